"""3-D F(2,3)^3 plans in 16-bit types with the width axis taken inside the product (csrc/conv.hip, `fold`).  The input
is transformed along depth and height only, over the pixel columns of the padded image (V: 16 elements per column of a
tile row), the three width taps lie side by side along the reduction of the shifted batched GEMM (one run of three
pieces, each one row of V further), and M too holds 16 elements per column: half of what F(2,3)^3 reads and writes.
The library takes the path by size; forced here (wc_test_gemm_override(12, .)) so that small shapes reach it, with each
of the kernels of the shifted product (rows_mode 0, 2, 3, 4).  Nothing the reference does (its 3-D path is F(2,3)^3
through three kernels: src/base_conv_launchers.cu); the convolution itself pins it."""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, K, pad
    ((2, 32, 6, 10, 12), 8, 1), ((1, 5, 4, 7, 9), 6, 1), ((2, 64, 5, 9, 8), 40, (0, 1, 1)), ((1, 128, 8, 12, 12), 128, 1),
    ((3, 16, 3, 3, 3), 8, 1), ((1, 40, 7, 11, 6), 33, (1, 0, 1)), ((2, 8, 9, 14, 15), 16, 0), ((1, 136, 4, 6, 6), 24, 1),
    ((2, 128, 8, 40, 40), 136, 1),       # more 512-row tiles than workgroups
]
DISC = {torch.float16: "fp16", torch.bfloat16: "bf16"}


def _rel(a, r):
    r = r.double()
    return float((a.double().cpu() - r).abs().max() / r.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("rows_mode", [0, 2, 3, 4])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_folded_product_against_fp64_and_the_three_kernel_path(dev, dtype, case, rows_mode, gemm_override, host_layer):
    xs, K, pad = case
    g = torch.Generator().manual_seed(31)
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(K, xs[1], 3, 3, 3, generator=g) * (2.0 / (27 * xs[1])) ** 0.5).to(dtype)
    b = torch.randn(K, generator=g).to(dtype)
    ref = F.conv3d(x.double(), w.double(), b.double(), padding=pad)
    gemm_override(config=11)
    y0 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2)
    gemm_override(config=12, rows_mode=rows_mode)
    y1 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2)
    tol = 2e-3 if dtype == torch.float16 else 1.6e-2
    assert tuple(y1.shape) == tuple(ref.shape)
    assert _rel(y1, ref) <= tol and _rel(y0, ref) <= tol
    assert _rel(y1, y0.double().cpu()) <= tol
    # with a transformed filter kept by the caller (the same U as for the three-kernel path), channel-first output
    U = engine.transform_filter(w.to(dev), xs, 1, pad, 2)
    assert torch.equal(engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, U=U), y1)
    ycf = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, channels_first_out=True)
    assert ycf.is_contiguous() and torch.equal(ycf, y1)


@pytest.mark.parametrize("rows_mode", [0, 2, 3, 4])
@pytest.mark.parametrize("case", [c for c in CASES if c[0][1] <= 64])
def test_folded_product_is_exact_on_small_integers(dev, case, rows_mode, gemm_override):
    """x in -3..3, taps multiples of 8 (G of F(2,3) halves per axis): every U, V and product is an integer and the sums
    stay below 2048 in fp16, whichever way they are grouped."""
    xs, K, pad = case
    g = torch.Generator().manual_seed(32)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = 8.0 * torch.randint(-1, 2, (K, xs[1], 3, 3, 3), generator=g).double()
    keep = (torch.rand(w.shape, generator=g) < 0.25).double()           # sparse taps keep the sums small
    w = w * keep
    b = torch.randint(-8, 9, (K,), generator=g).double()
    ref = F.conv3d(x, w, b, padding=pad)
    if float(ref.abs().max()) >= 2048:
        pytest.skip("sums beyond the exact range of fp16")
    gemm_override(config=12, rows_mode=rows_mode)
    y = engine.conv_forward(x.half().to(dev), w.half().to(dev), b.half().to(dev), 1, pad, 2)
    assert torch.equal(y.cpu(), ref.half())


def test_the_library_folds_by_size(dev, gemm_override):
    """Few channels over many tiles: the workspace of the folded path (V and M half as large, the folded filter beside
    U) is what wc_conv_workspace_bytes reports; against fp64 on a slice."""
    import ctypes
    from pytorch_winoconv_amd import _lib
    lib = _lib.load()
    xs, K = (3, 64, 16, 28, 28), 64
    n = {}
    for cfg in (11, 12, -1):
        gemm_override(config=cfg)
        d = engine.make_desc(xs, (K, xs[1], 3, 3, 3), torch.float16, 1, 1, 2)
        nb = ctypes.c_size_t()
        _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(d), ctypes.byref(nb)))
        n[cfg] = nb.value
    assert n[-1] == n[12] < n[11]
    gemm_override(config=-1)
    d = engine.make_desc((1, 256, 16, 28, 28), (256, 256, 3, 3, 3), torch.float16, 1, 1, 2)
    nb, nb11 = ctypes.c_size_t(), ctypes.c_size_t()
    _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(d), ctypes.byref(nb)))
    gemm_override(config=11)
    _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(d), ctypes.byref(nb11)))
    assert nb.value == nb11.value                                        # 256 channels over 1568 tiles: not folded
    gemm_override(config=-1)
    g = torch.Generator().manual_seed(33)
    x = torch.randn(*xs, generator=g).half()
    w = (torch.randn(K, xs[1], 3, 3, 3, generator=g) * (2.0 / (27 * xs[1])) ** 0.5).half()
    y = engine.conv_forward(x.to(dev), w.to(dev), None, 1, 1, 2)
    ref = F.conv3d(x[:1].double(), w.double(), None, padding=1)
    assert _rel(y[:1], ref) <= 2e-3
    assert _rel(y[:1, :, :2], ow.dwm_conv(x[:1, :, :3], w, None, 1, 1, 2, "fp16")[:, :, :2]) <= 2e-3


@pytest.mark.parametrize("chunk", [1, 2])
def test_folded_path_in_chunks_of_images(dev, chunk, gemm_override):
    """Batches cut into passes of `chunk` images (the last one partial) give what one pass gives, bit for bit: V and M of
    a pass are laid out by the images it holds."""
    g = torch.Generator().manual_seed(35)
    xs, K = (5, 64, 6, 12, 20), 72
    x = torch.randn(*xs, generator=g).half().to(dev)
    w = (torch.randn(K, xs[1], 3, 3, 3, generator=g) * (2.0 / (27 * xs[1])) ** 0.5).half().to(dev)
    b = torch.randn(K, generator=g).half().to(dev)
    gemm_override(config=12)
    whole = engine.conv_forward(x, w, b, 1, 1, 2)
    parts = engine.conv_forward(x, w, b, 1, 1, 2, chunk_images=chunk)
    assert torch.equal(whole, parts)
    ref = F.conv3d(x.double().cpu(), w.double().cpu(), b.double().cpu(), padding=1)
    assert _rel(parts, ref) <= 2e-3
