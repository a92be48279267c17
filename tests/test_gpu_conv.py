"""End-to-end parity of wc_conv_forward (through the C ABI) against fp64 torch convolution and
against the CPU oracle run in the same arithmetic discipline.

Tolerances (max |y - y64| / max |y64|, fp64 conv fed the same already-rounded inputs):
  fp32 F(2x2,3x3) and every fp32 F(2,r) plan: 1e-3 (measured ~1e-6),
  fp16 (any plan, F(4x4,3x3) included):       2e-2 (F(4,r) tiles: with 8 or more input channels; the
      rounding error of a tile-4 transform averages down over the channels, and with one or two
      channels unlucky data reach 3e-2 - the modules use tile 2 there).
"""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

TOL = {torch.float32: 1e-3, torch.float16: 2e-2}
DISC = {torch.float32: "fp32", torch.float16: "fp16"}


def _data(xs, ws, dtype, seed=0, uniform=False):
    g = torch.Generator().manual_seed(seed)
    if uniform:
        x, w = torch.rand(*xs, generator=g), torch.rand(*ws, generator=g)
    else:
        fan_in = 1
        for v in ws[1:]:
            fan_in *= v
        x = torch.randn(*xs, generator=g)
        w = torch.randn(*ws, generator=g) * (2.0 / fan_in) ** 0.5
    b = torch.randn(ws[0], generator=g)
    return x.to(dtype), w.to(dtype), b.to(dtype)


def _conv64(x, w, b, stride, pad):
    f = F.conv2d if x.dim() == 4 else F.conv3d
    return f(x.double(), w.double(), None if b is None else b.double(), stride=stride, padding=pad)


def _nerr(y, ref):
    return float((y.double().cpu() - ref).abs().max() / ref.abs().max())


CASES = [
    # reduced-size versions of the benchmark configurations and of the reference's own demos
    ((1, 64, 56, 56), (64, 64, 3, 3), 1, 1, 2),        # configs[0] at full size
    ((2, 64, 56, 56), (64, 64, 3, 3), 1, 1, 4),
    ((2, 3, 32, 32), (64, 3, 3, 3), 1, 1, 2),           # VGG first layer shape (C = 3)
    ((2, 3, 32, 32), (64, 3, 3, 3), 1, 1, 4),
    ((3, 128, 28, 28), (128, 128, 3, 3), 1, 1, 4),      # ResNet-style
    ((4, 256, 14, 14), (256, 256, 3, 3), 1, 1, 4),
    ((4, 512, 7, 7), (512, 512, 3, 3), 1, 1, 4),
    ((2, 32, 23, 21), (48, 32, 3, 3), 1, 1, 4),         # odd extents: partial edge tiles
    ((2, 32, 23, 21), (48, 32, 3, 3), 1, 0, 2),
    ((2, 32, 28, 28), (32, 32, 5, 5), 1, 2, 2),         # DWM
    ((2, 32, 28, 28), (32, 32, 7, 7), 1, 3, 2),
    ((2, 32, 28, 28), (32, 32, 3, 3), 2, 1, 2),
    ((2, 32, 28, 28), (32, 32, 7, 7), 2, 3, 2),
    ((2, 32, 28, 28), (32, 32, 5, 5), 1, 2, 4),         # DWM with output tile 4
    ((2, 32, 28, 28), (32, 32, 7, 7), 1, 3, 4),
    ((2, 32, 28, 28), (32, 32, 3, 3), 2, 1, 4),
    ((2, 32, 29, 27), (32, 32, 7, 7), 2, 3, 4),
    ((1, 224, 10, 10), (32, 224, 7, 7), 1, 0, 2),       # example.py:100-101
    ((1, 32, 10, 10, 10), (32, 32, 3, 3, 3), 1, 0, 2),  # example.py:112-113
    ((2, 32, 8, 14, 14), (32, 32, 3, 3, 3), 1, 1, 2),   # C3D-style
    ((2, 32, 8, 14, 14), (32, 32, 3, 3, 3), 1, 1, 4),   # ... with the tile 2 x 4 x 4
    ((1, 16, 5, 11, 9), (24, 16, 3, 3, 3), 1, 0, 4),
    ((1, 16, 6, 9, 9), (16, 16, 5, 5, 5), 1, 2, 2),
    ((1, 8, 12, 12), (8, 8, 9, 9), 1, 4, 2),
    ((1, 8, 14, 14), (8, 8, 4, 3), 1, 0, 2),
    ((1, 8, 9, 9, 9), (8, 8, 1, 3, 3), 1, 0, 2),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_conv_vs_fp64(dev, dtype, case):
    xs, ws, stride, pad, m = case
    x, w, b = _data(xs, ws, dtype)
    ref = _conv64(x, w, b, stride, pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m)
    assert tuple(y.shape) == tuple(ref.shape)
    assert y.dtype == dtype
    assert _nerr(y, ref) <= TOL[dtype]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", [c for c in CASES if c[0][0] * c[0][1] <= 256])
def test_conv_vs_oracle_same_discipline(dev, dtype, case):
    """HIP result against the CPU restatement with the same storage/rounding points: only the
    summation order differs.  fp32: <= 1e-5.  fp16: a different order flips single fp16
    roundings of M by one ulp (4.9e-4 relative), which A^T x A^T of F(4,3) amplifies by up to
    64: <= 1e-2 of the output range.  `unfused`: thin 16-bit 3x3 layers otherwise take the
    one-kernel path, which keeps the product in fp32 (test_gpu_thin.py)."""
    xs, ws, stride, pad, m = case
    x, w, _ = _data(xs, ws, dtype, seed=5)
    om = (2, 4, 4) if (m == 4 and len(xs) == 5) else m        # the engine's 3-D "tile 4" is 2 x 4 x 4
    want = ow.dwm_conv(x, w, None, stride, pad, om, DISC[dtype])
    y = engine.conv_forward(x.to(dev), w.to(dev), None, stride, pad, m, unfused=True)
    assert _nerr(y, want.double()) <= (1e-5 if dtype == torch.float32 else 1e-2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", [
    ((2, 16, 11, 12), (8, 16, 3, 3), 1, 1, 2, 4),
    ((2, 16, 12, 12), (8, 16, 5, 5), 1, 2, 2, 4),
    ((1, 16, 13, 12), (8, 16, 7, 7), 2, 3, 2, 4),
    ((1, 8, 6, 8, 8), (8, 8, 3, 3, 3), 1, 1, 2, 8),
])
def test_integer_exactness(dev, dtype, case):
    """With integer inputs and integer weights that are multiples of the common denominator of
    G x G (x G) (4 in 2-D, 8 in 3-D for F(2,r), whose G holds only 0, 1 and 1/2) every
    intermediate is exactly representable, so Winograd must equal direct convolution bit for bit.
    F(4,3) is left out: its G holds 1/6, 1/12 and 1/24, which binary floating point cannot
    represent, so no choice of inputs makes the filter transform exact."""
    xs, ws, stride, pad, m, wmul = case
    g = torch.Generator().manual_seed(7)
    x = torch.randint(-2, 3, xs, generator=g).to(dtype)
    w = (torch.randint(-2, 3, ws, generator=g) * wmul).to(dtype)
    ref = _conv64(x, w, None, stride, pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), None, stride, pad, m)
    assert torch.equal(y.double().cpu(), ref)


WHOLE = [
    # x shape, w shape, pad; whole-kernel tile F(2,k) x F(2,k) (reference: matrix_conv.py:112-135)
    ((2, 32, 28, 28), (32, 32, 4, 4), 1),
    ((2, 32, 28, 28), (32, 32, 5, 5), 2),
    ((2, 32, 27, 29), (32, 32, 6, 6), 0),
    ((2, 32, 28, 28), (32, 32, 7, 7), 3),
    ((1, 224, 10, 10), (32, 224, 7, 7), 0),             # example.py:100-101
]


@pytest.mark.parametrize("case", WHOLE)
def test_whole_kernel_tile_fp32(dev, case):
    """fp32 whole-kernel tiles against fp64 convolution and against the oracle run in the same
    discipline.  The tile's own rounding error grows with k (the oracle shows 1e-6 at k = 4 to
    5e-4 at k = 7 on these inputs), so the bound against fp64 is 2e-3, and the engine's error
    must stay within 3x that of the oracle's fp32 evaluation of the same formula (the two
    differ in summation order, so at k = 7 they differ from each other as much as from fp64)."""
    xs, ws, pad = case
    x, w, b = _data(xs, ws, torch.float32)
    ref = _conv64(x, w, b, 1, pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, whole_kernel=True)
    assert tuple(y.shape) == tuple(ref.shape)
    assert _nerr(y, ref) <= 2e-3
    yo = ow.dwm_conv(x, w, b, 1, pad, 2, "fp32", whole_kernel=True)
    assert _nerr(y, ref) <= 3 * _nerr(yo, ref) + 1e-6


def test_decomposition_keeps_fp16_accurate_where_the_whole_kernel_tile_does_not(dev):
    """The reference's claim (example.py:99-109): for a 7x7 kernel in half precision the DWM
    pieces stay accurate while one F(2,7) tile does not.  Same uniform inputs as the demo."""
    x, w, _ = _data((1, 224, 10, 10), (32, 224, 7, 7), torch.float16, uniform=True)
    ref = _conv64(x, w, None, 1, 0)
    xd, wd = x.to(dev), w.to(dev)
    e_dwm = _nerr(engine.conv_forward(xd, wd, None, 1, 0, 2), ref)
    e_whole = _nerr(engine.conv_forward(xd, wd, None, 1, 0, 2, whole_kernel=True), ref)
    e_oracle = _nerr(ow.dwm_conv(x, w, None, 1, 0, 2, "fp16", whole_kernel=True), ref)
    assert e_dwm <= 2e-3
    assert e_whole >= 20 * e_dwm                         # the tile really is that much worse
    assert 0.25 * e_oracle <= e_whole <= 4 * e_oracle    # and as bad as the same formula on the CPU


def test_reference_statistic(dev):
    """The reference's own accuracy statistic mean(|(y - y64) / y64|) on U(0,1) data at its own
    shapes (example.py:99-119); recorded for continuity, bounded loosely."""
    for xs, ws in [((1, 224, 10, 10), (32, 224, 7, 7)), ((1, 32, 10, 10, 10), (32, 32, 3, 3, 3))]:
        x, w, _ = _data(xs, ws, torch.float32, uniform=True)
        ref = _conv64(x, w, None, 1, 0)
        y = engine.conv_forward(x.to(dev), w.to(dev), None, 1, 0, 2)
        assert float(((y.double().cpu() - ref) / ref).abs().mean()) < 1e-5
        yh = engine.conv_forward(x.half().to(dev), w.half().to(dev), None, 1, 0, 2)
        refh = _conv64(x.half(), w.half(), None, 1, 0)
        assert float(((yh.double().cpu() - refh) / refh).abs().mean()) < 5e-3


@pytest.mark.parametrize("chunk", [1, 2, 5])
def test_chunking_is_invisible(dev, chunk):
    xs, ws = (5, 32, 20, 20), (32, 32, 3, 3)
    x, w, b = _data(xs, ws, torch.float16)
    y0 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, 1, 4, chunk_images=0)
    y1 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, 1, 4, chunk_images=chunk)
    assert torch.equal(y0, y1)


def test_channels_last_input_and_cached_filter(dev):
    xs, ws = (2, 32, 20, 20), (32, 32, 3, 3)
    x, w, b = _data(xs, ws, torch.float16)
    xd = x.to(dev)
    y0 = engine.conv_forward(xd, w.to(dev), b.to(dev), 1, 1, 4)
    xcl = xd.contiguous(memory_format=torch.channels_last)
    U = engine.transform_filter(w.to(dev), xs, 1, 1, 4)
    y1 = engine.conv_forward(xcl, w.to(dev), b.to(dev), 1, 1, 4, U=U)
    assert torch.equal(y0, y1)
    assert y1.is_contiguous(memory_format=torch.channels_last)


def test_empty_batch_and_single_pixel_outputs(dev):
    """Empty input (N = 0) gives an empty output of the right shape, like torch; outputs of one
    pixel and inputs smaller than a tile are handled by the edge rules."""
    w = torch.randn(6, 4, 3, 3).half().to(dev)
    y = engine.conv_forward(torch.empty(0, 4, 9, 7, dtype=torch.float16, device=dev), w, None, 1, 1, 4)
    assert tuple(y.shape) == (0, 6, 9, 7) and y.dtype == torch.float16
    y3 = engine.conv_forward(torch.empty(0, 4, 5, 9, 7, device=dev), torch.randn(6, 4, 3, 3, 3, device=dev), None, 2, 1, 2)
    assert tuple(y3.shape) == (0, 6, 3, 5, 4)
    for xs, ws, stride, pad, m in (((2, 4, 3, 3), (6, 4, 3, 3), 1, 0, 4), ((1, 4, 1, 1), (6, 4, 3, 3), 1, 1, 2),
                                   ((2, 4, 7, 7), (6, 4, 7, 7), 2, 0, 4), ((1, 4, 2, 3, 3), (6, 4, 3, 3, 3), 1, (1, 0, 0), 2)):
        x, wt, b = _data(xs, ws, torch.float32)
        ref = _conv64(x, wt, b, stride, pad)
        yy = engine.conv_forward(x.to(dev), wt.to(dev), b.to(dev), stride, pad, m)
        assert tuple(yy.shape) == tuple(ref.shape) and _nerr(yy, ref) <= 1e-3


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("m", [2, 4])
@pytest.mark.parametrize("shape", [
    # N, C, K, H, W
    (3, 64, 72, 13, 11),       # dense filter, channels split evenly: one launch for both transforms
    (2, 256, 40, 9, 9),
    (2, 36, 24, 10, 12),       # channels padded to 64
    (2, 30, 16, 8, 8),         # fp16: 30 channels are no multiple of the filter threads' 4: two launches
    (5, 8, 8, 30, 30),
])
def test_filter_transformed_beside_the_input_equals_the_separate_launches(dev, dtype, m, shape):
    """With a fresh filter the three-kernel path of a 3x3 layer transforms the filter in the first workgroups of the
    input transform's launch.  Same arithmetic, so: bit-equal to a call with the filter transformed beforehand, to
    the stage-by-stage (timed) call and to a call with a second chunk of images; a filter in the reference's (kH, kW, C, K)
    memory is read through strides by another kernel in a launch of its own; integer inputs come out exact."""
    N, C, K, H, W = shape
    g = torch.Generator().manual_seed(21)
    x = torch.randn(N, C, H, W, generator=g).to(dtype).to(dev)
    w = (torch.randn(K, C, 3, 3, generator=g) * (2.0 / (9 * C)) ** 0.5).to(dtype).to(dev)
    b = torch.randn(K, generator=g).to(dtype).to(dev)
    kw = dict(unfused=True)              # thin layers would take the one-kernel path
    y = engine.conv_forward(x, w, b, 1, 1, m, **kw)
    U = engine.transform_filter(w, x.shape, 1, 1, m)
    assert torch.equal(engine.conv_forward(x, w, b, 1, 1, m, U=U, **kw), y)
    yt, stages = engine.conv_forward_timed(x, w, b, 1, 1, m, **kw)
    assert torch.equal(yt, y) and stages["filter_transform"] > 0 and stages["input_transform"] > 0
    w_ref = w.permute(2, 3, 1, 0).contiguous().permute(3, 2, 0, 1)       # same values, (kH, kW, C, K) memory
    assert not w_ref.is_contiguous() and torch.equal(w_ref, w)
    y_ref = engine.conv_forward(x, w_ref, b, 1, 1, m, **kw)      # another filter kernel: equal to the last bit or two
    assert float((y_ref.double() - y.double()).abs().max() / y.double().abs().max()) <= {torch.float32: 1e-6, torch.float16: 4e-3, torch.bfloat16: 3e-2}[dtype]
    if N > 1:
        assert torch.equal(engine.conv_forward(x, w, b, 1, 1, m, chunk_images=N - 1, **kw), y)
    ref = F.conv2d(x.double().cpu(), w.double().cpu(), b.double().cpu(), padding=1)
    tol = {torch.float32: 1e-3, torch.float16: 2e-2, torch.bfloat16: 2e-2 if m == 2 else 2e-1}[dtype]      # bf16 with tile 4: as everywhere
    assert float((y.double().cpu() - ref).abs().max() / ref.abs().max()) <= tol
    xi = torch.randint(-3, 4, (N, C, H, W), generator=g).double()
    wi = (4.0 if m == 2 else 24.0) * torch.randint(-2, 3, (K, C, 3, 3), generator=g).double()      # G g G^T stays integral
    if float(F.conv2d(xi, wi, padding=1).abs().max()) < (2048 if dtype == torch.float16 else 256 if dtype == torch.bfloat16 else 1 << 24):
        yi = engine.conv_forward(xi.to(dtype).to(dev), wi.to(dtype).to(dev), None, 1, 1, m, **kw)
        if m == 2:
            assert torch.equal(yi.cpu().double(), F.conv2d(xi, wi, padding=1))
