"""The one-kernel F(2x2, 3x3) path that wc_conv_forward takes for thin fp16 / bf16 3x3 stride-1 layers
(at most 128 input channels; conv_thin.hip).  It computes what the three-kernel path computes
(input transform of src/split_kernel.cu:60-120, batched product of
src/base_conv_launchers.cu:353-367, output transform of src/split_kernel.cu:126-203) without V and M
in memory, so the product is not rounded to the storage type before the output transform.

Pinned three ways: bit-exact against an integer convolution on inputs for which every intermediate
is exactly representable (any wrong index, sign or dropped term changes an integer); against fp64
convolution and the CPU oracle on normal inputs (fp16 and bf16 2e-2 of the output range, the bound
of the three-kernel path with this tile); and against the three-kernel path itself."""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

SHAPES = [
    # N, C, K, H, W, pad
    (2, 64, 64, 8, 8, 1),
    (1, 64, 64, 7, 9, 1),        # odd output sizes: half-used tiles on both edges
    (3, 32, 64, 13, 11, 0),
    (2, 16, 48, 9, 9, 1),        # channels padded to 32, two per thread
    (2, 64, 128, 12, 12, 1),     # two groups of output channels
    (3, 32, 300, 20, 20, 1),     # five groups, the last one partly filled
    (2, 40, 20, 10, 10, 1),      # channels padded to 64; K no multiple of 16
    (1, 64, 6, 5, 5, 1),         # K no multiple of 4: element-wise stores
    (1, 8, 7, 4, 4, 1),
    (2, 64, 64, 3, 3, 0),        # one output pixel
    (1, 24, 32, 6, 20, 2),       # padding wider than the kernel needs
    (5, 64, 64, 30, 30, 1),      # more tiles than one round of workgroups' first blocks
    (2, 128, 64, 9, 11, 1),      # 128 channels: eight wavefronts, element rows split between two groups of four
    (3, 100, 130, 14, 14, 1),
    (6, 128, 128, 28, 28, 1),
]


def _rel(a, r):
    r = r.double()
    return float((a.double().cpu() - r).abs().max() / r.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_exact_on_small_integers(dev, dtype, shape):
    """x in -3..3, filter taps multiples of 4 (so G g G^T holds integers), integer bias: every
    transformed value, product and sum is an integer below 2^24, exact in both storage types and
    in the fp32 accumulators; the only rounding is the final one, of the exact result."""
    N, C, K, H, W, pad = shape
    g = torch.Generator().manual_seed(3)
    x = torch.randint(-3, 4, (N, C, H, W), generator=g).double()
    w = 4.0 * torch.randint(-2, 3, (K, C, 3, 3), generator=g).double()
    b = torch.randint(-8, 9, (K,), generator=g).double()
    ref = F.conv2d(x, w, b, padding=pad).float().to(dtype)
    y = engine.conv_forward(x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev), 1, pad, 2)
    assert tuple(y.shape) == tuple(ref.shape)
    assert torch.equal(y.cpu(), ref), float((y.cpu().double() - ref.double()).abs().max())


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", SHAPES)
def test_against_fp64_oracle_and_three_kernel_path(dev, dtype, shape):
    N, C, K, H, W, pad = shape
    g = torch.Generator().manual_seed(5)
    x = torch.randn(N, C, H, W, generator=g).to(dtype)
    w = (torch.randn(K, C, 3, 3, generator=g) * (2.0 / (9 * C)) ** 0.5).to(dtype)
    b = torch.randn(K, generator=g).to(dtype)
    ref = F.conv2d(x.double(), w.double(), b.double(), padding=pad)
    y_oracle = ow.dwm_conv(x, w, b, 1, pad, 2, "fp16" if dtype == torch.float16 else "bf16")
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    y = engine.conv_forward(xd, wd, bd, 1, pad, 2)
    y3 = engine.conv_forward(xd, wd, bd, 1, pad, 2, unfused=True)
    tol = 2e-2                                   # of the output range, both types, tile 2
    assert _rel(y, ref) <= tol and _rel(y3, ref) <= tol
    assert _rel(y, y_oracle) <= tol and _rel(y, y3.cpu()) <= tol
    # the product stays in fp32 here: no further from fp64 than the three-kernel path, rounding noise aside
    assert _rel(y, ref) <= 1.5 * _rel(y3, ref) + 1e-4
    no_bias = engine.conv_forward(xd, wd, None, 1, pad, 2)
    assert _rel(no_bias, F.conv2d(x.double(), w.double(), None, padding=pad)) <= tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_tile_request_and_cached_filter(dev, dtype):
    """The fused kernel is the F(2,3) one: it runs for tile 2, with or without a cached U, and
    never for tile 4."""
    g = torch.Generator().manual_seed(7)
    x = torch.randn(3, 48, 17, 15, generator=g).to(dtype).to(dev)
    w = (torch.randn(40, 48, 3, 3, generator=g) * 0.05).to(dtype).to(dev)
    b = torch.randn(40, generator=g).to(dtype).to(dev)
    y2 = engine.conv_forward(x, w, b, 1, 1, 2)
    U2 = engine.transform_filter(w, x.shape, 1, 1, 2)
    assert torch.equal(engine.conv_forward(x, w, b, 1, 1, 2, U=U2), y2)
    U4 = engine.transform_filter(w, x.shape, 1, 1, 4)
    y4 = engine.conv_forward(x, w, b, 1, 1, 4, unfused=True)
    assert torch.equal(engine.conv_forward(x, w, b, 1, 1, 4, U=U4), y4)
    assert torch.equal(engine.conv_forward(x, w, b, 1, 1, 4), y4)
    # unfused = stage by stage
    desc = engine.make_desc(x.shape, w.shape, dtype, 1, 1, 2)
    plan = engine.plan_conv(desc)
    V = engine.input_transform(desc, plan, engine.channel_last(x))
    M = engine.batched_gemm(V, engine.filter_transform(desc, plan, w))
    y_st = engine.output_transform(desc, plan, M, b, x.shape[0])
    y3 = engine.conv_forward(x, w, b, 1, 1, 2, unfused=True)
    assert torch.equal(y3.permute(0, 2, 3, 1), y_st[:, 0])
    assert not torch.equal(y3, y2)               # other roundings: the fused kernel did run above


@pytest.mark.parametrize("case", [
    # x shape, w shape, stride, dtype: outside the fused kernel's range, same result with and without `unfused`
    ((2, 5, 9, 9), (8, 5, 3, 3), 1, torch.float16),          # odd channel count above 4
    ((2, 96, 9, 9), (8, 96, 3, 3), 1, torch.float16),        # channels pad to 96: no kernel of that width
    ((2, 160, 9, 9), (8, 160, 3, 3), 1, torch.float16),      # more than 128 input channels
    ((2, 64, 9, 9), (520, 64, 3, 3), 1, torch.float16),      # more than 512 output channels
    ((2, 64, 12, 12), (8, 64, 3, 3), 2, torch.float16),      # stride 2
    ((2, 64, 12, 12), (8, 64, 5, 5), 1, torch.float16),      # DWM plan
    ((2, 96, 9, 9), (8, 96, 3, 3), 1, torch.float32),       # fp32 with more than 64 channels
    ((2, 64, 9, 9), (300, 64, 3, 3), 1, torch.float32),     # fp32, 64 channels, more than 256 output channels
    ((2, 64, 5, 9, 9), (8, 64, 3, 3, 3), 1, torch.float16),  # 3-D
])
def test_outside_the_range_nothing_changes(dev, case):
    xs, ws, stride, dtype = case
    g = torch.Generator().manual_seed(9)
    x = torch.randn(*xs, generator=g).to(dtype).to(dev)
    w = (torch.randn(*ws, generator=g) * 0.05).to(dtype).to(dev)
    assert torch.equal(engine.conv_forward(x, w, None, stride, 1, 2),
                       engine.conv_forward(x, w, None, stride, 1, 2, unfused=True))


def test_resnet_layer_at_full_size(dev):
    """N=64, C=K=64, 56x56 fp16 (the first ResNet-50 3x3 shape): fused against three kernels, and
    linearity in the filter (conv(x, w1 + w2) = conv(x, w1) + conv(x, w2) up to rounding)."""
    g = torch.Generator().manual_seed(1)
    x = torch.randn(64, 64, 56, 56, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    w1 = (torch.randn(64, 64, 3, 3, generator=g) * (2.0 / 576) ** 0.5).half().to(dev)
    w2 = (torch.randn(64, 64, 3, 3, generator=g) * (2.0 / 576) ** 0.5).half().to(dev)
    y1 = engine.conv_forward(x, w1, None, 1, 1, 2)
    y3 = engine.conv_forward(x, w1, None, 1, 1, 2, unfused=True)
    scale = float(y3.float().abs().max())
    assert float((y1.float() - y3.float()).abs().max()) <= 4e-3 * scale
    y2 = engine.conv_forward(x, w2, None, 1, 1, 2)
    y12 = engine.conv_forward(x, (w1.float() + w2.float()).half(), None, 1, 1, 2)
    assert float((y12.float() - y1.float() - y2.float()).abs().max()) <= 6e-3 * scale
    sample = F.conv2d(x[:2].double().cpu(), w1.double().cpu(), padding=1)
    assert _rel(y1[:2], sample) <= 2e-3


TINY = [
    # N, C, K, H, W, pad: at most 4 input channels, any storage type (tiny_conv3x3_kernel)
    (2, 3, 64, 12, 12, 1),
    (1, 1, 8, 7, 9, 1),
    (3, 4, 70, 13, 11, 0),
    (2, 2, 6, 9, 9, 1),
    (1, 3, 130, 20, 21, 2),
    (9, 3, 32, 17, 16, 1),       # more than one block of 64 tiles
    (2, 3, 64, 3, 3, 0),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", TINY)
def test_first_layers_exact_on_small_integers(dev, dtype, shape):
    """Same construction as above; the product of these layers runs in fp32 whatever the storage type."""
    N, C, K, H, W, pad = shape
    g = torch.Generator().manual_seed(13)
    x = torch.randint(-3, 4, (N, C, H, W), generator=g).double()
    w = 4.0 * torch.randint(-2, 3, (K, C, 3, 3), generator=g).double()
    b = torch.randint(-8, 9, (K,), generator=g).double()
    ref = F.conv2d(x, w, b, padding=pad).float().to(dtype)
    y = engine.conv_forward(x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev), 1, pad, 2)
    assert tuple(y.shape) == tuple(ref.shape) and torch.equal(y.cpu(), ref)
    assert torch.equal(engine.conv_forward(x.to(dtype).to(dev), w.to(dtype).to(dev), None, 1, pad, 2).cpu(),
                       F.conv2d(x, w, None, padding=pad).float().to(dtype))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("shape", TINY)
def test_first_layers_against_fp64_and_three_kernel_path(dev, dtype, shape):
    N, C, K, H, W, pad = shape
    g = torch.Generator().manual_seed(17)
    x = torch.randn(N, C, H, W, generator=g).to(dtype)
    w = (torch.randn(K, C, 3, 3, generator=g) * (2.0 / (9 * C)) ** 0.5).to(dtype)
    b = torch.randn(K, generator=g).to(dtype)
    ref = F.conv2d(x.double(), w.double(), b.double(), padding=pad)
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    y = engine.conv_forward(xd, wd, bd, 1, pad, 2)
    y3 = engine.conv_forward(xd, wd, bd, 1, pad, 2, unfused=True)
    tol = 1e-3 if dtype == torch.float32 else 2e-2
    assert _rel(y, ref) <= tol and _rel(y3, ref) <= tol and _rel(y, y3.cpu()) <= tol
    assert _rel(y, ref) <= 1.5 * _rel(y3, ref) + (1e-6 if dtype == torch.float32 else 1e-4)
    U = engine.transform_filter(wd, x.shape, 1, pad, 2)
    assert torch.equal(engine.conv_forward(xd, wd, bd, 1, pad, 2, U=U), y)
    if dtype != torch.float32:
        assert not torch.equal(y3, y)            # other roundings (M stays in fp32): the fused kernel did run


def test_misaligned_view_takes_the_three_kernel_path(dev):
    """x[1:] of a channel-last fp16 tensor with 6 channels and 7 x 7 images starts 588 bytes into the
    allocation: 4-byte aligned.  The one-kernel path needs 16-byte aligned operands, so the host layer
    sends such a view through the three kernels, with the same result as for an aligned copy."""
    g = torch.Generator().manual_seed(21)
    x = torch.randn(3, 6, 7, 7, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(8, 6, 3, 3, generator=g) * (2.0 / 54) ** 0.5).half().to(dev)
    view = x[1:]
    assert view.permute(0, 2, 3, 1).is_contiguous() and view.data_ptr() % 8 != 0
    y = engine.conv_forward(view, w, None, 1, 1, 2)
    y3 = engine.conv_forward(view.clone(memory_format=torch.channels_last), w, None, 1, 1, 2, unfused=True)
    assert torch.equal(y, y3)
    ref = F.conv2d(view.double().cpu(), w.double().cpu(), padding=1)
    assert float((y.double().cpu() - ref).abs().max() / ref.abs().max()) <= 2e-2


def test_fp16_input_transform_of_the_fused_kernel_at_large_magnitudes(dev):
    """The fused fp16 kernel transforms the input with fp16 adds (the reference kernels' arithmetic type,
    calculation_kernels.cu:786-806) where the three-kernel path adds in fp32 and rounds once.  With
    inputs of magnitude 1e3..1e4 (sums of four stay below the fp16 maximum) the two agree to fp16
    rounding of V, and both stay within the fp16 tolerance of the fp64 convolution."""
    g = torch.Generator().manual_seed(22)
    x = (torch.randn(2, 64, 20, 20, generator=g) * 3e3).clamp(-1.2e4, 1.2e4).half().to(dev)
    w = (torch.randn(64, 64, 3, 3, generator=g) * (2.0 / 576) ** 0.5).half().to(dev)
    y = engine.conv_forward(x, w, None, 1, 1, 2)
    y3 = engine.conv_forward(x, w, None, 1, 1, 2, unfused=True)
    ref = F.conv2d(x.double().cpu(), w.double().cpu(), padding=1)
    scale = float(ref.abs().max())
    assert torch.isfinite(y).all() and torch.isfinite(y3).all()
    assert float((y.double().cpu() - ref).abs().max()) / scale <= 2e-2
    assert float((y3.double().cpu() - ref).abs().max()) / scale <= 2e-2
    assert float((y.double() - y3.double()).abs().max()) / scale <= 5e-3


FP32_SHAPES = [s for s in SHAPES if s[1] <= 64 and s[1] % 2 == 0 and s[2] <= 256] + [
    (1, 64, 64, 56, 56, 1),      # the single-layer configuration of the benchmark suite
    (2, 32, 400, 10, 12, 1),     # 32 channels: up to 512 output channels
    (3, 50, 256, 14, 9, 1),
]


@pytest.mark.parametrize("shape", FP32_SHAPES)
def test_fp32_layers_of_at_most_64_channels(dev, shape):
    """fp32 with at most 64 input channels runs the same one kernel on v_mfma_f32_16x16x4_f32 (U of 32 channels in
    four wavefronts' registers, of 64 channels in eight).  Exact on small integers; on normal inputs within the fp32
    tolerance of the fp64 convolution and of the oracle, and as close to fp64 as the three-kernel path."""
    N, C, K, H, W, pad = shape
    assert engine.thin_layer(torch.float32, 2, C, K, (3, 3), 1)
    g = torch.Generator().manual_seed(11)
    xi = torch.randint(-3, 4, (N, C, H, W), generator=g).double()
    wi = 4.0 * torch.randint(-2, 3, (K, C, 3, 3), generator=g).double()
    bi = torch.randint(-8, 9, (K,), generator=g).double()
    yi = engine.conv_forward(xi.float().to(dev), wi.float().to(dev), bi.float().to(dev), 1, pad, 2)
    assert torch.equal(yi.cpu(), F.conv2d(xi, wi, bi, padding=pad).float())
    x = torch.randn(N, C, H, W, generator=g)
    w = torch.randn(K, C, 3, 3, generator=g) * (2.0 / (9 * C)) ** 0.5
    b = torch.randn(K, generator=g)
    ref = F.conv2d(x.double(), w.double(), b.double(), padding=pad)
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    y = engine.conv_forward(xd, wd, bd, 1, pad, 2)
    y3 = engine.conv_forward(xd, wd, bd, 1, pad, 2, unfused=True)
    assert _rel(y, ref) <= 1e-3 and _rel(y, ow.dwm_conv(x, w, b, 1, pad, 2, "fp32")) <= 1e-5
    assert _rel(y, ref) <= 1.5 * _rel(y3, ref) + 1e-6
    # the fused kernel did run: one product stage, no transform stages (its sums have the order of the three
    # kernels', so on a small layer the two results can agree bit for bit)
    yt, stages = engine.conv_forward_timed(xd, wd, bd, 1, pad, 2)
    assert torch.equal(yt, y)
    assert stages["product"] > 0 and stages["input_transform"] == 0 and stages["output_transform"] == 0
    U = engine.transform_filter(wd, x.shape, 1, pad, 2)
    assert torch.equal(engine.conv_forward(xd, wd, bd, 1, pad, 2, U=U), y)


@pytest.mark.parametrize("config", [8, 9])
@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("shape", SHAPES)
def test_both_workgroup_sizes_are_exact_on_small_integers(dev, dtype, shape, config, gemm_override):
    """The kernel has workgroups of 64 output channels and, for layers with few blocks of tiles, of 32 (half the
    wavefronts, each transforming twice the channels).  The library chooses by the number of tiles; here each form is
    forced on every shape (the small form falls back where a thread's channels would straddle C)."""
    N, C, K, H, W, pad = shape
    if not engine.thin_layer(dtype, 2, C, K, (3, 3), 1):
        pytest.skip("outside the range of the one-kernel path for this type")
    gemm_override(config=config)
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-3, 4, (N, C, H, W), generator=g).double()
    w = 4.0 * torch.randint(-2, 3, (K, C, 3, 3), generator=g).double()
    b = torch.randint(-8, 9, (K,), generator=g).double()
    ref = F.conv2d(x, w, b, padding=pad).float().to(dtype)
    xd, wd, bd = x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev)
    yt, stages = engine.conv_forward_timed(xd, wd, bd, 1, pad, 2)
    assert stages["product"] > 0 and stages["input_transform"] == 0 and stages["output_transform"] == 0
    assert torch.equal(yt.cpu(), ref)
    # normal data: both forms add in the same order, so they agree bit for bit
    x2 = torch.randn(N, C, H, W, generator=g).to(dtype).to(dev)
    w2 = (torch.randn(K, C, 3, 3, generator=g) * (2.0 / (9 * C)) ** 0.5).to(dtype).to(dev)
    y_forced = engine.conv_forward(x2, w2, bd, 1, pad, 2)
    gemm_override(config=8 if config == 9 else 9)
    assert torch.equal(engine.conv_forward(x2, w2, bd, 1, pad, 2), y_forced)
