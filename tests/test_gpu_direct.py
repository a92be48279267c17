"""The direct form (wc_conv_desc.direct): pieces of one tap on the tile F(1,1), i.e. the batched product reading the
pixels of x itself with the taps along its reduction axis.  The library chooses it for 1x1 kernels (every type) and for
16-bit stride-2 layers (which the reference does not implement: src/winograd_conv.cpp:122-126) where it measured
faster than the parity-phase Winograd plan the caller would otherwise get; on request it runs any 2-D kernel and stride.

Pinned bit for bit on small integers (every product and sum exact), against fp64 torch convolution and the oracle on
normal data, and against the Winograd / DWM plans of the same engine."""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, w shape, stride, pad
    ((2, 32, 12, 13), (8, 32, 3, 3), 2, 1), ((3, 64, 21, 20), (24, 64, 3, 3), 2, 1), ((1, 32, 9, 9), (16, 32, 3, 3), 2, 0),
    ((2, 32, 15, 14), (8, 32, 7, 7), 2, 3), ((1, 96, 17, 19), (40, 96, 5, 5), 2, 2), ((2, 32, 10, 11), (8, 32, 4, 6), 2, (1, 2)),
    ((1, 128, 30, 30), (136, 128, 3, 3), 2, 1), ((2, 32, 8, 9), (8, 32, 1, 1), 2, 0), ((2, 32, 9, 10), (72, 32, 2, 2), 2, 0),
    ((5, 64, 33, 31), (64, 64, 3, 3), 2, 1), ((1, 32, 7, 7), (8, 32, 7, 7), 2, 3), ((2, 32, 10, 10), (8, 32, 3, 3), 2, 3),
    ((40, 32, 28, 28), (32, 32, 3, 3), 2, 1),     # enough output pixels for the largest tile
    # stride 1 on request
    ((2, 32, 9, 11), (8, 32, 3, 3), 1, 1), ((1, 64, 12, 12), (16, 64, 5, 5), 1, 2), ((1, 32, 8, 8), (8, 32, 1, 3), 1, (0, 1)),
    # 1x1 kernels: the library's own choice at either stride
    ((3, 64, 13, 11), (40, 64, 1, 1), 1, 0), ((2, 32, 10, 10), (8, 32, 1, 1), 1, 1), ((6, 96, 28, 28), (256, 96, 1, 1), 1, 0),
]
DISC = {torch.float16: "fp16", torch.bfloat16: "bf16", torch.float32: "fp32"}


def _rel(a, b):
    return float((a.double().cpu() - b.double().cpu()).abs().max() / b.double().abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES)
def test_exact_on_small_integers(dev, dtype, case, host_layer):
    xs, ws, stride, pad = case
    g = torch.Generator().manual_seed(1)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = torch.randint(-2, 3, ws, generator=g).double()
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    ref = F.conv2d(x, w, b, stride=stride, padding=pad)
    assert float(ref.abs().max()) < {torch.float16: 2048, torch.bfloat16: 256, torch.float32: 1 << 21}[dtype] * 8      # representable after the one rounding
    y = engine.conv_forward(x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev), stride, pad, 2, direct=True)
    assert tuple(y.shape) == tuple(ref.shape)
    assert torch.equal(y.cpu(), ref.float().to(dtype))
    assert torch.equal(y.cpu(), ow.direct_conv(x, w, b, stride, pad, DISC[dtype]))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
@pytest.mark.parametrize("case", CASES)
def test_against_fp64_the_oracle_and_the_winograd_plans(dev, dtype, case):
    xs, ws, stride, pad = case
    g = torch.Generator().manual_seed(2)
    fan = ws[1] * ws[2] * ws[3]
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    y = engine.conv_forward(xd, wd, bd, stride, pad, 2, direct=True)
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.2e-2, torch.float32: 2e-6}[dtype]            # one rounding of an fp32 sum
    assert _rel(y, ref) <= tol
    assert _rel(y, ow.direct_conv(x, w, b, stride, pad, DISC[dtype])) <= tol
    yw = engine.conv_forward(xd, wd, bd, stride, pad, 2, direct=False)          # the Winograd / DWM plan
    assert _rel(yw, ref) <= (1e-3 if dtype == torch.float32 else 2e-2) and _rel(y, yw.cpu()) <= 2e-2
    # the library's own choice is one of the two: always the direct form for one tap, never for more taps at stride 1
    # or in fp32
    chosen = engine.make_desc(xs, ws, dtype, stride, pad, 2, stacked=None).direct
    if ws[2] * ws[3] == 1:
        assert chosen == 1
    elif stride == 1:
        assert chosen == 0
    ya = engine.conv_forward(xd, wd, bd, stride, pad, 2)
    assert torch.equal(ya, y if chosen else yw)
    # cached filter, no bias, channel-first in and out, one image per pass
    U = engine.transform_filter(wd, xs, stride, pad, 2, direct=True)
    assert tuple(U.shape) == (ws[0], ws[2], ws[3], ws[1])
    assert torch.equal(U, wd.permute(0, 2, 3, 1).contiguous())
    assert torch.equal(engine.conv_forward(xd, wd, bd, stride, pad, 2, U=U, direct=True), y)
    assert _rel(engine.conv_forward(xd, wd, None, stride, pad, 2, direct=True), F.conv2d(x.double(), w.double(), None, stride=stride, padding=pad)) <= tol
    xcl = xd.contiguous(memory_format=torch.channels_last)
    ycf = engine.conv_forward(xcl, wd, bd, stride, pad, 2, direct=True, channels_first_out=True, chunk_images=1)
    assert ycf.is_contiguous() and torch.equal(ycf, y)


def test_outside_its_range_the_direct_form_is_refused_or_not_chosen(dev):
    x = torch.randn(2, 20, 12, 12, device=dev).half()
    w = torch.randn(8, 20, 3, 3, device=dev).half()
    with pytest.raises(NotImplementedError, match="direct form"):
        engine.conv_forward(x, w, None, 2, 1, 2, direct=True)                   # 20 channels: no multiple of 32
    assert engine.make_desc(x.shape, w.shape, torch.float16, 2, 1, 2, stacked=None).direct == 0
    assert engine.make_desc((2, 32, 12, 12), (8, 32, 3, 3), torch.float16, 2, 1, 2, stacked=None).direct == 1
    assert engine.make_desc((2, 32, 12, 12), (8, 32, 3, 3), torch.float16, 1, 1, 2, stacked=None).direct == 0      # stride 1
    assert engine.make_desc((2, 32, 12, 12), (8, 32, 5, 5), torch.float32, 2, 2, 2, stacked=None).direct == 0      # fp32 beyond 3x3
    assert engine.make_desc((2, 32, 12, 12), (8, 32, 3, 3), torch.float16, 2, 1, 2, stacked=None, direct=False).direct == 0
    assert engine.make_desc((2, 32, 12, 12), (12, 32, 3, 3), torch.float16, 2, 1, 2, stacked=None).direct == 0     # K no multiple of 8
    assert engine.make_desc((2, 32, 12, 12), (8, 32, 3, 3), torch.float16, 2, 1, 2, stacked=True).direct == 0      # an explicit plan form


def test_c4_stride_2_layers_at_full_size(dev):
    """N=32, 128 channels, 112x112, 3x3 and 7x7 at stride 2, the library's choice (the direct form for both) and the
    direct form on request: the last image against fp64 on the CPU, and a permuted batch gives the permuted output
    bit for bit."""
    g = torch.Generator().manual_seed(3)
    x = torch.randn(32, 128, 112, 112, generator=g).half()
    xd = x.to(dev).contiguous(memory_format=torch.channels_last)
    for k, pad in ((3, 1), (7, 3)):
        w = (torch.randn(128, 128, k, k, generator=g) * (2.0 / (128 * k * k)) ** 0.5).half()
        assert engine.make_desc(x.shape, w.shape, torch.float16, 2, pad, 2, stacked=None).direct == 1
        ref = F.conv2d(x[31:].double(), w.double(), stride=2, padding=pad)
        perm = torch.randperm(32, generator=g).to(dev)
        xp = xd[perm].contiguous(memory_format=torch.channels_last)
        for direct, tol in ((None, 2e-3), (True, 2e-3)):
            y = engine.conv_forward(xd, w.to(dev), None, 2, pad, 2, direct=direct)
            assert _rel(y[31:], ref) <= tol
            assert torch.equal(engine.conv_forward(xp, w.to(dev), None, 2, pad, 2, direct=direct), y[perm])


ROWS_CASES = [
    # x shape, w shape, stride, pad: kernel rows of 4 to 8 taps, which the kernel with one operand tile per kernel row takes
    ((2, 32, 15, 14), (8, 32, 7, 7), 2, 3), ((1, 96, 17, 19), (40, 96, 5, 5), 2, 2), ((2, 32, 10, 11), (8, 32, 4, 6), 2, (1, 2)),
    ((3, 64, 30, 30), (136, 64, 7, 7), 2, 3),          # two channel tiles, the second 8 wide; 675 pixels: three pixel tiles
    ((1, 32, 40, 61), (16, 32, 3, 8), 2, (1, 3)),      # rows of 8 taps, odd width
    ((2, 64, 12, 12), (16, 64, 5, 5), 1, 2), ((1, 32, 9, 23), (8, 32, 2, 4), 1, (0, 2)), ((1, 32, 14, 14), (8, 32, 7, 7), 2, 3),
    ((2, 32, 20, 20), (24, 32, 6, 6), 2, 0), ((1, 32, 6, 120), (8, 32, 1, 5), 1, (0, 2)),     # 120 output pixels per row: few, long slots
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", ROWS_CASES)
def test_one_operand_tile_per_kernel_row_is_exact_on_small_integers(dev, dtype, case, gemm_override):
    """direct_rows_kernel, forced through the test hook on shapes far below the size at which the library takes it by
    itself: bit-equal to direct convolution on small integers (bias included), to the oracle, and to the kernel with
    one operand tile per tap."""
    xs, ws, stride, pad = case
    g = torch.Generator().manual_seed(5)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = torch.randint(-2, 3, ws, generator=g).double()
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    ref = F.conv2d(x, w, b, stride=stride, padding=pad)
    assert float(ref.abs().max()) < {torch.float16: 2048, torch.bfloat16: 256}[dtype] * 8
    xd, wd, bd = x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev)
    gemm_override(-1, 2)
    y = engine.conv_forward(xd, wd, bd, stride, pad, 2, direct=True)
    gemm_override(-1, 0)
    y_tap = engine.conv_forward(xd, wd, bd, stride, pad, 2, direct=True)
    assert tuple(y.shape) == tuple(ref.shape)
    assert torch.equal(y.cpu(), ref.float().to(dtype))
    assert torch.equal(y.cpu(), ow.direct_conv(x, w, b, stride, pad, DISC[dtype]))
    assert torch.equal(y, y_tap)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", ROWS_CASES)
def test_one_operand_tile_per_kernel_row_against_fp64_and_the_oracle(dev, dtype, case, gemm_override):
    xs, ws, stride, pad = case
    g = torch.Generator().manual_seed(6)
    fan = ws[1] * ws[2] * ws[3]
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    ref = F.conv2d(x.double(), w.double(), None, stride=stride, padding=pad)
    gemm_override(-1, 2)
    y = engine.conv_forward(x.to(dev), w.to(dev), None, stride, pad, 2, direct=True)
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.2e-2}[dtype]
    assert _rel(y, ref) <= tol
    assert _rel(y, ow.direct_conv(x, w, None, stride, pad, DISC[dtype])) <= tol


def test_strided_input_gradient_through_the_kernel_row_tiles(dev, gemm_override):
    """The input gradient of a 7x7 stride-2 layer is four stride-1 direct convolutions of dy, two of them with kernel
    rows of four taps, each writing every second pixel of dx: with the kernel-row tiles forced, on small integers,
    bit-equal to the gradient autograd gives in fp64."""
    g = torch.Generator().manual_seed(7)
    x = torch.zeros(2, 40, 18, 20, dtype=torch.double, requires_grad=True)
    w = torch.randint(-2, 3, (32, 40, 7, 7), generator=g).double()
    dy = torch.randint(-2, 3, (2, 32, 9, 10), generator=g).double()
    F.conv2d(x, w, None, stride=2, padding=3).backward(dy)
    gemm_override(-1, 2)
    dx = engine.conv_backward_input(dy.half().to(dev), w.half().to(dev), (18, 20), 2, 3, 2)
    assert float(x.grad.abs().max()) < 2048
    assert torch.equal(dx.cpu().double(), x.grad)


FIRST_CASES = [
    # x shape, w shape, pad: strided first layers (at most 4 channels, stride 2, 3 / 5 / 7 kernel rows, at most 8 columns)
    ((2, 3, 32, 32), (64, 3, 7, 7), 3), ((1, 3, 45, 51), (16, 3, 7, 7), 3), ((3, 1, 20, 33), (8, 1, 3, 3), 1),
    ((2, 4, 37, 18), (72, 4, 5, 8), (2, 3)), ((2, 2, 16, 16), (136, 2, 3, 5), (0, 2)), ((5, 3, 64, 64), (64, 3, 7, 7), 3),
    ((1, 3, 7, 9), (8, 3, 7, 7), 3), ((2, 3, 33, 34), (24, 3, 5, 5), 0),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", FIRST_CASES)
def test_strided_first_layers_are_exact_on_small_integers(dev, dtype, case, host_layer):
    """first_strided_kernel (csrc/direct_first.hip), the library's own choice for these layers: bit-equal to direct
    convolution on small integers, bias included, to the oracle, from channel-last and from channel-first memory."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(8)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = torch.randint(-2, 3, ws, generator=g).double()
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    ref = F.conv2d(x, w, b, stride=2, padding=pad)
    assert float(ref.abs().max()) < {torch.float16: 2048, torch.bfloat16: 256}[dtype]
    assert engine.make_desc(xs, ws, dtype, 2, pad, 4, stacked=None).direct == 1
    xd, wd, bd = x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev)
    y = engine.conv_forward(xd, wd, bd, 2, pad, 4)
    assert tuple(y.shape) == tuple(ref.shape)
    assert torch.equal(y.cpu(), ref.float().to(dtype))
    assert torch.equal(y.cpu(), ow.direct_conv(x, w, b, 2, pad, DISC[dtype]))
    ycl = engine.conv_forward(xd.contiguous(memory_format=torch.channels_last), wd, bd, 2, pad, 4)
    assert torch.equal(ycl, y)
    U = engine.transform_filter(wd, xs, 2, pad, 4)
    assert tuple(U.shape) == (ws[0], ws[2], 8, 4)
    assert torch.equal(U[:, :, :ws[3], :ws[1]], wd.permute(0, 2, 3, 1)) and float(U[:, :, ws[3]:].abs().sum()) == 0
    assert torch.equal(engine.conv_forward(xd, wd, bd, 2, pad, 4, U=U), y)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_resnet_first_layer_against_fp64_and_through_the_module(dev, dtype):
    """N=8, 3 -> 64, 7x7, stride 2, 224x224: against fp64 convolution and the oracle on normal data; WinoConv2d keeps the
    layer in the engine in 16-bit types and hands it to torch in fp32."""
    import pytorch_winoconv_amd as pkg
    g = torch.Generator().manual_seed(9)
    x = torch.randn(8, 3, 224, 224, generator=g).to(dtype)
    w = (torch.randn(64, 3, 7, 7, generator=g) * (2.0 / 147) ** 0.5).to(dtype)
    ref = F.conv2d(x.double(), w.double(), None, stride=2, padding=3)
    y = engine.conv_forward(x.to(dev), w.to(dev), None, 2, 3, 4)
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.2e-2}[dtype]
    assert _rel(y, ref) <= tol
    assert _rel(y[:1], ow.direct_conv(x[:1], w, None, 2, 3, DISC[dtype])) <= tol
    mod = pkg.WinoConv2d(3, 64, 7, 2, 3, bias=False, dtype=dtype, device=dev)
    with torch.no_grad():
        mod.weight.copy_(w.to(dev))
    assert torch.equal(mod(x.to(dev)), y) and mod._cache is not None
    mod32 = pkg.WinoConv2d(3, 64, 7, 2, 3, bias=False, device=dev)
    assert mod32(x.float().to(dev)).dtype == torch.float32 and mod32._cache is None


def test_first_layer_module_trains(dev):
    """Gradients of a strided first layer through the module: the weight gradient against fp64 autograd."""
    import pytorch_winoconv_amd as pkg
    torch.manual_seed(10)
    mod = pkg.WinoConv2d(3, 16, 7, 2, 3, dtype=torch.float16, device=dev)
    x = torch.randn(4, 3, 40, 40, device=dev).half()
    y = mod(x)
    dy = torch.randn_like(y)
    y.backward(dy)
    w64 = mod.weight.detach().double().cpu().requires_grad_(True)
    b64 = mod.bias.detach().double().cpu().requires_grad_(True)
    F.conv2d(x.double().cpu(), w64, b64, stride=2, padding=3).backward(dy.double().cpu())
    assert _rel(mod.weight.grad, w64.grad) <= 2e-2 and _rel(mod.bias.grad, b64.grad) <= 2e-2


FIRST3D_CASES = [
    # x shape, w shape, pad: 3-D first layers (at most 4 channels, 3x3x3 at stride 1, rows of at most 4 taps)
    ((2, 3, 6, 20, 21), (64, 3, 3, 3, 3), 1), ((1, 3, 4, 33, 18), (16, 3, 3, 3, 3), (1, 0, 1)), ((1, 1, 5, 16, 16), (8, 1, 3, 3, 3), 1),
    ((2, 4, 3, 9, 35), (72, 4, 3, 3, 4), (0, 1, 2)), ((1, 2, 7, 17, 17), (136, 2, 3, 3, 2), (1, 1, 0)), ((3, 3, 8, 40, 40), (32, 3, 3, 3, 3), 1),
    ((1, 3, 3, 3, 3), (8, 3, 3, 3, 3), 1),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", FIRST3D_CASES)
def test_3d_first_layers_are_exact_on_small_integers(dev, dtype, case, host_layer):
    """first3d_kernel (csrc/direct_first3d.hip), the library's own choice for these layers: bit-equal to direct
    convolution on small integers, bias included, to the oracle, from channel-last and from channel-first memory."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(18)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = torch.randint(-2, 3, ws, generator=g).double()
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    ref = F.conv3d(x, w, b, stride=1, padding=pad)
    assert float(ref.abs().max()) < {torch.float16: 2048, torch.bfloat16: 256}[dtype]
    assert engine.make_desc(xs, ws, dtype, 1, pad, 2, stacked=None).direct == 1
    xd, wd, bd = x.to(dtype).to(dev), w.to(dtype).to(dev), b.to(dtype).to(dev)
    y = engine.conv_forward(xd, wd, bd, 1, pad, 2)
    assert tuple(y.shape) == tuple(ref.shape)
    assert torch.equal(y.cpu(), ref.float().to(dtype))
    assert torch.equal(y.cpu(), ow.direct_conv(x, w, b, 1, pad, DISC[dtype]))
    ycl = engine.conv_forward(xd.contiguous(memory_format=torch.channels_last_3d), wd, bd, 1, pad, 2)
    assert torch.equal(ycl, y)
    U = engine.transform_filter(wd, xs, 1, pad, 2)
    assert tuple(U.shape) == (ws[0], 9, 4, 4)
    assert torch.equal(U[:, :, :ws[4], :ws[1]], wd.permute(0, 2, 3, 4, 1).reshape(ws[0], 9, ws[4], ws[1]))
    assert float(U[:, :, ws[4]:].abs().sum()) == 0 and float(U[:, :, :, ws[1]:].abs().sum()) == 0
    assert torch.equal(engine.conv_forward(xd, wd, bd, 1, pad, 2, U=U), y)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_3d_first_layer_against_fp64_and_through_the_module(dev, dtype):
    """N=2, 3 -> 64, 3x3x3 on 8 x 56 x 56 clips: against fp64 convolution and the oracle on normal data, values beside the
    window that are not finite do not leak into it, and WinoConv3d keeps the layer in the engine in 16-bit types."""
    import pytorch_winoconv_amd as pkg
    g = torch.Generator().manual_seed(19)
    x = torch.randn(2, 3, 8, 56, 56, generator=g).to(dtype)
    w = (torch.randn(64, 3, 3, 3, 3, generator=g) * (2.0 / 81) ** 0.5).to(dtype)
    ref = F.conv3d(x.double(), w.double(), None, stride=1, padding=1)
    y = engine.conv_forward(x.to(dev), w.to(dev), None, 1, 1, 2)
    tol = {torch.float16: 2e-3, torch.bfloat16: 1.2e-2}[dtype]
    assert _rel(y, ref) <= tol
    assert _rel(y[:1, :, :2], ow.direct_conv(x[:1, :, :3], w, None, 1, 1, DISC[dtype])[:, :, :2]) <= tol
    # an infinity one pixel to the right of a window (the fourth, padded tap of a row) stays out of it
    xi = x.clone()
    xi[0, :, 4, 20, 30] = float("inf")
    yi = engine.conv_forward(xi.to(dev), w.to(dev), None, 1, 1, 2)
    assert torch.isfinite(yi[0, :, 4, 20, :29]).all() and torch.equal(yi[0, :, 4, 20, :29], y[0, :, 4, 20, :29])
    mod = pkg.WinoConv3d(3, 64, 3, 1, 1, bias=False, dtype=dtype, device=dev)
    with torch.no_grad():
        mod.weight.copy_(w.to(dev))
    ym = mod(x.to(dev))
    assert mod._cache is not None and torch.equal(ym, y)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_3d_first_layer_module_trains(dev, dtype):
    """Gradients of a WinoConv3d first layer (forward on first3d_kernel, gradients in the transform domain) against fp64
    autograd of the same layer."""
    import pytorch_winoconv_amd as pkg
    g = torch.Generator().manual_seed(20)
    mod = pkg.WinoConv3d(3, 16, 3, 1, 1, bias=True, dtype=dtype, device=dev)
    x = torch.randn(2, 3, 6, 20, 22, generator=g).to(dtype).to(dev).requires_grad_(True)
    y = mod(x)
    dy = torch.randn(y.shape, generator=g).to(dtype).to(dev)
    y.backward(dy)
    xr = x.detach().double().requires_grad_(True)
    wr = mod.weight.detach().double().requires_grad_(True)
    br = mod.bias.detach().double().requires_grad_(True)
    F.conv3d(xr, wr, br, 1, 1).backward(dy.double())
    tol = {torch.float16: 4e-3, torch.bfloat16: 3e-2}[dtype]
    assert mod._cache is not None
    assert _rel(mod.weight.grad.detach(), wr.grad) <= tol and _rel(mod.bias.grad.detach(), br.grad) <= tol
    assert _rel(x.grad.detach(), xr.grad) <= tol
