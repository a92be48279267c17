"""Gradients of the convolution (the reference has no backward pass: src/back/utils.cu:15-24 is a
pointer-assign helper, include/split_functions_grad.h:3-6 is empty).  The oracle is what the
mathematics fixes: torch autograd through fp64 convolution of the same rounded inputs.
Bounds, as for the forward pass, in units of max |reference gradient|: fp32 1e-3, fp16 2e-2,
bf16 2e-2 with output tile 2 and 2e-1 with tile 4."""
import pytest
import torch
import torch.nn.functional as F

import pytorch_winoconv_amd as pkg
from pytorch_winoconv_amd import engine

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, w shape, stride, pad, m
    ((2, 8, 12, 13), (6, 8, 3, 3), 1, 1, 2),
    ((2, 8, 12, 13), (6, 8, 3, 3), 1, 1, 4),
    ((3, 16, 20, 20), (24, 16, 5, 5), 1, 2, 4),          # DWM pieces
    ((2, 8, 15, 14), (4, 8, 7, 7), 2, 3, 2),              # stride 2, odd remainder on one axis
    ((2, 8, 15, 14), (4, 8, 3, 3), 2, 1, 4),
    ((2, 5, 9, 11), (7, 5, 4, 3), 1, (1, 0), 2),          # non-square kernel, odd channel counts
    ((1, 6, 6, 9, 8), (8, 6, 3, 3, 3), 1, 1, 2),          # 3-D
    ((1, 6, 6, 9, 8), (8, 6, 3, 3, 3), 1, 1, 4),          # 3-D tile 2 x 4 x 4
    ((1, 4, 5, 7, 7), (4, 4, 2, 3, 1), 1, 0, 2),
    ((4, 64, 28, 28), (64, 64, 3, 3), 1, 1, 4),
    ((1, 3, 9, 9), (2, 3, 1, 1), 1, 0, 2),                # 1 x 1 kernel
    ((3, 32, 17, 19), (40, 32, 1, 1), 1, 0, 2),           # 1 x 1, whole vectors of channels: dw = dy^T x, no transforms
    ((9, 96, 28, 28), (136, 96, 1, 1), 1, 0, 4),          # the same with 128 x 128 product tiles and several parts
    ((2, 32, 10, 10), (8, 32, 1, 1), 2, 0, 2),            # 1 x 1 at stride 2: the same
    # stride 2 with the channel counts the library's own input gradient takes (one direct-form launch per parity class)
    ((2, 8, 15, 14), (32, 8, 3, 3), 2, 1, 2),
    ((3, 16, 21, 20), (64, 16, 7, 7), 2, 3, 2),
    ((2, 24, 12, 13), (32, 24, 1, 1), 2, 0, 2),           # one tap: three of the four classes are zero
    ((2, 8, 13, 16), (32, 8, 4, 2), 2, (1, 0), 2),
    ((2, 8, 10, 11), (32, 8, 2, 2), 2, 1, 2),             # padding that moves a class beyond the first row of dy
    ((2, 8, 9, 9), (32, 8, 3, 3), 2, 2, 2),
    ((4, 64, 56, 56), (64, 64, 3, 3), 2, 1, 4),
    ((6, 24, 40, 40), (40, 24, 3, 3), 1, 1, 2),           # tile sum split into 9 parts, the last one short
    ((8, 72, 40, 40), (136, 72, 3, 3), 1, 1, 4),          # 128 x 128 product tiles with partial edges, 3 parts
]
TOL = {torch.float32: (1e-3, 1e-3), torch.float16: (2e-2, 2e-2), torch.bfloat16: (2e-2, 2e-1)}


def _reference(x, w, dy, stride, pad):
    conv = F.conv2d if x.dim() == 4 else F.conv3d
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    y = conv(xr, wr, stride=stride, padding=pad)
    return torch.autograd.grad(y, (xr, wr), dy.double())


def _rel(a, b):
    return float((a.double().cpu() - b).abs().max() / b.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_gradients_against_fp64_autograd(dev, dtype, case):
    xs, ws, stride, pad, m = case
    g = torch.Generator().manual_seed(17)
    fan = ws[1]
    for v in ws[2:]:
        fan *= v
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    y_shape = (F.conv2d if len(xs) == 4 else F.conv3d)(x.float(), w.float(), stride=stride, padding=pad).shape
    dy = torch.randn(*y_shape, generator=g).to(dtype)
    gx, gw = _reference(x, w, dy, stride, pad)
    tol = TOL[dtype][0 if m == 2 else 1]
    dw = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, stride, pad, m)
    assert dw.dtype == dtype and tuple(dw.shape) == tuple(ws) and _rel(dw, gw) <= tol
    dx = engine.conv_backward_input(dy.to(dev), w.to(dev), xs[2:], stride, pad, m)
    assert dx.dtype == dtype and tuple(dx.shape) == tuple(xs) and _rel(dx, gx) <= tol


@pytest.mark.parametrize("k", [4, 5, 7])
def test_weight_gradient_through_a_whole_kernel_tile(dev, k):
    """One F(2,k) x F(2,k) tile instead of DWM pieces: the generic gradient kernels.  fp32; the
    bound grows with k as the forward error of these tiles does (1e-3 is the fp32 bound up to
    k = 5; F(2,7) loses another decimal digit)."""
    g = torch.Generator().manual_seed(5)
    xs, ws = (2, 6, 15, 14), (5, 6, k, k)
    x = torch.randn(*xs, generator=g)
    w = torch.randn(*ws, generator=g) * (2.0 / (6 * k * k)) ** 0.5
    dy = torch.randn(*F.conv2d(x, w, padding=k // 2).shape, generator=g)
    _, gw = _reference(x, w, dy, 1, k // 2)
    dw = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, 1, k // 2, 2, whole_kernel=True)
    assert _rel(dw, gw) <= (1e-3 if k <= 5 else 1e-2)
    ref = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, 1, k // 2, 2)
    assert _rel(ref, gw) <= 1e-3


def test_input_gradient_of_few_output_channels_uses_tile_2(dev):
    """With fewer than 8 output channels the sum behind each input-gradient element is too short to
    average the F(4,r) rounding error down (fp16, K = 1: up to 3e-2 of the range), so the engine
    computes it with tile 2 whatever tile the forward pass uses: 2e-3 here."""
    for seed in range(4):
        g = torch.Generator().manual_seed(seed)
        x = torch.randn(1, 32, 19, 9, generator=g).half()
        w = (torch.randn(1, 32, 5, 3, generator=g) * (2.0 / (32 * 15)) ** 0.5).half()
        dy = torch.randn(1, 1, 23, 9, generator=g).half()
        gx, _ = _reference(x, w, dy, 1, (4, 1))
        dx = engine.conv_backward_input(dy.to(dev), w.to(dev), (19, 9), 1, (4, 1), 4)
        assert _rel(dx, gx) <= 2e-3
        assert torch.equal(dx, engine.conv_backward_input(dy.to(dev), w.to(dev), (19, 9), 1, (4, 1), 2))


def test_weight_gradient_is_independent_of_the_image_chunking(dev):
    """The sum over tiles is split into parts and image chunks and added up in fp32: any chunking
    gives the same gradient up to fp32 summation order."""
    import ctypes
    from pytorch_winoconv_amd import _lib
    lib = _lib.load()
    g = torch.Generator().manual_seed(3)
    xs, ws = (5, 16, 58, 57), (24, 16, 3, 3)   # 225 tiles per image: passes of 4 images split their sum
    x = torch.randn(*xs, generator=g).to(dev).contiguous(memory_format=torch.channels_last)
    dy = torch.randn(5, 24, 58, 57, generator=g).to(dev).contiguous(memory_format=torch.channels_last)
    ref = engine.conv_backward_weight(x, dy, ws, 1, 1, 4)
    for chunk in (1, 2, 4):
        desc = engine.make_desc(xs, ws, torch.float32, 1, 1, 4, chunk)
        nbytes = ctypes.c_size_t()
        _lib.check(lib.wc_conv_backward_weight_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
        wsp = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
        dw = torch.full(ws, float("nan"), device=dev)
        _lib.check(lib.wc_conv_backward_weight(ctypes.byref(desc), engine.channel_last(x).data_ptr(),
                                               engine.channel_last(dy).data_ptr(), dw.data_ptr(), engine._w_strides(dw),
                                               wsp.data_ptr(), nbytes.value, engine._stream(x)))
        assert _rel(dw, ref.double().cpu()) <= 1e-5, chunk
    # too small a workspace is refused
    assert lib.wc_conv_backward_weight(ctypes.byref(desc), x.data_ptr(), dy.data_ptr(), dw.data_ptr(),
                                       engine._w_strides(dw), wsp.data_ptr(), 1024, engine._stream(x)) == _lib.WC_ERR_WORKSPACE


@pytest.mark.parametrize("k,stride,pad", [(3, 1, 1), (5, 1, 2), (3, 2, 1)])
def test_module_trains(dev, k, stride, pad):
    """loss.backward() through WinoConv2d gives the gradients of the same layer built on F.conv2d."""
    torch.manual_seed(0)
    mod = pkg.WinoConv2d(8, 12, k, stride, pad, device=dev)
    x = torch.randn(3, 8, 17, 16, device=dev, requires_grad=True)
    y = mod(x)
    target = torch.randn_like(y)
    ((y - target) ** 2).sum().backward()
    x2 = x.detach().double().cpu().requires_grad_(True)
    w2 = mod.weight.detach().double().cpu().requires_grad_(True)
    b2 = mod.bias.detach().double().cpu().requires_grad_(True)
    y2 = F.conv2d(x2, w2, b2, stride=stride, padding=pad)
    ((y2 - target.double().cpu()) ** 2).sum().backward()
    assert _rel(x.grad, x2.grad) <= 1e-3
    assert _rel(mod.weight.grad, w2.grad) <= 1e-3
    assert _rel(mod.bias.grad, b2.grad) <= 1e-3
    # no graph, no gradient bookkeeping
    with torch.no_grad():
        assert not mod(x).requires_grad
