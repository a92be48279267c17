"""Channel-first (NCHW / NCDHW contiguous) tensors, the layout torch tensors have by default, on either side of
the path (wc_conv_desc.x_layout / y_layout).  The reference permutes to channel-last and back with torch passes of
its own (dwm.py:129-133,143-144; Split_and_Concat.py:25,47,64,81); here single-piece 2-D plans read channel-first x
inside the input transform, and every other plan goes through the library's own copy kernel (wc_layout_copy).

Every check is against the oracle or fp64 torch convolution on the same values, and - because a change of layout
must not change a single bit - against the channel-last path of the same engine."""
import ctypes

import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import _lib, engine

pytestmark = pytest.mark.gpu

DISC = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}


def _rel(a, b):
    return float((a.double().cpu() - b.double().cpu()).abs().max() / b.double().abs().max())


@pytest.mark.parametrize("es", [2, 4])
@pytest.mark.parametrize("shape", [(2, 5, 7, 9), (1, 64, 64, 64), (3, 70, 1, 130), (2, 3, 4, 5, 6), (1, 129, 65, 3)])
def test_layout_copy_is_a_bit_exact_permute(dev, es, shape):
    lib = _lib.load()
    dtype = torch.float16 if es == 2 else torch.float32
    x = torch.randn(*shape, generator=torch.Generator().manual_seed(0)).to(dtype).to(dev)
    n, c = shape[:2]
    s = x[0, 0].numel()
    nd = len(shape) - 2
    to_cl = (0,) + tuple(range(2, 2 + nd)) + (1,)
    out = torch.full(tuple(x.permute(to_cl).shape), float("nan"), dtype=dtype, device=dev)
    _lib.check(lib.wc_layout_copy(engine._ptr(x), engine._ptr(out), n, c, s, 1, es, engine._stream(x)))
    assert torch.equal(out, x.permute(to_cl))
    back = torch.full(tuple(shape), float("nan"), dtype=dtype, device=dev)
    _lib.check(lib.wc_layout_copy(engine._ptr(out), engine._ptr(back), n, c, s, 0, es, engine._stream(x)))
    assert torch.equal(back, x)


# single-piece 2-D plans at stride 1: every tile pair the kernel is built for, even and odd widths (4-byte and
# 2-byte loads), channel counts that are no multiple of the block, tile rows cut into blocks (wide image)
DIRECT = [
    # x shape, w shape, pad, m   (images at least 16 columns wide: narrower ones take the copy, see below)
    ((2, 8, 9, 19), (12, 8, 3, 3), 1, 2), ((2, 8, 9, 20), (12, 8, 3, 3), 1, 4), ((1, 3, 10, 18), (5, 3, 3, 3), 0, 2),
    ((2, 70, 13, 22), (4, 70, 3, 3), 1, 4), ((1, 33, 7, 17), (4, 33, 3, 3), 1, 4), ((1, 5, 6, 200), (4, 5, 3, 3), 1, 2),
    ((1, 5, 9, 131), (4, 5, 3, 3), 1, 4), ((2, 6, 8, 24), (4, 6, 1, 1), 0, 2), ((2, 6, 8, 16), (4, 6, 2, 3), (1, 0), 2),
    ((2, 6, 8, 18), (4, 6, 3, 1), (0, 1), 4), ((1, 6, 11, 18), (4, 6, 2, 2), 1, 4), ((1, 6, 11, 26), (4, 6, 1, 2), 0, 4),
    ((1, 6, 11, 32), (4, 6, 3, 2), 2, 2), ((1, 6, 11, 17), (4, 6, 2, 1), 0, 4), ((1, 6, 11, 40), (4, 6, 1, 3), 1, 2),
    ((2, 40, 9, 56), (4, 40, 3, 3), 1, 4), ((1, 20, 5, 64), (4, 20, 3, 3), 1, 2),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", DIRECT)
def test_input_transform_reads_channel_first_memory(dev, dtype, case):
    xs, ws, pad, m = case
    g = torch.Generator().manual_seed(1)
    x = torch.randn(*xs, generator=g).to(dtype)
    w = torch.randn(*ws, generator=g).to(dtype)
    stages = {}
    ow.dwm_conv(x, w, None, 1, pad, m, DISC[dtype], stages)
    d_cf = engine.make_desc(xs, ws, dtype, 1, pad, m, x_layout=1)
    d_cl = engine.make_desc(xs, ws, dtype, 1, pad, m)
    plan = engine.plan_conv(d_cf)
    assert plan.n_pieces == 1
    xd = x.to(dev)
    V = engine.input_transform(d_cf, plan, xd)                          # NCHW memory as it is
    V_cl = engine.input_transform(d_cl, plan, engine.channel_last(xd))
    assert torch.equal(V, V_cl)
    C = xs[1]
    assert torch.count_nonzero(V[:, :, C:]) == 0
    tol = {torch.float32: 2e-6, torch.float16: 1.5e-3, torch.bfloat16: 1.2e-2}[dtype]
    assert _rel(V[:, :, :C], stages["V"]) <= tol
    # a view that starts 2 bytes into an allocation: the 4-byte loads of the even-width form do not apply
    if dtype != torch.float32:
        buf = torch.zeros(x.numel() + 1, dtype=dtype, device=dev)
        view = buf[1:].view(xs)
        view.copy_(xd)
        assert view.data_ptr() % 4 == 2
        assert torch.equal(engine.input_transform(d_cf, plan, view), V_cl)


def test_stage_refuses_channel_first_memory_for_other_plans(dev):
    """DWM plans, and images narrower than 16 columns (the copy and the channel-last kernel are faster there)."""
    for xs, ws, pad in (((1, 8, 12, 20), (8, 8, 5, 5), 2), ((1, 8, 12, 12), (8, 8, 3, 3), 1)):
        d = engine.make_desc(xs, ws, torch.float16, 1, pad, 2, x_layout=1)
        x = torch.zeros(*xs, dtype=torch.float16, device=dev)
        with pytest.raises(NotImplementedError, match="wc_layout_copy"):
            engine.input_transform(d, engine.plan_conv(d), x)


FORWARD = [
    # x shape, w shape, stride, pad, m: single piece (read directly), DWM pieces, stride 2, thin layers, 3-D
    ((3, 20, 15, 24), (24, 20, 3, 3), 1, 1, 4), ((3, 20, 15, 13), (24, 20, 3, 3), 1, 1, 2), ((2, 20, 15, 14), (24, 20, 5, 5), 1, 2, 2),
    ((2, 36, 9, 33), (24, 36, 3, 3), 1, 1, 2),
    ((2, 20, 15, 14), (24, 20, 7, 7), 1, 3, 4), ((2, 20, 21, 20), (24, 20, 7, 7), 2, 3, 2), ((2, 20, 15, 14), (24, 20, 3, 3), 2, 1, 2),
    ((2, 64, 12, 12), (64, 64, 3, 3), 1, 1, 2), ((2, 3, 20, 20), (16, 3, 3, 3), 1, 1, 2), ((2, 12, 6, 9, 10), (8, 12, 3, 3, 3), 1, 1, 2),
    ((1, 12, 6, 9, 10), (8, 12, 5, 4, 3), 1, 1, 2),
]


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.float16, 2e-2)])
@pytest.mark.parametrize("case", FORWARD)
def test_forward_with_channel_first_tensors(dev, dtype, tol, case, host_layer):
    xs, ws, stride, pad, m = case
    g = torch.Generator().manual_seed(2)
    fan = 1
    for v in ws[1:]:
        fan *= v
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    ref = conv(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    assert xd.is_contiguous()
    y = engine.conv_forward(xd, wd, bd, stride, pad, m)                                # channel-first in, channel-last out
    assert tuple(y.shape) == tuple(ref.shape) and _rel(y, ref) <= tol
    nd = len(xs) - 2
    fmt = torch.channels_last if nd == 2 else torch.channels_last_3d
    y_cl = engine.conv_forward(xd.contiguous(memory_format=fmt), wd, bd, stride, pad, m)
    assert torch.equal(y, y_cl)                                                         # the layout changes no bit
    y_cf = engine.conv_forward(xd, wd, bd, stride, pad, m, channels_first_out=True)    # channel-first out
    assert y_cf.is_contiguous() and torch.equal(y_cf, y)
    y_cf2 = engine.conv_forward(xd.contiguous(memory_format=fmt), wd, bd, stride, pad, m, channels_first_out=True)
    assert y_cf2.is_contiguous() and torch.equal(y_cf2, y)
    # the batch in chunks of one image: each chunk has its own scratch copies
    assert torch.equal(engine.conv_forward(xd, wd, bd, stride, pad, m, chunk_images=1, channels_first_out=True), y)
    form = engine._stack(None, dtype, nd, False, ws, stride, m)
    used = engine.make_desc(xs, ws, dtype, stride, pad, m, stacked=form).m     # tile 4 may have become 3 or 2
    om = (2, 4, 4) if (used == 4 and nd == 3) else used
    want = ow.dwm_conv(x, w, b, stride, pad, om, DISC[dtype], stacked=form)
    assert _rel(y, want) <= tol
