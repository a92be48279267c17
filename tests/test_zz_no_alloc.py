"""wc_conv_forward_static: the entry point that allocates nothing (its U, V and M live in a buffer inside
the library's device image) must give, bit for bit, what wc_conv_forward gives with a workspace from
the caller - on calls in a row that share the buffer, later ones with smaller inputs that leave the
earlier call's contents in most of it."""
import ctypes

import pytest
import torch
import torch.nn.functional as F

from pytorch_winoconv_amd import _lib, engine

pytestmark = pytest.mark.gpu

H16, F32 = torch.float16, torch.float32
CALLS = [
    # x shape, w shape, stride, pad, m, dtype, stacked
    ((48, 256, 28, 28), (256, 256, 3, 3), 1, 1, 4, H16, False),   # 87 MB of V + M: several chunks of images
    ((3, 40, 13, 11), (24, 40, 5, 5), 1, 2, 2, H16, 2),           # smaller; pieces share one V whose tail rows are stale
    ((2, 24, 9, 10), (16, 24, 3, 3), 1, 1, 2, F32, False),        # fp32, three kernels
    ((5, 64, 12, 12), (64, 64, 3, 3), 1, 1, 2, H16, False),       # thin layer: one fused kernel, only U in the buffer
    ((2, 16, 6, 10, 9), (8, 16, 3, 3, 3), 1, 1, 2, H16, False),   # 3-D
    ((2, 32, 21, 20), (16, 32, 7, 7), 2, 3, 2, H16, True),        # stride 2, stacked pieces
    ((4, 64, 21, 20), (32, 64, 3, 3), 2, 1, 2, H16, None),        # stride 2, the library's choice: the direct form, only U in the buffer
    ((3, 32, 10, 11), (16, 32, 1, 1), 1, 0, 2, F32, None),        # one tap, fp32: the direct form
]


def _both(dev, case, seed):
    xs, ws, stride, pad, m, dtype, stacked = case
    lib = _lib.load()
    g = torch.Generator().manual_seed(seed)
    fan = 1
    for v in ws[1:]:
        fan *= v
    x = torch.randn(*xs, generator=g).to(dtype).to(dev)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype).to(dev)
    b = torch.randn(ws[0], generator=g).to(dtype).to(dev)
    desc = engine.make_desc(xs, ws, dtype, stride, pad, m, 0, False, stacked)
    out, _ = engine.out_dims(desc)
    osp = out[1:] if desc.ndim == 2 else out
    x_cl = engine.channel_last(x)
    y_static = torch.full([xs[0]] + osp + [ws[0]], float("nan"), dtype=dtype, device=dev)
    _lib.check(lib.wc_conv_forward_static(ctypes.byref(desc), engine._ptr(x_cl), engine._ptr(w), engine._w_strides(w),
                                          None, engine._ptr(b), engine._ptr(y_static), engine._stream(x)))
    y = engine.channel_last(engine.conv_forward(x, w, b, stride, pad, m, stacked=stacked))
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    ref = engine.channel_last(conv(x.double(), w.double(), b.double(), stride=stride, padding=pad))
    return y_static, y, ref


def test_static_scratch_calls_in_a_row_equal_the_workspace_entry_point(dev):
    for rnd in range(2):                       # the second round starts from a buffer every case has written to
        for i, case in enumerate(CALLS):
            y_static, y, ref = _both(dev, case, 100 * rnd + i)
            assert tuple(y_static.shape) == tuple(y.shape)
            assert torch.equal(y_static, y), (rnd, case)
            tol = 1e-3 if case[5] == F32 else 2e-2
            assert float((y_static.double() - ref).abs().max() / ref.abs().max()) <= tol, (rnd, case)


def test_static_scratch_refuses_what_does_not_fit(dev):
    """One image of this layer needs 36 x 3136 x (256 + 256) x 2 B = 116 MB of V and M: more than the
    64 MiB buffer, so the call returns an error before it launches anything."""
    lib = _lib.load()
    desc = engine.make_desc((1, 256, 224, 224), (256, 256, 3, 3), H16, 1, 1, 4)
    x = torch.zeros(8, dtype=H16, device=dev)
    rc = lib.wc_conv_forward_static(ctypes.byref(desc), engine._ptr(x), engine._ptr(x), engine._w_strides(x.view(1, 1, 1, 8)),
                                    None, None, engine._ptr(x), engine._stream(x))
    assert rc == _lib.WC_ERR_WORKSPACE
    assert b"static buffer" in lib.wc_last_error()
