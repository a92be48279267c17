"""The compiled host layer: the pybind11 module MakePytorchBackend (csrc/host/make_pytorch_backend.cpp), which
stands in for the reference's extension of that name (pybind/bind.cpp:10-24, pybind/extern.hpp:3-9).  Every
function it exports is called here and checked against the oracle (tile copies: bit-exact; convolutions:
fp64 torch convolution and the CPU restatement of the reference algorithm), and against the ctypes binding
of the same C ABI, which must give the same bits."""
import threading

import numpy as np
import pytest
import torch
import torch.nn.functional as F

import pytorch_winoconv_amd as pkg
from pytorch_winoconv_amd import backend, engine
from oracle import tiles as ot
from oracle import winograd as ow

pytestmark = pytest.mark.gpu

ext = pytest.importorskip("pytorch_winoconv_amd.MakePytorchBackend")


def _nerr(y, ref):
    return float((y.double().cpu() - ref.double()).abs().max() / ref.double().abs().max())


def test_package_names_come_from_the_compiled_module():
    for name in ("Foo", "AddGPU", "WinoSplit", "WinoConcat", "DWM", "winograd_conv", "split_and_concat"):
        assert getattr(pkg, name) is getattr(ext, name)
    assert "gfx950" in ext.version()


def test_foo_and_add(dev):
    f = ext.Foo()
    f.setKey(7)
    assert f.getKey() == 7 and repr(f) == "< Foo, key: 7 > "          # src/foo.cpp
    a, b = torch.randn(5, 3, device=dev), torch.randn(15, device=dev)
    c = torch.empty(0, device=dev)
    ext.AddGPU(a, b, c)
    assert torch.equal(c, a + b.view(5, 3))
    with pytest.raises(ValueError):
        ext.AddGPU(a, b[:3], c)                                         # src/add.cpp:14-17


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("xs,ws,m", [((2, 24, 11, 14), (8, 24, 3, 3), 2), ((1, 7, 9, 9), (4, 7, 3, 3), 4),
                                     ((2, 9, 6, 9, 8), (4, 9, 3, 3, 3), 2)])
def test_split_and_concat_bit_exact(dev, dtype, xs, ws, m):
    g = torch.Generator().manual_seed(1)
    x = torch.randn(*xs, generator=g).to(dtype)
    want = torch.from_numpy(ot.wino_split(x.numpy(), ws, m))
    nd = len(xs) - 2
    blocks = [w + m - 1 for w in ws[2:]]
    n = ot.tile_counts(xs[2:], ws[2:], m)
    x_cl = engine.channel_last(x.to(dev))
    tiles = torch.zeros(want.shape, dtype=dtype, device=dev)
    b3, n3 = [1] * (3 - nd) + blocks, [1] * (3 - nd) + n
    ext.WinoSplit(x_cl, tiles, b3[0], b3[1], b3[2], m, n3[0], n3[1], n3[2], nd == 2)
    assert torch.equal(tiles.cpu(), want)
    tiles2 = torch.zeros_like(tiles)
    ext.split_and_concat("split", x_cl, tiles2, b3[0], b3[1], b3[2], m, n3[0], n3[1], n3[2], nd == 2)
    assert torch.equal(tiles2, tiles)
    # concat: tiles of the output block size back to an image, odd edges cropped
    osz = [2 * v - 1 for v in n]
    K = 5
    t = torch.randn([xs[0] * int(np.prod(n)), K] + [2] * nd, generator=g).to(dtype)
    want_y = torch.from_numpy(ot.wino_concat(t.numpy(), osz, 2))
    y = torch.zeros([xs[0]] + osz + [K], dtype=dtype, device=dev)
    ext.WinoConcat(t.to(dev), y, 2, nd == 2)
    perm = (0, nd + 1) + tuple(range(1, nd + 1))
    assert torch.equal(y.permute(perm).cpu(), want_y)
    y2 = torch.zeros_like(y)
    ext.split_and_concat("concat", t.to(dev), y2, 2, nd == 2)
    assert torch.equal(y2, y)
    # the ctypes binding of the same C ABI gives the same bits
    tiles3 = torch.zeros_like(tiles)
    backend.WinoSplit(x_cl, tiles3, b3[0], b3[1], b3[2], m, n3[0], n3[1], n3[2], nd == 2)
    assert torch.equal(tiles3, tiles)


@pytest.mark.parametrize("ks,stride", [((1, 3, 3), 1), ((1, 7, 7), 1), ((3, 3, 3), 1), ((1, 5, 4), 2), ((2, 5, 3), 1)])
def test_dwm_is_a_valid_convolution(dev, ks, stride):
    """DWM(Input, Weight, Output, stride, four scratch tensors): the reference's native entry point
    (src/winograd_conv.cpp:17-127), VALID padding, fp32, channel-last tensors, Weight (kD, kH, kW, C, K)."""
    g = torch.Generator().manual_seed(2)
    C, K = 12, 10
    sp = (1 if ks[0] == 1 else 7, 13, 12)
    x = torch.randn(2, C, *sp, generator=g)
    w = torch.randn(K, C, *ks, generator=g) * (2.0 / (C * ks[0] * ks[1] * ks[2])) ** 0.5
    ref = F.conv3d(x.double(), w.double(), stride=stride)
    Input = x.permute(0, 2, 3, 4, 1).contiguous().to(dev)
    Weight = w.permute(2, 3, 4, 1, 0).contiguous().to(dev)
    Output = torch.zeros(tuple(ref.permute(0, 2, 3, 4, 1).shape), device=dev)
    scratch = [torch.zeros(4, device=dev) for _ in range(3)] + [torch.zeros(4, dtype=torch.int64, device=dev)]
    ext.DWM(Input, Weight, Output, stride, *scratch)                    # dwm.py:135-136 call shape
    y = Output.permute(0, 4, 1, 2, 3)
    assert _nerr(y, ref) <= 1e-3
    two_d = ks[0] == 1
    xo, wo = (x[:, :, 0], w[:, :, 0]) if two_d else (x, w)
    want = ow.dwm_conv(xo, wo, None, stride, 0, 2, "fp32", stacked=engine._stack(None, torch.float32, 2 if two_d else 3, False,
                                                                                   tuple(wo.shape), stride, 2))
    want = want.unsqueeze(2) if two_d else want
    assert _nerr(y, want) <= 1e-5
    Out2 = torch.zeros_like(Output)
    backend.DWM(Input, Weight, Out2, stride, *scratch)
    assert torch.equal(Out2, Output)


@pytest.mark.parametrize("dtype,tol", [(torch.float32, 1e-3), (torch.float16, 2e-2), (torch.bfloat16, 2e-2)])
def test_winograd_conv_and_conv_forward(dev, dtype, tol):
    g = torch.Generator().manual_seed(3)
    x = torch.randn(3, 20, 15, 14, generator=g).to(dtype)
    for ws, stride, pad, m in (((24, 20, 3, 3), 1, 1, 2), ((24, 20, 3, 3), 1, 1, 4), ((24, 20, 5, 5), 1, 2, 2), ((24, 20, 7, 7), 2, 3, 2)):
        if dtype == torch.bfloat16 and m == 4:
            continue
        w = (torch.randn(*ws, generator=g) * (2.0 / (ws[1] * ws[2] * ws[3])) ** 0.5).to(dtype)
        b = torch.randn(ws[0], generator=g).to(dtype)
        ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
        y = ext.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m)
        assert tuple(y.shape) == tuple(ref.shape) and y.permute(0, 2, 3, 1).is_contiguous()
        assert _nerr(y, ref) <= tol
        disc = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}[dtype]
        form = engine._stack(None, dtype, 2, False, ws, stride, m)
        assert _nerr(y, ow.dwm_conv(x, w, b, stride, pad, m, disc, stacked=form)) <= tol
        # the ctypes path, and the channel-last entry point of both bindings: same bits
        engine_y = _ctypes_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m)
        assert torch.equal(engine_y, y)
        Input = x.to(dev).permute(0, 2, 3, 1).unsqueeze(1).contiguous()
        Weight = w.to(dev).permute(2, 3, 1, 0).unsqueeze(0)             # (kD, kH, kW, C, K) view, not contiguous
        Out = torch.zeros(tuple(y.permute(0, 2, 3, 1).unsqueeze(1).shape), dtype=dtype, device=dev)
        used = ext.winograd_conv(Input, Weight, Out, b.to(dev), stride, pad, m)
        assert torch.equal(Out[:, 0], y.permute(0, 2, 3, 1))
        assert used in (2, 3, 4) and (used == m or (m == 4 and max(ws[2:]) > 3))
        # a cached transformed filter
        U = engine.transform_filter(w.to(dev), x.shape, stride, pad, m)
        assert torch.equal(ext.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m, U), y)


def _ctypes_forward(*args, **kw):
    old = engine.USE_EXT
    engine.USE_EXT = False
    try:
        return engine.conv_forward(*args, **kw)
    finally:
        engine.USE_EXT = old


def test_errors_are_python_exceptions(dev):
    x = torch.randn(1, 4, 8, 8, device=dev)
    w = torch.randn(6, 4, 3, 3, device=dev)
    with pytest.raises(NotImplementedError):
        ext.conv_forward(x, w, None, 3, 1, 2)                          # stride 3
    with pytest.raises(NotImplementedError):
        ext.conv_forward(x, torch.randn(6, 4, 11, 3, device=dev), None, 1, 5, 2)
    with pytest.raises(ValueError):
        ext.conv_forward(x, w, torch.randn(5, device=dev))
    with pytest.raises(TypeError):
        ext.conv_forward(x, w.half())
    with pytest.raises(ValueError):
        ext.conv_forward(x.cpu(), w)
    Out = torch.zeros(1, 1, 5, 6, 6, device=dev)                        # wrong output shape
    with pytest.raises(ValueError, match="output must be"):
        ext.winograd_conv(x.permute(0, 2, 3, 1).unsqueeze(1).contiguous(), w.permute(2, 3, 1, 0).unsqueeze(0), Out)
    assert ext.conv_forward(x[:0], w, None, 1, 1, 2).shape == (0, 6, 8, 8)


def test_calls_release_the_gil_and_follow_the_current_stream(dev):
    """Two host threads, each on its own stream, call the compiled layer at the same time; each result equals
    the single-threaded one (the library is re-entrant and stream-ordered; the GIL is released around launches)."""
    g = torch.Generator().manual_seed(4)
    x = torch.randn(4, 32, 24, 24, generator=g).half().to(dev)
    w = (torch.randn(32, 32, 3, 3, generator=g) * 0.08).half().to(dev)
    want = ext.conv_forward(x, w, None, 1, 1, 4)
    torch.cuda.synchronize()
    got, errs = {}, []

    def work(i):
        try:
            s = torch.cuda.Stream()
            with torch.cuda.stream(s):
                for _ in range(20):
                    y = ext.conv_forward(x, w, None, 1, 1, 4)
                s.synchronize()
            got[i] = y
        except Exception as e:                                          # pragma: no cover
            errs.append(e)

    ts = [threading.Thread(target=work, args=(i,)) for i in range(2)]
    for t in ts:
        t.start()
    for t in ts:
        t.join()
    assert not errs and all(torch.equal(got[i], want) for i in range(2))
