"""The reference-shaped Python API (dwm, matrix_conv, matrix_conv3d, backend, modules) on the GPU,
checked against fp64 torch convolution and the oracle.  Tolerances as in test_gpu_conv.py."""
import pytest
import torch
import torch.nn.functional as F

import pytorch_winoconv_amd as pkg
from pytorch_winoconv_amd import engine
from oracle import winograd as ow

pytestmark = pytest.mark.gpu


def _nerr(y, ref):
    return float((y.double().cpu() - ref).abs().max() / ref.abs().max())


def _mk(xs, ws, seed=0):
    g = torch.Generator().manual_seed(seed)
    fan = 1
    for v in ws[1:]:
        fan *= v
    return (torch.randn(*xs, generator=g), torch.randn(*ws, generator=g) * (2.0 / fan) ** .5,
            torch.randn(ws[0], generator=g))


def test_dwm2d_matches_the_reference_demo(dev):
    """example.py:99-109: x (1,224,10,10) U(0,1), w (32,224,7,7); mean relative error vs fp64."""
    g = torch.Generator().manual_seed(0)
    x, w = torch.rand(1, 224, 10, 10, generator=g), torch.rand(32, 224, 7, 7, generator=g)
    ref = F.conv2d(x.double(), w.double())
    y = pkg.dwm.dwm2d(x.to(dev), w.to(dev), None, (1, 1))
    assert y.shape == ref.shape
    assert float(((y.double().cpu() - ref) / ref).abs().mean()) < 1e-6
    y16 = pkg.matrix_conv.conv16(x.to(dev), w.to(dev), None, (1, 1))
    assert y16.dtype == torch.float32                                     # matrix_conv.py:89
    ref16 = F.conv2d(x.half().double(), w.half().double())
    assert float(((y16.double().cpu() - ref16) / ref16).abs().mean()) < 5e-3


def test_dwm3d_and_module(dev):
    x, w, b = _mk((1, 32, 10, 10, 10), (32, 32, 3, 3, 3))                 # example.py:111-113
    ref = F.conv3d(x.double(), w.double(), b.double())
    y = pkg.dwm.dwm3d(x.to(dev), w.to(dev), b.to(dev), (1, 1, 1))
    assert _nerr(y, ref) < 1e-3
    y2 = pkg.Dwm().forward(x.to(dev), w.to(dev))                          # network.py:33-35
    assert _nerr(y2, F.conv3d(x.double(), w.double())) < 1e-3
    assert _nerr(pkg.dwm.dwm3d_(x.to(dev), w.to(dev)), F.conv3d(x.double(), w.double())) < 1e-3


@pytest.mark.parametrize("pad", [(1, 2), 2, 0])
def test_dwm2d_padding_bias_stride(dev, pad):
    x, w, b = _mk((2, 16, 21, 20), (24, 16, 5, 5))
    for stride in (1, 2):
        ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
        y = pkg.dwm.dwm2d(x.to(dev), w.to(dev), b.to(dev), (stride, stride), pad)
        assert y.shape == ref.shape and _nerr(y, ref) < 1e-3
    y4 = pkg.dwm.dwm2d(x.to(dev), w.to(dev), b.to(dev), (1, 1), pad, output_block=4)
    assert _nerr(y4, F.conv2d(x.double(), w.double(), b.double(), padding=pad)) < 1e-3
    yh = pkg.dwm.dwm2d(x.half().to(dev), w.half().to(dev), b.half().to(dev), (1, 1), pad)
    refh = F.conv2d(x.half().double(), w.half().double(), b.half().double(), padding=pad)
    assert yh.dtype == torch.float16 and _nerr(yh, refh) < 2e-2


def test_matrix_conv_functions(dev):
    x, w, b = _mk((2, 16, 18, 17), (8, 16, 3, 3))
    ref = F.conv2d(x.double(), w.double(), b.double(), padding=1)
    for ob in (2, 4):
        assert _nerr(pkg.matrix_conv.conv32(x.to(dev), w.to(dev), b.to(dev), (1, 1), (1, 1), 1, ob), ref) < 1e-3
        y16 = pkg.matrix_conv.conv16(x.to(dev), w.to(dev), b.to(dev), (1, 1), (1, 1), 1, ob)
        refh = F.conv2d(x.half().double(), w.half().double(), b.half().double(), padding=1)
        assert y16.dtype == torch.float32 and _nerr(y16, refh) < 2e-2
    assert _nerr(pkg.matrix_conv.conv(x.to(dev), w.to(dev), 2, 1), F.conv2d(x.double(), w.double())) < 1e-3
    assert _nerr(pkg.Wino().conv32(x.to(dev), w.to(dev), b.to(dev), 1, (1, 1)), ref) < 1e-3
    x3, w3, b3 = _mk((1, 8, 7, 10, 9), (8, 8, 3, 3, 3))
    ref3 = F.conv3d(x3.double(), w3.double(), b3.double(), padding=1)
    assert _nerr(pkg.matrix_conv3d.conv32(x3.to(dev), w3.to(dev), b3.to(dev), (1, 1, 1), (1, 1, 1)), ref3) < 1e-3


def test_matrix_conv_whole_kernel_tile_and_decompose_switch(dev):
    """matrix_conv.conv32 on a 5x5 kernel is one F(2,5) x F(2,5) tile like the reference
    (matrix_conv.py:112-135): bit-identical to the engine's whole-kernel plan; decompose=True
    is bit-identical to the DWM plan; wino_split -> base_conv32 -> wino_concat with 6x6 tiles
    gives the whole-kernel result too."""
    x, w, _ = _mk((2, 16, 18, 17), (8, 16, 5, 5))
    xd, wd = x.to(dev), w.to(dev)
    ref = F.conv2d(x.double(), w.double())
    y = pkg.matrix_conv.conv32(xd, wd)
    assert torch.equal(y, pkg.engine.conv_forward(xd, wd, whole_kernel=True))
    assert _nerr(y, ref) < 1e-3
    yd = pkg.matrix_conv.conv32(xd, wd, decompose=True)
    assert torch.equal(yd, pkg.engine.conv_forward(xd, wd))
    assert not torch.equal(y, yd)
    tiles = pkg.wino_split(xd, list(w.shape), 2)
    assert tuple(tiles.shape[2:]) == (6, 6)
    out = pkg.matrix_conv.base_conv32(tiles, wd, False, [2, 2], [5, 5])
    yc = pkg.wino_concat(out, [14, 13], 2)
    assert _nerr(yc, ref) < 1e-3 and _nerr(yc, y.double().cpu()) < 1e-5


def test_split_base_conv_concat_pipeline_like_the_reference(dev):
    """matrix_conv.conv's own sequence (matrix_conv.py:126-134): wino_split -> base_conv32 ->
    wino_concat, against the oracle's restatement of that path and fp64 convolution."""
    x, w, _ = _mk((2, 8, 11, 12), (6, 8, 3, 3))
    tiles = pkg.wino_split(x.to(dev), w.shape, 2)
    out = pkg.matrix_conv.base_conv32(tiles, w.to(dev), False, [2, 2], [3, 3])
    y = pkg.wino_concat(out, [9, 10], 2)
    ref = F.conv2d(x.double(), w.double())
    assert y.shape == ref.shape and _nerr(y, ref) < 1e-3
    assert _nerr(y, ow.matrix_conv(x, w, 2, "fp32").double()) < 1e-5
    x3, w3, _ = _mk((1, 4, 6, 7, 8), (5, 4, 3, 3, 3))
    t3 = pkg.wino_split(x3.to(dev), w3.shape, 2)
    o3 = pkg.matrix_conv3d.base_conv32(t3, w3.to(dev), False, [2, 2, 2], [3, 3, 3])
    y3 = pkg.wino_concat(o3, [4, 5, 6], 2)
    assert _nerr(y3, F.conv3d(x3.double(), w3.double())) < 1e-3


def test_backend_entry_points_with_reference_layouts(dev):
    """DWM / WinoSplit / WinoConcat called exactly as dwm2d_ and wino_split call them
    (dwm.py:122-136, Split_and_Concat.py:42-48,77-80)."""
    x, w, _ = _mk((2, 8, 12, 13), (6, 8, 5, 5))
    xd, wd = x.to(dev), w.to(dev)
    xin = xd.unsqueeze(2).permute(0, 2, 3, 4, 1).contiguous()             # NDHWC
    win = wd.unsqueeze(2).permute(2, 3, 4, 1, 0).contiguous()             # (kD,kH,kW,C,K)
    out = torch.zeros(2, 1, 8, 9, 6, device=dev)
    scratch = torch.zeros(4, device=dev)
    pkg.DWM(xin, win, out, 1, scratch, scratch, scratch, scratch.long())
    ref = F.conv2d(x.double(), w.double())
    assert _nerr(out[:, 0].permute(0, 3, 1, 2), ref) < 1e-3
    out2 = torch.zeros(2, 1, 4, 5, 6, device=dev)
    pkg.DWM(xin, win, out2, 2, scratch, scratch, scratch, scratch.long())
    assert _nerr(out2[:, 0].permute(0, 3, 1, 2), F.conv2d(x.double(), w.double(), stride=2)) < 1e-3
    # plain 3x3 through DWM: a key the reference's table lacks (base_conv_launchers.h:59-121)
    w3 = torch.randn(6, 8, 3, 3)
    out3 = torch.zeros(2, 1, 10, 11, 6, device=dev)
    pkg.DWM(xin, w3.to(dev).unsqueeze(2).permute(2, 3, 4, 1, 0).contiguous(), out3, 1)
    assert _nerr(out3[:, 0].permute(0, 3, 1, 2), F.conv2d(x.double(), w3.double())) < 1e-3
    # winograd_conv(x, w, out, bias, stride, padding, m, algo): padding, bias, tile 4 and the
    # whole-kernel algorithm on the same channel-last tensors
    b = torch.randn(6)
    refp = F.conv2d(x.double(), w.double(), b.double(), padding=2)
    for m, algo in ((2, "dwm"), (4, "dwm"), (2, "whole")):
        o = torch.zeros(2, 1, 12, 13, 6, device=dev)
        pkg.winograd_conv(xin, win, o, b.to(dev), 1, 2, m, algo)
        assert _nerr(o[:, 0].permute(0, 3, 1, 2), refp) < 1e-3, (m, algo)
    with pytest.raises(ValueError):
        pkg.winograd_conv(xin, win, out, None, 1, 0, 2, "fft")
    # tile copies
    a = xd.permute(0, 2, 3, 1).contiguous()
    tiles = torch.zeros(2 * 5 * 6, 8, 4, 4, device=dev)
    pkg.WinoSplit(a, tiles, 0, 4, 4, 2, 0, 5, 6, True)
    assert torch.equal(tiles, pkg.wino_split(xd, (6, 8, 3, 3), 2))
    back = torch.zeros(2, 10, 11, 8, device=dev)
    t2 = torch.randn(2 * 5 * 6, 8, 2, 2, device=dev)
    pkg.split_and_concat("concat", t2, back, 2, True)
    assert torch.equal(back.permute(0, 3, 1, 2), pkg.wino_concat(t2, [10, 11], 2))
    with pytest.raises(ValueError):
        pkg.WinoSplit(a, torch.zeros(3, device=dev), 0, 4, 4, 2, 0, 5, 6, True)
    c = pkg.add_gpu(xd, xd)
    assert torch.equal(c, xd + xd)


@pytest.mark.parametrize("k,stride,pad", [(3, 1, 1), (5, 1, 2), (7, 2, 3), (3, 2, 1)])
def test_winoconv2d_module_routes_and_caches(dev, k, stride, pad):
    torch.manual_seed(0)
    mod = pkg.WinoConv2d(16, 24, k, stride, pad, dtype=torch.float16, device=dev)
    x = torch.randn(2, 16, 20, 20, device=dev).half()
    ref = F.conv2d(x.double().cpu(), mod.weight.detach().double().cpu(), mod.bias.detach().double().cpu(),
                   stride=stride, padding=pad)
    y = mod(x)
    assert y.shape == ref.shape and _nerr(y, ref) < 2e-2
    U0 = mod._cache[1]
    mod(x)
    assert mod._cache[1] is U0                       # cached filter transform reused
    with torch.no_grad():
        mod.weight.mul_(2.0)
    y2 = mod(x)
    assert mod._cache[1] is not U0                   # weight changed: recomputed
    ref2 = F.conv2d(x.double().cpu(), mod.weight.detach().double().cpu(), mod.bias.detach().double().cpu(),
                    stride=stride, padding=pad)
    assert _nerr(y2, ref2) < 2e-2
    # dilation falls back to torch like the reference's cuDNN branch (conv.py:326-332)
    mod_d = pkg.WinoConv2d(16, 24, 3, 1, 2, dilation=2, dtype=torch.float16, device=dev)
    yd = mod_d(x)
    assert yd.shape == (2, 24, 20, 20)
    # so does a strided first layer with 5 to 8 input channels, or in fp32 (the reference sends every strided layer
    # there); with at most 4 channels in a 16-bit type the engine has a kernel of its own (test_gpu_direct.py)
    mod_s = pkg.WinoConv2d(6, 16, 7, 2, 3, dtype=torch.float16, device=dev)
    x6 = torch.randn(2, 6, 30, 30, device=dev).half()
    assert torch.equal(mod_s(x6), F.conv2d(x6, mod_s.weight, mod_s.bias, 2, 3)) and mod_s._cache is None
    mod_f = pkg.WinoConv2d(3, 16, 7, 2, 3, device=dev)
    x3 = torch.randn(2, 3, 30, 30, device=dev)
    assert torch.equal(mod_f(x3), F.conv2d(x3, mod_f.weight, mod_f.bias, 2, 3)) and mod_f._cache is None


def test_winoconv2d_module_follows_the_plan_form_when_the_batch_size_changes(dev):
    """The library takes the direct form for this strided layer at N = 32 and a Winograd plan at N = 8; the
    transformed filters of the two forms differ in size, so the module's cached one must follow the form."""
    torch.manual_seed(0)
    mod = pkg.WinoConv2d(128, 128, 7, 2, 3, bias=False, dtype=torch.float16, device=dev)
    forms = set()
    for n in (32, 8, 32):
        x = torch.randn(n, 128, 112, 112, device=dev).half()
        forms.add(engine.plan_form(x.shape, mod.weight.shape, x.dtype, 2, (3, 3), mod._tile_for(x.dtype)))
        y = mod(x)
        ref = F.conv2d(x[:2].double().cpu(), mod.weight.detach().double().cpu(), stride=2, padding=3)
        assert _nerr(y[:2], ref) < 2e-2
    assert len(forms) == 2


def test_winoconv3d_module(dev):
    torch.manual_seed(0)
    mod = pkg.WinoConv3d(8, 8, 3, 1, 1, device=dev)
    x = torch.randn(1, 8, 6, 10, 10, device=dev)
    ref = F.conv3d(x.double().cpu(), mod.weight.detach().double().cpu(), mod.bias.detach().double().cpu(), padding=1)
    assert _nerr(mod(x), ref) < 1e-3
    # a 3-D first layer with at most 4 input channels goes to torch (the reference sends every 3x3x3 layer there)
    mod3 = pkg.WinoConv3d(3, 8, 3, 1, 1, device=dev)
    x3 = torch.randn(1, 3, 6, 10, 10, device=dev)
    assert torch.equal(mod3(x3), F.conv3d(x3, mod3.weight, mod3.bias, 1, 1)) and mod3._cache is None


@pytest.mark.parametrize("ws,m,stacked,force", [
    ((48, 32, 5, 5), 4, 0, None),        # DWM pieces, four kernels
    ((48, 32, 5, 5), 2, 2, None),        # two-tap pieces sharing one transformed input (shifted GEMM operand)
    ((48, 32, 3, 3), 2, 0, None),        # thin 16-bit 3x3 layer: filter transform + the one fused kernel
    ((48, 32, 5, 5), 2, 2, (-1, 3)),     # ... the shifted product on its persistent LDS-DMA kernel
    ((256, 96, 3, 3), 4, 0, (10, 1)),    # the batched GEMM on its persistent LDS-DMA kernel
    ((256, 160, 3, 3), 4, 0, (13, 1)),   # ... with a tile's write-out riding on the next tile (buffer stores)
])
def test_forward_is_capturable_in_a_hip_graph(dev, ws, m, stacked, force, gemm_override):
    """The library allocates nothing, never synchronises and takes its stream from the caller, so a
    whole forward pass can be captured once and replayed.  The graph is replayed three times with new
    input contents, eager work and synchronisation between the replays, and every replay must equal
    the eager result bit for bit."""
    import ctypes
    from pytorch_winoconv_amd import _lib
    lib = _lib.load()
    if force:
        gemm_override(*force)
    xs = (2, ws[1], 20, 20)
    pad = ws[2] // 2
    g = torch.Generator().manual_seed(11)
    x = torch.randn(*xs, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(*ws, generator=g) * 0.05).half().to(dev)
    desc = pkg.engine.make_desc(xs, ws, torch.float16, 1, pad, m, stacked=stacked)
    nbytes = ctypes.c_size_t()
    _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
    wsp = torch.empty(nbytes.value, dtype=torch.uint8, device=dev)
    x_cl = pkg.engine.channel_last(x)
    y = torch.empty(2, 20, 20, ws[0], dtype=torch.float16, device=dev)
    strides = pkg.engine._w_strides(w)

    def forward():
        st = torch.cuda.current_stream().cuda_stream
        _lib.check(lib.wc_conv_forward(ctypes.byref(desc), x_cl.data_ptr(), w.data_ptr(), strides, None, None,
                                       y.data_ptr(), wsp.data_ptr(), nbytes.value, st))

    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        forward()                                         # warm-up outside the capture
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        forward()
    for i in range(3):
        x_cl.copy_(torch.randn(x_cl.shape, generator=g).half().to(dev))
        y.fill_(float("nan"))
        graph.replay()
        torch.cuda.synchronize()
        got = y.clone()
        want = pkg.engine.conv_forward(x_cl.permute(0, 3, 1, 2), w, None, 1, pad, m, stacked=stacked)   # eager, own buffers
        assert torch.equal(got.permute(0, 3, 1, 2), want), i


def test_plan_dump_with_winoconv_log(dev):
    """WINOCONV_LOG=1 makes wc_conv_forward print the plan it runs (one line per call, to stderr); without it
    the library prints nothing.  The variable is read once per process, so each case is a process of its own."""
    import os
    import subprocess
    import sys
    code = ("import torch, pytorch_winoconv_amd as p; x = torch.randn(2, 8, 20, 21, device='cuda').half(); "
            "w = torch.randn(4, 8, 7, 7, device='cuda').half(); p.engine.conv_forward(x, w, None, 1, 3, 4); "
            "torch.cuda.synchronize()")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    for flag, expect in (("1", True), ("0", False)):
        env = dict(os.environ, WINOCONV_LOG=flag, PYTHONPATH=root)
        r = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, timeout=300)
        assert r.returncode == 0, r.stderr
        lines = [ln for ln in r.stderr.splitlines() if ln.startswith("winoconv:")]
        assert bool(lines) == expect
        if expect:
            assert "tile m=1,3,3" in lines[0] and "pieces=9" in lines[0] and "stacked=2" in lines[0]
            assert "shifted batched GEMM" in lines[0] and "channel-first, copied" in lines[0]


@pytest.mark.parametrize("case", [
    # x shape, w shape, stride, pad, m, channel-first tensors, cached filter -> the stages that must have run
    ((4, 48, 20, 22), (40, 48, 3, 3), 1, 1, 4, False, False, {"filter_transform", "input_transform", "product", "output_transform"}),
    ((4, 48, 20, 22), (40, 48, 3, 3), 1, 1, 4, False, True, {"input_transform", "product", "output_transform"}),
    ((2, 32, 18, 18), (16, 32, 5, 5), 1, 2, 2, True, False, set(pkg.engine.STAGES)),
    ((4, 64, 20, 22), (64, 64, 3, 3), 1, 1, 2, False, False, {"filter_transform", "product"}),            # one fused kernel
    ((4, 64, 20, 22), (64, 64, 3, 3), 2, 1, 2, False, False, {"filter_transform", "product"}),            # the direct form
])
def test_timed_forward_reports_the_stages_that_ran(dev, case):
    """wc_conv_forward_timed: bit for bit the result of wc_conv_forward, a positive time for every stage the
    plan runs and zero for the others, and together no more than the wall time of the call."""
    import time
    xs, ws, stride, pad, m, channel_first, cached, ran = case
    g = torch.Generator().manual_seed(4)
    x = torch.randn(*xs, generator=g).half().to(dev)
    if not channel_first:
        x = x.contiguous(memory_format=torch.channels_last)
    w = torch.randn(*ws, generator=g).half().to(dev)
    U = pkg.engine.transform_filter(w, xs, stride, pad, m) if cached else None
    want = pkg.engine.conv_forward(x, w, None, stride, pad, m, U=U, channels_first_out=channel_first)
    pkg.engine.conv_forward_timed(x, w, None, stride, pad, m, U=U, channels_first_out=channel_first)    # warm
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    y, times = pkg.engine.conv_forward_timed(x, w, None, stride, pad, m, U=U, channels_first_out=channel_first)
    wall_ms = (time.perf_counter() - t0) * 1e3            # the call returns after the device has finished
    assert torch.equal(y, want)
    assert set(times) == set(pkg.engine.STAGES)
    for name, ms in times.items():
        assert (ms > 0) == (name in ran), (name, ms)
    assert sum(times.values()) <= wall_ms
