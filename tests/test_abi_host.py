"""CPU-only checks of the C-ABI library: it loads, exports every symbol the header declares,
plans exactly like the reference's table and the oracle, and reports errors by status code
(no GPU call is made here: every call below returns before its first launch)."""
import ctypes
import json
import os
import re

import pytest
import torch

import pytorch_winoconv_amd as pkg
from pytorch_winoconv_amd import _lib, engine
from oracle import split_plan as osp

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
LUT = json.load(open(os.path.join(ROOT, "tests", "golden", "split_lut.json")))


def test_library_exports_every_declared_symbol():
    header = open(os.path.join(ROOT, "include", "winoconv.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b(wc_[a-z0-9_]+)\s*\(", header))
    assert declared == set(_lib.SIGNATURES), declared ^ set(_lib.SIGNATURES)
    lib = ctypes.CDLL(_lib.LIB_PATH)
    for name in declared:
        assert hasattr(lib, name), name
    assert b"gfx950" in _lib.load().wc_version()


@pytest.mark.parametrize("key", sorted(LUT))
def test_wc_plan_dwm_matches_reference_table(key):
    kd, kh, kw = (int(v) for v in key.split("x"))
    p = engine.plan_dwm(kd, kh, kw)
    g = LUT[key]
    for a, b in [("D_s", "D_start"), ("D_e", "D_end"), ("H_s", "H_start"), ("H_e", "H_end"),
                 ("W_s", "W_start"), ("W_e", "W_end")]:
        assert g[a] == p[b], (key, a)
    o = osp.split_plan(kd, kh, kw)
    assert p["kernel_stride"] == o["kernel_stride"] and p["T_total"] == o["T_total"]


@pytest.mark.parametrize("xs,ws,stride,m", [
    ((1, 4, 20, 20), (4, 4, 3, 3), 1, 2), ((1, 4, 20, 20), (4, 4, 3, 3), 1, 4),
    ((1, 4, 20, 20), (4, 4, 7, 7), 1, 2), ((1, 4, 20, 20), (4, 4, 7, 7), 2, 2),
    ((1, 4, 20, 20), (4, 4, 3, 3), 2, 2), ((1, 4, 20, 20), (4, 4, 10, 9), 2, 2),
    ((1, 4, 20, 20), (4, 4, 7, 7), 1, 4), ((1, 4, 20, 20), (4, 4, 5, 4), 2, 4),
    ((1, 4, 9, 20, 20), (4, 4, 3, 3, 3), 1, 2), ((1, 4, 9, 20, 20), (4, 4, 5, 7, 4), 1, 2),
])
def test_wc_plan_conv_matches_oracle(xs, ws, stride, m):
    desc = engine.make_desc(xs, ws, torch.float16, stride, 1, m)
    plan = engine.plan_conv(desc)
    two_d = len(xs) == 4
    ks = ([1] if two_d else []) + list(ws[2:])
    pieces, T = osp.conv_pieces(ks, stride, m, degenerate_depth=two_d)
    assert plan.t_total == T and plan.n_pieces == len(pieces) and plan.tap_step == stride
    assert list(plan.m) == pieces[0]["ms"]
    for i, pc in enumerate(pieces):
        assert list(plan.piece[i].tap0) == [a[0] for a in pc["axes"]]
        assert list(plan.piece[i].r) == [a[2] for a in pc["axes"]]
        assert plan.piece[i].t_offset == pc["t_offset"]


def test_out_dims_follow_the_reference_arithmetic():
    """oX = X + 2 pad - kX + 1, nX = (oX + 1) / 2 (src/base_conv_launchers.cu:290-295)."""
    desc = engine.make_desc((2, 8, 10, 13), (4, 8, 7, 7), torch.float32, 1, 0, 2)
    out, grid = engine.out_dims(desc)
    assert out == [1, 4, 7] and grid == [1, 2, 4]
    desc = engine.make_desc((2, 8, 56, 56), (4, 8, 3, 3), torch.float16, 1, 1, 4)
    assert engine.out_dims(desc) == ([1, 56, 56], [1, 14, 14])
    desc = engine.make_desc((2, 8, 112, 112), (4, 8, 7, 7), torch.float16, 2, 3, 2)
    assert engine.out_dims(desc) == ([1, 56, 56], [1, 28, 28])


def test_errors_are_status_codes_with_messages_not_exits():
    lib = _lib.load()
    # unsupported: stride 3, tile 3, kernel extent 11, tile 4 in 3-D for a kernel that is not 3x3x3
    for kw in (dict(stride=3), dict(m=3), dict(w=(4, 4, 11, 3)), dict(m=4, x=(1, 4, 9, 20, 20), w=(4, 4, 3, 3, 5))):
        desc = engine.make_desc(kw.get("x", (1, 4, 20, 20)), kw.get("w", (4, 4, 3, 3)), torch.float32,
                                kw.get("stride", 1), 0, kw.get("m", 2))
        with pytest.raises(NotImplementedError):
            engine.plan_conv(desc)
        assert len(lib.wc_last_error()) > 0
    # bad argument: kernel larger than the padded input
    desc = engine.make_desc((1, 4, 2, 2), (4, 4, 3, 3), torch.float32, 1, 0, 2)
    with pytest.raises(ValueError):
        engine.out_dims(desc)
    # null pointers are rejected before any launch
    desc = engine.make_desc((1, 4, 8, 8), (4, 4, 3, 3), torch.float32, 1, 0, 2)
    plan = engine.plan_conv(desc)
    null = ctypes.c_void_p(0)
    assert lib.wc_input_transform(ctypes.byref(desc), ctypes.byref(plan), null, 1, null, null) == _lib.WC_ERR_BAD_ARG
    assert lib.wc_batched_gemm(null, null, null, 1, 1, 32, 1, 8, 0, null) == _lib.WC_ERR_BAD_ARG
    assert lib.wc_wino_split2d(null, null, 1, 4, 4, 4, 4, 4, 2, 1, 1, 4, null) == _lib.WC_ERR_BAD_ARG
    # workspace: missing / too small
    nbytes = ctypes.c_size_t()
    assert lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0 and nbytes.value > 0
    fake = ctypes.c_void_p(256)   # never dereferenced: the size check fails first
    strides = (ctypes.c_int64 * 5)(36, 9, 0, 3, 1)
    rc = lib.wc_conv_forward(ctypes.byref(desc), fake, fake, strides, null, null, fake, null, 0, null)
    assert rc == _lib.WC_ERR_WORKSPACE
    rc = lib.wc_conv_forward(ctypes.byref(desc), fake, fake, strides, null, null, fake, fake, 16, null)
    assert rc == _lib.WC_ERR_WORKSPACE and b"needed" in lib.wc_last_error()


def test_workspace_size_is_u_plus_v_plus_m():
    lib = _lib.load()
    desc = engine.make_desc((64, 256, 56, 56), (256, 256, 3, 3), torch.float16, 1, 1, 4)
    nbytes, ue = ctypes.c_size_t(), ctypes.c_size_t()
    assert lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0
    assert lib.wc_conv_u_elems(ctypes.byref(desc), ctypes.byref(ue)) == 0
    T, P = 36, 64 * 14 * 14
    assert ue.value == T * 256 * 256
    assert nbytes.value == 2 * (T * 256 * 256 + 2 * T * P * 256)
    desc.chunk_images = 8
    assert lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0
    assert nbytes.value == 2 * (T * 256 * 256 + 2 * T * (P // 8) * 256)
    # a layer the one-kernel path takes needs U only; with `unfused` all three buffers again
    thin = engine.make_desc((64, 64, 56, 56), (64, 64, 3, 3), torch.float16, 1, 1, 2)
    assert lib.wc_conv_workspace_bytes(ctypes.byref(thin), ctypes.byref(nbytes)) == 0
    assert nbytes.value == 2 * 16 * 64 * 64
    thin.unfused = 1
    assert lib.wc_conv_workspace_bytes(ctypes.byref(thin), ctypes.byref(nbytes)) == 0
    assert nbytes.value == 2 * (16 * 64 * 64 + 2 * 16 * 64 * 28 * 28 * 64)


def test_python_layer_refuses_cpu_tensors_and_bad_shapes(host_layer):
    x = torch.randn(1, 4, 8, 8)
    w = torch.randn(4, 4, 3, 3)
    with pytest.raises(ValueError, match="GPU only"):
        engine.conv_forward(x, w)
    with pytest.raises(ValueError, match="GPU only"):
        pkg.wino_split(x, w.shape, 2)
    with pytest.raises(ValueError):
        engine.make_desc((1, 4, 8, 8), (4, 5, 3, 3), torch.float32)        # channel mismatch
    with pytest.raises(NotImplementedError):
        engine.make_desc((1, 4, 8, 8), (4, 4, 3, 3), torch.float32, stride=(1, 2))
    with pytest.raises(NotImplementedError):
        pkg.dwm.dwm2d(x, w, groups=2)
    with pytest.raises(ValueError, match="GPU only"):                       # modules have no CPU path either
        pkg.WinoConv2d(4, 4, 3, 1, 1)(x)


def test_bias_and_cached_filter_are_checked_before_any_launch(host_layer):
    """The C ABI sees pointers only: a short bias would be read out of bounds and a transformed filter of
    another dtype misread, so the host layer refuses both (torch's own conv2d raises for them too)."""
    x = torch.randn(1, 4, 8, 8)
    w = torch.randn(6, 4, 3, 3)
    with pytest.raises(ValueError, match="bias must be a 1-D tensor of 6"):
        engine.conv_forward(x, w, torch.randn(5))
    with pytest.raises(ValueError, match="bias must be a 1-D tensor of 6"):
        engine.conv_forward(x, w, torch.randn(6, 1))
    with pytest.raises(TypeError, match="share one dtype"):
        engine.conv_forward(x, w, torch.randn(6).half())
    U16 = torch.zeros(16, 6, 32, dtype=torch.float16)
    with pytest.raises(TypeError, match="transformed filter is"):
        engine.conv_forward(x, w, None, 1, 1, 2, U=U16)
    xc, wc, out = torch.randn(1, 1, 8, 8, 4), torch.randn(1, 3, 3, 4, 6), torch.zeros(1, 1, 6, 6, 6)
    with pytest.raises(ValueError, match="bias must be a 1-D tensor of 6"):
        pkg.winograd_conv(xc, wc, out, bias=torch.randn(7))
    with pytest.raises(TypeError, match="transformed filter is"):
        pkg.winograd_conv(xc, wc, out, U=U16)


def test_static_scratch_entry_point_refuses_oversized_problems_before_any_gpu_call():
    """One image of this layer needs 116 MB of V and M, the static buffer holds 64 MiB: the size check comes
    before the first HIP call, so it can be seen without a GPU (the pointers are never touched)."""
    lib = _lib.load()
    desc = engine.make_desc((1, 256, 224, 224), (256, 256, 3, 3), torch.float16, 1, 1, 4)
    fake = ctypes.c_void_p(4096)
    strides = (ctypes.c_int64 * 5)(2304, 9, 0, 3, 1)
    rc = lib.wc_conv_forward_static(ctypes.byref(desc), fake, fake, strides, None, None, fake, None)
    assert rc == _lib.WC_ERR_WORKSPACE and b"static buffer" in lib.wc_last_error()
    assert _lib.WC_STATIC_SCRATCH_BYTES == 64 << 20
    header = open(os.path.join(ROOT, "include", "winoconv.h")).read()
    assert "#define WC_STATIC_SCRATCH_BYTES (64u * 1024u * 1024u)" in header


def test_effective_tile_tells_what_a_request_for_tile_4_becomes():
    """The plan whose pieces share one transformed input has tiles 2 and 3 only: fp16 callers who ask for 4 get 3
    where the three-tap pieces apply (kernels of 5..10 taps), bf16 callers and 4x4 kernels get 2; plain 3x3
    layers keep 4.  The choice is made by the library (wc_conv_auto) and reported back."""
    et = engine.effective_tile
    assert et((2, 8, 20, 21), (4, 8, 7, 7), torch.float16, 1, 3, 4) == (3, 2)
    assert et((2, 8, 20, 21), (4, 8, 7, 7), torch.bfloat16, 1, 3, 4) == (2, 2)
    assert et((2, 8, 20, 21), (4, 8, 4, 4), torch.float16, 1, 1, 4) == (2, 2)
    assert et((2, 8, 20, 21), (4, 8, 3, 3), torch.float16, 1, 1, 4)[0] == 4
    assert et((2, 8, 20, 21), (4, 8, 7, 7), torch.float32, 1, 3, 4) == (4, 0)
    assert et((2, 8, 20, 21), (4, 8, 7, 7), torch.float16, 1, 3, 4, stacked=True) == (4, 1)


def test_bfloat16_is_a_storage_type():
    d = engine.make_desc((2, 8, 20, 20), (4, 8, 3, 3), torch.bfloat16, 1, 1, 2)
    assert d.dtype == _lib.WC_BF16 == 2 and engine.plan_conv(d).t_total == 16
    d.dtype = 3
    with pytest.raises(ValueError):
        engine.plan_conv(d)


def test_3d_tile_4_is_2x4x4_for_3x3x3_only():
    d = engine.make_desc((2, 8, 7, 18, 21), (4, 8, 3, 3, 3), torch.float16, 1, 1, 4)
    plan = engine.plan_conv(d)
    assert list(plan.m) == [2, 4, 4] and plan.n_pieces == 1 and plan.t_total == 4 * 6 * 6
    out, grid = engine.out_dims(d)
    assert out == [7, 18, 21] and grid == [4, 5, 6]
    for ws, stride in (((4, 8, 5, 5, 5), 1), ((4, 8, 3, 3, 3), 2), ((4, 8, 1, 3, 3), 1)):
        with pytest.raises(NotImplementedError):
            engine.plan_conv(engine.make_desc((2, 8, 7, 18, 21), ws, torch.float16, stride, 1, 4))


def test_whole_kernel_plans():
    """One F(2,k) x F(2,k) piece for a k x k kernel (the reference's matrix_conv tile,
    matrix_conv.py:112-135) and the descriptor checks around it."""
    lib = _lib.load()
    for k in (4, 5, 6, 7):
        d = engine.make_desc((2, 8, 20, 20), (4, 8, k, k), torch.float32, 1, 0, 2, whole_kernel=True)
        plan = engine.plan_conv(d)
        assert plan.n_pieces == 1 and plan.t_total == (k + 1) ** 2
        assert list(plan.piece[0].r) == [1, k, k] and list(plan.piece[0].tap0) == [0, 0, 0]
        assert list(plan.m) == [1, 2, 2]
    d3 = engine.make_desc((2, 8, 20, 20), (4, 8, 3, 3), torch.float32, 1, 1, 2, whole_kernel=True)
    assert engine.plan_conv(d3).t_total == 16                       # 3x3 is a whole-kernel tile anyway
    for bad in (dict(x=(2, 8, 20, 20), w=(4, 8, 5, 5), stride=2, m=2),
                dict(x=(2, 8, 20, 20), w=(4, 8, 5, 5), stride=1, m=4),
                dict(x=(2, 8, 20, 20), w=(4, 8, 5, 7), stride=1, m=2),
                dict(x=(2, 8, 20, 20), w=(4, 8, 9, 9), stride=1, m=2),
                dict(x=(2, 8, 9, 20, 20), w=(4, 8, 5, 5, 5), stride=1, m=2)):
        d = engine.make_desc(bad["x"], bad["w"], torch.float32, bad["stride"], 0, bad["m"], whole_kernel=True)
        with pytest.raises(NotImplementedError):
            engine.plan_conv(d)


def test_stacked_plans():
    """Pieces that share one tile: element offset 0 for every piece, T of the tile of the longest
    piece per axis, U / V / workspace sized for the pieces side by side; 2-D DWM plans only."""
    lib = _lib.load()
    from oracle import winograd as ow
    for ws, stride, m in (((4, 8, 5, 5), 1, 4), ((4, 8, 7, 7), 1, 2), ((4, 8, 7, 7), 2, 4), ((4, 8, 3, 3), 2, 2),
                          ((4, 8, 4, 6), 1, 2), ((4, 8, 3, 3), 1, 4)):
        xs = (2, 8, 20, 21)
        plain = engine.plan_conv(engine.make_desc(xs, ws, torch.float16, stride, 1, m))
        d = engine.make_desc(xs, ws, torch.float16, stride, 1, m, stacked=True)
        plan = engine.plan_conv(d)
        pcs, T = ow.stacked_pieces(ow.conv_plan(xs, ws, stride, 1, m)["pieces"])
        assert plan.n_pieces == plain.n_pieces == len(pcs) and plan.t_total == T
        for i in range(plan.n_pieces):
            assert plan.piece[i].t_offset == 0
            assert list(plan.piece[i].r) == list(plain.piece[i].r) == pcs[i]["real"]
            assert list(plan.piece[i].tap0) == list(plain.piece[i].tap0)
        ue, nbytes = ctypes.c_size_t(), ctypes.c_size_t()
        assert lib.wc_conv_u_elems(ctypes.byref(d), ctypes.byref(ue)) == 0
        assert ue.value == T * 4 * 32 * plan.n_pieces
        assert lib.wc_conv_workspace_bytes(ctypes.byref(d), ctypes.byref(nbytes)) == 0
        out, grid = engine.out_dims(d)
        P = 2 * grid[1] * grid[2]
        r256 = lambda v: (v + 255) // 256 * 256                       # each buffer starts on a 256-byte boundary
        assert nbytes.value == r256(2 * ue.value) + r256(2 * T * P * 32 * plan.n_pieces) + r256(2 * T * P * 8)
    d3 = engine.make_desc((2, 8, 9, 20, 20), (4, 8, 5, 5, 5), torch.float32, 1, 0, 2, stacked=True)
    p3 = engine.plan_conv(d3)
    assert p3.n_pieces == 8 and p3.t_total == 64 and all(p3.piece[i].t_offset == 0 for i in range(8))
    with pytest.raises(NotImplementedError):
        engine.plan_conv(engine.make_desc((2, 8, 20, 20), (4, 8, 5, 5), torch.float32, 1, 0, 2, stacked=True,
                                          whole_kernel=True))


def test_modules_pick_tile_2_where_tile_4_loses_accuracy():
    import pytorch_winoconv_amd as pkg
    wide, thin = pkg.WinoConv2d(256, 256, 3, padding=1), pkg.WinoConv2d(3, 64, 3, padding=1)
    assert wide._tile_for(torch.float16) == 4 and wide._tile_for(torch.float32) == 4
    assert wide._tile_for(torch.bfloat16) == 2          # 8 mantissa bits
    assert thin._tile_for(torch.float16) == 2            # too few channels to average the rounding error down
    assert thin._tile_for(torch.float32) == 2            # 3 channels: the fused first-layer kernel, tile 2
    assert pkg.WinoConv2d(3, 64, 3, padding=1, output_block=4)._tile_for(torch.float16) == 4   # an explicit choice stands
    assert pkg.WinoConv3d(64, 64, 3, padding=1)._tile_for(torch.float16) == 2


def test_shared_input_plans():
    """stacked = 2: pieces of two taps on the tile F(2,2), one transformed input for all of them over a
    tile grid extended by the pieces' reach; 2-D, stride 1, output tile 2."""
    lib = _lib.load()
    d = engine.make_desc((2, 8, 20, 21), (4, 8, 7, 5), torch.float16, 1, (3, 2), 2, stacked=2)
    assert d.stacked == 2 and d.m == 2
    plan = engine.plan_conv(d)
    assert plan.n_pieces == 4 * 3 and plan.t_total == 9 and list(plan.m) == [1, 2, 2]
    want = [((0, 2 * a, 2 * b), (1, 2 if 2 * a + 2 <= 7 else 1, 2 if 2 * b + 2 <= 5 else 1)) for a in range(4) for b in range(3)]
    for i, (tap0, r) in enumerate(want):
        assert tuple(plan.piece[i].tap0) == tap0 and tuple(plan.piece[i].r) == r and plan.piece[i].t_offset == 0
    from oracle import split_plan as osp2
    pieces, T = osp2.conv_pieces([1, 7, 5], 1, 2, degenerate_depth=True, pairs=True)
    assert [tuple(a[0] for a in pc["axes"]) for pc in pieces] == [t for t, _ in want]
    out, grid = engine.out_dims(d)
    assert out == [1, 20, 21] and grid == [1, 10 + 3, 11 + 2]
    # workspace: U (9, K, 12 Cp) + V (9, P + tail, Cp) + M (9, P, 8), each rounded to 256 bytes
    nbytes = ctypes.c_size_t()
    assert lib.wc_conv_workspace_bytes(ctypes.byref(d), ctypes.byref(nbytes)) == 0
    P, tail = 2 * 13 * 13, 3 * 13 + 2
    r256 = lambda v: (v + 255) // 256 * 256
    assert nbytes.value == r256(2 * 9 * 4 * 12 * 32) + r256(2 * 9 * (P + tail) * 32) + r256(2 * 9 * P * 8)
    # one piece per axis: nothing is extended
    d1 = engine.make_desc((2, 8, 20, 21), (4, 8, 2, 1), torch.float16, 1, 0, 2, stacked=2)
    assert engine.plan_conv(d1).n_pieces == 1 and engine.out_dims(d1)[1] == [1, 10, 11]
    # 3-D: pieces depth-major, the grid extended on all three axes
    d3 = engine.make_desc((1, 8, 9, 20, 20), (4, 8, 3, 5, 4), torch.float16, 1, (1, 2, 1), 2, stacked=2)
    p3 = engine.plan_conv(d3)
    assert p3.n_pieces == 2 * 3 * 2 and p3.t_total == 27 and list(p3.m) == [2, 2, 2]
    assert tuple(p3.piece[7].tap0) == (2, 0, 2) and tuple(p3.piece[7].r) == (1, 2, 2)
    assert engine.out_dims(d3) == ([9, 20, 19], [5 + 1, 10 + 2, 10 + 1])
    bad = engine.make_desc((2, 8, 20, 21), (4, 8, 5, 5), torch.float16, 1, 2, 2, stacked=2)
    bad.m = 4
    with pytest.raises(NotImplementedError):
        engine.plan_conv(bad)
    # tile 3: the reference's three-tap pieces on the shared tile F(3,3); what a caller who asked for tile 4 gets
    # in fp16 (bf16: tile 2); 2-D, at least 3 taps per axis and more than 3 on one
    d = engine.make_desc((2, 8, 20, 21), (4, 8, 7, 5), torch.float16, 1, (3, 2), 4, stacked=2)
    assert d.m == 3 and engine.make_desc((2, 8, 20, 21), (4, 8, 7, 5), torch.bfloat16, 1, (3, 2), 4, stacked=2).m == 2
    plan = engine.plan_conv(d)
    assert plan.n_pieces == 3 * 2 and plan.t_total == 25 and list(plan.m) == [1, 3, 3]
    assert [tuple(plan.piece[i].tap0) for i in range(6)] == [(0, 3 * a, 3 * b) for a in range(3) for b in range(2)]
    assert [tuple(plan.piece[i].r) for i in range(6)] == [(1, 3, 3), (1, 3, 2), (1, 3, 3), (1, 3, 2), (1, 1, 3), (1, 1, 2)]
    assert engine.out_dims(d) == ([1, 20, 21], [1, 7 + 2, 7 + 1])
    for ws in ((4, 8, 3, 3), (4, 8, 5, 2)):
        bad = engine.make_desc((2, 8, 20, 21), ws, torch.float16, 1, 1, 3, stacked=2)
        with pytest.raises(NotImplementedError):
            engine.plan_conv(bad)
    bad = engine.make_desc((2, 8, 20, 21), (4, 8, 5, 5), torch.float16, 1, 1, 3)       # tile 3 without the shared plan
    with pytest.raises(NotImplementedError):
        engine.plan_conv(bad)
    # what the Python layer picks when nothing is said
    s = engine._stack
    assert s(None, torch.float16, 2, False, (128, 128, 5, 5), 1, 4) == 2 and s(None, torch.bfloat16, 2, False, (8, 100, 4, 8), 1, 2) == 2
    assert s(None, torch.float16, 2, False, (128, 128, 5, 5), 2, 4) is True        # stride 2
    assert s(None, torch.float16, 2, False, (128, 160, 5, 5), 1, 2) == 2 and s(None, torch.float16, 2, False, (128, 300, 5, 5), 1, 2) is True
    assert s(None, torch.float16, 2, False, (128, 160, 5, 5), 1, 4) == 2 and s(None, torch.float16, 2, False, (128, 300, 5, 5), 1, 4) is True
    assert s(None, torch.float16, 2, False, (128, 128, 9, 9), 1, 2) == 2 and s(None, torch.float16, 2, False, (128, 128, 9, 9), 1, 4) == 2
    assert s(None, torch.float16, 2, False, (128, 128, 11, 3), 1, 2) is True
    assert s(None, torch.float16, 3, False, (8, 160, 5, 5, 5), 1, 2) is True and s(None, torch.float16, 3, False, (8, 160, 4, 4, 4), 1, 2) == 2
    assert s(None, torch.bfloat16, 2, False, (128, 128, 9, 9), 1, 4) == 2 and s(None, torch.float16, 2, False, (8, 8, 3, 3), 1, 4) is True
    assert s(None, torch.float32, 2, False, (128, 128, 5, 5), 1, 4) is True and s(None, torch.float16, 3, False, (8, 8, 5, 5, 5), 1, 2) == 2
    assert s(None, torch.float16, 3, False, (8, 8, 3, 3, 3), 1, 2) is True and s(None, torch.float16, 3, False, (8, 8, 3, 3, 3), 1, 4) is False
    assert s(2, torch.float32, 2, False) == 2 and s(True, torch.float16, 2, False) is True and s(False, torch.float16, 2, False) is False


def test_shared_input_plans_at_stride_2():
    """Stride 2: positions of two phase taps per axis, inside a position the parity phases; a piece owns
    the taps q + 2 j (j = 2 pos, 2 pos + 1) that exist, pieces past a phase's last tap have none.  Every tap
    of the kernel is owned once; the grid grows by the positions beyond the first."""
    from pytorch_winoconv_amd import engine
    for kh, kw in ((7, 7), (5, 5), (3, 3), (8, 4), (2, 1), (10, 9)):
        d = engine.make_desc((2, 8, 30, 31), (4, 8, kh, kw), torch.float16, 2, (kh // 2, kw // 2), 2, stacked=2)
        plan = engine.plan_conv(d)
        ph = [2 if k >= 2 else 1 for k in (kh, kw)]
        pos = [((k + 1) // 2 + 1) // 2 for k in (kh, kw)]
        assert plan.n_pieces == ph[0] * ph[1] * pos[0] * pos[1] and plan.tap_step == 2
        owned = []
        for i in range(plan.n_pieces):
            pc = plan.piece[i]
            rest, q = divmod(i, ph[0] * ph[1])
            qh, qw = divmod(q, ph[1])
            a, b = divmod(rest, pos[1])
            if pc.r[1] and pc.r[2]:
                assert (pc.tap0[1], pc.tap0[2]) == (qh + 4 * a, qw + 4 * b) and pc.r[0] == 1
            else:
                assert tuple(pc.r) == (0, 0, 0)
            owned += [(pc.tap0[1] + 2 * i1, pc.tap0[2] + 2 * i2) for i1 in range(pc.r[1]) for i2 in range(pc.r[2])]
        assert sorted(owned) == [(i1, i2) for i1 in range(kh) for i2 in range(kw)]
        out, grid = engine.out_dims(d)
        oh, ow_ = (30 + 2 * (kh // 2) - kh) // 2 + 1, (31 + 2 * (kw // 2) - kw) // 2 + 1
        assert out == [1, oh, ow_] and grid == [1, (oh + 1) // 2 + pos[0] - 1, (ow_ + 1) // 2 + pos[1] - 1]
    bad = engine.make_desc((2, 8, 30, 31), (4, 8, 7, 7), torch.float16, 2, 3, 3, stacked=2)      # tile 3 is for stride 1
    with pytest.raises(NotImplementedError):
        engine.plan_conv(bad)
    s = engine._stack
    assert s(None, torch.float16, 2, False, (64, 64, 7, 7), 2, 4) == 2 and s(None, torch.bfloat16, 2, False, (64, 3, 8, 7), 2, 2) == 2
    assert s(None, torch.float16, 2, False, (64, 64, 5, 5), 2, 4) is True and s(None, torch.float16, 2, False, (64, 300, 7, 7), 2, 4) is True
    assert s(None, torch.float16, 3, False, (64, 64, 7, 7, 7), 2, 2) == 2 and s(None, torch.float16, 3, False, (64, 64, 3, 3, 3), 2, 2) is True and s(None, torch.float32, 2, False, (64, 64, 7, 7), 2, 2) is False


def test_modules_pick_tile_2_for_layers_the_fused_kernel_takes():
    """The cached U of a module must be the F(2,3) one wherever wc_conv_forward runs its fused kernel."""
    import pytorch_winoconv_amd as pkg
    from pytorch_winoconv_amd import engine
    assert pkg.WinoConv2d(64, 64, 3, padding=1)._tile_for(torch.float16) == 2
    assert pkg.WinoConv2d(64, 64, 3, padding=1)._tile_for(torch.float32) == 2       # fp32: fused where it beats F(4,3)
    assert pkg.WinoConv2d(64, 128, 3, padding=1)._tile_for(torch.float32) == 4 and pkg.WinoConv2d(32, 256, 3, padding=1)._tile_for(torch.float32) == 2
    assert pkg.WinoConv2d(64, 64, 3, padding=1, output_block=4)._tile_for(torch.float16) == 4
    assert pkg.WinoConv2d(64, 1024, 3, padding=1)._tile_for(torch.float16) == 4     # too many output channels
    assert pkg.WinoConv2d(96, 64, 3, padding=1)._tile_for(torch.float16) == 4       # no kernel for channels padded to 96
    assert pkg.WinoConv2d(128, 128, 3, padding=1)._tile_for(torch.float16) == 2 and pkg.WinoConv2d(160, 64, 3, padding=1)._tile_for(torch.float16) == 4
    assert pkg.WinoConv2d(64, 64, 5, padding=2)._tile_for(torch.float16) == 4
    assert pkg.WinoConv2d(64, 64, 3, stride=2, padding=1)._tile_for(torch.float16) == 4
    t = engine.thin_layer
    assert t(torch.float16, 2, 64, 512, (3, 3), 1) and not t(torch.float16, 2, 64, 513, (3, 3), 1)
    assert t(torch.float16, 2, 128, 256, (3, 3), 1) and not t(torch.float16, 2, 128, 257, (3, 3), 1) and not t(torch.float16, 2, 96, 8, (3, 3), 1)
    assert t(torch.float16, 2, 64, 128, (3, 3), 1) and t(torch.bfloat16, 2, 16, 8, (3, 3), (1, 1))
    assert t(torch.float16, 2, 40, 8, (3, 3), 1) and not t(torch.float16, 2, 42, 8, (3, 3), 1)   # 4 channels per thread
    assert t(torch.float16, 2, 30, 8, (3, 3), 1) and not t(torch.float16, 2, 7, 8, (3, 3), 1)    # 2 channels per thread
    assert t(torch.float16, 2, 3, 64, (3, 3), 1) and t(torch.float32, 2, 3, 64, (3, 3), 1) and t(torch.float32, 2, 1, 512, (3, 3), 1)   # first layers
    assert not t(torch.float32, 2, 5, 64, (3, 3), 1) and not t(torch.float32, 2, 3, 600, (3, 3), 1)
    assert not t(torch.float16, 3, 64, 64, (3, 3), 1)
    assert t(torch.float32, 2, 64, 256, (3, 3), 1) and not t(torch.float32, 2, 64, 257, (3, 3), 1)      # fp32: up to 64 channels
    assert t(torch.float32, 2, 32, 512, (3, 3), 1) and not t(torch.float32, 2, 66, 64, (3, 3), 1) and not t(torch.float32, 2, 33, 64, (3, 3), 1)
    tp = engine.thin_preferred
    assert tp(torch.float32, 2, 64, 64, (3, 3), 1) and not tp(torch.float32, 2, 64, 128, (3, 3), 1) and tp(torch.float32, 2, 32, 512, (3, 3), 1)
    assert tp(torch.float16, 2, 128, 256, (3, 3), 1) and tp(torch.float32, 2, 3, 64, (3, 3), 1)


def test_product_generator_equals_oracle_generator():
    """pytorch_winoconv_amd.wincnn (Lagrange-basis form) against oracle.cook_toom (the
    reference generator's steps), exact rationals, and against the reference's F(2,9) literals."""
    import json, os
    from fractions import Fraction
    from oracle import cook_toom
    from pytorch_winoconv_amd import wincnn
    cases = [((0, 1, -1), 2, 3), ((0, 1, -1, 2, -2), 4, 3), ((0, 1, -1, 2), 4, 2), ((0, 1, -1, 2), 2, 4),
             (cook_toom.POINTS_REF, 2, 6), (cook_toom.POINTS_REF, 2, 7), (cook_toom.POINTS_REF, 9, 5)]
    for pts, m, r in cases:
        a = wincnn.cookToomFilter(pts, m, r)
        b = cook_toom.cook_toom_exact(pts, m, r)
        assert a[0] == b[0] and a[1] == b[1] and a[2] == b[2], (m, r)
    with open(os.path.join(os.path.dirname(__file__), "golden", "cook_toom_f29.json")) as f:
        g = json.load(f)
    AT, G, BT = wincnn.cookToomFilter(g["points"], g["m"], g["r"])
    frac = lambda M: [[Fraction(v) for v in row] for row in M]
    assert AT == frac(g["AT"]) and G == frac(g["G"]) and BT == frac(g["BT"])
    with open(os.path.join(os.path.dirname(__file__), "golden", "cook_toom_reference_tables.json")) as f:
        for t in json.load(f)["tables"]:                             # the reference generator's own output
            got = wincnn.cookToomFilter(t["points"], t["m"], t["r"])
            assert got[0] == frac(t["AT"]) and got[1] == frac(t["G"]) and got[2] == frac(t["BT"])
    with pytest.raises(ValueError):
        wincnn.cookToomFilter((0, 1), 2, 3)                          # too few points


def test_reference_names_are_importable():
    for name in ("AddGPU", "Foo", "WinoSplit", "WinoConcat", "DWM", "add_gpu", "wino_split", "wino_concat",
                 "winograd_conv", "split_and_concat", "Wino", "Dwm", "WinoConv2d", "WinoConv3d"):
        assert hasattr(pkg, name), name
    for mod, names in (("dwm", ("dwm2d", "dwm3d", "dwm2d_", "dwm3d_")),
                       ("matrix_conv", ("conv16", "conv32", "conv", "base_conv32", "matrix_alloc", "A", "G", "B")),
                       ("matrix_conv3d", ("conv16", "conv32", "conv", "base_conv32"))):
        for n in names:
            assert hasattr(getattr(pkg, mod), n), (mod, n)
    f = pkg.Foo(); f.setKey(3)
    assert f.getKey() == 3 and "3" in repr(f)


def test_module_tables_equal_oracle_tables():
    import numpy as np
    from oracle import cook_toom
    for key in ((2, 1), (2, 2), (2, 3), (4, 1), (4, 2), (4, 3), (2, 4), (2, 5), (2, 6), (2, 7)):
        AT, G, BT = cook_toom.matrices(*key)
        assert np.allclose(pkg.matrix_conv.A[key], AT, atol=1e-16, rtol=0)
        assert np.allclose(pkg.matrix_conv.G[key], G, atol=1e-16, rtol=0)
        assert np.allclose(pkg.matrix_conv.B[key], BT, atol=1e-16, rtol=0)


@pytest.mark.parametrize("N,C,K,H,k,m,chosen", [
    # short reductions (kh kw C <= 3200): always
    (32, 128, 128, 112, 3, 2, 1), (64, 256, 256, 56, 3, 4, 1), (32, 128, 128, 112, 4, 4, 1), (32, 128, 128, 112, 5, 4, 1),
    (2, 64, 64, 28, 3, 2, 1), (2, 32, 64, 28, 5, 2, 1), (32, 64, 128, 112, 7, 2, 1),
    # at most 64 output channels: kernels of at most 25 taps only
    (32, 64, 64, 224, 7, 2, 0), (2, 32, 8, 28, 7, 2, 0), (32, 128, 64, 112, 7, 4, 0),
    # long reductions need pixels x channels >= 4 M
    (64, 512, 512, 14, 3, 4, 0), (128, 512, 512, 14, 3, 2, 0), (64, 256, 256, 28, 7, 2, 0), (2, 128, 128, 28, 7, 2, 0),
    # ... then: against the shared-input plan (7x7 and 8x8) yes
    (32, 128, 128, 112, 7, 2, 1), (32, 128, 128, 112, 7, 4, 1), (32, 96, 96, 112, 7, 4, 1), (32, 128, 128, 112, 8, 4, 1),
    # against stacked F(2,r) pieces always; against stacked F(4,r) pieces at 4x4, from 9x9 on, and between for
    # reductions of at most 4800
    (32, 128, 128, 112, 6, 2, 1), (32, 128, 128, 112, 6, 4, 1), (64, 256, 256, 56, 5, 2, 1), (64, 256, 256, 56, 5, 4, 0),
    (64, 256, 512, 28, 6, 4, 0), (32, 256, 256, 56, 4, 4, 1), (32, 128, 128, 112, 9, 4, 1), (32, 128, 128, 112, 9, 2, 1),
    (32, 64, 64, 112, 9, 2, 1)])
def test_the_library_chooses_the_direct_form_where_it_measured_faster(N, C, K, H, k, m, chosen):
    """Each stride-2 layer of the sweep behind the rule, on the side of the crossover it measured on."""
    d = engine.make_desc((N, C, H, H), (K, C, k, k), torch.float16, 2, k // 2, m, stacked=None)
    assert d.direct == chosen
    assert engine.make_desc((N, C, H, H), (K, C, k, k), torch.bfloat16, 2, k // 2, m, stacked=None).direct == chosen
    # fp32: 3x3 kernels over at most 128 channels only
    assert engine.make_desc((N, C, H, H), (K, C, k, k), torch.float32, 2, k // 2, m, stacked=None).direct == int(k <= 3 and C <= 128)


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16, torch.float32])
def test_one_tap_kernels_take_the_direct_form(dtype):
    """1x1 kernels at either stride, every type, where the operands allow it (whole reduction blocks of channels,
    16-byte rows of y); never when ruled out, never with an explicit plan form."""
    for stride in (1, 2):
        for m in (2, 4):
            assert engine.make_desc((4, 64, 28, 28), (128, 64, 1, 1), dtype, stride, 0, m, stacked=None).direct == 1
    assert engine.make_desc((4, 64, 28, 28), (128, 64, 1, 1), dtype, 1, 0, 2, stacked=None, direct=False).direct == 0
    assert engine.make_desc((4, 64, 28, 28), (128, 64, 1, 1), dtype, 1, 0, 2, stacked=False).direct == 0
    assert engine.make_desc((4, 20, 28, 28), (128, 20, 1, 1), dtype, 1, 0, 2, stacked=None).direct == 0          # 20 channels
    assert engine.make_desc((4, 64, 28, 28), (100, 64, 1, 1), dtype, 1, 0, 2, stacked=None).direct == 0          # K no multiple of 8
    assert engine.make_desc((4, 48, 28, 28), (128, 48, 1, 1), dtype, 1, 0, 2, stacked=None).direct == (1 if dtype == torch.float32 else 0)
    assert engine.make_desc((4, 64, 28, 28), (128, 64, 1, 3), dtype, 1, (0, 1), 2, stacked=None).direct == 0     # three taps, stride 1


def test_the_test_hook_is_inert_in_a_process_that_did_not_opt_in():
    """wc_test_gemm_override changes what launches do, so it works only where WINOCONV_TEST_HOOKS=1 was in the
    environment before its first call (this suite sets it in conftest.py); elsewhere it refuses."""
    import subprocess
    import sys
    code = ("import sys; sys.path.insert(0, %r)\n"
            "from pytorch_winoconv_amd import _lib\n"
            "lib = _lib.load()\n"
            "rc = lib.wc_test_gemm_override(0, 1)\n"
            "print(rc, lib.wc_last_error().decode())\n" % os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
    env = {k: v for k, v in os.environ.items() if k != "WINOCONV_TEST_HOOKS"}
    out = subprocess.run([sys.executable, "-c", code], env=env, capture_output=True, text=True, check=True).stdout
    assert out.split()[0] == str(_lib.WC_ERR_UNSUPPORTED) and "WINOCONV_TEST_HOOKS" in out
    lib = _lib.load()
    assert lib.wc_test_gemm_override(-1, 1) == 0            # this process opted in
