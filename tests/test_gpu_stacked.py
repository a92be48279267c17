"""DWM plans whose pieces are added by the batched GEMM (`stacked`): every piece is transformed
with the tile of the longest piece and the pieces lie side by side along the reduction axis of U
and V.  The reference adds the pieces after their output transforms (outputAggregate,
src/split_kernel.cu:184-203); the sum is the same.  Checked stage by stage against the CPU oracle
in the same arithmetic discipline, end to end against fp64 torch convolution (fp32 1e-3, fp16 2e-2,
bf16 2e-2 with tile 2 / 2e-1 with tile 4, as everywhere) and against the piece-by-piece path."""
import ctypes
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import _lib, engine

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, w shape, stride, pad, m
    ((2, 5, 13, 14), (6, 5, 5, 5), 1, 2, 4),
    ((1, 4, 15, 16), (3, 4, 7, 7), 1, 3, 2),
    ((2, 3, 15, 14), (4, 3, 7, 7), 2, 3, 4),
    ((1, 4, 12, 12), (3, 4, 3, 3), 2, 1, 2),
    ((1, 3, 10, 11), (2, 3, 4, 6), 1, (1, 2), 2),
    ((1, 3, 20, 21), (2, 3, 10, 9), 1, 4, 2),
    ((2, 40, 30, 30), (33, 40, 5, 5), 1, 2, 4),
    ((3, 64, 28, 28), (64, 64, 7, 7), 2, 3, 2),
    ((1, 3, 9, 9), (2, 3, 3, 3), 1, 1, 4),          # one piece: nothing to stack
]
DISC = {torch.float32: "fp32", torch.float16: "fp16", torch.bfloat16: "bf16"}
STAGE_TOL = {torch.float32: 2e-6, torch.float16: 1.5e-3, torch.bfloat16: 1.2e-2}


def _tol(dtype, m):
    return {torch.float32: 1e-3, torch.float16: 2e-2, torch.bfloat16: 2e-2 if m == 2 else 2e-1}[dtype]


def _rel(a, r):
    r = r.double()
    return float((a.double().cpu() - r).abs().max() / r.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_stacked_stages_and_result(dev, dtype, case):
    xs, ws, stride, pad, m = case
    g = torch.Generator().manual_seed(11)
    fan = ws[1] * ws[2] * ws[3]
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    st = {}
    ow.dwm_conv(x, w, b, stride, pad, m, DISC[dtype], st, stacked=True)

    desc = engine.make_desc(xs, ws, dtype, stride, pad, m, stacked=True)
    plan = engine.plan_conv(desc)
    n, C, K = plan.n_pieces, xs[1], ws[0]
    Cp = _lib.load().wc_padded_channels(C)
    xd, wd, bd = x.to(dev), w.to(dev), b.to(dev)
    U = engine.filter_transform(desc, plan, wd)
    V = engine.input_transform(desc, plan, engine.channel_last(xd))
    assert U.shape == (plan.t_total, K, n * Cp) and V.shape[0] == plan.t_total and V.shape[2] == n * Cp
    for i in range(n):
        # piece i occupies columns [i Cp, i Cp + C); the padding columns are zero
        assert _rel(U[:, :, i * Cp:i * Cp + C], st["U"][:, :, i * C:(i + 1) * C]) <= STAGE_TOL[dtype]
        assert _rel(V[:, :, i * Cp:i * Cp + C], st["V"][:, :, i * C:(i + 1) * C]) <= STAGE_TOL[dtype]
        assert not U[:, :, i * Cp + C:(i + 1) * Cp].any() and not V[:, :, i * Cp + C:(i + 1) * Cp].any()
    M = engine.batched_gemm(V, U)
    assert M.shape[0] == plan.t_total
    tol_m = STAGE_TOL[dtype] * (1 if dtype == torch.float32 else 4)
    assert _rel(M[:, :, :K], st["M"]) <= max(tol_m, 2e-5)
    y_st = engine.output_transform(desc, plan, M, bd, xs[0])
    y = engine.conv_forward(xd, wd, bd, stride, pad, m, stacked=True)
    assert torch.equal(y.permute(0, 2, 3, 1), y_st[:, 0])            # the one-call entry runs the same stages
    assert tuple(y.shape) == tuple(ref.shape) and _rel(y, ref) <= _tol(dtype, m)
    y_pieces = engine.conv_forward(xd, wd, bd, stride, pad, m, stacked=False)
    assert _rel(y, y_pieces.cpu()) <= 2 * _tol(dtype, m)


def test_cached_filter_chunks_and_size_check(dev):
    xs, ws = (5, 24, 30, 29), (16, 24, 5, 5)
    g = torch.Generator().manual_seed(4)
    x = torch.randn(*xs, generator=g).half().to(dev)
    w = (torch.randn(*ws, generator=g) * 0.05).half().to(dev)
    y = engine.conv_forward(x, w, None, 1, 2, 4, stacked=True)
    U = engine.transform_filter(w, xs, 1, 2, 4, stacked=True)
    for chunk in (0, 1, 2):
        assert torch.equal(engine.conv_forward(x, w, None, 1, 2, 4, U=U, chunk_images=chunk, stacked=True), y)
    # the default for 16-bit plans is a stacked form: at stride 2 this one, at stride 1 with 4..8 taps and
    # at most 128 channels the one whose pieces share the transformed input (test_gpu_shared.py)
    assert torch.equal(engine.conv_forward(x, w, None, 2, 2, 4), engine.conv_forward(x, w, None, 2, 2, 4, stacked=True))
    assert torch.equal(engine.transform_filter(w, xs, 2, 2, 4), engine.transform_filter(w, xs, 2, 2, 4, stacked=True))
    assert torch.equal(engine.conv_forward(x, w, None, 1, 2, 4), engine.conv_forward(x, w, None, 1, 2, 3, stacked=2))
    assert torch.equal(engine.conv_forward(x, w, None, 1, 2, 2), engine.conv_forward(x, w, None, 1, 2, 2, stacked=2))
    # a filter transformed for the other form has another size and is refused, not misread
    with pytest.raises(ValueError):
        engine.conv_forward(x, w, None, 1, 2, 4, U=U, stacked=False)
    U_pieces = engine.transform_filter(w, xs, 1, 2, 4, stacked=False)
    with pytest.raises(ValueError):
        engine.conv_forward(x, w, None, 1, 2, 4, U=U_pieces, stacked=True)
    # fp32: stacked by default up to four pieces (5x5), piece by piece beyond (7x7: nine)
    xf, wf = x.float(), w.float()
    assert torch.equal(engine.conv_forward(xf, wf, None, 1, 2, 4), engine.conv_forward(xf, wf, None, 1, 2, 4, stacked=True))
    w7 = torch.randn(16, 24, 7, 7, generator=g).to(dev) * 0.05
    assert torch.equal(engine.conv_forward(xf, w7, None, 1, 3, 4), engine.conv_forward(xf, w7, None, 1, 3, 4, stacked=False))


def _random_cases(seed, n):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        ks = [rng.choice([2, 3, 4, 5, 7, rng.randint(1, 10)]) for _ in range(2)]
        stride = rng.choice([1, 1, 2])
        pad = [rng.randint(0, k - 1) for k in ks]
        sp = [rng.randint(max(k - 2 * p, 1), 16) + rng.randint(0, 8) for k, p in zip(ks, pad)]
        N, C, K = rng.randint(1, 3), rng.choice([1, 3, 8, 17, 32, 40, 65]), rng.choice([1, 4, 6, 9, 32, 33, 72])
        out.append((N, C, K, tuple(sp), tuple(ks), stride, tuple(pad), rng.choice([2, 4]),
                    rng.choice([torch.float32, torch.float16, torch.bfloat16])))
    return out


RANDOM = _random_cases(77, 60)


@pytest.mark.parametrize("case", RANDOM, ids=[str(i) for i in range(len(RANDOM))])
def test_random_shapes_stacked(dev, case):
    N, C, K, sp, ks, stride, pad, m, dtype = case
    g = torch.Generator().manual_seed(hash(case[:8]) % (2 ** 31))
    x = torch.randn(N, C, *sp, generator=g).to(dtype)
    w = (torch.randn(K, C, *ks, generator=g) * (2.0 / (C * ks[0] * ks[1])) ** 0.5).to(dtype)
    b = torch.randn(K, generator=g).to(dtype)
    ref = F.conv2d(x.double(), w.double(), b.double(), stride=stride, padding=pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, m, stacked=True)
    assert tuple(y.shape) == tuple(ref.shape), case
    assert _rel(y, ref) <= _tol(dtype, m), case


GRAD_CASES = CASES[:7] + [((6, 24, 40, 40), (40, 24, 5, 5), 1, 2, 2),      # tile sum split into parts
                          ((8, 72, 40, 40), (136, 72, 5, 5), 1, 2, 4)]     # 128 x 128 product tiles, partial edges


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", GRAD_CASES)
def test_stacked_weight_gradient(dev, dtype, case):
    """The weight gradient of a stacked plan (one dM for all pieces, V with the pieces side by side,
    taps a piece lacks dropped at the end) against fp64 autograd, and against the piece-by-piece
    gradient: taps of pieces that already have the longest tile come out bit-identical."""
    xs, ws, stride, pad, m = case
    g = torch.Generator().manual_seed(21)
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / (ws[1] * ws[2] * ws[3])) ** 0.5).to(dtype)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    y = F.conv2d(xr, wr, stride=stride, padding=pad)
    dy = torch.randn(*y.shape, generator=g).to(dtype)
    gw, = torch.autograd.grad(y, (wr,), dy.double())
    dw = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, stride, pad, m, stacked=True)
    assert dw.dtype == dtype and tuple(dw.shape) == tuple(ws) and _rel(dw, gw) <= _tol(dtype, m)
    dw_pieces = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, stride, pad, m, stacked=False)
    plan = ow.conv_plan(xs, ws, stride, pad, m)
    rmax = [max(pc["axes"][ax][2] for pc in plan["pieces"]) for ax in (1, 2)]
    for pc in plan["pieces"]:
        (h0, hs, hr), (w0, wsx, wr_) = pc["axes"][1], pc["axes"][2]
        if [hr, wr_] == rmax:
            sel = (slice(None), slice(None), slice(h0, h0 + hr * hs, hs), slice(w0, w0 + wr_ * wsx, wsx))
            assert torch.equal(dw[sel], dw_pieces[sel])


CASES_3D = [
    ((1, 6, 7, 9, 8), (5, 6, 5, 5, 5), 1, 2),             # 8 pieces, all padded to F(2,3)^3
    ((2, 3, 6, 10, 9), (4, 3, 4, 5, 3), 1, (1, 2, 1)),    # 2+2, 3+2 and 3 taps: shared tile F(2,2) x F(2,3) x F(2,3)
    ((1, 8, 9, 9, 9), (6, 8, 3, 3, 3), 2, 1),             # stride 2: parity pieces of 2 and 1 taps
    ((1, 40, 6, 12, 12), (33, 40, 7, 3, 5), 1, (3, 1, 2)),
]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES_3D)
def test_stacked_3d(dev, dtype, case):
    """3-D DWM plans (output tile 2) stacked: forward against the oracle and fp64 convolution, the
    weight gradient against fp64 autograd."""
    xs, ws, stride, pad = case
    g = torch.Generator().manual_seed(31)
    fan = ws[1] * ws[2] * ws[3] * ws[4]
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    xr, wr = x.double().requires_grad_(True), w.double().requires_grad_(True)
    ref = F.conv3d(xr, wr, b.double(), stride=stride, padding=pad)
    st = {}
    yo = ow.dwm_conv(x, w, b, stride, pad, 2, DISC[dtype], st, stacked=True)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), stride, pad, 2, stacked=True)
    assert tuple(y.shape) == tuple(ref.shape) and _rel(y, ref.detach()) <= _tol(dtype, 2)
    assert _rel(y, yo) <= 4 * STAGE_TOL[dtype]
    desc = engine.make_desc(xs, ws, dtype, stride, pad, 2, stacked=True)
    plan = engine.plan_conv(desc)
    assert plan.t_total == st["plan"]["T_total"] and plan.n_pieces == len(st["plan"]["pieces"])
    n, C = plan.n_pieces, xs[1]
    Cp = _lib.load().wc_padded_channels(C)
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    U = engine.filter_transform(desc, plan, w.to(dev))
    for i in range(n):
        assert _rel(V[:, :, i * Cp:i * Cp + C], st["V"][:, :, i * C:(i + 1) * C]) <= STAGE_TOL[dtype]
        assert _rel(U[:, :, i * Cp:i * Cp + C], st["U"][:, :, i * C:(i + 1) * C]) <= STAGE_TOL[dtype]
    dy = torch.randn(*ref.shape, generator=g).to(dtype)
    gw, = torch.autograd.grad(ref, (wr,), dy.double())
    dw = engine.conv_backward_weight(x.to(dev), dy.to(dev), ws, stride, pad, 2, stacked=True)
    assert _rel(dw, gw) <= _tol(dtype, 2)
    # tile 4 does not exist for 3-D DWM plans, stacked or not
    with pytest.raises(NotImplementedError):
        engine.plan_conv(engine.make_desc(xs, ws, dtype, stride, pad, 4, stacked=True))
