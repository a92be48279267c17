"""Plans whose pieces share one transformed input (`wc_conv_desc.stacked = 2`): the kernel is cut
into pieces of two taps per axis on the tile F(2,2); a piece that starts at tap (2a, 2b) sees the
transformed input of the first piece a tile rows and b tiles further on, so V holds one piece over
an extended tile grid and the batched GEMM reads every piece's rows at that piece's tile offset.
Nothing the reference does (it splits into pieces of three taps, each with its own transforms:
src/base_conv_launchers.h:58-388); the sum over the pieces is the same convolution.

Pinned by: U and every shifted view of V bit-equal to the CPU oracle's per-piece transforms;
bit-exact integer convolution in fp16 on inputs whose every intermediate is an exactly
representable integer; fp64 convolution (fp16, bf16 2e-2 of the output range) on random shapes."""
import random

import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow
from pytorch_winoconv_amd import _lib, engine

pytestmark = pytest.mark.gpu

CASES = [
    # x shape, w shape, pad
    ((2, 32, 12, 12), (8, 32, 5, 5), 2),
    ((1, 64, 20, 17), (40, 64, 7, 7), 3),
    ((2, 16, 9, 14), (8, 16, 4, 6), (1, 2)),
    ((2, 5, 13, 11), (6, 5, 5, 3), (2, 0)),
    ((1, 40, 30, 30), (33, 40, 7, 7), 3),
    ((2, 32, 10, 10), (8, 32, 3, 3), 1),         # 2 x 2 pieces of a 3 x 3 kernel
    ((2, 24, 10, 10), (8, 24, 10, 9), 4),        # 25 pieces
    ((2, 24, 10, 10), (8, 24, 2, 1), 0),         # one piece: an ordinary plan
    ((3, 128, 28, 28), (128, 128, 5, 5), 2),
    # 3-D
    ((2, 16, 6, 9, 10), (8, 16, 3, 5, 5), (1, 2, 2)),
    ((1, 32, 8, 8, 8), (8, 32, 5, 5, 5), 2),
    ((1, 8, 7, 9, 9), (4, 8, 4, 7, 2), (1, 3, 0)),
    ((2, 32, 5, 10, 10), (8, 32, 1, 5, 5), (0, 2, 2)),       # one-tap depth axis of a 3-D problem
]


def _conv(x, w, b, pad):
    return (F.conv2d if x.dim() == 4 else F.conv3d)(x, w, b, padding=pad)


def _rel(a, r):
    r = r.double()
    return float((a.double().cpu() - r).abs().max() / r.abs().max().clamp_min(1e-30))


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", CASES)
def test_stages_against_the_oracle(dev, dtype, case):
    xs, ws, pad = case
    g = torch.Generator().manual_seed(21)
    x = torch.randn(*xs, generator=g).to(dtype)
    fan = 1
    for v in ws[1:]:
        fan *= v
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    st = {}
    y_oracle = ow.dwm_conv(x, w, b, 1, pad, 2, "fp16" if dtype == torch.float16 else "bf16", st, stacked=2)
    desc = engine.make_desc(xs, ws, dtype, 1, pad, 2, stacked=2)
    plan = engine.plan_conv(desc)
    nn = [1] * (5 - len(ws)) + [(k + 1) // 2 for k in ws[2:]]          # pieces per axis (depth, height, width)
    assert plan.n_pieces == nn[0] * nn[1] * nn[2] == len(st["plan"]["pieces"])
    for i, pc in enumerate(st["plan"]["pieces"]):
        assert list(plan.piece[i].tap0) == [a[0] for a in pc["axes"]] and plan.piece[i].t_offset == 0
    C, N = xs[1], xs[0]
    Cp = _lib.load().wc_padded_channels(C)
    U = engine.filter_transform(desc, plan, w.to(dev))
    assert U.shape == (plan.t_total, ws[0], plan.n_pieces * Cp)
    for i in range(plan.n_pieces):
        assert torch.equal(U[:, :, i * Cp:i * Cp + C].cpu(), st["U"][:, :, i * C:(i + 1) * C])
    # the grid the library reports covers the tiles the pieces reach: n - 1 more per axis than the output's
    out, grid = engine.out_dims(desc)
    own = [g - (n - 1) for g, n in zip(grid, nn)]
    assert own == [(o + 1) // 2 if m > 1 else o for o, m in zip(out, plan.m)]
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    if plan.n_pieces > 1:
        P = N * grid[0] * grid[1] * grid[2]
        assert V.shape == (plan.t_total, P + (nn[0] - 1) * grid[1] * grid[2] + (nn[1] - 1) * grid[2] + nn[2] - 1, Cp)
        Vg = V[:, :P, :C].cpu().reshape(plan.t_total, N, grid[0], grid[1], grid[2], C)
        for a in range(nn[0]):
            for bq in range(nn[1]):
                for c in range(nn[2]):
                    i = (a * nn[1] + bq) * nn[2] + c
                    want = st["V"][:, :, i * C:(i + 1) * C].reshape(plan.t_total, N, own[0], own[1], own[2], C)
                    # piece (a, b, c) = piece 0 moved by (a, b, c) tiles
                    assert torch.equal(Vg[:, :, a:a + own[0], bq:bq + own[1], c:c + own[2]], want), (a, bq, c)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, stacked=2)
    ref = _conv(x.double(), w.double(), b.double(), pad)
    assert tuple(y.shape) == tuple(ref.shape)
    assert _rel(y, ref) <= 2e-2 and _rel(y, y_oracle) <= 1e-2
    y1 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, stacked=True)
    assert _rel(y, y1.cpu()) <= 2e-2
    # a cached filter, and chunked passes, change nothing
    Uc = engine.transform_filter(w.to(dev), xs, 1, pad, 2, stacked=2)
    for chunk in (0, 1):
        assert torch.equal(engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 2, U=Uc, chunk_images=chunk,
                                               stacked=2), y)


@pytest.mark.parametrize("case", [c for c in CASES if c[0][1] <= 64])
def test_exact_on_small_integers(dev, case):
    """x in -3..3, taps multiples of 4 (G of F(2,2) halves): every U, V and product is an integer, and
    with at most 64 channels the sums stay below 2048, exact in fp16 too; only the result is rounded."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(3)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = (4.0 if len(ws) == 4 else 8.0) * torch.randint(-1, 2, ws, generator=g).double()    # G of F(2,2) halves per axis
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    ref = _conv(x, w, b, pad)
    y = engine.conv_forward(x.half().to(dev), w.half().to(dev), b.half().to(dev), 1, pad, 2, stacked=2)
    assert float(ref.abs().max()) < 4096
    assert torch.equal(y.cpu(), ref.half())


@pytest.mark.parametrize("case", [c for c in CASES if c[0][1] <= 64])
def test_one_operand_tile_per_run_is_exact_on_small_integers(dev, case, gemm_override):
    """The product kernel that serves all pieces of a run from one tile of V (chosen by size; here
    forced, so that small shapes with partial tiles, one to five pieces per run and 3-D plane jumps
    reach it): same integer inputs as above, so the other order of its sums changes nothing."""
    gemm_override(rows_mode=2)
    test_exact_on_small_integers(dev, case)


@pytest.mark.parametrize("case", [c for c in CASES if c[0][1] <= 64])
def test_dma_fed_tile_per_run_is_exact_on_small_integers(dev, case, gemm_override):
    """The 512 x 128 tile fed by LDS-DMA (runs of two to five pieces, 16-bit types; chosen by size, here forced so
    that partial tiles in both directions, 3-D plane jumps and tiles that end inside V's tail reach it)."""
    gemm_override(rows_mode=3)
    test_exact_on_small_integers(dev, case)


DMA_CASES = [
    # x shape, w shape, pad, tile: more than one 512-row tile, 128-channel blocks that end early, every run length
    ((2, 64, 40, 36), (136, 64, 7, 7), 3, 2), ((1, 96, 50, 47), (128, 96, 5, 5), 2, 2), ((1, 32, 66, 70), (200, 32, 9, 10), 4, 2),
    ((2, 64, 40, 36), (96, 64, 7, 7), 3, 3), ((1, 32, 80, 80), (64, 32, 5, 5), 2, 3), ((1, 32, 14, 20, 22), (40, 32, 5, 5, 5), 2, 2),
    ((1, 64, 45, 45), (256, 64, 3, 3), 1, 2),
    # more tiles than workgroups: a workgroup walks over two or three tiles of its XCD's range
    ((2, 32, 160, 160), (136, 32, 5, 5), 2, 3), ((1, 32, 200, 190), (128, 32, 7, 7), 3, 2),
    # tiles of enough steps for the write-out that rides on the next tile (runs of 2, 3 and 4 pieces), on more tiles
    # than workgroups
    ((1, 96, 80, 80), (64, 96, 5, 5), 2, 3), ((2, 96, 160, 160), (136, 96, 5, 5), 2, 3), ((2, 64, 200, 190), (128, 64, 7, 7), 3, 3),
    ((2, 64, 150, 150), (128, 64, 7, 7), 3, 2),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", DMA_CASES)
def test_dma_fed_tile_per_run_equals_the_register_staged_one(dev, dtype, case, gemm_override):
    """Both kernels add the pieces of a run and the channel blocks in the same order: bit-identical outputs; and
    against fp64 convolution."""
    xs, ws, pad, m = case
    g = torch.Generator().manual_seed(33)
    x = torch.randn(*xs, generator=g).to(dtype)
    fan = 1
    for v in ws[1:]:
        fan *= v
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    ref = _conv(x.double(), w.double(), b.double(), pad)
    gemm_override(rows_mode=2)
    y2 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, m, stacked=2)
    gemm_override(rows_mode=3)
    y3 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, m, stacked=2)
    assert torch.equal(y2, y3)
    gemm_override(rows_mode=4)          # ... with the write-out of a tile riding on the next one, where the tiles have the steps
    y4 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, m, stacked=2)
    assert torch.equal(y2, y4)
    tol = {2: (3e-3, 2e-2), 3: (1e-2, 5e-2)}[m]             # F(3,3) evaluates at 2 as well: 3.1e-3 in fp16, 2.6e-2 in bf16
    assert _rel(y3, ref) <= tol[dtype == torch.bfloat16]


TILE3 = [c for c in CASES if len(c[0]) == 4 and min(c[1][2:]) >= 3 and max(c[1][2:]) >= 4]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", TILE3)
def test_three_tap_pieces_on_the_shared_tile_f33(dev, dtype, case):
    """Output tile 3: the reference's pieces of three taps (3+3+1 for 7), every one on the tile F(3,3)
    (Cook-Toom over 0, 1, -1, 2), sharing one transformed input.  Stages against the oracle to the
    rounding of the storage type (the matrices are no longer 0 / +-1, so fp32 evaluation order shows);
    result against fp64: fp16 2e-2 of the output range (measured 3e-3), bf16 6e-2 (measured 2-4e-2:
    the Python layer never picks this tile for bf16)."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(31)
    x = torch.randn(*xs, generator=g).to(dtype)
    w = (torch.randn(*ws, generator=g) * (2.0 / (ws[1] * ws[2] * ws[3])) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    st = {}
    y_oracle = ow.dwm_conv(x, w, b, 1, pad, 3, "fp16" if dtype == torch.float16 else "bf16", st, stacked=2)
    desc = engine.make_desc(xs, ws, dtype, 1, pad, 3, stacked=2)
    plan = engine.plan_conv(desc)
    n_h, n_w = (ws[2] + 2) // 3, (ws[3] + 2) // 3
    assert list(plan.m) == [1, 3, 3] and plan.t_total == 25 and plan.n_pieces == n_h * n_w == len(st["plan"]["pieces"])
    C, N = xs[1], xs[0]
    Cp = _lib.load().wc_padded_channels(C)
    tol = 1.5e-3 if dtype == torch.float16 else 1.2e-2
    U = engine.filter_transform(desc, plan, w.to(dev))
    for i in range(plan.n_pieces):
        assert _rel(U[:, :, i * Cp:i * Cp + C], st["U"][:, :, i * C:(i + 1) * C]) <= tol
    (_, oH, oW), (_, gH, gW) = engine.out_dims(desc)
    nH, nW = (oH + 2) // 3, (oW + 2) // 3
    assert (gH, gW) == (nH + n_h - 1, nW + n_w - 1)
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    Vg = V[:, :N * gH * gW, :C].cpu().reshape(25, N, gH, gW, C)
    for a in range(n_h):
        for c in range(n_w):
            i = a * n_w + c
            want = st["V"][:, :, i * C:(i + 1) * C].reshape(25, N, nH, nW, C)
            assert _rel(Vg[:, :, a:a + nH, c:c + nW], want) <= tol, (a, c)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 3, stacked=2)
    ref = F.conv2d(x.double(), w.double(), b.double(), padding=pad)
    assert tuple(y.shape) == tuple(ref.shape)
    assert _rel(y, ref) <= (2e-2 if dtype == torch.float16 else 6e-2) and _rel(y, y_oracle) <= (1e-2 if dtype == torch.float16 else 6e-2)
    if dtype == torch.float16 and max(ws[2:]) >= 5:
        # what a caller who asks for tile 4 gets by default
        assert torch.equal(engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 4), y)
        Uc = engine.transform_filter(w.to(dev), xs, 1, pad, 4)
        assert torch.equal(engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 1, pad, 4, U=Uc, chunk_images=1), y)


def _random_cases(seed, n):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        ks = [rng.choice([2, 3, 4, 5, 7, rng.randint(1, 10)]) for _ in range(2)]
        pad = [rng.randint(0, k - 1) for k in ks]
        sp = [rng.randint(max(k - 2 * p, 1), 16) + rng.randint(0, 8) for k, p in zip(ks, pad)]
        N, C, K = rng.randint(1, 3), rng.choice([1, 3, 8, 17, 32, 40, 65, 128]), rng.choice([1, 4, 6, 9, 32, 33, 72])
        out.append((N, C, K, tuple(sp), tuple(ks), tuple(pad), rng.choice([torch.float16, torch.bfloat16])))
    return out


def _random_cases_3d(seed, n):
    rng = random.Random(seed)
    out = []
    while len(out) < n:
        ks = [rng.choice([1, 2, 3, 4, 5]) for _ in range(3)]
        pad = [rng.randint(0, k - 1) for k in ks]
        sp = [rng.randint(max(k - 2 * p, 1), 7) + rng.randint(0, 5) for k, p in zip(ks, pad)]
        N, C, K = rng.randint(1, 2), rng.choice([1, 3, 8, 17, 32, 40]), rng.choice([1, 4, 6, 9, 32, 33])
        out.append((N, C, K, tuple(sp), tuple(ks), tuple(pad), rng.choice([torch.float16, torch.bfloat16])))
    return out


RANDOM = _random_cases(5, 40) + _random_cases_3d(6, 20)


@pytest.mark.parametrize("case", RANDOM, ids=[str(i) for i in range(len(RANDOM))])
def test_random_shapes(dev, case):
    N, C, K, sp, ks, pad, dtype = case
    g = torch.Generator().manual_seed(N * 1000 + C)
    x = torch.randn(N, C, *sp, generator=g).to(dtype)
    fan = C
    for k in ks:
        fan *= k
    w = (torch.randn(K, C, *ks, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    ref = _conv(x.double(), w.double(), None, pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), None, 1, pad, 2, stacked=2)
    assert tuple(y.shape) == tuple(ref.shape) and _rel(y, ref) <= 2e-2
    if len(ks) == 2 and min(ks) >= 3 and max(ks) >= 4 and dtype == torch.float16:
        y3 = engine.conv_forward(x.to(dev), w.to(dev), None, 1, pad, 3, stacked=2)
        assert tuple(y3.shape) == tuple(ref.shape) and _rel(y3, ref) <= 2e-2


@pytest.mark.parametrize("case", RANDOM[::2], ids=[str(i) for i in range(0, len(RANDOM), 2)])
def test_random_shapes_with_one_operand_tile_per_run(dev, case, gemm_override):
    gemm_override(rows_mode=2)
    test_random_shapes(dev, case)


@pytest.mark.parametrize("case", RANDOM[1::2], ids=[str(i) for i in range(1, len(RANDOM), 2)])
def test_random_shapes_with_the_dma_fed_tile_per_run(dev, case, gemm_override):
    gemm_override(rows_mode=3)
    test_random_shapes(dev, case)


STRIDE2 = [
    # x shape, w shape, pad
    ((2, 8, 20, 21), (4, 8, 7, 7), 3), ((1, 5, 9, 12), (3, 5, 3, 3), 1), ((2, 16, 17, 14), (8, 16, 5, 4), (2, 1)),
    ((1, 8, 11, 13), (6, 8, 2, 1), 0), ((1, 40, 31, 30), (33, 40, 8, 7), (4, 3)), ((2, 24, 23, 25), (8, 24, 10, 9), 4),
    ((1, 8, 9, 10, 11), (4, 8, 3, 5, 3), 1), ((1, 4, 7, 9, 8), (5, 4, 4, 4, 4), (2, 1, 2)), ((1, 64, 33, 35), (72, 64, 7, 7), 3),
]


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("case", STRIDE2)
def test_stride_2_on_the_parity_phases(dev, dtype, case, gemm_override):
    """Stride 2 with a shared transformed input: the even and the odd samples of x are phases side
    by side in the rows of V, the pieces are pairs of a phase's taps.  Against fp64 convolution and
    against the CPU oracle's restatement (pieces with their own V) in the same storage type; once
    more through the product kernel that serves a run of pieces from one operand tile."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(11)
    x = torch.randn(*xs, generator=g).to(dtype)
    fan = ws[1]
    for k in ws[2:]:
        fan *= k
    w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype)
    b = torch.randn(ws[0], generator=g).to(dtype)
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    ref = conv(x.double(), w.double(), b.double(), 2, pad)
    y = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 2, pad, 2, stacked=2)
    assert tuple(y.shape) == tuple(ref.shape) and _rel(y, ref) <= 2e-2
    yo = ow.dwm_conv(x, w, b, 2, pad, 2, "fp16" if dtype == torch.float16 else "bf16", stacked=2)
    assert _rel(y, yo.double()) <= (3e-3 if dtype == torch.float16 else 2e-2)
    U = engine.transform_filter(w.to(dev), xs, 2, pad, 2, stacked=2)
    assert torch.equal(engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 2, pad, 2, U=U, stacked=2), y)
    gemm_override(rows_mode=2)
    y2 = engine.conv_forward(x.to(dev), w.to(dev), b.to(dev), 2, pad, 2, stacked=2)
    assert _rel(y2, ref) <= 2e-2 and _rel(y2, y.double().cpu()) <= (3e-3 if dtype == torch.float16 else 2e-2)


@pytest.mark.parametrize("case", [c for c in STRIDE2 if c[0][1] <= 16])
def test_stride_2_is_exact_on_small_integers(dev, case):
    """x in -3..3, taps multiples of 4 (8 in 3-D): every U, V and product is an integer; with at most 16
    channels in each of the 4 (8) phases the sums stay below 2048, exact in fp16."""
    xs, ws, pad = case
    g = torch.Generator().manual_seed(4)
    x = torch.randint(-3, 4, xs, generator=g).double()
    w = (4.0 if len(ws) == 4 else 8.0) * torch.randint(-1, 2, ws, generator=g).double()
    b = torch.randint(-8, 9, (ws[0],), generator=g).double()
    conv = F.conv2d if len(xs) == 4 else F.conv3d
    ref = conv(x, w, b, 2, pad)
    y = engine.conv_forward(x.half().to(dev), w.half().to(dev), b.half().to(dev), 2, pad, 2, stacked=2)
    assert float(ref.abs().max()) < 2048
    assert torch.equal(y.cpu(), ref.half())


def test_c4_stride_2_layer_at_full_size(dev):
    """Benchmark configuration c4, 7x7 stride 2 (fp16, N=32, 128 channels, 112x112): the default plan is
    the shared-input one; checked against torch's own GPU convolution accumulated in fp32."""
    g = torch.Generator().manual_seed(0)
    x = torch.randn(32, 128, 112, 112, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(128, 128, 7, 7, generator=g) * (2.0 / (128 * 49)) ** 0.5).half().to(dev)
    assert engine._stack(None, torch.float16, 2, False, w.shape, 2, 4) == 2
    y = engine.conv_forward(x, w, None, 2, 3, 4)
    ref = F.conv2d(x.float(), w.float(), None, 2, 3)
    assert tuple(y.shape) == tuple(ref.shape)
    assert float((y.float() - ref).abs().max() / ref.abs().max()) <= 2e-2


@pytest.mark.parametrize("nd,cin,cout,k,sp", [(2, 16, 24, 7, (37, 41)), (3, 8, 16, 7, (13, 12, 15)), (3, 8, 8, 4, (9, 12, 11))])
def test_modules_train_through_the_stride_2_plan(dev, nd, cin, cout, k, sp):
    """WinoConv2d / WinoConv3d at stride 2 with the kernel sizes whose default is the shared-input plan:
    output and all three gradients against fp64 autograd (the weight gradient has no shared-input form
    and runs on stacked pieces, the input gradient is a stride-1 convolution of the zero-filled dy)."""
    import pytorch_winoconv_amd as pkg
    torch.manual_seed(0)
    mod = (pkg.WinoConv2d if nd == 2 else pkg.WinoConv3d)(cin, cout, k, stride=2, padding=k // 2).to(dev).half()
    assert engine._stack(None, torch.float16, nd, False, mod.weight.shape, 2, 2) == 2
    x = torch.randn(2, cin, *sp, device=dev).half().requires_grad_(True)
    y = mod(x)
    xr, wr, br = (t.detach().double().requires_grad_(True) for t in (x, mod.weight, mod.bias))
    yr = (F.conv2d if nd == 2 else F.conv3d)(xr, wr, br, 2, k // 2)
    gy = torch.randn_like(yr)
    y.backward(gy.half())
    yr.backward(gy)
    for got, want in ((y, yr), (x.grad, xr.grad), (mod.weight.grad, wr.grad), (mod.bias.grad, br.grad)):
        assert float((got.detach().double() - want.detach()).abs().max() / want.detach().abs().max()) <= 2e-2


def _bad_tile_4(xs, ws):
    d = engine.make_desc(xs, ws, torch.float16, 1, 1, 2, stacked=2)
    d.m = 4
    return d


def test_what_the_plan_is_not_built_for(dev):
    x = torch.randn(2, 8, 12, 12).half().to(dev)
    w = torch.randn(4, 8, 5, 5).half().to(dev)
    with pytest.raises(NotImplementedError):
        engine.conv_forward(x, w, None, 2, 2, 3, stacked=2)                        # tile 3 at stride 2
    with pytest.raises(NotImplementedError):
        engine.conv_forward(x.float(), w.float(), None, 1, 2, 2, stacked=2)        # fp32 product
    x3, w3 = torch.randn(1, 8, 6, 12, 12).half().to(dev), torch.randn(4, 8, 3, 3, 3).half().to(dev)
    with pytest.raises(NotImplementedError):
        engine.plan_conv(_bad_tile_4(x3.shape, w3.shape))                          # no shared-input form of the 3-D tile 2 x 4 x 4
    # the weight gradient falls back to stacked pieces with their own V; the default picks this plan for the forward pass
    dy = torch.randn(2, 4, 12, 12).half().to(dev)
    dw = engine.conv_backward_weight(x, dy, w.shape, 1, 2, 2, stacked=2)
    assert torch.equal(dw, engine.conv_backward_weight(x, dy, w.shape, 1, 2, 2, stacked=True))
    assert torch.equal(engine.conv_forward(x, w, None, 1, 2, 2), engine.conv_forward(x, w, None, 1, 2, 2, stacked=2))
    assert torch.equal(engine.conv_forward(x, w, None, 1, 2, 4), engine.conv_forward(x, w, None, 1, 2, 3, stacked=2))


def test_c4_layer_at_full_size(dev):
    """N=32, C=K=128, 112x112, 7x7: against the stacked F(2,r) plan (own V per piece) and a sample of fp64."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(32, 128, 112, 112, generator=g).half().to(dev).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(128, 128, 7, 7, generator=g) * (2.0 / (128 * 49)) ** 0.5).half().to(dev)
    y = engine.conv_forward(x, w, None, 1, 3, 2, stacked=2)
    y1 = engine.conv_forward(x, w, None, 1, 3, 2, stacked=True)
    scale = float(y1.float().abs().max())
    assert float((y.float() - y1.float()).abs().max()) <= 4e-3 * scale
    y3 = engine.conv_forward(x, w, None, 1, 3, 3, stacked=2)                     # three-tap pieces on F(3,3)
    assert float((y3.float() - y1.float()).abs().max()) <= 1.5e-2 * scale
    sample = F.conv2d(x[:1].double().cpu(), w.double().cpu(), padding=3)
    assert _rel(y[:1], sample) <= 2e-3
