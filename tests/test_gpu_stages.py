"""Parity of every HIP stage (called through the C ABI) against the CPU oracle."""
import pytest
import torch

from oracle import tiles as otiles
from oracle import winograd as ow
from pytorch_winoconv_amd import engine, Split_and_Concat

pytestmark = pytest.mark.gpu

DISC = {torch.float32: "fp32", torch.float16: "fp16"}


def _rel(a, b):
    a, b = a.double().cpu(), b.double().cpu()
    return float((a - b).abs().max() / b.abs().max().clamp_min(1e-30))


# ------------------------------------------------------------------ split / concat: bit-exact
@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("shape,wshape,m", [
    ((2, 5, 9, 11), (3, 5, 3, 3), 2),
    ((1, 70, 8, 8), (3, 70, 3, 3), 2),
    ((2, 64, 14, 14), (3, 64, 3, 3), 4),
    ((1, 3, 12, 7), (3, 3, 5, 5), 2),
    ((2, 6, 6, 7, 9), (3, 6, 3, 3, 3), 2),
    ((1, 130, 5, 6, 6), (3, 130, 2, 3, 2), 2),
    # channel counts that take the vectorised kernels (a row of up to 8 tiles per workgroup):
    ((2, 64, 37, 41), (3, 64, 3, 3), 2),             # 20 tiles per row: full and partial groups
    ((1, 72, 30, 19), (3, 72, 3, 3), 4),             # a partial channel chunk (72 = 64 + 8), 6 x 6 tiles
    ((2, 8, 21, 23), (3, 8, 5, 5), 2),               # 6 x 6 tiles with step 2
    ((1, 136, 9, 11, 13), (3, 136, 3, 3, 3), 2),     # 4 x 4 x 4 tiles
    ((1, 16, 7, 20, 22), (3, 16, 3, 3, 3), 4),       # 6 x 6 x 6 tiles: few tiles fit the staging buffer
    ((3, 256, 14, 14), (3, 256, 1, 1), 2),           # 2 x 2 tiles without overlap
    ((1, 72, 20, 61), (3, 72, 3, 3), 4),             # 6 x 6 tiles, 15 per row (8 + 7), odd width, partial channel chunk
    ((2, 128, 18, 35), (3, 128, 3, 3), 2),           # 4 x 4 tiles, 17 per row (8 + 8 + 1)
])
def test_wino_split_bit_exact(dev, dtype, shape, wshape, m):
    torch.manual_seed(1)
    x = torch.randn(*shape).to(dtype)
    want = torch.from_numpy(otiles.wino_split(x.numpy(), wshape, m))
    got = Split_and_Concat.wino_split(x.to(dev), wshape, m)
    assert got.shape == want.shape
    assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("osize,K,B,m", [
    ((7, 9), 5, 2, 2), ((8, 8), 70, 1, 2), ((13, 10), 64, 2, 4), ((5, 7, 6), 6, 2, 2), ((4, 4, 5), 130, 1, 2),
    ((37, 41), 64, 2, 2), ((30, 19), 72, 1, 4), ((21, 23), 8, 2, 2), ((9, 11, 13), 136, 1, 2), ((7, 20, 22), 16, 1, 4),
    ((56, 56), 256, 2, 4), ((30, 61), 72, 1, 4), ((17, 35), 128, 2, 2),
])
def test_wino_concat_bit_exact(dev, dtype, osize, K, B, m):
    torch.manual_seed(2)
    n = [(o + m - 1) // m for o in osize]
    P = B
    for v in n:
        P *= v
    t = torch.randn(P, K, *([m] * len(osize))).to(dtype)
    want = torch.from_numpy(otiles.wino_concat(t.numpy(), osize, m))
    got = Split_and_Concat.wino_concat(t.to(dev), osize, m)
    assert got.shape == want.shape
    assert torch.equal(got.cpu(), want)


# ------------------------------------------------------------------ transforms and GEMM
CASES = [
    # x shape, w shape, stride, pad, m
    ((2, 8, 9, 11), (12, 8, 3, 3), 1, 1, 2),
    ((2, 8, 9, 11), (12, 8, 3, 3), 1, 1, 4),
    ((1, 3, 10, 10), (5, 3, 3, 3), 1, 0, 2),
    ((2, 16, 12, 13), (8, 16, 5, 5), 1, 2, 2),
    ((1, 8, 12, 12), (8, 8, 7, 7), 1, 3, 2),
    ((2, 8, 12, 13), (8, 8, 3, 3), 2, 1, 2),
    ((1, 8, 15, 14), (4, 8, 7, 7), 2, 3, 2),
    ((2, 16, 12, 13), (8, 16, 5, 5), 1, 2, 4),
    ((1, 8, 12, 12), (8, 8, 7, 7), 1, 3, 4),
    ((2, 8, 12, 13), (8, 8, 3, 3), 2, 1, 4),
    ((1, 8, 15, 14), (4, 8, 7, 7), 2, 3, 4),
    ((1, 6, 14, 14), (5, 6, 4, 3), 1, 0, 4),
    ((2, 8, 6, 9, 11), (8, 8, 3, 3, 3), 1, 1, 2),
    ((1, 4, 7, 9, 8), (4, 4, 5, 5, 5), 1, 2, 2),
    ((1, 6, 6, 8, 8), (5, 6, 2, 3, 1), 1, 0, 2),
    ((2, 8, 6, 9, 11), (8, 8, 3, 3, 3), 1, 1, 4),       # 3-D tile 2 x 4 x 4
    ((1, 5, 5, 10, 7), (6, 5, 3, 3, 3), 1, 0, 4),
    # whole-kernel tiles F(2,k) x F(2,k) (sixth entry), the reference's matrix_conv arithmetic
    ((2, 8, 12, 13), (8, 8, 4, 4), 1, 1, 2, True),
    ((2, 6, 12, 13), (8, 6, 5, 5), 1, 2, 2, True),
    ((1, 8, 13, 12), (4, 8, 6, 6), 1, 0, 2, True),
    ((1, 8, 12, 14), (8, 8, 7, 7), 1, 3, 2, True),
]


def _setup(case, dtype, dev, seed=0, integer=False):
    xs, ws, stride, pad, m = case[:5]
    whole = len(case) > 5 and case[5]
    g = torch.Generator().manual_seed(seed)
    if integer:
        x = torch.randint(-3, 4, xs, generator=g).float()
        w = torch.randint(-2, 3, ws, generator=g).float()
    else:
        x = torch.randn(*xs, generator=g)
        fan_in = 1
        for v in ws[1:]:
            fan_in *= v
        w = torch.randn(*ws, generator=g) * (2.0 / fan_in) ** 0.5
    x, w = x.to(dtype), w.to(dtype)
    stages = {}
    om = (2, 4, 4) if (m == 4 and len(xs) == 5) else m        # the engine's 3-D "tile 4" is 2 x 4 x 4
    ow.dwm_conv(x, w, None, stride, pad, om, DISC[dtype], stages, whole_kernel=whole)
    desc = engine.make_desc(xs, ws, dtype, stride, pad, m, whole_kernel=whole)
    plan = engine.plan_conv(desc)
    return x, w, stages, desc, plan


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_plan_matches_oracle(dev, dtype, case):
    _, _, stages, desc, plan = _setup(case, dtype, dev)
    op = stages["plan"]
    assert plan.t_total == op["T_total"] and plan.n_pieces == len(op["pieces"])
    for i, pc in enumerate(op["pieces"]):
        assert [a[0] for a in pc["axes"]] == list(plan.piece[i].tap0)
        assert [a[2] for a in pc["axes"]] == list(plan.piece[i].r)
        assert pc["t_offset"] == plan.piece[i].t_offset
    out, grid = engine.out_dims(desc)
    assert out == op["odims"] and grid == op["grid"]


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_filter_transform(dev, dtype, case):
    x, w, stages, desc, plan = _setup(case, dtype, dev)
    U = engine.filter_transform(desc, plan, w.to(dev))
    C = desc.C
    assert torch.count_nonzero(U[:, :, C:]) == 0          # channel padding is zero
    tol = 2e-6 if dtype == torch.float32 else 1.5e-3      # fp16: one rounding of a value <= a few ulp
    assert _rel(U[:, :, :C], stages["U"]) <= tol
    # the reference's (kD, kH, kW, C, K) filter layout (dwm.py:85,133) through strides
    w5 = w.to(dev) if w.dim() == 5 else w.to(dev).unsqueeze(2)
    w_ref_layout = w5.permute(2, 3, 4, 1, 0).contiguous().permute(4, 3, 0, 1, 2)
    if w.dim() == 4:
        w_ref_layout = w_ref_layout[:, :, 0]
    U2 = engine.filter_transform(desc, plan, w_ref_layout)
    assert torch.equal(U, U2)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_input_transform(dev, dtype, case):
    x, w, stages, desc, plan = _setup(case, dtype, dev)
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    C = desc.C
    assert torch.count_nonzero(V[:, :, C:]) == 0
    tol = 2e-6 if dtype == torch.float32 else 1.5e-3
    assert _rel(V[:, :, :C], stages["V"]) <= tol


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
def test_input_transform_integer_exact(dev, dtype, case):
    """BT of F(2,r), r <= 5, and F(4,r) is integer: small integer inputs give bit-identical V."""
    if len(case) > 5 and case[1][2] > 5:
        pytest.skip("BT of F(2,6) and F(2,7) holds thirds: not exact in binary")
    x, w, stages, desc, plan = _setup(case, dtype, dev, integer=True)
    V = engine.input_transform(desc, plan, engine.channel_last(x.to(dev)))
    assert torch.equal(V[:, :, :desc.C].cpu(), stages["V"])


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("T,P,C,K", [
    (4, 100, 32, 64), (16, 784, 64, 64), (3, 300, 96, 40), (2, 257, 160, 130), (36, 512, 256, 256),
    (1, 31, 32, 3), (5, 1000, 64, 512),
])
def test_batched_gemm(dev, dtype, T, P, C, K):
    g = torch.Generator().manual_seed(3)
    V = (torch.randn(T, P, C, generator=g)).to(dtype)
    U = (torch.randn(T, K, C, generator=g) / C ** 0.5).to(dtype)
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    M = engine.batched_gemm(V.to(dev), U.to(dev))
    assert M.shape[2] % 8 == 0
    tol = 1e-5 if dtype == torch.float32 else 2e-3
    assert _rel(M[:, :, :K], want) <= tol


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
def test_batched_gemm_long_reduction_tile(dev, dtype, gemm_override):
    """Cp >= 512 with many workgroups selects the 128 x 256 tile of eight wavefronts: checked
    against an fp64 product computed on the device, and bit for bit against the 256 x 128 tile
    (forced through wc_test_gemm_override), which adds the same products in the same order.
    P = 2001 and K = 264 leave partial tiles on both axes."""
    g = torch.Generator().manual_seed(5)
    T, P, C, K = 36, 2001, 512, 264
    V = torch.randn(T, P, C, generator=g).to(dtype).to(dev)
    U = (torch.randn(T, K, C, generator=g) / C ** 0.5).to(dtype).to(dev)
    M = engine.batched_gemm(V, U)
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    assert _rel(M[:, :, :K], want) <= (2e-3 if dtype == torch.float16 else 8e-3)
    gemm_override(config=0)
    M0 = engine.batched_gemm(V, U)
    assert torch.equal(M[:, :, :K], M0[:, :, :K])


@pytest.mark.parametrize("dtype", [torch.float16, torch.bfloat16])
@pytest.mark.parametrize("T,P,C,K", [
    (3, 1000, 96, 256),        # three reduction steps (the fewest), a partial tile of rows
    (5, 257, 256, 512),        # one row into the second tile, two tiles of channels
    (2, 4096, 160, 256),       # whole tiles
    (40, 300, 128, 256),       # more tiles than workgroups per XCD in a range that does not divide evenly
    (1, 31, 512, 256),         # fewer tiles than workgroups: most return at once
    (60, 1300, 96, 256),       # 360 tiles: some workgroups walk over two
    (41, 1100, 128, 512),      # 410 tiles, ranges of 51 and 52 tiles per XCD
    (60, 1300, 256, 256),      # reductions long enough for the write-out that rides on the next tile: 360 tiles
    (36, 3000, 160, 512),      # ... five steps (the fewest for it), 864 tiles
    (9, 2100, 512, 256),
])
@pytest.mark.parametrize("form", [10, 13])
def test_batched_gemm_persistent_tiles(dev, dtype, T, P, C, K, form, gemm_override):
    """The persistent 256 x 256 kernel (chosen by size for long reductions over many tiles; forced here through
    wc_test_gemm_override so that small shapes reach it): against an fp64 product, and bit for bit against the
    256 x 128 tile of gemm_kernel, which adds the same products in the same order.  Rows of M beyond K are not
    written by either.  Form 13: most of a tile's results ride on the workgroup's next tile (reductions of 160
    channels and more; as 10 below that)."""
    g = torch.Generator().manual_seed(6)
    V = torch.randn(T, P, C, generator=g).to(dtype).to(dev)
    U = (torch.randn(T, K, C, generator=g) / C ** 0.5).to(dtype).to(dev)
    gemm_override(config=form)
    M = engine.batched_gemm(V, U)
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    assert _rel(M[:, :, :K], want) <= (2e-3 if dtype == torch.float16 else 8e-3)
    gemm_override(config=0)
    M0 = engine.batched_gemm(V, U)
    assert torch.equal(M, M0)


def test_batched_gemm_persistent_tiles_integer_exact(dev, gemm_override):
    g = torch.Generator().manual_seed(7)
    V = torch.randint(-4, 5, (7, 700, 96), generator=g).half()
    U = torch.randint(-3, 4, (7, 256, 96), generator=g).half()
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    gemm_override(config=10)
    M = engine.batched_gemm(V.to(dev), U.to(dev))
    assert torch.equal(M.double().cpu(), want)


def test_batched_gemm_persistent_tiles_by_size(dev):
    """A long reduction over three and a half rounds of tiles (the F(4x4,3x3) product of a 512 -> 256 channel layer)
    takes the persistent kernel by itself: first and last batches against fp64."""
    g = torch.Generator().manual_seed(8)
    T, P, C, K = 36, 6500, 512, 256
    V = torch.randn(T, P, C, generator=g).half().to(dev)
    U = (torch.randn(T, K, C, generator=g) / C ** 0.5).half().to(dev)
    M = engine.batched_gemm(V, U)
    want = torch.bmm(V[:4].double(), U[:4].double().transpose(1, 2))
    assert _rel(M[:4], want) <= 2e-3
    want = torch.bmm(V[-2:].double(), U[-2:].double().transpose(1, 2))
    assert _rel(M[-2:], want) <= 2e-3


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
def test_batched_gemm_integer_exact(dev, dtype):
    g = torch.Generator().manual_seed(4)
    V = torch.randint(-4, 5, (6, 333, 64), generator=g).to(dtype)
    U = torch.randint(-3, 4, (6, 72, 64), generator=g).to(dtype)
    want = torch.bmm(V.double(), U.double().transpose(1, 2))
    M = engine.batched_gemm(V.to(dev), U.to(dev))
    assert torch.equal(M[:, :, :72].double().cpu(), want)


@pytest.mark.parametrize("dtype", [torch.float32, torch.float16])
@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("with_bias", [False, True])
def test_output_transform(dev, dtype, case, with_bias):
    x, w, stages, desc, plan = _setup(case, dtype, dev)
    Mo = stages["M"]
    K = desc.K
    ldm = engine._lib.load().wc_padded_channels8(K)
    M = torch.full((Mo.shape[0], Mo.shape[1], ldm), float("nan"), dtype=dtype)
    M[:, :, :K] = Mo
    bias = torch.randn(K).to(dtype) if with_bias else None
    op = stages["plan"]
    want = ow.output_transform(Mo, op["pieces"], desc.N, op["grid"], op["odims"], bias, DISC[dtype])
    got = engine.output_transform(desc, plan, M.to(dev), None if bias is None else bias.to(dev), desc.N)
    assert got.shape == want.shape
    tol = 2e-6 if dtype == torch.float32 else 1.5e-3
    if len(case) > 5:
        # A whole-kernel tile sums alpha^2 large terms that cancel: the fp32 sums of the engine and
        # of the oracle may differ by n * eps * sum |AT_i| |M_i| (n = alpha^2 terms), far more than
        # an ulp of the small result.  Bound the difference by that instead.
        from oracle import cook_toom
        k = case[1][2]
        amp = float(abs(cook_toom.matrices(2, k)[0]).sum(axis=1).max()) ** 2
        slack = (k + 1) ** 2 * 6e-8 * amp * float(Mo.abs().max())
        diff = float((got.double().cpu() - want.double()).abs().max())
        assert diff <= tol * float(want.abs().max()) + slack
        return
    assert _rel(got, want) <= tol
