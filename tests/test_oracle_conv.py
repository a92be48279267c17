"""Pins oracle.winograd: every stage composed must equal fp64 torch convolution, two
independently written pipelines must agree, and integer data must come out bit-exact."""
import pytest
import torch
import torch.nn.functional as F

from oracle import winograd as ow

CASES = [
    ((2, 5, 9, 11), (4, 5, 3, 3), 1, 1, 2), ((2, 5, 9, 11), (4, 5, 3, 3), 1, 1, 4),
    ((1, 3, 10, 10), (5, 3, 3, 3), 1, 0, 2), ((2, 4, 12, 13), (3, 4, 5, 5), 1, 2, 2),
    ((1, 4, 12, 12), (3, 4, 7, 7), 1, 3, 2), ((1, 2, 13, 13), (3, 2, 9, 9), 1, 4, 2),
    ((1, 2, 14, 14), (3, 2, 10, 10), 1, 0, 2), ((1, 2, 11, 12), (3, 2, 4, 3), 1, 0, 2),
    ((1, 2, 11, 12), (3, 2, 6, 8), 1, 2, 2),
    ((2, 4, 12, 13), (3, 4, 3, 3), 2, 1, 2), ((1, 4, 15, 14), (3, 4, 7, 7), 2, 3, 2),
    ((1, 4, 15, 14), (3, 4, 5, 5), 2, 2, 2),
    ((2, 4, 12, 13), (3, 4, 5, 5), 1, 2, 4), ((1, 4, 12, 12), (3, 4, 7, 7), 1, 3, 4),
    ((1, 2, 11, 12), (3, 2, 4, 3), 1, 0, 4), ((1, 4, 15, 14), (3, 4, 7, 7), 2, 3, 4),
    ((2, 4, 12, 13), (3, 4, 3, 3), 2, 1, 4),
    ((2, 4, 6, 9, 11), (3, 4, 3, 3, 3), 1, 1, 2), ((1, 3, 7, 9, 8), (2, 3, 5, 5, 5), 1, 2, 2),
    ((1, 3, 6, 8, 8), (2, 3, 2, 3, 1), 1, 0, 2), ((1, 2, 9, 9, 9), (2, 2, 3, 3, 3), 2, 1, 2),
]


def _conv(x, w, b, s, p):
    return (F.conv2d if x.dim() == 4 else F.conv3d)(x, w, b, stride=s, padding=p)


@pytest.mark.parametrize("case", CASES)
def test_dwm_conv_equals_fp64_convolution(case):
    xs, ws, s, p, m = case
    g = torch.Generator().manual_seed(0)
    x = torch.randn(*xs, dtype=torch.float64, generator=g)
    w = torch.randn(*ws, dtype=torch.float64, generator=g)
    b = torch.randn(ws[0], dtype=torch.float64, generator=g)
    y = ow.dwm_conv(x, w, b, s, p, m, "fp64")
    ref = _conv(x, w, b, s, p)
    assert y.shape == ref.shape
    assert float((y - ref).abs().max() / ref.abs().max()) < 1e-12


@pytest.mark.parametrize("case", [c for c in CASES if c[4] == 2])
def test_integer_data_is_bit_exact_in_fp32(case):
    """F(2,r): G holds only 0, 1, 1/2, BT and AT only 0, +-1.  Integer inputs and weights in units
    of 4 (2-D) / 8 (3-D) keep every intermediate an exactly representable integer, so fp32
    Winograd must equal direct convolution bit for bit (a dropped term, a wrong sign or a
    transposed index cannot hide behind a tolerance)."""
    xs, ws, s, p, m = case
    g = torch.Generator().manual_seed(1)
    unit = 4 if len(xs) == 4 else 8
    x = torch.randint(-3, 4, xs, generator=g).float()
    w = (torch.randint(-2, 3, ws, generator=g) * unit).float()
    y = ow.dwm_conv(x, w, None, s, p, m, "fp32")
    assert torch.equal(y.double(), _conv(x.double(), w.double(), None, s, p))


@pytest.mark.parametrize("xs,ws,m", [((2, 3, 10, 11), (4, 3, 3, 3), 2), ((1, 3, 14, 14), (4, 3, 3, 3), 4),
                                      ((1, 2, 12, 12), (3, 2, 2, 3), 2), ((2, 3, 6, 10, 11), (4, 3, 3, 3, 3), 2)])
def test_matrix_conv_pipeline_agrees_with_native_pipeline(xs, ws, m):
    """The (P,C,a,a)-tile PyTorch path (matrix_conv.py:112-254) and the channel-last native path
    (split_kernel.cu:14-203) are written separately here; on a single-piece kernel they must agree."""
    g = torch.Generator().manual_seed(2)
    x = torch.randn(*xs, dtype=torch.float64, generator=g)
    w = torch.randn(*ws, dtype=torch.float64, generator=g)
    a = ow.matrix_conv(x, w, m, "fp64")
    b = ow.dwm_conv(x, w, None, 1, 0, m, "fp64")
    assert a.shape == b.shape and float((a - b).abs().max()) < 1e-12
    assert float((a - _conv(x, w, None, 1, 0)).abs().max()) < 1e-12


def test_stage_layouts():
    """Buffer shapes of the native path: U (T,K,C), V (T,P,C), M (T,P,K), element order
    (d*a_h + h)*a_w + w; checked on a one-hot input against the kernel's window formula
    2*tile - pad + i (split_kernel.cu:78-100)."""
    x = torch.zeros(1, 2, 8, 8, dtype=torch.float64)
    x[0, 1, 3, 4] = 1.0
    w = torch.zeros(3, 2, 3, 3, dtype=torch.float64)
    st = {}
    ow.dwm_conv(x, w, None, 1, 1, 2, "fp64", st)
    V = st["V"]
    assert V.shape == (16, 16, 2) and st["U"].shape == (16, 3, 2) and st["M"].shape == (16, 16, 3)
    # tile (h=2, w=2) sees the pixel at window offset (3 - (2*2-1), 4 - (2*2-1)) = (0, 1)
    BT = torch.tensor([[1., 0, -1, 0], [0, 1, 1, 0], [0, -1, 1, 0], [0, 1, 0, -1]], dtype=torch.float64)
    d = torch.zeros(4, 4, dtype=torch.float64); d[0, 1] = 1
    want = (BT @ d @ BT.T).reshape(16)
    assert torch.equal(V[:, 2 * 4 + 2, 1], want)
    assert torch.count_nonzero(V[:, :, 0]) == 0


def test_fp16_discipline_is_within_the_stated_tolerance():
    g = torch.Generator().manual_seed(3)
    x = torch.randn(2, 32, 16, 16, generator=g).half()
    w = (torch.randn(32, 32, 3, 3, generator=g) * (2 / 288) ** .5).half()
    ref = _conv(x.double(), w.double(), None, 1, 1)
    for m in (2, 4):
        y = ow.dwm_conv(x, w, None, 1, 1, m, "fp16")
        assert y.dtype == torch.float16
        assert float((y.double() - ref).abs().max() / ref.abs().max()) < 2e-2


STACKED_CASES = [
    ((2, 5, 13, 14), (6, 5, 5, 5), 1, 2, 4), ((1, 4, 15, 16), (3, 4, 7, 7), 1, 3, 2),
    ((2, 3, 15, 14), (4, 3, 7, 7), 2, 3, 4), ((1, 4, 12, 12), (3, 4, 3, 3), 2, 1, 2),
    ((1, 3, 10, 11), (2, 3, 4, 6), 1, (1, 2), 2), ((1, 3, 20, 21), (2, 3, 10, 9), 1, 4, 2),
]


@pytest.mark.parametrize("case", STACKED_CASES)
def test_stacked_pieces_give_the_same_convolution(case):
    """Pieces summed by the batched product instead of after their output transforms: the same
    convolution in fp64, the integer-exact property of F(2,r) in fp32, and the buffer shapes
    (T of ONE shared tile, the pieces side by side along the reduction axis)."""
    xs, ws, s, p, m = case
    g = torch.Generator().manual_seed(2)
    x = torch.randn(*xs, dtype=torch.float64, generator=g)
    w = torch.randn(*ws, dtype=torch.float64, generator=g)
    b = torch.randn(ws[0], dtype=torch.float64, generator=g)
    st = {}
    y = ow.dwm_conv(x, w, b, s, p, m, "fp64", st, stacked=True)
    ref = _conv(x, w, b, s, p)
    assert y.shape == ref.shape and float((y - ref).abs().max() / ref.abs().max()) < 1e-12
    plain = ow.conv_plan(xs, ws, s, p, m)
    n = len(plain["pieces"])
    rmax = [max(pc["axes"][ax][2] for pc in plain["pieces"]) for ax in (1, 2)]
    T = (m + rmax[0] - 1) * (m + rmax[1] - 1)
    P = st["V"].shape[1]
    assert st["U"].shape == (T, ws[0], n * xs[1]) and st["V"].shape == (T, P, n * xs[1])
    assert st["M"].shape == (T, P, ws[0]) and T <= plain["T_total"]
    if m == 2:
        xi = torch.randint(-3, 4, xs, generator=g).float()
        wi = (torch.randint(-2, 3, ws, generator=g) * 4).float()
        yi = ow.dwm_conv(xi, wi, None, s, p, m, "fp32", stacked=True)
        assert torch.equal(yi.double(), _conv(xi.double(), wi.double(), None, s, p))


@pytest.mark.parametrize("case", [
    ((2, 3, 9, 10), (4, 3, 5, 5), 2), ((1, 2, 12, 11), (3, 2, 7, 4), (3, 1)), ((1, 3, 9, 9), (2, 3, 3, 3), 1),
    ((1, 2, 8, 9), (2, 2, 10, 2), (4, 0)), ((1, 2, 6, 8, 7), (3, 2, 3, 5, 4), (1, 2, 1)), ((2, 2, 5, 6, 6), (2, 2, 1, 5, 5), (0, 2, 2)),
])
def test_pair_pieces_give_the_same_convolution(case):
    """The split into pieces of two taps (not the reference's rule of three): pieces start at even
    taps 0, 2, 4, ..., together they own every tap once, the stacked sum over them is the convolution
    in fp64, and exactly so on small integers in fp32 (G of F(2,2) only halves)."""
    from oracle import split_plan as sp
    xs, ws, p = case
    for k in range(1, 11):
        pieces = sp.axis_pairs(k)
        assert [t for t, _, _ in pieces] == list(range(0, k, 2))
        assert sorted(t + j for t, _, n in pieces for j in range(n)) == list(range(k))
    g = torch.Generator().manual_seed(8)
    x = torch.randn(*xs, dtype=torch.float64, generator=g)
    w = torch.randn(*ws, dtype=torch.float64, generator=g)
    b = torch.randn(ws[0], dtype=torch.float64, generator=g)
    st = {}
    y = ow.dwm_conv(x, w, b, 1, p, 2, "fp64", st, stacked=2)
    ref = _conv(x, w, b, 1, p)
    assert y.shape == ref.shape and float((y - ref).abs().max() / ref.abs().max()) < 1e-12
    n = 1
    for k in ws[2:]:
        n *= (k + 1) // 2
    assert len(st["plan"]["pieces"]) == n and st["U"].shape[2] == n * xs[1]
    xi = torch.randint(-3, 4, xs, generator=g).float()
    wi = (torch.randint(-2, 3, ws, generator=g) * 8).float()
    yi = ow.dwm_conv(xi, wi, None, 1, p, 2, "fp32", stacked=2)
    assert torch.equal(yi.double(), _conv(xi.double(), wi.double(), None, 1, p))


@pytest.mark.parametrize("case", [
    ((2, 3, 13, 12), (4, 3, 7, 7), 3), ((1, 2, 12, 11), (3, 2, 5, 4), (2, 1)), ((1, 3, 9, 9), (2, 3, 3, 3), 1),
    ((1, 2, 15, 9), (2, 2, 8, 2), (4, 0)), ((1, 2, 8, 9, 7), (3, 2, 3, 5, 2), 1), ((1, 2, 9, 10), (2, 2, 1, 6), (0, 2)),
])
def test_pair_pieces_of_the_parity_phases_give_the_stride_2_convolution(case):
    """Stride 2 with two-tap pieces: the taps of an axis are separated by parity, then each parity's
    taps are cut into pairs.  Together the pieces own every tap once, their tap step is 2, and the
    stacked sum over them is the strided convolution: in fp64, and exactly on small integers in fp32."""
    from oracle import split_plan as sp
    xs, ws, p = case
    for k in range(1, 11):
        pieces, _ = sp.conv_pieces([1, 1, k], stride=2, m=2, degenerate_depth=True, pairs=True)
        taps = sorted(pc["axes"][2][0] + 2 * j for pc in pieces for j in range(pc["axes"][2][2]))
        assert taps == list(range(k)) and all(pc["axes"][2][1] == 2 and 1 <= pc["axes"][2][2] <= 2 for pc in pieces)
    g = torch.Generator().manual_seed(9)
    x = torch.randn(*xs, dtype=torch.float64, generator=g)
    w = torch.randn(*ws, dtype=torch.float64, generator=g)
    b = torch.randn(ws[0], dtype=torch.float64, generator=g)
    y = ow.dwm_conv(x, w, b, 2, p, 2, "fp64", stacked=2)
    ref = _conv(x, w, b, 2, p)
    assert y.shape == ref.shape and float((y - ref).abs().max() / ref.abs().max()) < 1e-12
    xi = torch.randint(-3, 4, xs, generator=g).float()
    wi = (torch.randint(-2, 3, ws, generator=g) * 8).float()
    yi = ow.dwm_conv(xi, wi, None, 2, p, 2, "fp32", stacked=2)
    assert torch.equal(yi.double(), _conv(xi.double(), wi.double(), None, 2, p))
