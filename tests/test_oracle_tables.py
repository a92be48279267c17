"""Pins oracle.cook_toom: the transform matrices every other oracle function builds on.

Independent facts used (none is a retyped copy of the generator's formula):
  * the literal F(2,1), F(2,2), F(2,3) tables of the reference (matrix_conv.py:15-30,
    matrix_convnd.py:20-27) - typed in here from the textbook definition of each and checked
    through the FIR identity rather than compared entry by entry with the oracle's copy;
  * the exact-rational FIR identity  AT . ((G g) o (BT d)) == valid correlation of d with g
    (what wincnn.filterVerify checks symbolically, wincnn.py:73-87), on basis vectors;
  * the published Lavin & Gray F(4x4,3x3) matrices, equal to the reference's commented B25 / G25
    literals (transform.py:29-40);
  * the reference's commented F(2,9) literals A29 / G29 / B29 (transform.py:41-61), kept as data
    in tests/golden/cook_toom_f29.json: a 10 x 10 case with the sign and scaling convention;
  * the output of the reference's own generator (wincnn.py:49-70) for the point sets it uses at
    import (matrix_conv.py:31-36), fractional points included, written once in the build
    container by tests/golden/make_cook_toom_tables.py into
    tests/golden/cook_toom_reference_tables.json (exact rationals);
  * spot formulas of the reference's unrolled kernels (transform_kernels.cu:1191,1587-1588,
    transform_kernels_3d.cu:4998).
"""
from fractions import Fraction

import numpy as np
import pytest

from oracle import cook_toom as ct


def _fir_identity_exact(AT, G, BT, m, r):
    alpha = m + r - 1
    for di in range(alpha):
        for gi in range(r):
            d = [Fraction(int(i == di)) for i in range(alpha)]
            g = [Fraction(int(i == gi)) for i in range(r)]
            U = [sum(Fraction(G[i][j]) * g[j] for j in range(r)) for i in range(alpha)]
            V = [sum(Fraction(BT[i][j]) * d[j] for j in range(alpha)) for i in range(alpha)]
            Y = [sum(Fraction(AT[o][i]) * U[i] * V[i] for i in range(alpha)) for o in range(m)]
            want = [sum(d[o + j] * g[j] for j in range(r)) for o in range(m)]
            assert Y == want, (m, r, di, gi)


@pytest.mark.parametrize("m,r,points", [
    (2, 2, (0, 1)), (2, 3, (0, 1, -1)), (4, 3, (0, 1, -1, 2, -2)), (2, 5, (0, 1, -1, 2, -2)),
    (6, 3, (0, 1, -1, 2, -2, Fraction(1, 2), Fraction(-1, 2))), (2, 4, (0, 1, -1, 2)),
])
def test_generator_satisfies_fir_identity_exactly(m, r, points):
    AT, G, BT = ct.cook_toom_exact(points, m, r)
    _fir_identity_exact(AT, G, BT, m, r)


@pytest.mark.parametrize("m,r", [(1, 1), (2, 1), (2, 2), (2, 3), (4, 1), (4, 2), (4, 3),
                                 (2, 4), (2, 5), (2, 6), (2, 7), (3, 3)])
def test_tables_in_use_satisfy_fir_identity_exactly(m, r):
    AT, G, BT = ct.matrices(m, r)
    as_frac = lambda M: [[Fraction(v).limit_denominator(1000) for v in row] for row in M]
    _fir_identity_exact(as_frac(AT), as_frac(G), as_frac(BT), m, r)


def test_f43_is_the_published_lavin_gray_matrix_set():
    AT, G, BT = ct.matrices(4, 3)
    # Lavin & Gray, "Fast Algorithms for Convolutional Neural Networks", F(4x4,3x3)
    BT_pub = [[4, 0, -5, 0, 1, 0], [0, -4, -4, 1, 1, 0], [0, 4, -4, -1, 1, 0],
              [0, -2, -1, 2, 1, 0], [0, 2, -1, -2, 1, 0], [0, 4, 0, -5, 0, 1]]
    G_pub = [[1 / 4, 0, 0], [-1 / 6, -1 / 6, -1 / 6], [-1 / 6, 1 / 6, -1 / 6],
             [1 / 24, 1 / 12, 1 / 6], [1 / 24, -1 / 12, 1 / 6], [0, 0, 1]]
    AT_pub = [[1, 1, 1, 1, 1, 0], [0, 1, -1, 2, -2, 0], [0, 1, 1, 4, 4, 0], [0, 1, -1, 8, -8, 1]]
    assert np.array_equal(BT, np.array(BT_pub, dtype=np.float64))
    assert np.allclose(G, np.array(G_pub), rtol=0, atol=1e-16)
    assert np.array_equal(AT, np.array(AT_pub, dtype=np.float64))


def test_f25_generator_reproduces_the_reference_literals():
    """F(2,5) over the points (0,1,-1,2,-2) is what the reference generates at import
    (matrix_conv.py:33); its commented literals A25/G25/B25 (transform.py:27-40) give the
    expected output of the generator, sign and scaling split included."""
    AT, G, BT = ct.cook_toom((0, 1, -1, 2, -2), 2, 5)
    A25 = [[1, 1, 1, 1, 1, 0], [0, 1, -1, 2, -2, 1]]
    G25 = [[1 / 4, 0, 0, 0, 0], [-1 / 6] * 5, [-1 / 6, 1 / 6, -1 / 6, 1 / 6, -1 / 6],
           [1 / 24, 1 / 12, 1 / 6, 1 / 3, 2 / 3], [1 / 24, -1 / 12, 1 / 6, -1 / 3, 2 / 3], [0, 0, 0, 0, 1]]
    B25 = [[4, 0, -5, 0, 1, 0], [0, -4, -4, 1, 1, 0], [0, 4, -4, -1, 1, 0],
           [0, -2, -1, 2, 1, 0], [0, 2, -1, -2, 1, 0], [0, 4, 0, -5, 0, 1]]
    assert np.array_equal(AT, np.array(A25, dtype=np.float64))
    assert np.allclose(G, np.array(G25), rtol=0, atol=1e-16)
    assert np.array_equal(BT, np.array(B25, dtype=np.float64))


def _golden_f29():
    import json, os
    with open(os.path.join(os.path.dirname(__file__), "golden", "cook_toom_f29.json")) as f:
        g = json.load(f)
    frac = lambda M: [[Fraction(v) for v in row] for row in M]
    return g["points"], g["m"], g["r"], frac(g["AT"]), frac(g["G"]), frac(g["BT"])


def test_f29_generator_reproduces_the_reference_literals():
    """A 10 x 10 known answer: the generator over the points 0, +-1 .. +-4 must give the
    reference's commented A29 / G29 / B29 exactly (rational arithmetic, no tolerance)."""
    points, m, r, AT, G, BT = _golden_f29()
    got = ct.cook_toom_exact(points, m, r)
    assert got[0] == AT and got[1] == G and got[2] == BT
    _fir_identity_exact(AT, G, BT, m, r)          # and the literals themselves are a valid F(2,9)


def test_generator_reproduces_the_reference_generator_output():
    """F(2,4), F(2,5), F(2,6), F(2,7) and F(9,5) exactly as the reference's generator returns
    them for its own point tuples - the split of the scaling between AT, G and BT for
    fractional points is a convention only that output shows."""
    import json, os
    with open(os.path.join(os.path.dirname(__file__), "golden", "cook_toom_reference_tables.json")) as f:
        tables = json.load(f)["tables"]
    assert sorted((t["m"], t["r"]) for t in tables) == [(2, 4), (2, 5), (2, 6), (2, 7), (9, 5)]
    frac = lambda M: [[Fraction(v) for v in row] for row in M]
    for t in tables:
        got = ct.cook_toom_exact([Fraction(p) for p in t["points"]], t["m"], t["r"])
        assert got[0] == frac(t["AT"]) and got[1] == frac(t["G"]) and got[2] == frac(t["BT"]), (t["m"], t["r"])
        if t["m"] == 2:                      # and these are the tables in use for whole-kernel tiles
            AT, G, BT = ct.matrices(2, t["r"])
            as_f = lambda M: np.array([[float(v) for v in row] for row in M])
            assert np.array_equal(AT, as_f(got[0])) and np.array_equal(G, as_f(got[1]))
            assert np.array_equal(BT, as_f(got[2]))


def test_whole_kernel_tables_use_the_reference_point_sets():
    """F(2,4..7) as the reference builds them (matrix_conv.py:31-35): the first alpha-1 entries of
    its point tuples.  AT rows are the powers of those points, which fixes the choice of points;
    the FIR identity above fixes the rest up to the scaling that the F(2,5)/F(2,9) literals fix."""
    long_points = [0, 1, -1, Fraction(1, 2), Fraction(-1, 2), Fraction(1, 3), Fraction(-1, 3)]
    want = {4: [0, 1, -1, 2], 5: [0, 1, -1, 2, -2], 6: long_points[:6], 7: long_points[:7]}
    for r, pts in want.items():
        AT, G, BT = ct.matrices(2, r)
        assert np.array_equal(AT[0], np.array([1.] * r + [0.]))
        assert np.allclose(AT[1], np.array([float(p) for p in pts] + [1.]), rtol=0, atol=0)
        assert np.array_equal(G[-1], np.eye(r)[-1]) and BT[-1][-1] == 1.0


def test_kernel_spot_formulas():
    """Kronecker products of the tables reproduce single lines of the reference's unrolled code."""
    AT, G, BT = ct.matrices(2, 3)
    # 2-D input element 0 = d0 - d2 - d8 + d10          (transform_kernels.cu:1191)
    row = np.kron(BT[0], BT[0])
    want = np.zeros(16); want[[0, 10]] = 1; want[[2, 8]] = -1
    assert np.array_equal(row, want)
    # 3-D input element 0 = d0 + d10 - d2 - d32 + d34 + d40 - d42 - d8   (transform_kernels_3d.cu:4998)
    row = np.kron(BT[0], np.kron(BT[0], BT[0]))
    want = np.zeros(64); want[[0, 10, 34, 40]] = 1; want[[2, 32, 42, 8]] = -1
    assert np.array_equal(row, want)
    # 2-D output y00 = m0+m1+m2+m4+m5+m6+m8+m9+m10      (transform_kernels.cu:1587-1588)
    row = np.kron(AT[0], AT[0])
    want = np.zeros(16); want[[0, 1, 2, 4, 5, 6, 8, 9, 10]] = 1
    assert np.array_equal(row, want)
    # filter, r = 3 along W: [g0, (g0+g1+g2)/2, (g0-g1+g2)/2, g2]   (calculation_kernels.cu:26-29)
    assert np.array_equal(G, np.array([[1, 0, 0], [.5, .5, .5], [.5, -.5, .5], [0, 0, 1]]))
    # r = 2: input [d0-d1, d1, d2-d1], output [m0+m1, m1+m2]        (calculation_kernels.cu:773-775, 1536-1537)
    AT2, G2, BT2 = ct.matrices(2, 2)
    assert np.array_equal(BT2, np.array([[1, -1, 0], [0, 1, 0], [0, -1, 1]]))
    assert np.array_equal(AT2, np.array([[1, 1, 0], [0, 1, 1]]))
    assert np.array_equal(G2, np.array([[1, 0], [1, 1], [0, 1]]))


def test_unsupported_pair_is_rejected():
    with pytest.raises(ValueError):
        ct.matrices(3, 2)


def test_f33_of_the_shared_input_plans():
    """F(3,3) over the points 0, 1, -1, 2 (the reference's point set for five-element tiles,
    matrix_conv.py:32): exact rationals of the generator against the literals the HIP tables hold."""
    AT, G, BT = ct.cook_toom_exact(ct.POINTS_F42, 3, 3)
    F_ = Fraction
    assert AT == [[1, 1, 1, 1, 0], [0, 1, -1, 2, 0], [0, 1, 1, 4, 1]]
    assert G == [[F_(1, 2), 0, 0], [F_(-1, 2), F_(-1, 2), F_(-1, 2)], [F_(-1, 6), F_(1, 6), F_(-1, 6)],
                 [F_(1, 6), F_(1, 3), F_(2, 3)], [0, 0, 1]]
    assert BT == [[2, -1, -2, 1, 0], [0, -2, -1, 1, 0], [0, 2, -3, 1, 0], [0, -1, 0, 1, 0], [0, 2, -1, -2, 1]]
    _fir_identity_exact(AT, G, BT, 3, 3)
