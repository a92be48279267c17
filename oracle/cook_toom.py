"""Winograd transform matrices AT (m x alpha), G (alpha x r), BT (alpha x alpha).

Test infrastructure only (see oracle/__init__.py).

`cook_toom(points, m, r)` restates the construction of the reference's vendored
generator (reference: wincnn.py:7-70, default fractionsIn=FractionsInG) in
exact rational arithmetic with `fractions.Fraction` instead of sympy:

  f_i   = prod_{k != i} (a_i - a_k)      i < alpha-1,  f_{alpha-1} = 1   (wincnn.py:22-33)
  f_0  *= -1 if f_0 < 0                                                  (wincnn.py:52-53)
  AT[j][i] = a_i**j,  last column e_{m-1}                                (wincnn.py:7-11, :55)
  G[i][j]  = a_i**j / f_i, last row e_{r-1}                              (wincnn.py:56)
  BT       = diag(f) * B(a, alpha)^T                                     (wincnn.py:35-45, :57)

The literal tables are the ones the reference hard-codes
(matrix_conv.py:15-30 for F(2,1), F(2,3); matrix_convnd.py:20-27 for F(2,2)).
"""
from fractions import Fraction
import numpy as np


def _poly_mul(p, q):
    out = [Fraction(0)] * (len(p) + len(q) - 1)
    for i, a in enumerate(p):
        for j, b in enumerate(q):
            out[i + j] += a * b
    return out


def cook_toom_exact(points, m, r):
    """Return (AT, G, BT) as nested lists of Fraction."""
    a = [Fraction(p) for p in points]
    alpha = m + r - 1
    n = alpha - 1
    assert len(a) >= n, "need alpha-1 interpolation points"
    a = a[:n]
    # f_i = prod_{k != i}(a_i - a_k); appended 1                (wincnn.py:22-33)
    F = []
    for i in range(n):
        v = Fraction(1)
        for k in range(n):
            if k != i:
                v *= a[i] - a[k]
        F.append(v)
    f = list(F) + [Fraction(1)]
    if f[0] < 0:                                               # (wincnn.py:52-53)
        f[0] = -f[0]

    def A(cols):                                               # (wincnn.py:7-11)
        rows = [[a[i] ** j for j in range(cols)] for i in range(n)]
        rows.append([Fraction(1) if j == cols - 1 else Fraction(0) for j in range(cols)])
        return rows

    Am, Ar = A(m), A(r)
    AT = [[Am[i][j] for i in range(alpha)] for j in range(m)]
    G = [[Ar[i][j] / f[i] for j in range(r)] for i in range(alpha)]

    # L[j][i] = coeff of x^j in prod_{k != i}(x - a_k), divided by F_i   (wincnn.py:17-38)
    L = [[Fraction(0)] * n for _ in range(n)]
    for i in range(n):
        poly = [Fraction(1)]
        for k in range(n):
            if k != i:
                poly = _poly_mul(poly, [-a[k], Fraction(1)])
        for j in range(n):
            L[j][i] = poly[j] / F[i]
    # T = [I_n | -a_i^n]; Bt = L * T  (n x alpha)                        (wincnn.py:13-15, :40-41)
    Bt = [[L[j][c] if c < n else -sum(L[j][i] * a[i] ** n for i in range(n))
           for c in range(alpha)] for j in range(n)]
    # B = Bt with the row e_{alpha-1} appended; BT = diag(f) * B^T       (wincnn.py:43-45, :57)
    Bm = Bt + [[Fraction(1) if c == alpha - 1 else Fraction(0) for c in range(alpha)]]
    BT = [[f[i] * Bm[j][i] for j in range(alpha)] for i in range(alpha)]
    return AT, G, BT


def _np(mat):
    return np.array([[float(v) for v in row] for row in mat], dtype=np.float64)


def cook_toom(points, m, r):
    AT, G, BT = cook_toom_exact(points, m, r)
    return _np(AT), _np(G), _np(BT)


# --- literal tables of the reference -------------------------------------------------------
_LIT = {
    (1, 1): (  # degenerate axis (a 2-D problem seen as 3-D with no depth transform)
        [[1.]], [[1.]], [[1.]]),
    (2, 1): (  # matrix_conv.py:15-20
        [[1., 0.], [0., 1.]],
        [[1.], [1.]],
        [[1., 0.], [0., 1.]]),
    (2, 2): (  # matrix_convnd.py:20-27
        [[1., 1., 0.], [0., 1., 1.]],
        [[1., 0.], [1., 1.], [0., 1.]],
        [[1., -1., 0.], [0., 1., 0.], [0., -1., 1.]]),
    (2, 3): (  # matrix_conv.py:21-30
        [[1., 1., 1., 0.], [0., 1., -1., -1.]],
        [[1., 0., 0.], [.5, .5, .5], [.5, -.5, .5], [0., 0., 1.]],
        [[1., 0., -1., 0.], [0., 1., 1., 0.], [0., -1., 1., 0.], [0., 1., 0., -1.]]),
}

# the reference's long point set (matrix_conv.py:31), used for F(2,6) and F(2,7) (matrix_conv.py:34-35)
POINTS_REF = (0, 1, -1, Fraction(1, 2), -Fraction(1, 2), Fraction(1, 3), -Fraction(1, 3),
              Fraction(3, 2), -Fraction(3, 2), -3, 2, -2)
# point sets of the whole-kernel tiles F(2,r), r = 4..7, as the reference builds them (matrix_conv.py:32-35)
POINTS_F2R = {4: (0, 1, -1, 2), 5: (0, 1, -1, 2, -2), 6: POINTS_REF, 7: POINTS_REF}
POINTS_F43 = (0, 1, -1, 2, -2)   # same point set the reference uses for F(2,5) (matrix_conv.py:33)
POINTS_F42 = (0, 1, -1, 2)       # the reference's point set for F(2,4) (matrix_conv.py:32)
_LIT[(4, 1)] = (                 # one tap: identity, like the reference's F(2,1) literal
    [[1., 0., 0., 0.], [0., 1., 0., 0.], [0., 0., 1., 0.], [0., 0., 0., 1.]],
    [[1.], [1.], [1.], [1.]],
    [[1., 0., 0., 0.], [0., 1., 0., 0.], [0., 0., 1., 0.], [0., 0., 0., 1.]])


def matrices(m, r):
    """(AT, G, BT) float64 for F(m, r).  F(2,1..3) and F(4,1) literal; F(4,2), F(4,3) and the
    whole-kernel tiles F(2,4..7) Cook-Toom."""
    if (m, r) in _LIT:
        AT, G, BT = _LIT[(m, r)]
        return (np.array(AT, dtype=np.float64), np.array(G, dtype=np.float64),
                np.array(BT, dtype=np.float64))
    if (m, r) == (4, 3):
        return cook_toom(POINTS_F43, 4, 3)
    if (m, r) == (4, 2):
        return cook_toom(POINTS_F42, 4, 2)
    if (m, r) == (3, 3):
        return cook_toom(POINTS_F42, 3, 3)      # the shared tile of three-tap pieces: same four finite points
    if m == 2 and r in POINTS_F2R:
        return cook_toom(POINTS_F2R[r], 2, r)
    raise ValueError("F(%d,%d) not on the hot path" % (m, r))
