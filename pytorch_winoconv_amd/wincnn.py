"""Cook-Toom construction of Winograd transform matrices in exact rational arithmetic, under
the names of the generator the reference vendors (reference: wincnn.py:49-70, which needs
sympy; this one needs only `fractions`).

For interpolation points a_0 .. a_{n-1} (n = alpha - 1, alpha = m + r - 1) let
M(x) = prod_k (x - a_k), M_i(x) = M(x) / (x - a_i) and N_i = M_i(a_i).  Then

  AT[j][i] = a_i**j                       (m x alpha; last column = e_{m-1}, the point at infinity)
  G[i][j]  = a_i**j / f_i                 (alpha x r; last row = e_{r-1}),  f_i = N_i, f_0 = |N_0|
  BT[i]    = (f_i / N_i) * coefficients of M_i, then 0   (i < n);   BT[n] = coefficients of M

which is the scaling the reference's generator produces (all of the division sits in G).
"""
from fractions import Fraction

import numpy as np


def _poly_from_roots(roots):
    """Coefficients, lowest power first, of prod (x - root)."""
    p = [Fraction(1)]
    for a in roots:
        q = [Fraction(0)] * (len(p) + 1)
        for i, c in enumerate(p):
            q[i] -= a * c
            q[i + 1] += c
        p = q
    return p


def cookToomFilter(a, n, r):
    """(AT, G, BT) of F(n, r) as nested lists of Fraction; `a` holds at least n + r - 2 points."""
    alpha = n + r - 1
    pts = [Fraction(str(v)) if not isinstance(v, (int, Fraction)) else Fraction(v) for v in a][:alpha - 1]
    if len(pts) < alpha - 1 or len(set(pts)) != len(pts):
        raise ValueError("F(%d,%d) needs %d distinct interpolation points" % (n, r, alpha - 1))
    AT = [[pts[i] ** j for i in range(alpha - 1)] + [Fraction(int(j == n - 1))] for j in range(n)]
    G, BT = [], []
    for i, ai in enumerate(pts):
        Mi = _poly_from_roots(pts[:i] + pts[i + 1:])
        Ni = sum(c * ai ** k for k, c in enumerate(Mi))
        fi = abs(Ni) if i == 0 else Ni
        G.append([ai ** j / fi for j in range(r)])
        BT.append([fi / Ni * c for c in Mi] + [Fraction(0)])
    G.append([Fraction(int(j == r - 1)) for j in range(r)])
    BT.append(_poly_from_roots(pts))
    return AT, G, BT


def showCookToomFilter(a, n, r):
    """(AT, G, BT) of F(n, r) as float64 arrays (reference: wincnn.py:72-89 prints them and the
    callers keep the returned matrices, matrix_conv.py:32-40)."""
    return tuple(np.array([[float(v) for v in row] for row in mat], dtype=np.float64)
                 for mat in cookToomFilter(a, n, r))
