"""Writes tests/golden/cook_toom_reference_tables.json: the transform matrices the reference's own
generator produces for the whole-kernel tiles it builds at import (matrix_conv.py:31-36).

Runs in the build container only (it imports /root/reference/wincnn.py, which needs sympy); the
JSON it writes is data (exact rationals as strings) and is what the tests read.  Needed because
the split of the scaling between AT, G and BT for the fractional point set is a convention of
that generator that no literal in the reference shows.

The generator divides a matrix by the diagonal matrix of the scale factors (wincnn.py:56,61:
`A(...).T/f`).  sympy 1.14 no longer defines matrix / matrix; the sympy of the reference's time
evaluated it as multiplication by the inverse, which is also the only meaning the expression
can have, so this script supplies exactly that for the duration of the run and changes nothing
else.

    python tests/golden/make_cook_toom_tables.py
"""
import importlib.util
import json
import os

from sympy import Rational
from sympy.matrices import MatrixBase

REF = "/root/reference/wincnn.py"
spec = importlib.util.spec_from_file_location("reference_wincnn", REF)
wincnn = importlib.util.module_from_spec(spec)
spec.loader.exec_module(wincnn)

# the point tuples of matrix_conv.py:31-35
points = (0, 1, -1, Rational(1, 2), -Rational(1, 2), Rational(1, 3), -Rational(1, 3),
          Rational(3, 2), -Rational(3, 2), -3, 2, -2)
cases = [((0, 1, -1, 2), 2, 4), ((0, 1, -1, 2, -2), 2, 5), (points, 2, 6), (points, 2, 7), (points, 9, 5)]

_truediv = MatrixBase.__truediv__


def _matrix_div(self, other):
    if isinstance(other, MatrixBase):
        return self * other.inv()
    return _truediv(self, other)


MatrixBase.__truediv__ = _matrix_div

out = {"source": "huangdi95/pytorch_winoconv wincnn.cookToomFilter (wincnn.py:49-70), default fractionsIn",
       "tables": []}
for pts, n, r in cases:
    AT, G, BT, f = wincnn.cookToomFilter(pts, n, r)
    as_rows = lambda M: [[str(Rational(M[i, j])) for j in range(M.shape[1])] for i in range(M.shape[0])]
    out["tables"].append({"points": [str(Rational(p)) for p in pts], "m": n, "r": r,
                          "AT": as_rows(AT), "G": as_rows(G), "BT": as_rows(BT)})
path = os.path.join(os.path.dirname(os.path.abspath(__file__)), "cook_toom_reference_tables.json")
with open(path, "w") as fh:
    json.dump(out, fh, indent=0)
print("wrote", path, [(t["m"], t["r"]) for t in out["tables"]])
