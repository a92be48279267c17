"""Pins oracle.split_plan against the reference's own integer table and against brute force."""
import itertools
import json
import os

import numpy as np
import pytest

from oracle import split_plan as sp

LUT = json.load(open(os.path.join(os.path.dirname(__file__), "golden", "split_lut.json")))


def test_lut_has_the_36_reference_keys():
    assert len(LUT) == 36


@pytest.mark.parametrize("key", sorted(LUT))
def test_rule_reproduces_every_lut_key(key):
    """splitControl (src/base_conv_launchers.h:58-388): all six arrays of every key."""
    kd, kh, kw = (int(v) for v in key.split("x"))
    p = sp.split_plan(kd, kh, kw)
    g = LUT[key]
    for a, b in [("D_s", "D_start"), ("D_e", "D_end"), ("H_s", "H_start"), ("H_e", "H_end"),
                 ("W_s", "W_start"), ("W_e", "W_end")]:
        assert g[a] == p[b], (key, a)


def test_kernel_stride_and_total_follow_the_launcher():
    """kernel_stride is the running sum of prod(size + 1) (base_conv_launchers.cu:307-313); the
    totals that follow from the table by hand: 7x7 -> 9 boxes of (1+1)(a+1)(b+1) = 200 and 5x5 -> 98
    with the reference's doubled depth, 3x3x3 -> 4^3 = 64."""
    p = sp.split_plan(1, 7, 7)
    assert p["kernel_stride"] == [0, 32, 64, 80, 112, 144, 160, 176, 192] and p["T_total"] == 200
    assert sp.split_plan(1, 5, 5)["T_total"] == 98
    assert sp.split_plan(3, 3, 3)["T_total"] == 64
    # the Python wrapper sizes its buffers with the same number (dwm.py:117)
    for k in (5, 7, 9):
        assert sp.split_plan(1, k, k)["T_total"] == (k + 1 + (k - 1) // 3) ** 2 * 2


@pytest.mark.parametrize("k", range(1, 11))
def test_axis_chunks_cover_the_axis(k):
    ch = sp.axis_chunks(k)
    assert all(1 <= z <= 3 for _, z in ch)
    assert [s for s, _ in ch] == list(np.cumsum([0] + [z for _, z in ch])[:-1])
    assert sum(z for _, z in ch) == k


@pytest.mark.parametrize("k,stride", list(itertools.product(range(1, 11), (1, 2))))
def test_axis_pieces_partition_the_taps(k, stride):
    taps = []
    for t0, step, n in sp.axis_pieces(k, stride):
        assert step == stride and 1 <= n <= 3
        taps += [t0 + step * i for i in range(n)]
    assert sorted(taps) == list(range(k))


@pytest.mark.parametrize("k,stride,pad,n", [(3, 2, 1, 12), (7, 2, 3, 15), (5, 2, 2, 9), (4, 2, 0, 10), (2, 2, 0, 8)])
def test_stride2_phase_identity_brute_force(k, stride, pad, n):
    """y[o] = sum_k x[s*o + k - pad] w[k] equals the sum over pieces of stride-1 correlations
    x[s*(o + j) + tap0 - pad] w[tap0 + s*j] - brute force with integers on one axis."""
    rng = np.random.default_rng(0)
    x = rng.integers(-5, 6, n)
    w = rng.integers(-5, 6, k)
    xp = lambda i: int(x[i]) if 0 <= i < n else 0
    no = (n + 2 * pad - k) // stride + 1
    direct = [sum(xp(stride * o + kk - pad) * int(w[kk]) for kk in range(k)) for o in range(no)]
    pieces = [0] * no
    for t0, step, r in sp.axis_pieces(k, stride):
        for o in range(no):
            pieces[o] += sum(xp(step * (o + j) + t0 - pad) * int(w[t0 + step * j]) for j in range(r))
    assert pieces == direct


def test_conv_pieces_offsets_and_order():
    pcs, T = sp.conv_pieces((1, 5, 5), 1, 2, degenerate_depth=True)
    assert [p["t_offset"] for p in pcs] == [0, 16, 28, 40] and T == 49
    assert [tuple(a[2] for a in p["axes"]) for p in pcs] == [(1, 3, 3), (1, 3, 2), (1, 2, 3), (1, 2, 2)]
    pcs, T = sp.conv_pieces((1, 3, 3), 1, 4, degenerate_depth=True)
    assert T == 36 and pcs[0]["alphas"] == [1, 6, 6]
    pcs, T = sp.conv_pieces((3, 3, 3), 1, 2)
    assert T == 64
