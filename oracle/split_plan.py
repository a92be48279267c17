"""DWM kernel split plan: which 3x3(-or-smaller) stride-1 pieces a kernel is cut into.

Test infrastructure only (see oracle/__init__.py).

Restates the rule implied by the reference's host look-up table
(reference: src/base_conv_launchers.h:58-388): per axis an extent k is cut into
chunks of 3 with the remainder last, except 4 -> [2, 2]; the boxes are the
Cartesian product of the per-axis chunks, depth outermost and width fastest.
`kernel_stride[s]` is the running sum of the tile sizes prod(size+1)
(reference: src/base_conv_launchers.cu:307-313).

For stride 2 (not implemented by the reference: src/winograd_conv.cpp:122-126
exits) the plan first separates the taps of each axis by parity - the identity
  y[o] = sum_k x[2o+k-pad] w[k] = sum_q sum_j x[2(o+j)+q-pad] w[2j+q]
turns a stride-2 correlation into two stride-1 correlations over the even and
odd samples - and then cuts each phase's taps by the same rule.
"""
from itertools import product


def axis_chunks(k):
    """[(start, size), ...] for one axis of extent k, stride 1."""
    if k == 4:
        sizes = [2, 2]
    else:
        sizes = [3] * (k // 3) + ([k % 3] if k % 3 else [])
    out, s = [], 0
    for z in sizes:
        out.append((s, z))
        s += z
    return out


def axis_pieces(k, stride):
    """[(first_tap, tap_step, n_taps), ...] for one axis."""
    if stride == 1:
        return [(s, 1, z) for s, z in axis_chunks(k)]
    out = []
    for q in range(stride):
        n = (k - q + stride - 1) // stride          # taps q, q+stride, ...
        if n <= 0:
            continue
        for s, z in axis_chunks(n):
            out.append((q + stride * s, stride, z))
    return out


def split_plan(kD, kH, kW):
    """Stride-1 plan in the reference's own vocabulary.

    Returns dict(D_start, D_end, H_start, H_end, W_start, W_end, kernel_stride,
    T_total), boxes half-open [start, end) as in the LUT.
    """
    boxes = list(product(axis_chunks(kD), axis_chunks(kH), axis_chunks(kW)))
    plan = {k: [] for k in ("D_start", "D_end", "H_start", "H_end", "W_start", "W_end",
                            "kernel_stride")}
    t = 0
    for (d0, dz), (h0, hz), (w0, wz) in boxes:
        plan["D_start"].append(d0); plan["D_end"].append(d0 + dz)
        plan["H_start"].append(h0); plan["H_end"].append(h0 + hz)
        plan["W_start"].append(w0); plan["W_end"].append(w0 + wz)
        plan["kernel_stride"].append(t)
        t += (dz + 1) * (hz + 1) * (wz + 1)
    plan["T_total"] = t
    return plan


def axis_pairs(k, n=2):
    """Chunks of n taps, the remainder last: [(first_tap, 1, n_taps), ...].  Not the split of the
    reference (chunks of three with 4 -> 2 + 2, base_conv_launchers.h:58-388): pieces that start at
    multiples of the output tile n see the same transformed input moved by whole tiles."""
    return [(s, 1, min(n, k - s)) for s in range(0, k, n)]


def conv_pieces(kernel, stride=1, m=2, degenerate_depth=False, whole_kernel=False, pairs=False):
    """General plan for a (kD, kH, kW) kernel with one stride for all axes.

    Each piece is one stride-1 sub-convolution: per axis (first_tap, tap_step,
    n_taps) and the Winograd tile F(m_axis, n_taps).  With `degenerate_depth`
    (a 2-D problem, D = kD = 1) the depth axis is F(1,1) - one element - rather
    than the reference's zero-padded alpha = 2 depth tile (dwm.py:117,
    src/split_kernel.cu:93-97), which only multiplies zeros.
    With `whole_kernel` the kernel is not decomposed: one piece, F(m, k) per axis - the
    arithmetic of the reference's PyTorch path (matrix_conv.py:112-135), stride 1 only.
    Returns (pieces, T_total); pieces[i] = dict(axes, ms, alphas, t_offset).
    """
    if whole_kernel:
        assert stride == 1
        per_axis = [[(0, 1, k)] for k in kernel]
    elif pairs and stride == 2:
        # parity phases first (as axis_pieces does), then pairs of a phase's taps: (q + 2 s, 2, <= 2 taps)
        per_axis = [[(q + 2 * s, 2, min(2, (k - q + 1) // 2 - s))
                     for q in range(min(2, k)) for s in range(0, (k - q + 1) // 2, 2)] for k in kernel]
    elif pairs:
        assert stride == 1
        per_axis = [axis_pairs(k, m if isinstance(m, int) else 2) for k in kernel]
    else:
        per_axis = [axis_pieces(k, stride) for k in kernel]
    # m: one output tile extent for all axes, or one per axis (depth, height, width)
    mt = [m] * 3 if isinstance(m, int) else list(m)
    ms = [1 if (ax == 0 and degenerate_depth) else mt[ax] for ax in range(3)]
    out, t = [], 0
    for combo in product(*per_axis):
        alphas = [ms[ax] + combo[ax][2] - 1 for ax in range(3)]
        out.append({"axes": list(combo), "ms": list(ms), "alphas": alphas, "t_offset": t})
        t += alphas[0] * alphas[1] * alphas[2]
    return out, t
