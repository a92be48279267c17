"""Winograd / DWM convolution on the CPU, stage by stage (torch CPU tensors).

Test infrastructure only (see oracle/__init__.py).

Two pipelines of the reference are restated:

* the pure-PyTorch `matrix_conv` path (reference: matrix_conv.py:112-254,
  matrix_conv3d.py:112-290): wino_split -> U = G g G^T, V = B^T d B as matmuls ->
  M = U V -> Y = A^T M A -> wino_concat; tile layout (P, C, alpha, alpha).
* the native DWM path (reference: src/winograd_conv.cpp:17-127,
  src/base_conv_launchers.cu:282-399, src/split_kernel.cu:14-203, dwm.py:5-145):
  channel-last input, per-piece shifted windows, element-major buffers
  V (T, P, C), M (T, P, K), sum over pieces.  Two deliberate differences from
  the reference's buffers, both layout only: the transformed filter is kept as
  U (T, K, C) (reference (T, C, K), split_kernel.cu:51) and a 2-D problem gets a
  one-element depth axis instead of the all-zero second depth slice
  (dwm.py:117, split_kernel.cu:93-97).

Element order inside a tile is (d * alpha_h + h) * alpha_w + w on the data side
and (d * r_h + h) * r_w + w on the filter side (reference: split_kernel.cu:34,94,
transform_kernels_3d.cu:4987).

`discipline` selects the arithmetic the stages use:
  "fp64"  everything in float64 (the mathematical definition),
  "fp32"  float32 storage and arithmetic,
  "fp16"  float16 storage of x, w, U, V, M, y with float32 arithmetic inside each
          stage and one rounding per stored value (the engine's fp16 contract;
          the reference's own half path rounds after every matmul,
          matrix_conv.py:160-251),
  "bf16"  the same contract with bfloat16 storage (the reference has no bfloat16 path).
"""
import math
import itertools

import torch

from . import cook_toom
from .split_plan import conv_pieces

_STORE = {"fp64": torch.float64, "fp32": torch.float32, "fp16": torch.float16, "bf16": torch.bfloat16}
_MATH = {"fp64": torch.float64, "fp32": torch.float32, "fp16": torch.float32, "bf16": torch.float32}


def _mats(m, r, dtype):
    AT, G, BT = cook_toom.matrices(m, r)
    return (torch.from_numpy(AT).to(dtype), torch.from_numpy(G).to(dtype),
            torch.from_numpy(BT).to(dtype))


def out_dims(spatial, kernel, pads, stride):
    return [(X + 2 * p - k) // stride + 1 for X, k, p in zip(spatial, kernel, pads)]


def tile_grid(odims, ms):
    """n_X = ceil(o_X / m_X) (reference for m = 2: src/winograd_conv.cpp:88-90)."""
    return [(o + m - 1) // m for o, m in zip(odims, ms)]


# ------------------------------------------------------------------ stages (native layouts)
def filter_transform(w, pieces, T_total, discipline="fp32"):
    """w (K, C, kD, kH, kW) -> U (T_total, K, C):  U = (G_d x G_h x G_w) g per piece.
    (reference: src/split_kernel.cu:14-53, calculation_kernels.cu:2-761)"""
    mt, st = _MATH[discipline], _STORE[discipline]
    K, C = w.shape[:2]
    U = torch.zeros(T_total, K, C, dtype=st)
    wf = w.to(mt)
    for pc in pieces:
        taps = []
        Gs = []
        for ax in range(3):
            t0, step, r = pc["axes"][ax]
            taps.append(torch.arange(r) * step + t0)
            Gs.append(_mats(pc["ms"][ax], r, mt)[1])
        g = wf[:, :, taps[0]][:, :, :, taps[1]][:, :, :, :, taps[2]]       # (K,C,rd,rh,rw)
        u = torch.einsum("ia,jb,kc,KCabc->ijkKC", Gs[0], Gs[1], Gs[2], g)
        n = u.shape[0] * u.shape[1] * u.shape[2]
        U[pc["t_offset"]:pc["t_offset"] + n] = u.reshape(n, K, C).to(st)
    return U


def _gather_axis(x, dim, idx):
    """Index `dim` of x with an integer grid idx (n, alpha); out-of-range -> 0.
    Result has dims (..., n, alpha, ...) in place of `dim`."""
    size = x.shape[dim]
    valid = (idx >= 0) & (idx < size)
    flat = idx.clamp(0, size - 1).reshape(-1)
    g = x.index_select(dim, flat)
    shape = list(x.shape[:dim]) + list(idx.shape) + list(x.shape[dim + 1:])
    g = g.reshape(shape)
    mshape = [1] * dim + list(idx.shape) + [1] * (x.dim() - dim - 1)
    return g * valid.reshape(mshape).to(g.dtype)


def input_transform(x, pieces, T_total, pads, stride, grid, discipline="fp32"):
    """x (B, D, H, W, C) channel-last -> V (T_total, P, C), P = B*nD*nH*nW.
    Window of tile t, element i on one axis: stride*(m*t + i) + first_tap - pad, 0 outside
    (reference, stride 1: src/split_kernel.cu:78-100).  V = (BT_d x BT_h x BT_w) d."""
    mt, st = _MATH[discipline], _STORE[discipline]
    B, D, H, W, C = x.shape
    nD, nH, nW = grid
    P = B * nD * nH * nW
    V = torch.zeros(T_total, P, C, dtype=st)
    xf = x.to(mt)
    for pc in pieces:
        g = xf
        BTs = []
        for ax in range(3):
            t0, step, r = pc["axes"][ax]
            m = pc["ms"][ax]
            a = pc["alphas"][ax]
            idx = stride * (m * torch.arange(grid[ax])[:, None] + torch.arange(a)[None, :]) + t0 - pads[ax]
            g = _gather_axis(g, 1 + 2 * ax, idx)
            BTs.append(_mats(m, r, mt)[2])
        # g: (B, nD, aD, nH, aH, nW, aW, C)
        v = torch.einsum("ia,jb,kc,BdahbwcC->ijkBdhwC", BTs[0], BTs[1], BTs[2], g)
        n = v.shape[0] * v.shape[1] * v.shape[2]
        V[pc["t_offset"]:pc["t_offset"] + n] = v.reshape(n, P, C).to(st)
    return V


def batched_product(V, U, discipline="fp32"):
    """M[t] (P x K) = V[t] (P x C) . U[t]^T (C x K)
    (reference: src/base_conv_launchers.cu:362-367, matrix_conv.py:205)."""
    mt, st = _MATH[discipline], _STORE[discipline]
    return torch.bmm(V.to(mt), U.to(mt).transpose(1, 2)).to(st)


def output_transform(M, pieces, B, grid, odims, bias=None, discipline="fp32"):
    """M (T_total, P, K) -> y (B, oD, oH, oW, K): per piece Y = (AT_d x AT_h x AT_w) m,
    pieces summed, partial edge tiles cropped
    (reference: src/split_kernel.cu:126-203; the sum over pieces is taken in the
    math type before the single store, the reference sums stored partials)."""
    mt, st = _MATH[discipline], _STORE[discipline]
    nD, nH, nW = grid
    K = M.shape[2]
    acc = None
    for pc in pieces:
        a = pc["alphas"]
        n = a[0] * a[1] * a[2]
        mm = M[pc["t_offset"]:pc["t_offset"] + n].to(mt).reshape(a[0], a[1], a[2], B, nD, nH, nW, K)
        ATs = [_mats(pc["ms"][ax], pc["axes"][ax][2], mt)[0] for ax in range(3)]
        y = torch.einsum("ai,bj,ck,ijkBdhwK->BdahbwcK", ATs[0], ATs[1], ATs[2], mm)
        acc = y if acc is None else acc + y
    ms = pieces[0]["ms"]
    y = acc.reshape(B, nD * ms[0], nH * ms[1], nW * ms[2], K)[:, :odims[0], :odims[1], :odims[2]]
    if bias is not None:
        y = y + bias.to(mt)
    return y.to(st).contiguous()


# ------------------------------------------------------------------ whole convolutions
def _as_3d(x, w):
    two_d = x.dim() == 4
    if two_d:
        x = x.unsqueeze(2)
        w = w.unsqueeze(2)
    return x, w, two_d


def conv_plan(x_shape, w_shape, stride=1, padding=0, m=2, whole_kernel=False, pairs=False):
    """Shapes and pieces for an NC[D]HW x (K, C, [kD,] kH, kW) convolution."""
    two_d = len(x_shape) == 4
    sp = ([1] if two_d else []) + list(x_shape[2:])
    ks = ([1] if two_d else []) + list(w_shape[2:])
    if isinstance(padding, int):
        padding = [padding] * (len(x_shape) - 2)
    pads = ([0] if two_d else []) + list(padding)
    pieces, T_total = conv_pieces(ks, stride, m, degenerate_depth=two_d, whole_kernel=whole_kernel, pairs=pairs)
    od = out_dims(sp, ks, pads, stride)
    grid = tile_grid(od, pieces[0]["ms"])
    return dict(spatial=sp, kernel=ks, pads=pads, pieces=pieces, T_total=T_total,
                odims=od, grid=grid, two_d=two_d, stride=stride)


def stacked_pieces(pieces):
    """The pieces of a plan re-tiled for summation in the transform domain: every piece gets the
    tile F(m, r_max) per axis (r_max = most taps of any piece on that axis), element offset 0, and
    remembers in "real" how many of those taps it has; the others count as zero.  The sum over
    the pieces of U_s . V_s then has ONE output transform, i.e. the pieces can lie side by side
    along the reduction axis of the batched product (linearity of A^T . A; nothing the reference
    does - it adds the pieces after their output transforms, src/split_kernel.cu:184-203)."""
    rp = [max(pc["axes"][ax][2] for pc in pieces) for ax in range(3)]
    out = []
    for pc in pieces:
        axes = [(pc["axes"][ax][0], pc["axes"][ax][1], rp[ax]) for ax in range(3)]
        out.append({"axes": axes, "ms": list(pc["ms"]), "alphas": [pc["ms"][ax] + rp[ax] - 1 for ax in range(3)],
                    "t_offset": 0, "real": [pc["axes"][ax][2] for ax in range(3)]})
    T = out[0]["alphas"][0] * out[0]["alphas"][1] * out[0]["alphas"][2]
    return out, T


def _own_taps(w, pc):
    """A filter that holds the taps the piece owns (tap0 + j*step, j < real) at their places and
    zero everywhere else, large enough for every tap index of the shared tile (j < r_max)."""
    need = [pc["axes"][ax][0] + (pc["axes"][ax][2] - 1) * pc["axes"][ax][1] + 1 for ax in range(3)]
    wz = torch.zeros(tuple(w.shape[:2]) + tuple(max(n, k) for n, k in zip(need, w.shape[2:])), dtype=w.dtype)
    i0, i1, i2 = [torch.arange(pc["real"][ax]) * pc["axes"][ax][1] + pc["axes"][ax][0] for ax in range(3)]
    sel = (slice(None), slice(None), i0[:, None, None], i1[None, :, None], i2[None, None, :])
    wz[sel] = w[sel]
    return wz


def dwm_conv(x, w, bias=None, stride=1, padding=0, m=2, discipline="fp32", stages=None,
             whole_kernel=False, stacked=False):
    """Native-layout Winograd/DWM convolution.  x NC[D]HW, w (K, C, [kD,] kH, kW).
    Returns y NC[D]HW in the storage type of `discipline`.  If `stages` is a dict the
    intermediate buffers U, V, M and the plan are stored in it.  `whole_kernel`: one F(m, k) tile
    per axis instead of the DWM pieces (the reference's matrix_conv arithmetic).  `stacked`: the
    pieces are summed by the batched product (see stacked_pieces); U and V then are
    (T, K, n_pieces * C) and (T, P, n_pieces * C).  `stacked=2`: the same with pieces of two taps
    (split_plan.axis_pairs; 2-D, stride 1, m = 2), the decomposition whose pieces share one
    transformed input in the product path."""
    st = _STORE[discipline]
    plan = conv_plan(tuple(x.shape), tuple(w.shape), stride, padding, m, whole_kernel, pairs=(stacked == 2))
    x3, w3, two_d = _as_3d(x.to(st), w.to(st))
    xl = x3.permute(0, 2, 3, 4, 1).contiguous()                      # dwm.py:84, :132
    if stacked and len(plan["pieces"]) > 1:
        pcs, T = stacked_pieces(plan["pieces"])
        Us, Vs = [], []
        for pc in pcs:
            wz = _own_taps(w3, pc)
            Us.append(filter_transform(wz, [pc], T, discipline))
            Vs.append(input_transform(xl, [pc], T, plan["pads"], stride, plan["grid"], discipline))
        U, V = torch.cat(Us, dim=2), torch.cat(Vs, dim=2)
        plan = dict(plan, pieces=pcs, T_total=T)
        M = batched_product(V, U, discipline)
        y = output_transform(M, pcs[:1], x.shape[0], plan["grid"], plan["odims"],
                             None if bias is None else bias, discipline)
    else:
        U = filter_transform(w3, plan["pieces"], plan["T_total"], discipline)
        V = input_transform(xl, plan["pieces"], plan["T_total"], plan["pads"], stride, plan["grid"], discipline)
        M = batched_product(V, U, discipline)
        y = output_transform(M, plan["pieces"], x.shape[0], plan["grid"], plan["odims"],
                             None if bias is None else bias, discipline)
    if stages is not None:
        stages.update(U=U, V=V, M=M, plan=plan, y_cl=y)
    y = y.permute(0, 4, 1, 2, 3)                                     # dwm.py:105, :144
    if two_d:
        y = y[:, :, 0]
    return y.contiguous()


def matrix_conv(x, w, m=2, discipline="fp32"):
    """The reference's PyTorch Winograd path for one un-split kernel, stride 1, no padding
    (reference: matrix_conv.py:112-254 for 2-D, matrix_conv3d.py:112-290 for 3-D):
    tiles (P, C, a, a) -> U (T, K, C), V (T, C, P), M = U V (T, K, P) -> (P, K, m, m)."""
    from . import tiles as tl
    mt, st = _MATH[discipline], _STORE[discipline]
    nd = x.dim() - 2
    K, C = w.shape[:2]
    rs = list(w.shape[2:])
    od = [X - r + 1 for X, r in zip(x.shape[2:], rs)]
    t = torch.from_numpy(tl.wino_split(x.to(st).numpy(), tuple(w.shape), m))   # matrix_conv.py:126
    P = t.shape[0]
    mats = [_mats(m, r, mt) for r in rs]
    letters = "abc"[:nd], "ijk"[:nd]
    sub_g = ",".join(o + i for o, i in zip(letters[1], letters[0]))
    U = torch.einsum("%s,KC%s->%sKC" % (sub_g, letters[0], letters[1]),
                     *[mm[1] for mm in mats], w.to(st).to(mt)).to(st)          # matrix_conv.py:150-153
    V = torch.einsum("%s,PC%s->%sCP" % (sub_g, letters[0], letters[1]),
                     *[mm[2] for mm in mats], t.to(mt)).to(st)                 # matrix_conv.py:158, :202-203
    T = int(math.prod(U.shape[:nd]))
    Mm = torch.bmm(U.reshape(T, K, C).to(mt), V.reshape(T, C, P).to(mt)).to(st)  # matrix_conv.py:205
    Mm = Mm.reshape(tuple(U.shape[:nd]) + (K, P))
    sub_a = ",".join(o + i for o, i in zip(letters[0], letters[1]))
    Y = torch.einsum("%s,%sKP->PK%s" % (sub_a, letters[1], letters[0]),
                     *[mm[0] for mm in mats], Mm.to(mt)).to(st)                # matrix_conv.py:207-211
    y = tl.wino_concat(Y.numpy(), od, m)                                       # matrix_conv.py:134
    return torch.from_numpy(y)


def direct_conv(x, w, bias=None, stride=1, padding=0, discipline="fp32"):
    """The degenerate end of the split: every piece is ONE tap on the trivial tile F(1,1), for which A^T, G and B^T
    are 1, so y[b, k, oy, ox] = sum over taps (ky, kx) and channels of x[b, c, stride oy + ky - pad, stride ox + kx - pad]
    w[k, c, ky, kx] with nothing transformed: the products are added tap by tap (ky outermost, the order the engine's
    product walks its reduction axis) in the arithmetic type of the discipline, the bias is added to the sum, and the
    result is rounded once to the storage type.  2-D, or 3-D with the kernel planes outermost.  The reference has no such
    form and no stride 2 at all (src/winograd_conv.cpp:122-126); the definition of the convolution itself (torch's
    conv2d / conv3d in fp64) pins it."""
    mt, st = _MATH[discipline], _STORE[discipline]
    nd = x.dim() - 2
    B, C = x.shape[:2]
    K = w.shape[0]
    sp, ks = tuple(x.shape[2:]), tuple(w.shape[2:])
    pads = (padding,) * nd if isinstance(padding, int) else tuple(padding)
    outs = out_dims(sp, ks, pads, stride)
    xp = torch.zeros(B, C, *[n + 2 * p + stride for n, p in zip(sp, pads)], dtype=mt)
    xp[(slice(None), slice(None)) + tuple(slice(p, p + n) for n, p in zip(sp, pads))] = x.to(st).to(mt)
    wm = w.to(st).to(mt)
    acc = torch.zeros(B, K, *outs, dtype=mt)
    letters = "hw" if nd == 2 else "dhw"
    for tap in itertools.product(*[range(k) for k in ks]):
        win = xp[(slice(None), slice(None)) + tuple(slice(t, t + stride * (o - 1) + 1, stride) for t, o in zip(tap, outs))]
        acc += torch.einsum("bc%s,kc->bk%s" % (letters, letters), win, wm[(slice(None), slice(None)) + tap])
    if bias is not None:
        acc += bias.to(st).to(mt).view(1, K, *([1] * nd))
    return acc.to(st)
