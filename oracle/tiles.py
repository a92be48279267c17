"""wino_split / wino_concat index maps on the CPU (numpy, exact copies).

Test infrastructure only (see oracle/__init__.py).

wino_split  (reference: Split_and_Concat.py:4-49, src/split_and_concat.cpp:14-40,
            src/split_and_concat_kernels.cu:8-37 and :76-101)
    tiles[(b, [d,] h, w), c, [k,] i, j] = x[b, [m*d+k,] m*h+i, m*w+j, c], 0 outside,
    n_X = int((X + 1 - block_X) / m + 1), block_X = w_X + m - 1.
    The reference kernel hard-codes the tile step 2 (kernels.cu:20-22, :87-88)
    while the wrapper derives n_X from output_block_size; both agree for m = 2,
    the only value the reference is correct for.  The step here is m.
wino_concat (reference: Split_and_Concat.py:51-82, src/split_and_concat.cpp:44-76,
            src/split_and_concat_kernels.cu:43-70 and :107-129)
    y[b, [m*d+k,] m*h+i, m*w+j, c] = tiles[(b,[d,]h,w), c, [k,] i, j] if inside.
Inputs/outputs are NCHW / NCDHW like the Python wrappers (the NHWC permutes
of Split_and_Concat.py:25,47,64,81 are folded into the index maps).
"""
import numpy as np


def tile_counts(spatial, w_spatial, m):
    """n_X of Split_and_Concat.py:21-23 / :40-41 (pads are 0 there)."""
    return [int((X + 1 - (wX + m - 1)) / m + 1) for X, wX in zip(spatial, w_spatial)]


def wino_split(a, w_shape, m):
    a = np.asarray(a)
    nd = a.ndim - 2
    B, C = a.shape[:2]
    spatial = a.shape[2:]
    w_sp = tuple(w_shape[2:])
    blocks = [w + m - 1 for w in w_sp]
    n = tile_counts(spatial, w_sp, m)
    out = np.zeros((B,) + tuple(n) + (C,) + tuple(blocks), dtype=a.dtype)
    # brute index loops over tile grid and in-tile offsets (small counts); vectorised over B, C
    grids = np.ndindex(*n)
    for t in grids:
        for off in np.ndindex(*blocks):
            src = [m * ti + oi for ti, oi in zip(t, off)]
            if all(0 <= s < X for s, X in zip(src, spatial)):
                out[(slice(None),) + t + (slice(None),) + off] = a[(slice(None), slice(None)) + tuple(src)]
    return out.reshape((B * int(np.prod(n)), C) + tuple(blocks))


def wino_concat(t, output_size, m):
    t = np.asarray(t)
    nd = len(output_size)
    N, K = t.shape[:2]
    n = [(int(o) + m - 1) // m for o in output_size]
    B = N // int(np.prod(n))
    t = t.reshape((B,) + tuple(n) + (K,) + (m,) * nd)
    out = np.zeros((B, K) + tuple(int(o) for o in output_size), dtype=t.dtype)
    for tile in np.ndindex(*n):
        for off in np.ndindex(*((m,) * nd)):
            dst = [m * ti + oi for ti, oi in zip(tile, off)]
            if all(d < int(o) for d, o in zip(dst, output_size)):
                out[(slice(None), slice(None)) + tuple(dst)] = t[(slice(None),) + tile + (slice(None),) + off]
    return out
