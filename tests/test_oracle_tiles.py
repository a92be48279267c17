"""Pins oracle.tiles (wino_split / wino_concat) against torch.unfold and brute-force loops."""
import numpy as np
import pytest
import torch

from oracle import tiles


@pytest.mark.parametrize("shape,w,m", [
    ((2, 3, 6, 6), (1, 3, 3, 3), 2), ((1, 2, 9, 11), (1, 2, 3, 3), 2), ((1, 2, 14, 10), (1, 2, 3, 3), 4),
    ((1, 1, 12, 7), (1, 1, 5, 5), 2), ((2, 2, 7, 8), (1, 2, 2, 3), 2),
])
def test_split_2d_equals_unfold_of_right_bottom_padded_input(shape, w, m):
    x = torch.arange(int(np.prod(shape)), dtype=torch.float32).reshape(shape) + 1
    blocks = [w[2] + m - 1, w[3] + m - 1]
    n = tiles.tile_counts(shape[2:], w[2:], m)
    need = [(n[i] - 1) * m + blocks[i] for i in range(2)]
    xp = torch.nn.functional.pad(x, (0, max(0, need[1] - shape[3]), 0, max(0, need[0] - shape[2])))
    u = xp.unfold(2, blocks[0], m).unfold(3, blocks[1], m)[:, :, :n[0], :n[1]]   # B,C,nH,nW,bH,bW
    want = u.permute(0, 2, 3, 1, 4, 5).reshape(-1, shape[1], *blocks)
    got = tiles.wino_split(x.numpy(), w, m)
    assert got.shape == tuple(want.shape)
    assert np.array_equal(got, want.numpy())


def test_split_tile_count_formula():
    """n = int((X + 1 - block) / m + 1), pads 0 (Split_and_Concat.py:21-23,40-41)."""
    assert tiles.tile_counts((58, 58), (3, 3), 2) == [28, 28]
    assert tiles.tile_counts((6, 6), (3, 3), 2) == [2, 2]
    assert tiles.tile_counts((7, 9), (3, 3), 2) == [3, 4]
    assert tiles.tile_counts((10, 10, 10), (3, 3, 3), 2) == [4, 4, 4]


def test_split_3d_brute_force():
    rng = np.random.default_rng(1)
    x = rng.standard_normal((2, 3, 5, 6, 7)).astype(np.float32)
    w, m = (1, 3, 3, 2, 3), 2
    got = tiles.wino_split(x, w, m)
    nD, nH, nW = tiles.tile_counts(x.shape[2:], w[2:], m)
    bD, bH, bW = 4, 3, 4
    assert got.shape == (2 * nD * nH * nW, 3, bD, bH, bW)
    for b in range(2):
        for d in range(nD):
            for h in range(nH):
                for ww in range(nW):
                    p = ((b * nD + d) * nH + h) * nW + ww          # split_and_concat_kernels.cu:33
                    for k in range(bD):
                        for i in range(bH):
                            for j in range(bW):
                                z, y, xx = 2 * d + k, 2 * h + i, 2 * ww + j
                                inside = z < 5 and y < 6 and xx < 7
                                want = x[b, :, z, y, xx] if inside else 0
                                assert np.array_equal(got[p, :, k, i, j], want + 0 * got[p, :, k, i, j])


@pytest.mark.parametrize("osize,m", [((7, 9), 2), ((8, 8), 2), ((13, 10), 4), ((5, 7, 6), 2)])
def test_concat_inverts_a_non_overlapping_split_and_crops(osize, m):
    rng = np.random.default_rng(2)
    K, B = 3, 2
    y = rng.standard_normal((B, K) + tuple(osize)).astype(np.float32)
    n = [(o + m - 1) // m for o in osize]
    padded = np.zeros((B, K) + tuple(v * m for v in n), dtype=np.float32)
    padded[(slice(None), slice(None)) + tuple(slice(0, o) for o in osize)] = y
    # cut the padded tensor into m^d blocks by reshape (independent of tiles.wino_concat's loops)
    nd = len(osize)
    shp = (B, K) + tuple(v for pair in zip(n, [m] * nd) for v in pair)
    t = padded.reshape(shp)
    perm = (0,) + tuple(2 + 2 * i for i in range(nd)) + (1,) + tuple(3 + 2 * i for i in range(nd))
    t = t.transpose(perm).reshape((B * int(np.prod(n)), K) + (m,) * nd)
    t = t + 0
    # garbage in the cropped part of edge tiles must not leak
    got = tiles.wino_concat(t, osize, m)
    assert got.shape == y.shape and np.array_equal(got, y)
