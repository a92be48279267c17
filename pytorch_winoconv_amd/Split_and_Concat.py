"""wino_split / wino_concat with the reference's signatures (reference: Split_and_Concat.py:4-82).

Differences from the reference, none visible in the results for output_block_size = 2:
the tile step follows output_block_size (the reference kernels hard-code 2:
src/split_and_concat_kernels.cu:20-22,87-88), float16 is accepted besides float32, the
tensors stay on the device of the input and a channel-last input is used without a copy.
"""
import ctypes

import torch

from . import _lib
from .engine import _ptr, _stream, _require_gpu, channel_last, channel_first_view


def wino_split(a, w_shape, output_block_size):
    """a (B, C, [D,] H, W) -> tiles (B*[nD*]nH*nW, C, [bD,] bH, bW), b = w + m - 1."""
    _require_gpu(a)
    lib = _lib.load()
    m = int(output_block_size)
    nd = a.dim() - 2
    if nd not in (2, 3) or len(w_shape) != nd + 2:
        raise ValueError("wino_split: expected a 4-D/5-D input and a matching filter shape")
    B, C = a.shape[:2]
    sp = list(a.shape[2:])
    blocks = [int(w) + m - 1 for w in w_shape[2:]]
    n = [int((X + 1 - b) / m + 1) for X, b in zip(sp, blocks)]      # Split_and_Concat.py:21-23,40-41
    a_cl = channel_last(a)                                          # Split_and_Concat.py:25,47
    n_tiles = B
    for v in n:
        n_tiles *= v
    out = torch.empty([n_tiles, C] + blocks, dtype=a.dtype, device=a.device)
    es = a.element_size()
    if nd == 2:
        _lib.check(lib.wc_wino_split2d(_ptr(a_cl), _ptr(out), B, sp[0], sp[1], C, blocks[0], blocks[1],
                                       m, n[0], n[1], es, _stream(a)))
    else:
        _lib.check(lib.wc_wino_split3d(_ptr(a_cl), _ptr(out), B, sp[0], sp[1], sp[2], C, blocks[0],
                                       blocks[1], blocks[2], m, n[0], n[1], n[2], es, _stream(a)))
    return out


def wino_concat(a, output_size, output_block_size):
    """a (B*[nD*]nH*nW, K, [m,] m, m) -> (B, K, [oD,] oH, oW) with partial edge tiles cropped."""
    _require_gpu(a)
    lib = _lib.load()
    m = int(output_block_size)
    nd = len(output_size)
    if nd not in (2, 3) or a.dim() != nd + 2:
        raise ValueError("wino_concat: tiles and output_size disagree")
    osz = [int(o) for o in output_size]
    n = [(o + m - 1) // m for o in osz]                              # Split_and_Concat.py:58-60,72-73
    per_image = 1
    for v in n:
        per_image *= v
    N, K = a.shape[:2]
    if N % per_image:
        raise ValueError("wino_concat: %d tiles is not a multiple of %d tiles per image" % (N, per_image))
    B = N // per_image
    a = a.contiguous()
    out = torch.empty([B] + osz + [K], dtype=a.dtype, device=a.device)
    es = a.element_size()
    if nd == 2:
        _lib.check(lib.wc_wino_concat2d(_ptr(a), _ptr(out), B, osz[0], osz[1], K, m, es, _stream(a)))
    else:
        _lib.check(lib.wc_wino_concat3d(_ptr(a), _ptr(out), B, osz[0], osz[1], osz[2], K, m, es, _stream(a)))
    return channel_first_view(out)                                   # Split_and_Concat.py:65,81
