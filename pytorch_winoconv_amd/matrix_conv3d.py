"""3-D conv32 / conv16 / conv / base_conv32 with the reference's signatures
(reference: matrix_conv3d.py:70-290).  Same engine and same differences as matrix_conv."""
import torch

from . import engine
from .matrix_conv import A, B, G, matrix_alloc, _run  # noqa: F401
from .Split_and_Concat import wino_split, wino_concat  # noqa: F401


def conv16(input, kernel, bias=None, stride=(1, 1, 1), padding=0, groups=1, output_block=2):
    """reference: matrix_conv3d.py:70-90"""
    return _run(input, kernel, bias, stride, padding, groups, output_block, torch.float16).float()


def conv32(input, kernel, bias=None, stride=(1, 1, 1), padding=0, groups=1, output_block=2):
    """reference: matrix_conv3d.py:92-110"""
    return _run(input, kernel, bias, stride, padding, groups, output_block, torch.float32)


def conv(input, kernel, output_block, stride, fp16=False):
    """reference: matrix_conv3d.py:112-137"""
    dtype = torch.float16 if fp16 else torch.float32
    out = _run(input, kernel, None, 1, 0, 1, output_block, dtype)
    return out.float() if fp16 else out


def base_conv32(input, kernel, fp16, m, r):
    """Tile-domain 3-D Winograd (reference: matrix_conv3d.py:139-290): tiles (P, C, a, a, a) ->
    (P, K, m, m, m)."""
    if list(input.shape[2:]) != [mi + ri - 1 for mi, ri in zip(m, r)]:
        raise ValueError("base_conv32: tiles do not match F(%r, %r)" % (m, r))
    dtype = torch.float16 if fp16 else input.dtype
    return engine.conv_forward(input.to(dtype), kernel.to(dtype), None, 1, 0, int(m[0])).contiguous()
