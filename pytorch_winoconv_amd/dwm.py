"""dwm2d / dwm3d with the reference's signatures (reference: dwm.py:5-145).

Differences from the reference: `stride` is honoured (1 or 2; the reference drops it,
dwm.py:13,32), `padding` may be an int as well as a tuple (the reference pads only for
tuples, dwm.py:6-8,26-28) and is applied inside the input transform instead of by F.pad,
the bias is added in fp32 inside the output transform, nothing is printed, float16 is
accepted, and the result is an NC[D]HW tensor in channel-last memory.
"""
import torch

from . import engine


def _norm_stride(stride, nd):
    if isinstance(stride, int):
        return stride
    s = tuple(int(v) for v in stride)
    if len(set(s)) != 1:
        raise NotImplementedError("dwm: stride must be equal on all axes, got %r" % (stride,))
    return s[0]


def _dwm(input, kernel, bias, stride, padding, groups, nd, output_block=2):
    if groups != 1:
        raise NotImplementedError("dwm: groups != 1 is not supported")
    if input.dim() != nd + 2 or kernel.dim() != nd + 2:
        raise ValueError("dwm%dd: expected %d-D input and kernel" % (nd, nd + 2))
    if bias is not None:
        bias = bias.type_as(input)                                   # dwm.py:18,36
    return engine.conv_forward(input, kernel.type_as(input), bias, _norm_stride(stride, nd), padding,
                               int(output_block))


def dwm3d(input, kernel, bias=None, stride=(1, 1, 1), padding=0, groups=1, output_block=2):
    """3-D DWM convolution (reference: dwm.py:5-23).  output_block = 2 is the reference's
    F(2,r)^3 arithmetic; 4 (3x3x3 kernels at stride 1 only) uses the tile 2 x 4 x 4 - F(2,3) along
    depth, F(4,3) along height and width - which moves 1.8x fewer transform-domain elements (fp16
    error about 1.3e-2 of the output range instead of 8e-4, inside the 2e-2 bound)."""
    return _dwm(input, kernel, bias, stride, padding, groups, 3, output_block)


def dwm2d(input, kernel, bias=None, stride=(1, 1), padding=0, groups=1, output_block=2):
    """2-D DWM convolution (reference: dwm.py:25-40).  output_block = 2 is the reference's F(2,r)
    decomposition; 4 uses F(4,r) pieces (about 1.3x faster for 5x5 / 7x7 kernels, fp16 error
    about 10x larger but inside the 2e-2 bound)."""
    return _dwm(input, kernel, bias, stride, padding, groups, 2, output_block)


def dwm3d_(x, w, stride=1):
    """VALID 3-D DWM convolution (reference: dwm.py:43-107)."""
    return _dwm(x, w, None, stride, 0, 1, 3)


def dwm2d_(x, w, stride=1):
    """VALID 2-D DWM convolution (reference: dwm.py:109-145)."""
    return _dwm(x, w, None, stride, 0, 1, 2)
