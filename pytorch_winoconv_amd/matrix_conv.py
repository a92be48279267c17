"""conv32 / conv16 / conv / base_conv32 with the reference's signatures
(reference: matrix_conv.py:70-254).

The reference expresses the transforms and the product as torch matmuls on tiles produced by
wino_split; here the same functions run the HIP engine.  Like the reference, a square 2-D
kernel of 4..7 taps at stride 1 and output_block 2 is one whole-kernel tile F(2,k) x F(2,k)
built from the reference's interpolation points (matrix_conv.py:31-35) - this is the
arithmetic whose loss of accuracy in fp16 the DWM decomposition (dwm.py) avoids; pass
decompose=True to get the decomposition here too.  Every other kernel larger than 3 (non-square,
above 7 taps, 3-D, output_block 4) and stride 2 - for which the reference falls back to
F.conv2d (matrix_conv.py:71-75,93-95) - is decomposed into pieces of <= 3 taps.
"""
import numpy as np
import torch

from . import engine, wincnn
from .Split_and_Concat import wino_split, wino_concat  # noqa: F401  (re-exported like the reference)

# transform tables under the reference's names: A = AT (m x alpha), G (alpha x r), B = BT
A, G, B = {}, {}, {}
A[(2, 1)] = np.array([[1., 0.], [0., 1.]])
G[(2, 1)] = np.array([[1.], [1.]])
B[(2, 1)] = np.array([[1., 0.], [0., 1.]])
A[(2, 2)] = np.array([[1., 1., 0.], [0., 1., 1.]])
G[(2, 2)] = np.array([[1., 0.], [1., 1.], [0., 1.]])
B[(2, 2)] = np.array([[1., -1., 0.], [0., 1., 0.], [0., -1., 1.]])
A[(2, 3)] = np.array([[1., 1., 1., 0.], [0., 1., -1., -1.]])
G[(2, 3)] = np.array([[1., 0., 0.], [.5, .5, .5], [.5, -.5, .5], [0., 0., 1.]])
B[(2, 3)] = np.array([[1., 0., -1., 0.], [0., 1., 1., 0.], [0., -1., 1., 0.], [0., 1., 0., -1.]])
A[(4, 1)] = np.eye(4)
G[(4, 1)] = np.ones((4, 1))
B[(4, 1)] = np.eye(4)
A[(4, 2)] = np.array([[1., 1., 1., 1., 0.], [0., 1., -1., 2., 0.], [0., 1., 1., 4., 0.], [0., 1., -1., 8., 1.]])
G[(4, 2)] = np.array([[1 / 2., 0.], [-1 / 2., -1 / 2.], [-1 / 6., 1 / 6.], [1 / 6., 1 / 3.], [0., 1.]])
B[(4, 2)] = np.array([[2., -1., -2., 1., 0.], [0., -2., -1., 1., 0.], [0., 2., -3., 1., 0.],
                      [0., -1., 0., 1., 0.], [0., 2., -1., -2., 1.]])
A[(4, 3)] = np.array([[1., 1., 1., 1., 1., 0.], [0., 1., -1., 2., -2., 0.],
                      [0., 1., 1., 4., 4., 0.], [0., 1., -1., 8., -8., 1.]])
G[(4, 3)] = np.array([[1 / 4., 0., 0.], [-1 / 6., -1 / 6., -1 / 6.], [-1 / 6., 1 / 6., -1 / 6.],
                      [1 / 24., 1 / 12., 1 / 6.], [1 / 24., -1 / 12., 1 / 6.], [0., 0., 1.]])
B[(4, 3)] = np.array([[4., 0., -5., 0., 1., 0.], [0., -4., -4., 1., 1., 0.], [0., 4., -4., -1., 1., 0.],
                      [0., -2., -1., 2., 1., 0.], [0., 2., -1., -2., 1., 0.], [0., 4., 0., -5., 0., 1.]])
# whole-kernel tiles, generated like the reference does (matrix_conv.py:31-35)
points = (0, 1, -1, "1/2", "-1/2", "1/3", "-1/3", "3/2", "-3/2", -3, 2, -2)
A[(2, 4)], G[(2, 4)], B[(2, 4)] = wincnn.showCookToomFilter((0, 1, -1, 2), 2, 4)
A[(2, 5)], G[(2, 5)], B[(2, 5)] = wincnn.showCookToomFilter((0, 1, -1, 2, -2), 2, 5)
A[(2, 6)], G[(2, 6)], B[(2, 6)] = wincnn.showCookToomFilter(points, 2, 6)
A[(2, 7)], G[(2, 7)], B[(2, 7)] = wincnn.showCookToomFilter(points, 2, 7)


def matrix_alloc(m, r):
    """Transform matrices for every axis (reference: matrix_conv.py:42-68); raises instead of
    sys.exit when a size is not available."""
    A_, B_, G_ = [], [], []
    for mi, ri in zip(m, r):
        if (mi, ri) not in A:
            raise NotImplementedError("Size Error: F(%d, %d) not implemented yet." % (ri, mi))
        A_.append(torch.from_numpy(A[(mi, ri)]))
        B_.append(torch.from_numpy(B[(mi, ri)]))
        G_.append(torch.from_numpy(G[(mi, ri)]))
    return A_, B_, G_


def _same_stride(stride):
    s = (stride,) if isinstance(stride, int) else tuple(int(v) for v in stride)
    if len(set(s)) != 1:
        raise NotImplementedError("stride must be equal on all axes, got %r" % (stride,))
    return s[0]


def _whole_kernel(kernel, stride, m, decompose):
    ks = tuple(kernel.shape[2:])
    return (not decompose and len(ks) == 2 and ks[0] == ks[1] and 4 <= ks[0] <= 7
            and stride == 1 and m == 2)


def _run(input, kernel, bias, stride, padding, groups, output_block, dtype, decompose=False):
    if groups != 1:
        raise NotImplementedError("groups != 1 is not supported")
    x = input.to(dtype)
    w = kernel.to(dtype)
    b = None if bias is None else bias.to(dtype)
    s = _same_stride(stride)
    m = int(output_block)
    return engine.conv_forward(x, w, b, s, padding, m, whole_kernel=_whole_kernel(w, s, m, decompose))


def conv16(input, kernel, bias=None, stride=(1, 1), padding=0, groups=1, output_block=2, decompose=False):
    """Half-precision Winograd convolution returning float32 (reference: matrix_conv.py:70-90)."""
    return _run(input, kernel, bias, stride, padding, groups, output_block, torch.float16, decompose).float()


def conv32(input, kernel, bias=None, stride=(1, 1), padding=0, groups=1, output_block=2, decompose=False):
    """Single-precision Winograd convolution (reference: matrix_conv.py:92-110)."""
    return _run(input, kernel, bias, stride, padding, groups, output_block, torch.float32, decompose)


def conv(input, kernel, output_block, stride, fp16=False, decompose=False):
    """VALID stride-1 convolution (reference: matrix_conv.py:112-135)."""
    dtype = torch.float16 if fp16 else torch.float32
    out = _run(input, kernel, None, 1, 0, 1, output_block, dtype, decompose)
    return out.float() if fp16 else out


def base_conv32(input, kernel, fp16, m, r):
    """Tile-domain Winograd: tiles (P, C, a_h, a_w) and kernel (K, C, r_h, r_w) -> (P, K, m_h, m_w)
    (reference: matrix_conv.py:137-254).  Each tile is a complete little VALID convolution
    problem with exactly one Winograd tile, so it runs through the same engine."""
    if len(set(m)) != 1:
        raise NotImplementedError("base_conv32: output tile must be square")
    if list(input.shape[2:]) != [mi + ri - 1 for mi, ri in zip(m, r)]:
        raise ValueError("base_conv32: tiles of shape %r do not match F(%r, %r)" % (tuple(input.shape[2:]), m, r))
    dtype = torch.float16 if fp16 else input.dtype
    return engine.conv_forward(input.to(dtype), kernel.to(dtype), None, 1, 0, int(m[0]),
                               whole_kernel=_whole_kernel(kernel, 1, int(m[0]), False)).contiguous()
