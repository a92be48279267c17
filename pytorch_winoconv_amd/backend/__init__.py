"""Stand-in for the reference's compiled extension module `MakePytorchBackend`
(reference: pybind/bind.cpp:10-24, pybind/extern.hpp:1-9): the same five names with the same
positional signatures - Foo, AddGPU, WinoSplit, WinoConcat, DWM - plus the two entry points
named after the reference's source files, `winograd_conv` (src/winograd_conv.cpp) and
`split_and_concat` (src/split_and_concat.cpp).

Every tensor function hands raw device pointers to libwinoconv_hip.so (include/winoconv.h) on
torch's current HIP stream.  Differences from the reference, all widening: float16 is
dispatched by tensor dtype (the reference binds float only: bind.cpp:19-23), errors raise
Python exceptions instead of exit(-1) (src/winograd_conv.cpp:80-84,116-126), stride 2 works,
and every kernel extent 1..10 works (the reference's table lacks e.g. 1x3x3:
src/base_conv_launchers.h:59-121).
"""
import ctypes

import torch

from .. import _lib, engine
from ..engine import (_ptr, _stream, _require_gpu, _w_strides, make_desc, out_dims)


class Foo:
    """Template-demo class of the reference extension (pybind/bind.cpp:11-16, src/foo.cpp)."""

    def __init__(self):
        self._key = 0

    def setKey(self, key):
        self._key = int(key)

    def getKey(self):
        return self._key

    def __repr__(self):
        return "< Foo, key: %d > " % self._key


def AddGPU(in_a, in_b, out_c):
    """Template-demo element-wise add (src/add.cpp:9-31): out_c is resized like in_a and
    receives in_a + in_b.  Tutorial scaffolding of the reference, kept importable; it is
    not part of the convolution path and simply uses torch's add."""
    if in_a.numel() != in_b.numel():
        raise ValueError("AddGPU: inputs must have the same number of elements")   # src/add.cpp:14-17
    out_c.resize_(in_a.shape)
    torch.add(in_a, in_b.view_as(in_a), out=out_c)


def _check_out(out, shape, like, what):
    if tuple(out.shape) != tuple(shape) or out.dtype != like.dtype or out.device != like.device \
            or not out.is_contiguous():
        raise ValueError("%s: output must be a contiguous %s tensor of shape %r on %s"
                         % (what, like.dtype, tuple(shape), like.device))


def WinoSplit(in_a, out, block_D, block_H, block_W, output_block_size, nD, nH, nW, two_dimension):
    """in_a channel-last (B, [D,] H, W, C) -> out (B*[nD*]nH*nW, C, [block_D,] block_H, block_W)
    (reference: src/split_and_concat.cpp:14-40)."""
    _require_gpu(in_a, out)
    if not in_a.is_contiguous():
        raise ValueError("WinoSplit: in_a must be contiguous channel-last")
    lib, m, es = _lib.load(), int(output_block_size), in_a.element_size()
    if two_dimension:
        B, H, W, C = in_a.shape
        _check_out(out, (B * nH * nW, C, block_H, block_W), in_a, "WinoSplit")
        _lib.check(lib.wc_wino_split2d(_ptr(in_a), _ptr(out), B, H, W, C, block_H, block_W, m, nH, nW,
                                       es, _stream(in_a)))
    else:
        B, D, H, W, C = in_a.shape
        _check_out(out, (B * nD * nH * nW, C, block_D, block_H, block_W), in_a, "WinoSplit")
        _lib.check(lib.wc_wino_split3d(_ptr(in_a), _ptr(out), B, D, H, W, C, block_D, block_H, block_W,
                                       m, nD, nH, nW, es, _stream(in_a)))


def WinoConcat(in_a, out, output_block_size, two_dimension):
    """in_a (B*[nD*]nH*nW, K, [m,] m, m) -> out channel-last (B, [oD,] oH, oW, K), cropped
    (reference: src/split_and_concat.cpp:44-76; like there, the output extents are read from
    `out` and B follows from the tile count)."""
    _require_gpu(in_a, out)
    if not in_a.is_contiguous() or not out.is_contiguous():
        raise ValueError("WinoConcat: tensors must be contiguous")
    lib, m, es = _lib.load(), int(output_block_size), in_a.element_size()
    N, K = in_a.shape[:2]
    osz = list(out.shape[1:-1])
    per = 1
    for o in osz:
        per *= (o + m - 1) // m
    B = N // per
    if B * per != N or out.shape[0] != B or out.shape[-1] != K or out.dtype != in_a.dtype:
        raise ValueError("WinoConcat: %d tiles of %d channels do not fill an output of shape %r"
                         % (N, K, tuple(out.shape)))
    if two_dimension:
        _lib.check(lib.wc_wino_concat2d(_ptr(in_a), _ptr(out), B, osz[0], osz[1], K, m, es, _stream(in_a)))
    else:
        _lib.check(lib.wc_wino_concat3d(_ptr(in_a), _ptr(out), B, osz[0], osz[1], osz[2], K, m, es,
                                        _stream(in_a)))


def split_and_concat(direction, in_a, out, *args):
    """One entry point for both tile copies: split_and_concat("split", in_a, out, block_D,
    block_H, block_W, output_block_size, nD, nH, nW, two_dimension) or
    split_and_concat("concat", in_a, out, output_block_size, two_dimension)."""
    if direction == "split":
        return WinoSplit(in_a, out, *args)
    if direction == "concat":
        return WinoConcat(in_a, out, *args)
    raise ValueError("split_and_concat: direction must be 'split' or 'concat'")


def winograd_conv(Input, Weight, Output, bias=None, stride=1, padding=0, m=2, algo="dwm", U=None,
                  chunk_images=0, stacked=None):
    """Whole convolution on channel-last tensors, written into `Output`.

    Input (B, D, H, W, C) contiguous; Weight any strided view whose dims are (kD, kH, kW, C, K)
    (the reference's layout, dwm.py:85,133); Output (B, oD, oH, oW, K) contiguous.  A 2-D
    problem has D = kD = 1.  `padding` is (pD, pH, pW) or one int; `m` is the Winograd output
    tile (4 allowed for 2-D 3x3 stride 1); kernels larger than 3 or stride 2 are decomposed
    (algo "dwm"); algo "whole" keeps a square 2-D kernel of 4..7 taps as one F(2,k) x F(2,k) tile,
    the arithmetic of the reference's matrix_conv path (matrix_conv.py:112-135).  `U` is an
    optional filter transformed earlier by engine.transform_filter with the same options;
    `stacked` as in engine.conv_forward (None chooses)."""
    if algo not in ("dwm", "whole"):
        raise ValueError("winograd_conv: algo must be 'dwm' or 'whole', got %r" % (algo,))
    whole = algo == "whole"
    if Weight.dim() == 5:
        if bias is not None and bias.dtype != Input.dtype and bias.dim() == 1 and bias.numel() == Weight.shape[4]:
            bias = bias.to(Input.dtype)
        engine.check_operands(Input, int(Weight.shape[4]), bias, U)
    _require_gpu(Input, Weight, Output, bias, U)
    if Input.dim() != 5 or Weight.dim() != 5 or Output.dim() != 5:
        raise ValueError("winograd_conv: expected 5-D channel-last Input/Output and a 5-D Weight")
    if not Input.is_contiguous() or not Output.is_contiguous():
        raise ValueError("winograd_conv: Input and Output must be contiguous")
    if Weight.dtype != Input.dtype or Output.dtype != Input.dtype:
        raise TypeError("winograd_conv: Input, Weight and Output must share one dtype")
    lib = _lib.load()
    B, D, H, W, C = Input.shape
    kD, kH, kW, Cw, K = Weight.shape
    if Cw != C:
        raise ValueError("winograd_conv: Input has %d channels, Weight expects %d" % (C, Cw))
    flat = D == 1 and kD == 1
    if isinstance(padding, int):
        padding = (0 if flat else padding, padding, padding)
    w_kc = Weight.permute(4, 3, 0, 1, 2)                 # (K, C, kD, kH, kW) view, no copy
    # `stacked` left open (None) goes to the library as it is, which then also may take the direct form: the same
    # call of wc_conv_auto that the compiled host layer makes, so both bindings run the same plan
    unfused = engine.misaligned(Input, Output, U)        # the one-kernel path of thin layers wants 16-byte alignment
    if flat:
        desc = make_desc((B, C, H, W), (K, C, kH, kW), Input.dtype, stride, padding[1:], m, chunk_images, whole,
                         stacked, unfused)
    else:
        desc = make_desc((B, C, D, H, W), (K, C, kD, kH, kW), Input.dtype, stride, padding, m, chunk_images, whole,
                         stacked, unfused)
    engine.check_u(desc, U)
    out, _ = out_dims(desc)
    _check_out(Output, (B, out[0], out[1], out[2], K), Input, "winograd_conv")
    nbytes = ctypes.c_size_t()
    _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=Input.device)
    strides = (ctypes.c_int64 * 5)(*w_kc.stride())
    if bias is not None:
        bias = bias.contiguous()
    _lib.check(lib.wc_conv_forward(ctypes.byref(desc), _ptr(Input), _ptr(w_kc), strides, _ptr(U),
                                   _ptr(bias), _ptr(Output), _ptr(ws), nbytes.value, _stream(Input)))


def DWM(Input, Weight, Output, stride, tmp_input_buffer=None, tmp_weight_buffer=None,
        tmp_product_buffer=None, tmp_ptr_buffer=None):
    """The reference's native entry point (pybind/extern.hpp:7-9, src/winograd_conv.cpp:17-127):
    VALID convolution of Input (B, D, H, W, C) with Weight (kD, kH, kW, C, K) into Output
    (B, oD, oH, oW, K).  The four scratch tensors of the reference signature are accepted and
    ignored: the engine sizes its own workspace (transformed buffers are laid out differently
    and no pointer table is needed)."""
    winograd_conv(Input, Weight, Output, None, int(stride), 0, 2, "dwm")
