"""Host-side orchestration over the C ABI: descriptors, plans, workspaces, streams.

torch is used for device memory (its caching allocator) and for the current HIP
stream only; all arithmetic is done by the HIP kernels behind libwinoconv_hip.so.
"""
import ctypes

import torch

from . import _lib
from ._lib import ConvDesc, Plan, check

# The compiled host layer (csrc/host/make_pytorch_backend.cpp, built by build()): conv_forward goes through it
# when it is there - same C ABI, a few microseconds of C++ per call instead of some twenty of Python.  Without
# it (a host with hipcc's output but no C++ build of the module) the ctypes path below does the same work.
try:
    from . import MakePytorchBackend as _ext
except ImportError:
    _ext = None
USE_EXT = _ext is not None

_DTYPES = {torch.float32: _lib.WC_F32, torch.float16: _lib.WC_F16, torch.bfloat16: _lib.WC_BF16}


def _ptr(t):
    return ctypes.c_void_p(t.data_ptr()) if t is not None else ctypes.c_void_p(0)


def _stream(t):
    return ctypes.c_void_p(torch.cuda.current_stream(t.device).cuda_stream)


def _require_gpu(*tensors):
    for t in tensors:
        if t is None:
            continue
        if not t.is_cuda:
            raise ValueError("winoconv runs on the GPU only: got a %s tensor" % t.device)
        if t.dtype not in _DTYPES:
            raise TypeError("winoconv supports float32, float16 and bfloat16, got %s" % t.dtype)


def check_operands(x, K, bias=None, U=None):
    """Shapes and types the C ABI cannot see: the bias must hold K values of x's dtype, a transformed
    filter must have x's dtype and device (its size is checked by check_u).  Raises before anything
    is launched; the kernels would read a short bias out of bounds and a filter of another type as
    garbage."""
    if bias is not None:
        if bias.dim() != 1 or bias.numel() != K:
            raise ValueError("bias must be a 1-D tensor of %d values (one per output channel), got shape %r"
                             % (K, tuple(bias.shape)))
        if bias.dtype != x.dtype:
            raise TypeError("bias is %s, the input is %s: they must share one dtype" % (bias.dtype, x.dtype))
        if bias.device != x.device:
            raise ValueError("bias is on %s, the input on %s" % (bias.device, x.device))
    if U is not None:
        if U.dtype != x.dtype:
            raise TypeError("the transformed filter is %s, the input is %s: transform the filter in the input's dtype"
                            % (U.dtype, x.dtype))
        if U.device != x.device:
            raise ValueError("the transformed filter is on %s, the input on %s" % (U.device, x.device))


def misaligned(*tensors):
    """True if one of the tensors does not start on a 16-byte boundary."""
    return any(t is not None and t.data_ptr() % 16 != 0 for t in tensors)


def _triple(v, nd, fill):
    if isinstance(v, int):
        v = (v,) * nd
    v = tuple(int(a) for a in v)
    if len(v) != nd:
        raise ValueError("expected %d values, got %r" % (nd, v))
    return ((fill,) if nd == 2 else ()) + v


def make_desc(x_shape, w_shape, dtype, stride=1, padding=0, m=2, chunk_images=0, whole_kernel=False, stacked=False,
              unfused=False, x_layout=0, y_layout=0, direct=None):
    """Descriptor for an NC[D]HW input and a (K, C, [kD,] kH, kW) filter.  `whole_kernel`: one
    F(2,k) tile per axis for a k x k kernel, k = 4..7, instead of the DWM pieces.  `stacked`: the
    DWM pieces share one tile and are added by the batched GEMM instead of by the output transform
    (2-D; same sum, fewer bytes moved for kernels above 3 x 3)."""
    nd = len(x_shape) - 2
    if nd not in (2, 3) or len(w_shape) != nd + 2:
        raise ValueError("expected 4-D or 5-D input and matching filter, got %r and %r"
                         % (tuple(x_shape), tuple(w_shape)))
    if x_shape[1] != w_shape[1]:
        raise ValueError("input has %d channels, filter expects %d (groups are not supported)"
                         % (x_shape[1], w_shape[1]))
    if isinstance(stride, (tuple, list)):
        if len(set(int(s) for s in stride)) != 1:
            raise NotImplementedError("stride must be the same on every axis, got %r" % (stride,))
        stride = int(stride[0])
    d = ConvDesc()
    d.ndim = nd
    d.N, d.C, d.K = int(x_shape[0]), int(x_shape[1]), int(w_shape[0])
    d.in_[:] = ((1,) if nd == 2 else ()) + tuple(int(v) for v in x_shape[2:])
    d.kernel[:] = ((1,) if nd == 2 else ()) + tuple(int(v) for v in w_shape[2:])
    d.pad[:] = _triple(padding, nd, 0)
    d.stride = int(stride)
    d.m = int(m)
    d.dtype = _DTYPES[dtype]
    d.chunk_images = int(chunk_images)
    d.whole_kernel = int(bool(whole_kernel))
    d.stacked = -1 if stacked is None else 2 if stacked == 2 else int(bool(stacked))
    # the direct form (wc_conv_desc.direct): True asks for it, False rules it out, None leaves it to the library,
    # which takes it for 16-bit stride-2 layers when `stacked` is left open too
    d.direct = 1 if direct else (-1 if direct is False else 0)
    # what is left open is filled in by the library: the form of the plan if `stacked` is None, and the tile
    # 3 or 2 where a caller asked for tile 4 and gets the shared-input plan, which has no such tile (d.m then
    # tells the tile really used)
    check(_lib.load().wc_conv_auto(ctypes.byref(d)))
    d.unfused = int(bool(unfused))
    d.x_layout, d.y_layout = int(x_layout), int(y_layout)     # 1: channel-first contiguous memory (wc_conv_desc.x_layout)
    return d


def effective_tile(x_shape, w_shape, dtype, stride=1, padding=0, m=2, whole_kernel=False, stacked=None):
    """The output tile conv_forward really uses for this problem and the plan form it picks: (m, stacked).  A
    caller who asks for tile 4 gets 3 or 2 where the plan whose pieces share one transformed input is chosen
    (that plan has no tile 4), and the accuracy is that of the smaller tile."""
    d = make_desc(x_shape, w_shape, dtype, stride, padding, m, 0, whole_kernel, stacked)
    return d.m, d.stacked


def plan_form(x_shape, w_shape, dtype, stride=1, padding=0, m=2):
    """(direct, stacked, tile) of the plan conv_forward runs for this problem with everything left to the library:
    what a cached transformed filter depends on beside the filter itself (the library's choice between the
    Winograd pieces and the direct form looks at the batch size)."""
    pad = padding if isinstance(padding, int) else tuple(padding)
    d = _forward_setup(tuple(x_shape), tuple(w_shape), dtype, stride, pad, m, 0, False, None)[0]
    return int(d.direct), int(d.stacked), int(d.m)


def plan_conv(desc):
    plan = Plan()
    check(_lib.load().wc_plan_conv(ctypes.byref(desc), ctypes.byref(plan)))
    return plan


def out_dims(desc):
    out = (ctypes.c_int * 3)()
    grid = (ctypes.c_int * 3)()
    check(_lib.load().wc_conv_out_dims(ctypes.byref(desc), out, grid))
    return list(out), list(grid)


def plan_dwm(kD, kH, kW):
    """The reference's splitControl() table for one kernel size, as a dict of lists."""
    arrs = [(ctypes.c_int * _lib.WC_MAX_PIECES)() for _ in range(7)]
    n, t = ctypes.c_int(), ctypes.c_int()
    check(_lib.load().wc_plan_dwm(kD, kH, kW, ctypes.byref(n), *arrs, ctypes.byref(t)))
    names = ("D_start", "D_end", "H_start", "H_end", "W_start", "W_end", "kernel_stride")
    out = {k: list(a[:n.value]) for k, a in zip(names, arrs)}
    out["T_total"] = t.value
    return out


def channel_last(x):
    """(N, C, *sp) tensor -> contiguous (N, *sp, C) view; zero-copy for channels_last memory."""
    nd = x.dim() - 2
    perm = (0,) + tuple(range(2, 2 + nd)) + (1,)
    v = x.permute(perm)
    return v if v.is_contiguous() else v.contiguous()


def channel_first_view(y_cl):
    """(N, *sp, K) contiguous tensor -> (N, K, *sp) view (channels_last memory format)."""
    nd = y_cl.dim() - 2
    return y_cl.permute((0, nd + 1) + tuple(range(1, nd + 1)))


def _w_strides(w):
    """Element strides of a (K, C, [kD,] kH, kW) filter view as (K, C, kD, kH, kW)."""
    s = list(w.stride())
    if w.dim() == 4:
        s = s[:2] + [0] + s[2:]
    return (ctypes.c_int64 * 5)(*s)


# ---------------------------------------------------------------- stages (used by the tests)
def _row(desc, plan):
    """Row length of U and V: the padded channel count, times the pieces of a stacked plan."""
    return _lib.load().wc_padded_channels(desc.C) * (plan.n_pieces if desc.stacked else 1)


def filter_transform(desc, plan, w):
    _require_gpu(w)
    U = torch.empty(plan.t_total, desc.K, _row(desc, plan), dtype=w.dtype, device=w.device)
    check(_lib.load().wc_filter_transform(ctypes.byref(desc), ctypes.byref(plan), _ptr(w),
                                          _w_strides(w), _ptr(U), _stream(w)))
    return U


def input_transform(desc, plan, x_cl):
    _require_gpu(x_cl)
    lib = _lib.load()
    _, grid = out_dims(desc)
    n = x_cl.shape[0]
    P = n * grid[0] * grid[1] * grid[2]
    if desc.stacked == 2 and plan.n_pieces > 1:
        # one piece over the extended tile grid, plus the rows the shifted reads of the last tiles reach
        # (stride 2: the even and the odd samples of each axis are phases side by side in a row of V,
        # and the pieces are cut from the ceil(k / 2) taps of a phase)
        taps = [(k + 1) // 2 if desc.stride == 2 else k for k in desc.kernel]
        phases = 1
        for k in desc.kernel:
            phases *= 2 if (desc.stride == 2 and k >= 2) else 1
        per = [(t + desc.m - 1) // desc.m for t in taps]               # pieces per axis
        tail = (per[0] - 1) * grid[1] * grid[2] + (per[1] - 1) * grid[2] + per[2] - 1
        V = torch.zeros(plan.t_total, P + tail, phases * lib.wc_padded_channels(desc.C), dtype=x_cl.dtype, device=x_cl.device)
    else:
        V = torch.empty(plan.t_total, P, _row(desc, plan), dtype=x_cl.dtype, device=x_cl.device)
    check(lib.wc_input_transform(ctypes.byref(desc), ctypes.byref(plan), _ptr(x_cl), n, _ptr(V), _stream(x_cl)))
    return V


def batched_gemm(V, U):
    _require_gpu(V, U)
    lib = _lib.load()
    T, P, Cp = V.shape
    K = U.shape[1]
    if U.shape[0] != T or U.shape[2] != Cp or not V.is_contiguous() or not U.is_contiguous():
        raise ValueError("V (T,P,Cp) and U (T,K,Cp) must be contiguous and agree on T and Cp")
    ldm = lib.wc_padded_channels8(K)
    M = torch.empty(T, P, ldm, dtype=V.dtype, device=V.device)
    check(lib.wc_batched_gemm(_ptr(V), _ptr(U), _ptr(M), T, P, Cp, K, ldm, _DTYPES[V.dtype], _stream(V)))
    return M


def output_transform(desc, plan, M, bias, n_images):
    _require_gpu(M, bias)
    lib = _lib.load()
    out, _ = out_dims(desc)
    y = torch.empty(n_images, out[0], out[1], out[2], desc.K, dtype=M.dtype, device=M.device)
    check(lib.wc_output_transform(ctypes.byref(desc), ctypes.byref(plan), _ptr(M), _ptr(bias),
                                  n_images, _ptr(y), _stream(M)))
    return y


# ---------------------------------------------------------------- whole convolution
def _stack(stacked, dtype, nd, whole_kernel, w_shape=None, stride=1, m=2):
    """`stacked=None` picks what measured faster on MI355X (the rule itself lives in the library, wc_conv_auto): pieces summed by the batched GEMM for
    16-bit plans (2-D: 1.15-1.3x for 5x5 and 7x7 kernels; 3-D: 1.05-1.4x; fewer bytes moved); for
    fp32, whose product is bound by the MFMA rate and to which stacking adds zero taps, only 2-D
    plans of up to four pieces (5x5: 1.1-1.15x; 7x7, nine pieces: 0.9-1.0x).  16-bit stride-1
    kernels of 4 to 10 taps over at most 256 input channels (3-D: 4 to 8 taps over at most 128, or
    4 taps over at most 256) get the plan whose two-tap pieces share one transformed input (2;
    make_desc then uses output tile 2).  Against stacked F(2,r) pieces it measured, in 2-D, 1.7x
    (4x4, 7x7), 1.5x (5x5) and 1.15x (9x9) faster at N=16, 256 channels, 56x56, 1.9x (9x9) and 3x
    (10x10) at N=32, 128 channels, 112x112, and the same speed at 512 channels; in 3-D 1.5x (5x5x5)
    to 2x (4x4x4, 7x7x7) with 64 and 128 channels, 1.5x (4x4x4) and 0.9x (5x5x5) with 256.  It is
    also 1.2x (5x5), 1.45x (4x4) and 1.6x (7x7) faster than stacked F(4,r) pieces at N=32, 128
    channels, 112x112.  Where the caller accepts tile 4 (fp16, 2-D, 5 to 10 taps, at
    least 3 on the other axis, at most 256 channels) the shared tile is F(3,3) with the reference's
    three-tap pieces (make_desc: output tile 3): 1.4x (5x5) to 1.8x (7x7, 9x9) faster than stacked
    F(4,r) pieces, also at 256 channels.  At stride 2 the shared-input plan works on the parity phases
    of x (four times the channels, half the taps) and pays where a phase has four taps: 7x7 and 8x8
    kernels, 2-D, at most 256 channels: 1.2x (7x7, 128 channels), 1.45-1.6x (64 channels, and 3 -> 64
    at 224x224) and 1.75x (8x8) faster than stacked F(4,r) pieces and as accurate as F(2,r) (equal
    speed at 256 channels, slower at 512); kernels of 5 or 6 taps (three per phase: pieces without
    taps) are 1.8x slower that way and keep their stacked pieces.  In 3-D (two or four taps per
    phase on every axis, at most 128 channels): 4x4x4 1.75x, 7x7x7 2.5x (64 channels) and 1.65x (128)
    faster than stacked F(2,r) pieces at N=4, 16x28x28."""
    if stacked is not None:
        return 2 if stacked == 2 else bool(stacked)
    if w_shape is None:
        return dtype != torch.float32 and not (whole_kernel or (nd == 3 and m != 2))
    if isinstance(stride, (tuple, list)):
        stride = stride[0]
    d = ConvDesc()
    d.ndim = nd
    d.N, d.C, d.K = 1, int(w_shape[1]), int(w_shape[0])
    d.kernel[:] = ((1,) if nd == 2 else ()) + tuple(int(v) for v in w_shape[2:])
    d.stride, d.m, d.dtype = int(stride), int(m), _DTYPES[dtype]
    d.whole_kernel, d.stacked, d.direct = int(bool(whole_kernel)), -1, -1     # the Winograd / DWM form, the direct one aside
    check(_lib.load().wc_conv_auto(ctypes.byref(d)))
    return 2 if d.stacked == 2 else bool(d.stacked)


def thin_layer(dtype, nd, in_channels, out_channels, kernel, stride):
    """True for the layers wc_conv_forward runs as one fused F(2x2, 3x3) kernel (wc_conv_desc.unfused):
    2-D, 3x3, stride 1 and either at most 4 input channels (any type, at most 512 output channels), or
    fp16 / bf16 with input channels padded to 32, 64 or 128 (an even number up to 32, a multiple of 4 in
    33..64 and 97..128) and at most 512 output channels (256 with 128 input channels), or fp32 with an
    even number of at most 64 input channels and at most 512 output channels (256 above 32 input
    channels).  Callers that cache U use it to transform the filter with tile 2."""
    if nd != 2 or tuple(kernel) != (3, 3):
        return False
    if (stride if isinstance(stride, int) else max(stride)) != 1:
        return False
    if in_channels <= 4:
        return out_channels <= 512
    cp = (in_channels + 31) // 32 * 32
    if dtype == torch.float32:
        return cp <= 64 and in_channels % 2 == 0 and out_channels <= (256 if cp == 64 else 512)
    return (cp in (32, 64, 128) and in_channels % (2 if cp == 32 else 4) == 0
            and out_channels <= (256 if cp == 128 else 512))


def thin_preferred(dtype, nd, in_channels, out_channels, kernel, stride):
    """True where the fused F(2x2, 3x3) kernel also beats the three-kernel path with tile 4, so that a caller
    free to choose the tile should take 2: every 16-bit layer the kernel takes (1.25-1.7x), first layers, and in
    fp32 (where the products run on the eight times slower fp32 MFMA and F(4,3) needs 2.25x fewer of them) layers
    with at most 32 input channels or at most 64 output channels (N=8, 64 -> 64 at 224x224: 160 against 231 us;
    64 -> 128 at 112x112: 92 against 93 us, a tie, so tile 4 there)."""
    if not thin_layer(dtype, nd, in_channels, out_channels, kernel, stride):
        return False
    if dtype != torch.float32 or in_channels <= 4:
        return True
    return in_channels <= 32 or out_channels <= 64


def check_u(desc, U):
    """A transformed filter made with other options (tile, stacking) has another size: refuse it
    rather than read it with the wrong layout."""
    if U is None:
        return
    n = ctypes.c_size_t()
    check(_lib.load().wc_conv_u_elems(ctypes.byref(desc), ctypes.byref(n)))
    if not U.is_contiguous() or U.numel() != n.value:
        raise ValueError("U has %d elements, this convolution needs a contiguous transformed filter of %d "
                         "(transform_filter must be called with the same options)" % (U.numel(), n.value))


def transform_filter(w, x_shape, stride=1, padding=0, m=2, whole_kernel=False, stacked=None, direct=None):
    """Transformed filter U for later calls of conv_forward(..., U=U) with the same options."""
    _require_gpu(w)
    desc = make_desc(x_shape, w.shape, w.dtype, stride, padding, m, 0, whole_kernel, stacked, direct=direct)
    if desc.direct:
        # the filter with its taps outermost and channels innermost, (K, kH, kW, C); strided first layers (at most 4
        # channels) pad every kernel row to 8 taps of 4 channels, (K, kH, 8, 4)
        n = ctypes.c_size_t()
        check(_lib.load().wc_conv_u_elems(ctypes.byref(desc), ctypes.byref(n)))
        shape = (desc.K, desc.kernel[1], desc.kernel[2], desc.C)
        if desc.ndim == 3:
            shape = (desc.K, desc.kernel[0] * desc.kernel[1], 4, 4)      # 3-D first layers: rows of 4 taps of 4 channels
        elif n.value != shape[0] * shape[1] * shape[2] * shape[3]:
            shape = (desc.K, desc.kernel[1], 8, 4)
        U = torch.empty(shape, dtype=w.dtype, device=w.device)
        plan = Plan()
        check(_lib.load().wc_filter_transform(ctypes.byref(desc), ctypes.byref(plan), _ptr(w), _w_strides(w), _ptr(U), _stream(w)))
        return U
    return filter_transform(desc, plan_conv(desc), w)


def conv_forward(x, w, bias=None, stride=1, padding=0, m=2, U=None, chunk_images=0, whole_kernel=False,
                 stacked=None, unfused=False, channels_first_out=False, direct=None):
    """Winograd / DWM convolution of an NC[D]HW tensor.  Returns an NC[D]HW tensor whose memory
    is channel-last (torch.channels_last / channels_last_3d), or, with `channels_first_out`, plain
    contiguous.  A channel-last input is used without a copy; a contiguous (channel-first) one is
    handed to the library as it is (wc_conv_desc.x_layout: small single-piece plans read it inside the
    input transform, the others copy it to channel-last scratch with the library's own kernel); any
    other layout is made contiguous first.  `stacked`: see make_desc; None chooses.
    `unfused=True` keeps thin 16-bit 3x3 layers on the three-kernel path (wc_conv_desc.unfused)."""
    if USE_EXT:
        return _ext.conv_forward(x, w, bias, stride, padding, m, U, chunk_images, bool(whole_kernel), stacked,
                                 bool(unfused), bool(channels_first_out), direct)
    return _conv_forward(x, w, bias, stride, padding, m, U, chunk_images, whole_kernel, stacked, unfused,
                         channels_first_out, direct, None)


STAGES = ("filter_transform", "layout_in", "input_transform", "product", "output_transform", "layout_out")


def conv_forward_timed(x, w, bias=None, stride=1, padding=0, m=2, U=None, chunk_images=0, whole_kernel=False,
                       stacked=None, unfused=False, channels_first_out=False, direct=None):
    """conv_forward through wc_conv_forward_timed: returns (y, {stage: milliseconds on the device}) with the
    stages of STAGES; waits for the device (the reference's timing prints: dwm.py:44-106)."""
    times = (ctypes.c_float * len(STAGES))()
    y = _conv_forward(x, w, bias, stride, padding, m, U, chunk_images, whole_kernel, stacked, unfused,
                      channels_first_out, direct, times)
    return y, dict(zip(STAGES, (float(t) for t in times)))


def _conv_forward(x, w, bias, stride, padding, m, U, chunk_images, whole_kernel, stacked, unfused,
                  channels_first_out, direct, times):
    check_operands(x, int(w.shape[0]), bias, U)
    _require_gpu(x, w, bias, U)
    if w.dtype != x.dtype or (bias is not None and bias.dtype != x.dtype):
        raise TypeError("input, filter and bias must share one dtype")
    lib = _lib.load()
    if x.shape[0] == 0:
        # empty batch: the shape arithmetic is checked on one image, nothing is launched
        out, _ = out_dims(make_desc((1,) + tuple(x.shape[1:]), w.shape, x.dtype, stride, padding, m, 0, whole_kernel,
                                    stacked, direct=direct))
        osp = out[1:] if x.dim() == 4 else out
        return channel_first_view(torch.empty([0] + osp + [w.shape[0]], dtype=x.dtype, device=x.device))
    # channel-last memory is used as it is, and so is contiguous channel-first memory (x_layout = 1)
    nd = x.dim() - 2
    v = x.permute((0,) + tuple(range(2, 2 + nd)) + (1,))
    x_layout = 0
    if v.is_contiguous():
        x_mem = v
    else:
        x_mem = x if x.is_contiguous() else x.contiguous()
        x_layout = 1
    y_layout = int(bool(channels_first_out))
    # the one-kernel path of thin layers needs 16-byte aligned operands; a legal view can start anywhere
    # (x[1:] of a channel-last tensor with 6 channels and 7 x 7 images is 4-byte aligned): three kernels then
    unfused = bool(unfused) or misaligned(x_mem, U)
    desc, y_shape, nbytes, u_elems = _forward_setup(tuple(x.shape), tuple(w.shape), x.dtype, stride, padding, m,
                                                    chunk_images, whole_kernel, stacked, unfused, x_layout, y_layout, direct)
    ws = torch.empty(nbytes, dtype=torch.uint8, device=x.device)
    if y_layout:
        y = torch.empty([y_shape[0], y_shape[-1]] + y_shape[1:-1], dtype=x.dtype, device=x.device)
    else:
        y = torch.empty(y_shape, dtype=x.dtype, device=x.device)
    if bias is not None:
        bias = bias.contiguous()
    if U is not None and (not U.is_contiguous() or U.numel() != u_elems):
        check_u(desc, U)                                  # raises with the sizes in the message
    if times is None:
        check(lib.wc_conv_forward(ctypes.byref(desc), _ptr(x_mem), _ptr(w), _w_strides(w), _ptr(U),
                                  _ptr(bias), _ptr(y), _ptr(ws), nbytes, _stream(x)))
    else:
        check(lib.wc_conv_forward_timed(ctypes.byref(desc), _ptr(x_mem), _ptr(w), _w_strides(w), _ptr(U),
                                        _ptr(bias), _ptr(y), _ptr(ws), nbytes, _stream(x), times))
    return y if y_layout else channel_first_view(y)


_SETUPS = {}


def _forward_setup(x_shape, w_shape, dtype, stride, padding, m, chunk_images, whole_kernel, stacked, unfused=False,
                   x_layout=0, y_layout=0, direct=None):
    """Descriptor, output shape (channel-last), workspace bytes and size of U for one problem.  Kept
    per problem: for small layers (a few tens of microseconds on the GPU) rebuilding them on every
    call costs as much host time as the launches themselves."""
    key = (x_shape, w_shape, dtype, stride if isinstance(stride, int) else tuple(stride),
           padding if isinstance(padding, int) else tuple(padding), m, chunk_images, whole_kernel, stacked, unfused,
           x_layout, y_layout, direct)
    hit = _SETUPS.get(key)
    if hit is None:
        lib = _lib.load()
        desc = make_desc(x_shape, w_shape, dtype, stride, padding, m, chunk_images, whole_kernel, stacked, unfused,
                         x_layout, y_layout, direct)
        out, _ = out_dims(desc)
        nbytes, ue = ctypes.c_size_t(), ctypes.c_size_t()
        check(lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
        check(lib.wc_conv_u_elems(ctypes.byref(desc), ctypes.byref(ue)))
        osp = out[1:] if desc.ndim == 2 else out
        if len(_SETUPS) >= 4096:
            _SETUPS.clear()
        hit = _SETUPS[key] = (desc, [desc.N] + osp + [desc.K], nbytes.value, ue.value)
    return hit


# ---------------------------------------------------------------- gradients
def conv_backward_weight(x, dy, w_shape, stride=1, padding=0, m=2, whole_kernel=False, stacked=None):
    """Gradient of sum(y * dy) with respect to the filter of conv_forward(x, w, ...): a tensor of
    shape `w_shape` (K, C, [kD,] kH, kW) in x's dtype.  The reference has no backward pass; this one
    works in the transform domain (see include/winoconv.h).  `stacked` as in conv_forward."""
    _require_gpu(x, dy)
    stacked = _stack(stacked, x.dtype, x.dim() - 2, whole_kernel, w_shape, stride, m)
    if stacked == 2:
        stacked = True               # the weight gradient has no shared-input form: pieces stacked with their own V
    if dy.dtype != x.dtype:
        raise TypeError("x and dy must share one dtype")
    lib = _lib.load()
    desc = make_desc(x.shape, w_shape, x.dtype, stride, padding, m, 0, whole_kernel, stacked)
    out, _ = out_dims(desc)
    osp = out[1:] if desc.ndim == 2 else out
    if tuple(dy.shape) != (x.shape[0], w_shape[0]) + tuple(osp):
        raise ValueError("dy has shape %r, the convolution gives %r"
                         % (tuple(dy.shape), (x.shape[0], w_shape[0]) + tuple(osp)))
    dw = torch.empty(tuple(w_shape), dtype=x.dtype, device=x.device)
    if x.shape[0] == 0:
        return dw.zero_()
    x_cl, dy_cl = channel_last(x), channel_last(dy)
    nbytes = ctypes.c_size_t()
    check(lib.wc_conv_backward_weight_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)))
    ws = torch.empty(nbytes.value, dtype=torch.uint8, device=x.device)
    check(lib.wc_conv_backward_weight(ctypes.byref(desc), _ptr(x_cl), _ptr(dy_cl), _ptr(dw), _w_strides(dw),
                                      _ptr(ws), nbytes.value, _stream(x)))
    return dw


def conv_backward_input(dy, w, x_spatial, stride=1, padding=0, m=2):
    """Gradient of sum(y * dy) with respect to the input: the convolution of dy (with zeros between
    its elements when stride is 2) with the filter flipped along every spatial axis and its two
    channel axes exchanged, padded by k - 1 - p - so it runs through conv_forward."""
    _require_gpu(dy, w)
    nd = w.dim() - 2
    ks = tuple(w.shape[2:])
    pads = _triple(padding, nd, 0)[3 - nd:]
    if isinstance(stride, (tuple, list)):
        stride = int(stride[0])
    if any(k - 1 - p < 0 for k, p in zip(ks, pads)):
        raise NotImplementedError("input gradient needs padding <= kernel - 1 on every axis")
    want = tuple(int(v) for v in x_spatial)
    if stride == 2 and nd == 2 and dy.shape[0] > 0:
        # the library's own input gradient of strided layers: one direct-form launch per parity class of the pixels of
        # dx (wc_conv_backward_input); where it does not apply, the zero-filled dy below
        lib = _lib.load()
        x_shape = (dy.shape[0], w.shape[1]) + want
        desc = make_desc(x_shape, w.shape, dy.dtype, 2, padding, 2, 0, False, False, direct=False)
        out, _ = out_dims(desc)
        if tuple(dy.shape[2:]) != tuple(out[1:]):
            raise ValueError("dy of shape %r does not belong to an input of extent %r" % (tuple(dy.shape), want))
        nbytes = ctypes.c_size_t()
        if lib.wc_conv_backward_input_workspace_bytes(ctypes.byref(desc), ctypes.byref(nbytes)) == 0:
            if w.dtype != dy.dtype:
                raise TypeError("dy and the filter must share one dtype")
            dy_cl = channel_last(dy)
            dx = torch.empty((x_shape[0],) + want + (x_shape[1],), dtype=dy.dtype, device=dy.device)
            ws = torch.empty(nbytes.value, dtype=torch.uint8, device=dy.device)
            check(lib.wc_conv_backward_input(ctypes.byref(desc), _ptr(dy_cl), _ptr(w), _w_strides(w), _ptr(dx), _ptr(ws),
                                             nbytes.value, _stream(dy)))
            return channel_first_view(dx)
    if stride == 2:
        # zeros between the elements of dy, and at the end as many as it takes for the result to have
        # the input's extent (one more when the strided forward pass left an odd remainder)
        up = [X - (k - 1 - 2 * p) for X, k, p in zip(want, ks, pads)]
        if any(u < 2 * (o - 1) + 1 for u, o in zip(up, dy.shape[2:])):
            raise ValueError("dy of shape %r does not belong to an input of extent %r" % (tuple(dy.shape), want))
        dyu = torch.zeros(tuple(dy.shape[:2]) + tuple(up), dtype=dy.dtype, device=dy.device)
        dyu[(slice(None), slice(None)) + tuple(slice(0, 2 * (o - 1) + 1, 2) for o in dy.shape[2:])] = dy
        dy = dyu
    elif stride != 1:
        raise NotImplementedError("stride must be 1 or 2")
    w_rot = w.flip(tuple(range(2, 2 + nd))).transpose(0, 1)
    # output tile: the caller's, except where the 3-D tile 4 does not exist, for stride 2, where
    # three quarters of the zero-filled dy are zeros and the F(4,r) rounding error is not averaged
    # down (fp16: 2.6e-2 of the gradient's range against 2e-3 with tile 2), and for fewer than 8
    # output channels, where the sum is too short to average it down either (fp16, K = 1: up to
    # 3e-2 with tile 4, 1e-3 with tile 2)
    mm = m if (stride == 1 and w.shape[0] >= 8 and (m == 2 or nd == 2 or ks == (3, 3, 3))) else 2
    dx = conv_forward(dy, w_rot, None, 1, tuple(k - 1 - p for k, p in zip(ks, pads)), mm)
    if tuple(dx.shape[2:]) != want:
        raise ValueError("dy of shape %r does not belong to an input of extent %r" % (tuple(dy.shape), want))
    return dx
