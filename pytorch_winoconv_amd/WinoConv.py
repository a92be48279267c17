"""The `Wino` function object of the reference (reference: WinoConv.py:8-229, whose code is
stale: it names `tf`, an undefined `A` and `fp16`) and the modules that give the patched
nn.Conv2d / nn.Conv3d of the reference (conv.py:324-339, 465-480) a working form.

Routing rule of the modules: groups == 1 and dilation == 1 are required for the Winograd
path; 3x3(x3) stride-1 kernels use plain Winograd, larger kernels and stride 2 the DWM
decomposition (output tile 4 in 2-D, 2 in 3-D); grouped, dilated, stride > 2 or kernel > 10
convolutions, which the Winograd algorithm here does not cover, go to
torch.nn.functional.conv2d/conv3d on the same device like the reference does (conv.py:326-332).
There is no CPU path: a CPU tensor, or a missing HIP library, raises.  The transformed filter
is cached and recomputed only when the weight changes.
"""
import torch
from torch import nn
import torch.nn.functional as F

from . import engine, matrix_conv, matrix_conv3d


class Wino:
    """conv32 / conv16 as methods (reference: WinoConv.py:43-109)."""

    def __init__(self):
        self.input = None
        self.kernel = None
        self.m = 0
        self.r = 0

    matrix_alloc = staticmethod(matrix_conv.matrix_alloc)

    def _mod(self, input):
        return matrix_conv if input.dim() == 4 else matrix_conv3d

    def conv16(self, input, kernel, bias=None, stride=1, padding=0, groups=1, output_block=2):
        return self._mod(input).conv16(input, kernel, bias, stride, padding, groups, output_block)

    def conv32(self, input, kernel, bias=None, stride=1, padding=0, groups=1, output_block=2):
        return self._mod(input).conv32(input, kernel, bias, stride, padding, groups, output_block)

    def conv(self, input, kernel, output_block, stride, fp16=False):
        return self._mod(input).conv(input, kernel, output_block, stride, fp16)


class WinoConvFunction(torch.autograd.Function):
    """conv_forward with gradients.  The reference has no backward pass (src/back/ holds only a
    pointer-assign helper, src/back/utils.cu:15-24); here the input gradient is a convolution run by
    the same engine and the weight gradient is computed in the transform domain."""

    @staticmethod
    def forward(ctx, x, w, bias, stride, padding, m, U):
        ctx.save_for_backward(x, w)
        ctx.conf = (stride, padding, m, bias is not None)
        return engine.conv_forward(x, w, bias, stride, padding, m, U=U)

    @staticmethod
    def backward(ctx, dy):
        x, w = ctx.saved_tensors
        stride, padding, m, has_bias = ctx.conf
        dx = dw = db = None
        if ctx.needs_input_grad[0]:
            dx = engine.conv_backward_input(dy, w, x.shape[2:], stride, padding, m)
        if ctx.needs_input_grad[1]:
            dw = engine.conv_backward_weight(x, dy, w.shape, stride, padding, m)
        if has_bias and ctx.needs_input_grad[2]:
            db = dy.sum(dim=[0] + list(range(2, dy.dim())))
        return dx, dw, db, None, None, None, None


class _WinoConvNd(nn.Module):
    nd = 2

    def __init__(self, in_channels, out_channels, kernel_size, stride=1, padding=0, dilation=1,
                 groups=1, bias=True, output_block=None, device=None, dtype=None):
        super().__init__()
        tup = lambda v: (v,) * self.nd if isinstance(v, int) else tuple(v)
        self.in_channels, self.out_channels = in_channels, out_channels
        self.kernel_size, self.stride = tup(kernel_size), tup(stride)
        self.padding, self.dilation, self.groups = tup(padding), tup(dilation), groups
        self.output_block = output_block
        self.weight = nn.Parameter(torch.empty((out_channels, in_channels // groups) + self.kernel_size,
                                               device=device, dtype=dtype))
        self.bias = nn.Parameter(torch.empty(out_channels, device=device, dtype=dtype)) if bias else None
        nn.init.kaiming_normal_(self.weight)
        if self.bias is not None:
            nn.init.zeros_(self.bias)
        self._cache = None

    def _winograd_ok(self, x):
        # The reference hands every strided or dilated layer (and every kernel up to 3 x 3) to the stock
        # convolution (conv.py:326-332, 467-473).  This engine keeps strided layers, with one exception: strided
        # first layers with at most 8 input channels, whose parity-phase plans pad the channels to 32 once per
        # phase (ResNet's 3 -> 64, 7 x 7, stride 2 at N = 32: 0.25 ms in fp16 and 1.0 ms in fp32 against 0.07 and
        # 0.12 ms for torch's own convolution); they go the reference's way.
        # ... except where the engine has a kernel for them: at most 4 channels in a 16-bit type, kernels of 3, 5 or 7
        # rows and at most 8 columns (the direct form's first-layer kernel: ResNet's layer in fp16).
        if self.stride[0] == 2 and self.in_channels <= 8:
            first = (self.nd == 2 and self.in_channels <= 4 and x.dtype in (torch.float16, torch.bfloat16)
                     and self.kernel_size[0] in (3, 5, 7) and self.kernel_size[1] <= 8 and self.out_channels % 8 == 0
                     and len(set(self.stride)) == 1 and self.groups == 1 and set(self.dilation) == {1})
            if not first:
                return False
        # ... and so do 3-D first layers with at most 4 input channels: F(2,3)^3 on 3 channels padded to 32 makes V eighty
        # times the input (N=2, 3 -> 64, 16x112x112: 0.27 ms in fp16 and 0.52 ms in fp32 against 0.12 and 0.11 ms) -
        # except 3x3x3 layers at stride 1 in a 16-bit type, for which the direct form has a kernel (N=8: 0.06 ms against
        # 0.41-0.57 ms)
        if self.nd == 3 and self.in_channels <= 4:
            first3d = (x.dtype in (torch.float16, torch.bfloat16) and tuple(self.kernel_size) == (3, 3, 3)
                       and set(self.stride) == {1} and self.out_channels % 8 == 0 and self.groups == 1
                       and set(self.dilation) == {1})
            if not first3d:
                return False
        return (self.groups == 1 and set(self.dilation) == {1} and len(set(self.stride)) == 1
                and self.stride[0] in (1, 2) and max(self.kernel_size) <= 10)

    def _tile(self):
        if self.output_block is not None:
            return int(self.output_block)
        return 4 if self.nd == 2 else 2

    def _tile_for(self, dtype):
        # F(4,r) tiles lose about 1e-1 of the output range in bfloat16 (8 mantissa bits): tile 2 there.
        # In float16 their rounding error averages down over the input channels (1e-2 of the range
        # at worst for 8 and more); with fewer it does not (3e-2 seen with one channel): tile 2 too.
        if self.output_block is None and (dtype == torch.bfloat16 or
                                          (dtype == torch.float16 and self.in_channels < 8)):
            return 2
        # thin 16-bit 3x3 layers run as one fused F(2,3) kernel; the cached U must be of that tile
        if self.output_block is None and engine.thin_preferred(dtype, self.nd, self.in_channels, self.out_channels,
                                                            self.kernel_size, self.stride):
            return 2
        return self._tile()

    def forward(self, x):
        conv = F.conv2d if self.nd == 2 else F.conv3d
        if not x.is_cuda:
            raise ValueError("WinoConv: the engine runs on the GPU only; got a CPU tensor")
        if x.dtype not in (torch.float16, torch.bfloat16, torch.float32):
            raise NotImplementedError(f"WinoConv: dtype {x.dtype} (float32, float16 and bfloat16 only)")
        if not self._winograd_ok(x):
            return conv(x, self.weight, self.bias, self.stride, self.padding, self.dilation, self.groups)
        w = self.weight.to(x.dtype)
        m = self._tile_for(x.dtype)
        # the form of the plan (Winograd pieces, or the direct form the library takes for large strided problems)
        # depends on the batch size too, and the transformed filter of one form does not fit the other
        form = engine.plan_form(x.shape, w.shape, x.dtype, self.stride[0], self.padding, m)
        key = (self.weight._version, self.weight.data_ptr(), tuple(x.shape[2:]), x.dtype, m, form)
        if self._cache is None or self._cache[0] != key:
            U = engine.transform_filter(w.detach(), x.shape, self.stride[0], self.padding, m)
            self._cache = (key, U)
        b = None if self.bias is None else self.bias.to(x.dtype)
        if torch.is_grad_enabled() and (x.requires_grad or w.requires_grad or (b is not None and b.requires_grad)):
            return WinoConvFunction.apply(x, w, b, self.stride[0], self.padding, m, self._cache[1])
        return engine.conv_forward(x, w.detach(), b, self.stride[0], self.padding, m, U=self._cache[1])


class WinoConv2d(_WinoConvNd):
    """nn.Conv2d whose forward runs the Winograd / DWM engine (reference: conv.py:324-339)."""
    nd = 2


class WinoConv3d(_WinoConvNd):
    """nn.Conv3d whose forward runs the Winograd / DWM engine (reference: conv.py:465-480)."""
    nd = 3
