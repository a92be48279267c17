// Direct form of a 2-D convolution (wc_conv_desc.direct): the degenerate end of the DWM split, pieces
// of ONE tap on the trivial tile F(1,1).  With one tap per piece there is nothing to transform - B^T, G and A^T
// are 1 - so the batched product reads the pixels of x itself as its V operand, walks the taps along its reduction
// axis (gemm_kernel<..., DIRECT> in gemm.hip) and writes y.  x is read once from HBM (the taps of neighbouring outputs
// meet in the caches), y written once, nothing else moves.
//
// Where it is used: 1x1 kernels of every type (a Winograd tile of one tap saves nothing, and its transforms are copies:
// three passes over memory instead of one), and 16-bit layers at stride 2.  The reference leaves stride 2 unimplemented (src/winograd_conv.cpp:122-126); the plans
// built here for it run Winograd tiles on the parity phases of x, which saves no multiplications for small kernels
// (F(2,2) on the phases of a 3x3 kernel needs the 9 products per output of the direct form) and moves V and M
// through HBM.  Stride-1 layers keep their Winograd plans, which need 2.25x to 4x fewer products.
//
// The filter goes to U (K, kh, kw, C) - taps outermost along the reduction, channels innermost - with a small copy
// kernel (the "filter transform" of this form; a caller may cache U like any other).
#include "wc_common.h"

namespace wc {

struct DirectFilterArgs {
  const void* w;
  void* U;
  long long s[5];     // element strides of w for (K, C, kD, kH, kW)
  int K, C, kh, kw;
  long long total;
};

template <typename T>
__global__ __launch_bounds__(256) void direct_filter_kernel(DirectFilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int c = (int)(idx % a.C);
  long long q = idx / a.C;
  const int kx = (int)(q % a.kw); q /= a.kw;
  const int ky = (int)(q % a.kh);
  const long long k = q / a.kh;
  static_cast<T*>(a.U)[idx] = static_cast<const T*>(a.w)[k * a.s[0] + c * a.s[1] + ky * a.s[3] + kx * a.s[4]];
}

bool direct_conv_fits(const wc_conv_desc* d) {
  if (d->ndim != 2) return false;
  if (d->C % (d->dtype == WC_F32 ? 16 : 32) != 0 || d->K % 8 != 0) return false;   // whole reduction blocks along C, 16-byte stores along K
  if (d->whole_kernel) return false;
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  if (wc_conv_out_dims(&e, out, grid) != WC_OK) return false;
  const long long P = (long long)d->N * out[1] * out[2];
  return P < (1ll << 31) && (long long)d->N * d->in[1] * d->in[2] < (1ll << 31);
}

int direct_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(w && w_strides && U, "direct filter copy: null pointer");
  DirectFilterArgs a;
  a.w = w; a.U = U;
  for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
  a.K = d->K; a.C = d->C; a.kh = d->kernel[1]; a.kw = d->kernel[2];
  a.total = (long long)d->K * d->kernel[1] * d->kernel[2] * d->C;
  const unsigned blocks = (unsigned)ceil_div_ll(a.total, 256);
  if (d->dtype == WC_F32) hipLaunchKernelGGL(direct_filter_kernel<float>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  else if (d->dtype == WC_F16) hipLaunchKernelGGL(direct_filter_kernel<half_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  else hipLaunchKernelGGL(direct_filter_kernel<bf16_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("direct_filter_kernel");
  return WC_OK;
}

int direct_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y, void* stream) {
  WC_CHECK_ARG(direct_conv_fits(d), "direct convolution: 2-D, input channels a multiple of 32 (fp32: 16), output "
               "channels a multiple of 8");
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  int rc = wc_conv_out_dims(&e, out, grid);
  if (rc) return rc;
  return gemm_direct_conv(x, U, bias, y, n_images, d->in[1], d->in[2], d->C, d->K, d->kernel[1], d->kernel[2], d->stride,
                          d->pad[1], d->pad[2], out[1], out[2], d->dtype, stream);
}

}  // namespace wc
