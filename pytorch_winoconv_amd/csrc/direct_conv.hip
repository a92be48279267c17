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

typedef uint32_t Chunk16z __attribute__((ext_vector_type(4)));   // one 16-byte store

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
  if (direct_first3d_fits(d)) return true;        // 3-D first layers: the only 3-D problems with a direct form (direct_first3d.hip)
  if (d->ndim != 2) return false;
  if (direct_first_fits(d)) return true;          // strided first layers: their own kernel and filter layout (direct_first.hip)
  if (d->C % (d->dtype == WC_F32 ? 16 : 32) != 0 || d->K % 8 != 0) return false;   // whole reduction blocks along C, 16-byte stores along K
  if (d->whole_kernel) return false;
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  if (wc_conv_out_dims(&e, out, grid) != WC_OK) return false;
  const long long P = (long long)d->N * out[1] * out[2];
  return P < (1ll << 31) && (long long)d->N * d->in[1] * d->in[2] < (1ll << 31);
}

size_t direct_u_elems(const wc_conv_desc* d) {
  if (direct_first3d_fits(d)) return direct_first3d_u_elems(d);
  return direct_first_fits(d) ? direct_first_u_elems(d) : (size_t)d->K * d->kernel[1] * d->kernel[2] * d->C;
}

int direct_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(w && w_strides && U, "direct filter copy: null pointer");
  if (direct_first3d_fits(d)) return direct_first3d_filter(d, w, w_strides, U, stream);
  if (direct_first_fits(d)) return direct_first_filter(d, w, w_strides, U, stream);
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
               "channels a multiple of 8 (or a first layer with at most 4 channels in a 16-bit type: 2-D at stride 2, 3-D 3x3x3 at stride 1)");
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  int rc = wc_conv_out_dims(&e, out, grid);
  if (rc) return rc;
  if (direct_first3d_fits(d)) return direct_first3d_conv(d, x, n_images, U, bias, y, out, stream);
  if (direct_first_fits(d)) return direct_first_conv(d, x, n_images, U, bias, y, out[1], out[2], stream);
  return gemm_direct_conv(x, U, bias, y, n_images, d->in[1], d->in[2], d->C, d->K, d->kernel[1], d->kernel[2], d->stride,
                          d->pad[1], d->pad[2], out[1], out[2], d->dtype, stream);
}

// ---- input gradient of a strided layer -------------------------------------------------------------------------
// dx[b, iy, ix, c] = sum over the taps (ky, kx) with iy + ph - ky and ix + pw - kx even, and over k, of
// dy[b, (iy + ph - ky) / 2, (ix + pw - kx) / 2, k] w[k, c, ky, kx].  The pixels of dx fall into four classes by the
// parity (py, px) of (iy + ph, ix + pw); a class only meets the taps of its own parity, ky = py + 2a, and with
// iy + ph = 2 qy + py it is a stride-1 direct convolution of dy with that sub-kernel, flipped, its channel axes
// exchanged: dx_class[qy, qx] = sum_a' sum_b' dy[qy - (A - 1) + a', qx - (B - 1) + b'] g[a', b'],
// g[a', b'] = w[., ., py + 2 (A - 1 - a'), px + 2 (B - 1 - b')].  One launch of the direct form per class, each writing
// every second pixel of dx: the multiplications of the forward pass and one pass over dy per class, where convolving a
// zero-filled dy at stride 1 multiplies four times as much.
struct SubFilterArgs {
  const void* w;
  void* U;            // (C, A, B, K): rows = input channels of the layer, reduction = its output channels
  long long s[5];
  int K, C, A, B, py, px;
  long long total;
};

template <typename T>
__global__ __launch_bounds__(256) void sub_filter_kernel(SubFilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.K);
  long long q = idx / a.K;
  const int b = (int)(q % a.B); q /= a.B;
  const int aa = (int)(q % a.A);
  const long long c = q / a.A;
  const int ky = a.py + 2 * (a.A - 1 - aa), kx = a.px + 2 * (a.B - 1 - b);
  static_cast<T*>(a.U)[idx] = static_cast<const T*>(a.w)[k * a.s[0] + c * a.s[1] + ky * a.s[3] + kx * a.s[4]];
}

template <typename T>
__global__ __launch_bounds__(256) void zero_class_kernel(T* dx, int H, int W, int C, int y0, int x0, int Qh, int Qw, long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;      // one thread per 16 bytes
  if (idx >= total) return;
  constexpr int V = 16 / sizeof(T);
  const int cv = (int)(idx % (C / V));
  long long q = idx / (C / V);
  const int qx = (int)(q % Qw); q /= Qw;
  const int qy = (int)(q % Qh);
  const long long b = q / Qh;
  Chunk16z z = {0u, 0u, 0u, 0u};
  *reinterpret_cast<Chunk16z*>(dx + ((b * H + 2 * qy + y0) * W + 2 * qx + x0) * C + cv * V) = z;
}

bool strided_input_grad_fits(const wc_conv_desc* d) {
  if (d->ndim != 2 || d->stride != 2 || d->whole_kernel) return false;
  // roles exchanged: the reduction runs over the layer's output channels, the rows of the result are its input channels
  if (d->K % (d->dtype == WC_F32 ? 16 : 32) != 0 || d->C % 8 != 0) return false;
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  if (wc_conv_out_dims(&e, out, grid) != WC_OK) return false;
  for (int a = 1; a < 3; ++a)
    if (d->pad[a] > d->kernel[a] - 1) return false;
  return (long long)d->N * d->in[1] * d->in[2] < (1ll << 31) && (long long)d->N * out[1] * out[2] < (1ll << 31);
}

}  // namespace wc

using namespace wc;

extern "C" int wc_conv_backward_input_workspace_bytes(const wc_conv_desc* d, size_t* bytes) {
  WC_CHECK_ARG(d && bytes, "wc_conv_backward_input_workspace_bytes: null pointer");
  if (!strided_input_grad_fits(d))
    return fail(WC_ERR_UNSUPPORTED, "wc_conv_backward_input: 2-D layers at stride 2 with output channels a multiple of 32 "
                "(fp32: 16), input channels a multiple of 8 and padding below the kernel extent");
  *bytes = ((size_t)d->kernel[1] * d->kernel[2] * d->K * d->C * (d->dtype == WC_F32 ? 4 : 2) + 255) / 256 * 256 + 4 * 256;
  return WC_OK;
}

extern "C" int wc_conv_backward_input(const wc_conv_desc* d, const void* dy, const void* w, const int64_t w_strides[5],
                                      void* dx, void* workspace, size_t workspace_bytes, void* stream) {
  size_t need = 0;
  int rc = wc_conv_backward_input_workspace_bytes(d, &need);
  if (rc) return rc;
  WC_CHECK_ARG(dy && w && w_strides && dx, "wc_conv_backward_input: null pointer");
  if (!workspace || workspace_bytes < need)
    return fail(WC_ERR_WORKSPACE, "wc_conv_backward_input: workspace of %zu bytes, %zu needed", workspace ? workspace_bytes : (size_t)0, need);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return fail(WC_ERR_WORKSPACE, "wc_conv_backward_input: workspace must be 256-byte aligned");
  int out[3], grid[3];
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  rc = wc_conv_out_dims(&e, out, grid);
  if (rc) return rc;
  const int H = d->in[1], W = d->in[2], kh = d->kernel[1], kw = d->kernel[2], ph = d->pad[1], pw = d->pad[2];
  const size_t es = d->dtype == WC_F32 ? 4 : 2;
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  hipStream_t s = as_stream(stream);
  for (int py = 0; py < 2; ++py) {
    for (int px = 0; px < 2; ++px) {
      const int A = (kh - py + 1) / 2, B = (kw - px + 1) / 2;                 // taps of this parity (may be none)
      const int qy0 = ph > py ? (ph - py + 1) / 2 : 0, qx0 = pw > px ? (pw - px + 1) / 2 : 0;
      const int y0 = 2 * qy0 + py - ph, x0 = 2 * qx0 + px - pw;              // first pixel of the class: 0 or 1
      if (y0 >= H || x0 >= W) continue;
      const int Qh = (H - y0 + 1) / 2, Qw = (W - x0 + 1) / 2;
      if (A <= 0 || B <= 0) {
        // a kernel of one tap along an axis never reaches the pixels of the other parity: their gradient is zero
        const long long total = (long long)d->N * Qh * Qw * (d->C * es / 16);
        dispatch_dtype(d->dtype, [&](auto t) {
          using T = decltype(t);
          hipLaunchKernelGGL(zero_class_kernel<T>, dim3((unsigned)ceil_div_ll(total, 256)), dim3(256), 0, s,
                             static_cast<T*>(dx), H, W, d->C, y0, x0, Qh, Qw, total);
          return 0;
        });
        WC_CHECK_LAUNCH("zero_class_kernel");
        continue;
      }
      SubFilterArgs a;
      a.w = w; a.U = ws;
      for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
      a.K = d->K; a.C = d->C; a.A = A; a.B = B; a.py = py; a.px = px;
      a.total = (long long)d->C * A * B * d->K;
      dispatch_dtype(d->dtype, [&](auto t) {
        using T = decltype(t);
        hipLaunchKernelGGL(sub_filter_kernel<T>, dim3((unsigned)ceil_div_ll(a.total, 256)), dim3(256), 0, s, a);
        return 0;
      });
      WC_CHECK_LAUNCH("sub_filter_kernel");
      rc = gemm_direct_conv(dy, ws, nullptr, dx, d->N, out[1], out[2], d->K, d->C, A, B, 1, A - 1 - qy0, B - 1 - qx0, Qh, Qw,
                            d->dtype, stream, 2, y0, x0, H, W);
      if (rc) return rc;
      ws += (a.total * es + 255) / 256 * 256;
    }
  }
  return WC_OK;
}

namespace wc {
}  // namespace wc
