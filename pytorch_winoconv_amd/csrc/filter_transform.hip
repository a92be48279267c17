// Filter transform U = (G_d x G_h x G_w) g for every piece of the plan, one launch.
//
// Replaces wNorm2WinoTransform + wNorm2WinoCalculation of the reference
// (src/split_kernel.cu:14-53, src/calculation_kernels.cu:2-761).  The filter is read through
// element strides, so both torch's (K, C, kD, kH, kW) and the reference's (kD, kH, kW, C, K)
// (dwm.py:85,133) are accepted without a copy.  Output U (T, K, Cp): element-major, the
// reduction axis C innermost and zero-padded to Cp so that the batched GEMM reads both of
// its operands along contiguous rows (the reference keeps (T, C, K): split_kernel.cu:51).
// Arithmetic in fp32, one rounding to the storage type.  Tiny (K*C*T outputs); run once per
// weight update by callers that cache U.
#include "wc_common.h"
#include "wc_tables.h"

namespace wc {

struct FilterArgs {
  const void* w;
  void* U;
  long long s[5];     // element strides of w for (K, C, kD, kH, kW)
  int C, Cp, K;
  int step;
  int m[3];
  int n_pieces;
  long long total;    // T * K * Cp
  wc_piece piece[WC_MAX_PIECES];
};

__device__ __forceinline__ int dev_kind(int m, int r) {
  return m == 1 ? KIND_11 : (m == 4 ? KIND_43 : KIND_21 + (r - 1));
}

template <typename T>
__global__ __launch_bounds__(256) void filter_transform_kernel(const FilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int c = (int)(idx % a.Cp);
  const long long q = idx / a.Cp;
  const int k = (int)(q % a.K);
  const int t = (int)(q / a.K);
  T* U = static_cast<T*>(a.U);
  if (c >= a.C) { U[idx] = static_cast<T>(0.f); return; }
  int s = 0;
  while (s + 1 < a.n_pieces && a.piece[s + 1].t_offset <= t) ++s;
  const wc_piece& pc = a.piece[s];
  const int e = t - pc.t_offset;
  const int a1n = a.m[1] + pc.r[1] - 1, a2n = a.m[2] + pc.r[2] - 1;
  const int i2 = e % a2n, i1 = (e / a2n) % a1n, i0 = e / (a2n * a1n);
  const int k0 = dev_kind(a.m[0], pc.r[0]), k1 = dev_kind(a.m[1], pc.r[1]), k2 = dev_kind(a.m[2], pc.r[2]);
  const T* w = static_cast<const T*>(a.w) + k * a.s[0] + c * a.s[1];
  float acc = 0.f;
  for (int j0 = 0; j0 < pc.r[0]; ++j0) {
    const float g0 = table_g(k0, i0, j0);
    for (int j1 = 0; j1 < pc.r[1]; ++j1) {
      const float g01 = g0 * table_g(k1, i1, j1);
      for (int j2 = 0; j2 < pc.r[2]; ++j2) {
        const float g = g01 * table_g(k2, i2, j2);
        const float v = static_cast<float>(w[(pc.tap0[0] + j0 * a.step) * a.s[2] +
                                            (pc.tap0[1] + j1 * a.step) * a.s[3] +
                                            (pc.tap0[2] + j2 * a.step) * a.s[4]]);
        acc = __builtin_fmaf(g, v, acc);
      }
    }
  }
  U[idx] = static_cast<T>(acc);
}

}  // namespace wc

using namespace wc;

extern "C" int wc_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const void* w,
                                   const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(d && plan && w && w_strides && U, "wc_filter_transform: null pointer");
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);   // validates the descriptor
  if (rc) return rc;
  WC_CHECK_ARG(plan->n_pieces > 0 && plan->n_pieces <= WC_MAX_PIECES, "wc_filter_transform: bad plan");
  FilterArgs a;
  a.w = w; a.U = U;
  for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
  a.C = d->C; a.Cp = wc_padded_channels(d->C); a.K = d->K;
  a.step = plan->tap_step;
  for (int i = 0; i < 3; ++i) a.m[i] = plan->m[i];
  a.n_pieces = plan->n_pieces;
  for (int i = 0; i < plan->n_pieces; ++i) a.piece[i] = plan->piece[i];
  a.total = (long long)plan->t_total * d->K * a.Cp;
  const long long blocks = ceil_div_ll(a.total, 256);
  WC_CHECK_ARG(blocks < (1ll << 31), "wc_filter_transform: problem too large");
  if (d->dtype == WC_F16)
    filter_transform_kernel<half_t><<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(a);
  else
    filter_transform_kernel<float><<<(unsigned)blocks, 256, 0, as_stream(stream)>>>(a);
  WC_CHECK_LAUNCH("filter_transform_kernel");
  return WC_OK;
}
