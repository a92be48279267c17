// Last step of the weight gradient: dg = (G^T x G^T x G^T) dU per piece, accumulated over image
// chunks into acc (taps, K, C) in fp32.  dU (T, S, K, ldc) holds, in part 0 of every transform
// element, the sum over the tiles.  No counterpart in the reference (its backward pass was never
// written: src/back/utils.cu:15-24); the adjoint of the filter transform of filter_transform.hip.
#include "wc_transform.h"

namespace wc {

namespace {

__device__ __forceinline__ int dev_kind_of(int m, int r) {
  return m == 1 ? KIND_11 : (m == 4 ? (r == 3 ? KIND_43 : r == 2 ? KIND_42 : KIND_41)
                                   : (r <= 3 ? KIND_21 + (r - 1) : KIND_24 + (r - 4)));
}

struct GradFilterArgs {
  const float* dU;           // (T, S, K, ldc), the parts already summed into part 0
  float* acc;                // (taps, K, C) running sum over image chunks
  int K, C, ldc, S;
  int kernel[3];
  int step;
  int m[3];
  int n_pieces;
  int stacked;               // pieces side by side along the rows of dU, all with the tile of rp taps
  int Cp;                    // columns of dU per piece of a stacked plan
  int rp[3];
  int first;                 // 1: overwrite acc, 0: add to it
  long long total;           // taps * K * C
  wc_piece piece[WC_MAX_PIECES];
};

// acc[tap][k][c] (+)= sum_i G[i0][j0] G[i1][j1] G[i2][j2] sum_s dU[t_off + e(i)][s][k][c] for the piece owning the tap
__global__ __launch_bounds__(256) void grad_filter_transform_kernel(const GradFilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int c = (int)(idx % a.C);
  long long q = idx / a.C;
  const int k = (int)(q % a.K);
  const int tap = (int)(q / a.K);
  const int x2 = tap % a.kernel[2], x1 = (tap / a.kernel[2]) % a.kernel[1], x0 = tap / (a.kernel[2] * a.kernel[1]);
  // the piece that owns this tap and the tap's index inside it
  int s = -1, j0 = 0, j1 = 0, j2 = 0;
  for (int i = 0; i < a.n_pieces && s < 0; ++i) {
    const wc_piece& pc = a.piece[i];
    const int d0 = x0 - pc.tap0[0], d1 = x1 - pc.tap0[1], d2 = x2 - pc.tap0[2];
    if (d0 < 0 || d1 < 0 || d2 < 0 || d0 % a.step || d1 % a.step || d2 % a.step) continue;
    j0 = d0 / a.step; j1 = d1 / a.step; j2 = d2 / a.step;
    if (j0 < pc.r[0] && j1 < pc.r[1] && j2 < pc.r[2]) s = i;
  }
  float val = 0.f;
  if (s >= 0) {
    const wc_piece& pc = a.piece[s];
    const int n0 = a.m[0] + pc.r[0] - 1, n1 = a.m[1] + pc.r[1] - 1, n2 = a.m[2] + pc.r[2] - 1;
    const int k0 = dev_kind_of(a.m[0], pc.r[0]), k1 = dev_kind_of(a.m[1], pc.r[1]), k2 = dev_kind_of(a.m[2], pc.r[2]);
    for (int i0 = 0; i0 < n0; ++i0) {
      const float g0 = table_g(k0, i0, j0);
      if (g0 == 0.f) continue;
      for (int i1 = 0; i1 < n1; ++i1) {
        const float g01 = g0 * table_g(k1, i1, j1);
        if (g01 == 0.f) continue;
        for (int i2 = 0; i2 < n2; ++i2) {
          const float g = g01 * table_g(k2, i2, j2);
          if (g == 0.f) continue;
          const long long t = pc.t_offset + (i0 * n1 + i1) * n2 + i2;
          val = __builtin_fmaf(g, a.dU[(t * a.S * a.K + k) * a.ldc + c], val);   // part 0 holds the sum
        }
      }
    }
  }
  a.acc[idx] = a.first ? val : a.acc[idx] + val;
}

// G^T (r x alpha) as an apply_axis matrix
template <int KIND>
struct MatGT {
  static constexpr int rows = Mats<KIND>::r;
  static constexpr int cols = Mats<KIND>::alpha;
  __host__ __device__ static constexpr float get(int i, int j) { return Mats<KIND>::g(j, i); }
  __host__ __device__ static constexpr int first_nz(int i) {
    for (int j = 0; j < cols; ++j)
      if (get(i, j) != 0.f) return j;
    return cols;
  }
};

// One (k, c) of one piece with compile-time kinds: loads the piece's alpha^d sums once (lanes
// along c: coalesced), applies G^T along each axis in registers and adds the result to the
// piece's taps.
template <int K0, int K1, int K2>
__device__ __forceinline__ void grad_taps(const float* __restrict__ src, long long t_stride, float* __restrict__ acc,
                                          long long plane, const int (&tap0)[3], int step, int kH, int kW, bool first,
                                          const int (&taps)[3]) {
  constexpr int R0 = Mats<K0>::r, R1 = Mats<K1>::r, R2 = Mats<K2>::r;
  constexpr int A0 = Mats<K0>::alpha, A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
  float u[A0 * A1 * A2][1];
  static_for<0, A0 * A1 * A2>([&](auto e_) {
    constexpr int e = decltype(e_)::value;
    u[e][0] = src[e * t_stride];
  });
  float g2[A0 * A1 * R2][1];
  apply_axis<MatGT<K2>, 2, A0, A1, A2, 1>(u, g2);
  float g1[A0 * R1 * R2][1];
  apply_axis<MatGT<K1>, 1, A0, A1, R2, 1>(g2, g1);
  float g0[R0 * R1 * R2][1];
  apply_axis<MatGT<K0>, 0, A0, R1, R2, 1>(g1, g0);
  static_for<0, R0>([&](auto j0_) {
    static_for<0, R1>([&](auto j1_) {
      static_for<0, R2>([&](auto j2_) {
        constexpr int j0 = decltype(j0_)::value, j1 = decltype(j1_)::value, j2 = decltype(j2_)::value;
        // (a stacked plan transforms with the tile of the longest piece: taps this piece lacks are dropped)
        if (j0 < taps[0] && j1 < taps[1] && j2 < taps[2]) {
          const int tap = ((tap0[0] + j0 * step) * kH + tap0[1] + j1 * step) * kW + tap0[2] + j2 * step;
          float* dst = acc + tap * plane;
          const float v = g0[(j0 * R1 + j1) * R2 + j2][0];
          *dst = first ? v : *dst + v;
        }
      });
    });
  });
}

// The same transform for plans whose pieces have 1..3 taps per axis (every DWM plan): blockIdx.y is
// the piece, one thread per (k, c); the piece's taps select a compile-time body (uniform over the
// workgroup).  M0 x MO x MO is the output tile: 1 x 2 x 2, 1 x 4 x 4, 2 x 2 x 2 or 2 x 4 x 4.
template <int M0, int MO>
__global__ __launch_bounds__(256) void grad_filter_pieces_kernel(const GradFilterArgs a) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.K * a.C) return;
  const wc_piece& pc = a.piece[blockIdx.y];
  const int c = idx % a.C, k = idx / a.C;
  const long long t_stride = (long long)a.S * a.K * a.ldc;
  const float* src = a.dU + pc.t_offset * t_stride + (long long)k * a.ldc + (a.stacked ? (int)blockIdx.y * a.Cp : 0) + c;
  const int r0 = a.stacked ? a.rp[0] : pc.r[0], r1 = a.stacked ? a.rp[1] : pc.r[1], r2 = a.stacked ? a.rp[2] : pc.r[2];
  float* acc = a.acc + idx;
  const long long plane = (long long)a.K * a.C;
  const bool first = a.first != 0;
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;
#define WC_BODY(K0, K1, K2) grad_taps<K0, K1, K2>(src, t_stride, acc, plane, pc.tap0, a.step, a.kernel[1], a.kernel[2], first, pc.r)
#define WC_ROW(K0, K1) \
  switch (r2) { case 1: WC_BODY(K0, K1, KA); break; case 2: WC_BODY(K0, K1, KB); break; default: WC_BODY(K0, K1, KC); }
#define WC_PLANE(K0) \
  switch (r1) { case 1: WC_ROW(K0, KA) break; case 2: WC_ROW(K0, KB) break; default: WC_ROW(K0, KC) }
  if constexpr (M0 == 1) {
    WC_PLANE(KIND_11)
  } else {
    switch (r0) { case 1: WC_PLANE(KIND_21) break; case 2: WC_PLANE(KIND_22) break; default: WC_PLANE(KIND_23) }
  }
#undef WC_PLANE
#undef WC_ROW
#undef WC_BODY
}

}  // namespace

int grad_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const float* dU, float* acc, int ldc, int S,
                          bool first, void* stream) {
  hipStream_t s = as_stream(stream);
  GradFilterArgs g;
  g.dU = dU; g.acc = acc;
  g.K = d->K; g.C = d->C; g.ldc = ldc; g.S = S;
  for (int i = 0; i < 3; ++i) { g.kernel[i] = d->kernel[i]; g.m[i] = plan->m[i]; }
  g.step = plan->tap_step;
  g.n_pieces = plan->n_pieces;
  for (int i = 0; i < plan->n_pieces; ++i) g.piece[i] = plan->piece[i];
  g.first = first;
  g.stacked = d->stacked && plan->n_pieces > 1;
  g.Cp = wc_padded_channels(d->C);
  stacked_taps(plan, g.rp);
  g.total = (long long)d->kernel[0] * d->kernel[1] * d->kernel[2] * d->K * d->C;
  const int m0 = plan->m[0], mo = plan->m[1];
  bool small_taps = true;
  for (int i = 0; i < plan->n_pieces; ++i)
    for (int q = 0; q < 3; ++q) small_taps = small_taps && plan->piece[i].r[q] <= 3;
  if (small_taps && plan->m[2] == mo && (mo == 2 || mo == 4) && (m0 == 1 || m0 == 2) &&
      (long long)d->K * d->C < (1ll << 31)) {
    void (*fn)(GradFilterArgs) = m0 == 1 ? (mo == 4 ? &grad_filter_pieces_kernel<1, 4> : &grad_filter_pieces_kernel<1, 2>)
                                         : (mo == 4 ? &grad_filter_pieces_kernel<2, 4> : &grad_filter_pieces_kernel<2, 2>);
    const dim3 grid((unsigned)ceil_div_ll((long long)d->K * d->C, 256), (unsigned)plan->n_pieces);
    hipLaunchKernelGGL(fn, grid, dim3(256), 0, s, g);
  } else {
    if (g.stacked) return fail(WC_ERR_UNSUPPORTED, "stacked weight gradient needs a 2-D plan with output tile 2 or 4");
    hipLaunchKernelGGL(grad_filter_transform_kernel, dim3((unsigned)ceil_div_ll(g.total, 256)), dim3(256), 0, s, g);
  }
  WC_CHECK_LAUNCH("grad_filter_transform_kernel");
  return WC_OK;
}

}  // namespace wc
