// Filter transform U = (G_d x G_h x G_w) g for every piece of the plan, one launch.
//
// Replaces wNorm2WinoTransform + wNorm2WinoCalculation of the reference
// (src/split_kernel.cu:14-53, src/calculation_kernels.cu:2-761).  The filter is read through
// element strides, so both torch's (K, C, kD, kH, kW) and the reference's (kD, kH, kW, C, K)
// (dwm.py:85,133) are accepted without a copy.  Output U (T, K, Cp): element-major, the
// reduction axis C innermost and zero-padded to Cp so that the batched GEMM reads both of
// its operands along contiguous rows (the reference keeps (T, C, K): split_kernel.cu:51).
// Arithmetic in fp32, one rounding to the storage type.  Tiny (K*C*T outputs); run once per
// weight update by callers that cache U.  Single-piece plans of the common shapes take a
// compile-time kernel (taps loaded once per (k, c)), DWM plans one launch whose workgroups pick the
// compile-time body of their piece; anything else (whole-kernel tiles) the generic kernel.
#include "filter_transform_impl.h"

namespace wc {

// Single piece with compile-time kinds: one thread per (k, VEC channels).
template <typename T, int K0, int K1, int K2, bool DENSE>
__global__ __launch_bounds__(256) void filter_transform_fast_kernel(const FilterFastArgs a) {
  filter_fast_body<T, K0, K1, K2, DENSE>(a, blockIdx.x * 256 + threadIdx.x);
}

using FilterFastKernel = void (*)(FilterFastArgs);

template <typename T, bool DENSE>
static FilterFastKernel pick_fast(int k0, int k1, int k2) {
  if (k0 == KIND_11 && k1 == KIND_43 && k2 == KIND_43) return &filter_transform_fast_kernel<T, KIND_11, KIND_43, KIND_43, DENSE>;
  if (k0 == KIND_11 && k1 == KIND_23 && k2 == KIND_23) return &filter_transform_fast_kernel<T, KIND_11, KIND_23, KIND_23, DENSE>;
  if (k0 == KIND_23 && k1 == KIND_23 && k2 == KIND_23) return &filter_transform_fast_kernel<T, KIND_23, KIND_23, KIND_23, DENSE>;
  if (k0 == KIND_23 && k1 == KIND_43 && k2 == KIND_43) return &filter_transform_fast_kernel<T, KIND_23, KIND_43, KIND_43, DENSE>;
  return nullptr;
}

// channels per thread of the kernel pick_fast returns (0: none)
static int fast_vec_of(int dtype, int k0, int k1, int k2) {
  const int es = dtype == WC_F32 ? 4 : 2;
  if (k0 == KIND_11) return 8 / es;
  if (k0 == KIND_23 && k1 == KIND_23) return 2;
  return 1;
}

struct FilterArgs {
  const void* w;
  void* U;
  long long s[5];     // element strides of w for (K, C, kD, kH, kW)
  int C, Cp, K;
  int step;
  int m[3];
  int n_pieces;
  long long total;    // T * K * Cp
  int stacked;        // pieces side by side along the rows of U, all with the tile of rp taps
  int rp[3];
  wc_piece piece[WC_MAX_PIECES];
};

__device__ __forceinline__ int dev_kind(int m, int r) {
  return m == 1 ? KIND_11 : (m == 4 ? (r == 3 ? KIND_43 : r == 2 ? KIND_42 : KIND_41)
                                   : (r <= 3 ? KIND_21 + (r - 1) : KIND_24 + (r - 4)));
}

// Any plan whose pieces have 1..3 taps per axis (every DWM plan): blockIdx.y is the piece, one
// thread per (k, c); the piece's taps-per-axis select one of the compile-time bodies (a branch
// that is uniform over the workgroup).  FLAT: one-element depth axis; MO: output tile 2 or 4.
template <typename T, bool FLAT, int MO>
__global__ __launch_bounds__(256) void filter_transform_pieces_kernel(const FilterArgs a) {
  const int idx = blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.K * a.Cp) return;
  const wc_piece& pc = a.piece[blockIdx.y];
  const int c = idx % a.Cp, k = idx / a.Cp;
  const int row = a.stacked ? a.Cp * a.n_pieces : a.Cp;          // row length of U
  const long long plane = (long long)a.K * row;
  T* U = static_cast<T*>(a.U) + (long long)pc.t_offset * plane + (long long)k * row +
         (a.stacked ? (int)blockIdx.y * a.Cp : 0) + c;
  const T* w = static_cast<const T*>(a.w);
  const int r0 = a.stacked ? a.rp[0] : pc.r[0], r1 = a.stacked ? a.rp[1] : pc.r[1], r2 = a.stacked ? a.rp[2] : pc.r[2];
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;
#define WC_BODY(K0, K1, K2) transform_taps<T, K0, K1, K2>(w, a.s, k, c, a.C, pc.tap0, a.step, U, plane, pc.r)
#define WC_ROW(K0, K1) \
  switch (r2) { case 1: WC_BODY(K0, K1, KA); break; case 2: WC_BODY(K0, K1, KB); break; default: WC_BODY(K0, K1, KC); }
#define WC_PLANE(K0) \
  switch (r1) { case 1: WC_ROW(K0, KA) break; case 2: WC_ROW(K0, KB) break; default: WC_ROW(K0, KC) }
  if constexpr (MO == 3) {
    WC_BODY(KIND_11, KIND_33, KIND_33);       // three-tap pieces on the shared tile F(3,3), 2-D only
  } else if constexpr (FLAT) {
    WC_PLANE(KIND_11)
  } else {
    switch (r0) { case 1: WC_PLANE(KIND_21) break; case 2: WC_PLANE(KIND_22) break; default: WC_PLANE(KIND_23) }
  }
#undef WC_PLANE
#undef WC_ROW
#undef WC_BODY
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

bool filter_fast_setup(const wc_conv_desc* d, const wc_plan* plan, const void* w, const int64_t w_strides[5], void* U,
                       FilterFastArgs* f, int* vec, bool* dense) {
  if (plan->n_pieces != 1) return false;
  const wc_piece& pc = plan->piece[0];
  const int k0 = kind_of(plan->m[0], pc.r[0]), k1 = kind_of(plan->m[1], pc.r[1]), k2 = kind_of(plan->m[2], pc.r[2]);
  if (!pick_fast<float, false>(k0, k1, k2)) return false;
  *vec = fast_vec_of(d->dtype, k0, k1, k2);
  // a contiguous (K, C, taps) filter whose channels split evenly among the threads is read in 8-byte pieces
  const long long taps = (long long)pc.r[0] * pc.r[1] * pc.r[2];
  *dense = w_strides[4] == 1 && w_strides[3] == pc.r[2] &&
           (pc.r[0] == 1 || w_strides[2] == (long long)pc.r[1] * pc.r[2]) && w_strides[1] == taps &&
           w_strides[0] == taps * d->C && plan->tap_step == 1 && pc.tap0[0] == 0 && pc.tap0[1] == 0 &&
           pc.tap0[2] == 0 && *vec > 1 && d->C % *vec == 0 && (reinterpret_cast<uintptr_t>(w) & 7) == 0;
  f->w = w; f->U = U;
  for (int i = 0; i < 5; ++i) f->s[i] = w_strides[i];
  f->C = d->C; f->Cp = wc_padded_channels(d->C); f->K = d->K;
  for (int i = 0; i < 3; ++i) f->tap0[i] = pc.tap0[i];
  f->step = plan->tap_step;
  f->t_offset = pc.t_offset;
  return true;
}

}  // namespace wc

using namespace wc;

extern "C" int wc_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const void* w,
                                   const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(d && plan && w && w_strides && U, "wc_filter_transform: null pointer");
  if (d->direct == 1) {
    // the direct form has nothing to transform: U is the filter with taps outermost, channels innermost
    if (!direct_conv_fits(d)) return fail(WC_ERR_UNSUPPORTED, "wc_filter_transform: problem outside the direct form's range");
    return direct_filter(d, w, w_strides, U, stream);
  }
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);   // validates the descriptor
  if (rc) return rc;
  WC_CHECK_ARG(plan->n_pieces > 0 && plan->n_pieces <= WC_MAX_PIECES, "wc_filter_transform: bad plan");
  {
    FilterFastArgs f;
    int vec = 1;
    bool dense = false;
    if (filter_fast_setup(d, plan, w, w_strides, U, &f, &vec, &dense)) {
      const wc_piece& pc = plan->piece[0];
      const int k0 = kind_of(plan->m[0], pc.r[0]), k1 = kind_of(plan->m[1], pc.r[1]), k2 = kind_of(plan->m[2], pc.r[2]);
      FilterFastKernel fn = dispatch_dtype(d->dtype, [&](auto t) {
        return dense ? pick_fast<decltype(t), true>(k0, k1, k2) : pick_fast<decltype(t), false>(k0, k1, k2);
      });
      const long long n = (long long)d->K * (f.Cp / vec);
      WC_CHECK_ARG(n < (1ll << 31), "wc_filter_transform: problem too large");
      hipLaunchKernelGGL(fn, dim3((unsigned)ceil_div_ll(n, 256)), dim3(256), 0, as_stream(stream), f);
      WC_CHECK_LAUNCH("filter_transform_fast_kernel");
      return WC_OK;
    }
  }
  FilterArgs a;
  a.w = w; a.U = U;
  for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
  a.C = d->C; a.Cp = wc_padded_channels(d->C); a.K = d->K;
  a.step = plan->tap_step;
  for (int i = 0; i < 3; ++i) a.m[i] = plan->m[i];
  a.n_pieces = plan->n_pieces;
  for (int i = 0; i < plan->n_pieces; ++i) a.piece[i] = plan->piece[i];
  a.total = (long long)plan->t_total * d->K * a.Cp;
  a.stacked = d->stacked && plan->n_pieces > 1;
  stacked_taps(plan, a.rp);
  bool small_taps = true;
  for (int i = 0; i < plan->n_pieces; ++i)
    for (int q = 0; q < 3; ++q)     // a stacked plan may hold pieces without taps (r = 0): their block of U is zero
      small_taps = small_taps && plan->piece[i].r[q] >= (a.stacked ? 0 : 1) && plan->piece[i].r[q] <= 3;
  const bool flat = plan->m[0] == 1;
  const int mo = plan->m[1];
  if (small_taps && plan->m[2] == mo && (flat ? (mo == 2 || mo == 4 || (mo == 3 && a.stacked)) : (mo == 2 && plan->m[0] == 2))) {
    const long long n = (long long)d->K * a.Cp;
    WC_CHECK_ARG(n < (1ll << 31), "wc_filter_transform: problem too large");
    const dim3 grid((unsigned)ceil_div_ll(n, 256), (unsigned)plan->n_pieces);
    void (*fn)(FilterArgs) = dispatch_dtype(d->dtype, [&](auto t) -> void (*)(FilterArgs) {
      using T = decltype(t);
      return !flat ? &filter_transform_pieces_kernel<T, false, 2>
                   : (mo == 4 ? &filter_transform_pieces_kernel<T, true, 4>
                      : mo == 3 ? &filter_transform_pieces_kernel<T, true, 3> : &filter_transform_pieces_kernel<T, true, 2>);
    });
    hipLaunchKernelGGL(fn, grid, dim3(256), 0, as_stream(stream), a);
    WC_CHECK_LAUNCH("filter_transform_pieces_kernel");
    return WC_OK;
  }
  if (a.stacked) return fail(WC_ERR_UNSUPPORTED, "stacked filter transform needs output tile 2 or 4 in 2-D, 2 in 3-D");
  const long long blocks = ceil_div_ll(a.total, 256);
  WC_CHECK_ARG(blocks < (1ll << 31), "wc_filter_transform: problem too large");
  void (*gen)(FilterArgs) = dispatch_dtype(d->dtype, [](auto t) -> void (*)(FilterArgs) {
    return &filter_transform_kernel<decltype(t)>;
  });
  hipLaunchKernelGGL(gen, dim3((unsigned)blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("filter_transform_kernel");
  return WC_OK;
}
