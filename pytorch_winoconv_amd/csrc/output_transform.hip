// Output transform y = sum over pieces of (AT_d x AT_h x AT_w) m, + bias, cropped at the edges.
//
// Replaces outputWino2NormTransform + outputWino2NormCalculation + outputAggregate of the
// reference (src/split_kernel.cu:126-203, src/calculation_kernels.cu:1524-1770).  The reference
// stores one partial output per piece (tmp_output, base_conv_launchers.cu:375-377) and sums
// them in a second pass; here every piece is accumulated in fp32 registers and y is written
// once.  Edge rule as in the reference (split_kernel.cu:162-176): an output position is
// written iff it lies inside (oD, oH, oW).
//
// HBM-bound: a thread owns one tile x VEC consecutive output channels (lanes along K).
// Three kernels: a separable compile-time one for single-piece plans (F(2,3)^2, F(4,3)^2,
// F(2,3)^3, whole-kernel tiles); one for 2-D DWM plans that runs the same compile-time body for
// every piece and sums the pieces in registers; and a streaming one for 3-D DWM plans, where
// each loaded tile row is transformed along the width and then scattered into the m^d
// accumulators with coefficients from a constant table.
#include "wc_transform.h"
#include <type_traits>

namespace wc {

struct OutArgs {
  const void* M;
  const void* bias;
  void* y;
  int oD, oH, oW, K, ldm;
  int nD, nH, nW;
  long long t_stride;   // P * ldm
  int t_offset;
  int n_kvec;           // K / VEC
  long long total;      // P * n_kvec
  int per_xcd;
};

struct Where { int tw, th, td; long long b; };

__device__ __forceinline__ Where decode_tile(long long p, int nD, int nH, int nW) {
  Where w;
  w.tw = (int)(p % nW); long long q = p / nW;
  w.th = (int)(q % nH); q /= nH;
  w.td = (int)(q % nD);
  w.b = q / nD;
  return w;
}

template <typename T, int M0, int M1, int M2, int VEC>
__device__ __forceinline__ void write_tile(const OutArgs& a, const Where& w, int k,
                                           float (&o)[M0 * M1 * M2][VEC]) {
  T* y = static_cast<T*>(a.y);
  float bias[VEC];
  if (a.bias) load_pack<T, VEC>(static_cast<const T*>(a.bias) + k, bias);
  static_for<0, M0>([&](auto a0_) {
    constexpr int a0 = decltype(a0_)::value;
    const int od = M0 * w.td + a0;
    static_for<0, M1>([&](auto a1_) {
      constexpr int a1 = decltype(a1_)::value;
      const int oh = M1 * w.th + a1;
      static_for<0, M2>([&](auto a2_) {
        constexpr int a2 = decltype(a2_)::value;
        constexpr int e = (a0 * M1 + a1) * M2 + a2;
        const int ow = M2 * w.tw + a2;
        if (od < a.oD && oh < a.oH && ow < a.oW) {
          if (a.bias) {
#pragma unroll
            for (int v = 0; v < VEC; ++v) o[e][v] += bias[v];
          }
          store_pack<T, VEC>(y + (((w.b * a.oD + od) * a.oH + oh) * a.oW + ow) * a.K + k, o[e]);
        }
      });
    });
  });
}

// ---- single piece, separable ------------------------------------------------------------------
template <typename T, int K0, int K1, int K2, int VEC>
__global__ __launch_bounds__(256) void output_transform_kernel(OutArgs a) {
  constexpr int A0 = Mats<K0>::alpha, A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
  constexpr int M0 = Mats<K0>::m, M1 = Mats<K1>::m, M2 = Mats<K2>::m;
  const int blk = xcd_remap(blockIdx.x, a.per_xcd);
  const long long idx = (long long)blk * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.n_kvec) * VEC;
  const long long p = idx / a.n_kvec;
  const Where w = decode_tile(p, a.nD, a.nH, a.nW);
  const T* M = static_cast<const T*>(a.M) + (long long)a.t_offset * a.t_stride + p * a.ldm + k;

  float m[A0 * A1 * A2][VEC];
  static_for<0, A0 * A1 * A2>([&](auto e_) {
    constexpr int e = decltype(e_)::value;
    load_pack<T, VEC>(M + e * a.t_stride, m[e]);
  });
  float s2[A0 * A1 * M2][VEC];
  apply_axis<MatSel<K2, true>, 2, A0, A1, A2, VEC>(m, s2);
  float s1[A0 * M1 * M2][VEC];
  apply_axis<MatSel<K1, true>, 1, A0, A1, M2, VEC>(s2, s1);
  if constexpr (A0 > 1) {
    float s0[M0 * M1 * M2][VEC];
    apply_axis<MatSel<K0, true>, 0, A0, M1, M2, VEC>(s1, s0);
    write_tile<T, M0, M1, M2, VEC>(a, w, k, s0);
  } else {
    write_tile<T, M0, M1, M2, VEC>(a, w, k, s1);
  }
}

// ---- any number of F(2, r) pieces, streaming -----------------------------------------------------
// AT of F(2, r) by [r][output a][element i] (r = 0 is the one-element depth axis)
__constant__ const float kAT2[4][2][4] = {
    {{1, 0, 0, 0}, {0, 0, 0, 0}},
    {{1, 0, 0, 0}, {0, 1, 0, 0}},
    {{1, 1, 0, 0}, {0, 1, 1, 0}},
    {{1, 1, 1, 0}, {0, 1, -1, -1}},
};

// A^T of F(4, r) by [r][output a][element i]
__constant__ const float kAT4[4][4][6] = {
    {{0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0}, {0, 0, 0, 0, 0, 0}},
    {{1, 0, 0, 0, 0, 0}, {0, 1, 0, 0, 0, 0}, {0, 0, 1, 0, 0, 0}, {0, 0, 0, 1, 0, 0}},
    {{1, 1, 1, 1, 0, 0}, {0, 1, -1, 2, 0, 0}, {0, 1, 1, 4, 0, 0}, {0, 1, -1, 8, 1, 0}},
    {{1, 1, 1, 1, 1, 0}, {0, 1, -1, 2, -2, 0}, {0, 1, 1, 4, 4, 0}, {0, 1, -1, 8, -8, 1}},
};

struct OutMultiArgs {
  OutArgs o;
  int n_pieces;
  int info[WC_MAX_PIECES];   // t_offset | r0 << 16 | r1 << 20 | r2 << 24 (r0 = 0: flat depth)
};

// MO: output tile extent on the image axes (2, or 4 for 2-D problems); FLAT: one-element depth axis
template <typename T, bool FLAT, int MO, int VEC>
__global__ __launch_bounds__(256) void output_multi_kernel(OutMultiArgs g) {
  constexpr int M0 = FLAT ? 1 : 2;
  static_assert(MO == 2 || (MO == 4 && FLAT), "tile 4 is 2-D only");
  const OutArgs& a = g.o;
  const int blk = xcd_remap(blockIdx.x, a.per_xcd);
  const long long idx = (long long)blk * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.n_kvec) * VEC;
  const long long p = idx / a.n_kvec;
  const Where w = decode_tile(p, a.nD, a.nH, a.nW);
  const T* M = static_cast<const T*>(a.M) + p * a.ldm + k;

  float acc[M0 * MO * MO][VEC];
#pragma unroll
  for (int e = 0; e < M0 * MO * MO; ++e)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[e][v] = 0.f;

  for (int s = 0; s < g.n_pieces; ++s) {
    const int info = g.info[s];
    const int r0 = (info >> 16) & 15, r1 = (info >> 20) & 15, r2 = (info >> 24) & 15;
    const int n0 = FLAT ? 1 : r0 + 1, n1 = r1 + MO - 1, n2 = r2 + MO - 1;
    const T* Ms = M + (long long)(info & 0xffff) * a.t_stride;
    // coefficients of this piece, fetched once (wave-uniform, they live in scalar registers)
    constexpr int NW = MO + 2;
    float cH[MO][NW], cW[MO][NW];
#pragma unroll
    for (int o = 0; o < MO; ++o)
#pragma unroll
      for (int i = 0; i < NW; ++i) {
        cH[o][i] = MO == 2 ? kAT2[r1][o & 1][i & 3] : kAT4[r1][o][i];
        cW[o][i] = MO == 2 ? kAT2[r2][o & 1][i & 3] : kAT4[r2][o][i];
      }
    // one tile row (up to MO + 2 elements) at a time: all its loads are issued before the first
    // FMA so that a thread keeps several requests in flight; width pass on the row, then the MO
    // results are scattered along height / depth
    for (int i0 = 0; i0 < n0; ++i0) {
#pragma unroll
      for (int i1 = 0; i1 < NW; ++i1) {
        if (i1 < n1) {
          const T* Mr = Ms + (long long)((i0 * n1 + i1) * n2) * a.t_stride;
          float v[NW][VEC];
#pragma unroll
          for (int i2 = 0; i2 < NW; ++i2)
            if (i2 < n2) load_pack<T, VEC>(Mr + (long long)i2 * a.t_stride, v[i2]);
          float rowres[MO][VEC];
#pragma unroll
          for (int a2 = 0; a2 < MO; ++a2)
#pragma unroll
            for (int q = 0; q < VEC; ++q) rowres[a2][q] = 0.f;
#pragma unroll
          for (int i2 = 0; i2 < NW; ++i2) {
            if (i2 < n2) {
#pragma unroll
              for (int a2 = 0; a2 < MO; ++a2)
#pragma unroll
                for (int q = 0; q < VEC; ++q) rowres[a2][q] = __builtin_fmaf(cW[a2][i2], v[i2][q], rowres[a2][q]);
            }
          }
#pragma unroll
          for (int a0 = 0; a0 < M0; ++a0)
#pragma unroll
            for (int a1 = 0; a1 < MO; ++a1) {
              const float c01 = kAT2[r0][a0][i0] * cH[a1][i1];
              if (c01 != 0.f) {
#pragma unroll
                for (int a2 = 0; a2 < MO; ++a2)
#pragma unroll
                  for (int q = 0; q < VEC; ++q)
                    acc[(a0 * MO + a1) * MO + a2][q] = __builtin_fmaf(c01, rowres[a2][q], acc[(a0 * MO + a1) * MO + a2][q]);
              }
            }
        }
      }
    }
  }
  write_tile<T, M0, MO, MO, VEC>(a, w, k, acc);
}

// ---- 3-D tile 2 x 4 x 4 of a 3x3x3 kernel ---------------------------------------------------------
// One depth plane (36 elements) at a time: height / width passes of F(4,3), then the plane is
// added to the two output planes with the coefficients of A^T of F(2,3)
// ([[1, 1, 1, 0], [0, 1, -1, -1]], matrix_conv.py:21-22).
template <typename T, int VEC>
__global__ __launch_bounds__(256) void output_transform_3d_m4_kernel(OutArgs a) {
  const int blk = xcd_remap(blockIdx.x, a.per_xcd);
  const long long idx = (long long)blk * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.n_kvec) * VEC;
  const long long p = idx / a.n_kvec;
  const Where w = decode_tile(p, a.nD, a.nH, a.nW);
  const T* M = static_cast<const T*>(a.M) + (long long)a.t_offset * a.t_stride + p * a.ldm + k;
  float acc[32][VEC];
#pragma unroll
  for (int e = 0; e < 32; ++e)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[e][v] = 0.f;
  static_for<0, 4>([&](auto i0_) {
    constexpr int i0 = decltype(i0_)::value;
    float m[36][VEC];
    static_for<0, 36>([&](auto e_) {
      constexpr int e = decltype(e_)::value;
      load_pack<T, VEC>(M + (long long)(i0 * 36 + e) * a.t_stride, m[e]);
    });
    float s2[24][VEC];
    apply_axis<MatSel<KIND_43, true>, 2, 1, 6, 6, VEC>(m, s2);
    float s1[16][VEC];
    apply_axis<MatSel<KIND_43, true>, 1, 1, 6, 4, VEC>(s2, s1);
    constexpr float c0 = Mats<KIND_23>::at(0, i0), c1 = Mats<KIND_23>::at(1, i0);
#pragma unroll
    for (int e = 0; e < 16; ++e)
#pragma unroll
      for (int v = 0; v < VEC; ++v) {
        if constexpr (c0 != 0.f) acc[e][v] += c0 * s1[e][v];
        if constexpr (c1 != 0.f) acc[16 + e][v] += c1 * s1[e][v];
      }
    // compiler fence: keeps the loads of the next plane below this point (hoisted, all 144 loads
    // of the tile are live at once and the kernel runs at one wavefront per SIMD)
    asm volatile("" ::: "memory");
  });
  write_tile<T, 2, 4, 4, VEC>(a, w, k, acc);
}

// ---- all pieces of a 2-D DWM plan, compile-time body per piece ------------------------------------
// Each piece is handled like a single-piece plan (all alpha_h x alpha_w loads of the tile issued
// together, separable AT passes in registers) and added to the m x m accumulators; the piece's
// taps per axis select the body, a branch that is uniform over the launch.
template <typename T, int MO, int VEC>
__global__ __launch_bounds__(256) void output_pieces_kernel(OutMultiArgs g) {
  const OutArgs& a = g.o;
  const int blk = xcd_remap(blockIdx.x, a.per_xcd);
  const long long idx = (long long)blk * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.n_kvec) * VEC;
  const long long p = idx / a.n_kvec;
  const Where w = decode_tile(p, a.nD, a.nH, a.nW);
  const T* M = static_cast<const T*>(a.M) + p * a.ldm + k;
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;

  float acc[MO * MO][VEC];
#pragma unroll
  for (int e = 0; e < MO * MO; ++e)
#pragma unroll
    for (int v = 0; v < VEC; ++v) acc[e][v] = 0.f;

  auto piece = [&](auto k1_, auto k2_, const T* Ms) {
    constexpr int K1 = decltype(k1_)::value, K2 = decltype(k2_)::value;
    constexpr int A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
    float m[A1 * A2][VEC];
    static_for<0, A1 * A2>([&](auto e_) {
      constexpr int e = decltype(e_)::value;
      load_pack<T, VEC>(Ms + e * a.t_stride, m[e]);
    });
    float s2[A1 * MO][VEC];
    apply_axis<MatSel<K2, true>, 2, 1, A1, A2, VEC>(m, s2);
    float s1[MO * MO][VEC];
    apply_axis<MatSel<K1, true>, 1, 1, A1, MO, VEC>(s2, s1);
#pragma unroll
    for (int e = 0; e < MO * MO; ++e)
#pragma unroll
      for (int v = 0; v < VEC; ++v) acc[e][v] += s1[e][v];
  };
  using IA = std::integral_constant<int, KA>;
  using IB = std::integral_constant<int, KB>;
  using IC = std::integral_constant<int, KC>;
  for (int s = 0; s < g.n_pieces; ++s) {
    const int info = g.info[s];
    const int r1 = (info >> 20) & 15, r2 = (info >> 24) & 15;
    const T* Ms = M + (long long)(info & 0xffff) * a.t_stride;
#define WC_ROW(I1) \
  switch (r2) { case 1: piece(I1{}, IA{}, Ms); break; case 2: piece(I1{}, IB{}, Ms); break; default: piece(I1{}, IC{}, Ms); }
    switch (r1) { case 1: WC_ROW(IA) break; case 2: WC_ROW(IB) break; default: WC_ROW(IC) }
#undef WC_ROW
  }
  write_tile<T, 1, MO, MO, VEC>(a, w, k, acc);
}

template <typename T>
static void (*pick_pieces(int m, int vec))(OutMultiArgs) {
  if (m == 4) return vec == 2 ? &output_pieces_kernel<T, 4, 2> : &output_pieces_kernel<T, 4, 1>;
  return vec == 4 ? &output_pieces_kernel<T, 2, 4> : &output_pieces_kernel<T, 2, 1>;
}

using OutKernel = void (*)(OutArgs);
using OutMultiKernel = void (*)(OutMultiArgs);

template <typename T>
static OutKernel pick_single(int k0, int k1, int k2, int vec) {
  if (k0 == KIND_11 && k1 == KIND_23 && k2 == KIND_23)
    return vec == 4 ? &output_transform_kernel<T, KIND_11, KIND_23, KIND_23, 4>
                    : &output_transform_kernel<T, KIND_11, KIND_23, KIND_23, 1>;
  if (k0 == KIND_11 && k1 == KIND_43 && k2 == KIND_43)
    return vec == 4 ? &output_transform_kernel<T, KIND_11, KIND_43, KIND_43, 2>
                    : &output_transform_kernel<T, KIND_11, KIND_43, KIND_43, 1>;
  if (k0 == KIND_23 && k1 == KIND_23 && k2 == KIND_23)
    return vec == 4 ? &output_transform_kernel<T, KIND_23, KIND_23, KIND_23, 2>
                    : &output_transform_kernel<T, KIND_23, KIND_23, KIND_23, 1>;
  if (k0 == KIND_23 && k1 == KIND_43 && k2 == KIND_43)
    return vec == 4 ? &output_transform_3d_m4_kernel<T, 2> : &output_transform_3d_m4_kernel<T, 1>;
  // whole-kernel tiles F(2,r) x F(2,r), r = 4..7
#define WC_WHOLE(KD) \
  if (k0 == KIND_11 && k1 == KD && k2 == KD) \
    return vec == 4 ? &output_transform_kernel<T, KIND_11, KD, KD, 2> : &output_transform_kernel<T, KIND_11, KD, KD, 1>;
  WC_WHOLE(KIND_24) WC_WHOLE(KIND_25) WC_WHOLE(KIND_26) WC_WHOLE(KIND_27)
  WC_WHOLE(KIND_33)       // the shared tile of three-tap pieces
#undef WC_WHOLE
  return nullptr;
}

template <typename T>
static OutMultiKernel pick_multi(bool flat, int m, int vec) {
  if (flat && m == 4) return vec == 4 ? &output_multi_kernel<T, true, 4, 4> : &output_multi_kernel<T, true, 4, 1>;
  if (flat) return vec == 4 ? &output_multi_kernel<T, true, 2, 4> : &output_multi_kernel<T, true, 2, 1>;
  return vec == 4 ? &output_multi_kernel<T, false, 2, 4> : &output_multi_kernel<T, false, 2, 1>;
}

}  // namespace wc

using namespace wc;

extern "C" int wc_output_transform(const wc_conv_desc* d, const wc_plan* plan_in, const void* M,
                                   const void* bias, int n_images, void* y, void* stream) {
  WC_CHECK_ARG(d && plan_in && M && y, "wc_output_transform: null pointer");
  // a stacked plan has one set of products (the batched GEMM has added the pieces): the output
  // transform of a single piece with the shared tile
  wc_plan one;
  const wc_plan* plan = plan_in;
  if (d->stacked && plan_in->n_pieces > 1 && plan_in->n_pieces <= WC_MAX_PIECES) {
    one = *plan_in;
    one.n_pieces = 1;
    stacked_taps(plan_in, one.piece[0].r);
    one.piece[0].t_offset = 0;
    plan = &one;
  }
  WC_CHECK_ARG(n_images > 0, "wc_output_transform: n_images %d", n_images);
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);
  if (rc) return rc;
  WC_CHECK_ARG(plan->n_pieces > 0 && plan->n_pieces <= WC_MAX_PIECES, "wc_output_transform: bad plan");
  const int ldm = wc_padded_channels8(d->K);
  const long long P = (long long)n_images * grid[0] * grid[1] * grid[2];
  const int vec = (d->K % 4 == 0) ? 4 : 1;
  OutArgs a;
  a.M = M; a.bias = bias; a.y = y;
  a.oD = out[0]; a.oH = out[1]; a.oW = out[2]; a.K = d->K; a.ldm = ldm;
  a.nD = grid[0]; a.nH = grid[1]; a.nW = grid[2];
  a.t_stride = P * ldm;
  a.t_offset = 0;
  hipStream_t s = as_stream(stream);

  int k[3] = {0, 0, 0};
  OutKernel single = nullptr;
  if (plan->n_pieces == 1) {
    for (int q = 0; q < 3; ++q) k[q] = kind_of(plan->m[q], plan->piece[0].r[q]);
    single = dispatch_dtype(d->dtype, [&](auto t) { return pick_single<decltype(t)>(k[0], k[1], k[2], vec); });
  }
  if (single) {
    // 3-D tiles, F(4,3) tiles (36 live elements per channel) and whole-kernel tiles use 2 channels per thread:
    // more wavefronts in flight (measured 64.8 vs 69.2 us at N=64, K=256, 56x56 fp16)
    const int v = ((k[0] == KIND_23 || k[1] == KIND_43 || k[1] >= KIND_24) && vec == 4) ? 2 : vec;
    a.n_kvec = d->K / v;
    a.total = P * a.n_kvec;
    a.per_xcd = (int)ceil_div_ll(ceil_div_ll(a.total, 256), kXcds);
    a.t_offset = plan->piece[0].t_offset;
    hipLaunchKernelGGL(single, dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), 0, s, a);
    WC_CHECK_LAUNCH("output_transform_kernel");
    return WC_OK;
  }
  const bool tile4 = plan->m[0] == 1 && plan->m[1] == 4 && plan->m[2] == 4;
  const bool tile2 = plan->m[1] == 2 && plan->m[2] == 2 && (plan->m[0] == 1 || plan->m[0] == 2);
  if (!tile2 && !tile4)
    return fail(WC_ERR_UNSUPPORTED, "multi-piece output transform needs output tile 2, or 4 in 2-D");
  if (plan->t_total > 0xffff)
    return fail(WC_ERR_UNSUPPORTED, "plan with %d transform elements is too large", plan->t_total);
  OutMultiArgs g;
  const bool flat = plan->m[0] == 1;
  a.n_kvec = d->K / vec;
  a.total = P * a.n_kvec;
  a.per_xcd = (int)ceil_div_ll(ceil_div_ll(a.total, 256), kXcds);
  g.o = a;
  g.n_pieces = plan->n_pieces;
  for (int i = 0; i < plan->n_pieces; ++i) {
    const wc_piece& pc = plan->piece[i];
    for (int q = 0; q < 3; ++q)
      if (pc.r[q] < 1 || pc.r[q] > 3) return fail(WC_ERR_UNSUPPORTED, "piece with %d taps", pc.r[q]);
    g.info[i] = pc.t_offset | ((flat ? 0 : pc.r[0]) << 16) | (pc.r[1] << 20) | (pc.r[2] << 24);
  }
  if (flat) {
    // 2-D plans: compile-time body per piece; F(4,r) tiles use 2 channels per thread
    const int v = (tile4 && vec == 4) ? 2 : vec;
    g.o.n_kvec = d->K / v;
    g.o.total = P * g.o.n_kvec;
    g.o.per_xcd = (int)ceil_div_ll(ceil_div_ll(g.o.total, 256), kXcds);
    OutMultiKernel fp = dispatch_dtype(d->dtype, [&](auto t) { return pick_pieces<decltype(t)>(plan->m[1], v); });
    hipLaunchKernelGGL(fp, dim3((unsigned)(g.o.per_xcd * kXcds)), dim3(256), 0, s, g);
    WC_CHECK_LAUNCH("output_pieces_kernel");
    return WC_OK;
  }
  OutMultiKernel fn = dispatch_dtype(d->dtype, [&](auto t) { return pick_multi<decltype(t)>(flat, plan->m[1], vec); });
  hipLaunchKernelGGL(fn, dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), 0, s, g);
  WC_CHECK_LAUNCH("output_multi_kernel");
  return WC_OK;
}

// M (16, P, ldm) over pixel columns: P = n_images x tiles in depth x tiles in height x grid_w columns, of which the
// first oW hold outputs (input_transform_columns, the product with the width taps along its reduction: gemm.hip)
int wc::output_transform_columns(const wc_conv_desc* d, const void* M, const void* bias, int n_images, void* y, void* stream) {
  WC_CHECK_ARG(d && M && y && n_images > 0, "output_transform_columns: null pointer or no images");
  WC_CHECK_ARG(d->ndim == 3 && d->stride == 1 && d->y_layout == 0 && d->kernel[0] == 3 && d->kernel[1] == 3 && d->kernel[2] == 3 &&
               d->dtype != WC_F32, "output_transform_columns: 3x3x3 kernels at stride 1 on channel-last 16-bit tensors");
  int out[3], grid[3];
  wc_conv_desc t = *d;
  t.m = 2;
  int rc = wc_conv_out_dims(&t, out, grid);
  if (rc) return rc;
  const int Wx = columns_width(d);
  const long long P = (long long)n_images * grid[0] * grid[1] * Wx;
  const int vec = d->K % 4 == 0 ? 4 : 1;           // (2 and 8 channels per thread measured the same)
  OutArgs a;
  a.M = M; a.bias = bias; a.y = y;
  a.oD = out[0]; a.oH = out[1]; a.oW = out[2]; a.K = d->K; a.ldm = wc_padded_channels8(d->K);
  a.nD = grid[0]; a.nH = grid[1]; a.nW = Wx;
  a.t_stride = P * a.ldm;
  a.t_offset = 0;
  a.n_kvec = d->K / vec;
  a.total = P * a.n_kvec;
  a.per_xcd = (int)ceil_div_ll(ceil_div_ll(a.total, 256), kXcds);
  WC_CHECK_ARG((long long)a.per_xcd * kXcds < (1ll << 31), "output_transform_columns: problem too large");
  OutKernel fn = dispatch_dtype(d->dtype, [&](auto t_) -> OutKernel {
    using T = decltype(t_);
    return vec == 4 ? &output_transform_kernel<T, KIND_23, KIND_23, KIND_11, 4> : &output_transform_kernel<T, KIND_23, KIND_23, KIND_11, 1>;
  });
  hipLaunchKernelGGL(fn, dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("output_transform_kernel (pixel columns)");
  return WC_OK;
}
