// Weight gradient of the Winograd / DWM convolution, in the transform domain.
//
// The reference never implemented a backward pass (it holds only a pointer-assign helper for one,
// src/back/utils.cu:15-24, and an empty header, include/split_functions_grad.h:3-6).  With
// y = sum over pieces of A^T [ (G g G^T) . (B^T d B) ] A, the gradient with respect to g is
//
//   dU[t][k][c] = sum over tiles p of dM[t][p][k] * V[t][p][c]     dM = A dy A^T per tile
//   dg          = G^T dU G                                         per piece, onto its taps
//
// V is the forward input transform (same kernels) and dM comes from a gather kernel of the same
// shape; both keep the forward layout (rows = tiles, channels contiguous).  The contraction over
// the tiles runs on MFMA straight from those layouts (gemm_tn.hip: operands in their storage type,
// whose products are exact in fp32; the sum over up to millions of tiles is kept in fp32 from the
// first product to the last addition), split into parts that are added here, and a last kernel
// applies G^T . G and accumulates over image chunks (backward_filter.hip).
#include "wc_transform.h"
#include <algorithm>

namespace wc {

__device__ __forceinline__ int dev_kind_of(int m, int r) {
  return m == 1 ? KIND_11 : (m == 4 ? (r == 3 ? KIND_43 : r == 2 ? KIND_42 : KIND_41)
                                   : (r <= 3 ? KIND_21 + (r - 1) : KIND_24 + (r - 4)));
}

struct GradOutArgs {
  const void* dy;
  void* dM;
  int oD, oH, oW, K, ldm;
  int nD, nH, nW;
  long long P;
  int m[3];
  int n_pieces;
  long long total;           // T * P * ldm
  wc_piece piece[WC_MAX_PIECES];
};

// dM[t][p][k] = sum_a AT[a0][i0] AT[a1][i1] AT[a2][i2] dy[b, m0 td + a0, m1 th + a1, m2 tw + a2, k]
template <typename T>
__global__ __launch_bounds__(256) void grad_output_transform_kernel(const GradOutArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int k = (int)(idx % a.ldm);
  long long q = idx / a.ldm;
  const long long p = q % a.P;
  const int t = (int)(q / a.P);
  T* dM = static_cast<T*>(a.dM);
  if (k >= a.K) { dM[idx] = static_cast<T>(0.f); return; }
  int s = 0;
  while (s + 1 < a.n_pieces && a.piece[s + 1].t_offset <= t) ++s;
  const wc_piece& pc = a.piece[s];
  const int e = t - pc.t_offset;
  const int a1n = a.m[1] + pc.r[1] - 1, a2n = a.m[2] + pc.r[2] - 1;
  const int i2 = e % a2n, i1 = (e / a2n) % a1n, i0 = e / (a2n * a1n);
  const int k0 = dev_kind_of(a.m[0], pc.r[0]), k1 = dev_kind_of(a.m[1], pc.r[1]), k2 = dev_kind_of(a.m[2], pc.r[2]);
  const int tw = (int)(p % a.nW); long long r = p / a.nW;
  const int th = (int)(r % a.nH); r /= a.nH;
  const int td = (int)(r % a.nD);
  const long long b = r / a.nD;
  const T* dy = static_cast<const T*>(a.dy);
  float acc = 0.f;
  for (int a0 = 0; a0 < a.m[0]; ++a0) {
    const int od = a.m[0] * td + a0;
    if (od >= a.oD) continue;
    const float c0 = table_at(k0, a0, i0);
    for (int a1 = 0; a1 < a.m[1]; ++a1) {
      const int oh = a.m[1] * th + a1;
      if (oh >= a.oH) continue;
      const float c01 = c0 * table_at(k1, a1, i1);
      for (int a2 = 0; a2 < a.m[2]; ++a2) {
        const int ow = a.m[2] * tw + a2;
        if (ow >= a.oW) continue;
        const float c = c01 * table_at(k2, a2, i2);
        if (c != 0.f)
          acc = __builtin_fmaf(c, static_cast<float>(dy[(((b * a.oD + od) * a.oH + oh) * a.oW + ow) * a.K + k]), acc);
      }
    }
  }
  dM[idx] = static_cast<T>(acc);
}

// A (alpha x m) = transpose of A^T, as an apply_axis matrix
template <int KIND>
struct MatA {
  static constexpr int rows = Mats<KIND>::alpha;
  static constexpr int cols = Mats<KIND>::m;
  __host__ __device__ static constexpr float get(int i, int j) { return Mats<KIND>::at(j, i); }
  __host__ __device__ static constexpr int first_nz(int i) {
    for (int j = 0; j < cols; ++j)
      if (get(i, j) != 0.f) return j;
    return cols;
  }
};

// The same for plans whose pieces have 1..3 taps per axis (every DWM plan): a thread owns one tile x
// VEC output channels, loads its m^d values of dy once and writes dM = (A x A x A) dy for every
// piece; the piece's taps select a compile-time body (a branch that is uniform over the launch).
// M0 x MO x MO is the output tile: 1 x 2 x 2, 1 x 4 x 4, 2 x 2 x 2 or 2 x 4 x 4.
template <typename T, int M0, int MO, int VEC>
__global__ __launch_bounds__(256) void grad_output_pieces_kernel(const GradOutArgs a) {
  const int n_kvec = a.ldm / VEC;
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.P * n_kvec) return;
  const int k = (int)(idx % n_kvec) * VEC;
  const long long p = idx / n_kvec;
  const int tw = (int)(p % a.nW); long long r = p / a.nW;
  const int th = (int)(r % a.nH); r /= a.nH;
  const int td = (int)(r % a.nD);
  const long long b = r / a.nD;
  const T* dy = static_cast<const T*>(a.dy);
  const bool k_ok = k < a.K;                       // ldm - K padding columns are written as zeros
  float g[M0 * MO * MO][VEC];
  static_for<0, M0>([&](auto a0_) {
    constexpr int a0 = decltype(a0_)::value;
    const int od = M0 * td + a0;
    static_for<0, MO>([&](auto a1_) {
      constexpr int a1 = decltype(a1_)::value;
      const int oh = MO * th + a1;
      static_for<0, MO>([&](auto a2_) {
        constexpr int a2 = decltype(a2_)::value;
        const int ow = MO * tw + a2;
        constexpr int e = (a0 * MO + a1) * MO + a2;
        const bool ok = k_ok && od < a.oD && oh < a.oH && ow < a.oW;
        const long long off = (((b * a.oD + min(od, a.oD - 1)) * a.oH + min(oh, a.oH - 1)) * a.oW + min(ow, a.oW - 1)) * a.K + (k_ok ? k : 0);
        if constexpr (VEC == 1) {
          g[e][0] = ok ? static_cast<float>(dy[off]) : 0.f;
        } else {
          load_pack<T, VEC>(dy + off, g[e]);
#pragma unroll
          for (int v = 0; v < VEC; ++v) g[e][v] = ok ? g[e][v] : 0.f;
        }
      });
    });
  });
  T* dM = static_cast<T*>(a.dM) + p * a.ldm + k;
  const long long t_stride = a.P * a.ldm;
  auto piece = [&](auto k0_, auto k1_, auto k2_, int t_offset) {
    constexpr int K0 = decltype(k0_)::value, K1 = decltype(k1_)::value, K2 = decltype(k2_)::value;
    constexpr int A0 = Mats<K0>::alpha, A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
    float s2[M0 * MO * A2][VEC];
    apply_axis<MatA<K2>, 2, M0, MO, MO, VEC>(g, s2);
    float s1[M0 * A1 * A2][VEC];
    apply_axis<MatA<K1>, 1, M0, MO, A2, VEC>(s2, s1);
    T* out = dM + (long long)t_offset * t_stride;
    if constexpr (M0 > 1) {
      float s0[A0 * A1 * A2][VEC];
      apply_axis<MatA<K0>, 0, M0, A1, A2, VEC>(s1, s0);
      static_for<0, A0 * A1 * A2>([&](auto e_) {
        constexpr int e = decltype(e_)::value;
        store_pack<T, VEC>(out + e * t_stride, s0[e]);
      });
    } else {
      static_for<0, A1 * A2>([&](auto e_) {
        constexpr int e = decltype(e_)::value;
        store_pack<T, VEC>(out + e * t_stride, s1[e]);
      });
    }
  };
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;
  using IA = ic<KA>; using IB = ic<KB>; using IC = ic<KC>;
  for (int s = 0; s < a.n_pieces; ++s) {
    const wc_piece& pc = a.piece[s];
    const int t0 = pc.t_offset;
    if constexpr (M0 == 1) {
#define WC_ROW(I1) \
  switch (pc.r[2]) { case 1: piece(ic<KIND_11>{}, I1{}, IA{}, t0); break; case 2: piece(ic<KIND_11>{}, I1{}, IB{}, t0); break; \
                     default: piece(ic<KIND_11>{}, I1{}, IC{}, t0); }
      switch (pc.r[1]) { case 1: WC_ROW(IA) break; case 2: WC_ROW(IB) break; default: WC_ROW(IC) }
#undef WC_ROW
    } else if constexpr (MO == 4) {
      piece(ic<KIND_23>{}, IC{}, IC{}, t0);        // the only 3-D plan with tile 4: one 3x3x3 piece
    } else {
#define WC_ROW(I0, I1) \
  switch (pc.r[2]) { case 1: piece(I0{}, I1{}, IA{}, t0); break; case 2: piece(I0{}, I1{}, IB{}, t0); break; \
                     default: piece(I0{}, I1{}, IC{}, t0); }
#define WC_PLANE(I0) \
  switch (pc.r[1]) { case 1: WC_ROW(I0, IA) break; case 2: WC_ROW(I0, IB) break; default: WC_ROW(I0, IC) }
      switch (pc.r[0]) { case 1: WC_PLANE(IA) break; case 2: WC_PLANE(IB) break; default: WC_PLANE(IC) }
#undef WC_PLANE
#undef WC_ROW
    }
  }
}

// dU[t][0][i] = sum over s of dU[t][s][i], i in [0, n): the parts of the split reduction, added in
// a fixed order.  4 elements per thread; n is a multiple of 4.
__global__ __launch_bounds__(256) void sum_parts_kernel(float* __restrict__ dU, int S, long long n, long long total4) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total4) return;
  const long long n4 = n / 4;
  const long long t = idx / n4, i = (idx % n4) * 4;
  float* base = dU + t * S * n + i;
  float4 sum = *reinterpret_cast<const float4*>(base);
  for (int sp = 1; sp < S; ++sp) {
    const float4 v = *reinterpret_cast<const float4*>(base + sp * n);
    sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
  }
  *reinterpret_cast<float4*>(base) = sum;
}

// acc[t][i] = sum over s of dU[t][s][i]: the same sum, written densely (the layout grad_filter_store_kernel reads)
__global__ __launch_bounds__(256) void sum_parts_out_kernel(const float* __restrict__ dU, float* __restrict__ acc, int S,
                                                            long long n, long long total4) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total4) return;
  const long long n4 = n / 4;
  const long long t = idx / n4, i = (idx % n4) * 4;
  const float* base = dU + t * S * n + i;
  float4 sum = *reinterpret_cast<const float4*>(base);
  for (int sp = 1; sp < S; ++sp) {
    const float4 v = *reinterpret_cast<const float4*>(base + sp * n);
    sum.x += v.x; sum.y += v.y; sum.z += v.z; sum.w += v.w;
  }
  *reinterpret_cast<float4*>(acc + t * n + i) = sum;
}

// dw[k][c][tap] through element strides <- acc (taps, K, C)
template <typename T>
__global__ __launch_bounds__(256) void grad_filter_store_kernel(const float* __restrict__ acc, T* __restrict__ dw,
                                                               long long s0, long long s1, long long s2, long long s3,
                                                               long long s4, int K, int C, int kD, int kH, int kW,
                                                               long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int c = (int)(idx % C);
  long long q = idx / C;
  const int k = (int)(q % K);
  const int tap = (int)(q / K);
  const int x2 = tap % kW, x1 = (tap / kW) % kH, x0 = tap / (kW * kH);
  dw[k * s0 + c * s1 + x0 * s2 + x1 * s3 + x2 * s4] = static_cast<T>(acc[idx]);
}

}  // namespace wc

using namespace wc;

namespace {

size_t round256(size_t v) { return (v + 255) / 256 * 256; }

// Parts the reduction over the tiles is split into.  The product's workgroups run in rounds of as many as the chip
// holds at once (two per CU for 128 x 128 tiles, four for 64 x 64: what their LDS stages allow), and a round that is nearly empty costs as much
// as a full one: the most parts that still fit r rounds, for the r with the least work per round-limited workgroup
// (metric shape, 144 tiles: 7 parts = 1008 workgroups in two rounds, where 8 parts made 1152 = three rounds).
int pick_parts(long long tiles, long long rows, bool big_tiles) {
  const long long slots = big_tiles ? 512 : 1024;
  long long best = 1;
  double best_cost = 1e30;
  for (int r = 1; r <= 4; ++r) {
    long long S = slots * r / tiles;
    S = std::max(1ll, std::min(S, std::min(64ll, rows / 256)));
    const double cost = (double)((tiles * S + slots - 1) / slots) / (double)S;
    if (cost < best_cost * (1.0 - 1e-9)) { best = S; best_cost = cost; }
  }
  return (int)best;
}

struct BwdLayout {
  wc_plan plan;
  int out[3], grid[3];
  int Cp, ldm, ldc, chunk, S, Pq;   // Cp: row length of V; ldc: row length of dU (both span the pieces of a stacked plan)
  int ncol;                         // columns of dU that are computed
  wc_plan dm_plan;                  // the plan dM follows: the plan itself, or its one shared tile when stacked
  long long tiles_per_image;
  size_t es;
  size_t v_bytes, dm_bytes, du_bytes, acc_bytes;
  bool one_tap;                     // 1x1 kernel, stride 1, no padding: dw = dy^T x, no transforms
  bool gathered;                    // 2-D stride 2: dw[tap] = dy^T (the pixels of x that tap reads), no transforms
};

// A 2-D layer at stride 2: the transform-domain gradient runs Winograd tiles on the parity phases of x (V and dM
// through memory, few multiplications saved); taken directly, tap (ky, kx) is one transposed product of dy with the
// pixels of x that tap reads, gathered row by row inside the product (fp16 N=32, 128 channels, 112x112, 3x3: 159 us
// in the transform domain).
bool gathered_layout(const wc_conv_desc* d, BwdLayout* L) {
  if (d->ndim != 2 || d->stride != 2 || d->whole_kernel) return false;
  if (d->C % 8 != 0 || d->K % 8 != 0) return false;
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2;
  if (wc_conv_out_dims(&e, L->out, L->grid) != WC_OK) return false;
  const long long P = (long long)d->N * L->out[1] * L->out[2];
  if (P >= (1ll << 31) || (long long)d->N * d->in[1] * d->in[2] >= (1ll << 31)) return false;
  const int taps = d->kernel[1] * d->kernel[2];
  L->gathered = true;
  L->es = d->dtype == WC_F32 ? 4 : 2;
  L->ldm = d->K; L->Cp = d->C; L->ncol = d->C; L->ldc = d->C; L->chunk = d->N;
  L->tiles_per_image = (long long)L->out[1] * L->out[2];
  const int bt = (d->K > 64 && d->C > 64) ? 128 : 64;
  const long long tiles = (long long)taps * ((d->K + bt - 1) / bt) * ((d->C + bt - 1) / bt);
  const long long S = pick_parts(tiles, P, bt == 128);
  L->S = (int)S;
  L->Pq = (int)(((P + S - 1) / S + 31) / 32 * 32);
  L->v_bytes = L->dm_bytes = 0;
  L->du_bytes = round256((size_t)taps * S * d->K * d->C * 4);
  L->acc_bytes = round256((size_t)taps * d->K * d->C * 4);
  return true;
}

// A kernel of one tap at stride 1 without padding: y = x w^T pixel by pixel, so dw (K x C) = sum over the pixels of
// dy (x) x is the transposed product of the two tensors as they lie in memory, rows = pixels; F(m,1) has nothing to
// transform and its dM and V would be copies (fp16 N=64, 64 -> 256 channels, 56x56: 92 us that way).
bool one_tap_layout(const wc_conv_desc* d, BwdLayout* L) {
  if (d->ndim != 2 || d->stride != 1 || d->whole_kernel) return false;
  for (int a = 0; a < 3; ++a)
    if (d->kernel[a] != 1 || d->pad[a] != 0) return false;
  if (d->C % 8 != 0 || d->K % 8 != 0) return false;
  const long long P = (long long)d->N * d->in[1] * d->in[2];
  if (P >= (1ll << 31)) return false;
  L->one_tap = true;
  L->es = d->dtype == WC_F32 ? 4 : 2;
  L->ldm = d->K; L->Cp = d->C; L->ncol = d->C; L->ldc = d->C; L->chunk = d->N;
  L->tiles_per_image = (long long)d->in[1] * d->in[2];
  const int bt = (d->K > 64 && d->C > 64) ? 128 : 64;
  const long long tiles = (long long)((d->K + bt - 1) / bt) * ((d->C + bt - 1) / bt);
  const long long S = pick_parts(tiles, P, bt == 128);
  L->S = (int)S;
  L->Pq = (int)(((P + S - 1) / S + 31) / 32 * 32);
  L->v_bytes = L->dm_bytes = L->acc_bytes = 0;
  L->du_bytes = round256((size_t)S * d->K * d->C * 4);
  return true;
}

int make_bwd_layout(const wc_conv_desc* d, BwdLayout* L) {
  WC_CHECK_ARG(d != nullptr, "null descriptor");
  WC_CHECK_ARG(d->dtype == WC_F32 || d->dtype == WC_F16 || d->dtype == WC_BF16, "dtype %d", d->dtype);
  WC_CHECK_ARG((d->ndim == 2 || d->ndim == 3) && d->N > 0 && d->C > 0 && d->K > 0, "ndim %d, N %d, C %d, K %d", d->ndim, d->N, d->C, d->K);
  L->one_tap = L->gathered = false;
  if (one_tap_layout(d, L)) return WC_OK;
  if (gathered_layout(d, L)) return WC_OK;
  if (d && d->stacked == 2)
    return fail(WC_ERR_UNSUPPORTED, "the weight gradient is not built for plans with a shared transformed input (stacked = 2)");
  int rc = wc_plan_conv(d, &L->plan);
  if (rc) return rc;
  rc = wc_conv_out_dims(d, L->out, L->grid);
  if (rc) return rc;
  if (L->plan.t_total > 0xffff) return fail(WC_ERR_UNSUPPORTED, "plan with %d transform elements is too large", L->plan.t_total);
  const bool stacked = d->stacked && L->plan.n_pieces > 1;
  L->Cp = stacked_row(d, &L->plan);
  L->ldm = wc_padded_channels8(d->K);
  L->ncol = stacked ? L->Cp : d->C;
  L->ldc = wc_padded_channels8(L->ncol);
  L->dm_plan = L->plan;
  if (stacked) {
    // one set of dM for all pieces: the adjoint of the single output transform of the stacked forward pass
    L->dm_plan.n_pieces = 1;
    stacked_taps(&L->plan, L->dm_plan.piece[0].r);
    L->dm_plan.piece[0].t_offset = 0;
  }
  L->es = d->dtype == WC_F32 ? 4 : 2;
  L->tiles_per_image = (long long)L->grid[0] * L->grid[1] * L->grid[2];
  const long long T = L->plan.t_total;
  // images per pass: the two large buffers of one pass stay below about 8 GiB
  const double per_image = (double)T * L->tiles_per_image * (L->Cp + L->ldm) * L->es * 1.1;
  int chunk = d->chunk_images > 0 ? d->chunk_images : (int)(8192.0 * 1024 * 1024 / per_image);
  chunk = std::max(1, std::min(chunk, d->N));
  if (d->chunk_images <= 0 && chunk < d->N) {   // equal passes rather than full ones and a short last one
    const int passes = (d->N + chunk - 1) / chunk;
    chunk = (d->N + passes - 1) / passes;
  }
  L->chunk = chunk;
  const long long Pc = L->tiles_per_image * chunk;
  if (Pc >= (1ll << 31)) return fail(WC_ERR_UNSUPPORTED, "chunk of %d images has too many tiles", chunk);
  // split of the tile axis: whole rounds of resident workgroups, every part >= 256 tiles
  const int bt = (d->K > 64 && L->ncol > 64) ? 128 : 64;
  const long long tiles = T * ((d->K + bt - 1) / bt) * ((L->ncol + bt - 1) / bt);
  const long long S = pick_parts(tiles, Pc, bt == 128);
  L->S = (int)S;
  L->Pq = (int)(((Pc + S - 1) / S + 31) / 32 * 32);
  L->v_bytes = round256((size_t)T * Pc * L->Cp * L->es);
  L->dm_bytes = round256((size_t)T * Pc * L->ldm * L->es);
  L->du_bytes = round256((size_t)T * S * d->K * L->ldc * 4);
  L->acc_bytes = round256((size_t)d->kernel[0] * d->kernel[1] * d->kernel[2] * d->K * d->C * 4);
  return WC_OK;
}

}  // namespace

extern "C" {

int wc_conv_backward_weight_workspace_bytes(const wc_conv_desc* d, size_t* bytes) {
  WC_CHECK_ARG(bytes != nullptr, "wc_conv_backward_weight_workspace_bytes: null output");
  BwdLayout L{};
  int rc = make_bwd_layout(d, &L);
  if (rc) return rc;
  *bytes = L.v_bytes + L.dm_bytes + L.du_bytes + L.acc_bytes;
  return WC_OK;
}

int wc_conv_backward_weight(const wc_conv_desc* d, const void* x, const void* dy, void* dw,
                            const int64_t dw_strides[5], void* workspace, size_t workspace_bytes, void* stream) {
  BwdLayout L{};
  int rc = make_bwd_layout(d, &L);
  if (rc) return rc;
  WC_CHECK_ARG(x && dy && dw && dw_strides, "wc_conv_backward_weight: null pointer");
  if (!workspace) return fail(WC_ERR_WORKSPACE, "wc_conv_backward_weight: null workspace");
  const size_t need = L.v_bytes + L.dm_bytes + L.du_bytes + L.acc_bytes;
  if (workspace_bytes < need)
    return fail(WC_ERR_WORKSPACE, "wc_conv_backward_weight: workspace of %zu bytes, %zu needed", workspace_bytes, need);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return fail(WC_ERR_WORKSPACE, "wc_conv_backward_weight: workspace must be 256-byte aligned");
  hipStream_t s = as_stream(stream);
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  void* V = ws;
  void* dM = ws + L.v_bytes;
  float* dU = reinterpret_cast<float*>(ws + L.v_bytes + L.dm_bytes);
  float* acc = reinterpret_cast<float*>(ws + L.v_bytes + L.dm_bytes + L.du_bytes);
  const int T = L.plan.t_total;
  const size_t x_image = (size_t)d->in[0] * d->in[1] * d->in[2] * d->C * L.es;
  const size_t y_image = (size_t)L.out[0] * L.out[1] * L.out[2] * d->K * L.es;
  const int taps = d->kernel[0] * d->kernel[1] * d->kernel[2];

  if (L.one_tap) {
    const long long P = L.tiles_per_image * d->N;
    rc = batched_gemm_tn(dy, x, dU, 1, P, d->K, d->C, d->K, d->C, d->C, L.S, L.Pq, d->dtype, stream);
    if (rc) return rc;
    if (L.S > 1) {
      const long long n = (long long)d->K * d->C, total4 = n / 4;
      hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)ceil_div_ll(total4, 256)), dim3(256), 0, s, dU, L.S, n, total4);
      WC_CHECK_LAUNCH("sum_parts_kernel");
    }
    acc = dU;
  }
  if (L.gathered) {
    rc = gemm_tn_conv(dy, x, dU, d->N, d->in[1], d->in[2], d->C, d->K, d->kernel[1], d->kernel[2], d->stride, d->pad[1],
                      d->pad[2], L.out[1], L.out[2], L.S, L.Pq, d->dtype, stream);
    if (rc) return rc;
    const long long n = (long long)d->K * d->C, total4 = (long long)taps * n / 4;
    hipLaunchKernelGGL(sum_parts_out_kernel, dim3((unsigned)ceil_div_ll(total4, 256)), dim3(256), 0, s, dU, acc, L.S, n, total4);
    WC_CHECK_LAUNCH("sum_parts_out_kernel");
  }
  for (int b0 = 0; b0 < d->N && !L.one_tap && !L.gathered; b0 += L.chunk) {
    const int n = std::min(L.chunk, d->N - b0);
    const long long P = L.tiles_per_image * n;
    rc = wc_input_transform(d, &L.plan, static_cast<const unsigned char*>(x) + b0 * x_image, n, V, stream);
    if (rc) return rc;
    {
      GradOutArgs a;
      a.dy = static_cast<const unsigned char*>(dy) + b0 * y_image;
      a.dM = dM;
      a.oD = L.out[0]; a.oH = L.out[1]; a.oW = L.out[2]; a.K = d->K; a.ldm = L.ldm;
      a.nD = L.grid[0]; a.nH = L.grid[1]; a.nW = L.grid[2];
      a.P = P;
      const wc_plan& gp = L.dm_plan;
      for (int i = 0; i < 3; ++i) a.m[i] = gp.m[i];
      a.n_pieces = gp.n_pieces;
      for (int i = 0; i < gp.n_pieces; ++i) a.piece[i] = gp.piece[i];
      a.total = (long long)T * P * L.ldm;
      const long long blocks = ceil_div_ll(a.total, 256);
      WC_CHECK_ARG(blocks < (1ll << 31), "wc_conv_backward_weight: problem too large");
      bool small_taps = true;
      for (int i = 0; i < gp.n_pieces; ++i)
        for (int q = 0; q < 3; ++q) small_taps = small_taps && gp.piece[i].r[q] <= 3;
      const int m0 = L.plan.m[0], mo = L.plan.m[1];
      void (*fn)(GradOutArgs) = nullptr;
      long long threads = a.total;
      if (small_taps && L.plan.m[2] == mo && (mo == 2 || mo == 4) && (m0 == 1 || m0 == 2)) {
        // 2 channels per thread when K is even, except for the 144-element tile of the 3-D tile 4
        const int vec = ((m0 == 2 && mo == 4) || d->K % 2) ? 1 : 2;
        threads = P * (L.ldm / vec);
        fn = dispatch_dtype(d->dtype, [&](auto t) -> void (*)(GradOutArgs) {
          using TT = decltype(t);
          if (m0 == 2 && mo == 4) return &grad_output_pieces_kernel<TT, 2, 4, 1>;
          if (vec == 2) {
            if (m0 == 1) return mo == 4 ? &grad_output_pieces_kernel<TT, 1, 4, 2> : &grad_output_pieces_kernel<TT, 1, 2, 2>;
            return &grad_output_pieces_kernel<TT, 2, 2, 2>;
          }
          if (m0 == 1) return mo == 4 ? &grad_output_pieces_kernel<TT, 1, 4, 1> : &grad_output_pieces_kernel<TT, 1, 2, 1>;
          return &grad_output_pieces_kernel<TT, 2, 2, 1>;
        });
      } else {
        fn = dispatch_dtype(d->dtype, [](auto t) -> void (*)(GradOutArgs) {
          return &grad_output_transform_kernel<decltype(t)>;
        });
      }
      const long long nblocks = ceil_div_ll(threads, 256);
      hipLaunchKernelGGL(fn, dim3((unsigned)nblocks), dim3(256), 0, s, a);
      WC_CHECK_LAUNCH("grad_output_transform_kernel");
    }
    // the part length of this pass (the last pass may hold fewer images)
    const int Pq = (int)(((P + L.S - 1) / L.S + 31) / 32 * 32);
    // dU[(t, s)] (K x C, fp32) = sum over the tiles of part s of dM[t][p][.] (x) V[t][p][.]: operands in
    // the storage type (their values already are), products summed in fp32
    rc = batched_gemm_tn(dM, V, dU, T, P, L.ldm, L.Cp, d->K, L.ncol, L.ldc, L.S, Pq, d->dtype, stream);
    if (rc) return rc;
    if (L.S > 1) {
      const long long n = (long long)d->K * L.ldc, total4 = (long long)T * n / 4;
      hipLaunchKernelGGL(sum_parts_kernel, dim3((unsigned)ceil_div_ll(total4, 256)), dim3(256), 0, s, dU, L.S, n, total4);
      WC_CHECK_LAUNCH("sum_parts_kernel");
    }
    rc = grad_filter_transform(d, &L.plan, dU, acc, L.ldc, L.S, b0 == 0, stream);
    if (rc) return rc;
  }
  const long long total = (long long)taps * d->K * d->C;
  dispatch_dtype(d->dtype, [&](auto t) {
    using TT = decltype(t);
    hipLaunchKernelGGL(grad_filter_store_kernel<TT>, dim3((unsigned)ceil_div_ll(total, 256)), dim3(256), 0, s, acc,
                       static_cast<TT*>(dw), (long long)dw_strides[0], (long long)dw_strides[1],
                       (long long)dw_strides[2], (long long)dw_strides[3], (long long)dw_strides[4], d->K, d->C,
                       d->kernel[0], d->kernel[1], d->kernel[2], total);
    return 0;
  });
  WC_CHECK_LAUNCH("grad_filter_store_kernel");
  return WC_OK;
}

}  // extern "C"
