// Shared host/device helpers for the gfx950 Winograd engine.
#pragma once
#include <hip/hip_runtime.h>
#include <cstdint>
#include <cstdio>
#include <cstdarg>
#include <type_traits>
#include "../../include/winoconv.h"

namespace wc {

// ---- error reporting (thread-local message behind wc_last_error) -------------------------
void set_error(const char* fmt, ...);
int fail(int code, const char* fmt, ...);

#define WC_CHECK_ARG(cond, ...) \
  do { if (!(cond)) return ::wc::fail(WC_ERR_BAD_ARG, __VA_ARGS__); } while (0)
#define WC_CHECK_HIP(expr)                                                               \
  do { hipError_t e_ = (expr);                                                           \
       if (e_ != hipSuccess)                                                             \
         return ::wc::fail(WC_ERR_HIP, "%s failed: %s", #expr, hipGetErrorString(e_));   \
  } while (0)
#define WC_CHECK_LAUNCH(name)                                                            \
  do { hipError_t e_ = hipGetLastError();                                                \
       if (e_ != hipSuccess)                                                             \
         return ::wc::fail(WC_ERR_HIP, "launch of %s failed: %s", name, hipGetErrorString(e_)); \
  } while (0)

// hipFuncSetAttribute(MaxDynamicSharedMemorySize) once per (device, kernel) for kernels above 64 KB of LDS
int ensure_dynamic_lds(const void* fn, size_t bytes);
// what wc_test_gemm_override last set: tile shape forced on wc_batched_gemm (-1: none) and the
// choice between the two shifted-operand kernels (1: by size)
int test_gemm_config();
int test_gemm_rows();

inline hipStream_t as_stream(void* s) { return reinterpret_cast<hipStream_t>(s); }
inline int ceil_div(int a, int b) { return (a + b - 1) / b; }
inline long long ceil_div_ll(long long a, long long b) { return (a + b - 1) / b; }

// ---- compile-time loops ---------------------------------------------------------------------
template <int I> using ic = std::integral_constant<int, I>;

template <int Begin, int End, typename F>
__host__ __device__ __forceinline__ void static_for(F&& f) {
  if constexpr (Begin < End) {
    f(ic<Begin>{});
    static_for<Begin + 1, End>(static_cast<F&&>(f));
  }
}

// ---- packed element vectors -------------------------------------------------------------------
template <typename T, int N>
struct alignas(sizeof(T) * N) Pack {
  T v[N];
};

using half_t = _Float16;
using bf16_t = __bf16;

// f(T{}) with the storage type that `dtype` (a wc_dtype) names
template <typename F>
inline auto dispatch_dtype(int dtype, F&& f) {
  switch (dtype) {
    case WC_F16: return f(half_t{});
    case WC_BF16: return f(bf16_t{});
    default: return f(float{});
  }
}

// Taps per axis of the tile that the pieces of a stacked plan share.
inline void stacked_taps(const wc_plan* plan, int rp[3]) {
  rp[0] = rp[1] = rp[2] = 1;
  for (int s = 0; s < plan->n_pieces; ++s)
    for (int q = 0; q < 3; ++q)
      if (plan->piece[s].r[q] > rp[q]) rp[q] = plan->piece[s].r[q];
}
// Row length of U and V in elements: the pieces of a stacked plan lie side by side.
inline int stacked_row(const wc_conv_desc* d, const wc_plan* plan) {
  return wc_padded_channels(d->C) * (d->stacked ? plan->n_pieces : 1);
}

// Plans with stacked == 2: the pieces start at multiples of the output tile m (2, or 3 in 2-D) and use one tile
// F(m, m or less) per axis, so the transformed input of the piece that starts at tap (m a, m b) is that of the first piece
// a tile rows and b tiles further on.  V then holds one piece (row length Cp) over a tile grid
// extended by the largest shifts (wc_conv_out_dims reports that grid), followed by `tail` rows that
// only the products of the extension tiles read; the batched GEMM reads piece (a, b) of tile row p
// at row p + a * grid_w + b (3-D: the depth axis likewise, whole planes of the grid further on).
// At stride 2 the taps of each axis are first separated by parity (y[o] = sum_q sum_j x[2 (o + j) + q - pad] w[2 j + q]):
// the even and the odd samples of x are the "phases" of a stride-1 problem whose kernel has ceil(k / 2) taps per
// axis and 2^d times the channels.  A row of V then holds the phases side by side (depth parity outermost), and
// the pieces are (position, phase) pairs, the phases of one position next to each other along the rows of U.
inline bool shared_input(const wc_conv_desc* d, const wc_plan* plan) { return d->stacked == 2 && plan->n_pieces > 1; }
inline int shared_taps(const wc_conv_desc* d, int axis) {
  return d->stride == 2 ? (d->kernel[axis] + 1) / 2 : d->kernel[axis];
}
inline int shared_phases(const wc_conv_desc* d, int axis) { return d->stride == 2 && d->kernel[axis] >= 2 ? 2 : 1; }
inline int shared_phases(const wc_conv_desc* d) { return shared_phases(d, 0) * shared_phases(d, 1) * shared_phases(d, 2); }
inline int v_row(const wc_conv_desc* d, const wc_plan* plan) {
  return shared_input(d, plan) ? wc_padded_channels(d->C) * shared_phases(d) : stacked_row(d, plan);
}
struct SharedShift {          // pieces (a, b, c) of the depth, height and width axes; tiles (d, h, w) of the extended grid
  int n_run, n_runs, n_planes;  // pieces per axis: width, height, depth
  int run_rows, plane_rows;     // tile rows of V between two tiles that are neighbours in height / in depth
  int tail;                     // rows beyond the grid that the shifted reads of its last tiles reach
};
inline SharedShift shared_shift(const wc_conv_desc* d, const int grid[3]) {
  SharedShift s;
  const int len = d->m;                           // taps per piece = output tile (3 only in 2-D: one depth piece)
  s.n_run = (shared_taps(d, 2) + len - 1) / len;
  s.n_runs = (shared_taps(d, 1) + len - 1) / len;
  s.n_planes = (shared_taps(d, 0) + len - 1) / len;
  s.run_rows = grid[2];
  s.plane_rows = grid[1] * grid[2];
  s.tail = (s.n_planes - 1) * s.plane_rows + (s.n_runs - 1) * s.run_rows + s.n_run - 1;
  return s;
}
// M[t] (P x K, row stride ldm) = sum over pieces (a, b, c) of V[t][p + a plane_rows + b run_rows + c][.] x
// U[t][k][((a n_runs + b) n_run + c) Cp + .]; V (T, P + tail, Cp), U (T, K, n_pieces Cp); 16-bit types (gemm.hip)
int batched_gemm_shifted(const void* V, const void* U, void* M, int T, int P, int Cp, SharedShift sh, int K, int ldm,
                         int dtype, void* stream);

// 3-D F(2,3)^3 plans with the width axis inside the product: transforms along depth and height only, over the pixel
// columns of the padded image (columns_width per tile row); V (16, P + 2, Cp), U (64, K, Cp) -> Uw (16, K, 3 Cp)
// (gemm.hip), the product by batched_gemm_shifted with one run of three pieces, M (16, P, ldm)
int columns_width(const wc_conv_desc* d);
int input_transform_columns(const wc_conv_desc* d, const void* x, int n_images, void* V, void* stream);
int fold_filter_w(const void* U, void* Uw, int K, int Cp, int dtype, void* stream);
int output_transform_columns(const wc_conv_desc* d, const void* M, const void* bias, int n_images, void* y, void* stream);
// wc_batched_gemm on persistent 256 x 256 tiles fed by LDS-DMA (gemm_persistent.hip): 16-bit types, K a multiple of 256
bool gemm_persistent_fits(int T, int P, int Cp, int K, int dtype);
bool gemm_persistent_deferred_fits(int P, int Cp, int K, int ldm);      // ... with a tile written out during the next tile's first steps
int gemm_persistent(const void* V, const void* U, void* M, int T, int P, int Cp, int K, int ldm, int dtype, bool deferred, void* stream);
// The same product on tiles of 512 x 128 fed by LDS-DMA (gemm_rows_dma.hip): runs of 2 to 5 pieces
bool gemm_rows_dma_fits(SharedShift sh, int P, int Cp, int K, int dtype);
// ... with a tile's results written out during the first steps of the workgroup's next tile: tiles of enough steps
bool gemm_rows_dma_deferred_fits(SharedShift sh, int P, int Cp, int ldm);
int gemm_rows_dma(const void* V, const void* U, void* M, int T, int P, int Cp, SharedShift sh, int K, int ldm, int dtype,
                  bool deferred, void* stream);

// Input transform of single-piece 2-D plans at stride 1 that reads channel-first x (input_transform_2d_nchw.hip):
// whether the plan is in its range, and the launch.
bool input_transform_nchw_fits(const wc_conv_desc* d, const wc_plan* plan);
int input_transform_nchw(const wc_conv_desc* d, const wc_plan* plan, const void* x, int n_images, void* V, void* stream);
// src (n, R, Q) -> dst (n, Q, R), elements of 2 or 4 bytes (layout_copy.hip)
int transpose_images(const void* src, void* dst, long long n, long long R, long long Q, int elem_size, void* stream);

// Direct form (wc_conv_desc.direct; direct_conv.hip, gemm.hip): whether a problem is in its range, the copy of the
// filter to U (K, kh, kw, C), and the product that reads x itself.
bool direct_conv_fits(const wc_conv_desc* d);
int direct_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream);
int direct_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y, void* stream);
size_t direct_u_elems(const wc_conv_desc* d);     // elements of the direct form's U
// Strided first layers (direct_first.hip): at most 4 input channels, stride 2, kernels of 3, 5 or 7 rows and at most 8
// columns, 16-bit types.  U is (K, kh, 8 taps, 4 channels), zero where the filter has no tap or channel.
bool direct_first_fits(const wc_conv_desc* d);
size_t direct_first_u_elems(const wc_conv_desc* d);
int direct_first_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream);
int direct_first_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y,
                      int oH, int oW, void* stream);
// 3-D first layers (direct_first3d.hip): at most 4 input channels, a 3x3x3 kernel (rows of at most 4 taps) at stride 1,
// 16-bit types; U is (K, 9, 4, 4)
bool direct_first3d_fits(const wc_conv_desc* d);
size_t direct_first3d_u_elems(const wc_conv_desc* d);
int direct_first3d_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream);
int direct_first3d_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y,
                        const int out[3], void* stream);
// o_step > 0: row (b, oy, ox) of the result goes to pixel (o_step oy + o_y0, o_step ox + o_x0) of image b of an
// (o_H, o_W) tensor instead of to row b oH oW + oy oW + ox
int gemm_direct_conv(const void* x, const void* U, const void* bias, void* y, int N, int H, int W, int C, int K,
                     int kh, int kw, int stride, int pad_h, int pad_w, int oH, int oW, int dtype, void* stream,
                     int o_step = 0, int o_y0 = 0, int o_x0 = 0, int o_H = 0, int o_W = 0);

// The direct form with one operand tile per kernel row (direct_rows.hip; 16-bit types, kernel rows of 4 to 8 taps, stride
// 1 or 2): whether a problem is in its range (the input rows that 256 consecutive output pixels read, with their
// padding, must fit a stage of kDirectRowsPixels pixels), and the launch, with the arguments of gemm_direct_conv.
constexpr int kDirectRowsPixels = 768;
bool direct_rows_fits(int N, int C, int K, int kw, int stride, int oH, int oW, int dtype);
int direct_rows_conv(const void* x, const void* U, const void* bias, void* y, int N, int H, int W, int C, int K, int kh,
                     int kw, int stride, int pad_h, int pad_w, int oH, int oW, int dtype, void* stream, int o_step,
                     int o_y0, int o_x0, int o_H, int o_W);

// Number of XCDs (L2 domains) a launch is spread over round-robin by workgroup id.
constexpr int kXcds = 8;
constexpr int kCus = 256;                  // compute units of an MI355X

// Maps the hardware workgroup id to a logical one so that each XCD owns one contiguous
// range of logical ids (neighbouring tiles then share that XCD's L2).  `per_xcd` is
// ceil(n_logical / 8); the launch uses 8 * per_xcd workgroups, ids >= n_logical idle.
__device__ __forceinline__ int xcd_remap(int hw_id, int per_xcd) {
  return (hw_id % kXcds) * per_xcd + hw_id / kXcds;
}

// acc (taps, K, C) (+)= G^T dU G per piece of the plan; dU (T, S, K, ldc) with the parts already
// summed into part 0; `first` overwrites acc instead of adding (backward_filter.hip).
// wc_input_transform and wc_filter_transform of one call: one launch where a kernel holds both (single-piece 2-D
// plans of 3x3 kernels with a dense filter), two launches otherwise
int input_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const void* x, int n_images, void* V,
                           const void* w, const int64_t w_strides[5], void* U, void* stream);
int grad_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const float* dU, float* acc, int ldc, int S,
                          bool first, void* stream);

// D[t][s] (na x nb, fp32, row stride ldd) = sum over rows p in [s Pq, (s + 1) Pq) of
// A[t][p][.] (x) B[t][p][.], operands (T, P, ld) of storage type `dtype` (gemm_tn.hip).
int batched_gemm_tn(const void* A, const void* B, float* D, int T, long long P, int lda, int ldb, int na, int nb,
                    int ldd, int S, int Pq, int dtype, void* stream);
// The weight gradient of a 2-D convolution taken directly: dW[(ky, kx)][s] (K x C) = sum over the output pixels of
// part s of dy (x) the pixel of x that tap reads (gemm_tn.hip)
int gemm_tn_conv(const void* dy, const void* x, float* D, int N, int H, int W, int C, int K, int kh, int kw, int stride,
                 int pad_h, int pad_w, int oH, int oW, int S, int Pq, int dtype, void* stream);

// One-kernel F(2x2, 3x3) forward pass for thin 16-bit layers (conv_thin.hip): whether the problem
// with this single-piece plan is in its range, and the launch.  U (16, K, Cp) from wc_filter_transform.
bool thin_conv_fits(const wc_conv_desc* d, const wc_plan* plan);
int thin_conv_forward(const wc_conv_desc* d, const wc_plan* plan, const void* x, const void* U, const void* bias,
                      void* y, void* stream);

}  // namespace wc
