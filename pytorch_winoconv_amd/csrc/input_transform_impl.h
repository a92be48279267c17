// Input transform kernel (included by the per-shape translation units).
// Input transform V = (BT_d x BT_h x BT_w) d, channel-last input; one launch per piece, or one
// launch for all pieces of a 2-D DWM plan.
//
// Replaces inputNorm2WinoTransform + inputNorm2WinoCalculation of the reference
// (src/split_kernel.cu:60-120, src/calculation_kernels.cu:763-1522).  Window of tile t,
// element i on one axis: step*(m*t + i) + tap0 - pad, zero outside (split_kernel.cu:78-100).
//
// HBM-bound: each thread owns one tile x VEC consecutive channels (lanes run along C, so a
// wavefront reads and writes contiguous runs), transforms in fp32 registers with compile-time
// tile sizes (no run-time indexed private arrays) and stores each transform-domain element once.
// Workgroup ids are remapped so that one XCD walks a contiguous range of tiles: the halo rows
// and columns shared by neighbouring tiles are then served by that XCD's L2.
#pragma once
#include "wc_transform.h"

namespace wc {

struct InArgs {
  const void* x;
  void* V;
  int D, H, W, C, Cp;
  int nD, nH, nW;
  int base0, base1, base2;   // tap0 - pad per axis
  int step;                  // convolution stride
  long long t_stride;        // P * Cp
  int t_offset;
  int n_cvec;                // Cp / VEC
  long long total;           // P * n_cvec
  int per_xcd;
  int x_bytes;               // bytes of the images one launch covers (kernels that read x through a buffer descriptor)
  // input_transform_kernel only: blockIdx.y enumerates the parity phases of a stride-2 plan whose
  // pieces share one transformed input (depth parity outermost; 1, 1, 0 otherwise): phase
  // (q0, q1, q2) reads from base + q and writes its own q_cols columns of a row of V
  int nq1, nq2, q_cols;
};

// Tile coordinates and channel offset of one thread
struct InWhere {
  int td, th, tw, c;
  long long b, p;
  bool c_ok;
};

// blk: logical workgroup index (after the XCD remap)
__device__ __forceinline__ bool in_decode(const InArgs& a, int blk, int vec, InWhere& w) {
  const long long idx = (long long)blk * 256 + threadIdx.x;
  if (idx >= a.total) return false;
  const int cv = (int)(idx % a.n_cvec);
  w.p = idx / a.n_cvec;
  w.tw = (int)(w.p % a.nW); long long q = w.p / a.nW;
  w.th = (int)(q % a.nH); q /= a.nH;
  w.td = (int)(q % a.nD);
  w.b = q / a.nD;
  w.c = cv * vec;
  w.c_ok = w.c < a.C;
  return true;
}

// One window (tile x VEC channels) of one piece: load, transform, store.
template <typename T, int K0, int K1, int K2, int VEC>
__device__ __forceinline__ void transform_window(const InArgs& a, const InWhere& w, int base0, int base1,
                                                 int base2, int t_offset, int col0 = 0) {
  constexpr int A0 = Mats<K0>::alpha, A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
  constexpr int m0 = Mats<K0>::m, m1 = Mats<K1>::m, m2 = Mats<K2>::m;
  const T* x = static_cast<const T*>(a.x);

  // Every load is issued unconditionally from a clamped address and zeroed afterwards if the
  // window element lies outside the image: the loads of a tile are then all in flight together
  // instead of one per divergent branch.
  float d[A0 * A1 * A2][VEC];
  const int cc = w.c_ok ? w.c : 0;
  static_for<0, A0>([&](auto i0_) {
    constexpr int i0 = decltype(i0_)::value;
    const int z = a.step * (m0 * w.td + i0) + base0;
    const bool z_ok = w.c_ok && (unsigned)z < (unsigned)a.D;
    const int zc = min(max(z, 0), a.D - 1);
    static_for<0, A1>([&](auto i1_) {
      constexpr int i1 = decltype(i1_)::value;
      const int yy = a.step * (m1 * w.th + i1) + base1;
      const bool y_ok = z_ok && (unsigned)yy < (unsigned)a.H;
      const int yc = min(max(yy, 0), a.H - 1);
      const long long row = ((w.b * a.D + zc) * a.H + yc) * a.W;
      static_for<0, A2>([&](auto i2_) {
        constexpr int i2 = decltype(i2_)::value;
        constexpr int e = (i0 * A1 + i1) * A2 + i2;
        const int xx = a.step * (m2 * w.tw + i2) + base2;
        const bool ok = y_ok && (unsigned)xx < (unsigned)a.W;
        const int xc = min(max(xx, 0), a.W - 1);
        load_pack<T, VEC>(x + (row + xc) * a.C + cc, d[e]);
#pragma unroll
        for (int v = 0; v < VEC; ++v) d[e][v] = ok ? d[e][v] : 0.f;
      });
    });
  });

  // W, then H, then D (reference order: matrix_conv3d.py:162-163)
  float t2[A0 * A1 * A2][VEC];
  apply_axis<MatSel<K2, false>, 2, A0, A1, A2, VEC>(d, t2);
  apply_axis<MatSel<K1, false>, 1, A0, A1, A2, VEC>(t2, d);
  if constexpr (A0 > 1) {
    apply_axis<MatSel<K0, false>, 0, A0, A1, A2, VEC>(d, t2);
  }
  T* V = static_cast<T*>(a.V) + (long long)t_offset * a.t_stride + w.p * a.Cp + col0 + w.c;
  static_for<0, A0 * A1 * A2>([&](auto e_) {
    constexpr int e = decltype(e_)::value;
    if constexpr (A0 > 1) store_pack<T, VEC>(V + e * a.t_stride, t2[e]);
    else store_pack<T, VEC>(V + e * a.t_stride, d[e]);
  });
}

template <typename T, int K0, int K1, int K2, int VEC>
__global__ __launch_bounds__(256) void input_transform_kernel(InArgs a) {
  InWhere w;
  if (!in_decode(a, xcd_remap(blockIdx.x, a.per_xcd), VEC, w)) return;
  const int ph = blockIdx.y;
  const int q2 = ph % a.nq2, q1 = (ph / a.nq2) % a.nq1, q0 = ph / (a.nq2 * a.nq1);
  transform_window<T, K0, K1, K2, VEC>(a, w, a.base0 + q0, a.base1 + q1, a.base2 + q2, a.t_offset, ph * a.q_cols);
}

// All pieces of a 2-D DWM plan in one launch: a thread transforms the windows of its tile piece
// after piece, so the overlapping windows of the pieces are read from HBM once and then served
// by the caches (a launch per piece reads the whole input once per piece; giving each piece its
// own workgroup next to the others on one XCD measured 8-16 % slower than this loop).
struct InPiecesArgs {
  InArgs o;                       // base0/1/2 and t_offset unused
  int n_pieces;
  int pad1, pad2;
  int col_step;                   // columns of V between two pieces (stacked plans), else 0
  int info[WC_MAX_PIECES];        // t_offset | tap0_h << 16 | tap0_w << 20 | r_h << 24 | r_w << 28
};
using InPiecesKernel = void (*)(InPiecesArgs);
InPiecesKernel pick_in_2d_pieces(int dtype, int m, int vec);     // nullptr if the combination is not built
InPiecesKernel pick_in_2d_stacked(int dtype, int m, int vec);    // stacked plans: one thread per (tile, piece, channels)

using InKernel = void (*)(InArgs);

template <typename T, int VEC, int K0, int K1, int K2>
constexpr InKernel in_kernel() { return &input_transform_kernel<T, K0, K1, K2, VEC>; }

// Kernel look-up, one translation unit per depth kind so that they compile in parallel.
InKernel pick_in_2d(int dtype, int k1, int k2, int vec);          // depth kind KIND_11 (2-D problems)
InKernel pick_in_2d_m4(int dtype, int k1, int k2, int vec);       // ... with output tile 4, vec 2 or 1
InKernel pick_in_2d_whole(int dtype, int k1, int k2, int vec);    // ... whole-kernel tiles F(2,4..7), vec 2 or 1
InKernel pick_in_3d_21(int dtype, int k1, int k2, int vec);       // depth kind KIND_21, vec 2 or 1
InKernel pick_in_3d_22(int dtype, int k1, int k2, int vec);
InKernel pick_in_3d_23(int dtype, int k1, int k2, int vec);
InKernel pick_in_columns(int dtype, int vec);                      // kinds F(2,3), F(2,3), F(1,1); vec 8, 4, 2 or 1
struct FilterFastArgs;
// channels per thread of the filter part of that launch
constexpr int in_filter_vec(int elem_bytes, int k1) { return elem_bytes == 4 && k1 == KIND_43 ? 1 : 8 / elem_bytes; }
using InFilterKernel = void (*)(InArgs, FilterFastArgs, int);
InFilterKernel pick_in_filter_2d(int dtype, int k1, int k2, int vec);   // 3x3 kernels, tile 2 or 4, with the filter transform in the same launch; nullptr otherwise
InKernel pick_in_3d_planes(int dtype, int vec);                   // tile 2 x 4 x 4 of a 3x3x3 kernel, plane by plane, vec 2 or 1

}  // namespace wc
