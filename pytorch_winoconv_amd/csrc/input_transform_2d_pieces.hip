// Input transform of every piece of a 2-D DWM plan (pieces of 1..3 taps per axis) in one launch.
#include "input_transform_impl.h"

namespace wc {

template <typename T, int MO, int VEC>
__global__ __launch_bounds__(256) void input_transform_pieces_kernel(InPiecesArgs g) {
  const InArgs& a = g.o;
  InWhere w;
  if (!in_decode(a, xcd_remap(blockIdx.x, a.per_xcd), VEC, w)) return;
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;
  for (int s = 0; s < g.n_pieces; ++s) {
    const int info = g.info[s];
    const int t_offset = info & 0xffff;
    const int base1 = ((info >> 16) & 15) - g.pad1, base2 = ((info >> 20) & 15) - g.pad2;
    const int r1 = (info >> 24) & 15, r2 = (info >> 28) & 15;
#define WC_BODY(K1, K2) transform_window<T, KIND_11, K1, K2, VEC>(a, w, 0, base1, base2, t_offset, s * g.col_step)
#define WC_ROW(K1) \
  switch (r2) { case 1: WC_BODY(K1, KA); break; case 2: WC_BODY(K1, KB); break; default: WC_BODY(K1, KC); }
    switch (r1) { case 1: WC_ROW(KA) break; case 2: WC_ROW(KB) break; default: WC_ROW(KC) }
#undef WC_ROW
#undef WC_BODY
  }
}

// Stacked plans (every piece transformed with the same tile, the pieces side by side along the rows
// of V): one thread per (tile, piece, VEC channels), the piece next to the channels in the thread
// index, so that neighbouring wavefronts write neighbouring columns of one row of V.
template <typename T, int MO, int VEC>
__global__ __launch_bounds__(256) void input_transform_stacked_kernel(InPiecesArgs g) {
  const InArgs& a = g.o;
  const long long idx = (long long)xcd_remap(blockIdx.x, a.per_xcd) * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int cols = g.n_pieces * a.n_cvec;               // channel groups of one row of V
  const int col = (int)(idx % cols);
  const int s = col / a.n_cvec;
  InWhere w;
  w.p = idx / cols;
  w.tw = (int)(w.p % a.nW); long long q = w.p / a.nW;
  w.th = (int)(q % a.nH); q /= a.nH;
  w.td = 0;
  w.b = q;
  w.c = (col % a.n_cvec) * VEC;
  w.c_ok = w.c < a.C;
  constexpr int KA = MO == 4 ? KIND_41 : KIND_21, KB = MO == 4 ? KIND_42 : KIND_22, KC = MO == 4 ? KIND_43 : KIND_23;
  const int info = g.info[s];
  const int base1 = ((info >> 16) & 15) - g.pad1, base2 = ((info >> 20) & 15) - g.pad2;
  const int r1 = (info >> 24) & 15, r2 = (info >> 28) & 15;      // the shared tile: the same for every piece
#define WC_BODY(K1, K2) transform_window<T, KIND_11, K1, K2, VEC>(a, w, 0, base1, base2, 0, s * g.col_step)
#define WC_ROW(K1) \
  switch (r2) { case 1: WC_BODY(K1, KA); break; case 2: WC_BODY(K1, KB); break; default: WC_BODY(K1, KC); }
  switch (r1) { case 1: WC_ROW(KA) break; case 2: WC_ROW(KB) break; default: WC_ROW(KC) }
#undef WC_ROW
#undef WC_BODY
}

template <typename T>
static InPiecesKernel pick_stacked(int m, int vec) {
  if (m == 4) return vec == 2 ? &input_transform_stacked_kernel<T, 4, 2> : vec == 1 ? &input_transform_stacked_kernel<T, 4, 1> : nullptr;
  if (vec == 8 && sizeof(T) == 2) return &input_transform_stacked_kernel<T, 2, 8>;
  if (vec == 4) return &input_transform_stacked_kernel<T, 2, 4>;
  if (vec == 2) return &input_transform_stacked_kernel<T, 2, 2>;
  return vec == 1 ? &input_transform_stacked_kernel<T, 2, 1> : nullptr;
}

InPiecesKernel pick_in_2d_stacked(int dtype, int m, int vec) {
  return dispatch_dtype(dtype, [&](auto t) { return pick_stacked<decltype(t)>(m, vec); });
}

template <typename T>
static InPiecesKernel pick(int m, int vec) {
  if (m == 4) return vec == 2 ? &input_transform_pieces_kernel<T, 4, 2> : vec == 1 ? &input_transform_pieces_kernel<T, 4, 1> : nullptr;
  if (vec == 8 && sizeof(T) == 2) return &input_transform_pieces_kernel<T, 2, 8>;
  if (vec == 4) return &input_transform_pieces_kernel<T, 2, 4>;
  if (vec == 2) return &input_transform_pieces_kernel<T, 2, 2>;
  return vec == 1 ? &input_transform_pieces_kernel<T, 2, 1> : nullptr;
}

InPiecesKernel pick_in_2d_pieces(int dtype, int m, int vec) {
  return dispatch_dtype(dtype, [&](auto t) { return pick<decltype(t)>(m, vec); });
}

}  // namespace wc
