// Register-resident separable transforms shared by the input and output transform kernels.
#pragma once
#include "wc_common.h"
#include "wc_tables.h"

namespace wc {

template <int KIND, bool IS_AT>
struct MatSel {
  static constexpr int rows = IS_AT ? Mats<KIND>::m : Mats<KIND>::alpha;
  static constexpr int cols = Mats<KIND>::alpha;
  __host__ __device__ static constexpr float get(int i, int j) {
    return IS_AT ? Mats<KIND>::at(i, j) : Mats<KIND>::bt(i, j);
  }
  // first column with a non-zero coefficient in row i
  __host__ __device__ static constexpr int first_nz(int i) {
    for (int j = 0; j < cols; ++j)
      if (get(i, j) != 0.f) return j;
    return cols;
  }
};

// out = Mat applied along AXIS of the N0 x N1 x N2 block `in`; every index is a compile-time
// constant, zero coefficients are skipped and +-1 coefficients become plain adds.
template <typename MS, int AXIS, int N0, int N1, int N2, int VEC>
__device__ __forceinline__ void apply_axis(
    const float (&in)[N0 * N1 * N2][VEC],
    float (&out)[(AXIS == 0 ? MS::rows : N0) * (AXIS == 1 ? MS::rows : N1) * (AXIS == 2 ? MS::rows : N2)][VEC]) {
  constexpr int O0 = AXIS == 0 ? MS::rows : N0;
  constexpr int O1 = AXIS == 1 ? MS::rows : N1;
  constexpr int O2 = AXIS == 2 ? MS::rows : N2;
  static_assert(MS::cols == (AXIS == 0 ? N0 : AXIS == 1 ? N1 : N2), "axis extent mismatch");
  static_for<0, O0>([&](auto o0_) {
    static_for<0, O1>([&](auto o1_) {
      static_for<0, O2>([&](auto o2_) {
        constexpr int o0 = decltype(o0_)::value, o1 = decltype(o1_)::value, o2 = decltype(o2_)::value;
        constexpr int row = AXIS == 0 ? o0 : AXIS == 1 ? o1 : o2;
        constexpr int first = MS::first_nz(row);
        float acc[VEC];
        static_for<0, MS::cols>([&](auto j_) {
          constexpr int j = decltype(j_)::value;
          constexpr float c = MS::get(row, j);
          if constexpr (c != 0.f) {
            constexpr int i0 = AXIS == 0 ? j : o0, i1 = AXIS == 1 ? j : o1, i2 = AXIS == 2 ? j : o2;
            constexpr int idx = (i0 * N1 + i1) * N2 + i2;
#pragma unroll
            for (int v = 0; v < VEC; ++v) {
              if constexpr (j == first) acc[v] = c * in[idx][v];
              else acc[v] = __builtin_fmaf(c, in[idx][v], acc[v]);
            }
          }
        });
#pragma unroll
        for (int v = 0; v < VEC; ++v) out[(o0 * O1 + o1) * O2 + o2][v] = acc[v];
      });
    });
  });
}

template <typename T, int VEC>
__device__ __forceinline__ void load_pack(const T* p, float (&dst)[VEC]) {
  const Pack<T, VEC> v = *reinterpret_cast<const Pack<T, VEC>*>(p);
#pragma unroll
  for (int i = 0; i < VEC; ++i) dst[i] = static_cast<float>(v.v[i]);
}

template <typename T, int VEC>
__device__ __forceinline__ void store_pack(T* p, const float (&src)[VEC]) {
  Pack<T, VEC> v;
#pragma unroll
  for (int i = 0; i < VEC; ++i) v.v[i] = static_cast<T>(src[i]);
  *reinterpret_cast<Pack<T, VEC>*>(p) = v;
}

}  // namespace wc
