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

// VEC consecutive elements through one buffer load: the buffer descriptor carries the base and
// the size of the input, the per-lane address is one 32-bit offset (half the registers of a 64-bit
// pointer per load), and an offset beyond the size - which is how a window element outside the
// image is encoded - reads as zero in hardware, so no select is needed afterwards.
template <typename T, int VEC>
__device__ __forceinline__ Pack<T, VEC> buffer_load_pack(__amdgpu_buffer_rsrc_t rsrc, unsigned off) {
  if constexpr (sizeof(T) * VEC == 2) {
    const unsigned short raw = __builtin_amdgcn_raw_buffer_load_b16(rsrc, off, 0, 0);
    return __builtin_bit_cast(Pack<T, VEC>, raw);
  } else if constexpr (sizeof(T) * VEC == 4) {
    const unsigned raw = __builtin_amdgcn_raw_buffer_load_b32(rsrc, off, 0, 0);
    return __builtin_bit_cast(Pack<T, VEC>, raw);
  } else if constexpr (sizeof(T) * VEC == 8) {
    typedef unsigned u2 __attribute__((ext_vector_type(2)));
    const u2 raw = __builtin_amdgcn_raw_buffer_load_b64(rsrc, off, 0, 0);
    return __builtin_bit_cast(Pack<T, VEC>, raw);
  } else {
    static_assert(sizeof(T) * VEC == 16, "buffer_load_pack: 2, 4, 8 or 16 bytes per lane");
    typedef unsigned u4 __attribute__((ext_vector_type(4)));
    const u4 raw = __builtin_amdgcn_raw_buffer_load_b128(rsrc, off, 0, 0);
    return __builtin_bit_cast(Pack<T, VEC>, raw);
  }
}

constexpr unsigned kOutside = 0x80000000u;   // >= the descriptor's size (the host keeps it below 2 GiB)

// Division of 0 <= n < 2^31 by a divisor fixed on the host: q = (n * mul) >> (31 + shift) with
// shift = ceil(log2 d) and mul = floor(2^(31 + shift) / d) + 1 (exact: the excess of mul * d over
// 2^(31 + shift) is at most d <= 2^shift, so n times it stays below 2^(31 + shift)).
struct FastDiv {
  unsigned mul, shift;
};
inline FastDiv make_fast_div(int d) {
  unsigned s = 0;
  while ((1ll << s) < d) ++s;
  return FastDiv{(unsigned)((1ull << (31 + s)) / (unsigned)d + 1), s};
}
__device__ __forceinline__ int fast_div(int n, FastDiv f) {
  return (int)(((unsigned long long)(unsigned)n * f.mul) >> (31 + f.shift));
}

}  // namespace wc
