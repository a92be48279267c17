// Device body of the filter transform of one piece with compile-time tile kinds (shared by the kernels of
// filter_transform.hip and by the launch that runs it beside the input transform).
#pragma once
#include "wc_transform.h"

namespace wc {

// G of one kind as an apply_axis matrix (alpha x r)
template <int KIND>
struct MatG {
  static constexpr int rows = Mats<KIND>::alpha;
  static constexpr int cols = Mats<KIND>::r;
  __host__ __device__ static constexpr float get(int i, int j) { return Mats<KIND>::g(i, j); }
  __host__ __device__ static constexpr int first_nz(int i) {
    for (int j = 0; j < cols; ++j)
      if (get(i, j) != 0.f) return j;
    return cols;
  }
};

struct FilterFastArgs {
  const void* w;
  void* U;
  long long s[5];
  int C, Cp, K;
  int tap0[3];
  int step;
  int t_offset;
};

// VEC channels of one k of one piece with compile-time kinds: loads the taps once, transforms in registers
// and writes the alpha^d elements (lanes along c: coalesced rows of U).
// `taps`: how many of the tile's taps per axis the piece really has; the others count as zero (a
// stacked plan transforms every piece with the tile of the longest one).
// DENSE: w is a contiguous (K, C, taps) array, the piece is the whole kernel and C a multiple of VEC, so the
// VEC * taps values of a thread are one contiguous run, read 8 (or 4) bytes at a time.
template <typename T, int K0, int K1, int K2, int VEC = 1, bool DENSE = false>
__device__ __forceinline__ void transform_taps(const T* __restrict__ w, const long long (&s)[5], int k, int c,
                                               int C, const int (&tap0)[3], int step, T* __restrict__ U,
                                               long long plane, const int (&taps)[3]) {
  constexpr int R0 = Mats<K0>::r, R1 = Mats<K1>::r, R2 = Mats<K2>::r;
  constexpr int A0 = Mats<K0>::alpha, A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
  constexpr int R = R0 * R1 * R2;
  float g[R][VEC];
  if constexpr (DENSE && VEC > 1) {
    constexpr int BYTES = VEC * R * (int)sizeof(T);
    constexpr int CH = BYTES % 8 == 0 ? 8 : 4;             // bytes per load
    static_assert(BYTES % CH == 0, "a thread's taps are whole 4-byte words");
    constexpr int EPL = CH / (int)sizeof(T);               // elements per load
    T flat[VEC * R];                                        // [channel][tap]
    if (c < C) {
      const T* wp = w + ((long long)k * C + c) * R;
#pragma unroll
      for (int i = 0; i < BYTES / CH; ++i) {
        const Pack<T, EPL> q = *reinterpret_cast<const Pack<T, EPL>*>(wp + i * EPL);
#pragma unroll
        for (int e = 0; e < EPL; ++e) flat[i * EPL + e] = q.v[e];
      }
    }
#pragma unroll
    for (int j = 0; j < R; ++j)
#pragma unroll
      for (int v = 0; v < VEC; ++v) g[j][v] = c < C ? static_cast<float>(flat[v * R + j]) : 0.f;
  } else {
#pragma unroll
    for (int v = 0; v < VEC; ++v) {
      const bool ok = c + v < C;
      const T* wp = w + k * s[0] + (ok ? c + v : 0) * s[1];
      static_for<0, R0>([&](auto j0_) {
        static_for<0, R1>([&](auto j1_) {
          static_for<0, R2>([&](auto j2_) {
            constexpr int j0 = decltype(j0_)::value, j1 = decltype(j1_)::value, j2 = decltype(j2_)::value;
            const bool real = j0 < taps[0] && j1 < taps[1] && j2 < taps[2];
            const float val = static_cast<float>(wp[(tap0[0] + (real ? j0 : 0) * step) * s[2] +
                                                   (tap0[1] + (real ? j1 : 0) * step) * s[3] +
                                                   (tap0[2] + (real ? j2 : 0) * step) * s[4]]);
            g[(j0 * R1 + j1) * R2 + j2][v] = (ok && real) ? val : 0.f;
          });
        });
      });
    }
  }
  float u2[R0 * R1 * A2][VEC];
  apply_axis<MatG<K2>, 2, R0, R1, R2, VEC>(g, u2);
  float u1[R0 * A1 * A2][VEC];
  apply_axis<MatG<K1>, 1, R0, R1, A2, VEC>(u2, u1);
  float u0[A0 * A1 * A2][VEC];
  apply_axis<MatG<K0>, 0, R0, A1, A2, VEC>(u1, u0);
  static_for<0, A0 * A1 * A2>([&](auto e_) {
    constexpr int e = decltype(e_)::value;
    store_pack<T, VEC>(U + e * plane, u0[e]);
  });
}

// Channels per thread of the single-piece kernel: 8-byte stores for 2-D tiles, 2 channels for the 64 elements of
// F(2,3)^3, one for the 144 of F(2,3) x F(4,3)^2 (registers).
template <typename T, int K0, int K1, int K2>
constexpr int fast_vec() {
  constexpr int elems = Mats<K0>::alpha * Mats<K1>::alpha * Mats<K2>::alpha;
  return elems <= 36 ? 8 / (int)sizeof(T) : elems <= 64 ? 2 : 1;
}

// One thread per (k, VEC channels) of a single-piece plan; idx enumerates them.
template <typename T, int K0, int K1, int K2, bool DENSE, int VEC = fast_vec<T, K0, K1, K2>()>
__device__ __forceinline__ void filter_fast_body(const FilterFastArgs& a, int idx) {
  const int cvecs = a.Cp / VEC;
  if (idx >= a.K * cvecs) return;
  const int c = (idx % cvecs) * VEC, k = idx / cvecs;
  T* U = static_cast<T*>(a.U) + (long long)a.t_offset * a.K * a.Cp + (long long)k * a.Cp + c;
  const int all[3] = {Mats<K0>::r, Mats<K1>::r, Mats<K2>::r};
  transform_taps<T, K0, K1, K2, VEC, DENSE>(static_cast<const T*>(a.w), a.s, k, c, a.C, a.tap0, a.step, U,
                                            (long long)a.K * a.Cp, all);
}

// Host side: the arguments of the single-piece kernel for this plan, the channels per thread of that kernel and
// whether the filter is a contiguous (K, C, taps) array it can read in 8-byte pieces.  False if the plan has no
// compile-time kernel.
bool filter_fast_setup(const wc_conv_desc* d, const wc_plan* plan, const void* w, const int64_t w_strides[5], void* U,
                       FilterFastArgs* f, int* vec, bool* dense);

}  // namespace wc
