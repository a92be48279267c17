// Input transform of a 3x3x3 kernel for the tile 2 x 4 x 4, one depth plane at a time: F(2,3)
// along depth, F(4,3) along height and width (4 x 6 x 6 = 144 elements per channel; the plane
// kind is a template parameter).
//
// The depth pass of F(2,3) only adds or subtracts two input planes
//   o0 = p0 - p2,  o1 = p1 + p2,  o2 = p2 - p1,  o3 = p1 - p3      (BT of matrix_conv.py:27-30)
// so it is done first on two planes at a time (kept in storage precision until combined),
// and each resulting plane goes through the height / width passes and is stored at once.  Plane p1
// is read twice (the second time from cache).
#include "input_transform_impl.h"

namespace wc {

// One plane in storage precision (a 16-bit pair stays packed in one register until it is used).
// KP: kind of the plane axes, A x A elements, output tile MP.
template <typename T, int KP, int VEC>
__device__ __forceinline__ void load_plane(const InArgs& a, __amdgpu_buffer_rsrc_t rsrc, const InWhere& w, int i0,
                                           Pack<T, VEC> (&d)[Mats<KP>::alpha * Mats<KP>::alpha]) {
  constexpr int A = Mats<KP>::alpha, MP = Mats<KP>::m;
  const int cc = w.c_ok ? w.c : 0;
  const int z = 2 * w.td + i0 + a.base0;
  const bool z_ok = w.c_ok && (unsigned)z < (unsigned)a.D;
  static_for<0, A>([&](auto i1_) {
    constexpr int i1 = decltype(i1_)::value;
    const int yy = MP * w.th + i1 + a.base1;
    const bool y_ok = z_ok && (unsigned)yy < (unsigned)a.H;
    const unsigned row = (((unsigned)w.b * a.D + z) * a.H + yy) * a.W;
    static_for<0, A>([&](auto i2_) {
      constexpr int i2 = decltype(i2_)::value;
      const int xx = MP * w.tw + i2 + a.base2;
      const bool ok = y_ok && (unsigned)xx < (unsigned)a.W;
      const unsigned off = ok ? ((row + xx) * a.C + cc) * (unsigned)sizeof(T) : kOutside;
      d[i1 * A + i2] = buffer_load_pack<T, VEC>(rsrc, off);
    });
  });
}

// One output depth plane: o = sp * p + sq * q (fp32), width pass row by row as the rows are
// combined, height pass column by column with each result stored at once - the fp32 copy of the
// combined plane never exists as a whole.
template <typename T, int KP, int VEC>
__device__ __forceinline__ void emit_plane(const InArgs& a, const InWhere& w, int i0,
                                           const Pack<T, VEC> (&p)[Mats<KP>::alpha * Mats<KP>::alpha],
                                           const Pack<T, VEC> (&q)[Mats<KP>::alpha * Mats<KP>::alpha], float sp, float sq) {
  using BT = MatSel<KP, false>;
  constexpr int A = Mats<KP>::alpha;
  float t[A * A][VEC];
  static_for<0, A>([&](auto r_) {
    constexpr int r = decltype(r_)::value;
    float in[A][VEC];
#pragma unroll
    for (int i = 0; i < A; ++i)
#pragma unroll
      for (int v = 0; v < VEC; ++v)
        in[i][v] = sp * static_cast<float>(p[r * A + i].v[v]) + sq * static_cast<float>(q[r * A + i].v[v]);
    static_for<0, A>([&](auto j_) {
      constexpr int j = decltype(j_)::value;
      constexpr int first = BT::first_nz(j);
      static_for<0, A>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        constexpr float c = BT::get(j, i);
        if constexpr (c != 0.f) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            if constexpr (i == first) t[r * A + j][v] = c * in[i][v];
            else t[r * A + j][v] = __builtin_fmaf(c, in[i][v], t[r * A + j][v]);
          }
        }
      });
    });
  });
  T* V = static_cast<T*>(a.V) + (long long)(a.t_offset + i0 * A * A) * a.t_stride + w.p * a.Cp + w.c;
  static_for<0, A>([&](auto j_) {           // column j of the plane
    constexpr int j = decltype(j_)::value;
    static_for<0, A>([&](auto o_) {         // output row o
      constexpr int o = decltype(o_)::value;
      constexpr int first = BT::first_nz(o);
      float acc[VEC];
      static_for<0, A>([&](auto i_) {
        constexpr int i = decltype(i_)::value;
        constexpr float c = BT::get(o, i);
        if constexpr (c != 0.f) {
#pragma unroll
          for (int v = 0; v < VEC; ++v) {
            if constexpr (i == first) acc[v] = c * t[i * A + j][v];
            else acc[v] = __builtin_fmaf(c, t[i * A + j][v], acc[v]);
          }
        }
      });
      store_pack<T, VEC>(V + (long long)(o * A + j) * a.t_stride, acc);
    });
  });
}

template <typename T, int KP, int VEC>
__global__ __launch_bounds__(256, (KP == KIND_43 ? 2 : 1)) void input_transform_3d_planes_kernel(InArgs a) {
  constexpr int AA = Mats<KP>::alpha * Mats<KP>::alpha;
  InWhere w;
  if (!in_decode(a, xcd_remap(blockIdx.x, a.per_xcd), VEC, w)) return;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.x), 0, a.x_bytes, 0x00020000);
  Pack<T, VEC> p[AA], q[AA];
  load_plane<T, KP, VEC>(a, rsrc, w, 1, p);
  load_plane<T, KP, VEC>(a, rsrc, w, 2, q);
  emit_plane<T, KP, VEC>(a, w, 1, p, q, 1.f, 1.f);    // o1 = p1 + p2
  emit_plane<T, KP, VEC>(a, w, 2, p, q, -1.f, 1.f);   // o2 = p2 - p1
  // (compiler fences: without them the loads of the later planes are hoisted and the register
  // count of the 6 x 6 version grows to one wavefront per SIMD)
  asm volatile("" ::: "memory");
  load_plane<T, KP, VEC>(a, rsrc, w, 0, p);           // q still holds p2
  emit_plane<T, KP, VEC>(a, w, 0, p, q, 1.f, -1.f);   // o0 = p0 - p2
  asm volatile("" ::: "memory");
  load_plane<T, KP, VEC>(a, rsrc, w, 1, p);
  load_plane<T, KP, VEC>(a, rsrc, w, 3, q);
  emit_plane<T, KP, VEC>(a, w, 3, p, q, 1.f, -1.f);   // o3 = p1 - p3
}

// F(4,3) planes; vec: channels per thread (2 for 16-bit types, else 1)
InKernel pick_in_3d_planes(int dtype, int vec) {
  return dispatch_dtype(dtype, [&](auto t) -> InKernel {
    using T = decltype(t);
    if constexpr (sizeof(T) == 2) return vec == 2 ? &input_transform_3d_planes_kernel<T, KIND_43, 2> : &input_transform_3d_planes_kernel<T, KIND_43, 1>;
    else return &input_transform_3d_planes_kernel<T, KIND_43, 1>;
  });
}

}  // namespace wc
