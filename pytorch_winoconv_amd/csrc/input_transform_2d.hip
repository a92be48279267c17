// Input transform kernels for 2-D problems (one-element depth axis).
#include "input_transform_impl.h"

namespace wc {

template <typename T, int VEC>
static InKernel pick2d_m2(int k1, int k2) {
#define WC_CASE(a, b) if (k1 == a && k2 == b) return in_kernel<T, VEC, KIND_11, a, b>();
  WC_CASE(KIND_21, KIND_21) WC_CASE(KIND_21, KIND_22) WC_CASE(KIND_21, KIND_23)
  WC_CASE(KIND_22, KIND_21) WC_CASE(KIND_22, KIND_22) WC_CASE(KIND_22, KIND_23)
  WC_CASE(KIND_23, KIND_21) WC_CASE(KIND_23, KIND_22) WC_CASE(KIND_23, KIND_23)
  if constexpr (VEC <= 2) { WC_CASE(KIND_33, KIND_33) }     // the shared tile of three-tap pieces
#undef WC_CASE
  return nullptr;
}

// output tile 2: 8 (fp16) / 4 (fp32) / 2 / 1 channels per thread
InKernel pick_in_2d(int dtype, int k1, int k2, int vec) {
  if (kind_m(k1) == 4) return pick_in_2d_m4(dtype, k1, k2, vec);
  if ((k1 >= KIND_24 && k1 <= KIND_27) || (k2 >= KIND_24 && k2 <= KIND_27)) return pick_in_2d_whole(dtype, k1, k2, vec);
  if (dtype == WC_F16 || dtype == WC_BF16) {
    return dispatch_dtype(dtype, [&](auto t) -> InKernel {
      using T = decltype(t);
      if constexpr (sizeof(T) == 2) {
        if (vec == 8) return pick2d_m2<T, 8>(k1, k2);
        if (vec == 4) return pick2d_m2<T, 4>(k1, k2);
        return vec == 2 ? pick2d_m2<T, 2>(k1, k2) : pick2d_m2<T, 1>(k1, k2);
      } else {
        return nullptr;
      }
    });
  }
  if (vec == 4) return pick2d_m2<float, 4>(k1, k2);
  return vec == 2 ? pick2d_m2<float, 2>(k1, k2) : pick2d_m2<float, 1>(k1, k2);
}

}  // namespace wc
