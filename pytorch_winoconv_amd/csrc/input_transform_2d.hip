// Input transform kernels for 2-D problems (one-element depth axis).
#include "input_transform_impl.h"

namespace wc {

template <typename T, int VEC>
static InKernel pick2d(int k1, int k2) {
#define WC_CASE(a, b) if (k1 == a && k2 == b) return in_kernel<T, VEC, KIND_11, a, b>();
  WC_CASE(KIND_21, KIND_21) WC_CASE(KIND_21, KIND_22) WC_CASE(KIND_21, KIND_23)
  WC_CASE(KIND_22, KIND_21) WC_CASE(KIND_22, KIND_22) WC_CASE(KIND_22, KIND_23)
  WC_CASE(KIND_23, KIND_21) WC_CASE(KIND_23, KIND_22) WC_CASE(KIND_23, KIND_23)
  WC_CASE(KIND_43, KIND_43)
#undef WC_CASE
  return nullptr;
}

InKernel pick_in_2d(int dtype, int k1, int k2, int vec) {
  if (dtype == WC_F16) {
    if (vec == 8) return pick2d<half_t, 8>(k1, k2);
    if (vec == 2) return pick2d<half_t, 2>(k1, k2);
    return vec == 4 ? pick2d<half_t, 4>(k1, k2) : pick2d<half_t, 1>(k1, k2);
  }
  if (vec == 2) return pick2d<float, 2>(k1, k2);
  return vec == 4 ? pick2d<float, 4>(k1, k2) : pick2d<float, 1>(k1, k2);
}

}  // namespace wc
