// Input transform kernels for 2-D problems with output tile 4: F(4,r) x F(4,s), r, s in 1..3.
#include "input_transform_impl.h"

namespace wc {

template <typename T, int VEC>
static InKernel pick2d_m4(int k1, int k2) {
#define WC_CASE(a, b) if (k1 == a && k2 == b) return in_kernel<T, VEC, KIND_11, a, b>();
  WC_CASE(KIND_41, KIND_41) WC_CASE(KIND_41, KIND_42) WC_CASE(KIND_41, KIND_43)
  WC_CASE(KIND_42, KIND_41) WC_CASE(KIND_42, KIND_42) WC_CASE(KIND_42, KIND_43)
  WC_CASE(KIND_43, KIND_41) WC_CASE(KIND_43, KIND_42) WC_CASE(KIND_43, KIND_43)
#undef WC_CASE
  return nullptr;
}

// 2 channels per thread (1 when C is odd): up to 36 live elements per channel
InKernel pick_in_2d_m4(int dtype, int k1, int k2, int vec) {
  return dispatch_dtype(dtype, [&](auto t) -> InKernel {
    using T = decltype(t);
    return vec == 2 ? pick2d_m4<T, 2>(k1, k2) : pick2d_m4<T, 1>(k1, k2);
  });
}

}  // namespace wc
