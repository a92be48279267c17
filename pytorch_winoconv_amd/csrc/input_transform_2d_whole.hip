// Input transform kernels for 2-D whole-kernel tiles F(2,r) x F(2,r), r = 4..7 (the tiles of the
// reference's PyTorch path, matrix_conv.py:112-135).
#include "input_transform_impl.h"

namespace wc {

template <typename T, int VEC>
static InKernel pick2d_whole(int k1, int k2) {
#define WC_CASE(a) if (k1 == a && k2 == a) return in_kernel<T, VEC, KIND_11, a, a>();
  WC_CASE(KIND_24) WC_CASE(KIND_25) WC_CASE(KIND_26) WC_CASE(KIND_27)
#undef WC_CASE
  return nullptr;
}

// 2 channels per thread (1 when C is odd): up to 64 live elements per channel
InKernel pick_in_2d_whole(int dtype, int k1, int k2, int vec) {
  return dispatch_dtype(dtype, [&](auto t) -> InKernel {
    using T = decltype(t);
    return vec == 2 ? pick2d_whole<T, 2>(k1, k2) : pick2d_whole<T, 1>(k1, k2);
  });
}

}  // namespace wc
