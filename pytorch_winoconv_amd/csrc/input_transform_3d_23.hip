#define WC_K0 KIND_23
#define WC_PICK_NAME pick_in_3d_23
#include "input_transform_3d.inc"

namespace wc {
// pixel columns: depth and height in F(2,3) tiles, nothing along the width (one row of V per column); vec 8, 4, 2 or 1
InKernel pick_in_columns(int dtype, int vec) {
  return dispatch_dtype(dtype, [&](auto t) -> InKernel {
    using T = decltype(t);
    return vec == 8 ? in_kernel<T, 8, KIND_23, KIND_23, KIND_11>() : vec == 4 ? in_kernel<T, 4, KIND_23, KIND_23, KIND_11>()
         : vec == 2 ? in_kernel<T, 2, KIND_23, KIND_23, KIND_11>() : in_kernel<T, 1, KIND_23, KIND_23, KIND_11>();
  });
}
}  // namespace wc
