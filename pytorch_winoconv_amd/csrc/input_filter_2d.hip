// Input transform of a single-piece 2-D plan with the filter transform of the same call riding in the first
// workgroups of the launch.  The two transforms are independent and both feed the batched product; as two
// launches on one stream they run one after the other, and for layers with few tiles and many channels the
// filter transform is as long as everything else (N=64, 512 channels, 7x7: 11 of 40 us).
#include "filter_transform_impl.h"
#include "input_transform_impl.h"

namespace wc {

// The last f_blocks workgroups of the launch transform the filter (at the front or at the back of the launch
// measured the same).  The filter part takes one channel per thread for the fp32 F(4,3) tile: with two, the kernel
// needs more registers than the input transform alone and one wavefront fewer fits a SIMD.
template <typename T, int K1, int K2, int VEC>
__global__ __launch_bounds__(256) void input_filter_kernel(InArgs a, FilterFastArgs f, int f_blocks) {
  const int first_f = gridDim.x - f_blocks;
  if ((int)blockIdx.x >= first_f) {
    constexpr int FV = in_filter_vec(sizeof(T), K1);
    filter_fast_body<T, KIND_11, K1, K2, (FV > 1), FV>(f, (blockIdx.x - first_f) * 256 + threadIdx.x);
    return;
  }
  InWhere w;
  if (!in_decode(a, xcd_remap(blockIdx.x, a.per_xcd), VEC, w)) return;
  transform_window<T, KIND_11, K1, K2, VEC>(a, w, a.base0, a.base1, a.base2, a.t_offset, 0);
}

template <typename T>
static InFilterKernel pick(int k1, int k2, int vec) {
  constexpr int V2 = sizeof(T) == 4 ? 4 : 8;          // channels per thread of the F(2,3) input transform
  if (k1 == KIND_43 && k2 == KIND_43 && vec == 2) return &input_filter_kernel<T, KIND_43, KIND_43, 2>;
  if (k1 == KIND_23 && k2 == KIND_23 && vec == V2) return &input_filter_kernel<T, KIND_23, KIND_23, V2>;
  return nullptr;
}

InFilterKernel pick_in_filter_2d(int dtype, int k1, int k2, int vec) {
  return dispatch_dtype(dtype, [&](auto t) -> InFilterKernel { return pick<decltype(t)>(k1, k2, vec); });
}

}  // namespace wc
