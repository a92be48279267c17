// Change of layout between channel-first (N, C, S) and channel-last (N, S, C) memory, S = [D] H W: a bit-exact
// copy.  Replaces the permute passes the reference runs in torch on both sides of its kernels
// (dwm.py:129-133,143-144; Split_and_Concat.py:25,47,64,81) for the plans whose transform kernels cannot read or
// write channel-first memory themselves.
//
// Per image this is the transpose of an R x Q matrix into a Q x R one.  A workgroup moves a 64 x 64 tile
// through LDS (pitch 65 elements: the row-wise writes and the column-wise reads both touch every bank once);
// lanes run along the contiguous axis on both sides.
#include "wc_common.h"

namespace wc {

struct TransposeArgs {
  const void* src;     // (n, R, Q)
  void* dst;           // (n, Q, R)
  long long R, Q;
  int tiles_r, tiles_q;
  long long n_blocks;
};

template <typename U>
__global__ __launch_bounds__(256) void transpose_kernel(TransposeArgs a) {
  __shared__ U tile[64][65];
  const long long blk = blockIdx.x;
  const int tq = (int)(blk % a.tiles_q);
  const long long rest = blk / a.tiles_q;
  const int tr = (int)(rest % a.tiles_r);
  const long long n = rest / a.tiles_r;
  const long long r0 = (long long)tr * 64, q0 = (long long)tq * 64;
  const U* src = static_cast<const U*>(a.src) + n * a.R * a.Q;
  U* dst = static_cast<U*>(a.dst) + n * a.R * a.Q;
  const int lx = threadIdx.x & 63, ly = threadIdx.x >> 6;
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int r = ly + 4 * i;
    if (r0 + r < a.R && q0 + lx < a.Q) tile[r][lx] = src[(r0 + r) * a.Q + q0 + lx];
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 16; ++i) {
    const int qq = ly + 4 * i;
    if (q0 + qq < a.Q && r0 + lx < a.R) dst[(q0 + qq) * a.R + r0 + lx] = tile[lx][qq];
  }
}

// The same for 2-byte elements with both extents even and 4-byte aligned tensors: every global access moves a
// pair of elements (a wavefront reads and writes 256 contiguous bytes per tile row instead of 128).  The tile
// sits in LDS as [r][q] with a pitch of 66 elements: the pair-wise writes along q are consecutive words, and
// the reads of one column q for two consecutive rows land in 32 different banks across the 32 row pairs.
__global__ __launch_bounds__(256) void transpose_pairs_kernel(TransposeArgs a) {
  __shared__ unsigned short tile[64 * 66];
  const long long blk = blockIdx.x;
  const int tq = (int)(blk % a.tiles_q);
  const long long rest = blk / a.tiles_q;
  const int tr = (int)(rest % a.tiles_r);
  const long long n = rest / a.tiles_r;
  const long long r0 = (long long)tr * 64, q0 = (long long)tq * 64;
  const unsigned short* src = static_cast<const unsigned short*>(a.src) + n * a.R * a.Q;
  unsigned short* dst = static_cast<unsigned short*>(a.dst) + n * a.R * a.Q;
  const int lx = threadIdx.x & 31, ly = threadIdx.x >> 5;      // 32 pairs per row, 8 rows per pass
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int r = ly + 8 * i;
    if (r0 + r < a.R && q0 + 2 * lx < a.Q)
      *reinterpret_cast<unsigned*>(&tile[r * 66 + 2 * lx]) = *reinterpret_cast<const unsigned*>(src + (r0 + r) * a.Q + q0 + 2 * lx);
  }
  __syncthreads();
#pragma unroll
  for (int i = 0; i < 8; ++i) {
    const int qq = ly + 8 * i;
    if (q0 + qq < a.Q && r0 + 2 * lx < a.R) {
      const unsigned v = (unsigned)tile[(2 * lx) * 66 + qq] | ((unsigned)tile[(2 * lx + 1) * 66 + qq] << 16);
      *reinterpret_cast<unsigned*>(dst + (q0 + qq) * a.R + r0 + 2 * lx) = v;
    }
  }
}

// src (n, R, Q) -> dst (n, Q, R), elements of 2 or 4 bytes
int transpose_images(const void* src, void* dst, long long n, long long R, long long Q, int elem_size, void* stream) {
  WC_CHECK_ARG(src && dst && n > 0 && R > 0 && Q > 0, "layout copy: null pointer or empty tensor");
  WC_CHECK_ARG(elem_size == 2 || elem_size == 4, "layout copy: element size %d", elem_size);
  TransposeArgs a;
  a.src = src; a.dst = dst; a.R = R; a.Q = Q;
  a.tiles_r = (int)ceil_div_ll(R, 64); a.tiles_q = (int)ceil_div_ll(Q, 64);
  a.n_blocks = n * a.tiles_r * a.tiles_q;
  WC_CHECK_ARG(a.n_blocks < (1ll << 31), "layout copy: problem too large");
  const bool pairs = elem_size == 2 && R % 2 == 0 && Q % 2 == 0 &&
                     ((reinterpret_cast<uintptr_t>(src) | reinterpret_cast<uintptr_t>(dst)) & 3) == 0;
  if (pairs)
    hipLaunchKernelGGL(transpose_pairs_kernel, dim3((unsigned)a.n_blocks), dim3(256), 0, as_stream(stream), a);
  else if (elem_size == 2)
    hipLaunchKernelGGL(transpose_kernel<unsigned short>, dim3((unsigned)a.n_blocks), dim3(256), 0, as_stream(stream), a);
  else
    hipLaunchKernelGGL(transpose_kernel<unsigned>, dim3((unsigned)a.n_blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("transpose_kernel");
  return WC_OK;
}

}  // namespace wc

using namespace wc;

extern "C" int wc_layout_copy(const void* src, void* dst, int n_images, int channels, long long spatial,
                              int to_channel_last, int elem_size, void* stream) {
  WC_CHECK_ARG(n_images > 0 && channels > 0 && spatial > 0, "wc_layout_copy: %d images, %d channels, %lld positions",
               n_images, channels, spatial);
  // channel-first (n, C, S) -> channel-last (n, S, C) is the transpose of C x S matrices, and back
  return to_channel_last ? transpose_images(src, dst, n_images, channels, spatial, elem_size, stream)
                         : transpose_images(src, dst, n_images, spatial, channels, elem_size, stream);
}
