// Input transform that reads a channel-FIRST input (N, C, H, W contiguous) directly: single-piece
// 2-D plans at stride 1, F(2,r) x F(2,s) and F(4,r) x F(4,s), r, s in 1..3.
//
// The reference permutes the whole input to channel-last with a torch pass of its own before its
// kernels see it (dwm.py:129-133, Split_and_Concat.py:25,47); here the change of layout happens
// inside the transform.  A workgroup owns one row of tiles (all of it, or a block of neighbouring
// tiles when the image is wide) and 32 words of channels (64 channels of a 16-bit type as channel
// pairs, 32 channels of fp32).  Phase 1: lanes run along W, where channel-first memory is
// contiguous - the window rows of a tile row are one contiguous run per channel - and put the
// patch into LDS as [row][column][word], the word index innermost with a row pitch of 33 words,
// which is free of bank conflicts for the column-wise writes of this phase and the word-wise
// reads of the next.  Phase 2: a thread takes one tile and one word of channels, reads its window
// from LDS and runs the same register transform as the channel-last kernel
// (input_transform_impl.h), then stores V with the channels innermost.  Positions outside the
// image (padding) and channels beyond C (the zero columns that pad V to a multiple of 32) are
// zero words in LDS.  Results are bit-identical to the channel-last kernel on the permuted input.
#include "input_transform_impl.h"
#include <algorithm>

namespace wc {

constexpr int kNchwWords = 32;               // words of channels per workgroup
constexpr int kNchwPitch = kNchwWords + 1;   // LDS words per patch position

struct InNchwArgs {
  const void* x;
  void* V;
  int H, W, C, Cp;           // Cp: row length of V
  int nH, nW;
  int base1, base2;          // tap0 - pad
  long long t_stride;        // P * Cp
  int t_offset;
  int nWb, wblocks, cblocks; // tiles of a row per workgroup; workgroups per tile row; channel blocks
  int PW;                    // patch columns: m (nWb - 1) + alpha
  int n_blocks, per_xcd;
};

template <typename T, int K1, int K2, bool PAIR>
__global__ __launch_bounds__(256) void input_transform_nchw_kernel(InNchwArgs a) {
  constexpr int A1 = Mats<K1>::alpha, A2 = Mats<K2>::alpha;
  constexpr int m1 = Mats<K1>::m, m2 = Mats<K2>::m;
  constexpr int VEC = 4 / sizeof(T);                 // channels per word
  extern __shared__ __attribute__((aligned(16))) unsigned lds_words[];

  const int blk = xcd_remap(blockIdx.x, a.per_xcd);
  if (blk >= a.n_blocks) return;
  // neighbouring tile rows of one image and channel block are neighbours in the launch order
  const int th = blk % a.nH;
  int q = blk / a.nH;
  const int wb = q % a.wblocks; q /= a.wblocks;
  const int cb = q % a.cblocks;
  const long long b = q / a.cblocks;
  const int tw0 = wb * a.nWb;
  const int ntw = min(a.nWb, a.nW - tw0);
  const int c0 = cb * kNchwWords * VEC;
  const int y0 = m1 * th + a.base1, x0 = m2 * tw0 + a.base2;
  const int PW = a.PW;
  const T* x = static_cast<const T*>(a.x);
  const long long plane = (long long)a.H * a.W;
  const int tid = threadIdx.x;

  // ---- phase 1: patch (A1 rows x PW columns x 32 words) from channel-first memory into LDS
  if constexpr (sizeof(T) == 2 && PAIR) {
    // image columns in aligned pairs: one 4-byte load per channel, two words out
    const int xs = x0 & ~1;
    const int NP = (x0 + PW - xs + 1) >> 1;
    const int total = kNchwWords * A1 * NP;
    for (int it = tid; it < total; it += 256) {
      const int pq = it % NP;
      const int r = (it / NP) % A1;
      const int w = it / (NP * A1);
      const int ic = xs + 2 * pq, yy = y0 + r;
      const int c = c0 + 2 * w;
      const bool in_img = (unsigned)yy < (unsigned)a.H && ic >= 0 && ic + 1 < a.W;   // W is even, so is ic
      unsigned lo = 0, hi = 0;
      if (in_img) {
        const T* p = x + (b * a.C + c) * plane + (long long)yy * a.W + ic;
        if (c < a.C) lo = *reinterpret_cast<const unsigned*>(p);
        if (c + 1 < a.C) hi = *reinterpret_cast<const unsigned*>(p + plane);
      }
      const int j0 = ic - x0;
      if (j0 >= 0 && j0 < PW) lds_words[(r * PW + j0) * kNchwPitch + w] = (lo & 0xffffu) | (hi << 16);
      if (j0 + 1 >= 0 && j0 + 1 < PW) lds_words[(r * PW + j0 + 1) * kNchwPitch + w] = (lo >> 16) | (hi & 0xffff0000u);
    }
  } else {
    const int total = kNchwWords * A1 * PW;
    for (int it = tid; it < total; it += 256) {
      const int j = it % PW;
      const int r = (it / PW) % A1;
      const int w = it / (PW * A1);
      const int ic = x0 + j, yy = y0 + r;
      const int c = c0 + VEC * w;
      const bool in_img = (unsigned)yy < (unsigned)a.H && (unsigned)ic < (unsigned)a.W;
      unsigned word = 0;
      if (in_img) {
        const T* p = x + (b * a.C + c) * plane + (long long)yy * a.W + ic;
        if constexpr (sizeof(T) == 2) {
          unsigned lo = 0, hi = 0;
          if (c < a.C) lo = *reinterpret_cast<const unsigned short*>(p);
          if (c + 1 < a.C) hi = *reinterpret_cast<const unsigned short*>(p + plane);
          word = lo | (hi << 16);
        } else {
          if (c < a.C) word = *reinterpret_cast<const unsigned*>(p);
        }
      }
      lds_words[(r * PW + j) * kNchwPitch + w] = word;
    }
  }
  __syncthreads();

  // ---- phase 2: one tile x one word of channels per item
  const int items = ntw * kNchwWords;
  for (int it = tid; it < items; it += 256) {
    const int w = it % kNchwWords, j = it / kNchwWords;
    const int c = c0 + VEC * w;
    if (c >= a.Cp) continue;
    float d[A1 * A2][VEC];
    static_for<0, A1>([&](auto i1_) {
      static_for<0, A2>([&](auto i2_) {
        constexpr int i1 = decltype(i1_)::value, i2 = decltype(i2_)::value;
        const unsigned word = lds_words[(i1 * PW + m2 * j + i2) * kNchwPitch + w];
        if constexpr (sizeof(T) == 2) {
          const Pack<T, 2> v = __builtin_bit_cast(Pack<T, 2>, word);
          d[i1 * A2 + i2][0] = static_cast<float>(v.v[0]);
          d[i1 * A2 + i2][1] = static_cast<float>(v.v[1]);
        } else {
          d[i1 * A2 + i2][0] = __builtin_bit_cast(float, word);
        }
      });
    });
    // W, then H: the order of the channel-last kernel, so that the two agree bit for bit
    float t2[A1 * A2][VEC];
    apply_axis<MatSel<K2, false>, 2, 1, A1, A2, VEC>(d, t2);
    apply_axis<MatSel<K1, false>, 1, 1, A1, A2, VEC>(t2, d);
    const long long p = (b * a.nH + th) * a.nW + tw0 + j;
    T* V = static_cast<T*>(a.V) + (long long)a.t_offset * a.t_stride + p * a.Cp + c;
    static_for<0, A1 * A2>([&](auto e_) {
      constexpr int e = decltype(e_)::value;
      store_pack<T, VEC>(V + e * a.t_stride, d[e]);
    });
  }
}

using InNchwKernel = void (*)(InNchwArgs);

template <typename T, bool PAIR>
static InNchwKernel pick_nchw(int k1, int k2) {
#define WC_CASE(a, b) if (k1 == a && k2 == b) return &input_transform_nchw_kernel<T, a, b, PAIR>;
  WC_CASE(KIND_21, KIND_21) WC_CASE(KIND_21, KIND_22) WC_CASE(KIND_21, KIND_23)
  WC_CASE(KIND_22, KIND_21) WC_CASE(KIND_22, KIND_22) WC_CASE(KIND_22, KIND_23)
  WC_CASE(KIND_23, KIND_21) WC_CASE(KIND_23, KIND_22) WC_CASE(KIND_23, KIND_23)
  WC_CASE(KIND_41, KIND_41) WC_CASE(KIND_41, KIND_42) WC_CASE(KIND_41, KIND_43)
  WC_CASE(KIND_42, KIND_41) WC_CASE(KIND_42, KIND_42) WC_CASE(KIND_42, KIND_43)
  WC_CASE(KIND_43, KIND_41) WC_CASE(KIND_43, KIND_42) WC_CASE(KIND_43, KIND_43)
#undef WC_CASE
  return nullptr;
}

bool input_transform_nchw_fits(const wc_conv_desc* d, const wc_plan* plan) {
  if (d->ndim != 2 || plan->n_pieces != 1 || plan->tap_step != 1 || d->whole_kernel || d->stacked == 2) return false;
  if (plan->m[0] != 1 || plan->m[1] != plan->m[2] || (plan->m[1] != 2 && plan->m[1] != 4)) return false;
  const wc_piece& pc = plan->piece[0];
  return pc.r[1] >= 1 && pc.r[1] <= 3 && pc.r[2] >= 1 && pc.r[2] <= 3;
}

int input_transform_nchw(const wc_conv_desc* d, const wc_plan* plan, const void* x, int n_images, void* V, void* stream) {
  WC_CHECK_ARG(input_transform_nchw_fits(d, plan), "input_transform_nchw: plan outside the kernel's range");
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);
  if (rc) return rc;
  const wc_piece& pc = plan->piece[0];
  const int k1 = kind_of(plan->m[1], pc.r[1]), k2 = kind_of(plan->m[2], pc.r[2]);
  const int A1 = kind_alpha(k1), A2 = kind_alpha(k2), m2 = plan->m[2];
  const int es = d->dtype == WC_F32 ? 4 : 2;
  const int Cp = wc_padded_channels(d->C);
  InNchwArgs a;
  a.x = x; a.V = V;
  a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.Cp = Cp;
  a.nH = grid[1]; a.nW = grid[2];
  a.base1 = pc.tap0[1] - d->pad[1]; a.base2 = pc.tap0[2] - d->pad[2];
  const long long P = (long long)n_images * grid[1] * grid[2];
  a.t_stride = P * Cp;
  a.t_offset = pc.t_offset;
  // tiles of a row per workgroup: as many as keep the patch below 48 KB of LDS, in equal blocks
  const int max_pw = 48 * 1024 / (kNchwPitch * 4 * A1);
  const int cap = std::max(1, (max_pw - A2) / m2 + 1);
  a.wblocks = ceil_div(grid[2], cap);
  a.nWb = ceil_div(grid[2], a.wblocks);
  a.PW = m2 * (a.nWb - 1) + A2;
  a.cblocks = ceil_div(Cp, kNchwWords * (4 / es));
  const long long blocks = (long long)n_images * a.cblocks * a.wblocks * grid[1];
  WC_CHECK_ARG(blocks < (1ll << 30), "input_transform_nchw: problem too large");
  a.n_blocks = (int)blocks;
  a.per_xcd = ceil_div((int)blocks, kXcds);
  const bool pair = es == 2 && d->in[2] % 2 == 0 && (reinterpret_cast<uintptr_t>(x) & 3) == 0;
  InNchwKernel fn = dispatch_dtype(d->dtype, [&](auto t) -> InNchwKernel {
    using T = decltype(t);
    if constexpr (sizeof(T) == 2) return pair ? pick_nchw<T, true>(k1, k2) : pick_nchw<T, false>(k1, k2);
    else return pick_nchw<T, false>(k1, k2);
  });
  if (!fn) return fail(WC_ERR_UNSUPPORTED, "channel-first input transform for kinds (%d, %d) not built", k1, k2);
  const size_t lds = (size_t)A1 * a.PW * kNchwPitch * 4;
  hipLaunchKernelGGL(fn, dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), lds, as_stream(stream), a);
  WC_CHECK_LAUNCH("input_transform_nchw_kernel");
  return WC_OK;
}

}  // namespace wc
