// Input transform that reads a channel-FIRST input (N, C, H, W contiguous) directly: single-piece
// 2-D plans at stride 1, F(2,r) x F(2,s) and F(4,r) x F(4,s), r, s in 1..3.
//
// The reference permutes the whole input to channel-last with a torch pass of its own before its
// kernels see it (dwm.py:129-133, Split_and_Concat.py:25,47); here the change of layout happens
// inside the transform.  A workgroup owns one row of tiles (all of it, or a block of neighbouring
// tiles when the image is wide) and 32 words of channels (64 channels of a 16-bit type as channel
// pairs, 32 channels of fp32).  Phase 1: lanes run along W, where channel-first memory is
// contiguous (16-byte loads where the row pitch allows, all loads of a pass in flight together), and put the
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

// CE: image columns per global load (the 16-, 4- or 2/4-byte form: the row pitch W must be a multiple of CE and
// x aligned to the load size)
template <typename T, int K1, int K2, int CE>
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
  // positions outside the image are zero words: whole rows, then the columns left and right of the image
  const int nl = max(0, -x0), nr = max(0, x0 + PW - a.W);
  static_for<0, A1>([&](auto r_) {
    constexpr int r = decltype(r_)::value;
    if ((unsigned)(y0 + r) >= (unsigned)a.H) {
      for (int i = tid; i < PW * kNchwWords; i += 256) lds_words[(r * PW + (i >> 5)) * kNchwPitch + (i & 31)] = 0;
    } else {
      for (int i = tid; i < (nl + nr) * kNchwWords; i += 256) {
        const int k = i >> 5;
        const int j = k < nl ? k : PW - nr + (k - nl);
        lds_words[(r * PW + j) * kNchwPitch + (i & 31)] = 0;
      }
    }
  });
  // the image part: lanes along W in chunks of CE columns, LPR lanes per row of the patch, the rows of
  // 256 / LPR words of channels per pass; all loads of a pass are requested before the first is used
  constexpr int LPR = 64 / CE;                       // lanes per patch row: 64 columns
  constexpr int WPP = 256 / LPR;                     // words of channels per pass
  using Raw = Pack<T, CE>;
  const int lane_q = tid % LPR, lane_w = tid / LPR;
  const int q_first = max(0, x0) / CE;               // first chunk with a column of the patch
  const int col_end = min(a.W, x0 + PW);             // one past the last image column of the patch
  for (int w = lane_w; w < kNchwWords; w += WPP) {
    const int c = c0 + VEC * w;
    for (int qq = q_first + lane_q; qq * CE < col_end; qq += LPR) {
      const int ic0 = qq * CE;
      Raw lo[A1], hi[A1];
      static_for<0, A1>([&](auto r_) {
        constexpr int r = decltype(r_)::value;
        const int yy = y0 + r;
        lo[r] = Raw{};
        hi[r] = Raw{};
        if ((unsigned)yy < (unsigned)a.H) {
          const T* p = x + (b * a.C + c) * plane + (long long)yy * a.W + ic0;
          if (c < a.C) lo[r] = *reinterpret_cast<const Raw*>(p);
          if constexpr (VEC == 2) {
            if (c + 1 < a.C) hi[r] = *reinterpret_cast<const Raw*>(p + plane);
          }
        }
      });
      static_for<0, A1>([&](auto r_) {
        constexpr int r = decltype(r_)::value;
        if ((unsigned)(y0 + r) < (unsigned)a.H) {
#pragma unroll
          for (int i = 0; i < CE; ++i) {
            const int j = ic0 + i - x0;
            if (j >= 0 && j < PW) {
              unsigned word;
              if constexpr (VEC == 2) {
                const Pack<T, 2> pr{{lo[r].v[i], hi[r].v[i]}};
                word = __builtin_bit_cast(unsigned, pr);
              } else {
                word = __builtin_bit_cast(unsigned, lo[r].v[i]);
              }
              lds_words[(r * PW + j) * kNchwPitch + w] = word;
            }
          }
        }
      });
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

template <typename T, int CE>
static InNchwKernel pick_nchw(int k1, int k2) {
#define WC_CASE(a, b) if (k1 == a && k2 == b) return &input_transform_nchw_kernel<T, a, b, CE>;
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
  if (!(pc.r[1] >= 1 && pc.r[1] <= 3 && pc.r[2] >= 1 && pc.r[2] <= 3)) return false;
  // the lanes of the loading phase run along W: images narrower than 16 columns leave most of them idle, and the
  // copy to channel-last memory followed by the channel-last kernel measured faster (N=64, 512 channels, 7x7)
  return d->in[2] >= 16;
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
  // columns per load: 16-byte loads where the row pitch and the base allow them, else 4-byte, else single elements
  const uintptr_t addr = reinterpret_cast<uintptr_t>(x);
  const int W = d->in[2];
  int ce = 1;
  if (W % (16 / es) == 0 && (addr & 15) == 0) ce = 16 / es;
  else if (es == 2 && W % 2 == 0 && (addr & 3) == 0) ce = 2;
  InNchwKernel fn = dispatch_dtype(d->dtype, [&](auto t) -> InNchwKernel {
    using T = decltype(t);
    if constexpr (sizeof(T) == 2) return ce == 8 ? pick_nchw<T, 8>(k1, k2) : ce == 2 ? pick_nchw<T, 2>(k1, k2) : pick_nchw<T, 1>(k1, k2);
    else return ce == 4 ? pick_nchw<T, 4>(k1, k2) : pick_nchw<T, 1>(k1, k2);
  });
  if (!fn) return fail(WC_ERR_UNSUPPORTED, "channel-first input transform for kinds (%d, %d) not built", k1, k2);
  const size_t lds = (size_t)A1 * a.PW * kNchwPitch * 4;
  hipLaunchKernelGGL(fn, dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), lds, as_stream(stream), a);
  WC_CHECK_LAUNCH("input_transform_nchw_kernel");
  return WC_OK;
}

}  // namespace wc
