// Batched product with the reduction along the rows of both operands:
//
//   D[t][s] (na x nb, fp32) = sum over rows p of part s of  A[t][p][0..na) (x) B[t][p][0..nb)
//
// This is the contraction over the tiles in the weight gradient (dU = dM^T V per transform
// element): both operands are stored the way the forward kernels write them, rows = tiles,
// channels contiguous, and nothing is transposed in memory.  The reference has no counterpart
// (its backward pass was never written: src/back/utils.cu:15-24).
//
// A stage holds BK rows of each operand exactly as they lie in memory (16-byte loads and LDS
// stores of whole rows).  The MFMA operands need 8 consecutive reduction elements per lane, which
// in this layout are a column: for 16-bit types ds_read_b64_tr_b16 delivers exactly that (16 lanes
// read 4 rows x 32 bytes, and lane j receives column j of the 4 x 16 block), for fp32 the operand
// of v_mfma_f32_32x32x2_f32 is a single element and a plain 4-byte read of a row does.  LDS rows
// are padded by 32 bytes so that the 4 rows of a transposing read fall into different banks.
//
// The reduction is split into S parts of Pq rows (few outputs, a long reduction: the parts are
// what fills the chip); the caller adds the parts.  Workgroup = 4 wavefronts (2 x 2), each owning
// W x W blocks of 32 x 32.  V feeds the MFMA "A" side, so a lane ends up with 4 consecutive
// columns of D and stores them as one 16-byte write.
#include "wc_common.h"
#include "wc_transform.h"

namespace wc {

namespace {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef short short4v __attribute__((ext_vector_type(4)));
typedef short short8v __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t Chunk16 __attribute__((ext_vector_type(4)));

struct GemmTnArgs {
  const void* A;             // (T, P, lda)
  const void* B;             // (T, P, ldb)
  float* D;                  // (T, S, na, ldd)
  long long P;
  int lda, ldb, na, nb, ldd;
  int S, Pq;
  int tiles_a, tiles_b;
  int n_blocks, per_xcd;
  // GATHER (the weight gradient of a convolution taken directly, one batch per tap): A is dy (P = N oH oW rows, the
  // same for every batch), B is x itself, and row p = (b, oy, ox) of batch t = (ky, kx) is the pixel
  // (stride oy + ky - pad_h, stride ox + kx - pad_w) of image b, zeros outside the image
  int H, W, oH, oW, conv_stride, pad_h, pad_w, kw;
  FastDiv div_per, div_oW;
};

__device__ __forceinline__ floatx16 mfma16(short8v a, short8v b, floatx16 c, half_t) {
  return __builtin_amdgcn_mfma_f32_32x32x16_f16(__builtin_bit_cast(half8, a), __builtin_bit_cast(half8, b), c, 0, 0, 0);
}
__device__ __forceinline__ floatx16 mfma16(short8v a, short8v b, floatx16 c, bf16_t) {
  return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(bf16x8, a), __builtin_bit_cast(bf16x8, b), c, 0, 0, 0);
}

template <typename T, int W, int BK, bool GATHER = false>
__global__ __launch_bounds__(256, 2) void gemm_tn_kernel(GemmTnArgs g) {
  constexpr int BT = 64 * W;                       // tile extent on both output axes
  constexpr int EPC = 16 / sizeof(T);              // elements per 16-byte chunk
  constexpr int PITCH = BT + 32 / sizeof(T);       // LDS row, elements
  constexpr int CPR = BT / EPC;                    // chunks per row
  constexpr int RPP = 256 / CPR;                   // rows per load pass
  constexpr int NL = BK / RPP;                     // load passes per operand
  constexpr int STAGE = 2 * BK * PITCH;            // A rows, then B rows
  static_assert(RPP * CPR == 256 && NL * RPP == BK && NL >= 1, "tile shape");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const int blk = xcd_remap(blockIdx.x, g.per_xcd);
  if (blk >= g.n_blocks) return;
  const int tb = blk % g.tiles_b;
  const int ta = (blk / g.tiles_b) % g.tiles_a;
  const int ts = blk / (g.tiles_b * g.tiles_a);
  const int s = ts % g.S;
  const int t = ts / g.S;
  const int a0 = ta * BT, b0 = tb * BT;
  const long long p_begin = (long long)s * g.Pq;
  const long long p_end = min(g.P, p_begin + g.Pq);
  const int nk = p_end > p_begin ? (int)((p_end - p_begin + BK - 1) / BK) : 0;

  const T* Ap = static_cast<const T*>(g.A) + (GATHER ? 0 : (long long)t * g.P * g.lda);
  const T* Bp = static_cast<const T*>(g.B) + (GATHER ? 0 : (long long)t * g.P * g.ldb);
  const int tap_y = GATHER ? t / g.kw : 0, tap_x = GATHER ? t - tap_y * g.kw : 0;

  const int tid = threadIdx.x;
  const int lrow = tid / CPR, lcol = (tid % CPR) * EPC;
  const bool a_in = a0 + lcol < g.lda, b_in = b0 + lcol < g.ldb;   // ld is a multiple of 8: whole chunks

  Chunk16 ra[NL], rb[NL];
  auto gload = [&](int kt) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const long long p = p_begin + (long long)kt * BK + lrow + i * RPP;
      const Chunk16 zero = {0u, 0u, 0u, 0u};
      ra[i] = (p < p_end && a_in) ? *reinterpret_cast<const Chunk16*>(Ap + p * g.lda + a0 + lcol) : zero;
      if constexpr (GATHER) {
        const int pi = (int)min(p, g.P - 1);
        const int b = fast_div(pi, g.div_per), rem = pi - b * (g.oH * g.oW);
        const int oy = fast_div(rem, g.div_oW), ox = rem - oy * g.oW;
        const int iy = oy * g.conv_stride + tap_y - g.pad_h, ix = ox * g.conv_stride + tap_x - g.pad_w;
        const bool inside = (unsigned)iy < (unsigned)g.H && (unsigned)ix < (unsigned)g.W;
        rb[i] = (p < p_end && b_in && inside)
                    ? *reinterpret_cast<const Chunk16*>(Bp + (((long long)b * g.H + iy) * g.W + ix) * g.ldb + b0 + lcol) : zero;
      } else {
        rb[i] = (p < p_end && b_in) ? *reinterpret_cast<const Chunk16*>(Bp + p * g.ldb + b0 + lcol) : zero;
      }
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NL; ++i) {
      const int off = buf * STAGE + (lrow + i * RPP) * PITCH + lcol;
      *reinterpret_cast<Chunk16*>(lds + off) = ra[i];
      *reinterpret_cast<Chunk16*>(lds + off + BK * PITCH) = rb[i];
    }
  };

  const int lane = tid & 63, wave = tid >> 6;
  const int wa = wave >> 1, wb = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  floatx16 acc[W][W];
#pragma unroll
  for (int i = 0; i < W; ++i)
#pragma unroll
    for (int j = 0; j < W; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // offset of a lane's fragment source inside a stage, for block 0 of its wavefront and step 0
  int fa, fb;
  if constexpr (sizeof(T) == 2) {
    // 16-lane group b reads rows 8*lhi + (0..3), columns 16*(b&1) + (0..15); lane s of the group
    // supplies the 4 elements at row s/4, columns 4*(s%4)..+3 and receives column s of the block
    const int b = lane >> 4, sl = lane & 15;
    const int row = 8 * lhi + (sl >> 2), col = 16 * (b & 1) + 4 * (sl & 3);
    fa = row * PITCH + wa * W * 32 + col;
    fb = BK * PITCH + row * PITCH + wb * W * 32 + col;
  } else {
    fa = lhi * PITCH + wa * W * 32 + l32;
    fb = BK * PITCH + lhi * PITCH + wb * W * 32 + l32;
  }

  if (nk > 0) {
    gload(0);
    lstore(0);
  }
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if (kt + 1 < nk) gload(kt + 1);
    const T* st = lds + cur * STAGE;
    if constexpr (sizeof(T) == 2) {
      typedef short4v __attribute__((address_space(3))) * LdsVec;
#pragma unroll
      for (int kk = 0; kk < BK / 16; ++kk) {
        short8v af[W], bf[W];
#pragma unroll
        for (int i = 0; i < W; ++i) {
          const T* src = st + fa + kk * 16 * PITCH + i * 32;
          const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsVec)(src));
          const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsVec)(src + 4 * PITCH));
          af[i] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int j = 0; j < W; ++j) {
          const T* src = st + fb + kk * 16 * PITCH + j * 32;
          const short4v lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsVec)(src));
          const short4v hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((LdsVec)(src + 4 * PITCH));
          bf[j] = __builtin_shufflevector(lo, hi, 0, 1, 2, 3, 4, 5, 6, 7);
        }
#pragma unroll
        for (int i = 0; i < W; ++i)
#pragma unroll
          for (int j = 0; j < W; ++j) acc[i][j] = mfma16(bf[j], af[i], acc[i][j], T{});
      }
    } else {
#pragma unroll
      for (int kk = 0; kk < BK / 2; ++kk) {
        float af[W], bf[W];
#pragma unroll
        for (int i = 0; i < W; ++i) af[i] = st[fa + kk * 2 * PITCH + i * 32];
#pragma unroll
        for (int j = 0; j < W; ++j) bf[j] = st[fb + kk * 2 * PITCH + j * 32];
#pragma unroll
        for (int i = 0; i < W; ++i)
#pragma unroll
          for (int j = 0; j < W; ++j)
            acc[i][j] = __builtin_amdgcn_mfma_f32_32x32x2f32(bf[j], af[i], acc[i][j], 0, 0, 0);
      }
    }
    if (kt + 1 < nk) lstore(cur ^ 1);
    __syncthreads();
  }

  // accumulator (i, j), register 4q + e: row a0 + 32 (W wa + i) + l32, column b0 + 32 (W wb + j) + 8q + 4 lhi + e
  float* Dt = g.D + ((long long)t * g.S + s) * g.na * g.ldd;
#pragma unroll
  for (int i = 0; i < W; ++i) {
    const int row = a0 + (wa * W + i) * 32 + l32;
    if (row >= g.na) continue;
#pragma unroll
    for (int j = 0; j < W; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        const int col = b0 + (wb * W + j) * 32 + 8 * q + 4 * lhi;
        if (col < g.ldd) {
          floatx4 o = {acc[i][j][4 * q], acc[i][j][4 * q + 1], acc[i][j][4 * q + 2], acc[i][j][4 * q + 3]};
          *reinterpret_cast<floatx4*>(Dt + (long long)row * g.ldd + col) = o;
        }
      }
  }
}

template <typename T, int W, bool GATHER = false>
int launch_tn(GemmTnArgs g, int T_, void* stream) {
  constexpr int BT = 64 * W;
  constexpr int BK = sizeof(T) == 2 ? 64 : 16;     // reduction rows per stage (64: measured 5 % faster than 32)
  constexpr size_t lds = (size_t)2 * 2 * BK * (BT + 32 / sizeof(T)) * sizeof(T);
  g.tiles_a = ceil_div(g.na, BT);
  g.tiles_b = ceil_div(g.nb, BT);
  const long long blocks = (long long)g.tiles_a * g.tiles_b * g.S * T_;
  WC_CHECK_ARG(blocks < (1ll << 30), "batched_gemm_tn: problem too large");
  g.n_blocks = (int)blocks;
  g.per_xcd = ceil_div((int)blocks, kXcds);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(&gemm_tn_kernel<T, W, BK, GATHER>), lds)) return rc;
  hipLaunchKernelGGL((gemm_tn_kernel<T, W, BK, GATHER>), dim3((unsigned)(g.per_xcd * kXcds)), dim3(256), lds, as_stream(stream), g);
  WC_CHECK_LAUNCH("gemm_tn_kernel");
  return WC_OK;
}

}  // namespace

int batched_gemm_tn(const void* A, const void* B, float* D, int T_, long long P, int lda, int ldb, int na, int nb,
                    int ldd, int S, int Pq, int dtype, void* stream) {
  WC_CHECK_ARG(A && B && D, "batched_gemm_tn: null pointer");
  WC_CHECK_ARG(T_ > 0 && P > 0 && na > 0 && nb > 0 && S > 0 && Pq > 0, "batched_gemm_tn: empty problem");
  WC_CHECK_ARG(lda % 8 == 0 && ldb % 8 == 0 && ldd % 4 == 0 && lda >= na && ldb >= nb && ldd >= nb,
               "batched_gemm_tn: row strides %d, %d, %d", lda, ldb, ldd);
  WC_CHECK_ARG((long long)S * Pq >= P, "batched_gemm_tn: %d parts of %d rows do not cover %lld rows", S, Pq, P);
  GemmTnArgs g;
  g.A = A; g.B = B; g.D = D; g.P = P;
  g.lda = lda; g.ldb = ldb; g.na = na; g.nb = nb; g.ldd = ldd;
  g.S = S; g.Pq = Pq;
  g.H = g.W = g.oH = g.oW = g.conv_stride = g.pad_h = g.pad_w = g.kw = 0;
  g.div_per = g.div_oW = make_fast_div(1);
  const bool big = na > 64 && nb > 64;
  return dispatch_dtype(dtype, [&](auto t) {
    using TT = decltype(t);
    return big ? launch_tn<TT, 2>(g, T_, stream) : launch_tn<TT, 1>(g, T_, stream);
  });
}

// dW[(ky, kx)][s] (K x C, fp32) = sum over the output pixels p = (b, oy, ox) of part s of dy[p][0..K) (x)
// x[b][stride oy + ky - pad_h][stride ox + kx - pad_w][0..C): the weight gradient taken directly, one batch per tap,
// x gathered row by row (zeros outside the image).  dy (N oH oW, K) and x (N, H, W, C) as they lie in memory.
int gemm_tn_conv(const void* dy, const void* x, float* D, int N, int H, int W, int C, int K, int kh, int kw, int stride,
                 int pad_h, int pad_w, int oH, int oW, int S, int Pq, int dtype, void* stream) {
  WC_CHECK_ARG(dy && x && D, "gemm_tn_conv: null pointer");
  WC_CHECK_ARG(C % 8 == 0 && K % 8 == 0 && S > 0 && Pq > 0, "gemm_tn_conv: C %d, K %d (multiples of 8)", C, K);
  const long long P = (long long)N * oH * oW;
  WC_CHECK_ARG(P > 0 && P < (1ll << 31) && (long long)S * Pq >= P, "gemm_tn_conv: %d parts of %d rows and %lld rows", S, Pq, P);
  GemmTnArgs g;
  g.A = dy; g.B = x; g.D = D; g.P = P;
  g.lda = K; g.ldb = C; g.na = K; g.nb = C; g.ldd = C;
  g.S = S; g.Pq = Pq;
  g.H = H; g.W = W; g.oH = oH; g.oW = oW; g.conv_stride = stride; g.pad_h = pad_h; g.pad_w = pad_w; g.kw = kw;
  g.div_per = make_fast_div(oH * oW); g.div_oW = make_fast_div(oW);
  const bool big = K > 64 && C > 64;
  return dispatch_dtype(dtype, [&](auto t) {
    using TT = decltype(t);
    return big ? launch_tn<TT, 2, true>(g, kh * kw, stream) : launch_tn<TT, 1, true>(g, kh * kw, stream);
  });
}

}  // namespace wc
