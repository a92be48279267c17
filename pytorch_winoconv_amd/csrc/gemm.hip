// Batched GEMM of the Winograd domain: M[t] (P x K) = V[t] (P x Cp) . U[t]^T, t in [0, T).
//
// Replaces forwardAssign + cublas{S,H}gemmBatched of the reference (src/utils.cu:5-12,
// src/base_conv_launchers.cu:353-367, src/base_conv_launchers_half.cu:231-236): batches are
// addressed by stride, so no pointer arrays.  Both operands keep the reduction axis C
// innermost, which is the layout MFMA wants for both: a lane feeds 8 consecutive halves
// (one 16-byte LDS read) per operand per v_mfma_f32_32x32x16_f16.
//
// Workgroup = 4 wavefronts (2 x 2), each owning WM x WN MFMA blocks of 32 x 32, so the
// macro tile is (64 WM) tiles x (64 WN) output channels.  Operand tiles go global -> registers ->
// LDS with two LDS stages (one barrier per reduction step; the global loads of step k+1 are in
// flight while step k is multiplied).  LDS rows are 64 bytes with their 16-byte chunks swizzled
// by row, which keeps both the row-wise stores and the column-wise fragment reads free of bank
// conflicts.  The MFMA "A" operand is the
// filter block and "B" the input block: a lane then holds 4 consecutive output channels of
// one tile row per accumulator group and stores them as one 8-byte (fp16) / 16-byte (fp32)
// write.  fp16 and bf16 accumulate in fp32; fp32 uses v_mfma_f32_32x32x2_f32.
//
// Plans whose pieces share one transformed input read V at a row offset per piece: gemm_kernel
// with SHIFT walks the operand pointer piece by piece; gemm_rows_kernel serves the pieces of one
// run (neighbours along the width) from a single operand tile that is n_run - 1 rows taller.
#include "wc_common.h"

namespace wc {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx16 __attribute__((ext_vector_type(16)));
typedef float floatx4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma;
template <> struct Mfma<half_t> {
  using Frag = half8;
  static constexpr int kpack = 8;    // consecutive reduction elements a lane supplies
  static constexpr int kstep = 16;   // reduction elements per instruction
  __device__ static __forceinline__ floatx16 run(Frag a, Frag b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma<bf16_t> {
  using Frag = bf16x8;
  static constexpr int kpack = 8;
  static constexpr int kstep = 16;
  __device__ static __forceinline__ floatx16 run(Frag a, Frag b, floatx16 c) {
    return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0);
  }
};
// fp32: a lane reads four consecutive reduction elements with one 16-byte LDS access and feeds
// them to four v_mfma_f32_32x32x2_f32, each of which pairs element e of the lower lanes' chunk
// with element e of the upper lanes' chunk (4 elements further along the reduction axis).
template <> struct Mfma<float> {
  using Frag = floatx4;
  static constexpr int kpack = 4;
  static constexpr int kstep = 8;
  __device__ static __forceinline__ floatx16 run(Frag a, Frag b, floatx16 c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_32x32x2f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
};

struct GemmArgs {
  const void* V;
  const void* U;
  void* M;
  int P, K, Cp, ldm;
  long long sV, sU, sM;     // batch strides in elements
  int tiles_p, tiles_k, T;
  int n_blocks, per_xcd;
  // shifted operand (plans whose pieces share one transformed input): rows of V are ldv apart, and
  // after every run_blocks reduction blocks the V operand jumps on by `jump` elements
  // (one run = the pieces along the width: consecutive rows of V), and after every plane_runs runs
  // by jump2 more (3-D plans: on to the next depth plane of the tile grid)
  int ldv, run_blocks, plane_runs;
  long long jump, jump2;
  // the same plans for gemm_rows_kernel: pieces per run, runs in all, and what the first row of
  // a run moves by from one run to the next / beyond that from one plane to the next (rows of V)
  int n_run, total_runs, run_rows, plane_extra;
  // direct form (gemm_kernel<..., DIRECT>): the rows of the V operand are the pixels of x itself, row p of the product
  // is output pixel (b, oy, ox) and starts at input pixel (stride oy - pad_h, stride ox - pad_w); the reduction walks
  // the taps (kx fastest: the next pixel, then the next image row) with cblocks reduction blocks per tap; taps that
  // fall outside the image contribute zeros; `bias` (K values, may be null) is added before the result is rounded
  int H, W, oH, oW, conv_stride, pad_h, pad_w, kw, cblocks;
  const void* bias;
  // direct form writing every o_step-th pixel of a larger image (the input gradient of a strided layer, one launch per
  // parity class of its pixels): row (b, oy, ox) of the product goes to pixel (o_step oy + o_y0, o_step ox + o_x0) of
  // image b of an (o_H, o_W) tensor; o_step == 0: rows are written one after the other
  int o_step, o_y0, o_x0, o_H, o_W;
};

typedef uint32_t Chunk16 __attribute__((ext_vector_type(4)));   // one 16-byte global/LDS access

// Operand rows in LDS are 64 bytes (four 16-byte chunks) with no padding; chunk c of row r sits
// at position c ^ swizzle(r).  A workgroup pass writes whole rows, so stores touch every bank
// once.  Fragment reads take the same chunk of consecutive rows: the swizzle gives rows of equal
// r mod 2 among 8 consecutive rows, and rows of equal r mod 4 among 16, distinct positions, which
// is conflict-free for 128-byte and for 256-byte wide bank sets alike.
__device__ __forceinline__ int swizzle(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }

template <typename T, int WM, int WN, int BK, int NWP = 2, int NWK = 2, bool SHIFT = false, bool DIRECT = false>
__global__ __launch_bounds__(64 * NWP * NWK, (WM * WN <= 8 && NWP * NWK == 4 ? 2 : 1)) void gemm_kernel(GemmArgs g) {
  static_assert(!DIRECT || SHIFT, "the direct form walks the taps like the shifted operand");
  using MF = Mfma<T>;
  constexpr int NT = 64 * NWP * NWK;               // threads: NWP x NWK wavefronts
  constexpr int BM = 32 * NWP * WM, BN = 32 * NWK * WN;
  constexpr int EPC = 16 / sizeof(T);              // elements per 16-byte chunk
  constexpr int CPR = BK / EPC;                    // chunks per tile row
  constexpr int LDS_STRIDE = BK;                   // unpadded row; the chunks of a row are swizzled
  constexpr int ROWS = BM + BN;
  constexpr int RPP = NT / CPR;                    // rows covered by one pass of the workgroup
  constexpr int NLOAD = ROWS / RPP;
  constexpr int STAGE = ROWS * LDS_STRIDE;         // elements per LDS stage
  static_assert(ROWS % RPP == 0 && BM % RPP == 0, "tile rows must be a multiple of the load pass");
  static_assert(CPR == 4 && RPP % 16 == 0, "the swizzle assumes 64-byte rows and passes of whole 16-row groups");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);

  const int blk = xcd_remap(blockIdx.x, g.per_xcd);
  if (blk >= g.n_blocks) return;
  const int kt_ = blk % g.tiles_k;
  const int pt = (blk / g.tiles_k) % g.tiles_p;
  const int t = blk / (g.tiles_k * g.tiles_p);
  const int p0 = pt * BM, k0 = kt_ * BN;

  const T* Vt = static_cast<const T*>(g.V) + (long long)t * g.sV;
  const T* Ut = static_cast<const T*>(g.U) + (long long)t * g.sU;

  const int tid = threadIdx.x;
  const int lrow = tid / CPR, lpart = tid % CPR;
  const T* gptr[NLOAD];
  int loff[NLOAD];
  int iy0[DIRECT ? BM / RPP : 1], ix0[DIRECT ? BM / RPP : 1];   // first input pixel of each V row this thread loads
#pragma unroll
  for (int i = 0; i < NLOAD; ++i) {
    const int row = lrow + i * RPP;                // row of the stacked [X ; W] tile
    if (row < BM) {
      const int p = min(p0 + row, g.P - 1);
      if constexpr (DIRECT) {
        const int per = g.oH * g.oW;
        const int b = p / per, rem = p - b * per;
        const int oy = rem / g.oW, ox = rem - oy * g.oW;
        iy0[i] = oy * g.conv_stride - g.pad_h;
        ix0[i] = ox * g.conv_stride - g.pad_w;
        gptr[i] = Vt + (((long long)b * g.H + iy0[i]) * g.W + ix0[i]) * g.ldv + lpart * EPC;
      } else {
        gptr[i] = Vt + (long long)p * (SHIFT ? g.ldv : g.Cp) + lpart * EPC;
      }
    } else {
      const int k = min(k0 + row - BM, g.K - 1);
      gptr[i] = Ut + (long long)k * g.Cp + lpart * EPC;
    }
    loff[i] = row * LDS_STRIDE + (lpart ^ swizzle(row)) * EPC;
  }

  Chunk16 regs[NLOAD];
  // `vshift`: what the V operand has jumped by at reduction block kt (rows i < BM / RPP are V's)
  int tap_y = 0, tap_x = 0, tap_cb = 0;             // direct form: the tap and channel block of the next load
  auto gload = [&](int kt, long long vshift) {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) {
      if constexpr (DIRECT) {
        if (i < BM / RPP) {
          const int j = i < BM / RPP ? i : 0;
          const bool inside = (unsigned)(iy0[j] + tap_y) < (unsigned)g.H && (unsigned)(ix0[j] + tap_x) < (unsigned)g.W;
          regs[i] = Chunk16{0u, 0u, 0u, 0u};
          if (inside) regs[i] = *reinterpret_cast<const Chunk16*>(gptr[i] + kt * BK + vshift);
          continue;
        }
      }
      regs[i] = *reinterpret_cast<const Chunk16*>(gptr[i] + kt * BK + (SHIFT && i < BM / RPP ? vshift : 0));
    }
    if constexpr (DIRECT) {
      if (++tap_cb == g.cblocks) {
        tap_cb = 0;
        if (++tap_x == g.kw) { tap_x = 0; ++tap_y; }
      }
    }
  };
  auto lstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NLOAD; ++i) *reinterpret_cast<Chunk16*>(lds + buf * STAGE + loff[i]) = regs[i];
  };

  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave / NWK, wk = wave % NWK;
  const int l32 = lane & 31, lhi = lane >> 5;
  // fragment read offsets inside a stage (elements); all rows a lane reads share l32's swizzle
  const int xoff = (wp * WM * 32 + l32) * LDS_STRIDE;
  const int woff = (BM + wk * WN * 32 + l32) * LDS_STRIDE;
  const int fz = swizzle(l32);
  auto koff = [&](int kk) {                        // element kk*kstep + lhi*kpack of a swizzled row
    const int e = kk * MF::kstep + lhi * MF::kpack;
    return (((e / EPC) ^ fz) * EPC) + e % EPC;
  };

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  const int nk = g.Cp / BK;
  long long vshift = 0;
  int run_left = SHIFT ? g.run_blocks : 0, plane_left = SHIFT ? g.plane_runs : 0;
  gload(0, 0);
  lstore(0);
  __syncthreads();
  for (int kt = 0; kt < nk; ++kt) {
    const int cur = kt & 1;
    if constexpr (SHIFT) {
      if (--run_left == 0) {
        vshift += g.jump;
        run_left = g.run_blocks;
        if (--plane_left == 0) { vshift += g.jump2; plane_left = g.plane_runs; }
      }
    }
    if (kt + 1 < nk) gload(kt + 1, vshift);
    const T* st = lds + cur * STAGE;
    // fragments of step kk+1 are read from LDS while the MFMAs of step kk run
    constexpr int KK = BK / MF::kstep;
    typename MF::Frag xf[2][WM], wf[2][WN];
    auto fload = [&](int kk, int b) {
      const int ko = koff(kk);
#pragma unroll
      for (int i = 0; i < WM; ++i)
        xf[b][i] = *reinterpret_cast<const typename MF::Frag*>(st + xoff + i * 32 * LDS_STRIDE + ko);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        wf[b][j] = *reinterpret_cast<const typename MF::Frag*>(st + woff + j * 32 * LDS_STRIDE + ko);
    };
    fload(0, 0);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) fload(kk + 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);   // keep the LDS reads above ahead of the MFMAs below
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = MF::run(wf[kk & 1][j], xf[kk & 1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
    if (kt + 1 < nk) lstore(cur ^ 1);
    __syncthreads();
  }

  // Epilogue through LDS so that global stores are whole rows.  Accumulator (i, j), register
  // 4q + e holds output channel 32j + 8q + 4*lhi + e of tile row 32i + l32.  The tile is staged
  // EI accumulator rows at a time (all of them for fp16; one for fp32, whose full tile would need
  // 135 KB and leave room for only one workgroup per CU).
  constexpr int EI = sizeof(T) == 4 ? 1 : (NWP * NWK == 4 ? WM : WM / 2);
  constexpr int CS = BN + EPC;                     // padded row of the staged output tile
  constexpr int SROWS = 32 * NWP * EI;             // staged rows per pass: NWP wavefront rows x EI x 32
  T* cs = lds;   // operand stages are free after the last barrier; the launch sizes LDS for both uses
  T* Mt = static_cast<T*>(g.M) + (long long)t * g.sM;
  constexpr int CPRO = BN / EPC;                   // 16-byte chunks per output row
  constexpr int RPPO = NT / CPRO;                  // rows per pass
  static_assert(NT % CPRO == 0 && SROWS % RPPO == 0, "output tile shape");
  const int orow = tid / CPRO, ocol = (tid % CPRO) * EPC;
#pragma unroll
  for (int i0 = 0; i0 < WM; i0 += EI) {
    if (i0 > 0) __syncthreads();                   // the previous pass has been read out
#pragma unroll
    for (int ii = 0; ii < EI; ++ii)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          Pack<T, 4> o;
          float bv[4] = {0.f, 0.f, 0.f, 0.f};
          if constexpr (DIRECT) {
            if (g.bias) {
              const int kb = k0 + wk * WN * 32 + j * 32 + 8 * q + 4 * lhi;
#pragma unroll
              for (int e = 0; e < 4; ++e)
                if (kb + e < g.K) bv[e] = static_cast<float>(static_cast<const T*>(g.bias)[kb + e]);
            }
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i0 + ii][j][4 * q + e] + bv[e]);
          *reinterpret_cast<Pack<T, 4>*>(cs + (wp * EI * 32 + ii * 32 + l32) * CS + wk * WN * 32 + j * 32 + 8 * q + 4 * lhi) = o;
        }
    __syncthreads();
    if (k0 + ocol < g.ldm) {
#pragma unroll
      for (int r = 0; r < SROWS / RPPO; ++r) {
        const int srow = orow + r * RPPO;            // staged row: wavefront row, then (ii, l32)
        const int row = (srow / (EI * 32)) * WM * 32 + i0 * 32 + srow % (EI * 32);
        if (p0 + row < g.P) {
          long long orow = p0 + row;
          if constexpr (DIRECT) {
            if (g.o_step) {
              const int per = g.oH * g.oW;
              const int b = (p0 + row) / per, rem = (p0 + row) - b * per;
              const int oy = rem / g.oW, ox = rem - oy * g.oW;
              orow = ((long long)b * g.o_H + oy * g.o_step + g.o_y0) * g.o_W + ox * g.o_step + g.o_x0;
            }
          }
          *reinterpret_cast<Chunk16*>(Mt + orow * g.ldm + k0 + ocol) =
              *reinterpret_cast<const Chunk16*>(cs + srow * CS + ocol);
        }
      }
    }
  }
}

using GemmKernel = void (*)(GemmArgs);

struct GemmConfig {
  GemmKernel fn;
  int bm, bn, bk;
  size_t lds;
  int threads;
};

template <typename T, int WM, int WN, int BK, int NWP = 2, int NWK = 2, bool SHIFT = false, bool DIRECT = false>
static GemmConfig make_config() {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int BM = 32 * NWP * WM, BN = 32 * NWK * WN;
  constexpr int EI = sizeof(T) == 4 ? 1 : (NWP * NWK == 4 ? WM : WM / 2);
  constexpr size_t stages = (size_t)2 * (BM + BN) * BK * sizeof(T);
  constexpr size_t out_tile = (size_t)32 * NWP * EI * (BN + EPC) * sizeof(T);
  return GemmConfig{&gemm_kernel<T, WM, WN, BK, NWP, NWK, SHIFT, DIRECT>, BM, BN, BK,
                    stages > out_tile ? stages : out_tile, 64 * NWP * NWK};
}

// The shifted product with the pieces of one run served by ONE operand tile.  Piece b of a run
// multiplies rows p + b of V, so a tile of BM + n_run - 1 rows holds what all n_run pieces of the
// run need from one block of 32 channels: the reduction runs (run, channel block, piece) with the
// piece innermost, V is loaded once per (run, channel block) instead of once per piece, and only
// the filter block changes from step to step.  The shifted gemm_kernel is bound by L2-to-LDS
// traffic (every piece loads its own copy of nearly the same rows); this form loads
// (BM + n_run - 1 + n_run BN) rows per run and channel block instead of n_run (BM + BN).
// LDS: two stages of V (BM + kRunExtra rows) and two of U (BN rows); the V block of the next
// (run, channel block) is requested at the first piece of the current one and parked in
// registers until the last piece.  The accumulation order differs from gemm_kernel's (pieces of a
// run alternate), so results agree to fp32 rounding, not bit for bit.
constexpr int kRunExtra = 8;       // pieces per run are at most kRunExtra + 1

template <typename T, int WM, int WN, int NWP, int NWK>
__global__ __launch_bounds__(64 * NWP * NWK, (WM * WN <= 8 && NWP * NWK == 4 ? 2 : 1)) void gemm_rows_kernel(GemmArgs g) {
  using MF = Mfma<T>;
  constexpr int BK = 32;
  constexpr int NT = 64 * NWP * NWK;
  constexpr int BM = 32 * NWP * WM, BN = 32 * NWK * WN;
  constexpr int EPC = 16 / sizeof(T);
  constexpr int CPR = BK / EPC;
  constexpr int RPP = NT / CPR;                    // rows covered by one pass of the workgroup
  constexpr int NLV = BM / RPP, NLU = BN / RPP;
  constexpr int VSTAGE = (BM + kRunExtra) * BK, USTAGE = BN * BK;
  static_assert(sizeof(T) == 2 && CPR == 4 && RPP % 16 == 0, "16-bit operands in 64-byte swizzled rows");
  static_assert(BM % RPP == 0 && BN % RPP == 0 && kRunExtra <= RPP, "tile rows must be a multiple of the load pass");

  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  T* lds = reinterpret_cast<T*>(lds_raw);
  T* ldsV = lds;
  T* ldsU = lds + 2 * VSTAGE;

  const int blk = xcd_remap(blockIdx.x, g.per_xcd);
  if (blk >= g.n_blocks) return;
  const int kt_ = blk % g.tiles_k;
  const int pt = (blk / g.tiles_k) % g.tiles_p;
  const int t = blk / (g.tiles_k * g.tiles_p);
  const int p0 = pt * BM, k0 = kt_ * BN;
  const int n_run = g.n_run;

  const T* Vt = static_cast<const T*>(g.V) + (long long)t * g.sV;
  const T* Ut = static_cast<const T*>(g.U) + (long long)t * g.sU;

  const int tid = threadIdx.x;
  const int lrow = tid / CPR, lpart = tid % CPR;
  // rows past the last tile of the grid still lie inside V's tail for every piece of the run
  const int last_row = g.P - 1 + n_run - 1;
  const T* vptr[NLV + 1];
  int vloff[NLV + 1];
#pragma unroll
  for (int i = 0; i <= NLV; ++i) {
    const int row = lrow + i * RPP;                // i == NLV: the n_run - 1 rows beyond the tile
    vptr[i] = Vt + (long long)min(p0 + row, last_row) * g.ldv + lpart * EPC;
    vloff[i] = row * BK + (lpart ^ swizzle(row)) * EPC;
  }
  const bool has_extra = lrow < n_run - 1;
  const T* uptr[NLU];
  int uloff[NLU];
#pragma unroll
  for (int i = 0; i < NLU; ++i) {
    const int row = lrow + i * RPP;
    uptr[i] = Ut + (long long)min(k0 + row, g.K - 1) * g.Cp + lpart * EPC;
    uloff[i] = row * BK + (lpart ^ swizzle(row)) * EPC;
  }

  Chunk16 vregs[NLV + 1], uregs[NLU];
  auto vload_extra = [&](long long off) {
    if (has_extra) vregs[NLV] = *reinterpret_cast<const Chunk16*>(vptr[NLV] + off);
  };
  auto vload = [&](long long off) {
#pragma unroll
    for (int i = 0; i < NLV; ++i) vregs[i] = *reinterpret_cast<const Chunk16*>(vptr[i] + off);
  };
  auto vstore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NLV; ++i) *reinterpret_cast<Chunk16*>(ldsV + buf * VSTAGE + vloff[i]) = vregs[i];
    if (has_extra) *reinterpret_cast<Chunk16*>(ldsV + buf * VSTAGE + vloff[NLV]) = vregs[NLV];
  };
  auto uload = [&](long long off) {
#pragma unroll
    for (int i = 0; i < NLU; ++i) uregs[i] = *reinterpret_cast<const Chunk16*>(uptr[i] + off);
  };
  auto ustore = [&](int buf) {
#pragma unroll
    for (int i = 0; i < NLU; ++i) *reinterpret_cast<Chunk16*>(ldsU + buf * USTAGE + uloff[i]) = uregs[i];
  };

  const int lane = tid & 63, wave = tid >> 6;
  const int wp = wave / NWK, wk = wave % NWK;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int xrow = wp * WM * 32 + l32;             // first V row of this lane (piece 0)
  const int woff = (wk * WN * 32 + l32) * BK;
  const int fzw = swizzle(l32);
  auto koff = [&](int kk, int fz) {                // element kk*kstep + lhi*kpack of a swizzled row
    const int e = kk * MF::kstep + lhi * MF::kpack;
    return (((e / EPC) ^ fz) * EPC) + e % EPC;
  };

  floatx16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  // A group is one (run, channel block); its V block sits at element offset nv of a V row, the
  // filter block of its piece b at offset (run n_run + b) ldv + 32 cc of a U row.  Every group
  // is the same straight line of loads, waits and stores (first piece, middle pieces, last piece;
  // the last group requests a block it never uses), so that the compiler can count what is in
  // flight at each wait.  Loads return in order: the filter block of the next step is requested
  // BEFORE the V block of the next group, and the end of the first step waits for it alone.
  const int ncc = g.ldv / BK;
  const int groups = g.total_runs * ncc;
  long long nv = 0;                                // V offset of the next group
  int ncc_left = ncc, plane_left = g.plane_runs;
  long long row_shift = 0;
  auto advance_v = [&]() {
    if (--ncc_left > 0) { nv += BK; return; }
    ncc_left = ncc;
    row_shift += g.run_rows;
    if (--plane_left == 0) { row_shift += g.plane_extra; plane_left = g.plane_runs; }
    nv = row_shift * g.ldv;
  };
  long long lu_run = 0;                            // U cursor: the next step to request
  int lu_b = 0, lu_cc = 0, lu_left = groups * n_run;
  auto next_u = [&]() {                            // its offset (0 past the end), then move it on
    const long long off = lu_left > 0 ? lu_run + (long long)lu_b * g.ldv + lu_cc * BK : 0;
    --lu_left;
    if (++lu_b == n_run) {
      lu_b = 0;
      if (++lu_cc == ncc) { lu_cc = 0; lu_run += (long long)n_run * g.ldv; }
    }
    return off;
  };
  auto multiply = [&](const T* stv, const T* stu, int b) {
    const int xoff = (xrow + b) * BK;
    const int fzx = swizzle(l32 + b);
    constexpr int KK = BK / MF::kstep;
    typename MF::Frag xf[2][WM], wf[2][WN];
    auto fload = [&](int kk, int sb) {
      const int kx = koff(kk, fzx), kw = koff(kk, fzw);
#pragma unroll
      for (int i = 0; i < WM; ++i)
        xf[sb][i] = *reinterpret_cast<const typename MF::Frag*>(stv + xoff + i * 32 * BK + kx);
#pragma unroll
      for (int j = 0; j < WN; ++j)
        wf[sb][j] = *reinterpret_cast<const typename MF::Frag*>(stu + woff + j * 32 * BK + kw);
    };
    fload(0, 0);
#pragma unroll
    for (int kk = 0; kk < KK; ++kk) {
      if (kk + 1 < KK) fload(kk + 1, (kk + 1) & 1);
      __builtin_amdgcn_sched_barrier(0);
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) acc[i][j] = MF::run(wf[kk & 1][j], xf[kk & 1][i], acc[i][j]);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  vload_extra(0);
  uload(next_u());
  vload(0);
  advance_v();
  vstore(0);
  ustore(0);
  __syncthreads();
  int ub = 0;                                      // U stage of the current step
  for (int gi = 0; gi < groups; ++gi) {
    const long long vnext = gi + 1 < groups ? nv : 0;
    const T* stv = ldsV + (gi & 1) * VSTAGE;
    // first piece: request the next filter block, then the next group's V block
    vload_extra(vnext);
    uload(next_u());
    vload(vnext);
    multiply(stv, ldsU + ub * USTAGE, 0);
    ustore(ub ^ 1);
    __syncthreads();
    ub ^= 1;
    for (int b = 1; b < n_run - 1; ++b) {
      uload(next_u());
      multiply(stv, ldsU + ub * USTAGE, b);
      ustore(ub ^ 1);
      __syncthreads();
      ub ^= 1;
    }
    // last piece: the V block moves from registers to the other stage
    uload(next_u());
    multiply(stv, ldsU + ub * USTAGE, n_run - 1);
    vstore((gi + 1) & 1);
    ustore(ub ^ 1);
    __syncthreads();
    ub ^= 1;
    advance_v();
  }

  // Epilogue as in gemm_kernel: the tile goes through LDS so that global stores are whole rows.
  constexpr int EI = NWP * NWK == 4 ? WM : WM / 2;
  constexpr int CS = BN + EPC;
  constexpr int SROWS = 32 * NWP * EI;
  T* cs = lds;
  T* Mt = static_cast<T*>(g.M) + (long long)t * g.sM;
  constexpr int CPRO = BN / EPC;
  constexpr int RPPO = NT / CPRO;
  static_assert(EI >= 1 && WM % EI == 0 && NT % CPRO == 0 && SROWS % RPPO == 0, "output tile shape");
  const int orow = tid / CPRO, ocol = (tid % CPRO) * EPC;
#pragma unroll
  for (int i0 = 0; i0 < WM; i0 += EI) {
    if (i0 > 0) __syncthreads();
#pragma unroll
    for (int ii = 0; ii < EI; ++ii)
#pragma unroll
      for (int j = 0; j < WN; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          Pack<T, 4> o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i0 + ii][j][4 * q + e]);
          *reinterpret_cast<Pack<T, 4>*>(cs + (wp * EI * 32 + ii * 32 + l32) * CS + wk * WN * 32 + j * 32 + 8 * q + 4 * lhi) = o;
        }
    __syncthreads();
    if (k0 + ocol < g.ldm) {
#pragma unroll
      for (int r = 0; r < SROWS / RPPO; ++r) {
        const int srow = orow + r * RPPO;
        const int row = (srow / (EI * 32)) * WM * 32 + i0 * 32 + srow % (EI * 32);
        if (p0 + row < g.P)
          *reinterpret_cast<Chunk16*>(Mt + (long long)(p0 + row) * g.ldm + k0 + ocol) =
              *reinterpret_cast<const Chunk16*>(cs + srow * CS + ocol);
      }
    }
  }
}

template <typename T, int WM, int WN, int NWP, int NWK>
static GemmConfig make_rows_config() {
  constexpr int EPC = 16 / sizeof(T);
  constexpr int BM = 32 * NWP * WM, BN = 32 * NWK * WN;
  constexpr int EI = NWP * NWK == 4 ? WM : WM / 2;
  constexpr size_t stages = (size_t)2 * (BM + kRunExtra + BN) * 32 * sizeof(T);
  constexpr size_t out_tile = (size_t)32 * NWP * EI * (BN + EPC) * sizeof(T);
  return GemmConfig{&gemm_rows_kernel<T, WM, WN, NWP, NWK>, BM, BN, 32, stages > out_tile ? stages : out_tile,
                    64 * NWP * NWK};
}

// Tile shapes: 0..4 four wavefronts, largest first; 5 (16-bit types) 128 x 256 with eight wavefronts.
template <typename T> struct Configs;
template <> struct Configs<half_t> {
  static constexpr int n = 7;
  static GemmConfig get(int i) {
    switch (i) {
      case 6: return make_config<half_t, 4, 4, 32>();   // 256 x 256, four wavefronts of 128 x 128
      case 0: return make_config<half_t, 4, 2, 32>();   // 256 x 128
      case 1: return make_config<half_t, 2, 2, 32>();   // 128 x 128
      case 2: return make_config<half_t, 4, 1, 32>();   // 256 x 64
      case 3: return make_config<half_t, 2, 1, 32>();   // 128 x 64
      case 4: return make_config<half_t, 1, 1, 32>();   // 64 x 64
      default: return make_config<half_t, 2, 2, 32, 2, 4>();  // 128 x 256, 8 wavefronts
    }
  }
};
template <> struct Configs<bf16_t> {
  static constexpr int n = 6;
  static GemmConfig get(int i) {
    switch (i) {
      case 0: return make_config<bf16_t, 4, 2, 32>();
      case 1: return make_config<bf16_t, 2, 2, 32>();
      case 2: return make_config<bf16_t, 4, 1, 32>();
      case 3: return make_config<bf16_t, 2, 1, 32>();
      case 4: return make_config<bf16_t, 1, 1, 32>();
      default: return make_config<bf16_t, 2, 2, 32, 2, 4>();
    }
  }
};
template <> struct Configs<float> {
  static constexpr int n = 5;
  static GemmConfig get(int i) {
    switch (i) {
      case 0: return make_config<float, 4, 2, 16>();
      case 1: return make_config<float, 2, 2, 16>();
      case 2: return make_config<float, 4, 1, 16>();
      case 3: return make_config<float, 2, 1, 16>();
      default: return make_config<float, 1, 1, 16>();
    }
  }
};

// fp16: the largest tile that still gives the 256 CUs about two workgroups each and does not
// waste more than half a tile on the channel axis (the big tile moves the fewest bytes, and the
// fp16 product is bound by memory).  fp32: always the 64 x 64 tile.  One reduction step of an
// fp32 stage is only 16 deep, so a big tile has too little work per stage to cover the load
// latency with one or two workgroups per CU; the small tile runs 4+ workgroups per CU and
// measured 1.0-1.3x faster than every larger tile on all VGG-16 layer shapes (N = 8), within 4 %
// of the best tile on each.
template <typename T>
static GemmConfig choose(int T_, int P, int K, int Cp) {
  const int force = test_gemm_config();
  if (force >= 0 && force < Configs<T>::n) return Configs<T>::get(force);
  constexpr int n_auto = 5;
  // fp32 is bound by the MFMA rate: the 64 x 64 tile fills the chip best, except for long
  // reductions with thousands of tiles, where 128 x 128 halves the LDS traffic (measured 5-9 %
  // faster at Cp >= 256).  A reduction of <= 64 channels is one or two stages: small tiles again.
  if constexpr (sizeof(T) == 4) {
    if (Cp >= 256 && K >= 128 && (long long)ceil_div(P, 128) * ceil_div(K, 128) * T_ >= 2048) return Configs<T>::get(1);
  }
  if (sizeof(T) == 4 || Cp <= 64) return Configs<T>::get(n_auto - 1);
  // Long reductions over many output channels: the 128 x 256 tile of eight wavefronts reads V
  // once per 256 channels (measured 3-13 % faster than any four-wavefront tile for Cp >= 512 from four rounds of
  // tiles on; at 576 tiles - N = 64, 512 -> 512 channels at 14 x 14 - the 128 x 128 tile is 6 % ahead, 0.055 against
  // 0.059 ms per layer).
  if constexpr (sizeof(T) == 2) {
    if (Cp >= 512 && K >= 256 && (long long)ceil_div(P, 128) * ceil_div(K, 256) * T_ >= 1024) return Configs<T>::get(5);
  }
  GemmConfig best = Configs<T>::get(n_auto - 1);
  for (int i = 0; i < n_auto; ++i) {
    GemmConfig c = Configs<T>::get(i);
    if (c.bn > 64 && c.bn / 2 >= K) continue;                 // half of the tile would be padding
    const long long blocks = (long long)ceil_div(P, c.bm) * ceil_div(K, c.bn) * T_;
    // The 256 x 128 tile runs two workgroups per CU: 512 are resident at once.  It is the best tile when it fills
    // that once (fp16 N = 64, F(4,3): 384 -> 384 channels at 14 x 14, 432 tiles, 0.040 ms per layer against 0.044 for the
    // next best; 128 -> 128 and 256 -> 128 at 28 x 28, 468 tiles, 0.036 | 0.038 and 0.046 | 0.048) and the worst when a few
    // tiles are left for a second round (512 -> 512 at 14 x 14, 576 tiles: 0.062 against 0.055 on 128 x 128; N = 32
    // 256 -> 384 at 28 x 28, 756 tiles: 0.052 | 0.050); from two full rounds on the tail no longer decides.
    const bool ok = i == 0 ? (blocks >= 1024 || (blocks >= 400 && blocks <= 512)) : blocks >= 512;
    if (ok || i == n_auto - 1) { best = c; break; }
  }
  return best;
}

// Tiles for the shifted operand (16-bit types).  Measured at N=32, 112x112, 5x5 / 7x7 kernels: 256 x 128 with
// eight wavefronts is 2-6 % faster than with four, 256 x 64 is 25 % faster than either for 64 output
// channels; smaller tiles where those would leave CUs idle.
template <typename T>
static GemmConfig choose_shifted(int T_, int P, int K) {
  auto blocks = [&](const GemmConfig& c) { return (long long)ceil_div(P, c.bm) * ceil_div(K, c.bn) * T_; };
  if (K > 64) {
    GemmConfig big = make_config<T, 2, 2, 32, 4, 2, true>();   // 256 x 128, eight wavefronts
    if (blocks(big) >= 512) return big;
    GemmConfig mid = make_config<T, 2, 2, 32, 2, 2, true>();   // 128 x 128
    if (blocks(mid) >= 512) return mid;
  } else if (K > 32) {
    GemmConfig tall = make_config<T, 4, 1, 32, 2, 2, true>();  // 256 x 64
    if (blocks(tall) >= 512) return tall;
  }
  return make_config<T, 1, 1, 32, 2, 2, true>();               // 64 x 64
}

// Tiles of gemm_rows_kernel.  Measured at N=32, 128 channels, 112x112, 5x5 / 7x7 kernels and at
// 3-D 5x5x5 kernels: 256 x 128 with four wavefronts is 8-15 % faster than the tile per piece
// (eight wavefronts are slower than either: their 64 x 64 wavefront tiles read more of LDS per
// MFMA, and that is the bound once the operand traffic is halved); 128 x 128 wins 8-10 % below about
// 2000 big tiles (256 channels at 56x56, small 3-D problems); small problems keep the tile per
// piece (no kernel: fn == nullptr).
template <typename T>
static GemmConfig choose_rows(int T_, int P, int K, bool always) {
  auto blocks = [&](const GemmConfig& c) { return (long long)ceil_div(P, c.bm) * ceil_div(K, c.bn) * T_; };
  if (K <= 64 && !always) {
    GemmConfig tall = make_rows_config<T, 4, 1, 2, 2>();       // 256 x 64
    if (blocks(tall) >= 512) return tall;
    return GemmConfig{nullptr, 0, 0, 0, 0, 0};
  }
  GemmConfig big = make_rows_config<T, 4, 2, 2, 2>();       // 256 x 128
  if (blocks(big) >= 2048 && !always) return big;                         // four rounds of two workgroups per CU
  GemmConfig mid = make_rows_config<T, 2, 2, 2, 2>();       // 128 x 128
  if (blocks(mid) >= 512 || always) return mid;
  return GemmConfig{nullptr, 0, 0, 0, 0, 0};
}

int batched_gemm_shifted(const void* V, const void* U, void* M, int T_, int P, int Cp, SharedShift sh, int K, int ldm,
                         int dtype, void* stream) {
  WC_CHECK_ARG(V && U && M, "batched_gemm_shifted: null pointer");
  WC_CHECK_ARG(T_ > 0 && P > 0 && K > 0 && Cp > 0 && Cp % 32 == 0, "batched_gemm_shifted: T %d, P %d, K %d, Cp %d", T_, P, K, Cp);
  WC_CHECK_ARG(sh.n_run > 0 && sh.n_runs > 0 && sh.n_planes > 0 && sh.run_rows >= sh.n_run &&
                   sh.plane_rows >= sh.n_runs * sh.run_rows &&
                   sh.tail == (sh.n_planes - 1) * sh.plane_rows + (sh.n_runs - 1) * sh.run_rows + sh.n_run - 1,
               "batched_gemm_shifted: bad shift description");
  WC_CHECK_ARG(ldm >= K && ldm % 8 == 0, "batched_gemm_shifted: row stride %d", ldm);
  if (dtype != WC_F16 && dtype != WC_BF16) return fail(WC_ERR_UNSUPPORTED, "batched_gemm_shifted: 16-bit types only");
  GemmConfig c = dtype == WC_F16 ? choose_shifted<half_t>(T_, P, K) : choose_shifted<bf16_t>(T_, P, K);
  // Runs of two and more pieces over more than 64 output channels, on problems that fill the chip
  // with 128-row tiles: one operand tile per run.  wc_test_gemm_override(., 0) keeps the tile per
  // piece, (., 2) takes the 128 x 128 tile of gemm_rows_kernel for every plan with runs (what the
  // tests use to reach it with small shapes).
  const int rows_mode = test_gemm_rows();
  // Runs of two to five pieces on at least two rounds of 512 x 128 tiles whose last block of 128 channels is at least
  // three quarters full: the persistent kernel fed by LDS-DMA (3-13 % ahead of gemm_rows_kernel there, behind it on
  // fewer tiles and on 64 channels), with a tile's results written out during the next tile's first steps wherever a
  // tile has the steps for that (2-6 % again).  wc_test_gemm_override(., 3) takes the kernel wherever it runs with the
  // write-out at the end of each tile, (., 4) with the write-out riding on the next tile wherever that fits.
  if (gemm_rows_dma_fits(sh, P, Cp, K, dtype) &&
      (rows_mode >= 3 || (rows_mode == 1 && (K % 128 == 0 || K % 128 >= 96) &&
                          (long long)ceil_div(P, 512) * ceil_div(K, 128) * T_ >= 2 * kCus)))
    return gemm_rows_dma(V, U, M, T_, P, Cp, sh, K, ldm, dtype, rows_mode != 3 && gemm_rows_dma_deferred_fits(sh, P, Cp, ldm), stream);
  bool rows = sh.n_run >= 2 && sh.n_run <= kRunExtra + 1 && rows_mode != 0 && (K > 32 || rows_mode == 2);
  if (rows) {
    GemmConfig r = dtype == WC_F16 ? choose_rows<half_t>(T_, P, K, rows_mode == 2) : choose_rows<bf16_t>(T_, P, K, rows_mode == 2);
    if (r.fn) c = r; else rows = false;
  }
  GemmArgs g;
  g.V = V; g.U = U; g.M = M;
  g.P = P; g.K = K; g.ldm = ldm;
  g.Cp = sh.n_planes * sh.n_runs * sh.n_run * Cp;        // reduction length = row length of U
  g.ldv = Cp;
  g.run_blocks = sh.n_run * Cp / c.bk;                   // one run: the pieces of one piece row, contiguous rows of V
  g.jump = (long long)(sh.run_rows - sh.n_run) * Cp;     // on to the same tile one grid row further
  g.plane_runs = sh.n_runs;
  g.jump2 = (long long)(sh.plane_rows - sh.n_runs * sh.run_rows) * Cp;   // ... and one grid plane further
  g.H = g.W = g.oH = g.oW = g.conv_stride = g.pad_h = g.pad_w = g.kw = g.cblocks = 0; g.bias = nullptr;
  g.o_step = g.o_y0 = g.o_x0 = g.o_H = g.o_W = 0;
  g.n_run = sh.n_run; g.total_runs = sh.n_planes * sh.n_runs;
  g.run_rows = sh.run_rows; g.plane_extra = sh.plane_rows - sh.n_runs * sh.run_rows;
  g.sV = (long long)(P + sh.tail) * Cp; g.sU = (long long)K * g.Cp; g.sM = (long long)P * ldm;
  g.tiles_p = ceil_div(P, c.bm); g.tiles_k = ceil_div(K, c.bn); g.T = T_;
  const long long blocks = (long long)g.tiles_p * g.tiles_k * T_;
  WC_CHECK_ARG(blocks < (1ll << 30), "batched_gemm_shifted: problem too large");
  g.n_blocks = (int)blocks;
  g.per_xcd = ceil_div((int)blocks, kXcds);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(c.fn), c.lds)) return rc;
  hipLaunchKernelGGL(c.fn, dim3((unsigned)(g.per_xcd * kXcds)), dim3(c.threads), c.lds, as_stream(stream), g);
  WC_CHECK_LAUNCH(rows ? "gemm_rows_kernel" : "gemm_kernel (shifted operand)");
  return WC_OK;
}

// ---- 3-D F(2,3)^3 plans with the width axis taken directly inside the product ----------------------------------------
// Along the width nothing is transformed: V' = (B^T d B over depth and height) of every input pixel column, 16 elements
// per tile of 2 x 2 x 1 outputs, one row of V' per pixel column of the padded image; the filter Uw (16, K, 3 Cp) holds,
// per (depth, height) element g, the three width taps side by side, each transformed along depth and height only.
// Output column x is then
//   M'[g][x] = sum over the taps kx of V'[g][x + kx] times Uw[g][kx]:
// the product of a plan whose pieces share one transformed input, with one run of three pieces (batched_gemm_shifted).
// M' has 16 elements per 2 x 2 x 1 outputs where F(2,3)^3 has 64 per 2 x 2 x 2, the output transform has nothing left
// to do along the width, and V' is read and written at half the size: 12 multiplications per output where F(2,3)^3 has
// 8, in a pipeline that waits for memory in every stage.  Uw comes from the ordinary U (64, K, Cp): with G of F(2,3) =
// [1 0 0; .5 .5 .5; .5 -.5 .5; 0 0 1] its width elements are g0, (g0 + g1 + g2) / 2, (g0 - g1 + g2) / 2, g2, so tap 0
// is element 0, tap 2 element 3, and tap 1 element 1 minus element 2.
__global__ __launch_bounds__(256) void fold_filter_kernel(const uint16_t* __restrict__ U, uint16_t* __restrict__ Uw, int K, int Cp,
                                                          int is_bf16, long long total) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= total) return;
  const int cv = Cp / 8;
  const int c8 = (int)(idx % cv);
  long long q = idx / cv;
  const int piece = (int)(q % 3); q /= 3;
  const int k = (int)(q % K);
  const int g = (int)(q / K);
  auto plane = [&](int e) { return U + ((long long)(4 * g + e) * K + k) * Cp + c8 * 8; };
  Chunk16 v;
  if (piece != 1) v = *reinterpret_cast<const Chunk16*>(plane(piece == 0 ? 0 : 3));
  else {
    const Chunk16 a = *reinterpret_cast<const Chunk16*>(plane(1)), b = *reinterpret_cast<const Chunk16*>(plane(2));
    uint16_t av[8], bv[8], ov[8];
    __builtin_memcpy(av, &a, 16); __builtin_memcpy(bv, &b, 16);
#pragma unroll
    for (int e = 0; e < 8; ++e) {
      if (is_bf16) {
        bf16_t x, y; __builtin_memcpy(&x, &av[e], 2); __builtin_memcpy(&y, &bv[e], 2);
        const bf16_t d = static_cast<bf16_t>(static_cast<float>(x) - static_cast<float>(y));
        __builtin_memcpy(&ov[e], &d, 2);
      } else {
        half_t x, y; __builtin_memcpy(&x, &av[e], 2); __builtin_memcpy(&y, &bv[e], 2);
        const half_t d = static_cast<half_t>(static_cast<float>(x) - static_cast<float>(y));
        __builtin_memcpy(&ov[e], &d, 2);
      }
    }
    __builtin_memcpy(&v, ov, 16);
  }
  *reinterpret_cast<Chunk16*>(Uw + (((long long)g * K + k) * 3 + piece) * Cp + c8 * 8) = v;
}

int fold_filter_w(const void* U, void* Uw, int K, int Cp, int dtype, void* stream) {
  WC_CHECK_ARG(U && Uw && K > 0 && Cp > 0 && Cp % 32 == 0 && (dtype == WC_F16 || dtype == WC_BF16), "fold_filter_w: K %d, Cp %d", K, Cp);
  const long long total = 16ll * K * 3 * (Cp / 8);
  hipLaunchKernelGGL(fold_filter_kernel, dim3((unsigned)ceil_div_ll(total, 256)), dim3(256), 0, as_stream(stream),
                     static_cast<const uint16_t*>(U), static_cast<uint16_t*>(Uw), K, Cp, dtype == WC_BF16, total);
  WC_CHECK_LAUNCH("fold_filter_kernel");
  return WC_OK;
}

// Tiles of the direct form, chosen like those of the shifted operand.
template <typename T>
static GemmConfig choose_direct(int P, int K) {
  constexpr int BK = sizeof(T) == 4 ? 16 : 32;
  auto blocks = [&](const GemmConfig& c) { return (long long)ceil_div(P, c.bm) * ceil_div(K, c.bn); };
  switch (test_gemm_config()) {                       // wc_test_gemm_override: a tile shape forced by a test
    case 0: return make_config<T, 2, 2, BK, 4, 2, true, true>();
    case 1: return make_config<T, 2, 2, BK, 2, 2, true, true>();
    case 2: return make_config<T, 4, 1, BK, 2, 2, true, true>();
    case 3: return make_config<T, 1, 1, BK, 2, 2, true, true>();
    case 4: return make_config<T, 4, 2, BK, 2, 2, true, true>();   // 256 x 128, four wavefronts
    default: break;
  }
  // Measured on MI355X (fp16, stride 2): the largest tile that still gives every compute unit a workgroup
  // wins: 256 x 128 over 128 x 128 by 15-25 % at 392 workgroups (N=32, C=K=128, 112x112: 54.9 against
  // 63.7 us; C=K=256, 56x56: 93.5 against 115 us), and loses by 40 % at 196.  Four wavefronts of 128 x 64
  // beat eight of 64 x 64 for the large tile (54.9 against 73.0 us): half the LDS reads per MFMA.
  // fp32 products are bound by the MFMA rate and fill the chip best with small tiles (as in choose()).
  if constexpr (sizeof(T) == 4) {
    GemmConfig mid = make_config<T, 2, 2, BK, 2, 2, true, true>();     // 128 x 128
    if (K > 64 && blocks(mid) >= 2048) return mid;
    return make_config<T, 1, 1, BK, 2, 2, true, true>();               // 64 x 64
  }
  if (K > 64) {
    GemmConfig big = make_config<T, 4, 2, BK, 2, 2, true, true>();   // 256 x 128, four wavefronts
    if (blocks(big) >= kCus) return big;
    GemmConfig mid = make_config<T, 2, 2, BK, 2, 2, true, true>();   // 128 x 128
    if (blocks(mid) >= kCus) return mid;
  }
  return make_config<T, 1, 1, BK, 2, 2, true, true>();               // 64 x 64
}

// y (N, oH, oW, K) = direct convolution of x (N, H, W, C) with U (K, kh kw C): the batched product with the
// pixels of x as its V operand (no transform, no intermediate in memory); C a multiple of the reduction block (32
// elements of a 16-bit type, 16 of fp32), K a multiple of 8.
int gemm_direct_conv(const void* x, const void* U, const void* bias, void* y, int N, int H, int W, int C, int K,
                     int kh, int kw, int stride, int pad_h, int pad_w, int oH, int oW, int dtype, void* stream,
                     int o_step, int o_y0, int o_x0, int o_H, int o_W) {
  WC_CHECK_ARG(x && U && y, "gemm_direct_conv: null pointer");
  WC_CHECK_ARG(dtype == WC_F16 || dtype == WC_BF16 || dtype == WC_F32, "gemm_direct_conv: dtype %d", dtype);
  const int cq = dtype == WC_F32 ? 16 : 32;
  WC_CHECK_ARG(C > 0 && C % cq == 0 && K > 0 && K % 8 == 0, "gemm_direct_conv: C %d (multiple of %d), K %d (multiple of 8)", C, cq, K);
  const long long P = (long long)N * oH * oW;
  WC_CHECK_ARG(P > 0 && P < (1ll << 31) && (long long)kh * kw * C < (1ll << 24), "gemm_direct_conv: problem too large");
  // Kernel rows of four and more taps over enough output to give a quarter of the CUs a 256 x 128 tile: one operand
  // tile per kernel row (direct_rows.hip).  Measured against the tile per tap, fp16, stride 2, ms: N=32, 128 channels,
  // 112x112: 4x4 0.091 | 0.102, 5x5 0.116 | 0.151, 7x7 0.181 | 0.264, 8x8 0.222 | 0.340; N=8: 7x7 0.081 | 0.122;
  // 256 channels on 56x56: 7x7 0.166 | 0.249; 256 -> 512 on 28x28, N=64: 5x5 0.100 | 0.137; stride 1, 128 channels
  // on 56x56: 5x5 0.103 | 0.135.  wc_test_gemm_override(., 2) takes it wherever it fits, (., 0) never.
  if (direct_rows_fits(N, C, K, kw, stride, oH, oW, dtype)) {
    const int mode = test_gemm_rows();
    const long long tiles = ceil_div_ll(P, 256) * ceil_div(K, 128);
    const bool k_fills = K % 128 == 0 || K % 128 >= 96;      // the last 128-channel tile is at least three quarters full
    if (mode == 2 || (mode != 0 && tiles >= 64 && k_fills))
      return direct_rows_conv(x, U, bias, y, N, H, W, C, K, kh, kw, stride, pad_h, pad_w, oH, oW, dtype, stream, o_step, o_y0,
                              o_x0, o_H, o_W);
  }
  GemmConfig c = dispatch_dtype(dtype, [&](auto t) { return choose_direct<decltype(t)>((int)P, K); });
  GemmArgs g;
  g.V = x; g.U = U; g.M = y; g.bias = bias;
  g.P = (int)P; g.K = K; g.ldm = K;
  g.Cp = kh * kw * C;                                    // reduction length = row length of U
  g.ldv = C;
  g.run_blocks = kw * C / c.bk;                          // one run: the taps of one kernel row, neighbouring pixels
  g.jump = (long long)(W - kw) * C;                      // on to the same column one image row further
  g.plane_runs = kh + 1; g.jump2 = 0;                    // one plane: never left
  g.n_run = kw; g.total_runs = kh; g.run_rows = W; g.plane_extra = 0;
  g.H = H; g.W = W; g.oH = oH; g.oW = oW; g.conv_stride = stride; g.pad_h = pad_h; g.pad_w = pad_w;
  g.kw = kw; g.cblocks = C / c.bk;
  g.o_step = o_step; g.o_y0 = o_y0; g.o_x0 = o_x0; g.o_H = o_H; g.o_W = o_W;
  g.sV = 0; g.sU = 0; g.sM = 0;
  g.tiles_p = ceil_div((int)P, c.bm); g.tiles_k = ceil_div(K, c.bn); g.T = 1;
  const long long blocks = (long long)g.tiles_p * g.tiles_k;
  g.n_blocks = (int)blocks;
  g.per_xcd = ceil_div((int)blocks, kXcds);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(c.fn), c.lds)) return rc;
  hipLaunchKernelGGL(c.fn, dim3((unsigned)(g.per_xcd * kXcds)), dim3(c.threads), c.lds, as_stream(stream), g);
  WC_CHECK_LAUNCH("gemm_kernel (direct form)");
  return WC_OK;
}

}  // namespace wc

using namespace wc;

extern "C" int wc_batched_gemm(const void* V, const void* U, void* M, int T_, int P, int Cp, int K,
                               int ldm, int dtype, void* stream) {
  WC_CHECK_ARG(V && U && M, "wc_batched_gemm: null pointer");
  WC_CHECK_ARG(T_ > 0 && P > 0 && K > 0, "wc_batched_gemm: T %d, P %d, K %d", T_, P, K);
  WC_CHECK_ARG(Cp > 0 && Cp % 32 == 0, "wc_batched_gemm: reduction extent %d is not a multiple of 32", Cp);
  WC_CHECK_ARG(ldm >= K && ldm % 8 == 0, "wc_batched_gemm: row stride %d (needs >= K, multiple of 8)", ldm);
  WC_CHECK_ARG(dtype == WC_F16 || dtype == WC_F32 || dtype == WC_BF16, "wc_batched_gemm: dtype %d", dtype);
  // Persistent 256 x 256 tiles (gemm_persistent.hip) where whole layers measured faster with them than with every
  // tile below.  With most of a tile's write-out riding on the workgroup's next tile (reductions of 160 channels and
  // more): from one and a half rounds of tiles on, the last round mostly full - fp16 N = 64, ms per layer against the
  // tiles below: 256 -> 256 channels at 56 x 56 0.218 | 0.233 (F(2,3): 0.369 | 0.396), at 28 x 28 0.065 | 0.067, 256 -> 512 at
  // 28 x 28 0.100 | 0.107, 512 -> 512 at 28 x 28 0.143 | 0.147, 512 -> 256 at 56 x 56 0.338 | 0.346, N = 32 192 -> 256 at 56 x 56
  // 0.104 | 0.108; equal at 252 tiles (N = 32 at 28 x 28, N = 8 at 56 x 56), behind below that (N = 64 at 14 x 14
  // 0.034 | 0.033).  Without that (batches of 2 GB and more): reductions of 512 and more channels over at least three
  // and a half rounds.  wc_test_gemm_override(10, .) takes the kernel wherever it runs with every tile written out when
  // it is done, (13, .) with the write-out riding on the next tile wherever that fits.
  if (gemm_persistent_fits(T_, P, Cp, K, dtype)) {
    const int force = test_gemm_config();
    const long long tiles = (long long)ceil_div(P, 256) * (K / 256) * T_, rounds = ceil_div_ll(tiles, kCus);
    const bool last_round_full = tiles * 100 >= rounds * kCus * 85;
    const bool rides = gemm_persistent_deferred_fits(P, Cp, K, ldm);
    const bool by_size = last_round_full && (rides ? tiles >= 384 : (Cp >= 512 && tiles >= 896));
    if (force == 10 || force == 13 || (force < 0 && by_size))
      return gemm_persistent(V, U, M, T_, P, Cp, K, ldm, dtype, force != 10 && rides, stream);
  }
  GemmConfig c = dispatch_dtype(dtype, [&](auto t) { return choose<decltype(t)>(T_, P, K, Cp); });
  GemmArgs g;
  g.V = V; g.U = U; g.M = M;
  g.P = P; g.K = K; g.Cp = Cp; g.ldm = ldm;
  g.sV = (long long)P * Cp; g.sU = (long long)K * Cp; g.sM = (long long)P * ldm;
  g.ldv = Cp; g.run_blocks = 0; g.jump = 0; g.plane_runs = 0; g.jump2 = 0;
  g.n_run = 0; g.total_runs = 0; g.run_rows = 0; g.plane_extra = 0;
  g.H = g.W = g.oH = g.oW = g.conv_stride = g.pad_h = g.pad_w = g.kw = g.cblocks = 0; g.bias = nullptr;
  g.o_step = g.o_y0 = g.o_x0 = g.o_H = g.o_W = 0;
  g.tiles_p = ceil_div(P, c.bm); g.tiles_k = ceil_div(K, c.bn); g.T = T_;
  const long long blocks = (long long)g.tiles_p * g.tiles_k * T_;
  WC_CHECK_ARG(blocks < (1ll << 30), "wc_batched_gemm: problem too large");
  WC_CHECK_ARG(Cp % c.bk == 0, "wc_batched_gemm: tile depth %d does not divide %d", c.bk, Cp);
  g.n_blocks = (int)blocks;
  g.per_xcd = ceil_div((int)blocks, kXcds);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(c.fn), c.lds)) return rc;
  hipLaunchKernelGGL(c.fn, dim3((unsigned)(g.per_xcd * kXcds)), dim3(c.threads), c.lds, as_stream(stream), g);
  WC_CHECK_LAUNCH("gemm_kernel");
  return WC_OK;
}
