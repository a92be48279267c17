// Direct form with ONE operand tile per kernel row (16-bit types, kernel rows of 4 to 8 taps).
//
// gemm_kernel<..., DIRECT> (gemm.hip) loads, for every tap, its own tile of 256 pixels x 32 channels of x: the taps of
// one kernel row read nearly the same pixels, and the rate at which a CU can pull operands in is what bounds that
// kernel (c4 7x7 at stride 2: x fetched 5.75 times from beyond L2).  Here a workgroup owns 256 consecutive output
// pixels x 128 output channels (four wavefronts of 128 x 64, one workgroup per CU), and for every group (kernel row
// ky, block of 32 channels) the input rows those pixels read are brought to LDS ONCE, with their zero padding, and
// serve all KW taps of the row: tap kx of output pixel (oy, ox) is pixel stride ox + kx of the slot of row oy.  Only
// the 128 x 32 filter block changes from tap to tap.  Same sum as the other direct kernel in another order (kernel
// row, channel block, tap), so the two agree to fp32 rounding and exactly on small integers.
//
// Everything arrives by LDS-DMA (global_load_lds_dwordx4, inline assembly: the compiler cannot know which LDS bytes such
// a load fills and would wait for all of them before every LDS read): the pixel tile of the next group a whole
// group ahead into the other of two 48 KB stages, the filter blocks six taps ahead into a ring of eight 8 KB stages.
// Pixels outside the image are copied from a 64-byte block of zeros.  One barrier per tap; what may still be in flight
// at each barrier is a compile-time count per tap (the taps of a group are unrolled), handed to s_waitcnt.  The last
// groups queue loads nobody uses (the last group again, into free stages) so that those counts hold to the end.
// LDS pixel layout: groups of 16 pixels, chunk-major inside a group - what one DMA instruction fills, lane l = 16 c +
// position - with the position XORed by the parity of the group, so that the sixteen lanes of a fragment read that take
// every second pixel (stride 2) meet sixteen different bank groups.  Fragment addresses are fixed per lane, tap and
// row block and held in registers.  Fragments of the next sub-step are read between the products of the current one.
#include "wc_common.h"

namespace wc {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct Mfma16;
template <> struct Mfma16<half_t> {
  using Frag = f16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct Mfma16<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

__device__ __attribute__((aligned(64))) unsigned char rows_zeros[64];   // source of every pixel outside the image

struct RowsArgs {
  const void* x; const void* U; const void* bias; void* y;
  int H, W, C, K, kh, stride, pad_h, pad_w, oH, oW;
  int P, total_rows;          // N oH oW, N oH
  int SR, VR;                 // pixels per slot (one input row with its padding), pixels of the whole tile
  int cblocks, Cp;            // C / 32, kh KW C (row length of U)
  int tiles_k, n_blocks, per_xcd;
  int o_step, o_y0, o_x0, o_H, o_W;
};

__device__ __forceinline__ int row_swizzle(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }
// one wavefront-wide LDS-DMA load: lane l copies 16 bytes from its own global address to LDS byte lds_addr + 16 l
__device__ __forceinline__ void dma16(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(gptr), "s"(lds_addr) : "memory");
}
// byte offset of pixel r (its first chunk) inside a pixel stage
__device__ __forceinline__ int pixel_offset(int r) { return (r >> 4) * 1024 + (((r & 15) ^ ((r >> 4) & 1)) << 4); }

constexpr int kVInstr = kDirectRowsPixels / 64;   // DMA instructions per wavefront and pixel tile (16 pixels each)
constexpr int kUStages = 8, kUAhead = 6;
constexpr int kUStage = 128 * 64;                 // bytes: 128 filter rows of 32 channels
constexpr int kVStage = kDirectRowsPixels * 64;   // bytes

// pixel-tile instructions queued at tap j of a group: half the tile at taps 0 and 1
constexpr int v_share(int j) { return j <= 1 ? kVInstr / 2 : 0; }
constexpr int step_count(int KW, int j) { return v_share(((j % KW) + KW) % KW) + 2; }
// Loads that may still be in flight at the barrier of tap kx: everything queued after the filter block of tap kx + 1
// (queued five taps ago, as the last loads of that tap), and at the last tap of a group - during which the first
// fragments of the next group are read - nothing of the next pixel tile (queued at taps 0 and 1 of this group).
constexpr int in_flight(int KW, int kx) {
  int a = 0;
  for (int d = 1; d <= 4; ++d) a += step_count(KW, kx - d);
  if (kx == KW - 1) {
    int b = 2;
    for (int j = 2; j <= KW - 2; ++j) b += step_count(KW, j);
    if (b < a) a = b;
  }
  return a;
}

template <typename T, int KW>
__global__ __launch_bounds__(256, 1) void direct_rows_kernel(RowsArgs g) {
  static_assert(KW >= 4 && sizeof(T) == 2, "kernel rows of at least four taps, 16-bit types");
  using MF = Mfma16<T>;
  constexpr int WM = 4, WN = 2, BM = 256, BN = 128;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;
  const unsigned u_base = lds_base + 2 * kVStage;

  const int blk = xcd_remap(blockIdx.x, g.per_xcd);
  if (blk >= g.n_blocks) return;
  const int kt_ = blk % g.tiles_k, pt = blk / g.tiles_k;
  const int p0 = pt * BM, k0 = kt_ * BN;
  const int gr0 = p0 / g.oW;                       // first output row (over all images) the tile touches: slot 0
  const int s = g.stride;
  const T* xb = static_cast<const T*>(g.x);

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wp = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- pixel tile: instruction n of this wavefront fills the 16-pixel group wave + 4 n; lane l: position l & 15, chunk l >> 4
  const T* vptr[kVInstr];
  int viy[kVInstr];
  const int vchunk = lane >> 4;
#pragma unroll
  for (int n = 0; n < kVInstr; ++n) {
    const int grp = wave + 4 * n;
    const int r = grp * 16 + ((lane & 15) ^ (grp & 1));
    const int slot = r / g.SR, col = r - slot * g.SR;
    const int gr = gr0 + slot;
    const int ix = col - g.pad_w;
    const bool ok = r < g.VR && gr < g.total_rows && (unsigned)ix < (unsigned)g.W;
    const int b = gr / g.oH, oy = gr - b * g.oH;
    const int iy0 = s * oy - g.pad_h;              // input row of kernel row 0
    vptr[n] = xb + (((long long)b * g.H + iy0) * g.W + ix) * g.C + vchunk * 8;
    viy[n] = ok ? iy0 : -(1 << 24);                // never inside the image
  }
  const T* zsrc = reinterpret_cast<const T*>(rows_zeros) + vchunk * 8;
  // ---- filter blocks: instruction n (0, 1) fills rows 16 (wave + 4 n) .. + 15; lane l: row l >> 2, stored position l & 3
  const T* uptr[2];
#pragma unroll
  for (int n = 0; n < 2; ++n) {
    const int row = (wave + 4 * n) * 16 + (lane >> 2);
    uptr[n] = static_cast<const T*>(g.U) + (long long)min(k0 + row, g.K - 1) * g.Cp + (((lane & 3) ^ row_swizzle(row)) * 8);
  }

  // element offsets of the groups gi .. gi + 3 (the last group again beyond the end) and their kernel rows, moved on
  // one group at a time
  const int G = g.kh * g.cblocks;
  long long voffs[4];
  int uoffs[4], kys[4];
  int q_ky = 0, q_cb = 0, q_g = 0;
  auto make_entry = [&](int e) {
    voffs[e] = (long long)q_ky * g.W * g.C + q_cb * 32;
    uoffs[e] = q_ky * KW * g.C + q_cb * 32;
    kys[e] = q_ky;
    if (q_g + 1 < G) {
      ++q_g;
      if (++q_cb == g.cblocks) { q_cb = 0; ++q_ky; }
    }
  };
#pragma unroll
  for (int e = 0; e < 4; ++e) make_entry(e);
  auto advance = [&]() {
#pragma unroll
    for (int e = 0; e < 3; ++e) { voffs[e] = voffs[e + 1]; uoffs[e] = uoffs[e + 1]; kys[e] = kys[e + 1]; }
    make_entry(3);
  };
  auto issue_v = [&](int dg, int stage, int n_begin, int n_end) {
    const unsigned dst = lds_base + stage * kVStage + wave * 1024;
#pragma unroll
    for (int n = 0; n < kVInstr; ++n) {
      if (n < n_begin || n >= n_end) continue;
      const bool in = (unsigned)(viy[n] + kys[dg]) < (unsigned)g.H;
      const T* src = in ? vptr[n] + voffs[dg] : zsrc;
      dma16(src, dst + n * 4096);
    }
  };
  auto issue_u = [&](int dg, int kx, int stage) {
    const unsigned dst = u_base + stage * kUStage + wave * 1024;
#pragma unroll
    for (int n = 0; n < 2; ++n) dma16(uptr[n] + uoffs[dg] + kx * g.C, dst + n * 4096);
  };

  // ---- fragments: this lane's pixel of row block i at tap kx (with its half of the chunk pair); its filter row
  int vaddr[KW][WM];
#pragma unroll
  for (int i = 0; i < WM; ++i) {
    const int p = min(p0 + wp * 128 + 32 * i + l32, g.P - 1);
    const int gr = p / g.oW, ox = p - gr * g.oW;
    const int vbase = (gr - gr0) * g.SR + s * ox;
#pragma unroll
    for (int kx = 0; kx < KW; ++kx) vaddr[kx][i] = pixel_offset(vbase + kx) + lhi * 256;
  }
  int uoffk[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) uoffk[kk] = (wk * 64 + l32) * 64 + (((kk * 2 + lhi) ^ row_swizzle(l32)) * 16);

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;

  typename MF::Frag vf[2][WM], uf[2][WN];
  // fragments of (pixel stage vs, tap kx, filter stage us, sub-step kk) into buffer b, in the order the products use them
  auto fload = [&](int vs, auto kxc, int us, int kk, int b) {
    constexpr int kx = decltype(kxc)::value;
    const unsigned char* vst = lds + vs * kVStage + kk * 512;
    const unsigned char* ust = lds + 2 * kVStage + us * kUStage + uoffk[kk];
    uf[b][0] = *reinterpret_cast<const typename MF::Frag*>(ust);
    vf[b][0] = *reinterpret_cast<const typename MF::Frag*>(vst + vaddr[kx][0]);
    uf[b][1] = *reinterpret_cast<const typename MF::Frag*>(ust + 2048);
#pragma unroll
    for (int i = 1; i < WM; ++i) vf[b][i] = *reinterpret_cast<const typename MF::Frag*>(vst + vaddr[kx][i]);
  };
  auto products = [&](int b) {
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[i][j] = MF::run(uf[b][j], vf[b][i], acc[i][j]);
  };
  // two LDS reads behind each of the first three products, the other five products behind them: the last fragment
  // is requested five products before the first product of the next sub-step
  auto interleave = [&]() {
#pragma unroll
    for (int r = 0; r < 3; ++r) {
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 2, 0);
    }
    __builtin_amdgcn_sched_group_barrier(0x008, WM * WN - 3, 0);
  };

  // ---- the pixel tile of group 0 and the filter blocks of steps 0 .. 5
  issue_v(0, 0, 0, kVInstr);
  static_for<0, kUAhead>([&](auto sc) {
    constexpr int st = decltype(sc)::value;
    issue_u(st / KW, st % KW, st);
  });
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");
  fload(0, ic<0>{}, 0, 0, 0);

#pragma unroll 1
  for (int gi = 0; gi < G; ++gi) {
    const int st0 = gi * KW;
    static_for<0, KW>([&](auto kxc) {
      constexpr int kx = decltype(kxc)::value;
      // the filter block of the next step has landed everywhere (at the last tap the next pixel tile too), and nobody
      // reads the filter stage of the previous step any more
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(in_flight(KW, kx)) : "memory");
      if constexpr (v_share(kx) > 0) issue_v(1, (gi + 1) & 1, kx * (kVInstr / 2), kx * (kVInstr / 2) + v_share(kx));
      issue_u((kx + kUAhead) / KW, (kx + kUAhead) % KW, (st0 + kx + kUAhead) & (kUStages - 1));
      __builtin_amdgcn_sched_barrier(0);
      const int us = (st0 + kx) & (kUStages - 1), usn = (st0 + kx + 1) & (kUStages - 1);
      fload(gi & 1, ic<kx>{}, us, 1, 1);
      products(0);
      interleave();
      if constexpr (kx + 1 < KW) fload(gi & 1, ic<kx + 1>{}, usn, 0, 0);
      else fload((gi + 1) & 1, ic<0>{}, usn, 0, 0);
      products(1);
      interleave();
      __builtin_amdgcn_sched_barrier(0);
    });
    advance();
  }
  asm volatile("s_waitcnt vmcnt(0)\n\ts_barrier" ::: "memory");

  // ---- epilogue: every wavefront stages 32 rows x 64 channels of its own (128 bytes per row, chunks swizzled by row)
  // in what was the first pixel stage and writes whole 128-byte row segments.  Accumulator (i, j), register 4 q + e holds
  // output channel 32 j + 8 q + 4 lhi + e of tile row 32 i + l32.
  unsigned char* stg = lds + wave * (32 * WN * 64);
  constexpr int CPR = WN * 4;            // 16-byte chunks per staged row
  constexpr int RPI = 64 / CPR;          // rows per read-back instruction
  T* yb = static_cast<T*>(g.y);
#pragma unroll
  for (int i = 0; i < WM; ++i) {
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q) {
        Pack<T, 4> o;
        float bv[4] = {0.f, 0.f, 0.f, 0.f};
        if (g.bias) {
          const int kb = k0 + wk * 64 + j * 32 + 8 * q + 4 * lhi;
#pragma unroll
          for (int e = 0; e < 4; ++e)
            if (kb + e < g.K) bv[e] = static_cast<float>(static_cast<const T*>(g.bias)[kb + e]);
        }
#pragma unroll
        for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e] + bv[e]);
        const int chunk = (4 * j + q) ^ (l32 & (CPR - 1));
        *reinterpret_cast<Pack<T, 4>*>(stg + l32 * (CPR * 16) + chunk * 16 + lhi * 8) = o;
      }
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPI) {
      const int row = r0 + lane / CPR, c = lane % CPR;
      const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * (CPR * 16) + ((c ^ (row & (CPR - 1))) * 16));
      const int p = p0 + wp * 128 + i * 32 + row;
      const int k = k0 + wk * 64 + c * 8;
      if (p < g.P && k < g.K) {
        long long orow = p;
        if (g.o_step) {
          const int per = g.oH * g.oW;
          const int b = p / per, rem = p - b * per;
          const int oy = rem / g.oW, ox = rem - oy * g.oW;
          orow = ((long long)b * g.o_H + oy * g.o_step + g.o_y0) * g.o_W + ox * g.o_step + g.o_x0;
        }
        *reinterpret_cast<u32x4*>(yb + orow * g.K + k) = val;
      }
    }
  }
}

using RowsKernel = void (*)(RowsArgs);

template <typename T>
RowsKernel pick_rows(int kw) {
  switch (kw) {
    case 4: return &direct_rows_kernel<T, 4>;
    case 5: return &direct_rows_kernel<T, 5>;
    case 6: return &direct_rows_kernel<T, 6>;
    case 7: return &direct_rows_kernel<T, 7>;
    case 8: return &direct_rows_kernel<T, 8>;
    default: return nullptr;
  }
}

}  // namespace

// Pixels of the tile one workgroup keeps per group: the slots of every output row that 256 consecutive output pixels
// can touch, each one input row with its padding.
static int rows_tile_pixels(int stride, int oW, int kw) { return (255 / oW + 2) * (stride * (oW - 1) + kw); }

bool direct_rows_fits(int N, int C, int K, int kw, int stride, int oH, int oW, int dtype) {
  if (dtype != WC_F16 && dtype != WC_BF16) return false;
  if (kw < 4 || kw > 8 || (stride != 1 && stride != 2)) return false;
  if (C % 32 != 0 || K % 8 != 0 || oW < 1 || oW > 256) return false;
  return rows_tile_pixels(stride, oW, kw) <= kDirectRowsPixels && (long long)N * oH * oW < (1ll << 31);
}

int direct_rows_conv(const void* x, const void* U, const void* bias, void* y, int N, int H, int W, int C, int K, int kh,
                     int kw, int stride, int pad_h, int pad_w, int oH, int oW, int dtype, void* stream, int o_step,
                     int o_y0, int o_x0, int o_H, int o_W) {
  WC_CHECK_ARG(x && U && y, "direct_rows_conv: null pointer");
  WC_CHECK_ARG(direct_rows_fits(N, C, K, kw, stride, oH, oW, dtype), "direct_rows_conv: problem outside the kernel's range");
  WC_CHECK_ARG(kh >= 1 && (long long)kh * kw * C < (1ll << 24), "direct_rows_conv: kernel %d x %d", kh, kw);
  WC_CHECK_ARG((long long)N * H * W < (1ll << 31), "direct_rows_conv: input too large");
  RowsArgs g;
  g.x = x; g.U = U; g.bias = bias; g.y = y;
  g.H = H; g.W = W; g.C = C; g.K = K; g.kh = kh; g.stride = stride; g.pad_h = pad_h; g.pad_w = pad_w; g.oH = oH; g.oW = oW;
  g.P = N * oH * oW; g.total_rows = N * oH;
  g.SR = stride * (oW - 1) + kw;
  g.VR = rows_tile_pixels(stride, oW, kw);
  g.cblocks = C / 32; g.Cp = kh * kw * C;
  g.tiles_k = ceil_div(K, 128);
  g.n_blocks = ceil_div(g.P, 256) * g.tiles_k;
  g.per_xcd = ceil_div(g.n_blocks, kXcds);
  g.o_step = o_step; g.o_y0 = o_y0; g.o_x0 = o_x0; g.o_H = o_H; g.o_W = o_W;
  RowsKernel fn = dtype == WC_F16 ? pick_rows<half_t>(kw) : pick_rows<bf16_t>(kw);
  WC_CHECK_ARG(fn != nullptr, "direct_rows_conv: kernel rows of %d taps", kw);
  constexpr size_t lds = 2 * (size_t)kVStage + (size_t)kUStages * kUStage;
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
  hipLaunchKernelGGL(fn, dim3((unsigned)(g.per_xcd * kXcds)), dim3(256), lds, as_stream(stream), g);
  WC_CHECK_LAUNCH("direct_rows_kernel");
  return WC_OK;
}

}  // namespace wc
