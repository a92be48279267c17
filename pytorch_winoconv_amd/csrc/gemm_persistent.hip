// Batched GEMM M[t] = V[t] x U[t]^T for 16-bit types on persistent workgroups: 256 x 256 tiles, four wavefronts of
// 128 x 128 (accumulators in 256 registers: eight fragment reads per sixteen MFMAs where gemm_kernel's 128 x 64 wavefront
// tiles need twelve, and a third fewer operand bytes per product than its 256 x 128 tile), one workgroup per CU walking
// over its share of the tiles.  Operands arrive by global_load_lds_dwordx4 (inline assembly: the compiler would wait
// for every outstanding load before each LDS read) in a ring of four 32-deep stages, three steps ahead; the ring runs on
// across tile boundaries, so the first steps of the next tile are in flight while this tile is written out (through a
// staging block per wavefront, whole 256-byte row segments).  One barrier per step; what may be in flight at each
// barrier is a fixed count handed to s_waitcnt - the loads of the step after next, and during the first two steps of
// a tile the stores of the tile before (loads and stores share the counter and return in order).  That is why every
// tile issues the same number of stores: rows beyond the problem are written as copies of its last row, and K must
// be a multiple of 256.  Same order of additions as gemm_kernel: bit-identical results.
//
// Measured against gemm_kernel's choice (fp16, three rotating operand sets): T = 36, P = 12544, C = K = 256 125 us
// against 140; P = 3136, C = K = 512 94 against 111.
#include "wc_common.h"

namespace wc {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct MfmaP;
template <> struct MfmaP<half_t> {
  using Frag = f16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaP<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

struct PersistentArgs {
  const void* V; const void* U; void* M;
  int P, K, Cp, ldm;
  long long sV, sU, sM;     // batch strides in elements
  int tiles_p, tiles_k, n_tiles;
  int n_wg;                 // workgroups (a multiple of the number of XCDs)
};

__device__ __forceinline__ int swizzle(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }
__device__ __forceinline__ void dma16(const void* gptr, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(gptr), "s"(lds_addr) : "memory");
}

constexpr int WM = 4, WN = 4, BM = 256, BN = 256, ROWS = BM + BN;
constexpr int STAGE = ROWS * 64;      // bytes: 64-byte rows (32 channels), chunks swizzled by the row as in gemm_kernel
constexpr int S = 4;
constexpr int GPW = ROWS / 64;        // DMA instructions per wavefront and step (8)
constexpr int VG = BM / 64;
constexpr int STORES = WM * 32 / (64 / (WN * 4));   // global stores per wavefront and tile: 4 row blocks x 8 instructions
constexpr size_t kPersistentLds = (size_t)S * STAGE + 4 * 32 * WN * 64;

template <typename T>
__global__ __launch_bounds__(256, 1) void gemm_persistent_kernel(PersistentArgs g) {
  using MF = MfmaP<T>;
  using Frag = typename MF::Frag;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;

  // each XCD (hardware id % 8) owns a contiguous range of tiles; its workgroups take them round robin
  const int xcd = blockIdx.x % kXcds, in_xcd = blockIdx.x / kXcds, per_xcd_wg = g.n_wg / kXcds;
  const int t_begin = (int)((long long)g.n_tiles * xcd / kXcds), t_end = (int)((long long)g.n_tiles * (xcd + 1) / kXcds);
  const int first = t_begin + in_xcd;
  if (first >= t_end) return;
  const int my_tiles = (t_end - first + per_xcd_wg - 1) / per_xcd_wg;
  const int NK = g.Cp / 32;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wp = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- issue side
  const T* src0[GPW];           // operand rows of this lane for the tile being multiplied ...
  const T* src1[GPW];           // ... and for the one after it
  auto set_tile = [&](const T* (&src)[GPW], int tile) {
    const int kt_ = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
    const T* Vt = static_cast<const T*>(g.V) + (long long)t * g.sV;
    const T* Ut = static_cast<const T*>(g.U) + (long long)t * g.sU;
#pragma unroll
    for (int gi = 0; gi < GPW; ++gi) {
      const int row = (wave + 4 * gi) * 16 + (lane >> 2);
      const int chunk = (lane & 3) ^ swizzle(row);
      if (gi < VG) src[gi] = Vt + (long long)min(pt * BM + row, g.P - 1) * g.Cp + chunk * 8;
      else src[gi] = Ut + (long long)min(kt_ * BN + row - BM, g.K - 1) * g.Cp + chunk * 8;
    }
  };
  // the loads of reduction step `ks` of tile set `which` into the ring stage of global step `gstep`; share q of 8
  auto issue_part = [&](bool next, int ks, int gstep, int q) {
    const unsigned dst = lds_base + (gstep & (S - 1)) * STAGE + wave * 1024;
    const T* p = next ? src1[q] : src0[q];
    dma16(p + ks * 32, dst + q * 4096);
  };

  int voff[2], uoff[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const int phys = ((kk * 2 + lhi) ^ swizzle(l32)) * 16;
    voff[kk] = (wp * WM * 32 + l32) * 64 + phys;
    uoff[kk] = (BM + wk * WN * 32 + l32) * 64 + phys;
  }

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  Frag vf[2][WM], uf[2][WN];

  // One 16-deep sub-step in WM quarters: quarter q multiplies row block q by all column blocks from buffer b, reads its
  // share of the fragments (stage rstage, sub-step rkk) into the other buffer and queues one DMA load of the step
  // three ahead.
  auto substep = [&](int b, int rstage, int rkk, bool which, int iks, int gstep, int half) {
    const unsigned char* st = lds + rstage * STAGE;
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[b ^ 1][q] = *reinterpret_cast<const Frag*>(st + voff[rkk] + q * 2048);
      uf[b ^ 1][q] = *reinterpret_cast<const Frag*>(st + uoff[rkk] + q * 2048);
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[q][j] = MF::run(uf[b][j], vf[b][q], acc[q][j]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, WN - 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      issue_part(which, iks, gstep, half * WM + q);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- epilogue of one tile through this wavefront's private staging block
  unsigned char* stg = lds + S * STAGE + wave * (32 * WN * 64);
  auto epilogue = [&](int tile) {
    const int kt_ = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
    T* Mt = static_cast<T*>(g.M) + (long long)t * g.sM;
    constexpr int CPR = WN * 4;
    constexpr int RPI = 64 / CPR;
    // the lane's row and column offsets are the same for every tile: keep the compiler from computing all 32 store
    // addresses once and holding them in registers across the reduction loops (an opaque copy of the lane id)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
#pragma unroll
    for (int i = 0; i < WM; ++i) {
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        // the block is read here, not before: without this the reads of all 256 accumulators are moved to the top of
        // the epilogue, and the registers they need are spilled; a reload from scratch waits for every load and store
        // in flight
        asm volatile("" : "+a"(acc[i][j]));
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          Pack<T, 4> o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e]);
          const int chunk = (4 * j + q) ^ (l32 & (CPR - 1));
          *reinterpret_cast<Pack<T, 4>*>(stg + l32 * (CPR * 16) + chunk * 16 + lhi * 8) = o;
          if (q == 3) __builtin_amdgcn_sched_barrier(0);      // one accumulator block at a time: few registers live
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;          // for the next tile
      }
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += RPI) {
        const int row = r0 + lane_e / CPR, c = lane_e % CPR;
        const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * (CPR * 16) + ((c ^ (row & (CPR - 1))) * 16));
        // rows beyond the problem are written to its last row instead of being skipped - they hold that row's values,
        // their operand rows were clamped to it - so that the number of stores per tile is fixed (it is part of the
        // count of loads and stores in flight); K is a multiple of the tile width
        const int p = min(pt * BM + wp * WM * 32 + i * 32 + row, g.P - 1);
        const int k = kt_ * BN + wk * WN * 32 + c * 8;
        *reinterpret_cast<u32x4*>(Mt + (long long)p * g.ldm + k) = val;
        if ((r0 / RPI) % 2 == 1) __builtin_amdgcn_sched_barrier(0);
      }
    }
  };

  // ---- steps 0 .. 2 of the first tile in flight
  set_tile(src0, first);
  set_tile(src1, my_tiles > 1 ? first + per_xcd_wg : first);
  int gstep = 0;                       // global step counter: stage = gstep & 3
  {
#pragma unroll
    for (int s3 = 0; s3 < 3; ++s3) {
#pragma unroll
      for (int q = 0; q < GPW; ++q) issue_part(false, s3, s3, q);      // (a tile has at least three steps)
    }
  }
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(2 * GPW) : "memory");
  {
    const unsigned char* st = lds;
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[0][q] = *reinterpret_cast<const Frag*>(st + voff[0] + q * 2048);
      uf[0][q] = *reinterpret_cast<const Frag*>(st + uoff[0] + q * 2048);
    }
  }

#pragma unroll 1
  for (int ti = 0; ti < my_tiles; ++ti) {
#pragma unroll 1
    for (int ks = 0; ks < NK; ++ks) {
      // stage gstep + 1 has landed everywhere and nobody reads stage gstep - 1 any more.  In flight may be: the loads of
      // step gstep + 2, and behind the first two steps of a tile the stores of the tile before it.
      if (ti > 0 && ks < 2) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(GPW + STORES) : "memory");
      else asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(GPW) : "memory");
      // the loads of step gstep + 3: this tile's, or the next tile's first steps (the last tile queues its own again)
      const bool which = ks + 3 >= NK;
      const int iks = ks + 3 < NK ? ks + 3 : ks + 3 - NK;
      const int cs = gstep & (S - 1), ns = (gstep + 1) & (S - 1);
      substep(0, cs, 1, which, iks, gstep + 3, 0);
      substep(1, ns, 0, which, iks, gstep + 3, 1);
      ++gstep;
    }
    epilogue(first + ti * per_xcd_wg);
    // the tile after the next one
#pragma unroll
    for (int gi = 0; gi < GPW; ++gi) src0[gi] = src1[gi];
    set_tile(src1, ti + 2 < my_tiles ? first + (ti + 2) * per_xcd_wg : first + (my_tiles - 1) * per_xcd_wg);
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}


// ---- the same kernel with a tile's results written out during the first four steps of the workgroup's next tile.
// With one workgroup per CU nobody multiplies, and nothing is requested, while a tile is written out; here a finished
// tile is only packed to 16 bits - three of its four 32-row blocks into 96 registers, the fourth into the wavefront's
// staging area - and each of the next tile's first four steps stores one block (eight instructions per wavefront)
// between its sub-steps: first the one that waits in the staging area, then the others, each staged before the first
// sub-step of its step.  The stores are
// buffer stores: rows beyond the problem are dropped by the bounds check of the tile's descriptor, and before the first
// tile an empty descriptor drops everything, so every wavefront issues every one of them and they are counted with the
// loads: behind a step that carried stores, eight more operations may be in flight.  To make room for the registers
// the operand addresses are a scalar base and a lane offset computed when a load is queued (batches of V, U and M below
// 2 GB; all four blocks in registers spill).  A tile needs at least five steps.  Same order of additions: bit-identical results.
__device__ __forceinline__ void dma16s(const void* base, unsigned offset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(offset), "s"(base), "s"(lds_addr) : "memory");
}

template <typename T, int HR>
__global__ __launch_bounds__(256, 1) void gemm_persistent_deferred_kernel(PersistentArgs g) {
  static_assert(HR >= 1 && HR <= WM, "row blocks of a tile that ride on the next one");
  using MF = MfmaP<T>;
  using Frag = typename MF::Frag;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;

  const int xcd = blockIdx.x % kXcds, in_xcd = blockIdx.x / kXcds, per_xcd_wg = g.n_wg / kXcds;
  const int t_begin = (int)((long long)g.n_tiles * xcd / kXcds), t_end = (int)((long long)g.n_tiles * (xcd + 1) / kXcds);
  const int first = t_begin + in_xcd;
  if (first >= t_end) return;
  const int my_tiles = (t_end - first + per_xcd_wg - 1) / per_xcd_wg;
  const int NK = g.Cp / 32;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int wp = wave >> 1, wk = wave & 1;
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- issue side: the tile being multiplied (0) and the one after it (1) as scalars
  const T* tV[2]; const T* tU[2];
  int tp0[2], tk0[2];
  auto set_tile = [&](int w, int tile) {
    const int kt_ = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
    tV[w] = static_cast<const T*>(g.V) + (long long)t * g.sV;
    tU[w] = static_cast<const T*>(g.U) + (long long)t * g.sU;
    tp0[w] = pt * BM; tk0[w] = kt_ * BN;
  };
  const unsigned chunk16 = ((lane & 3) ^ swizzle(lane >> 2)) * 16;       // (rows 16 n + r share r's swizzle)
  const unsigned row_bytes = (unsigned)g.Cp * 2;
  // the loads of reduction step `ks` of tile set `next` into the ring stage of global step `gstep`; share q of 8
  auto issue_part = [&](bool next, int ks, int gstep, int q) {
    const unsigned dst = lds_base + (gstep & (S - 1)) * STAGE + wave * 1024 + q * 4096;
    int rl = lane >> 2;
    asm volatile("" : "+v"(rl));          // computed here, load by load: eight offsets per tile would otherwise be kept in registers
    const int row = (wave + 4 * q) * 16 + rl;
    const int w = next ? 1 : 0;
    if (q < VG) dma16s(tV[w], (unsigned)min(tp0[w] + row, g.P - 1) * row_bytes + chunk16 + (unsigned)ks * 64, dst);
    else dma16s(tU[w], (unsigned)min(tk0[w] + row - BM, g.K - 1) * row_bytes + chunk16 + (unsigned)ks * 64, dst);
  };

  int voff[2], uoff[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) {
    const int phys = ((kk * 2 + lhi) ^ swizzle(l32)) * 16;
    voff[kk] = (wp * WM * 32 + l32) * 64 + phys;
    uoff[kk] = (BM + wk * WN * 32 + l32) * 64 + phys;
  }

  f32x16 acc[WM][WN];
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  Frag vf[2][WM], uf[2][WN];

  auto substep = [&](int b, int rstage, int rkk, bool which, int iks, int gstep, int half) {
    const unsigned char* st = lds + rstage * STAGE;
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[b ^ 1][q] = *reinterpret_cast<const Frag*>(st + voff[rkk] + q * 2048);
      uf[b ^ 1][q] = *reinterpret_cast<const Frag*>(st + uoff[rkk] + q * 2048);
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[q][j] = MF::run(uf[b][j], vf[b][q], acc[q][j]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, WN - 2, 0);
      __builtin_amdgcn_sched_barrier(0);
      issue_part(which, iks, gstep, half * WM + q);
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- the previous tile's results (packed) and where they go.  Accumulator (i, j), register 4 q + e holds output
  // channel 32 j + 8 q + 4 lhi + e of tile row 32 i + l32; held[i][j][2 q], [2 q + 1] are its registers 4 q .. 4 q + 3 as
  // 16-bit pairs.  A 32-row block (i, 0 .. 3) is staged as rows of 256 bytes, chunks swizzled by the row.
  constexpr int CPR = WN * 4, RPI = 64 / CPR;
  uint32_t held[HR][WN][8];
  __amdgpu_buffer_rsrc_t hdesc = __builtin_amdgcn_make_buffer_rsrc(g.M, 0, 0, 0x00020000);   // no tile yet: every store is dropped
  unsigned held_off = 0;
  // (staging addresses are computed where they are used, behind an opaque copy of the lane id: sixteen write and eight
  // read addresses per lane would otherwise be kept in registers across the reduction loops)
  auto stage_rows = [&](auto ic_) {
    constexpr int i = decltype(ic_)::value;
    typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
    int le = lane;
    asm volatile("" : "+v"(le));
    const int z = le & (CPR - 1);
    unsigned char* row = lds + S * STAGE + wave * (32 * WN * 64) + (le & 31) * (CPR * 16) + (le >> 5) * 8;
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int q = 0; q < 4; ++q)
        *reinterpret_cast<u32x2*>(row + (((4 * j + q) ^ z) * 16)) = u32x2{held[i][j][2 * q], held[i][j][2 * q + 1]};
  };
  auto store_rows = [&](auto ic_) {
    constexpr int i = decltype(ic_)::value;
    int le = lane;
    asm volatile("" : "+v"(le));
    const int c = le % CPR, r = le / CPR;
    const unsigned char* blk = lds + S * STAGE + wave * (32 * WN * 64);
#pragma unroll
    for (int r0 = 0; r0 < 32; r0 += RPI) {
      const int row = r0 + r;
      const u32x4 val = *reinterpret_cast<const u32x4*>(blk + row * (CPR * 16) + ((c ^ (row & (CPR - 1))) * 16));
      __builtin_amdgcn_raw_buffer_store_b128(val, hdesc, held_off + (unsigned)((i * 32 + r0) * g.ldm * 2), 0, 0);
      if ((r0 / RPI) % 2 == 1) __builtin_amdgcn_sched_barrier(0);       // two at a time: few registers live
    }
  };

  // ---- steps 0 .. 2 of the first tile in flight
  set_tile(0, first);
  set_tile(1, my_tiles > 1 ? first + per_xcd_wg : first);
  int gstep = 0;
#pragma unroll
  for (int s3 = 0; s3 < 3; ++s3)
#pragma unroll
    for (int q = 0; q < GPW; ++q) issue_part(false, s3, s3, q);
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(2 * GPW) : "memory");
  {
    const unsigned char* st = lds;
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[0][q] = *reinterpret_cast<const Frag*>(st + voff[0] + q * 2048);
      uf[0][q] = *reinterpret_cast<const Frag*>(st + uoff[0] + q * 2048);
    }
  }

  constexpr int IM = (WM - HR - 1) * 2 * WM;  // stores per wavefront that follow a tile at once (row blocks HR + 1 .. 3)
  constexpr int SU = HR + 2;                  // steps whose counts differ from the plain one
#pragma unroll 1
  for (int ti = 0; ti < my_tiles; ++ti) {
    // Step 0 carries the previous tile's row block HR, which has waited in the staging area; steps 1 .. HR carry its row
    // blocks 0 .. HR - 1 from the registers (eight stores each, between the sub-steps).  Stage gstep + 1 has landed
    // everywhere and nobody reads stage gstep - 1 any more when all that is in flight is what was queued behind the last
    // load of step gstep - 2: the loads of step gstep - 1, the stores it carried, and behind the first two steps of a
    // tile the stores that followed the tile before at once.
    static_for<0, SU>([&](auto kc) {
      constexpr int ks = decltype(kc)::value;
      constexpr int carried = ks >= 1 && ks - 1 <= HR ? 2 * WM : 0;
      if (ti > 0) asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(GPW + carried + (ks < 2 ? IM : 0)) : "memory");
      else asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(GPW + carried) : "memory");
      const bool which = ks + 3 >= NK;
      const int iks = ks + 3 < NK ? ks + 3 : ks + 3 - NK;
      const int cs = gstep & (S - 1), ns = (gstep + 1) & (S - 1);
      if constexpr (ks >= 1 && ks <= HR) { stage_rows(ic<(ks >= 1 && ks <= HR ? ks - 1 : 0)>{}); __builtin_amdgcn_sched_barrier(0); }
      substep(0, cs, 1, which, iks, gstep + 3, 0);
      if constexpr (ks <= HR) { store_rows(ic<(ks == 0 ? HR : ks <= HR ? ks - 1 : 0)>{}); __builtin_amdgcn_sched_barrier(0); }
      substep(1, ns, 0, which, iks, gstep + 3, 1);
      ++gstep;
    });
#pragma unroll 1
    for (int ks = SU; ks < NK; ++ks) {
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(GPW) : "memory");
      const bool which = ks + 3 >= NK;
      const int iks = ks + 3 < NK ? ks + 3 : ks + 3 - NK;
      const int cs = gstep & (S - 1), ns = (gstep + 1) & (S - 1);
      substep(0, cs, 1, which, iks, gstep + 3, 0);
      substep(1, ns, 0, which, iks, gstep + 3, 1);
      ++gstep;
    }
    // ---- the tile's results: row blocks 0 .. HR - 1 into `held`, the others through the staging area - the last ones
    // out at once, row block HR left there for step 0 of the next tile
    {
      const int tile = first + ti * per_xcd_wg;
      const int kt_ = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      hdesc = __builtin_amdgcn_make_buffer_rsrc(static_cast<T*>(g.M) + (long long)t * g.sM, 0, (int)((unsigned)g.P * (unsigned)g.ldm * 2u), 0x00020000);
      held_off = (unsigned)(((pt * BM + wp * WM * 32 + lane_e / CPR) * g.ldm + kt_ * BN + wk * WN * 32 + (lane_e % CPR) * 8) * 2);
      // (descending: the block that stays in the staging area is written there last)
      static_for<0, WM>([&](auto rc) {
        constexpr int i = WM - 1 - decltype(rc)::value;
        unsigned char* row = lds + S * STAGE + wave * (32 * WN * 64) + (lane_e & 31) * (CPR * 16) + (lane_e >> 5) * 8;
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          asm volatile("" : "+a"(acc[i][j]));
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            Pack<T, 4> o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e]);
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const u32x2 w2 = __builtin_bit_cast(u32x2, o);
            if constexpr (i < HR) { held[i < HR ? i : 0][j][2 * q] = w2[0]; held[i < HR ? i : 0][j][2 * q + 1] = w2[1]; }
            else *reinterpret_cast<u32x2*>(row + (((4 * j + q) ^ (lane_e & (CPR - 1))) * 16)) = w2;
          }
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
          __builtin_amdgcn_sched_barrier(0);
        }
        if constexpr (i > HR) store_rows(ic<i>{});
      });
    }
    // the tile after the next one
    tV[0] = tV[1]; tU[0] = tU[1]; tp0[0] = tp0[1]; tk0[0] = tk0[1];
    set_tile(1, ti + 2 < my_tiles ? first + (ti + 2) * per_xcd_wg : first + (my_tiles - 1) * per_xcd_wg);
  }
  // the last tile's results: nothing to ride on
  if constexpr (HR < WM) store_rows(ic<(HR < WM ? HR : 0)>{});
  static_for<0, HR>([&](auto kc) {
    stage_rows(kc);
    store_rows(kc);
  });
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");
}

}  // namespace

// 16-bit types, output channels in whole tiles, at least three reduction steps, and enough tiles for two rounds
bool gemm_persistent_fits(int T_, int P, int Cp, int K, int dtype) {
  return (dtype == WC_F16 || dtype == WC_BF16) && K % BN == 0 && Cp % 32 == 0 && Cp >= 96 &&
         (long long)ceil_div(P, BM) * (K / BN) * T_ < (1ll << 30);
}

constexpr int kHeldRows = 3;      // row blocks of a tile kept in registers (four spill)
// ... with the write-out riding on the next tile: at least five steps per tile, batches below 2 GB
bool gemm_persistent_deferred_fits(int P, int Cp, int K, int ldm) {
  return Cp >= 160 && (long long)P * Cp * 2 < (1ll << 31) && (long long)K * Cp * 2 < (1ll << 31) && (long long)P * ldm * 2 < (1ll << 31);
}

int gemm_persistent(const void* V, const void* U, void* M, int T_, int P, int Cp, int K, int ldm, int dtype, bool deferred, void* stream) {
  WC_CHECK_ARG(gemm_persistent_fits(T_, P, Cp, K, dtype), "gemm_persistent: P %d, K %d, reduction %d", P, K, Cp);
  WC_CHECK_ARG(!deferred || gemm_persistent_deferred_fits(P, Cp, K, ldm), "gemm_persistent: reduction %d too short for the deferred write-out", Cp);
  PersistentArgs a;
  a.V = V; a.U = U; a.M = M;
  a.P = P; a.K = K; a.Cp = Cp; a.ldm = ldm;
  a.sV = (long long)P * Cp; a.sU = (long long)K * Cp; a.sM = (long long)P * ldm;
  a.tiles_p = ceil_div(P, BM); a.tiles_k = K / BN;
  a.n_tiles = a.tiles_p * a.tiles_k * T_;
  a.n_wg = kCus;
  auto fn = deferred ? (dtype == WC_F16 ? &gemm_persistent_deferred_kernel<half_t, kHeldRows> : &gemm_persistent_deferred_kernel<bf16_t, kHeldRows>)
                     : (dtype == WC_F16 ? &gemm_persistent_kernel<half_t> : &gemm_persistent_kernel<bf16_t>);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), kPersistentLds)) return rc;
  hipLaunchKernelGGL(fn, dim3((unsigned)a.n_wg), dim3(256), kPersistentLds, as_stream(stream), a);
  WC_CHECK_LAUNCH("gemm_persistent_kernel");
  return WC_OK;
}

}  // namespace wc
