// The shifted product of plans whose pieces share one transformed input, with one operand tile per run (as
// gemm_rows_kernel, gemm.hip) on tiles of 512 tile rows x 128 output channels fed by LDS-DMA, persistent.
//
// gemm_rows_kernel (256 x 128, four wavefronts of 128 x 64, two workgroups per CU, operands through registers one step
// ahead) is bound by LDS: six fragment reads per eight MFMAs, and every operand byte written to LDS by a VALU store.
// Here one workgroup per CU walks over tiles of 512 x 128: four wavefronts of 128 x 128 (accumulators in 256 registers),
// eight fragment reads per sixteen MFMAs, and half the filter bytes per product.  Operands arrive by
// global_load_lds_dwordx4 (inline assembly: the compiler would wait for every outstanding load before each LDS read;
// scalar base + 32-bit lane offset): the V tile (512 + n_run - 1 rows x 32 channels) of the group two groups ahead into a
// ring of three stages, spread over the steps of a group; the 128 x 32 filter block of the step four steps ahead into a
// ring of six stages.  A group is one (run, channel block) of a tile; its steps are the n_run pieces of the run, which
// read the same V tile b rows further down.  The queue of groups runs on from the last group of a tile to the first of
// the workgroup's next tile, so that tile's first operands arrive while this one is written out (per-wavefront staging
// of 32 x 32 blocks in LDS, rows of 64 bytes).  One barrier per step; what may still be in flight at each barrier is a
// compile-time count per piece position (the steps of a group are unrolled), handed to s_waitcnt: loads return in order,
// and the stores of a tile's results, which share the counter, can only make a wait longer.  Beyond the last tile the
// queue holds loads of one and the same 16 bytes that nobody reads, so that the counts hold to the end.  Rows of 64
// bytes with their 16-byte chunks swizzled by the row, as in gemm_kernel; the swizzle of a fragment read depends on the
// piece (rows l + b), so fragment addresses are held per (piece, sub-step).  Same order of additions as
// gemm_rows_kernel: bit-identical results.
//
// With one workgroup per CU nobody multiplies while a tile is written out.  Where a tile has enough steps (DG > 0
// below) its results are therefore only packed to 16 bits when it is done (128 registers), and go out during the first
// eight steps of the workgroup's next tile, two 32 x 32 blocks per step, each staged before a sub-step and stored
// behind it; the last tile's follow the loop.  Those stores are counted with the loads (memory operations of both
// kinds retire in order on this part), so the waits of the steps that carry them stay exact.
#include "wc_common.h"

namespace wc {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));

template <typename T> struct MfmaR;
template <> struct MfmaR<half_t> {
  using Frag = f16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaR<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

struct RowsDmaArgs {
  const void* V; const void* U; void* M;
  int P, K, ldv, Cu, ldm;        // rows of a batch of V (without its tail), output channels, row lengths of V and U, of M
  long long sV, sU, sM;          // batch strides in elements
  int last_row;                  // P - 1 + n_run - 1: the last row of V any piece of a run may read
  int total_runs, plane_runs, run_rows, plane_extra;
  int tiles_p, tiles_k, n_tiles;
  int per_xcd, wgs_per_xcd;      // tiles an XCD owns (a contiguous range), workgroups that share them
};

__device__ __forceinline__ int row_swizzle(int r) { return (((r >> 1) ^ (r >> 3)) & 1) | (((r >> 2) & 1) << 1); }
__device__ __forceinline__ void dma16(const void* base, unsigned offset, unsigned lds_addr) {
  asm volatile("s_mov_b32 m0, %2\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, %1" :: "v"(offset), "s"(base), "s"(lds_addr) : "memory");
}

constexpr int BM = 512, BN = 128, WM = 4, WN = 4;
constexpr int kVI = 9;                           // DMA instructions per wavefront and V tile: 16-row groups wave + 4 n
constexpr int kVStage = 33 * 1024;               // 528 rows of 64 bytes: the tile and up to 16 more for the pieces of a run
constexpr int kVStages = 3;                      // the V tile of group g + 2 is queued during group g
constexpr int kJunk = kVStages * kVStage;        // where the ninth load of wavefronts 1 to 3 lands (rows nobody reads)
constexpr int kUBase = kJunk + 3 * 1024;
constexpr int kUStage = BN * 64;
constexpr int kUStages = 6, kUAhead = 4;
constexpr int kStaging = kUBase + kUStages * kUStage;     // 2 KB per wavefront
constexpr int kLdsBytes = kStaging + 4 * 2048;
static_assert(kLdsBytes <= 160 * 1024, "LDS of one CU");

// V instructions queued at piece position j of a group: an even share of the kVI
constexpr int v_begin(int KW, int j) { return j * kVI / KW; }
constexpr int v_share(int KW, int j) { return v_begin(KW, j + 1) - v_begin(KW, j); }
constexpr int step_count(int KW, int j) { return v_share(KW, ((j % KW) + KW) % KW) + 2; }
// Loads that may still be in flight at the barrier of piece position kx.  The filter block of the NEXT step must have
// landed (its fragments are read during this step): it was queued kUAhead - 1 steps ago as the last loads of that step,
// so everything queued in the kUAhead - 2 steps since may be in flight.  At the last piece of a group the V tile of the
// next group must have landed too: it was queued during the previous group, its last load at that group's last position
// with a share, followed by that step's two filter loads, the rest of that group and this group up to here.
constexpr int in_flight(int KW, int kx) {
  int a = 0;
  for (int d = 1; d <= kUAhead - 2; ++d) a += step_count(KW, kx - d);
  if (kx == KW - 1) {
    int jl = KW - 1;
    while (v_share(KW, jl) == 0) --jl;
    int b = 2;
    for (int j = jl + 1; j <= KW - 1; ++j) b += step_count(KW, j);
    for (int j = 0; j <= KW - 2; ++j) b += step_count(KW, j);
    if (b < a) a = b;
  }
  return a;
}
// ... before the loop: everything queued in the steps after the one that holds the later of the last load of V tile 0
// (step -KW - 1) and the filter block of step 0 (step -kUAhead)
constexpr int prologue_in_flight(int KW) {
  const int from = (-KW - 1 > -kUAhead ? -KW - 1 : -kUAhead) + 1;
  int n = 0;
  for (int s = from; s < 0; ++s) n += v_share(KW, ((s % KW) + KW) % KW) + (s + kUAhead >= 0 ? 2 : 0);
  return n;
}

// ---- deferred write-out (DG > 0).  A tile's results are packed into 128 registers when its last step is done, and go
// out during the first kNS steps of the workgroup's NEXT tile, two 32 x 32 blocks per step (each through the wavefront's
// staging area: staged before a sub-step, read back and stored behind it), so that the matrix cores do not wait for the
// write-out.  The stores are buffer stores - lanes beyond the tensor are dropped by the bounds check of the descriptor, an
// empty descriptor drops all of them before the first tile - so each of them is issued by every wavefront at every such
// step and the counts below hold.  The first DG groups of a tile are unrolled (their steps know which blocks they
// carry); the unrolled part ends late enough behind the last store that the steps of the rolled part, and the first steps
// of the next tile, see no store in the window they count (dg_steps_ok).
constexpr int kNS = 8;
constexpr int imod(int a, int n) { return ((a % n) + n) % n; }
constexpr int stores_at(int DG, int r) {      // r: step of a tile (group * KW + piece); negative: a step of the tile before
  return DG > 0 && r >= 0 && r < kNS ? 4 : 0;
}
constexpr int ops_at(int KW, int DG, int r) { return v_share(KW, imod(r, KW)) + 2 + stores_at(DG, r); }
// in_flight() with the stores counted: the order inside a step is V loads, filter loads, stores
constexpr int in_flight_at(int KW, int DG, int s) {
  int a = stores_at(DG, s - (kUAhead - 1));
  for (int d = 1; d <= kUAhead - 2; ++d) a += ops_at(KW, DG, s - d);
  if (imod(s, KW) == KW - 1) {
    int jl = KW - 1;
    while (v_share(KW, jl) == 0) --jl;
    const int sp = s - 2 * KW + 1 + jl;          // the step of the previous group that queued the last load of the next V tile
    int b = 2 + stores_at(DG, sp);
    for (int x = sp + 1; x <= s - 1; ++x) b += ops_at(KW, DG, x);
    if (b < a) a = b;
  }
  return a;
}
constexpr bool counts_agree(int KW) {
  for (int kx = 0; kx < KW; ++kx)
    if (in_flight_at(KW, 0, kx) != in_flight(KW, kx) || in_flight_at(KW, 0, kx + 3 * KW) != in_flight(KW, kx)) return false;
  return true;
}
static_assert(counts_agree(2) && counts_agree(3) && counts_agree(4) && counts_agree(5), "the two ways of counting agree without stores");
// how many steps back the count of a step reaches
constexpr int count_reach(int KW) {
  int jl = KW - 1;
  while (v_share(KW, jl) == 0) --jl;
  const int b = 2 * KW - 1 - jl;
  return b > kUAhead - 1 ? b : kUAhead - 1;
}
constexpr bool dg_steps_ok(int KW, int DG) { return DG * KW - count_reach(KW) >= kNS; }
constexpr int deferred_groups(int KW) { return (kNS + count_reach(KW) + KW - 1) / KW; }     // the fewest unrolled groups

template <typename T, int KW, int DG = 0>
__global__ __launch_bounds__(256, 1) void gemm_rows_dma_kernel(RowsDmaArgs g) {
  static_assert(KW >= 2 && KW <= 9 && sizeof(T) == 2, "runs of 2 to 9 pieces, 16-bit types");
  static_assert(DG == 0 || dg_steps_ok(KW, DG), "unrolled groups cover the stores and their wake");
  using MF = MfmaR<T>;
  extern __shared__ __attribute__((aligned(1024))) unsigned char lds[];
  const unsigned lds_base = (unsigned)(size_t)(__attribute__((address_space(3))) unsigned char*)lds;

  const int tid = threadIdx.x, lane = tid & 63;
  const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
  const int l32 = lane & 31, lhi = lane >> 5;

  // ---- the tiles of this workgroup: local indices wg, wg + wgs_per_xcd, ... of its XCD's range
  const int xcd = blockIdx.x % kXcds;
  const int tile0 = xcd * g.per_xcd;
  const int local_end = min(g.per_xcd, g.n_tiles - tile0);
  const int local_first = blockIdx.x / kXcds;
  if (local_first >= local_end) return;

  // ---- the queue of groups: entries 0 .. 2 are the group the loop is at and the two after it, across tiles.  Kept
  // small (scalar registers are scarce beside 512 vector registers): offsets in units of 64 bytes, tile coordinates packed.
  const int ncc = g.ldv / 32;
  const int G = g.total_runs * ncc;
  constexpr unsigned kPast = 1u << 31;   // entry flag: no such group, one and the same 16 bytes are fetched
  unsigned vb[3], ub[3];           // V / U of the entry's batch at its (run, channel block), first piece, from g.V / g.U
  unsigned ept[3];                 // tile: index along P | index along K << 20 | kPast
  int q_local = local_first, q_g = 0, q_cb = 0, q_plane_left = g.plane_runs;
  unsigned q_v = 0, q_u = 0, q_vrun = 0, q_urun = 0, q_pt = 0;
  const unsigned run_step = (unsigned)g.run_rows * ncc, plane_step = (unsigned)g.plane_extra * ncc, urun_step = (unsigned)KW * ncc;
  auto open_tile = [&]() {
    if (q_local >= local_end) { q_pt = kPast; q_v = q_u = 0; }
    else {
      const int tile = tile0 + q_local;
      const int kt = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
      q_pt = (unsigned)pt | (unsigned)kt << 20;
      q_v = (unsigned)((long long)t * g.sV / 32); q_u = (unsigned)((long long)t * g.sU / 32);
    }
    q_g = 0; q_cb = 0; q_plane_left = g.plane_runs; q_vrun = 0; q_urun = 0;
  };
  auto make_entry = [&](int e) {
    ept[e] = q_pt;
    vb[e] = q_v + q_vrun + q_cb;
    ub[e] = q_u + q_urun + q_cb;
    if (q_pt & kPast) return;
    if (++q_g == G) { q_local += g.wgs_per_xcd; open_tile(); return; }
    if (++q_cb == ncc) {
      q_cb = 0;
      q_vrun += run_step;
      if (--q_plane_left == 0) { q_vrun += plane_step; q_plane_left = g.plane_runs; }
      q_urun += urun_step;
    }
  };
  open_tile();
#pragma unroll
  for (int e = 0; e < 3; ++e) make_entry(e);
  auto advance = [&]() {
#pragma unroll
    for (int e = 0; e < 2; ++e) { vb[e] = vb[e + 1]; ub[e] = ub[e + 1]; ept[e] = ept[e + 1]; }
    make_entry(2);
  };
  auto entry_p0 = [&](int e) { return (int)(ept[e] & 0xFFFFFu) * BM; };
  auto entry_k0 = [&](int e) { return (int)((ept[e] >> 20) & 0x7FFu) * BN; };

  // ---- issue side.  V: instruction n of this wavefront fills the 16-row group wave + 4 n of a stage; lane l: row l >> 2,
  // stored position l & 3.  Lane offsets for the tile whose first row is p0: rows past the last one a piece reads fetch
  // that row again, rows beyond the last one a run may read are clamped (nobody multiplies them).
  const unsigned chunk16 = ((lane & 3) ^ row_swizzle(lane >> 2)) * 16;
  const unsigned row_bytes = (unsigned)g.ldv * 2, urow_bytes = (unsigned)g.Cu * 2;
  auto issue_v = [&](int dg, int stage, int n_begin, int n_end) {
    const int p0 = entry_p0(dg);
#pragma unroll
    for (int n = 0; n < kVI; ++n) {
      if (n < n_begin || n >= n_end) continue;
      const int row = min((wave + 4 * n) * 16 + (lane >> 2), BM + KW - 2);
      const unsigned voff_n = (unsigned)min(p0 + row, g.last_row) * row_bytes + chunk16;
      const unsigned dst = n == 8 && wave != 0 ? lds_base + kJunk + (wave - 1) * 1024
                                               : lds_base + stage * kVStage + (wave + 4 * n) * 1024;
      dma16(static_cast<const char*>(g.V) + ((unsigned long long)vb[dg] << 6), (ept[dg] & kPast) ? 0u : voff_n, dst);
    }
  };
  auto issue_u = [&](int dg, int b, int stage) {
#pragma unroll
    for (int n = 0; n < 2; ++n) {
      const int row = (wave + 4 * n) * 16 + (lane >> 2);
      const unsigned off = (unsigned)min(entry_k0(dg) + row, g.K - 1) * urow_bytes + (unsigned)b * row_bytes + chunk16;
      dma16(static_cast<const char*>(g.U) + ((unsigned long long)ub[dg] << 6), (ept[dg] & kPast) ? 0u : off, lds_base + kUBase + stage * kUStage + (wave + 4 * n) * 1024);
    }
  };

  // ---- fragment addresses: V rows 128 wave + 32 i + l32 + b (piece b), both sub-steps; U rows 32 j + l32
  int vaddr[KW][2];
#pragma unroll
  for (int b = 0; b < KW; ++b)
#pragma unroll
    for (int kk = 0; kk < 2; ++kk)
      vaddr[b][kk] = (wave * 128 + l32 + b) * 64 + (((kk * 2 + lhi) ^ row_swizzle(l32 + b)) * 16);
  int uaddr[2];
#pragma unroll
  for (int kk = 0; kk < 2; ++kk) uaddr[kk] = kUBase + l32 * 64 + (((kk * 2 + lhi) ^ row_swizzle(l32)) * 16);

  f32x16 acc[WM][WN];
  typename MF::Frag vf[2][WM], uf[2][WN];
  // One 16-deep sub-step in WM quarters: quarter q multiplies row block q by all column blocks from buffer bf and reads
  // its share of the next fragments (V stage vs, piece rb, filter stage us, sub-step rkk) into the other buffer.
  auto substep = [&](int bf, int vs, auto rbc, int us, int rkk) {
    constexpr int rb = decltype(rbc)::value;
    const unsigned char* vst = lds + vs * kVStage + vaddr[rb][rkk];
    const unsigned char* ust = lds + us * kUStage + uaddr[rkk];
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[bf ^ 1][q] = *reinterpret_cast<const typename MF::Frag*>(vst + q * 2048);
      uf[bf ^ 1][q] = *reinterpret_cast<const typename MF::Frag*>(ust + q * 2048);
#pragma unroll
      for (int j = 0; j < WN; ++j) acc[q][j] = MF::run(uf[bf][j], vf[bf][q], acc[q][j]);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);
      __builtin_amdgcn_sched_group_barrier(0x008, WN - 2, 0);
    }
  };

  // ---- what the steps -2 KW .. -1 of the loop below would have queued, in its order (so that its counts hold from the
  // first step on): the V tiles of groups 0 and 1 in their shares, the filter blocks of steps 0 .. kUAhead - 1.  The
  // first fragments need the V tile of group 0 and the filter block of step 0: what later steps queued may stay in flight.
  static_for<0, 2 * KW>([&](auto sc) {
    constexpr int s = decltype(sc)::value - 2 * KW, gv = (s + 2 * KW) / KW, j = (s + 2 * KW) % KW;
    if constexpr (v_share(KW, j) > 0) issue_v(gv, gv, v_begin(KW, j), v_begin(KW, j + 1));
    if constexpr (s + kUAhead >= 0) issue_u((s + kUAhead) / KW, (s + kUAhead) % KW, s + kUAhead);
  });
  asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(prologue_in_flight(KW)) : "memory");
  {
    const unsigned char* vst = lds + vaddr[0][0];
    const unsigned char* ust = lds + uaddr[0];
#pragma unroll
    for (int q = 0; q < WM; ++q) {
      vf[0][q] = *reinterpret_cast<const typename MF::Frag*>(vst + q * 2048);
      uf[0][q] = *reinterpret_cast<const typename MF::Frag*>(ust + q * 2048);
    }
  }

  int vs0 = 0, vs1 = 1, vs2 = 2;          // V stages of this group, the next one, and the one being filled
  int ust = 0;                            // filter stage of the current step
#pragma unroll
  for (int i = 0; i < WM; ++i)
#pragma unroll
    for (int j = 0; j < WN; ++j)
#pragma unroll
      for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
  // ---- deferred write-out: the previous tile's results (packed), where they go, and the two halves of a block's trip
  // through the staging area.  Accumulator (i, j), register 4 q + e holds output channel 32 j + 8 q + 4 lhi + e of tile row
  // 32 i + l32; held[i][j][2 q], [2 q + 1] are its registers 4 q .. 4 q + 3 as 16-bit pairs.
  uint32_t held[DG > 0 ? WM : 1][DG > 0 ? WN : 1][8];
  __amdgpu_buffer_rsrc_t hdesc = __builtin_amdgcn_make_buffer_rsrc(g.M, 0, 0, 0x00020000);   // no tile yet: every store is dropped
  unsigned held_off = 0;           // byte offset in the batch of M of what this lane stores first
  int held_kleft = 0;              // this lane stores channel blocks j with 32 j below this
  int stg_w = 0, stg_r = 0;        // this lane's staging addresses: writes (q = 0), reads (h = 0)
  int stg_z = 0;
  if constexpr (DG > 0) {
    stg_z = (l32 >> 2) & 3;
    stg_w = kStaging + wave * 2048 + l32 * 64 + lhi * 8;
    stg_r = kStaging + wave * 2048 + (lane >> 2) * 64 + (((lane & 3) ^ ((lane >> 4) & 3)) * 16);
  }
  auto stage_block = [&](auto blkc) {
    constexpr int blk = decltype(blkc)::value, i = blk / WN, j = blk % WN;
#pragma unroll
    for (int q = 0; q < 4; ++q) {
      typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
      *reinterpret_cast<u32x2*>(lds + stg_w + ((q ^ stg_z) * 16)) = u32x2{held[i][j][2 * q], held[i][j][2 * q + 1]};
    }
  };
  auto store_block = [&](auto blkc) {
    constexpr int blk = decltype(blkc)::value, i = blk / WN, j = blk % WN;
#pragma unroll
    for (int h = 0; h < 2; ++h) {
      const u32x4 val = *reinterpret_cast<const u32x4*>(lds + stg_r + h * 1024);
      unsigned off = held_off + (unsigned)(((i * 32 + h * 16) * g.ldm + j * 32) * 2);
      if (j * 32 >= held_kleft) off = 0xFFFFFFF0u;                 // beyond the row: out of bounds, dropped
      __builtin_amdgcn_raw_buffer_store_b128(val, hdesc, off, 0, 0);
    }
  };

  auto run_group = [&](auto dgc) {
    constexpr int dg = decltype(dgc)::value;          // the group's index in its tile where that is unrolled, else -1
    static_for<0, KW>([&](auto bc) {
      constexpr int b = decltype(bc)::value;
      constexpr int s = dg * KW + b;
      constexpr bool carries = dg >= 0 && s < kNS;    // this step writes blocks 2 s and 2 s + 1 of the previous tile
      // the filter block of the next step has landed everywhere (at the last piece the next V tile too), and nobody
      // reads the filter stage of the previous step or the V stage of the previous group any more
      asm volatile("s_waitcnt vmcnt(%0)\n\ts_barrier" :: "n"(dg >= 0 ? in_flight_at(KW, DG, s) : in_flight(KW, b)) : "memory");
      if constexpr (v_share(KW, b) > 0) issue_v(2, vs2, v_begin(KW, b), v_begin(KW, b + 1));
      int uis = ust + kUAhead;
      if (uis >= kUStages) uis -= kUStages;
      issue_u((b + kUAhead) / KW, (b + kUAhead) % KW, uis);
      __builtin_amdgcn_sched_barrier(0);
      int usn = ust + 1;
      if (usn == kUStages) usn = 0;
      if constexpr (carries) { stage_block(ic<2 * (carries ? s : 0)>{}); __builtin_amdgcn_sched_barrier(0); }
      substep(0, vs0, ic<b>{}, ust, 1);                       // sub-step 0 multiplies; reads sub-step 1 of this step
      if constexpr (carries) {
        __builtin_amdgcn_sched_barrier(0);
        store_block(ic<2 * (carries ? s : 0)>{});
        stage_block(ic<2 * (carries ? s : 0) + 1>{});
        __builtin_amdgcn_sched_barrier(0);
      }
      if constexpr (b + 1 < KW) substep(1, vs0, ic<b + 1>{}, usn, 0);   // sub-step 1; reads sub-step 0 of the next step
      else substep(1, vs1, ic<0>{}, usn, 0);
      if constexpr (carries) { __builtin_amdgcn_sched_barrier(0); store_block(ic<2 * (carries ? s : 0) + 1>{}); }
      __builtin_amdgcn_sched_barrier(0);
      ust = usn;
    });
    advance();
    const int f = vs0; vs0 = vs1; vs1 = vs2; vs2 = f;
  };

#pragma unroll 1
  for (int local = local_first; local < local_end; local += g.wgs_per_xcd) {
    if constexpr (DG > 0) {
      static_for<0, DG>([&](auto dgc) { run_group(dgc); });
#pragma unroll 1
      for (int gi = DG; gi < G; ++gi) run_group(ic<-1>{});
    } else {
#pragma unroll 1
      for (int gi = 0; gi < G; ++gi) run_group(ic<-1>{});
    }

    const int tile = tile0 + local;
    const int kt = tile % g.tiles_k, pt = (tile / g.tiles_k) % g.tiles_p, t = tile / (g.tiles_k * g.tiles_p);
    if constexpr (DG > 0) {
      // ---- the tile's results into `held` (the write-out rides on the next tile's first steps, or follows the loop)
      int lane_e = lane;
      asm volatile("" : "+v"(lane_e));
      const int row_first = pt * BM + wave * 128, k_first = kt * BN;
      hdesc = __builtin_amdgcn_make_buffer_rsrc(static_cast<T*>(g.M) + (long long)t * g.sM, 0, (int)((unsigned)g.P * (unsigned)g.ldm * 2u), 0x00020000);
      held_off = (unsigned)(((row_first + (lane_e >> 2)) * g.ldm + k_first + (lane_e & 3) * 8) * 2);
      held_kleft = g.ldm - k_first - (lane_e & 3) * 8;
#pragma unroll
      for (int i = 0; i < WM; ++i)
#pragma unroll
        for (int j = 0; j < WN; ++j) {
          asm volatile("" : "+a"(acc[i][j]));      // read here, block by block
#pragma unroll
          for (int q = 0; q < 4; ++q) {
            Pack<T, 4> o;
#pragma unroll
            for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e]);
            typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
            const u32x2 w = __builtin_bit_cast(u32x2, o);
            held[i][j][2 * q] = w[0]; held[i][j][2 * q + 1] = w[1];
          }
#pragma unroll
          for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;          // for the next tile
          __builtin_amdgcn_sched_barrier(0);
        }
    } else {
    // ---- the tile's results: every wavefront stages one 32 x 32 block at a time (64-byte rows, chunks swizzled by the
    // row) and writes 64-byte row segments.  Accumulator (i, j), register 4 q + e holds output channel 32 j + 8 q + 4 lhi + e
    // of tile row 32 i + l32.  The loads of the next tile's first groups are in flight meanwhile.
    // scalar base of the tile + one lane offset: no per-store 64-bit lane addresses (which the compiler would compute
    // before the loop over the tiles and keep in registers that the loop needs)
    // lane-derived values of this part are computed here, tile by tile (behind an opaque copy of the lane id), so that
    // they do not occupy registers during the loop above
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    const int srow = lane_e >> 2, sc = lane_e & 3, e32 = lane_e & 31, ehi = lane_e >> 5;
    unsigned char* stg = lds + kStaging + wave * 2048;
    const int row_first = pt * BM + wave * 128, k_first = kt * BN;
    unsigned long long tile_base = (unsigned long long)(static_cast<T*>(g.M) + (long long)t * g.sM + (long long)row_first * g.ldm + k_first);
    asm volatile("" : "+s"(tile_base));
    const unsigned lane_off = (unsigned)(srow * g.ldm + sc * 8) * 2;
    const int rows_left = g.P - row_first - srow, k_left = g.ldm - k_first - sc * 8;     // this lane stores rows / channels below these
#pragma unroll
    for (int i = 0; i < WM; ++i)
#pragma unroll
      for (int j = 0; j < WN; ++j) {
        asm volatile("" : "+a"(acc[i][j]));      // read here, block by block: not all 256 accumulators copied out up front
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          Pack<T, 4> o;
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e]);
          *reinterpret_cast<Pack<T, 4>*>(stg + e32 * 64 + ((q ^ ((e32 >> 2) & 3)) * 16) + ehi * 8) = o;
        }
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;          // for the next tile
#pragma unroll
        for (int h = 0; h < 2; ++h) {
          const int row = h * 16 + srow;
          const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * 64 + ((sc ^ ((row >> 2) & 3)) * 16));
          char* base = reinterpret_cast<char*>(tile_base) + ((long long)(i * 32 + h * 16) * g.ldm + j * 32) * 2;
          if (i * 32 + h * 16 < rows_left && j * 32 < k_left) *reinterpret_cast<u32x4*>(base + lane_off) = val;
        }
        __builtin_amdgcn_sched_barrier(0);     // block by block: not all 256 accumulators read and converted up front
      }
      }
  }
  if constexpr (DG > 0) {
    // the last tile's results: the same trips through the staging area, with nothing to ride on
    static_for<0, WM * WN>([&](auto blkc) {
      stage_block(blkc);
      store_block(blkc);
    });
  }
  asm volatile("s_waitcnt vmcnt(0)" ::: "memory");       // the queue's last loads write LDS: not after this workgroup has gone
}

using RowsDmaKernel = void (*)(RowsDmaArgs);
template <typename T>
RowsDmaKernel pick_rows_dma(int n_run, bool deferred) {
  if (deferred)
    switch (n_run) {
      case 2: return &gemm_rows_dma_kernel<T, 2, deferred_groups(2)>;
      case 3: return &gemm_rows_dma_kernel<T, 3, deferred_groups(3)>;
      case 4: return &gemm_rows_dma_kernel<T, 4, deferred_groups(4)>;
      case 5: return &gemm_rows_dma_kernel<T, 5, deferred_groups(5)>;
      default: return nullptr;
    }
  switch (n_run) {
    case 2: return &gemm_rows_dma_kernel<T, 2>;
    case 3: return &gemm_rows_dma_kernel<T, 3>;
    case 4: return &gemm_rows_dma_kernel<T, 4>;
    case 5: return &gemm_rows_dma_kernel<T, 5>;
    default: return nullptr;
  }
}

}  // namespace

// Lane offsets are 32-bit: a batch of V and a batch of U below 2 GB each
bool gemm_rows_dma_fits(SharedShift sh, int P, int Cp, int K, int dtype) {
  const int n_run = sh.n_run, tail = sh.tail, n_pieces = sh.n_planes * sh.n_runs * sh.n_run;
  return (dtype == WC_F16 || dtype == WC_BF16) && n_run >= 2 && n_run <= 5 && Cp % 32 == 0 &&
         (long long)(P + tail) * Cp * 2 < (1ll << 31) && (long long)K * n_pieces * Cp * 2 < (1ll << 31) && K <= (1 << 17);
}

// The deferred write-out needs a tile of at least deferred_groups groups and a batch of M below 2 GB (32-bit offsets
// into a buffer descriptor)
bool gemm_rows_dma_deferred_fits(SharedShift sh, int P, int Cp, int ldm) {
  const int groups = sh.n_planes * sh.n_runs * (Cp / 32);
  int need = 1 << 30;
  switch (sh.n_run) {
    case 2: need = deferred_groups(2); break;
    case 3: need = deferred_groups(3); break;
    case 4: need = deferred_groups(4); break;
    case 5: need = deferred_groups(5); break;
    default: break;
  }
  return groups >= need && (long long)P * ldm * 2 < (1ll << 31);
}

int gemm_rows_dma(const void* V, const void* U, void* M, int T_, int P, int Cp, SharedShift sh, int K, int ldm, int dtype,
                  bool deferred, void* stream) {
  const int n_pieces = sh.n_planes * sh.n_runs * sh.n_run;
  WC_CHECK_ARG(gemm_rows_dma_fits(sh, P, Cp, K, dtype), "gemm_rows_dma: runs of %d pieces, rows of %d", sh.n_run, Cp);
  WC_CHECK_ARG(!deferred || gemm_rows_dma_deferred_fits(sh, P, Cp, ldm), "gemm_rows_dma: too few steps per tile for the deferred write-out");
  RowsDmaArgs g;
  g.V = V; g.U = U; g.M = M;
  g.P = P; g.K = K; g.ldv = Cp; g.Cu = n_pieces * Cp; g.ldm = ldm;
  g.sV = (long long)(P + sh.tail) * Cp; g.sU = (long long)K * g.Cu; g.sM = (long long)P * ldm;
  g.last_row = P - 1 + sh.n_run - 1;
  g.total_runs = sh.n_planes * sh.n_runs; g.plane_runs = sh.n_runs;
  g.run_rows = sh.run_rows; g.plane_extra = sh.plane_rows - sh.n_runs * sh.run_rows;
  g.tiles_p = ceil_div(P, BM); g.tiles_k = ceil_div(K, BN);
  const long long tiles = (long long)g.tiles_p * g.tiles_k * T_;
  WC_CHECK_ARG(tiles < (1ll << 30), "gemm_rows_dma: problem too large");
  g.n_tiles = (int)tiles;
  g.per_xcd = ceil_div(g.n_tiles, kXcds);
  g.wgs_per_xcd = g.per_xcd < kCus / kXcds ? g.per_xcd : kCus / kXcds;

  RowsDmaKernel fn = dtype == WC_F16 ? pick_rows_dma<half_t>(sh.n_run, deferred) : pick_rows_dma<bf16_t>(sh.n_run, deferred);
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), kLdsBytes)) return rc;
  hipLaunchKernelGGL(fn, dim3((unsigned)(g.wgs_per_xcd * kXcds)), dim3(256), kLdsBytes, as_stream(stream), g);
  WC_CHECK_LAUNCH("gemm_rows_dma_kernel");
  return WC_OK;
}

}  // namespace wc
