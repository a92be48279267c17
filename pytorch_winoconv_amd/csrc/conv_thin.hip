// One-kernel F(2x2, 3x3) convolution for thin layers: fp16 / bf16 with at most 128 input channels, fp32 with at
// most 64, and any storage type with at most 4 (tiny_conv3x3_kernel, further down).
//
// Same arithmetic as the three-kernel path (input transform of src/split_kernel.cu:60-120, the
// batched product of src/base_conv_launchers.cu:353-367, output transform of
// src/split_kernel.cu:126-203), without V and M in HBM.  With few channels the product has so
// little arithmetic per byte that the transform-domain buffers (4x the input and 4x the output
// for this tile) are all the cost; here x is read once and y written once.
//
// What makes it fit: U of one wavefront's 16 output channels (16 elements x 16 x Cp) stays in
// registers for the life of the workgroup, so LDS only carries the transformed input of the
// 16 tiles in flight.  A workgroup (4 wavefronts, 16 output channels each) walks over blocks of
// 16 tiles: every thread loads the 4 x 4 window of one tile for a few channels, transforms it
// (fp16: packed fp16 adds; bf16: fp32) and stores the 16 elements to LDS in the storage type; after
// one barrier every wavefront multiplies all 16 elements by its part of U on v_mfma_f32_16x16x32
// (U as the row operand, so a lane ends up with 4 consecutive output channels of one tile).  The
// width half of the output transform happens in the MFMA accumulators (A^T has only 0 and +-1:
// a product is added into the accumulators it belongs to), the height half in fp32 registers.  The
// window of the next block is requested before the products of this one, and LDS is
// double-buffered, so there is one barrier per block.  With 128 channels U would take the whole
// register file: eight wavefronts then share a block, four per pair of element rows, and the
// upper four hand their share of each output tile to the lower four through LDS (a second barrier).
// Launches with few blocks of tiles use workgroups of half the size (32 output channels), and U reaches the
// registers through LDS: see thin_conv3x3_kernel.
#include "wc_transform.h"
#include <algorithm>

namespace wc {

typedef _Float16 half8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float floatx4 __attribute__((ext_vector_type(4)));
typedef uint32_t uint4v __attribute__((ext_vector_type(4)));

namespace {

template <typename T> struct Mfma16;
template <> struct Mfma16<half_t> {
  using Frag = half8;
  __device__ static __forceinline__ floatx4 run(Frag a, Frag b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_f16(a, b, c, 0, 0, 0);
  }
};
template <> struct Mfma16<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ floatx4 run(Frag a, Frag b, floatx4 c) {
    return __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, b, c, 0, 0, 0);
  }
};
// fp32: a lane's 16-byte fragment holds four consecutive channels and feeds four v_mfma_f32_16x16x4_f32, each
// of which pairs channel e of the four lane groups' fragments (both operands are cut the same way, so every
// channel of a 16-channel step meets its partner exactly once).
template <> struct Mfma16<float> {
  using Frag = floatx4;
  __device__ static __forceinline__ floatx4 run(Frag a, Frag b, floatx4 c) {
#pragma unroll
    for (int e = 0; e < 4; ++e) c = __builtin_amdgcn_mfma_f32_16x16x4f32(a[e], b[e], c, 0, 0, 0);
    return c;
  }
};

// The accumulator scheme below is written for these matrices.
static_assert(Mats<KIND_23>::at(0, 0) == 1 && Mats<KIND_23>::at(0, 1) == 1 && Mats<KIND_23>::at(0, 2) == 1 &&
              Mats<KIND_23>::at(0, 3) == 0 && Mats<KIND_23>::at(1, 0) == 0 && Mats<KIND_23>::at(1, 1) == 1 &&
              Mats<KIND_23>::at(1, 2) == -1 && Mats<KIND_23>::at(1, 3) == -1, "A^T of F(2,3)");

constexpr int kThinTiles = 16;      // tiles per block
constexpr int kThinK = 64;          // output channels per workgroup

struct ThinArgs {
  const void* x;
  const void* U;
  const void* bias;
  void* y;
  int H, W, C, K, Cp;
  int oH, oW, nH, nW;
  int pad1, pad2;
  int P;          // tiles of the whole batch
  int n_blocks;   // ceil(P / 16)
  int per_xcd;    // gridDim.x / 8
  int x_bytes;    // size of x, below 1 GiB
  int y_bytes;    // size of y, below 2 GiB
  int row_bytes;  // W * C * sizeof(T)
  int k_whole;    // K is a multiple of 4: a lane's 4 output channels go out in one store
  FastDiv div_nW, div_nH;
};

// Store of one lane's share of an output tile: tile p, output channels ko .. ko + 4, the 2 x 2 output positions
// in out[oa][ob], bias bv added.  Stores go through a buffer descriptor and are issued unconditionally: a
// position outside (oH, oW), a tile beyond the last or a lane without work (`live` false) gets an offset beyond
// the buffer and is dropped by the hardware.  No branch around the stores matters for speed: loads and stores
// share one in-order counter, and only with straight-line code can the wait for the next block's window leave
// this block's stores in flight.
template <typename T, bool KW>
__device__ __forceinline__ void store_tile(const ThinArgs& a, __amdgpu_buffer_rsrc_t ydesc, int p, int ko, bool live,
                                           const float (&bv)[4], const floatx4 (&out)[2][2]) {
  const int q = fast_div(p, a.div_nW);
  const int tw = p - q * a.nW;
  const int b = fast_div(q, a.div_nH);
  const int th = q - b * a.nH;
  const unsigned o00 = (((unsigned)b * a.oH + 2 * th) * a.oW + 2 * tw) * a.K + ko;   // in elements
  const bool h1 = 2 * th + 1 < a.oH, w1 = 2 * tw + 1 < a.oW;
#pragma unroll
  for (int oa = 0; oa < 2; ++oa) {
#pragma unroll
    for (int ob = 0; ob < 2; ++ob) {
      const floatx4 s4 = out[oa][ob];
      const bool inside = live && (oa == 0 || h1) && (ob == 0 || w1);
      const unsigned off = o00 + (oa * a.oW + ob) * a.K;
      Pack<T, 4> o;
#pragma unroll
      for (int r = 0; r < 4; ++r) o.v[r] = static_cast<T>(s4[r] + bv[r]);
      if constexpr (KW) {
        const unsigned byte_off = inside ? off * (unsigned)sizeof(T) : kOutside;
        if constexpr (sizeof(T) == 4) {
          __builtin_amdgcn_raw_buffer_store_b128(__builtin_bit_cast(uint4v, o), ydesc, byte_off, 0, 0);
        } else {
          typedef unsigned u2 __attribute__((ext_vector_type(2)));
          __builtin_amdgcn_raw_buffer_store_b64(__builtin_bit_cast(u2, o), ydesc, byte_off, 0, 0);
        }
      } else {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
          const unsigned byte_off = inside && ko + r < a.K ? (off + r) * (unsigned)sizeof(T) : kOutside;
          if constexpr (sizeof(T) == 4)
            __builtin_amdgcn_raw_buffer_store_b32(__builtin_bit_cast(unsigned, o.v[r]), ydesc, byte_off, 0, 0);
          else
            __builtin_amdgcn_raw_buffer_store_b16(__builtin_bit_cast(unsigned short, o.v[r]), ydesc, byte_off, 0, 0);
        }
      }
    }
  }
}

// The bias of a lane's four output channels, loaded once per kernel.
template <typename T>
__device__ __forceinline__ void load_bias(const ThinArgs& a, int ko, float (&bv)[4]) {
  const T* bias = static_cast<const T*>(a.bias);
#pragma unroll
  for (int r = 0; r < 4; ++r) bv[r] = bias && ko + r < a.K ? static_cast<float>(bias[ko + r]) : 0.f;
}

typedef _Float16 half2v __attribute__((ext_vector_type(2)));

// B^T of F(2,3) along one axis of a 4 x 4 block (STRIDE: distance between the four elements,
// OTHER: distance between the four lines).
template <int STRIDE, int OTHER, typename V>
__device__ __forceinline__ void bt23(const V (&in)[16], V (&out)[16]) {
#pragma unroll
  for (int l = 0; l < 4; ++l) {
    const V d0 = in[l * OTHER], d1 = in[l * OTHER + STRIDE], d2 = in[l * OTHER + 2 * STRIDE], d3 = in[l * OTHER + 3 * STRIDE];
    out[l * OTHER] = d0 - d2;
    out[l * OTHER + STRIDE] = d1 + d2;
    out[l * OTHER + 2 * STRIDE] = d2 - d1;
    out[l * OTHER + 3 * STRIDE] = d1 - d3;
  }
}
static_assert(Mats<KIND_23>::bt(0, 0) == 1 && Mats<KIND_23>::bt(0, 2) == -1 && Mats<KIND_23>::bt(1, 1) == 1 &&
              Mats<KIND_23>::bt(1, 2) == 1 && Mats<KIND_23>::bt(2, 1) == -1 && Mats<KIND_23>::bt(2, 2) == 1 &&
              Mats<KIND_23>::bt(3, 1) == 1 && Mats<KIND_23>::bt(3, 3) == -1, "B^T of F(2,3)");

// KW: K is a multiple of 4, a lane's 4 output channels go out in one store (a compile-time choice: a branch
// around the stores, even a uniform one, makes the compiler wait for all memory operations at the loop top).
// KSUB: groups of 16 output channels per workgroup, 4 or 2.  With 2 a workgroup has half the wavefronts, half of
// U to fetch and half the products, and the launch has twice the workgroups: for layers whose blocks of tiles
// would leave more than half of the CUs idle (a workgroup with one block spends most of its time fetching U and,
// in fp32, multiplying).
template <typename T, int CP, bool KW, int KSUB>
__global__ __launch_bounds__((CP * sizeof(T) > 128 ? 128 : 64) * KSUB) __attribute__((amdgpu_waves_per_eu(KSUB / 2, KSUB / 2))) void thin_conv3x3_kernel(ThinArgs a) {
  // Up to 64 channels a wavefront holds U of all 16 elements (4 wavefronts).  With 128 that is twice
  // the register file, so SPLIT: 8 wavefronts, the upper four take the element rows 2 and 3 and hand
  // their share of the output tile to the lower four through LDS.
  constexpr bool SPLIT = CP * sizeof(T) > 128;       // 128 channels of a 16-bit type, 64 of fp32
  constexpr bool PLAIN = sizeof(T) == 4;             // one accumulator per element, width transform in VALU (measured: no gain for 16-bit types)
  constexpr int EPF = 16 / sizeof(T);                // channels per 16-byte fragment
  constexpr int NT = (SPLIT ? 128 : 64) * KSUB;
  constexpr int NROW = SPLIT ? 2 : 4;     // element rows per wavefront
  constexpr int VEC = kThinTiles * CP / NT;   // channels per thread in the transform
  constexpr int CVECS = CP / VEC;
  constexpr int KS = CP / (4 * EPF);      // fragment steps along the channels (four lane groups x EPF channels each)
  // Bytes per (element, tile) row in LDS: no padding; the 16-byte chunks of a row are permuted by the row instead.
  // A fragment read takes one chunk from each of 16 consecutive rows; the LDS of this part delivers 16-byte reads
  // at 256 bytes per clock only if those 16 chunks fall into 16 different 16-byte columns of a 256-byte line
  // (rows padded by 16 bytes, which are conflict-free for 128-byte wide LDS, measured half that rate).  With R rows
  // per 256 bytes, chunk c of row r sits at position c ^ ((r / R) mod chunks per row).
  constexpr int PITCH = CP * sizeof(T);
  constexpr int CPRW = PITCH / 16;             // chunks per row: 4, 8 or 16
  constexpr int RPL = 16 / CPRW;               // rows per 256-byte line
  static_assert(CPRW == 4 || CPRW == 8 || CPRW == 16, "rows of 64, 128 or 256 bytes");
  static_assert(VEC * sizeof(T) <= 16, "a thread's channels stay inside one chunk");
  constexpr int BUF = 16 * kThinTiles * PITCH;
  using MF = Mfma16<T>;
  using Frag = typename MF::Frag;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kbase = (blockIdx.y * KSUB + wave % KSUB) * 16;
  const int row0i = SPLIT ? 2 * (wave / KSUB) : 0;       // first element row of this wavefront

  // transform role: tile pl of the block, channels c .. c + VEC.  x is read through a buffer descriptor:
  // one 32-bit offset per load, and a window element outside the image is an offset beyond the
  // buffer, which reads as zero.
  const int pl = tid / CVECS;
  const int c = (tid % CVECS) * VEC;
  const bool c_ok = c < a.C;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ydesc = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
  Pack<T, VEC> raw[16];

  // Offset of a window element = row part + column part.  A row outside the image contributes
  // 2^31 and a column outside 2^30: with x below 1 GiB every sum that contains one of them lies
  // beyond the buffer, so no per-element select is needed.
  auto load_window = [&](int blk) {
    const int p = blk * kThinTiles + pl;
    const bool valid = p < a.P && c_ok;
    const int q = fast_div(p, a.div_nW);
    const int tw = p - q * a.nW;
    const int b = fast_div(q, a.div_nH);
    const int th = q - b * a.nH;
    const int y0 = 2 * th - a.pad1, x0 = 2 * tw - a.pad2;
    const unsigned row0 = (unsigned)(b * a.H + y0) * (unsigned)a.row_bytes;
    const unsigned col0 = (unsigned)(x0 * a.C + c) * (unsigned)sizeof(T);
    unsigned rowoff[4], coloff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      rowoff[i] = valid && (unsigned)(y0 + i) < (unsigned)a.H ? row0 + i * a.row_bytes : 0x80000000u;
      coloff[i] = (unsigned)(x0 + i) < (unsigned)a.W ? col0 + i * a.C * (unsigned)sizeof(T) : 0x40000000u;
    }
#pragma unroll
    for (int i1 = 0; i1 < 4; ++i1)
#pragma unroll
      for (int i2 = 0; i2 < 4; ++i2) raw[i1 * 4 + i2] = buffer_load_pack<T, VEC>(rsrc, rowoff[i1] + coloff[i2]);
  };

  const int nwg = gridDim.x;
  int blk = xcd_remap(blockIdx.x, a.per_xcd);
  if (blk < a.n_blocks) load_window(blk);   // in flight while U arrives

  // this wavefront's part of U: row operand, lane = output channel kbase + lane % 16, 8 channels
  // from 8 * (lane / 16).  Rows beyond K repeat row K - 1: a row of U only reaches the same row of the
  // product, and those rows are never stored.
  // Memory is read in whole rows (consecutive lanes take consecutive 16 bytes) and the fragments go to the lanes
  // that need them through this wavefront's own slice of LDS, which nothing else uses yet: a load whose
  // neighbouring lanes address different rows, as the operand layout would have it, measured 3.8 times slower per
  // byte with every line in L2, and for a workgroup with one block of tiles that load is most of the kernel.
  Frag u[NROW * 4][KS];
  {
    constexpr int NW = NT / 64;
    constexpr int SLICE = 2 * BUF / NW;                // bytes of LDS per wavefront
    constexpr int EPR = SLICE / (16 * PITCH);          // elements per round: 16 rows of U each
    constexpr int NEL = NROW * 4;
    static_assert(EPR >= 1 && NEL % EPR == 0 && KS == PITCH / 64, "staging of U");
    unsigned char* slice = lds + wave * SLICE;
    const unsigned char* Ub = static_cast<const unsigned char*>(a.U);
    uint4v tmp[NEL][KS];
    int srow[KS], scol[KS];
#pragma unroll
    for (int i = 0; i < KS; ++i) {
      const int off = (i * 64 + lane) * 16;            // byte of the 16-row block
      srow[i] = off / PITCH;
      scol[i] = off % PITCH;
    }
    static_for<0, NEL>([&](auto t_) {
      constexpr int t = decltype(t_)::value;
#pragma unroll
      for (int i = 0; i < KS; ++i) {
        const long long row = (long long)(row0i * 4 + t) * a.K + min(kbase + srow[i], a.K - 1);
        tmp[t][i] = *reinterpret_cast<const uint4v*>(Ub + row * PITCH + scol[i]);
      }
    });
    const int fswz = ((lane & 15) / RPL) & (CPRW - 1);
    static_for<0, NEL / EPR>([&](auto r_) {
      constexpr int rd = decltype(r_)::value;
      static_for<0, EPR>([&](auto e_) {
        constexpr int e = decltype(e_)::value;
#pragma unroll
        for (int i = 0; i < KS; ++i)
          *reinterpret_cast<uint4v*>(slice + (e * 16 + srow[i]) * PITCH +
                                     (((scol[i] >> 4) ^ ((srow[i] / RPL) & (CPRW - 1))) << 4)) = tmp[rd * EPR + e][i];
      });
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
      static_for<0, EPR>([&](auto e_) {
        constexpr int e = decltype(e_)::value;
        static_for<0, KS>([&](auto s_) {
          constexpr int s2 = decltype(s_)::value;
          u[rd * EPR + e][s2] = *reinterpret_cast<const Frag*>(slice + (e * 16 + (lane & 15)) * PITCH +
                                                              ((((lane >> 4) + 4 * s2) ^ fswz) << 4));
        });
      });
      __builtin_amdgcn_fence(__ATOMIC_RELEASE, "wavefront");
      __builtin_amdgcn_wave_barrier();
      __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "wavefront");
    });
  }

  // U and the bias have arrived before the loop starts: a wait for them inside the loop would also wait, on
  // every pass, for the window loads of the next block, which are younger (loads return in order).
  float bv[4];
  load_bias<T>(a, kbase + 4 * (lane >> 4), bv);
#pragma unroll
  for (int t = 0; t < NROW * 4; ++t)
#pragma unroll
    for (int s2 = 0; s2 < KS; ++s2) asm volatile("" : "+v"(u[t][s2]));
#pragma unroll
  for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(bv[r]));
  __syncthreads();   // the first block's V goes where other wavefronts staged their U

  for (int it = 0; blk < a.n_blocks; blk += nwg, ++it) {
    unsigned char* buf = lds + (it & 1) * BUF;
    // Input transform, two channels at a time.  fp16 adds pairs of channels
    // in fp16 like the reference's kernels (calculation_kernels.cu:786-806 computes in T); bf16,
    // which has no packed add, goes through fp32.
    // all channels of this thread lie in one chunk
    const int cb = c * (int)sizeof(T);
    T* vdst = reinterpret_cast<T*>(buf + pl * PITCH + ((((cb >> 4) ^ ((pl / RPL) & (CPRW - 1))) << 4) | (cb & 15)));
    static_for<0, VEC / 2>([&](auto h_) {
      constexpr int h = decltype(h_)::value;
      if constexpr (std::is_same<T, half_t>::value) {
        half2v d[16], t2[16];
#pragma unroll
        for (int e = 0; e < 16; ++e) d[e] = half2v{raw[e].v[2 * h], raw[e].v[2 * h + 1]};
        bt23<1, 4>(d, t2);
        bt23<4, 1>(t2, d);
#pragma unroll
        for (int e = 0; e < 16; ++e)
          *reinterpret_cast<half2v*>(vdst + e * (kThinTiles * PITCH / (int)sizeof(T)) + 2 * h) = d[e];
      } else {
        typedef float float2v __attribute__((ext_vector_type(2)));
        float2v d[16], t2[16];
#pragma unroll
        for (int e = 0; e < 16; ++e)
          d[e] = float2v{static_cast<float>(raw[e].v[2 * h]), static_cast<float>(raw[e].v[2 * h + 1])};
        bt23<1, 4>(d, t2);
        bt23<4, 1>(t2, d);
#pragma unroll
        for (int e = 0; e < 16; ++e) {
          const float o[2] = {d[e][0], d[e][1]};
          store_pack<T, 2>(vdst + e * (kThinTiles * PITCH / (int)sizeof(T)) + 2 * h, o);
        }
      }
    });
    __syncthreads();
    if (blk + nwg < a.n_blocks) load_window(blk + nwg);

    // The products M[i][j] = U[i][j] V[i][j] over the channels, and the width half of the output transform,
    // zw[i][0] = M[i][0] + M[i][1] + M[i][2], zw[i][1] = M[i][1] - M[i][2] - M[i][3].  16-bit types do the sums in
    // the accumulators (z0 takes j = 0, 1, 2; zp takes j = 1 and zn j = 2, 3, so that no operand needs its sign
    // changed): 24 MFMAs per channel step instead of 16, 12 accumulators instead of 16, no VALU work - their
    // MFMAs are cheap and registers are what is short.  fp32, whose MFMAs are sixteen times slower and bound the
    // kernel, keeps one accumulator per element and adds in VALU.  Consecutive MFMAs write different accumulators.
    floatx4 zw[NROW][2];
    const unsigned char* vrow = buf + (lane & 15) * PITCH + row0i * 4 * kThinTiles * PITCH;
    const int vswz = ((lane & 15) / RPL) & (CPRW - 1);
    if constexpr (PLAIN) {
      floatx4 mm[NROW][4];
#pragma unroll
      for (int i = 0; i < NROW; ++i)
#pragma unroll
        for (int j = 0; j < 4; ++j) mm[i][j] = floatx4{0.f, 0.f, 0.f, 0.f};
      static_for<0, KS>([&](auto s_) {
        constexpr int s = decltype(s_)::value;
        static_for<0, 4>([&](auto j_) {
          constexpr int j = decltype(j_)::value;
          Frag v[NROW];
          static_for<0, NROW>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            v[i] = *reinterpret_cast<const Frag*>(vrow + (i * 4 + j) * kThinTiles * PITCH + ((((lane >> 4) + 4 * s) ^ vswz) << 4));
          });
          static_for<0, NROW>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            mm[i][j] = MF::run(u[i * 4 + j][s], v[i], mm[i][j]);
          });
        });
      });
#pragma unroll
      for (int i = 0; i < NROW; ++i) {
        zw[i][0] = mm[i][0] + mm[i][1] + mm[i][2];
        zw[i][1] = mm[i][1] - mm[i][2] - mm[i][3];
      }
    } else {
      floatx4 z0[NROW], zp[NROW], zn[NROW];
#pragma unroll
      for (int i = 0; i < NROW; ++i) z0[i] = zp[i] = zn[i] = floatx4{0.f, 0.f, 0.f, 0.f};
      static_for<0, KS>([&](auto s_) {
        constexpr int s = decltype(s_)::value;
        static_for<0, 4>([&](auto j_) {
          constexpr int j = decltype(j_)::value;
          Frag v[NROW];
          static_for<0, NROW>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            v[i] = *reinterpret_cast<const Frag*>(vrow + (i * 4 + j) * kThinTiles * PITCH + ((((lane >> 4) + 4 * s) ^ vswz) << 4));
          });
          static_for<0, NROW>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            if constexpr (j <= 2) z0[i] = MF::run(u[i * 4 + j][s], v[i], z0[i]);
          });
          static_for<0, NROW>([&](auto i_) {
            constexpr int i = decltype(i_)::value;
            if constexpr (j == 1) zp[i] = MF::run(u[i * 4 + j][s], v[i], zp[i]);
            if constexpr (j >= 2) zn[i] = MF::run(u[i * 4 + j][s], v[i], zn[i]);
          });
        });
      });
#pragma unroll
      for (int i = 0; i < NROW; ++i) {
        zw[i][0] = z0[i];
        zw[i][1] = zp[i] - zn[i];
      }
    }

    // Height half of the output transform: out[0][b] = zw[0][b] + zw[1][b] + zw[2][b], out[1][b] = zw[1][b] -
    // zw[2][b] - zw[3][b].
    floatx4 out[2][2];
    if constexpr (!SPLIT) {
#pragma unroll
      for (int ob = 0; ob < 2; ++ob) {
        out[0][ob] = zw[0][ob] + zw[1][ob] + zw[2][ob];
        out[1][ob] = zw[1][ob] - zw[2][ob] - zw[3][ob];
      }
    } else {
      // the upper wavefronts (rows 2, 3) pass their share through LDS to the lower ones (rows 0, 1)
      floatx4* xch = reinterpret_cast<floatx4*>(lds + 2 * BUF) + ((wave % KSUB) * 4) * 64 + lane;
      const bool upper = wave >= KSUB;
#pragma unroll
      for (int ob = 0; ob < 2; ++ob) {
        const floatx4 za = zw[0][ob], zb = zw[1][ob];
        out[0][ob] = upper ? za : za + zb;
        out[1][ob] = upper ? -za - zb : zb;
      }
      if (upper) {
#pragma unroll
        for (int q = 0; q < 4; ++q) xch[q * 64] = out[q >> 1][q & 1];
      }
      __syncthreads();
      if (!upper) {
#pragma unroll
        for (int q = 0; q < 4; ++q) out[q >> 1][q & 1] += xch[q * 64];
      }
    }

    // lane = tile lane % 16, output channels ko .. ko + 4
    const int p = blk * kThinTiles + (lane & 15);
    const int ko = kbase + 4 * (lane >> 4);
    store_tile<T, KW>(a, ydesc, p, ko, p < a.P && ko < a.K && (!SPLIT || wave < KSUB), bv, out);
  }
}

// The same for at most 4 input channels (first layers: grey or RGB images), any storage type.  Padding 3
// channels to the 32 of the batched GEMM makes V ten times the input, and M is 4x the output whatever
// the channel count, so the three-kernel path spends its time on buffers; here the product runs on
// v_mfma_f32_16x16x4_f32 in fp32 with a reduction of exactly 4 channels, U (16 elements x 16 output
// channels x 4) is 16 registers per lane, and a block is 64 tiles: a thread transforms one channel of
// one tile, a wavefront multiplies four column blocks of 16 tiles.
template <typename T, bool KW>
__global__ __launch_bounds__(256) void tiny_conv3x3_kernel(ThinArgs a) {
  constexpr int TILES = 64;
  constexpr int BUF = 16 * TILES * 4;     // floats per buffer, [element][tile][channel]
  extern __shared__ __attribute__((aligned(16))) unsigned char lds[];
  float* ldsf = reinterpret_cast<float*>(lds);
  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int kbase = blockIdx.y * kThinK + wave * 16;
  const int pl = tid >> 2, c = tid & 3;
  const bool c_ok = c < a.C;
  const __amdgpu_buffer_rsrc_t rsrc =
      __builtin_amdgcn_make_buffer_rsrc(const_cast<void*>(a.x), 0, a.x_bytes, 0x00020000);
  const __amdgpu_buffer_rsrc_t ydesc = __builtin_amdgcn_make_buffer_rsrc(a.y, 0, a.y_bytes, 0x00020000);
  Pack<T, 1> raw[16];

  auto load_window = [&](int blk) {      // offsets as in thin_conv3x3_kernel
    const int p = blk * TILES + pl;
    const bool valid = p < a.P && c_ok;
    const int q = fast_div(p, a.div_nW);
    const int tw = p - q * a.nW;
    const int b = fast_div(q, a.div_nH);
    const int th = q - b * a.nH;
    const int y0 = 2 * th - a.pad1, x0 = 2 * tw - a.pad2;
    const unsigned row0 = (unsigned)(b * a.H + y0) * (unsigned)a.row_bytes;
    const unsigned col0 = (unsigned)(x0 * a.C + c) * (unsigned)sizeof(T);
    unsigned rowoff[4], coloff[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
      rowoff[i] = valid && (unsigned)(y0 + i) < (unsigned)a.H ? row0 + i * a.row_bytes : 0x80000000u;
      coloff[i] = (unsigned)(x0 + i) < (unsigned)a.W ? col0 + i * a.C * (unsigned)sizeof(T) : 0x40000000u;
    }
#pragma unroll
    for (int i1 = 0; i1 < 4; ++i1)
#pragma unroll
      for (int i2 = 0; i2 < 4; ++i2) raw[i1 * 4 + i2] = buffer_load_pack<T, 1>(rsrc, rowoff[i1] + coloff[i2]);
  };

  const int nwg = gridDim.x;
  int blk = xcd_remap(blockIdx.x, a.per_xcd);
  if (blk < a.n_blocks) load_window(blk);

  // U as the row operand: lane = output channel kbase + lane % 16, input channel lane / 16 (U's rows are
  // Cp long, channels beyond C hold zeros)
  float u[16];
  {
    const int ko = min(kbase + (lane & 15), a.K - 1);
    const T* U = static_cast<const T*>(a.U) + (long long)ko * a.Cp + (lane >> 4);
#pragma unroll
    for (int t = 0; t < 16; ++t) u[t] = static_cast<float>(U[(long long)t * a.K * a.Cp]);
  }

  float bv[4];
  load_bias<T>(a, kbase + 4 * (lane >> 4), bv);
#pragma unroll
  for (int t = 0; t < 16; ++t) asm volatile("" : "+v"(u[t]));
#pragma unroll
  for (int r = 0; r < 4; ++r) asm volatile("" : "+v"(bv[r]));

  for (int it = 0; blk < a.n_blocks; blk += nwg, ++it) {
    float* buf = ldsf + (it & 1) * BUF;
    {
      float d[16], t2[16];
#pragma unroll
      for (int e = 0; e < 16; ++e) d[e] = static_cast<float>(raw[e].v[0]);
      bt23<1, 4>(d, t2);
      bt23<4, 1>(t2, d);
#pragma unroll
      for (int e = 0; e < 16; ++e) buf[(e * TILES + pl) * 4 + c] = d[e];
    }
    __syncthreads();
    if (blk + nwg < a.n_blocks) load_window(blk + nwg);

#pragma unroll 1
    for (int cb = 0; cb < TILES / 16; ++cb) {
      floatx4 z0[4], zp[4], zn[4];
#pragma unroll
      for (int i = 0; i < 4; ++i) z0[i] = zp[i] = zn[i] = floatx4{0.f, 0.f, 0.f, 0.f};
      const float* vcol = buf + (cb * 16 + (lane & 15)) * 4 + (lane >> 4);
      static_for<0, 4>([&](auto j_) {
        constexpr int j = decltype(j_)::value;
        float v[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) v[i] = vcol[(i * 4 + j) * TILES * 4];
#pragma unroll
        for (int i = 0; i < 4; ++i)
          if constexpr (j <= 2) z0[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(u[i * 4 + j], v[i], z0[i], 0, 0, 0);
#pragma unroll
        for (int i = 0; i < 4; ++i) {
          if constexpr (j == 1) zp[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(u[i * 4 + j], v[i], zp[i], 0, 0, 0);
          if constexpr (j >= 2) zn[i] = __builtin_amdgcn_mfma_f32_16x16x4f32(u[i * 4 + j], v[i], zn[i], 0, 0, 0);
        }
      });
      floatx4 out[2][2];
#pragma unroll
      for (int ob = 0; ob < 2; ++ob) {
        floatx4 z[4];
#pragma unroll
        for (int i = 0; i < 4; ++i) z[i] = ob == 0 ? z0[i] : zp[i] - zn[i];
        out[0][ob] = z[0] + z[1] + z[2];
        out[1][ob] = z[1] - z[2] - z[3];
      }
      const int p = blk * TILES + cb * 16 + (lane & 15);
      const int ko = kbase + 4 * (lane >> 4);
      store_tile<T, KW>(a, ydesc, p, ko, p < a.P && ko < a.K, bv, out);
    }
  }
}

template <typename T>
int launch_tiny(ThinArgs a, int k_groups, void* stream) {
  constexpr int lds = 2 * 16 * 64 * 4 * 4;
  a.n_blocks = ceil_div(a.P, 64);
  int wgs = std::min(a.n_blocks, std::max(kXcds, 1024 / k_groups / kXcds * kXcds));
  a.per_xcd = ceil_div(wgs, kXcds);
  if (a.k_whole)
    hipLaunchKernelGGL((tiny_conv3x3_kernel<T, true>), dim3((unsigned)(a.per_xcd * kXcds), (unsigned)k_groups), dim3(256), lds,
                       as_stream(stream), a);
  else
    hipLaunchKernelGGL((tiny_conv3x3_kernel<T, false>), dim3((unsigned)(a.per_xcd * kXcds), (unsigned)k_groups), dim3(256), lds,
                       as_stream(stream), a);
  WC_CHECK_LAUNCH("tiny_conv3x3_kernel");
  return WC_OK;
}

template <typename T, int CP, int KSUB>
int launch_thin_groups(ThinArgs a, void* stream) {
  constexpr bool split = CP * sizeof(T) > 128;
  constexpr int lds = 2 * 16 * kThinTiles * CP * (int)sizeof(T) + (split ? KSUB * 4 * 64 * 16 : 0);
  const int k_groups = ceil_div(a.K, 16 * KSUB);
  // workgroups that stay resident (registers and LDS): two per CU, one of the eight-wavefront form;
  // shared among the groups of output channels, in whole multiples of the 8 XCDs
  int wgs = std::min(a.n_blocks, std::max(kXcds, (split ? 256 : 512) / k_groups / kXcds * kXcds));
  a.per_xcd = ceil_div(wgs, kXcds);
  auto fn = a.k_whole ? &thin_conv3x3_kernel<T, CP, true, KSUB> : &thin_conv3x3_kernel<T, CP, false, KSUB>;
  if (int rc = ensure_dynamic_lds(reinterpret_cast<const void*>(fn), lds)) return rc;
  hipLaunchKernelGGL(fn, dim3((unsigned)(a.per_xcd * kXcds), (unsigned)k_groups),
                     dim3((split ? 128 : 64) * KSUB), lds, as_stream(stream), a);
  WC_CHECK_LAUNCH("thin_conv3x3_kernel");
  return WC_OK;
}

template <typename T, int CP>
int launch_thin(ThinArgs a, void* stream) {
  // half-size workgroups while the full-size ones would fill at most half of the CUs (their threads transform
  // twice the channels each, and a thread's channels must be all inside C or all outside)
  constexpr int vec2 = kThinTiles * CP / ((CP * sizeof(T) > 128 ? 128 : 64) * 2);
  const int forced = test_gemm_config();            // wc_test_gemm_override: 8 = full size, 9 = half size
  const bool half = forced == 9 || (forced != 8 && (long long)a.n_blocks * ceil_div(a.K, kThinK) * 2 <= kCus);
  if (half && a.C % vec2 == 0) return launch_thin_groups<T, CP, 2>(a, stream);
  return launch_thin_groups<T, CP, 4>(a, stream);
}

}  // namespace

bool thin_conv_fits(const wc_conv_desc* d, const wc_plan* plan) {
  if (d->ndim != 2 || d->whole_kernel) return false;
  if (plan->n_pieces != 1 || plan->tap_step != 1 || plan->m[0] != 1 || plan->m[1] != 2 || plan->m[2] != 2) return false;
  const wc_piece& pc = plan->piece[0];
  if (pc.r[0] != 1 || pc.r[1] != 3 || pc.r[2] != 3) return false;
  const long long es = d->dtype == WC_F32 ? 4 : 2;
  if ((long long)d->N * d->in[1] * d->in[2] * d->C * es >= (1ll << 30)) return false;   // 32-bit offsets into x, two spare bits
  int out[3], grid[3];
  if (wc_conv_out_dims(d, out, grid) != WC_OK) return false;
  if ((long long)d->N * out[1] * out[2] * d->K * es >= (1ll << 31)) return false;      // and into y
  if (d->C <= 4) return d->K <= 8 * kThinK;          // tiny_conv3x3_kernel, any storage type
  const int Cp = wc_padded_channels(d->C);
  if (d->dtype == WC_F32) {
    // fp32: U of 32 channels fits four wavefronts, of 64 channels eight (the products run on fp32 MFMA)
    if (Cp > 64 || d->C % 2 != 0) return false;
    return d->K <= (Cp == 64 ? 4 : 8) * kThinK;
  }
  if (Cp > 128 || (Cp == 96) || d->C % (Cp == 32 ? 2 : 4) != 0) return false;
  return d->K <= (Cp == 128 ? 4 : 8) * kThinK;   // measured: no gain beyond (K = 512 at 128 channels: 0.97x)
}

int thin_conv_forward(const wc_conv_desc* d, const wc_plan* plan, const void* x, const void* U, const void* bias,
                      void* y, void* stream) {
  WC_CHECK_ARG(thin_conv_fits(d, plan), "thin_conv_forward: problem outside the kernel's range");
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);
  if (rc) return rc;
  const int Cp = wc_padded_channels(d->C);
  const long long P = (long long)d->N * grid[1] * grid[2];
  WC_CHECK_ARG(P < (1ll << 31) - kThinTiles, "thin_conv_forward: too many tiles");
  WC_CHECK_ARG((reinterpret_cast<uintptr_t>(x) & 7) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
                   (reinterpret_cast<uintptr_t>(U) & 15) == 0,
               "thin_conv_forward: x must be 8-byte aligned, y and U 16-byte aligned");
  const int es = d->dtype == WC_F32 ? 4 : 2;
  ThinArgs a;
  a.x = x; a.U = U; a.bias = bias; a.y = y;
  a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.K = d->K; a.Cp = Cp;
  a.oH = out[1]; a.oW = out[2]; a.nH = grid[1]; a.nW = grid[2];
  a.pad1 = d->pad[1]; a.pad2 = d->pad[2];
  a.P = (int)P;
  a.n_blocks = (int)ceil_div_ll(P, kThinTiles);
  a.per_xcd = 0;
  a.x_bytes = (int)((long long)d->N * d->in[1] * d->in[2] * d->C * es);
  a.y_bytes = (int)((long long)d->N * out[1] * out[2] * d->K * es);
  a.k_whole = d->K % 4 == 0;
  a.row_bytes = d->in[2] * d->C * es;
  a.div_nW = make_fast_div(a.nW);
  a.div_nH = make_fast_div(a.nH);
  const int k_groups = ceil_div(d->K, kThinK);
  if (d->C <= 4) return dispatch_dtype(d->dtype, [&](auto t) -> int { return launch_tiny<decltype(t)>(a, k_groups, stream); });
  return dispatch_dtype(d->dtype, [&](auto t) -> int {
    using T = decltype(t);
    if constexpr (sizeof(T) == 2) {
      if (Cp == 128) return launch_thin<T, 128>(a, stream);
      return Cp == 64 ? launch_thin<T, 64>(a, stream) : launch_thin<T, 32>(a, stream);
    } else {
      return Cp == 64 ? launch_thin<T, 64>(a, stream) : launch_thin<T, 32>(a, stream);
    }
  });
}

}  // namespace wc
