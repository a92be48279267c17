// Direct form for 3-D first layers: at most 4 input channels, a 3x3x3 kernel at stride 1, 16-bit types (the stem of
// C3D / I3D style networks: 3 -> 64 on 16 x 112 x 112 clips).
//
// The reference sends every 3x3x3 layer to the stock convolution (conv.py:467-473).  The Winograd plans of this engine
// pad 3 channels to 32 and make V, at F(2,3)^3, eighty times the input (N=8, 3 -> 64, 16x112x112 in fp16: 1.05 ms,
// MIOpen 0.41-0.57 ms); the layer itself is bound by writing y.  Here, as in first_strided_kernel (direct_first.hip), the
// reduction axis is (kernel plane, kernel row, tap, channel) with the channels and the taps of a row both padded to 4:
// one kernel row is 16 elements, one MFMA step, and a lane's 8-element fragment is two neighbouring pixels of the padded
// input row (two 8-byte LDS reads: at stride 1 the first tap of output column ox is input column ox, any parity).
//
// A workgroup (four wavefronts) owns tiles of 16 x 16 output pixels of one output plane x 64 output channels and walks
// over tiles persistently.  Per tile the input patch (3 planes of 18 rows of 19 pixels) goes global -> registers ->
// LDS with the channels padded to 4 (zero outside the image; patches are requested two tiles ahead, into two sets of
// registers, and LDS holds two patches); the filter fragments of the workgroup's 64 output channels (9 rows x 2
// channel blocks) stay in LDS; 36 `v_mfma_f32_32x32x16` per wavefront and tile; the result leaves through LDS as
// whole 128-byte pixel rows with the bias added before the one rounding.  The taps a kernel row does not have meet
// zeros on both sides (the filter's padding, and the fragment's half for them is cleared: a pixel beside the window
// may hold anything, infinities included).  x may be channel-last or channel-first (five element strides).
#include "wc_common.h"

namespace wc {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct MfmaG;
template <> struct MfmaG<half_t> {
  using Frag = f16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaG<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

constexpr int kTile = 16;                 // output pixels per tile edge
constexpr int kPatchW = kTile + 3;        // input pixels per patch row (kernel rows of at most 4 taps)
constexpr int kPitch = 20;                // patch row pitch in pixels (8 bytes each)

struct First3dArgs {
  const void* x; const void* U; const void* bias; void* y;
  int N, D, H, W, C, K, kw, pad_d, pad_h, pad_w, oD, oH, oW;
  long long sb, sz, sy, sx, sc;           // element strides of x: clip, plane, row, pixel, channel
  int tiles_x, tiles_y, n_tiles;          // tiles per plane row / column, tiles in all (over planes and clips)
};

template <typename T, int KD, int KH>
__global__ __launch_bounds__(256, 3) void first3d_kernel(First3dArgs a) {
  using MF = MfmaG<T>;
  using Frag = typename MF::Frag;
  constexpr int R = KD * KH;                               // kernel rows = MFMA steps
  constexpr int PH = kTile + KH - 1;                       // patch rows per plane
  constexpr int PLANE = PH * kPitch * 8;                   // bytes
  constexpr int PATCH = KD * PLANE;
  constexpr int NPIX = KD * PH * kPatchW;                  // pixels a patch loads
  constexpr int NL = (NPIX + 255) / 256;                   // pixels per thread
  constexpr int UBYTES = 2 * R * 64 * 16;                  // the filter fragments of 64 output channels: (block, row, lane) x 16 bytes
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * PATCH + 4 * 32 * 128 + UBYTES];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int k0 = blockIdx.y * 64;
  const uint16_t* xb = static_cast<const uint16_t*>(a.x);

  // filter fragments of the workgroup's 64 output channels, in LDS in the order the lanes read them (block j, row r,
  // lane: the 16 bytes of output channel k0 + 32 j + l32, taps 2 lhi and 2 lhi + 1 of U (K, R, 4 taps, 4 channels));
  // in registers they would cost 8 R registers and a wavefront per SIMD
  unsigned char* ulds = lds + 2 * PATCH + 4 * 32 * 128;
  for (int q = tid; q < 2 * R * 64; q += 256) {
    const int ln = q & 63, r = (q >> 6) % R, j = q / (64 * R);
    const int k = min(k0 + 32 * j + (ln & 31), a.K - 1);
    *reinterpret_cast<u32x4*>(ulds + q * 16) =
        *reinterpret_cast<const u32x4*>(static_cast<const T*>(a.U) + ((long long)k * R + r) * 16 + (ln >> 5) * 8);
  }
  const unsigned char* ufrag = ulds + lane * 16;

  // patch pixels of this thread: q = tid + 256 n -> (plane, row, column)
  int pz[NL], prow[NL], pcol[NL];
#pragma unroll
  for (int n = 0; n < NL; ++n) {
    const int q = tid + 256 * n;
    const int zz = q / (PH * kPatchW), rem = q - zz * (PH * kPatchW);
    pz[n] = q < NPIX ? zz : -1;
    prow[n] = rem / kPatchW;
    pcol[n] = rem - prow[n] * kPatchW;
  }
  uint16_t pva[NL][4], pvb[NL][4];             // the patches of the next two tiles, on their way
  auto decode = [&](int tile, int& tx, int& ty, int& od, int& b) {
    tx = tile % a.tiles_x;
    int q = tile / a.tiles_x;
    ty = q % a.tiles_y; q /= a.tiles_y;
    od = q % a.oD;
    b = q / a.oD;
  };
  auto load_patch = [&](int tile, uint16_t (&pv)[NL][4]) {
    int tx, ty, od, b;
    decode(tile, tx, ty, od, b);
    const int iz0 = od - a.pad_d, iy0 = ty * kTile - a.pad_h, ix0 = tx * kTile - a.pad_w;
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int iz = iz0 + pz[n], iy = iy0 + prow[n], ix = ix0 + pcol[n];
      const bool ok = pz[n] >= 0 && (unsigned)iz < (unsigned)a.D && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
      const uint16_t* p = xb + b * a.sb + (ok ? iz : 0) * a.sz + (ok ? iy : 0) * a.sy + (ok ? ix : 0) * a.sx;
#pragma unroll
      for (int c = 0; c < 4; ++c) {
        uint16_t v = 0;
        if (c < a.C) v = p[c * a.sc];              // (uniform branch: C is the same for every lane)
        pv[n][c] = ok ? v : (uint16_t)0;
      }
    }
  };
  auto store_patch = [&](int buf, const uint16_t (&pv)[NL][4]) {
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      if (pz[n] < 0) continue;
      u32x2 w;
      w[0] = (uint32_t)pv[n][0] | ((uint32_t)pv[n][1] << 16);
      w[1] = (uint32_t)pv[n][2] | ((uint32_t)pv[n][3] << 16);
      *reinterpret_cast<u32x2*>(lds + buf * PATCH + pz[n] * PLANE + (prow[n] * kPitch + pcol[n]) * 8) = w;
    }
  };

  // this lane's pixels of the tile: wavefront w owns tile rows 4 w .. 4 w + 3; block i, lane l32: row 4 w + 2 i + l32 / 16
  int frag_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ty = 4 * wave + 2 * i + (l32 >> 4), tx = l32 & 15;
    frag_off[i] = (ty * kPitch + tx + 2 * lhi) * 8;
  }
  // which of the lane's two taps the kernel row has
  const bool tap0_real = 2 * lhi < a.kw, tap1_real = 2 * lhi + 1 < a.kw;
  unsigned char* stg = lds + 2 * PATCH + wave * (32 * 128);
  T* yb = static_cast<T*>(a.y);

  int tile = blockIdx.x;
  if (tile >= a.n_tiles) return;
  load_patch(tile, pva);
  if (tile + (int)gridDim.x < a.n_tiles) load_patch(tile + gridDim.x, pvb);
  int buf = 0;
  // one tile; `mine`: the registers its patch arrived in, refilled with the patch of the tile after next (the memory
  // latency under load is longer than one tile's work: with one tile ahead every tile waited for its patch)
  auto do_tile = [&](int tile, uint16_t (&mine)[NL][4]) {
    store_patch(buf, mine);
    __syncthreads();                                    // the patch is complete; the other buffer is free (its tile is done)
    const int next = tile + 2 * gridDim.x;
    if (next < a.n_tiles) load_patch(next, mine);
    f32x16 acc[2][2];
#pragma unroll
    for (int i = 0; i < 2; ++i)
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int e = 0; e < 16; ++e) acc[i][j][e] = 0.f;
    const unsigned char* patch = lds + buf * PATCH;
#pragma unroll
    for (int kz = 0; kz < KD; ++kz)
#pragma unroll
      for (int ky = 0; ky < KH; ++ky) {
        Frag vf[2], uf[2];
#pragma unroll
        for (int j = 0; j < 2; ++j) uf[j] = *reinterpret_cast<const Frag*>(ufrag + (j * R + kz * KH + ky) * (64 * 16));
#pragma unroll
        for (int i = 0; i < 2; ++i) {
          const unsigned char* p = patch + kz * PLANE + ky * kPitch * 8 + frag_off[i];
          u32x2 lo = *reinterpret_cast<const u32x2*>(p), hi = *reinterpret_cast<const u32x2*>(p + 8);
          u32x4 both;
          both[0] = tap0_real ? lo[0] : 0u; both[1] = tap0_real ? lo[1] : 0u;
          both[2] = tap1_real ? hi[0] : 0u; both[3] = tap1_real ? hi[1] : 0u;
          __builtin_memcpy(&vf[i], &both, 16);
        }
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = MF::run(uf[j], vf[i], acc[i][j]);
      }
    // epilogue: 32 pixels x 64 channels per block row through this wavefront's staging block (128-byte rows, the
    // 16-byte chunks of a row swizzled by the row), then whole pixel rows to y
    int tx, ty, od, b;
    decode(tile, tx, ty, od, b);
    const int tx0 = tx * kTile, ty0 = ty * kTile;
#pragma unroll
    for (int i = 0; i < 2; ++i) {
#pragma unroll
      for (int j = 0; j < 2; ++j)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
          Pack<T, 4> o;
          float bv[4] = {0.f, 0.f, 0.f, 0.f};
          if (a.bias) {
            const int kb = k0 + j * 32 + 8 * q + 4 * lhi;
#pragma unroll
            for (int e = 0; e < 4; ++e)
              if (kb + e < a.K) bv[e] = static_cast<float>(static_cast<const T*>(a.bias)[kb + e]);
          }
#pragma unroll
          for (int e = 0; e < 4; ++e) o.v[e] = static_cast<T>(acc[i][j][4 * q + e] + bv[e]);
          const int chunk = (4 * j + q) ^ (l32 & 7);
          *reinterpret_cast<Pack<T, 4>*>(stg + l32 * 128 + chunk * 16 + lhi * 8) = o;
        }
#pragma unroll
      for (int r0 = 0; r0 < 32; r0 += 8) {
        const int row = r0 + (lane >> 3), c = lane & 7;
        const u32x4 val = *reinterpret_cast<const u32x4*>(stg + row * 128 + ((c ^ (row & 7)) * 16));
        const int oy = ty0 + 4 * wave + 2 * i + (row >> 4), ox = tx0 + (row & 15);
        const int k = k0 + c * 8;
        if (oy < a.oH && ox < a.oW && k < a.K)
          *reinterpret_cast<u32x4*>(yb + ((((long long)b * a.oD + od) * a.oH + oy) * a.oW + ox) * a.K + k) = val;
      }
    }
    buf ^= 1;
  };
  for (; tile < a.n_tiles; tile += 2 * gridDim.x) {
    do_tile(tile, pva);
    if (tile + (int)gridDim.x < a.n_tiles) do_tile(tile + gridDim.x, pvb);
  }
}

struct First3dFilterArgs {
  const void* w; void* U;
  long long s[5];
  int K, C, kd, kh, kw;
  long long total;       // K kd kh 16
};

// U (K, kd kh rows, 4 taps, 4 channels) = the filter with zeros for the taps and channels it does not have
template <typename T>
__global__ __launch_bounds__(256) void first3d_filter_kernel(First3dFilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int c = (int)(idx & 3), kx = (int)((idx >> 2) & 3);
  long long q = idx >> 4;
  const int ky = (int)(q % a.kh); q /= a.kh;
  const int kz = (int)(q % a.kd);
  const long long k = q / a.kd;
  T v = static_cast<T>(0.f);
  if (c < a.C && kx < a.kw) v = static_cast<const T*>(a.w)[k * a.s[0] + c * a.s[1] + kz * a.s[2] + ky * a.s[3] + kx * a.s[4]];
  static_cast<T*>(a.U)[idx] = v;
}

}  // namespace

bool direct_first3d_fits(const wc_conv_desc* d) {
  if (d->ndim != 3 || d->stride != 1 || d->whole_kernel) return false;
  if (d->dtype != WC_F16 && d->dtype != WC_BF16) return false;
  if (d->C < 1 || d->C > 4 || d->K % 8 != 0) return false;
  return d->kernel[0] == 3 && d->kernel[1] == 3 && d->kernel[2] >= 1 && d->kernel[2] <= 4;
}

size_t direct_first3d_u_elems(const wc_conv_desc* d) { return (size_t)d->K * d->kernel[0] * d->kernel[1] * 16; }

int direct_first3d_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(w && w_strides && U, "3-D first-layer filter copy: null pointer");
  First3dFilterArgs a;
  a.w = w; a.U = U;
  for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
  a.K = d->K; a.C = d->C; a.kd = d->kernel[0]; a.kh = d->kernel[1]; a.kw = d->kernel[2];
  a.total = (long long)direct_first3d_u_elems(d);
  const unsigned blocks = (unsigned)ceil_div_ll(a.total, 256);
  if (d->dtype == WC_F16) hipLaunchKernelGGL(first3d_filter_kernel<half_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  else hipLaunchKernelGGL(first3d_filter_kernel<bf16_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("first3d_filter_kernel");
  return WC_OK;
}

int direct_first3d_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y,
                        const int out[3], void* stream) {
  WC_CHECK_ARG(x && U && y, "direct_first3d_conv: null pointer");
  WC_CHECK_ARG(direct_first3d_fits(d), "direct_first3d_conv: problem outside the kernel's range");
  WC_CHECK_ARG((reinterpret_cast<uintptr_t>(U) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
               (reinterpret_cast<uintptr_t>(x) & 1) == 0, "direct_first3d_conv: U and y must be 16-byte aligned");
  First3dArgs a;
  a.x = x; a.U = U; a.bias = bias; a.y = y;
  a.N = n_images; a.D = d->in[0]; a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.K = d->K; a.kw = d->kernel[2];
  a.pad_d = d->pad[0]; a.pad_h = d->pad[1]; a.pad_w = d->pad[2];
  a.oD = out[0]; a.oH = out[1]; a.oW = out[2];
  const long long plane = (long long)a.H * a.W, clip = plane * a.D;
  if (d->x_layout == 1) { a.sb = clip * a.C; a.sc = clip; a.sz = plane; a.sy = a.W; a.sx = 1; }
  else { a.sb = clip * a.C; a.sz = plane * a.C; a.sy = (long long)a.W * a.C; a.sx = a.C; a.sc = 1; }
  a.tiles_x = ceil_div(a.oW, kTile); a.tiles_y = ceil_div(a.oH, kTile);
  const long long tiles = (long long)a.tiles_x * a.tiles_y * a.oD * n_images;
  WC_CHECK_ARG(tiles > 0 && tiles < (1ll << 30) && (long long)n_images * clip < (1ll << 31), "direct_first3d_conv: problem too large");
  a.n_tiles = (int)tiles;
  auto fn = d->dtype == WC_F16 ? &first3d_kernel<half_t, 3, 3> : &first3d_kernel<bf16_t, 3, 3>;
  const int k_blocks = ceil_div(d->K, 64);
  // persistent workgroups: three per CU, fewer where the tiles do not fill them
  int grid = 3 * kCus / k_blocks;
  if (grid < 1) grid = 1;
  if (grid > a.n_tiles) grid = a.n_tiles;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid, (unsigned)k_blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("first3d_kernel");
  return WC_OK;
}

}  // namespace wc
