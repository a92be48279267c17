// Direct form for strided first layers: at most 4 input channels, stride 2, kernels of 3, 5 or 7 rows and at most 8
// columns, 16-bit types (ResNet's 3 -> 64, 7x7, stride 2).
//
// The reference hands every strided layer to the stock convolution (conv.py:326-332) and exits on stride 2 in its own
// launcher (src/winograd_conv.cpp:122-126).  The Winograd plans of this engine pad 3 channels to 32 once per parity phase
// and the other direct kernels want whole blocks of 32 channels, so neither fits a layer whose whole reduction is
// 7 x 7 x 3 = 147 long.  Here the reduction axis is (kernel row, tap, channel) with the channels padded to 4 and the
// taps of a row to 8: one kernel row is 32 elements, two MFMA steps of 16, and a lane's 8-element fragment is two
// neighbouring pixels of the padded input row - 16 bytes at a 16-byte aligned address, because at stride 2 the first
// tap of output column ox is input column 2 ox.
//
// A workgroup (four wavefronts) owns tiles of 16 x 16 output pixels x 64 output channels and walks over tiles
// persistently.  Per tile the input patch (2 x 15 + kh rows of 2 x 15 + 8 pixels) goes global -> registers -> LDS with
// the channels padded to 4 (zero outside the image; patches are requested two tiles ahead, into two sets of registers,
// and LDS holds two patches); the filter fragments of a wavefront's 64 output channels (kh x 2 x 2
// fragments) stay in registers for the life of the workgroup; 8 kh `v_mfma_f32_32x32x16` per wavefront and tile; the
// result leaves through LDS as whole 128-byte pixel rows with the bias added before the one rounding.  x is read once
// (plus the halo of the tiles), y written once, nothing else touches memory.  x may be channel-last or channel-first
// (wc_conv_desc.x_layout): the patch loader takes the four element strides, so a torch tensor in its default layout
// needs no copy (N=32, 3 -> 64, 224x224: 0.026 ms either way; a channel-last copy of x first costs 0.04 ms more).
#include "wc_common.h"

namespace wc {

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef __bf16 bf16x8 __attribute__((ext_vector_type(8)));
typedef float f32x16 __attribute__((ext_vector_type(16)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));

template <typename T> struct MfmaF;
template <> struct MfmaF<half_t> {
  using Frag = f16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_f16(a, b, c, 0, 0, 0); }
};
template <> struct MfmaF<bf16_t> {
  using Frag = bf16x8;
  __device__ static __forceinline__ f32x16 run(Frag a, Frag b, f32x16 c) { return __builtin_amdgcn_mfma_f32_32x32x16_bf16(a, b, c, 0, 0, 0); }
};

constexpr int kTile = 16;                       // output pixels per tile edge
constexpr int kPatchW = 2 * (kTile - 1) + 8;    // 38 input pixels per patch row
constexpr int kPitch = 40;                      // patch row pitch in pixels (8 bytes each)

struct FirstArgs {
  const void* x; const void* U; const void* bias; void* y;
  int N, H, W, C, K, pad_h, pad_w, oH, oW;
  long long sb, sy, sx, sc;                    // element strides of x: image, row, pixel, channel (channel-last or channel-first)
  int tiles_x, tiles_y, n_tiles;               // tiles per image row / column, tiles in all (over the images)
};

template <typename T, int KH>
__global__ __launch_bounds__(256, 2) void first_strided_kernel(FirstArgs a) {
  using MF = MfmaF<T>;
  constexpr int PH = 2 * (kTile - 1) + KH;                 // patch rows
  constexpr int PATCH = PH * kPitch * 8;                   // bytes
  constexpr int NPIX = PH * kPatchW;                       // pixels a patch loads
  constexpr int NL = (NPIX + 255) / 256;                   // pixels per thread
  __shared__ __attribute__((aligned(16))) unsigned char lds[2 * PATCH + 4 * 32 * 128];

  const int tid = threadIdx.x, lane = tid & 63, wave = tid >> 6;
  const int l32 = lane & 31, lhi = lane >> 5;
  const int k0 = blockIdx.y * 64;
  const uint16_t* xb = static_cast<const uint16_t*>(a.x);

  // filter fragments of this lane's two output channels (k0 + l32, k0 + 32 + l32): U is (K, KH, 4, 8), the 8
  // elements of (ky, n) being taps 2 n and 2 n + 1 with their 4 channels
  typename MF::Frag uf[2][KH][2];
#pragma unroll
  for (int j = 0; j < 2; ++j) {
    const int k = min(k0 + 32 * j + l32, a.K - 1);
#pragma unroll
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk)
        uf[j][ky][kk] = *reinterpret_cast<const typename MF::Frag*>(static_cast<const T*>(a.U) + (((long long)k * KH + ky) * 4 + 2 * kk + lhi) * 8);
  }

  // patch pixels of this thread: q = tid + 256 n -> (row, column)
  int prow[NL], pcol[NL];
#pragma unroll
  for (int n = 0; n < NL; ++n) {
    const int q = tid + 256 * n;
    prow[n] = q < NPIX ? q / kPatchW : -1;
    pcol[n] = q - (q / kPatchW) * kPatchW;
  }
  uint16_t pva[NL][4], pvb[NL][4];             // the patches of the next two tiles, on their way
  auto load_patch = [&](int tile, uint16_t (&pv)[NL][4]) {
    const int tx = tile % a.tiles_x, ty = (tile / a.tiles_x) % a.tiles_y, b = tile / (a.tiles_x * a.tiles_y);
    const int iy0 = 2 * ty * kTile - a.pad_h, ix0 = 2 * tx * kTile - a.pad_w;
#pragma unroll
    for (int n = 0; n < NL; ++n) {
      const int iy = iy0 + prow[n], ix = ix0 + pcol[n];
      const bool ok = prow[n] >= 0 && (unsigned)iy < (unsigned)a.H && (unsigned)ix < (unsigned)a.W;
      const uint16_t* p = xb + b * a.sb + (ok ? iy : 0) * a.sy + (ok ? ix : 0) * a.sx;
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
      if (prow[n] < 0) continue;
      u32x2 w;
      w[0] = (uint32_t)pv[n][0] | ((uint32_t)pv[n][1] << 16);
      w[1] = (uint32_t)pv[n][2] | ((uint32_t)pv[n][3] << 16);
      *reinterpret_cast<u32x2*>(lds + buf * PATCH + (prow[n] * kPitch + pcol[n]) * 8) = w;
    }
  };

  // this lane's pixels of the tile: wavefront w owns tile rows 4 w .. 4 w + 3; block i, lane l32: row 4 w + 2 i + l32 / 16
  int frag_off[2];
#pragma unroll
  for (int i = 0; i < 2; ++i) {
    const int ty = 4 * wave + 2 * i + (l32 >> 4), tx = l32 & 15;
    frag_off[i] = (2 * ty * kPitch + 2 * tx + 2 * lhi) * 8;
  }
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
    for (int ky = 0; ky < KH; ++ky)
#pragma unroll
      for (int kk = 0; kk < 2; ++kk) {
        typename MF::Frag vf[2];
#pragma unroll
        for (int i = 0; i < 2; ++i)
          vf[i] = *reinterpret_cast<const typename MF::Frag*>(patch + frag_off[i] + (ky * kPitch + 4 * kk) * 8);
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
          for (int j = 0; j < 2; ++j) acc[i][j] = MF::run(uf[j][ky][kk], vf[i], acc[i][j]);
      }
    // epilogue: 32 pixels x 64 channels per block row through this wavefront's staging block (128-byte rows, the
    // 16-byte chunks of a row swizzled by the row), then whole pixel rows to y
    const int tx0 = (tile % a.tiles_x) * kTile, ty0 = ((tile / a.tiles_x) % a.tiles_y) * kTile, b = tile / (a.tiles_x * a.tiles_y);
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
          *reinterpret_cast<u32x4*>(yb + (((long long)b * a.oH + oy) * a.oW + ox) * a.K + k) = val;
      }
    }
    buf ^= 1;
  };
  for (; tile < a.n_tiles; tile += 2 * gridDim.x) {
    do_tile(tile, pva);
    if (tile + (int)gridDim.x < a.n_tiles) do_tile(tile + gridDim.x, pvb);
  }
}

using FirstKernel = void (*)(FirstArgs);
template <typename T>
FirstKernel pick_first(int kh) {
  switch (kh) {
    case 3: return &first_strided_kernel<T, 3>;
    case 5: return &first_strided_kernel<T, 5>;
    case 7: return &first_strided_kernel<T, 7>;
    default: return nullptr;
  }
}

struct FirstFilterArgs {
  const void* w; void* U;
  long long s[5];
  int K, C, kh, kw;
  long long total;       // K kh 32
};

// U (K, kh, 8 taps, 4 channels) = the filter with zeros for the taps and channels it does not have
template <typename T>
__global__ __launch_bounds__(256) void first_filter_kernel(FirstFilterArgs a) {
  const long long idx = (long long)blockIdx.x * 256 + threadIdx.x;
  if (idx >= a.total) return;
  const int c = (int)(idx & 3), kx = (int)((idx >> 2) & 7);
  long long q = idx >> 5;
  const int ky = (int)(q % a.kh);
  const long long k = q / a.kh;
  T v = static_cast<T>(0.f);
  if (c < a.C && kx < a.kw) v = static_cast<const T*>(a.w)[k * a.s[0] + c * a.s[1] + ky * a.s[3] + kx * a.s[4]];
  static_cast<T*>(a.U)[idx] = v;
}

}  // namespace

bool direct_first_fits(const wc_conv_desc* d) {
  if (d->ndim != 2 || d->stride != 2 || d->whole_kernel) return false;
  if (d->dtype != WC_F16 && d->dtype != WC_BF16) return false;
  if (d->C < 1 || d->C > 4 || d->K % 8 != 0) return false;
  const int kh = d->kernel[1], kw = d->kernel[2];
  if ((kh != 3 && kh != 5 && kh != 7) || kw < 1 || kw > 8) return false;
  return d->in[0] == 1 && d->kernel[0] == 1 && d->pad[0] == 0;
}

size_t direct_first_u_elems(const wc_conv_desc* d) { return (size_t)d->K * d->kernel[1] * 32; }

int direct_first_filter(const wc_conv_desc* d, const void* w, const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(w && w_strides && U, "first-layer filter copy: null pointer");
  FirstFilterArgs a;
  a.w = w; a.U = U;
  for (int i = 0; i < 5; ++i) a.s[i] = w_strides[i];
  a.K = d->K; a.C = d->C; a.kh = d->kernel[1]; a.kw = d->kernel[2];
  a.total = (long long)direct_first_u_elems(d);
  const unsigned blocks = (unsigned)ceil_div_ll(a.total, 256);
  if (d->dtype == WC_F16) hipLaunchKernelGGL(first_filter_kernel<half_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  else hipLaunchKernelGGL(first_filter_kernel<bf16_t>, dim3(blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("first_filter_kernel");
  return WC_OK;
}

int direct_first_conv(const wc_conv_desc* d, const void* x, int n_images, const void* U, const void* bias, void* y,
                      int oH, int oW, void* stream) {
  WC_CHECK_ARG(x && U && y, "direct_first_conv: null pointer");
  WC_CHECK_ARG(direct_first_fits(d), "direct_first_conv: problem outside the kernel's range");
  WC_CHECK_ARG((reinterpret_cast<uintptr_t>(U) & 15) == 0 && (reinterpret_cast<uintptr_t>(y) & 15) == 0 &&
               (reinterpret_cast<uintptr_t>(x) & 1) == 0, "direct_first_conv: U and y must be 16-byte aligned");
  FirstArgs a;
  a.x = x; a.U = U; a.bias = bias; a.y = y;
  a.N = n_images; a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.K = d->K; a.pad_h = d->pad[1]; a.pad_w = d->pad[2];
  a.oH = oH; a.oW = oW;
  if (d->x_layout == 1) { a.sb = (long long)a.C * a.H * a.W; a.sc = (long long)a.H * a.W; a.sy = a.W; a.sx = 1; }
  else { a.sb = (long long)a.H * a.W * a.C; a.sy = (long long)a.W * a.C; a.sx = a.C; a.sc = 1; }
  a.tiles_x = ceil_div(oW, kTile); a.tiles_y = ceil_div(oH, kTile);
  const long long tiles = (long long)a.tiles_x * a.tiles_y * n_images;
  WC_CHECK_ARG(tiles > 0 && tiles < (1ll << 30) && (long long)n_images * a.H * a.W < (1ll << 31), "direct_first_conv: problem too large");
  a.n_tiles = (int)tiles;
  FirstKernel fn = d->dtype == WC_F16 ? pick_first<half_t>(d->kernel[1]) : pick_first<bf16_t>(d->kernel[1]);
  WC_CHECK_ARG(fn != nullptr, "direct_first_conv: kernels of %d rows", d->kernel[1]);
  const int k_blocks = ceil_div(d->K, 64);
  // persistent workgroups: two per CU, fewer where the tiles do not fill them
  int grid = 2 * kCus / k_blocks;
  if (grid < 1) grid = 1;
  if (grid > a.n_tiles) grid = a.n_tiles;
  hipLaunchKernelGGL(fn, dim3((unsigned)grid, (unsigned)k_blocks), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("first_strided_kernel");
  return WC_OK;
}

}  // namespace wc
