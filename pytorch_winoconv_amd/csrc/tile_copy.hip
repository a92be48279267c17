// wino_split / wino_concat: overlapping-tile gather and cropped tile scatter (bit-exact copies).
//
// Index maps follow the reference kernels (src/split_and_concat_kernels.cu:8-129) with the
// tile step taken from m instead of the reference's hard-coded 2:
//   split : tiles[((b*nD+d)*nH+h)*nW+w][c][k][i][j] = x[b][m*d+k][m*h+i][m*w+j][c], 0 outside
//   concat: y[b][m*d+k][m*h+i][m*w+j][c] = tiles[((b*nD+d)*nH+h)*nW+w][c][k][i][j] if inside
//
// Both are pure HBM-bound copies.  One workgroup moves one tile x 64 channels through LDS so
// that the channel-last side is accessed with lanes along C and the tile side as one
// contiguous run of 64*E elements (the reference writes E scalars per lane with stride E).
#include "wc_common.h"

namespace wc {

constexpr int kCC = 64;        // channels per workgroup
constexpr int kMaxE = 216;     // largest tile (6x6x6) staged in LDS

struct TileArgs {
  const void* src;
  void* dst;
  int B, D, H, W, C;          // channel-last tensor (input of split / output of concat)
  int bD, bH, bW;             // tile extents
  int m;                      // tile step
  int nD, nH, nW;
  int c_chunks;
};

template <typename U>
__global__ __launch_bounds__(256) void wino_split_kernel(TileArgs a) {
  extern __shared__ unsigned char lds_raw[];
  U* lds = reinterpret_cast<U*>(lds_raw);
  const int E = a.bD * a.bH * a.bW;
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks;
  int p = blk / a.c_chunks;
  const int tw = p % a.nW; int q = p / a.nW;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  const U* x = static_cast<const U*>(a.src);
  // gather: lanes along channels
  for (int idx = threadIdx.x; idx < E * kCC; idx += 256) {
    const int c = idx % kCC, e = idx / kCC;
    const int j = e % a.bW; const int r = e / a.bW;
    const int i = r % a.bH, k = r / a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx = a.m * tw + j;
    U v = 0;
    if (c < cn && z < a.D && yy < a.H && xx < a.W)
      v = x[((((long long)b * a.D + z) * a.H + yy) * a.W + xx) * a.C + c0 + c];
    lds[e * (kCC + 1) + c] = v;
  }
  __syncthreads();
  // tiles[p][c0 + c][e] for c < cn is one contiguous run of cn*E elements
  U* out = static_cast<U*>(a.dst) + ((long long)p * a.C + c0) * E;
  for (int o = threadIdx.x; o < cn * E; o += 256) {
    const int c = o / E, e = o % E;
    out[o] = lds[e * (kCC + 1) + c];
  }
}

template <typename U>
__global__ __launch_bounds__(256) void wino_concat_kernel(TileArgs a) {
  extern __shared__ unsigned char lds_raw[];
  U* lds = reinterpret_cast<U*>(lds_raw);
  const int E = a.bD * a.bH * a.bW;
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks;
  int p = blk / a.c_chunks;
  const int tw = p % a.nW; int q = p / a.nW;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  const U* in = static_cast<const U*>(a.src) + ((long long)p * a.C + c0) * E;
  for (int o = threadIdx.x; o < cn * E; o += 256) {
    const int c = o / E, e = o % E;
    lds[e * (kCC + 1) + c] = in[o];
  }
  __syncthreads();
  U* y = static_cast<U*>(a.dst);
  for (int idx = threadIdx.x; idx < E * kCC; idx += 256) {
    const int c = idx % kCC, e = idx / kCC;
    const int j = e % a.bW; const int r = e / a.bW;
    const int i = r % a.bH, k = r / a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx = a.m * tw + j;
    if (c < cn && z < a.D && yy < a.H && xx < a.W)
      y[((((long long)b * a.D + z) * a.H + yy) * a.W + xx) * a.C + c0 + c] = lds[e * (kCC + 1) + c];
  }
}

static int launch_tiles(bool split, const void* src, void* dst, int B, int D, int H, int W, int C,
                        int bD, int bH, int bW, int m, int nD, int nH, int nW, int elem_size,
                        void* stream) {
  const char* name = split ? "wino_split" : "wino_concat";
  WC_CHECK_ARG(src && dst, "%s: null pointer", name);
  WC_CHECK_ARG(B > 0 && D > 0 && H > 0 && W > 0 && C > 0, "%s: non-positive tensor extent", name);
  WC_CHECK_ARG(bD > 0 && bH > 0 && bW > 0 && m > 0, "%s: non-positive tile extent", name);
  WC_CHECK_ARG(nD > 0 && nH > 0 && nW > 0, "%s: non-positive tile count", name);
  WC_CHECK_ARG(elem_size == 2 || elem_size == 4, "%s: element size %d (2 or 4)", name, elem_size);
  if (bD * bH * bW > kMaxE)
    return fail(WC_ERR_UNSUPPORTED, "%s: tile of %d elements exceeds %d", name, bD * bH * bW, kMaxE);
  const long long blocks = (long long)B * nD * nH * nW * ceil_div(C, kCC);
  WC_CHECK_ARG(blocks < (1ll << 31), "%s: too many tiles", name);
  TileArgs a{src, dst, B, D, H, W, C, bD, bH, bW, m, nD, nH, nW, ceil_div(C, kCC)};
  hipStream_t s = as_stream(stream);
  const size_t lds = (size_t)bD * bH * bW * (kCC + 1) * elem_size;   // <= 56 KB
  if (split) {
    if (elem_size == 4) wino_split_kernel<uint32_t><<<(unsigned)blocks, 256, lds, s>>>(a);
    else wino_split_kernel<uint16_t><<<(unsigned)blocks, 256, lds, s>>>(a);
  } else {
    if (elem_size == 4) wino_concat_kernel<uint32_t><<<(unsigned)blocks, 256, lds, s>>>(a);
    else wino_concat_kernel<uint16_t><<<(unsigned)blocks, 256, lds, s>>>(a);
  }
  WC_CHECK_LAUNCH(name);
  return WC_OK;
}

}  // namespace wc

using namespace wc;

extern "C" {

int wc_wino_split2d(const void* x, void* tiles, int B, int H, int W, int C, int block_H,
                    int block_W, int m, int nH, int nW, int elem_size, void* stream) {
  return launch_tiles(true, x, tiles, B, 1, H, W, C, 1, block_H, block_W, m, 1, nH, nW, elem_size, stream);
}
int wc_wino_split3d(const void* x, void* tiles, int B, int D, int H, int W, int C, int block_D,
                    int block_H, int block_W, int m, int nD, int nH, int nW, int elem_size,
                    void* stream) {
  return launch_tiles(true, x, tiles, B, D, H, W, C, block_D, block_H, block_W, m, nD, nH, nW, elem_size, stream);
}
int wc_wino_concat2d(const void* tiles, void* y, int B, int oH, int oW, int K, int m,
                     int elem_size, void* stream) {
  WC_CHECK_ARG(m > 0, "wino_concat: non-positive tile extent");
  return launch_tiles(false, tiles, y, B, 1, oH, oW, K, 1, m, m, m, 1, ceil_div(oH, m), ceil_div(oW, m), elem_size, stream);
}
int wc_wino_concat3d(const void* tiles, void* y, int B, int oD, int oH, int oW, int K, int m,
                     int elem_size, void* stream) {
  WC_CHECK_ARG(m > 0, "wino_concat: non-positive tile extent");
  return launch_tiles(false, tiles, y, B, oD, oH, oW, K, m, m, m, m, ceil_div(oD, m), ceil_div(oH, m), ceil_div(oW, m), elem_size, stream);
}

}  // extern "C"
