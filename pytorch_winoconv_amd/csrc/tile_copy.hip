// wino_split / wino_concat: overlapping-tile gather and cropped tile scatter (bit-exact copies).
//
// Index maps follow the reference kernels (src/split_and_concat_kernels.cu:8-129) with the
// tile step taken from m instead of the reference's hard-coded 2:
//   split : tiles[((b*nD+d)*nH+h)*nW+w][c][k][i][j] = x[b][m*d+k][m*h+i][m*w+j][c], 0 outside
//   concat: y[b][m*d+k][m*h+i][m*w+j][c] = tiles[((b*nD+d)*nH+h)*nW+w][c][k][i][j] if inside
//
// Both are pure HBM-bound copies.  A workgroup moves a row of up to 8 neighbouring tiles x 64
// channels through LDS: the channel-last side is accessed in 16-byte vectors along C (the
// overlapping window columns of neighbouring tiles are read once), the tile side as contiguous
// runs of 64*E elements per tile in 16-byte vectors (the reference writes E scalars per lane with
// stride E).  LDS holds the row channel-major in 4-byte words (wino_split_cm_kernel /
// wino_concat_cm_kernel); odd tile extents of 2-byte types keep the older pixel-major staging
// (wino_split_row_kernel / wino_concat_row_kernel).  Channel counts that are not a multiple of
// the vector length take the scalar kernels below, one tile per workgroup.
#include "wc_common.h"
#include "wc_transform.h"
#include <algorithm>

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


typedef uint32_t Vec16 __attribute__((ext_vector_type(4)));   // one 16-byte access

struct RowArgs {
  TileArgs t;
  int TW;                 // tiles along W per workgroup
  int w_groups;           // ceil(nW / TW)
  int cols;               // window columns of the workgroup's tiles together: m (TW - 1) + bW
};

// pixel (k, i, col) of the staged region -> offset of its first channel in LDS
template <typename U>
__device__ __forceinline__ int pix_off(int pixel) {
  constexpr int V = 16 / sizeof(U);
  return pixel * (kCC + V);                      // rows stay 16-byte aligned; the pad spreads the banks
}

// e -> pixel of tile 0 of the row: the table all threads use instead of dividing by runtime extents
__device__ __forceinline__ void fill_table(int* table, int E, int bH, int bW, int cols) {
  for (int e = threadIdx.x; e < E; e += 256) {
    const int j = e % bW; const int r = e / bW;
    table[e] = ((r / bH) * bH + r % bH) * cols + j;
  }
}

template <typename U>
__global__ __launch_bounds__(256) void wino_split_row_kernel(RowArgs g) {
  constexpr int V = 16 / sizeof(U);              // elements per vector
  constexpr int VPC = kCC / V;                   // vectors per pixel
  const TileArgs& a = g.t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int E = a.bD * a.bH * a.bW;
  int* table = reinterpret_cast<int*>(lds_raw);
  U* lds = reinterpret_cast<U*>(lds_raw + (E * 4 + 15) / 16 * 16);
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks; blk /= a.c_chunks;
  const int wg = blk % g.w_groups; int q = blk / g.w_groups;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int tw0 = wg * g.TW;
  const int ntw = min(g.TW, a.nW - tw0);
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  fill_table(table, E, a.bH, a.bW, g.cols);
  // gather the window of the tile row: 16-byte vectors along the channels
  const U* x = static_cast<const U*>(a.src);
  const int cols = a.m * (ntw - 1) + a.bW;
  const int pixels = a.bD * a.bH * cols;
  for (int idx = threadIdx.x; idx < pixels * VPC; idx += 256) {
    const int cv = idx % VPC, px = idx / VPC;
    const int col = px % cols; const int r = px / cols;
    const int i = r % a.bH, k = r / a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx = a.m * tw0 + col;
    Vec16 v = {0u, 0u, 0u, 0u};
    if (cv * V < cn && z < a.D && yy < a.H && xx < a.W)
      v = *reinterpret_cast<const Vec16*>(x + ((((long long)b * a.D + z) * a.H + yy) * a.W + xx) * a.C + c0 + cv * V);
    *reinterpret_cast<Vec16*>(lds + pix_off<U>((k * a.bH + i) * g.cols + col) + cv * V) = v;
  }
  __syncthreads();
  // tiles[p][c0 + c][e], c < cn: one contiguous run of cn * E elements per tile
  const long long p0 = (((long long)b * a.nD + td) * a.nH + th) * a.nW + tw0;
  const int run = cn * E;                        // a multiple of V
  for (int o = threadIdx.x * V; o < ntw * run; o += 256 * V) {
    const int t = o / run; const int w = o % run;
    int c = w / E, e = w % E;
    alignas(16) U out[V];
#pragma unroll
    for (int v = 0; v < V; ++v) {
      out[v] = lds[pix_off<U>(table[e] + a.m * t) + c];
      if (++e == E) { e = 0; ++c; }
    }
    *reinterpret_cast<Vec16*>(static_cast<U*>(a.dst) + ((p0 + t) * a.C + c0) * E + w) = *reinterpret_cast<const Vec16*>(out);
  }
}

template <typename U>
__global__ __launch_bounds__(256) void wino_concat_row_kernel(RowArgs g) {
  constexpr int V = 16 / sizeof(U);
  constexpr int VPC = kCC / V;
  const TileArgs& a = g.t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  const int E = a.bD * a.bH * a.bW;
  int* table = reinterpret_cast<int*>(lds_raw);
  U* lds = reinterpret_cast<U*>(lds_raw + (E * 4 + 15) / 16 * 16);
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks; blk /= a.c_chunks;
  const int wg = blk % g.w_groups; int q = blk / g.w_groups;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int tw0 = wg * g.TW;
  const int ntw = min(g.TW, a.nW - tw0);
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  fill_table(table, E, a.bH, a.bW, g.cols);
  __syncthreads();
  const long long p0 = (((long long)b * a.nD + td) * a.nH + th) * a.nW + tw0;
  const int run = cn * E;
  for (int o = threadIdx.x * V; o < ntw * run; o += 256 * V) {
    const int t = o / run; const int w = o % run;
    int c = w / E, e = w % E;
    alignas(16) U in[V];
    *reinterpret_cast<Vec16*>(in) = *reinterpret_cast<const Vec16*>(static_cast<const U*>(a.src) + ((p0 + t) * a.C + c0) * E + w);
#pragma unroll
    for (int v = 0; v < V; ++v) {
      lds[pix_off<U>(table[e] + a.m * t) + c] = in[v];
      if (++e == E) { e = 0; ++c; }
    }
  }
  __syncthreads();
  U* y = static_cast<U*>(a.dst);
  const int cols = a.m * ntw;                    // tiles do not overlap: bW == m
  const int pixels = a.bD * a.bH * cols;
  for (int idx = threadIdx.x; idx < pixels * VPC; idx += 256) {
    const int cv = idx % VPC, px = idx / VPC;
    const int col = px % cols; const int r = px / cols;
    const int i = r % a.bH, k = r / a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx = a.m * tw0 + col;
    if (cv * V < cn && z < a.D && yy < a.H && xx < a.W)
      *reinterpret_cast<Vec16*>(y + ((((long long)b * a.D + z) * a.H + yy) * a.W + xx) * a.C + c0 + cv * V) =
          *reinterpret_cast<const Vec16*>(lds + pix_off<U>((k * a.bH + i) * g.cols + col) + cv * V);
  }
}

// The same row of tiles with LDS held channel-major, in 4-byte words: word [c][r][w] holds the 4 / sizeof(U)
// neighbouring pixels of window row r (depth and height taken together) for channel c.  The tile layout
// (p, c, k, i, j) of the reference keeps one channel's window together, so channel-major LDS turns every word of
// a 16-byte tile-side access into ONE word-sized LDS access at a computed address (the pixel-major staging above
// needs one 2-byte access and a table lookup per element: 16 LDS instructions per 16 bytes of fp16 tiles, which
// bounded it at 3.4 TB/s).  The transposition happens on the channel-last side, where a thread that holds the 16
// bytes of two neighbouring pixels packs them into words of (pixel, pixel + 1) per channel.  The pitch of a
// channel row is odd: the words of 8 consecutive channel vectors x 8 consecutive pixel groups, and the words of
// 64 consecutive channels, fall into distinct banks.  Needs even bW and m for 2-byte elements.
struct CmArgs {
  TileArgs t;
  int TW, w_groups;
  int rows;               // bD * bH
  int dpr;                // words per window row of the whole tile row: (m (TW - 1) + bW) / EPD
  int pitch;              // words per channel: rows * dpr, made odd
  int dpc;                // words per channel of one tile: E / EPD
  int bWd, md;            // bW / EPD, m / EPD
  FastDiv div_dpr, div_bH, div_dpc, div_bWd;
  FastDiv div_vecs;       // 16-byte vectors per tile of a full channel chunk: kCC * dpc / 4
  FastDiv div_last;       // concat: words per row of the last, possibly shorter, group of tiles
};

template <typename U> struct Words;
template <> struct Words<uint32_t> {
  // one pixel per word: the 4 channels of a vector go to 4 channel rows
  static __device__ __forceinline__ void scatter(uint32_t* w, int pitch, const Vec16 (&v)[1]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) w[k * pitch] = v[0][k];
  }
  static __device__ __forceinline__ void gather(const uint32_t* w, int pitch, Vec16 (&v)[1]) {
#pragma unroll
    for (int k = 0; k < 4; ++k) v[0][k] = w[k * pitch];
  }
};
template <> struct Words<uint16_t> {
  // two pixels per word: word d of a pixel's vector holds channels 2d (low half) and 2d + 1
  static __device__ __forceinline__ void scatter(uint32_t* w, int pitch, const Vec16 (&v)[2]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t a = v[0][d], b = v[1][d];
      w[(2 * d) * pitch] = (a & 0xffffu) | (b << 16);
      w[(2 * d + 1) * pitch] = (a >> 16) | (b & 0xffff0000u);
    }
  }
  static __device__ __forceinline__ void gather(const uint32_t* w, int pitch, Vec16 (&v)[2]) {
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      const uint32_t e = w[(2 * d) * pitch], o = w[(2 * d + 1) * pitch];
      v[0][d] = (e & 0xffffu) | (o << 16);
      v[1][d] = (e >> 16) | (o & 0xffff0000u);
    }
  }
};

// Compile-time tile shapes (ROWS = bD bH, BW, M, TW tiles per workgroup; 0: taken from the arguments) turn the index
// arithmetic of both sides into shifts and constants.
template <int ROWS, int BW, int M, int TW, int EPD>
struct CmShape {
  static constexpr bool fixed = ROWS > 0;
  const CmArgs& g;
  __device__ __forceinline__ int rows() const { return fixed ? ROWS : g.rows; }
  __device__ __forceinline__ int dpr() const { return fixed ? (M * (TW - 1) + BW) / EPD : g.dpr; }
  __device__ __forceinline__ int pitch() const { return fixed ? ((ROWS * ((M * (TW - 1) + BW) / EPD)) | 1) : g.pitch; }
  __device__ __forceinline__ int dpc() const { return fixed ? ROWS * BW / EPD : g.dpc; }
  __device__ __forceinline__ int bWd() const { return fixed ? BW / EPD : g.bWd; }
  __device__ __forceinline__ int md() const { return fixed ? M / EPD : g.md; }
  __device__ __forceinline__ int div_dpr(int n) const { return fixed ? n / ((M * (TW - 1) + BW) / EPD) : fast_div(n, g.div_dpr); }
  __device__ __forceinline__ int div_dpc(int n) const { return fixed ? n / (ROWS * BW / EPD) : fast_div(n, g.div_dpc); }
  __device__ __forceinline__ int div_bWd(int n) const { return fixed ? n / (BW / EPD) : fast_div(n, g.div_bWd); }
  __device__ __forceinline__ int div_vecs(int n) const { return fixed ? n / (kCC * (ROWS * BW / EPD) / 4) : fast_div(n, g.div_vecs); }
};

template <typename U, int ROWS = 0, int BW = 0, int M = 0, int TWC = 0>
__global__ __launch_bounds__(256) void wino_split_cm_kernel(CmArgs g) {
  constexpr int V = 16 / sizeof(U), EPD = 4 / sizeof(U), VPC = kCC / V;
  const CmShape<ROWS, BW, M, TWC, EPD> sh{g};
  const TileArgs& a = g.t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint32_t* ldsw = reinterpret_cast<uint32_t*>(lds_raw);
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks; blk /= a.c_chunks;
  const int wg = blk % g.w_groups; int q = blk / g.w_groups;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int tw0 = wg * g.TW;
  const int ntw = min(g.TW, a.nW - tw0);
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  const U* x = static_cast<const U*>(a.src);
  // channel-last side: a thread takes the vectors of EPD neighbouring pixels
  const int groups = sh.rows() * sh.dpr();
  for (int idx = threadIdx.x; idx < groups * VPC; idx += 256) {
    const int cv = idx % VPC, pg = idx / VPC;
    const int r = sh.div_dpr(pg), pc = pg - r * sh.dpr();
    const int k = fast_div(r, g.div_bH), i = r - k * a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx0 = a.m * tw0 + pc * EPD;
    const bool row_ok = cv * V < cn && z < a.D && yy < a.H;
    const U* src = x + ((((long long)b * a.D + z) * a.H + yy) * a.W + xx0) * a.C + c0 + cv * V;
    Vec16 v[EPD];
#pragma unroll
    for (int e = 0; e < EPD; ++e) {
      v[e] = Vec16{0u, 0u, 0u, 0u};
      if (row_ok && xx0 + e < a.W) v[e] = *reinterpret_cast<const Vec16*>(src + (long long)e * a.C);
    }
    Words<U>::scatter(ldsw + cv * V * sh.pitch() + r * sh.dpr() + pc, sh.pitch(), v);
  }
  __syncthreads();
  // tile side: tiles[p][c0 + c][e], c < cn, is one contiguous run of cn * dpc words per tile
  const long long p0 = (((long long)b * a.nD + td) * a.nH + th) * a.nW + tw0;
  const int E = a.bD * a.bH * a.bW;
  const int vecs = cn * sh.dpc() / 4;               // 16-byte vectors per tile
  uint32_t* dst = static_cast<uint32_t*>(a.dst);
  for (int ov = threadIdx.x; ov < ntw * vecs; ov += 256) {
    const int t = cn == kCC ? sh.div_vecs(ov) : ov / vecs;
    const int q0 = (ov - t * vecs) * 4;
    int c = sh.div_dpc(q0);
    const int rem = q0 - c * sh.dpc();
    int i = sh.div_bWd(rem), j = rem - i * sh.bWd();
    const uint32_t* w = ldsw + sh.md() * t;
    Vec16 vec;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      vec[d] = w[c * sh.pitch() + i * sh.dpr() + j];
      if (++j == sh.bWd()) { j = 0; if (++i == sh.rows()) { i = 0; ++c; } }
    }
    *reinterpret_cast<Vec16*>(dst + ((p0 + t) * a.C + c0) * E / EPD + q0) = vec;
  }
}

template <typename U, int ROWS = 0, int BW = 0, int M = 0, int TWC = 0>
__global__ __launch_bounds__(256) void wino_concat_cm_kernel(CmArgs g) {
  constexpr int V = 16 / sizeof(U), EPD = 4 / sizeof(U), VPC = kCC / V;
  const CmShape<ROWS, BW, M, TWC, EPD> sh{g};
  const TileArgs& a = g.t;
  extern __shared__ __attribute__((aligned(16))) unsigned char lds_raw[];
  uint32_t* ldsw = reinterpret_cast<uint32_t*>(lds_raw);
  int blk = blockIdx.x;
  const int cc = blk % a.c_chunks; blk /= a.c_chunks;
  const int wg = blk % g.w_groups; int q = blk / g.w_groups;
  const int th = q % a.nH; q /= a.nH;
  const int td = q % a.nD;
  const int b = q / a.nD;
  const int tw0 = wg * g.TW;
  const int ntw = min(g.TW, a.nW - tw0);
  const int c0 = cc * kCC;
  const int cn = min(kCC, a.C - c0);
  const long long p0 = (((long long)b * a.nD + td) * a.nH + th) * a.nW + tw0;
  const int E = a.bD * a.bH * a.bW;
  const int vecs = cn * sh.dpc() / 4;
  const uint32_t* src = static_cast<const uint32_t*>(a.src);
  for (int ov = threadIdx.x; ov < ntw * vecs; ov += 256) {
    const int t = cn == kCC ? sh.div_vecs(ov) : ov / vecs;
    const int q0 = (ov - t * vecs) * 4;
    int c = sh.div_dpc(q0);
    const int rem = q0 - c * sh.dpc();
    int i = sh.div_bWd(rem), j = rem - i * sh.bWd();
    const Vec16 vec = *reinterpret_cast<const Vec16*>(src + ((p0 + t) * a.C + c0) * E / EPD + q0);
    uint32_t* w = ldsw + sh.md() * t;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
      w[c * sh.pitch() + i * sh.dpr() + j] = vec[d];
      if (++j == sh.bWd()) { j = 0; if (++i == sh.rows()) { i = 0; ++c; } }
    }
  }
  __syncthreads();
  U* y = static_cast<U*>(a.dst);
  const int dpr = sh.md() * ntw;                    // tiles do not overlap: bW == m
  const int groups = sh.rows() * dpr;
  const FastDiv div_row = wg == g.w_groups - 1 ? g.div_last : g.div_dpr;
  for (int idx = threadIdx.x; idx < groups * VPC; idx += 256) {
    const int cv = idx % VPC, pg = idx / VPC;
    const int r = fast_div(pg, div_row), pc = pg - r * dpr;
    const int k = fast_div(r, g.div_bH), i = r - k * a.bH;
    const int z = a.m * td + k, yy = a.m * th + i, xx0 = a.m * tw0 + pc * EPD;
    if (!(cv * V < cn && z < a.D && yy < a.H)) continue;
    Vec16 v[EPD];
    Words<U>::gather(ldsw + cv * V * sh.pitch() + r * sh.dpr() + pc, sh.pitch(), v);
    U* dst = y + ((((long long)b * a.D + z) * a.H + yy) * a.W + xx0) * a.C + c0 + cv * V;
#pragma unroll
    for (int e = 0; e < EPD; ++e)
      if (xx0 + e < a.W) *reinterpret_cast<Vec16*>(dst + (long long)e * a.C) = v[e];
  }
}

template <int R, int BW, int M, int T> struct TileShape { static constexpr int rows = R, bw = BW, m = M, tw = T; };

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
  const int V = 16 / elem_size;
  const bool aligned = (reinterpret_cast<uintptr_t>(src) % 16 == 0) && (reinterpret_cast<uintptr_t>(dst) % 16 == 0);
  const int EPD = 4 / elem_size;
  if (C % V == 0 && aligned && (split || bW == m) && bW % EPD == 0 && m % EPD == 0 && (long long)C * bD * bH * bW * elem_size % 16 == 0) {
    // a row of tiles per workgroup, staged channel-major: at most 8 tiles, fewer for large tiles (LDS)
    const int E = bD * bH * bW;
    CmArgs g;
    g.t = a;
    g.rows = bD * bH;
    auto pitch_of = [&](int t) { return (g.rows * ((m * (t - 1) + bW) / EPD)) | 1; };
    auto lds_bytes = [&](int t) { return (size_t)kCC * pitch_of(t) * 4; };
    int tw = std::min(8, nW);
    while (tw > 2 && lds_bytes(tw) > 20 * 1024) --tw;       // eight workgroups per CU when the tile allows
    while (tw > 1 && lds_bytes(tw) > 56 * 1024) --tw;
    if (lds_bytes(tw) <= 56 * 1024) {
      g.TW = tw;
      g.w_groups = ceil_div(nW, tw);
      g.dpr = (m * (tw - 1) + bW) / EPD;
      g.pitch = pitch_of(tw);
      g.dpc = E / EPD;
      g.bWd = bW / EPD;
      g.md = m / EPD;
      g.div_dpr = make_fast_div(g.dpr); g.div_bH = make_fast_div(bH);
      g.div_dpc = make_fast_div(g.dpc); g.div_bWd = make_fast_div(g.bWd);
      g.div_vecs = make_fast_div(kCC * g.dpc / 4);
      g.div_last = make_fast_div(g.md * (nW - (g.w_groups - 1) * tw));
      const long long rows = (long long)B * nD * nH * g.w_groups * a.c_chunks;
      WC_CHECK_ARG(rows < (1ll << 31), "%s: too many tiles", name);
      const size_t lb = lds_bytes(tw);
      // the 2-D tiles of F(2,3) and F(4,3), with the number of tiles per workgroup the rule above gives them when
      // the rows are long enough, have compile-time index arithmetic (1.1-1.2x over the generic form)
      bool done = false;
      auto pick = [&](auto u, auto shape) {
        using U = decltype(u);
        constexpr int R = decltype(shape)::rows, BW = decltype(shape)::bw, M = decltype(shape)::m, T = decltype(shape)::tw;
        if (done || bD != 1 || bH != R || bW != BW || m != M || tw != T || elem_size != (int)sizeof(U)) return;
        if (split) wino_split_cm_kernel<U, R, BW, M, T><<<(unsigned)rows, 256, lb, s>>>(g);
        else wino_concat_cm_kernel<U, R, BW, M, T><<<(unsigned)rows, 256, lb, s>>>(g);
        done = true;
      };
      if (split) {
        pick(uint16_t{}, TileShape<4, 4, 2, 8>{}); pick(uint32_t{}, TileShape<4, 4, 2, 8>{});
        pick(uint16_t{}, TileShape<6, 6, 4, 6>{}); pick(uint32_t{}, TileShape<6, 6, 4, 2>{});
      } else {
        pick(uint16_t{}, TileShape<2, 2, 2, 8>{}); pick(uint32_t{}, TileShape<2, 2, 2, 8>{});
        pick(uint16_t{}, TileShape<4, 4, 4, 8>{}); pick(uint32_t{}, TileShape<4, 4, 4, 4>{});
      }
      if (!done) {
        if (elem_size == 4) {
          if (split) wino_split_cm_kernel<uint32_t><<<(unsigned)rows, 256, lb, s>>>(g);
          else wino_concat_cm_kernel<uint32_t><<<(unsigned)rows, 256, lb, s>>>(g);
        } else {
          if (split) wino_split_cm_kernel<uint16_t><<<(unsigned)rows, 256, lb, s>>>(g);
          else wino_concat_cm_kernel<uint16_t><<<(unsigned)rows, 256, lb, s>>>(g);
        }
      }
      WC_CHECK_LAUNCH(name);
      return WC_OK;
    }
  }
  if (C % V == 0 && aligned && (split || bW == m)) {
    // pixel-major staging: odd tile extents in 2-byte types
    const int E = bD * bH * bW;
    RowArgs g;
    g.t = a;
    int tw = std::min(8, nW);
    auto lds_bytes = [&](int t) {
      return (size_t)(E * 4 + 15) / 16 * 16 + (size_t)bD * bH * (m * (t - 1) + bW) * (kCC + V) * elem_size;
    };
    while (tw > 2 && lds_bytes(tw) > 36 * 1024) --tw;       // four workgroups per CU when the tile allows
    while (tw > 1 && lds_bytes(tw) > 56 * 1024) --tw;
    if (lds_bytes(tw) <= 56 * 1024) {
      g.TW = tw;
      g.w_groups = ceil_div(nW, tw);
      g.cols = m * (tw - 1) + bW;
      const long long rows = (long long)B * nD * nH * g.w_groups * a.c_chunks;
      WC_CHECK_ARG(rows < (1ll << 31), "%s: too many tiles", name);
      const size_t lb = lds_bytes(tw);
      if (split) {
        if (elem_size == 4) wino_split_row_kernel<uint32_t><<<(unsigned)rows, 256, lb, s>>>(g);
        else wino_split_row_kernel<uint16_t><<<(unsigned)rows, 256, lb, s>>>(g);
      } else {
        if (elem_size == 4) wino_concat_row_kernel<uint32_t><<<(unsigned)rows, 256, lb, s>>>(g);
        else wino_concat_row_kernel<uint16_t><<<(unsigned)rows, 256, lb, s>>>(g);
      }
      WC_CHECK_LAUNCH(name);
      return WC_OK;
    }
  }
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
