// Host-side planning and error reporting (no device code).
//
// The split rule replaces the reference's 36-key look-up table
// (reference: src/base_conv_launchers.h:58-388): per axis an extent k is cut into chunks of
// 3 with the remainder last, except 4 -> 2 + 2; boxes are the Cartesian product of the
// per-axis chunks, depth outermost and width fastest; the transform-domain offset of a box
// is the running sum of prod(size + m - 1) (reference: src/base_conv_launchers.cu:307-313).
// Stride 2 - which the reference rejects (src/winograd_conv.cpp:122-126) - is handled by
// separating the taps of each axis by parity first:
//   y[o] = sum_k x[2o + k - pad] w[k] = sum_q sum_j x[2(o + j) + q - pad] w[2j + q].
#include "wc_common.h"

#include <cstdlib>
#include "wc_tables.h"
#include <atomic>
#include <cstring>
#include <mutex>
#include <string>
#include <unordered_set>

namespace wc {

static thread_local std::string g_err;

void set_error(const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_err = buf;
}

int fail(int code, const char* fmt, ...) {
  char buf[512];
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(buf, sizeof(buf), fmt, ap);
  va_end(ap);
  g_err = buf;
  return code;
}

// Kernels that need more than 64 KB of LDS must be told so once per device; the set remembers
// which (device, kernel) pairs have been, so that launches after the first pay one lookup.
int ensure_dynamic_lds(const void* fn, size_t bytes) {
  if (bytes <= 64 * 1024) return WC_OK;
  static std::mutex mu;
  static std::unordered_set<uintptr_t> done;
  int dev = 0;
  WC_CHECK_HIP(hipGetDevice(&dev));
  const uintptr_t key = reinterpret_cast<uintptr_t>(fn) * 64 + (uintptr_t)dev;
  std::lock_guard<std::mutex> lock(mu);
  if (done.count(key)) return WC_OK;
  WC_CHECK_HIP(hipFuncSetAttribute(fn, hipFuncAttributeMaxDynamicSharedMemorySize, (int)bytes));
  done.insert(key);
  return WC_OK;
}

// State of the test hook wc_test_gemm_override: per host thread, and writable only in a process whose environment
// holds WINOCONV_TEST_HOOKS=1 when the hook is first called (the test suite sets it); elsewhere the hook refuses and
// these stay at their defaults, so no caller can change what another caller's launches do.
thread_local int t_gemm_config = -1, t_gemm_rows = 1;
int test_gemm_config() { return t_gemm_config; }
int test_gemm_rows() { return t_gemm_rows; }
static bool test_hooks_enabled() {
  static const bool on = [] { const char* e = std::getenv("WINOCONV_TEST_HOOKS"); return e && e[0] == '1'; }();
  return on;
}

struct AxisPiece { int tap0, r; };

// chunks of one axis at stride 1: fills (start, size), returns the count
static int axis_chunks(int k, int* start, int* size) {
  int n = 0, s = 0;
  if (k == 4) {
    start[0] = 0; size[0] = 2; start[1] = 2; size[1] = 2;
    return 2;
  }
  while (k - s >= 3) { start[n] = s; size[n] = 3; s += 3; ++n; }
  if (k - s > 0) { start[n] = s; size[n] = k - s; ++n; }
  return n;
}

// chunks of `len` taps, the remainder last (plans whose pieces share one transformed input: len = output tile)
static int axis_even_chunks(int k, int len, AxisPiece* out) {
  int n = 0;
  for (int s = 0; s < k; s += len) { out[n].tap0 = s; out[n].r = k - s >= len ? len : k - s; ++n; }
  return n;
}

static int axis_pieces(int k, int stride, AxisPiece* out) {
  int n = 0;
  int start[8], size[8];
  for (int q = 0; q < stride; ++q) {
    int taps = (k - q + stride - 1) / stride;
    if (taps <= 0) continue;
    int c = axis_chunks(taps, start, size);
    for (int i = 0; i < c; ++i) { out[n].tap0 = q + stride * start[i]; out[n].r = size[i]; ++n; }
  }
  return n;
}

}  // namespace wc

using namespace wc;

extern "C" {

int wc_test_gemm_override(int config, int rows_mode) {
  WC_CHECK_ARG(config >= -1 && config < 16 && rows_mode >= 0 && rows_mode <= 4,
               "wc_test_gemm_override: config %d, rows_mode %d", config, rows_mode);
  if (!test_hooks_enabled())
    return fail(WC_ERR_UNSUPPORTED, "wc_test_gemm_override: test hooks are off (set WINOCONV_TEST_HOOKS=1 before the first call)");
  t_gemm_config = config;
  t_gemm_rows = rows_mode;
  return WC_OK;
}

const char* wc_version(void) { return "winoconv-hip 0.1 (gfx950)"; }
const char* wc_last_error(void) { return g_err.c_str(); }

int wc_padded_channels(int C) { return (C + 31) / 32 * 32; }
int wc_padded_channels8(int K) { return (K + 7) / 8 * 8; }

int wc_plan_dwm(int kD, int kH, int kW, int* num_split, int* D_start, int* D_end, int* H_start,
                int* H_end, int* W_start, int* W_end, int* kernel_stride, int* t_total) {
  WC_CHECK_ARG(num_split && D_start && D_end && H_start && H_end && W_start && W_end &&
                   kernel_stride && t_total, "wc_plan_dwm: null output pointer");
  if (kD < 1 || kH < 1 || kW < 1 || kD > 10 || kH > 10 || kW > 10)
    return fail(WC_ERR_UNSUPPORTED, "wc_plan_dwm: kernel %dx%dx%d outside 1..10", kD, kH, kW);
  int ds[8], dz[8], hs[8], hz[8], ws[8], wz[8];
  int nd = axis_chunks(kD, ds, dz), nh = axis_chunks(kH, hs, hz), nw = axis_chunks(kW, ws, wz);
  if (nd * nh * nw > WC_MAX_PIECES)
    return fail(WC_ERR_UNSUPPORTED, "wc_plan_dwm: %d pieces exceed %d", nd * nh * nw, WC_MAX_PIECES);
  int n = 0, t = 0;
  for (int a = 0; a < nd; ++a)
    for (int b = 0; b < nh; ++b)
      for (int c = 0; c < nw; ++c) {
        D_start[n] = ds[a]; D_end[n] = ds[a] + dz[a];
        H_start[n] = hs[b]; H_end[n] = hs[b] + hz[b];
        W_start[n] = ws[c]; W_end[n] = ws[c] + wz[c];
        kernel_stride[n] = t;
        t += (dz[a] + 1) * (hz[b] + 1) * (wz[c] + 1);
        ++n;
      }
  *num_split = n;
  *t_total = t;
  return WC_OK;
}

static int check_desc(const wc_conv_desc* d) {
  WC_CHECK_ARG(d != nullptr, "null descriptor");
  WC_CHECK_ARG(d->ndim == 2 || d->ndim == 3, "ndim must be 2 or 3, got %d", d->ndim);
  WC_CHECK_ARG(d->N > 0 && d->C > 0 && d->K > 0, "N, C, K must be positive (%d, %d, %d)", d->N, d->C, d->K);
  WC_CHECK_ARG(d->dtype == WC_F32 || d->dtype == WC_F16 || d->dtype == WC_BF16, "unknown dtype %d", d->dtype);
  for (int a = 0; a < 3; ++a) {
    WC_CHECK_ARG(d->in[a] > 0 && d->kernel[a] > 0 && d->pad[a] >= 0,
                 "axis %d: input %d, kernel %d, pad %d", a, d->in[a], d->kernel[a], d->pad[a]);
    if (d->kernel[a] > 10)
      return fail(WC_ERR_UNSUPPORTED, "kernel extent %d > 10 on axis %d", d->kernel[a], a);
    if (d->in[a] + 2 * d->pad[a] < d->kernel[a])
      return fail(WC_ERR_BAD_ARG, "axis %d: padded input %d smaller than kernel %d", a,
                  d->in[a] + 2 * d->pad[a], d->kernel[a]);
  }
  if (d->ndim == 2)
    WC_CHECK_ARG(d->in[0] == 1 && d->kernel[0] == 1 && d->pad[0] == 0,
                 "2-D problem needs depth extent 1, kernel 1, pad 0");
  if (d->stride != 1 && d->stride != 2)
    return fail(WC_ERR_UNSUPPORTED, "stride %d not implemented (1 or 2)", d->stride);
  if (d->m != 2 && d->m != 4 && !(d->m == 3 && d->stacked == 2))
    return fail(WC_ERR_UNSUPPORTED, "output tile %d not implemented (2 or 4; 3 with stacked = 2)", d->m);
  if (d->m == 4 && d->ndim == 3 &&
      !(d->stride == 1 && d->kernel[0] == 3 && d->kernel[1] == 3 && d->kernel[2] == 3))
    return fail(WC_ERR_UNSUPPORTED, "output tile 4 in 3-D (2 x 4 x 4) is implemented for 3x3x3 kernels at stride 1");
  WC_CHECK_ARG(d->chunk_images >= 0, "chunk_images must be >= 0");
  WC_CHECK_ARG(d->whole_kernel == 0 || d->whole_kernel == 1, "whole_kernel must be 0 or 1");
  WC_CHECK_ARG(d->stacked >= 0 && d->stacked <= 2, "stacked must be 0, 1 or 2");
  WC_CHECK_ARG(d->direct == 0 || d->direct == 1, "direct must be 0 or 1");
  WC_CHECK_ARG((d->x_layout == 0 || d->x_layout == 1) && (d->y_layout == 0 || d->y_layout == 1),
               "x_layout and y_layout must be 0 (channel-last) or 1 (channel-first)");
  if (d->stacked && (d->whole_kernel || (d->ndim == 3 && d->m != 2)))
    return fail(WC_ERR_UNSUPPORTED, "stacked plans are built for DWM plans with output tile 2, or 4 in 2-D");
  if (d->stacked == 2 && d->m != 2 && !(d->m == 3 && d->stride == 1))
    return fail(WC_ERR_UNSUPPORTED, "plans with a shared transformed input need output tile 2, or 3 at stride 1");
  if (d->stacked == 2 && d->m == 3 &&
      (d->ndim != 2 || d->kernel[1] < 3 || d->kernel[2] < 3 || (d->kernel[1] == 3 && d->kernel[2] == 3)))
    return fail(WC_ERR_UNSUPPORTED, "output tile 3 is built for 2-D kernels of at least 3 taps per axis and more than 3 on one");
  if (d->whole_kernel) {
    if (d->ndim != 2 || d->stride != 1 || d->m != 2)
      return fail(WC_ERR_UNSUPPORTED, "whole-kernel tiles need a 2-D problem, stride 1 and output tile 2");
    if (d->kernel[1] != d->kernel[2] || d->kernel[1] > 7)
      return fail(WC_ERR_UNSUPPORTED, "whole-kernel tiles are built for square kernels up to 7x7, got %dx%d",
                  d->kernel[1], d->kernel[2]);
  }
  return WC_OK;
}

// Stride 2 with a shared transformed input (see shared_phases in wc_common.h): positions of two
// phase taps per axis, depth outermost; inside a position the 2^d parity phases, depth parity
// outermost.  Piece (position, phase) owns the taps q + 2 j, j in [2 pos, 2 pos + 2) that the
// kernel has; a phase that runs out of taps before the others leaves pieces without any (r = 0:
// their block of U is zero).  All pieces use the tile F(2, 2) (F(2, 1) on an axis of one or two taps).
static int plan_shared_stride2(const wc_conv_desc* d, wc_plan* plan) {
  int npos[3], nq[3];
  for (int a = 0; a < 3; ++a) {
    nq[a] = shared_phases(d, a);
    npos[a] = (shared_taps(d, a) + 1) / 2;
  }
  const int np_total = npos[0] * npos[1] * npos[2] * nq[0] * nq[1] * nq[2];
  if (np_total > WC_MAX_PIECES) return fail(WC_ERR_UNSUPPORTED, "%d pieces exceed %d", np_total, WC_MAX_PIECES);
  std::memset(plan, 0, sizeof(*plan));
  plan->tap_step = 2;
  const bool flat_depth = (d->in[0] == 1 && d->kernel[0] == 1 && d->pad[0] == 0);
  plan->m[0] = flat_depth ? 1 : 2;
  plan->m[1] = plan->m[2] = 2;
  int np = 0;
  int pos[3], q[3];
  for (pos[0] = 0; pos[0] < npos[0]; ++pos[0])
    for (pos[1] = 0; pos[1] < npos[1]; ++pos[1])
      for (pos[2] = 0; pos[2] < npos[2]; ++pos[2])
        for (q[0] = 0; q[0] < nq[0]; ++q[0])
          for (q[1] = 0; q[1] < nq[1]; ++q[1])
            for (q[2] = 0; q[2] < nq[2]; ++q[2]) {
              wc_piece& p = plan->piece[np++];
              bool empty = false;
              for (int a = 0; a < 3; ++a) {
                const int taps = (d->kernel[a] - q[a] + 1) / 2;     // taps of this parity
                int r = taps - 2 * pos[a];
                r = r < 0 ? 0 : (r > 2 ? 2 : r);
                p.r[a] = r;
                p.tap0[a] = q[a] + 4 * pos[a];
                empty = empty || r == 0;
              }
              if (empty)
                for (int a = 0; a < 3; ++a) { p.r[a] = 0; p.tap0[a] = 0; }
              p.t_offset = 0;
            }
  plan->n_pieces = np;
  int t = 1;
  for (int a = 0; a < 3; ++a) {
    const int rp = shared_taps(d, a) >= 2 ? 2 : 1;
    if (kind_of(plan->m[a], rp) < 0) return fail(WC_ERR_UNSUPPORTED, "F(%d,%d) not implemented", plan->m[a], rp);
    t *= plan->m[a] + rp - 1;
  }
  plan->t_total = t;
  return WC_OK;
}

int wc_plan_conv(const wc_conv_desc* d, wc_plan* plan) {
  int rc = check_desc(d);
  if (rc) return rc;
  WC_CHECK_ARG(plan != nullptr, "wc_plan_conv: null plan");
  if (d->stacked == 2 && d->stride == 2) return plan_shared_stride2(d, plan);
  AxisPiece ax[3][8];
  int n[3];
  for (int a = 0; a < 3; ++a) {
    if (d->whole_kernel) { ax[a][0].tap0 = 0; ax[a][0].r = d->kernel[a]; n[a] = 1; }
    else if (d->stacked == 2) n[a] = axis_even_chunks(d->kernel[a], d->m, ax[a]);
    else n[a] = axis_pieces(d->kernel[a], d->stride, ax[a]);
  }
  if (n[0] * n[1] * n[2] > WC_MAX_PIECES)
    return fail(WC_ERR_UNSUPPORTED, "%d pieces exceed %d", n[0] * n[1] * n[2], WC_MAX_PIECES);
  std::memset(plan, 0, sizeof(*plan));
  plan->tap_step = d->stride;
  const bool flat_depth = (d->in[0] == 1 && d->kernel[0] == 1 && d->pad[0] == 0);
  plan->m[0] = flat_depth ? 1 : (d->m == 4 ? 2 : d->m);   // 3-D tile 4 is 2 x 4 x 4
  plan->m[1] = d->m;
  plan->m[2] = d->m;
  int np = 0, t = 0;
  for (int a = 0; a < n[0]; ++a)
    for (int b = 0; b < n[1]; ++b)
      for (int c = 0; c < n[2]; ++c) {
        wc_piece& p = plan->piece[np++];
        p.tap0[0] = ax[0][a].tap0; p.r[0] = ax[0][a].r;
        p.tap0[1] = ax[1][b].tap0; p.r[1] = ax[1][b].r;
        p.tap0[2] = ax[2][c].tap0; p.r[2] = ax[2][c].r;
        p.t_offset = t;
        int e = 1;
        for (int q = 0; q < 3; ++q) {
          if (!d->stacked && kind_of(plan->m[q], p.r[q]) < 0)      // stacked: only the shared tile counts (below)
            return fail(WC_ERR_UNSUPPORTED, "F(%d,%d) on axis %d not implemented", plan->m[q], p.r[q], q);
          e *= plan->m[q] + p.r[q] - 1;
        }
        t += e;
      }
  plan->n_pieces = np;
  plan->t_total = t;
  if (d->stacked) {
    int rp[3];
    stacked_taps(plan, rp);
    t = 1;
    for (int q = 0; q < 3; ++q) {
      if (rp[q] > 3 || kind_of(plan->m[q], rp[q]) < 0)
        return fail(WC_ERR_UNSUPPORTED, "stacked plans need pieces of at most 3 taps and a tile F(%d,%d)", plan->m[q], rp[q]);
      t *= plan->m[q] + rp[q] - 1;
    }
    for (int s = 0; s < np; ++s) plan->piece[s].t_offset = 0;
    plan->t_total = t;
  }
  return WC_OK;
}

// Which form of a DWM plan measured fastest on MI355X (wc_conv_auto, stacked == -1):
//  * 16-bit: pieces added by the batched GEMM (2-D 1.15-1.3x for 5x5 and 7x7 kernels, 3-D 1.05-1.4x: fewer
//    bytes moved); stride-1 kernels of 4 to 10 taps over at most 256 input channels (3-D: 4 to 8 taps over at
//    most 128, or 4 taps over at most 256) get the two-tap pieces that share one transformed input (against
//    stacked F(2,r) pieces 1.15-3x in 2-D at 128 and 256 channels, equal at 512; 1.5-2x in 3-D); where the
//    caller accepts tile 4 (fp16, 2-D, 5 to 10 taps, at least 3 on the other axis, at most 256 channels) the
//    shared tile is F(3,3) with three-tap pieces (1.4-1.8x faster than stacked F(4,r) pieces).  At stride 2
//    the shared-input plan works on the parity phases of x and pays where every phase has four taps (2-D 7x7
//    and 8x8 kernels, at most 256 channels: 1.2-1.75x) or, in 3-D, two or four (at most 128 channels:
//    1.65-2.5x); kernels with three taps per phase are 1.8x slower that way and keep their stacked pieces.
//  * fp32 (product bound by the MFMA rate, to which stacking adds zero taps): only 2-D plans of two to four
//    pieces are stacked (5x5: 1.1-1.15x; 7x7 with nine pieces: 0.9-1.0x).
static int auto_stacked(const wc_conv_desc* d) {
  const int nd = d->ndim;
  if (d->whole_kernel || (nd == 3 && d->m != 2)) return 0;
  const int* ks = d->kernel + (3 - nd);
  int kmax = 0, kmin = 99;
  for (int a = 0; a < nd; ++a) { kmax = ks[a] > kmax ? ks[a] : kmax; kmin = ks[a] < kmin ? ks[a] : kmin; }
  if (d->dtype != WC_F32) {
    if (d->stride == 2) {
      bool all4 = true, all24 = true;
      for (int a = 0; a < nd; ++a) {
        const int t = (ks[a] + 1) / 2;
        all4 = all4 && t == 4;
        all24 = all24 && (t == 2 || t == 4);
      }
      if (nd == 2 && all4 && d->C <= 256) return 2;
      if (nd == 3 && all24 && kmax >= 4 && d->C <= 128) return 2;
    }
    if (d->stride == 1) {
      const int cp = wc_padded_channels(d->C);
      const bool tile3 = d->dtype == WC_F16 && nd == 2 && d->m == 4 && kmin >= 3 && kmax >= 5 && kmax <= 10 && cp <= 256;
      const bool tile2 = nd == 2 ? (kmax >= 4 && kmax <= 10 && cp <= 256)
                                 : ((kmax >= 4 && kmax <= 8 && cp <= 128) || (kmax == 4 && cp <= 256));
      if (tile3 || tile2) return 2;
    }
    return 1;
  }
  if (nd != 2) return 0;
  int n = 1;
  for (int a = 0; a < nd; ++a) {
    int sum = 0;
    for (int q = 0; q < (d->stride == 2 ? 2 : 1); ++q) {
      const int t = d->stride == 2 ? (ks[a] + 1 - q) / 2 : ks[a];
      if (t > 0) sum += t == 4 ? 2 : (t + 2) / 3;
    }
    n *= sum;
  }
  return n > 1 && n <= 4 ? 1 : 0;
}

// Where the direct form measured faster than the Winograd plan the caller would otherwise get.  Stride 2 in 16-bit,
// against the parity-phase plans (MI355X, fp16, warmed clocks, filter conversion included on both sides; us,
// direct | F(2,r) plan | F(4,r) plan):
//  * Short reductions (kh kw C <= 3200) always: 3x3 at N=32, C=K=128, 112x112 57 | 160 | 126; C=K=256, 56x56
//    94 | 193 | 156; 256 -> 512 at 28x28 53 | 81 | 86; 5x5 at C=128 131 | 261 | 154; small layers too (N=8, 128 channels,
//    56x56: 22 | 28 | 29).
//  * With 64 output channels or fewer it runs 64 x 64 tiles only and loses beyond 5x5 kernels (7x7, C=K=64,
//    224x224: 382 | 372; 128 -> 64 at 112x112: 209 | 201).
//  * A long reduction needs enough output (pixels x channels >= 4 M, i.e. 256 tiles of 128 x 128) to keep the chip
//    busy, else the latency of its k-steps decides: 3x3 at C=K=512 on 14x14 images 90 | 66, 7x7 at C=K=256 on 28x28
//    240 | 139.  With that, and with one operand tile per kernel row for rows of 4 to 8 taps (direct_rows.hip): against
//    the plan that shares one transformed input (7 and 8 taps) it wins (C=K=128, 112x112: 7x7 181 | 270, 8x8 234 | 284;
//    96 channels 7x7 146 | 214, 8x8 182 | 224; 256 -> 512 on 28x28 7x7 173 | 228, 8x8 230 | 277); against stacked
//    F(2,r) pieces it wins (128 channels, 112x112: 6x6 168 | 281, 9x9 421 | 845; 256 -> 512 on 28x28 5x5 111 | 115);
//    against stacked F(4,r) pieces it wins at 4x4 (128 channels: 91 | 143; 256 -> 512: 77 | 83), from 9x9 on
//    (414 | 554) and between while the reduction stays short of 4800 (6x6 at 128 channels 152 | 182, at 96 118 | 141),
//    and loses beyond (256 -> 512 on 28x28: 5x5 101 | 98, 6x6 143 | 99).
//  * A kernel of one tap at either stride, every type: the tile F(m,1) has nothing to save and its transforms are
//    copies (fp16 N=64, 64 -> 256 channels, 56x56: three kernels 78 us).
static bool direct_preferred(const wc_conv_desc* d) {
  // 3-D first layers (direct_first3d.hip; N=8, 3 -> 64, 16x112x112 in fp16: the Winograd plan 1.05 ms)
  if (direct_first3d_fits(d)) return true;
  const int taps = d->kernel[1] * d->kernel[2];
  if (taps == 1) return true;
  if (d->stride != 2) return false;
  // fp32 products are bound by the MFMA rate, where the multiplications F(4,r) tiles save count: the direct form wins
  // for 3x3 kernels over at most 128 channels only (N=64, 128 channels, 56x56: 163 | 220 | 170; N=16, 64 channels,
  // 112x112: 55 | 77 | 65; 32 -> 64 at 112x112: 49 | 86 | 75; 256 channels on 28x28: 187 | 173 | 176; 5x5 at 128: 798 | 708 | 426)
  if (d->dtype == WC_F32) return taps <= 9 && d->C <= 128;
  // strided first layers have a kernel of their own (direct_first.hip; N=32, 3 -> 64, 7x7 on 224x224: the parity-phase
  // plans pad the 3 channels to 32 per phase)
  if (direct_first_fits(d)) return true;
  if (d->K <= 64 && taps > 25 && taps < 81) return false;      // (9x9, 64 channels, 112x112: 180 | 482 | 286)
  if ((long long)taps * d->C <= 3200) return true;
  wc_conv_desc e = *d;
  e.direct = 0; e.stacked = 0; e.m = 2; e.whole_kernel = 0;
  int out[3], grid[3];
  if (wc_conv_out_dims(&e, out, grid) != WC_OK) return false;
  if ((long long)d->N * out[1] * out[2] * d->K < (4ll << 20)) return false;
  if (auto_stacked(d) == 2) return taps <= 64;
  if (d->m == 2) return true;
  return taps <= 16 || taps >= 81 || (long long)taps * d->C <= 4800;
}

int wc_conv_auto(wc_conv_desc* d) {
  WC_CHECK_ARG(d != nullptr, "wc_conv_auto: null descriptor");
  WC_CHECK_ARG(d->ndim == 2 || d->ndim == 3, "ndim must be 2 or 3, got %d", d->ndim);
  WC_CHECK_ARG(d->stacked >= -1 && d->stacked <= 2, "stacked must be -1 (choose), 0, 1 or 2");
  WC_CHECK_ARG(d->direct >= -1 && d->direct <= 1, "direct must be -1 (never), 0 (may be chosen) or 1");
  const bool never_direct = d->direct == -1;
  if (never_direct) d->direct = 0;
  if (d->stacked == -1) {
    if (!d->direct && !never_direct && direct_conv_fits(d) && direct_preferred(d)) d->direct = 1;
    d->stacked = d->direct ? 0 : auto_stacked(d);
  }
  if (d->stacked == 2 && d->m == 4) {
    // the shared-input plan exists for output tiles 2 and 3: tile 3 (F(3,3): fp16 error 3e-3 of the output
    // range, between F(2,r) and F(4,r); too coarse for bf16) where its three-tap pieces apply, else 2
    const int kh = d->kernel[1], kw = d->kernel[2];
    const bool tile3 = d->ndim == 2 && d->stride == 1 && d->dtype == WC_F16 && (kh < kw ? kh : kw) >= 3 && (kh > kw ? kh : kw) >= 5;
    d->m = tile3 ? 3 : 2;
  }
  return WC_OK;
}

int wc_conv_out_dims(const wc_conv_desc* d, int out[3], int grid[3]) {
  int rc = check_desc(d);
  if (rc) return rc;
  WC_CHECK_ARG(out && grid, "wc_conv_out_dims: null output");
  const bool flat_depth = (d->in[0] == 1 && d->kernel[0] == 1 && d->pad[0] == 0);
  for (int a = 0; a < 3; ++a) {
    out[a] = (d->in[a] + 2 * d->pad[a] - d->kernel[a]) / d->stride + 1;
    int m = a == 0 ? (flat_depth ? 1 : (d->m == 4 ? 2 : d->m)) : d->m;
    grid[a] = (out[a] + m - 1) / m;
    // a shared transformed input covers the tiles that the pieces reach beyond the output's own
    if (d->stacked == 2) grid[a] += (shared_taps(d, a) + m - 1) / m - 1;
  }
  return WC_OK;
}

}  // extern "C"
