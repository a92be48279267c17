// Whole convolution: filter transform -> per image chunk (input transform -> batched GEMM ->
// output transform).  Replaces DWM<T> (src/winograd_conv.cpp:17-127) and
// convLauncherStrideOneLarge<T> (src/base_conv_launchers.cu:282-399) of the reference, minus
// its per-call cudaMalloc/cudaMemcpy/cudaFree of the split tables and of tmp_output
// (base_conv_launchers.cu:323-336, :375-376, :384-391) and its per-call cuBLAS handle
// (:360-361, :383): the plan travels in kernel arguments, scratch comes from the caller and
// everything is enqueued on the caller's stream.
//
// The batch is processed in chunks of images, which bounds the size of the two large
// intermediates V and M (each written once and read once).
#include "wc_common.h"

#include <cstdlib>
#include <mutex>
#include <vector>

using namespace wc;

// Scratch of wc_conv_forward_static: lives in the library's device image, one copy per GPU at that
// GPU's own address, held until the process ends.  Host code never uses this name as an address:
// static_scratch() asks the runtime for the device address once per device and hands that out.
static __device__ __align__(256) unsigned char scratch[WC_STATIC_SCRATCH_BYTES];

namespace {

constexpr int kMaxDevices = 64;
void* g_scratch_ptr[kMaxDevices];      // device address of `scratch` on each GPU, null until first asked
std::mutex g_scratch_mu;

// Device address of `scratch` on the current device.
int static_scratch(void** out) {
  int dev = 0;
  WC_CHECK_HIP(hipGetDevice(&dev));
  if (dev < 0 || dev >= kMaxDevices) return fail(WC_ERR_UNSUPPORTED, "wc_conv_forward_static: device %d", dev);
  std::lock_guard<std::mutex> lock(g_scratch_mu);
  if (!g_scratch_ptr[dev]) {
    void* ptr = nullptr;
    WC_CHECK_HIP(hipGetSymbolAddress(&ptr, HIP_SYMBOL(scratch)));
    if (!ptr || (reinterpret_cast<uintptr_t>(ptr) & 255) != 0)
      return fail(WC_ERR_HIP, "wc_conv_forward_static: bad address %p for the static scratch", ptr);
    g_scratch_ptr[dev] = ptr;
  }
  *out = g_scratch_ptr[dev];
  return WC_OK;
}

struct Layout {
  wc_plan plan;
  int out[3], grid[3];
  int Cp, ldm, chunk;   // Cp: row length of U, and of V unless the pieces share one transformed input
  int vrow;             // row length of V
  bool shared;
  SharedShift shift;
  long long tiles_per_image;
  size_t es;
  size_t u_bytes, v_bytes, m_bytes;   // each rounded up to 256
  bool thin;                          // the one-kernel path runs: V and M are not needed
  bool direct;                        // the direct form: the product reads x itself, V and M are not needed
  bool x_direct;                      // channel-first x is read by the input transform itself
  size_t xcl_bytes, ycl_bytes;        // channel-last scratch copies of a chunk of x / of y (0 if not needed)
  // 3-D F(2,3)^3 plans in 16-bit types: the width axis is taken inside the product (fold_filter_w, gemm.hip).  V and M
  // hold 16 elements per pixel column of a tile row (depth and height transformed only), half of what the plan's V and
  // M hold; the workspace also holds the filter with the width taps side by side
  bool fold;
  size_t fold_bytes;
  SharedShift fold_shift;             // one run of three pieces, each one row of V further
  long long fold_rows_per_image;      // rows of V and M: the pixel columns of all tile rows (tiles_per_image where the plan is not folded)
  size_t need() const { return (thin || direct ? u_bytes : u_bytes + fold_bytes + v_bytes + m_bytes) + xcl_bytes + ycl_bytes; }
};

size_t round256(size_t v) { return (v + 255) / 256 * 256; }

// WINOCONV_LOG=1 in the environment (read once, at the first call): wc_conv_forward prints the plan it runs to
// stderr - silent otherwise (the reference prints from inside its launchers on every call:
// src/winograd_conv.cpp:106).
bool log_enabled() {
  static const bool on = [] { const char* e = std::getenv("WINOCONV_LOG"); return e && e[0] == '1'; }();
  return on;
}

int make_layout(const wc_conv_desc* d_in, Layout* L) {
  WC_CHECK_ARG(d_in != nullptr, "null descriptor");
  // the direct form has no tiles: its shapes are those of the plain plan with the same kernel, stride and padding
  wc_conv_desc plain = *d_in;
  L->direct = d_in->direct == 1;
  if (L->direct) {
    if (!direct_conv_fits(d_in))
      return fail(WC_ERR_UNSUPPORTED, "direct form: 2-D, input channels a multiple of 32 (fp32: 16; or at most 4 at stride 2 in a 16-bit type), "
                  "output channels a multiple of 8");
    plain.direct = 0; plain.stacked = 0; plain.m = 2; plain.whole_kernel = 0; plain.unfused = 1;
  }
  const wc_conv_desc* d = &plain;
  int rc = wc_plan_conv(d, &L->plan);
  if (rc) return rc;
  rc = wc_conv_out_dims(d, L->out, L->grid);
  if (rc) return rc;
  L->Cp = stacked_row(d, &L->plan);
  L->vrow = v_row(d, &L->plan);
  L->shared = shared_input(d, &L->plan);
  L->shift = shared_shift(d, L->grid);
  L->ldm = wc_padded_channels8(d->K);
  L->es = d->dtype == WC_F32 ? 4 : 2;
  L->tiles_per_image = (long long)L->grid[0] * L->grid[1] * L->grid[2];
  const long long T = L->plan.t_total;
  int chunk = d->chunk_images;
  if (chunk <= 0) {
    // Measured on MI355X (N=64, C=K=256, 56x56, fp16): one pass over the whole batch is fastest,
    // smaller chunks lose more to partially filled launches than they gain from cache residency.
    // The chunk only bounds the scratch footprint: V + M of one chunk stay below 8 GiB.
    const double per_image = (double)T * L->tiles_per_image * (L->vrow + L->ldm) * L->es;
    chunk = (int)(8192.0 * 1024 * 1024 / per_image);
    if (chunk < 1) chunk = 1;
    // equal passes rather than full ones and a short last one
    if (chunk < d->N) chunk = (d->N + (d->N + chunk - 1) / chunk - 1) / ((d->N + chunk - 1) / chunk);
  }
  if (chunk > d->N) chunk = d->N;
  L->chunk = chunk;
  const long long Pc = L->tiles_per_image * chunk;
  if (T * Pc * (long long)(L->Cp > L->ldm ? L->Cp : L->ldm) >= (1ll << 40))
    return fail(WC_ERR_UNSUPPORTED, "chunk of %d images is too large", chunk);
  L->u_bytes = L->direct ? round256(direct_u_elems(d) * L->es)
                         : round256((size_t)T * d->K * L->Cp * L->es);
  L->v_bytes = round256((size_t)T * (Pc + (L->shared ? L->shift.tail : 0)) * L->vrow * L->es);
  L->m_bytes = round256((size_t)T * Pc * L->ldm * L->es);
  L->thin = !L->direct && !d->unfused && thin_conv_fits(d, &L->plan);
  L->fold = false; L->fold_bytes = 0;
  L->fold_rows_per_image = L->tiles_per_image;
  {
    const wc_plan& pl = L->plan;
    const bool cube = !L->direct && !L->shared && !d->whole_kernel && d->ndim == 3 && pl.n_pieces == 1 &&
                      pl.tap_step == 1 && pl.m[0] == 2 && pl.m[1] == 2 && pl.m[2] == 2 && pl.piece[0].r[0] == 3 &&
                      pl.piece[0].r[1] == 3 && pl.piece[0].r[2] == 3 && (d->dtype == WC_F16 || d->dtype == WC_BF16);
    // Half the V and M traffic for half more multiplications and one more launch: it pays where the pipeline waits
    // for memory, the more channels the larger the problem has to be.  Measured fp16, ms folded | not: N=8 16x56x56
    // 128 -> 128 channels 0.437 | 0.712, 64 -> 128 0.317 | 0.590, 64 -> 64 0.205 | 0.371; N=8 16x112x112 32 -> 32 0.455 | 0.712;
    // one 8x28x28 clip 128 -> 128 0.027 | 0.031; 8x28x28 256 -> 256 N=16 0.284 | 0.415, N=4 0.093 | 0.105, 256 -> 512 N=2
    // 0.091 | 0.094, 320 -> 320 N=4 0.138 | 0.156, 384 -> 384 N=8 0.291 | 0.367, 192 -> 192 N=4 unpadded 0.057 | 0.057;
    // 8x14x14 384 -> 384 N=4 0.062 | 0.063, 512 -> 512 N=4 0.085 | 0.077, 512 -> 128 N=8 0.087 | 0.069; 4x14x14 512 -> 512
    // N=16 0.151 | 0.130; 8x14x14 64 -> 64 N=1 0.017 | 0.016.
    // wc_test_gemm_override(11, .) switches it off, (12, .) on for every such plan.
    const int force = test_gemm_config();
    const long long min_tiles = L->Cp <= 128 ? 512 : L->Cp <= 384 ? 3000 : (1ll << 40);
    if (cube && force != 11 && (force == 12 || Pc >= min_tiles)) {
      const int Wx = columns_width(d);
      L->fold = true;
      L->fold_rows_per_image = (long long)L->grid[0] * L->grid[1] * Wx;
      L->fold_shift.n_run = 3; L->fold_shift.n_runs = 1; L->fold_shift.n_planes = 1;
      L->fold_shift.run_rows = Wx; L->fold_shift.plane_rows = Wx; L->fold_shift.tail = 2;
      const long long Pw = L->fold_rows_per_image * chunk;
      L->fold_bytes = round256((size_t)16 * d->K * 3 * L->Cp * L->es);
      L->v_bytes = round256((size_t)16 * (Pw + 2) * L->Cp * L->es);
      L->m_bytes = round256((size_t)16 * Pw * L->ldm * L->es);
    }
  }
  // channel-first tensors: the input transform of small single-piece plans reads x as it is; everything else goes
  // through a channel-last copy of one chunk (the one-kernel path: of the whole batch)
  L->x_direct = d->x_layout == 1 && ((!L->thin && !L->direct && input_transform_nchw_fits(d, &L->plan)) ||
                                     (L->direct && (direct_first_fits(d_in) || direct_first3d_fits(d_in))));      // ... and so do the first-layer kernels
  const size_t images = L->thin || L->direct ? d->N : chunk;
  const size_t x_image = (size_t)d->in[0] * d->in[1] * d->in[2] * d->C * L->es;
  const size_t y_image = (size_t)L->out[0] * L->out[1] * L->out[2] * d->K * L->es;
  L->xcl_bytes = d->x_layout == 1 && !L->x_direct ? round256(images * x_image) : 0;
  L->ycl_bytes = d->y_layout == 1 ? round256(images * y_image) : 0;
  return WC_OK;
}

// Opt-in timing of the stages of one call: a pair of events around every stage on the caller's stream, read
// after one synchronisation at the end (the reference times its phases with perf_counter and device-wide
// synchronisations around each: dwm.py:44-106).
struct StageTimer {
  struct Span { int stage; hipEvent_t t0, t1; };
  std::vector<Span> spans;
  hipStream_t stream;
  bool on;
  StageTimer(bool enabled, void* s) : stream(as_stream(s)), on(enabled) {}
  ~StageTimer() {
    for (Span& sp : spans) { (void)hipEventDestroy(sp.t0); (void)hipEventDestroy(sp.t1); }
  }
  template <typename F>
  int run(int stage, F&& f) {
    if (!on) return f();
    Span sp; sp.stage = stage;
    if (hipEventCreate(&sp.t0) != hipSuccess) return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipEventCreate failed");
    if (hipEventCreate(&sp.t1) != hipSuccess) { (void)hipEventDestroy(sp.t0); return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipEventCreate failed"); }
    spans.push_back(sp);
    if (hipEventRecord(sp.t0, stream) != hipSuccess) return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipEventRecord failed");
    const int rc = f();
    if (hipEventRecord(sp.t1, stream) != hipSuccess) return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipEventRecord failed");
    return rc;
  }
  int collect(float* stage_ms) {
    for (int i = 0; i < WC_N_STAGES; ++i) stage_ms[i] = 0.f;
    if (hipStreamSynchronize(stream) != hipSuccess) return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipStreamSynchronize failed");
    for (Span& sp : spans) {
      float ms = 0.f;
      if (hipEventElapsedTime(&ms, sp.t0, sp.t1) != hipSuccess) return fail(WC_ERR_HIP, "wc_conv_forward_timed: hipEventElapsedTime failed");
      stage_ms[sp.stage] += ms;
    }
    return WC_OK;
  }
};

int forward_impl(const wc_conv_desc* d, const void* x, const void* w, const int64_t w_strides[5],
                 const void* U_cached, const void* bias, void* y, void* workspace,
                 size_t workspace_bytes, void* stream, float* stage_ms);

}  // namespace

extern "C" {

int wc_conv_workspace_bytes(const wc_conv_desc* d, size_t* bytes) {
  WC_CHECK_ARG(bytes != nullptr, "wc_conv_workspace_bytes: null output");
  Layout L;
  int rc = make_layout(d, &L);
  if (rc) return rc;
  *bytes = L.need();
  return WC_OK;
}

int wc_conv_u_elems(const wc_conv_desc* d, size_t* elems) {
  WC_CHECK_ARG(elems != nullptr, "wc_conv_u_elems: null output");
  Layout L;
  int rc = make_layout(d, &L);
  if (rc) return rc;
  *elems = L.direct ? direct_u_elems(d) : (size_t)L.plan.t_total * d->K * L.Cp;
  return WC_OK;
}

int wc_conv_forward(const wc_conv_desc* d, const void* x, const void* w, const int64_t w_strides[5],
                    const void* U_cached, const void* bias, void* y, void* workspace,
                    size_t workspace_bytes, void* stream) {
  return forward_impl(d, x, w, w_strides, U_cached, bias, y, workspace, workspace_bytes, stream, nullptr);
}

int wc_conv_forward_timed(const wc_conv_desc* d, const void* x, const void* w, const int64_t w_strides[5],
                          const void* U_cached, const void* bias, void* y, void* workspace,
                          size_t workspace_bytes, void* stream, float stage_ms[WC_N_STAGES]) {
  WC_CHECK_ARG(stage_ms != nullptr, "wc_conv_forward_timed: null stage_ms");
  return forward_impl(d, x, w, w_strides, U_cached, bias, y, workspace, workspace_bytes, stream, stage_ms);
}

}  // extern "C"

namespace {

int forward_impl(const wc_conv_desc* d, const void* x, const void* w, const int64_t w_strides[5],
                 const void* U_cached, const void* bias, void* y, void* workspace,
                 size_t workspace_bytes, void* stream, float* stage_ms) {
  Layout L;
  int rc = make_layout(d, &L);
  if (rc) return rc;
  WC_CHECK_ARG(x && y, "wc_conv_forward: null input or output");
  WC_CHECK_ARG(U_cached || (w && w_strides), "wc_conv_forward: neither a filter nor a transformed filter");
  if (!workspace) return fail(WC_ERR_WORKSPACE, "wc_conv_forward: null workspace");
  const size_t need = L.need();
  if (workspace_bytes < need)
    return fail(WC_ERR_WORKSPACE, "wc_conv_forward: workspace of %zu bytes, %zu needed", workspace_bytes, need);
  if ((reinterpret_cast<uintptr_t>(workspace) & 255) != 0)
    return fail(WC_ERR_WORKSPACE, "wc_conv_forward: workspace must be 256-byte aligned");

  if (log_enabled()) {
    static const char* const dt[] = {"f32", "f16", "bf16"};
    std::fprintf(stderr, "winoconv: %dD %s N=%d C=%d K=%d in=%dx%dx%d kernel=%dx%dx%d stride=%d pad=%d,%d,%d | tile m=%d,%d,%d "
                 "pieces=%d T=%d stacked=%d%s | %s | chunk=%d images, tiles/image=%lld, workspace=%zu B (U %zu, V %zu, M %zu, "
                 "x copy %zu, y copy %zu) | x %s, y %s, filter %s\n",
                 d->ndim, dt[d->dtype], d->N, d->C, d->K, d->in[0], d->in[1], d->in[2], d->kernel[0], d->kernel[1], d->kernel[2],
                 d->stride, d->pad[0], d->pad[1], d->pad[2], L.plan.m[0], L.plan.m[1], L.plan.m[2], L.plan.n_pieces, L.plan.t_total,
                 d->stacked, d->whole_kernel ? " whole-kernel tile" : "",
                 L.direct ? "direct form: the product reads x" : L.thin ? "one fused kernel" : L.fold ? "input transform (depth, height), shifted batched GEMM with the width taps along its reduction, output transform" : (L.shared ? "input transform, shifted batched GEMM, output transform"
                                                         : "input transform, batched GEMM, output transform"),
                 L.thin || L.direct ? d->N : L.chunk, L.tiles_per_image, need, L.u_bytes, L.thin || L.direct ? (size_t)0 : L.v_bytes,
                 L.thin || L.direct ? (size_t)0 : L.m_bytes, L.xcl_bytes, L.ycl_bytes,
                 d->x_layout ? (L.x_direct ? "channel-first, read by the input transform" : "channel-first, copied") : "channel-last",
                 d->y_layout ? "channel-first, copied" : "channel-last", U_cached ? "transformed by the caller" : "transformed here");
  }
  unsigned char* ws = static_cast<unsigned char*>(workspace);
  void* Uws = ws;
  void* Ufold = ws + L.u_bytes;
  void* V = ws + L.u_bytes + L.fold_bytes;
  void* M = ws + L.u_bytes + L.fold_bytes + L.v_bytes;
  unsigned char* tail = ws + (L.thin || L.direct ? L.u_bytes : L.u_bytes + L.fold_bytes + L.v_bytes + L.m_bytes);
  bool folded = false;
  void* Xcl = tail;                       // channel-last copies of channel-first tensors, one chunk each
  void* Ycl = tail + L.xcl_bytes;
  StageTimer timer(stage_ms != nullptr, stream);
  const void* U = U_cached;
  // the three-kernel path transforms the filter in the launch of the first chunk's input transform (unless the
  // stages are being timed one by one)
  bool filter_with_input = !U && !stage_ms && !L.thin && !L.direct;
  if (!U && !filter_with_input) {
    rc = timer.run(WC_STAGE_FILTER, [&] { return wc_filter_transform(d, &L.plan, w, w_strides, Uws, stream); });
    if (rc) return rc;
  }
  if (!U) U = Uws;
  wc_conv_desc dcl = *d;                  // the stages behind a scratch copy see channel-last tensors
  dcl.x_layout = L.x_direct ? 1 : 0;
  dcl.y_layout = 0;
  const long long in_pos = (long long)d->in[0] * d->in[1] * d->in[2];
  const long long out_pos = (long long)L.out[0] * L.out[1] * L.out[2];
  const size_t x_image = (size_t)in_pos * d->C * L.es;
  const size_t y_image = (size_t)out_pos * d->K * L.es;
  const int step = L.thin || L.direct ? d->N : L.chunk;
  for (int b0 = 0; b0 < d->N; b0 += step) {
    const int n = (d->N - b0 < step) ? d->N - b0 : step;
    const void* xin = static_cast<const unsigned char*>(x) + b0 * x_image;
    void* yout = static_cast<unsigned char*>(y) + b0 * y_image;
    if (L.xcl_bytes) {
      rc = timer.run(WC_STAGE_LAYOUT_IN, [&] { return transpose_images(xin, Xcl, n, d->C, in_pos, (int)L.es, stream); });
      if (rc) return rc;
      xin = Xcl;
    }
    void* ydst = L.ycl_bytes ? Ycl : yout;
    if (L.direct) {
      rc = timer.run(WC_STAGE_PRODUCT, [&] { return direct_conv(&dcl, xin, n, U, bias, ydst, stream); });
      if (rc) return rc;
    } else if (L.thin) {
      // thin F(2x2, 3x3) layers: one kernel, no V and M
      rc = timer.run(WC_STAGE_PRODUCT, [&] { return thin_conv_forward(&dcl, &L.plan, xin, U, bias, ydst, stream); });
      if (rc) return rc;
    } else {
      const long long P = L.fold_rows_per_image * n;
      WC_CHECK_ARG(P < (1ll << 31), "wc_conv_forward: chunk has too many tiles");
      if (L.fold && filter_with_input) {     // the input transform below is not the plan's
        rc = wc_filter_transform(d, &L.plan, w, w_strides, Uws, stream);
        if (rc) return rc;
        filter_with_input = false;
      }
      rc = timer.run(WC_STAGE_INPUT, [&] {
        if (L.fold) return input_transform_columns(&dcl, xin, n, V, stream);
        return filter_with_input ? input_filter_transform(&dcl, &L.plan, xin, n, V, w, w_strides, Uws, stream)
                                 : wc_input_transform(&dcl, &L.plan, xin, n, V, stream);
      });
      if (rc) return rc;
      filter_with_input = false;
      if (L.fold && !folded) {
        rc = timer.run(WC_STAGE_FILTER, [&] { return fold_filter_w(U, Ufold, d->K, L.Cp, d->dtype, stream); });
        if (rc) return rc;
        folded = true;
      }
      rc = timer.run(WC_STAGE_PRODUCT, [&] {
        if (L.fold) return batched_gemm_shifted(V, Ufold, M, 16, (int)P, L.Cp, L.fold_shift, d->K, L.ldm, d->dtype, stream);
        return L.shared ? batched_gemm_shifted(V, U, M, L.plan.t_total, (int)P, L.vrow, L.shift, d->K, L.ldm, d->dtype, stream)
                        : wc_batched_gemm(V, U, M, L.plan.t_total, (int)P, L.Cp, d->K, L.ldm, d->dtype, stream);
      });
      if (rc) return rc;
      rc = timer.run(WC_STAGE_OUTPUT, [&] {
        if (L.fold) return output_transform_columns(&dcl, M, bias, n, ydst, stream);
        return wc_output_transform(&dcl, &L.plan, M, bias, n, ydst, stream);
      });
      if (rc) return rc;
    }
    if (L.ycl_bytes) {
      rc = timer.run(WC_STAGE_LAYOUT_OUT, [&] { return transpose_images(Ycl, yout, n, out_pos, d->K, (int)L.es, stream); });
      if (rc) return rc;
    }
  }
  return stage_ms ? timer.collect(stage_ms) : WC_OK;
}

}  // namespace

extern "C" {

int wc_conv_forward_static(const wc_conv_desc* d, const void* x, const void* w, const int64_t w_strides[5],
                           const void* U_cached, const void* bias, void* y, void* stream) {
  WC_CHECK_ARG(d != nullptr, "wc_conv_forward_static: null descriptor");
  // the largest chunk of images whose V and M fit beside U; the caller's own chunk if that is smaller
  wc_conv_desc dd = *d;
  dd.chunk_images = 1;
  Layout L;
  int rc = make_layout(&dd, &L);
  if (rc) return rc;
  const size_t cap = WC_STATIC_SCRATCH_BYTES;
  if (L.need() > cap)
    return fail(WC_ERR_WORKSPACE, "wc_conv_forward_static: one image needs %zu bytes of scratch, the static buffer "
                "holds %zu; use wc_conv_forward with a caller-provided workspace", L.need(), cap);
  if (!L.thin) {
    // v_bytes carries a fixed tail for plans that share one transformed input; the rest grows with the chunk
    Layout L2;
    dd.chunk_images = d->N >= 2 ? 2 : 1;
    rc = make_layout(&dd, &L2);
    if (rc) return rc;
    const size_t per_image = dd.chunk_images == 2 ? L2.need() - L.need() + 512 : 0;   // rounding of V and M to 256 each
    long long fit = per_image ? 1 + (long long)((cap - L.need()) / per_image) : 1;
    if (fit > d->N) fit = d->N;
    if (d->chunk_images > 0 && d->chunk_images < fit) fit = d->chunk_images;
    // the estimate ignores that V, M and the layout copies are each rounded up to 256 bytes: step down until it fits
    for (;;) {
      dd.chunk_images = (int)fit;
      rc = make_layout(&dd, &L);
      if (rc) return rc;
      if (L.need() <= cap || fit <= 1) break;
      --fit;
    }
    if (L.need() > cap) return fail(WC_ERR_WORKSPACE, "wc_conv_forward_static: chunk of %d images needs %zu bytes", dd.chunk_images, L.need());
  }
  void* ws = nullptr;
  rc = static_scratch(&ws);
  if (rc) return rc;
  return wc_conv_forward(&dd, x, w, w_strides, U_cached, bias, y, ws, cap, stream);
}

}  // extern "C"
