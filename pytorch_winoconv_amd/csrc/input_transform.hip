// Host entry of the input transform: picks the kernel of each piece and launches it.
#include "filter_transform_impl.h"
#include "input_transform_impl.h"
#include <algorithm>

using namespace wc;

namespace {

// filt: the filter transform of the same call, to be run in the same launch where a kernel for that exists;
// *filt_done tells whether it was
int input_transform_impl(const wc_conv_desc* d, const wc_plan* plan, const void* x, int n_images, void* V, void* stream,
                         const FilterFastArgs* filt, bool* filt_done) {
  WC_CHECK_ARG(d && plan && x && V, "wc_input_transform: null pointer");
  WC_CHECK_ARG(n_images > 0, "wc_input_transform: n_images %d", n_images);
  int out[3], grid[3];
  int rc = wc_conv_out_dims(d, out, grid);
  if (rc) return rc;
  WC_CHECK_ARG(plan->n_pieces > 0 && plan->n_pieces <= WC_MAX_PIECES, "wc_input_transform: bad plan");
  if (d->x_layout == 1) {
    if (!input_transform_nchw_fits(d, plan))
      return fail(WC_ERR_UNSUPPORTED, "wc_input_transform: channel-first x is read directly by single-piece 2-D plans at "
                  "stride 1 only; copy it with wc_layout_copy, or let wc_conv_forward do so");
    return input_transform_nchw(d, plan, x, n_images, V, stream);
  }
  const int Cp = wc_padded_channels(d->C);
  const long long P = (long long)n_images * grid[0] * grid[1] * grid[2];
  const bool flat = plan->m[0] == 1;
  const bool shared = shared_input(d, plan);         // one piece's transform serves all pieces (see wc_common.h)
  const bool stacked = d->stacked && plan->n_pieces > 1 && !shared;
  const int row = v_row(d, plan);                    // row length of V
  int rp[3];
  stacked_taps(plan, rp);
  // Channels per thread.  Measured on MI355X at N=64, C=256, 56x56 fp16: F(4,3) tiles (36 live
  // elements per channel) run best with 2 channels per thread (more wavefronts in flight),
  // F(2,r) tiles with 16-byte accesses; 3-D tiles and whole-kernel tiles (up to 64 elements) use 2.
  int want;
  if (!flat) want = 2;
  else if (plan->m[1] >= 3 || plan->piece[0].r[1] > 3 || plan->piece[0].r[2] > 3) want = 2;
  else want = d->dtype == WC_F32 ? 4 : 8;
  int vec = 1;
  for (int v = want; v > 1; v /= 2)
    if (d->C % v == 0) { vec = v; break; }
  InArgs a;
  a.x = x; a.V = V;
  a.D = d->in[0]; a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.Cp = row;
  a.nD = grid[0]; a.nH = grid[1]; a.nW = grid[2];
  a.step = plan->tap_step;
  a.t_stride = (P + (shared ? shared_shift(d, grid).tail : 0)) * row;
  a.n_cvec = Cp / vec;
  a.total = P * a.n_cvec;
  const long long blocks = ceil_div_ll(a.total, 256);
  a.per_xcd = (int)ceil_div_ll(blocks, kXcds);
  a.x_bytes = 0;
  a.nq1 = a.nq2 = 1; a.q_cols = 0;
  WC_CHECK_ARG((long long)a.per_xcd * kXcds < (1ll << 31), "wc_input_transform: problem too large");
  const dim3 launch_grid((unsigned)(a.per_xcd * kXcds));

  if (shared) {
    // the first piece with the tile all pieces share, over the extended tile grid
    const int k0 = kind_of(plan->m[0], rp[0]), k1 = kind_of(plan->m[1], rp[1]), k2 = kind_of(plan->m[2], rp[2]);
    InKernel fn = nullptr;
    switch (k0) {
      case KIND_11: fn = pick_in_2d(d->dtype, k1, k2, vec); break;
      case KIND_21: fn = pick_in_3d_21(d->dtype, k1, k2, vec); break;
      case KIND_22: fn = pick_in_3d_22(d->dtype, k1, k2, vec); break;
      default: break;
    }
    if (!fn) return fail(WC_ERR_UNSUPPORTED, "input transform for the shared tile (%d, %d, %d taps) not built", rp[0], rp[1], rp[2]);
    a.t_offset = 0;
    // stride 2: the parity phases are the second grid dimension, each writes its own columns of V
    const int n0 = shared_phases(d, 0), n1 = shared_phases(d, 1), n2 = shared_phases(d, 2);
    a.base0 = -d->pad[0]; a.base1 = -d->pad[1]; a.base2 = -d->pad[2];
    a.nq1 = n1; a.nq2 = n2; a.q_cols = Cp;
    hipLaunchKernelGGL(fn, dim3(launch_grid.x, (unsigned)(n0 * n1 * n2)), dim3(256), 0, as_stream(stream), a);
    WC_CHECK_LAUNCH("input_transform_kernel");
    return WC_OK;
  }
  // 2-D DWM plans: all pieces in one launch
  bool small_taps = plan->n_pieces > 1 && flat && plan->t_total <= 0xffff;
  for (int s = 0; s < plan->n_pieces && small_taps; ++s) {
    const wc_piece& pc = plan->piece[s];
    small_taps = pc.r[1] >= 1 && pc.r[1] <= 3 && pc.r[2] >= 1 && pc.r[2] <= 3 && pc.tap0[1] < 16 && pc.tap0[2] < 16;
  }
  if (small_taps && plan->m[1] == plan->m[2]) {
    // Stacked plans of small problems give every piece its own threads (one thread per tile and
    // channel group, looping over the pieces, then leaves most of the chip idle: 2.2x faster at
    // N=8, C=24, 56x56, 7x7); large ones keep the loop, which reads each window from cache once per
    // piece and measured 7-30 % faster there.
    const bool per_piece_threads = stacked && a.total < 512 * 1024;
    InPiecesKernel fn = per_piece_threads ? pick_in_2d_stacked(d->dtype, plan->m[1], vec)
                                          : pick_in_2d_pieces(d->dtype, plan->m[1], vec);
    if (fn) {
      InPiecesArgs g;
      a.base0 = a.base1 = a.base2 = 0; a.t_offset = 0;
      dim3 launch = launch_grid;
      if (per_piece_threads) {
        a.total = P * a.n_cvec * plan->n_pieces;
        a.per_xcd = (int)ceil_div_ll(ceil_div_ll(a.total, 256), kXcds);
        WC_CHECK_ARG((long long)a.per_xcd * kXcds < (1ll << 31), "wc_input_transform: problem too large");
        launch = dim3((unsigned)(a.per_xcd * kXcds));
      }
      g.o = a;
      g.n_pieces = plan->n_pieces;
      g.pad1 = d->pad[1]; g.pad2 = d->pad[2];
      g.col_step = stacked ? Cp : 0;
      for (int s = 0; s < plan->n_pieces; ++s) {
        const wc_piece& pc = plan->piece[s];
        const int r1 = stacked ? rp[1] : pc.r[1], r2 = stacked ? rp[2] : pc.r[2];
        g.info[s] = pc.t_offset | (pc.tap0[1] << 16) | (pc.tap0[2] << 20) | (r1 << 24) | (r2 << 28);
      }
      hipLaunchKernelGGL(fn, launch, dim3(256), 0, as_stream(stream), g);
      WC_CHECK_LAUNCH("input_transform_pieces_kernel");
      return WC_OK;
    }
  }
  if (stacked && (flat || plan->m[1] != 2))
    return fail(WC_ERR_UNSUPPORTED, "stacked input transform needs output tile 2 or 4 in 2-D, 2 in 3-D");
  // one launch per piece (3-D plans); the pieces of a stacked plan all use the shared tile and
  // write their own columns of V
  for (int s = 0; s < plan->n_pieces; ++s) {
    const wc_piece& pc = plan->piece[s];
    int k[3];
    for (int q = 0; q < 3; ++q) {
      k[q] = kind_of(plan->m[q], stacked ? rp[q] : pc.r[q]);
      if (k[q] < 0) return fail(WC_ERR_UNSUPPORTED, "F(%d,%d) not implemented", plan->m[q], pc.r[q]);
    }
    InKernel fn = nullptr;
    const bool cube3 = !flat && plan->n_pieces == 1 && plan->tap_step == 1 && k[0] == KIND_23 &&
                       k[1] == KIND_43 && k[2] == KIND_43;
    const long long es = d->dtype == WC_F32 ? 4 : 2;
    const long long image_bytes = (long long)d->in[0] * d->in[1] * d->in[2] * d->C * es;
    if (!flat && plan->m[1] == 4 && !(cube3 && image_bytes < (1ll << 31)))
      return fail(WC_ERR_UNSUPPORTED, "3-D output tile 4 is built for 3x3x3 kernels and images below 2 GiB");
    if (cube3 && image_bytes < (1ll << 31)) {
      // tile 2 x 4 x 4 of a 3x3x3 kernel: plane by plane (the same scheme measured slower than the
      // whole-window kernel for the 2 x 2 x 2 tile: 272 against 205 us at N=8, C=128, 16x56x56).
      // The kernel reads x through a buffer descriptor with 32-bit offsets, so the batch is cut
      // into launches of images that together stay below 2 GiB.
      const int v3 = (es == 2 && d->C % 2 == 0) ? 2 : 1;   // channels per thread: 4 bytes per lane
      InKernel f3 = pick_in_3d_planes(d->dtype, v3);
      a.n_cvec = Cp / v3;
      const int per_launch = (int)std::max<long long>(1, ((1ll << 31) - 1) / image_bytes);
      const long long tiles_per_image = (long long)grid[0] * grid[1] * grid[2];
      a.base0 = pc.tap0[0] - d->pad[0]; a.base1 = pc.tap0[1] - d->pad[1]; a.base2 = pc.tap0[2] - d->pad[2];
      a.t_offset = pc.t_offset;
      for (int b0 = 0; b0 < n_images; b0 += per_launch) {
        const int nb = std::min(per_launch, n_images - b0);
        InArgs c = a;
        c.x = static_cast<const char*>(x) + (long long)b0 * image_bytes;
        c.V = static_cast<char*>(V) + (long long)b0 * tiles_per_image * Cp * es;
        c.x_bytes = (int)(nb * image_bytes);
        c.total = (long long)nb * tiles_per_image * c.n_cvec;
        c.per_xcd = (int)ceil_div_ll(ceil_div_ll(c.total, 256), kXcds);
        hipLaunchKernelGGL(f3, dim3((unsigned)(c.per_xcd * kXcds)), dim3(256), 0, as_stream(stream), c);
        WC_CHECK_LAUNCH("input_transform_3d_planes_kernel");
      }
      continue;
    }
    switch (k[0]) {
      case KIND_11: fn = pick_in_2d(d->dtype, k[1], k[2], vec); break;
      case KIND_21: fn = pick_in_3d_21(d->dtype, k[1], k[2], vec); break;
      case KIND_22: fn = pick_in_3d_22(d->dtype, k[1], k[2], vec); break;
      case KIND_23: fn = pick_in_3d_23(d->dtype, k[1], k[2], vec); break;
      default: break;
    }
    if (!fn) return fail(WC_ERR_UNSUPPORTED, "input transform for kinds (%d,%d,%d) not built", k[0], k[1], k[2]);
    a.base0 = pc.tap0[0] - d->pad[0]; a.base1 = pc.tap0[1] - d->pad[1]; a.base2 = pc.tap0[2] - d->pad[2];
    a.t_offset = pc.t_offset;
    a.V = static_cast<char*>(V) + (stacked ? (long long)s * Cp * (d->dtype == WC_F32 ? 4 : 2) : 0);
    if (filt && plan->n_pieces == 1 && k[0] == KIND_11) {
      if (InFilterKernel both = pick_in_filter_2d(d->dtype, k[1], k[2], vec)) {
        const int fv = in_filter_vec(d->dtype == WC_F32 ? 4 : 2, k[1]);
        const long long fb = ceil_div_ll((long long)filt->K * (filt->Cp / fv), 256);
        if (fb + launch_grid.x < (1ll << 31)) {
          hipLaunchKernelGGL(both, dim3((unsigned)(fb + launch_grid.x)), dim3(256), 0, as_stream(stream), a, *filt, (int)fb);
          WC_CHECK_LAUNCH("input_filter_kernel");
          *filt_done = true;
          continue;
        }
      }
    }
    hipLaunchKernelGGL(fn, launch_grid, dim3(256), 0, as_stream(stream), a);
    WC_CHECK_LAUNCH("input_transform_kernel");
  }
  return WC_OK;
}

}  // namespace

extern "C" int wc_input_transform(const wc_conv_desc* d, const wc_plan* plan, const void* x,
                                  int n_images, void* V, void* stream) {
  return input_transform_impl(d, plan, x, n_images, V, stream, nullptr, nullptr);
}

namespace wc {

int columns_width(const wc_conv_desc* d) { return d->in[2] + 2 * d->pad[2]; }

int input_transform_columns(const wc_conv_desc* d, const void* x, int n_images, void* V, void* stream) {
  WC_CHECK_ARG(d && x && V && n_images > 0, "input_transform_columns: null pointer or no images");
  WC_CHECK_ARG(d->ndim == 3 && d->stride == 1 && d->x_layout == 0 && d->kernel[0] == 3 && d->kernel[1] == 3 && d->kernel[2] == 3 &&
               d->dtype != WC_F32, "input_transform_columns: 3x3x3 kernels at stride 1 on channel-last 16-bit tensors");
  int out[3], grid[3];
  wc_conv_desc t = *d;
  t.m = 2;
  int rc = wc_conv_out_dims(&t, out, grid);
  if (rc) return rc;
  const int Cp = wc_padded_channels(d->C);
  const int Wx = columns_width(d);
  const long long P = (long long)n_images * grid[0] * grid[1] * Wx;
  // 16 window elements per thread: 16-byte accesses fit (measured at N=8, 128 channels, 16x56x56 fp16: 8 channels per
  // thread 118 us, 4 125, 2 133)
  int vec = 1;
  for (int v = 8; v > 1; v /= 2)
    if (d->C % v == 0) { vec = v; break; }
  InArgs a;
  a.x = x; a.V = V;
  a.D = d->in[0]; a.H = d->in[1]; a.W = d->in[2]; a.C = d->C; a.Cp = Cp;
  a.nD = grid[0]; a.nH = grid[1]; a.nW = Wx;
  a.base0 = -d->pad[0]; a.base1 = -d->pad[1]; a.base2 = -d->pad[2];
  a.step = 1;
  a.t_stride = (P + 2) * Cp;
  a.t_offset = 0;
  a.n_cvec = Cp / vec;
  a.total = P * a.n_cvec;
  a.per_xcd = (int)ceil_div_ll(ceil_div_ll(a.total, 256), kXcds);
  a.x_bytes = 0;
  a.nq1 = a.nq2 = 1; a.q_cols = 0;
  WC_CHECK_ARG((long long)a.per_xcd * kXcds < (1ll << 31), "input_transform_columns: problem too large");
  hipLaunchKernelGGL(pick_in_columns(d->dtype, vec), dim3((unsigned)(a.per_xcd * kXcds)), dim3(256), 0, as_stream(stream), a);
  WC_CHECK_LAUNCH("input_transform_kernel (pixel columns)");
  return WC_OK;
}

int input_filter_transform(const wc_conv_desc* d, const wc_plan* plan, const void* x, int n_images, void* V,
                           const void* w, const int64_t w_strides[5], void* U, void* stream) {
  WC_CHECK_ARG(w && w_strides && U, "input_filter_transform: null pointer");
  FilterFastArgs f;
  int vec = 1;
  bool dense = false, done = false;
  const bool try_both = d->x_layout == 0 && filter_fast_setup(d, plan, w, w_strides, U, &f, &vec, &dense) && dense;
  int rc = input_transform_impl(d, plan, x, n_images, V, stream, try_both ? &f : nullptr, &done);
  if (rc || done) return rc;
  return wc_filter_transform(d, plan, w, w_strides, U, stream);
}

}  // namespace wc
