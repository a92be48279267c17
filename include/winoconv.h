/*
 * winoconv.h - C ABI of libwinoconv_hip.so, a Winograd / DWM convolution engine
 * for AMD gfx950 (MI355X).
 *
 * Plain pointers, ints and sizes only: no torch, no HIP types (a stream is passed
 * as `void*` holding a hipStream_t; NULL is the default stream).  Every function
 * returns 0 on success or a negative wc_status; wc_last_error() then gives a
 * thread-local message.  No function allocates device memory or synchronises the
 * device: work is enqueued on the caller's stream and scratch memory comes from the
 * caller (`workspace`).  Nothing a call computes depends on earlier calls; the library
 * only remembers which of its kernels it has already granted more than 64 KB of LDS on
 * which device (the test hook wc_test_gemm_override is inert unless the process opts in).
 *
 * Data layouts (row-major, innermost last).  "Channel-last" means NHWC / NDHWC.
 *   x   (N, D, H, W, C)        D = 1 for 2-D problems (or channel-first, see wc_conv_desc.x_layout)
 *   w   any strided (K, C, kD, kH, kW) view: element strides are passed in
 *   y   (N, oD, oH, oW, K)
 *   U   (T, K,  Cp)            transformed filter, Cp = wc_padded_channels(C)
 *   V   (T, P,  Cp)            transformed input,  P = N*nD*nH*nW tiles
 *   M   (T, P,  ldm)           per-element products, ldm = wc_padded_channels8(K)
 * T is the number of transform-domain elements summed over all pieces of the
 * DWM plan; element order inside a piece is (d*alpha_h + h)*alpha_w + w.
 *
 * Each declaration cites the interface of the reference implementation
 * (huangdi95/pytorch_winoconv) that it stands in for.
 */
#ifndef WINOCONV_H_
#define WINOCONV_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Storage type of every tensor of a call.  Sums and products inside the kernels are fp32 (MFMA
 * accumulators included), and values are rounded to the storage type once, when V, M and y are
 * written - with one exception: the one-kernel path of thin fp16 layers (wc_conv_desc.unfused = 0)
 * transforms its input windows with fp16 adds, the arithmetic type of the reference's own kernels
 * (src/calculation_kernels.cu:786-806); its bf16 form and everything else add in fp32. */
typedef enum { WC_F32 = 0, WC_F16 = 1, WC_BF16 = 2 } wc_dtype;

typedef enum {
  WC_OK = 0,
  WC_ERR_BAD_ARG = -1,      /* null pointer, non-positive size, inconsistent shapes   */
  WC_ERR_UNSUPPORTED = -2,  /* kernel size / stride / tile size outside the engine     */
  WC_ERR_WORKSPACE = -3,    /* workspace missing or too small                          */
  WC_ERR_HIP = -4           /* a HIP runtime call failed (message carries its text)    */
} wc_status;

#define WC_MAX_PIECES 64

/* One stride-1 sub-convolution of the DWM plan. */
typedef struct {
  int tap0[3];   /* first kernel tap per axis (D, H, W)                      */
  int r[3];      /* taps per axis, 1..3 (4..7 for a whole-kernel tile); taps are tap0 + i*tap_step */
  int t_offset;  /* first transform-domain element of this piece             */
} wc_piece;

typedef struct {
  int n_pieces;
  int t_total;                 /* sum over pieces of prod(m + r - 1)                  */
  int tap_step;                /* = convolution stride                                */
  int m[3];                    /* output tile extent per axis (1 on a size-1 depth)   */
  wc_piece piece[WC_MAX_PIECES];
} wc_plan;

typedef struct {
  int ndim;        /* 2 or 3                                                   */
  int N, C, K;
  int in[3];       /* D, H, W of the input (D = 1 when ndim == 2)               */
  int kernel[3];   /* kD, kH, kW (kD = 1 when ndim == 2)                        */
  int pad[3];      /* symmetric zero padding per axis                           */
  int stride;      /* 1 or 2, same on every axis                                */
  int m;           /* Winograd output tile: 2, or 4 (2-D: 4 x 4; 3-D: 2 x 4 x 4, 3x3x3 stride 1 only), or 3 (with stacked = 2) */
  int dtype;       /* wc_dtype                                                  */
  int chunk_images;/* images per pass of wc_conv_forward; 0 = choose automatically */
  int whole_kernel;/* 0: kernels > 3 are decomposed into pieces of <= 3 taps (DWM, dwm.py:107-146);
                    * 1: one F(2,k) x F(2,k) tile for the whole k x k kernel, k = 4..7, the arithmetic
                    *    of the reference's PyTorch path (matrix_conv.py:112-135, tables :31-35):
                    *    2-D, stride 1, m = 2 only; loses accuracy quickly with k, fp16 above all */
  int stacked;     /* 0: every piece of a DWM plan has its own transform-domain elements and products, and
                    *    the output transform adds the pieces (the reference's structure: outputAggregate,
                    *    src/split_kernel.cu:184-203);
                    * 1: all pieces share one tile F(m, r_max) per axis (r_max = most taps of any piece on
                    *    that axis; shorter pieces count their missing taps as zero) and lie side by side
                    *    along the reduction axis of U and V (row length n_pieces * Cp), so the batched
                    *    GEMM adds them: M shrinks to one piece's size.  Same sum, other rounding.
                    *    Output tile 2, or 4 in 2-D.  The plan then reports t_offset = 0 for every piece and
                    *    t_total = prod(m + r_max - 1).
                    * 2: (stride 1, m = 2; wc_conv_forward and the stages, fp16 / bf16 products) the kernel is cut
                    *    into pieces of two taps per axis (the last one of an odd extent has one), all on the tile
                    *    F(2,2).  Pieces that start at even taps see the same transformed input, moved by whole
                    *    tiles: V holds ONE piece, over a tile grid extended by the largest moves (wc_conv_out_dims
                    *    reports that grid) plus the rows that the moved reads of its last tiles reach, U holds the
                    *    pieces side by side as for 1, and the batched GEMM reads each piece's rows of V at that
                    *    piece's tile offset.  Same sum as 0 and 1; V is written and read once instead of once
                    *    per piece.  With m = 3 (2-D, at least 3 taps per axis and more than 3 on one) the pieces
                    *    have three taps, the reference's split without its 4 -> 2 + 2 exception, on the tile F(3,3). */
  int unfused;     /* wc_conv_forward only.  0: 3x3 stride-1 2-D layers with m = 2 run as ONE kernel (input transform,
                    *    products and output transform of F(2x2, 3x3) without V and M in memory, the product
                    *    kept in fp32; x below 1 GiB) if they have
                    *    - at most 4 input channels (any dtype, at most 512 output channels): first layers, or
                    *    - fp16 / bf16 data and input channels that pad to 32, 64 or 128 (an even number up to
                    *      32, a multiple of 4 in 33..64 or 97..128), at most 512 output channels (256 with
                    *      128 input channels), or
                    *    - fp32 data, an even number of at most 64 input channels, at most 512 output channels (256
                    *      above 32 input channels): the products on fp32 MFMA;
                    * 1: always filter transform -> input transform -> batched GEMM -> output transform. */
  int x_layout;    /* 0: x is channel-last (N, D, H, W, C); 1: x is channel-first contiguous (N, C, D, H, W), the layout
                    *    torch tensors have by default.  Single-piece 2-D plans at stride 1 (kernels of at most 3 taps
                    *    per axis) then read x as it is inside the input transform; every other plan copies it to
                    *    channel-last scratch first (wc_conv_forward: the workspace grows by the size of x).  The
                    *    reference always runs that copy, as a torch pass of its own (dwm.py:129-133). */
  int y_layout;    /* the same for y: 1 = channel-first contiguous (N, K, oD, oH, oW); wc_conv_forward then writes the
                    *    output transform's channel-last result to scratch and copies it (dwm.py:143-144). */
  int direct;      /* 1: the direct form, the degenerate end of the split: pieces of one tap on the trivial tile F(1,1),
                    *    for which there is nothing to transform, so the batched product reads the pixels of x as its V
                    *    operand, walks the taps along its reduction axis and writes y; no V or M in memory, U is the
                    *    filter as (K, kH, kW, C).  2-D, C a multiple of 32 (fp32: 16), K a multiple of 8; m, stacked
                    *    and whole_kernel are ignored.  wc_conv_auto chooses it for kernels of one tap (every type: the
                    *    tile F(m,1) saves nothing and its transforms are copies), for 16-bit layers at stride 2 (short
                    *    reductions always, longer ones where the output fills the chip) and for fp32 3x3 layers at
                    *    stride 2 over at most 128 channels: strides the reference does not implement
                    *    (src/winograd_conv.cpp:122-126) and where Winograd tiles on the parity phases save few or no
                    *    multiplications; and for first layers with at most 4 channels in a 16-bit type - 2-D at stride 2
                    *    (3 / 5 / 7 kernel rows of at most 8 taps, U (K, kH, 8, 4)) and 3-D 3x3x3 at stride 1 (rows of at
                    *    most 4 taps, U (K, 9, 4, 4)) - which have kernels of their own.  wc_conv_forward, wc_filter_transform,
                    *    wc_conv_workspace_bytes and wc_conv_u_elems honour it; the other stage functions do not apply. */
} wc_conv_desc;

/* ---- library ------------------------------------------------------------------------- */
const char* wc_version(void);
/* Replaces the reference's cout + exit(-1) error convention
 * (src/winograd_conv.cpp:80-84,116-126; src/base_conv_launchers.h:384-387). */
const char* wc_last_error(void);

/* Test hook, no counterpart in the reference: forces tile shape `config` (an index into the
 * library's list of shapes; -1 = choose by problem size) on wc_batched_gemm, and for plans that
 * share one transformed input the kernel with one operand tile per piece (rows_mode 0), the
 * choice by size (1, the default), one tile per run of pieces wherever the plan has runs (2), or
 * the persistent kernel with one tile per run fed by LDS-DMA wherever it runs (runs of 2 to 5
 * pieces, else as 1): 3 with every tile written out when it is done, 4 with the write-out riding on
 * the workgroup's next tile wherever the tiles have the steps for that (what the choice by size takes).
 * config 10: wc_batched_gemm on persistent 256 x 256 tiles wherever that kernel runs (16-bit types, K a
 * multiple of 256, reductions of 96 and more), every tile written out when it is done; config 13: the
 * same with most of a tile's write-out riding on the workgroup's next tile (reductions of 160 and more;
 * what the choice by size takes).
 * config 11 / 12: 3-D F(2,3)^3 plans in 16-bit types never / always take the width axis inside the product
 * (transforms along depth and height only, the three width taps along the reduction; by size otherwise).
 * config 8 / 9: the one-kernel F(2x2,3x3) path with workgroups of 64 / 32 output channels whatever
 * the number of tiles (9 only where the channel count allows it).
 * Works only in a process started with WINOCONV_TEST_HOOKS=1 in its environment (WC_ERR_UNSUPPORTED
 * otherwise, and nothing changes); what it sets holds for the calling host thread only, so a caller
 * cannot change what the launches of another thread do.  Production code never calls it. */
int wc_test_gemm_override(int config, int rows_mode);

/* ---- planning (host only) --------------------------------------------------------------- */
/* Stride-1 split plan in the reference's own terms; replaces splitControl()
 * (src/base_conv_launchers.h:58-388) and the kernel_stride prefix sums
 * (src/base_conv_launchers.cu:307-313).  Arrays must hold WC_MAX_PIECES ints.
 * Boxes are half-open [start, end).  Works for every extent 1..10, not just the
 * reference's 36 keys. */
int wc_plan_dwm(int kD, int kH, int kW, int* num_split,
                int* D_start, int* D_end, int* H_start, int* H_end,
                int* W_start, int* W_end, int* kernel_stride, int* t_total);
/* General plan of a convolution (stride 1 or 2; tile 2 with F(2,r) pieces, or tile 4 with
 * F(4,r) pieces in 2-D). */
int wc_plan_conv(const wc_conv_desc* desc, wc_plan* plan);
/* Fills in what a caller leaves open.  desc->stacked == -1 on entry: replaced by the form of the plan
 * (0, 1 or 2, see wc_conv_desc.stacked; or desc->direct = 1 with stacked = 0) that measured fastest on MI355X
 * for this dtype, kernel, stride and channel count.  desc->m == 4 with stacked == 2 (a tile that plan does not have): replaced by 3 where the
 * three-tap pieces on F(3,3) apply (fp16, 2-D, stride 1, at least 3 taps per axis and 5 on one), else by 2;
 * desc->direct == -1 on entry: the direct form is never chosen (and the field comes back 0).
 * The caller reads the tile that will really be used back from desc->m.  No counterpart in the reference,
 * which has one form only (src/base_conv_launchers.cu:282-399).  Every other function wants stacked >= 0. */
int wc_conv_auto(wc_conv_desc* desc);
/* Output extent and tile grid: replaces the shape arithmetic of DWM<T>
 * (src/winograd_conv.cpp:71-90) and of dwm2d_/dwm3d_ (dwm.py:56-61,118-121). */
int wc_conv_out_dims(const wc_conv_desc* desc, int out[3], int grid[3]);
int wc_padded_channels(int C);   /* channel stride of U and V (multiple of 32) */
int wc_padded_channels8(int K);  /* row stride of M (multiple of 8)             */

/* ---- tile split / concat (bit-exact copies) ----------------------------------------------- */
/* Replaces WinoSplit<T> (pybind/extern.hpp:3-4, src/split_and_concat.cpp:14-40) and the
 * kernels winoSplitKernel2d / winoSplitKernel (src/split_and_concat_kernels.cu:76-101, :8-37).
 * x channel-last (B, [D,] H, W, C) -> tiles (B*[nD*]nH*nW, C, [block_D,] block_H, block_W),
 * tile step = m on every axis, zero outside the input.  elem_size is 2 or 4 bytes. */
int wc_wino_split2d(const void* x, void* tiles, int B, int H, int W, int C,
                    int block_H, int block_W, int m, int nH, int nW,
                    int elem_size, void* stream);
int wc_wino_split3d(const void* x, void* tiles, int B, int D, int H, int W, int C,
                    int block_D, int block_H, int block_W, int m, int nD, int nH, int nW,
                    int elem_size, void* stream);
/* Replaces WinoConcat<T> (pybind/extern.hpp:5-6, src/split_and_concat.cpp:44-76) and the
 * kernels winoConcatKernel2d / winoConcatKernel (src/split_and_concat_kernels.cu:107-129, :43-70).
 * tiles (B*[nD*]nH*nW, K, [m,] m, m) -> y channel-last (B, [oD,] oH, oW, K); partial edge
 * tiles are cropped.  n_X = ceil(o_X / m). */
int wc_wino_concat2d(const void* tiles, void* y, int B, int oH, int oW, int K, int m,
                     int elem_size, void* stream);
int wc_wino_concat3d(const void* tiles, void* y, int B, int oD, int oH, int oW, int K, int m,
                     int elem_size, void* stream);

/* Bit-exact copy between channel-first (n, C, S) and channel-last (n, S, C) memory, S = [D] H W positions;
 * to_channel_last = 1 for the first direction.  Replaces the permute passes of the reference's Python callers
 * (dwm.py:129-133,143-144; Split_and_Concat.py:25,47,64,81).  elem_size is 2 or 4 bytes. */
int wc_layout_copy(const void* src, void* dst, int n_images, int channels, long long spatial,
                   int to_channel_last, int elem_size, void* stream);

/* ---- pipeline stages ---------------------------------------------------------------------- */
/* U = (G x G x G) g for every piece.  Replaces wNorm2WinoTransform + wNorm2WinoCalculation
 * (src/split_kernel.cu:14-53, src/calculation_kernels.cu:2-761) and matrix_conv.py:150-153.
 * w_strides: element strides of w for (K, C, kD, kH, kW). */
int wc_filter_transform(const wc_conv_desc* desc, const wc_plan* plan,
                        const void* w, const int64_t w_strides[5], void* U, void* stream);
/* V = (BT x BT x BT) d for `n_images` images starting at x (channel-first x, desc->x_layout = 1, only for the
 * plans named there: WC_ERR_UNSUPPORTED otherwise).  Replaces
 * inputNorm2WinoTransform + inputNorm2WinoCalculation (src/split_kernel.cu:60-120,
 * src/calculation_kernels.cu:763-1522) and matrix_conv.py:158-203. */
int wc_input_transform(const wc_conv_desc* desc, const wc_plan* plan,
                       const void* x, int n_images, void* V, void* stream);
/* M[t] (P x K) = V[t] (P x Cp) . U[t]^T for t in [0, T).  Replaces forwardAssign +
 * cublas{S,H}gemmBatched (src/utils.cu:5-12, src/base_conv_launchers.cu:353-367,
 * src/base_conv_launchers_half.cu:231-236).  fp16 accumulates in fp32. */
int wc_batched_gemm(const void* V, const void* U, void* M, int T, int P, int Cp, int K, int ldm,
                    int dtype, void* stream);
/* y = sum over pieces of (AT x AT x AT) m, + bias, cropped.  Replaces outputWino2NormTransform +
 * outputWino2NormCalculation + outputAggregate (src/split_kernel.cu:126-203,
 * src/calculation_kernels.cu:1524-1770) and matrix_conv.py:207-253.  bias may be NULL
 * (K values of the tensor dtype otherwise). */
int wc_output_transform(const wc_conv_desc* desc, const wc_plan* plan,
                        const void* M, const void* bias, int n_images, void* y, void* stream);

/* ---- whole convolution -------------------------------------------------------------------- */
/* Replaces DWM<T> (pybind/extern.hpp:7-9, src/winograd_conv.cpp:17-127) and
 * convLauncherStrideOneLarge<T> (src/base_conv_launchers.cu:282-399).
 * The workspace holds U, V and M (the reference's tmp_weight_buffer, tmp_input_buffer,
 * tmp_product_buffer: dwm.py:122-125); images are processed in chunks that bound the size
 * of V and M.  `U_cached` (may be NULL) is a filter already transformed
 * by wc_filter_transform; `w` may then be NULL.  Thin 3x3 layers take one fused kernel
 * instead (see wc_conv_desc.unfused); the workspace then only holds U. */
int wc_conv_workspace_bytes(const wc_conv_desc* desc, size_t* bytes);
int wc_conv_u_elems(const wc_conv_desc* desc, size_t* elems);
int wc_conv_forward(const wc_conv_desc* desc, const void* x,
                    const void* w, const int64_t w_strides[5], const void* U_cached,
                    const void* bias, void* y, void* workspace, size_t workspace_bytes,
                    void* stream);

/* wc_conv_forward with the time every stage took on the device: a pair of events around each stage on `stream`,
 * read after the stream has been waited for, so the call returns when the convolution is done (opt-in: it
 * serialises the host with the device).  Replaces the perf_counter / synchronize pairs the reference puts
 * around its phases (dwm.py:44-106).  stage_ms[s] is the sum over the image chunks; stages that did not run
 * read 0.  The one-kernel forms (thin layers, the direct form) count as WC_STAGE_PRODUCT.  Same results
 * as wc_conv_forward, bit for bit. */
enum {
  WC_STAGE_FILTER = 0,      /* filter transform (0 with U_cached) */
  WC_STAGE_LAYOUT_IN = 1,   /* channel-first x copied to channel-last scratch */
  WC_STAGE_INPUT = 2,       /* input transform */
  WC_STAGE_PRODUCT = 3,     /* batched GEMM, or the one fused kernel */
  WC_STAGE_OUTPUT = 4,      /* output transform */
  WC_STAGE_LAYOUT_OUT = 5,  /* channel-last scratch copied to channel-first y */
  WC_N_STAGES = 6
};
int wc_conv_forward_timed(const wc_conv_desc* desc, const void* x,
                          const void* w, const int64_t w_strides[5], const void* U_cached,
                          const void* bias, void* y, void* workspace, size_t workspace_bytes,
                          void* stream, float stage_ms[WC_N_STAGES]);

/* wc_conv_forward without a workspace argument.  No counterpart in the reference; it is for callers
 * that cannot allocate device memory: code under HIP graph capture, tight serving loops, harnesses
 * that forbid hipMalloc.  U, V and M live in a buffer of WC_STATIC_SCRATCH_BYTES inside the
 * library's device image (each GPU the library runs on holds its own copy until the process ends),
 * and the batch is processed in as many chunks of images as it takes for them to fit.  Returns
 * WC_ERR_WORKSPACE, before anything is launched, if U plus the V and M of a single image exceed the
 * buffer.  Allocates nothing and frees nothing.  The first call on a device looks up the buffer's
 * address (make it outside graph capture).  All calls on one GPU share the buffer: calls that
 * overlap in time on one GPU (two streams, two host threads) race; nothing in it needs to start at
 * zero, a call only reads what it has written.  Same results as wc_conv_forward, bit for bit. */
#define WC_STATIC_SCRATCH_BYTES (64u * 1024u * 1024u)
int wc_conv_forward_static(const wc_conv_desc* desc, const void* x,
                           const void* w, const int64_t w_strides[5], const void* U_cached,
                           const void* bias, void* y, void* stream);

/* ---- weight gradient -------------------------------------------------------------------------- */
/* No counterpart in the reference: it never implemented a backward pass (only a pointer-assign
 * helper exists for one, src/back/utils.cu:15-24; include/split_functions_grad.h:3-6 is empty).
 * dw[k][c][taps] = gradient of sum(y * dy) with respect to the filter, for the same descriptor as
 * the forward call: x (N, D, H, W, C) and dy (N, oD, oH, oW, K) channel-last contiguous, dw written
 * through element strides for the axes (K, C, kD, kH, kW).  Computed in the transform domain
 * (dU = sum over tiles of dM x V, dw = G^T dU G) with every sum in fp32.  The input gradient needs
 * no entry point of its own: it is wc_conv_forward of dy with the flipped, transposed filter. */
int wc_conv_backward_weight_workspace_bytes(const wc_conv_desc* desc, size_t* bytes);
/* Input gradient of a 2-D layer at stride 2 (no counterpart in the reference either): dx (N, H, W, C) from dy
 * (N, oH, oW, K) channel-last contiguous and the filter through its element strides, for the descriptor of the
 * forward call.  The pixels of dx fall into four classes by their parity; each class is a stride-1 direct convolution
 * of dy with the taps of its parity (flipped, channel axes exchanged), one launch of the direct form each, writing every
 * second pixel: the multiplications of the forward pass, where convolving a zero-filled dy multiplies four times as
 * much.  K a multiple of 32 (fp32: 16), C a multiple of 8, padding below the kernel extent; WC_ERR_UNSUPPORTED
 * otherwise (a caller then runs wc_conv_forward on the zero-filled dy).  Sums in fp32, one rounding. */
int wc_conv_backward_input_workspace_bytes(const wc_conv_desc* desc, size_t* bytes);
int wc_conv_backward_input(const wc_conv_desc* desc, const void* dy, const void* w, const int64_t w_strides[5],
                           void* dx, void* workspace, size_t workspace_bytes, void* stream);
int wc_conv_backward_weight(const wc_conv_desc* desc, const void* x, const void* dy, void* dw,
                            const int64_t dw_strides[5], void* workspace, size_t workspace_bytes,
                            void* stream);
#ifdef __cplusplus
}
#endif
#endif /* WINOCONV_H_ */
