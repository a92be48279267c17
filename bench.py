#!/usr/bin/env python3
"""Benchmark of the Winograd convolution hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu]

Workload (the configuration the headline metric is quoted on): one 3x3 stride-1 pad-1
convolution, fp16 storage with fp32 accumulation, N=64, C=K=256, 56x56, Winograd
F(4x4,3x3); x ~ N(0,1), w Kaiming-normal (fan_in = 2304), seed 0, generated on the CPU and
copied, channel-last (NHWC) in HBM before the timed region starts.

A step is one pass of the whole path over the batch: filter transform, input transform,
batched GEMM, output transform - the same C-ABI calls, in the same order and on the same
stream, that wc_conv_forward makes for a one-chunk batch - with a HIP event between the
stages so that each kernel's duration is measured inside the timed region.  Exactly K steps
are timed between two device synchronisations.

Prints ONE JSON line.  `value` is effective TFLOP/s = direct-convolution FLOPs
(2*N*K*C*oH*oW*9) / time per step.  `roofline` describes the batched GEMM (the dominant
kernel): achieved = 2*T*P*C*K flops per launch / its mean duration, against the published
dense fp16 MFMA peak.  `cpu_baseline` times the CPU restatement of the reference algorithm
(oracle.winograd.dwm_conv, fp32) on a bounded sample of the same layer on the host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N, C, K, H, W, R, PAD, M_TILE = 64, 256, 256, 56, 56, 3, 1, 4
MFMA_FP16_PEAK_TFLOPS = 2500.0      # MI355X published dense fp16 matrix peak
# HBM bytes per GEMM launch from rocprofv3 --pmc FETCH_SIZE (116734 KiB, x2.00 by the copy
# probe) + WRITE_SIZE (225792 KiB, x1.00); runs and scale factors are recorded in
# profiles/conv3x3_f16_n64_c256_56x56_all_kernels.md.
GEMM_HBM_TRAFFIC_BYTES = int((116734 * 2.0 + 225792 * 1.0) * 1024)


def synthetic(n):
    import torch
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n, C, H, W, generator=g)
    w = torch.randn(K, C, R, R, generator=g) * (2.0 / (C * R * R)) ** 0.5
    return x, w


def cpu_baseline(sample_images=32, repeats=3):
    """CPU restatement of the reference algorithm on `sample_images` images of the workload."""
    import torch
    from oracle import winograd as ow
    x, w = synthetic(sample_images)
    ow.dwm_conv(x[:1], w, None, 1, PAD, M_TILE, "fp32")          # warm-up
    best = float("inf")
    for _ in range(repeats):
        t0 = time.perf_counter()
        ow.dwm_conv(x, w, None, 1, PAD, M_TILE, "fp32")
        best = min(best, time.perf_counter() - t0)
    flops = 2.0 * sample_images * K * C * H * W * R * R
    t0 = time.perf_counter()
    torch.nn.functional.conv2d(x, w, padding=PAD)
    t_direct = time.perf_counter() - t0
    return {
        "value": flops / best / 1e12, "unit": "effective TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port",
        "sample": "%d of the %d images of the same layer, fp32, oracle.winograd.dwm_conv F(4x4,3x3), "
                  "best of %d; torch CPU conv2d fp32 on the same sample: %.4f effective TFLOP/s"
                  % (sample_images, N, repeats, flops / t_direct / 1e12),
    }


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--copy-probe", action="store_true",
                    help="also run three 128 MiB device-to-device copies before the timed region "
                         "(the known-size kernel that scales rocprofv3's FETCH_SIZE / WRITE_SIZE)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py: this engine is a single-GPU operator with no collectives; it is "
                 "measured on one GPU only (use --gpus 1). Batch sharding across GPUs needs no "
                 "exchange step and is not part of this benchmark.")
    import torch
    from pytorch_winoconv_amd import _lib, engine
    if not torch.cuda.is_available():
        sys.exit("bench.py: no GPU visible")
    lib = _lib.load()
    dev = torch.device("cuda:0")
    dtype = torch.float16

    x, w = synthetic(N)
    x = x.to(dtype).to(dev).contiguous(memory_format=torch.channels_last)
    w = w.to(dtype).to(dev)
    desc = engine.make_desc(x.shape, w.shape, dtype, 1, PAD, M_TILE)
    plan = engine.plan_conv(desc)
    out, grid = engine.out_dims(desc)
    x_cl = engine.channel_last(x)
    T, P = plan.t_total, N * grid[1] * grid[2]
    Cp, ldm = lib.wc_padded_channels(C), lib.wc_padded_channels8(K)
    U = torch.empty(T, K, Cp, dtype=dtype, device=dev)
    V = torch.empty(T, P, Cp, dtype=dtype, device=dev)
    Mb = torch.empty(T, P, ldm, dtype=dtype, device=dev)
    y = torch.empty(N, out[1], out[2], K, dtype=dtype, device=dev)
    st = engine._stream(x)
    d_, p_ = ctypes.byref(desc), ctypes.byref(plan)
    ws = engine._w_strides(w)
    px, pw, pU, pV, pM, py = (engine._ptr(t) for t in (x_cl, w, U, V, Mb, y))

    def step(ev=None):
        if ev: ev[0].record()
        _lib.check(lib.wc_filter_transform(d_, p_, pw, ws, pU, st))
        if ev: ev[1].record()
        _lib.check(lib.wc_input_transform(d_, p_, px, N, pV, st))
        if ev: ev[2].record()
        _lib.check(lib.wc_batched_gemm(pV, pU, pM, T, P, Cp, K, ldm, desc.dtype, st))
        if ev: ev[3].record()
        _lib.check(lib.wc_output_transform(d_, p_, pM, None, N, py, st))
        if ev: ev[4].record()

    if args.copy_probe:
        src = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    events = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(args.steps)]
    t0 = time.perf_counter()
    for ev in events:
        step(ev)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    names = ("filter_transform", "input_transform", "batched_gemm", "output_transform")
    stage_us = {n: sum(ev[i].elapsed_time(ev[i + 1]) for ev in events) / args.steps * 1e3
                for i, n in enumerate(names)}

    # the product's one-call entry point on the same inputs, for comparison
    def one_call():
        return engine.conv_forward(x, w, None, 1, PAD, M_TILE)
    y1 = one_call()
    torch.cuda.synchronize()
    same = bool(torch.equal(y1.permute(0, 2, 3, 1), y))
    t0 = time.perf_counter()
    for _ in range(args.steps):
        one_call()
    torch.cuda.synchronize()
    ms_one_call = (time.perf_counter() - t0) / args.steps * 1e3

    direct_flops = 2.0 * N * K * C * out[1] * out[2] * R * R
    gemm_flops = 2.0 * T * P * C * K
    gemm_tflops = gemm_flops / (stage_us["batched_gemm"] * 1e-6) / 1e12
    es = 2
    hbm = {
        "input_transform": (x.numel() + V.numel()) * es,
        "output_transform": (Mb.numel() + y.numel()) * es,
    }
    result = {
        "metric": "effective TFLOP/s (direct-conv-equivalent), 3x3 conv fp16 N=64 C=K=256 56x56, 1 MI355X",
        "value": direct_flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "conv2d 3x3 s1 p1, N=64 C=K=256 56x56, fp16 in / fp32 accumulate, "
                               "Winograd F(4x4,3x3), T=36 P=12544, NHWC resident in HBM, filter "
                               "transform included in every step"},
        "roofline": {"bound": "mfma", "achieved": gemm_tflops, "peak": MFMA_FP16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": gemm_tflops / MFMA_FP16_PEAK_TFLOPS,
                     "traffic": GEMM_HBM_TRAFFIC_BYTES, "kernel": "wc::gemm_kernel (batched_gemm)",
                     "flops_per_launch": gemm_flops, "avg_us": stage_us["batched_gemm"]},
        "stage_us": stage_us,
        "stage_hbm_tb_s": {k: v / (stage_us[k] * 1e-6) / 1e12 for k, v in hbm.items()},
        "ms_per_layer_one_call": ms_one_call,
        "one_call_matches_stages": same,
    }
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
