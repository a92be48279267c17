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
stages of every fourth step (--event-every) so that each kernel's duration is measured inside
the timed region.  Exactly K steps are timed between two device synchronisations.

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
HBM_PEAK_GB_S = 8000.0              # MI355X published HBM3E bandwidth
# HBM bytes per GEMM launch from rocprofv3 --pmc FETCH_SIZE (127139 KiB, x2.00 by the copy
# probe) + WRITE_SIZE (225792 KiB, x1.00); runs and scale factors are recorded in
# profiles/conv3x3_f16_n64_c256_56x56_all_kernels.md.
GEMM_HBM_TRAFFIC_BYTES = int((127139 * 2.0 + 225792 * 1.0) * 1024)


def synthetic(n):
    import torch
    g = torch.Generator().manual_seed(0)
    x = torch.randn(n, C, H, W, generator=g)
    w = torch.randn(K, C, R, R, generator=g) * (2.0 / (C * R * R)) ** 0.5
    return x, w


def cpu_model():
    """Model name of the host CPU as the kernel reports it."""
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or "unknown"


def cpu_baseline(sample_images=32, repeats=3):
    """CPU restatement of the reference algorithm on `sample_images` images of the workload, and
    torch's own CPU convolution on the same sample (each warmed, then the median of `repeats`)."""
    import statistics
    import torch
    from oracle import winograd as ow
    x, w = synthetic(sample_images)

    def timed(fn):
        fn()                                                     # warm-up
        ts = []
        for _ in range(repeats):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return statistics.median(ts), min(ts)

    flops = 2.0 * sample_images * K * C * H * W * R * R
    med, best = timed(lambda: ow.dwm_conv(x, w, None, 1, PAD, M_TILE, "fp32"))
    d_med, d_best = timed(lambda: torch.nn.functional.conv2d(x, w, padding=PAD))
    return {
        "value": flops / med / 1e12, "unit": "effective TFLOP/s", "cores": torch.get_num_threads(),
        "kind": "port", "cpu_model": cpu_model(),
        "sample": "%d of the %d images of the same layer, fp32, oracle.winograd.dwm_conv F(4x4,3x3), warmed, "
                  "median of %d" % (sample_images, N, repeats),
        "best": flops / best / 1e12,
        "torch_cpu_conv2d": {"value": flops / d_med / 1e12, "best": flops / d_best / 1e12,
                             "unit": "effective TFLOP/s", "sample": "the same %d images, fp32, warmed, median of %d"
                                                                    % (sample_images, repeats)},
    }


SUITE = [
    # name, x shape, w shape, stride, pad, m, dtype  (the five benchmark configurations c1..c5 at full size).
    # c3, 64 and 128 channels: the default is the fused F(2,3) kernel; the three-kernel F(4,3) line stands beside it.
    # c4: the 16-bit default adds the DWM pieces in the batched GEMM; at stride 1 the pieces share one
    # transformed input (tile 3 / F(3,3) with the reference's three-tap pieces where the caller asks for tile 4,
    # tile 2 / F(2,2) with two-tap pieces where it asks for 2; 7x7 at stride 2: F(2,2) on the parity phases of x;
    # 3x3 at stride 2: the direct form, the product reading x itself, with the Winograd plans beside it),
    # else each has its own ("stacked"); two lines with
    # the reference's structure (pieces added after their output transforms) stand beside them.
    ("c1 fp32 N1 C64 56x56 F(2,3)", (1, 64, 56, 56), (64, 64, 3, 3), 1, 1, 2, "f32"),
    ("c2 vgg16 fp32 N8 F(2,3) x13 (first layer: one fused kernel)", "vgg", None, 1, 1, 2, "f32"),
    ("c2 vgg16 fp32 N8 F(4,3) x12 + fused F(2,3) first layer", "vgg", None, 1, 1, 4, "f32"),
    ("c3 fp16 N64 C64 56x56 F(2,3) one kernel", (64, 64, 56, 56), (64, 64, 3, 3), 1, 1, 2, "f16"),
    ("c3 fp16 N64 C64 56x56 F(4,3) three kernels", (64, 64, 56, 56), (64, 64, 3, 3), 1, 1, 4, "f16-unfused"),
    ("c3 fp16 N64 C128 28x28 F(2,3) one kernel", (64, 128, 28, 28), (128, 128, 3, 3), 1, 1, 2, "f16"),
    ("c3 fp16 N64 C128 28x28 F(4,3) three kernels", (64, 128, 28, 28), (128, 128, 3, 3), 1, 1, 4, "f16"),
    ("c3 fp16 N64 C256 14x14 F(4,3)", (64, 256, 14, 14), (256, 256, 3, 3), 1, 1, 4, "f16"),
    ("c3 fp16 N64 C512 7x7 F(4,3)", (64, 512, 7, 7), (512, 512, 3, 3), 1, 1, 4, "f16"),
    ("c4 fp16 N32 C128 112x112 5x5 s1 DWM shared input F(3,3)", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 4, "f16"),
    ("c4 fp16 N32 C128 112x112 7x7 s1 DWM shared input F(3,3)", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 4, "f16"),
    ("c4 fp16 N32 C128 112x112 5x5 s1 DWM shared input F(2,2)", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 2, "f16"),
    ("c4 fp16 N32 C128 112x112 7x7 s1 DWM shared input F(2,2)", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 2, "f16"),
    ("c4 fp16 N32 C128 112x112 5x5 s1 DWM F(2,r) stacked", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 2, "f16-stacked"),
    ("c4 fp16 N32 C128 112x112 7x7 s1 DWM F(2,r) stacked", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 2, "f16-stacked"),
    ("c4 fp16 N32 C128 112x112 5x5 s1 DWM F(4,r) stacked", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 4, "f16-stacked"),
    ("c4 fp16 N32 C128 112x112 7x7 s1 DWM F(4,r) stacked", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 4, "f16-stacked"),
    ("c4 fp16 N32 C128 112x112 3x3 s2 direct form (the default)", (32, 128, 112, 112), (128, 128, 3, 3), 2, 1, 2, "f16"),
    ("c4 fp16 N32 C128 112x112 3x3 s2 DWM F(2,r) stacked", (32, 128, 112, 112), (128, 128, 3, 3), 2, 1, 2, "f16-nodirect"),
    ("c4 fp16 N32 C128 112x112 3x3 s2 DWM F(4,r) stacked", (32, 128, 112, 112), (128, 128, 3, 3), 2, 1, 4, "f16-nodirect"),
    ("c4 fp16 N32 C128 112x112 7x7 s2 direct form (the default)", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 2, "f16"),
    ("c4 fp16 N32 C128 112x112 7x7 s2 DWM shared input F(2,2) on the parity phases", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 4, "f16-nodirect"),
    ("c4 fp16 N32 C128 112x112 7x7 s2 DWM F(2,r) stacked", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 2, "f16-stacked-nodirect"),
    ("c4 fp16 N32 C128 112x112 7x7 s2 DWM F(4,r) stacked", (32, 128, 112, 112), (128, 128, 7, 7), 2, 3, 4, "f16-stacked-nodirect"),
    ("c4 fp16 N32 C128 112x112 5x5 s1 DWM F(4,r) piece by piece", (32, 128, 112, 112), (128, 128, 5, 5), 1, 2, 4, "f16-pieces"),
    ("c4 fp16 N32 C128 112x112 7x7 s1 DWM F(4,r) piece by piece", (32, 128, 112, 112), (128, 128, 7, 7), 1, 3, 4, "f16-pieces"),
    ("first layer fp16 N32 3->64 224x224 7x7 s2 (the direct form's first-layer kernel)", (32, 3, 224, 224), (64, 3, 7, 7), 2, 3, 4, "f16"),
    ("3-D first layer fp16 N8 3->64 16x112x112 3x3x3 (the direct form's 3-D first-layer kernel)", (8, 3, 16, 112, 112), (64, 3, 3, 3, 3), 1, 1, 2, "f16"),
    ("c5 fp16 N8 C128 16x56x56 3x3x3 F(2,3)^3", (8, 128, 16, 56, 56), (128, 128, 3, 3, 3), 1, 1, 2, "f16"),
    ("c5 fp16 N8 C128 16x56x56 3x3x3 F(2,3)xF(4,3)^2", (8, 128, 16, 56, 56), (128, 128, 3, 3, 3), 1, 1, 4, "f16"),
    ("3-D DWM fp16 N4 C64 16x28x28 5x5x5 shared input F(2,2)^3", (4, 64, 16, 28, 28), (64, 64, 5, 5, 5), 1, 2, 2, "f16"),
    ("3-D DWM fp16 N4 C64 16x28x28 5x5x5 F(2,r)^3 stacked", (4, 64, 16, 28, 28), (64, 64, 5, 5, 5), 1, 2, 2, "f16-stacked"),
    ("metric fp16 N64 C256 56x56 F(2,3)", (64, 256, 56, 56), (256, 256, 3, 3), 1, 1, 2, "f16"),
    ("fp16 N64 C512 28x28 F(4,3) (batched GEMM on persistent 256x256 tiles)", (64, 512, 28, 28), (512, 512, 3, 3), 1, 1, 4, "f16"),
]
VGG16 = [(3, 64, 224), (64, 64, 224), (64, 128, 112), (128, 128, 112), (128, 256, 56), (256, 256, 56),
         (256, 256, 56), (256, 512, 28), (512, 512, 28), (512, 512, 28), (512, 512, 14), (512, 512, 14),
         (512, 512, 14)]


# the default form of every benchmark configuration (c1..c5): what a plain `python bench.py` adds to its JSON line
DEFAULTS = ("c1 ", "c2 vgg16 fp32 N8 F(4,3)", "c2 vgg16 fp32 N8 F(2,3)", "c3 fp16 N64 C64 56x56 F(2,3)", "c3 fp16 N64 C128 28x28 F(2,3)",
            "c3 fp16 N64 C64 56x56 F(4,3)", "c3 fp16 N64 C128 28x28 F(4,3)", "c3 fp16 N64 C256", "c3 fp16 N64 C512", "5x5 s1 DWM shared input F(3,3)", "7x7 s1 DWM shared input F(3,3)",
            "3x3 s2 direct form", "7x7 s2 direct form", "first layer fp16", "c5 fp16 N8 C128 16x56x56 3x3x3 F(2,3)^3")


def run_suite(steps=10, only=None, defaults=False):
    """ms per layer (whole forward through the one-call entry point, filter transform included;
    `ms_filter_cached`: with the filter transformed beforehand) and direct-convolution-equivalent
    TFLOP/s for every other benchmark configuration (`only`: just the configurations whose name
    contains that text)."""
    import torch
    from pytorch_winoconv_amd import engine
    dev = torch.device("cuda:0")
    out = []

    def one(xs, ws, stride, pad, m, dt, steps=steps):
        dtype = torch.float32 if dt == "f32" else torch.float16
        # None: the engine's default (16-bit: stride-1 kernels of 4..8 taps share one transformed input,
        # other DWM plans are stacked)
        stacked = False if "-pieces" in dt else True if "-stacked" in dt else None
        unfused = "-unfused" in dt                                 # thin layers: keep the three-kernel path
        direct = False if dt.endswith("-nodirect") else True if dt.endswith("-direct") else None
        g = torch.Generator().manual_seed(0)
        fan = 1
        for v in ws[1:]:
            fan *= v
        x = torch.randn(*xs, generator=g).to(dtype).to(dev)
        x = x.contiguous(memory_format=torch.channels_last if len(xs) == 4 else torch.channels_last_3d)
        w = (torch.randn(*ws, generator=g) * (2.0 / fan) ** 0.5).to(dtype).to(dev)
        # warm-up by time, not by count: a configuration measured in the first few milliseconds after another one
        # runs before the clocks have settled (fp32 layers measured 8-10 % slower that way)
        y = engine.conv_forward(x, w, None, stride, pad, m, stacked=stacked, unfused=unfused, direct=direct)
        torch.cuda.synchronize()
        t_warm = time.perf_counter()
        warm_calls = 0
        while time.perf_counter() - t_warm < 0.15:
            for _ in range(5):
                engine.conv_forward(x, w, None, stride, pad, m, stacked=stacked, unfused=unfused, direct=direct)
            torch.cuda.synchronize()
            warm_calls += 5
        # calls per timed round: at least `steps`, and enough of them for about 3 ms, so that the one wait for the
        # device at the end of a round is not a visible part of a layer that takes 10 us (it was, at 10 calls)
        per_call = (time.perf_counter() - t_warm) / warm_calls
        steps = max(steps, min(1000, int(3e-3 / per_call) + 1))
        # best of three rounds: a single round now and then includes a stall of tens of milliseconds
        # (the caching allocator returning memory between configurations of very different sizes)
        ms = float("inf")
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                engine.conv_forward(x, w, None, stride, pad, m, stacked=stacked, unfused=unfused, direct=direct)
            torch.cuda.synchronize()
            ms = min(ms, (time.perf_counter() - t0) / steps * 1e3)
        U = engine.transform_filter(w, xs, stride, pad, m, stacked=stacked, direct=direct)
        engine.conv_forward(x, w, None, stride, pad, m, U=U, stacked=stacked, unfused=unfused, direct=direct)
        msc = float("inf")
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                engine.conv_forward(x, w, None, stride, pad, m, U=U, stacked=stacked, unfused=unfused, direct=direct)
            torch.cuda.synchronize()
            msc = min(msc, (time.perf_counter() - t0) / steps * 1e3)
        flops = 2.0 * xs[0] * ws[0] * ws[1]
        for v in list(y.shape[2:]) + list(ws[2:]):
            flops *= v
        # the stock library on the same box and tensors (torch's convolution: MIOpen), as a yardstick; a failure
        # there (it has refused shapes before) must not cost the line
        conv = torch.nn.functional.conv2d if len(xs) == 4 else torch.nn.functional.conv3d
        mst = float("inf")
        try:
            for _ in range(3):
                conv(x, w, None, stride, pad)
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    conv(x, w, None, stride, pad)
                torch.cuda.synchronize()
                mst = min(mst, (time.perf_counter() - t0) / steps * 1e3)
        except RuntimeError:
            mst = float("nan")
        return ms, flops, msc, mst

    for name, xs, ws, stride, pad, m, dt in SUITE:
        if only and only not in name:
            continue
        if defaults and not any(key in name for key in DEFAULTS):
            continue
        try:
            if xs == "vgg":
                ms = fl = msc = mst = 0.0
                for c, k, hw in VGG16:
                    # like the modules: tile 2 where wc_conv_forward has a fused kernel for it (the 3-channel first layer)
                    tile = 2 if engine.thin_preferred(torch.float32 if dt == "f32" else torch.float16, 2, c, k, (3, 3), stride) else m
                    a, b, c_, d_ = one((8, c, hw, hw), (k, c, 3, 3), stride, pad, tile, dt)
                    ms, fl, msc, mst = ms + a, fl + b, msc + c_, mst + d_
            else:
                ms, fl, msc, mst = one(xs, ws, stride, pad, m, dt)
            out.append({"config": name, "ms": round(ms, 4), "effective_tflops": round(fl / ms / 1e9, 1),
                        "ms_filter_cached": round(msc, 4), "torch_conv_ms": None if mst != mst else round(mst, 4)})
        except Exception as e:                          # one configuration failing must not cost the others
            out.append({"config": name, "error": "%s: %s" % (type(e).__name__, e)})
    return out


def run_backward(steps=20):
    """us per call of the two gradients of the metric layer, next to the forward pass through the
    same Python entry points."""
    import torch
    from pytorch_winoconv_amd import engine
    dev = torch.device("cuda:0")
    x, w = synthetic(N)
    x = x.half().to(dev).contiguous(memory_format=torch.channels_last)
    w = w.half().to(dev)
    dy = torch.randn(N, K, H, W, generator=torch.Generator().manual_seed(1)).half().to(dev)
    dy = dy.contiguous(memory_format=torch.channels_last)
    calls = {
        "forward": lambda: engine.conv_forward(x, w, None, 1, PAD, M_TILE),
        "weight_gradient": lambda: engine.conv_backward_weight(x, dy, tuple(w.shape), 1, PAD, M_TILE),
        "input_gradient": lambda: engine.conv_backward_input(dy, w, (H, W), 1, PAD, M_TILE),
    }
    out = {}
    for name, fn in calls.items():
        for _ in range(3):
            fn()
        best = float("inf")
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(steps):
                fn()
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) / steps * 1e6)
        out[name] = round(best, 1)
    return out


def run_host_overhead(calls=300):
    """Host side of a small layer (c1: fp32, N=1, C=K=64, 56x56, F(2,3): four kernels of about 5 us): us per
    call of conv_forward through the compiled host layer (the pybind11 module MakePytorchBackend) and through
    the ctypes binding of the same C ABI.  `enqueue_us`: the loop of calls alone, before the device has been
    waited for (what the host spends per call); `wall_us`: the same loop including the final synchronisation."""
    import torch
    from pytorch_winoconv_amd import engine
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    x = torch.randn(1, 64, 56, 56, generator=g).to(dev).contiguous(memory_format=torch.channels_last)
    w = (torch.randn(64, 64, 3, 3, generator=g) * (2.0 / 576) ** 0.5).to(dev)
    out = {}
    for name, use_ext in (("compiled", True), ("ctypes", False)):
        if use_ext and engine._ext is None:
            continue
        engine.USE_EXT = use_ext
        try:
            for _ in range(20):
                engine.conv_forward(x, w, None, 1, 1, 2)
            best_q = best_w = float("inf")
            for _ in range(5):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(calls):
                    engine.conv_forward(x, w, None, 1, 1, 2)
                t1 = time.perf_counter()
                torch.cuda.synchronize()
                t2 = time.perf_counter()
                best_q, best_w = min(best_q, (t1 - t0) / calls * 1e6), min(best_w, (t2 - t0) / calls * 1e6)
            out[name] = {"enqueue_us": round(best_q, 1), "wall_us": round(best_w, 1)}
        finally:
            engine.USE_EXT = engine._ext is not None
    return out


def run_layouts(steps=50):
    """ms per layer with the input in channel-last memory (used as it is), in channel-first contiguous memory
    handed to the library (read inside the input transform, or copied by the library's kernel), and in
    channel-first memory permuted by a torch pass first (what the reference does: dwm.py:129-133); then the
    first again with a channel-first output."""
    import torch
    from pytorch_winoconv_amd import engine
    dev = torch.device("cuda:0")
    shapes = [("c1 fp32 N1 C64 56x56 F(2,3)", (1, 64, 56, 56), (64, 64, 3, 3), 2, torch.float32),
              ("c3 fp16 N64 C64 56x56 F(2,3) one kernel", (64, 64, 56, 56), (64, 64, 3, 3), 2, torch.float16),
              ("c3 fp16 N64 C128 28x28 F(4,3)", (64, 128, 28, 28), (128, 128, 3, 3), 4, torch.float16),
              ("c3 fp16 N64 C256 14x14 F(4,3)", (64, 256, 14, 14), (256, 256, 3, 3), 4, torch.float16),
              ("c3 fp16 N64 C512 7x7 F(4,3)", (64, 512, 7, 7), (512, 512, 3, 3), 4, torch.float16),
              ("metric fp16 N64 C256 56x56 F(4,3)", (64, 256, 56, 56), (256, 256, 3, 3), 4, torch.float16),
              ("c2 vgg fp32 N8 64->64 224x224 F(4,3)", (8, 64, 224, 224), (64, 64, 3, 3), 4, torch.float32)]
    out = []
    for name, xs, ws, m, dtype in shapes:
        g = torch.Generator().manual_seed(0)
        x_cf = torch.randn(*xs, generator=g).to(dtype).to(dev)
        x_cl = x_cf.contiguous(memory_format=torch.channels_last)
        w = (torch.randn(*ws, generator=g) * (2.0 / (ws[1] * 9)) ** 0.5).to(dtype).to(dev)
        calls = {
            "channel_last_in": lambda: engine.conv_forward(x_cl, w, None, 1, 1, m),
            "channel_first_in": lambda: engine.conv_forward(x_cf, w, None, 1, 1, m),
            "channel_first_in_torch_permute": lambda: engine.conv_forward(x_cf.contiguous(memory_format=torch.channels_last), w, None, 1, 1, m),
            "channel_first_in_and_out": lambda: engine.conv_forward(x_cf, w, None, 1, 1, m, channels_first_out=True),
            "channel_first_in_and_out_torch_permutes": lambda: engine.conv_forward(
                x_cf.contiguous(memory_format=torch.channels_last), w, None, 1, 1, m).contiguous(),
        }
        row = {"config": name}
        for what, fn in calls.items():
            for _ in range(5):
                fn()
            best = float("inf")
            for _ in range(3):
                torch.cuda.synchronize()
                t0 = time.perf_counter()
                for _ in range(steps):
                    fn()
                torch.cuda.synchronize()
                best = min(best, (time.perf_counter() - t0) / steps * 1e3)
            row[what] = round(best, 4)
        out.append(row)
    return out


def run_chunk_residency(iters=40):
    """The three kernels of the metric layer on chunks of its batch, with V and M in the same buffers every iteration
    (a chunk's V and M then sit in the 256 MB last-level cache when the next kernel reads them) and with V and M rotated
    over more than 700 MB of buffers (served by HBM): us per chunk and per 64 images.  x and y always rotate over three
    batches.  What a forward pass blocked per image chunk could gain from cache residency."""
    import torch
    from pytorch_winoconv_amd import _lib, engine
    lib = _lib.load()
    dev = torch.device("cuda:0")
    g = torch.Generator().manual_seed(0)
    xs = [torch.randn(N, H, W, C, generator=g).half().to(dev) for _ in range(3)]
    ys = [torch.empty(N, H, W, K, dtype=torch.float16, device=dev) for _ in range(3)]
    w = (torch.randn(K, C, R, R, generator=g) * (2.0 / (C * R * R)) ** 0.5).half().to(dev)
    out = []
    for nc in (64, 16, 8, 4):
        desc = engine.make_desc((nc, C, H, W), w.shape, torch.float16, 1, PAD, M_TILE)
        plan = engine.plan_conv(desc)
        U = engine.filter_transform(desc, plan, w)
        _, grid = engine.out_dims(desc)
        P, T = nc * grid[1] * grid[2], plan.t_total
        Cp, ldm = lib.wc_padded_channels(C), lib.wc_padded_channels8(K)
        st = engine._stream(xs[0])
        for mode in ("hot", "cold"):
            nset = 1 if mode == "hot" else max(2, int(700e6 // (2 * T * P * Cp * 2)) + 1)
            Vs = [torch.empty(T, P, Cp, dtype=torch.float16, device=dev) for _ in range(nset)]
            Ms = [torch.empty(T, P, ldm, dtype=torch.float16, device=dev) for _ in range(nset)]
            ev = [[torch.cuda.Event(enable_timing=True) for _ in range(4)] for _ in range(iters)]

            def one(i, e=None):
                V, Mb = Vs[i % nset], Ms[i % nset]
                b0 = (i * nc) % N
                xi, yi = xs[i % 3][b0:b0 + nc], ys[i % 3][b0:b0 + nc]
                if e: e[0].record()
                _lib.check(lib.wc_input_transform(ctypes.byref(desc), ctypes.byref(plan), engine._ptr(xi), nc, engine._ptr(V), st))
                if e: e[1].record()
                _lib.check(lib.wc_batched_gemm(engine._ptr(V), engine._ptr(U), engine._ptr(Mb), T, P, Cp, K, ldm, desc.dtype, st))
                if e: e[2].record()
                _lib.check(lib.wc_output_transform(ctypes.byref(desc), ctypes.byref(plan), engine._ptr(Mb), None, nc, engine._ptr(yi), st))
                if e: e[3].record()
            t0, i = time.perf_counter(), 0
            while time.perf_counter() - t0 < 0.3:
                one(i); i += 1
            torch.cuda.synchronize()
            for j in range(iters):
                one(i + j, ev[j])
            torch.cuda.synchronize()
            us = [sum(e[k].elapsed_time(e[k + 1]) for e in ev) / iters * 1e3 for k in range(3)]
            out.append({"chunk_images": nc, "V_M": mode, "buffer_sets": nset,
                        "us_per_chunk": {"input_transform": round(us[0], 1), "batched_gemm": round(us[1], 1), "output_transform": round(us[2], 1)},
                        "us_per_64_images": round(sum(us) * N / nc, 1)})
            del Vs, Ms
    return out


def run_split_concat(steps=20):
    """Tile split / concat (bit-exact copies) at the metric layer's shape: us per call and HBM GB/s
    of the algorithmic bytes (input once + tiles once; tiles once + output once)."""
    import torch
    from pytorch_winoconv_amd import backend
    dev = torch.device("cuda:0")
    out = {}
    for name, dtype in (("f32", torch.float32), ("f16", torch.float16)):
        for alpha, m in ((4, 2), (6, 4)):
            x = torch.randn(N, H + 2, W + 2, C, device=dev).to(dtype)            # padded by one, channel-last
            nH, nW = (H + m - 1) // m, (W + m - 1) // m
            tiles = torch.empty(N * nH * nW, C, alpha, alpha, dtype=dtype, device=dev)
            yt = torch.randn(N * nH * nW, K, m, m, device=dev).to(dtype)
            y = torch.empty(N, H, W, K, dtype=dtype, device=dev)
            calls = {
                "split": (lambda: backend.WinoSplit(x, tiles, 1, alpha, alpha, m, 1, nH, nW, True),
                          (x.numel() + tiles.numel()) * x.element_size()),
                "concat": (lambda: backend.WinoConcat(yt, y, m, True), (yt.numel() + y.numel()) * y.element_size()),
            }
            for what, (fn, nbytes) in calls.items():
                for _ in range(3):
                    fn()
                best = float("inf")
                for _ in range(3):
                    torch.cuda.synchronize()
                    t0 = time.perf_counter()
                    for _ in range(steps):
                        fn()
                    torch.cuda.synchronize()
                    best = min(best, (time.perf_counter() - t0) / steps)
                out["%s %s %dx%d tiles, step %d" % (what, name, alpha if what == "split" else m,
                                                    alpha if what == "split" else m, m)] = {
                    "us": round(best * 1e6, 1), "MB": round(nbytes / 1e6, 1), "GB_s": round(nbytes / best / 1e9, 0)}
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--prewarm", type=float, default=0.5, metavar="SECONDS",
                    help="run untimed steps for this long before the warm-up steps (clocks settle)")
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--gemm-config", type=int, default=-1, metavar="I",
                    help="force tile shape I of the batched GEMM through the library's test hook (-1: its own choice)")
    ap.add_argument("--suite", action="store_true",
                    help="time every form of every other benchmark configuration (the 'suite' list); without it the "
                         "list holds the default form of each benchmark configuration (c1..c5), about 20 s")
    ap.add_argument("--no-suite", action="store_true", help="no 'suite' list at all: the metric layer only")
    ap.add_argument("--event-every", type=int, default=4, metavar="N",
                    help="record the per-stage HIP events on every N-th timed step (an event record between two "
                         "kernels keeps the second from starting under the tail of the first: about 13 us per "
                         "step with events, measured; 1 = every step)")
    ap.add_argument("--suite-only", default=None, metavar="TEXT",
                    help="with --suite: only the configurations whose name contains TEXT")
    ap.add_argument("--backward", action="store_true",
                    help="also time the weight and input gradients of the metric layer")
    ap.add_argument("--split-concat", action="store_true",
                    help="also time the tile split / concat kernels at the metric layer's shape")
    ap.add_argument("--host-overhead", action="store_true",
                    help="also time the host side of a small layer (c1) through the compiled host layer and through ctypes")
    ap.add_argument("--layouts", action="store_true",
                    help="also time small and large layers with channel-last and channel-first tensors")
    ap.add_argument("--chunk-residency", action="store_true",
                    help="also time the three kernels of the metric layer on chunks of 64 / 16 / 8 / 4 images with V and M "
                         "kept in one set of buffers (last-level cache resident) and rotated over 700 MB (from HBM)")
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
    if args.gemm_config >= 0:
        os.environ["WINOCONV_TEST_HOOKS"] = "1"      # the tile-shape hook is inert in a process that does not opt in
    lib = _lib.load()
    if args.gemm_config >= 0:
        _lib.check(lib.wc_test_gemm_override(args.gemm_config, 1))
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
    # U, V and M laid out as wc_conv_forward lays them out in its workspace (each 256-byte aligned)
    nb = ctypes.c_size_t()
    _lib.check(lib.wc_conv_workspace_bytes(ctypes.byref(desc), ctypes.byref(nb)))
    wsbuf = torch.empty(nb.value, dtype=torch.uint8, device=dev)
    r256 = lambda v: (v + 255) // 256 * 256
    ub, vb = r256(T * K * Cp * 2), r256(T * P * Cp * 2)
    U = wsbuf[:T * K * Cp * 2].view(dtype).view(T, K, Cp)
    V = wsbuf[ub:ub + T * P * Cp * 2].view(dtype).view(T, P, Cp)
    Mb = wsbuf[ub + vb:ub + vb + T * P * ldm * 2].view(dtype).view(T, P, ldm)
    y = torch.empty(N, out[1], out[2], K, dtype=dtype, device=dev)
    st = engine._stream(x)
    d_, p_ = ctypes.byref(desc), ctypes.byref(plan)
    ws = engine._w_strides(w)
    px, pw, pU, pV, pM, py = (engine._ptr(t) for t in (x_cl, w, U, V, Mb, y))

    pws, nws = engine._ptr(wsbuf), nb.value

    def step(ev=None):
        """One pass of the layer into y.  Without events: one call of wc_conv_forward, the entry point a caller of
        the reference's DWM binds, on the caller-provided workspace.  With events: the same four stages through
        their own entry points (what wc_conv_forward runs inside, except that it transforms the filter in the
        launch of the input transform), with a record between them."""
        if not ev:
            _lib.check(lib.wc_conv_forward(d_, px, pw, ws, None, None, py, pws, nws, st))
            return
        if ev[0]: ev[0].record()
        _lib.check(lib.wc_filter_transform(d_, p_, pw, ws, pU, st))
        if ev[1]: ev[1].record()
        _lib.check(lib.wc_input_transform(d_, p_, px, N, pV, st))
        ev[2].record()
        _lib.check(lib.wc_batched_gemm(pV, pU, pM, T, P, Cp, K, ldm, desc.dtype, st))
        ev[3].record()
        _lib.check(lib.wc_output_transform(d_, p_, pM, None, N, py, st))
        if ev[4]: ev[4].record()

    if args.copy_probe:
        src = torch.empty(128 * 1024 * 1024, dtype=torch.uint8, device=dev)
        dst = torch.empty_like(src)
        for _ in range(3):
            dst.copy_(src)
    # Untimed steps for a fixed wall time first: a GPU that has been idle needs a few tenths of a second of
    # work to reach its steady clocks, far more than a handful of 0.25 ms warm-up steps provide.
    # The untimed steps mix the two forms of a step like the timed ones (a kernel's first launch loads its code).
    spare = [torch.cuda.Event(enable_timing=True) for _ in range(5)]
    t_pre = time.perf_counter()
    while time.perf_counter() - t_pre < args.prewarm:
        for i in range(10):
            step(spare if i % args.event_every == 0 else None)
        torch.cuda.synchronize()
    prewarm_s = time.perf_counter() - t_pre
    for i in range(args.warmup):
        step(spare if i % args.event_every == 0 else None)
    torch.cuda.synchronize()
    # The batched GEMM, the kernel of the roofline figure, is bracketed by two HIP events inside the timed region,
    # on every fourth step by default (--event-every); its average agrees with the profiler's kernel duration
    # (120.6 against 120.4 us on one box).  Those steps run the four stage entry points; the steps without
    # records are single calls of wc_conv_forward.  The other stages are timed the same way, with a record between
    # every two of them, in a few untimed steps right afterwards (a step with five records takes about 13 us
    # longer than one with none, because each record sits between two kernels).
    sampled = [i % args.event_every == 0 for i in range(args.steps)]
    def gemm_events():
        return [None, None, torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True), None]
    events = [gemm_events() if s else None for s in sampled]
    t0 = time.perf_counter()
    for ev in events:
        step(ev)
    torch.cuda.synchronize()
    elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3

    names = ("filter_transform", "input_transform", "batched_gemm", "output_transform")
    timed = [ev for ev in events if ev]
    gemm_us = sum(ev[2].elapsed_time(ev[3]) for ev in timed) / len(timed) * 1e3
    after = [[torch.cuda.Event(enable_timing=True) for _ in range(5)] for _ in range(8)]
    for ev in after:
        step(ev)
    torch.cuda.synchronize()
    stage_us = {n: sum(ev[i].elapsed_time(ev[i + 1]) for ev in after) / len(after) * 1e3
                for i, n in enumerate(names)}
    stage_us["batched_gemm"] = gemm_us          # the one measured inside the timed region

    # the product's one-call entry point on the same inputs, for comparison
    def one_call():
        return engine.conv_forward(x, w, None, 1, PAD, M_TILE)
    y1 = one_call()
    y.zero_()
    step([torch.cuda.Event(enable_timing=True) for _ in range(5)])      # y from the four stage entry points
    torch.cuda.synchronize()
    same = bool(torch.equal(y1.permute(0, 2, 3, 1), y))
    def best_of_three(fn):
        # a single round now and then includes a stall of tens of milliseconds (the caching
        # allocator growing or returning memory): the best of three rounds of `steps` calls
        # at least 50 calls per round after five untimed ones: the first calls through the Python layer get their
        # workspace and output from the allocator for the first time
        calls = max(args.steps, 50)
        for _ in range(5):
            fn()
        best = float("inf")
        for _ in range(3):
            torch.cuda.synchronize()
            t0 = time.perf_counter()
            for _ in range(calls):
                fn()
            torch.cuda.synchronize()
            best = min(best, (time.perf_counter() - t0) / calls * 1e3)
        return best

    ms_one_call = best_of_three(one_call)
    # the same with the filter transformed once beforehand (what a module with fixed weights does)
    U_cached = engine.transform_filter(w, x.shape, 1, PAD, M_TILE)
    ms_cached = best_of_three(lambda: engine.conv_forward(x, w, None, 1, PAD, M_TILE, U=U_cached))

    direct_flops = 2.0 * N * K * C * out[1] * out[2] * R * R
    gemm_flops = 2.0 * T * P * C * K
    gemm_tflops = gemm_flops / (stage_us["batched_gemm"] * 1e-6) / 1e12
    es = 2
    # The GEMM's algorithmic bytes (V and U read once, M written once): at 127 flop/byte the
    # kernel sits left of the ridge of the MI355X roofline (2500 TFLOP/s / 8 TB/s = 312 flop/byte),
    # so the HBM view is reported beside the MFMA one.
    gemm_bytes = (V.numel() + U.numel() + Mb.numel()) * es
    gemm_gb_s = gemm_bytes / (stage_us["batched_gemm"] * 1e-6) / 1e9
    hbm = {
        "input_transform": (x.numel() + V.numel()) * es,
        "output_transform": (Mb.numel() + y.numel()) * es,
    }
    result = {
        "metric": "effective TFLOP/s (direct-conv-equivalent), 3x3 conv fp16 N=64 C=K=256 56x56, 1 MI355X",
        "value": direct_flops / (ms_per_step * 1e-3) / 1e12,
        "unit": "TFLOP/s",
        "n_gpus": 1, "steps": args.steps, "warmup": args.warmup, "prewarm_s": round(prewarm_s, 3),
        "ms_per_step": ms_per_step,
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "conv2d 3x3 s1 p1, N=64 C=K=256 56x56, fp16 in / fp32 accumulate, "
                               "Winograd F(4x4,3x3), T=36 P=12544, NHWC resident in HBM, filter "
                               "transform included in every step"},
        "roofline": {"bound": "mfma", "achieved": gemm_tflops, "peak": MFMA_FP16_PEAK_TFLOPS,
                     "unit": "TFLOP/s", "frac": gemm_tflops / MFMA_FP16_PEAK_TFLOPS,
                     "traffic": GEMM_HBM_TRAFFIC_BYTES, "kernel": "wc::gemm_persistent_deferred_kernel (wc_batched_gemm)",
                     "flops_per_launch": gemm_flops, "avg_us": stage_us["batched_gemm"],
                     "hbm_view": {"bytes_per_launch": gemm_bytes, "achieved": gemm_gb_s, "peak": HBM_PEAK_GB_S,
                                  "unit": "GB/s", "frac": gemm_gb_s / HBM_PEAK_GB_S}},
        "stage_us": stage_us,
        "stage_hbm_tb_s": {k: v / (stage_us[k] * 1e-6) / 1e12 for k, v in hbm.items()},
        "ms_per_layer_one_call": ms_one_call,
        "ms_per_layer_filter_cached": ms_cached,
        "effective_tflops_filter_cached": direct_flops / (ms_cached * 1e-3) / 1e12,
        "one_call_matches_stages": same,
        "timed_steps": {"wc_conv_forward": sampled.count(False), "four_stage_calls_with_events": sampled.count(True)},
    }
    if args.suite or args.suite_only:
        result["suite"] = run_suite(only=args.suite_only)
    elif not args.no_suite:
        result["suite"] = run_suite(defaults=True)
    if args.backward:
        result["backward_us"] = run_backward()
    if args.split_concat:
        result["split_concat"] = run_split_concat()
    if args.layouts:
        result["layouts_ms"] = run_layouts()
    if args.chunk_residency:
        result["chunk_residency"] = run_chunk_residency()
    if args.host_overhead:
        result["host_overhead_c1"] = run_host_overhead()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline()
    print(json.dumps(result))


if __name__ == "__main__":
    main()
