#!/usr/bin/env python3
"""Benchmark: batch-1 latency of the PET-optimised dilated-conv block on one MI355X.

Workload (benchmark configuration 2): six fp32 3x3 convolutions, dilation 2 / pad 2,
channels 512->512->512->512->256->128->64 on a 1x512x64x64 input, ReLU after
each, weights N(0, 0.01). The PET-optimised program is space-to-batch (4 phase
images of 32x32), six dense convolutions (dilation 1, pad 1) with fused ReLU,
batch-to-space. One "step" is one launch of that program as a HIP graph with
inputs and weights resident in HBM.

Prints one JSON line: the latency (`value`, ms), the roofline of the dominant
kernel (the 512->512 implicit-GEMM convolution, against the fp32 MFMA peak) from
HIP events around that kernel alone, and the CPU oracle timed on a bounded
sample of the same workload on this box's host cores.
"""
import argparse
import ctypes
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

CHANNELS = [512, 512, 512, 512, 256, 128, 64]
HW = 64
DIL = 2
MFMA_FP32_PEAK_TFLOPS = 157.3
HBM_PEAK_GBS = 8000.0


def conv_flop(n, f, oh, ow, c, r, s):
    return 2.0 * n * f * oh * ow * c * r * s


DOMINANT_PROFILE = os.path.join(ROOT, "profiles", "conv_plane_64x64_rs9_c2_layer_512to512.txt")


def dominant_traffic_bytes():
    """HBM-side bytes one launch of the dominant kernel moves, read from the committed
    rocprofv3 --pmc summary of `bench.py --dominant-only 20` (a counter cannot be read from
    inside this process): FETCH_SIZE and WRITE_SIZE in KiB per dispatch of the convolution,
    each scaled by what the same counter reads for the 256 MiB plain copy of the same run.
    None when the summary is missing or does not parse."""
    import re
    try:
        text = open(DOMINANT_PROFILE).read()
    except OSError:
        return None
    val = {}
    for kernel, key in (("conv_plane_kernel", "conv"), ("view_direct_kernel", "copy")):
        for counter in ("FETCH_SIZE", "WRITE_SIZE"):
            m = re.search(r"^[^\n]*%s[^\n]*\s%s\s+dispatches=\d+\s+avg_KiB=([0-9.]+)"
                          % (kernel, counter), text, re.M)
            if not m:
                return None
            val[key, counter] = float(m.group(1))
    copy_kib = 256.0 * 1024
    fetch = val["conv", "FETCH_SIZE"] * copy_kib / val["copy", "FETCH_SIZE"]
    write = val["conv", "WRITE_SIZE"] * copy_kib / val["copy", "WRITE_SIZE"]
    return int((fetch + write) * 1024)


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--cpu-seconds", type=float, default=15.0)
    ap.add_argument("--unfolded-layout", action="store_true",
                    help="run space-to-batch and batch-to-space as launches of their own "
                         "instead of as the neighbouring convolutions' addressing")
    ap.add_argument("--no-configs", action="store_true",
                    help="skip the latency table of the other four configurations")
    ap.add_argument("--config-only", default="", metavar="c1|c3|c4|c5[:pet]",
                    help="replay that configuration's graph 20 times and exit (for rocprofv3)")
    ap.add_argument("--layout-only", type=int, default=0, metavar="N",
                    help="launch only the 1 GiB layout operators N times each and exit (for rocprofv3)")
    ap.add_argument("--dominant-only", type=int, default=0, metavar="N",
                    help="launch only the dominant kernel N times and exit (for rocprofv3)")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one MI355X; this build has no multi-GPU path "
                 "(run with --gpus 1)")

    import numpy as np
    import torch
    from pet_amd import abi, ops

    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    torch.cuda.set_device(0)
    abi.init(0)
    dev = torch.device("cuda:0")

    g = torch.Generator(device="cpu").manual_seed(0)
    x = torch.randn((1, CHANNELS[0], HW, HW), generator=g).to(dev)
    ws = [(0.01 * torch.randn((CHANNELS[i + 1], CHANNELS[i], 3, 3), generator=g)).to(dev)
          for i in range(6)]

    hs = HW // DIL
    s2b_flat, s2b_perm = [1, CHANNELS[0], hs, DIL, hs, DIL], [3, 5, 0, 1, 2, 4]
    b2s_flat, b2s_perm = [DIL, DIL, 1, CHANNELS[-1], hs, hs], [2, 3, 4, 0, 5, 1]

    # pre-allocated activations: nothing is allocated inside a step
    t_s2b = torch.empty((DIL * DIL, CHANNELS[0], hs, hs), device=dev)
    t_act = [torch.empty((DIL * DIL, CHANNELS[i + 1], hs, hs), device=dev) for i in range(6)]
    t_out = torch.empty((1, CHANNELS[-1], HW, HW), device=dev)
    o_act = [torch.empty((1, CHANNELS[i + 1], HW, HW), device=dev) for i in range(6)]

    # What the graph runtime of the host layer plans for this chain (code_engine.cc,
    # planLaunchFlags), done by hand for the six calls: the outputs of the convolutions that
    # add partial sums into their output are initialised by one batched launch up front, and
    # such a convolution leaves its ReLU to the convolution that reads it.
    from pet_amd import abi as _abi
    accum = [ops.conv2d_accumulates((DIL * DIL, CHANNELS[i], hs, hs),
                                    (CHANNELS[i + 1], CHANNELS[i], 3, 3), 1, 1) for i in range(6)]
    fills = [(t_act[i], None, DIL * DIL, CHANNELS[i + 1], hs * hs) for i in range(6) if accum[i]]
    flags = []
    for i in range(6):
        fl = _abi.Y_INITIALISED if accum[i] else 0
        if accum[i] and i < 5:
            fl |= _abi.DEFER_RELU
        if i > 0 and accum[i - 1]:
            fl |= _abi.X_RELU
        flags.append(fl)

    # The two layout operators of the program are addressing modes of the convolutions next
    # to them (pet_hip_conv2d_view_f32): the first convolution reads x through the strides of
    # the space-to-batch Transpose, the last one writes through those of batch-to-space.
    # --unfolded-layout keeps them as launches of their own.
    folded = not args.unfolded_layout and \
        ops.conv2d_view_supported((DIL * DIL, CHANNELS[0], hs, hs), tuple(ws[0].shape), 1, 1) and \
        ops.conv2d_view_supported((DIL * DIL, CHANNELS[5], hs, hs), tuple(ws[5].shape), 1, 1)
    view_in = ops.interleave_view(1, CHANNELS[0], hs, hs, DIL)
    view_out = ops.interleave_view(1, CHANNELS[-1], hs, hs, DIL)
    if folded and accum[5]:
        fills[-1] = (t_out, None, 1, CHANNELS[-1], HW * HW)

    def optimised():
        if fills:
            ops.bias_fill_batch(fills)
        if not folded:
            ops.permute_flat(x, s2b_flat, s2b_perm, out=t_s2b)
            cur = t_s2b
            for i in range(6):
                ops.conv2d(cur, ws[i], 1, 1, act="relu", out=t_act[i], flags=flags[i])
                cur = t_act[i]
            ops.permute_flat(cur, b2s_flat, b2s_perm, out=t_out)
            return
        ops.conv2d(x, ws[0], 1, 1, act="relu", out=t_act[0], flags=flags[0], x_view=view_in,
                   x_shape=tuple(t_s2b.shape))
        for i in range(1, 5):
            ops.conv2d(t_act[i - 1], ws[i], 1, 1, act="relu", out=t_act[i], flags=flags[i])
        ops.conv2d(t_act[4], ws[5], 1, 1, act="relu", out=t_out, flags=flags[5], y_view=view_out)

    def original():
        cur = x
        for i in range(6):
            ops.conv2d(cur, ws[i], DIL, DIL, 1, 1, DIL, DIL, act="relu", out=o_act[i])
            cur = o_act[i]

    stream = torch.cuda.Stream()
    sp = ctypes.c_void_p(stream.cuda_stream)

    if args.config_only:
        # profiling aid: one configuration (original program, or PET's with ":pet") as a graph
        from pet_amd import programs
        name, _, variant = args.config_only.partition(":")
        run, params = getattr(programs, "run_" + name), getattr(programs, "params_" + name)(0)
        ns, table = programs.GpuNS(keep=True), {}
        with torch.cuda.stream(stream):
            run(ns, params, variant == "pet", T=table)
            stream.synchronize()
            ns.kept.clear()
            abi.call("pet_hip_graph_begin_capture", sp)
            try:
                run(ns, params, variant == "pet", T=table)
            finally:
                gh = ctypes.c_void_p(0)
                abi.call("pet_hip_graph_end_capture", sp, ctypes.byref(gh))
        for _ in range(20):
            abi.call("pet_hip_graph_launch", gh, sp)
        torch.cuda.synchronize()
        return

    if args.layout_only:
        # profiling aid: a 256 MiB calibration copy, then the 1 GiB layout operators
        cal = torch.zeros((64, 1024, 1024), device=dev)
        cal_out = torch.empty_like(cal)
        ops.pad(cal, [0, 0, 0], [0, 0, 0], out=cal_out)
        del cal, cal_out
        big = torch.randn((1, 4096, 256, 256), device=dev)
        big_out = torch.empty((4, 4096, 128, 128), device=dev)
        halo_chain = [("split", 2, 128, 0, 1), ("reorder", [0, 2, 1, 3, 4]), ("fuse", 0, 0, 0)]
        halo_out = ops.trans_chain(big, halo_chain)
        for _ in range(args.layout_only):
            ops.permute_flat(big, [1, 4096, 128, 2, 128, 2], [3, 5, 0, 1, 2, 4], out=big_out)
            ops.permute_flat(big_out, [2, 2, 1, 4096, 128, 128], [2, 3, 4, 0, 5, 1], out=big)
            ops.permute_flat(big, [1, 4096, 2, 128, 256], [0, 2, 1, 3, 4], out=big_out)
            ops.trans_chain(big, halo_chain, out=halo_out)
        del big_out, halo_out
        # odd rows: zero-pad 126x126 planes to 128x128 and crop them back
        odd = big.reshape(-1)[:64 * 256 * 126 * 126].reshape(64, 256, 126, 126)
        padded = torch.empty((64, 256, 128, 128), device=dev)
        for _ in range(args.layout_only):
            ops.pad(odd, [0, 0, 1, 1], [0, 0, 1, 1], out=padded)
            ops.slice_(padded, [0, 0, 1, 1], [0, 0, 1, 1], out=odd)
        torch.cuda.synchronize()
        return

    if args.dominant_only:
        # profiling aid: the 512->512 layer of the optimised program, nothing else
        # plus one plain copy of 256 MiB (a pad by zero) that calibrates the
        # FETCH_SIZE / WRITE_SIZE counters
        cal = torch.zeros((64, 1024, 1024), device=dev)
        cal_out = torch.empty_like(cal)
        ops.pad(cal, [0, 0, 0], [0, 0, 0], out=cal_out)
        ops.permute_flat(x, s2b_flat, s2b_perm, out=t_s2b)
        for _ in range(args.dominant_only):
            ops.conv2d(t_s2b, ws[0], 1, 1, act="relu", out=t_act[0])
        torch.cuda.synchronize()
        return

    def capture(fn):
        with torch.cuda.stream(stream):
            fn()  # eager once (also warms up code objects)
            stream.synchronize()
            abi.call("pet_hip_graph_begin_capture", sp)
            fn()
            gh = ctypes.c_void_p(0)
            abi.call("pet_hip_graph_end_capture", sp, ctypes.byref(gh))
        return gh

    def time_graph(gh, steps, warmup):
        for _ in range(warmup):
            abi.call("pet_hip_graph_launch", gh, sp)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(steps):
            abi.call("pet_hip_graph_launch", gh, sp)
        torch.cuda.synchronize()
        return (time.perf_counter() - t0) * 1e3 / steps

    g_opt = capture(optimised)
    g_org = capture(original)
    # the two programs agree (fp32 summation order differs between them)
    torch.cuda.synchronize()
    diff = (t_out - o_act[-1]).abs().max().item()
    scale = o_act[-1].abs().max().item()
    if not diff <= 1e-4 * max(scale, 1e-30):
        sys.exit("optimised and original programs disagree: %g vs scale %g" % (diff, scale))

    # `steps` launches are timed as one block; the block is repeated and the median block
    # is the value (a single block of 200 launches is a 0.13 s sample)
    REPEATS = 5
    blocks = sorted(time_graph(g_opt, args.steps, args.warmup if r == 0 else 0)
                    for r in range(REPEATS))
    ms_opt = blocks[REPEATS // 2]
    ms_org = time_graph(g_org, max(10, args.steps // 4), max(2, args.warmup // 4))

    # ---- per-kernel timing with HIP events on the launch stream
    ev0, ev1 = ctypes.c_void_p(0), ctypes.c_void_p(0)
    abi.call("pet_hip_event_create", ctypes.byref(ev0))
    abi.call("pet_hip_event_create", ctypes.byref(ev1))

    def time_kernel(fn, reps=50, warm=5):
        with torch.cuda.stream(stream):
            for _ in range(warm):
                fn()
            abi.call("pet_hip_event_record", ev0, sp)
            for _ in range(reps):
                fn()
            abi.call("pet_hip_event_record", ev1, sp)
            abi.call("pet_hip_event_sync", ev1)
            ms = ctypes.c_float(0)
            abi.call("pet_hip_event_elapsed_ms", ctypes.byref(ms), ev0, ev1)
        return ms.value / reps

    per_op = []
    s2b_bytes = 4.0 * 2 * x.numel()
    ms = time_kernel(lambda: ops.permute_flat(x, s2b_flat, s2b_perm, out=t_s2b))
    per_op.append({"op": "space_to_batch 1x512x64x64", "ms": ms, "GB/s": s2b_bytes / ms / 1e6,
                   "frac_hbm": s2b_bytes / ms / 1e6 / HBM_PEAK_GBS})
    conv_ms = []
    for i in range(6):
        src = t_s2b if i == 0 else t_act[i - 1]
        fl = conv_flop(DIL * DIL, CHANNELS[i + 1], hs, hs, CHANNELS[i], 3, 3)
        ms = time_kernel(lambda s=src, i=i: ops.conv2d(s, ws[i], 1, 1, act="relu", out=t_act[i]))
        conv_ms.append(ms)
        per_op.append({"op": "conv3x3 %d->%d @4x32x32" % (CHANNELS[i], CHANNELS[i + 1]),
                       "ms": ms, "TFLOP/s": fl / ms / 1e9,
                       "frac_mfma": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS})
    b2s_bytes = 4.0 * 2 * t_out.numel()
    ms = time_kernel(lambda: ops.permute_flat(t_act[5], b2s_flat, b2s_perm, out=t_out))
    per_op.append({"op": "batch_to_space 4x64x32x32", "ms": ms, "GB/s": b2s_bytes / ms / 1e6,
                   "frac_hbm": b2s_bytes / ms / 1e6 / HBM_PEAK_GBS})
    # the first and the last convolution as the timed program runs them: through the strides
    # of the layout operator next to them
    if folded:
        fl = conv_flop(DIL * DIL, CHANNELS[1], hs, hs, CHANNELS[0], 3, 3)
        ms = time_kernel(lambda: ops.conv2d(x, ws[0], 1, 1, act="relu", out=t_act[0],
                                            x_view=view_in, x_shape=tuple(t_s2b.shape)))
        per_op.append({"op": "conv3x3 %d->%d reading 1x%dx%dx%d through the space-to-batch "
                             "strides" % (CHANNELS[0], CHANNELS[1], CHANNELS[0], HW, HW),
                       "ms": ms, "TFLOP/s": fl / ms / 1e9,
                       "frac_mfma": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS})
        fl = conv_flop(DIL * DIL, CHANNELS[6], hs, hs, CHANNELS[5], 3, 3)
        ms = time_kernel(lambda: ops.conv2d(t_act[4], ws[5], 1, 1, act="relu", out=t_out,
                                            y_view=view_out))
        per_op.append({"op": "conv3x3 %d->%d writing 1x%dx%dx%d through the batch-to-space "
                             "strides" % (CHANNELS[5], CHANNELS[6], CHANNELS[6], HW, HW),
                       "ms": ms, "TFLOP/s": fl / ms / 1e9,
                       "frac_mfma": fl / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS})
    # HBM-bound layout kernel at a size that cannot hide in cache: 1 GiB each way
    big = torch.empty((1, 4096, 256, 256), device=dev)
    big_out = torch.empty((4, 4096, 128, 128), device=dev)
    bflat, bperm = [1, 4096, 128, 2, 128, 2], [3, 5, 0, 1, 2, 4]
    big_bytes = 4.0 * 2 * big.numel()
    ms = time_kernel(lambda: ops.permute_flat(big, bflat, bperm, out=big_out), reps=10, warm=2)
    per_op.append({"op": "space_to_batch 1x4096x256x256 (1 GiB)", "ms": ms,
                   "GB/s": big_bytes / ms / 1e6, "frac_hbm": big_bytes / ms / 1e6 / HBM_PEAK_GBS})
    # ... its inverse, the H2N transform (an outer-dimension move), and the same H2N with
    # the one-row halo that makes the transformed convolution exact
    ms = time_kernel(lambda: ops.permute_flat(big_out, [2, 2, 1, 4096, 128, 128],
                                              [2, 3, 4, 0, 5, 1], out=big), reps=10, warm=2)
    per_op.append({"op": "batch_to_space 4x4096x128x128 (1 GiB)", "ms": ms,
                   "GB/s": big_bytes / ms / 1e6, "frac_hbm": big_bytes / ms / 1e6 / HBM_PEAK_GBS})
    ms = time_kernel(lambda: ops.permute_flat(big, [1, 4096, 2, 128, 256], [0, 2, 1, 3, 4],
                                              out=big_out), reps=10, warm=2)
    per_op.append({"op": "H2N 1x4096x256x256 -> 2x4096x128x256 (1 GiB)", "ms": ms,
                   "GB/s": big_bytes / ms / 1e6, "frac_hbm": big_bytes / ms / 1e6 / HBM_PEAK_GBS})
    del big_out
    halo_chain = [("split", 2, 128, 0, 1), ("reorder", [0, 2, 1, 3, 4]), ("fuse", 0, 0, 0)]
    halo_out = ops.trans_chain(big, halo_chain)
    halo_bytes = 4.0 * (big.numel() + halo_out.numel())
    ms = time_kernel(lambda: ops.trans_chain(big, halo_chain, out=halo_out), reps=10, warm=2)
    per_op.append({"op": "H2N with 1-row halo, same tensor", "ms": ms,
                   "GB/s": halo_bytes / ms / 1e6, "frac_hbm": halo_bytes / ms / 1e6 / HBM_PEAK_GBS})
    del halo_out
    # rows at odd dword alignment: zero-pad 126x126 planes to 128x128 and crop them back
    odd = big.reshape(-1)[:64 * 256 * 126 * 126].reshape(64, 256, 126, 126)
    padded = torch.empty((64, 256, 128, 128), device=dev)
    odd_bytes = 4.0 * (odd.numel() + padded.numel())
    ms = time_kernel(lambda: ops.pad(odd, [0, 0, 1, 1], [0, 0, 1, 1], out=padded), reps=10, warm=2)
    per_op.append({"op": "pad 64x256x126x126 -> 64x256x128x128", "ms": ms,
                   "GB/s": odd_bytes / ms / 1e6, "frac_hbm": odd_bytes / ms / 1e6 / HBM_PEAK_GBS})
    ms = time_kernel(lambda: ops.slice_(padded, [0, 0, 1, 1], [0, 0, 1, 1], out=odd), reps=10,
                     warm=2)
    per_op.append({"op": "slice 64x256x128x128 -> 64x256x126x126", "ms": ms,
                   "GB/s": odd_bytes / ms / 1e6, "frac_hbm": odd_bytes / ms / 1e6 / HBM_PEAK_GBS})
    del big, odd, padded

    # the other operator families of the library, one launch each at a representative size:
    # transposed convolution (the reference's perf-test shape, src/Test/transposeconv_test_1.cc,
    # and a generator layer), the band matmuls at a long-sequence shape (12 heads, 4096
    # tokens, window 2 x 256 + 1), the fused attention core at BERT-base's shape, and a
    # MemBound expression (the stride-2 gather in front of ResNet-18's 1x1 downsample)
    def family(name, fn, flop=None, nbytes=None, reps=20):
        try:
            ms = time_kernel(fn, reps=reps, warm=3)
        except Exception as exc:  # report, do not lose the main measurement
            per_op.append({"op": name, "error": str(exc)[:200]})
            return
        line = {"op": name, "ms": ms}
        if flop:
            line["TFLOP/s"] = flop / ms / 1e9
            line["frac_mfma"] = flop / ms / 1e9 / MFMA_FP32_PEAK_TFLOPS
        if nbytes:
            line["GB/s"] = nbytes / ms / 1e6
            line["frac_hbm"] = nbytes / ms / 1e6 / HBM_PEAK_GBS
        per_op.append(line)

    if not args.no_configs:
        for (n_, h_, f_, r_, c_, p_, s_) in ((1, 2, 448, 4, 256, 0, 1), (16, 16, 256, 4, 128, 1, 2)):
            xt = torch.randn((n_, h_, h_, f_), device=dev)
            wt = torch.randn((r_, r_, f_, c_), device=dev) * 0.05
            oh_ = ops.conv_trans_out_dim(h_, r_, p_, s_, 1, 0)
            yt = torch.empty((n_, oh_, oh_, c_), device=dev)
            family("conv_trans %dx%dx%dx%d, %dx%d filters -> %d, stride %d" % (n_, h_, h_, f_, r_, r_, c_, s_),
                   lambda: ops.conv_trans(xt, wt, p_, p_, s_, s_, out=yt),
                   flop=2.0 * n_ * h_ * h_ * f_ * r_ * r_ * c_,
                   nbytes=4.0 * (xt.numel() + wt.numel() + yt.numel()))
        for dil in (1, 4):
            qa = torch.randn((12, 4096, 64), device=dev)
            kb = torch.randn((12, 4096, 64), device=dev)
            band = torch.empty((12, 4096, 513), device=dev)
            family("g2bmm 12x4096x64, width 256, dilation %d" % dil,
                   lambda: ops.g2bmm(qa, kb, 256, dil, out=band),
                   flop=2.0 * 12 * 4096 * 513 * 64, nbytes=4.0 * (2 * qa.numel() + band.numel()))
            ctx = torch.empty((12, 4096, 64), device=dev)
            family("gbmml 12x4096x513 x 12x4096x64, dilation %d" % dil,
                   lambda: ops.gbmml(band, kb, dil, out=ctx),
                   flop=2.0 * 12 * 4096 * 513 * 64, nbytes=4.0 * (band.numel() + 2 * kb.numel()))
        qkv = torch.randn((3, 128, 768), device=dev)
        att = torch.empty((128, 768), device=dev)
        family("attention 12 heads x 128 x 64 (scores, softmax, context)",
               lambda: ops.attention(qkv[0], qkv[1], qkv[2], 12, 0.125, out=att),
               flop=2.0 * 2 * 12 * 128 * 128 * 64, nbytes=4.0 * 4 * 128 * 768)
        from pet_amd import expr_programs as ep
        gx = torch.randn((1, 128, 28, 28), device=dev)
        gy = torch.empty((1, 128, 196), device=dev)
        gather = ops.ExprProgram(ep.assemble(
            [(1, 128, 28, 28)],
            ep.R([("b", 0, 1), ("c", 0, 128), ("p", 0, 196)], [],
                 ep.T(0, [ep.C(0), ep.I("c"), (ep.I("p") // 14) * 2, (ep.I("p") % 14) * 2]))))
        family("membound: stride-2 gather 1x128x28x28 -> 1x128x196",
               lambda: ops.expr(gather, [gx], out=gy), nbytes=4.0 * 2 * gy.numel())

    # ---- the other configurations: batch-1 latency of the original network and of
    # its PET-transformed program, each replayed as one HIP graph
    other = {}
    if not args.no_configs:
        from pet_amd import programs
        specs = [("c1_conv_56x56", programs.run_c1, programs.params_c1(0), 0.2312),
                 ("c3_resnet18", programs.run_c3, programs.params_c3(0), 3.628),
                 ("c4_bert_base_seq128", programs.run_c4, programs.params_c4(0), 22.347),
                 ("c5_resnet3d18", programs.run_c5, programs.params_c5(0), 81.393)]
        for name, run, params, gflop in specs:
            entry = {"GFLOP": gflop}
            for label, transformed in (("original_ms", False), ("pet_ms", True)):
                try:
                    ns = programs.GpuNS(keep=True)
                    table = {}
                    with torch.cuda.stream(stream):
                        run(ns, params, transformed, T=table)  # uploads, weight-side ops
                        stream.synchronize()
                        ns.kept.clear()  # back to the allocator's pool for the captured run
                        abi.call("pet_hip_graph_begin_capture", sp)
                        try:
                            run(ns, params, transformed, T=table)
                        finally:
                            gh = ctypes.c_void_p(0)
                            abi.call("pet_hip_graph_end_capture", sp, ctypes.byref(gh))
                    reps = max(10, args.steps // 10)
                    entry[label] = time_graph(gh, reps, 3)
                    abi.call("pet_hip_graph_destroy", gh)
                    del ns, table
                except Exception as exc:  # report, do not lose the main measurement
                    entry[label] = None
                    entry[label + "_error"] = str(exc)[:200]
            if entry.get("pet_ms"):
                entry["pet_TFLOP/s"] = gflop / entry["pet_ms"]
            if name.startswith("c1"):
                # a graph of one 7 us kernel mostly measures the replay's own launch cost:
                # the same convolution launched on the stream, 50 in a row
                try:
                    ns, table = programs.GpuNS(keep=False), {}
                    with torch.cuda.stream(stream):
                        run(ns, params, False, T=table)
                    entry["original_stream_launch_ms"] = time_kernel(
                        lambda: run(ns, params, False, T=table))
                    del ns, table
                except Exception as exc:
                    entry["original_stream_launch_error"] = str(exc)[:200]
            other[name] = entry

    # ---- every distinct contraction of the other configurations by itself: 20 launches
    # captured into one graph (so that Python's call overhead stays out), replayed, with
    # the roofline it sits under: min(fp32 MFMA peak, arithmetic intensity x HBM peak)
    cfg_layers = []
    if not args.no_configs:
        def time_in_graph(fn, reps=20):
            with torch.cuda.stream(stream):
                for _ in range(3):
                    fn()
                stream.synchronize()
                abi.call("pet_hip_graph_begin_capture", sp)
                try:
                    for _ in range(reps):
                        fn()
                finally:
                    gh = ctypes.c_void_p(0)
                    abi.call("pet_hip_graph_end_capture", sp, ctypes.byref(gh))
            ms = time_graph(gh, 5, 2) / reps
            abi.call("pet_hip_graph_destroy", gh)
            return ms

        def layer_line(name, ms, flop, nbytes):
            tf = flop / ms / 1e9
            roof = min(MFMA_FP32_PEAK_TFLOPS, flop / nbytes * HBM_PEAK_GBS / 1e3)
            cfg_layers.append({"layer": name, "ms": ms, "TFLOP/s": tf, "GFLOP": flop / 1e9,
                           "roof_TFLOP/s": roof, "frac_roof": tf / roof})

        def conv2_layer(name, c, h, f, r, st, pad):
            lx = torch.randn((1, c, h, h), device=dev)
            lw = torch.randn((f, c, r, r), device=dev) * 0.05
            ly = ops.conv2d(lx, lw, pad, pad, st, st, act="relu")
            ms = time_in_graph(lambda: ops.conv2d(lx, lw, pad, pad, st, st, act="relu", out=ly))
            layer_line(name, ms, 2.0 * ly.numel() * c * r * r,
                       4.0 * (lx.numel() + lw.numel() + ly.numel()))

        def conv3_layer(name, c, t, h, f, k, st, pad):
            lx = torch.randn((1, c, t, h, h), device=dev)
            lw = torch.randn((f, c) + k, device=dev) * 0.05
            pk = ops.conv3d_pack_filters(lw) or lw
            ly = ops.conv3d(lx, pk, pad, st, act="relu")
            ms = time_in_graph(lambda: ops.conv3d(lx, pk, pad, st, act="relu", out=ly))
            layer_line(name, ms, 2.0 * ly.numel() * c * k[0] * k[1] * k[2],
                       4.0 * (lx.numel() + lw.numel() + ly.numel()))

        def mm_layer(name, b, m, n, k, tb=False):
            la = torch.randn((b, m, k), device=dev)
            lb = torch.randn((b, n, k) if tb else (b, k, n), device=dev)
            lc = ops.matmul(la, lb, False, tb)
            ms = time_in_graph(lambda: ops.matmul(la, lb, False, tb, out=lc))
            layer_line(name, ms, 2.0 * b * m * n * k, 4.0 * b * (m * k + k * n + m * n))

        try:
            conv2_layer("c1/c3 conv3x3 64->64 @56", 64, 56, 64, 3, 1, 1)
            conv2_layer("c3 stem 7x7/2 3->64 @224", 3, 224, 64, 7, 2, 3)
            for c, h, f, st in [(64, 56, 128, 2), (128, 28, 128, 1), (128, 28, 256, 2),
                                (256, 14, 256, 1), (256, 14, 512, 2), (512, 7, 512, 1)]:
                conv2_layer("c3 conv3x3/%d %d->%d @%d" % (st, c, f, h), c, h, f, 3, st, 1)
            for c, h, f in [(64, 56, 128), (128, 28, 256), (256, 14, 512)]:
                conv2_layer("c3 conv1x1/2 %d->%d @%d" % (c, f, h), c, h, f, 1, 2, 0)
            mm_layer("c3 fc 1x512x1000", 1, 1, 1000, 512)
            mm_layer("c4 qkv b3 128x768x768", 3, 128, 768, 768)
            mm_layer("c4 scores b12 128x128x64 (B transposed)", 12, 128, 128, 64, True)
            mm_layer("c4 probs x V b12 128x64x128", 12, 128, 64, 128)
            mm_layer("c4 out-proj 128x768x768", 1, 128, 768, 768)
            mm_layer("c4 ffn1 128x3072x768", 1, 128, 3072, 768)
            mm_layer("c4 ffn2 128x768x3072", 1, 128, 768, 3072)
            conv3_layer("c5 stem 3x7x7/(1,2,2) 3->64 @16x112", 3, 16, 112, 64, (3, 7, 7),
                        (1, 2, 2), (1, 3, 3))
            for c, t, h, f, st in [(64, 16, 56, 64, 1), (64, 16, 56, 128, 2), (128, 8, 28, 128, 1),
                                   (128, 8, 28, 256, 2), (256, 4, 14, 256, 1),
                                   (256, 4, 14, 512, 2), (512, 2, 7, 512, 1)]:
                conv3_layer("c5 conv3x3x3/%d %d->%d @%dx%d" % (st, c, f, t, h), c, t, h, f,
                            (3, 3, 3), (st, st, st), (1, 1, 1))
            for c, t, h, f in [(64, 16, 56, 128), (128, 8, 28, 256), (256, 4, 14, 512)]:
                conv3_layer("c5 conv1x1x1/2 %d->%d @%dx%d" % (c, f, t, h), c, t, h, f, (1, 1, 1),
                            (2, 2, 2), (0, 0, 0))
        except Exception as exc:  # report, do not lose the main measurement
            cfg_layers.append({"error": str(exc)[:200]})

    # ---- the same networks through the C++ host layer (tpm::Graph -> SubGraph ->
    # CodeEngine::instantiate -> HIP graph replay), the path a PET user takes
    host_path = {}
    run_model = os.path.join(ROOT, "pet_amd", "lib", "pet_run_model")
    if not args.no_configs and os.path.exists(run_model):
        import subprocess
        torch.cuda.synchronize()
        # plain, and with --tune: Operator::perf on every operator first, so that each
        # contraction runs with the algorithm that timed fastest for it (what PET's search
        # leaves in its PerfEngine)
        for model in ("dilated:pet", "dilated", "resnet18", "resnet18:pet", "bert", "bert:pet",
                      "resnet3d18"):
            for key, extra in ((model, []), (model + " tuned", ["--tune"])):
                try:
                    res = subprocess.run([run_model, model, "--rounds", str(max(50, args.steps)),
                                          "--warmup", "10"] + extra, capture_output=True,
                                         text=True, timeout=300)
                    host_path[key] = (json.loads(res.stdout.strip().splitlines()[-1])
                                      if res.returncode == 0 else {"error": res.stderr[-200:]})
                except Exception as exc:
                    host_path[key] = {"error": str(exc)[:200]}

        # beside each configuration's plain call-by-call program: the same original network
        # as the graph runtime launches it (aliases, folded tails, hoisted initialisations,
        # fused attention)
        for name, model in (("c3_resnet18", "resnet18"), ("c4_bert_base_seq128", "bert"),
                            ("c5_resnet3d18", "resnet3d18")):
            got = host_path.get(model, {})
            if name in other and "ms" in got:
                other[name]["graph_runtime_ms"] = got["ms"]
                other[name]["graph_runtime_kernels"] = got.get("kernels")
            pet = host_path.get(model + ":pet", {})
            if name in other and "ms" in pet:
                other[name]["graph_runtime_pet_ms"] = pet["ms"]
                other[name]["graph_runtime_pet_kernels"] = pet.get("kernels")

    dom_flop = conv_flop(DIL * DIL, 512, hs, hs, 512, 3, 3)
    dom_ms = conv_ms[0]
    achieved = dom_flop / dom_ms / 1e9
    roofline = {"bound": "mfma", "kernel": "conv_plane_kernel<64x64, RS=9, CB=8> (512->512, 4x32x32, 3x3, ReLU)",
                "achieved": achieved, "peak": MFMA_FP32_PEAK_TFLOPS, "unit": "TFLOP/s",
                "frac": achieved / MFMA_FP32_PEAK_TFLOPS,
                "traffic": dominant_traffic_bytes(), "traffic_unit": "bytes per launch",
                "traffic_source": "profiles/" + os.path.basename(DOMINANT_PROFILE),
                "flop_per_launch": dom_flop, "avg_launch_ms": dom_ms}

    total_flop = sum(conv_flop(1, CHANNELS[i + 1], HW, HW, CHANNELS[i], 3, 3) for i in range(6))

    # ---- CPU baseline: the oracle's conv loop nest on the original (dilated) program
    cpu = None
    if not args.no_cpu:
        import oracle
        xs = [x.cpu().numpy()] + [t.cpu().numpy() for t in o_act[:-1]]
        wn = [w.cpu().numpy() for w in ws]
        spent, done_flop, layers = 0.0, 0.0, []
        for i in reversed(range(6)):  # cheapest layers first
            fl = conv_flop(1, CHANNELS[i + 1], HW, HW, CHANNELS[i], 3, 3)
            if layers and spent > 0 and spent + fl * (spent / done_flop) > args.cpu_seconds:
                break
            t0 = time.perf_counter()
            y = oracle.conv2d(xs[i], wn[i], DIL, DIL, 1, 1, DIL, DIL)
            oracle.activation(y, "relu")
            spent += time.perf_counter() - t0
            done_flop += fl
            layers.append(i + 1)
        cpu = {"value": spent * 1e3 * total_flop / done_flop, "unit": "ms",
               "cores": oracle.num_threads(), "kind": "port",
               "sample": "oracle conv+ReLU on layers %s of the original dilated block "
                         "(%.2f of %.2f GFLOP, %.1f s measured), scaled to the whole block by FLOP"
                         % (sorted(layers), done_flop / 1e9, total_flop / 1e9, spent),
               "measured_s": spent, "GFLOP/s": done_flop / spent / 1e9}

    out = {
        "metric": "batch-1 e2e latency ms per PET-optimized graph",
        "value": ms_opt,
        "unit": "ms",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": ms_opt,
        "higher_is_better": False,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f32",
        "data": "synthetic",
        "config": {"workload": "dilated-conv block (CSRNet back-end), six 3x3 convs "
                               "512-512-512-512-256-128-64 on 1x512x64x64, PET space-to-batch "
                               "program (4x32x32 dense convs + fused ReLU, launches planned "
                               "as the graph runtime plans them%s) as one HIP graph"
                               % (", the two layout operators as the addressing of the first "
                                  "and last convolution" if folded else ""),
                   "global_batch": 1},
        "value_is": "median of %d blocks of %d launches" % (REPEATS, args.steps),
        "block_ms_min": blocks[0],
        "block_ms_max": blocks[-1],
        "planned_launches": {"layout_operators_folded": bool(folded),
                             "accumulating_convs": [i + 1 for i in range(6) if accum[i]],
                             "batched_initialisations": len(fills)},
        "original_graph_ms": ms_org,
        "e2e_TFLOP/s": total_flop / ms_opt / 1e9,
        "e2e_frac_mfma": total_flop / ms_opt / 1e9 / MFMA_FP32_PEAK_TFLOPS,
        "roofline": roofline,
        "cpu_baseline": cpu,
        "per_op": per_op,
        "configs": other,
        "config_layers": cfg_layers,
        "host_layer_graphs": host_path,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
