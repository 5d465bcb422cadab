#!/usr/bin/env python3
"""Benchmark of the hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A step is one pass of the hot path over configuration c3 of BASELINE.json:
activation reorder-quantize (bf16 [4096, 4096] -> packed MXFP4/6/8 + E8M0
scales) followed by the mixed GEMM against MXFP4 weights [14336, 4096] into bf16
[4096, 14336], with every input already resident in HBM and the weights quantized
once outside the timed region (as bench_reorder_gemm.cu:163-167 of the reference
does).  Prints ONE JSON line.  `roofline` describes the dominant kernel (the mixed
GEMM, MFMA-bound); `extra` carries the memory-bound configurations c1 (reorder-
quantize alone) and c2 (decode GEMM) with their own rooflines; `cpu_baseline` is
the oracle's fake-quant + fp32 matmul timed on the host cores over a bounded
sample of the same workload.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0
# dense MFMA peaks, TFLOP/s: an E4M3 operand halves the f8f6f4 rate
P46, P8 = 10100.0, 5000.0


# HBM bytes per launch measured with rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, each scaled by the same
# counter's reading for `bench.py --calibrate-copy`.  These are figures of an earlier profiling run, not of
# this one: each entry names the summary under profiles/ it comes from and the SHA-256 (first 16 hex digits)
# of the kernel source it was taken with; when the source has changed since, the JSON carries null and says so.
PROFILE = "profiles/hbm_traffic_fetch_write_size.txt"
MEASURED_TRAFFIC = {
    "gemm_c3": {"bytes": int((110300.3 * 1.99981 + 114703.1 * 1.0) * 1024),      # 343 MB against 159 MB algorithmic: operands re-read 5.5x past L2
                "source": "mixedgemm_amd/csrc/mixed_gemm_256.hip", "sha": "edd444588cd9c90b"},
    "quant_c1": {"bytes": int((16465.5 * 1.99981 + 10522.4 * 1.0) * 1024),       # 44.5 MB against 44.2 MB algorithmic
                 "source": "mixedgemm_amd/csrc/reorder_quant.hip", "sha": "76e172a1ba32b3ef"},
    "quant_w_c3": {"bytes": int((57430.5 * 1.99981 + 30855.0 * 1.0) * 1024),     # 149.2 MB against 148.6 MB algorithmic
                   "source": "mixedgemm_amd/csrc/reorder_quant.hip", "sha": "76e172a1ba32b3ef"},
    "tile_w_c3": {"bytes": int((14412.5 * 1.99981 + 28672.0 * 1.0) * 1024),      # 58.9 MB against 58.7 MB (three launches)
                  "source": "mixedgemm_amd/csrc/mixed_gemm_256.hip", "sha": "edd444588cd9c90b"},
    "decode_c2": {"bytes": int((15429.0 * 1.99981 + 224.0 * 1.0) * 1024),        # 31.8 MB against 31.4 MB algorithmic (tile-major weights)
                  "source": "mixedgemm_amd/csrc/mixed_gemm.hip", "sha": "8acb521f32f6708a"},
    "calibrate_c1": {"bytes": int(((16422.5 + 286.5) * 1.99981 + (64.0 + 56.2) * 1.0) * 1024),   # two kernels: 34.3 MB against 33.6 MB
                     "source": "mixedgemm_amd/csrc/calibrate.hip", "sha": "6b06f434b6263d8d"},
}


def source_sha(rel):
    import hashlib
    with open(os.path.join(ROOT, rel), "rb") as f:
        return hashlib.sha256(f.read()).hexdigest()[:16]


def traffic(key):
    """(bytes or None, provenance string) of a kernel's profiled HBM traffic."""
    e = MEASURED_TRAFFIC[key]
    now = source_sha(e["source"])
    if now != e["sha"]:
        return None, f"not re-profiled since {e['source']} changed (figure in {PROFILE} was taken at source sha256 {e['sha']}, now {now})"
    return e["bytes"], f"rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE figure from {PROFILE}, taken at {e['source']} sha256 {e['sha']} (unchanged since); not measured by this run"


def bench_lib():
    """The measurement kernels (libmixedgemm_bench.so): MFMA register loop, streaming copy, empty launch."""
    import ctypes
    path = os.path.join(ROOT, "mixedgemm_amd", "lib", "libmixedgemm_bench.so")
    L = ctypes.CDLL(path)
    p, i, z = ctypes.c_void_p, ctypes.c_int, ctypes.c_size_t
    L.mgb_measure_mfma_ceiling.restype = i
    L.mgb_measure_mfma_ceiling.argtypes = [i, i, ctypes.POINTER(ctypes.c_double), ctypes.POINTER(ctypes.c_double)]
    L.mgb_stream.restype, L.mgb_stream.argtypes = i, [p, z, p, z, i, p]
    L.mgb_empty_launch.restype, L.mgb_empty_launch.argtypes = i, [i, i, p]
    return L


def measure_mfma_ceiling(L, random_operands, iters=4000):
    import ctypes
    tf, ghz = ctypes.c_double(0.0), ctypes.c_double(0.0)
    rc = L.mgb_measure_mfma_ceiling(int(bool(random_operands)), iters, ctypes.byref(tf), ctypes.byref(ghz))
    assert rc == 0, f"mgb_measure_mfma_ceiling: {rc}"
    return tf.value, ghz.value


def blended_peak(kn, ks, ko):
    return (kn + ks + ko) / ((kn + ks) / P46 + ko / P8)


def quant_bytes(m, k, kn, ks, ko):
    """Algorithmic bytes of one activation reorder-quantize launch."""
    return m * (2 * k + kn // 2 + 3 * ks // 4 + ko + k // 32) + 2 * k


def gemm_bytes(m, n, kn, ks, ko):
    k = kn + ks + ko
    return n * k // 2 + n * k // 32 + m * (kn // 2 + 3 * ks // 4 + ko) + m * k // 32 + m * n * 2


def weight_quant_bytes(n, k):
    """Algorithmic bytes of one weight reorder-quantize launch: bf16 rows in, E2M1 codes and E8M0 scales out, the index once."""
    return n * (2 * k + k // 2 + k // 32) + 2 * k


def event_ms(pairs):
    return sum(a.elapsed_time(b) for a, b in pairs) / len(pairs)


GRAPH_WARM_S = 0.15   # untimed replays in front of a graph measurement (0 with --no-clock-warmup)


def graph_ms(launch, iters, warmup=3, repeats=5, warm_s=None):
    """Time of one launch when `iters` back-to-back launches (launch(i), i = 0..iters-1, no
    allocation inside) are replayed as one HIP graph: the host's per-call cost (10-15 us through ctypes)
    is out of the measurement, which a 10 us kernel needs.  The graph is first replayed untimed for
    GRAPH_WARM_S seconds (after the host-side set-up of a leg the GPU has idled and runs the first
    milliseconds at other clocks, as the headline's warm-up steps account for); then the median over
    `repeats` timed replays.  warm_s = 0 for legs that alternate two graphs back to back on a GPU that is busy anyway."""
    import time
    import torch
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    g = torch.cuda.CUDAGraph()
    with torch.cuda.stream(side):
        for i in range(warmup):
            launch(i)
        side.synchronize()
        with torch.cuda.graph(g, stream=side):
            for i in range(iters):
                launch(i)
    torch.cuda.synchronize()
    g.replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    while time.perf_counter() - t0 < (GRAPH_WARM_S if warm_s is None else warm_s):
        for _ in range(4):
            g.replay()
        torch.cuda.synchronize()
    times = []
    for _ in range(repeats):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        times.append(e0.elapsed_time(e1))
    del g
    return sorted(times)[len(times) // 2] / iters


def main():
    global GRAPH_WARM_S
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-extra", action="store_true")
    ap.add_argument("--no-zero-operand-leg", action="store_true",
                    help="skip the c3 launches on all-zero operand codes (same kernel and grid as c3: in a kernel trace "
                         "they would be averaged into c3's row)")
    ap.add_argument("--no-clock-warmup", action="store_true",
                    help="skip the 0.4 s of untimed steps in front (for counter runs, where every launch is slow)")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="only run a plain device copy of known size (256 MiB read + 256 MiB written per launch): "
                         "the reference point for scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import numpy as np
    import torch

    from mixedgemm_amd import abi
    from tests import helpers as H

    abi.lib()
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.calibrate_copy:
        src = torch.full((64 << 20,), 3, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            dst.copy_(src)
        torch.cuda.synchronize()
        print(json.dumps({"calibration": "torch copy_ int32", "bytes_read": src.numel() * 4, "bytes_written": dst.numel() * 4,
                          "launches": 5}))
        return

    # ---------------------------------------------------------------- c3
    m, n, k, kn, ks, ko = H.CONFIGS["c3"]
    x = H.make_activations(m, k, 1234 + 3)
    w = H.make_weights(n, k, 2234 + 3)
    idx = H.absmax_sort_index(x)
    xd, wd, idd = x.to(dev), w.to(dev), idx.to(dev)
    # weights: quantized and put in tile-major order once, outside the timed region (the offline pack)
    bq = abi.reorder_quantize_w(wd, idd, kn, ks, ko)
    bt = abi.tile_weights(*bq[:3])
    aq = abi.alloc_quant_outputs(m, kn, ks, ko, abi.MG_OPERAND_A, dev)
    d = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
    ws = torch.empty(abi.fused_workspace_bytes(m, kn, ks, ko), dtype=torch.uint8, device=dev)
    torch.cuda.synchronize()

    # The step: ONE call of mg_fused_linear_ex (reorder-quantize into the preallocated workspace, then the
    # GEMM, on torch's current stream), arguments converted once.
    import ctypes
    L = abi.lib()
    vp = lambda t: ctypes.c_void_p(t.data_ptr())
    stream = ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)
    fused_args = (vp(xd), vp(idd), vp(bt[0]), vp(bt[1]), vp(bt[2]), vp(bq[3]), vp(bq[4]), vp(bq[5]), m, n, kn, ks, ko,
                  abi.MG_FLAG_W_TILED, vp(d), vp(ws), ctypes.c_size_t(ws.numel()), stream)

    def step():
        rc = L.mg_fused_linear_ex(*fused_args)
        if rc:
            abi.check(rc, "mg_fused_linear_ex")

    def quant_then_gemm(pair):
        """The same two kernels through the two separate entry points, with an event pair around the GEMM."""
        abi.reorder_quantize_x(xd, idd, kn, ks, ko, out=aq)
        pair[0].record()
        abi.matmul(aq[0], bt[0], aq[1], bt[1], aq[2], bt[2], aq[3], bq[3], aq[4], bq[4], aq[5], bq[5], out=d, w_tiled=True)
        pair[1].record()

    # Clock warm-up by time, whatever --warmup says: the first ~10 ms after an idle period run at other clocks
    # than the steady state, and the counted warm-up may be a handful of steps.
    t_warm = time.perf_counter()
    warm_steps = 0
    if args.no_clock_warmup:
        GRAPH_WARM_S = 0.0
    while time.perf_counter() - t_warm < (0.0 if args.no_clock_warmup else 0.4):
        for _ in range(20):
            step()
        torch.cuda.synchronize()
        warm_steps += 20
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()

    # Timed region: exactly --steps steps between two synchronizes.  Up to five event marks split it into
    # sub-loops whose median is reported next to the whole region's mean.
    nsub = min(5, args.steps)
    bounds = [round(i * args.steps / nsub) for i in range(nsub + 1)]
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(nsub + 1)]
    t0 = time.perf_counter()
    for j in range(nsub):
        marks[j].record()
        for _ in range(bounds[j], bounds[j + 1]):
            step()
    marks[nsub].record()
    torch.cuda.synchronize()
    t1 = time.perf_counter()
    ms_per_step = (t1 - t0) * 1e3 / args.steps
    sub_ms = sorted(marks[j].elapsed_time(marks[j + 1]) / (bounds[j + 1] - bounds[j]) for j in range(nsub))
    flops = 2.0 * m * n * k
    value = flops / (ms_per_step * 1e-3) / 1e12

    # The GEMM kernel, timed with events on the launch stream: five sub-loops of back-to-back GEMM launches (the
    # launch mg_fused_linear_ex makes, on the workspace the step just filled), one event pair around each
    # sub-loop, the median of the sub-loop means.  (An event pair around every single launch inside the step
    # adds about 5 us to a 140 us kernel: that figure is reported next to this one.)
    per_sub = max(4, (max(args.steps, 20) + 4) // 5)
    aq_ws = abi.alloc_quant_outputs(m, kn, ks, ko, abi.MG_OPERAND_A, dev)
    abi.reorder_quantize_x(xd, idd, kn, ks, ko, out=aq_ws)

    def gemm_only():
        abi.matmul(aq_ws[0], bt[0], aq_ws[1], bt[1], aq_ws[2], bt[2], aq_ws[3], bq[3], aq_ws[4], bq[4], aq_ws[5], bq[5],
                   out=d, w_tiled=True)

    for _ in range(per_sub):
        gemm_only()
    torch.cuda.synchronize()
    sub_gemm = []
    for _ in range(5):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(per_sub):
            gemm_only()
        e1.record()
        torch.cuda.synchronize()
        sub_gemm.append(e0.elapsed_time(e1) / per_sub)
    gemm_ms = sorted(sub_gemm)[2]
    in_step = []
    for _ in range(3):
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(per_sub)]
        for pair in ev:
            quant_then_gemm(pair)
        torch.cuda.synchronize()
        in_step.append(event_ms(ev))
    peak = blended_peak(kn, ks, ko)
    gemm_tflops = flops / (gemm_ms * 1e-3) / 1e12
    t_bytes, t_note = traffic("gemm_c3")
    roofline = {
        "kernel": "mixed GEMM (c3)", "bound": "mfma", "achieved": round(gemm_tflops, 2), "peak": round(peak, 1),
        "unit": "TFLOP/s", "frac": round(gemm_tflops / peak, 4), "traffic": t_bytes, "traffic_source": t_note,
        "avg_kernel_ms": round(gemm_ms, 4), "algorithmic_flops": flops,
        "protocol": f"clock warm-up {warm_steps} steps (>= 0.4 s), the timed steps, then 5 sub-loops of {per_sub} back-to-back "
                    "GEMM launches with one event pair around each sub-loop on the launch stream; median of the sub-loop means",
        "sub_loop_ms": [round(v, 4) for v in sub_gemm],
        "event_pair_around_each_gemm_inside_the_step_ms": round(sorted(in_step)[1], 4),
    }

    extra = {}
    if not args.no_extra:
        BL = bench_lib()
        # ------------------------------------------------------------ c3 GEMM with the weights as reorder_quantize_w leaves them
        rm, tl = [], []
        for it in range(5):   # alternate: the chip's clock drifts with load, medians of interleaved runs compare fairly
            rm.append(graph_ms(lambda i: abi.matmul(aq[0], bq[0], aq[1], bq[1], aq[2], bq[2], aq[3], bq[3], aq[4], bq[4],
                                                    aq[5], bq[5], out=d), 20, repeats=2, warm_s=None if it == 0 else 0.0))
            tl.append(graph_ms(lambda i: abi.matmul(aq[0], bt[0], aq[1], bt[1], aq[2], bt[2], aq[3], bq[3], aq[4], bq[4],
                                                    aq[5], bq[5], out=d, w_tiled=True), 20, repeats=2, warm_s=0.0))
        rm_ms, tl_ms = sorted(rm)[2], sorted(tl)[2]
        extra["gemm_c3_weight_layouts"] = {
            "note": "c3 GEMM alone, 20 launches replayed as a HIP graph (no host launch gaps), median of 5 interleaved runs",
            "row_major_runs_ms": [round(v, 5) for v in rm], "tile_major_runs_ms": [round(v, 5) for v in tl],
            "row_major_ms": round(rm_ms, 5), "row_major_tflops": round(flops / (rm_ms * 1e-3) / 1e12, 1),
            "tile_major_ms": round(tl_ms, 5), "tile_major_tflops": round(flops / (tl_ms * 1e-3) / 1e12, 1)}
        # ------------------------------------------------------------ the same launch on all-zero operands: same
        # instructions, addresses and bytes moved, but the multiplier arrays do not toggle -- separates what the
        # kernel's structure costs from what the chip's power limit costs on real operand bits
        if not args.no_zero_operand_leg:
            zq = abi.reorder_quantize_x(torch.zeros_like(xd), idd, kn, ks, ko)
            zw = abi.reorder_quantize_w(torch.zeros_like(wd), idd, kn, ks, ko)
            zb = abi.tile_weights(*zw[:3])
            zr, rr = [], []
            for _ in range(5):   # straight after the leg above: the GPU has not idled
                zr.append(graph_ms(lambda i: abi.matmul(zq[0], zb[0], zq[1], zb[1], zq[2], zb[2], zq[3], zw[3], zq[4], zw[4],
                                                        zq[5], zw[5], out=d, w_tiled=True), 20, repeats=2, warm_s=0.0))
                rr.append(graph_ms(lambda i: abi.matmul(aq[0], bt[0], aq[1], bt[1], aq[2], bt[2], aq[3], bq[3], aq[4], bq[4],
                                                        aq[5], bq[5], out=d, w_tiled=True), 20, repeats=2, warm_s=0.0))
            z_ms, r_ms = sorted(zr)[2], sorted(rr)[2]
            extra["gemm_c3_zero_operands"] = {
                "note": "c3 GEMM launch with all-zero operand codes against the bench operands, medians of 5 interleaved runs of 20 launches",
                "zero_ms": round(z_ms, 5), "zero_tflops": round(flops / (z_ms * 1e-3) / 1e12, 1),
                "bench_operands_ms": round(r_ms, 5), "bench_operands_tflops": round(flops / (r_ms * 1e-3) / 1e12, 1)}
            del zq, zw, zb
        # ------------------------------------------------------------ the weight side of the reorder-quantize kernel
        # (run_reorder_bf16_fp4, timed by bench_reorder.cu:143-166 of the reference next to the activation side):
        # c3's W[14336, 4096] -> three E2M1 segments + scales, then the tile-major rewrite of the codes; offline work
        # in deployment, so outside the headline's step.  Three rotating W (352 MB) and five rotating code sets
        # (5 x 2 x 29.4 MB) keep the bytes out of the 256 MB Infinity Cache.
        wsets = [wd] + [H.make_weights(n, k, 2300 + i).to(dev) for i in range(2)]
        wouts = [abi.alloc_quant_outputs(n, kn, ks, ko, abi.MG_OPERAND_B, dev) for _ in range(3)]
        for i in range(3):
            abi.reorder_quantize_w(wsets[i], idd, kn, ks, ko, out=wouts[i])
        torch.cuda.synchronize()
        wq_ms = graph_ms(lambda i: abi.reorder_quantize_w(wsets[i % 3], idd, kn, ks, ko, out=wouts[i % 3]), 12)
        wqb = weight_quant_bytes(n, k)
        extra["reorder_quant_w_c3"] = {
            "workload": "weight reorder-quantize of c3's W[14336, 4096] (all E2M1, segments 2560/1408/128), 3 rotating inputs, "
                        "12 launches replayed as a HIP graph",
            "value": round(wqb / (wq_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "avg_kernel_ms": round(wq_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(wqb / (wq_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(wqb / (wq_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": traffic("quant_w_c3")[0],
                         "traffic_source": traffic("quant_w_c3")[1], "algorithmic_bytes": wqb}}
        del wsets
        csets = [tuple(t.clone() for t in bq[:3]) for _ in range(5)]
        tsets = [tuple(torch.empty_like(t) for t in bq[:3]) for _ in range(5)]

        def tile(i):
            for src, dst in zip(csets[i % 5], tsets[i % 5]):
                abi.check(L.mg_tile_weights(vp(src), vp(dst), src.shape[0], src.shape[1] * 2,
                                            ctypes.c_void_p(torch.cuda.current_stream(dev).cuda_stream)), "mg_tile_weights")

        tw_ms = graph_ms(tile, 20)
        twb = 2 * sum(t.numel() for t in bq[:3])
        extra["tile_weights_c3"] = {
            "workload": "tile-major rewrite of c3's weight codes (three launches, one per segment: 29.4 MB read + 29.4 MB written), "
                        "5 rotating sets, 20 calls replayed as a HIP graph",
            "value": round(twb / (tw_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "avg_ms": round(tw_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(twb / (tw_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(twb / (tw_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": traffic("tile_w_c3")[0],
                         "traffic_source": traffic("tile_w_c3")[1], "algorithmic_bytes": twb}}
        del csets, tsets, wouts
        # ------------------------------------------------------------ c1: reorder-quantize alone, HBM-bound
        m1, _, k1, kn1, ks1, ko1 = H.CONFIGS["c1"]
        nsets = 8                                    # 8 x 44 MB > 256 MB Infinity Cache
        idx1 = H.random_index(k1, 4321).to(dev)
        base = H.make_activations(m1, k1, 1234 + 1).to(dev)
        xs = [base.clone() for _ in range(nsets)]
        outs = [abi.alloc_quant_outputs(m1, kn1, ks1, ko1, abi.MG_OPERAND_A, dev) for _ in range(nsets)]
        iters = max(args.steps, 80)
        for i in range(args.warmup + nsets):
            abi.reorder_quantize_x(xs[i % nsets], idx1, kn1, ks1, ko1, out=outs[i % nsets])
        torch.cuda.synchronize()
        q_ms = graph_ms(lambda i: abi.reorder_quantize_x(xs[i % nsets], idx1, kn1, ks1, ko1, out=outs[i % nsets]), iters)
        qb = quant_bytes(m1, k1, kn1, ks1, ko1)
        q_gbs = qb / (q_ms * 1e-3) / 1e9
        extra["reorder_quant_c1"] = {
            "workload": "c1 reorder-quantize M=4096 K=4096 (2560/1408/128), random-permutation index, 8 rotating buffer sets, 80 launches replayed as a HIP graph",
            "value": round(q_gbs, 1), "unit": "GB/s", "avg_kernel_ms": round(q_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(q_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(q_gbs / HBM_PEAK_GBS, 4), "traffic": traffic("quant_c1")[0], "traffic_source": traffic("quant_c1")[1],
                         "algorithmic_bytes": qb},
        }
        # ------------------------------------------------------------ what a plain streaming kernel reaches on c1's bytes
        # reads the same 33.6 MB per launch from the same rotating inputs and writes 10.6 MB into the same
        # rotating outputs (one launch of 2048 workgroups of 256, 16 bytes per lane and access), and an empty
        # launch of the quantizer's grid: the two figures the c1 fraction is to be read against
        rb, wb = m1 * k1 * 2, (qb - m1 * k1 * 2 - 2 * k1) // 16 * 16
        st = ctypes.c_void_p(0)

        def stream_copy(i):
            st.value = torch.cuda.current_stream(dev).cuda_stream
            rc = BL.mgb_stream(vp(xs[i % nsets]), rb, vp(outs[i % nsets][0]), min(wb, outs[i % nsets][0].numel() // 16 * 16), 2048, st)
            assert rc == 0

        def empty(i):
            st.value = torch.cuda.current_stream(dev).cuda_stream
            assert BL.mgb_empty_launch(1024, 128, st) == 0

        s_ms = graph_ms(stream_copy, iters)
        e_ms = graph_ms(empty, iters)
        wrote = min(wb, outs[0][0].numel() // 16 * 16)
        extra["reorder_quant_c1"]["streaming_reference"] = {
            "note": "plain streaming kernel on c1's input bytes (same rotation, same graph replay): reads X once, writes "
                    f"{wrote} bytes; and an empty launch of 1024 workgroups x 128 lanes (the quantizer's launch shape)",
            "stream_ms": round(s_ms, 5), "stream_gbs": round((rb + wrote) / (s_ms * 1e-3) / 1e9, 1),
            "empty_launch_ms": round(e_ms, 5)}
        # ------------------------------------------------------------ c1 with an RMSNorm fused into the row pass
        gamma1 = torch.ones(k1, dtype=torch.bfloat16, device=dev)
        n_ms = graph_ms(lambda i: abi.rmsnorm_reorder_quantize_x(xs[i % nsets], gamma1, 1e-5, idx1, kn1, ks1, ko1,
                                                                 out=outs[i % nsets]), iters)
        extra["rmsnorm_reorder_quant_c1"] = {
            "workload": "c1 with an RMSNorm in front, same pass (a separate RMSNorm kernel would read and write X once more)",
            "value": round((qb + 2 * k1) / (n_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "avg_kernel_ms": round(n_ms, 5)}
        # ------------------------------------------------------------ calibration: column absmax + sort (reads X once)
        wsp = torch.empty(int(abi.lib().mg_calibrate_workspace_bytes(k1)), dtype=torch.uint8, device=dev)
        idx_out = torch.empty(k1, dtype=torch.int16, device=dev)
        for i in range(args.warmup):
            abi.calibrate_reorder_index(xs[i % nsets], out=idx_out, workspace=wsp)
        torch.cuda.synchronize()
        c_ms = graph_ms(lambda i: abi.calibrate_reorder_index(xs[i % nsets], out=idx_out, workspace=wsp), iters)
        cb = m1 * k1 * 2 + k1 * 2
        extra["calibrate_index_c1"] = {
            "workload": "reorder index of the c1 activations: per-channel absmax over M=4096 rows + sort of K=4096 channels",
            "value": round(cb / (c_ms * 1e-3) / 1e9, 1), "unit": "GB/s", "avg_ms": round(c_ms, 5),
            "roofline": {"bound": "hbm", "achieved": round(cb / (c_ms * 1e-3) / 1e9, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(cb / (c_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4), "traffic": traffic("calibrate_c1")[0], "traffic_source": traffic("calibrate_c1")[1],
                         "algorithmic_bytes": cb},
        }
        del xs, outs, base

        # ------------------------------------------------------------ c2: decode GEMM, HBM-bound
        m2, n2, k2, kn2, ks2, ko2 = H.CONFIGS["c2"]
        x2 = H.make_activations(m2, k2, 1234 + 2)
        idx2 = H.absmax_sort_index(x2).to(dev)
        aq2 = abi.reorder_quantize_x(x2.to(dev), idx2, kn2, ks2, ko2)
        nsets2 = 10                                  # 10 x 31 MB of weights > 256 MB
        wq_rm = [abi.reorder_quantize_w(H.make_weights(n2, k2, 3000 + i).to(dev), idx2, kn2, ks2, ko2) for i in range(nsets2)]
        # tile-major codes: the layout the packed weights of a layer are stored in (as in the headline's step)
        wq = [abi.tile_weights(*b[:3]) + b[3:] for b in wq_rm]
        d2 = torch.empty((m2, n2), dtype=torch.bfloat16, device=dev)

        def decode(i):
            b = wq[i % nsets2]
            abi.matmul(aq2[0], b[0], aq2[1], b[1], aq2[2], b[2], aq2[3], b[3], aq2[4], b[4], aq2[5], b[5], out=d2, w_tiled=True)

        def decode_rm(i):
            b = wq_rm[i % nsets2]
            abi.matmul(aq2[0], b[0], aq2[1], b[1], aq2[2], b[2], aq2[3], b[3], aq2[4], b[4], aq2[5], b[5], out=d2)

        for i in range(args.warmup + nsets2):
            decode(i)
            decode_rm(i)
        torch.cuda.synchronize()
        g_rm_ms = graph_ms(decode_rm, iters)
        g_ms = graph_ms(decode, iters)
        gb = gemm_bytes(m2, n2, kn2, ks2, ko2)
        g_gbs = gb / (g_ms * 1e-3) / 1e9
        extra["decode_gemm_c2"] = {
            "workload": "c2 mixed GEMM M=8 K=4096 (2560/1408/128) N=14336, tile-major weight codes, 10 rotating weight sets",
            "value": round(g_gbs, 1), "unit": "GB/s", "avg_kernel_ms": round(g_ms, 5), "row_major_weights_ms": round(g_rm_ms, 5),
            "tflops": round(2.0 * m2 * n2 * k2 / (g_ms * 1e-3) / 1e12, 3),
            "roofline": {"bound": "hbm", "achieved": round(g_gbs, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                         "frac": round(g_gbs / HBM_PEAK_GBS, 4), "traffic": traffic("decode_c2")[0], "traffic_source": traffic("decode_c2")[1],
                         "algorithmic_bytes": gb},
        }
        del wq, wq_rm

        # ------------------------------------------------------------ the other layer shapes of the reference's K list
        # fused step (activation reorder-quantize + mixed GEMM) per shape; weights quantized outside the timing
        from mixedgemm_amd import linear as caller
        matrix = []
        shapes = [("c0", 128, 4096, 4096), ("c4", 2048, 4096, 14336), ("reference bench_gemm.cu:23-27", 1024, 4096, 4096),
                  ("", 4096, 13824, 5120), ("", 4096, 5120, 13824),
                  ("", 4096, 18944, 3584), ("", 4096, 3584, 18944), ("", 4096, 4096, 12288)]
        for tag, mm, nn, kk in shapes:
            knm, ksm, kom = caller.default_split(kk)
            xm = H.make_activations(mm, kk, 1234 + 4, student_t=(tag == "c4")).to(dev)
            idm = abi.calibrate_reorder_index(xm)
            wqm = abi.reorder_quantize_w(H.make_weights(nn, kk, 2234 + 4).to(dev), idm, knm, ksm, kom)
            tiled = abi.weights_tileable(nn, knm, ksm, kom)
            if tiled:
                wqm = abi.tile_weights(*wqm[:3]) + wqm[3:]
            aqm = abi.alloc_quant_outputs(mm, knm, ksm, kom, abi.MG_OPERAND_A, dev)
            dm = torch.empty((mm, nn), dtype=torch.bfloat16, device=dev)

            def quant():
                abi.reorder_quantize_x(xm, idm, knm, ksm, kom, out=aqm)

            def gemm():
                abi.matmul(aqm[0], wqm[0], aqm[1], wqm[1], aqm[2], wqm[2], aqm[3], wqm[3], aqm[4], wqm[4], aqm[5], wqm[5], out=dm,
                           w_tiled=tiled)

            times = [graph_ms(lambda i: quant(), 20), graph_ms(lambda i: gemm(), 20)]
            flops = 2.0 * mm * nn * kk
            matrix.append({"config": tag, "M": mm, "N": nn, "K": kk, "split": [knm, ksm, kom], "weights_tiled": bool(tiled),
                           "quant_ms": round(times[0], 5), "gemm_ms": round(times[1], 5),
                           "gemm_tflops": round(flops / (times[1] * 1e-3) / 1e12, 1),
                           "fused_tflops": round(flops / ((times[0] + times[1]) * 1e-3) / 1e12, 1),
                           "gemm_frac_of_peak": round(flops / (times[1] * 1e-3) / 1e12 / blended_peak(knm, ksm, kom), 4),
                           "quant_gbs": round(quant_bytes(mm, kk, knm, ksm, kom) / (times[0] * 1e-3) / 1e9, 1)})
            del xm, wqm, aqm, dm
        extra["shape_matrix"] = {"note": "back-to-back launches on one buffer set (operands may sit in the 256 MB "
                                         "Infinity Cache); 20 launches per kernel replayed as a HIP graph: 0.15 s of untimed replays, then the median of 5", "rows": matrix}

        # ------------------------------------------------------------ one activation format at a time (c3's M, N, K)
        # splits that run the kernel family c3 runs (segment-boundary copies compiled in: at least three stages in every
        # segment that another follows), tile-major weights; the other formats get few stages, and the last segments
        # differ in length (2, 3 stages; no E3M2 at all) so that each leg is a kernel of its own in a trace
        per_format = []
        for name, (knf, ksf, kof) in (("e2m1", (3456, 384, 256)), ("e3m2", (384, 3328, 384)), ("e4m3", (768, 0, 3328))):
            aqf = abi.reorder_quantize_x(xd, idd, knf, ksf, kof)
            wqf = abi.reorder_quantize_w(wd, idd, knf, ksf, kof)
            wqf = abi.tile_weights(*wqf[:3]) + wqf[3:]
            df = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            f_ms = graph_ms(lambda i: abi.matmul(aqf[0], wqf[0], aqf[1], wqf[1], aqf[2], wqf[2], aqf[3], wqf[3],
                                                 aqf[4], wqf[4], aqf[5], wqf[5], out=df, w_tiled=True), 20)
            pk = blended_peak(knf, ksf, kof)
            tf = 2.0 * m * n * k / (f_ms * 1e-3) / 1e12
            per_format.append({"activations": name, "split": [knf, ksf, kof], "gemm_ms": round(f_ms, 5),
                               "tflops": round(tf, 1), "peak": round(pk, 1), "frac": round(tf / pk, 4)})
            del aqf, wqf, df
        extra["per_format_gemm"] = {"note": "c3's M, N and K with 3456 / 3328 / 3328 of the 4096 channels in one activation format, "
                                            "on the kernel family c3 runs; peak = the same blended nominal formula", "rows": per_format}

        # ------------------------------------------------------------ plans without one or two of the activation formats
        # (the last three: pure E3M2 x E2M1 and E4M3 x E2M1 products, what matmul_host6 / matmul_host8 of the
        # reference compute on their own, bench_fp6.cu:109-122 and bench_fp8.cu, and E3M2 + E4M3)
        partial = []
        for knf, ksf, kof in ((4096, 0, 0), (3968, 0, 128), (2560, 1536, 0), (0, 4096, 0), (0, 0, 4096), (0, 3968, 128)):
            aqf = abi.reorder_quantize_x(xd, idd, knf, ksf, kof)
            wqf = abi.reorder_quantize_w(wd, idd, knf, ksf, kof)
            wtf = abi.tile_weights(*wqf[:3])
            df = torch.empty((m, n), dtype=torch.bfloat16, device=dev)
            f_ms = graph_ms(lambda i: abi.matmul(aqf[0], wtf[0], aqf[1], wtf[1], aqf[2], wtf[2], aqf[3], wqf[3],
                                                 aqf[4], wqf[4], aqf[5], wqf[5], out=df, w_tiled=True), 20)
            pk = blended_peak(knf, ksf, kof)
            tf = 2.0 * m * n * k / (f_ms * 1e-3) / 1e12
            partial.append({"split": [knf, ksf, kof], "gemm_ms": round(f_ms, 5), "tflops": round(tf, 1),
                            "peak": round(pk, 1), "frac": round(tf / pk, 4)})
            del aqf, wqf, wtf, df
        extra["plans_without_a_segment"] = {"note": "c3's M, N and K, tile-major weights, whole-tile kernel", "rows": partial}

        # ------------------------------------------------------------ what the matrix cores sustain on this box
        # register-resident scaled-MFMA loop on all CUs: with pseudo-random operand bits the chip hits its
        # power limit and clocks down, which bounds any GEMM on real data below the nominal peak
        c_tf, c_ghz = measure_mfma_ceiling(BL, False)
        r_tf, r_ghz = measure_mfma_ceiling(BL, True)
        extra["mfma_e2m1_register_loop"] = {
            "constant_operands": {"tflops": round(c_tf, 1), "shader_ghz": round(c_ghz, 3)},
            "random_operands": {"tflops": round(r_tf, 1), "shader_ghz": round(r_ghz, 3)},
            "nominal_peak_tflops": P46,
        }

    # ---------------------------------------------------------------- CPU baseline (oracle, host cores)
    cpu = None
    if not args.no_cpu_baseline:
        from oracle import mx_oracle as mo
        from oracle import scalar as sc
        torch_threads = torch.get_num_threads()
        rows = m          # the whole c3 workload: a step takes the host cores well under a second
        wq_host = sc.quantize_w(H.bf16_bits(w), idx.numpy(), kn, ks, ko)          # offline, as on the GPU
        wdeq = torch.from_numpy(np.concatenate([
            mo.dequantize(mo.unpack_fp4(wq_host[q]), mo.sf_gather(wq_host[s], n, kk), "e2m1")
            for q, s, kk in (("qn", "sfn", kn), ("qs", "sfs", ks), ("qo", "sfo", ko))], axis=1))
        xs_bits = H.bf16_bits(x[:rows])

        def cpu_step():
            q = sc.quantize_x(xs_bits, idx.numpy(), kn, ks, ko)
            xdeq = np.concatenate([
                mo.dequantize(mo.unpack_fp4(q["qn"]), mo.sf_gather(q["sfn"], rows, kn), "e2m1"),
                mo.dequantize(mo.unpack_fp6(q["qs"]), mo.sf_gather(q["sfs"], rows, ks), "e3m2"),
                mo.dequantize(q["qo"], mo.sf_gather(q["sfo"], rows, ko), "e4m3")], axis=1)
            return (torch.from_numpy(xdeq) @ wdeq.T).to(torch.bfloat16)

        cpu_step()
        reps = 30
        c0 = time.perf_counter()
        for _ in range(reps):
            cpu_step()
        c_s = (time.perf_counter() - c0) / reps
        cpu = {
            "value": round(2.0 * rows * n * k / c_s / 1e12, 4), "unit": "TFLOP/s",
            "cores": torch_threads, "kind": "port",
            "sample": f"all {rows} token rows of c3 (N={n}, K={k}): C-oracle reorder-quantize + NumPy "
                      f"dequantize + torch fp32 matmul, weights quantized offline; 1 warm-up + {reps} repeats "
                      f"({c_s * reps:.1f} s of host work); os.cpu_count()={os.cpu_count()}",
        }
        if "reorder_quant_c1" in extra:
            m1, _, k1, kn1, ks1, ko1 = H.CONFIGS["c1"]
            r1 = m1
            reps1 = 500
            x1b = H.bf16_bits(H.make_activations(m1, k1, 1234 + 1)[:r1])
            i1 = H.random_index(k1, 4321).numpy()
            sc.quantize_x(x1b, i1, kn1, ks1, ko1)
            c0 = time.perf_counter()
            for _ in range(reps1):
                sc.quantize_x(x1b, i1, kn1, ks1, ko1)
            c1_s = (time.perf_counter() - c0) / reps1
            extra["reorder_quant_c1"]["cpu_baseline"] = {
                "value": round(quant_bytes(r1, k1, kn1, ks1, ko1) / c1_s / 1e9, 3), "unit": "GB/s",
                "cores": int(os.environ.get("OMP_NUM_THREADS", os.cpu_count())), "kind": "port",
                "sample": f"all {r1} rows of c1, scalar C oracle with OpenMP over rows, {reps1} repeats "
                          f"({c1_s * reps1:.1f} s of host work)",
            }

    out = {
        "metric": "mixed_mx_gemm_tflops", "value": round(value, 2), "unit": "TFLOP/s", "n_gpus": 1,
        "steps": args.steps, "warmup": args.warmup, "ms_per_step": round(ms_per_step, 4),
        "ms_per_step_sub_loops": [round(v, 4) for v in sub_ms], "ms_per_step_median_sub_loop": round(sub_ms[len(sub_ms) // 2], 4),
        "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "mxfp4/mxfp6/mxfp8 x mxfp4 -> f32 accumulate -> bf16", "data": "synthetic",
        "config": {"workload": "c3 prefill: reorder-quantize bf16 X[4096,4096] + mixed GEMM vs MXFP4 W[14336,4096] "
                               "(K split 2560 fp4 / 1408 fp6 / 128 fp8), bf16 out; weight codes packed tile-major offline; "
                               "one mg_fused_linear_ex call per step",
                   "M": m, "N": n, "K": k, "KN": kn, "KS": ks, "KO": ko},
        "roofline": roofline, "cpu_baseline": cpu, "extra": extra,
    }
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
