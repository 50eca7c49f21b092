#!/usr/bin/env python3
"""Throughput of the per-rank data-parallel compute path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--only fold|all]

A "step" is one pass of the hot path over one batch of synthetic input with the
inputs already resident in HBM: the fp32 ring reduce-scatter fold of a
96,510,024-element gradient held by 8 simulated ranks (25 MiB buckets, 8 chunks
per bucket, 7 folds per chunk slot in ring-step order, then AVG x 1/8).  The one
JSON line printed at the end carries that figure as `value`, its roofline
block, the CPU baseline timed on this box's host cores, and (under `extra`) the
other workloads of the path: the binary fold of one bucket, the step-wise
drop-in sequence, the bf16/fp16 folds, top-k 1 % compression and the
decompress-accumulate.
"""
from __future__ import annotations

import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

N_GRAD = 96_510_024          # HeavyDummyModel parameter count of the reference
BUCKET = 6_553_600           # 25 MiB of fp32: DDP's default bucket
HBM_PEAK_GBPS = 8000.0       # MI355X published HBM3E peak


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=20)
    ap.add_argument("--warmup", type=int, default=3)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--only", default="all", choices=["all", "fold", "topk", "sparse"],
                    help="fold / topk / sparse: the headline workload plus only that part (profiling runs)")
    ap.add_argument("--elems", type=int, default=N_GRAD, help="gradient elements (default: the full 96.5 M)")
    return ap.parse_args()


def main() -> int:
    a = parse()
    if a.gpus != 1:
        print("bench.py measures one GPU: every rank's buffer lives in that GPU's HBM and nothing "
              "here uses a second device; run with --gpus 1", file=sys.stderr)
        return 2

    import numpy as np
    import torch
    from mccl_amd import hip_ops as ops
    import bench_traffic as hbm_traffic

    # HBM bytes per launch from the committed counter runs; None (with the reason) when they were
    # taken on other versions of the kernel sources or another workload size
    traffic, traffic_note = hbm_traffic.load_for_bench()
    if a.elems != N_GRAD:
        traffic, traffic_note = None, "counter runs exist for the default workload size only"

    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        return 2
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    N = a.elems
    W = 8
    K, WU = a.steps, a.warmup

    def gpu_time(fn, steps=K, warmup=WU):
        """Returns (wall ms per step, list of per-launch-group event ms)."""
        for _ in range(warmup):
            fn()
        torch.cuda.synchronize()
        evs = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(steps)]
        t0 = time.perf_counter()
        for s, e in evs:
            s.record()
            fn()
            e.record()
        torch.cuda.synchronize()
        wall = (time.perf_counter() - t0) * 1e3 / steps
        return wall, [s.elapsed_time(e) for s, e in evs]

    def stats(ms_list):
        arr = sorted(ms_list)
        return {"avg_ms": sum(arr) / len(arr), "median_ms": arr[len(arr) // 2], "min_ms": arr[0]}

    def rate(nbytes, ms):
        return nbytes / (ms * 1e-3) / 1e9

    extra = {}
    roofline_topk = None

    # ---- config 2: the headline workload -----------------------------------
    gens = [torch.Generator(device=dev).manual_seed(1000 + r) for r in range(W)]
    ranks = [torch.randn(N, generator=gens[r], device=dev).mul_(1e-3) for r in range(W)]
    out = torch.empty(N, device=dev)
    fold_bytes = (W + 1) * 4 * N

    def step_fold():
        ops.ring_fold(out, ranks, ops.AVG, ops.RING_BASIC, bucket_elems=BUCKET, scale_by=0.125)

    wall_ms, ev_ms = gpu_time(step_fold)
    st = stats(ev_ms)
    fold_gbps = rate(fold_bytes, wall_ms)
    roofline = {
        "bound": "hbm", "kernel": "k_ring_fold<f32,add>",
        "achieved": rate(fold_bytes, st["avg_ms"]), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
        "frac": rate(fold_bytes, st["avg_ms"]) / HBM_PEAK_GBPS,
        "traffic": traffic["ring_fold_f32_w8"] if traffic else None, "traffic_source": traffic_note,
        "bytes_per_launch": fold_bytes, "avg_launch_ms": st["avg_ms"], "min_launch_ms": st["min_ms"],
    }

    # device-to-device copy ceiling with the same timing method (read N, write N)
    cpy_ms = stats(gpu_time(lambda: out.copy_(ranks[0]))[1])
    extra["d2d_copy_GBps"] = rate(8 * N, cpy_ms["avg_ms"])

    if a.only in ("all", "fold"):
        # other world sizes (the reference's tests use 3 and 6); each has an unrolled instance
        for ws_rt in (3, 5, 6, 7):
            inv = float(np.float32(1.0 / ws_rt))
            r = stats(gpu_time(lambda: ops.ring_fold(out, ranks[:ws_rt], ops.AVG, ops.RING_BASIC,
                                                     bucket_elems=BUCKET, scale_by=inv))[1])
            b = (ws_rt + 1) * 4 * N
            extra[f"ring_fold_f32_w{ws_rt}"] = {"ms": r["avg_ms"], "GBps": rate(b, r["avg_ms"]),
                                                "frac": rate(b, r["avg_ms"]) / HBM_PEAK_GBPS}

    if a.only == "all":
        # ---- step-wise drop-in sequence: 7 binary folds per chunk view + scale --
        work = [r.clone() for r in ranks[:2]]  # only shapes matter for timing; reuse two buffers
        nb = (N + BUCKET - 1) // BUCKET

        def step_stepwise():
            for b in range(nb):
                lo, hi = b * BUCKET, min(N, (b + 1) * BUCKET)
                ce = (hi - lo + W - 1) // W
                for c in range(W):
                    s, e = lo + c * ce, min(hi, lo + (c + 1) * ce)
                    if s >= e:
                        continue
                    for j in range(1, W):
                        ops.fold2(out[s:e], ranks[(c + j) % W][s:e], ops.SUM)
                ops.scale(out[lo:hi], 0.125)

        sw = stats(gpu_time(step_stepwise, steps=max(2, K // 5), warmup=1)[1])
        extra["stepwise_dropin"] = {"ms": sw["avg_ms"], "GBps": rate((12 * (W - 1) + 8) * N, sw["avg_ms"]),
                                    "bytes_per_elem": 12 * (W - 1) + 8, "launches": nb * (W * (W - 1) + 1)}

        # the same sequence with the folds of one ring step handed over as one list
        # (mccl_hip_fold2_batch): W - 1 list calls and one scale instead of 855 launches
        lists = []
        for j in range(1, W):
            dl, sl = [], []
            for b in range(nb):
                lo, hi = b * BUCKET, min(N, (b + 1) * BUCKET)
                ce = (hi - lo + W - 1) // W
                for c in range(W):
                    s, e = lo + c * ce, min(hi, lo + (c + 1) * ce)
                    if s < e:
                        dl.append(out[s:e]); sl.append(ranks[(c + j) % W][s:e])
            lists.append((dl, sl))

        def step_batched():
            for dl, sl in lists:
                ops.fold2_batch(dl, sl, ops.SUM)
            ops.scale(out, 0.125)

        sb = stats(gpu_time(step_batched, steps=max(3, K // 4), warmup=1)[1])
        extra["stepwise_batched"] = {"ms": sb["avg_ms"], "GBps": rate((12 * (W - 1) + 8) * N, sb["avg_ms"]),
                                     "frac": rate((12 * (W - 1) + 8) * N, sb["avg_ms"]) / HBM_PEAK_GBPS,
                                     "bytes_per_elem": 12 * (W - 1) + 8, "launches": W,
                                     "note": "host time of building the pointer lists included"}

        # ---- config 1: one 25 MiB bucket, W=2, fused (x0 + x1) * 0.5 ------------
        b0, b1 = ranks[0][:BUCKET].clone(), ranks[1][:BUCKET].clone()
        c1 = stats(gpu_time(lambda: ops.fold2_scale(b0, b1, 0.5))[1])
        extra["config1_fold2_scale_bucket"] = {"ms": c1["avg_ms"], "GBps": rate(12 * BUCKET, c1["avg_ms"]),
                                               "note": "78.6 MB working set: Infinity-Cache resident"}
        # same kernel over the whole gradient: HBM-resident figure
        c1w = stats(gpu_time(lambda: ops.fold2_scale(work[0], work[1], 0.5))[1])
        extra["fold2_scale_whole_gradient"] = {"ms": c1w["avg_ms"], "GBps": rate(12 * N, c1w["avg_ms"]),
                                               "frac": rate(12 * N, c1w["avg_ms"]) / HBM_PEAK_GBPS}
        c1f = stats(gpu_time(lambda: ops.fold2(work[0], work[1], ops.SUM))[1])
        extra["fold2_whole_gradient"] = {"ms": c1f["avg_ms"], "GBps": rate(12 * N, c1f["avg_ms"]),
                                         "frac": rate(12 * N, c1f["avg_ms"]) / HBM_PEAK_GBPS}
        del work, b0, b1

        # ---- config 3: bf16 / fp16, W = 4, SUM (+ x0.25) and MAX ----------------
        for name, tdt in (("bf16", torch.bfloat16), ("fp16", torch.float16)):
            hs = []
            for r in range(4):
                x = torch.randn(N, generator=gens[r], device=dev).mul_(1e-3)
                m = torch.rand(N, generator=gens[r], device=dev) < 1e-3
                x[m] *= 1e3
                hs.append(x.to(tdt))
                del x, m
            ho = torch.empty(N, device=dev, dtype=tdt)
            res = {}
            for label, kw in (("sum_avg_single_rounding", dict(op=ops.AVG, scale_by=0.25, stepwise=False)),
                              ("sum_avg_stepwise", dict(op=ops.AVG, scale_by=0.25, stepwise=True)),
                              ("max", dict(op=ops.MAX))):
                s3 = stats(gpu_time(lambda: ops.ring_fold(ho, hs, schedule=ops.RING_BASIC,
                                                          bucket_elems=2 * BUCKET, **kw))[1])
                res[label] = {"ms": s3["avg_ms"], "GBps": rate(10 * N, s3["avg_ms"]),
                              "frac": rate(10 * N, s3["avg_ms"]) / HBM_PEAK_GBPS}
            extra[f"config3_{name}_w4"] = res
            del hs, ho

    if a.only in ("all", "topk", "sparse"):
        # ---- config 4: top-k 1 % with error feedback, per 25 MiB bucket ----------
        g = torch.randn(N, generator=gens[0], device=dev)
        chi = sum(torch.randn(N, generator=gens[1], device=dev).square_() for _ in range(3)).div_(3).sqrt_()
        grad = g.div_(chi).mul_(1e-3)
        del chi
        m = N // 100
        dst = torch.randint(0, N, (m,), generator=gens[2], device=dev)
        src = torch.randint(0, N, (m,), generator=gens[2], device=dev)
        sign = torch.where(torch.rand(m, generator=gens[2], device=dev) < 0.5, -1.0, 1.0)
        grad[dst] = grad[src] * sign
        residual0 = torch.randn(N, generator=gens[3], device=dev).mul_(1e-4)
        residual = residual0.clone()
        stride = ops.topk_wire_stride(BUCKET, 0.01)
        nb = (N + BUCKET - 1) // BUCKET
        wire = torch.empty(nb * stride, dtype=torch.uint8, device=dev)
        wsb = ops.topk_workspace(N, BUCKET, 0.01, dev)
        ks = [ops.topk_k(min(BUCKET, N - b * BUCKET), 0.01) for b in range(nb)]
        topk_bytes = 12 * N + sum(8 * k + 4 for k in ks)

        def step_topk():
            ops.topk_compress(grad, residual, 0.01, bucket_elems=BUCKET, wire=wire, workspace=wsb,
                              wire_stride=stride)

        tk = stats(gpu_time(step_topk)[1])
        extra["config4_topk_compress"] = {"ms": tk["avg_ms"], "GBps": rate(topk_bytes, tk["avg_ms"]),
                                          "frac": rate(topk_bytes, tk["avg_ms"]) / HBM_PEAK_GBPS,
                                          "elems_per_s": N / (tk["avg_ms"] * 1e-3),
                                          "bytes": topk_bytes, "buckets": nb, "k_per_bucket": ks[0],
                                          "single_pass_buckets": ops.topk_path_report(wsb, N, BUCKET, 0.01)[0]}
        # second half of the headline metric: same fields as `roofline`, for the whole
        # compress call (two launches: streaming with sample and binning, selection)
        roofline_topk = {"bound": "hbm", "kernel": "mccl_hip_topk_compress (2 launches, dominant k_topk_stream)",
                         "achieved": rate(topk_bytes, tk["avg_ms"]), "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                         "frac": rate(topk_bytes, tk["avg_ms"]) / HBM_PEAK_GBPS,
                         "traffic": traffic["topk_compress"] if traffic else None, "traffic_source": traffic_note,
                         "bytes_per_launch": topk_bytes, "avg_launch_ms": tk["avg_ms"],
                         "median_launch_ms": tk["median_ms"], "min_launch_ms": tk["min_ms"]}
        # one bucket alone (the reference's call granularity; cache resident)
        r1 = residual0[:BUCKET].clone()
        ws1 = ops.topk_workspace(BUCKET, BUCKET, 0.01, dev)
        w1 = torch.empty(stride, dtype=torch.uint8, device=dev)
        tb = stats(gpu_time(lambda: ops.topk_compress(grad[:BUCKET], r1, 0.01, wire=w1, workspace=ws1,
                                                      wire_stride=stride))[1])
        extra["config4_topk_one_bucket"] = {"ms": tb["avg_ms"],
                                            "GBps": rate(12 * BUCKET + 8 * ks[0] + 4, tb["avg_ms"]),
                                            "frac": rate(12 * BUCKET + 8 * ks[0] + 4, tb["avg_ms"]) / HBM_PEAK_GBPS}
        # the reference compresses bucket by bucket (TopKCompressor::compress per DDP bucket): the 15
        # buckets as 15 separate buffers, through 15 calls and through one list call
        import torch.distributed  # noqa: F401
        from mccl_amd import _C
        bufs = [grad[b * BUCKET: min(N, (b + 1) * BUCKET)] for b in range(nb)]
        ids = list(range(1, nb + 1))
        comp = _C.TopKCompressor(0.01)
        per = stats(gpu_time(lambda: [comp.compress(t, stable_id=i) for t, i in zip(bufs, ids)],
                             steps=max(3, K // 2))[1])
        extra["config4_15_compress_calls"] = {"ms": per["avg_ms"], "GBps": rate(topk_bytes, per["avg_ms"]),
                                              "frac": rate(topk_bytes, per["avg_ms"]) / HBM_PEAK_GBPS,
                                              "note": "15 x TopKCompressor::compress, 30 launches: bound by launch latency"}
        comp = _C.TopKCompressor(0.01)
        many = stats(gpu_time(lambda: comp.compress_many(bufs, stable_ids=ids))[1])
        extra["config4_compress_many"] = {"ms": many["avg_ms"], "GBps": rate(topk_bytes, many["avg_ms"]),
                                          "frac": rate(topk_bytes, many["avg_ms"]) / HBM_PEAK_GBPS,
                                          "note": "TopKCompressor::compress_many on the same 15 buffers: 2 launches"}
        del comp, bufs

        # ---- config 5: decompress-accumulate of 8 ranks' payloads -----------------
        shared = torch.rand(N, generator=gens[4], device=dev) < 0.004
        wires = []
        for r in range(W):
            gr = torch.randn(N, generator=gens[r], device=dev).mul_(1e-2)
            gr[shared] *= 50.0
            rz = torch.zeros(N, device=dev)
            wr = torch.empty(nb * stride, dtype=torch.uint8, device=dev)
            ops.topk_compress(gr, rz, 0.01, bucket_elems=BUCKET, wire=wr, workspace=wsb, wire_stride=stride)
            wires.append(wr)
            del gr, rz
        status = torch.zeros(1, dtype=torch.int32, device=dev)
        acc = torch.empty(N, device=dev)
        acc_bytes = 4 * N + 8 * sum(ks) * W
        sws = ops.sparse_workspace(N, BUCKET, W, dev)
        sa = stats(gpu_time(lambda: ops.sparse_accumulate(acc, wires, stride, bucket_elems=BUCKET,
                                                          scale_by=0.125, status=status, workspace=sws))[1])
        extra["config5_sparse_accumulate"] = {"ms": sa["avg_ms"], "GBps": rate(acc_bytes, sa["avg_ms"]),
                                              "frac": rate(acc_bytes, sa["avg_ms"]) / HBM_PEAK_GBPS,
                                              "bytes": acc_bytes, "status": int(status),
                                              "traffic": traffic["sparse_accumulate"] if traffic else None,
                                              "traffic_source": traffic_note}
        # the other kernels of the same entry point: no workspace (block-per-tile kernels that
        # search the payloads themselves), and 12 ranks (more than the runs-of-tiles kernel takes)
        sn = stats(gpu_time(lambda: ops.sparse_accumulate(acc, wires, stride, bucket_elems=BUCKET, scale_by=0.125,
                                                          status=status, workspace=None))[1])
        extra["config5_sparse_accumulate_no_workspace"] = {"ms": sn["avg_ms"], "GBps": rate(acc_bytes, sn["avg_ms"]),
                                                           "frac": rate(acc_bytes, sn["avg_ms"]) / HBM_PEAK_GBPS}
        w12 = wires + wires[:4]
        b12 = 4 * N + 8 * sum(ks) * 12
        sws12 = ops.sparse_workspace(N, BUCKET, 12, dev)
        s12 = stats(gpu_time(lambda: ops.sparse_accumulate(acc, w12, stride, bucket_elems=BUCKET, scale_by=1.0 / 12,
                                                           status=status, workspace=sws12))[1])
        extra["sparse_accumulate_12_ranks_tile_kernels"] = {"ms": s12["avg_ms"], "GBps": rate(b12, s12["avg_ms"]),
                                                            "frac": rate(b12, s12["avg_ms"]) / HBM_PEAK_GBPS, "bytes": b12}
        cfg5_host = None
        if not a.no_cpu:
            cfg5_host = [wv[:stride].cpu().numpy() for wv in wires]   # bucket 0 of every rank, for the CPU leg

    if a.only == "all":
        # ---- FP16 compressor casts over the whole gradient (6 B / element each way) ----
        half = torch.empty(N, dtype=torch.float16, device=dev)
        c1 = stats(gpu_time(lambda: ops.cast_f32_to_f16(ranks[0], half))[1])
        c2 = stats(gpu_time(lambda: ops.cast_f16_to_f32(half, out))[1])
        extra["fp16_compress_cast"] = {"ms": c1["avg_ms"], "GBps": rate(6 * N, c1["avg_ms"]),
                                       "frac": rate(6 * N, c1["avg_ms"]) / HBM_PEAK_GBPS}
        extra["fp16_decompress_cast"] = {"ms": c2["avg_ms"], "GBps": rate(6 * N, c2["avg_ms"]),
                                         "frac": rate(6 * N, c2["avg_ms"]) / HBM_PEAK_GBPS}
        del half

    # ---- CPU baseline: the reference's CPU fold path restated, same workload ----
    cpu = None
    if not a.no_cpu:
        import oracle
        nbk = min(2, (N + BUCKET - 1) // BUCKET)     # bounded sample: 2 buckets of the 15
        cn = min(N, nbk * BUCKET)
        host = [r[:cn].cpu().numpy() for r in ranks]
        # The reference folds in place: a rank's chunk is `local`, the partial that arrived is
        # `incoming`, and local (op)= incoming (csrc/backend/ProcessGroupMCCL.cpp:492-512).  The
        # simulated ranks' buffers are therefore folded where they lie - no allocation or copy in
        # the timed loop - and only throughput is read off (the values drift from pass to pass).
        times = []
        t_all = time.perf_counter()
        while True:
            t0 = time.perf_counter()
            for b in range(nbk):
                lo, hi = b * BUCKET, min(cn, (b + 1) * BUCKET)
                ce = (hi - lo + W - 1) // W
                for c in range(W):
                    s, e = lo + c * ce, min(hi, lo + (c + 1) * ce)
                    if s >= e:
                        continue
                    part = host[c][s:e]
                    for j in range(1, W):
                        local = host[(c + j) % W][s:e]
                        oracle.fold2(local, part, oracle.F32, oracle.OP_SUM, threads=0)  # reference job split
                        part = local
                    oracle.scale(part, oracle.F32, 0.125, threads=0)
            times.append(time.perf_counter() - t0)
            spent = time.perf_counter() - t_all
            if spent > 10.0 or (len(times) >= 12 and spent > 3.0):   # at least 3 s of folding, at most 10
                break
        reps = len(times)
        cpu_s = sum(times) / reps
        cpu_med = sorted(times)[reps // 2]
        cpu = {"value": (W + 1) * 4 * cn / cpu_s / 1e9, "median": (W + 1) * 4 * cn / cpu_med / 1e9,
               "unit": "GB/s", "cores": min(8, os.cpu_count() or 1), "kind": "port",
               "sample": f"{nbk} of {(N + BUCKET - 1) // BUCKET} buckets ({cn} elements), {reps} repetitions; "
                         "step-wise ring folds in place with the reference's job split (>= 1 Mi floats per job, "
                         "<= 8 jobs), timed loop = folds and scale only, same 36 B/element numerator",
               "host_cores_visible": os.cpu_count()}
        if a.only in ("all", "topk") and oracle.RefCompressor.available():
            ref = oracle.RefCompressor(2, 0.01)
            gh = grad[:BUCKET].cpu().numpy()
            ref.compress(gh, stable_id=1)
            t0 = time.perf_counter()
            reps = 0
            while time.perf_counter() - t0 < 8.0 and reps < 6:
                ref.compress(gh, stable_id=1)
                reps += 1
            s_ref = (time.perf_counter() - t0) / reps
            extra["config4_cpu_reference_topk"] = {
                "GBps": (12 * BUCKET + 8 * 65_536 + 4) / s_ref / 1e9, "ms_per_bucket": s_ref * 1e3,
                "cores": 1, "kind": "reference",
                "sample": f"one 25 MiB bucket, {reps} repetitions of the reference's compiled TopKCompressor::compress"}

        if a.only in ("all", "sparse") and cfg5_host is not None:
            # leg (iii): decompress + accumulate in the reference's form - memset and scatter per rank
            # (csrc/compression/TopKCompression.cpp:122-152), a dense add per rank and x 1/W
            # (csrc/backend/ProcessGroupMCCL.cpp:2272-2296) - on bucket 0 of the 8 payloads of config 5
            use_ref = oracle.RefCompressor.available()
            refc = oracle.RefCompressor(2, 0.01) if use_ref else None
            accb = np.zeros(BUCKET, np.float32)
            kb0 = ops.topk_k(BUCKET, 0.01)
            t0 = time.perf_counter()
            reps = 0
            while time.perf_counter() - t0 < 6.0 and reps < 8:
                accb[:] = 0.0
                for hw in cfg5_host:
                    dense = refc.decompress(hw[:4 + 8 * kb0], BUCKET)[0] if use_ref else oracle.topk_decompress(hw, BUCKET)[0]
                    oracle.fold2(accb, dense, oracle.F32, oracle.OP_SUM, threads=0)
                oracle.scale(accb, oracle.F32, 0.125, threads=0)
                reps += 1
            s3 = (time.perf_counter() - t0) / reps
            b3 = 4 * BUCKET + 8 * kb0 * W
            extra["config5_cpu_reference_form"] = {
                "GBps": b3 / s3 / 1e9, "ms_per_bucket": s3 * 1e3, "cores": min(8, os.cpu_count() or 1),
                "kind": "reference" if use_ref else "port", "bytes": b3,
                "sample": f"bucket 0 of the 8 payloads of config 5, {reps} repetitions: per rank the reference's "
                          "decompress (memset + scatter, one core) and a dense fold with the reference's job split, "
                          "then x 1/8; same 4 n + 8 k W numerator as the GPU figure"}
        if a.only in ("all", "fold"):
            # cross-check of the fold port with torch's CPU kernels on the same host buffers, in the
            # same ring-step order and with the same numerator: in-place add_ per fold, mul_ per chunk
            import torch as _t
            th = [_t.from_numpy(h) for h in host]
            t0 = time.perf_counter()
            reps = 0
            while time.perf_counter() - t0 < 4.0 and reps < 12:
                for b in range(nbk):
                    lo, hi = b * BUCKET, min(cn, (b + 1) * BUCKET)
                    ce = (hi - lo + W - 1) // W
                    for c in range(W):
                        s, e = lo + c * ce, min(hi, lo + (c + 1) * ce)
                        if s >= e:
                            continue
                        part = th[c][s:e]
                        for j in range(1, W):
                            local = th[(c + j) % W][s:e]
                            local.add_(part)
                            part = local
                        part.mul_(0.125)
                reps += 1
            s4 = (time.perf_counter() - t0) / reps
            extra["cpu_torch_fold_crosscheck"] = {
                "GBps": (W + 1) * 4 * cn / s4 / 1e9, "threads": _t.get_num_threads(),
                "working_set_MiB": W * 4 * cn / 2 ** 20,
                "sample": f"the cpu_baseline sample ({nbk} buckets x {W} ranks) folded with torch's CPU add_ and "
                          f"mul_ in the same ring-step order, {reps} repetitions, same 36 B/element numerator; "
                          "a working set that fits the host's last-level cache is served from it"}

    if a.only == "all":
        # ---- step-wise ring driver: 8 ranks, chunked ring allreduce (reduce-scatter folds,
        # all-gather copies, AVG scale on every rank), one HIP stream per rank with fences.
        # Runs last: it reduces `ranks` in place.
        import torch.distributed  # noqa: F401
        from mccl_amd import _C
        group = _C.LoopbackGroup(W)
        rd = stats(gpu_time(lambda: group.allreduce_ring(ranks, ops.AVG, True), steps=max(3, K // 4), warmup=1)[1])
        rd_bytes = ((W - 1) * 12 + (W - 1) * 8 + W * 8) * N
        extra["ring_driver_allreduce_w8"] = {"ms": rd["avg_ms"], "GBps": rate(rd_bytes, rd["avg_ms"]),
                                             "bytes": rd_bytes, "launches": 2 * W * 2 * (W - 1) + W}

    line = {
        "metric": "HBM GB/s (% of peak) for fp32 bucket fold and top-k 1% compress, 1 GPU",
        "value": fold_gbps, "unit": "GB/s", "n_gpus": 1, "steps": K, "warmup": WU,
        "ms_per_step": wall_ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic (seeded device generators; values as the configs specify)",
        "config": {"workload": "configs[1]: fp32 ring reduce-scatter fold, 8 simulated ranks in one GPU's HBM, "
                               f"{N}-element gradient, 25 MiB buckets x 8 chunks, 7 folds per chunk slot in "
                               "ring-step order, AVG x 1/8 fused",
                   "elements": N, "world_size": W, "bucket_elems": BUCKET, "bytes_per_element": 36,
                   "elements_per_s": N / (wall_ms * 1e-3), "pct_of_hbm_peak": 100.0 * fold_gbps / HBM_PEAK_GBPS},
        "roofline": roofline,
        "roofline_topk": roofline_topk,
        "cpu_baseline": cpu,
        "extra": extra,
    }
    print(json.dumps(line))
    return 0


if __name__ == "__main__":
    sys.exit(main())
