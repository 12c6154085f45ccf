#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

One *step* = one decode pass (batch 1) over the linear projections of one
27B/32B-class dense decoder layer, the workload BASELINE.json's metric is quoted
on: Q8_1-quantise the hidden state, fused Q/K/V GEMV (Q4_K, Q4_K, Q6_K),
quantise, O GEMV (Q4_K), quantise, fused gate+up GEMV (Q4_K), SwiGLU + quantise,
down GEMV (Q6_K).  All inputs and weights are resident in HBM before the timed
region.  Steps rotate over several layers' worth of distinct weights (more than
the 256 MB Infinity Cache), and each layer's step is replayed as a HIP graph so
the figure is not bounded by host launch overhead.

Prints ONE JSON line: whole-job effective GB/s (algorithmic bytes / time), a
`roofline` object for the dominant kernel (Q4_K GEMV 25600x5120, timed with HIP
events on the launch stream over back-to-back launches on rotating weights) and a
`cpu_baseline` object (the reference CPU path timed on this host by
oracle/cpu_baseline.py on a bounded sample).
"""
from __future__ import annotations

import argparse
import json
import os
import subprocess
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

# HBM bytes per launch of the dominant kernel, from rocprofv3 --pmc FETCH_SIZE and WRITE_SIZE
# runs of this script (profiles/gemv_q4k_25600x5120_batch1_pmc.txt): (36104.2 KiB x 2.000 +
# 104.4 KiB x 1.000), the factors being what the same counters read for a plain 256 MiB kernel.
DOMINANT_TRAFFIC_BYTES = 74048307

HIDDEN, QDIM, KVDIM, FFN = 5120, 8192, 1024, 25600


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--batch", type=int, default=1, help="activation rows per step (1 or 8)")
    ap.add_argument("--layers", type=int, default=4, help="distinct weight sets rotated through")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--pmc-calibration", action="store_true",
                    help="also run a plain 256 MiB read + 256 MiB write elementwise kernel a few times, so a rocprofv3 --pmc run of this "
                         "command records FETCH_SIZE / WRITE_SIZE for a kernel of known traffic")
    return ap.parse_args()


def main():
    args = parse()
    if args.gpus != 1:
        print("bench.py measures one GPU: this build has no multi-GPU path (run with --gpus 1)", file=sys.stderr)
        sys.exit(2)

    import torch

    from llaminar_amd import capi, synth
    from llaminar_amd.capi import FMT_Q4_K, FMT_Q6_K

    capi.load()
    if not torch.cuda.is_available():
        print("bench.py needs a GPU", file=sys.stderr)
        sys.exit(2)
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)
    M = args.batch
    assert 1 <= M <= capi.MAX_GEMV_M

    projs = [("q", QDIM, HIDDEN, FMT_Q4_K), ("k", KVDIM, HIDDEN, FMT_Q4_K), ("v", KVDIM, HIDDEN, FMT_Q6_K),
             ("o", HIDDEN, QDIM, FMT_Q4_K), ("gate", FFN, HIDDEN, FMT_Q4_K), ("up", FFN, HIDDEN, FMT_Q4_K),
             ("down", HIDDEN, FFN, FMT_Q6_K)]
    layers = []
    for l in range(args.layers):
        w = {}
        for i, (name, N, K, fmt) in enumerate(projs):
            raw = synth.weights_torch(fmt, N, K, 1000 * l + i, dev)
            w[name] = capi.prepare_weights(fmt, raw, N, K)
            del raw
        layers.append(w)
    torch.cuda.synchronize()

    g = torch.Generator(device=dev)
    g.manual_seed(7)
    x = torch.randn(M, HIDDEN, device=dev, generator=g)
    attn = torch.randn(M, QDIM, device=dev, generator=g)
    x2 = torch.randn(M, HIDDEN, device=dev, generator=g)
    q8_x = torch.empty(M * (HIDDEN // 32) * 36, dtype=torch.uint8, device=dev)
    q8_attn = torch.empty(M * (QDIM // 32) * 36, dtype=torch.uint8, device=dev)
    q8_x2 = torch.empty(M * (HIDDEN // 32) * 36, dtype=torch.uint8, device=dev)
    q8_act = torch.empty(M * (FFN // 32) * 36, dtype=torch.uint8, device=dev)
    qkv = torch.empty(M, QDIM + 2 * KVDIM, device=dev)
    o_out = torch.empty(M, HIDDEN, device=dev)
    gate = torch.empty(M, FFN, device=dev)
    up = torch.empty(M, FFN, device=dev)
    down = torch.empty(M, HIDDEN, device=dev)
    lib = capi.load()

    def step(w):
        capi.quantize_q8_1(x, out=q8_x)
        capi.gemv_fused([(FMT_Q4_K, w["q"], qkv[:, :QDIM]), (FMT_Q4_K, w["k"], qkv[:, QDIM:QDIM + KVDIM]),
                         (FMT_Q6_K, w["v"], qkv[:, QDIM + KVDIM:])], q8_x, M, HIDDEN)
        capi.quantize_q8_1(attn, out=q8_attn)
        capi.gemv(FMT_Q4_K, w["o"], q8_attn, M, HIDDEN, QDIM, out=o_out)
        capi.quantize_q8_1(x2, out=q8_x2)
        capi.gemv_fused([(FMT_Q4_K, w["gate"], gate), (FMT_Q4_K, w["up"], up)], q8_x2, M, HIDDEN)
        ok = lib.llam_ql_swiglu_quantize(gate.data_ptr(), up.data_ptr(), None, q8_act.data_ptr(), M, FFN, 0,
                                         torch.cuda.current_stream().cuda_stream)
        assert ok, capi.last_error()
        capi.gemv(FMT_Q6_K, w["down"], q8_act, M, HIDDEN, FFN, out=down)

    bytes_per_step = sum(synth.gemv_bytes(fmt, N, K, M) for _, N, K, fmt in projs)
    bytes_per_step += M * (2 * HIDDEN + QDIM) * 4 + M * 2 * FFN * 4  # fp32 read by the quantisers

    stream = torch.cuda.Stream()
    graphs = None
    with torch.cuda.stream(stream):
        for i in range(max(args.warmup, 1)):
            step(layers[i % args.layers])
        stream.synchronize()
        if not args.no_graph:
            graphs = []
            for w in layers:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    step(w)
                graphs.append(gr)
            for gr in graphs:
                gr.replay()
            stream.synchronize()

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if graphs is not None:
            for i in range(args.steps):
                graphs[i % args.layers].replay()
        else:
            for i in range(args.steps):
                step(layers[i % args.layers])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms_per_step = (t1 - t0) * 1e3 / args.steps
        value = bytes_per_step / (ms_per_step * 1e-3) / 1e9

        # ---- roofline of the dominant kernel: Q4_K GEMV 25600 x 5120, batch 1 ------------------
        # back-to-back launches over 2*layers distinct matrices (gate and up of every layer),
        # bracketed by HIP events on the launch stream
        mats = [l[n] for l in layers for n in ("gate", "up")]
        q8_1 = q8_x2[: (HIDDEN // 32) * 36]
        y = torch.empty(1, FFN, device=dev)
        reps = max(50, min(400, args.steps))
        for i in range(10):
            capi.gemv(FMT_Q4_K, mats[i % len(mats)], q8_1, 1, FFN, HIDDEN, out=y)
        e0 = torch.cuda.Event(enable_timing=True)
        e1 = torch.cuda.Event(enable_timing=True)
        stream.synchronize()
        e0.record(stream)
        for i in range(reps):
            capi.gemv(FMT_Q4_K, mats[i % len(mats)], q8_1, 1, FFN, HIDDEN, out=y)
        e1.record(stream)
        stream.synchronize()
        k_us = e0.elapsed_time(e1) * 1e3 / reps
        k_bytes = synth.gemv_bytes(FMT_Q4_K, FFN, HIDDEN, 1)
        achieved = k_bytes / (k_us * 1e-6) / 1e9

    if args.pmc_calibration:
        # a plain streaming kernel: reads 256 MiB, writes 256 MiB
        src = torch.arange(64 << 20, dtype=torch.int32, device=dev)
        dst = torch.empty_like(src)
        for _ in range(5):
            torch.add(src, 1, out=dst)
        torch.cuda.synchronize()

    cpu = None
    if not args.no_cpu_baseline:
        try:
            env = dict(os.environ)
            env.setdefault("QL_CPU_BASELINE_SECONDS", "12")
            p = subprocess.run([sys.executable, str(ROOT / "oracle" / "cpu_baseline.py")], capture_output=True,
                               text=True, timeout=300, env=env)
            if p.returncode == 0:
                cpu = json.loads(p.stdout.strip().splitlines()[-1])
            else:
                cpu = {"value": None, "unit": "GB/s", "cores": None, "kind": "port",
                       "sample": f"cpu baseline failed (exit {p.returncode}): {p.stderr.strip()[-200:]}"}
        except Exception as e:  # noqa: BLE001 - the GPU figure must still be reported
            cpu = {"value": None, "unit": "GB/s", "cores": None, "kind": "port", "sample": f"cpu baseline error: {e}"}

    out = {
        "metric": "Q4_K GEMV effective GB/s (% of 8 TB/s HBM); decode tokens/s at batch 1",
        "value": round(value, 1),
        "unit": "GB/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": "one 27B/32B-class dense decoder layer's linear projections, decode batch %d: "
                        "Q 5120->8192, K/V 5120->1024, O 8192->5120, gate/up 5120->25600 in Q4_K, V 5120->1024 and "
                        "down 25600->5120 in Q6_K; Q8_1 activations" % M,
            "batch": M,
            "bytes_per_step": bytes_per_step,
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "distinct_weight_sets": args.layers,
            "launch": "eager" if graphs is None else "hip-graph replay",
        },
        "roofline": {
            "kernel": "gemv_stream_kernel<Q4KTraits,1,5,2> N=25600 K=5120",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": DOMINANT_TRAFFIC_BYTES,
            "bytes_per_launch": k_bytes,
            "us_per_launch": round(k_us, 3),
            "launches_timed": reps,
        },
        "cpu_baseline": cpu,
    }
    print(json.dumps(out))


if __name__ == "__main__":
    main()
