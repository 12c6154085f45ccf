#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

One *step* = one launch of the kernel BASELINE.json's metric is quoted on, the
Q4_K decode GEMV 25600 x 5120 at batch 1 (the gate/up projection of a 27B/32B-class
dense decoder layer), Q8_1 activations.  All inputs and weights are resident in
HBM before the timed region; the steps rotate over eight distinct matrices (more
than the 256 MB Infinity Cache) and are replayed as a HIP graph, so the figure is
not bounded by host launch overhead.  `value` = algorithmic bytes / time.

`config.layer_step` holds the whole layer the kernel belongs to (config 2 of the
baseline): Q8_1-quantise the hidden state, fused Q/K/V GEMV (Q4_K, Q4_K, Q6_K),
quantise, O GEMV (Q4_K), quantise, fused gate+up GEMV (Q4_K), SwiGLU + quantise,
down GEMV (Q6_K), rotating over several layers' weights.

Prints ONE JSON line with a `roofline` object for the same kernel (HIP events on
the launch stream around graph replays of 40 launches, at least 200 launches
whatever --steps says: mean, median and minimum) and a `cpu_baseline` object (the
reference CPU path timed on this host by oracle/cpu_baseline.py on a bounded
sample).  The default run appends short runs of the other configurations to
`config` (decode step at batch 1 and 8, prefill GEMM, MoE decode).
"""
from __future__ import annotations

import argparse
import json
import os
import re
import subprocess
import sys
import time
from pathlib import Path

ROOT = Path(__file__).resolve().parent
sys.path.insert(0, str(ROOT))

HBM_PEAK_GBS = 8000.0  # MI355X published HBM3E bandwidth

DOMINANT_PROFILE = ROOT / "profiles" / "gemv_q4k_25600x5120_batch1_pmc.txt"


def dominant_traffic_bytes():
    """HBM bytes per launch of the dominant kernel as measured with rocprofv3 --pmc (FETCH_SIZE and
    WRITE_SIZE runs of this script, scaled by what the same counters read for a plain copy
    kernel): the `traffic_bytes_per_launch = N` line of the committed profile summary.  None
    when the summary is missing."""
    try:
        m = re.search(r"^traffic_bytes_per_launch\s*=\s*(\d+)", DOMINANT_PROFILE.read_text(), re.M)
    except OSError:
        return None
    return int(m.group(1)) if m else None

HIDDEN, QDIM, KVDIM, FFN = 5120, 8192, 1024, 25600


INT8_MFMA_PEAK_TOPS = 5000.0  # MI355X published dense int8 rate


def _time_launches(torch, stream, fn, reps, warm=5):
    """Average duration in microseconds of fn(i), timed with events on the launch stream."""
    for i in range(warm):
        fn(i)
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    stream.synchronize()
    e0.record(stream)
    for i in range(reps):
        fn(i)
    e1.record(stream)
    stream.synchronize()
    return e0.elapsed_time(e1) * 1e3 / reps


def _common(args, metric, value, unit, ms, dtype, config, roofline):
    return {"metric": metric, "value": value, "unit": unit, "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
            "ms_per_step": ms, "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": dtype,
            "data": "synthetic", "config": config, "roofline": roofline, "cpu_baseline": None}


def bench_gemm(args, torch, capi, synth, dev):
    """Prefill: M x 5120 Q8_1 activations times Q4_K [25600 x 5120], int8 MFMA."""
    from llaminar_amd.capi import FMT_Q4_K

    M = args.batch if args.batch > 8 else 512
    N, K = FFN, HIDDEN
    mats = [capi.prepare_weights(FMT_Q4_K, synth.weights_torch(FMT_Q4_K, N, K, 50 + i, dev), N, K) for i in range(2)]
    g = torch.Generator(device=dev)
    g.manual_seed(9)
    x = torch.randn(M, K, device=dev, generator=g)
    q8 = capi.quantize_q8_1(x)
    y = torch.empty(M, N, device=dev)
    stream = torch.cuda.Stream()
    steps = min(args.steps, 50)
    with torch.cuda.stream(stream):
        us = _time_launches(torch, stream, lambda i: capi.gemm(FMT_Q4_K, mats[i % 2], q8, M, N, K, out=y), steps,
                            max(2, min(args.warmup, 5)))
        us_q = _time_launches(torch, stream, lambda i: capi.quantize_q8_1(x, out=q8), steps)
    ops = 2.0 * M * N * K
    tops = ops / (us * 1e-6) / 1e12
    return _common(args, "prefill int8 GEMM TOPS", round(tops, 2), "TOP/s", round(us * 1e-3, 5), "int8",
                   {"workload": "prefill GEMM of the gate/up projection: M=%d tokens x K=5120 x N=25600, Q4_K weights, "
                                "Q8_1 activations" % M, "M": M, "N": N, "K": K, "ops_per_step": ops,
                    "quantize_us": round(us_q, 2)},
                   {"kernel": "gemm_kernel<Q4KTraits> M=%d N=25600 K=5120" % M, "bound": "mfma",
                    "achieved": round(tops, 2), "peak": INT8_MFMA_PEAK_TOPS, "unit": "TOP/s",
                    "frac": round(tops / INT8_MFMA_PEAK_TOPS, 4), "traffic": None, "ops_per_launch": ops,
                    "us_per_launch": round(us, 2), "launches_timed": steps})


def bench_moe(args, torch, capi, synth, dev):
    """MoE expert FFN decode: route (+ Q8_1 of the hidden state), gate/up, SwiGLU+quantise, down, shared expert."""
    from llaminar_amd.capi import FMT_IQ3_S

    T = args.batch
    H, I, E, TOPK = 2048, 512, 256, 8
    fmt = FMT_IQ3_S
    experts = []
    for e in range(E + 1):  # the last one is the shared expert
        experts.append(tuple(capi.prepare_weights(fmt, synth.weights_torch(fmt, n, k, 10 * e + j, dev), n, k)
                             for j, (n, k) in enumerate(((I, H), (I, H), (H, I)))))
    # the shared expert is entry E of the table and sits in a ninth slot of every token
    # (weight 1) that the router leaves alone: one gate/up and one down launch serve all
    table = capi.expert_table(experts, dev)
    # Several independent token sets (own hidden states, router logits and buffers), so that
    # consecutive steps route to different experts and their weights are not served from the
    # caches: 1 token x 9 experts x 1.35 MB per step against 256 MB of Infinity Cache.  All sets
    # are captured in ONE graph, the way a decode pass captures all of its MoE layers.
    nsets = 32 if T == 1 else 4
    g = torch.Generator(device=dev)
    g.manual_seed(11)
    sets = []
    for _ in range(nsets):
        sets.append({"x": torch.randn(T, H, device=dev, generator=g),
                     "logits": torch.randn(T, E, device=dev, generator=g),
                     "q8": torch.empty(T * (H // 32) * 36, dtype=torch.uint8, device=dev),
                     "out": torch.empty(T, H, device=dev),
                     "ids": torch.full((T, TOPK + 1), E, dtype=torch.int32, device=dev),
                     "w": torch.ones(T, TOPK + 1, device=dev)})

    # Batches sort the (token, slot) pairs by expert on the device and read every distinct
    # expert's matrices once (6 launches); a single token has nothing to group (2 launches).
    # (measured, grouped against per slot: 32 tokens 115 / 107 us, 48 tokens 142 / 144, 64 tokens 155 / 188, 128 tokens 228 / 340)
    path = args.moe_path if args.moe_path != "auto" else ("grouped" if T * (TOPK + 1) >= 432 else "slots")
    S = TOPK + 1
    for s_ in sets:
        s_["group"] = torch.empty(int(capi.load().llam_ql_moe_group_bytes(T, S)), dtype=torch.uint8, device=dev)
        s_["gate"] = torch.empty(T * S, I, device=dev)
        s_["up"] = torch.empty(T * S, I, device=dev)
        s_["pair_out"] = torch.empty(T * S, H, device=dev)
        s_["qa"] = torch.empty(T * S * (I // 32) * 36, dtype=torch.uint8, device=dev)

    def step(s):
        if path == "slots":
            # router, Q8_1 of the hidden state, gate/up, SwiGLU and the Q8_1 quantiser of the result in one launch
            # (from a few tokens on the library runs the router + quantiser as a launch of its own)
            qa = capi.moe_route_gate_up_swiglu(fmt, table, E + 1, s["logits"], TOPK, s["x"], s["ids"], s["w"], I,
                                               q8_out=s["qa"], q8_hidden=s["q8"])
        else:
            capi.moe_route_quantize(s["logits"], TOPK, s["x"], s["q8"], ids=s["ids"], weights=s["w"])
            capi.moe_group(s["ids"], E + 1, group=s["group"])
            gate, up = capi.moe_gate_up_grouped(fmt, table, E + 1, s["group"], s["q8"], T, S, H, I, gate=s["gate"],
                                                up=s["up"])
            qa = capi.swiglu_quantize(gate, up)
        if path == "grouped":
            capi.moe_down_grouped(fmt, table, E + 1, s["group"], s["ids"], s["w"], qa, s["pair_out"], s["out"], T, S,
                                  H, I)
        else:
            capi.moe_down(fmt, table, E + 1, s["ids"], s["w"], qa, s["out"], T, S, H, I, accumulate=False)

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        for i in range(max(args.warmup, 2)):
            step(sets[i % nsets])
        stream.synchronize()
        gr = torch.cuda.CUDAGraph()
        with torch.cuda.graph(gr, stream=stream):
            for s_ in sets:
                step(s_)
        reps = max(1, (args.steps + nsets - 1) // nsets)
        us = _time_launches(torch, stream, lambda i: gr.replay(), reps, 2) / nsets
        distinct = len(set(int(v) for s_ in sets for v in s_["ids"][:, :TOPK].flatten().tolist()))
        per_set = [len(set(int(v) for v in s_["ids"].flatten().tolist())) for s_ in sets]
    blk = 112  # device bytes per IQ3_S super-block
    per_expert = 3 * I * (H // 256) * blk
    slot_bytes = S * T * per_expert                       # every token slot streams its expert's matrices
    distinct_bytes = sum(per_set) / nsets * per_expert    # every distinct expert of a step once (incl. the shared one)
    # algorithmic bytes: the distinct experts a step touches (a single token touches S of them)
    w_bytes = distinct_bytes
    value = w_bytes / (us * 1e-6) / 1e9
    launches = {"slots": 2 if T * S * (I // 32) < 512 else 3, "grouped-gate-up": 5, "grouped": 6}[path]
    return _common(args, "MoE expert FFN decode effective GB/s", round(value, 1), "GB/s", round(us * 1e-3, 5), "int8",
                   {"workload": "MoE expert FFN decode: hidden 2048, 256 routed experts + 1 shared, top-8, expert "
                                "intermediate 512, IQ3_S, %d token(s); route + quantise, gate/up + SwiGLU + quantise (one launch with the router inside at 1-2 tokens), down; shared expert in a ninth slot" % T,
                    "tokens": T, "weight_bytes_per_step": round(w_bytes), "slot_bytes_per_step": slot_bytes,
                    "distinct_experts_per_step": round(sum(per_set) / nsets, 1),
                    "tokens_per_s": round(T / (us * 1e-6), 1), "path": path,
                    "token_sets_rotated": nsets, "distinct_routed_experts_over_sets": distinct,
                    "launch": "hip-graph replay of all token sets' steps"},
                   {"kernel": "moe step (%d launches)" % launches, "bound": "hbm", "achieved": round(value, 1),
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": round(value / HBM_PEAK_GBS, 4), "traffic": None,
                    "bytes_per_launch": round(w_bytes), "us_per_launch": round(us, 2), "launches_timed": args.steps})


def bench_gemv(args, torch, capi, synth, dev):
    """Single GEMVs: every format on the layer shapes, rotating over matrices beyond the cache."""
    from llaminar_amd.capi import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K

    M = args.batch
    rows = []
    stream = torch.cuda.Stream()
    names = {FMT_Q4_K: "Q4_K", FMT_Q6_K: "Q6_K", FMT_IQ3_S: "IQ3_S"}
    for fmt in (FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S):
        for N, K in ((FFN, HIDDEN), (HIDDEN, FFN), (QDIM, HIDDEN), (HIDDEN, QDIM), (KVDIM, HIDDEN)):
            nmat = max(2, min(8, int(600e6 // synth.gemv_bytes(fmt, N, K, 1)) + 1))
            mats = [capi.prepare_weights(fmt, synth.weights_torch(fmt, N, K, 70 + i, dev), N, K) for i in range(nmat)]
            # batches of 5..8: with the matrices' batch planes where the shape has them (--no-batch-planes: without)
            planes = [None] * nmat
            if M >= 5 and N >= 4096 and not args.no_batch_planes and capi.batch_plane_bytes(fmt, N, K) > 0:
                planes = [capi.build_batch_plane(fmt, w, N, K) for w in mats]
            x = torch.randn(M, K, device=dev)
            q8 = capi.quantize_q8_1(x)
            y = torch.empty(M, N, device=dev)
            with torch.cuda.stream(stream):
                us = _time_launches(torch, stream,
                                    lambda i: capi.gemv(fmt, mats[i % nmat], q8, M, N, K, out=y, plane=planes[i % nmat]),
                                    args.steps, 60)
            b = synth.gemv_bytes(fmt, N, K, M)
            rows.append({"fmt": names[fmt], "N": N, "K": K, "M": M, "us": round(us, 2),
                         "GBps": round(b / (us * 1e-6) / 1e9, 1), "frac": round(b / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
            if planes[0] is not None:
                rows[-1]["batch_plane"] = True
            del mats, planes
    head = rows[0]
    return _common(args, "GEMV effective GB/s per shape", head["GBps"], "GB/s", round(head["us"] * 1e-3, 5), "int8",
                   {"workload": "single decode GEMVs, batch %d, all formats x layer shapes" % M, "shapes": rows},
                   {"kernel": "Q4_K GEMV N=25600 K=5120", "bound": "hbm", "achieved": head["GBps"],
                    "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": head["frac"], "traffic": None,
                    "us_per_launch": head["us"], "launches_timed": args.steps})


def bench_decode(args, torch, capi, synth, dev):
    """End-to-end greedy decode step of the random-init 64-layer dense model (the layer
    workload's shapes, RMSNorm, RoPE, GQA attention over an fp16 KV cache at context 4096,
    Q6_K lm_head 5120 -> 152064): tokens per second, with the share of the step that the
    quantized-linear launches take when they run alone."""
    from llaminar_amd.capi import FMT_Q4_K, FMT_Q6_K
    from llaminar_amd.decoder import DenseDecoder, Shape

    B = args.batch
    shape = Shape(n_layers=args.decode_layers)
    ctx = args.context
    cap = (ctx + args.steps + args.warmup + 8 + 31) // 32 * 32   # the caches are kept in tiles of 16 and 32 positions
    t_build = time.perf_counter()
    dec = DenseDecoder(shape, B, cap, dev, seed=11, keep_prepared=True, batch_planes=False if args.no_batch_planes else None)
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    for l in range(shape.n_layers):   # a cache as `ctx - 1` earlier tokens would have left it
        k, v = dec.buffer("kcache", l), dec.buffer("vcache", l)
        # (random values: the tiles' order inside the caches does not matter to what the step costs)
        k.copy_(torch.randn(B, shape.n_kv, cap, shape.head_dim, device=dev, generator=g))
        v.copy_(torch.randn(B, shape.n_kv, cap, shape.head_dim, device=dev, generator=g))
    ids0 = torch.randint(0, shape.vocab, (B,), generator=torch.Generator().manual_seed(5)).numpy()
    dec.set_state(ids0, [ctx - 1] * B)
    torch.cuda.synchronize()
    t_build = time.perf_counter() - t_build

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        dec.step(stream)
        stream.synchronize()
        graph = None
        if not args.no_graph:
            graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(graph, stream=stream):
                dec.step(stream)
        run = (lambda: graph.replay()) if graph is not None else (lambda: dec.step(stream))
        if graph is not None:
            dec.advance(max(args.warmup - 1, 1) + args.steps)  # replays do not pass through dec.step()
        for _ in range(max(args.warmup - 1, 1)):
            run()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        ms = (t1 - t0) * 1e3 / args.steps
        tokens = dec.buffer("ids").cpu().tolist()
        last_pos = dec.buffer("pos").cpu().tolist()

        # the quantized-linear launches of the same step alone (quantisers, GEMVs, lm_head)
        H, QD, KV, F = shape.hidden, shape.n_heads * shape.head_dim, shape.n_kv * shape.head_dim, shape.ffn
        x = torch.randn(B, H, device=dev)
        attn = torch.randn(B, QD, device=dev)
        q8 = torch.empty(B * (max(H, QD) // 32) * 36, dtype=torch.uint8, device=dev)
        q8a = torch.empty(B * (F // 32) * 36, dtype=torch.uint8, device=dev)
        qkv = torch.empty(B, QD + 2 * KV, device=dev)
        o = torch.empty(B, H, device=dev)
        gate = torch.randn(B, F, device=dev)
        up = torch.randn(B, F, device=dev)
        logits = torch.empty(B, shape.vocab, device=dev)
        W = dec.prepared
        P = lambda name: dec.planes.get(name)   # the matrix's batch plane, if the decoder built one

        fused_ffn = (capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, B, F, H) and
                     (P("0.wgate") is None) == (P("0.wup") is None))
        split_down = capi.gemv_plane_split_supported(FMT_Q6_K, B, H, F)
        o_hi = torch.empty(B, H, device=dev)

        def linear_only():
            for l in range(shape.n_layers):
                capi.quantize_q8_1(x, out=q8)
                capi.gemv_fused([(FMT_Q4_K, W[f"{l}.wq"], qkv[:, :QD], P(f"{l}.wq")),
                                 (FMT_Q4_K, W[f"{l}.wk"], qkv[:, QD:QD + KV], P(f"{l}.wk")),
                                 (FMT_Q6_K, W[f"{l}.wv"], qkv[:, QD + KV:], P(f"{l}.wv"))], q8, B, H)
                capi.gemv_fused_f32([(FMT_Q4_K, W[f"{l}.wo"], o, P(f"{l}.wo"))], attn, B, QD, q8_scratch=q8)
                capi.quantize_q8_1(x, out=q8)
                if fused_ffn:   # as the decoder does at these batches: gate, up, SwiGLU and its quantiser in one launch
                    capi.gemv_gate_up_swiglu(FMT_Q4_K, W[f"{l}.wgate"], W[f"{l}.wup"], q8, B, F, H,
                                             plane_gate=P(f"{l}.wgate"), plane_up=P(f"{l}.wup"), q8_out=q8a)
                    if split_down and P(f"{l}.wdown") is not None:
                        capi.gemv_plane_split(FMT_Q6_K, P(f"{l}.wdown"), q8a, B, H, F, out_lo=o, out_hi=o_hi)
                    else:
                        capi.gemv(FMT_Q6_K, W[f"{l}.wdown"], q8a, B, H, F, out=o, plane=P(f"{l}.wdown"))
                    continue
                capi.gemv_fused([(FMT_Q4_K, W[f"{l}.wgate"], gate, P(f"{l}.wgate")),
                                 (FMT_Q4_K, W[f"{l}.wup"], up, P(f"{l}.wup"))], q8, B, H)
                capi.gemv_swiglu_f32(FMT_Q6_K, W[f"{l}.wdown"], gate, up, B, H, F, out=o, q8_scratch=q8a,
                                     plane=P(f"{l}.wdown"))
            capi.quantize_q8_1(x, out=q8)
            capi.gemv(FMT_Q6_K, W["lm_head"], q8, B, shape.vocab, H, out=logits, plane=P("lm_head"))

        linear_only()
        stream.synchronize()
        lin = torch.cuda.CUDAGraph()
        with torch.cuda.graph(lin, stream=stream):
            linear_only()
        for _ in range(3):
            lin.replay()
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        reps = max(5, args.steps // 4)
        for _ in range(reps):
            lin.replay()
        torch.cuda.synchronize()
        ms_lin = (time.perf_counter() - t0) * 1e3 / reps

    wbytes = shape.weight_bytes_per_token()
    kv_bytes = shape.n_layers * B * 2 * shape.n_kv * ctx * shape.head_dim * 2
    achieved = (wbytes + kv_bytes) / (ms * 1e-3) / 1e9
    value = B * 1e3 / ms
    cfg = {"workload": "end-to-end greedy decode step, random-init %d-layer dense model (hidden 5120, 64x128 heads, "
                       "8 KV heads, ffn 25600; Q4_K projections, Q6_K V/down/lm_head 5120->152064, Q4_K embedding), "
                       "RMSNorm, RoPE theta 1e6, fp16 KV cache at context %d, batch %d" % (shape.n_layers, ctx, B),
           "batch": B, "context": ctx, "layers": shape.n_layers, "batch_planes": bool(dec.planes),
           "weight_bytes_per_step": wbytes, "kv_bytes_per_step": kv_bytes,
           "linear_only_ms": round(ms_lin, 4), "gemv_share_of_step": round(ms_lin / ms, 4),
           "hbm_bound_tokens_per_s": round(B * HBM_PEAK_GBS * 1e9 / (wbytes + kv_bytes), 1),
           "launch": "eager" if graph is None else "hip-graph replay of the whole step",
           "build_seconds": round(t_build, 1), "device_bytes_buffers": dec.device_bytes(),
           "last_tokens": tokens, "last_positions": last_pos}
    roof = {"kernel": "whole decode step (weights of every projection and the KV cache read once)", "bound": "hbm",
            "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS, "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4), "traffic": None,
            "bytes_per_launch": wbytes + kv_bytes, "us_per_launch": round(ms * 1e3, 1), "launches_timed": args.steps}
    out = _common(args, "decode tokens/s (greedy, batch %d)" % B, round(value, 2), "tokens/s", round(ms, 4), "int8",
                  cfg, roof)
    dec.close()
    return out


def bench_read_order(args, torch, capi, synth, dev):
    """What the order of a GEMV's reads is worth on its own: read-only kernels over 25600 x 5120 Q4_K-sized buffers
    (73.7 MB each, eight rotated so nothing is served from a previous launch), no arithmetic."""
    from tests.probe import binding as probe   # measurement-only library, not part of the product

    lib = probe.load()
    N, K = FFN, HIDDEN
    nbytes = N * (K // 256) * 144
    bufs = [torch.randint(0, 256, (nbytes,), dtype=torch.uint8, device=dev) for _ in range(8)]
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    stream = torch.cuda.Stream()
    # (label, pattern, rows per wavefront, wavefronts per workgroup, depth, workgroups)
    cases = [("quad-lane loads, 13 contiguous rows per wavefront, 2 steps in flight", 0, 13, 8, 2, 0),
             ("quad-lane loads, rows dealt round robin, 2 steps in flight", 1, 13, 8, 2, 0),
             ("quad-lane loads, contiguous rows, 1 step in flight", 0, 13, 8, 1, 0),
             ("quad-lane loads, round robin, 1 step in flight", 1, 13, 8, 1, 0),
             ("quad-lane loads, contiguous rows, 4 steps in flight", 0, 13, 8, 4, 0),
             ("quad-lane loads, round robin, 4 steps in flight", 1, 13, 8, 4, 0),
             ("quad-lane loads, 7 contiguous rows, 16 wavefronts, 1 step in flight", 0, 7, 16, 1, 0),
             ("quad-lane loads, 7 rows round robin, 16 wavefronts, 1 step in flight", 1, 7, 16, 1, 0),
             ("three planes, round robin, 2 steps in flight", 5, 13, 8, 2, 0),
             ("three planes, round robin, 3 steps in flight", 5, 13, 8, 3, 0),
             ("three planes, round robin, 4 steps in flight", 5, 13, 8, 4, 0),
             ("three planes, contiguous rows, 2 steps in flight", 4, 13, 8, 2, 0),
             ("three planes, 7 rows round robin, 16 wavefronts, 1 step in flight", 5, 7, 16, 1, 0),
             ("three planes, 7 rows round robin, 16 wavefronts, 2 steps in flight", 5, 7, 16, 2, 0),
             ("quad-lane loads, round robin, 3 steps in flight", 1, 13, 8, 3, 0),
             ("1 KB stream, region per wavefront, 256 x 1024 threads, 3 loads in flight", 2, 0, 16, 3, 256),
             ("1 KB stream, grid-stride, 256 x 1024 threads, 3 loads in flight", 3, 0, 16, 3, 256),
             ("1 KB stream, region per wavefront, 256 x 1024 threads, 6 loads in flight", 2, 0, 16, 6, 256),
             ("1 KB stream, grid-stride, 256 x 1024 threads, 6 loads in flight", 3, 0, 16, 6, 256),
             ("1 KB stream, grid-stride, 256 x 1024 threads, 9 loads in flight", 3, 0, 16, 9, 256)]
    rows = []
    with torch.cuda.stream(stream):
        for label, pattern, rpw, wpw, depth, wgs in cases:
            def launch(i):
                ok = lib.llam_probe_read(bufs[i % 8].data_ptr(), N, K, pattern, rpw, wpw, depth, wgs,
                                            sink.data_ptr(), 0, stream.cuda_stream)
                assert ok, capi.last_error()
            us = min(_time_launches(torch, stream, launch, args.steps, 20) for _ in range(3))
            rows.append({"pattern": label, "us": round(us, 2), "frac": round(nbytes / (us * 1e-6) / 1e9 / HBM_PEAK_GBS, 4)})
    best = min(rows, key=lambda r: r["us"])
    gbs = round(nbytes / (best["us"] * 1e-6) / 1e9, 1)
    return _common(args, "read-only stream GB/s by order of reads", gbs, "GB/s", round(best["us"] * 1e-3, 5), "u8",
                   {"workload": "read-only probes over 25600 x 5120 Q4_K-sized buffers (73.7 MB), 8 rotated", "patterns": rows},
                   {"kernel": best["pattern"], "bound": "hbm", "achieved": gbs, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                    "frac": best["frac"], "traffic": None, "us_per_launch": best["us"], "launches_timed": args.steps})


OTHER_WORKLOADS = {"gemm": bench_gemm, "moe": bench_moe, "gemv": bench_gemv, "decode": bench_decode,
                   "read-order": bench_read_order}


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--moe-path", choices=["auto", "slots", "grouped-gate-up", "grouped"], default="auto",
                    help="moe workload: per-slot launches, or tokens grouped by expert (gate/up only, or down as well)")
    ap.add_argument("--workload", choices=["layer", "gemm", "moe", "gemv", "decode", "read-order"], default="layer",
                    help="layer: the headline decode-layer step (default); gemm: prefill int8 GEMM 512x25600x5120 Q4_K; "
                         "moe: 256-expert top-8 IQ3_S expert FFN decode; gemv: single GEMVs of every format and layer shape; "
                         "read-order: read-only probes of the GEMV's load stream in several orders")
    ap.add_argument("--batch", type=int, default=1, help="activation rows / tokens per step")
    ap.add_argument("--layers", type=int, default=4, help="distinct weight sets rotated through")
    ap.add_argument("--no-graph", action="store_true", help="launch eagerly instead of replaying HIP graphs")
    ap.add_argument("--context", type=int, default=4096, help="decode workload: tokens in the KV cache")
    ap.add_argument("--decode-layers", type=int, default=64, help="decode workload: layers of the model")
    ap.add_argument("--separate-quantise", action="store_true",
                    help="layer workload: quantiser kernels of their own instead of the fp32-input GEMV calls")
    ap.add_argument("--no-batch-planes", action="store_true",
                    help="batches of 5..8: no batch planes beside the prepared matrices (llam_ql_build_batch_plane)")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-decode", action="store_true",
                    help="layer workload at batch 1: skip the short run of the 64-layer decode step")
    ap.add_argument("--no-extras", action="store_true",
                    help="layer workload at batch 1: skip the short runs of the prefill GEMM and the MoE decode")
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
    if args.workload != "layer":
        print(json.dumps(OTHER_WORKLOADS[args.workload](args, torch, capi, synth, dev)))
        return
    assert 1 <= M <= capi.MAX_GEMV_M

    projs = [("q", QDIM, HIDDEN, FMT_Q4_K), ("k", KVDIM, HIDDEN, FMT_Q4_K), ("v", KVDIM, HIDDEN, FMT_Q6_K),
             ("o", HIDDEN, QDIM, FMT_Q4_K), ("gate", FFN, HIDDEN, FMT_Q4_K), ("up", FFN, HIDDEN, FMT_Q4_K),
             ("down", HIDDEN, FFN, FMT_Q6_K)]
    layers = []
    n_planes = 0
    for l in range(args.layers):
        w = {}
        for i, (name, N, K, fmt) in enumerate(projs):
            raw = synth.weights_torch(fmt, N, K, 1000 * l + i, dev)
            w[name] = capi.prepare_weights(fmt, raw, N, K)
            del raw
            # batches of 5..8 rows: the projections of 4096 rows and more read their weights from batch planes; batches
            # of 2..4: the feed-forward matrices only (the launches that name the matrix unit serve them)
            w["plane_" + name] = None
            if ((M >= 5 or (M >= 2 and name in ("gate", "up", "down"))) and N >= 4096 and not args.no_batch_planes and
                    capi.batch_plane_bytes(fmt, N, K) > 0):
                w["plane_" + name] = capi.build_batch_plane(fmt, w[name], N, K)
                n_planes += 1
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

    # batches the matrix unit serves: gate, up, SwiGLU and the Q8_1 quantiser of the result as one launch
    fused_ffn = capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, M, FFN, HIDDEN)
    split_down = capi.gemv_plane_split_supported(FMT_Q6_K, M, HIDDEN, FFN)
    down_hi = torch.empty(M, HIDDEN, device=dev)

    def ffn_fused(w):
        capi.quantize_q8_1(x2, out=q8_x2)
        capi.gemv_gate_up_swiglu(FMT_Q4_K, w["gate"], w["up"], q8_x2, M, FFN, HIDDEN, plane_gate=w["plane_gate"],
                                 plane_up=w["plane_up"], q8_out=q8_act)
        if split_down and w["plane_down"] is not None:   # the rows' halves as two partial sums (the next norm adds them)
            capi.gemv_plane_split(FMT_Q6_K, w["plane_down"], q8_act, M, HIDDEN, FFN, out_lo=down, out_hi=down_hi)
        else:
            capi.gemv(FMT_Q6_K, w["down"], q8_act, M, HIDDEN, FFN, out=down, plane=w["plane_down"])

    def step_separate(w):
        # quantiser kernels of their own, Q8_1 blocks through memory
        capi.quantize_q8_1(x, out=q8_x)
        capi.gemv_fused([(FMT_Q4_K, w["q"], qkv[:, :QDIM], w["plane_q"]),
                         (FMT_Q4_K, w["k"], qkv[:, QDIM:QDIM + KVDIM], w["plane_k"]),
                         (FMT_Q6_K, w["v"], qkv[:, QDIM + KVDIM:], w["plane_v"])], q8_x, M, HIDDEN)
        capi.quantize_q8_1(attn, out=q8_attn)
        capi.gemv(FMT_Q4_K, w["o"], q8_attn, M, HIDDEN, QDIM, out=o_out, plane=w["plane_o"])
        if fused_ffn:
            return ffn_fused(w)
        capi.quantize_q8_1(x2, out=q8_x2)
        capi.gemv_fused([(FMT_Q4_K, w["gate"], gate, w["plane_gate"]), (FMT_Q4_K, w["up"], up, w["plane_up"])],
                        q8_x2, M, HIDDEN)
        ok = lib.llam_ql_swiglu_quantize(gate.data_ptr(), up.data_ptr(), None, q8_act.data_ptr(), M, FFN, 0,
                                         torch.cuda.current_stream().cuda_stream)
        assert ok, capi.last_error()
        capi.gemv(FMT_Q6_K, w["down"], q8_act, M, HIDDEN, FFN, out=down, plane=w["plane_down"])

    def step_fp32(w):
        # the operator's fp32-input calls: every GEMV quantises its input itself (same bits)
        capi.gemv_fused_f32([(FMT_Q4_K, w["q"], qkv[:, :QDIM], w["plane_q"]),
                             (FMT_Q4_K, w["k"], qkv[:, QDIM:QDIM + KVDIM], w["plane_k"]),
                             (FMT_Q6_K, w["v"], qkv[:, QDIM + KVDIM:], w["plane_v"])], x, M, HIDDEN, q8_scratch=q8_x)
        capi.gemv_fused_f32([(FMT_Q4_K, w["o"], o_out, w["plane_o"])], attn, M, QDIM, q8_scratch=q8_attn)
        if fused_ffn:
            return ffn_fused(w)
        capi.gemv_fused_f32([(FMT_Q4_K, w["gate"], gate, w["plane_gate"]), (FMT_Q4_K, w["up"], up, w["plane_up"])],
                            x2, M, HIDDEN, q8_scratch=q8_x2)
        capi.gemv_swiglu_f32(FMT_Q6_K, w["down"], gate, up, M, HIDDEN, FFN, out=down, q8_scratch=q8_act,
                             plane=w["plane_down"])
        # (with the scratch buffers given, the library quantises inside the GEMV only where that is
        # cheaper than a quantiser launch: single short rows)

    step = step_separate if args.separate_quantise else step_fp32

    bytes_per_step = sum(synth.gemv_bytes(fmt, N, K, M) for _, N, K, fmt in projs)
    bytes_per_step += M * (2 * HIDDEN + QDIM) * 4 + M * 2 * FFN * 4  # fp32 read by the quantisers

    stream = torch.cuda.Stream()
    graphs = None
    with torch.cuda.stream(stream):
        for i in range(max(args.warmup, 1)):
            step(layers[i % args.layers])
        stream.synchronize()
        group = None
        if not args.no_graph:
            # one graph per weight set, and one graph of `layers` consecutive steps (a decode
            # pass captures all of its layers in one graph: one graph launch per pass)
            graphs = []
            for w in layers:
                gr = torch.cuda.CUDAGraph()
                with torch.cuda.graph(gr, stream=stream):
                    step(w)
                graphs.append(gr)
            group = torch.cuda.CUDAGraph()
            with torch.cuda.graph(group, stream=stream):
                for w in layers:
                    step(w)
            for gr in graphs + [group]:
                gr.replay()
            stream.synchronize()

        torch.cuda.synchronize()
        t0 = time.perf_counter()
        if graphs is not None:
            whole, rest = divmod(args.steps, args.layers)
            for i in range(whole):
                group.replay()
            for i in range(rest):
                graphs[i].replay()
        else:
            for i in range(args.steps):
                step(layers[i % args.layers])
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        layer_ms = (t1 - t0) * 1e3 / args.steps
        layer_gbs = bytes_per_step / (layer_ms * 1e-3) / 1e9

        # ---- the metric's own shape: Q4_K GEMV 25600 x 5120 at batch 1 ---------------------------
        # One step = one launch.  The launches rotate over 2*layers distinct matrices (gate and up
        # of every layer: 8 x 73.7 MB, beyond the 256 MB Infinity Cache).  The K timed steps are
        # one HIP graph of K launches (no host launch gaps), bracketed by synchronisation on both
        # sides and timed with events on the launch stream.
        mats = [l[n] for l in layers for n in ("gate", "up")]
        q8_1 = q8_x2[: (HIDDEN // 32) * 36]
        y = torch.empty(1, FFN, device=dev)
        k_bytes = synth.gemv_bytes(FMT_Q4_K, FFN, HIDDEN, 1)

        def launches(n, first=0):
            for i in range(n):
                capi.gemv(FMT_Q4_K, mats[(first + i) % len(mats)], q8_1, 1, FFN, HIDDEN, out=y)

        def timed(fn):
            e0 = torch.cuda.Event(enable_timing=True)
            e1 = torch.cuda.Event(enable_timing=True)
            torch.cuda.synchronize()
            e0.record(stream)
            fn()
            e1.record(stream)
            torch.cuda.synchronize()
            return e0.elapsed_time(e1) * 1e3  # microseconds

        launches(max(args.warmup, 50))   # W untimed warm-up steps (at least 50: clocks and caches settle)
        if args.no_graph:
            k_total_us = timed(lambda: launches(args.steps))
        else:
            kgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(kgraph, stream=stream):
                launches(args.steps)
            kgraph.replay()   # untimed: the first replay of a graph pays its upload
            k_total_us = timed(kgraph.replay)
        ms_per_step = k_total_us * 1e-3 / args.steps
        value = k_bytes / (ms_per_step * 1e-3) / 1e9

        # ---- roofline of that kernel: at least 200 launches whatever --steps says -----------------
        # chunks of 40 launches (five rounds over the eight matrices), each chunk one graph replay
        # timed with its own pair of events: mean over all launches, median and minimum of the chunks
        chunk = 5 * len(mats)
        n_chunks = max(5, (max(args.steps, 200) + chunk - 1) // chunk)
        if args.no_graph:
            run_chunk = lambda: launches(chunk)
        else:
            cgraph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(cgraph, stream=stream):
                launches(chunk)
            run_chunk = cgraph.replay
        run_chunk()
        run_chunk()
        chunk_us = sorted(timed(run_chunk) / chunk for _ in range(n_chunks))
        reps = n_chunks * chunk
        k_us = sum(chunk_us) / n_chunks
        k_us_median = chunk_us[n_chunks // 2]
        k_us_min = chunk_us[0]
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
        "ms_per_step": round(ms_per_step, 6),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8",
        "data": "synthetic",
        "config": {
            "workload": "Q4_K decode GEMV 25600 x 5120 (the gate/up projection of a 27B/32B-class dense decoder layer), "
                        "batch 1, Q8_1 activations; one step = one launch, %d distinct matrices rotated" % len(mats),
            "batch": 1,
            "bytes_per_step": k_bytes,
            "pct_of_hbm_peak": round(100.0 * value / HBM_PEAK_GBS, 2),
            "launch": "eager" if graphs is None else "hip-graph replay of the K steps",
            # the whole layer the kernel belongs to (BASELINE config 2): all seven projections of one layer
            "layer_step": {
                "workload": "one dense decoder layer's linear projections, decode batch %d: Q 5120->8192, K/V 5120->1024, "
                            "O 8192->5120, gate/up 5120->25600 in Q4_K, V 5120->1024 and down 25600->5120 in Q6_K; "
                            "Q8_1 activations" % M,
                "batch": M,
                "value": round(layer_gbs, 1),
                "unit": "GB/s",
                "us_per_step": round(layer_ms * 1e3, 2),
                "bytes_per_step": bytes_per_step,
                "pct_of_hbm_peak": round(100.0 * layer_gbs / HBM_PEAK_GBS, 2),
                "distinct_weight_sets": args.layers,
                "batch_planes": n_planes // max(args.layers, 1),   # projections per layer read from batch planes (batches of 5..8)
                "fused_ffn": bool(fused_ffn),   # gate + up + SwiGLU + Q8_1 in one launch (batches of 5..8)
                "split_down": bool(split_down and n_planes > 0),   # down projection summed in two halves (batches of 5..8)
                "steps": args.steps,
                "launch": "eager" if graphs is None else "hip-graph replay",
            },
        },
        "roofline": {
            "kernel": "gemv_quad_kernel<Q4KQuad, 1 activation row, 1 step per load chunk, Q8_1 input, row sums "
                      "through the LDS ring> N=25600 K=5120",
            "bound": "hbm",
            "achieved": round(achieved, 1),
            "peak": HBM_PEAK_GBS,
            "unit": "GB/s",
            "frac": round(achieved / HBM_PEAK_GBS, 4),
            "traffic": dominant_traffic_bytes(),
            "bytes_per_launch": k_bytes,
            "us_per_launch": round(k_us, 3),
            "us_per_launch_median": round(k_us_median, 3),
            "us_per_launch_min": round(k_us_min, 3),
            "frac_median": round(k_bytes / (k_us_median * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "frac_best": round(k_bytes / (k_us_min * 1e-6) / 1e9 / HBM_PEAK_GBS, 4),
            "launches_timed": reps,
            "timing": "HIP events on the launch stream around graph replays of %d launches each" % chunk,
        },
        "cpu_baseline": cpu,
    }
    if M == 1 and not args.no_decode:
        # the metric's second figure: tokens per second of the whole 64-layer decode step at
        # batch 1 (the `decode` workload, a shorter run of it), reported beside the headline
        layers = graphs = group = None
        torch.cuda.empty_cache()
        try:
            sub = argparse.Namespace(**vars(args))
            sub.steps, sub.warmup = 24, 4
            d = bench_decode(sub, torch, capi, synth, dev)
            out["config"]["decode_step"] = {
                "tokens_per_s": d["value"], "ms_per_token": d["ms_per_step"], "layers": d["config"]["layers"],
                "context": d["config"]["context"], "gemv_share_of_step": d["config"]["gemv_share_of_step"],
                "frac_of_hbm_bound": round(d["value"] / d["config"]["hbm_bound_tokens_per_s"], 4),
                "steps": sub.steps, "workload": "bench.py --workload decode"}
        except Exception as e:  # noqa: BLE001 - the headline figure must still be reported
            out["config"]["decode_step"] = {"error": str(e)[:200]}
    if M == 1 and not args.no_decode and not args.no_extras:
        # the same step for eight sequences at once (the matrix-unit kernels and, unless --no-batch-planes, the
        # batch planes beside the prepared matrices)
        torch.cuda.empty_cache()
        try:
            sub = argparse.Namespace(**vars(args))
            sub.steps, sub.warmup, sub.batch = 24, 4, 8
            d = bench_decode(sub, torch, capi, synth, dev)
            out["config"]["decode_step_batch8"] = {
                "tokens_per_s": d["value"], "ms_per_step": d["ms_per_step"], "batch_planes": d["config"]["batch_planes"],
                "steps": sub.steps, "workload": "bench.py --workload decode --batch 8"}
        except Exception as e:  # noqa: BLE001
            out["config"]["decode_step_batch8"] = {"error": str(e)[:200]}
    if M == 1 and not args.no_extras:
        # the other configurations of the baseline, short runs of their own workloads, each with
        # its own roofline fraction: the prefill GEMM (int8 matrix-unit peak) and the MoE expert
        # FFN decode at 1 and 16 tokens (HBM peak over the distinct experts' bytes)
        layers = graphs = group = mats = None
        torch.cuda.empty_cache()

        def brief(d, extra):
            r = d["roofline"]
            o = {"value": d["value"], "unit": d["unit"], "us_per_step": round(d["ms_per_step"] * 1e3, 2),
                 "roofline": {"bound": r["bound"], "achieved": r["achieved"], "peak": r["peak"], "unit": r["unit"],
                              "frac": r["frac"]}}
            o.update(extra)
            return o

        try:
            sub = argparse.Namespace(**vars(args))
            sub.workload, sub.batch, sub.steps, sub.warmup = "gemm", 512, 20, 3
            d = bench_gemm(sub, torch, capi, synth, dev)
            out["config"]["prefill_gemm"] = brief(d, {"M": 512, "N": FFN, "K": HIDDEN, "fmt": "Q4_K",
                                                      "workload": "bench.py --workload gemm"})
        except Exception as e:  # noqa: BLE001
            out["config"]["prefill_gemm"] = {"error": str(e)[:200]}
        torch.cuda.empty_cache()
        moe = []
        for tokens in (1, 16):
            try:
                sub = argparse.Namespace(**vars(args))
                sub.workload, sub.batch, sub.steps, sub.warmup = "moe", tokens, 128, 4
                d = bench_moe(sub, torch, capi, synth, dev)
                moe.append(brief(d, {"tokens": tokens, "path": d["config"]["path"],
                                     "distinct_experts_per_step": d["config"]["distinct_experts_per_step"],
                                     "tokens_per_s": d["config"]["tokens_per_s"],
                                     "workload": "bench.py --workload moe --batch %d" % tokens}))
            except Exception as e:  # noqa: BLE001
                moe.append({"tokens": tokens, "error": str(e)[:200]})
            torch.cuda.empty_cache()
        out["config"]["moe_decode"] = moe
    print(json.dumps(out))


if __name__ == "__main__":
    main()
