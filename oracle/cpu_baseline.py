"""TEST/BENCH INFRASTRUCTURE: time the CPU path on a bounded sample and print one
JSON object.  Run as a subprocess by bench.py's cpu_baseline leg.

kind "reference": the reference's own AVX512-VNNI GEMV (oracle/_ref), when that
library was built and this host has the instruction sets it was compiled for;
kind "port": the scalar C restatement (oracle/ql_oracle.c, OpenMP over rows).

Sample: the headline kernel's shape -- Q4_K GEMV, N=25600 x K=5120, batch 1 --
on seeded synthetic blocks; GB/s counts the same algorithmic bytes as the GPU
figure (GGUF weight bytes + Q8_1 activations + fp32 outputs).
"""
from __future__ import annotations

import json
import os
import sys
import time
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent
sys.path.insert(0, str(ROOT))

from oracle.binding import BLOCK_BYTES, FMT_Q4_K, Oracle, Ref  # noqa: E402

NEEDED = {"avx512f", "avx512bw", "avx512vl", "avx512dq", "avx512_vnni", "avx2", "fma", "f16c"}


def cpu_flags() -> set:
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("flags"):
                return set(line.split(":", 1)[1].split())
    except OSError:
        pass
    return set()


def cpu_topology() -> dict:
    """Sockets, physical cores and logical CPUs of this host, from /proc/cpuinfo."""
    cores, sockets, logical, model = set(), set(), 0, ""
    phys = core = None
    try:
        for line in open("/proc/cpuinfo"):
            key, _, val = line.partition(":")
            key, val = key.strip(), val.strip()
            if key == "processor":
                logical += 1
                phys = core = None
            elif key == "model name" and not model:
                model = val
            elif key == "physical id":
                phys = val
                sockets.add(val)
            elif key == "core id":
                core = val
            if phys is not None and core is not None:
                cores.add((phys, core))
    except OSError:
        pass
    return {"sockets": len(sockets) or None, "physical_cores": len(cores) or None, "logical_cpus": logical or None,
            "model": model}


def main():
    N, K, fmt = 25600, 5120, FMT_Q4_K
    budget_s = float(os.environ.get("QL_CPU_BASELINE_SECONDS", "12"))
    rng = np.random.default_rng(1)
    W = rng.integers(0, 256, size=(N, K // 256, BLOCK_BYTES[fmt]), dtype=np.uint8)
    for off in (0, 2):
        d = rng.uniform(0.001, 0.02, size=(N, K // 256)).astype(np.float16)
        W[:, :, off:off + 2] = d.view(np.uint8).reshape(N, K // 256, 2)
    x = rng.standard_normal((1, K)).astype(np.float32)
    o = Oracle()
    q8 = o.quantize(x)
    nbytes = N * (K // 256) * BLOCK_BYTES[fmt] + (K // 32) * 36 + N * 4
    threads = int(os.environ.get("OMP_NUM_THREADS", os.cpu_count() or 1))

    use_ref = Ref.available() and NEEDED <= cpu_flags() and os.environ.get("QL_CPU_BASELINE_KIND", "") != "port"
    times = []
    # Like the reference's own perf harness (tests/v2/performance/kernels/cpu/native_vnni/
    # Perf__CPUNativeVNNI_GEMV.cpp:856) the packed weights are pushed out of the caches before
    # every timed call: sweep a buffer larger than any last-level cache.
    flush = np.zeros(int(os.environ.get("QL_CPU_FLUSH_MB", "768")) * (1 << 20) // 8, np.float64)

    def flush_caches():
        np.add(flush, 1.0, out=flush)

    flush_caches()  # first touch of the pages happens outside the timed budget

    if use_ref:
        r = Ref()
        threads = r.omp_threads()
        h = r.pack(fmt, W, N, K)
        packed = r.pack_bytes(h)
        C = np.zeros((1, N), np.float32)
        for _ in range(3):
            r.gemm_packed(h, q8, N, isa=0, out=C)
        t_end = time.perf_counter() + budget_s
        while time.perf_counter() < t_end and len(times) < 5000:
            flush_caches()
            t0 = time.perf_counter()
            r.gemm_packed(h, q8, N, isa=0, out=C)
            times.append(time.perf_counter() - t0)
        r.pack_free(h)
        kind = "reference"
        detail = f"reference AVX512-VNNI gemv_native_vnni_preq, packed {packed / 1e6:.1f} MB"
    else:
        # scalar port: decode + dot per call (the restatement keeps no packed form)
        rows = 2048  # bounded sample of the rows; GB/s scales linearly in rows
        nbytes = rows * (K // 256) * BLOCK_BYTES[fmt] + (K // 32) * 36 + rows * 4
        Wp = np.ascontiguousarray(W[:rows])
        o.gemm(fmt, Wp, K, q8)
        t_end = time.perf_counter() + budget_s
        while time.perf_counter() < t_end and len(times) < 200:
            flush_caches()
            t0 = time.perf_counter()
            o.gemm(fmt, Wp, K, q8)
            times.append(time.perf_counter() - t0)
        kind = "port"
        detail = f"scalar C restatement on {rows} of {N} rows, OpenMP over rows"
    med = float(np.median(times))
    del flush
    try:
        stream_gbs = round(o.stream_triad_gbs(), 1)
    except Exception:  # noqa: BLE001 - an older oracle library without the routine
        stream_gbs = None
    topo = cpu_topology()
    print(json.dumps({
        "value": nbytes / med / 1e9,
        "unit": "GB/s",
        "cores": threads,
        "kind": kind,
        "host": topo,
        "host_dram_stream_triad_gbs": stream_gbs,
        "frac_of_host_dram": (round(nbytes / med / 1e9 / stream_gbs, 3) if stream_gbs else None),
        "sample": f"Q4_K GEMV N={N} K={K} batch 1, {len(times)} timed calls with the caches flushed before each "
                  f"(median {med * 1e3:.3f} ms, min {min(times) * 1e3:.3f} ms), {detail}",
    }))


if __name__ == "__main__":
    main()
