"""Writes tests/golden/ql_goldens.npz from the REFERENCE's own CPU code.

Runs only where oracle/_ref/libllaminar_ref.so exists (it is compiled from the
reference's headers by oracle/Makefile and cannot travel).  Every output array
below is produced by reference routines -- the fp16 converters, the Q8_1
quantisers (dispatch / scalar / AVX2 / AVX512 variants), the per-format
super-block unpackers and the AVX512 / AVX2 GEMV and GEMM kernels -- on seeded
inputs that include the edge cases the reference's tests use (zero and
near-zero blocks, clamping, tails, ties, uniform / alternating / ramp data).
The only derived quantity is `*_bsums`: int64 brute-force dot products of the
reference-produced int8 weights with the reference-produced Q8_1 quants.

Usage: python tests/golden/make_goldens.py
"""
from __future__ import annotations

import sys
from pathlib import Path

import numpy as np

ROOT = Path(__file__).resolve().parent.parent.parent
sys.path.insert(0, str(ROOT))

from oracle.binding import BLOCK_BYTES, FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K, Ref  # noqa: E402

OUT = Path(__file__).resolve().parent / "ql_goldens.npz"
FMTS = {"q4k": FMT_Q4_K, "q6k": FMT_Q6_K, "iq3s": FMT_IQ3_S}


def weights(rng, fmt, n, sb, d_lo=0.001, d_hi=0.02):
    bb = BLOCK_BYTES[fmt]
    w = rng.integers(0, 256, size=(n, sb, bb), dtype=np.uint8)
    offs = {FMT_Q4_K: (0, 2), FMT_Q6_K: (208,), FMT_IQ3_S: (0,)}[fmt]
    for off in offs:
        d = rng.uniform(d_lo, d_hi, size=(n, sb)).astype(np.float16)
        w[:, :, off:off + 2] = d.view(np.uint8).reshape(n, sb, 2)
    return w


def q8_inputs(rng):
    """[n,32] fp32 rows covering the reference quantiser tests' cases."""
    rows = []
    rows.append(rng.standard_normal((64, 32)).astype(np.float32))                      # random
    rows.append(rng.uniform(-1, 1, (16, 32)).astype(np.float32))                       # uniform
    rows.append(np.tile(np.array([1.0, -1.0], np.float32), 16)[None])                  # alternating
    rows.append(np.linspace(-3, 3, 32, dtype=np.float32)[None])                        # ramp
    rows.append(np.zeros((1, 32), np.float32))                                         # zero block
    rows.append(np.full((1, 32), 5e-11, np.float32))                                   # below threshold
    rows.append(np.full((1, 32), 2e-10, np.float32))                                   # just above threshold
    rows.append((rng.standard_normal((8, 32)) * 1e-7).astype(np.float32))              # fp16-subnormal d
    rows.append((rng.standard_normal((8, 32)) * 3e4).astype(np.float32))               # large magnitudes
    x = np.zeros((1, 32), np.float32); x[0, 5] = 127.0; x[0, 6] = -127.0               # exact +-127
    rows.append(x)
    # exact .5 ties after scaling: amax = 127 -> id == 1, values k + 0.5
    t = np.arange(32, dtype=np.float32) - 15.5
    t[0] = 127.0
    rows.append(t[None])
    rows.append(-t[None])
    return np.concatenate(rows, 0)


def main():
    if not Ref.available():
        raise SystemExit("oracle/_ref is not built here: run `make -C oracle` where the reference tree exists")
    r = Ref()
    rng = np.random.default_rng(20251125)
    out = {}

    # ---- fp16 converters ---------------------------------------------------------------
    xs = np.concatenate([
        (rng.standard_normal(4000) * s).astype(np.float32) for s in (1.0, 1e-2, 1e-4, 3e-5, 1e-6, 1e-8, 1e3, 7e4)
    ] + [np.array([0.0, -0.0, 65504.0, 65519.9, 65520.0, 1e9, 6.1035156e-05, 6.0975552e-05, 5.9604645e-08,
                   2.9802322e-08, 2.9802326e-08, 8.940697e-08, 1.4901161e-07], np.float32)])
    out["f16_in"] = xs
    out["f16_sw"] = np.array([r.f32_to_f16(x) for x in xs], np.uint16)        # FP16Utils.h fp32_to_fp16
    out["f16_f16c"] = np.array([r.f32_to_f16_f16c(x) for x in xs], np.uint16)  # _mm_cvtps_ph RNE
    hs = rng.integers(0, 65536, 4000).astype(np.uint16)
    hs = hs[(hs & 0x7C00) != 0x7C00]
    out["h_in"] = hs
    out["h_f32"] = np.array([r.f16_to_f32(int(h)) for h in hs], np.float32)

    # ---- get_scale_min_k4 ----------------------------------------------------------------
    sc12 = rng.integers(0, 256, size=(64, 12), dtype=np.uint8)
    out["k4_in"] = sc12
    out["k4_out"] = np.array([[r.scale_min_k4(j, s) for j in range(8)] for s in sc12], np.uint8)

    # ---- iq3s grid -------------------------------------------------------------------------
    out["iq3s_grid"] = r.iq3s_grid().astype(np.uint32)

    # ---- Q8_1 -------------------------------------------------------------------------------
    x = q8_inputs(rng)
    out["q8_in"] = x
    for name, variant in (("dispatch", 0), ("scalar", 1), ("avx2", 2), ("avx512", 3)):
        out[f"q8_{name}"] = np.stack([r.quantize_block(row, 32, variant) for row in x])
    # tails: valid < 32 always takes the scalar path
    tails = rng.standard_normal((12, 32)).astype(np.float32)
    valid = np.array([1, 2, 3, 5, 8, 13, 16, 17, 24, 30, 31, 31], np.int32)
    out["q8_tail_in"] = tails
    out["q8_tail_valid"] = valid
    out["q8_tail"] = np.stack([r.quantize_block(tails[i], int(valid[i]), 0) for i in range(12)])
    # whole rows through quantize_activations_to_q8_1 (pairs + odd tail block + K % 32 != 0)
    for K in (256, 288, 300):
        a = rng.standard_normal((3, K)).astype(np.float32)
        out[f"q8_rows_in_{K}"] = a
        out[f"q8_rows_{K}"] = r.quantize(a)

    # ---- per-format: effective sub-blocks, GEMV and GEMM --------------------------------------
    N, K = 96, 1024
    act = rng.standard_normal((5, K)).astype(np.float32)
    act[1] *= 0.01
    act[2, 64:128] = 0.0
    q8 = r.quantize(act)
    out["act"] = act
    out["act_q8"] = q8
    qs = q8[:, :, 4:].view(np.int8).astype(np.int64)  # [M, KB, 32]
    for name, fmt in FMTS.items():
        W = weights(rng, fmt, N, K // 256)
        # a few hand-made extremes
        if fmt == FMT_Q4_K:
            W[0, 0, 4:16] = 0          # all scales and mins zero
            W[1, 0, 2:4] = 0           # dmin = 0
            W[2, 1, 16:] = 0xFF        # all nibbles 15
            W[3, 0, 0:2] = np.array([0x0001], np.uint16).view(np.uint8)  # subnormal d -> truncating fp16 branch
        elif fmt == FMT_Q6_K:
            W[0, 0, 192:208] = 0       # all sub-scales zero
            W[1, 0, 192:194] = 0       # one sub-block with max_sc == 0
            W[2, 1, 192:208] = 0x80    # scales -128
            W[3, 0, 192:208] = np.array([1, 16, 3, 16, 16, 1, 16, 3, 127, 2, 5, 10, 7, 14, 9, 18], np.uint8)  # .5 ties
            W[4, 0, 0:192] = 0xFF      # q = 63 everywhere
            W[5, 0, 0:192] = 0x00      # q = 0 everywhere
        else:
            W[0, 0, 106:110] = 0       # all sub-scales nibble 0
            W[1, 0, 0:2] = np.array([0x0400], np.uint16).view(np.uint8)  # d = 2^-14: scale lands in fp16 subnormals
            W[2, 0, 2:66] = 0          # index 0 everywhere (gmax = 1)
            W[2, 0, 66:74] = 0
            W[3, 0, 0:2] = np.array([0x0001], np.uint16).view(np.uint8)  # tiny d: zero-block threshold
        out[f"{name}_w"] = W
        ints, scs, mns = [], [], []
        for n in range(N):
            for s in range(K // 256):
                w, sc, mn = r.unpack_superblock(fmt, W[n, s])
                ints.append(w)
                scs.append([r.f32_to_f16(float(v)) for v in sc])
                mns.append([r.f32_to_f16(float(v)) for v in mn])
        ints = np.array(ints, np.int8).reshape(N, K)
        out[f"{name}_int8"] = ints
        out[f"{name}_scale_h"] = np.array(scs, np.uint16).reshape(N, K // 32)
        out[f"{name}_min_h"] = np.array(mns, np.uint16).reshape(N, K // 32)
        if fmt == FMT_Q6_K:
            # the scalar variant is NOT the definition (may differ by 1); keep it to document that
            out["q6k_int8_scalar_variant"] = np.array(
                [r.unpack_superblock(fmt, W[n, s], 1)[0] for n in range(8) for s in range(K // 256)], np.int8)
            out["q6k_int8_avx2_variant"] = np.array(
                [r.unpack_superblock(fmt, W[n, s], 2)[0] for n in range(8) for s in range(K // 256)], np.int8)
        wi = ints.astype(np.int64).reshape(N, K // 32, 32)
        out[f"{name}_bsums"] = np.einsum("mkb,nkb->mnk", qs, wi).astype(np.int32)
        for M in (1, 4, 5):
            out[f"{name}_c_avx512_m{M}"] = r.gemm(fmt, W, N, K, q8[:M], isa=1)
            out[f"{name}_c_avx2_m{M}"] = r.gemm(fmt, W, N, K, q8[:M], isa=2)

    np.savez_compressed(OUT, **out)
    print(f"wrote {OUT} ({OUT.stat().st_size} bytes, {len(out)} arrays)")


if __name__ == "__main__":
    main()
