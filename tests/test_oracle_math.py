"""Pins on the oracle that need no reference build: library routines, closed
forms, invariants and brute force, chosen so a dropped term, wrong nibble order,
wrong sign or wrong rounding fails one of them."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import BLOCK_BYTES, FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K


def _f16(bits):
    return np.array(bits, np.uint16).view(np.float16).astype(np.float32)


def test_f16_rne_equals_numpy(oracle):
    rng = np.random.default_rng(1)
    xs = np.concatenate([(rng.standard_normal(3000) * s).astype(np.float32)
                         for s in (1, 1e-3, 1e-5, 1e-7, 1e-8, 100, 6e4)])
    with np.errstate(over="ignore"):
        want = xs.astype(np.float16).view(np.uint16)
    got = np.array([oracle.f32_to_f16_rne(x) for x in xs], np.uint16)
    assert np.array_equal(got, want)


def test_f16_sw_truncates_subnormals(oracle):
    # normal range: identical to RNE; subnormal range: floor of |x| / 2^-24
    for x in (1.0, 0.333, 1e-3, 6.2e-5, 65504.0):
        assert oracle.f32_to_f16_sw(x) == oracle.f32_to_f16_rne(x)
    for k in (1, 2, 3, 100, 1023):
        x = np.float32((k + 0.75) * 2.0 ** -24)
        assert oracle.f32_to_f16_sw(x) == k
        assert oracle.f32_to_f16_rne(x) == k + 1
        assert oracle.f32_to_f16_sw(-x) == (0x8000 | k)
    assert oracle.f32_to_f16_sw(np.float32(2.0 ** -26)) == 0
    assert oracle.f16_to_f32(0x0001) == 2.0 ** -24 and oracle.f16_to_f32(0x3C00) == 1.0


def test_q8_1_invariants(oracle):
    x = synth.activations_numpy(16, 1024, 3)
    q = oracle.quantize(x)
    d = _f16(q[:, :, 0:2].copy().view(np.uint16)[..., 0])
    s = q[:, :, 2:4].copy().view(np.int16)[..., 0]
    qs = q[:, :, 4:].view(np.int8)
    xb = x.reshape(16, 32, 32)
    amax = np.abs(xb).max(-1)
    assert np.abs(qs.astype(int)).max() <= 127
    assert np.array_equal(s, qs.astype(np.int32).sum(-1))
    with np.errstate(over="ignore"):
        assert np.array_equal(d, (amax / np.float32(127.0)).astype(np.float16).astype(np.float32))
    # the element holding amax quantises to +-127; dequantised error is at most half a step
    assert (np.abs(qs.astype(int)).max(-1) == 127).all()
    step = (amax / np.float32(127.0))[..., None]
    assert (np.abs(qs * step - xb) <= 0.5001 * step).all()
    # brute force on one block: exact formula in float32
    blk = xb[3, 7]
    dd = np.float32(np.abs(blk).max()) / np.float32(127.0)
    idd = np.float32(1.0) / dd
    want = np.rint(blk * idd).astype(np.int8)
    assert np.array_equal(qs[3, 7], want)


def test_q8_1_zero_and_threshold(oracle):
    assert not oracle.quantize_block(np.zeros(32, np.float32)).any()
    assert not oracle.quantize_block(np.full(32, 9.9e-11, np.float32)).any()
    b = oracle.quantize_block(np.full(32, 1.1e-10, np.float32))
    assert (b[4:].view(np.int8) == 127).all() and b[0:2].view(np.uint16)[0] == 0  # d underflows fp16


def _dequant_q4k(W):
    """Textbook Q4_K dequantisation (ggml dequantize_row_q4_K), float64."""
    N, SB, _ = W.shape
    out = np.zeros((N, SB * 256))
    for n in range(N):
        for s in range(SB):
            b = W[n, s]
            d = float(b[0:2].view(np.float16)[0])
            dmin = float(b[2:4].view(np.float16)[0])
            sc = b[4:16]
            q = b[16:]
            for j in range(8):
                if j < 4:
                    scale, mn = sc[j] & 63, sc[j + 4] & 63
                else:
                    scale = (sc[j + 4] & 0xF) | ((sc[j - 4] >> 6) << 4)
                    mn = (sc[j + 4] >> 4) | ((sc[j] >> 6) << 4)
                src = q[32 * (j // 2):32 * (j // 2) + 32]
                nib = (src >> 4) if (j & 1) else (src & 0xF)
                out[n, 256 * s + 32 * j:256 * s + 32 * j + 32] = d * scale * nib - dmin * mn
    return out


def test_q4k_effective_blocks_are_the_textbook_dequantisation(oracle):
    W = synth.weights_numpy(FMT_Q4_K, 8, 512, 5)
    want = _dequant_q4k(W)
    for n in range(8):
        for s in range(2):
            w, sc, mn = oracle.subblocks(FMT_Q4_K, W[n, s])
            got = (w.reshape(8, 32) * _f16(sc)[:, None] + _f16(mn)[:, None]).reshape(-1)
            ref = want[n, 256 * s:256 * (s + 1)]
            # only difference: fp16 rounding of d*sc and dmin*m (2^-11 relative each)
            assert np.abs(got - ref).max() <= 2.0 ** -10 * np.abs(ref).max()


def test_q6k_requantisation_closed_form(oracle):
    """Exhaustive over (q, sc, msc): w = ((q-32)*f+128)>>8 with f = rne(sc*1016/msc),
    and the dequantised value tracks the native d*sc*(q-32) within one requant step."""
    rng = np.random.default_rng(9)
    for trial in range(40):
        blk = rng.integers(0, 256, BLOCK_BYTES[FMT_Q6_K], dtype=np.uint8)
        blk[208:210] = np.array([0.01], np.float16).view(np.uint8)
        w, sc_h, mn_h = oracle.subblocks(FMT_Q6_K, blk)
        ql, qh, scales = blk[:128], blk[128:192], blk[192:208].view(np.int8)
        for j in range(8):
            half, s = j >> 2, j & 3
            lo = ql[64 * half + 32 * (s & 1):64 * half + 32 * (s & 1) + 32]
            nib = (lo >> 4) if s >= 2 else (lo & 0xF)
            hi = (qh[32 * half:32 * half + 32] >> (2 * s)) & 3
            q = (nib | (hi << 4)).astype(int) - 32
            sc0, sc1 = int(scales[8 * half + 2 * s]), int(scales[8 * half + 2 * s + 1])
            msc = max(abs(sc0), abs(sc1))
            if msc == 0:
                assert not w[32 * j:32 * j + 32].any() and sc_h[j] == 0
                continue

            def rne_div(a, b):  # round-half-even of a/b for integers, b > 0
                qq, rr = divmod(a, b)
                return qq + (1 if (2 * rr > b or (2 * rr == b and (qq & 1))) else 0)

            f = [rne_div(sc0 * 1016, msc), rne_div(sc1 * 1016, msc)]
            want = np.array([((int(q[i]) * f[i >> 4] + 128) >> 8) for i in range(32)])
            assert np.array_equal(w[32 * j:32 * j + 32].astype(int), want)
            assert mn_h[j] == 0
            native = 0.01 * np.array([sc0] * 16 + [sc1] * 16) * q
            scale = float(_f16([sc_h[j]])[0])
            # half a step of rounding + 32*0.5/256 of a step from the 8.8 factor + fp16 scale rounding
            assert np.abs(w[32 * j:32 * j + 32] * scale - native).max() <= 0.6 * scale + 1e-3 * np.abs(native).max()


def test_division_free_forms_of_the_q6k_factors(oracle):
    """The GPU kernels compute the Q6_K block scale and the 8.8 factor of the smaller sub-scale
    without divisions; the same IEEE operations on the host, over every input they can see:
    x/127 for every fp16 d and max sub-scale, and rne(s*1016/msc) for every (s, msc) with any
    reciprocal within 4 units in the last place of the true one."""
    assert oracle.check_div127() == 0
    # every fp32 significand: the IQ3_S block scale divides d * (odd products up to 465) by 127
    assert oracle.check_div127_all_significands() == 0
    for ulps in (0, 1, 4):
        assert oracle.check_q6k_factor(ulps) == 0


def test_iq3s_requantisation_is_an_integer_map(oracle):
    """w = +-round(g*127/gmax) and scale = f16(gmax*db/127): a pure function of the codebook."""
    import re
    from pathlib import Path

    text = (Path(__file__).resolve().parent.parent / "include" / "llaminar_amd" / "iq3s_grid.h").read_text()
    grid = np.array([int(v, 16) for v in re.findall(r"0x([0-9a-f]{8})u", text)], np.uint32)
    rng = np.random.default_rng(4)
    seen_gmax = set()
    for trial in range(200):
        blk = rng.integers(0, 256, BLOCK_BYTES[FMT_IQ3_S], dtype=np.uint8)
        blk[0:2] = np.array([rng.uniform(0.001, 0.02)], np.float16).view(np.uint8)
        if trial % 4 == 0:  # force small gmax: restrict indices to entries whose bytes are small
            small = np.where([max((g >> (8 * t)) & 255 for t in range(4)) <= 2 * (trial % 7) + 1 for g in grid])[0]
            small = small[small < 256]
            if len(small):
                blk[2:66] = rng.choice(small, 64).astype(np.uint8)
                blk[66:74] = 0
        w, sc_h, mn_h = oracle.subblocks(FMT_IQ3_S, blk)
        d = float(blk[0:2].view(np.float16)[0])
        qs, qh, signs, scales = blk[2:66], blk[66:74], blk[74:106], blk[106:110]
        for j in range(8):
            g = []
            for l in range(8):
                idx = int(qs[8 * j + l]) | (((int(qh[j]) >> l) & 1) << 8)
                g += [(int(grid[idx]) >> (8 * t)) & 255 for t in range(4)]
            g = np.array(g)
            sb = int.from_bytes(bytes(signs[4 * j:4 * j + 4]), "little")
            sgn = np.array([-1 if (sb >> e) & 1 else 1 for e in range(32)])
            gmax = int(g.max())
            seen_gmax.add(gmax)
            want = sgn * ((2 * g * 127 + gmax) // (2 * gmax))
            assert np.array_equal(w[32 * j:32 * j + 32].astype(int), want)
            nib = (int(scales[j >> 1]) >> (4 * (j & 1))) & 0xF
            db = np.float32(d) * np.float32(1 + 2 * nib)
            scale = np.float32(gmax) * db / np.float32(127.0)
            assert sc_h[j] == oracle.f32_to_f16_sw(scale) and mn_h[j] == 0
    assert len(seen_gmax) >= 3  # the small-gmax branches were exercised


@pytest.mark.parametrize("fmt", [FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S])
def test_gemm_is_the_sum_over_blocks(oracle, fmt):
    """Block sums by int64 brute force; fp32 output equals the float64 evaluation of
    the same sum of products to fp32 accumulation accuracy; linear in the activations' d."""
    N, K, M = 24, 768, 3
    W = synth.weights_numpy(fmt, N, K, 21)
    x = synth.activations_numpy(M, K, 22)
    q8 = oracle.quantize(x)
    C, sums = oracle.gemm(fmt, W, K, q8, want_sums=True)
    a_d = _f16(q8[:, :, 0:2].copy().view(np.uint16)[..., 0]).astype(np.float64)
    a_s = q8[:, :, 2:4].copy().view(np.int16)[..., 0].astype(np.float64)
    a_q = q8[:, :, 4:].view(np.int8).astype(np.int64)
    want = np.zeros((M, N))
    for n in range(N):
        wi = np.zeros((K // 32, 32), np.int64)
        sc = np.zeros(K // 32)
        mn = np.zeros(K // 32)
        for s in range(K // 256):
            w, a, b = oracle.subblocks(fmt, W[n, s])
            wi[8 * s:8 * s + 8] = w.reshape(8, 32)
            sc[8 * s:8 * s + 8] = _f16(a)
            mn[8 * s:8 * s + 8] = _f16(b)
        bs = np.einsum("mkb,kb->mk", a_q, wi)
        assert np.array_equal(sums[:, n, :], bs)
        want[:, n] = (bs * a_d * sc).sum(-1) + (a_s * a_d * mn).sum(-1)
    assert np.abs(C - want).max() <= 2e-6 * np.abs(want).max()
    # k_tiles variant: same blocks, different association
    C4 = oracle.gemm(fmt, W, K, q8, k_tiles=4)
    assert np.abs(C4 - want).max() <= 2e-6 * np.abs(want).max()


def test_route_topk_properties(oracle):
    rng = np.random.default_rng(2)
    logits = rng.standard_normal((16, 256)).astype(np.float32)
    ids, w, probs = oracle.route(logits, 8, True)
    assert np.allclose(probs.sum(-1), 1.0, atol=1e-5)
    for t in range(16):
        order = np.argsort(-logits[t], kind="stable")[:8]
        assert np.array_equal(ids[t], order)
        e = np.exp(logits[t, order].astype(np.float64))
        assert np.allclose(w[t], e / e.sum(), rtol=1e-5)
    assert np.allclose(w.sum(-1), 1.0, atol=1e-6)
    ids2, w2, _ = oracle.route(logits, 8, False)
    assert np.array_equal(ids, ids2) and np.allclose(w2, np.take_along_axis(probs, ids, 1))
    # ties resolve to the lower expert id
    tie = np.zeros((1, 16), np.float32)
    ids3, _, _ = oracle.route(tie, 4, True)
    assert np.array_equal(ids3[0], [0, 1, 2, 3])


def test_epilogue(oracle):
    rng = np.random.default_rng(3)
    C = rng.standard_normal((3, 8)).astype(np.float32)
    T = rng.standard_normal((3, 8)).astype(np.float32)
    b = rng.standard_normal(8).astype(np.float32)
    assert np.allclose(oracle.epilogue(C, T, 0.5, 2.0, b), 2.0 * C + 0.5 * T + b, rtol=1e-6)
    assert np.array_equal(oracle.epilogue(np.full((3, 8), np.nan, np.float32), T, 1.0, 0.0), T)
