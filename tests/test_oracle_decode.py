"""Pins oracle/decode_oracle.c: what the mathematics fixes (closed forms in float64,
invariants, special cases), the reference's own compiled primitives where oracle/_ref was
built, and the committed vectors those primitives produced (tests/golden/decode_goldens.npz)."""
from pathlib import Path

import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_Q4_K

GOLD = Path(__file__).parent / "golden" / "decode_goldens.npz"


def f16_bits_to_f32(a):
    return np.asarray(a, dtype=np.uint16).view(np.float16).astype(np.float32)


# ---- Q4_K rows ------------------------------------------------------------------------------
def test_dequant_q4k_matches_pinned_subblock_decoder(oracle):
    """y = (d*sc)*q - dmin*m with q, sc, m as the pinned int8 sub-block decoder reads them."""
    W = synth.weights_numpy(FMT_Q4_K, 6, 1024, 77)
    y = oracle.dequant_rows_q4k(W)
    for n in range(6):
        for s in range(4):
            blk = W[n, s]
            d = f16_bits_to_f32(blk[0:2].view(np.uint16))[0]
            dmin = f16_bits_to_f32(blk[2:4].view(np.uint16))[0]
            w, _, _ = oracle.subblocks(FMT_Q4_K, blk)  # nibble order pinned on the reference's vectors
            for j in range(8):
                sc, m = oracle.scale_min_k4(j, blk[4:16]) if hasattr(oracle, "scale_min_k4") else (None, None)
                if sc is None:
                    pytest.skip("no scale accessor")
                exp = np.float32(d * np.float32(sc)) * w[32 * j:32 * j + 32].astype(np.float32) - np.float32(
                    dmin * np.float32(m))
                got = y[n, s * 256 + 32 * j: s * 256 + 32 * j + 32]
                assert np.array_equal(got, exp.astype(np.float32))


def test_dequant_q4k_special_cases(oracle):
    blk = np.zeros((1, 1, 144), np.uint8)
    blk[0, 0, 0:2] = np.array([np.float16(0.5)]).view(np.uint8)   # d
    blk[0, 0, 2:4] = np.array([np.float16(0.25)]).view(np.uint8)  # dmin
    blk[0, 0, 4:8] = 3    # scales of sub-blocks 0..3
    blk[0, 0, 8:12] = 2   # mins of sub-blocks 0..3
    blk[0, 0, 16:48] = 0x21  # group 0: low nibble 1 (sub-block 0), high nibble 2 (sub-block 1)
    y = oracle.dequant_rows_q4k(blk)[0]
    assert np.all(y[0:32] == 0.5 * 3 * 1 - 0.25 * 2)
    assert np.all(y[32:64] == 0.5 * 3 * 2 - 0.25 * 2)
    assert np.all(y[64:128] == 0.5 * 3 * 0 - 0.25 * 2)
    assert np.all(y[128:] == 0.0)  # scales and mins 4..7 are zero


# ---- RMSNorm -------------------------------------------------------------------------------------
def test_rmsnorm_closed_form_and_invariants(oracle):
    rng = np.random.default_rng(5)
    x = rng.standard_normal((4, 5120)).astype(np.float32)
    g = rng.uniform(0.5, 1.5, 5120).astype(np.float32)
    y, x_after = oracle.rmsnorm(x, g, 1e-6)
    assert np.array_equal(x_after, x)
    ref = x.astype(np.float64) / np.sqrt((x.astype(np.float64) ** 2).mean(axis=1, keepdims=True) + 1e-6) * g
    assert np.abs(y - ref).max() <= 4e-7 * np.abs(ref).max()
    # a constant row normalises to +-gamma; a dropped eps or a sum instead of a mean would not
    c = np.full((1, 256), -3.0, np.float32)
    yc, _ = oracle.rmsnorm(c, np.ones(256, np.float32), 0.0)
    assert np.allclose(yc, -1.0, atol=1e-7)
    # eps matters for tiny rows: x = 1e-4, eps = 1e-6 -> 1e-4 / sqrt(1e-8 + 1e-6)
    t = np.full((1, 64), 1e-4, np.float32)
    yt, _ = oracle.rmsnorm(t, np.ones(64, np.float32), 1e-6)
    assert np.allclose(yt, 1e-4 / np.sqrt(1e-8 + 1e-6), rtol=1e-6)
    # the residual add comes first and is returned
    d = rng.standard_normal((4, 5120)).astype(np.float32)
    y2, x2 = oracle.rmsnorm(x, g, 1e-6, delta=d)
    assert np.array_equal(x2, x + d)
    y3, _ = oracle.rmsnorm(x + d, g, 1e-6)
    assert np.array_equal(y2, y3)


# ---- RoPE ----------------------------------------------------------------------------------------
def test_rope_closed_form_and_invariants(oracle):
    hd, theta = 128, 1e6
    f = oracle.rope_inv_freq(hd, theta)
    i = np.arange(hd // 2)
    assert np.allclose(f, theta ** (-2.0 * i / hd), rtol=2e-6)
    assert f[0] == 1.0
    rng = np.random.default_rng(6)
    h = rng.standard_normal(hd).astype(np.float32)
    assert np.array_equal(oracle.rope_head(h, 0, f), h)  # position 0 is the identity
    for pos in (1, 17, 4095):
        r = oracle.rope_head(h, pos, f)
        ang = pos * f.astype(np.float64)
        exp0 = h[:64] * np.cos(ang) - h[64:] * np.sin(ang)   # pairs (i, i+64): not interleaved
        exp1 = h[:64] * np.sin(ang) + h[64:] * np.cos(ang)
        # float32 angles at position 4095 carry up to 4095 * 2^-24 absolute error
        tol = 1e-6 + pos * 1.2e-7
        assert np.abs(r[:64] - exp0).max() <= tol * 4 and np.abs(r[64:] - exp1).max() <= tol * 4
        assert np.allclose(r[:64] ** 2 + r[64:] ** 2, h[:64] ** 2 + h[64:] ** 2, rtol=1e-5)
    # composition: rotating by 5 then by 7 is rotating by 12 (up to fp32 rounding)
    assert np.allclose(oracle.rope_head(oracle.rope_head(h, 5, f), 7, f), oracle.rope_head(h, 12, f), atol=2e-5)


def test_rope_kv_append_layout(oracle):
    n_heads, n_kv, hd, cap = 4, 2, 128, 8
    rng = np.random.default_rng(8)
    qkv = rng.standard_normal((n_heads + 2 * n_kv) * hd).astype(np.float32)
    f = oracle.rope_inv_freq(hd, 1e6)
    kc = np.zeros((n_kv, cap, hd), np.uint16)
    vc = np.zeros((n_kv, cap, hd), np.uint16)
    out = oracle.rope_kv_append(qkv, f, 3, kc, vc, n_heads, n_kv, hd)
    for h in range(n_heads + n_kv):
        assert np.array_equal(out[h * hd:(h + 1) * hd], oracle.rope_head(qkv[h * hd:(h + 1) * hd], 3, f))
    assert np.array_equal(out[(n_heads + n_kv) * hd:], qkv[(n_heads + n_kv) * hd:])  # V untouched
    for kh in range(n_kv):
        k = out[(n_heads + kh) * hd:(n_heads + kh + 1) * hd]
        v = qkv[(n_heads + n_kv + kh) * hd:(n_heads + n_kv + kh + 1) * hd]
        assert np.array_equal(kc[kh, 3], k.astype(np.float16).view(np.uint16))
        assert np.array_equal(vc[kh, 3], v.astype(np.float16).view(np.uint16))
    assert not kc[:, [0, 1, 2, 4, 5, 6, 7]].any() and not vc[:, [0, 1, 2, 4, 5, 6, 7]].any()


# ---- attention -----------------------------------------------------------------------------------
def test_attention_closed_form_and_special_cases(oracle):
    n_heads, n_kv, hd, cap = 8, 2, 128, 64
    rng = np.random.default_rng(9)
    q = rng.standard_normal(n_heads * hd).astype(np.float32)
    kc = rng.standard_normal((n_kv, cap, hd)).astype(np.float16)
    vc = rng.standard_normal((n_kv, cap, hd)).astype(np.float16)
    ku, vu = kc.view(np.uint16), vc.view(np.uint16)
    # one position: the output is that V row, whatever q is
    o = oracle.attention_decode(q, ku, vu, 0, n_heads, n_kv, hd).reshape(n_heads, hd)
    for h in range(n_heads):
        assert np.array_equal(o[h], vc[h // 4, 0].astype(np.float32))
    # general case against float64 numpy; heads 0..3 use KV head 0, 4..7 KV head 1; last is inclusive
    last = 40
    o = oracle.attention_decode(q, ku, vu, last, n_heads, n_kv, hd).reshape(n_heads, hd)
    for h in range(n_heads):
        K = kc[h // 4, :last + 1].astype(np.float64)
        V = vc[h // 4, :last + 1].astype(np.float64)
        s = K @ q[h * hd:(h + 1) * hd].astype(np.float64) / np.sqrt(hd)
        p = np.exp(s - s.max())
        assert np.allclose(o[h], (p / p.sum()) @ V, rtol=0, atol=1e-6)
    # identical keys: uniform weights, the mean of V
    kc2 = np.repeat(kc[:, :1], cap, axis=1)
    o = oracle.attention_decode(q, kc2.view(np.uint16), vu, cap - 1, n_heads, n_kv, hd).reshape(n_heads, hd)
    assert np.allclose(o[0], vc[0].astype(np.float64).mean(axis=0), atol=1e-6)


# ---- argmax --------------------------------------------------------------------------------------
def test_argmax_ties_and_nan(oracle):
    rng = np.random.default_rng(10)
    x = rng.standard_normal(152064).astype(np.float32)
    assert oracle.argmax(x) == int(np.argmax(x))
    x[[7, 100, 90000]] = 50.0
    assert oracle.argmax(x) == 7          # ties: the lowest index
    x[3] = np.nan
    assert oracle.argmax(x) == 7          # NaN never wins
    # nothing beats the start value (-FLT_MAX, INT_MAX): the reference's kernels return INT_MAX then
    assert oracle.argmax(np.array([-np.inf, -np.inf], np.float32)) == 2**31 - 1


# ---- the reference's own primitives ----------------------------------------------------------------
def _decode_ref(ref):
    if not getattr(ref, "has_decode", False):
        pytest.skip("reference primitives not in this build of oracle/_ref")
    return ref


def test_rmsnorm_against_reference_rows(oracle, ref):
    ref = _decode_ref(ref)
    rng = np.random.default_rng(11)
    for cols in (5120, 8192, 128, 1000):
        x = (rng.standard_normal(cols) * rng.uniform(0.01, 30)).astype(np.float32)
        g = rng.uniform(0.2, 2.0, cols).astype(np.float32)
        y, _ = oracle.rmsnorm(x[None], g, 1e-6)
        # scalar row: the same operations in the same order
        assert np.array_equal(y[0], ref.rmsnorm_row(x, g, 1e-6, variant=1))
        # SIMD rows sum the squares in another order (in double): the float rms almost always agrees
        for variant in (2, 3):
            r = ref.rmsnorm_row(x, g, 1e-6, variant=variant)
            assert np.abs(y[0] - r).max() <= 2.4e-7 * np.abs(r).max()
        d = rng.standard_normal(cols).astype(np.float32)
        y2, x2 = oracle.rmsnorm(x[None], g, 1e-6, delta=d[None])
        r2, xr = ref.residual_rmsnorm_row(d, x, g, 1e-6)
        assert np.array_equal(x2[0], xr)
        assert np.abs(y2[0] - r2).max() <= 2.4e-7 * np.abs(r2).max()


def test_rope_against_reference(oracle, ref):
    ref = _decode_ref(ref)
    hd, theta = 128, 1e6
    f = oracle.rope_inv_freq(hd, theta)
    assert np.array_equal(f, ref.rope_inv_freq(hd, theta))
    rng = np.random.default_rng(12)
    q = rng.standard_normal(8 * hd).astype(np.float32)
    k = rng.standard_normal(2 * hd).astype(np.float32)
    for pos in (0, 1, 333, 4095):
        # scalar head routine: same libm and angles; the reference's build may fuse one of the
        # two products of a rotation into the subtraction, the restatement rounds both
        a, b = oracle.rope_head(q[:hd], pos, f), ref.rope_head_scalar(q[:hd], pos, theta)
        assert np.abs(a - b).max() <= 2.4e-7 * np.abs(q[:hd]).max() * 2
        # the path a decode step takes (SIMD sin/cos): last bits only
        rq, rk = ref.rope_token(q, k, hd, pos, theta)
        mine_q = np.concatenate([oracle.rope_head(q[h * hd:(h + 1) * hd], pos, f) for h in range(8)])
        mine_k = np.concatenate([oracle.rope_head(k[h * hd:(h + 1) * hd], pos, f) for h in range(2)])
        assert np.abs(mine_q - rq).max() <= 5e-6 and np.abs(mine_k - rk).max() <= 5e-6


def test_swiglu_against_reference(oracle, ref):
    """silu(gate) * up: the reference's vector path (a degree-5 exp polynomial, rcp14 plus one
    Newton step; SwiGLUPrimitives.cpp:137-208) stays within a few 1e-6 of the mathematical
    function the restatement computes; its scalar tail is that function itself."""
    if not getattr(ref, "has_swiglu", False):
        pytest.skip("reference SwiGLU not in this build of oracle/_ref")
    rng = np.random.default_rng(13)
    for n, spread in ((25600, 3.0), (512, 1.0), (2048, 8.0)):
        g = (rng.standard_normal(n) * spread).astype(np.float32)
        u = rng.standard_normal(n).astype(np.float32)
        mine, theirs = oracle.swiglu(g, u), ref.swiglu(g, u)
        assert np.abs(mine - theirs).max() <= 1e-5 * np.maximum(np.abs(mine), 1e-3).max()
        assert (np.abs(mine - theirs) <= 8e-6 * np.abs(mine) + 1e-30).all()
    # fewer than one vector: the scalar routine, the same expression on the same libm
    g = (rng.standard_normal(13) * 4).astype(np.float32)
    u = rng.standard_normal(13).astype(np.float32)
    assert np.array_equal(oracle.swiglu(g, u), ref.swiglu(g, u))
    # closed form in float64, and the special values
    g = np.array([-30, -8, -1, -1e-3, 0, 1e-3, 1, 8, 30], np.float32)
    u = np.full(g.size, 1.5, np.float32)
    want = (g.astype(np.float64) / (1 + np.exp(-g.astype(np.float64)))) * 1.5
    assert np.abs(oracle.swiglu(g, u) - want).max() <= 3e-7 * np.abs(want).max()
    assert oracle.swiglu(np.zeros(4, np.float32), np.ones(4, np.float32)).tolist() == [0, 0, 0, 0]


def test_committed_reference_vectors(oracle):
    """Outputs of the reference's primitives written by tests/golden/make_decode_goldens.py."""
    if not GOLD.exists():
        pytest.skip("decode goldens not generated")
    z = np.load(GOLD)
    y, _ = oracle.rmsnorm(z["rms_x"], z["rms_gamma"], float(z["rms_eps"]))
    assert np.array_equal(y, z["rms_y_scalar"])
    assert np.abs(y - z["rms_y_avx512"]).max() <= 2.4e-7 * np.abs(y).max()
    y2, x2 = oracle.rmsnorm(z["rms_x"], z["rms_gamma"], float(z["rms_eps"]), delta=z["rms_delta"])
    assert np.array_equal(x2, z["rms_res_after"])
    assert np.abs(y2 - z["rms_res_y_avx512"]).max() <= 2.4e-7 * np.abs(y2).max()
    f = oracle.rope_inv_freq(128, 1e6)
    assert np.array_equal(f, z["rope_inv_freq"])
    for i, pos in enumerate(z["rope_positions"]):
        got = oracle.rope_head(z["rope_head"], int(pos), f)
        assert np.abs(got - z["rope_scalar"][i]).max() <= 4.8e-7 * np.abs(z["rope_head"]).max()
        assert np.abs(got - z["rope_token_q"][i][:128]).max() <= 5e-6
    if "route_ids" in z:
        # the router: the reference's softmax (as its dispatcher runs it), selection and renormalisation
        ids, w, probs = oracle.route(z["route_logits"], 8, True)
        assert np.array_equal(ids, z["route_ids"]) and np.array_equal(probs, z["route_probs"])
        assert np.array_equal(w, z["route_weights"])
        assert np.array_equal(oracle.route(z["route_logits"], 8, False)[1], z["route_weights_unnormalised"])
    if "swiglu_out" in z:
        mine = oracle.swiglu(z["swiglu_gate"], z["swiglu_up"])
        assert (np.abs(mine - z["swiglu_out"]) <= 8e-6 * np.abs(mine) + 1e-30).all()
        assert np.array_equal(mine[1024:], z["swiglu_out"][1024:])  # the scalar tail
