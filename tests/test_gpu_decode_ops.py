"""Decode-step operators on the GPU through the C-ABI against the CPU restatement
(oracle/decode_oracle.c).  Floating point: tolerances relative to the largest expected
value, stated per test; the sampler's index and the Q8_1 bytes of an exactly matching
RMSNorm row are exact."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_Q4_K
from tests.helpers import sync

pytestmark = pytest.mark.gpu


def close(got, exp, tol):
    exp = np.asarray(exp, dtype=np.float64)
    return np.abs(np.asarray(got, dtype=np.float64) - exp).max() <= tol * max(np.abs(exp).max(), 1e-30)


def test_embed_q4k_rows(capi, dev, oracle):
    import torch

    vocab, H = 300, 5120
    W = synth.weights_numpy(FMT_Q4_K, vocab, H, 41)
    table = torch.from_numpy(W.reshape(-1)).to(dev)
    ids_h = np.array([0, 299, 17, 17, -1, 300, 5], np.int32)
    ids = torch.from_numpy(ids_h).to(dev)
    out = torch.full((len(ids_h), H + 8), 7.0, device=dev)
    capi.embed_q4k(table, vocab, ids, H, out=out[:, :H])
    sync()
    got = out.cpu().numpy()
    exp = oracle.dequant_rows_q4k(W)
    for b, i in enumerate(ids_h):
        if 0 <= i < vocab:
            # the product (d*sc)*q may be fused into the subtraction: one rounding less
            assert close(got[b, :H], exp[i], 2e-7), b
        else:
            assert not got[b, :H].any()
    assert (got[:, H:] == 7.0).all()


@pytest.mark.parametrize("M,H", [(1, 5120), (8, 5120), (3, 8192), (2, 256), (5, 25600)])
def test_rmsnorm_q8_1(capi, dev, oracle, M, H):
    import torch

    rng = np.random.default_rng(M * 100 + H)
    x = (rng.standard_normal((M, H)) * rng.uniform(0.05, 20, (M, 1))).astype(np.float32)
    g = rng.uniform(0.2, 2.0, H).astype(np.float32)
    d = rng.standard_normal((M, H)).astype(np.float32)
    gd = torch.from_numpy(g).to(dev)
    for delta in (None, d):
        xd = torch.from_numpy(x).to(dev)
        dd = torch.from_numpy(delta).to(dev) if delta is not None else None
        y, q8 = capi.rmsnorm_q8_1(xd, gd, 1e-6, delta=dd)
        sync()
        exp_y, exp_x = oracle.rmsnorm(x, g, 1e-6, delta=delta)
        assert np.array_equal(xd.cpu().numpy(), exp_x)            # residual add: one fp32 add, exact
        got = y.cpu().numpy()
        assert close(got, exp_y, 2.4e-7)                           # double sum in another order: <= 1 ulp of rms
        # the quantiser behind it is the bit-exact one: its bytes are those of quantising the row it saw
        assert np.array_equal(q8.cpu().numpy().reshape(M, H // 32, 36), oracle.quantize(got))
        # only one of the two outputs
        y2, none = capi.rmsnorm_q8_1(torch.from_numpy(exp_x).to(dev), gd, 1e-6, want_q8=False)
        assert none is None and torch.equal(y2, y)
        none, q82 = capi.rmsnorm_q8_1(torch.from_numpy(exp_x).to(dev), gd, 1e-6, want_y=False)
        assert none is None and torch.equal(q82, q8)
    sync()


@pytest.mark.parametrize("M,H", [(8, 5120), (5, 9216)])
def test_rmsnorm_with_the_delta_in_two_partial_sums(capi, dev, M, H):
    """llam_dec_rmsnorm2_q8_1: x += (delta + delta2), then the norm: the bits of the one-delta call on the sum of
    the two (rows longer than the registers hold included)."""
    import torch

    rng = np.random.default_rng(7 * M + H)
    x = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).to(dev)
    g = torch.from_numpy(rng.uniform(0.2, 2.0, H).astype(np.float32)).to(dev)
    d1 = torch.from_numpy(rng.standard_normal((M, H)).astype(np.float32)).to(dev)
    d2 = torch.from_numpy((rng.standard_normal((M, H)) * 1e-3).astype(np.float32)).to(dev)
    xa, xb = x.clone(), x.clone()
    ya, qa = capi.rmsnorm_q8_1(xa, g, 1e-6, delta=d1, delta2=d2)
    yb, qb = capi.rmsnorm_q8_1(xb, g, 1e-6, delta=d1 + d2)
    sync()
    assert torch.equal(xa, xb) and torch.equal(xa, x + (d1 + d2))
    assert torch.equal(ya, yb) and torch.equal(qa, qb)
    with pytest.raises(capi.QLError, match="second delta"):
        capi.rmsnorm_q8_1(x.clone(), g, 1e-6, delta=None, delta2=d2)


@pytest.mark.parametrize("B,n_heads,n_kv", [(1, 64, 8), (8, 64, 8), (3, 4, 1), (2, 6, 6)])
def test_rope_kv_append(capi, dev, oracle, B, n_heads, n_kv):
    import torch

    hd, cap, theta = 128, 64, 1e6
    rng = np.random.default_rng(B + n_heads)
    width = (n_heads + 2 * n_kv) * hd
    qkv = rng.standard_normal((B, width + 16)).astype(np.float32)
    pos_h = rng.integers(0, cap, B).astype(np.int32)
    pos_h[0] = cap - 1
    inv = capi.rope_inv_freq(hd, theta, dev)
    assert np.array_equal(inv.cpu().numpy(), oracle.rope_inv_freq(hd, theta))
    kc = torch.zeros(B, n_kv, cap, hd, dtype=torch.float16, device=dev)   # both caches are kept in tiles
    vc = torch.zeros(B, n_kv, cap, hd, dtype=torch.float16, device=dev)
    qd = torch.from_numpy(qkv).to(dev)
    capi.rope_kv_append(qd, inv, torch.from_numpy(pos_h).to(dev), kc, vc, n_heads, n_kv, hd)
    sync()
    got = qd.cpu().numpy()
    kg = capi.kcache_logical(kc).cpu().numpy().view(np.uint16)   # as [cap][hd]
    vg = capi.vcache_logical(vc).cpu().numpy().view(np.uint16)
    f = oracle.rope_inv_freq(hd, theta)
    for b in range(B):
        ke = np.zeros((n_kv, cap, hd), np.uint16)
        ve = np.zeros((n_kv, cap, hd), np.uint16)
        exp = oracle.rope_kv_append(qkv[b, :width], f, int(pos_h[b]), ke, ve, n_heads, n_kv, hd)
        # device sin/cos against the host's: a few ulp of values of magnitude <= ~5
        assert np.abs(got[b, :n_heads * hd] - exp[:n_heads * hd]).max() <= 3e-6
        assert np.array_equal(got[b, n_heads * hd:], qkv[b, n_heads * hd:])   # K, V and the padding stay
        assert np.array_equal(vg[b], ve)                                        # V: a plain fp16 rounding
        kdiff = np.abs(kg[b].view(np.float16).astype(np.float32) - ke.view(np.float16).astype(np.float32))
        assert kdiff.max() <= 4e-3            # one fp16 ulp at magnitude <= 4 where the fp32 values straddle a tie
        assert (kdiff > 0).mean() < 0.01
        untouched = np.ones(cap, bool)
        untouched[pos_h[b]] = False
        assert not kg[b][:, untouched].any() and not vg[b][:, untouched].any()


@pytest.mark.parametrize("B,n_heads,n_kv,cap,positions", [
    (1, 64, 8, 4224, [4095]), (2, 64, 8, 608, [0, 607]), (3, 8, 2, 320, [127, 128, 255]),
    (2, 4, 4, 160, [5, 129]), (1, 2, 1, 128, [64]), (4, 16, 2, 288, [6, 7, 8, 287]),
    (2, 3, 3, 64, [30, 63])])
def test_attention_decode(capi, dev, oracle, B, n_heads, n_kv, cap, positions):
    import torch

    hd = 128
    g = torch.Generator(device=dev)
    g.manual_seed(cap + n_heads)
    kl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()   # position-major values
    vl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()
    for b, p in enumerate(positions):      # what lies past the newest position must not matter, whatever it is
        kl[b, :, p + 1:] = float("nan")
        vl[b, :, p + 1:] = float("nan")
    kc, vc = capi.kcache_tiled(kl), capi.vcache_tiled(vl)                # as the device keeps them
    q = torch.randn(B, n_heads * hd + 32, device=dev, generator=g) * 1.5
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    out = torch.full((B, n_heads * hd + 4), float("nan"), device=dev)
    q8 = torch.zeros(B * (n_heads * hd // 32) * 36, dtype=torch.uint8, device=dev)
    capi.attention(q[:, :n_heads * hd], kc, vc, pos, n_heads, n_kv, hd, out=out[:, :n_heads * hd], q8_out=q8)
    sync()
    got = out.cpu().numpy()
    # the Q8_1 side output: the bit-exact quantiser applied to the fp32 rows it wrote
    assert np.array_equal(q8.cpu().numpy().reshape(B, n_heads * hd // 32, 36),
                          oracle.quantize(np.ascontiguousarray(got[:, :n_heads * hd])))
    assert np.isnan(got[:, n_heads * hd:]).all()
    kh = kl.cpu().numpy().view(np.uint16)   # the oracle's [cap][hd]
    vh = vl.cpu().numpy().view(np.uint16)
    qh = q.cpu().numpy()
    for b in range(B):
        exp = oracle.attention_decode(qh[b, :n_heads * hd], kh[b], vh[b], positions[b], n_heads, n_kv, hd)
        assert close(got[b, :n_heads * hd], exp, 1e-5), (b, positions[b])


def test_attention_follows_the_position_in_memory(capi, dev, oracle):
    """The position is read on the device: the same launch arguments serve every step."""
    import torch

    B, n_heads, n_kv, hd, cap = 1, 8, 1, 128, 512
    g = torch.Generator(device=dev)
    g.manual_seed(3)
    kl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()
    vl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()
    kc, vc = capi.kcache_tiled(kl), capi.vcache_tiled(vl)
    q = torch.randn(B, n_heads * hd, device=dev, generator=g)
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    v_rows = vl.cpu().numpy().view(np.uint16)[0]
    scratch = capi.attention_scratch(B, n_heads, hd, cap, dev)
    for p in (0, 1, 130, 511):
        pos.fill_(p)
        out = capi.attention(q, kc, vc, pos, n_heads, n_kv, hd, scratch=scratch)
        exp = oracle.attention_decode(q.cpu().numpy()[0], kl.cpu().numpy().view(np.uint16)[0],
                                      v_rows, p, n_heads, n_kv, hd)
        assert close(out.cpu().numpy()[0], exp, 1e-5), p


@pytest.mark.parametrize("B,n_heads,n_kv,cap,positions", [
    (1, 64, 8, 4224, [4095]), (8, 64, 8, 544, [0, 1, 127, 128, 255, 256, 300, 543]), (3, 8, 2, 320, [7, 8, 319]),
    (2, 4, 4, 160, [5, 129]), (2, 2, 1, 128, [64, 127]), (2, 3, 3, 64, [0, 63])])
def test_rope_attention_is_append_then_attention(capi, dev, oracle, B, n_heads, n_kv, cap, positions):
    """The fused operator leaves the outputs and the caches that the two separate calls leave."""
    import torch

    hd = 128
    g = torch.Generator(device=dev)
    g.manual_seed(cap + n_heads + 1)
    kl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()
    vl = torch.randn(B, n_kv, cap, hd, device=dev, generator=g).half()
    for b, p in enumerate(positions):      # the slot of the new token and everything after it: anything at all
        kl[b, :, p:] = float("nan")
        vl[b, :, p:] = float("nan")
    kc, vc = capi.kcache_tiled(kl), capi.vcache_tiled(vl)
    width = (n_heads + 2 * n_kv) * hd
    qkv = torch.randn(B, width + 8, device=dev, generator=g) * 1.5
    pos = torch.tensor(positions, dtype=torch.int32, device=dev)
    inv = capi.rope_inv_freq(hd, 1e6, dev)

    kc1, vc1, qkv1 = kc.clone(), vc.clone(), qkv.clone()
    capi.rope_kv_append(qkv1, inv, pos, kc1, vc1, n_heads, n_kv, hd)
    q8_1 = torch.zeros(B * (n_heads * hd // 32) * 36, dtype=torch.uint8, device=dev)
    out1 = capi.attention(qkv1[:, :n_heads * hd], kc1, vc1, pos, n_heads, n_kv, hd, q8_out=q8_1)

    kc2, vc2, qkv2 = kc.clone(), vc.clone(), qkv.clone()
    q8_2 = torch.zeros_like(q8_1)
    table = capi.rope_table(pos, inv, hd)
    out2 = capi.rope_attention(qkv2, table, pos, kc2, vc2, n_heads, n_kv, hd, q8_out=q8_2)
    sync()
    assert torch.equal(qkv2, qkv)                                   # only read
    # K: the sines and cosines come from another kernel; where a rotated value lies on an fp16 tie
    # its last bit may differ.  Slots that were not appended keep their bits.
    k1, k2 = kc1.float().cpu().numpy(), kc2.float().cpu().numpy()
    assert np.array_equal(np.isnan(k1), np.isnan(k2))
    kdiff = np.abs(np.nan_to_num(k1) - np.nan_to_num(k2))
    assert kdiff.max() <= 8e-3 and (kdiff > 0).sum() <= 0.01 * B * n_kv * hd
    assert torch.equal(vc1.view(torch.int16), vc2.view(torch.int16))
    assert torch.isfinite(out2).all()
    # the rotated Q is computed in another kernel: the last bit of a sine may differ
    assert close(out2.cpu().numpy(), out1.cpu().numpy(), 1e-6)
    assert np.array_equal(q8_2.cpu().numpy().reshape(B, n_heads * hd // 32, 36), oracle.quantize(out2.cpu().numpy()))
    # and against the oracle: its rotation of Q, its attention over the caches the device wrote (a rotated
    # K value on an fp16 tie may round the other way on the host; test_rope_kv_append bounds that)
    f = oracle.rope_inv_freq(hd, 1e6)
    qh = qkv.cpu().numpy()
    kh = capi.kcache_logical(kc2).cpu().numpy().view(np.uint16)
    vh = capi.vcache_logical(vc2).cpu().numpy().view(np.uint16)
    got = out2.cpu().numpy()
    for b in range(B):
        rot = oracle.rope_kv_append(qh[b, :width], f, positions[b], kh[b].copy(), vh[b].copy(), n_heads, n_kv, hd)
        exp = oracle.attention_decode(rot[:n_heads * hd], kh[b], vh[b], positions[b], n_heads, n_kv, hd)
        assert close(got[b], exp, 2e-5), (b, positions[b])


def test_attention_refuses_a_cache_it_cannot_read(capi, dev):
    import torch

    hd, cap = 128, 136   # not a multiple of 32: the caches are kept in tiles of 16 and 32 positions
    kc = torch.zeros(1, 1, cap, hd, dtype=torch.float16, device=dev)
    vc = torch.zeros(1, 1, cap, hd, dtype=torch.float16, device=dev)
    q = torch.zeros(1, hd, device=dev)
    pos = torch.zeros(1, dtype=torch.int32, device=dev)
    with pytest.raises(RuntimeError, match="multiple of 32"):
        capi.attention(q, kc, vc, pos, 1, 1, hd)


def test_argmax(capi, dev, oracle):
    import torch

    n, B = 152064, 4
    rng = np.random.default_rng(2)
    x = rng.standard_normal((B, n + 8)).astype(np.float32)
    x[1, [9, 100000, 152063]] = 60.0       # ties: lowest index
    x[2, 5] = np.nan                        # NaN never wins
    x[2, 152063] = 70.0                     # last element
    x[3, :n] = -np.inf                      # nothing beats the start value: INT_MAX, as the reference's kernels
    x[:, n:] = 1e9                          # beyond n: ignored
    xd = torch.from_numpy(x).to(dev)
    pos = torch.tensor([5, 6, 7, 8], dtype=torch.int32, device=dev)
    ids = capi.argmax(xd[:, :n], n, pos=pos)
    sync()
    exp = [oracle.argmax(x[b, :n]) for b in range(B)]
    assert ids.cpu().tolist() == exp
    assert exp[1] == 9 and exp[2] == 152063 and exp[3] == 2**31 - 1
    assert pos.cpu().tolist() == [6, 7, 8, 9]
    small = torch.tensor([[1.0, 3.0, 3.0, 2.0]], device=dev)
    assert capi.argmax(small, 4).cpu().tolist() == [1]
