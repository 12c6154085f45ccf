"""The host library's decode step (dense_decoder.h) against a numpy walk through the same
operators built from the CPU restatements: same weights, same cache, three tokens.

The step chains about a dozen operators per layer whose fp32 results differ from the
restatement's in the last bits (summation order, device sin/cos/exp); each Q8_1 quantiser on
the way turns such a difference into at most one int8 step on a few elements.  The logits
are therefore compared at 5e-3 of the largest logit, and the greedy token wherever the
restatement's top-2 gap exceeds that."""
import numpy as np
import pytest

from llaminar_amd.capi import FMT_Q4_K, FMT_Q6_K
from tests.helpers import sync

pytestmark = pytest.mark.gpu


class NumpyDecoder:
    """One sequence at a time through oracle/*.c, in the order of llam_decoder_step."""

    def __init__(self, oracle, shape, raw, ctx_cap):
        self.o, self.s, self.cap = oracle, shape, ctx_cap
        self.w = {k: v.cpu().numpy() for k, v in raw.items()}
        self.inv_freq = oracle.rope_inv_freq(shape.head_dim, shape.rope_theta)

    def gemv(self, name, fmt, K, x):
        return self.o.gemm(fmt, self.w[name], K, self.o.quantize(x[None]))[0]

    def step(self, token, pos, kcache, vcache):
        """kcache/vcache: uint16 [n_layers, n_kv, cap, hd] of this sequence, updated in place."""
        o, s = self.o, self.s
        H, hd = s.hidden, s.head_dim
        qd, kvd = s.n_heads * hd, s.n_kv * hd
        x = o.dequant_rows_q4k(self.w["embed"].reshape(s.vocab, H // 256, 144)[token][None])[0]
        delta = None
        for l in range(s.n_layers):
            h, x2 = o.rmsnorm(x[None], self.w[f"{l}.attn_norm"], s.rms_eps, delta=None if delta is None else delta[None])
            x = x2[0]
            qkv = np.concatenate([self.gemv(f"{l}.wq", FMT_Q4_K, H, h[0]), self.gemv(f"{l}.wk", FMT_Q4_K, H, h[0]),
                                  self.gemv(f"{l}.wv", FMT_Q6_K, H, h[0])])
            qkv = o.rope_kv_append(qkv, self.inv_freq, pos, kcache[l], vcache[l], s.n_heads, s.n_kv, hd)
            a = o.attention_decode(qkv[:qd], kcache[l], vcache[l], pos, s.n_heads, s.n_kv, hd)
            delta = self.gemv(f"{l}.wo", FMT_Q4_K, qd, a)
            h2, x2 = o.rmsnorm(x[None], self.w[f"{l}.ffn_norm"], s.rms_eps, delta=delta[None])
            x = x2[0]
            g = self.gemv(f"{l}.wgate", FMT_Q4_K, H, h2[0])
            u = self.gemv(f"{l}.wup", FMT_Q4_K, H, h2[0])
            delta = self.gemv(f"{l}.wdown", FMT_Q6_K, s.ffn, o.swiglu(g, u))
        hf, xf = o.rmsnorm(x[None], self.w["final_norm"], s.rms_eps, delta=delta[None])
        self.last_residual = xf[0]   # the residual stream with every layer's output added
        logits = self.gemv("lm_head", FMT_Q6_K, H, hf[0])
        return logits


@pytest.mark.parametrize("batch", [1, 3])
def test_three_tokens_against_numpy_walk(capi, dev, oracle, batch):
    import torch

    from llaminar_amd.decoder import DenseDecoder, Shape

    shape = Shape(hidden=4096, n_heads=8, n_kv=2, head_dim=128, ffn=4096, vocab=2048, n_layers=2)
    cap, start = 192, 130   # the newest position lies in the second 128-position chunk
    # block scales large enough that activations stay O(1) through the layers
    dec = DenseDecoder(shape, batch, cap, dev, seed=5, keep_raw=True, d_lo=0.002, d_hi=0.004, norm_scale=1.0)
    ref = NumpyDecoder(oracle, shape, dec.raw, cap)
    rng = np.random.default_rng(1)
    ids = rng.integers(0, shape.vocab, batch).astype(np.int32)
    pos = (start + np.arange(batch)).astype(np.int32)   # sequences at different positions
    kc_h = np.zeros((batch, shape.n_layers, shape.n_kv, cap, 128), np.float16)
    vc_h = np.zeros_like(kc_h)
    for b in range(batch):
        kc_h[b, :, :, :pos[b]] = rng.standard_normal((shape.n_layers, shape.n_kv, pos[b], 128)).astype(np.float16)
        vc_h[b, :, :, :pos[b]] = rng.standard_normal((shape.n_layers, shape.n_kv, pos[b], 128)).astype(np.float16)
    for l in range(shape.n_layers):
        # the device keeps both caches in tiles
        dec.buffer("kcache", l).copy_(capi.kcache_tiled(torch.from_numpy(kc_h[:, l])).to(dev))
        dec.buffer("vcache", l).copy_(capi.vcache_tiled(torch.from_numpy(vc_h[:, l])).to(dev))
    dec.set_state(ids, pos)
    kc_u, vc_u = kc_h.view(np.uint16).copy(), vc_h.view(np.uint16).copy()

    for step in range(3):
        dec.step()
        sync()
        logits = dec.buffer("logits").cpu().numpy()
        new_ids = dec.buffer("ids").cpu().numpy()
        resid = dec.buffer("x").cpu().numpy()   # wherever the step left the residual stream
        assert dec.buffer("pos").cpu().tolist() == [int(p) + step + 1 for p in pos]
        assert np.isfinite(logits).all()
        for b in range(batch):
            exp = ref.step(int(ids[b]), int(pos[b]) + step, kc_u[b], vc_u[b])
            scale = np.abs(exp).max()
            err = np.abs(logits[b] - exp).max()
            assert err <= 5e-3 * scale, (step, b, err, scale)
            assert np.abs(resid[b] - ref.last_residual).max() <= 5e-3 * np.abs(ref.last_residual).max(), (step, b)
            assert new_ids[b] == int(np.argmax(logits[b]))           # the sampler on the device's own logits
            top2 = np.sort(exp)[-2:]
            if top2[1] - top2[0] > 2 * 5e-3 * scale:
                assert new_ids[b] == int(np.argmax(exp)), (step, b)
            # the appended K/V rows: fp16 of nearly equal fp32 values
            for l in range(shape.n_layers):
                kg = capi.kcache_logical(dec.buffer("kcache", l))[b, :, int(pos[b]) + step].cpu().numpy().astype(np.float32)
                ke = kc_u[b, l, :, int(pos[b]) + step].view(np.float16).astype(np.float32)
                assert np.abs(kg - ke).max() <= 2e-2 * max(np.abs(ke).max(), 1.0), (step, b, l)
                vg = capi.vcache_logical(dec.buffer("vcache", l))[b, :, int(pos[b]) + step].cpu().numpy().astype(np.float32)
                ve = vc_u[b, l, :, int(pos[b]) + step].view(np.float16).astype(np.float32)
                assert np.abs(vg - ve).max() <= 2e-2 * max(np.abs(ve).max(), 1.0), (step, b, l)
        ids = new_ids.copy()   # both sides continue from the device's tokens
    dec.close()


@pytest.mark.parametrize("ffn,n_layers", [(4096, 2), (16384, 1)], ids=["ffn4096", "ffn16384-split-down"])
def test_batch_eight_against_numpy_walk(capi, dev, oracle, ffn, n_layers):
    """One step at batch 8 (the matrix-unit GEMV kernels: Q with K and V in one launch, gate + up + SwiGLU in one
    launch; the batched attention and sampler) against the numpy walk, sequence by sequence: logits, greedy token
    and the appended K row.  With a feed-forward width of 16384 the down projection's rows are long enough to be
    summed in two halves, which the following norm adds."""
    import torch

    from llaminar_amd.decoder import DenseDecoder, Shape

    batch = 8
    shape = Shape(hidden=4096, n_heads=8, n_kv=2, head_dim=128, ffn=ffn, vocab=2048, n_layers=n_layers)
    assert capi.gemv_plane_split_supported(FMT_Q6_K, batch, shape.hidden, ffn) == (ffn >= 16384)
    cap, start = 64, 20
    dec = DenseDecoder(shape, batch, cap, dev, seed=9, keep_raw=True, d_lo=0.002, d_hi=0.004, norm_scale=1.0)
    ref = NumpyDecoder(oracle, shape, dec.raw, cap)
    rng = np.random.default_rng(2)
    ids = rng.integers(0, shape.vocab, batch).astype(np.int32)
    pos = (start + 3 * np.arange(batch)).astype(np.int32)
    kc_h = np.zeros((batch, shape.n_layers, shape.n_kv, cap, 128), np.float16)
    vc_h = np.zeros_like(kc_h)
    for b in range(batch):
        kc_h[b, :, :, :pos[b]] = rng.standard_normal((shape.n_layers, shape.n_kv, pos[b], 128)).astype(np.float16)
        vc_h[b, :, :, :pos[b]] = rng.standard_normal((shape.n_layers, shape.n_kv, pos[b], 128)).astype(np.float16)
    for l in range(shape.n_layers):
        dec.buffer("kcache", l).copy_(capi.kcache_tiled(torch.from_numpy(kc_h[:, l])).to(dev))
        dec.buffer("vcache", l).copy_(capi.vcache_tiled(torch.from_numpy(vc_h[:, l])).to(dev))
    dec.set_state(ids, pos)
    kc_u, vc_u = kc_h.view(np.uint16).copy(), vc_h.view(np.uint16).copy()
    dec.step()
    sync()
    logits = dec.buffer("logits").cpu().numpy()
    new_ids = dec.buffer("ids").cpu().numpy()
    assert dec.buffer("pos").cpu().tolist() == [int(p) + 1 for p in pos]
    for b in range(batch):
        exp = ref.step(int(ids[b]), int(pos[b]), kc_u[b], vc_u[b])
        scale = np.abs(exp).max()
        assert np.abs(logits[b] - exp).max() <= 5e-3 * scale, b
        assert new_ids[b] == int(np.argmax(logits[b]))
        top2 = np.sort(exp)[-2:]
        if top2[1] - top2[0] > 2 * 5e-3 * scale:
            assert new_ids[b] == int(np.argmax(exp)), b
        for l in range(shape.n_layers):
            kg = capi.kcache_logical(dec.buffer("kcache", l))[b, :, int(pos[b])].cpu().numpy().astype(np.float32)
            ke = kc_u[b, l, :, int(pos[b])].view(np.float16).astype(np.float32)
            assert np.abs(kg - ke).max() <= 2e-2 * max(np.abs(ke).max(), 1.0), (b, l)
    dec.close()


def test_a_full_context_is_reported(capi, dev):
    """The last position of the cache can still be decoded; the step after it fails with a clear
    error and enqueues nothing (ids, positions and logits keep their values); replays of a
    captured step are accounted through advance()."""
    from llaminar_amd.decoder import DenseDecoder, Shape

    shape = Shape(hidden=1024, n_heads=8, n_kv=2, head_dim=128, ffn=1024, vocab=512, n_layers=1)
    cap = 32
    dec = DenseDecoder(shape, 2, cap, dev, seed=3)
    dec.set_state([5, 6], [cap - 3, cap - 1])          # the furthest sequence sits on the last position
    assert dec.steps_left() == 1
    dec.step()
    sync()
    assert dec.buffer("pos").cpu().tolist() == [cap - 2, cap]
    assert dec.steps_left() == 0
    ids = dec.buffer("ids").cpu().tolist()
    logits = dec.buffer("logits").clone()
    with pytest.raises(capi.QLError, match="context full"):
        dec.step()
    sync()
    assert dec.buffer("pos").cpu().tolist() == [cap - 2, cap] and dec.buffer("ids").cpu().tolist() == ids
    import torch

    assert torch.equal(dec.buffer("logits"), logits)
    with pytest.raises(capi.QLError, match="context full"):
        dec.advance(1)
    dec.set_state([1, 2], [0, 3])
    assert dec.steps_left() == cap - 3
    dec.advance(cap - 4)
    assert dec.steps_left() == 1
    with pytest.raises(capi.QLError, match="outside"):
        dec.set_state([1, 2], [0, cap])
    dec.close()


@pytest.mark.parametrize("batch,ffn", [(2, 4096), (6, 4096), (6, 16384)])
def test_step_replays_as_a_graph(capi, dev, batch, ffn):
    """A captured step replayed gives the tokens of eager steps (batch 6: the matrix-unit kernels and their merged
    launches; feed-forward width 16384: the down projection summed in two halves)."""
    import torch

    from llaminar_amd.decoder import DenseDecoder, Shape

    shape = Shape(hidden=4096, n_heads=8, n_kv=2, head_dim=128, ffn=ffn, vocab=2048, n_layers=2)
    dec = DenseDecoder(shape, batch, 160, dev, seed=6)
    ids0 = np.array([7, 1999, 3, 1024, 77, 500][:batch], np.int32)
    pos0 = np.array([0, 0, 5, 17, 1, 130][:batch], np.int32)

    def run(n, graph):
        for l in range(shape.n_layers):
            dec.buffer("kcache", l).zero_()
            dec.buffer("vcache", l).zero_()
        dec.set_state(ids0, pos0)
        toks, lg = [], []
        for _ in range(n):
            if graph is None:
                dec.step()
            else:
                graph.replay()
            torch.cuda.synchronize()
            toks.append(dec.buffer("ids").cpu().tolist())
            lg.append(dec.buffer("logits").clone())
            # unrelated eager work between replays
            torch.ones(1000, device=dev).sum().item()
        return toks, lg

    eager_t, eager_l = run(4, None)
    stream = torch.cuda.Stream()
    gr = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        dec.step(stream)          # warm-up on the capture stream
        stream.synchronize()
        with torch.cuda.graph(gr, stream=stream):
            dec.step(stream)
    graph_t, graph_l = run(4, gr)
    assert graph_t == eager_t
    for a, b in zip(eager_l, graph_l):
        assert torch.equal(a, b)
    dec.close()


def test_bad_configurations_are_refused(capi, dev):
    from llaminar_amd import decoder

    L = decoder.load()
    bad = decoder.Config(5000, 64, 8, 128, 25600, 1000, 1, 32, 1, 1e6, 1e-6, 0)  # hidden not a multiple of 256
    assert not L.llam_decoder_create(bad)
    assert b"multiples of 256" in L.llam_decoder_last_error()
    bad = decoder.Config(512, 6, 4, 128, 512, 1000, 1, 32, 1, 1e6, 1e-6, 0)       # 6 heads on 4 KV heads
    assert not L.llam_decoder_create(bad)
    ok = decoder.Config(512, 4, 4, 128, 512, 1000, 1, 32, 9, 1e6, 1e-6, 0)        # batch 9
    assert not L.llam_decoder_create(ok)
    assert not L.llam_decoder_create(decoder.Config(512, 4, 4, 128, 512, 1000, 1, 24, 1, 1e6, 1e-6, 0))
    assert b"multiple of 32" in L.llam_decoder_last_error()                       # 24 cache positions
    h = L.llam_decoder_create(decoder.Config(512, 4, 4, 128, 512, 1000, 1, 32, 1, 1e6, 1e-6, 0))
    assert h
    assert not L.llam_decoder_step(h, None) and b"globals not set" in L.llam_decoder_last_error()
    L.llam_decoder_destroy(h)
