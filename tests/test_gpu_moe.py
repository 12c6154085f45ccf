"""P4 on the GPU: router, routed gate/up GEMVs from device-resident ids, fused
SwiGLU + Q8_1, weighted down GEMVs -- each stage against the oracle, then the
whole expert FFN at the BASELINE MoE shape (hidden 2048, 256+1 experts, top-8,
intermediate 512, IQ3_S) for 1 and 16 tokens."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import FMTS, TOL, rel_err, sync, upload_q8, upload_weights

pytestmark = pytest.mark.gpu


def test_router(capi, dev, oracle):
    import torch

    rng = np.random.default_rng(12)
    for T, E, k in ((1, 256, 8), (16, 256, 8), (3, 64, 4), (2, 1000, 6), (1, 8, 8)):
        logits = rng.standard_normal((T, E)).astype(np.float32)
        ids, w = capi.moe_route(torch.from_numpy(logits).to(dev), k, True)
        ids_n, w_n = capi.moe_route(torch.from_numpy(logits).to(dev), k, False)
        sync()
        rids, rw, probs = oracle.route(logits, k, True)
        assert np.array_equal(ids.cpu().numpy(), rids)
        assert np.allclose(w.cpu().numpy(), rw, rtol=2e-6, atol=1e-8)
        assert np.array_equal(ids_n.cpu().numpy(), rids)
        assert np.allclose(w_n.cpu().numpy(), np.take_along_axis(probs, rids, 1), rtol=2e-6, atol=1e-9)
    tie = torch.zeros(1, 16, device=dev)
    ids, w = capi.moe_route(tie, 4, True)
    sync()
    assert ids.cpu().numpy().tolist() == [[0, 1, 2, 3]]
    assert np.allclose(w.cpu().numpy(), 0.25)


def test_router_logits(capi, dev):
    """fp32 router matrix times hidden states against float64 numpy (floating point: 1e-5 of
    the largest logit; the reference's SIMD dot sums in another order as well)."""
    import torch

    rng = np.random.default_rng(4)
    for T, D, E in ((1, 2048, 256), (16, 2048, 257), (3, 5120, 7)):
        h = rng.standard_normal((T, D)).astype(np.float32)
        w = (rng.standard_normal((E, D)) * 0.05).astype(np.float32)
        got = capi.moe_router_logits(torch.from_numpy(h).to(dev), torch.from_numpy(w).to(dev)).cpu().numpy()
        exp = h.astype(np.float64) @ w.astype(np.float64).T
        assert np.abs(got - exp).max() <= 1e-5 * np.abs(exp).max(), (T, D, E)


def test_swiglu_quantize(capi, dev, oracle):
    import torch

    rng = np.random.default_rng(3)
    g = (rng.standard_normal((9, 512)) * 3).astype(np.float32)
    u = rng.standard_normal((9, 512)).astype(np.float32)
    q8, act = capi.swiglu_quantize(torch.from_numpy(g).to(dev), torch.from_numpy(u).to(dev), want_act=True)
    sync()
    act_h = act.cpu().numpy()
    want = oracle.swiglu(g, u)
    assert np.abs(act_h - want).max() <= 4e-6 * max(1.0, np.abs(want).max())
    # the quantiser stage is bit-exact on the activations the GPU actually produced
    assert np.array_equal(q8.cpu().numpy().reshape(9, 16, 36), oracle.quantize(act_h))


def _experts(capi, dev, fmt, n_exp, hidden, inter, seed):
    host, devs = [], []
    for e in range(n_exp):
        g = synth.weights_numpy(fmt, inter, hidden, seed + 3 * e)
        u = synth.weights_numpy(fmt, inter, hidden, seed + 3 * e + 1)
        d = synth.weights_numpy(fmt, hidden, inter, seed + 3 * e + 2)
        host.append((g, u, d))
        devs.append(tuple(upload_weights(capi, dev, fmt, w) for w in (g, u, d)))
    return host, devs, capi.expert_table(devs, dev)


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_stages_small(capi, dev, oracle, fmt):
    """Every stage against the oracle on a 6-expert toy (hidden 512, inter 256, top-3, 4 tokens)."""
    import torch

    n_exp, hidden, inter, k, T = 6, 512, 256, 3, 4
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 40)
    rng = np.random.default_rng(8)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, n_exp)).astype(np.float32)
    ids, w = capi.moe_route(torch.from_numpy(logits).to(dev), k, True)
    qd = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
    gate, up = capi.moe_gate_up(fmt, table, n_exp, ids, qd, T, k, hidden, inter)
    q8a, act = capi.swiglu_quantize(gate, up, want_act=True)
    out = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down(fmt, table, n_exp, ids, w, q8a, out, T, k, hidden, inter, accumulate=False)
    sync()
    rids, rw, _ = oracle.route(logits, k, True)
    assert np.array_equal(ids.cpu().numpy(), rids)
    q8 = oracle.quantize(x)
    gate_h, up_h, act_h = gate.cpu().numpy(), up.cpu().numpy(), act.cpu().numpy()
    q8a_h = q8a.cpu().numpy().reshape(T * k, inter // 32, 36)
    want_out = np.zeros((T, hidden), np.float64)
    for t in range(T):
        for s in range(k):
            e = int(rids[t, s])
            g_ref = oracle.gemm(fmt, host[e][0], hidden, q8[t:t + 1])[0]
            u_ref = oracle.gemm(fmt, host[e][1], hidden, q8[t:t + 1])[0]
            assert rel_err(gate_h[t * k + s], g_ref) <= TOL[fmt] * 1e-2
            assert rel_err(up_h[t * k + s], u_ref) <= TOL[fmt] * 1e-2
            # down: same Q8_1 input on both sides (the GPU's), so the stage is checked tightly
            d_ref = oracle.gemm(fmt, host[e][2], inter, q8a_h[t * k + s][None])[0]
            want_out[t] += float(rw[t, s]) * d_ref
    assert rel_err(out.cpu().numpy(), want_out.astype(np.float32)) <= TOL[fmt] * 1e-2
    # accumulate mode adds onto the existing output
    base = torch.ones((T, hidden), device=dev)
    capi.moe_down(fmt, table, n_exp, ids, w, q8a, base, T, k, hidden, inter, accumulate=True)
    sync()
    assert rel_err(base.cpu().numpy() - 1.0, want_out.astype(np.float32)) <= 1e-5


def test_out_of_range_expert_ids_are_skipped(capi, dev, oracle):
    import torch

    fmt, n_exp, hidden, inter, k, T = FMT_Q4_K, 2, 256, 256, 2, 1
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 90)
    x = synth.activations_numpy(T, hidden, 1)
    qd = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
    ids = torch.tensor([[1, 7]], dtype=torch.int32, device=dev)   # 7 is not a valid expert
    gate, up = capi.moe_gate_up(fmt, table, n_exp, ids, qd, T, k, hidden, inter)
    gate2 = torch.full_like(gate, 5.0)
    up2 = torch.full_like(up, 5.0)
    lib = capi.load()
    assert lib.llam_ql_moe_gate_up(fmt, table.data_ptr(), n_exp, ids.data_ptr(), qd.data_ptr(), gate2.data_ptr(),
                                   up2.data_ptr(), T, k, hidden, inter, 0, None)
    sync()
    assert (gate2[1] == 5.0).all() and (up2[1] == 5.0).all()      # untouched
    q8 = oracle.quantize(x)
    assert rel_err(gate2[0].cpu().numpy(), oracle.gemm(fmt, host[1][0], hidden, q8)[0]) <= 1e-5


@pytest.mark.parametrize("T", [1, 16])
def test_expert_ffn_baseline_shape(capi, dev, oracle, T):
    """Config 4: hidden 2048, 256 routed + 1 shared expert, top-8, intermediate 512, IQ3_S."""
    import torch

    fmt, n_exp, hidden, inter, k = FMT_IQ3_S, 256, 2048, 512, 8
    rng = np.random.default_rng(100 + T)
    # one big seeded slab per matrix kind, generated on the device; expert e is a slice
    def slab(rows, cols, seed):
        raw = synth.weights_torch(fmt, (n_exp + 1) * rows, cols, seed, dev)
        per = rows * (cols // 256) * 110
        return raw, per
    graw, gper = slab(inter, hidden, 1)
    uraw, uper = slab(inter, hidden, 2)
    draw, dper = slab(hidden, inter, 3)
    devs = []
    for e in range(n_exp + 1):
        devs.append((capi.prepare_weights(fmt, graw[e * gper:(e + 1) * gper].clone(), inter, hidden),
                     capi.prepare_weights(fmt, uraw[e * uper:(e + 1) * uper].clone(), inter, hidden),
                     capi.prepare_weights(fmt, draw[e * dper:(e + 1) * dper].clone(), hidden, inter)))
    table = capi.expert_table(devs, dev)
    x = rng.standard_normal((T, hidden)).astype(np.float32)
    logits = rng.standard_normal((T, n_exp)).astype(np.float32)
    xd = torch.from_numpy(x).to(dev)

    ids, w = capi.moe_route(torch.from_numpy(logits).to(dev), k, True)
    qd = capi.quantize_q8_1(xd)
    # routing and the quantiser of the hidden state in one launch: the bits of the two calls
    qd2 = torch.zeros_like(qd)
    ids2, w2 = capi.moe_route_quantize(torch.from_numpy(logits).to(dev), k, xd, qd2)
    sync()
    assert torch.equal(ids2, ids) and torch.equal(w2, w) and torch.equal(qd2, qd)
    gate, up = capi.moe_gate_up(fmt, table, n_exp + 1, ids, qd, T, k, hidden, inter)
    q8a = capi.swiglu_quantize(gate, up)
    out = torch.empty((T, hidden), device=dev)
    capi.moe_down(fmt, table, n_exp + 1, ids, w, q8a, out, T, k, hidden, inter, accumulate=False)
    # shared expert (id n_exp) for every token with weight 1, added ungated
    sid = torch.full((T, 1), n_exp, dtype=torch.int32, device=dev)
    sw = torch.ones((T, 1), device=dev)
    sg, su = capi.moe_gate_up(fmt, table, n_exp + 1, sid, qd, T, 1, hidden, inter)
    sq = capi.swiglu_quantize(sg, su)
    capi.moe_down(fmt, table, n_exp + 1, sid, sw, sq, out, T, 1, hidden, inter, accumulate=True)
    # the same in one gate/up and one down launch: the shared expert sits in a ninth slot
    # that the router leaves alone
    ids9 = torch.full((T, k + 1), n_exp, dtype=torch.int32, device=dev)
    w9 = torch.ones((T, k + 1), device=dev)
    capi.moe_route(torch.from_numpy(logits).to(dev), k, True, ids=ids9, weights=w9)
    gate9, up9 = capi.moe_gate_up(fmt, table, n_exp + 1, ids9, qd, T, k + 1, hidden, inter)
    out9 = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down(fmt, table, n_exp + 1, ids9, w9, capi.swiglu_quantize(gate9, up9), out9, T, k + 1, hidden, inter,
                  accumulate=False)
    sync()
    assert torch.equal(ids9[:, :k], ids) and torch.equal(w9[:, :k], w)
    assert (ids9[:, k] == n_exp).all() and (w9[:, k] == 1.0).all()
    assert rel_err(out9.cpu().numpy(), out.cpu().numpy()) <= 2e-6

    # oracle: the same chain on the CPU (own SwiGLU, own quantisation of it)
    rids, rw, _ = oracle.route(logits, k, True)
    assert np.array_equal(ids.cpu().numpy(), rids)
    q8 = oracle.quantize(x)
    gh, uh, dh = graw.cpu().numpy(), uraw.cpu().numpy(), draw.cpu().numpy()
    want = np.zeros((T, hidden), np.float32)
    for t in range(T):
        for e, wt in list(zip(rids[t].tolist(), rw[t].tolist())) + [(n_exp, 1.0)]:
            g = oracle.gemm(fmt, gh[e * gper:(e + 1) * gper], hidden, q8[t:t + 1])[0]
            u = oracle.gemm(fmt, uh[e * uper:(e + 1) * uper], hidden, q8[t:t + 1])[0]
            a = oracle.swiglu(g, u)
            d = oracle.gemm(fmt, dh[e * dper:(e + 1) * dper], inter, oracle.quantize(a[None]))[0]
            want[t] += np.float32(wt) * d
    # chained end to end: the SwiGLU differs by ulps between CPU and GPU, which can flip a
    # Q8_1 rounding in the down input; the IQ3_S output contract (1e-2) holds with margin
    assert rel_err(out.cpu().numpy(), want) <= 1e-3


def test_token_without_live_slot_gets_zeros(capi, dev):
    """accumulate == 0 overwrites: a token whose ids are all out of range (or whose experts
    live elsewhere) must end up zero, not keep what the buffer held (both down kernels and the
    grouped path); with accumulate != 0 its row is left alone."""
    import torch

    fmt, n_exp, T = FMT_Q4_K, 3, 3
    for hidden, inter, k in ((256, 256, 2), (512, 2304, 2)):  # multi-slot kernel / slot-by-slot kernel
        host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 7)
        ids = torch.tensor([[0, 2], [9, -1], [1, 9]], dtype=torch.int32, device=dev)
        w = torch.full((T, k), 0.5, device=dev)
        q8a = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(T * k, inter, 3)).to(dev))
        out = torch.full((T, hidden), 7.0, device=dev)
        capi.moe_down(fmt, table, n_exp, ids, w, q8a, out, T, k, hidden, inter, accumulate=False)
        acc = torch.full((T, hidden), 7.0, device=dev)
        capi.moe_down(fmt, table, n_exp, ids, w, q8a, acc, T, k, hidden, inter, accumulate=True)
        grp = capi.moe_group(ids, n_exp)
        pair_out = torch.full((T * k, hidden), float("nan"), device=dev)
        out_g = torch.full((T, hidden), 7.0, device=dev)
        capi.moe_down_grouped(fmt, table, n_exp, grp, ids, w, q8a, pair_out, out_g, T, k, hidden, inter)
        acc_g = torch.full((T, hidden), 7.0, device=dev)
        capi.moe_down_grouped(fmt, table, n_exp, grp, ids, w, q8a, pair_out, acc_g, T, k, hidden, inter, accumulate=True)
        sync()
        assert float(out[1].abs().max()) == 0.0 and float(out[0].abs().max()) > 0.0
        assert float((acc[1] - 7.0).abs().max()) == 0.0
        assert torch.equal(out_g, out)
        assert torch.equal(acc_g, acc)   # accumulate: ((out + v0) + v1) + .. on both paths


def test_group_tokens_by_expert(capi, dev):
    """The device-side sort of (token, slot) pairs by expert against numpy's stable argsort:
    segment table, order inside a segment, ids out of range left out."""
    import torch

    rng = np.random.default_rng(21)
    for T, S, E in ((1, 9, 257), (16, 9, 257), (5, 3, 4), (64, 9, 257), (7, 1, 2)):
        ids = rng.integers(-1, E + 2, size=(T, S)).astype(np.int32)  # -1, E and E+1 are invalid
        g = capi.moe_group(torch.from_numpy(ids).to(dev), E)
        sync()
        P = T * S
        w = g.cpu().numpy().view(np.int32)
        flat = ids.reshape(-1)
        valid = np.flatnonzero((flat >= 0) & (flat < E))
        order = valid[np.argsort(flat[valid], kind="stable")]
        experts = np.unique(flat[valid])
        n_seg, n_valid = int(w[0]), int(w[1])
        assert n_valid == len(valid) and n_seg == len(experts)
        seg_expert, seg_begin, pair_sorted = w[4:4 + P], w[4 + P:4 + 2 * P + 1], w[4 + 2 * P + 1:4 + 3 * P + 1]
        assert np.array_equal(seg_expert[:n_seg], experts)
        assert np.array_equal(pair_sorted[:n_valid], order)
        begins = np.searchsorted(flat[order], experts)
        assert np.array_equal(seg_begin[:n_seg], begins) and seg_begin[n_seg] == n_valid
        # chunks: every segment cut into runs of at most `per` pairs (2 below 512 pairs, else 4), in segment order
        per = 4 if P >= 512 else 2
        assert int(w[3]) == per
        c0 = 4 + 3 * P + 1
        chunk_expert, chunk_begin, chunk_count = w[c0:c0 + P], w[c0 + P:c0 + 2 * P], w[c0 + 2 * P:c0 + 3 * P]
        want = []
        ends = list(begins[1:]) + [n_valid]
        for e, b, en in zip(experts, begins, ends):
            for j in range(b, en, per):
                want.append((e, j, min(per, en - j)))
        assert int(w[2]) == len(want)
        got = list(zip(chunk_expert[:len(want)].tolist(), chunk_begin[:len(want)].tolist(), chunk_count[:len(want)].tolist()))
        assert got == [(int(e), int(b), int(c)) for e, b, c in want]


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_grouped_launches_equal_ungrouped(capi, dev, fmt):
    """Tokens grouped by expert: every gate/up row and every token output carries the bits of
    the ungrouped launches (12 tokens on 5 experts + an always-on slot: segments of 1..12 tokens,
    an expert missing from the table, an id out of range).  Rows of 4 and 2 super-blocks: both paths run the
    quad-lane decoders, the grouped one decoding each step once per chunk of an expert's tokens."""
    import torch

    def same(a, b):
        return torch.equal(a, b)

    n_exp, hidden, inter, k, T = 6, 1024, 512, 3, 12
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 60)
    tab = table.clone()
    tab.view(torch.int64).view(n_exp, 3)[4] = 0      # expert 4 lives elsewhere: null matrices
    rng = np.random.default_rng(9)
    ids = rng.integers(0, n_exp - 1, size=(T, k + 1)).astype(np.int32)
    ids[:, k] = n_exp - 1                             # the always-on expert in the extra slot
    ids[3, 1] = 77                                    # out of range
    idd = torch.from_numpy(ids).to(dev)
    w = torch.from_numpy(rng.random((T, k + 1)).astype(np.float32)).to(dev)
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(T, hidden, 4)).to(dev))
    S = k + 1
    gate = torch.full((T * S, inter), 3.0, device=dev)
    up = torch.full((T * S, inter), 3.0, device=dev)
    lib = capi.load()
    assert lib.llam_ql_moe_gate_up(fmt, tab.data_ptr(), n_exp, idd.data_ptr(), qd.data_ptr(), gate.data_ptr(),
                                   up.data_ptr(), T, S, hidden, inter, 0, None)
    grp = capi.moe_group(idd, n_exp)
    gate_g = torch.full((T * S, inter), 3.0, device=dev)
    up_g = torch.full((T * S, inter), 3.0, device=dev)
    capi.moe_gate_up_grouped(fmt, tab, n_exp, grp, qd, T, S, hidden, inter, gate=gate_g, up=up_g)
    sync()
    assert same(gate_g, gate) and same(up_g, up)
    q8a = capi.swiglu_quantize(gate, up)
    out = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down(fmt, tab, n_exp, idd, w, q8a, out, T, S, hidden, inter, accumulate=False)
    out_g = torch.full((T, hidden), float("nan"), device=dev)
    pair_out = torch.empty((T * S, hidden), device=dev)
    capi.moe_down_grouped(fmt, tab, n_exp, grp, idd, w, q8a, pair_out, out_g, T, S, hidden, inter)
    base = torch.from_numpy(rng.standard_normal((T, hidden)).astype(np.float32)).to(dev)
    acc, acc_g = base.clone(), base.clone()
    capi.moe_down(fmt, tab, n_exp, idd, w, q8a, acc, T, S, hidden, inter, accumulate=True)
    capi.moe_down_grouped(fmt, tab, n_exp, grp, idd, w, q8a, pair_out, acc_g, T, S, hidden, inter, accumulate=True)
    sync()
    assert same(out_g, out)
    assert same(acc_g, acc)   # the accumulate mode adds the slots onto the output in the same order
    assert bool(torch.isfinite(out).all())


def test_shared_expert_gate(capi, dev):
    import torch

    rng = np.random.default_rng(5)
    T, D = 3, 2048
    out = rng.standard_normal((T, D)).astype(np.float32)
    sh = rng.standard_normal((T, D)).astype(np.float32)
    h = rng.standard_normal((T, D)).astype(np.float32)
    gi = (rng.standard_normal(D) * 0.05).astype(np.float32)
    od = torch.from_numpy(out.copy()).to(dev)
    capi.shared_expert_add(od, torch.from_numpy(sh).to(dev), torch.from_numpy(h).to(dev), torch.from_numpy(gi).to(dev))
    sync()
    gate = 1.0 / (1.0 + np.exp(-(h.astype(np.float64) @ gi.astype(np.float64))))
    want = out + gate[:, None] * sh
    assert np.allclose(od.cpu().numpy(), want, rtol=1e-5, atol=1e-5)


def test_token_batching_helpers(capi, dev, oracle):
    """The remaining device helpers of the MoE operator interface: gather of token rows into an
    expert's batch (exact copy, rows with a bad index read as zeros), weighted scatter-add back
    (rows taken in order, so a token listed twice gets both contributions; bad indices skipped),
    the shared expert's sigmoid gate in place, and SwiGLU in place (the restatement's values,
    any count: the last count % 4 values take the scalar path)."""
    import torch

    lib = capi.load()
    rng = np.random.default_rng(6)
    T, D = 7, 2048
    hidden = rng.standard_normal((T, D)).astype(np.float32)
    idx = np.array([3, 0, 6, 3, -1, 7, 2], dtype=np.int32)       # 3 twice, two indices out of range
    hd = torch.from_numpy(hidden).to(dev)
    idx_d = torch.from_numpy(idx).to(dev)
    batch = torch.full((len(idx), D), float("nan"), device=dev)
    assert lib.llam_ql_moe_gather_rows(hd.data_ptr(), batch.data_ptr(), idx_d.data_ptr(), len(idx), T, D, 0, None), \
        capi.last_error()
    sync()
    want = np.stack([hidden[i] if 0 <= i < T else np.zeros(D, np.float32) for i in idx])
    assert np.array_equal(batch.cpu().numpy(), want)

    expert_out = rng.standard_normal((len(idx), D)).astype(np.float32)
    w = rng.uniform(0.1, 1.0, len(idx)).astype(np.float32)
    out0 = rng.standard_normal((T, D)).astype(np.float32)
    out = torch.from_numpy(out0.copy()).to(dev)
    assert lib.llam_ql_moe_scatter_add_weighted(out.data_ptr(), torch.from_numpy(expert_out).to(dev).data_ptr(),
                                                idx_d.data_ptr(), torch.from_numpy(w).to(dev).data_ptr(), len(idx), T,
                                                D, 0, None), capi.last_error()
    sync()
    want = out0.astype(np.float64)
    for i, t in enumerate(idx):
        if 0 <= t < T:
            want[t] += np.float64(w[i]) * expert_out[i]
    assert np.allclose(out.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    assert np.array_equal(out.cpu().numpy()[[1, 4, 5]], out0[[1, 4, 5]])   # tokens no row names are untouched

    sh = rng.standard_normal((T, D)).astype(np.float32)
    gi = (rng.standard_normal(D) * 0.05).astype(np.float32)
    shd = torch.from_numpy(sh.copy()).to(dev)
    assert lib.llam_ql_shared_expert_gate(shd.data_ptr(), hd.data_ptr(), torch.from_numpy(gi).to(dev).data_ptr(), T, D,
                                          0, None), capi.last_error()
    sync()
    gate = 1.0 / (1.0 + np.exp(-(hidden.astype(np.float64) @ gi.astype(np.float64))))
    assert np.allclose(shd.cpu().numpy(), gate[:, None] * sh, rtol=1e-5, atol=1e-6)

    for count in (4096, 1027, 3):
        g = (rng.standard_normal(count) * 3).astype(np.float32)
        u = rng.standard_normal(count).astype(np.float32)
        gd = torch.from_numpy(g.copy()).to(dev)
        assert lib.llam_ql_swiglu_inplace(gd.data_ptr(), torch.from_numpy(u).to(dev).data_ptr(), count, 0, None), \
            capi.last_error()
        sync()
        ref = oracle.swiglu(g, u)
        assert np.allclose(gd.cpu().numpy(), ref, rtol=2e-6, atol=1e-7), count
    assert not lib.llam_ql_swiglu_inplace(gd.data_ptr() + 4, gd.data_ptr(), 8, 0, None)
    assert "aligned" in capi.last_error()


def test_short_row_quad_lane_kernels_against_the_oracle(capi, dev, oracle):
    """IQ3_S with enough work for the quad-lane kernels on both stages (48 tokens, rows of 4 and 2 super-blocks):
    gate/up rows and the weighted down sums against the CPU restatement, with an id out of range, an expert whose
    matrices live elsewhere, a token without a live slot (zeros when overwriting, untouched when accumulating), and
    the accumulate mode."""
    import torch
    from oracle.binding import FMT_IQ3_S as fmt

    n_exp, hidden, inter, k, T = 6, 1024, 512, 4, 48
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 21)
    tab = table.clone()
    tab.view(torch.int64).view(n_exp, 3)[4] = 0       # expert 4 lives elsewhere: null matrices
    rng = np.random.default_rng(17)
    ids = rng.integers(0, n_exp, size=(T, k)).astype(np.int32)
    ids[3, 1] = 77                                     # out of range
    ids[5] = [-1, 9, 4, 99]                            # no live slot at all
    w = rng.random((T, k)).astype(np.float32)
    x = synth.activations_numpy(T, hidden, 4)
    idd, wd = torch.from_numpy(ids).to(dev), torch.from_numpy(w).to(dev)
    qd = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
    gate = torch.full((T * k, inter), 3.0, device=dev)
    up = torch.full((T * k, inter), 3.0, device=dev)
    lib = capi.load()
    assert lib.llam_ql_moe_gate_up(fmt, tab.data_ptr(), n_exp, idd.data_ptr(), qd.data_ptr(), gate.data_ptr(),
                                   up.data_ptr(), T, k, hidden, inter, 0, None)
    q8a = capi.swiglu_quantize(gate, up)
    out = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down(fmt, tab, n_exp, idd, wd, q8a, out, T, k, hidden, inter, accumulate=False)
    acc = torch.full((T, hidden), 2.0, device=dev)
    capi.moe_down(fmt, tab, n_exp, idd, wd, q8a, acc, T, k, hidden, inter, accumulate=True)
    sync()
    q8 = oracle.quantize(x)
    gate_h, up_h = gate.cpu().numpy(), up.cpu().numpy()
    q8a_h = q8a.cpu().numpy().reshape(T * k, inter // 32, 36)
    want = np.zeros((T, hidden), np.float64)
    for t in range(T):
        for s in range(k):
            e = int(ids[t, s])
            if e < 0 or e >= n_exp or e == 4:
                assert (gate_h[t * k + s] == 3.0).all() and (up_h[t * k + s] == 3.0).all()   # untouched
                continue
            if t % 6 == 0:                                                                     # a sample of the rows
                assert rel_err(gate_h[t * k + s], oracle.gemm(fmt, host[e][0], hidden, q8[t:t + 1])[0]) <= TOL[fmt] * 1e-2
                assert rel_err(up_h[t * k + s], oracle.gemm(fmt, host[e][1], hidden, q8[t:t + 1])[0]) <= TOL[fmt] * 1e-2
            want[t] += float(w[t, s]) * oracle.gemm(fmt, host[e][2], inter, q8a_h[t * k + s][None])[0]
    got = out.cpu().numpy()
    assert not got[5].any()                                                                    # the dead token: zeros
    assert rel_err(got, want.astype(np.float32)) <= TOL[fmt] * 1e-2
    acc_h = acc.cpu().numpy()
    assert (acc_h[5] == 2.0).all()
    assert rel_err(acc_h - 2.0, want.astype(np.float32)) <= 1e-5


@pytest.mark.parametrize("fmt,hidden", [(FMT_IQ3_S, 512), (FMT_IQ3_S, 1024), (FMT_IQ3_S, 2048), (FMT_IQ3_S, 4096),
                                        (FMT_Q4_K, 512), (FMT_Q4_K, 2048), (FMT_Q6_K, 1024), (FMT_Q6_K, 4096)])
def test_gate_up_swiglu_in_one_launch_has_the_bits_of_the_two(capi, dev, fmt, hidden):
    """Rows of 2, 4, 8 and 16 super-blocks: the Q8_1 blocks of the one-launch gate/up + SwiGLU + quantiser are
    the bytes of llam_ql_moe_gate_up followed by llam_ql_swiglu_quantize; blocks of a slot with an id out of range
    or an expert that lives elsewhere keep what the buffer held.  No scratch rows are needed (or touched)."""
    import torch

    n_exp, inter, k, T = 5, 768, 3, 5
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 33)
    tab = table.clone()
    tab.view(torch.int64).view(n_exp, 3)[2] = 0       # expert 2 lives elsewhere
    rng = np.random.default_rng(hidden)
    ids = rng.integers(0, n_exp, size=(T, k)).astype(np.int32)
    ids[1, 2] = -3
    ids[4, 0] = n_exp
    idd = torch.from_numpy(ids).to(dev)
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(T, hidden, 6)).to(dev))
    gate, up = capi.moe_gate_up(fmt, tab, n_exp, idd, qd, T, k, hidden, inter)
    want = capi.swiglu_quantize(gate, up).view(T * k, -1)
    got = torch.full((T * k * (inter // 32) * 36,), 0x5A, dtype=torch.uint8, device=dev)
    capi.moe_gate_up_swiglu(fmt, tab, n_exp, idd, qd, T, k, hidden, inter, q8_out=got)
    sync()
    got = got.view(T * k, -1)
    live = ((ids >= 0) & (ids < n_exp) & (ids != 2)).reshape(-1)
    assert live.sum() < T * k
    for r in range(T * k):
        if live[r]:
            assert torch.equal(got[r], want[r]), r
        else:
            assert bool((got[r] == 0x5A).all()), r


@pytest.mark.parametrize("fmt,hidden,T", [(FMT_IQ3_S, 2048, 24), (FMT_IQ3_S, 512, 40), (FMT_Q4_K, 1024, 24), (FMT_Q6_K, 2048, 30),
                                          (FMT_IQ3_S, 2048, 64), (FMT_IQ3_S, 2048, 70), (FMT_IQ3_S, 4096, 24)])
def test_gate_up_swiglu_many_slots_of_few_experts(capi, dev, fmt, hidden, T):
    """Many slots (72..210) of five experts, one of them used by every token: the launch shape for much work (two
    steps in flight per wavefront).  Every slot's blocks are the bytes of the two-launch path; dead slots keep what
    the buffer held."""
    import torch

    n_exp, inter, k = 5, 768, 3
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 71)
    tab = table.clone()
    tab.view(torch.int64).view(n_exp, 3)[3] = 0       # expert 3 lives elsewhere
    rng = np.random.default_rng(hidden + T)
    ids = rng.integers(0, n_exp, size=(T, k)).astype(np.int32)
    ids[1, 2] = -3
    ids[T - 1, 0] = n_exp
    ids[:, 1] = 4                                     # an expert every token uses (the always-on expert of a model)
    idd = torch.from_numpy(ids).to(dev)
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(T, hidden, 8)).to(dev))
    gate, up = capi.moe_gate_up(fmt, tab, n_exp, idd, qd, T, k, hidden, inter)
    want = capi.swiglu_quantize(gate, up).view(T * k, -1)
    got = torch.full((T * k * (inter // 32) * 36,), 0x5A, dtype=torch.uint8, device=dev)
    capi.moe_gate_up_swiglu(fmt, tab, n_exp, idd, qd, T, k, hidden, inter, q8_out=got)
    sync()
    got = got.view(T * k, -1)
    live = ((ids >= 0) & (ids < n_exp) & (ids != 3)).reshape(-1)
    assert 0 < live.sum() < T * k
    for r in range(T * k):
        if live[r]:
            assert torch.equal(got[r], want[r]), r
        else:
            assert bool((got[r] == 0x5A).all()), r


def test_gate_up_swiglu_other_row_lengths_run_the_two_launches(capi, dev):
    """Rows that are no power of two of super-blocks go through the caller's fp32 scratch rows; without them the
    call is refused."""
    import torch

    for fmt, hidden in ((FMT_Q4_K, 768), (FMT_IQ3_S, 768)):
        n_exp, inter, k, T = 3, 256, 2, 3
        host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 12)
        ids = torch.tensor([[0, 1], [2, 0], [1, 2]], dtype=torch.int32, device=dev)
        qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(T, hidden, 2)).to(dev))
        gate, up = capi.moe_gate_up(fmt, table, n_exp, ids, qd, T, k, hidden, inter)
        want = capi.swiglu_quantize(gate, up)
        scratch = (torch.empty_like(gate), torch.empty_like(up))
        got = capi.moe_gate_up_swiglu(fmt, table, n_exp, ids, qd, T, k, hidden, inter, scratch=scratch)
        sync()
        assert torch.equal(got, want)
        with pytest.raises(capi.QLError, match="scratch"):
            capi.moe_gate_up_swiglu(fmt, table, n_exp, ids, qd, T, k, hidden, inter)


@pytest.mark.parametrize("shape", [(FMT_IQ3_S, 2048, 512, 9, 1), (FMT_IQ3_S, 2048, 512, 9, 4), (FMT_IQ3_S, 1024, 1024, 4, 2),
                                   (FMT_IQ3_S, 512, 2048, 16, 1), (FMT_IQ3_S, 768, 512, 3, 3), (FMT_Q4_K, 1024, 512, 5, 2),
                                   (FMT_Q6_K, 512, 1024, 3, 1), (FMT_Q4_K, 768, 4096, 2, 3)])
def test_down_of_a_few_tokens_wavefront_per_slot(capi, dev, oracle, shape):
    """Down projection with little work per compute unit (a wavefront per slot): weighted sums against the CPU
    restatement on the same Q8_1 input, overwrite and accumulate, with a dead slot, a dead token when there are
    several, and the grouped path's bits to 1e-5 (its kernel adds a row's blocks in another order)."""
    import torch

    fmt, hidden, inter, k, T = shape
    n_exp = 5
    host, devs, table = _experts(capi, dev, fmt, n_exp, hidden, inter, 70 + k)
    tab = table.clone()
    tab.view(torch.int64).view(n_exp, 3)[3] = 0       # expert 3 lives elsewhere
    rng = np.random.default_rng(31 + T)
    ids = rng.integers(0, n_exp, size=(T, k)).astype(np.int32)
    ids[0, k - 1] = 42
    if T > 1:
        ids[T - 1] = -1
    w = rng.random((T, k)).astype(np.float32)
    idd, wd = torch.from_numpy(ids).to(dev), torch.from_numpy(w).to(dev)
    act = synth.activations_numpy(T * k, inter, 5)
    q8a = capi.quantize_q8_1(torch.from_numpy(act).to(dev))
    out = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down(fmt, tab, n_exp, idd, wd, q8a, out, T, k, hidden, inter, accumulate=False)
    base = rng.standard_normal((T, hidden)).astype(np.float32)
    acc = torch.from_numpy(base).to(dev)
    capi.moe_down(fmt, tab, n_exp, idd, wd, q8a, acc, T, k, hidden, inter, accumulate=True)
    grp = capi.moe_group(idd, n_exp)
    pair_out = torch.empty((T * k, hidden), device=dev)
    out_g = torch.full((T, hidden), float("nan"), device=dev)
    capi.moe_down_grouped(fmt, tab, n_exp, grp, idd, wd, q8a, pair_out, out_g, T, k, hidden, inter)
    sync()
    q8a_h = oracle.quantize(act)
    assert np.array_equal(q8a.cpu().numpy().reshape(q8a_h.shape), q8a_h)
    want = np.zeros((T, hidden), np.float64)
    for t in range(T):
        for s in range(k):
            e = int(ids[t, s])
            if 0 <= e < n_exp and e != 3:
                want[t] += float(w[t, s]) * oracle.gemm(fmt, host[e][2], inter, q8a_h[t * k + s][None])[0]
    got = out.cpu().numpy()
    assert np.isfinite(got).all()
    assert rel_err(got, want.astype(np.float32)) <= TOL[fmt] * 1e-2
    if T > 1:
        assert not got[T - 1].any()
        assert np.array_equal(acc.cpu().numpy()[T - 1], base[T - 1])
    assert rel_err(acc.cpu().numpy() - base, want.astype(np.float32)) <= 1e-5
    assert float((out_g - out).abs().max()) <= 1e-5 * float(out.abs().max())


@pytest.mark.parametrize("fmt,T,n_route,hidden", [(FMT_IQ3_S, 1, 256, 2048), (FMT_IQ3_S, 16, 256, 2048), (FMT_IQ3_S, 3, 60, 512),
                                                  (FMT_IQ3_S, 5, 300, 1024), (FMT_Q4_K, 2, 128, 1024), (FMT_Q6_K, 1, 64, 2048)])
def test_router_inside_the_gate_up_launch(capi, dev, fmt, T, n_route, hidden):
    """llam_ql_moe_route_gate_up_swiglu against llam_ql_moe_route_quantize + llam_ql_moe_gate_up_swiglu: the same
    ids and weights in the routed columns, the always-on column left as the caller set it, the same Q8_1 bytes for
    every slot (up to 512 routed experts: four or eight per lane of the routing wavefront)."""
    import torch

    inter, k = 256, 4
    n_tab = n_route + 1                                  # the last table entry is the always-on expert
    rng = np.random.default_rng(T + n_route)
    # few distinct expert matrices, many table entries: the table repeats them
    host, devs, _ = _experts(capi, dev, fmt, 7, hidden, inter, 50)
    table = capi.expert_table([devs[e % 7] for e in range(n_tab)], dev)
    x = torch.from_numpy(rng.standard_normal((T, hidden)).astype(np.float32)).to(dev)
    logits = torch.from_numpy(rng.standard_normal((T, n_route)).astype(np.float32)).to(dev)

    def fresh():
        ids = torch.full((T, k + 1), n_route, dtype=torch.int32, device=dev)
        w = torch.ones((T, k + 1), device=dev)
        return ids, w

    ids0, w0 = fresh()
    q8h = torch.empty(T * (hidden // 32) * 36, dtype=torch.uint8, device=dev)
    capi.moe_route_quantize(logits, k, x, q8h, ids=ids0, weights=w0)
    want = capi.moe_gate_up_swiglu(fmt, table, n_tab, ids0, q8h, T, k + 1, hidden, inter)
    ids1, w1 = fresh()
    got = capi.moe_route_gate_up_swiglu(fmt, table, n_tab, logits, k, x, ids1, w1, inter, q8_hidden=torch.empty_like(q8h))
    sync()
    assert torch.equal(ids1, ids0) and torch.equal(w1, w0)
    assert bool((ids1[:, k] == n_route).all()) and bool((w1[:, k] == 1.0).all())
    assert torch.equal(got, want)


def test_router_inside_other_row_lengths_run_the_launches_one_by_one(capi, dev):
    import torch

    fmt, T, n_route, hidden, inter, k = FMT_Q4_K, 2, 5, 768, 256, 2   # rows of three super-blocks: no quad-lane launch
    host, devs, table = _experts(capi, dev, fmt, n_route, hidden, inter, 77)
    rng = np.random.default_rng(5)
    x = torch.from_numpy(rng.standard_normal((T, hidden)).astype(np.float32)).to(dev)
    logits = torch.from_numpy(rng.standard_normal((T, n_route)).astype(np.float32)).to(dev)
    ids0 = torch.zeros((T, k), dtype=torch.int32, device=dev)
    w0 = torch.zeros((T, k), device=dev)
    q8h = torch.empty(T * (hidden // 32) * 36, dtype=torch.uint8, device=dev)
    capi.moe_route_quantize(logits, k, x, q8h, ids=ids0, weights=w0)
    gate, up = capi.moe_gate_up(fmt, table, n_route, ids0, q8h, T, k, hidden, inter)
    want = capi.swiglu_quantize(gate, up)
    ids1, w1 = torch.zeros_like(ids0), torch.zeros_like(w0)
    got = capi.moe_route_gate_up_swiglu(fmt, table, n_route, logits, k, x, ids1, w1, inter, q8_hidden=torch.empty_like(q8h),
                                        scratch=(torch.empty_like(gate), torch.empty_like(up)))
    sync()
    assert torch.equal(ids1, ids0) and torch.equal(w1, w0) and torch.equal(got, want)
    with pytest.raises(capi.QLError, match="scratch"):
        capi.moe_route_gate_up_swiglu(fmt, table, n_route, logits, k, x, ids1, w1, inter)
