"""The entry points under HIP-graph capture: a decode step (quantise, fused Q/K/V
GEMV, O projection, gate+up, SwiGLU+quantise, down) captured once and replayed
several times with new inputs and eager work in between; every replay must equal
the eager result bit for bit (the kernels are deterministic and the library neither
allocates nor synchronises, so capture must not change anything)."""
import numpy as np
import pytest
import torch

from llaminar_amd import synth
from oracle.binding import FMT_Q4_K, FMT_Q6_K

pytestmark = pytest.mark.gpu


def test_decode_step_graph_replays_match_eager(capi, dev):
    d_model, d_ff, n_kv = 1024, 2816, 256
    mk = lambda fmt, N, K, seed: capi.prepare_weights(
        fmt, torch.from_numpy(synth.weights_numpy(fmt, N, K, seed).reshape(-1)).to(dev), N, K)
    wq, wk, wv = mk(FMT_Q4_K, d_model, d_model, 1), mk(FMT_Q4_K, n_kv, d_model, 2), mk(FMT_Q4_K, n_kv, d_model, 3)
    wo = mk(FMT_Q4_K, d_model, d_model, 4)
    wg, wu = mk(FMT_Q4_K, d_ff, d_model, 5), mk(FMT_Q4_K, d_ff, d_model, 6)
    wd = mk(FMT_Q6_K, d_model, d_ff, 7)

    x = torch.empty(1, d_model, device=dev)
    q8 = torch.empty((d_model // 32) * 36, dtype=torch.uint8, device=dev)
    q = torch.empty(1, d_model, device=dev)
    k = torch.empty(1, n_kv, device=dev)
    v = torch.empty(1, n_kv, device=dev)
    q8o = torch.empty_like(q8)
    o = torch.empty(1, d_model, device=dev)
    g = torch.empty(1, d_ff, device=dev)
    u = torch.empty(1, d_ff, device=dev)
    q8a = torch.empty((d_ff // 32) * 36, dtype=torch.uint8, device=dev)
    y = torch.empty(1, d_model, device=dev)
    lib = capi.load()

    def step(stream):
        s = stream.cuda_stream
        capi.quantize_q8_1(x, out=q8, stream=s)
        capi.gemv_fused([(FMT_Q4_K, wq, q), (FMT_Q4_K, wk, k), (FMT_Q4_K, wv, v)], q8, 1,
                        d_model, stream=s)
        capi.quantize_q8_1(q, out=q8o, stream=s)  # stands in for the attention output
        capi.gemv(FMT_Q4_K, wo, q8o, 1, d_model, d_model, out=o, stream=s)
        capi.gemv_fused([(FMT_Q4_K, wg, g), (FMT_Q4_K, wu, u)], q8, 1, d_model, stream=s)
        assert lib.llam_ql_swiglu_quantize(g.data_ptr(), u.data_ptr(), 0, q8a.data_ptr(), 1, d_ff, 0, s)
        capi.gemv(FMT_Q6_K, wd, q8a, 1, d_model, d_ff, out=y, stream=s)

    inputs = [torch.from_numpy(synth.activations_numpy(1, d_model, 100 + i)).to(dev) for i in range(4)]
    stream = torch.cuda.Stream()

    eager = []
    with torch.cuda.stream(stream):
        for inp in inputs:
            x.copy_(inp)
            step(stream)
            stream.synchronize()
            eager.append((o.clone(), k.clone(), y.clone()))

    graph = torch.cuda.CUDAGraph()
    with torch.cuda.stream(stream):
        x.copy_(inputs[0])
        step(stream)  # warm-up outside capture
        stream.synchronize()
        with torch.cuda.graph(graph, stream=stream):
            step(stream)
    torch.cuda.synchronize()

    scratch = torch.zeros(1 << 20, device=dev)
    for rep in range(3):
        for i, inp in enumerate(inputs):
            x.copy_(inp)
            for t in (q, k, v, o, g, u, y):
                t.fill_(float("nan"))  # a replay has to rewrite every output
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            eo, ek, ey = eager[i]
            assert torch.equal(o, eo) and torch.equal(k, ek) and torch.equal(y, ey), (rep, i)
            # the program's own eager work between replays
            scratch.add_(1.0)
            capi.gemv(FMT_Q4_K, wo, q8o, 1, d_model, d_model)
            torch.cuda.synchronize()
    assert np.isfinite(y.cpu().numpy()).all()


def test_batch_plane_launches_replay(capi, dev):
    """Batches of eight rows launched with their matrices' batch planes, captured once: every replay equals the
    eager result, with eager launches of the same matrices (without a plane) between the replays."""
    M, H, F = 8, 2048, 4096
    mk = lambda fmt, N, K, seed: capi.prepare_weights(
        fmt, torch.from_numpy(synth.weights_numpy(fmt, N, K, seed).reshape(-1)).to(dev), N, K)
    wu, wd = mk(FMT_Q4_K, F, H, 11), mk(FMT_Q6_K, F, H, 12)
    pu, pd = capi.build_batch_plane(FMT_Q4_K, wu, F, H), capi.build_batch_plane(FMT_Q6_K, wd, F, H)
    assert pu is not None and pd is not None
    x = torch.empty(M, H, device=dev)
    q8 = torch.empty(M * (H // 32) * 36, dtype=torch.uint8, device=dev)
    a, b = torch.empty(M, F, device=dev), torch.empty(M, F, device=dev)

    def step(stream):
        s = stream.cuda_stream
        capi.quantize_q8_1(x, out=q8, stream=s)
        capi.gemv(FMT_Q4_K, wu, q8, M, F, H, out=a, stream=s, plane=pu)
        capi.gemv(FMT_Q6_K, wd, q8, M, F, H, out=b, stream=s, plane=pd)

    inputs = [torch.from_numpy(synth.activations_numpy(M, H, 200 + i)).to(dev) for i in range(3)]
    stream = torch.cuda.Stream()
    eager = []
    with torch.cuda.stream(stream):
        for inp in inputs:
            x.copy_(inp)
            step(stream)
            stream.synchronize()
            eager.append((a.clone(), b.clone()))
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=stream):
            step(stream)
    torch.cuda.synchronize()
    for rep in range(2):
        for i, inp in enumerate(inputs):
            x.copy_(inp)
            a.fill_(float("nan"))
            b.fill_(float("nan"))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            assert torch.equal(a, eager[i][0]) and torch.equal(b, eager[i][1]), (rep, i)
            capi.gemv(FMT_Q6_K, wd, q8, M, F, H)   # eager work between the replays, now without a plane
            torch.cuda.synchronize()
