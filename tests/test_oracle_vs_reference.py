"""The restatement against the reference's own compiled CPU kernels (oracle/_ref),
on larger seeded sweeps than the committed fixtures hold.  Skipped on machines
that never saw the reference tree; the golden-vector tests cover those."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K

FMTS = [FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S]


def test_q8_1_rows_bit_exact(oracle, ref):
    for seed, scale in ((1, 1.0), (2, 1e-4), (3, 1e-8), (4, 1e3)):
        x = synth.activations_numpy(32, 5120, seed) * np.float32(scale)
        x[0, :64] = 0
        assert np.array_equal(oracle.quantize(x), ref.quantize(x))


@pytest.mark.parametrize("fmt", FMTS)
def test_subblocks_bit_exact(oracle, ref, fmt):
    for seed, (lo, hi) in enumerate([(0.001, 0.02), (1e-6, 1e-4), (1.0, 50.0)]):
        W = synth.weights_numpy(fmt, 48, 1024, 100 + seed, d_lo=lo, d_hi=hi)
        for n in range(48):
            for s in range(4):
                w, sc, mn = oracle.subblocks(fmt, W[n, s])
                w2, sc2, mn2 = ref.unpack_superblock(fmt, W[n, s])
                assert np.array_equal(w, w2)
                assert [ref.f32_to_f16(float(v)) for v in sc2] == list(sc)
                assert [ref.f32_to_f16(float(v)) for v in mn2] == list(mn)


@pytest.mark.parametrize("fmt", FMTS)
@pytest.mark.parametrize("M", [1, 2, 7])
def test_gemm_float_exact(oracle, ref, fmt, M, monkeypatch):
    # one accumulation chain per output: keep the reference from K-tiling the GEMV
    N, K = 320, 2048
    W = synth.weights_numpy(fmt, N, K, 31)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 32))
    for isa in (1, 2):
        C2 = ref.gemm(fmt, W, N, K, q8, isa=isa)
        C = oracle.gemm(fmt, W, K, q8)
        assert np.array_equal(C.view(np.uint32), C2.view(np.uint32))


def test_router_bit_exact(oracle, ref):
    """qlo_moe_route against CPUMoEKernel::route from the logits on (the reference's softmax_row_fp32 in every ISA
    variant, its partial_sort and renormalisation): probabilities, ids and weights bit for bit.  With exactly equal
    probabilities the reference's partial_sort leaves the order to the library; the restatement (and the GPU
    kernel) take the lower expert id first, so ties are compared as sets of weights only."""
    if not ref.has_route:
        pytest.skip("oracle/_ref predates the router door")
    rng = np.random.default_rng(3)
    for spread in (0.5, 1.0, 8.0, 30.0):   # (wider spreads underflow to exact zeros: ties, below)
        lg = (rng.standard_normal((64, 256)) * spread).astype(np.float32)
        for variant in (0, 1, 2, 3):
            for normalize in (True, False):
                ids, w, probs = ref.moe_route(lg, 8, normalize, variant)
                oi, ow, op = oracle.route(lg, 8, normalize)
                assert np.array_equal(op, probs) and np.array_equal(oi, ids) and np.array_equal(ow, w), (spread, variant)
    lg = rng.standard_normal((32, 256)).astype(np.float32)
    for t in range(32):
        top = np.argsort(-lg[t])[:10]
        lg[t, top[3]] = lg[t, top[4]] = lg[t, top[5]]
        lg[t, top[7]] = lg[t, top[8]]          # a tie across the cut after the eighth
    ids, w, probs = ref.moe_route(lg, 8, True, 0)
    oi, ow, op = oracle.route(lg, 8, True)
    assert np.array_equal(op, probs) and np.array_equal(ow, w)
    for t in range(32):
        assert np.array_equal(np.sort(op[t][oi[t]]), np.sort(probs[t][ids[t]]))
        order = np.lexsort((oi[t], -op[t][oi[t]]))          # by probability, ties by expert id
        assert np.array_equal(order, np.arange(8)), t
