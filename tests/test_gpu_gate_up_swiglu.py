"""The feed-forward block's first half in one launch at batches of 2..8 (llam_ql_gemv_gate_up_swiglu): gate and
up projection on the matrix unit, SwiGLU and the Q8_1 quantiser of the down projection's input in the workgroup
that holds both operands.  The projections are checked against the oracle and the unfused launches, the Q8_1
blocks bit for bit against the stand-alone SwiGLU quantiser on the launch's own projections."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import TOL, rel_err, sync, upload_q8, upload_weights

pytestmark = pytest.mark.gpu

# (M, N, K): one pair of tiles per workgroup and several; a count of pairs that leaves the last workgroup
# partly empty (129 pairs); the shortest rows served (8 super-blocks); rows of 32 super-blocks;
# the longest rows served with few tiles (two tiles of eight wavefronts would not fit the LDS: fewer per tile)
# batches of 2..4 (served for callers that do not need the bits of single-row calls)
_CASES = [(8, 4096, 2048), (5, 4128, 5120), (7, 8192, 8192), (6, 12800, 5120), (8, 4096, 10240), (5, 4096, 11520),
          (2, 4096, 5120), (3, 8192, 4096), (4, 25600, 5120)]


@pytest.mark.parametrize("with_planes", [False, True], ids=["prepared", "planes"])
@pytest.mark.parametrize("M,N,K", _CASES)
def test_blocks_are_the_quantised_swiglu_of_the_launchs_projections(capi, dev, oracle, M, N, K, with_planes):
    fmt = FMT_Q4_K
    assert capi.gemv_gate_up_swiglu_supported(fmt, M, N, K)
    Wg = synth.weights_numpy(fmt, N, K, 1000 + N)
    Wu = synth.weights_numpy(fmt, N, K, 2000 + N)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 3000 + K))
    wg, wu, qd = upload_weights(capi, dev, fmt, Wg), upload_weights(capi, dev, fmt, Wu), upload_q8(dev, q8)
    pg = capi.build_batch_plane(fmt, wg, N, K) if with_planes else None
    pu = capi.build_batch_plane(fmt, wu, N, K) if with_planes else None
    assert (pg is not None) == with_planes
    blocks, yg, yu = capi.gemv_gate_up_swiglu(fmt, wg, wu, qd, M, N, K, plane_gate=pg, plane_up=pu,
                                              want_projections=True)
    sync()
    # the projections: the reference's arithmetic within the fp32 contract, on a window of rows the oracle finishes
    # quickly, and the unfused launches to re-association accuracy everywhere
    for W, y in ((Wg, yg), (Wu, yu)):
        for n0 in (0, N - 96):
            C = oracle.gemm(fmt, W, K, q8, n0=n0, n1=n0 + 96)
            assert rel_err(y.cpu().numpy()[:, n0:n0 + 96], C) <= TOL[fmt] * 1e-2
    assert rel_err(yg.cpu().numpy(), capi.gemv(fmt, wg, qd, M, N, K, plane=pg).cpu().numpy()) <= 2e-6
    assert rel_err(yu.cpu().numpy(), capi.gemv(fmt, wu, qd, M, N, K, plane=pu).cpu().numpy()) <= 2e-6
    # the blocks: the stand-alone quantiser on the same projections, bit for bit
    want = capi.swiglu_quantize(yg, yu)
    sync()
    assert np.array_equal(blocks.cpu().numpy(), want.cpu().numpy())
    # without the fp32 outputs the same blocks
    only = capi.gemv_gate_up_swiglu(fmt, wg, wu, qd, M, N, K, plane_gate=pg, plane_up=pu)
    sync()
    assert np.array_equal(only.cpu().numpy(), blocks.cpu().numpy())


def test_planes_and_prepared_matrices_give_the_same_bits(capi, dev, oracle):
    fmt, M, N, K = FMT_Q4_K, 8, 5120, 5120
    Wg = synth.weights_numpy(fmt, N, K, 11)
    Wu = synth.weights_numpy(fmt, N, K, 12)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 13))
    wg, wu, qd = upload_weights(capi, dev, fmt, Wg), upload_weights(capi, dev, fmt, Wu), upload_q8(dev, q8)
    pg, pu = capi.build_batch_plane(fmt, wg, N, K), capi.build_batch_plane(fmt, wu, N, K)
    a = capi.gemv_gate_up_swiglu(fmt, wg, wu, qd, M, N, K, want_projections=True)
    b = capi.gemv_gate_up_swiglu(fmt, wg, wu, qd, M, N, K, plane_gate=pg, plane_up=pu, want_projections=True)
    sync()
    for x, y in zip(a, b):
        assert np.array_equal(x.cpu().numpy(), y.cpu().numpy())


def test_full_size_block_against_the_oracles_swiglu(capi, dev, oracle):
    """Config 2's gate/up shape at batch 8: the dequantised blocks lie within the Q8_1 step of the oracle's
    silu(gate) * up of the oracle's own projections (a window of rows)."""
    fmt, M, N, K = FMT_Q4_K, 8, 25600, 5120
    wg = synth.weights_torch(fmt, N, K, 21, dev)
    wu = synth.weights_torch(fmt, N, K, 22, dev)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 23))
    qd = upload_q8(dev, q8)
    pg, pu = capi.build_batch_plane(fmt, wg, N, K), capi.build_batch_plane(fmt, wu, N, K)
    blocks = capi.gemv_gate_up_swiglu(fmt, wg, wu, qd, M, N, K, plane_gate=pg, plane_up=pu)
    sync()
    raw = blocks.cpu().numpy().reshape(M, N // 32, 36)
    d = raw[:, :, :2].copy().view(np.float16).astype(np.float32)[:, :, 0]
    qs = raw[:, :, 4:].view(np.int8).astype(np.float32)
    got = (qs * d[:, :, None]).reshape(M, N)
    Wg, Wu = wg.cpu().numpy(), wu.cpu().numpy()
    for n0 in (0, 12800, N - 64):
        g = oracle.gemm(fmt, Wg, K, q8, n0=n0, n1=n0 + 64)
        u = oracle.gemm(fmt, Wu, K, q8, n0=n0, n1=n0 + 64)
        act = oracle.swiglu(g, u)
        for b in range(2):
            blk = slice(32 * b, 32 * b + 32)
            step = np.abs(act[:, blk]).max(axis=1, keepdims=True) / 127.0
            assert (np.abs(got[:, n0:n0 + 64][:, blk] - act[:, blk]) <= 0.51 * step + 1e-3 * np.abs(act[:, blk]).max()).all()
    # sum_qs of every block is the sum of its quants
    sums = raw[:, :, 2:4].copy().view(np.int16)[:, :, 0]
    assert np.array_equal(sums, raw[:, :, 4:].view(np.int8).astype(np.int32).sum(axis=2))


def test_shapes_that_are_not_served(capi, dev):
    import torch

    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, 1, 8192, 5120)      # a single row: the quad-lane kernel
    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, 8, 8200, 5120)      # N not a multiple of 32
    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, 8, 2048, 5120)      # too few rows for the matrix unit
    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, 8, 5120, 25600)     # rows walked in chunks
    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q4_K, 8, 8192, 11776)     # (from 46 super-blocks on)
    assert not capi.gemv_gate_up_swiglu_supported(FMT_Q6_K, 8, 8192, 5120)
    assert not capi.gemv_gate_up_swiglu_supported(FMT_IQ3_S, 8, 8192, 5120)
    w = torch.zeros(8192 * 20 * 144, dtype=torch.uint8, device=dev)
    q = torch.zeros(160 * 36, dtype=torch.uint8, device=dev)
    with pytest.raises(capi.QLError, match="not served"):
        capi.gemv_gate_up_swiglu(FMT_Q4_K, w, w, q, 1, 8192, 5120)
    # a plane for one matrix only
    q = torch.zeros(8 * 160 * 36, dtype=torch.uint8, device=dev)
    plane = torch.zeros(capi.batch_plane_bytes(FMT_Q4_K, 8192, 5120), dtype=torch.uint8, device=dev)
    with pytest.raises(capi.QLError, match="both matrices"):
        capi.gemv_gate_up_swiglu(FMT_Q4_K, w, w, q, 8, 8192, 5120, plane_gate=plane)
