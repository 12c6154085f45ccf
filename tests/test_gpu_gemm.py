"""P3 on the GPU: prefill GEMM (int8 MFMA, per-block fp32 rescale) through the
C-ABI against the oracle, and against the decode GEMV whose per-block integer
pipeline is separately pinned bit-exact."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import FMTS, TOL, rel_err, sync, upload_q8, upload_weights

pytestmark = pytest.mark.gpu

GOLD = {FMT_Q4_K: "q4k", FMT_Q6_K: "q6k", FMT_IQ3_S: "iq3s"}


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_golden_fixture(capi, dev, golden, fmt):
    name = GOLD[fmt]
    W = golden[f"{name}_w"]
    N, K = W.shape[0], W.shape[1] * 256
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, golden["act_q8"])
    for M in (1, 4, 5):
        y = capi.gemm(fmt, wd, qd, M, N, K)
        sync()
        assert rel_err(y.cpu().numpy(), golden[f"{name}_c_avx512_m{M}"]) <= TOL[fmt] * 1e-2


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
@pytest.mark.parametrize("M,N,K", [(1, 128, 256), (17, 100, 512), (128, 128, 1024), (130, 257, 768), (300, 64, 2048),
                                   # launches of few tokens run tiles of 32 tokens: one, two (the second
                                   # holds one token) and three rows of tiles, then the first 128-token launch
                                   (32, 200, 1024), (33, 130, 5120), (96, 64, 2048), (97, 64, 2048)])
def test_random_shapes(capi, dev, oracle, fmt, M, N, K):
    W = synth.weights_numpy(fmt, N, K, 7 + M + N)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 9 + K))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    y = capi.gemm(fmt, wd, qd, M, N, K)
    sync()
    C = oracle.gemm(fmt, W, K, q8)
    assert rel_err(y.cpu().numpy(), C) <= TOL[fmt] * 1e-2


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_gemm_rows_equal_gemv(capi, dev, oracle, fmt):
    """Integer parity by transitivity: the GEMV's block sums are bit-exact, and every GEMM
    row must reproduce the GEMV output of that row to fp32 re-association accuracy."""
    M, N, K = 8, 384, 5120
    W = synth.weights_numpy(fmt, N, K, 71)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 72))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    yg = capi.gemm(fmt, wd, qd, M, N, K)
    yv = capi.gemv(fmt, wd, qd, M, N, K)
    sync()
    assert rel_err(yg.cpu().numpy(), yv.cpu().numpy()) <= 2e-6


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
@pytest.mark.parametrize("M,N,K,r0,nr", [(1, 128, 256, 0, 128), (17, 100, 512, 37, 63), (130, 257, 768, 190, 67),
                                         (300, 200, 2048, 60, 70), (40, 130, 1280, 60, 70), (96, 70, 512, 0, 70)])
def test_block_sums_of_the_gemm_kernel(capi, dev, oracle, fmt, M, N, K, r0, nr):
    """The matrix unit's per-block results of llam_ql_gemm's own kernel (block-sum variant) are
    the reference's int32 sums bit for bit: ragged tiles, windows that start and end inside a
    64-row tile, token tails, and the 32-token tiles that launches of up to 96 tokens run (there four
    wavefronts share a tile's blocks of a step)."""
    W = synth.weights_numpy(fmt, N, K, 70 + M + N)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 90 + K))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    s = capi.gemm_block_sums(fmt, wd, qd, M, N, K, r0, nr)
    sync()
    _, sums = oracle.gemm(fmt, W, K, q8, n0=r0, n1=r0 + nr, want_sums=True)
    assert np.array_equal(s.cpu().numpy(), sums)


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_more_tiles_than_the_chip_holds(capi, dev, oracle, fmt):
    """More tiles than the chip holds at once, with a sparsely filled last round of workgroups
    (580 tiles of 128 x 64 on 512 workgroup slots), ragged in both directions (130 tokens: the
    second token tile holds two; 18550 rows: the last row tile holds 54): every output element
    written exactly once and equal to the oracle's."""
    import torch

    M, N, K = 130, 18550, 512
    W = synth.weights_numpy(fmt, N, K, 4242)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 4243))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    y = torch.full((M, N), float("nan"), device=dev)
    capi.gemm(fmt, wd, qd, M, N, K, out=y)
    sync()
    got = y.cpu().numpy()
    assert np.isfinite(got).all()
    C = oracle.gemm(fmt, W, K, q8)
    assert rel_err(got, C) <= TOL[fmt] * 1e-2
    # the worst single element, too: a misplaced tile would hide in a norm
    assert np.abs(got - C).max() <= 1e-4 * np.abs(C).max()
    y2 = torch.full((M, N), float("nan"), device=dev)
    capi.gemm(fmt, wd, qd, M, N, K, out=y2)
    sync()
    assert torch.equal(y, y2)


def test_prefill_config_full_size(capi, dev, oracle):
    """Config 3: M=512, K=5120, N=25600, Q4_K.  Oracle on a window of weight rows for all
    512 tokens; determinism over the whole output."""
    import torch

    M, N, K = 512, 25600, 5120
    fmt = FMT_Q4_K
    wd = synth.weights_torch(fmt, N, K, 31337, dev)
    x = synth.activations_numpy(M, K, 5)
    xd = torch.from_numpy(x).to(dev)
    qd = capi.quantize_q8_1(xd)
    y = capi.gemm(fmt, wd, qd, M, N, K)
    y2 = capi.gemm(fmt, wd, qd, M, N, K)
    sync()
    assert torch.equal(y, y2)
    q8 = oracle.quantize(x)
    assert np.array_equal(qd.cpu().numpy().reshape(q8.shape), q8)
    Wh = wd.cpu().numpy()
    for n0 in (0, 12800 - 32, N - 64):
        C, sums = oracle.gemm(fmt, Wh, K, q8, n0=n0, n1=n0 + 64, want_sums=True)
        assert rel_err(y.cpu().numpy()[:, n0:n0 + 64], C) <= TOL[fmt] * 1e-2
        s = capi.gemm_block_sums(fmt, wd, qd, M, N, K, n0, 64)
        sync()
        assert np.array_equal(s.cpu().numpy(), sums), f"block sums of rows from {n0}"
    assert np.isfinite(y.cpu().numpy()).all()


def test_epilogue_alpha_beta_bias(capi, dev, oracle):
    import torch

    rng = np.random.default_rng(4)
    C = rng.standard_normal((5, 96)).astype(np.float32)
    T = rng.standard_normal((5, 96)).astype(np.float32)
    b = rng.standard_normal(96).astype(np.float32)
    for alpha, beta, bias in ((1.0, 0.0, None), (0.5, 2.0, b), (2.0, 1.0, None)):
        cd = torch.from_numpy(C.copy()).to(dev)
        capi.epilogue(cd, torch.from_numpy(T).to(dev), None if bias is None else torch.from_numpy(bias).to(dev),
                      alpha, beta)
        sync()
        want = oracle.epilogue(C, T, alpha, beta, bias)
        assert np.allclose(cd.cpu().numpy(), want, rtol=1e-6, atol=1e-6)
    # beta == 0 must overwrite NaNs, like the reference's zero-fill
    cd = torch.full((5, 96), float("nan"), device=dev)
    capi.epilogue(cd, torch.from_numpy(T).to(dev), None, 1.0, 0.0)
    sync()
    assert np.array_equal(cd.cpu().numpy(), T)


def test_empty_and_errors(capi, dev):
    import torch

    lib = capi.load()
    w = torch.zeros(4096, dtype=torch.uint8, device=dev)
    y = torch.zeros(64, device=dev)
    assert lib.llam_ql_gemm(FMT_Q4_K, w.data_ptr(), w.data_ptr(), y.data_ptr(), 0, 4, 256, 4, 0, None)
    assert not lib.llam_ql_gemm(FMT_Q4_K, w.data_ptr(), w.data_ptr(), y.data_ptr(), 2, 4, 255, 4, 0, None)
