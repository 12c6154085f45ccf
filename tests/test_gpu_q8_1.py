"""P1 on the GPU: the Q8_1 activation quantiser, through the C-ABI, must write the
same bytes as the reference's CPU quantiser (oracle + golden fixtures)."""
import numpy as np
import pytest

from llaminar_amd import synth
from tests.helpers import sync

pytestmark = pytest.mark.gpu


def _gpu_quantize(capi, dev, x):
    import torch

    xd = torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(dev)
    q = capi.quantize_q8_1(xd)
    sync()
    M, K = x.shape
    return q.cpu().numpy().reshape(M, (K + 31) // 32, 36)


def test_golden_blocks(capi, dev, golden):
    x = golden["q8_in"]                       # [n,32] incl. zero, threshold, subnormal-d, clamp and tie rows
    got = _gpu_quantize(capi, dev, x)[:, 0, :]
    assert np.array_equal(got, golden["q8_avx512"])


@pytest.mark.parametrize("K", [256])
def test_golden_rows(capi, dev, golden, K):
    got = _gpu_quantize(capi, dev, golden[f"q8_rows_in_{K}"])
    assert np.array_equal(got, golden[f"q8_rows_{K}"])


@pytest.mark.parametrize("M,K,scale", [(1, 5120, 1.0), (8, 5120, 1.0), (1, 25600, 1.0), (3, 8192, 1e-4),
                                       (5, 2048, 1e-8), (2, 512, 3e4), (7, 32, 1.0), (1, 96, 1.0)])
def test_random_rows_bit_exact(capi, dev, oracle, M, K, scale):
    x = synth.activations_numpy(M, K, 1000 + M + K) * np.float32(scale)
    x[0, :32] = 0.0
    if K >= 96:
        x[M - 1, 32:64] = 1e-11
    assert np.array_equal(_gpu_quantize(capi, dev, x), oracle.quantize(x))


@pytest.mark.parametrize("M,K", [(1, 1), (1, 31), (3, 33), (2, 48), (5, 100), (1, 5121), (4, 5151)])
def test_partial_last_block_bit_exact(capi, dev, oracle, M, K):
    """Rows whose length is not a multiple of 32: the last block of a row holds K % 32 values and
    follows the reference's scalar quantiser (round half away from zero, software fp16, zero
    padding), the full blocks before it the SIMD one.  Row 0 is built so that x * id lands on
    exact .5 ties in both kinds of block (amax 127 makes d = id = 1): the two roundings differ there."""
    x = synth.activations_numpy(M, K, 3000 + M + K)
    ties = (np.arange(K) % 32).astype(np.float32) - 15.5     # -15.5 .. 15.5
    x[0] = ties
    x[0, (np.arange(K) % 32) == 0] = 127.0                    # every block's amax
    if K > 32 * 2 and M > 1:
        x[1, 32 * ((K - 1) // 32):] = 1e-11                   # a partial block below the zero threshold
        x[M - 1, 32 * ((K - 1) // 32):] *= np.float32(1e-7)   # its d is an fp16 subnormal (truncated)
    want = oracle.quantize(x)
    got = _gpu_quantize(capi, dev, x)
    assert np.array_equal(got, want)
    tail = K % 32
    assert (got[:, -1, 4 + tail:] == 0).all()                 # zero padding


def test_prefill_size_bit_exact(capi, dev, oracle):
    x = synth.activations_numpy(512, 5120, 7)      # config 3: 81,920 blocks
    assert np.array_equal(_gpu_quantize(capi, dev, x), oracle.quantize(x))


def test_invariants_at_full_size(capi, dev):
    x = synth.activations_numpy(512, 5120, 8)
    q = _gpu_quantize(capi, dev, x)
    qs = q[:, :, 4:].view(np.int8)
    s = q[:, :, 2:4].copy().view(np.int16)[..., 0]
    d = q[:, :, 0:2].copy().view(np.float16)[..., 0].astype(np.float32)
    assert np.array_equal(s, qs.astype(np.int32).sum(-1))
    assert (np.abs(qs.astype(int)).max(-1) == 127).all()
    amax = np.abs(x.reshape(512, 160, 32)).max(-1)
    assert np.array_equal(d, (amax / np.float32(127)).astype(np.float16).astype(np.float32))


def test_empty_and_errors(capi, dev):
    import torch

    lib = capi.load()
    assert lib.llam_ql_quantize_q8_1(None, None, 0, 5120, 0, None)
    x = torch.zeros(64, device=dev)
    out = torch.zeros(72, dtype=torch.uint8, device=dev)
    assert not lib.llam_ql_quantize_q8_1(x.data_ptr() + 4, out.data_ptr(), 1, 32, 0, None)
    assert "16-byte aligned" in capi.last_error()
    assert not lib.llam_ql_quantize_q8_1(x.data_ptr(), out.data_ptr(), 1, 64, 99, None)
    assert "device_id" in capi.last_error()
