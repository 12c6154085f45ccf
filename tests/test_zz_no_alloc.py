"""llam_ql_gemv_f32_static: the fp32-input GEMV with the library's built-in Q8_1 scratch.

It must give the bits of llam_ql_gemv_f32 called with a caller-owned scratch buffer, on
calls in a row that share the built-in buffer (the second smaller than the first, so stale
blocks of the first stay behind it), allocate nothing and refuse what exceeds the buffer.
Collected last on purpose: a failure here must not hide the tests of the reference path.
"""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import TOL, rel_err, sync, upload_weights

pytestmark = pytest.mark.gpu

# (format, N, K, M): every pair runs big then small on the same GPU.  IQ3_S always takes the
# scratch; Q4_K / Q6_K take it for M*K > 6144 (quantiser launch + Q8_1 kernels) and for K < 4096.
PAIRS = [
    ((FMT_IQ3_S, 512, 2048, 4), (FMT_IQ3_S, 200, 1024, 1)),
    ((FMT_Q4_K, 1024, 5120, 4), (FMT_Q4_K, 300, 4096, 2)),
    ((FMT_Q6_K, 640, 8192, 8), (FMT_Q6_K, 96, 2048, 3)),
    ((FMT_Q4_K, 256, 32768, 8), (FMT_Q4_K, 64, 512, 1)),  # first call fills the whole buffer
]


def _run_both(capi, dev, oracle, fmt, N, K, M, seed):
    import torch

    W = synth.weights_numpy(fmt, N, K, seed)
    x = synth.activations_numpy(M, K, seed + 1)
    wd = upload_weights(capi, dev, fmt, W)
    xd = torch.from_numpy(x).to(dev)
    scratch = torch.empty(M * (K // 32) * 36, dtype=torch.uint8, device=dev)
    y_ref = torch.full((M, N), float("nan"), device=dev)
    y = torch.full((M, N), float("nan"), device=dev)
    capi.gemv_f32(fmt, wd, xd, M, N, K, out=y_ref, q8_scratch=scratch)
    sync()
    capi.gemv_f32_static(fmt, wd, xd, M, N, K, out=y)
    sync()
    # (a kernel's first launch in a process makes the runtime load its code: measured on a repeat)
    y2 = torch.full((M, N), float("nan"), device=dev)
    free0 = torch.cuda.mem_get_info()[0]
    capi.gemv_f32_static(fmt, wd, xd, M, N, K, out=y2)
    sync()
    assert torch.cuda.mem_get_info()[0] == free0, "the call changed the amount of free device memory"
    assert torch.equal(y, y2)
    a, b = y.cpu().numpy(), y_ref.cpu().numpy()
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32)), f"fmt {fmt} N={N} K={K} M={M}: bits differ"
    C = oracle.gemm(fmt, W, K, oracle.quantize(x))
    assert rel_err(a, C) <= TOL[fmt] * 1e-2
    return a


@pytest.mark.parametrize("big,small", PAIRS, ids=[f"fmt{b[0]}_K{b[2]}_then_K{s[2]}" for b, s in PAIRS])
def test_two_calls_in_a_row_share_the_buffer(capi, dev, oracle, big, small):
    print(f"[no_alloc] big {big} small {small}", flush=True)
    _run_both(capi, dev, oracle, *big, seed=11)
    first = _run_both(capi, dev, oracle, *small, seed=23)
    # and once more: same input, same bits (the buffer's leftovers do not leak in)
    again = _run_both(capi, dev, oracle, *small, seed=23)
    assert np.array_equal(first.view(np.uint32), again.view(np.uint32))


def test_strided_rows_and_padded_output(capi, dev, oracle):
    """ldx > K takes the row-by-row quantiser calls into the built-in buffer."""
    import torch

    fmt, N, K, M = FMT_IQ3_S, 128, 1024, 3
    W = synth.weights_numpy(fmt, N, K, 5)
    x = synth.activations_numpy(M, K, 6)
    wd = upload_weights(capi, dev, fmt, W)
    xd = torch.zeros(M, K + 64, device=dev)
    xd[:, :K] = torch.from_numpy(x).to(dev)
    out = torch.zeros(M, N + 8, device=dev)
    capi.gemv_f32_static(fmt, wd, xd[:, :K], M, N, K, out=out[:, :N])
    sync()
    C = oracle.gemm(fmt, W, K, oracle.quantize(x))
    assert rel_err(out[:, :N].cpu().numpy(), C) <= TOL[fmt] * 1e-2
    assert float(out[:, N:].abs().max()) == 0.0


def test_oversize_is_refused_with_a_message(capi, dev):
    import torch

    K = 32768 + 256  # 8 rows of it are one super-block per row beyond the buffer
    w = torch.zeros(capi.prepared_bytes(FMT_Q4_K, 1, K), dtype=torch.uint8, device=dev)
    x = torch.zeros(8, K, device=dev)
    out = torch.zeros(8, 1, device=dev)
    with pytest.raises(capi.QLError) as e:
        capi.gemv_f32_static(FMT_Q4_K, w, x, 8, 1, K, out=out)
    assert "built-in buffer" in str(e.value)
    capi.gemv_f32_static(FMT_Q4_K, w, x[:7], 7, 1, K, out=out[:7])  # 7 rows fit
    sync()
    assert float(out.abs().max()) == 0.0
