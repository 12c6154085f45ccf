"""Shared plumbing of the GPU parity tests: upload, prepare, compare."""
import numpy as np

from llaminar_amd import synth
from oracle.binding import BLOCK_BYTES, FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K

FMTS = {"q4_k": FMT_Q4_K, "q6_k": FMT_Q6_K, "iq3_s": FMT_IQ3_S}
# fp32 output contract: max |y - ref| / max |ref|
TOL = {FMT_Q4_K: 1e-3, FMT_Q6_K: 1e-3, FMT_IQ3_S: 1e-2}


def upload_weights(capi, dev, fmt, W):
    """raw GGUF bytes (numpy) -> prepared device tensor"""
    import torch

    N, SB, _ = W.shape
    raw = torch.from_numpy(np.ascontiguousarray(W).reshape(-1)).to(dev)
    return capi.prepare_weights(fmt, raw, N, SB * 256)


def upload_q8(dev, q8):
    import torch

    return torch.from_numpy(np.ascontiguousarray(q8).reshape(-1)).to(dev)


def rel_err(y, ref):
    denom = float(np.abs(ref).max())
    if denom == 0.0:
        return float(np.abs(y).max())
    return float(np.abs(y.astype(np.float64) - ref.astype(np.float64)).max() / denom)


def sync():
    import torch

    torch.cuda.synchronize()
