"""Seeded synthetic GGUF weight blocks and activations.

Block fields are uniform over their whole range: every packed byte uniform
0..255 (which makes Q4_K's 6-bit scales/mins uniform 0..63, its nibbles uniform
0..15, Q6_K's int8 sub-scales uniform -128..127 and IQ3_S's 9-bit codebook
indices uniform 0..511 with random signs and 4-bit sub-scales), and the fp16
super-block scales d (and dmin) uniform in [0.001, 0.02).  Activations and
router logits are N(0,1).
"""
from __future__ import annotations

import numpy as np

from .capi import BLOCK_BYTES, FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K

# byte offsets of the fp16 scale fields inside one super-block
_FP16_FIELDS = {FMT_Q4_K: (0, 2), FMT_Q6_K: (208,), FMT_IQ3_S: (0,)}


def weights_numpy(fmt: int, N: int, K: int, seed: int, d_lo: float = 0.001, d_hi: float = 0.02) -> np.ndarray:
    """uint8 array [N, K/256, block_bytes] of raw GGUF super-blocks."""
    assert K % 256 == 0
    rng = np.random.default_rng(seed)
    bb = BLOCK_BYTES[fmt]
    sb = K // 256
    w = rng.integers(0, 256, size=(N, sb, bb), dtype=np.uint8)
    for off in _FP16_FIELDS[fmt]:
        d = rng.uniform(d_lo, d_hi, size=(N, sb)).astype(np.float16)
        w[:, :, off:off + 2] = d.view(np.uint8).reshape(N, sb, 2)
    return w


def weights_torch(fmt: int, N: int, K: int, seed: int, device, d_lo: float = 0.001, d_hi: float = 0.02):
    """Same distribution generated directly on `device` (for matrices too big to
    build on the host every run).  uint8 tensor of N*(K/256)*block_bytes bytes."""
    import torch

    g = torch.Generator(device=device)
    g.manual_seed(seed)
    bb = BLOCK_BYTES[fmt]
    sb = K // 256
    w = torch.randint(0, 256, (N * sb, bb), dtype=torch.uint8, device=device, generator=g)
    for off in _FP16_FIELDS[fmt]:
        d = (torch.rand(N * sb, device=device, generator=g) * (d_hi - d_lo) + d_lo).to(torch.float16)
        w[:, off:off + 2] = d.view(torch.uint8).reshape(N * sb, 2)
    return w.reshape(-1)


def activations_numpy(M: int, K: int, seed: int) -> np.ndarray:
    rng = np.random.default_rng(seed)
    return rng.standard_normal((M, K)).astype(np.float32)


def gemv_bytes(fmt: int, N: int, K: int, M: int = 1) -> int:
    """Algorithmic bytes of one GEMV: weights + Q8_1 activations + fp32 outputs."""
    return N * (K // 256) * BLOCK_BYTES[fmt] + M * (K // 32) * 36 + M * N * 4
