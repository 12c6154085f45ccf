"""TEST INFRASTRUCTURE ONLY: ctypes doors onto the checkers.

``Oracle``  -> oracle/libql_oracle.so        (scalar C restatement, ql_oracle.c)
``Ref``     -> oracle/_ref/libllaminar_ref.so (the reference's own CPU kernels,
                                               present only where it was built)

Only tests, the smoke check and the benchmark's cpu_baseline leg import this.
"""
from __future__ import annotations

import ctypes
import os
import subprocess
from ctypes import POINTER, c_float, c_int, c_int32, c_long, c_uint8, c_uint16, c_void_p
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
ORACLE_LIB = HERE / "libql_oracle.so"
REF_LIB = HERE / "_ref" / "libllaminar_ref.so"

FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S = 5, 8, 11
BLOCK_BYTES = {FMT_Q4_K: 144, FMT_Q6_K: 210, FMT_IQ3_S: 110}


def build(reference: str = "/root/reference") -> None:
    """Compile the restatement (always) and the reference shim (when the tree is there)."""
    subprocess.run(["make", "-C", str(HERE), f"REFERENCE={reference}", "all"], check=True,
                   stdout=subprocess.DEVNULL)


def _p(a: np.ndarray):
    return a.ctypes.data_as(c_void_p)


class Oracle:
    def __init__(self):
        if not ORACLE_LIB.exists():
            build()
        L = ctypes.CDLL(str(ORACLE_LIB))
        L.qlo_f16_to_f32.restype = c_float
        L.qlo_f16_to_f32.argtypes = [c_uint16]
        L.qlo_f32_to_f16_sw.restype = c_uint16
        L.qlo_f32_to_f16_sw.argtypes = [c_float]
        L.qlo_f32_to_f16_rne.restype = c_uint16
        L.qlo_f32_to_f16_rne.argtypes = [c_float]
        L.qlo_quantize_block_q8_1.argtypes = [c_void_p, c_int, c_void_p]
        L.qlo_quantize_q8_1.argtypes = [c_void_p, c_int, c_int, c_void_p]
        L.qlo_get_scale_min_k4.argtypes = [c_int, c_void_p, c_void_p, c_void_p]
        L.qlo_subblocks.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_void_p]
        L.qlo_gemm_rows.argtypes = [c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p, c_int,
                                    c_void_p, c_int]
        L.qlo_epilogue.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_void_p]
        L.qlo_moe_route.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
        L.qlo_swiglu.argtypes = [c_void_p, c_void_p, c_int, c_void_p]
        L.qlo_check_div127.restype = ctypes.c_long
        L.qlo_check_div127_all_significands.restype = ctypes.c_long
        L.qlo_stream_triad.restype = ctypes.c_double
        L.qlo_stream_triad.argtypes = [c_void_p, c_void_p, c_void_p, ctypes.c_long, c_int]
        L.qlo_check_q6k_factor.restype = ctypes.c_long
        L.qlo_check_q6k_factor.argtypes = [c_int]
        L.qlo_dequant_row_q4k.argtypes = [c_void_p, c_int, c_void_p]
        L.qlo_rmsnorm.argtypes = [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int, c_int]
        L.qlo_rope_inv_freq.argtypes = [c_int, c_float, c_void_p]
        L.qlo_rope_head.argtypes = [c_void_p, c_int, c_void_p, c_int]
        L.qlo_rope_kv_append.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int]
        L.qlo_attention_decode.argtypes = [c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int]
        L.qlo_argmax.restype = c_int
        L.qlo_argmax.argtypes = [c_void_p, c_int]
        self.L = L

    # -- fp16 ---------------------------------------------------------------
    def f16_to_f32(self, h: int) -> float:
        return float(self.L.qlo_f16_to_f32(h))

    def f32_to_f16_sw(self, f: float) -> int:
        return int(self.L.qlo_f32_to_f16_sw(np.float32(f)))

    def f32_to_f16_rne(self, f: float) -> int:
        return int(self.L.qlo_f32_to_f16_rne(np.float32(f)))

    # -- Q8_1 ---------------------------------------------------------------
    def quantize_block(self, x: np.ndarray, valid: int = 32) -> np.ndarray:
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.zeros(36, dtype=np.uint8)
        self.L.qlo_quantize_block_q8_1(_p(x), valid, _p(out))
        return out

    def quantize(self, x: np.ndarray) -> np.ndarray:
        """fp32 [M,K] -> uint8 [M, ceil(K/32), 36]"""
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None]
        M, K = x.shape
        out = np.zeros((M, (K + 31) // 32, 36), dtype=np.uint8)
        self.L.qlo_quantize_q8_1(_p(x), M, K, _p(out))
        return out

    # -- weights --------------------------------------------------------------
    def scale_min_k4(self, j: int, scales12: np.ndarray):
        sc = np.zeros(1, np.uint8)
        m = np.zeros(1, np.uint8)
        s = np.ascontiguousarray(scales12, dtype=np.uint8)
        self.L.qlo_get_scale_min_k4(j, _p(s), _p(sc), _p(m))
        return int(sc[0]), int(m[0])

    def subblocks(self, fmt: int, sb: np.ndarray):
        """one super-block's bytes -> (int8[256], fp16-bits scales[8], fp16-bits mins[8])"""
        sb = np.ascontiguousarray(sb, dtype=np.uint8)
        assert sb.size == BLOCK_BYTES[fmt]
        w = np.zeros(256, np.int8)
        sc = np.zeros(8, np.uint16)
        mn = np.zeros(8, np.uint16)
        self.L.qlo_subblocks(fmt, _p(sb), _p(w), _p(sc), _p(mn))
        return w, sc, mn

    # -- GEMV / GEMM ------------------------------------------------------------
    def gemm(self, fmt: int, W: np.ndarray, K: int, q8: np.ndarray, n0: int = 0, n1: int | None = None,
             want_sums: bool = False, k_tiles: int = 0):
        """W: uint8 raw GGUF rows; q8: uint8 [M, K/32, 36].  Returns C[M, n1-n0] (and sums[M, n1-n0, K/32])."""
        W = np.ascontiguousarray(W, dtype=np.uint8).reshape(-1)
        row_bytes = (K // 256) * BLOCK_BYTES[fmt]
        N = W.size // row_bytes
        if n1 is None:
            n1 = N
        q8 = np.ascontiguousarray(q8, dtype=np.uint8)
        M = q8.shape[0]
        C = np.zeros((M, N), np.float32)
        sums = np.zeros((M, n1 - n0, K // 32), np.int32) if want_sums else None
        self.L.qlo_gemm_rows(fmt, _p(W), K, n0, n1, _p(q8), M, _p(C), N, _p(sums) if want_sums else None, k_tiles)
        C = C[:, n0:n1].copy()
        return (C, sums) if want_sums else C

    def epilogue(self, C: np.ndarray, T: np.ndarray, alpha: float, beta: float, bias=None) -> np.ndarray:
        C = np.ascontiguousarray(C, dtype=np.float32).copy()
        T = np.ascontiguousarray(T, dtype=np.float32)
        M, N = T.shape
        b = np.ascontiguousarray(bias, dtype=np.float32) if bias is not None else None
        self.L.qlo_epilogue(_p(C), _p(T), M, N, N, alpha, beta, _p(b) if b is not None else None)
        return C

    # -- MoE ----------------------------------------------------------------------
    def route(self, logits: np.ndarray, top_k: int, normalize: bool = True):
        logits = np.ascontiguousarray(logits, dtype=np.float32)
        T, E = logits.shape
        ids = np.zeros((T, top_k), np.int32)
        w = np.zeros((T, top_k), np.float32)
        probs = np.zeros((T, E), np.float32)
        self.L.qlo_moe_route(_p(logits), T, E, top_k, int(normalize), _p(ids), _p(w), _p(probs))
        return ids, w, probs

    def stream_triad_gbs(self, mib_per_array: int = 256, reps: int = 5) -> float:
        """Host DRAM bandwidth (STREAM triad, every OpenMP thread), GB/s."""
        n = mib_per_array * (1 << 20) // 8
        a, b, c = np.zeros(n), np.ones(n), np.full(n, 2.0)
        return float(self.L.qlo_stream_triad(_p(a), _p(b), _p(c), n, reps)) / 1e9

    def check_div127(self) -> int:
        return int(self.L.qlo_check_div127())

    def check_div127_all_significands(self) -> int:
        return int(self.L.qlo_check_div127_all_significands())

    def check_q6k_factor(self, ulps: int) -> int:
        return int(self.L.qlo_check_q6k_factor(ulps))

    def swiglu(self, gate: np.ndarray, up: np.ndarray) -> np.ndarray:
        gate = np.ascontiguousarray(gate, dtype=np.float32)
        up = np.ascontiguousarray(up, dtype=np.float32)
        out = np.zeros_like(gate)
        self.L.qlo_swiglu(_p(gate), _p(up), gate.size, _p(out))
        return out

    # -- decode-step operators ------------------------------------------------------
    def dequant_rows_q4k(self, blocks: np.ndarray) -> np.ndarray:
        """blocks: uint8 [..., nsb, 144] -> float32 [..., nsb*256]."""
        blocks = np.ascontiguousarray(blocks, dtype=np.uint8)
        n = blocks.size // 144
        out = np.zeros(n * 256, np.float32)
        self.L.qlo_dequant_row_q4k(_p(blocks), n, _p(out))
        return out.reshape(blocks.shape[:-2] + (blocks.shape[-2] * 256,))

    def rmsnorm(self, x: np.ndarray, gamma: np.ndarray, eps: float, delta=None):
        """Returns (y, x_after): x_after = x + delta when delta is given."""
        x = np.ascontiguousarray(x, dtype=np.float32).copy()
        rows, cols = x.shape
        g = np.ascontiguousarray(gamma, dtype=np.float32)
        d = np.ascontiguousarray(delta, dtype=np.float32) if delta is not None else None
        y = np.zeros_like(x)
        self.L.qlo_rmsnorm(_p(x), _p(d) if d is not None else None, _p(g), eps, _p(y), rows, cols)
        return y, x

    def rope_inv_freq(self, head_dim: int, theta: float) -> np.ndarray:
        out = np.zeros(head_dim // 2, np.float32)
        self.L.qlo_rope_inv_freq(head_dim, theta, _p(out))
        return out

    def rope_head(self, head: np.ndarray, position: int, inv_freq: np.ndarray) -> np.ndarray:
        h = np.ascontiguousarray(head, dtype=np.float32).copy()
        self.L.qlo_rope_head(_p(h), position, _p(inv_freq), h.size)
        return h

    def rope_kv_append(self, qkv: np.ndarray, inv_freq, position: int, kcache: np.ndarray, vcache: np.ndarray,
                       n_heads: int, n_kv: int, head_dim: int) -> np.ndarray:
        """qkv: [(n_heads+2 n_kv)*head_dim]; caches uint16 [n_kv, ctx_cap, head_dim], updated in place."""
        q = np.ascontiguousarray(qkv, dtype=np.float32).copy()
        assert kcache.dtype == np.uint16 and kcache.flags.c_contiguous and vcache.flags.c_contiguous
        self.L.qlo_rope_kv_append(_p(q), _p(inv_freq), position, _p(kcache), _p(vcache), n_heads, n_kv, head_dim,
                                  kcache.shape[1])
        return q

    def attention_decode(self, q: np.ndarray, kcache: np.ndarray, vcache: np.ndarray, last: int, n_heads: int,
                         n_kv: int, head_dim: int) -> np.ndarray:
        q = np.ascontiguousarray(q, dtype=np.float32)
        out = np.zeros(n_heads * head_dim, np.float32)
        self.L.qlo_attention_decode(_p(q), _p(kcache), _p(vcache), last, _p(out), n_heads, n_kv, head_dim,
                                    kcache.shape[1])
        return out

    def argmax(self, x: np.ndarray) -> int:
        x = np.ascontiguousarray(x, dtype=np.float32)
        return int(self.L.qlo_argmax(_p(x), x.size))


class Ref:
    """The reference's own code.  `available()` is False where it was not built
    (for instance on a machine that never saw the reference tree)."""

    @staticmethod
    def available() -> bool:
        return REF_LIB.exists()

    def __init__(self):
        L = ctypes.CDLL(str(REF_LIB), mode=os.RTLD_LAZY)
        L.ref_f16_to_f32.restype = c_float
        L.ref_f16_to_f32.argtypes = [c_uint16]
        L.ref_f32_to_f16.restype = c_uint16
        L.ref_f32_to_f16.argtypes = [c_float]
        L.ref_f32_to_f16_f16c.restype = c_uint16
        L.ref_f32_to_f16_f16c.argtypes = [c_float]
        L.ref_iq3s_grid.restype = POINTER(ctypes.c_uint32)
        L.ref_get_scale_min_k4.argtypes = [c_int, c_void_p, c_void_p, c_void_p]
        L.ref_quantize_block_q8_1.argtypes = [c_void_p, c_int, c_void_p, c_int]
        L.ref_quantize_q8_1.argtypes = [c_void_p, c_int, c_int, c_void_p]
        L.ref_unpack_superblock.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int]
        L.ref_pack.restype = c_void_p
        L.ref_pack.argtypes = [c_int, c_void_p, c_int, c_int]
        L.ref_pack_free.argtypes = [c_void_p]
        L.ref_pack_bytes.restype = c_long
        L.ref_pack_bytes.argtypes = [c_void_p]
        L.ref_gemm_packed.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int, c_int]
        L.ref_gemm_fp32_packed.argtypes = [c_void_p, c_void_p, c_int, c_void_p, c_int]
        L.ref_gemm.restype = c_int
        L.ref_gemm.argtypes = [c_int, c_void_p, c_int, c_int, c_void_p, c_int, c_void_p, c_int, c_int]
        L.ref_omp_threads.restype = c_int
        self.has_decode = hasattr(L, "ref_rmsnorm_row")
        if self.has_decode:
            L.ref_rmsnorm_row.argtypes = [c_int, c_void_p, c_void_p, c_void_p, c_long, c_float]
            L.ref_residual_rmsnorm_row.argtypes = [c_void_p, c_void_p, c_void_p, c_void_p, c_long, c_float]
            L.ref_rope_inv_freq.argtypes = [c_int, c_float, c_void_p]
            L.ref_rope_token.argtypes = [c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_float]
            L.ref_rope_head_scalar.argtypes = [c_void_p, c_int, c_int, c_float]
        self.has_swiglu = hasattr(L, "ref_swiglu")
        if self.has_swiglu:
            L.ref_swiglu.argtypes = [c_void_p, c_void_p, c_void_p, c_int]
        self.has_route = hasattr(L, "ref_moe_route")
        if self.has_route:
            L.ref_softmax_row.argtypes = [c_void_p, c_int, c_int]
            L.ref_moe_route.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p]
        self.L = L

    def softmax_row(self, row, variant=0):
        """primitives::softmax_row_fp32 on one row; variant 0 dispatch, 1 scalar, 2 AVX2, 3 AVX512."""
        r = np.ascontiguousarray(row, dtype=np.float32).copy()
        self.L.ref_softmax_row(_p(r), r.size, variant)
        return r

    def moe_route(self, logits, top_k, normalize=True, variant=0):
        """CPUMoEKernel::route from the logits on: (ids, weights, probabilities)."""
        lg = np.ascontiguousarray(logits, dtype=np.float32)
        T, E = lg.shape
        ids = np.zeros((T, top_k), np.int32)
        w = np.zeros((T, top_k), np.float32)
        probs = np.zeros((T, E), np.float32)
        self.L.ref_moe_route(_p(lg), T, E, top_k, int(normalize), variant, _p(ids), _p(w), _p(probs))
        return ids, w, probs

    def f16_to_f32(self, h):
        return float(self.L.ref_f16_to_f32(h))

    def f32_to_f16(self, f):
        return int(self.L.ref_f32_to_f16(np.float32(f)))

    def f32_to_f16_f16c(self, f):
        return int(self.L.ref_f32_to_f16_f16c(np.float32(f)))

    def iq3s_grid(self) -> np.ndarray:
        return np.ctypeslib.as_array(self.L.ref_iq3s_grid(), shape=(512,)).copy()

    def scale_min_k4(self, j, scales12):
        sc = np.zeros(1, np.uint8)
        m = np.zeros(1, np.uint8)
        s = np.ascontiguousarray(scales12, dtype=np.uint8)
        self.L.ref_get_scale_min_k4(j, _p(s), _p(sc), _p(m))
        return int(sc[0]), int(m[0])

    def quantize_block(self, x, valid=32, variant=0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.zeros(36, np.uint8)
        self.L.ref_quantize_block_q8_1(_p(x), valid, _p(out), variant)
        return out

    def quantize(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        if x.ndim == 1:
            x = x[None]
        M, K = x.shape
        out = np.zeros((M, (K + 31) // 32, 36), np.uint8)
        self.L.ref_quantize_q8_1(_p(x), M, K, _p(out))
        return out

    def unpack_superblock(self, fmt, sb, variant=0):
        sb = np.ascontiguousarray(sb, dtype=np.uint8)
        w = np.zeros(256, np.int8)
        sc = np.zeros(8, np.float32)
        mn = np.zeros(8, np.float32)
        self.L.ref_unpack_superblock(fmt, _p(sb), _p(w), _p(sc), _p(mn), variant)
        return w, sc, mn

    def gemm(self, fmt, W, N, K, q8, isa=0):
        W = np.ascontiguousarray(W, dtype=np.uint8).reshape(-1)
        q8 = np.ascontiguousarray(q8, dtype=np.uint8)
        M = q8.shape[0]
        C = np.zeros((M, N), np.float32)
        ok = self.L.ref_gemm(fmt, _p(W), N, K, _p(q8), M, _p(C), N, isa)
        assert ok
        return C

    def pack(self, fmt, W, N, K):
        W = np.ascontiguousarray(W, dtype=np.uint8).reshape(-1)
        h = self.L.ref_pack(fmt, _p(W), N, K)
        assert h
        return h

    def pack_free(self, h):
        self.L.ref_pack_free(h)

    def pack_bytes(self, h) -> int:
        return int(self.L.ref_pack_bytes(h))

    def gemm_packed(self, h, q8, N, isa=0, out=None):
        q8 = np.ascontiguousarray(q8, dtype=np.uint8)
        M = q8.shape[0]
        C = out if out is not None else np.zeros((M, N), np.float32)
        self.L.ref_gemm_packed(h, _p(q8), M, _p(C), N, isa)
        return C

    def omp_threads(self) -> int:
        return int(self.L.ref_omp_threads())

    # -- decode-step primitives --------------------------------------------------------
    def rmsnorm_row(self, x, gamma, eps, variant=3):
        x = np.ascontiguousarray(x, dtype=np.float32)
        g = np.ascontiguousarray(gamma, dtype=np.float32)
        y = np.zeros_like(x)
        self.L.ref_rmsnorm_row(variant, _p(x), _p(g), _p(y), x.size, eps)
        return y

    def residual_rmsnorm_row(self, delta, residual, gamma, eps):
        d = np.ascontiguousarray(delta, dtype=np.float32)
        r = np.ascontiguousarray(residual, dtype=np.float32).copy()
        g = np.ascontiguousarray(gamma, dtype=np.float32)
        y = np.zeros_like(r)
        self.L.ref_residual_rmsnorm_row(_p(d), _p(r), _p(g), _p(y), r.size, eps)
        return y, r

    def swiglu(self, gate, up):
        g = np.ascontiguousarray(gate, dtype=np.float32)
        u = np.ascontiguousarray(up, dtype=np.float32)
        out = np.zeros_like(g)
        self.L.ref_swiglu(_p(g), _p(u), _p(out), g.size)
        return out

    def rope_inv_freq(self, head_dim, theta):
        out = np.zeros(head_dim // 2, np.float32)
        self.L.ref_rope_inv_freq(head_dim, theta, _p(out))
        return out

    def rope_token(self, q, k, head_dim, n_past, theta):
        q = np.ascontiguousarray(q, dtype=np.float32).copy()
        k = np.ascontiguousarray(k, dtype=np.float32).copy()
        self.L.ref_rope_token(_p(q), _p(k), head_dim, q.size // head_dim, k.size // head_dim, n_past, theta)
        return q, k

    def rope_head_scalar(self, head, position, theta):
        h = np.ascontiguousarray(head, dtype=np.float32).copy()
        self.L.ref_rope_head_scalar(_p(h), position, h.size, theta)
        return h
