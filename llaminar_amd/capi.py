"""ctypes binding of the C-ABI in ``include/llaminar_amd/ql_api.h``.

Python here is plumbing only: PyTorch supplies device memory and streams, every
computation happens in the HIP library.  There is no fallback: if the shared
object is missing or fails to load, importing the binding raises.
"""
from __future__ import annotations

import ctypes
import os
from ctypes import POINTER, c_bool, c_char_p, c_float, c_int, c_int32, c_size_t, c_uint8, c_void_p
from pathlib import Path

FMT_Q4_K = 5
FMT_Q6_K = 8
FMT_IQ3_S = 11
FORMATS = {"q4_k": FMT_Q4_K, "q6_k": FMT_Q6_K, "iq3_s": FMT_IQ3_S}
BLOCK_BYTES = {FMT_Q4_K: 144, FMT_Q6_K: 210, FMT_IQ3_S: 110}
MAX_GEMV_M = 8
MAX_FUSED = 16

LIB_PATH = Path(__file__).resolve().parent / "lib" / "libllaminar_ql.so"


class QLError(RuntimeError):
    """A C-ABI call returned false; the message is llam_ql_last_error()."""


class Proj(ctypes.Structure):
    _fields_ = [("d_w", c_void_p), ("d_y", c_void_p), ("N", c_int), ("ldy", c_int), ("fmt", c_uint8),
                ("d_plane", c_void_p)]


class GemvPlan(ctypes.Structure):
    _fields_ = [("kernel", c_int), ("m_first", c_int), ("slice_sb", c_int), ("rows_per_wave", c_int),
                ("decode_equivalent", c_int)]


KERNEL_GENERIC, KERNEL_CHUNKED, KERNEL_QUAD, KERNEL_MFMA = 0, 1, 2, 3


class Expert(ctypes.Structure):
    _fields_ = [("d_gate", c_void_p), ("d_up", c_void_p), ("d_down", c_void_p)]


# name -> (restype, argtypes); mirrors ql_api.h declaration by declaration
SIGNATURES = {
    "llam_ql_last_error": (c_char_p, []),
    "llam_ql_abi_version": (c_int, []),
    "llam_ql_set_gemv_tuning": (None, [c_int, c_int]),
    "llam_ql_reset_gemv_tuning": (None, []),
    "llam_ql_batch_plane_bytes": (c_size_t, [c_uint8, c_int, c_int]),
    "llam_ql_build_batch_plane": (c_bool, [c_uint8, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_quantize_q8_1": (c_bool, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_prepared_bytes": (c_size_t, [c_uint8, c_int, c_int]),
    "llam_ql_prepare_weights": (c_bool, [c_uint8, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemv": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemv_plane": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                    c_void_p]),
    "llam_ql_gemv_fused": (c_bool, [POINTER(Proj), c_int, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemv_f32": (c_bool, [c_uint8, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p,
                                  c_int, c_void_p]),
    "llam_ql_gemv_f32_static": (c_bool, [c_uint8, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_int,
                                         c_int, c_void_p]),
    "llam_ql_gemv_accumulate_supported": (c_bool, [c_uint8, c_int, c_int, c_int, c_int]),
    "llam_ql_gemv_accumulate": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemv_fused_rmsnorm_supported": (c_bool, [POINTER(Proj), c_int, c_int, c_int]),
    "llam_ql_gemv_fused_rmsnorm": (c_bool, [POINTER(Proj), c_int, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_int,
                                            c_int, c_int, c_void_p]),
    "llam_ql_gemv_fused_f32": (c_bool, [POINTER(Proj), c_int, c_void_p, c_int, c_int, c_int, c_void_p, c_int,
                                        c_void_p]),
    "llam_ql_gemv_swiglu_f32": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_int, c_int,
                                         c_int, c_int, c_void_p, c_int, c_void_p]),
    "llam_ql_gemv_block_sums": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                         c_int, c_int, c_void_p]),
    "llam_ql_gemv_describe": (c_bool, [c_uint8, c_int, c_int, c_int, c_int, c_int, POINTER(GemvPlan)]),
    "llam_ql_gemm": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemm_block_sums": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                         c_int, c_void_p]),
    "llam_ql_epilogue": (c_bool, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_float, c_float, c_int,
                                  c_void_p]),
    "llam_ql_moe_router_logits": (c_bool, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_route_ex": (c_bool, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "llam_ql_moe_route": (c_bool, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p]),
    "llam_ql_moe_route_quantize": (c_bool, [c_void_p, c_int, c_int, c_int, c_int, c_void_p, c_void_p, c_int, c_void_p,
                                            c_int, c_void_p, c_int, c_void_p]),
    "llam_ql_moe_gate_up": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                     c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_gate_up_swiglu": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                            c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_route_gate_up_swiglu": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_int, c_int, c_int, c_void_p,
                                                  c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                                  c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_gemv_plane_split_supported": (c_bool, [c_uint8, c_int, c_int, c_int]),
    "llam_ql_gemv_plane_split": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int,
                                          c_void_p]),
    "llam_ql_gemv_gate_up_swiglu_supported": (c_bool, [c_uint8, c_int, c_int, c_int]),
    "llam_ql_gemv_gate_up_swiglu": (c_bool, [c_uint8, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                             c_int, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_swiglu_quantize": (c_bool, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_down": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int,
                                  c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_group_bytes": (c_size_t, [c_int, c_int]),
    "llam_ql_moe_group": (c_bool, [c_void_p, c_int, c_int, c_int, c_void_p, c_int, c_void_p]),
    "llam_ql_moe_gate_up_grouped": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                             c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_down_grouped": (c_bool, [c_uint8, c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p,
                                          c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_ids_from_f32": (c_bool, [c_void_p, c_void_p, c_int, c_int, c_void_p]),
    "llam_ql_moe_publish_routing": (c_bool, [c_void_p, c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p,
                                             c_int, c_int, c_void_p]),
    "llam_ql_shared_expert_add": (c_bool, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_shared_expert_gate": (c_bool, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_gather_rows": (c_bool, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_ql_moe_scatter_add_weighted": (c_bool, [c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_int,
                                                  c_void_p]),
    "llam_ql_swiglu_inplace": (c_bool, [c_void_p, c_void_p, ctypes.c_long, c_int, c_void_p]),
    # decode_api.h
    "llam_dec_embed_q4k": (c_bool, [c_void_p, c_int, c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_dec_rmsnorm_q8_1": (c_bool, [c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int, c_int,
                                       c_void_p]),
    "llam_dec_rmsnorm2_q8_1": (c_bool, [c_void_p, c_void_p, c_void_p, c_void_p, c_float, c_void_p, c_void_p, c_int, c_int,
                                        c_int, c_void_p]),
    "llam_dec_rope_inv_freq": (None, [c_int, c_float, c_void_p]),
    "llam_dec_rope_kv_append": (c_bool, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_int, c_int,
                                         c_int, c_int, c_int, c_void_p]),
    "llam_dec_attention_scratch_floats": (c_size_t, [c_int, c_int, c_int, c_int]),
    "llam_dec_attention": (c_bool, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_int, c_void_p, c_void_p,
                                    c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_dec_rope_table": (c_bool, [c_void_p, c_void_p, c_void_p, c_int, c_int, c_int, c_void_p]),
    "llam_dec_rope_attention": (c_bool, [c_void_p, c_int, c_void_p, c_void_p, c_void_p, c_void_p, c_void_p, c_int,
                                         c_void_p, c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p]),
    "llam_dec_argmax_scratch_bytes": (c_size_t, [c_int, c_int]),
    "llam_dec_argmax": (c_bool, [c_void_p, c_int, c_int, c_int, c_void_p, c_void_p, c_void_p, c_int, c_void_p]),
}

_lib = None


def load() -> ctypes.CDLL:
    """Load the HIP library (once).  Raises if it has not been built."""
    global _lib
    if _lib is not None:
        return _lib
    if not LIB_PATH.exists():
        raise ImportError(
            f"{LIB_PATH} is missing: build it with `python -m llaminar_amd.build` "
            "(hipcc --offload-arch=gfx950).  There is no CPU fallback.")
    # PyTorch ships its own copy of the HIP runtime under the same soname as the
    # system one.  A process must use exactly one of them: import torch first so the
    # dynamic loader binds this library to the runtime torch's allocator uses.
    import torch  # noqa: F401

    lib = ctypes.CDLL(str(LIB_PATH))
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)  # AttributeError if the library does not export it
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def last_error() -> str:
    return load().llam_ql_last_error().decode()


def _check(ok: bool, what: str) -> None:
    if not ok:
        raise QLError(f"{what}: {last_error()}")


def _ptr(t) -> int:
    """Device (or host) address of a torch tensor, or a raw int."""
    if t is None:
        return 0
    if isinstance(t, int):
        return t
    return t.data_ptr()


def _stream(stream=None) -> int:
    if stream is None:
        import torch

        return torch.cuda.current_stream().cuda_stream
    if isinstance(stream, int):
        return stream
    return stream.cuda_stream


def _dev(t) -> int:
    return t.device.index if t.device.index is not None else 0


# ---------------------------------------------------------------------------
# Thin call wrappers (tensor in, tensor out; all allocation is the caller's or
# torch's, never the library's)
# ---------------------------------------------------------------------------

def quantize_q8_1(x, out=None, stream=None):
    """fp32 [M,K] (or [K]) on the GPU -> uint8 tensor of M*ceil(K/32) 36-byte Q8_1 blocks."""
    import torch

    x2 = x.reshape(1, -1) if x.dim() == 1 else x
    M, K = x2.shape
    assert x2.dtype == torch.float32 and x2.is_contiguous() and x2.is_cuda
    if out is None:
        out = torch.empty(M * ((K + 31) // 32) * 36, dtype=torch.uint8, device=x.device)
    _check(load().llam_ql_quantize_q8_1(_ptr(x2), _ptr(out), M, K, _dev(x2), _stream(stream)), "quantize_q8_1")
    return out


def prepared_bytes(fmt: int, N: int, K: int) -> int:
    return int(load().llam_ql_prepared_bytes(fmt, N, K))


def prepare_weights(fmt: int, gguf, N: int, K: int, stream=None):
    """Raw GGUF super-block bytes (uint8 GPU tensor) -> device layout the kernels read."""
    import torch

    assert gguf.dtype == torch.uint8 and gguf.is_cuda and gguf.is_contiguous()
    assert gguf.numel() == N * (K // 256) * BLOCK_BYTES[fmt], "weight byte count does not match N,K,fmt"
    nbytes = prepared_bytes(fmt, N, K)
    out = torch.empty(nbytes, dtype=torch.uint8, device=gguf.device)
    _check(load().llam_ql_prepare_weights(fmt, _ptr(gguf), _ptr(out), N, K, _dev(gguf), _stream(stream)),
           "prepare_weights")
    return out


def batch_plane_bytes(fmt: int, N: int, K: int) -> int:
    """Size of the optional int8 batch plane of a prepared matrix; 0 where the shape has none."""
    return int(load().llam_ql_batch_plane_bytes(fmt, N, K))


def build_batch_plane(fmt: int, w, N: int, K: int, stream=None):
    """Builds the batch plane of the prepared matrix `w`: hand it to the launches of that matrix (`plane=`)
    and batches of 5..8 rows read weights laid out for the matrix unit.  Returns the plane, finished (the
    building stream is waited for, so a launch on any stream may read it), or None where the format or shape
    has no plane.  The caller keeps it alive as long as launches use it."""
    import torch

    nbytes = batch_plane_bytes(fmt, N, K)
    if nbytes == 0:
        return None
    plane = torch.empty(nbytes, dtype=torch.uint8, device=w.device)
    _check(load().llam_ql_build_batch_plane(fmt, _ptr(w), _ptr(plane), N, K, _dev(w), _stream(stream)), "build_batch_plane")
    (stream if stream is not None and not isinstance(stream, int) else torch.cuda.current_stream()).synchronize()
    return plane


def _proj(p):
    """(fmt, w, out[M,N]) or (fmt, w, out[M,N], plane) -> Proj."""
    fmt, w, out = p[0], p[1], p[2]
    plane = p[3] if len(p) > 3 else None
    return Proj(_ptr(w), _ptr(out), out.shape[-1], out.stride(0) if out.dim() == 2 else out.shape[-1], fmt, _ptr(plane))


def gemv(fmt: int, w, q8, M: int, N: int, K: int, out=None, stream=None, plane=None):
    """out[M,N] from Q8_1 activations; `plane`: the matrix's batch plane (build_batch_plane) or None."""
    import torch

    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=w.device)
    ldy = out.stride(0) if out.dim() == 2 else N
    if plane is None:
        _check(load().llam_ql_gemv(fmt, _ptr(w), _ptr(q8), _ptr(out), M, N, K, ldy, _dev(w), _stream(stream)), "gemv")
    else:
        _check(load().llam_ql_gemv_plane(fmt, _ptr(w), _ptr(plane), _ptr(q8), _ptr(out), M, N, K, ldy, _dev(w),
                                         _stream(stream)), "gemv_plane")
    return out


def gemv_fused(projs, q8, M: int, K: int, stream=None):
    """projs: list of (fmt, w, out[M,N]) or (fmt, w, out[M,N], plane) sharing one quantised input."""
    arr = _proj_array(projs)
    dev = _dev(q8)
    _check(load().llam_ql_gemv_fused(arr, len(projs), _ptr(q8), M, K, dev, _stream(stream)), "gemv_fused")


def _ld(t) -> int:
    return t.stride(0) if t.dim() == 2 else t.shape[-1]


def gemv_f32(fmt: int, w, x, M: int, N: int, K: int, out=None, q8_scratch=None, stream=None):
    """out[M,N] from fp32 activations x[M,K] (quantised inside the kernel)."""
    import torch

    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=w.device)
    _check(load().llam_ql_gemv_f32(fmt, _ptr(w), _ptr(x), _ld(x), _ptr(out), M, N, K, _ld(out), _ptr(q8_scratch),
                                   _dev(w), _stream(stream)), "gemv_f32")
    return out


STATIC_SCRATCH_BYTES = 8 * (32768 // 32) * 36


def gemv_f32_static(fmt: int, w, x, M: int, N: int, K: int, out, stream=None):
    """llam_ql_gemv_f32 with the library's built-in Q8_1 scratch; `out` is caller-provided."""
    _check(load().llam_ql_gemv_f32_static(fmt, _ptr(w), _ptr(x), _ld(x), _ptr(out), M, N, K, _ld(out), _dev(w),
                                          _stream(stream)), "gemv_f32_static")
    return out


def gemv_fused_f32(projs, x, M: int, K: int, q8_scratch=None, stream=None):
    """projs: list of (fmt, w, out[M,N]) or (fmt, w, out[M,N], plane) sharing the fp32 input x[M,K]."""
    arr = _proj_array(projs)
    _check(load().llam_ql_gemv_fused_f32(arr, len(projs), _ptr(x), _ld(x), M, K, _ptr(q8_scratch), _dev(x),
                                         _stream(stream)), "gemv_fused_f32")


def gemv_accumulate_supported(fmt: int, M: int, N: int, K: int, device: int = 0) -> bool:
    return bool(load().llam_ql_gemv_accumulate_supported(fmt, M, N, K, device))


def gemv_accumulate(fmt: int, w, q8, M: int, N: int, K: int, out, stream=None):
    """out[M,N] += Q8_1 activations times W^T, inside the GEMV's launch."""
    _check(load().llam_ql_gemv_accumulate(fmt, _ptr(w), _ptr(q8), _ptr(out), M, N, K, _ld(out), _dev(w),
                                          _stream(stream)), "gemv_accumulate")
    return out


def _proj_array(projs):
    arr = (Proj * len(projs))()
    for i, p in enumerate(projs):
        arr[i] = _proj(p)
    return arr


def gemv_fused_rmsnorm_supported(projs, M: int, K: int) -> bool:
    """Whether every projection of the list (fmt, w, out[M,N]) can run the norm inside its own kernel."""
    return bool(load().llam_ql_gemv_fused_rmsnorm_supported(_proj_array(projs), len(projs), M, K))


def gemv_fused_rmsnorm(projs, x, delta, gamma, eps: float, x_out, M: int, K: int, stream=None):
    """projs: list of (fmt, w, out[M,N]) on RMSNorm(x (+ delta)) * gamma; x + delta goes to x_out."""
    _check(load().llam_ql_gemv_fused_rmsnorm(_proj_array(projs), len(projs), _ptr(x), _ptr(delta), _ptr(gamma), eps,
                                             _ptr(x_out), M, K, _dev(x), _stream(stream)), "gemv_fused_rmsnorm")


def gemv_swiglu_f32(fmt: int, w, gate, up, M: int, N: int, K: int, out=None, q8_scratch=None, stream=None,
                    plane=None):
    """out[M,N] = (silu(gate) * up)[M,K] @ W^T."""
    import torch

    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=w.device)
    assert _ld(gate) == _ld(up)
    _check(load().llam_ql_gemv_swiglu_f32(fmt, _ptr(w), _ptr(plane), _ptr(gate), _ptr(up), _ld(gate), _ptr(out), M, N, K, _ld(out),
                                          _ptr(q8_scratch), _dev(w), _stream(stream)), "gemv_swiglu_f32")
    return out


def gemv_block_sums(fmt: int, w, q8, M: int, N: int, K: int, row0: int, nrows: int, stream=None, plane=None):
    """The exact int32 block sums of the kernel a launch with these arguments (plane included) runs."""
    import torch

    out = torch.empty(M, nrows, K // 32, dtype=torch.int32, device=w.device)
    _check(load().llam_ql_gemv_block_sums(fmt, _ptr(w), _ptr(plane), _ptr(q8), _ptr(out), M, N, K, row0, nrows, _dev(w),
                                          _stream(stream)), "gemv_block_sums")
    return out


def gemv_describe(fmt: int, M: int, N: int, K: int, device_id: int = 0, has_plane: bool = False) -> GemvPlan:
    """The launch plan for a shape, without or with the matrix's batch plane (no GPU work)."""
    plan = GemvPlan()
    _check(load().llam_ql_gemv_describe(fmt, M, N, K, int(has_plane), device_id, ctypes.byref(plan)), "gemv_describe")
    return plan


def gemm(fmt: int, w, q8, M: int, N: int, K: int, out=None, stream=None):
    import torch

    if out is None:
        out = torch.empty(M, N, dtype=torch.float32, device=w.device)
    _check(load().llam_ql_gemm(fmt, _ptr(w), _ptr(q8), _ptr(out), M, N, K, out.stride(0), _dev(w), _stream(stream)),
           "gemm")
    return out


def gemm_block_sums(fmt: int, w, q8, M: int, N: int, K: int, row0: int, nrows: int, stream=None):
    import torch

    out = torch.empty(M, nrows, K // 32, dtype=torch.int32, device=w.device)
    _check(load().llam_ql_gemm_block_sums(fmt, _ptr(w), _ptr(q8), _ptr(out), M, N, K, row0, nrows, _dev(w),
                                          _stream(stream)), "gemm_block_sums")
    return out


def epilogue(c, t, bias, alpha: float, beta: float, stream=None):
    M, N = t.shape
    _check(load().llam_ql_epilogue(_ptr(c), _ptr(t), _ptr(bias), M, N, c.stride(0), alpha, beta, _dev(c),
                                   _stream(stream)), "epilogue")
    return c


def moe_router_logits(hidden, gate_w, stream=None):
    """logits[T, E] = hidden[T, D] @ gate_w[E, D]^T in fp32."""
    import torch

    T, D = hidden.shape
    E = gate_w.shape[0]
    out = torch.empty(T, E, dtype=torch.float32, device=hidden.device)
    _check(load().llam_ql_moe_router_logits(_ptr(hidden), _ptr(gate_w), _ptr(out), T, D, E, _dev(hidden),
                                            _stream(stream)), "moe_router_logits")
    return out


def moe_route(logits, top_k: int, normalize: bool = True, stream=None, ids=None, weights=None):
    """Top-k routing.  With preallocated ids / weights [T, S >= top_k] only the first top_k
    columns are written (the rest can hold always-on experts such as a shared expert)."""
    import torch

    T, E = logits.shape
    if ids is None:
        ids = torch.empty(T, top_k, dtype=torch.int32, device=logits.device)
        weights = torch.empty(T, top_k, dtype=torch.float32, device=logits.device)
    assert ids.shape == weights.shape and ids.shape[0] == T and ids.is_contiguous() and weights.is_contiguous()
    _check(load().llam_ql_moe_route_ex(_ptr(logits), T, E, top_k, int(normalize), _ptr(ids), _ptr(weights),
                                       ids.shape[1], _dev(logits), _stream(stream)), "moe_route")
    return ids, weights


def moe_route_quantize(logits, top_k: int, hidden, q8_out, normalize: bool = True, stream=None, ids=None,
                       weights=None):
    """moe_route and quantize_q8_1(hidden) in one launch."""
    import torch

    T, E = logits.shape
    if ids is None:
        ids = torch.empty(T, top_k, dtype=torch.int32, device=logits.device)
        weights = torch.empty(T, top_k, dtype=torch.float32, device=logits.device)
    assert ids.shape == weights.shape and ids.shape[0] == T and ids.is_contiguous() and weights.is_contiguous()
    assert hidden.shape[0] == T and hidden.is_contiguous()
    _check(load().llam_ql_moe_route_quantize(_ptr(logits), T, E, top_k, int(normalize), _ptr(ids), _ptr(weights),
                                             ids.shape[1], _ptr(hidden), hidden.shape[1], _ptr(q8_out), _dev(logits),
                                             _stream(stream)), "moe_route_quantize")
    return ids, weights


def expert_table(experts, device):
    """experts: list of (gate, up, down) prepared-weight tensors -> device table (uint8 tensor)."""
    import torch

    arr = (Expert * len(experts))()
    for i, (g, u, d) in enumerate(experts):
        arr[i] = Expert(_ptr(g), _ptr(u), _ptr(d))
    host = torch.frombuffer(bytearray(bytes(arr)), dtype=torch.uint8)
    return host.to(device)


def moe_gate_up(fmt: int, table, n_experts: int, ids, q8, n_tokens: int, top_k: int, hidden: int, inter: int,
                stream=None):
    import torch

    gate = torch.empty(n_tokens * top_k, inter, dtype=torch.float32, device=q8.device)
    up = torch.empty_like(gate)
    _check(load().llam_ql_moe_gate_up(fmt, _ptr(table), n_experts, _ptr(ids), _ptr(q8), _ptr(gate), _ptr(up),
                                      n_tokens, top_k, hidden, inter, _dev(q8), _stream(stream)), "moe_gate_up")
    return gate, up


def moe_gate_up_swiglu(fmt: int, table, n_experts: int, ids, q8, n_tokens: int, top_k: int, hidden: int, inter: int,
                       q8_out=None, scratch=None, stream=None):
    """Q8_1 of silu(gate) * up for every token slot; scratch: (gate, up) fp32 rows for the shapes that need them."""
    import torch

    if q8_out is None:
        q8_out = torch.zeros(n_tokens * top_k * (inter // 32) * 36, dtype=torch.uint8, device=q8.device)
    g, u = scratch if scratch is not None else (None, None)
    _check(load().llam_ql_moe_gate_up_swiglu(fmt, _ptr(table), n_experts, _ptr(ids), _ptr(q8), _ptr(g), _ptr(u),
                                             _ptr(q8_out), n_tokens, top_k, hidden, inter, _dev(q8), _stream(stream)),
           "moe_gate_up_swiglu")
    return q8_out


def moe_route_gate_up_swiglu(fmt: int, table, n_experts: int, logits, top_k: int, x, ids, weights, inter: int,
                             normalize: bool = True, q8_out=None, q8_hidden=None, scratch=None, stream=None):
    """Router, Q8_1 of the hidden rows x, gate/up, SwiGLU and its quantiser; ids / weights [T, slot_stride] are
    written in their first top_k columns and read in the others (always-on slots)."""
    import torch

    T, hidden = x.shape
    stride = ids.shape[1]
    if q8_out is None:
        q8_out = torch.zeros(T * stride * (inter // 32) * 36, dtype=torch.uint8, device=x.device)
    g, u = scratch if scratch is not None else (None, None)
    _check(load().llam_ql_moe_route_gate_up_swiglu(fmt, _ptr(table), n_experts, _ptr(logits), logits.shape[1], top_k,
                                                   int(normalize), _ptr(ids), _ptr(weights), stride, _ptr(x),
                                                   _ptr(q8_hidden), _ptr(g), _ptr(u), _ptr(q8_out), T, hidden, inter,
                                                   _dev(x), _stream(stream)), "moe_route_gate_up_swiglu")
    return q8_out


def gemv_plane_split_supported(fmt: int, M: int, N: int, K: int) -> bool:
    return bool(load().llam_ql_gemv_plane_split_supported(fmt, M, N, K))


def gemv_plane_split(fmt: int, plane, q8, M: int, N: int, K: int, out_lo=None, out_hi=None, stream=None):
    """The sums over the first and the second half of every row's super-blocks as two outputs [M,N] (batches of
    2..8 on long Q6_K rows, 5..8 on Q4_K, from the matrix's batch plane); their sum is the projection."""
    import torch

    if out_lo is None:
        out_lo = torch.empty(M, N, dtype=torch.float32, device=plane.device)
    if out_hi is None:
        out_hi = torch.empty(M, N, dtype=torch.float32, device=plane.device)
    _check(load().llam_ql_gemv_plane_split(fmt, _ptr(plane), _ptr(q8), _ptr(out_lo), _ptr(out_hi), M, N, K, _ld(out_lo),
                                           _dev(plane), _stream(stream)), "gemv_plane_split")
    return out_lo, out_hi


def gemv_gate_up_swiglu_supported(fmt: int, M: int, N: int, K: int) -> bool:
    return bool(load().llam_ql_gemv_gate_up_swiglu_supported(fmt, M, N, K))


def gemv_gate_up_swiglu(fmt: int, w_gate, w_up, q8, M: int, N: int, K: int, plane_gate=None, plane_up=None,
                        want_projections: bool = False, q8_out=None, stream=None):
    """Q8_1 blocks [M x N/32] of silu(W_gate a) * (W_up a) in one launch (batches of 2..8); with
    want_projections also the fp32 projections the blocks were formed from."""
    import torch

    if q8_out is None:
        q8_out = torch.empty(M * (N // 32) * 36, dtype=torch.uint8, device=w_gate.device)
    yg = torch.empty(M, N, dtype=torch.float32, device=w_gate.device) if want_projections else None
    yu = torch.empty(M, N, dtype=torch.float32, device=w_gate.device) if want_projections else None
    _check(load().llam_ql_gemv_gate_up_swiglu(fmt, _ptr(w_gate), _ptr(plane_gate), _ptr(w_up), _ptr(plane_up), _ptr(q8),
                                              _ptr(yg), _ptr(yu), N, _ptr(q8_out), M, N, K, _dev(w_gate),
                                              _stream(stream)), "gemv_gate_up_swiglu")
    return (q8_out, yg, yu) if want_projections else q8_out


def swiglu_quantize(gate, up, want_act: bool = False, stream=None):
    import torch

    rows, inter = gate.shape
    q8 = torch.empty(rows * (inter // 32) * 36, dtype=torch.uint8, device=gate.device)
    act = torch.empty_like(gate) if want_act else None
    _check(load().llam_ql_swiglu_quantize(_ptr(gate), _ptr(up), _ptr(act), _ptr(q8), rows, inter, _dev(gate),
                                          _stream(stream)), "swiglu_quantize")
    return (q8, act) if want_act else q8


def moe_down(fmt: int, table, n_experts: int, ids, weights, q8_act, out, n_tokens: int, top_k: int, hidden: int,
             inter: int, accumulate: bool = False, stream=None):
    _check(load().llam_ql_moe_down(fmt, _ptr(table), n_experts, _ptr(ids), _ptr(weights), _ptr(q8_act), _ptr(out),
                                   n_tokens, top_k, hidden, inter, int(accumulate), _dev(out), _stream(stream)),
           "moe_down")
    return out


def moe_group(ids, n_experts: int, group=None, stream=None):
    """Sort the (token, slot) pairs of ids [T, S] by expert on the device -> workspace tensor."""
    import torch

    T, S = ids.shape
    if group is None:
        group = torch.empty(int(load().llam_ql_moe_group_bytes(T, S)), dtype=torch.uint8, device=ids.device)
    _check(load().llam_ql_moe_group(_ptr(ids), T, S, n_experts, _ptr(group), _dev(ids), _stream(stream)), "moe_group")
    return group


def moe_gate_up_grouped(fmt: int, table, n_experts: int, group, q8, n_tokens: int, slots: int, hidden: int, inter: int,
                        gate=None, up=None, stream=None):
    import torch

    if gate is None:
        gate = torch.empty(n_tokens * slots, inter, dtype=torch.float32, device=q8.device)
        up = torch.empty_like(gate)
    _check(load().llam_ql_moe_gate_up_grouped(fmt, _ptr(table), n_experts, _ptr(group), _ptr(q8), _ptr(gate), _ptr(up),
                                              n_tokens, slots, hidden, inter, _dev(q8), _stream(stream)),
           "moe_gate_up_grouped")
    return gate, up


def moe_down_grouped(fmt: int, table, n_experts: int, group, ids, weights, q8_act, pair_out, out, n_tokens: int,
                     slots: int, hidden: int, inter: int, accumulate: bool = False, stream=None):
    _check(load().llam_ql_moe_down_grouped(fmt, _ptr(table), n_experts, _ptr(group), _ptr(ids), _ptr(weights),
                                           _ptr(q8_act), _ptr(pair_out), _ptr(out), n_tokens, slots, hidden, inter,
                                           int(accumulate), _dev(out), _stream(stream)), "moe_down_grouped")
    return out


def shared_expert_add(out, shared, hidden=None, gate_inp=None, stream=None):
    T, D = out.shape
    _check(load().llam_ql_shared_expert_add(_ptr(out), _ptr(shared), _ptr(hidden), _ptr(gate_inp), T, D, _dev(out),
                                            _stream(stream)), "shared_expert_add")
    return out


# ---- decode-step operators (decode_api.h) -----------------------------------------------------
def embed_q4k(table, vocab: int, ids, H: int, out=None, stream=None):
    import torch

    B = ids.numel()
    if out is None:
        out = torch.empty(B, H, dtype=torch.float32, device=ids.device)
    _check(load().llam_dec_embed_q4k(_ptr(table), vocab, _ptr(ids), _ptr(out), B, H, _ld(out), _dev(ids),
                                     _stream(stream)), "embed_q4k")
    return out


def rmsnorm_q8_1(x, gamma, eps: float, delta=None, want_y: bool = True, want_q8: bool = True, y=None, q8=None,
                 stream=None, delta2=None):
    """x [M,H] contiguous; with delta, x += delta in place first (x += delta + delta2 when the delta comes as two
    partial sums).  Returns (y, q8)."""
    import torch

    M, H = x.shape
    assert x.is_contiguous()
    if want_y and y is None:
        y = torch.empty_like(x)
    if want_q8 and q8 is None:
        q8 = torch.empty(M * (H // 32) * 36, dtype=torch.uint8, device=x.device)
    if delta2 is not None:
        _check(load().llam_dec_rmsnorm2_q8_1(_ptr(x), _ptr(delta), _ptr(delta2), _ptr(gamma), eps, _ptr(y), _ptr(q8), M, H,
                                             _dev(x), _stream(stream)), "rmsnorm2_q8_1")
    else:
        _check(load().llam_dec_rmsnorm_q8_1(_ptr(x), _ptr(delta), _ptr(gamma), eps, _ptr(y), _ptr(q8), M, H, _dev(x),
                                            _stream(stream)), "rmsnorm_q8_1")
    return y, q8


def rope_inv_freq(head_dim: int, theta: float, device=None):
    import numpy as np
    import torch

    f = np.zeros(head_dim // 2, np.float32)
    load().llam_dec_rope_inv_freq(head_dim, theta, f.ctypes.data)
    t = torch.from_numpy(f)
    return t.to(device) if device is not None else t


def kcache_tiled(k):
    """[..., cap, head_dim] position-major values -> the K cache's tiles (same shape, same values):
    [cap/16][head_dim/8][16 positions][8 dims] per (sequence, head)."""
    *lead, cap, hd = k.shape
    assert cap % 32 == 0 and hd % 16 == 0, "cap a multiple of 32, head_dim of 16"
    t = k.reshape(*lead, cap // 16, 16, hd // 8, 8)
    n = len(lead)
    return t.permute(*range(n), n, n + 2, n + 1, n + 3).reshape(*lead, cap, hd).contiguous()


def kcache_logical(k):
    """The inverse of kcache_tiled."""
    *lead, cap, hd = k.shape
    t = k.reshape(*lead, cap // 16, hd // 8, 16, 8)
    n = len(lead)
    return t.permute(*range(n), n, n + 2, n + 1, n + 3).reshape(*lead, cap, hd).contiguous()


def vcache_tiled(v):
    """[..., cap, head_dim] position-major values -> the V cache's tiles (same shape, same values):
    [cap/32][head_dim/16][4 groups of 8 positions][16 dims][8 positions] per (sequence, head)."""
    *lead, cap, hd = v.shape
    assert cap % 32 == 0 and hd % 16 == 0, "cap a multiple of 32, head_dim of 16"
    t = v.reshape(*lead, cap // 32, 4, 8, hd // 16, 16)   # p32, group, p8, d16 tile, d
    n = len(lead)
    return t.permute(*range(n), n, n + 3, n + 1, n + 4, n + 2).reshape(*lead, cap, hd).contiguous()


def vcache_logical(v):
    """The inverse of vcache_tiled."""
    *lead, cap, hd = v.shape
    t = v.reshape(*lead, cap // 32, hd // 16, 4, 16, 8)   # p32, d16 tile, group, d, p8
    n = len(lead)
    return t.permute(*range(n), n, n + 2, n + 4, n + 1, n + 3).reshape(*lead, cap, hd).contiguous()


def rope_kv_append(qkv, inv_freq, pos, kcache, vcache, n_heads: int, n_kv: int, head_dim: int, stream=None):
    """qkv [B, >= (n_heads+2 n_kv)*head_dim] fp32, rotated in place; kcache and vcache [B, n_kv, cap, head_dim]
    fp16 in the tiles of kcache_tiled / vcache_tiled."""
    B = qkv.shape[0]
    cap = kcache.shape[2]
    _check(load().llam_dec_rope_kv_append(_ptr(qkv), _ld(qkv), _ptr(inv_freq), _ptr(pos), _ptr(kcache), _ptr(vcache),
                                          B, n_heads, n_kv, head_dim, cap, _dev(qkv), _stream(stream)),
           "rope_kv_append")


def attention_scratch(B: int, n_heads: int, head_dim: int, cap: int, device):
    import torch

    n = load().llam_dec_attention_scratch_floats(B, n_heads, head_dim, cap)
    return torch.empty(n, dtype=torch.float32, device=device)


def attention(q, kcache, vcache, pos, n_heads: int, n_kv: int, head_dim: int, out=None, scratch=None, stream=None,
              q8_out=None):
    """out [B, n_heads*head_dim] fp32; q8_out (optional) receives the Q8_1 blocks of the same rows.
    kcache and vcache [B, n_kv, cap, head_dim] fp16 in the tiles of kcache_tiled / vcache_tiled."""
    import torch

    B = q.shape[0]
    cap = kcache.shape[2]
    assert tuple(vcache.shape) == tuple(kcache.shape), "both caches are [B, n_kv, cap, head_dim]"
    if out is None:
        out = torch.empty(B, n_heads * head_dim, dtype=torch.float32, device=q.device)
    if scratch is None:
        scratch = attention_scratch(B, n_heads, head_dim, cap, q.device)
    _check(load().llam_dec_attention(_ptr(q), _ld(q), _ptr(kcache), _ptr(vcache), _ptr(pos), _ptr(out), _ld(out),
                                     _ptr(q8_out), _ptr(scratch), B, n_heads, n_kv, head_dim, cap, _dev(q),
                                     _stream(stream)), "attention")
    return out


def rope_table(pos, inv_freq, head_dim: int, stream=None):
    """[B, head_dim/2, 2] fp32: cos and sin of pos[b] * inv_freq[i], for rope_attention."""
    import torch

    B = pos.shape[0]
    table = torch.empty(B, head_dim // 2, 2, dtype=torch.float32, device=pos.device)
    _check(load().llam_dec_rope_table(_ptr(pos), _ptr(inv_freq), _ptr(table), B, head_dim, _dev(pos), _stream(stream)),
           "rope_table")
    return table


def rope_attention(qkv, table, pos, kcache, vcache, n_heads: int, n_kv: int, head_dim: int, out=None,
                   scratch=None, stream=None, q8_out=None):
    """rope_kv_append and attention as one operator; qkv [B, >= (n_heads+2 n_kv)*head_dim] is only read,
    table = rope_table(pos, inv_freq, head_dim)."""
    import torch

    B = qkv.shape[0]
    cap = kcache.shape[2]
    assert tuple(vcache.shape) == tuple(kcache.shape), "both caches are [B, n_kv, cap, head_dim]"
    if out is None:
        out = torch.empty(B, n_heads * head_dim, dtype=torch.float32, device=qkv.device)
    if scratch is None:
        scratch = attention_scratch(B, n_heads, head_dim, cap, qkv.device)
    _check(load().llam_dec_rope_attention(_ptr(qkv), _ld(qkv), _ptr(table), _ptr(pos), _ptr(kcache), _ptr(vcache),
                                          _ptr(out), _ld(out), _ptr(q8_out), _ptr(scratch), B, n_heads, n_kv,
                                          head_dim, cap, _dev(qkv), _stream(stream)), "rope_attention")
    return out


def argmax(logits, n: int, ids=None, pos=None, scratch=None, stream=None):
    import torch

    B = logits.shape[0]
    if ids is None:
        ids = torch.empty(B, dtype=torch.int32, device=logits.device)
    if scratch is None:
        scratch = torch.empty(load().llam_dec_argmax_scratch_bytes(B, n), dtype=torch.uint8, device=logits.device)
    _check(load().llam_dec_argmax(_ptr(logits), _ld(logits), n, B, _ptr(ids), _ptr(pos), _ptr(scratch), _dev(logits),
                                  _stream(stream)), "argmax")
    return ids
