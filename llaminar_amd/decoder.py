"""ctypes door onto the host library's dense decoder (include/llaminar_amd/dense_decoder.h)
for the tests and the benchmark: build a random-init model in device memory, run steps."""
from __future__ import annotations

import ctypes
from ctypes import c_bool, c_char_p, c_float, c_int, c_size_t, c_uint8, c_void_p
from dataclasses import dataclass
from pathlib import Path

from . import capi, synth
from .capi import FMT_Q4_K, FMT_Q6_K

HOST_LIB = Path(__file__).resolve().parent / "lib" / "libllaminar_ql_host.so"


class Config(ctypes.Structure):
    _fields_ = [("hidden", c_int), ("n_heads", c_int), ("n_kv", c_int), ("head_dim", c_int), ("ffn", c_int),
                ("vocab", c_int), ("n_layers", c_int), ("ctx_cap", c_int), ("batch", c_int),
                ("rope_theta", c_float), ("rms_eps", c_float), ("device_id", c_int)]


class Layer(ctypes.Structure):
    _fields_ = [(n, c_void_p) for n in ("wq", "wk", "wv", "wo", "wgate", "wup", "wdown")] + \
               [(n, c_uint8) for n in ("fmt_q", "fmt_k", "fmt_v", "fmt_o", "fmt_gate", "fmt_up", "fmt_down")] + \
               [("attn_norm", c_void_p), ("ffn_norm", c_void_p)] + \
               [(n, c_void_p) for n in ("plane_q", "plane_k", "plane_v", "plane_o", "plane_gate", "plane_up", "plane_down")]


class Globals(ctypes.Structure):
    _fields_ = [("embed_q4k", c_void_p), ("final_norm", c_void_p), ("lm_head", c_void_p), ("fmt_lm_head", c_uint8),
                ("plane_lm_head", c_void_p)]


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        capi.load()  # the kernel library first (and torch before it, for the HIP runtime)
        if not HOST_LIB.exists():
            raise capi.QLError(f"{HOST_LIB} is missing: run python -m llaminar_amd.build")
        L = ctypes.CDLL(str(HOST_LIB))
        L.llam_decoder_create.restype = c_void_p
        L.llam_decoder_create.argtypes = [ctypes.POINTER(Config)]
        L.llam_decoder_destroy.argtypes = [c_void_p]
        L.llam_decoder_set_layer.restype = c_bool
        L.llam_decoder_set_layer.argtypes = [c_void_p, c_int, ctypes.POINTER(Layer)]
        L.llam_decoder_set_globals.restype = c_bool
        L.llam_decoder_set_globals.argtypes = [c_void_p, ctypes.POINTER(Globals)]
        L.llam_decoder_set_state.restype = c_bool
        L.llam_decoder_set_state.argtypes = [c_void_p, c_void_p, c_void_p]
        L.llam_decoder_step.restype = c_bool
        L.llam_decoder_step.argtypes = [c_void_p, c_void_p]
        L.llam_decoder_steps_left.restype = c_int
        L.llam_decoder_steps_left.argtypes = [c_void_p]
        L.llam_decoder_advance.restype = c_bool
        L.llam_decoder_advance.argtypes = [c_void_p, c_int]
        L.llam_decoder_buffer.restype = c_void_p
        L.llam_decoder_buffer.argtypes = [c_void_p, c_char_p, c_int]
        L.llam_decoder_device_bytes.restype = c_size_t
        L.llam_decoder_device_bytes.argtypes = [c_void_p]
        L.llam_decoder_last_error.restype = c_char_p
        _lib = L
    return _lib


# projections of a layer: name, rows, columns (as attributes of the shape), GGUF format
@dataclass
class Shape:
    hidden: int = 5120
    n_heads: int = 64
    n_kv: int = 8
    head_dim: int = 128
    ffn: int = 25600
    vocab: int = 152064
    n_layers: int = 64
    rope_theta: float = 1e6
    rms_eps: float = 1e-6

    def projections(self):
        q, kv = self.n_heads * self.head_dim, self.n_kv * self.head_dim
        return [("wq", q, self.hidden, FMT_Q4_K), ("wk", kv, self.hidden, FMT_Q4_K), ("wv", kv, self.hidden, FMT_Q6_K),
                ("wo", self.hidden, q, FMT_Q4_K), ("wgate", self.ffn, self.hidden, FMT_Q4_K),
                ("wup", self.ffn, self.hidden, FMT_Q4_K), ("wdown", self.hidden, self.ffn, FMT_Q6_K)]

    def weight_bytes_per_token(self) -> int:
        """GGUF bytes one decode step streams: all layers' projections and the lm_head."""
        per = {FMT_Q4_K: 144, FMT_Q6_K: 210}
        layer = sum(n * (k // 256) * per[f] for _, n, k, f in self.projections())
        return self.n_layers * layer + self.vocab * (self.hidden // 256) * per[FMT_Q6_K]


class DenseDecoder:
    """Random-init model of the given shape: Q4_K/Q6_K projections, Q4_K embedding, Q6_K lm_head,
    norm weights ~U(0.5,1.5) * norm_scale.  Weights are generated on the device, seeded; `raw` keeps the GGUF
    bytes (device tensors) when keep_raw is set, for the CPU check."""

    def __init__(self, shape: Shape, batch: int, ctx_cap: int, device, seed: int = 0, keep_raw: bool = False,
                 d_lo: float = 0.001, d_hi: float = 0.02, keep_prepared: bool = False, norm_scale: float | None = None,
                 batch_planes: bool | None = None):
        import torch

        self.shape, self.batch, self.ctx_cap, self.device = shape, batch, ctx_cap, device
        self.L = load()
        cfg = Config(shape.hidden, shape.n_heads, shape.n_kv, shape.head_dim, shape.ffn, shape.vocab, shape.n_layers,
                     ctx_cap, batch, shape.rope_theta, shape.rms_eps, device.index or 0)
        self.h = self.L.llam_decoder_create(ctypes.byref(cfg))
        if not self.h:
            raise capi.QLError(self.L.llam_decoder_last_error().decode())
        self.keep = []   # device tensors the handle borrows
        self.raw = {} if keep_raw else None
        self.prepared = {} if keep_prepared else None   # name -> prepared weight tensor
        # Matrices of 4096 rows and more get a batch plane where the batch is 5..8 rows (capi.build_batch_plane):
        # Q6_K ones (down, lm_head) an int8 copy, Q4_K ones (Q, O, gate, up) their bytes in the matrix unit's
        # operand order; same results, less work per launch.  At batches of 2..4 only the feed-forward matrices get
        # one: the step runs them on the launches that name the matrix unit (gate + up + SwiGLU in one, the down
        # projection in two halves), the other projections stay on the quad-lane kernel, which reads no plane.
        if batch_planes is None:
            batch_planes = batch >= 2
        ffn_only = batch < 5
        self.planes = {}   # name -> batch plane of that matrix
        g = torch.Generator(device=device)
        g.manual_seed(seed)

        # Random block fields give weights of mean ~2 and spread ~2.8 (at d ~ U(0.001, 0.02)), so a
        # projection multiplies the norm of its input by about 2.8 sqrt(K).  Norm weights of
        # that inverse size keep q, k, v and the feed-forward activations O(1): inside fp16
        # range for the KV cache and away from SwiGLU's flat tail.
        if norm_scale is None:
            norm_scale = 1.0 / (2.8 * shape.hidden ** 0.5)

        def norm_weight(name):
            t = (torch.rand(shape.hidden, device=device, generator=g) + 0.5) * norm_scale
            self.keep.append(t)
            if keep_raw:
                self.raw[name] = t
            return t.data_ptr()

        def weights(name, fmt, n, k, sd, prepare=True):
            raw = synth.weights_torch(fmt, n, k, sd, device, d_lo=d_lo, d_hi=d_hi)
            w = capi.prepare_weights(fmt, raw, n, k) if prepare else raw
            self.keep.append(w)
            plane = None
            wanted = not ffn_only or name.endswith((".wgate", ".wup", ".wdown"))
            if prepare and batch_planes and wanted and n >= 4096 and capi.batch_plane_bytes(fmt, n, k) > 0:
                plane = capi.build_batch_plane(fmt, w, n, k)
                if plane is not None:
                    self.planes[name] = plane
            if keep_raw:
                self.raw[name] = raw
            if keep_prepared:
                self.prepared[name] = w
            return w.data_ptr(), (plane.data_ptr() if plane is not None else None)

        for l in range(shape.n_layers):
            lw = Layer()
            for i, (name, n, k, fmt) in enumerate(shape.projections()):
                w_ptr, plane_ptr = weights(f"{l}.{name}", fmt, n, k, seed * 100003 + l * 16 + i)
                setattr(lw, name, w_ptr)
                setattr(lw, "fmt_" + name[1:], fmt)
                setattr(lw, "plane_" + name[1:], plane_ptr)
            lw.attn_norm = norm_weight(f"{l}.attn_norm")
            lw.ffn_norm = norm_weight(f"{l}.ffn_norm")
            if not self.L.llam_decoder_set_layer(self.h, l, ctypes.byref(lw)):
                raise capi.QLError(self.L.llam_decoder_last_error().decode())
        gl = Globals()
        gl.embed_q4k, _ = weights("embed", FMT_Q4_K, shape.vocab, shape.hidden, seed * 100003 + 900001, prepare=False)
        gl.final_norm = norm_weight("final_norm")
        gl.lm_head, gl.plane_lm_head = weights("lm_head", FMT_Q6_K, shape.vocab, shape.hidden, seed * 100003 + 900002)
        gl.fmt_lm_head = FMT_Q6_K
        if not self.L.llam_decoder_set_globals(self.h, ctypes.byref(gl)):
            raise capi.QLError(self.L.llam_decoder_last_error().decode())
        torch.cuda.synchronize()

    def close(self):
        if self.h:
            self.L.llam_decoder_destroy(self.h)
            self.h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def buffer(self, name: str, layer: int = 0):
        """A device buffer of the handle as a torch tensor sharing its memory."""
        import torch

        s, B = self.shape, self.batch
        ptr = self.L.llam_decoder_buffer(self.h, name.encode(), layer)
        if not ptr:
            raise capi.QLError(self.L.llam_decoder_last_error().decode())
        shapes = {"ids": ((B,), torch.int32), "pos": ((B,), torch.int32), "logits": ((B, s.vocab), torch.float32),
                  "x": ((B, s.hidden), torch.float32),
                  "kcache": ((B, s.n_kv, self.ctx_cap, s.head_dim), torch.float16),
                  "vcache": ((B, s.n_kv, self.ctx_cap, s.head_dim), torch.float16)}   # both in tiles (capi.kcache_tiled, vcache_tiled)
        shp, dt = shapes[name]
        n = 1
        for v in shp:
            n *= v
        return _tensor_from_ptr(ptr, n, dt, self.device).view(shp)

    def set_state(self, ids, pos):
        import numpy as np

        i = np.ascontiguousarray(ids, dtype=np.int32)
        p = np.ascontiguousarray(pos, dtype=np.int32)
        assert i.size == self.batch and p.size == self.batch
        if not self.L.llam_decoder_set_state(self.h, i.ctypes.data, p.ctypes.data):
            raise capi.QLError(self.L.llam_decoder_last_error().decode())

    def step(self, stream=None):
        if not self.L.llam_decoder_step(self.h, capi._stream(stream)):
            raise capi.QLError(self.L.llam_decoder_last_error().decode())

    def steps_left(self) -> int:
        """Steps before the furthest sequence reaches the end of the cache (the host's count)."""
        return int(self.L.llam_decoder_steps_left(self.h))

    def advance(self, n: int):
        """Report n replays of a captured step (they do not pass through step())."""
        if not self.L.llam_decoder_advance(self.h, n):
            raise capi.QLError(self.L.llam_decoder_last_error().decode())

    def device_bytes(self) -> int:
        return int(self.L.llam_decoder_device_bytes(self.h))


def _tensor_from_ptr(ptr: int, numel: int, dtype, device):
    """Torch view of device memory owned elsewhere (the decoder handle outlives the view)."""
    import torch

    itemsize = torch.empty(0, dtype=dtype).element_size()

    class _Mem:
        __cuda_array_interface__ = {"shape": (numel * itemsize,), "typestr": "|u1", "data": (ptr, False),
                                    "version": 2, "strides": None}

    return torch.as_tensor(_Mem(), device=device).view(dtype)
