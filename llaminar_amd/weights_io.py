"""ctypes view of the host library's GGUF reader and prepared-weights container
(include/llaminar_amd/weights_io.h)."""
from __future__ import annotations

import ctypes
from ctypes import c_bool, c_char_p, c_double, c_int, c_int32, c_uint8, c_uint32, c_uint64, c_void_p

import numpy as np

from . import decoder


class GgufTensor(ctypes.Structure):
    _fields_ = [("name", c_char_p), ("ggml_type", c_uint32), ("fmt", c_uint8), ("n_dims", c_uint32),
                ("dims", c_uint64 * 4), ("nbytes", c_uint64), ("data", c_void_p)]


class PreparedHeader(ctypes.Structure):
    _fields_ = [("magic", c_uint32), ("version", c_uint32), ("fmt", c_uint8), ("reserved0", c_uint8 * 3),
                ("N", c_int32), ("K", c_int32), ("block_bytes", c_uint32), ("prepared_bytes", c_uint64),
                ("gguf_bytes", c_uint64), ("checksum", c_uint64), ("reserved1", c_uint8 * 16)]


assert ctypes.sizeof(PreparedHeader) == 64

_bound = False


def lib() -> ctypes.CDLL:
    global _bound
    L = decoder.load()
    if not _bound:
        L.llam_weights_last_error.restype = c_char_p
        L.llam_gguf_open.restype = c_void_p
        L.llam_gguf_open.argtypes = [c_char_p]
        L.llam_gguf_close.argtypes = [c_void_p]
        L.llam_gguf_tensor_count.restype = c_uint64
        L.llam_gguf_tensor_count.argtypes = [c_void_p]
        L.llam_gguf_tensor_at.restype = c_bool
        L.llam_gguf_tensor_at.argtypes = [c_void_p, c_uint64, ctypes.POINTER(GgufTensor)]
        L.llam_gguf_find.restype = c_bool
        L.llam_gguf_find.argtypes = [c_void_p, c_char_p, ctypes.POINTER(GgufTensor)]
        L.llam_gguf_meta_u64.restype = c_bool
        L.llam_gguf_meta_u64.argtypes = [c_void_p, c_char_p, ctypes.POINTER(c_uint64)]
        L.llam_gguf_meta_f64.restype = c_bool
        L.llam_gguf_meta_f64.argtypes = [c_void_p, c_char_p, ctypes.POINTER(c_double)]
        L.llam_gguf_meta_str.restype = c_char_p
        L.llam_gguf_meta_str.argtypes = [c_void_p, c_char_p]
        L.llam_weights_checksum.restype = c_uint64
        L.llam_weights_checksum.argtypes = [c_void_p, c_uint64]
        L.llam_prepared_header_build.restype = c_bool
        L.llam_prepared_header_build.argtypes = [c_uint8, c_int, c_int, c_void_p, ctypes.POINTER(PreparedHeader)]
        L.llam_prepared_buffer_check.restype = c_bool
        L.llam_prepared_buffer_check.argtypes = [c_void_p, c_uint64, c_bool]
        L.llam_prepared_save.restype = c_bool
        L.llam_prepared_save.argtypes = [c_char_p, c_uint8, c_int, c_int, c_void_p, c_int]
        L.llam_prepared_load.restype = c_bool
        L.llam_prepared_load.argtypes = [c_char_p, ctypes.POINTER(PreparedHeader), c_void_p, c_uint64, c_int]
        _bound = True
    return L


class WeightsError(RuntimeError):
    pass


def _err() -> str:
    return lib().llam_weights_last_error().decode()


class GgufFile:
    """A GGUF file mapped read-only; tensors come back as numpy views of the mapping."""

    def __init__(self, path):
        self._h = lib().llam_gguf_open(str(path).encode())
        if not self._h:
            raise WeightsError(_err())

    def close(self):
        if self._h:
            lib().llam_gguf_close(self._h)
            self._h = None

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    def __len__(self):
        return int(lib().llam_gguf_tensor_count(self._h))

    @staticmethod
    def _view(t: GgufTensor):
        data = None
        if t.nbytes:
            data = np.ctypeslib.as_array(ctypes.cast(t.data, ctypes.POINTER(c_uint8)), shape=(int(t.nbytes),))
        return {"name": t.name.decode(), "ggml_type": int(t.ggml_type), "fmt": int(t.fmt),
                "dims": [int(t.dims[d]) for d in range(t.n_dims)], "nbytes": int(t.nbytes), "data": data}

    def tensor_at(self, i: int):
        t = GgufTensor()
        if not lib().llam_gguf_tensor_at(self._h, i, ctypes.byref(t)):
            raise WeightsError(_err())
        return self._view(t)

    def find(self, name: str):
        t = GgufTensor()
        if not lib().llam_gguf_find(self._h, name.encode(), ctypes.byref(t)):
            raise WeightsError(_err())
        return self._view(t)

    def meta_int(self, key: str) -> int:
        v = c_uint64()
        if not lib().llam_gguf_meta_u64(self._h, key.encode(), ctypes.byref(v)):
            raise WeightsError(_err())
        return int(v.value)

    def meta_float(self, key: str) -> float:
        v = c_double()
        if not lib().llam_gguf_meta_f64(self._h, key.encode(), ctypes.byref(v)):
            raise WeightsError(_err())
        return float(v.value)

    def meta_str(self, key: str) -> str:
        s = lib().llam_gguf_meta_str(self._h, key.encode())
        if s is None:
            raise WeightsError(_err())
        return s.decode()


def checksum(buf: np.ndarray) -> int:
    buf = np.ascontiguousarray(buf).view(np.uint8)
    return int(lib().llam_weights_checksum(buf.ctypes.data, buf.size))


def header_build(fmt: int, N: int, K: int, payload: np.ndarray) -> PreparedHeader:
    h = PreparedHeader()
    payload = np.ascontiguousarray(payload).view(np.uint8)
    if not lib().llam_prepared_header_build(fmt, N, K, payload.ctypes.data, ctypes.byref(h)):
        raise WeightsError(_err())
    return h


def buffer_check(buf: np.ndarray, verify_checksum: bool = True) -> None:
    buf = np.ascontiguousarray(buf).view(np.uint8)
    if not lib().llam_prepared_buffer_check(buf.ctypes.data, buf.size, verify_checksum):
        raise WeightsError(_err())


def save_prepared(path, fmt: int, N: int, K: int, prepared) -> None:
    """prepared: a torch uint8 tensor on the GPU, as prepare_weights returned it."""
    if not lib().llam_prepared_save(str(path).encode(), fmt, N, K, prepared.data_ptr(), prepared.device.index or 0):
        raise WeightsError(_err())


def load_prepared(path, device):
    """Returns (header, torch uint8 tensor on `device` holding the prepared matrix)."""
    import torch

    h = PreparedHeader()
    if not lib().llam_prepared_load(str(path).encode(), ctypes.byref(h), None, 0, device.index or 0):
        raise WeightsError(_err())
    out = torch.empty(int(h.prepared_bytes), dtype=torch.uint8, device=device)
    if not lib().llam_prepared_load(str(path).encode(), ctypes.byref(h), out.data_ptr(), out.numel(),
                                    device.index or 0):
        raise WeightsError(_err())
    return h, out
