"""ctypes door onto tests/probe/libql_probe.so: the read-only load-stream probes of
``bench.py --workload read-order`` and the tile-rows sweep override of the matrix-unit
kernels.  Measurement and test infrastructure; the product library does not contain it."""
from __future__ import annotations

import ctypes
from ctypes import c_bool, c_int, c_void_p
from pathlib import Path

LIB_PATH = Path(__file__).resolve().parent / "libql_probe.so"
_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        from llaminar_amd import capi

        capi.load()  # the product library (and torch's HIP runtime) first
        if not LIB_PATH.exists():
            raise ImportError(f"{LIB_PATH} is missing: make -C tests/probe")
        lib = ctypes.CDLL(str(LIB_PATH))
        lib.llam_probe_read.restype = c_bool
        lib.llam_probe_read.argtypes = [c_void_p, c_int, c_int, c_int, c_int, c_int, c_int, c_int, c_void_p, c_int,
                                        c_void_p]
        lib.llam_probe_set_batch_tile_rows.restype = None
        lib.llam_probe_set_batch_tile_rows.argtypes = [c_int]
        _lib = lib
    return _lib
