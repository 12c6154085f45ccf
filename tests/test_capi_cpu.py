"""CPU-side checks of the boundary: the built library exports every symbol the
header declares, the Python binding mirrors it, argument validation fails with
the documented error text, and without a GPU a valid call fails loudly instead of
falling back to anything."""
import ctypes
import re
from pathlib import Path

import numpy as np
import pytest

ROOT = Path(__file__).resolve().parent.parent
HEADER = ROOT / "include" / "llaminar_amd" / "ql_api.h"
DECODE_HEADER = ROOT / "include" / "llaminar_amd" / "decode_api.h"


def declared_symbols():
    text = HEADER.read_text() + DECODE_HEADER.read_text()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(llam_(?:ql|dec)_[a-z0-9_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol():
    from llaminar_amd import capi

    assert capi.LIB_PATH.exists(), "build the library first: python -m llaminar_amd.build"
    lib = ctypes.CDLL(str(capi.LIB_PATH))
    names = declared_symbols()
    assert len(names) >= 14
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ but not exported"
    assert set(names) == set(capi.SIGNATURES), "capi.SIGNATURES out of step with the headers"


def test_host_library_exports_every_declared_symbol():
    """dense_decoder.h and weights_io.h are the C ABI of the host library."""
    from llaminar_amd import capi, decoder

    capi.load()
    assert decoder.HOST_LIB.exists(), "build the library first: python -m llaminar_amd.build"
    lib = ctypes.CDLL(str(decoder.HOST_LIB))
    text = "".join((ROOT / "include" / "llaminar_amd" / h).read_text() for h in ("dense_decoder.h", "weights_io.h"))
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    names = sorted(set(re.findall(r"\b(llam_(?:decoder|gguf|weights|prepared)_[a-z0-9_]+)\s*\(", text)))
    assert len(names) >= 20, names
    for n in names:
        assert hasattr(lib, n), f"{n} declared in include/ but not exported by the host library"


def test_block_layouts_match_header():
    from llaminar_amd import capi

    text = (ROOT / "include" / "llaminar_amd" / "ql_blocks.h").read_text()
    for fmt, size in capi.BLOCK_BYTES.items():
        assert re.search(rf"== {size},", text)
    assert re.search(r"LLAM_FMT_Q4_K = 5", text) and capi.FMT_Q4_K == 5
    assert re.search(r"LLAM_FMT_Q6_K = 8", text) and capi.FMT_Q6_K == 8
    assert re.search(r"LLAM_FMT_IQ3_S = 11", text) and capi.FMT_IQ3_S == 11


def test_argument_validation_and_error_text():
    from llaminar_amd import capi

    lib = capi.load()
    assert lib.llam_ql_abi_version() == 2
    buf = np.zeros(4096, np.uint8)
    p = buf.ctypes.data
    p16 = p + (-p % 16)
    assert not lib.llam_ql_quantize_q8_1(p16 + 4, p16, 1, 64, 0, None)
    assert "16-byte aligned" in capi.last_error() and "llam_ql_quantize_q8_1" in capi.last_error()
    assert not lib.llam_ql_quantize_q8_1(p16 + 2, p16, 1, 33, 0, None)
    assert "4-byte aligned" in capi.last_error()
    assert not lib.llam_ql_gemv(capi.FMT_Q4_K, p16, p16, p16, 9, 4, 256, 4, 0, None)
    assert "M=9" in capi.last_error()
    assert not lib.llam_ql_gemv(capi.FMT_Q4_K, p16, p16, p16, 1, 4, 100, 4, 0, None)
    assert "multiple of 256" in capi.last_error()
    assert not lib.llam_ql_gemv(77, p16, p16, p16, 1, 4, 256, 4, 0, None)
    assert "unsupported weight format" in capi.last_error()
    assert not lib.llam_ql_gemv(capi.FMT_Q4_K, p16 + 4, p16, p16, 1, 4, 256, 4, 0, None)
    assert "aligned" in capi.last_error()
    assert not lib.llam_ql_gemv(capi.FMT_Q4_K, p16, p16, p16, 1, 4, 256, 3, 0, None)
    assert "ldy" in capi.last_error()
    assert not lib.llam_ql_moe_route(p16, 1, 8, 9, 1, p16, p16, 0, None)
    assert "top_k" in capi.last_error()
    # Q6_K: the 210 bytes of a block in planes, padded to 16, then 8 four-byte factor records per block
    assert lib.llam_ql_prepared_bytes(capi.FMT_Q6_K, 4, 512) == 4 * 2 * 210 + 4 * 2 * 32
    assert lib.llam_ql_prepared_bytes(capi.FMT_Q6_K, 3, 256) == 640 + 3 * 32
    assert lib.llam_ql_prepared_bytes(capi.FMT_IQ3_S, 4, 512) == 4 * 2 * 112
    assert lib.llam_ql_prepared_bytes(capi.FMT_Q4_K, 4, 100) == 0
    # empty problems are a successful no-op
    assert lib.llam_ql_quantize_q8_1(None, None, 0, 0, 0, None)


def test_valid_call_without_gpu_fails_loudly():
    import torch

    if torch.cuda.is_available():
        pytest.skip("a GPU is present")
    from llaminar_amd import capi

    lib = capi.load()
    buf = np.zeros(4096, np.uint8)
    p16 = buf.ctypes.data + (-buf.ctypes.data % 16)
    assert not lib.llam_ql_quantize_q8_1(p16, p16, 1, 32, 0, None)
    assert "no HIP device" in capi.last_error()


def test_synthetic_generators_are_seeded_and_in_range():
    from llaminar_amd import capi, synth

    for fmt in (capi.FMT_Q4_K, capi.FMT_Q6_K, capi.FMT_IQ3_S):
        a = synth.weights_numpy(fmt, 8, 512, 3)
        b = synth.weights_numpy(fmt, 8, 512, 3)
        assert np.array_equal(a, b) and a.shape == (8, 2, capi.BLOCK_BYTES[fmt])
        off = {capi.FMT_Q4_K: 0, capi.FMT_Q6_K: 208, capi.FMT_IQ3_S: 0}[fmt]
        d = a[:, :, off:off + 2].copy().view(np.float16).astype(np.float32)
        assert d.min() >= 0.000999 and d.max() <= 0.02
    assert synth.gemv_bytes(capi.FMT_Q4_K, 25600, 5120) == 25600 * 20 * 144 + 160 * 36 + 25600 * 4


def test_cache_tiles_follow_the_documented_offsets():
    """capi.kcache_tiled / vcache_tiled (the host-side views of the KV caches) against the element offsets
    include/llaminar_amd/decode_api.h gives for llam_dec_rope_kv_append, and their inverses."""
    import torch

    from llaminar_amd import capi

    cap, hd = 96, 128
    x = torch.arange(2 * 3 * cap * hd, dtype=torch.float32).reshape(2, 3, cap, hd)
    kt, vt = capi.kcache_tiled(x), capi.vcache_tiled(x)
    assert kt.shape == x.shape and vt.shape == x.shape
    assert torch.equal(capi.kcache_logical(kt), x) and torch.equal(capi.vcache_logical(vt), x)
    kf, vf = kt.reshape(2, 3, -1), vt.reshape(2, 3, -1)
    rng = np.random.default_rng(0)
    for _ in range(3000):
        p, d = int(rng.integers(cap)), int(rng.integers(hd))
        k_off = (p // 16) * 16 * hd + (d // 8) * 128 + (p % 16) * 8 + d % 8
        v_off = (p // 32) * 32 * hd + (d // 16) * 512 + ((p // 8) % 4) * 128 + (d % 16) * 8 + p % 8
        assert kf[1, 2, k_off] == x[1, 2, p, d] and vf[0, 1, v_off] == x[0, 1, p, d]
    with pytest.raises(AssertionError):
        capi.kcache_tiled(torch.zeros(1, 1, 40, 128))   # capacities are multiples of 32
