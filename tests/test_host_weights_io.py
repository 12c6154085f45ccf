"""GGUF reader and prepared-weights container of the host library (weights_io.h).

No GGUF file ships with the reference and none can be fetched here, so the files are written by
this module from the published layout of the format (header, metadata pairs, tensor directory,
aligned data section); the tensors hold the synthetic super-blocks every other test uses."""
import struct

import numpy as np
import pytest

from llaminar_amd import synth
from llaminar_amd.capi import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import TOL, rel_err, sync, upload_q8

GGML = {FMT_Q4_K: 12, FMT_Q6_K: 14, FMT_IQ3_S: 21}
U8, I8, U16, I16, U32, I32, F32, BOOL, STR, ARR, U64, I64, F64 = range(13)
_SCALAR = {U8: "<B", I8: "<b", U16: "<H", I16: "<h", U32: "<I", I32: "<i", F32: "<f", BOOL: "<B", U64: "<Q",
           I64: "<q", F64: "<d"}


def _s(text: str) -> bytes:
    b = text.encode()
    return struct.pack("<Q", len(b)) + b


def _value(vtype, v) -> bytes:
    if vtype == STR:
        return _s(v)
    if vtype == ARR:
        etype, items = v
        return struct.pack("<IQ", etype, len(items)) + b"".join(_value(etype, x) for x in items)
    return struct.pack(_SCALAR[vtype], v)


def gguf_bytes(meta, tensors, version=3, alignment=32, declare_alignment=True) -> bytes:
    """meta: [(key, type, value)]; tensors: [(name, ggml_type, dims, payload bytes)]."""
    meta = list(meta)
    if declare_alignment and alignment != 32:
        meta.append(("general.alignment", U32, alignment))
    out = struct.pack("<IIQQ", 0x46554747, version, len(tensors), len(meta))
    for key, vtype, v in meta:
        out += _s(key) + struct.pack("<I", vtype) + _value(vtype, v)
    offsets, at = [], 0
    for _, _, _, payload in tensors:
        offsets.append(at)
        at = (at + len(payload) + alignment - 1) // alignment * alignment
    for (name, gtype, dims, _), off in zip(tensors, offsets):
        out += _s(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", gtype, off)
    out += b"\0" * (-len(out) % alignment)
    for (_, _, _, payload), off in zip(tensors, offsets):
        out += payload + b"\0" * (-len(payload) % alignment)
    return out


@pytest.fixture()
def wio():
    from llaminar_amd import weights_io

    weights_io.lib()
    return weights_io


def _sample_file():
    w4 = synth.weights_numpy(FMT_Q4_K, 3, 512, 1)
    w6 = synth.weights_numpy(FMT_Q6_K, 5, 256, 2)
    f32 = np.arange(7, dtype=np.float32)
    meta = [("general.architecture", STR, "qwen3"), ("qwen3.block_count", U32, 64),
            ("qwen3.rope.freq_base", F32, 1e6), ("qwen3.attention.layer_norm_rms_epsilon", F64, 1e-6),
            ("some.flag", BOOL, 1), ("a.small", I8, 5), ("a.negative", I32, -3), ("a.big", U64, 1 << 40),
            ("tokenizer.ggml.tokens", ARR, (STR, ["a", "bc", ""])), ("tokenizer.ggml.scores", ARR, (F32, [0.5, 1.5])),
            ("nested", ARR, (ARR, [(U16, [1, 2]), (U16, [])]))]
    tensors = [("blk.0.attn_q.weight", 12, [512, 3], w4.tobytes()), ("output_norm.weight", 0, [7], f32.tobytes()),
               ("blk.0.ffn_down.weight", 14, [256, 5], w6.tobytes())]
    return meta, tensors, (w4, w6, f32)


def test_gguf_directory_and_metadata(wio, tmp_path):
    meta, tensors, (w4, w6, f32) = _sample_file()
    for version, alignment in ((3, 32), (2, 64), (3, 4096)):
        p = tmp_path / f"m{version}_{alignment}.gguf"
        p.write_bytes(gguf_bytes(meta, tensors, version, alignment))
        with wio.GgufFile(p) as g:
            assert len(g) == 3
            t = g.tensor_at(0)
            assert (t["name"], t["ggml_type"], t["fmt"], t["dims"]) == ("blk.0.attn_q.weight", 12, FMT_Q4_K, [512, 3])
            assert t["nbytes"] == 3 * 2 * 144 and np.array_equal(t["data"], w4.reshape(-1).view(np.uint8))
            assert t["data"].ctypes.data % alignment == 0 or alignment > 4096
            t = g.find("blk.0.ffn_down.weight")
            assert (t["fmt"], t["dims"], t["nbytes"]) == (FMT_Q6_K, [256, 5], 5 * 210)
            assert np.array_equal(t["data"], w6.reshape(-1).view(np.uint8))
            t = g.find("output_norm.weight")
            assert t["fmt"] == 0 and np.array_equal(t["data"].view(np.float32), f32)
            assert g.meta_str("general.architecture") == "qwen3"
            assert g.meta_int("qwen3.block_count") == 64 and g.meta_int("a.big") == 1 << 40
            assert g.meta_int("some.flag") == 1 and g.meta_int("a.small") == 5
            assert g.meta_float("qwen3.rope.freq_base") == 1e6
            assert g.meta_float("qwen3.attention.layer_norm_rms_epsilon") == 1e-6
            for call, key in ((g.meta_int, "a.negative"), (g.meta_int, "general.architecture"),
                              (g.meta_float, "qwen3.block_count"), (g.meta_str, "qwen3.block_count"),
                              (g.meta_int, "absent"), (g.meta_int, "tokenizer.ggml.tokens"), (g.find, "absent")):
                with pytest.raises(wio.WeightsError):
                    call(key)
            with pytest.raises(wio.WeightsError):
                g.tensor_at(3)


def test_gguf_unknown_type_is_listed_without_a_size(wio, tmp_path):
    p = tmp_path / "u.gguf"
    p.write_bytes(gguf_bytes([], [("x", 99, [32], b"\1" * 32), ("y", 8, [64, 2], b"\2" * 136)]))
    with wio.GgufFile(p) as g:
        assert g.tensor_at(0)["nbytes"] == 0 and g.tensor_at(0)["data"] is None
        assert g.tensor_at(1)["nbytes"] == 136 and g.tensor_at(1)["fmt"] == 0   # Q8_0: known size, no kernel here


def test_gguf_malformed_files_are_refused(wio, tmp_path):
    meta, tensors, _ = _sample_file()
    good = gguf_bytes(meta, tensors)
    p = tmp_path / "bad.gguf"

    def refused(data, what):
        p.write_bytes(data)
        with pytest.raises(wio.WeightsError, match=what):
            wio.GgufFile(p)

    refused(b"GGML" + good[4:], "magic")
    refused(good[:4] + struct.pack("<I", 1) + good[8:], "version")
    refused(good[:8] + struct.pack("<Q", 1 << 60) + good[16:], "exceed")
    refused(good[:16] + struct.pack("<Q", 1 << 60) + good[24:], "exceed")
    refused(good[:10], "too short")
    # a tensor that runs past the end, an unaligned offset, a row that is no whole number of blocks
    w4 = tensors[0][3]
    refused(gguf_bytes([], [("a", 12, [512, 3], w4)])[:-64], "past the end")
    refused(gguf_bytes([], [("a", 12, [512, 4], w4)]), "past the end")
    refused(gguf_bytes([], [("a", 12, [500, 3], w4)]), "multiple of the block")
    refused(gguf_bytes([], [("a", 0, [1 << 40, 1 << 40], b"")]), "overflows")
    refused(gguf_bytes([], [("a", 0, [4], b"\0" * 16), ("a", 0, [4], b"\0" * 16)]), "twice")
    refused(gguf_bytes([], [("a", 0, [0], b"")]), "dimension")
    refused(gguf_bytes([("general.alignment", U32, 48)], [("a", 0, [4], b"\0" * 16)], declare_alignment=False),
            "power of two")
    unaligned = bytearray(gguf_bytes([], [("a", 0, [4], b"\0" * 16), ("b", 0, [4], b"\0" * 16)]))
    # the second tensor's offset field is the last 8 bytes of its directory entry
    entry_end = unaligned.index(b"\x01\0\0\0\0\0\0\0b") + 8 + 1 + 4 + 8 + 4 + 8
    unaligned[entry_end - 8:entry_end] = struct.pack("<Q", 36)
    refused(bytes(unaligned), "not aligned")
    # every truncation of a valid file either opens (the cut fell into trailing padding) or is refused
    for cut in list(range(0, 700, 7)) + [len(good) - 1, len(good) - 40]:
        p.write_bytes(good[:cut])
        try:
            wio.GgufFile(p).close()
        except wio.WeightsError:
            pass


def test_checksum_and_container_header(wio, capi):
    capi_cpu = capi.load()
    rng = np.random.default_rng(3)
    a = rng.integers(0, 256, 1003, dtype=np.uint8)
    h = 0xcbf29ce484222325
    padded = np.concatenate([a, np.zeros(-a.size % 8, np.uint8)]).view("<u8")
    for w in padded:
        h = ((h ^ int(w)) * 0x100000001b3) & (2 ** 64 - 1)
    assert wio.checksum(a) == h
    assert wio.checksum(a[:0]) == 0xcbf29ce484222325

    N, K = 3, 512
    for fmt, block in ((FMT_Q4_K, 144), (FMT_Q6_K, 210), (FMT_IQ3_S, 110)):
        nbytes = capi_cpu.llam_ql_prepared_bytes(fmt, N, K)
        payload = rng.integers(0, 256, nbytes, dtype=np.uint8)
        hdr = wio.header_build(fmt, N, K, payload)
        assert (hdr.magic, hdr.version, hdr.fmt, hdr.N, hdr.K) == (0x5750514C, 2, fmt, N, K)
        assert (hdr.block_bytes, hdr.prepared_bytes, hdr.gguf_bytes) == (block, nbytes, N * 2 * block)
        assert hdr.checksum == wio.checksum(payload)
        blob = np.concatenate([np.frombuffer(bytes(hdr), np.uint8), payload])
        wio.buffer_check(blob)
        bad = blob.copy()
        bad[64 + nbytes // 2] ^= 1
        wio.buffer_check(bad, verify_checksum=False)
        with pytest.raises(wio.WeightsError, match="checksum"):
            wio.buffer_check(bad)
        for off, val, what in ((0, 0, "magic"), (4, 9, "version"), (8, 77, "format"), (9, 1, "reserved"),
                               (12, 0, "shape"), (16, 1, "shape"), (20, 1, "block size"), (24, 1, "payload size"),
                               (32, 1, "source size"), (60, 1, "reserved")):
            bad = blob.copy()
            bad[off] = val
            with pytest.raises(wio.WeightsError, match=what):
                wio.buffer_check(bad)
        with pytest.raises(wio.WeightsError, match="does not fit"):
            wio.buffer_check(blob[:-1])
        with pytest.raises(wio.WeightsError, match="shorter than the header"):
            wio.buffer_check(blob[:63])
    with pytest.raises(wio.WeightsError):
        wio.header_build(FMT_Q4_K, 3, 500, np.zeros(16, np.uint8))
    with pytest.raises(wio.WeightsError):
        wio.header_build(3, 3, 512, np.zeros(16, np.uint8))


@pytest.mark.gpu
@pytest.mark.parametrize("fmt", [FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S])
def test_gguf_tensor_to_prepared_to_file_and_back(capi, dev, oracle, wio, tmp_path, fmt):
    """A tensor read from a GGUF file, uploaded and prepared multiplies as the oracle does on the same
    bytes; the prepared matrix survives a round trip through the container bit for bit; a damaged
    container is refused."""
    import torch

    N, K = 96, 1024
    W = synth.weights_numpy(fmt, N, K, 50 + fmt)
    path = tmp_path / "model.gguf"
    path.write_bytes(gguf_bytes([("general.architecture", STR, "test")],
                                [("pad", 0, [3], np.zeros(3, np.float32).tobytes()),
                                 ("blk.0.w", GGML[fmt], [K, N], W.tobytes())]))
    with wio.GgufFile(path) as g:
        t = g.find("blk.0.w")
        assert t["fmt"] == fmt and t["dims"] == [K, N]
        raw = torch.from_numpy(t["data"].copy()).to(dev)
    wd = capi.prepare_weights(fmt, raw, N, K)
    q8 = oracle.quantize(synth.activations_numpy(2, K, 9))
    y = capi.gemv(fmt, wd, upload_q8(dev, q8), 2, N, K)
    sync()
    assert rel_err(y.cpu().numpy(), oracle.gemm(fmt, W, K, q8)) <= TOL[fmt] * 1e-2

    blob = tmp_path / "w.lqpw"
    wio.save_prepared(blob, fmt, N, K, wd)
    hdr, back = wio.load_prepared(blob, dev)
    assert (hdr.fmt, hdr.N, hdr.K, hdr.prepared_bytes) == (fmt, N, K, wd.numel())
    assert torch.equal(back, wd.view(torch.uint8).reshape(-1)[:back.numel()])
    y2 = capi.gemv(fmt, back, upload_q8(dev, q8), 2, N, K)
    assert torch.equal(y, y2)
    data = bytearray(blob.read_bytes())
    wio.buffer_check(np.frombuffer(bytes(data), np.uint8))
    data[64 + 1000] ^= 0x10
    blob.write_bytes(bytes(data))
    with pytest.raises(wio.WeightsError, match="checksum"):
        wio.load_prepared(blob, dev)
    blob.write_bytes(bytes(data[:2000]))
    with pytest.raises(wio.WeightsError, match="less than its header"):
        wio.load_prepared(blob, dev)
