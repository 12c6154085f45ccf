"""The CPU restatement (oracle/ql_oracle.c) against golden vectors produced by the
reference's own code (tests/golden/make_goldens.py).  Everything here is
bit-exact: integers, bytes, fp16 bit patterns and fp32 outputs alike."""
import numpy as np
import pytest

from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K

FMTS = {"q4k": FMT_Q4_K, "q6k": FMT_Q6_K, "iq3s": FMT_IQ3_S}


def test_f16_conversions(oracle, golden):
    xs = golden["f16_in"]
    sw = np.array([oracle.f32_to_f16_sw(x) for x in xs], np.uint16)
    rne = np.array([oracle.f32_to_f16_rne(x) for x in xs], np.uint16)
    assert np.array_equal(sw, golden["f16_sw"])
    assert np.array_equal(rne, golden["f16_f16c"])
    # the two converters genuinely differ (subnormal range): the fixture must exercise that
    assert (golden["f16_sw"] != golden["f16_f16c"]).any()
    back = np.array([oracle.f16_to_f32(int(h)) for h in golden["h_in"]], np.float32)
    assert np.array_equal(back.view(np.uint32), golden["h_f32"].view(np.uint32))


def test_scale_min_k4(oracle, golden):
    got = np.array([[oracle.scale_min_k4(j, s) for j in range(8)] for s in golden["k4_in"]], np.uint8)
    assert np.array_equal(got, golden["k4_out"])


def test_iq3s_grid_table(golden):
    import re
    from pathlib import Path

    text = (Path(__file__).resolve().parent.parent / "include" / "llaminar_amd" / "iq3s_grid.h").read_text()
    vals = np.array([int(v, 16) for v in re.findall(r"0x([0-9a-f]{8})u", text)], np.uint32)
    assert vals.size == 512
    assert np.array_equal(vals, golden["iq3s_grid"])


def test_q8_1_blocks(oracle, golden):
    x = golden["q8_in"]
    got = np.stack([oracle.quantize_block(r) for r in x])
    # the path the GEMV takes for full blocks is the dispatcher == AVX512 == AVX2
    assert np.array_equal(golden["q8_dispatch"], golden["q8_avx512"])
    assert np.array_equal(golden["q8_avx2"], golden["q8_avx512"])
    assert np.array_equal(got, golden["q8_avx512"])
    # the scalar variant differs only on exact .5 ties and subnormal d: the last two rows are tie rows
    diff_rows = np.where((golden["q8_scalar"] != golden["q8_avx512"]).any(axis=1))[0]
    assert len(diff_rows) > 0


def test_q8_1_tails(oracle, golden):
    for i, v in enumerate(golden["q8_tail_valid"]):
        got = oracle.quantize_block(golden["q8_tail_in"][i], int(v))
        assert np.array_equal(got, golden["q8_tail"][i]), f"tail valid={v}"


@pytest.mark.parametrize("K", [256, 288, 300])
def test_q8_1_rows(oracle, golden, K):
    got = oracle.quantize(golden[f"q8_rows_in_{K}"])
    assert np.array_equal(got, golden[f"q8_rows_{K}"])


@pytest.mark.parametrize("name", list(FMTS))
def test_effective_subblocks(oracle, golden, name):
    fmt = FMTS[name]
    W = golden[f"{name}_w"]
    N, SB, _ = W.shape
    ints = np.zeros((N, SB * 256), np.int8)
    sc = np.zeros((N, SB * 8), np.uint16)
    mn = np.zeros((N, SB * 8), np.uint16)
    for n in range(N):
        for s in range(SB):
            w, a, b = oracle.subblocks(fmt, W[n, s])
            ints[n, 256 * s:256 * (s + 1)] = w
            sc[n, 8 * s:8 * (s + 1)] = a
            mn[n, 8 * s:8 * (s + 1)] = b
    assert np.array_equal(ints, golden[f"{name}_int8"])
    assert np.array_equal(sc, golden[f"{name}_scale_h"])
    assert np.array_equal(mn, golden[f"{name}_min_h"])


def test_q6k_scalar_variant_is_not_the_definition(golden):
    """The reference's scalar Q6_K unpack may differ from the SIMD one by 1 LSB;
    the fixed-point SIMD path is what the packer runs (AVX2 == AVX512)."""
    simd = golden["q6k_int8"][:8].reshape(-1, 256)
    assert np.array_equal(golden["q6k_int8_avx2_variant"], simd)
    d = np.abs(golden["q6k_int8_scalar_variant"].astype(int) - simd.astype(int))
    assert d.max() <= 1


@pytest.mark.parametrize("name", list(FMTS))
@pytest.mark.parametrize("M", [1, 4, 5])
def test_gemm_outputs_and_block_sums(oracle, golden, name, M):
    fmt = FMTS[name]
    W = golden[f"{name}_w"]
    K = W.shape[1] * 256
    C, sums = oracle.gemm(fmt, W, K, golden["act_q8"][:M], want_sums=True)
    assert np.array_equal(sums, golden[f"{name}_bsums"][:M])
    ref = golden[f"{name}_c_avx512_m{M}"]
    assert np.array_equal(golden[f"{name}_c_avx2_m{M}"].view(np.uint32), ref.view(np.uint32))
    assert np.array_equal(C.view(np.uint32), ref.view(np.uint32)), np.abs(C - ref).max()
