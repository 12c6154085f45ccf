"""P2 on the GPU: decode GEMV for Q4_K / Q6_K / IQ3_S through the C-ABI against
the oracle: per-block int32 sums bit-exact, fp32 outputs within 1e-3 (1e-2 IQ3_S)."""
import numpy as np
import pytest

from llaminar_amd import synth
from oracle.binding import FMT_IQ3_S, FMT_Q4_K, FMT_Q6_K
from tests.helpers import FMTS, TOL, rel_err, sync, upload_q8, upload_weights

pytestmark = pytest.mark.gpu

GOLDEN_PATH = __import__("pathlib").Path(__file__).resolve().parent / "golden" / "ql_goldens.npz"
GOLD = {FMT_Q4_K: "q4k", FMT_Q6_K: "q6k", FMT_IQ3_S: "iq3s"}


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_golden_fixture(capi, dev, golden, fmt):
    """The committed reference vectors (edge-case blocks included): sums exact, outputs close."""
    name = GOLD[fmt]
    W = golden[f"{name}_w"]
    N, K = W.shape[0], W.shape[1] * 256
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, golden["act_q8"])
    for M in (1, 4, 5):
        y = capi.gemv(fmt, wd, qd, M, N, K)
        s = capi.gemv_block_sums(fmt, wd, qd, M, N, K, 0, N)
        sync()
        assert np.array_equal(s.cpu().numpy(), golden[f"{name}_bsums"][:M])
        assert rel_err(y.cpu().numpy(), golden[f"{name}_c_avx512_m{M}"]) <= TOL[fmt] * 1e-2


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
@pytest.mark.parametrize("N,K", [(64, 256), (33, 512), (257, 1024), (100, 2048), (1024, 5120), (96, 8192)])
def test_random_shapes(capi, dev, oracle, fmt, N, K):
    W = synth.weights_numpy(fmt, N, K, 17 + N + K)
    q8 = oracle.quantize(synth.activations_numpy(8, K, 3 + N))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    for M in (1, 3, 8):
        y = capi.gemv(fmt, wd, qd, M, N, K)
        s = capi.gemv_block_sums(fmt, wd, qd, M, N, K, 0, N)
        sync()
        C, sums = oracle.gemm(fmt, W, K, q8[:M], want_sums=True)
        assert np.array_equal(s.cpu().numpy(), sums), f"block sums differ M={M}"
        assert rel_err(y.cpu().numpy(), C) <= TOL[fmt] * 1e-2


# config 2: one dense decoder layer's projections (N, K, format)
LAYER = [("q", 8192, 5120, FMT_Q4_K), ("k", 1024, 5120, FMT_Q4_K), ("v", 1024, 5120, FMT_Q6_K),
         ("o", 5120, 8192, FMT_Q4_K), ("gate_up", 25600, 5120, FMT_Q4_K), ("down", 5120, 25600, FMT_Q6_K)]


@pytest.mark.parametrize("name,N,K,fmt", LAYER, ids=[l[0] for l in LAYER])
def test_layer_projections_full_size(capi, dev, oracle, name, N, K, fmt):
    """Full BASELINE shapes, batch 1 and 8: oracle on a window of rows (the CPU
    finishes it in seconds), plus size-independent properties over all rows."""
    import torch

    wd_raw = synth.weights_torch(fmt, N, K, 4242 + N, dev)
    wd = capi.prepare_weights(fmt, wd_raw, N, K)
    x = synth.activations_numpy(8, K, 99)
    q8 = oracle.quantize(x)
    qd = upload_q8(dev, q8)
    y1 = capi.gemv(fmt, wd, qd, 1, N, K)
    y8 = capi.gemv(fmt, wd, qd, 8, N, K)
    y1b = capi.gemv(fmt, wd, qd, 1, N, K)
    y2 = capi.gemv(fmt, wd, qd, 2, N, K)
    row0, nrows = N - 192, 192
    s = capi.gemv_block_sums(fmt, wd, qd, 2, N, K, row0, nrows)
    sync()
    Wh = wd_raw.cpu().numpy()
    C, sums = oracle.gemm(fmt, Wh, K, q8[:8], n0=row0, n1=N, want_sums=True)
    assert np.array_equal(s.cpu().numpy(), sums[:2])
    assert rel_err(y8.cpu().numpy()[:, row0:], C) <= TOL[fmt] * 1e-2
    # determinism: bitwise-stable repeated runs; small-batch rows equal the batch-1 result bit
    # for bit (the reference's decode-equivalent rows); batch 8 may split K into LDS slices,
    # which only re-associates the fp32 sum
    assert torch.equal(y1, y1b)
    assert torch.equal(y2[0], y1[0])
    assert rel_err(y8[0].cpu().numpy(), y1[0].cpu().numpy()) <= 2e-6
    # first window too (different workgroups)
    C0 = oracle.gemm(fmt, Wh, K, q8[:1], n0=0, n1=64)
    assert rel_err(y1.cpu().numpy()[:, :64], C0) <= TOL[fmt] * 1e-2
    assert np.isfinite(y8.cpu().numpy()).all()


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_k_slicing_and_row_tails(capi, dev, oracle, fmt):
    """M=8 with K=25600 needs several LDS slices; N not a multiple of the workgroup's rows."""
    N, K = 45, 25600
    W = synth.weights_numpy(fmt, N, K, 5)
    q8 = oracle.quantize(synth.activations_numpy(8, K, 6))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    y = capi.gemv(fmt, wd, qd, 8, N, K)
    s = capi.gemv_block_sums(fmt, wd, qd, 8, N, K, 3, 40)
    sync()
    C, sums = oracle.gemm(fmt, W, K, q8, n0=3, n1=43, want_sums=True)
    assert np.array_equal(s.cpu().numpy(), sums)
    assert rel_err(y.cpu().numpy()[:, 3:43], C) <= TOL[fmt] * 1e-2


@pytest.mark.parametrize("fmt", list(FMTS.values()), ids=list(FMTS))
def test_tuning_override_does_not_change_results(capi, dev, oracle, fmt):
    import torch

    N, K = 777, 2048
    W = synth.weights_numpy(fmt, N, K, 8)
    q8 = oracle.quantize(synth.activations_numpy(2, K, 9))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    base = capi.gemv(fmt, wd, qd, 2, N, K)
    lib = capi.load()
    try:
        # rows per wavefront only changes which wavefront owns a row: bitwise identical
        for rpw in (1, 3, 8):
            lib.llam_ql_set_gemv_tuning(rpw, 0)
            assert torch.equal(capi.gemv(fmt, wd, qd, 2, N, K), base)
        # the unroll depth does not change the per-lane accumulation order either
        for unroll in (1, 2, 3, 4):
            lib.llam_ql_set_gemv_tuning(0, unroll)
            assert torch.equal(capi.gemv(fmt, wd, qd, 2, N, K), base)
    finally:
        lib.llam_ql_reset_gemv_tuning()
    sync()


def test_fused_projections(capi, dev, oracle):
    """QKV-style fused launch: one quantised input, mixed formats, strided outputs."""
    import torch

    K = 5120
    q8 = oracle.quantize(synth.activations_numpy(2, K, 11))
    qd = upload_q8(dev, q8)
    specs = [(FMT_Q4_K, 512), (FMT_Q4_K, 128), (FMT_Q6_K, 128)]
    out = torch.zeros(2, 768, device=dev)
    projs, hosts, col = [], [], 0
    for i, (fmt, N) in enumerate(specs):
        W = synth.weights_numpy(fmt, N, K, 50 + i)
        hosts.append((fmt, W, col, N))
        projs.append((fmt, upload_weights(capi, dev, fmt, W), out[:, col:col + N]))
        col += N
    capi.gemv_fused(projs, qd, 2, K)
    sync()
    got = out.cpu().numpy()
    for fmt, W, c0, N in hosts:
        assert rel_err(got[:, c0:c0 + N], oracle.gemm(fmt, W, K, q8)) <= TOL[fmt] * 1e-2


@pytest.mark.parametrize("M", [1, 2, 5, 7, 8])
def test_fused_groups_equal_separate_calls(capi, dev, M):
    """Neighbouring projections of one format share a launch; every output must carry the
    bits of its own llam_ql_gemv call.  Groups here: five Q4_K (four + one, the last joined by
    two Q6_K in a two-format launch), two IQ3_S (one launch), a Q4_K again, and a Q4_K of
    4096 rows, which from batch 5 on runs alone on the matrix unit; ragged N, a strided output."""
    import torch

    K = 5120
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(8, K, 23)).to(dev))
    specs = [(FMT_Q4_K, 700), (FMT_Q4_K, 37), (FMT_Q4_K, 1), (FMT_Q4_K, 2048), (FMT_Q4_K, 129),
             (FMT_Q6_K, 300), (FMT_Q6_K, 64), (FMT_IQ3_S, 96), (FMT_IQ3_S, 33), (FMT_Q4_K, 250), (FMT_Q4_K, 4096), (FMT_Q6_K, 40)]
    total = sum(n for _, n in specs)
    out = torch.full((M, total + 5), float("nan"), device=dev)
    projs, singles, col = [], [], 0
    for i, (fmt, N) in enumerate(specs):
        wd = capi.prepare_weights(fmt, synth.weights_torch(fmt, N, K, 900 + i, dev), N, K)
        projs.append((fmt, wd, out[:, col:col + N]))
        singles.append((col, N, capi.gemv(fmt, wd, qd, M, N, K)))
        col += N
    capi.gemv_fused(projs, qd, M, K)
    sync()
    for c0, N, y in singles:
        assert torch.equal(out[:, c0:c0 + N], y), f"projection at column {c0} differs"
    assert torch.isnan(out[:, total:]).all()


@pytest.mark.parametrize("with_plane", [False, True], ids=["prepared", "plane"])
@pytest.mark.parametrize("M", [5, 6, 7, 8])
def test_matrix_unit_matrix_and_quad_lane_group_in_one_launch(capi, dev, M, with_plane):
    """Batches of 5..8: a Q4_K matrix of thousands of rows (the matrix unit) followed by small matrices for the
    quad-lane kernel (Q, then K and V) go out as ONE launch whose first workgroups run the matrix-unit body;
    every output carries the bits of its own llam_ql_gemv call.  Followers: Q4_K and Q6_K, Q6_K only, Q4_K
    only; ragged row counts; a batch plane for the large matrix."""
    import torch

    K = 5120
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(8, K, 123)).to(dev))
    for g, specs in enumerate([[(FMT_Q4_K, 8192), (FMT_Q4_K, 1024), (FMT_Q6_K, 1024)],
                               [(FMT_Q4_K, 4100), (FMT_Q6_K, 333), (FMT_Q6_K, 64)],
                               [(FMT_Q4_K, 5120), (FMT_Q4_K, 77), (FMT_Q4_K, 512), (FMT_Q4_K, 640)]]):
        total = sum(n for _, n in specs)
        out = torch.full((M, total + 3), float("nan"), device=dev)
        projs, singles, col = [], [], 0
        for i, (fmt, N) in enumerate(specs):
            wd = capi.prepare_weights(fmt, synth.weights_torch(fmt, N, K, 1900 + 10 * g + i, dev), N, K)
            plane = capi.build_batch_plane(fmt, wd, N, K) if (with_plane and i == 0) else None
            assert (plane is not None) == (with_plane and i == 0)
            projs.append((fmt, wd, out[:, col:col + N], plane))
            singles.append((col, N, capi.gemv(fmt, wd, qd, M, N, K, plane=plane)))
            col += N
        capi.gemv_fused(projs, qd, M, K)
        sync()
        for c0, N, y in singles:
            assert torch.equal(out[:, c0:c0 + N], y), f"group {g}: projection at column {c0} differs"
        assert torch.isnan(out[:, total:]).all()


@pytest.mark.parametrize("fmt,M,N,K", [(FMT_Q6_K, 8, 5120, 25600), (FMT_Q6_K, 5, 1000, 16384), (FMT_Q6_K, 6, 130, 17408),
                                       (FMT_Q6_K, 2, 5120, 25600), (FMT_Q6_K, 3, 700, 16384),
                                       (FMT_Q4_K, 8, 5120, 25600), (FMT_Q4_K, 8, 4100, 17408)],
                         ids=["q6k-m8", "q6k-m5", "q6k-m6-few-rows", "q6k-m2", "q6k-m3", "q4k-m8", "q4k-m8-ragged"])
def test_long_rows_summed_in_two_halves(capi, dev, oracle, fmt, M, N, K):
    """llam_ql_gemv_plane_split (rows of 64 super-blocks and more, from the batch plane; Q6_K at batches of 2..8, and
    Q4_K matrices of 4096 rows and more at batches of 5..8): the first output is the projection over the first half of every row's
    super-blocks, the second over the second half -- each checked against the oracle on that half of the matrix and
    of the activations -- and their sum is the projection (the one-launch plane kernel to re-association accuracy)."""
    assert capi.gemv_plane_split_supported(fmt, M, N, K)
    W = synth.weights_numpy(fmt, N, K, 4000 + N)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 4100 + K))
    wd, qd = upload_weights(capi, dev, fmt, W), upload_q8(dev, q8)
    plane = capi.build_batch_plane(fmt, wd, N, K)
    lo, hi = capi.gemv_plane_split(fmt, plane, qd, M, N, K)
    y = capi.gemv(fmt, wd, qd, M, N, K, plane=plane)   # (batches of up to 4: the quad-lane kernel)
    sync()
    lo, hi, y = lo.cpu().numpy(), hi.cpu().numpy(), y.cpu().numpy()
    assert rel_err(lo + hi, y) <= 2e-6
    half = K // 2
    rows = slice(0, min(N, 96))
    q8r = q8.reshape(M, K // 32, -1)
    for part, got in ((0, lo), (1, hi)):
        Wp = np.ascontiguousarray(W[rows, part * (half // 256):(part + 1) * (half // 256)])
        qp = np.ascontiguousarray(q8r[:, part * (half // 32):(part + 1) * (half // 32)])
        C = oracle.gemm(fmt, Wp, half, qp)
        assert rel_err(got[:, rows], C) <= TOL[fmt] * 1e-2
    # not served: short rows, batches of 1..4, other formats, an odd number of super-blocks
    assert not capi.gemv_plane_split_supported(fmt, M, N, 8192)
    assert not capi.gemv_plane_split_supported(fmt, 1, N, K)
    assert not capi.gemv_plane_split_supported(FMT_IQ3_S, M, N, K)
    assert not capi.gemv_plane_split_supported(FMT_Q4_K, M, 1024, K)    # too few rows for the matrix unit
    assert not capi.gemv_plane_split_supported(fmt, M, N, 16640)


@pytest.mark.parametrize("M", [1, 3, 8])
def test_fp32_input_equals_quantise_then_gemv(capi, dev, M):
    """llam_ql_gemv_f32 / _fused_f32 / _swiglu_f32 quantise inside the kernel: bits of the
    two-step path, for kernels that quantise themselves (K >= 4096), for the ones
    that need the scratch buffer (short K), with padded input rows, and with tiny
    and zero blocks in the input."""
    import torch

    for K in (5120, 1024):
        ldx = K + 64
        xbuf = torch.from_numpy(synth.activations_numpy(8, ldx, 31 + K)).to(dev)
        xbuf[:, 32:64] = 0.0          # an all-zero block
        xbuf[:, 64:96] *= 1e-12       # below the quantiser's zero threshold
        xbuf[:, 96:128] *= 1e4
        x = xbuf[:M, :K]
        gbuf = torch.from_numpy(synth.activations_numpy(8, ldx, 77 + K)).to(dev) * 3.0
        g = gbuf[:M, :K]
        qd = capi.quantize_q8_1(x.contiguous())
        qa = capi.swiglu_quantize(g.contiguous(), x.contiguous())
        scratch = torch.empty(M * (K // 32) * 36, dtype=torch.uint8, device=dev)
        specs = [(FMT_Q4_K, 300), (FMT_Q4_K, 65), (FMT_Q6_K, 130), (FMT_IQ3_S, 70), (FMT_Q4_K, 40)]
        total = sum(n for _, n in specs)
        out = torch.full((M, total), float("nan"), device=dev)
        projs, col = [], 0
        for i, (fmt, N) in enumerate(specs):
            wd = capi.prepare_weights(fmt, synth.weights_torch(fmt, N, K, 300 + i, dev), N, K)
            projs.append((fmt, wd, out[:, col:col + N]))
            ref = capi.gemv(fmt, wd, qd, M, N, K)
            ref_s = capi.gemv(fmt, wd, qa, M, N, K)
            # with a scratch buffer the library picks the cheaper way; without one the kernel
            # has to quantise for itself, which short rows cannot
            for sc in (scratch, None) if K >= 4096 else (scratch,):
                assert torch.equal(capi.gemv_f32(fmt, wd, x, M, N, K, q8_scratch=sc), ref), (K, fmt, "f32")
                assert torch.equal(capi.gemv_swiglu_f32(fmt, wd, g, x, M, N, K, q8_scratch=sc), ref_s), (K, fmt)
            col += N
        if K >= 4096:
            capi.gemv_fused_f32(projs[:4], x, M, K)  # no scratch: one launch per format group
            col = 0
            for (fmt, N), (_, wd, _) in zip(specs[:4], projs[:4]):
                assert torch.equal(out[:, col:col + N], capi.gemv(fmt, wd, qd, M, N, K)), (K, fmt, "fused/self")
                col += N
            out.fill_(float("nan"))
        capi.gemv_fused_f32(projs, x, M, K, q8_scratch=scratch)
        col = 0
        for (fmt, N), (_, wd, _) in zip(specs, projs):
            assert torch.equal(out[:, col:col + N], capi.gemv(fmt, wd, qd, M, N, K)), (K, fmt, "fused")
            col += N
    sync()


def test_fp32_input_without_scratch_fails_cleanly(capi, dev):
    import torch

    K, N = 1024, 64   # too short for the self-quantising kernel
    wd = capi.prepare_weights(FMT_Q4_K, synth.weights_torch(FMT_Q4_K, N, K, 1, dev), N, K)
    x = torch.zeros(1, K, device=dev)
    with pytest.raises(capi.QLError, match="d_q8_scratch"):
        capi.gemv_f32(FMT_Q4_K, wd, x, 1, N, K)
    with pytest.raises(capi.QLError, match="aligned"):
        capi.gemv_f32(FMT_Q4_K, wd, torch.zeros(1, K + 1, device=dev)[:, 1:], 1, N, K)


def test_q4k_prepare_is_identity(capi, dev):
    import torch

    raw = synth.weights_torch(FMT_Q4_K, 16, 512, 1, dev)
    assert torch.equal(capi.prepare_weights(FMT_Q4_K, raw, 16, 512), raw)


@pytest.mark.parametrize("fmt", [FMT_Q6_K, FMT_IQ3_S], ids=["q6_k", "iq3_s"])
def test_prepare_moves_every_byte(capi, dev, oracle, fmt):
    """Plane layout: a permutation of the input bytes (plus zero padding for IQ3_S).  Q6_K also
    gets a plane of per-block records, the 8.8 factors of the two sub-scales of a block and its
    scale, which must be the closed form of the requantisation the reference performs."""
    N, K = 5, 768
    W = synth.weights_numpy(fmt, N, K, 2)
    wd = upload_weights(capi, dev, fmt, W)
    sync()
    P = wd.cpu().numpy()
    T = N * (K // 256)
    B = W.reshape(T, -1)
    if fmt == FMT_Q6_K:
        assert np.array_equal(P[:T * 128].reshape(T, 128), B[:, :128])
        assert np.array_equal(P[T * 128:T * 192].reshape(T, 64), B[:, 128:192])
        assert np.array_equal(P[T * 192:T * 208].reshape(T, 16), B[:, 192:208])
        assert np.array_equal(P[T * 208:T * 210].reshape(T, 2), B[:, 208:210])
        off = (T * 210 + 15) & ~15
        assert P.size == off + T * 32
        rec = P[off:].view(np.uint32).reshape(T, 8)
        sc = B[:, 192:208].view(np.int8).astype(int)

        def rne_div(a, b):  # round-half-even of a/b for integers, b > 0
            qq, rr = divmod(a, b)
            return qq + (1 if (2 * rr > b or (2 * rr == b and (qq & 1))) else 0)

        for t in range(T):
            _, sc_h, _ = oracle.subblocks(fmt, B[t])
            for j in range(8):
                c = int(rec[t, (j & 4) | ((j & 1) << 1) | ((j >> 1) & 1)])
                s0, s1 = sc[t, 2 * j], sc[t, 2 * j + 1]
                msc = max(abs(s0), abs(s1))
                assert (c >> 16) == int(sc_h[j]), (t, j)
                if msc == 0:
                    assert (c & 0xFFFF) == 0
                    continue
                big1 = abs(s1) > abs(s0)
                small, big = (s0, s1) if big1 else (s1, s0)
                fs = c & 0xFFF
                fs -= 4096 if fs & 0x800 else 0
                assert fs == rne_div(small * 1016, msc) and bool(c & (1 << 12)) == big1
                assert (c >> 13) & 3 == (3 if big < 0 else 1)   # the larger sub-scale's sign: -1 or +1 in two bits
    else:
        assert np.array_equal(P[:T * 64].reshape(T, 64), B[:, 2:66])
        assert np.array_equal(P[T * 64:T * 96].reshape(T, 32), B[:, 74:106])
        meta = P[T * 96:].reshape(T, 16)
        assert np.array_equal(meta[:, 0:8], B[:, 66:74])
        assert np.array_equal(meta[:, 8:12], B[:, 106:110])
        assert np.array_equal(meta[:, 12:14], B[:, 0:2])
        # the two spare bytes carry the hints: two bits per 32-element block, 7 - k for the block's
        # largest codebook magnitude 2k+1 when k >= 5 and the block's scale is an ordinary fp16
        # number (normal, below the clamp), else 3
        grid = np.load(GOLDEN_PATH, allow_pickle=False)["iq3s_grid"].astype(np.uint32).reshape(-1)[:512]
        kmax = np.max(np.stack([(grid >> (8 * b)) & 0xFF for b in range(4)]), axis=0) >> 1
        hints = meta[:, 14].astype(np.uint32) | (meta[:, 15].astype(np.uint32) << 8)
        for t in range(T):
            qs, qh = B[t, 2:66].astype(np.uint32), B[t, 66:74].astype(np.uint32)
            d = np.float32(B[t, 0:2].view(np.float16)[0])
            for j in range(8):
                idx = qs[8 * j:8 * j + 8] | (((qh[j] >> np.arange(8)) & 1) << 8)
                k = int(kmax[idx].max())
                nib = (int(B[t, 106 + (j >> 1)]) >> (4 * (j & 1))) & 15
                with np.errstate(all="ignore"):
                    scale = np.float32(d * np.float32((2 * k + 1) * (2 * nib + 1))) / np.float32(127.0)
                regular = bool(scale >= np.float32(6.103515625e-05)) and bool(scale < np.float32(65504.0))
                assert (int(hints[t]) >> (2 * j)) & 3 == (7 - k if k >= 5 and regular else 3), (t, j)


def test_error_paths(capi, dev):
    import torch

    lib = capi.load()
    w = torch.zeros(4096, dtype=torch.uint8, device=dev)
    y = torch.zeros(64, device=dev)
    assert not lib.llam_ql_gemv(FMT_Q4_K, w.data_ptr(), w.data_ptr(), y.data_ptr(), 0, 4, 256, 4, 0, None)
    assert not lib.llam_ql_gemv(FMT_Q4_K, w.data_ptr(), w.data_ptr(), None, 1, 4, 256, 4, 0, None)
    assert not lib.llam_ql_gemv_block_sums(FMT_Q4_K, w.data_ptr(), None, w.data_ptr(), y.data_ptr(), 1, 4, 256, 2, 3, 0, None)
    assert "row window" in capi.last_error()


@pytest.mark.parametrize("N,K", [(1, 4096), (37, 4096), (250, 4352), (129, 5120), (64, 8192), (19, 25600)])
def test_q4k_long_rows_all_batches(capi, dev, oracle, N, K):
    """Rows of 16 and more super-blocks take the kernel that walks a wavefront's rows as one
    run: row ends inside a step (K/256 not a multiple of 16), ragged last steps, wavefronts
    without rows, every batch size; up to four rows (the decode-equivalent verifier rows of
    the reference) a batch row equals the single-row result bit for bit.  Batches of 5..8 run
    on the matrix unit, which adds a row's blocks in ascending order: same values up to the
    association of the fp32 sum, and independent of what else is in the batch."""
    import torch

    fmt = FMT_Q4_K
    W = synth.weights_numpy(fmt, N, K, 31 + N)
    q8 = oracle.quantize(synth.activations_numpy(8, K, 7 + N))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    C = oracle.gemm(fmt, W, K, q8)
    y1 = [capi.gemv(fmt, wd, upload_q8(dev, q8[m:m + 1]), 1, N, K) for m in range(8)]
    for M in range(1, 9):
        y = capi.gemv(fmt, wd, qd, M, N, K)
        sync()
        assert rel_err(y.cpu().numpy(), C[:M]) <= TOL[fmt] * 1e-2, M
        for m in range(M):
            if M <= 4:
                assert torch.equal(y[m], y1[m][0]), (M, m)
            else:
                assert rel_err(y[m].cpu().numpy(), y1[m][0].cpu().numpy()) <= TOL[fmt] * 1e-2, (M, m)
        if M == 5:
            y5 = y.clone()
        if M > 5:
            assert torch.equal(y[:5], y5), M   # a row does not depend on the batch it rides in
    lib = capi.load()
    try:
        # another row partition moves rows to other lanes: same values up to summation order
        for rpw in (1, 2, 5, 64):
            lib.llam_ql_set_gemv_tuning(rpw, 0)
            y = capi.gemv(fmt, wd, qd, 3, N, K)
            sync()
            assert rel_err(y.cpu().numpy(), C[:3]) <= TOL[fmt] * 1e-2, rpw
    finally:
        lib.llam_ql_reset_gemv_tuning()


@pytest.mark.parametrize("fmt", [FMT_Q4_K, FMT_Q6_K, FMT_IQ3_S], ids=["q4_k", "q6_k", "iq3_s"])
@pytest.mark.parametrize("N,K", [(100, 512), (33, 1024), (300, 2048), (257, 3840), (64, 4096), (40, 25600)],
                         ids=["generic_k512", "generic_k1024", "chunked_k2048", "chunked_k3840", "quad_k4096",
                              "quad_k25600"])
def test_rows_of_small_batches_equal_the_single_row_call(capi, dev, fmt, N, K):
    """What the operator's decode-equivalent verifier rows rely on: for up to four activation
    rows the launcher reports decode_equivalent (same kernel, row partition and K slices as the
    single-row call) and every row of the batch carries the bits of its own single-row call --
    on the generic, the chunked and the quad-lane kernel, all formats, K = 25600 included."""
    import torch

    W = synth.weights_torch(fmt, N, K, 400 + N, dev)
    wd = capi.prepare_weights(fmt, W, N, K)
    qd = capi.quantize_q8_1(torch.from_numpy(synth.activations_numpy(4, K, 401 + K)).to(dev))
    rb = (K // 32) * 36
    one = [capi.gemv(fmt, wd, qd[m * rb:(m + 1) * rb], 1, N, K) for m in range(4)]
    for M in (2, 3, 4):
        plan = capi.gemv_describe(fmt, M, N, K)
        assert plan.decode_equivalent == 1, (M, plan.kernel, plan.slice_sb)
        y = capi.gemv(fmt, wd, qd, M, N, K)
        sync()
        for m in range(M):
            assert torch.equal(y[m], one[m][0]), (M, m)
    # five and more rows of a large Q4_K matrix go to the matrix unit, which adds blocks in another order
    if fmt == FMT_Q4_K:
        assert capi.gemv_describe(fmt, 8, 8192, 5120).decode_equivalent == 0


@pytest.mark.parametrize("N,K", [(19, 25600), (70, 17408), (33, 30720)])
def test_q6k_long_rows_large_batches(capi, dev, oracle, N, K):
    """Q6_K rows too long for eight activation rows in LDS: batches the quad-lane kernel would
    split run on the matrix unit in one pass, the row walked in chunks staged by producer
    wavefronts (K = 17408 and 30720: the last chunk is short; N = 19: one partial tile).  Same
    block sums, blocks added in ascending order per wavefront: values agree with the oracle and
    with the single-row result up to the association of the fp32 sum, a row does not depend on
    the batch it rides in, and fp32 input quantised inside the kernel gives the same bits."""
    import torch

    fmt = FMT_Q6_K
    W = synth.weights_numpy(fmt, N, K, 91 + N)
    x = synth.activations_numpy(8, K, 17 + N)
    q8 = oracle.quantize(x)
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    xd = torch.from_numpy(x).to(dev)
    C = oracle.gemm(fmt, W, K, q8)
    y1 = [capi.gemv(fmt, wd, upload_q8(dev, q8[m:m + 1]), 1, N, K) for m in range(8)]
    ys = {}
    for M in (4, 5, 7, 8):
        y = capi.gemv(fmt, wd, qd, M, N, K)
        sync()
        ys[M] = y
        assert rel_err(y.cpu().numpy(), C[:M]) <= TOL[fmt] * 1e-2, M
        for m in range(M):
            assert rel_err(y[m].cpu().numpy(), y1[m][0].cpu().numpy()) <= TOL[fmt] * 1e-2, (M, m)
        assert torch.equal(capi.gemv(fmt, wd, qd, M, N, K), y), M  # bitwise repeatable
        assert torch.equal(capi.gemv_f32(fmt, wd, xd[:M], M, N, K), y), (M, "fp32 input, no scratch")
    if K >= 25600:  # seven rows of a shorter row still fit the quad-lane kernel's LDS
        assert torch.equal(ys[8][:7], ys[7])
    sync()


def _q6k_one_live_block_per_row(pairs, K, seed):
    """Q6_K rows whose sub-scales are zero except for ONE block per row, which carries the
    given pair: every other block contributes an exact zero, so a row's output is one
    multiply-add and its bits do not depend on how a kernel orders the blocks."""
    rng = np.random.default_rng(seed)
    N, SB = len(pairs), K // 256
    W = rng.integers(0, 256, size=(N, SB, 210), dtype=np.uint8)
    W[:, :, 192:208] = 0
    d = rng.uniform(0.0005, 0.05, size=(N, SB)).astype(np.float16)
    d[::97] = np.float16(3e-6)   # block scales below the fp16 normal range (truncating conversion)
    W[:, :, 208:210] = d.view(np.uint8).reshape(N, SB, 2)
    sb = rng.integers(0, SB, N)
    j = rng.integers(0, 8, N)
    sc = W[:, :, 192:208].view(np.int8)
    sc[np.arange(N), sb, 2 * j] = pairs[:, 0]
    sc[np.arange(N), sb, 2 * j + 1] = pairs[:, 1]
    return W


def test_q6k_every_pair_of_subscales_bit_exact(capi, dev, oracle):
    """All 65536 (sub-scale, sub-scale) pairs of a Q6_K block, one live block per row, through
    the quad-lane kernel (K = 4096): the 8.8 factors (ties and signs included), the block scale
    and its fp16 rounding must be the reference's exactly, so every output bit matches."""
    import torch

    v = np.arange(-128, 128, dtype=np.int8)
    pairs = np.stack(np.meshgrid(v, v, indexing="ij"), -1).reshape(-1, 2)
    K = 4096
    W = _q6k_one_live_block_per_row(pairs, K, 5)
    q8 = oracle.quantize(synth.activations_numpy(2, K, 6))
    wd = upload_weights(capi, dev, FMT_Q6_K, W)
    y = capi.gemv(FMT_Q6_K, wd, upload_q8(dev, q8), 2, len(pairs), K)
    sync()
    C = oracle.gemm(FMT_Q6_K, W, K, q8)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), C.view(np.uint32))
    assert np.count_nonzero(C) > 0.9 * C.size


def test_q6k_subscale_pairs_on_the_matrix_unit_bit_exact(capi, dev, oracle):
    """The same construction on rows long enough for the matrix-unit kernel at batch 8
    (K = 16640: 65 super-blocks), 4096 pairs that include every tie of the factor rounding."""
    rng = np.random.default_rng(8)
    v = np.arange(-128, 128)
    a, b = np.meshgrid(v, v, indexing="ij")
    m = np.maximum(np.abs(a), np.abs(b))
    s = np.where(np.abs(a) >= np.abs(b), b, a)
    tie = (m > 0) & ((2 * s * 1016) % np.maximum(m, 1) == 0) & (((2 * s * 1016) // np.maximum(m, 1)) % 2 != 0)
    ties = np.stack([a[tie], b[tie]], -1)
    rest = rng.integers(-128, 128, size=(4096 - min(len(ties), 2048), 2))
    pairs = np.concatenate([ties[:2048], rest]).astype(np.int8)
    K = 16640
    W = _q6k_one_live_block_per_row(pairs, K, 9)
    q8 = oracle.quantize(synth.activations_numpy(8, K, 10))
    wd = upload_weights(capi, dev, FMT_Q6_K, W)
    y = capi.gemv(FMT_Q6_K, wd, upload_q8(dev, q8), 8, len(pairs), K)
    sync()
    C = oracle.gemm(FMT_Q6_K, W, K, q8)
    assert np.array_equal(y.cpu().numpy().view(np.uint32), C.view(np.uint32))


# ---- the block sums come from the kernel that serves the shape -------------------------------
# llam_ql_gemv_block_sums executes llam_ql_gemv's launch plan with the chosen kernel's block-sum
# variant, so each case below pins the integer pipeline of one production kernel; the expected
# kernel is asserted through llam_ql_gemv_describe so that a change of the dispatch shows up here.
def _production_cases():
    from llaminar_amd.capi import KERNEL_CHUNKED as CH, KERNEL_GENERIC as GE, KERNEL_MFMA as MF, KERNEL_QUAD as QU

    return [
        ("q4k_quad_m1", FMT_Q4_K, 777, 5120, 1, QU),
        ("q4k_quad_m4_row_ends_inside_steps", FMT_Q4_K, 1030, 4352, 4, QU),
        ("q4k_quad_batch_split_m5", FMT_Q4_K, 100, 25600, 5, QU),
        ("q6k_quad_m1", FMT_Q6_K, 1024, 5120, 1, QU),
        ("q6k_quad_m8", FMT_Q6_K, 700, 5120, 8, QU),
        ("q6k_quad_m4_long_rows", FMT_Q6_K, 64, 25600, 4, QU),
        ("q4k_mfma_m8", FMT_Q4_K, 4100, 5120, 8, MF),
        ("q4k_mfma_m5", FMT_Q4_K, 4096, 4096, 5, MF),
        ("q4k_mfma_m6_chunked_row", FMT_Q4_K, 4100, 25600, 6, MF),
        ("q4k_mfma_m8_short_last_chunk", FMT_Q4_K, 4096, 17408, 8, MF),
        ("q4k_mfma_m8_chunked_row_that_would_fit", FMT_Q4_K, 4100, 12800, 8, MF),
        ("q4k_quad_m5_long_rows_in_one_launch", FMT_Q4_K, 4100, 25600, 5, QU),
        ("q6k_mfma_m8_chunked_row", FMT_Q6_K, 200, 25600, 8, MF),
        ("q6k_mfma_m8_short_last_chunk", FMT_Q6_K, 70, 17408, 8, MF),
        ("iq3s_quad_m1", FMT_IQ3_S, 1000, 5120, 1, QU),
        ("iq3s_quad_m8", FMT_IQ3_S, 300, 5120, 8, QU),
        ("iq3s_quad_m4_long_rows", FMT_IQ3_S, 50, 25600, 4, QU),
        ("iq3s_quad_m3_row_ends_inside_steps", FMT_IQ3_S, 515, 4352, 3, QU),
        ("iq3s_chunked_m1", FMT_IQ3_S, 1000, 3072, 1, CH),
        ("iq3s_chunked_m8", FMT_IQ3_S, 300, 2048, 8, CH),
        ("q4k_chunked_m3", FMT_Q4_K, 500, 2048, 3, CH),
        ("q6k_chunked_m6_batch_split", FMT_Q6_K, 90, 3072, 6, CH),
        ("q6k_generic_m2", FMT_Q6_K, 100, 512, 2, GE),
        ("iq3s_generic_m1", FMT_IQ3_S, 33, 1024, 1, GE),
    ]


@pytest.mark.parametrize("case", _production_cases(), ids=[c[0] for c in _production_cases()])
def test_block_sums_of_the_production_kernels(capi, dev, oracle, case):
    name, fmt, N, K, M, kernel = case
    print(f"[block sums] {name}: fmt {fmt} N={N} K={K} M={M}", flush=True)
    plan = capi.gemv_describe(fmt, M, N, K)
    assert plan.kernel == kernel, f"{name}: the dispatcher now picks kernel {plan.kernel}"
    W = synth.weights_numpy(fmt, N, K, 1000 + N + M)
    q8 = oracle.quantize(synth.activations_numpy(M, K, 2000 + K))
    wd = upload_weights(capi, dev, fmt, W)
    qd = upload_q8(dev, q8)
    y = capi.gemv(fmt, wd, qd, M, N, K)
    windows = [(0, min(N, 40)), (max(0, N - 33), N)] + ([(N // 2 - 7, N // 2 + 30)] if N > 200 else [])
    for r0, r1 in windows:
        s = capi.gemv_block_sums(fmt, wd, qd, M, N, K, r0, r1 - r0)
        sync()
        C, sums = oracle.gemm(fmt, W, K, q8, n0=r0, n1=r1, want_sums=True)
        assert np.array_equal(s.cpu().numpy(), sums), f"{name}: block sums of rows [{r0},{r1}) differ"
        assert rel_err(y.cpu().numpy()[:, r0:r1], C) <= TOL[fmt] * 1e-2


def test_config1_q4k_5120x5120(capi, dev, oracle):
    """BASELINE config 1: one Q4_K GEMV, N = K = 5120, batch 1.  Block sums of the quad-lane
    kernel on row windows, fp32 over ALL rows against the oracle, bitwise repeatability, and the
    fp32-input entry point (quantiser inside the kernel) with the same bits."""
    import torch

    fmt, N, K = FMT_Q4_K, 5120, 5120
    assert capi.gemv_describe(fmt, 1, N, K).kernel == capi.KERNEL_QUAD
    W = synth.weights_numpy(fmt, N, K, 20240)
    x = synth.activations_numpy(1, K, 20241)
    q8 = oracle.quantize(x)
    wd = upload_weights(capi, dev, fmt, W)
    xd = torch.from_numpy(x).to(dev)
    qd = capi.quantize_q8_1(xd)
    sync()
    assert np.array_equal(qd.cpu().numpy().reshape(q8.shape), q8), "Q8_1 bytes differ from the oracle"
    y = capi.gemv(fmt, wd, qd, 1, N, K)
    y_again = capi.gemv(fmt, wd, qd, 1, N, K)
    y_f32 = capi.gemv_f32(fmt, wd, xd, 1, N, K)
    sync()
    C = oracle.gemm(fmt, W, K, q8)
    assert rel_err(y.cpu().numpy(), C) <= TOL[fmt] * 1e-2
    assert torch.equal(y, y_again) and torch.equal(y, y_f32)
    for r0 in (0, 2537, N - 64):
        s = capi.gemv_block_sums(fmt, wd, qd, 1, N, K, r0, 64)
        sync()
        _, sums = oracle.gemm(fmt, W, K, q8, n0=r0, n1=r0 + 64, want_sums=True)
        assert np.array_equal(s.cpu().numpy(), sums), f"rows from {r0}"
    # doubling the activations doubles d of every Q8_1 block and leaves the quants alone:
    # the output doubles exactly (a size-independent check of the whole row range)
    y2 = capi.gemv_f32(fmt, wd, 2.0 * xd, 1, N, K)
    sync()
    assert torch.equal(y2, 2.0 * y)


@pytest.mark.parametrize("M", [1, 8])
def test_lm_head_shape_q6k_152064x5120(capi, dev, oracle, M):
    """The lm_head of config 5 at full size: oracle on row windows at both ends and in the
    middle (block sums bit-exact, fp32 close), properties over all 152064 rows."""
    import torch

    fmt, N, K = FMT_Q6_K, 152064, 5120
    raw = synth.weights_torch(fmt, N, K, 777, dev)
    wd = capi.prepare_weights(fmt, raw, N, K)
    x = synth.activations_numpy(8, K, 778)
    q8 = oracle.quantize(x)
    qd = upload_q8(dev, q8[:M])
    y = capi.gemv(fmt, wd, qd, M, N, K)
    y_again = capi.gemv(fmt, wd, qd, M, N, K)
    sync()
    assert torch.equal(y, y_again)
    assert bool(torch.isfinite(y).all())
    bb = 210 * (K // 256)
    for r0 in (0, 76000, N - 48):
        Wh = raw[r0 * bb:(r0 + 48) * bb].cpu().numpy().reshape(48, K // 256, 210)
        s = capi.gemv_block_sums(fmt, wd, qd, M, N, K, r0, 48)
        sync()
        C, sums = oracle.gemm(fmt, Wh, K, q8[:M], want_sums=True)
        assert np.array_equal(s.cpu().numpy(), sums), f"rows from {r0}"
        assert rel_err(y.cpu().numpy()[:, r0:r0 + 48], C) <= TOL[fmt] * 1e-2
    if M == 8:
        # a batch row has the bits of its single-row call (Q6_K rows of this length stay on
        # the quad-lane kernel at every batch size)
        assert capi.gemv_describe(fmt, 8, N, K).decode_equivalent == 1
        y1 = capi.gemv(fmt, wd, upload_q8(dev, q8[5:6]), 1, N, K)
        sync()
        assert torch.equal(y[5], y1[0])


# (formats, Ns) of the projections, K, M: the decoder's two uses (Q and K in Q4_K with V in Q6_K; gate and up),
# a format with decode tables, matrices whose workgroups are smaller than the norm's 512 threads, rows too long
# for the registers
_NORM_CASES = [
    ((FMT_Q4_K, FMT_Q4_K, FMT_Q6_K), (8192, 1024, 1024), 5120, 1),
    ((FMT_Q4_K, FMT_Q4_K), (25600, 25600), 5120, 1),
    ((FMT_Q4_K, FMT_Q4_K, FMT_Q6_K), (2048, 512, 512), 4096, 1),
    ((FMT_Q4_K, FMT_Q4_K), (6400, 6400), 8192, 1),
    ((FMT_IQ3_S,), (4096,), 5120, 1),
    ((FMT_Q6_K,), (384,), 8192, 1),
    ((FMT_Q4_K,), (3000,), 12800, 1),
    # rows of 64 super-blocks and more (plain launches take two steps per load chunk there; the norm source one)
    ((FMT_Q6_K,), (640,), 16384, 1),
    ((FMT_Q4_K, FMT_Q4_K), (768, 512), 20480, 1),
]


@pytest.mark.parametrize("fmts,Ns,K,M", _NORM_CASES)
def test_norm_inside_the_projections_equals_norm_then_projections(capi, dev, fmts, Ns, K, M):
    """llam_ql_gemv_fused_rmsnorm against llam_dec_rmsnorm_q8_1 followed by llam_ql_gemv_fused: the same bits in
    every output and in the updated residual, with and without a delta, whatever the workgroup size of the launch."""
    import torch

    rng = np.random.default_rng(K + M + sum(Ns))
    x = torch.from_numpy((rng.standard_normal((M, K)) * rng.uniform(0.05, 20, (M, 1))).astype(np.float32)).to(dev)
    d = torch.from_numpy(rng.standard_normal((M, K)).astype(np.float32)).to(dev)
    g = torch.from_numpy(rng.uniform(0.2, 2.0, K).astype(np.float32)).to(dev)
    ws = [capi.prepare_weights(f, synth.weights_torch(f, N, K, 300 + i, dev), N, K) for i, (f, N) in enumerate(zip(fmts, Ns))]
    for delta in (None, d):
        sep = [torch.full((M, N), 3.0, device=dev) for N in Ns]
        fus = [torch.full((M, N), 5.0, device=dev) for N in Ns]
        projs_sep = [(f, w, o) for f, w, o in zip(fmts, ws, sep)]
        projs_fus = [(f, w, o) for f, w, o in zip(fmts, ws, fus)]
        assert capi.gemv_fused_rmsnorm_supported(projs_fus, M, K)
        x_sep = x.clone()
        _, q8 = capi.rmsnorm_q8_1(x_sep, g, 1e-6, delta=delta, want_y=False)
        capi.gemv_fused(projs_sep, q8, M, K)
        x_in = x.clone()
        x_out = torch.full((M, K), 9.0, device=dev)
        capi.gemv_fused_rmsnorm(projs_fus, x_in, delta, g, 1e-6, x_out if delta is not None else None, M, K)
        sync()
        for a, b in zip(sep, fus):
            assert torch.equal(a, b)
        assert torch.equal(x_in, x)                      # the input rows are read only
        if delta is not None:
            assert torch.equal(x_out, x_sep)             # x + delta, as the stand-alone norm leaves it
        else:
            assert (x_out == 9.0).all()                  # no delta: nothing to store


def test_norm_inside_the_projections_is_refused_where_no_kernel_fuses_it(capi, dev):
    import torch

    K = 5120
    w = capi.prepare_weights(FMT_Q4_K, synth.weights_torch(FMT_Q4_K, 8192, K, 1, dev), 8192, K)
    x = torch.randn(8, K, device=dev)
    g = torch.ones(K, device=dev)
    out = torch.empty(8, 8192, device=dev)
    for M in (2, 8):                                                               # one row only
        assert not capi.gemv_fused_rmsnorm_supported([(FMT_Q4_K, w, out[:M])], M, K)
        with pytest.raises(capi.QLError):
            capi.gemv_fused_rmsnorm([(FMT_Q4_K, w, out[:M])], x[:M], None, g, 1e-6, None, M, K)
    small = torch.empty(1, 64, device=dev)
    w2 = capi.prepare_weights(FMT_Q4_K, synth.weights_torch(FMT_Q4_K, 64, 1024, 2, dev), 64, 1024)
    assert not capi.gemv_fused_rmsnorm_supported([(FMT_Q4_K, w2, small)], 1, 1024)  # rows too short for the quad-lane kernel
    with pytest.raises(capi.QLError):                                              # x + delta must not land on x
        capi.gemv_fused_rmsnorm([(FMT_Q4_K, w, out[:1])], x[:1], x[1:2], g, 1e-6, x[:1], 1, K)


@pytest.mark.parametrize("fmt,N,K,M", [(FMT_Q4_K, 5120, 8192, 1), (FMT_Q6_K, 5120, 25600, 1), (FMT_IQ3_S, 4096, 5120, 1),
                                       (FMT_Q4_K, 5120, 8192, 2), (FMT_Q6_K, 1000, 4096, 1)])
def test_accumulating_launch_equals_gemv_then_add(capi, dev, fmt, N, K, M):
    """llam_ql_gemv_accumulate: y += W a inside the launch has the bits of llam_ql_gemv followed by one fp32 add."""
    import torch

    assert capi.gemv_accumulate_supported(fmt, M, N, K)
    w = capi.prepare_weights(fmt, synth.weights_torch(fmt, N, K, 77, dev), N, K)
    x = torch.randn(M, K, device=dev, generator=torch.Generator(device=dev).manual_seed(N + K))
    q8 = capi.quantize_q8_1(x)
    y0 = torch.randn(M, N + 8, device=dev)                 # a residual with a row stride of its own
    delta = capi.gemv(fmt, w, q8, M, N, K)
    got = y0.clone()
    capi.gemv_accumulate(fmt, w, q8, M, N, K, got[:, :N])
    sync()
    assert torch.equal(got[:, :N], y0[:, :N] + delta)
    assert torch.equal(got[:, N:], y0[:, N:])


def test_accumulating_launch_is_refused_where_the_kernel_cannot(capi, dev):
    import torch

    # the lm_head shape: a wavefront walks more rows than one flush of the ring holds; batch 8: the matrix unit;
    # short rows: not the quad-lane kernel
    for fmt, M, N, K in ((FMT_Q6_K, 1, 152064, 5120), (FMT_Q4_K, 8, 25600, 5120), (FMT_Q4_K, 1, 512, 1024)):
        assert not capi.gemv_accumulate_supported(fmt, M, N, K)
    N, K = 512, 1024
    w = capi.prepare_weights(FMT_Q4_K, synth.weights_torch(FMT_Q4_K, N, K, 5, dev), N, K)
    q8 = capi.quantize_q8_1(torch.randn(1, K, device=dev))
    with pytest.raises(capi.QLError):
        capi.gemv_accumulate(FMT_Q4_K, w, q8, 1, N, K, torch.zeros(1, N, device=dev))


def test_read_probe_runs_and_checks_its_arguments(capi, dev):
    """The read-only probes behind bench.py --workload read-order (tests/probe, not part of the product library):
    every pattern runs on a small buffer (they read inside N * K/256 * 144 bytes and write nothing), bad arguments
    are refused."""
    import torch

    from tests.probe import binding as probe

    lib = probe.load()
    N, K = 96, 4096
    buf = torch.randint(0, 256, (N * (K // 256) * 144 + 64,), dtype=torch.uint8, device=dev)
    guard = buf[-64:].clone()
    sink = torch.zeros(1, dtype=torch.int32, device=dev)
    for pattern, rpw, depth, wgs in ((0, 3, 2, 0), (1, 3, 1, 0), (1, 5, 4, 0), (2, 0, 3, 4), (3, 0, 6, 4), (3, 0, 9, 2), (4, 3, 3, 0),
                                     (5, 5, 2, 0)):
        assert lib.llam_probe_read(buf.data_ptr(), N, K, pattern, rpw, 4, depth, wgs, sink.data_ptr(), 0, None), capi.last_error()
    sync()
    assert torch.equal(buf[-64:], guard) and int(sink[0]) in (0, 1)
    for args in ((buf.data_ptr(), N, K, 7, 3, 4, 2, 0), (buf.data_ptr(), N, K, 0, 3, 4, 5, 0), (buf.data_ptr(), N, 1024, 0, 3, 4, 2, 0),
                 (buf.data_ptr(), N, K, 2, 0, 4, 3, 0), (0, N, K, 0, 3, 4, 2, 0), (buf.data_ptr(), N, K, 0, 3, 17, 2, 0)):
        assert not lib.llam_probe_read(*args, sink.data_ptr(), 0, None)


@pytest.mark.parametrize("fmt,N,K", [(FMT_Q4_K, 8192 + 40, 5120), (FMT_Q6_K, 1000, 25600)])
def test_batch_tile_heights_agree(capi, dev, oracle, fmt, N, K):
    """The matrix-unit kernels of batches 5..8 with tiles of 16..32 weight rows (the sweep override of tests/probe):
    every height against the CPU restatement on a row window, and the exact block sums of the kernel that serves
    the shape unchanged by the height (rows that do not fill the last tile included), without and with the
    matrix's batch plane."""
    import torch

    from tests.probe import binding as probe

    M = 8
    plib = probe.load()
    assert capi.gemv_describe(fmt, M, N, K).kernel == 3
    W = synth.weights_numpy(fmt, N, K, 31)
    w = capi.prepare_weights(fmt, torch.from_numpy(W.reshape(-1)).to(dev), N, K)
    plane = capi.build_batch_plane(fmt, w, N, K)
    assert plane is not None
    x = synth.activations_numpy(M, K, 6)
    q8 = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
    rows = slice(N - 70, N)
    exp, exp_sums = oracle.gemm(fmt, W[rows], K, oracle.quantize(x), want_sums=True)
    try:
        for tr in (0, 32, 27, 20, 16):
            plib.llam_probe_set_batch_tile_rows(tr)
            for pl in (None, plane):
                y = capi.gemv(fmt, w, q8, M, N, K, plane=pl)
                s = capi.gemv_block_sums(fmt, w, q8, M, N, K, N - 70, 70, plane=pl)
                sync()
                assert rel_err(y.cpu().numpy()[:, rows], exp) <= TOL[fmt] * 1e-2, (tr, pl is not None)
                assert np.array_equal(s.cpu().numpy(), exp_sums), (tr, pl is not None)   # bit-exact whatever the tile height
    finally:
        plib.llam_probe_set_batch_tile_rows(0)


# ---- batch planes (llam_ql_build_batch_plane; handed to the launches that may use them) ------------------------
def _plane_rows(plane: np.ndarray, N: int, nsb: int):
    """The plane's int8 weights as [rows][nsb][256] and fp16 scale bits as [rows][nsb][8], rows = 4 ceil(N / 4):
    group g = row / 4 keeps, per super-block, eight 128-byte lines (block j: its four rows' 32 bytes in turn), and
    in a second plane the rows' eight scales."""
    G = (N + 3) // 4
    w = plane[:G * nsb * 1024].reshape(G, nsb, 8, 4, 32).transpose(0, 3, 1, 2, 4).reshape(G * 4, nsb, 256)
    s = plane[G * nsb * 1024:].view(np.uint16).reshape(G, nsb, 4, 8).transpose(0, 2, 1, 3).reshape(G * 4, nsb, 8)
    return w.view(np.int8), s


@pytest.mark.parametrize("N,K", [(37, 2048), (8, 5120), (130, 25600)])
def test_q6k_batch_plane_holds_the_requantised_weights(capi, dev, oracle, N, K):
    """The plane is the reference's packed Q6_K matrix: every int8 weight and every fp16 block scale equals the CPU
    restatement's (subblocks), rows that pad the last group of four are zero."""
    import torch

    nsb = K // 256
    W = synth.weights_numpy(FMT_Q6_K, N, K, 5 + N)
    w = capi.prepare_weights(FMT_Q6_K, torch.from_numpy(W.reshape(-1)).to(dev), N, K)
    assert capi.batch_plane_bytes(FMT_Q6_K, N, K) == ((N + 3) // 4) * nsb * 1088
    plane = capi.build_batch_plane(FMT_Q6_K, w, N, K)
    sync()
    got_w, got_s = _plane_rows(plane.cpu().numpy(), N, nsb)
    for r in range(N):
        for t in range(nsb):
            ew, es, _ = oracle.subblocks(FMT_Q6_K, W[r, t])
            assert np.array_equal(got_w[r, t], ew), (r, t)
            assert np.array_equal(got_s[r, t], es), (r, t)
    assert not got_w[N:].any() and not got_s[N:].any()


def test_q6k_batch_plane_launches_match(capi, dev, oracle):
    """Batches of 5..8 rows launched with the matrix's plane: the exact block sums of the plane kernel equal the
    CPU restatement's; the fp32 results are bit-identical to the launch without a plane where that is the
    matrix-unit kernel as well (K = 25600, batches the quad-lane kernel cannot hold), within the format's tolerance
    of the CPU restatement everywhere (K = 5120 and batch 5 of K = 25600 leave the quad-lane kernel for it);
    batches of 1..4 do not look at the plane; the same call without the plane is the old launch."""
    import torch

    for N, K in ((1030, 25600), (4100, 5120), (50, 2048)):
        W = synth.weights_numpy(FMT_Q6_K, N, K, 77 + N)
        w = capi.prepare_weights(FMT_Q6_K, torch.from_numpy(W.reshape(-1)).to(dev), N, K)
        x = synth.activations_numpy(8, K, 9)
        q8 = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
        r0 = max(N - 70, 0)
        rows = slice(r0, N)
        exp, exp_sums = oracle.gemm(FMT_Q6_K, W[rows], K, oracle.quantize(x), want_sums=True)
        before = {M: capi.gemv(FMT_Q6_K, w, q8, M, N, K).clone() for M in (1, 4, 5, 7, 8)}
        plane = capi.build_batch_plane(FMT_Q6_K, w, N, K)
        assert plane is not None
        for M in (1, 4, 5, 7, 8):
            y = capi.gemv(FMT_Q6_K, w, q8, M, N, K, plane=plane)
            s = capi.gemv_block_sums(FMT_Q6_K, w, q8, M, N, K, r0, N - r0, plane=plane)
            sync()
            assert np.array_equal(s.cpu().numpy(), exp_sums[:M]), (N, K, M)
            assert rel_err(y.cpu().numpy()[:, rows], exp[:M]) <= TOL[FMT_Q6_K] * 1e-2, (N, K, M)
            with_plane = capi.gemv_describe(FMT_Q6_K, M, N, K, has_plane=True)
            assert (with_plane.kernel == 3 and with_plane.decode_equivalent == 0) if M >= 5 else with_plane.kernel != 3
            if M <= 4 or capi.gemv_describe(FMT_Q6_K, M, N, K).kernel == 3:
                assert torch.equal(y, before[M]), (N, K, M)
        # fp32 input quantised inside the launch takes the plane too
        xf = torch.from_numpy(x).to(dev)
        scratch = torch.empty(8 * (K // 32) * 36, dtype=torch.uint8, device=dev)
        out = torch.empty(8, N, device=dev)
        capi.gemv_fused_f32([(FMT_Q6_K, w, out, plane)], xf, 8, K, q8_scratch=scratch)
        sync()
        assert torch.equal(out, capi.gemv(FMT_Q6_K, w, q8, 8, N, K, plane=plane))
        y = capi.gemv(FMT_Q6_K, w, q8, 8, N, K)
        sync()
        assert torch.equal(y, before[8])


def test_a_plane_is_an_argument_not_a_registration(capi, dev, oracle):
    """Nothing is remembered between calls: two matrices that follow each other AT THE SAME ADDRESS (what a caching
    allocator hands out after a free) each multiply against the plane passed with them, and a launch without a
    plane never reads one."""
    import torch

    N, K, M = 4100, 5120, 8
    x = synth.activations_numpy(M, K, 3)
    q8 = capi.quantize_q8_1(torch.from_numpy(x).to(dev))
    buf = torch.empty(capi.prepared_bytes(FMT_Q6_K, N, K), dtype=torch.uint8, device=dev)
    results = []
    for seed in (1, 2):
        W = synth.weights_numpy(FMT_Q6_K, N, K, seed)
        buf.copy_(capi.prepare_weights(FMT_Q6_K, torch.from_numpy(W.reshape(-1)).to(dev), N, K))   # same address, new matrix
        plane = capi.build_batch_plane(FMT_Q6_K, buf, N, K)
        y = capi.gemv(FMT_Q6_K, buf, q8, M, N, K, plane=plane)
        y0 = capi.gemv(FMT_Q6_K, buf, q8, M, N, K)
        sync()
        exp = oracle.gemm(FMT_Q6_K, W[-64:], K, oracle.quantize(x))
        assert rel_err(y.cpu().numpy()[:, -64:], exp) <= TOL[FMT_Q6_K] * 1e-2, seed
        assert rel_err(y0.cpu().numpy()[:, -64:], exp) <= TOL[FMT_Q6_K] * 1e-2, seed
        results.append(y.clone())
        del plane
    assert not torch.equal(results[0], results[1])


def test_batch_plane_refusals(capi, dev):
    import torch

    lib = capi.load()
    assert capi.batch_plane_bytes(FMT_IQ3_S, 5120, 25600) == 0      # Q4_K and Q6_K only
    assert capi.batch_plane_bytes(FMT_Q4_K, 1024, 5120) == 0        # Q4_K: where batches go to the matrix unit
    assert capi.batch_plane_bytes(FMT_Q4_K, 25600, 5120) == 6400 * 20 * 576
    assert capi.batch_plane_bytes(FMT_Q6_K, 5120, 1024) == 0        # rows of eight super-blocks and more
    assert capi.batch_plane_bytes(FMT_Q6_K, 5120, 25600) == 1280 * 100 * 1088
    buf = torch.zeros(4096, dtype=torch.uint8, device=dev)
    y = torch.zeros(64, device=dev)
    assert not lib.llam_ql_build_batch_plane(FMT_Q4_K, buf.data_ptr(), buf.data_ptr(), 4, 2048, 0, None)   # too few rows
    assert not lib.llam_ql_build_batch_plane(FMT_Q6_K, None, buf.data_ptr(), 4, 2048, 0, None)
    # a plane for a shape that has none, or a misaligned one, is refused by the launches
    assert not lib.llam_ql_gemv_plane(FMT_Q6_K, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), y.data_ptr(), 5, 4, 1024, 4, 0, None)
    assert "no batch plane" in capi.last_error()
    assert not lib.llam_ql_gemv_plane(FMT_IQ3_S, buf.data_ptr(), buf.data_ptr(), buf.data_ptr(), y.data_ptr(), 5, 4, 2048, 4, 0, None)
    assert not lib.llam_ql_gemv_plane(FMT_Q6_K, buf.data_ptr(), buf.data_ptr() + 4, buf.data_ptr(), y.data_ptr(), 5, 4, 2048, 4, 0, None)
    assert "16-byte aligned" in capi.last_error()


def test_q4k_batch_plane_is_the_prepared_matrix_regrouped(capi, dev):
    """The Q4_K plane holds the bytes of the super-blocks, not new ones: per group of four rows and super-block four
    128-byte lines (the rows' two 16-byte halves of one 32-byte group of quants each), then the rows' heads."""
    import torch

    N, K = 4098, 2048   # a last group of two rows
    nsb = K // 256
    W = synth.weights_numpy(FMT_Q4_K, N, K, 3)           # [N][nsb][144]
    w = capi.prepare_weights(FMT_Q4_K, torch.from_numpy(W.reshape(-1)).to(dev), N, K)
    G = (N + 3) // 4
    assert capi.batch_plane_bytes(FMT_Q4_K, N, K) == G * nsb * 576
    plane = capi.build_batch_plane(FMT_Q4_K, w, N, K)
    sync()
    p = plane.cpu().numpy()
    pad = np.zeros((G * 4, nsb, 144), np.uint8)
    pad[:N] = W.reshape(N, nsb, 144)
    quants = pad[:, :, 16:].reshape(G, 4, nsb, 4, 32).transpose(0, 2, 3, 1, 4)   # [g][sb][group of quants][row][32]
    heads = pad[:, :, :16].reshape(G, 4, nsb, 16).transpose(0, 2, 1, 3)          # [g][sb][row][16]
    assert np.array_equal(p[:G * nsb * 512], quants.reshape(-1))
    assert np.array_equal(p[G * nsb * 512:], heads.reshape(-1))


def test_q4k_batch_plane_launches_match(capi, dev, oracle):
    """Q4_K batches of 5..8 launched with the matrix's plane: the plane kernel's exact block sums equal the CPU
    restatement's, its results the matrix-unit kernel's bit for bit; rows that do not fill the last tile or group
    included; fp32 and SwiGLU input as well."""
    import torch

    for N, K in ((4100, 5120), (4097, 8192)):
        W = synth.weights_numpy(FMT_Q4_K, N, K, 21 + N)
        w = capi.prepare_weights(FMT_Q4_K, torch.from_numpy(W.reshape(-1)).to(dev), N, K)
        x = synth.activations_numpy(8, K, 4)
        xd = torch.from_numpy(x).to(dev)
        q8 = capi.quantize_q8_1(xd)
        rows = slice(N - 70, N)
        exp, exp_sums = oracle.gemm(FMT_Q4_K, W[rows], K, oracle.quantize(x), want_sums=True)
        scratch = torch.empty(8 * (K // 32) * 36, dtype=torch.uint8, device=dev)
        before = {M: capi.gemv(FMT_Q4_K, w, q8, M, N, K).clone() for M in (4, 5, 6, 8)}
        before_f32 = capi.gemv_f32(FMT_Q4_K, w, xd, 8, N, K, q8_scratch=scratch).clone()
        g, u = torch.randn(8, K, device=dev), torch.randn(8, K, device=dev)
        before_swiglu = capi.gemv_swiglu_f32(FMT_Q4_K, w, g, u, 8, N, K, q8_scratch=scratch).clone()
        assert capi.gemv_describe(FMT_Q4_K, 5, N, K).kernel == 3
        plane = capi.build_batch_plane(FMT_Q4_K, w, N, K)
        for M in (4, 5, 6, 8):
            y = capi.gemv(FMT_Q4_K, w, q8, M, N, K, plane=plane)
            s = capi.gemv_block_sums(FMT_Q4_K, w, q8, M, N, K, N - 70, 70, plane=plane)
            sync()
            assert np.array_equal(s.cpu().numpy(), exp_sums[:M]), (N, K, M)
            assert torch.equal(y, before[M]), (N, K, M)
            assert rel_err(y.cpu().numpy()[:, rows], exp[:M]) <= TOL[FMT_Q4_K] * 1e-2
        out = torch.empty(8, N, device=dev)
        capi.gemv_fused_f32([(FMT_Q4_K, w, out, plane)], xd, 8, K, q8_scratch=scratch)
        y = capi.gemv_swiglu_f32(FMT_Q4_K, w, g, u, 8, N, K, q8_scratch=scratch, plane=plane)
        sync()
        assert torch.equal(out, before_f32) and torch.equal(y, before_swiglu)


@pytest.mark.parametrize("M", [6, 8])
def test_q4k_long_rows_on_the_matrix_unit(capi, dev, oracle, M):
    """Q4_K rows of 100 super-blocks at batches of 5..8: eight activation rows do not fit the LDS, so the matrix-unit
    kernel walks the row in chunks that producer wavefronts stage.  Repeatable; with the matrix's batch plane the same
    bits; the fp32-input call gives the bits of quantise + GEMV; block sums (plain and from the plane) and a window
    of rows against the CPU restatement."""
    import torch

    fmt, N, K = FMT_Q4_K, 4100, 25600
    plan = capi.gemv_describe(fmt, M, N, K)
    assert plan.kernel == capi.KERNEL_MFMA and not plan.decode_equivalent
    assert capi.gemv_describe(fmt, M, N, K, has_plane=True).kernel == capi.KERNEL_MFMA
    W = synth.weights_numpy(fmt, N, K, 4242)
    x = synth.activations_numpy(M, K, 4243)
    wd = upload_weights(capi, dev, fmt, W)
    xd = torch.from_numpy(x).to(dev)
    qd = capi.quantize_q8_1(xd)
    y = capi.gemv(fmt, wd, qd, M, N, K)
    again = capi.gemv(fmt, wd, qd, M, N, K)
    plane = capi.build_batch_plane(fmt, wd, N, K)
    yp = capi.gemv(fmt, wd, qd, M, N, K, plane=plane)
    yf = capi.gemv_f32(fmt, wd, xd, M, N, K)
    s0 = capi.gemv_block_sums(fmt, wd, qd, M, N, K, 4000, 100)
    sp = capi.gemv_block_sums(fmt, wd, qd, M, N, K, 4000, 100, plane=plane)
    sync()
    assert torch.equal(y, again) and torch.equal(y, yp) and torch.equal(y, yf)
    q8 = oracle.quantize(x)
    C, sums = oracle.gemm(fmt, W, K, q8, n0=4000, n1=4100, want_sums=True)
    assert np.array_equal(s0.cpu().numpy(), sums) and np.array_equal(sp.cpu().numpy(), sums)
    assert rel_err(y.cpu().numpy()[:, 4000:4100], C) <= TOL[fmt] * 1e-2
