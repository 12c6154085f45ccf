"""Writes tests/golden/decode_goldens.npz: inputs and the outputs of the reference's own
RMSNorm, RoPE, SwiGLU and softmax primitives and of the router built on the last (compiled into oracle/_ref from the reference tree by
oracle/Makefile).  Run in a container that holds the reference; the fixture is data only."""
from pathlib import Path
import sys

import numpy as np

sys.path.insert(0, str(Path(__file__).resolve().parents[2]))
from oracle.binding import Ref, build  # noqa: E402


def main():
    build()
    ref = Ref()
    assert ref.has_decode
    rng = np.random.default_rng(20240)
    rows, cols = 3, 5120
    x = (rng.standard_normal((rows, cols)) * np.array([[1.0], [0.02], [25.0]])).astype(np.float32)
    gamma = rng.uniform(0.2, 2.0, cols).astype(np.float32)
    delta = rng.standard_normal((rows, cols)).astype(np.float32)
    eps = np.float32(1e-6)
    out = {"rms_x": x, "rms_gamma": gamma, "rms_delta": delta, "rms_eps": eps}
    out["rms_y_scalar"] = np.stack([ref.rmsnorm_row(x[r], gamma, eps, 1) for r in range(rows)])
    out["rms_y_avx512"] = np.stack([ref.rmsnorm_row(x[r], gamma, eps, 3) for r in range(rows)])
    ys, rs = zip(*[ref.residual_rmsnorm_row(delta[r], x[r], gamma, eps) for r in range(rows)])
    out["rms_res_y_avx512"] = np.stack(ys)
    out["rms_res_after"] = np.stack(rs)
    hd, theta = 128, 1e6
    out["rope_inv_freq"] = ref.rope_inv_freq(hd, theta)
    head = rng.standard_normal(hd).astype(np.float32)
    k = rng.standard_normal(hd).astype(np.float32)
    pos = np.array([0, 1, 2, 77, 1024, 4095], np.int32)
    out["rope_head"] = head
    out["rope_positions"] = pos
    out["rope_scalar"] = np.stack([ref.rope_head_scalar(head, int(p), theta) for p in pos])
    out["rope_token_q"] = np.stack([ref.rope_token(np.tile(head, 2), k, hd, int(p), theta)[0] for p in pos])
    assert ref.has_swiglu
    g = (rng.standard_normal(1037) * 4).astype(np.float32)  # 64 vectors and a scalar tail of 13
    g[:8] = [-100, -88, -20, -1e-3, 0, 1e-3, 20, 88]
    u = rng.standard_normal(1037).astype(np.float32)
    out["swiglu_gate"], out["swiglu_up"], out["swiglu_out"] = g, u, ref.swiglu(g, u)
    # the router from the logits on (CPUMoEKernel::route: softmax_row_fp32 as the dispatcher runs it,
    # partial_sort, renormalisation): 256 experts, top-8, logits of three spreads; no exact ties
    assert ref.has_route
    lg = np.concatenate([(rng.standard_normal((6, 256)) * s).astype(np.float32) for s in (1.0, 6.0, 40.0)])
    ids, w, probs = ref.moe_route(lg, 8, True, 0)
    _, w_raw, _ = ref.moe_route(lg, 8, False, 0)
    out["route_logits"], out["route_ids"], out["route_weights"], out["route_probs"] = lg, ids, w, probs
    out["route_weights_unnormalised"] = w_raw
    np.savez_compressed(Path(__file__).with_name("decode_goldens.npz"), **out)
    print("wrote decode_goldens.npz", {k: np.asarray(v).shape for k, v in out.items()})


if __name__ == "__main__":
    main()
