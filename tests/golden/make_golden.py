#!/usr/bin/env python3
"""Writes tests/golden/vectors.npz: small seeded inputs with the CPU oracle's
outputs for every operator of the path.

Run from the repository root after the oracle passes its known-answer tests
(tests/test_oracle_kats.py):   python tests/golden/make_golden.py

The file holds data only (numpy arrays, loaded with allow_pickle=False).  The
reference-held known answers (hand-computed blocks of the reference's own
tests) are restated byte by byte in tests/test_oracle_kats.py; this file adds
seeded cases, so that a change of the oracle or of a kernel that moves any
output shows up against a frozen copy.
"""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
sys.path.insert(0, ROOT)
import oracle as O  # noqa: E402

OUT = os.path.join(os.path.dirname(os.path.abspath(__file__)), "vectors.npz")


def main():
    v = {}
    # Q4_0: 24 x 256 (pair kernel) and 5 x 96 (odd block count, generic kernel)
    for tag, rows, cols, seed in (("q4_0_a", 24, 256, 101), ("q4_0_b", 5, 96, 102)):
        w = O.synth_q4_0(seed, rows * cols // 32, 0.02)
        x = O.normal(cols, seed + 1000)
        v[tag + "_w"], v[tag + "_x"] = w, x
        v[tag + "_dims"] = np.array([rows, cols], dtype=np.int64)
        v[tag + "_dequant_bits"] = O.q4_0_dequant(w).view(np.uint32)
        v[tag + "_y_f64"] = O.q4_0_matvec_f64(w, rows, cols, x)
        v[tag + "_y_ref_bits"] = O.q4_0_matvec_ref(w, rows, cols, x).view(np.uint32)
    # Q6_K: 12 x 512 with argmax and margin
    rows, cols = 12, 512
    w = O.synth_q6_k(103, rows * cols // 256, 0.01)
    x = O.normal(cols, 1103)
    y32 = O.q6_k_matvec_ref(w, rows, cols, x)
    v.update(q6_k_w=w, q6_k_x=x, q6_k_dims=np.array([rows, cols], dtype=np.int64),
             q6_k_dequant_bits=O.q6_k_dequant(w).view(np.uint32),
             q6_k_y_f64=O.q6_k_matvec_f64(w, rows, cols, x),
             q6_k_y_ref_bits=y32.view(np.uint32),
             q6_k_argmax=np.array([O.argmax(y32)], dtype=np.int64))
    # Q4_K: 16 x 512, three columns, fused RMSNorm
    rows, cols, ncol = 16, 512, 3
    w = O.synth_q4_k(104, rows * cols // 256, 0.01)
    x = O.normal(ncol * cols, 1104).reshape(ncol, cols)
    gain = O.normal(cols, 2104, 1.0, 0.1)
    y = np.stack([O.q4_k_matvec_f64(w, rows, cols, O.rmsnorm(x[c], gain, 1e-6)) for c in range(ncol)])
    v.update(q4_k_w=w, q4_k_x=x, q4_k_gain=gain, q4_k_dims=np.array([rows, cols, ncol], dtype=np.int64),
             q4_k_dequant_bits=O.q4_k_dequant(w).view(np.uint32), q4_k_y_f64=y,
             q4_k_y_plain_f64=np.stack([O.q4_k_matvec_f64(w, rows, cols, x[c]) for c in range(ncol)]))
    # prefill GEMM oracle: 5 tokens, every row
    xh = O.normal(5 * cols, 3104).astype(np.float16).reshape(5, cols)
    v.update(gemm_x_f16_bits=xh.view(np.uint16),
             gemm_y_f64=O.q4_k_gemm_f16_oracle(w, rows, cols, xh.view(np.uint16), 5, 0, 1))
    # int8-activation path: quantiser behind the RMSNorm of the Q4_K case's activations, the Q4_K
    # product on those codes, and the Q6_K product on the plainly quantised Q6_K activation
    q8 = [O.quantize_q8(O.rmsnorm(x[c], gain, 1e-6)) for c in range(ncol)]
    v.update(q8_codes=np.stack([q for q, d, s in q8]), q8_d_bits=np.stack([d for q, d, s in q8]).view(np.uint32),
             q8_s_bits=np.stack([s for q, d, s in q8]).view(np.uint32),
             q8_q4_k_y_f64=np.stack([O.q4_k_matvec_q8_f64(w, rows, cols, q, d) for q, d, s in q8]))
    q6, d6, s6 = O.quantize_q8(v["q6_k_x"])
    r6, c6 = (int(t) for t in v["q6_k_dims"])
    v.update(q8_q6_k_codes=q6, q8_q6_k_d_bits=d6.view(np.uint32),
             q8_q6_k_y_f64=O.q6_k_matvec_q8_f64(v["q6_k_w"], r6, c6, q6, d6))
    # elementwise
    g = np.array([1.0, -20.0, 1e30, -1e30, 1e-30, 1e20, 0.5, -0.5, 3.25, -7.5], dtype=np.float32)
    u = np.array([1.0, 3.0, 2.0, 2.0, 2.0, 2.0, 4.0, 4.0, -1.5, 0.25], dtype=np.float32)
    v.update(gelu_g=g, gelu_u=u, gelu_y_bits=np.array([O.gelu_up_f32(float(a), float(b)) for a, b in zip(g, u)],
                                  dtype=np.float32).view(np.uint32))
    xr = O.normal(2 * 320, 105).reshape(2, 320)
    gr = O.normal(320, 1105, 1.0, 0.1)
    v.update(rms_x=xr, rms_gain=gr, rms_y_f64=np.stack([O.rmsnorm_f64(xr[i], gr, 1e-6) for i in range(2)]))
    # router: 16 experts, top 4, three tokens, with an exact tie in token 2
    hidden, experts, top_k = 64, 16, 4
    wr = O.normal(experts * hidden, 106, 0.0, 0.02).reshape(experts, hidden)
    wr[9] = wr[3]                                    # experts 3 and 9 always tie: 3 must win
    xt = O.normal(3 * hidden, 1106).reshape(3, hidden)
    ids, wts, scores = [], [], []
    for t in range(3):
        s = O.f32_matvec(wr, experts, hidden, xt[t])
        i, wgt = O.router_topk(s, top_k)
        scores.append(s); ids.append(i); wts.append(wgt)
    v.update(router_w=wr, router_x=xt, router_ids=np.stack(ids).astype(np.int32),
             router_weights=np.stack(wts), router_scores=np.stack(scores))
    # MoE experts: hidden 128, inter 64, 6 experts, top 2, two tokens
    hidden, inter, experts, top_k = 128, 64, 6, 2
    gu, dn = inter * (hidden // 32) * 18, hidden * (inter // 32) * 18
    gate = O.synth_q4_0(107, experts * gu // 18, 0.02)
    up = O.synth_q4_0(108, experts * gu // 18, 0.02)
    down = O.synth_q4_0(109, experts * dn // 18, 0.02)
    xm = O.normal(2 * hidden, 1107).reshape(2, hidden)
    mids = np.array([[4, 1], [0, 5]], dtype=np.int32)
    mw = np.array([[0.7, 0.3], [0.55, 0.45]], dtype=np.float32)
    refs = [O.moe_experts_f64(gate, up, down, hidden, inter, mids[t], mw[t], xm[t]) for t in range(2)]
    v.update(moe_gate=gate, moe_up=up, moe_down=down, moe_x=xm, moe_ids=mids, moe_weights=mw,
             moe_dims=np.array([hidden, inter, experts, top_k], dtype=np.int64),
             moe_y_f64=np.stack([r["y"] for r in refs]), moe_act_f64=np.stack([r["act"] for r in refs]))
    np.savez_compressed(OUT, **v)
    print(OUT, os.path.getsize(OUT), "bytes,", len(v), "arrays")


if __name__ == "__main__":
    main()
