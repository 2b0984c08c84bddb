"""Committed golden vectors (tests/golden/vectors.npz, written by
tests/golden/make_golden.py from the CPU oracle once it passed the reference's
known-answer tests).

CPU: the oracle still reproduces the frozen outputs bit for bit.
GPU: the HIP library, through the C ABI, meets the parity bars against them:
dequantised weights, expert ids and argmax bit-exact; f32 outputs within
max|got-ref|/max(1,|ref|) < 1e-4 of the frozen FP64 outputs (1e-3 for the
fp16-input GEMM).
"""
import os

import numpy as np
import pytest

import oracle as O

G = np.load(os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "vectors.npz"),
            allow_pickle=False)
TOL = 1e-4


# ------------------------------------------------------------------ CPU

def test_oracle_reproduces_golden_q4_0():
    for tag in ("q4_0_a", "q4_0_b"):
        rows, cols = (int(v) for v in G[tag + "_dims"])
        w, x = G[tag + "_w"], G[tag + "_x"]
        assert np.array_equal(O.q4_0_dequant(w).view(np.uint32), G[tag + "_dequant_bits"])
        assert np.array_equal(O.q4_0_matvec_f64(w, rows, cols, x), G[tag + "_y_f64"])
        assert np.array_equal(O.q4_0_matvec_ref(w, rows, cols, x).view(np.uint32), G[tag + "_y_ref_bits"])


def test_oracle_reproduces_golden_k_quants():
    rows, cols = (int(v) for v in G["q6_k_dims"])
    w, x = G["q6_k_w"], G["q6_k_x"]
    assert np.array_equal(O.q6_k_dequant(w).view(np.uint32), G["q6_k_dequant_bits"])
    assert np.array_equal(O.q6_k_matvec_f64(w, rows, cols, x), G["q6_k_y_f64"])
    y32 = O.q6_k_matvec_ref(w, rows, cols, x)
    assert np.array_equal(y32.view(np.uint32), G["q6_k_y_ref_bits"])
    assert O.argmax(y32) == int(G["q6_k_argmax"][0])
    rows, cols, ncol = (int(v) for v in G["q4_k_dims"])
    w, x, gain = G["q4_k_w"], G["q4_k_x"], G["q4_k_gain"]
    assert np.array_equal(O.q4_k_dequant(w).view(np.uint32), G["q4_k_dequant_bits"])
    for c in range(ncol):
        assert np.array_equal(O.q4_k_matvec_f64(w, rows, cols, O.rmsnorm(x[c], gain, 1e-6)), G["q4_k_y_f64"][c])
    assert np.array_equal(O.q4_k_gemm_f16_oracle(w, rows, cols, G["gemm_x_f16_bits"], 5, 0, 1), G["gemm_y_f64"])


def test_oracle_reproduces_golden_int8_path():
    rows, cols, ncol = (int(v) for v in G["q4_k_dims"])
    w, x, gain = G["q4_k_w"], G["q4_k_x"], G["q4_k_gain"]
    for c in range(ncol):
        q, d, s = O.quantize_q8(O.rmsnorm(x[c], gain, 1e-6))
        assert np.array_equal(q, G["q8_codes"][c]) and np.array_equal(d.view(np.uint32), G["q8_d_bits"][c])
        assert np.array_equal(s.view(np.uint32), G["q8_s_bits"][c])
        assert np.array_equal(O.q4_k_matvec_q8_f64(w, rows, cols, q, d), G["q8_q4_k_y_f64"][c])
    r6, c6 = (int(v) for v in G["q6_k_dims"])
    q, d, s = O.quantize_q8(G["q6_k_x"])
    assert np.array_equal(q, G["q8_q6_k_codes"]) and np.array_equal(d.view(np.uint32), G["q8_q6_k_d_bits"])
    assert np.array_equal(O.q6_k_matvec_q8_f64(G["q6_k_w"], r6, c6, q, d), G["q8_q6_k_y_f64"])


def test_oracle_reproduces_golden_moe_and_elementwise():
    got = np.array([O.gelu_up_f32(float(a), float(b)) for a, b in zip(G["gelu_g"], G["gelu_u"])],
                   dtype=np.float32)
    assert np.array_equal(got.view(np.uint32), G["gelu_y_bits"])
    for i in range(2):
        assert np.array_equal(O.rmsnorm_f64(G["rms_x"][i], G["rms_gain"], 1e-6), G["rms_y_f64"][i])
    wr, xt = G["router_w"], G["router_x"]
    experts, hidden = wr.shape
    for t in range(xt.shape[0]):
        s = O.f32_matvec(wr, experts, hidden, xt[t])
        assert np.array_equal(s, G["router_scores"][t])
        ids, wts = O.router_topk(s, G["router_ids"].shape[1])
        assert np.array_equal(ids, G["router_ids"][t]) and np.array_equal(wts, G["router_weights"][t])
        assert 9 not in ids or 3 in ids                       # tie between 3 and 9: 3 first
    hidden, inter, experts, top_k = (int(v) for v in G["moe_dims"])
    for t in range(2):
        r = O.moe_experts_f64(G["moe_gate"], G["moe_up"], G["moe_down"], hidden, inter,
                              G["moe_ids"][t], G["moe_weights"][t], G["moe_x"][t])
        assert np.array_equal(r["y"], G["moe_y_f64"][t]) and np.array_equal(r["act"], G["moe_act_f64"][t])


# ------------------------------------------------------------------ GPU

@pytest.fixture(scope="module")
def ctx():
    from leviathan_amd import ops
    c = ops.Context(0)
    yield c
    c.close()


def dev(a):
    import torch
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def host(t):
    return t.cpu().numpy()


@pytest.mark.gpu
def test_gpu_golden_q4_0(ctx):
    from leviathan_amd import capi
    for tag in ("q4_0_a", "q4_0_b"):
        rows, cols = (int(v) for v in G[tag + "_dims"])
        w, x = dev(G[tag + "_w"]), dev(G[tag + "_x"])
        dq = ctx.dequant(capi.TYPE_Q4_0, w, rows * cols // 32)
        y = ctx.q4_0_gemv(w, x, cols, rows)
        ctx.sync()
        assert np.array_equal(host(dq).view(np.uint32), G[tag + "_dequant_bits"])
        assert O.max_rel_err(host(y), G[tag + "_y_f64"]) < TOL


@pytest.mark.gpu
def test_gpu_golden_q6_k(ctx):
    from leviathan_amd import capi
    rows, cols = (int(v) for v in G["q6_k_dims"])
    w, x = dev(G["q6_k_w"]), dev(G["q6_k_x"])
    dq = ctx.dequant(capi.TYPE_Q6_K, w, rows * cols // 256)
    y, idx, margin = ctx.q6_k_gemv(w, x, cols, rows, argmax=True)
    ctx.sync()
    assert np.array_equal(host(dq).view(np.uint32), G["q6_k_dequant_bits"])
    yh = host(y)
    assert O.max_rel_err(yh, G["q6_k_y_f64"]) < TOL
    assert int(idx.item()) == O.argmax(yh) == int(G["q6_k_argmax"][0])
    assert abs(float(margin.item()) - O.top_margin(yh)) <= 1e-6 * max(1.0, abs(O.top_margin(yh)))


@pytest.mark.gpu
def test_gpu_golden_q4_k(ctx):
    from leviathan_amd import capi
    rows, cols, ncol = (int(v) for v in G["q4_k_dims"])
    w, x, gain = dev(G["q4_k_w"]), dev(G["q4_k_x"]), dev(G["q4_k_gain"])
    dq = ctx.dequant(capi.TYPE_Q4_K, w, rows * cols // 256)
    y = ctx.q4_k_gemv_ncol(w, x, cols, rows, ncol, gain=gain)
    yp = ctx.q4_k_gemv_ncol(w, x, cols, rows, ncol)
    xh = dev(G["gemm_x_f16_bits"].view(np.float16))
    yg = ctx.q4_k_gemm_prefill(w, xh, cols, rows, 5)
    ctx.sync()
    assert np.array_equal(host(dq).view(np.uint32), G["q4_k_dequant_bits"])
    for c in range(ncol):
        assert O.max_rel_err(host(y)[c], G["q4_k_y_f64"][c]) < TOL
        assert O.max_rel_err(host(yp)[c], G["q4_k_y_plain_f64"][c]) < TOL
    for t in range(5):
        assert O.max_rel_err(host(yg)[t], G["gemm_y_f64"][t]) < 1e-3      # fp16 inputs: 1e-3


@pytest.mark.gpu
def test_gpu_golden_int8_path(ctx):
    rows, cols, ncol = (int(v) for v in G["q4_k_dims"])
    w, x, gain = dev(G["q4_k_w"]), dev(G["q4_k_x"].copy()), dev(G["q4_k_gain"])
    xq, xs = ctx.norm_quant_q8(x, cols, ncol, gain=gain)
    y = ctx.q4_k_gemv_q8(w, xq, xs, cols, rows, ncol)
    r6, c6 = (int(v) for v in G["q6_k_dims"])
    xq6, xs6 = ctx.norm_quant_q8(dev(G["q6_k_x"].copy()), c6, 1)
    y6 = ctx.q6_k_gemv_q8(dev(G["q6_k_w"]), xq6, xs6, c6, r6, 1)
    ctx.sync()
    assert np.array_equal(host(xq), G["q8_codes"])                       # codes, scales, sums: bit-exact
    assert np.array_equal(host(xs)[..., 0].view(np.uint32), G["q8_d_bits"])
    assert np.array_equal(host(xs)[..., 1].view(np.uint32), G["q8_s_bits"])
    assert np.array_equal(host(xq6)[0], G["q8_q6_k_codes"])
    assert np.array_equal(host(xs6)[0, :, 0].view(np.uint32), G["q8_q6_k_d_bits"])
    for c in range(ncol):
        assert O.max_rel_err(host(y)[c], G["q8_q4_k_y_f64"][c]) < TOL
    assert O.max_rel_err(host(y6)[0], G["q8_q6_k_y_f64"]) < TOL


@pytest.mark.gpu
def test_gpu_golden_elementwise(ctx):
    g, u = G["gelu_g"], G["gelu_u"]
    y = host(ctx.gelu_up(dev(np.concatenate([g, u])), g.size))
    want = G["gelu_y_bits"].view(np.float32)
    assert np.all(np.isfinite(y))
    assert np.all(np.abs(y - want) <= 1e-6 * np.maximum(1.0, np.abs(want)))
    r = host(ctx.rmsnorm(dev(G["rms_x"]), G["rms_x"].shape[1], 2, weight=dev(G["rms_gain"])))
    for i in range(2):
        assert O.max_rel_err(r.reshape(2, -1)[i], G["rms_y_f64"][i]) < 1e-5


@pytest.mark.gpu
def test_gpu_golden_router_and_experts(ctx):
    from leviathan_amd import ops
    wr, xt = G["router_w"], G["router_x"]
    experts, hidden = wr.shape
    top_k = G["router_ids"].shape[1]
    for tokens in (1, xt.shape[0]):                     # both the few-token and the batched path
        ids, wts = ctx.moe_route_topk(dev(wr), dev(xt[:tokens]), hidden, experts, top_k, tokens)
        ctx.sync()
        assert np.array_equal(host(ids), G["router_ids"][:tokens])                 # bit-exact
        assert np.all(np.abs(host(wts) - G["router_weights"][:tokens]) <= 1e-6)
    hidden, inter, experts, top_k = (int(v) for v in G["moe_dims"])
    pool = np.concatenate([G["moe_gate"], G["moe_up"], G["moe_down"]])
    pool_d = dev(pool)
    pools = ops.Context.moe_pools(pool_d, hidden, inter, experts, 0, G["moe_gate"].size,
                                  G["moe_gate"].size + G["moe_up"].size)
    y, act = ctx.moe_experts_q4_0(pools, dev(G["moe_x"]), dev(G["moe_ids"]), dev(G["moe_weights"]),
                                  top_k, 2, want_act=True)
    ctx.sync()
    for t in range(2):
        assert O.max_rel_err(host(y)[t], G["moe_y_f64"][t]) < TOL
        assert O.max_rel_err(host(act)[t].reshape(-1), G["moe_act_f64"][t].reshape(-1)) < TOL
