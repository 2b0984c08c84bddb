"""GPU: every matvec / GEMM / MoE entry point on seeded random shapes against the oracle.

The fixed-shape tests sit on the shapes the kernels were written for; this sweep
draws shapes that sit on none of their tile sizes (odd row counts, row lengths
of an odd number of blocks, column counts either side of the kernels' limits).
Bars as elsewhere: max|got-ref|/max(1,|ref|) < 1e-4 against the FP64 oracle
(lev-cli/src/main.rs:12), 1e-3 for the fp16 GEMM (main.rs:1266-1278), expert ids
bit-exact, greedy token bit-exact.
"""
import numpy as np
import pytest
import torch

import oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

GATE = 1e-4
GEMM_TOL = 1e-3


@pytest.fixture(scope="module")
def ctx():
    from leviathan_amd import ops
    c = ops.Context(0)
    yield c
    c.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def shapes(seed, count, block, max_rows, max_blocks):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        rows = int(rng.integers(1, max_rows + 1))
        cols = block * int(rng.integers(1, max_blocks + 1))
        out.append((rows, cols))
    return out


@pytest.mark.parametrize("rows,cols", shapes(101, 16, 32, 900, 260))
def test_q4_0_gemv_random(ctx, rows, cols):
    w = O.synth_q4_0(rows * 7 + cols, rows * cols // 32, 0.02)
    x = O.normal(cols, rows + 1)
    y = torch.full((rows,), float("nan"), device="cuda")
    ctx.q4_0_gemv(dev(w), dev(x), cols, rows, y=y)
    ctx.sync()
    assert O.max_rel_err(y.cpu().numpy(), O.q4_0_matvec_f64(w, rows, cols, x)) < GATE


@pytest.mark.parametrize("rows,cols", shapes(102, 12, 256, 700, 24))
def test_q6_k_gemv_random_with_greedy_token(ctx, rows, cols):
    w = O.synth_q6_k(rows * 5 + cols, rows * cols // 256, 0.01)
    x = O.normal(cols, rows + 2)
    y, idx, margin = ctx.q6_k_gemv(dev(w), dev(x), cols, rows, argmax=True)
    ctx.sync()
    got = y.cpu().numpy()
    ref = O.q6_k_matvec_f64(w, rows, cols, x)
    # the sums are formed without rounding: the reference's gate holds whatever the row's magnitudes
    assert O.max_rel_err(got, ref) < GATE
    assert int(idx.cpu()) == int(np.argmax(got))       # first maximum of the values it wrote


@pytest.mark.parametrize("rows,cols", shapes(105, 12, 256, 600, 40))
def test_q6_k_gemv_random_columns_and_norm(ctx, rows, cols):
    rng = np.random.default_rng(rows * 29 + cols)
    ncol = int(rng.integers(1, 17))
    with_norm = bool(rng.integers(0, 2))
    w = O.synth_q6_k(rows + cols, rows * cols // 256, 0.01)
    x = O.normal(ncol * cols, rows + 7).reshape(ncol, cols)
    gain = O.normal(cols, rows + 8, 1.0, 0.1) if with_norm else None
    y = torch.full((ncol, rows), float("nan"), device="cuda")
    ctx.q6_k_gemv_ncol(dev(w), dev(x), cols, rows, ncol, gain=None if gain is None else dev(gain), y=y)
    ctx.sync()
    got = y.cpu().numpy()
    for c in range(ncol):
        xc = O.rmsnorm(x[c], gain, 1e-6) if with_norm else x[c]
        assert O.max_rel_err(got[c], O.q6_k_matvec_f64(w, rows, cols, xc)) < GATE, (c, ncol, with_norm)


@pytest.mark.parametrize("rows,cols", shapes(103, 12, 256, 500, 20))
def test_q4_k_gemv_random_columns_and_norm(ctx, rows, cols):
    rng = np.random.default_rng(rows * 31 + cols)
    ncol = int(rng.integers(1, 17))
    with_norm = bool(rng.integers(0, 2))
    w = O.synth_q4_k(rows + cols, rows * cols // 256, 0.01)
    x = O.normal(ncol * cols, rows + 3).reshape(ncol, cols)
    gain = O.normal(cols, rows + 4, 1.0, 0.1) if with_norm else None
    y = torch.full((ncol, rows), float("nan"), device="cuda")
    ctx.q4_k_gemv_ncol(dev(w), dev(x), cols, rows, ncol, gain=None if gain is None else dev(gain), y=y)
    ctx.sync()
    got = y.cpu().numpy()
    for c in range(ncol):
        xc = O.rmsnorm(x[c], gain, 1e-6) if with_norm else x[c]
        assert O.max_rel_err(got[c], O.q4_k_matvec_f64(w, rows, cols, xc)) < GATE, (c, ncol, with_norm)


@pytest.mark.parametrize("rows,cols", shapes(104, 12, 256, 500, 20))
def test_int8_path_random(ctx, rows, cols):
    rng = np.random.default_rng(rows * 17 + cols)
    ncol = int(rng.integers(1, 17))
    x = O.signed_units(ncol * cols, rows + cols).reshape(ncol, cols)
    xq, xs = ctx.norm_quant_q8(dev(x), cols, ncol)
    w4 = O.synth_q4_k(rows + 5, rows * cols // 256, 0.01)
    w6 = O.synth_q6_k(rows + 6, rows * cols // 256, 0.01)
    y4 = torch.full((ncol, rows), float("nan"), device="cuda")
    y6 = torch.full((ncol, rows), float("nan"), device="cuda")
    ctx.q4_k_gemv_q8(dev(w4), xq, xs, cols, rows, ncol, y=y4)
    ctx.q6_k_gemv_q8(dev(w6), xq, xs, cols, rows, ncol, y=y6)
    ctx.sync()
    q, s = xq.cpu().numpy(), xs.cpu().numpy()
    for c in range(ncol):
        codes, d, _ = O.quantize_q8(x[c])
        assert np.array_equal(q[c], codes)
        assert O.max_rel_err(y4[c].cpu().numpy(), O.q4_k_matvec_q8_f64(w4, rows, cols, q[c], s[c, :, 0])) < GATE
        assert O.max_rel_err(y6[c].cpu().numpy(), O.q6_k_matvec_q8_f64(w6, rows, cols, q[c], s[c, :, 0])) < GATE


@pytest.mark.parametrize("rows,cols", shapes(105, 10, 256, 330, 8))
def test_prefill_gemm_random(ctx, rows, cols):
    tokens = int(np.random.default_rng(rows + cols).integers(1, 600))
    w, x = H.config4(rows, cols, tokens, seed=rows + tokens)
    y = torch.full((tokens, rows), float("nan"), device="cuda")
    ctx.q4_k_gemm_prefill(dev(w), dev(x), cols, rows, tokens, y=y)
    ctx.sync()
    ref = O.q4_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(y.cpu().numpy(), ref) < GEMM_TOL, tokens


@pytest.mark.parametrize("rows,cols", shapes(107, 10, 256, 330, 8))
def test_q6_k_prefill_gemm_random(ctx, rows, cols):
    tokens = int(np.random.default_rng(rows + cols + 1).integers(1, 600))
    w = O.synth_q6_k(rows + tokens, rows * cols // 256, 0.01)
    x = O.normal(tokens * cols, rows + 1000).astype(np.float16).reshape(tokens, cols)
    y = torch.full((tokens, rows), float("nan"), device="cuda")
    ctx.q6_k_gemm_prefill(dev(w), dev(x), cols, rows, tokens, y=y)
    ctx.sync()
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(y.cpu().numpy(), ref) < GEMM_TOL, tokens


def moe_cases(seed, count):
    rng = np.random.default_rng(seed)
    out = []
    for _ in range(count):
        hidden = 64 * int(rng.integers(1, 17))
        inter = 64 * int(rng.integers(1, 9))
        experts = int(rng.integers(1, 70))
        top_k = int(rng.integers(1, min(8, experts) + 1))
        tokens = int(rng.integers(1, 24))
        out.append((hidden, inter, experts, top_k, tokens))
    return out


@pytest.mark.parametrize("hidden,inter,experts,top_k,tokens", moe_cases(106, 14))
def test_moe_layer_random(ctx, hidden, inter, experts, top_k, tokens):
    from leviathan_amd import ops
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=hidden + experts + tokens)
    pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                  offs["down_off"])
    y, ids, wts = ctx.moe_layer_q4_0(pools, dev(wr), dev(x), top_k, tokens)
    ctx.sync()
    y, ids, wts = y.cpu().numpy(), ids.cpu().numpy(), wts.cpu().numpy()
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        scores = O.f32_matvec(wr, experts, hidden, x[t])
        ref_ids, ref_w = O.router_topk(scores, top_k, None)
        H.check_moe_layer_token(y[t], ids[t], wts[t], ref_ids, ref_w, g, u, d, hidden, inter, x[t], GATE)
