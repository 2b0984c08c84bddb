"""GPU parity: MoE router/top-k + routed Q4_0 experts, and the Q4_K prefill GEMM.

Bars: expert ids bit-exact; fp32 outputs max|got-ref|/max(1,|ref|) < 1e-4
against the FP64 oracle (MoESIMDOracle.contract, MoESIMDLowering.swift:930);
prefill GEMM < 1e-3 against the fp16-rounded FP64 oracle
(rust/crates/lev-cli/src/main.rs:1278).
"""
import numpy as np
import pytest
import torch

import oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

TOL = 1e-4
GEMM_TOL = 1e-3


@pytest.fixture(scope="module")
def ctx():
    from leviathan_amd import ops
    c = ops.Context(0)
    yield c
    c.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def cpu_route(wr, x, top_k, scale=None):
    """Reference path: F32 router matvec + CPU softmax/top-k (Gemma4.swift:3795-3810)."""
    scores = O.f32_matvec(wr, wr.shape[0], wr.shape[1], x)
    ids, wts = O.router_topk(scores, top_k, scale)
    return scores, ids, wts


# -------------------------------------------------------------- router ----

@pytest.mark.parametrize("hidden,experts,top_k,tokens", [(2048, 128, 8, 1), (2048, 128, 8, 64),
                                                         (256, 16, 3, 5), (2816, 128, 8, 3),
                                                         (96, 8, 8, 2), (130, 200, 64, 2),
                                                         (512, 20, 4, 33), (768, 130, 8, 16), (2080, 64, 8, 40),
                                                         (256, 600, 16, 2), (128, 2000, 64, 3), (256, 1024, 8, 17),
                                                         (64, 4096, 32, 1)])
def test_router_ids_bit_exact_weights_close(ctx, hidden, experts, top_k, tokens):
    wr = O.normal(experts * hidden, 7 + hidden, 0.0, 0.02).reshape(experts, hidden)
    x = O.normal(tokens * hidden, 8 + experts).reshape(tokens, hidden)
    ids, wts, scores = ctx.moe_route_topk(dev(wr), dev(x), hidden, experts, top_k, tokens,
                                          want_scores=True)
    ctx.sync()
    ids, wts, scores = ids.cpu().numpy(), wts.cpu().numpy(), scores.cpu().numpy()
    for t in range(tokens):
        ref_scores, ref_ids, ref_w = cpu_route(wr, x[t], top_k)
        ref64 = O.f32_matvec_f64(wr, experts, hidden, x[t])
        mag = np.abs(wr.astype(np.float64)) @ np.abs(x[t].astype(np.float64))
        # main.swift:2615-2647: |delta| <= 1e-4 * sum|w_i x_i| + 1e-6 against FP64
        assert np.all(np.abs(scores[t] - ref64) <= 1e-4 * mag + 1e-6)
        # ids can only be compared when the reference's own selection is not
        # decided by summation-order noise: gap at the top-k boundary >> |delta|
        order = np.sort(ref_scores)[::-1]
        if top_k < experts:
            gap = float(order[top_k - 1] - order[top_k])
            assert gap > 50 * float(np.max(np.abs(scores[t] - ref_scores))), "degenerate seed"
        inner = float(np.min(np.diff(-order[:top_k]))) if top_k > 1 else 1.0
        if inner > 50 * float(np.max(np.abs(scores[t] - ref_scores))):
            assert ids[t].tolist() == ref_ids.tolist()
        else:
            assert sorted(ids[t].tolist()) == sorted(ref_ids.tolist())
        assert len(set(ids[t].tolist())) == top_k
        assert abs(float(wts[t].astype(np.float64).sum()) - 1.0) < 1e-6
        assert np.allclose(wts[t], ref_w, rtol=2e-5, atol=1e-7)


def test_router_topk_is_exact_on_its_own_scores(ctx):
    """Selection, tie rule and renormalisation are exact given the scores the
    kernel produced: feed rows that make the scores exact small integers."""
    experts, hidden, top_k = 16, 64, 5
    wr = np.zeros((experts, hidden), np.float32)
    vals = [0, 1, 0, 1, 0, 0, 0, 0, 0, 1, 0, 0, 0, 0, 0, 0]          # ties at 1.0: ids 1, 3, 9
    for e, v in enumerate(vals):
        wr[e, 0] = v
    x = np.zeros((1, hidden), np.float32)
    x[0, 0] = 1.0
    scale = np.arange(1, experts + 1, dtype=np.float32)
    ids, wts = ctx.moe_route_topk(dev(wr), dev(x), hidden, experts, top_k, 1, expert_scale=dev(scale))
    ctx.sync()
    ref_ids, ref_w = O.router_topk(np.array(vals, np.float32), top_k, scale)
    assert ids.cpu().numpy()[0].tolist() == ref_ids.tolist() == [1, 3, 9, 0, 2]
    assert np.allclose(wts.cpu().numpy()[0], ref_w, rtol=1e-6)


ORDER_CASES = {
    # exp() saturates at 1.0 for every score: all probabilities tie, index order wins
    "saturating_exp": [3e-20, 1e-20, 2e-20, 0.0, 5e-21, 4e-20, 0.0, 1e-21],
    # exp() underflows to 0 below about -745: those tie at 0, index order wins
    "underflow": [0.0, -800.0, -900.0, -1000.0, -750.0, -700.0, -2000.0, -760.0],
    # the ordinary range, with exact ties and a negative maximum
    "plain": [-3.0, -1.5, -3.0, -1.5, -7.25, -1.5, -20.0, -3.0],
    # one score just below the maximum (the gap is smaller than 1e-6), the rest ordinary
    "near_max": [1.0, 1.0 - 2.0 ** -24, -1.0, 1.0 - 2.0 ** -23, 0.5, 1.0, -4.0, 0.25],
}


@pytest.mark.parametrize("case", sorted(ORDER_CASES))
@pytest.mark.parametrize("experts", [8, 128, 200])
def test_router_selection_order_edge_cases(ctx, case, experts):
    """Selection order where the probabilities tie although the scores differ,
    and where they do not: one-hot x makes the scores exactly the chosen values,
    so ids are compared bit for bit, from the stand-alone router and from the
    selection the single-token layer runs inside its gate/up kernel."""
    from leviathan_amd import ops
    hidden, inter, top_k = 64, 64, 5
    vals = np.array(ORDER_CASES[case], np.float32)
    rng = np.random.default_rng(experts)
    scores = np.resize(vals, experts).astype(np.float32)
    scores[8:] = rng.permutation(scores[8:])
    wr = np.zeros((experts, hidden), np.float32)
    wr[:, 3] = scores
    x = np.zeros((1, hidden), np.float32)
    x[0, 3] = 1.0
    ref_ids, ref_w = O.router_topk(scores, top_k)
    ids, wts, got = ctx.moe_route_topk(dev(wr), dev(x), hidden, experts, top_k, 1, want_scores=True)
    ctx.sync()
    assert np.array_equal(got.cpu().numpy()[0], scores)
    assert ids.cpu().numpy()[0].tolist() == ref_ids.tolist()
    assert np.allclose(wts.cpu().numpy()[0], ref_w, rtol=1e-6, atol=0)

    gu, dn = inter * (hidden // 32) * 18, hidden * (inter // 32) * 18
    pool = rng.integers(0, 256, experts * (2 * gu + dn), dtype=np.uint8)
    pool.reshape(-1, 18)[:, 1] = 0x20          # fp16 scales of ordinary size
    pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, 0, experts * gu, 2 * experts * gu)
    _, ids2, wts2 = ctx.moe_layer_q4_0(pools, dev(wr), dev(x), top_k, 1)
    ctx.sync()
    assert ids2.cpu().numpy()[0].tolist() == ref_ids.tolist()
    assert np.allclose(wts2.cpu().numpy()[0], ref_w, rtol=1e-6, atol=0)


@pytest.mark.parametrize("experts,top_k", [(8, 3), (64, 8), (128, 8), (200, 16), (256, 5), (1000, 32)])
def test_router_selection_matches_the_oracle_on_adversarial_scores(ctx, experts, top_k):
    """256 score vectors per expert count, built to sit on the edges of the
    selection's two orderings: few distinct values (ties), neighbours one ulp
    apart, magnitudes from 1e-30 to 1e3, gaps below 1e-6 and beyond 690.  One-hot
    activations make the scores exactly the chosen values; ids must match the
    reference's order bit for bit."""
    cases = 256
    rng = np.random.default_rng(1000 + experts)
    scores = np.empty((cases, experts), np.float32)
    for t in range(cases):
        kind = t % 8
        if kind == 0:      # few distinct values: many exact ties
            scores[t] = rng.choice(np.array([-2.5, 0.0, 0.75, 3.0], np.float32), experts)
        elif kind == 1:    # one-ulp neighbours of one value
            base = np.float32(rng.uniform(-4, 4))
            scores[t] = base
            up = rng.random(experts) < 0.3
            scores[t][up] = np.nextafter(base, np.float32(np.inf))
            scores[t][rng.random(experts) < 0.2] = np.nextafter(base, np.float32(-np.inf))
        elif kind == 2:    # tiny magnitudes: exp saturates at 1 for every score.  (Differences
            # between 1e-19 and 1e-9 are left out on purpose: there the last bit of exp()
            # decides which probabilities tie, and neither this build's nor the reference's
            # libm promises that bit.)
            scores[t] = (rng.standard_normal(experts) * 10.0 ** rng.integers(-30, -20)).astype(np.float32)
        elif kind == 3:    # huge spread: exp underflows
            scores[t] = (-rng.random(experts) * 1500.0).astype(np.float32)
        elif kind == 4:    # ordinary router scores
            scores[t] = (rng.standard_normal(experts) * 2.0).astype(np.float32)
        elif kind == 5:    # ordinary, a handful within 1e-6 of the maximum
            scores[t] = (rng.standard_normal(experts) * 2.0).astype(np.float32)
            m = scores[t].max()
            near = rng.choice(experts, min(4, experts), replace=False)
            scores[t][near] = m - np.float32(1e-7) * rng.integers(0, 8, near.size).astype(np.float32)
        elif kind == 6:    # gaps right at the edges of the fast ordering
            scores[t] = rng.choice(np.array([0.0, -1e-6, -9.5e-7, -1.05e-6, -690.0, -689.9, -690.1, -5.0],
                                            np.float32), experts)
        else:              # all equal
            scores[t] = np.float32(rng.uniform(-3, 3))
    hidden = cases
    wr = np.ascontiguousarray(scores.T)                 # [experts, hidden]: score[t][e] = wr[e][t]
    x = np.eye(cases, dtype=np.float32)
    ids, wts, got = ctx.moe_route_topk(dev(wr), dev(x), hidden, experts, top_k, cases, want_scores=True)
    ctx.sync()
    assert np.array_equal(got.cpu().numpy(), scores)
    ids, wts = ids.cpu().numpy(), wts.cpu().numpy()
    for t in range(cases):
        ref_ids, ref_w = O.router_topk(scores[t], top_k)
        assert ids[t].tolist() == ref_ids.tolist(), (t, t % 8)
        assert np.allclose(wts[t], ref_w, rtol=2e-6, atol=0), (t, t % 8)


# ------------------------------------------------------------- experts ----

def run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts):
    from leviathan_amd import ops
    pool_d = dev(pool)
    pools = ops.Context.moe_pools(pool_d, hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                  offs["down_off"], offs.get("gate_stride"), offs.get("up_stride"),
                                  offs.get("down_stride"))
    tokens, top_k = ids.shape
    y, act = ctx.moe_experts_q4_0(pools, dev(x), dev(ids.astype(np.int32)), dev(wts.astype(np.float32)),
                                  top_k, tokens, want_act=True)
    ctx.sync()
    return y.cpu().numpy(), act.cpu().numpy()


def test_moe_hand_computed_composite(ctx):
    """main.swift:8925-8946: gate 16, up 2, act 32, down 512 -- exact."""
    gate, up, down = H.hand_moe()
    pool = np.concatenate([gate, up, down])
    offs = dict(gate_off=0, up_off=gate.size, down_off=gate.size + up.size)
    x = np.ones((1, 32), np.float32)
    y, act = run_experts(ctx, pool, offs, 32, 32, 1, x, np.array([[0]]), np.array([[1.0]]))
    assert np.array_equal(act[0, 0], np.full(32, 32.0, np.float32))
    assert np.array_equal(y[0], np.full(32, 512.0, np.float32))
    y, _ = run_experts(ctx, pool, offs, 32, 32, 1, x, np.array([[0]]), np.array([[0.5]]))
    assert np.array_equal(y[0], np.full(32, 256.0, np.float32))


def test_moe_tail_region_fused_gate_up_layout(ctx):
    """main.swift:6551-6615: hidden 96, inter 32, topK 3, the reference's fused
    gate|up tensor [2I, H] per expert, synthetic bytes SplitMix64(0x5A4C4F57),
    x from SplitMix64(70004); inside the FP64 contract."""
    hidden, inter, top_k = 96, 32, 3
    gu_stride = (hidden // 32) * 18 * 2 * inter
    dn_stride = (inter // 32) * 18 * hidden
    rng = O.SplitMix64(0x5A4C4F57)
    gu = H.swift_synthetic_blocks(rng, gu_stride * top_k // 18)
    dn = H.swift_synthetic_blocks(rng, dn_stride * top_k // 18)
    x = O.seeded_input(hidden, 1, 70004)[None]
    pool = np.concatenate([gu, dn])
    up_rel = inter * (hidden // 32) * 18
    offs = dict(gate_off=0, up_off=up_rel, down_off=gu.size, gate_stride=gu_stride,
                up_stride=gu_stride, down_stride=dn_stride)
    ids, wts = np.array([[0, 1, 2]]), np.array([[1.0, 1.0, 1.0]])
    y, act = run_experts(ctx, pool, offs, hidden, inter, top_k, x, ids, wts)
    # The reference gates this region STAGE BY STAGE (oracleRels,
    # MoELowering.swift:1818-1888): gate|up rows against FP64 of x, the
    # activation against the FP64 formula applied to the GPU's own gate|up
    # outputs, the down rows against FP64 of the GPU's own activation.  The raw
    # random fp16 scales of this fixture reach 6e4, so values grow to 1e15 and
    # only a stage-wise comparison is meaningful.
    gu_d = dev(gu)
    y_ref = np.zeros(hidden)
    for slot in range(top_k):
        gu_gpu = ctx.q4_0_gemv(gu_d, dev(x[0]), hidden, 2 * inter, w_off=slot * gu_stride)
        ctx.sync()
        gu_gpu = gu_gpu.cpu().numpy()
        gu_ref = O.q4_0_matvec_f64(gu[slot * gu_stride:(slot + 1) * gu_stride], 2 * inter, hidden, x[0])
        assert O.max_rel_err(gu_gpu, gu_ref) < TOL
        act_ref = [O.gelu_up_f64(float(g), float(u)) for g, u in zip(gu_gpu[:inter], gu_gpu[inter:])]
        assert O.max_rel_err(act[0, slot], np.array(act_ref)) < TOL
        # the slot's down rows on their own (one routed slot, weight 1)
        dn_gpu, act1 = run_experts(ctx, pool, offs, hidden, inter, top_k, x, np.array([[slot]]),
                                   np.array([[1.0]]))
        assert np.array_equal(act1[0, 0], act[0, slot])
        dn_ref = O.q4_0_matvec_f64_xd(dn, slot * dn_stride, hidden, inter, act[0, slot].astype(np.float64))
        assert O.max_rel_err(dn_gpu[0], dn_ref) < TOL
        y_ref += dn_ref
    # merged output: three terms of up to 1e15 cancel, so the bound is relative
    # to the largest term
    assert np.max(np.abs(y[0] - y_ref)) <= 1e-5 * np.max(np.abs(y_ref))
    # end to end against the full FP64 oracle (MoESIMDOracle.reference): the activation
    # may differ by the 1e-4 of its own stage plus what the (gated) error of the gate|up
    # stage moves it: d(gelu(g)*u) <= |gelu'|*|u|*dg + |gelu(g)|*du with |gelu'| < 1.13
    # and |gelu(g)| <= |g|.  With values up to 1e15 no fixed constant says that.
    ref = O.moe_experts_f64(gu, gu[up_rel:], dn, hidden, inter, [0, 1, 2], [1, 1, 1], x[0],
                            (gu_stride, gu_stride, dn_stride))
    for slot in range(top_k):
        gu_gpu = ctx.q4_0_gemv(gu_d, dev(x[0]), hidden, 2 * inter, w_off=slot * gu_stride)
        ctx.sync()
        gu_gpu = gu_gpu.cpu().numpy().astype(np.float64)
        g_ref, u_ref = ref["gate"][slot], ref["up"][slot]
        dg, du = np.abs(gu_gpu[:inter] - g_ref), np.abs(gu_gpu[inter:] - u_ref)
        slack = TOL * np.maximum(1.0, np.abs(ref["act"][slot])) + 1.2 * (np.abs(u_ref) * dg + np.abs(g_ref) * du)
        assert np.all(np.abs(act[0, slot] - ref["act"][slot]) <= slack)
    assert np.max(np.abs(y[0] - ref["y"])) <= 1e-3 * np.max(np.abs(ref["y"]))


@pytest.mark.parametrize("hidden,inter,experts,top_k,tokens", [(2048, 768, 16, 8, 1), (2048, 768, 16, 8, 5),
                                                               (2816, 704, 8, 8, 2), (256, 128, 6, 2, 3),
                                                               (64, 64, 4, 1, 1), (4096, 1024, 4, 3, 2)])
def test_moe_experts_vs_fp64(ctx, hidden, inter, experts, top_k, tokens):
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=hidden + inter)
    rng = np.random.default_rng(experts)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    y, act = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        ref = O.moe_experts_f64(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        assert O.max_rel_err(y[t], ref["y"]) < TOL
        # the reference's serial f32 CPU order on the same inputs, for scale:
        # the HIP path must not be less accurate than it
        y32, _ = O.moe_experts_f32(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(y[t], ref["y"]) <= max(TOL / 2, 1.5 * O.max_rel_err(y32, ref["y"]))


@pytest.mark.parametrize("experts", [300, 1500, 4096])
def test_moe_grouped_path_many_experts(ctx, experts):
    """Five tokens and up group the pairs by expert: the per-expert offsets are an
    exclusive scan over up to 4096 counts, cut into four experts per thread and
    sixteen waves.  Expert counts beyond one wave's 256, beyond several waves and
    at the 4096 limit (whose total is the one entry past the last thread's share),
    with the last expert and experts of every wave routed."""
    hidden, inter, top_k, tokens = 256, 256, 4, 6
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=experts)
    rng = np.random.default_rng(experts)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    ids[0, 0], ids[1, 1], ids[2, 2] = experts - 1, 0, experts // 2
    ids[3] = [experts - 1, experts - 2, 1, experts // 3]            # the last expert twice in the batch
    for t in range(tokens):
        assert len(set(ids[t].tolist())) == top_k
    wts = rng.random((tokens, top_k)).astype(np.float32)
    y, act = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        ref = O.moe_experts_f64(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        assert O.max_rel_err(y[t], ref["y"]) < TOL


@pytest.mark.parametrize("experts,tokens,again", [(16, 2100, 64), (1500, 2100, 2080), (1500, 1400, 64), (40, 36, 20)])
def test_moe_grouped_path_many_tokens(ctx, experts, tokens, again):
    """Many tokens through the grouped path.  More than five and a half pairs per expert on average take the
    fp16 kernels: with 16 experts every expert takes many passes of twelve columns over its weights,
    with 1500 the scan over the expert counts crosses waves.  Fewer pairs per expert take the
    integer kernels (1400 tokens over 1500 experts: work items of one to eight pairs, those of more
    than four in front of the others; 36 tokens of which most go to two experts: several whole
    items per expert).  Sampled tokens against the FP64 chain, and the first `again` tokens as a
    batch of their own, on the same kernels, bit for bit: a pair's result does not depend on the
    batch."""
    hidden, inter, top_k = 256, 256, 4
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=experts + 7)
    rng = np.random.default_rng(experts + 7)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    ids[0, 0], ids[1, 1] = experts - 1, 0
    if experts == 40:
        # experts 3 and 4 in nearly every token: 30 and 27 pairs -> three whole items and a remainder
        for t in range(tokens):
            if t % 6 != 5:
                ids[t] = [3, 5 + t % 30, 4 if t % 10 else 36, 37 + t % 3]
        for t in range(tokens):
            assert len(set(ids[t].tolist())) == top_k
    # which kernels a batch takes (integer matrix cores up to 5.5 pairs per expert on average)
    assert (2 * tokens * top_k <= 11 * experts) == (2 * again * top_k <= 11 * experts)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    y, act = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in list(range(0, tokens, 97 if tokens > 100 else 5)) + [1, tokens - 1]:
        ref = O.moe_experts_f64(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        assert O.max_rel_err(y[t], ref["y"]) < TOL
    y2, act2 = run_experts(ctx, pool, offs, hidden, inter, experts, x[:again], ids[:again], wts[:again])
    assert np.array_equal(y2.view(np.uint32), y[:again].view(np.uint32))
    assert np.array_equal(act2.view(np.uint32), act[:again].view(np.uint32))


@pytest.mark.parametrize("experts,tokens,top_k", [(16, 2, 2), (16, 6, 2), (4, 12, 2)])
def test_moe_non_finite_activation_stays_in_its_token(ctx, experts, tokens, top_k):
    """A NaN or an infinity in one token's activations makes every output of THAT token non-finite
    (as the reference's f32 dot products do: each of them contains the element) and leaves the
    other tokens' bits alone, on the per-pair kernels (2 tokens), the integer grouped kernels
    (6 tokens over 16 experts) and the fp16 grouped kernels (12 tokens over 4 experts)."""
    hidden, inter = 256, 256
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=91 + tokens)
    rng = np.random.default_rng(91 + tokens)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    y_good, _ = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    assert np.isfinite(y_good).all()
    for bad_value, where in ((np.float32(np.nan), 77), (np.float32(np.inf), 3), (np.float32(-np.inf), 255)):
        xb = x.copy()
        xb[1, where] = bad_value
        y, _ = run_experts(ctx, pool, offs, hidden, inter, experts, xb, ids, wts)
        assert not np.isfinite(y[1]).any(), (bad_value, where)
        for t in range(tokens):
            if t != 1:
                assert np.array_equal(y[t].view(np.uint32), y_good[t].view(np.uint32)), (bad_value, t)


@pytest.mark.parametrize("experts,tokens,top_k", [(16, 2, 2), (16, 6, 2), (4, 12, 2)])
def test_moe_block_scale_edge_cases(ctx, experts, tokens, top_k):
    """Block scales the synthetic pools do not draw: zero, negative, the smallest fp16 subnormal
    and a large one, sprinkled over every matrix, and activations spanning forty-six binades within a
    row; the three schedules (per-pair, integer grouped, fp16 grouped) against the FP64 chain."""
    hidden, inter = 256, 256
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=311 + tokens)
    pool = pool.copy()
    d = np.ascontiguousarray(pool.reshape(-1, 18)[:, 0:2]).view(np.float16).reshape(-1)   # one scale per block
    n = d.size
    d[0:n:7] = np.float16(0.0)
    d[3:n:11] = -d[3:n:11]
    d[5:n:13] = np.float16(5.96e-8)                                     # 2^-24: the smallest subnormal
    d[6:n:17] = np.float16(0.0625)
    pool.reshape(-1, 18)[:, 0:2] = d.view(np.uint8).reshape(-1, 2)
    x = x.copy()
    x[:, 0::5] *= np.float32(2.0 ** -40)
    x[:, 1::9] *= np.float32(2.0 ** 6)
    rng = np.random.default_rng(311 + tokens)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    y, act = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    g, u, dwn = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        ref = O.moe_experts_f64(g, u, dwn, hidden, inter, ids[t], wts[t], x[t])
        assert np.isfinite(ref["y"]).all()
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        # y sums f32 activations of mixed sign and size 1e3: the reference's own f32 chain is off by up
        # to 5e-4 of small outputs here; the HIP path must stay within the gate or within that chain's error
        y32, _ = O.moe_experts_f32(g, u, dwn, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(y[t], ref["y"]) <= max(TOL, 1.5 * O.max_rel_err(y32, ref["y"]))


@pytest.mark.parametrize("hidden,inter", [(1280, 512), (1536, 1280), (1792, 256), (768, 1792), (2048, 2048)])
def test_moe_grouped_integer_kernels_wave_geometries(ctx, hidden, inter):
    """The integer grouped kernels give a wave one 256-value column task of its row groups: rows of
    three, five, six, seven and eight tasks, whose workgroups hold five to twelve waves in one to
    four row-group slots (gate/up over hidden, down over the intermediate size).  Seven tokens over
    six experts; one expert takes six pairs (a second product), one a single pair."""
    experts, top_k, tokens = 6, 2, 7
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=hidden + inter)
    ids = np.array([[0, 1], [0, 2], [0, 3], [0, 4], [0, 1], [0, 2], [5, 3]], dtype=np.int32)
    rng = np.random.default_rng(hidden + inter)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    assert 2 * tokens * top_k <= 11 * experts            # the integer kernels' share of the grouped path
    y, act = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        ref = O.moe_experts_f64(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        assert O.max_rel_err(y[t], ref["y"]) < TOL


@pytest.mark.parametrize("experts,top_k,tokens", [(40, 12, 6), (9, 1, 40), (24, 8, 5)])
def test_moe_grouped_integer_kernels_fused_layout_and_top_k(ctx, experts, top_k, tokens):
    """The integer grouped kernels on the reference's fused gate|up tensor ([2I, H] per expert: the up
    rows of an expert lie behind its gate rows, both strides are the fused record's size) and with
    more and fewer slots per token than eight: twelve (the merge and the duplicate check take the
    slots in runs of eight), one, and five tokens, the fewest the grouped path takes."""
    hidden, inter = 512, 256
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=experts + top_k)
    gu = offs["gate_stride"]
    g, u, d = (pool[offs["gate_off"]:offs["up_off"]], pool[offs["up_off"]:offs["down_off"]], pool[offs["down_off"]:])
    fused = np.concatenate([np.concatenate([g[e * gu:(e + 1) * gu], u[e * gu:(e + 1) * gu]]) for e in range(experts)])
    pool2 = np.concatenate([fused, d])
    offs2 = dict(gate_off=0, up_off=gu, down_off=fused.size, gate_stride=2 * gu, up_stride=2 * gu,
                 down_stride=offs["down_stride"])
    rng = np.random.default_rng(experts + top_k)
    ids = np.stack([rng.permutation(experts)[:top_k] for _ in range(tokens)]).astype(np.int32)
    wts = rng.random((tokens, top_k)).astype(np.float32)
    assert tokens >= 5 and 2 * tokens * top_k <= 11 * experts
    y, act = run_experts(ctx, pool2, offs2, hidden, inter, experts, x, ids, wts)
    y_packed, act_packed = run_experts(ctx, pool, offs, hidden, inter, experts, x, ids, wts)
    assert np.array_equal(y.view(np.uint32), y_packed.view(np.uint32))          # the layout does not show
    assert np.array_equal(act.view(np.uint32), act_packed.view(np.uint32))
    for t in range(tokens):
        ref = O.moe_experts_f64(g, u, d, hidden, inter, ids[t], wts[t], x[t])
        assert O.max_rel_err(act[t], ref["act"]) < TOL
        assert O.max_rel_err(y[t], ref["y"]) < TOL


def test_moe_grouped_path_rejects_bad_expert_ids(ctx):
    """The same rule on the many-token path: a pair whose id is out of range or repeats another
    slot of its token is dropped (it adds nothing to its token) and reported; the other tokens
    are computed."""
    from leviathan_amd import capi, ops
    from leviathan_amd.ops import LevError
    hidden, inter, experts, top_k, tokens = 256, 256, 8, 2, 6
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=11)
    good = np.array([[0, 1], [2, 3], [4, 5], [6, 7], [1, 2], [3, 4]], np.int32)
    wts = np.full((tokens, top_k), 0.5, np.float32)
    y_good, _ = run_experts(ctx, pool, offs, hidden, inter, experts, x, good, wts)
    for bad_row in ([5, 5], [1, 9], [-1, 2]):
        ids = good.copy()
        ids[2] = bad_row
        pool_d = dev(pool)
        pools = ops.Context.moe_pools(pool_d, hidden, inter, experts, offs["gate_off"], offs["up_off"], offs["down_off"])
        y = ctx.moe_experts_q4_0(pools, dev(x), dev(ids), dev(wts), top_k, tokens)
        with pytest.raises(LevError) as e:
            ctx.sync()
        assert e.value.status == capi.BAD_DIMENSIONS
        y = y.cpu().numpy()
        for t in (0, 1, 3, 4, 5):
            assert np.array_equal(y[t].view(np.uint32), y_good[t].view(np.uint32))
        assert np.all(np.isfinite(y[2]))


def test_moe_rejects_bad_expert_ids(ctx):
    """MoEModelBinding.offsets (MoEModelBinding.swift:174-214): ids must be in
    range and distinct; nothing is written through a bad id."""
    from leviathan_amd import capi
    from leviathan_amd.ops import LevError
    wr, pool, offs, x = H.config5(64, 64, 4, 1, seed=3)
    for bad in ([[0, 0]], [[1, 9]], [[-1, 2]]):
        run_y = None
        with pytest.raises(LevError) as e:
            run_y = run_experts(ctx, pool, offs, 64, 64, 4, x, np.array(bad), np.array([[0.5, 0.5]]))
        assert e.value.status == capi.BAD_DIMENSIONS and run_y is None
    y, _ = run_experts(ctx, pool, offs, 64, 64, 4, x, np.array([[2, 1]]), np.array([[0.5, 0.5]]))
    assert np.all(np.isfinite(y))                                   # the context recovers


@pytest.mark.parametrize("tokens", [1, 64])
def test_moe_layer_config5(ctx, tokens):
    """128 experts, top-8, hidden 2048, intermediate 768, T in {1, 64}."""
    from leviathan_amd import ops
    hidden, inter, experts, top_k = 2048, 768, 128, 8
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens)
    pool_d = dev(pool)
    pools = ops.Context.moe_pools(pool_d, hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                  offs["down_off"])
    y, ids, wts = ctx.moe_layer_q4_0(pools, dev(wr), dev(x), top_k, tokens)
    ctx.sync()
    y, ids, wts = y.cpu().numpy(), ids.cpu().numpy(), wts.cpu().numpy()
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        ref_scores, ref_ids, ref_w = cpu_route(wr, x[t], top_k)
        order = np.sort(ref_scores)[::-1]
        assert float(np.min(np.diff(-order[:top_k + 1]))) > 1e-5, "degenerate seed"
        H.check_moe_layer_token(y[t], ids[t], wts[t], ref_ids, ref_w, g, u, d, hidden, inter, x[t], TOL)
    # batch invariance (main.swift:9053-9056: a schedule gives the same bits whatever
    # else is in the batch).  Three schedules exist here: up to four tokens every
    # (token, slot) streams its expert alone; from five tokens pairs are grouped
    # by expert on the matrix cores, by the integer kernels up to 5.5 pairs per
    # expert on average (64 and 8 tokens over 128 experts both) and by the fp16
    # kernels beyond.  Within a schedule a token's bits do not depend on the rest
    # of the batch; across schedules the same token agrees to the
    # summation-order noise.
    if tokens > 1:
        y8, _, _ = ctx.moe_layer_q4_0(pools, dev(wr), dev(x[:8]), top_k, 8)
        y1, _, _ = ctx.moe_layer_q4_0(pools, dev(wr), dev(x[:1]), top_k, 1)
        ctx.sync()
        assert np.array_equal(y8.cpu().numpy()[0].view(np.uint32), y[0].view(np.uint32))
        assert O.max_rel_err(y1.cpu().numpy()[0], y[0].astype(np.float64)) < TOL


@pytest.mark.parametrize("hidden,inter,experts,top_k,tokens", [(1024, 256, 8, 2, 1), (256, 256, 16, 3, 4),
                                                             (512, 256, 70, 5, 2), (256, 256, 200, 8, 3),
                                                             (1024, 256, 8, 2, 9), (256, 256, 40, 4, 20),
                                                             (256, 256, 4, 2, 40), (512, 512, 3, 1, 30)])
def test_moe_layer_small_and_odd_expert_counts(ctx, hidden, inter, experts, top_k, tokens):
    """The whole block (router in the gate/up kernel up to four tokens, separate
    selection kernel above) for expert counts well below and between the table
    sizes the selection is instantiated for; the last two give every expert more
    tokens than one pass of the grouped kernel takes."""
    from leviathan_amd import ops
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=experts + tokens)
    pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                  offs["down_off"])
    y, ids, wts = ctx.moe_layer_q4_0(pools, dev(wr), dev(x), top_k, tokens)
    ctx.sync()
    y, ids, wts = y.cpu().numpy(), ids.cpu().numpy(), wts.cpu().numpy()
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    for t in range(tokens):
        _, ref_ids, ref_w = cpu_route(wr, x[t], top_k)
        H.check_moe_layer_token(y[t], ids[t], wts[t], ref_ids, ref_w, g, u, d, hidden, inter, x[t], TOL)


# ---------------------------------------------------------- prefill GEMM ----

def gemm(ctx, w, x16, rows, cols, tokens):
    y = torch.full((tokens, rows), float("nan"), device="cuda")
    ctx.q4_k_gemm_prefill(dev(w), dev(x16), cols, rows, tokens, y=y)
    ctx.sync()
    return y.cpu().numpy()


@pytest.mark.parametrize("rows,cols,tokens", [(128, 256, 32), (96, 512, 64), (200, 1024, 37),
                                              (33, 256, 1), (256, 4096, 300),
                                              # either side of the 96-row x 256-token workgroup tile
                                              (97, 256, 257), (95, 512, 255), (192, 256, 256), (289, 768, 511)])
def test_gemm_small_shapes_every_row(ctx, rows, cols, tokens):
    w, x = H.config4(rows, cols, tokens, seed=rows + tokens)
    got = gemm(ctx, w, x, rows, cols, tokens)
    ref = O.q4_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(got, ref) < GEMM_TOL


def test_gemm_config4_full_size_sampled_rows(ctx):
    """lev-cli main.rs:1266-1278: every 13th row, every token, gate 1e-3."""
    rows, cols, tokens = 12288, 4096, 512
    w, x = H.config4(rows, cols, tokens)
    got = gemm(ctx, w, x, rows, cols, tokens)
    assert np.all(np.isfinite(got))
    ref = O.q4_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 13)
    assert O.max_rel_err(got[:, 0::13], ref) < GEMM_TOL
    # linearity over the whole output: 2X gives exactly 2Y (power-of-two scaling)
    got2 = gemm(ctx, w, (x * np.float16(2)), rows, cols, tokens)
    assert np.array_equal(got2.view(np.uint32), (got * 2).view(np.uint32))


def test_f32_to_f16_then_gemm_matches_direct(ctx):
    """act_f16 (coopmat.rs:49) in front of the GEMM, as the prefill path runs it."""
    rows, cols, tokens = 64, 512, 16
    w = O.synth_q4_k(8, rows * cols // 256)
    x32 = O.normal(tokens * cols, 9).reshape(tokens, cols)
    x16 = ctx.f32_to_f16(dev(x32))
    ctx.sync()
    assert np.array_equal(x16.cpu().numpy().view(np.uint16), x32.astype(np.float16).view(np.uint16))
    y = ctx.q4_k_gemm_prefill(dev(w), x16, cols, rows, tokens)
    ctx.sync()
    ref = O.q4_k_gemm_f16_oracle(w, rows, cols, x32.astype(np.float16).view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(y.cpu().numpy(), ref) < GEMM_TOL


# --------------------------------------------------- Q6_K prefill GEMM ----

def gemm6(ctx, w, x16, rows, cols, tokens, w_off=0):
    y = torch.full((tokens, rows), float("nan"), device="cuda")
    ctx.q6_k_gemm_prefill(dev(w), dev(x16), cols, rows, tokens, y=y, w_off=w_off)
    ctx.sync()
    return y.cpu().numpy()


def config4_q6(rows, cols, tokens, seed):
    w = O.synth_q6_k(seed, rows * cols // 256, 0.01)
    x = O.normal(tokens * cols, seed + 1000).astype(np.float16).reshape(tokens, cols)
    return w, x


@pytest.mark.parametrize("rows,cols,tokens", [(128, 256, 128), (64, 512, 32), (200, 1024, 37), (33, 256, 1),
                                              # either side of the 128-row x 256-token workgroup tile
                                              (129, 256, 129), (127, 512, 127), (256, 768, 256),
                                              (300, 4096, 150), (97, 1280, 257), (260, 256, 300)])
def test_q6_gemm_small_shapes_every_row(ctx, rows, cols, tokens):
    """coopmat.rs:333-425 against the gate of lev-cli main.rs:1201-1217 (W and X
    rounded to fp16, f64 accumulation), every row and token."""
    w, x = config4_q6(rows, cols, tokens, seed=rows + tokens)
    got = gemm6(ctx, w, x, rows, cols, tokens)
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(got, ref) < GEMM_TOL


def test_q6_gemm_weights_at_a_2_byte_offset(ctx):
    """GGUF aligns Q6_K tensors to 2 bytes only (210-byte blocks)."""
    rows, cols, tokens = 96, 512, 48
    w, x = config4_q6(rows, cols, tokens, seed=77)
    shifted = np.concatenate([np.zeros(2, np.uint8), w])
    got = gemm6(ctx, shifted, x, rows, cols, tokens, w_off=2)
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert O.max_rel_err(got, ref) < GEMM_TOL


def test_q6_gemm_lm_head_size_sampled_rows(ctx):
    """The 32000 x 4096 head at 256 tokens: every 13th row (lev-cli main.rs:1266-1278,
    gate 1e-3), and exact linearity under a power-of-two scaling of X."""
    rows, cols, tokens = 32000, 4096, 256
    w, x = config4_q6(rows, cols, tokens, seed=6)
    got = gemm6(ctx, w, x, rows, cols, tokens)
    assert np.all(np.isfinite(got))
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 13)
    assert O.max_rel_err(got[:, 0::13], ref) < GEMM_TOL
    got2 = gemm6(ctx, w, (x * np.float16(2)), rows, cols, tokens)
    assert np.array_equal(got2.view(np.uint32), (got * 2).view(np.uint32))


def test_q6_gemm_token_tiles_taken_in_turn(ctx):
    """More workgroup tiles than CUs with the row tiles alone nearly filling the chip: a workgroup
    takes its rows' token tiles one after the other (three here, the last one ragged).  Every tile
    is the product the kernel forms when that tile is the whole call, bit for bit, and sampled rows
    meet the gate."""
    rows, cols, tokens = 32000, 4096, 600
    w, x = config4_q6(rows, cols, tokens, seed=16)
    got = gemm6(ctx, w, x, rows, cols, tokens)
    assert np.all(np.isfinite(got))
    for lo, hi in ((0, 256), (256, 512), (512, 600)):
        part = gemm6(ctx, w, x[lo:hi].copy(), rows, cols, hi - lo)
        assert np.array_equal(part.view(np.uint32), got[lo:hi].view(np.uint32)), (lo, hi)
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 97)
    assert O.max_rel_err(got[:, 0::97], ref) < GEMM_TOL
    # two token tiles side by side, four in turn (100 row tiles x 8 token tiles on 256 CUs)
    rows, cols, tokens = 12800, 1024, 2000
    w, x = config4_q6(rows, cols, tokens, seed=17)
    got = gemm6(ctx, w, x, rows, cols, tokens)
    for lo, hi in ((0, 256), (768, 1024), (1792, 2000)):
        part = gemm6(ctx, w, x[lo:hi].copy(), rows, cols, hi - lo)
        assert np.array_equal(part.view(np.uint32), got[lo:hi].view(np.uint32)), (lo, hi)
    ref = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 211)
    assert O.max_rel_err(got[:, 0::211], ref) < GEMM_TOL


def test_q6_gemm_one_token_matches_the_gemv_within_rounding(ctx):
    """One token through the GEMM against the f64 GEMV oracle on the same fp16
    activations: the only difference is the fp16 rounding of W (2^-11 relative
    per weight)."""
    rows, cols = 160, 2048
    w, x = config4_q6(rows, cols, 1, seed=12)
    got = gemm6(ctx, w, x, rows, cols, 1)[0]
    ref = O.q6_k_matvec_f64(w, rows, cols, x[0].astype(np.float32))
    mag = np.abs(O.q6_k_dequant(w).reshape(rows, cols).astype(np.float64)) @ np.abs(x[0].astype(np.float64))
    assert np.all(np.abs(got - ref) <= 2.0 ** -10 * mag)


def test_q6_gemm_rejects_bad_arguments(ctx):
    from leviathan_amd import ops
    w, x = config4_q6(32, 256, 4, seed=3)
    with pytest.raises(ops.LevError):
        ctx.q6_k_gemm_prefill(dev(w), dev(x), 255, 32, 4)            # in_dim not a multiple of 256
    with pytest.raises(ops.LevError):
        ctx.q6_k_gemm_prefill(dev(w), dev(x), 256, 33, 4)            # weights too short for 33 rows
    with pytest.raises(ops.LevError):
        ctx.q6_k_gemm_prefill(dev(w), dev(x), 256, 32, 5)            # x too short for 5 tokens
    with pytest.raises(ops.LevError):
        ctx.q6_k_gemm_prefill(dev(w), dev(x), 256, 32, 0)


@pytest.mark.parametrize("kind", ["q4_k", "q6_k"])
def test_gemm_weights_are_exactly_the_fp16_rounded_decode(ctx, kind):
    """X = identity reads the fp16 weights the kernel multiplies with back out:
    they must be the f32 decode rounded once to fp16 (coopmat.rs:236-323, 333-425),
    exactly, wide scale range included."""
    rows, cols = 70, 512
    if kind == "q4_k":
        w = O.synth_q4_k(31, rows * cols // 256, 0.3)
        want = O.q4_k_dequant(w)
        run = gemm
    else:
        w = O.synth_q6_k(32, rows * cols // 256, 0.3)
        want = O.q6_k_dequant(w)
        run = gemm6
    want16 = want.reshape(rows, cols).astype(np.float16).astype(np.float32)
    x = np.eye(cols, dtype=np.float16)
    got = run(ctx, w, x, rows, cols, cols)            # [cols tokens][rows]
    assert np.array_equal(got.T, want16)              # as values: the sign of a zero weight is immaterial
