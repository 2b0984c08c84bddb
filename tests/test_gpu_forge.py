"""GPU: schedule candidates and per-shape selection behind the matvec entry points.

The library side of the forge loop (schedule::derive, lev-forge/src/schedule.rs:83-105;
selection rule lev-cli/src/main.rs:1977-2022).  Every candidate must pass the
reference's gate max|y - oracle| / max(1, |oracle|) < 1e-4 on the forge's own
input (SplitMix64(0x4C455649) signed units); candidate 0 is the built-in choice;
a selection changes which kernel runs for exactly one shape and nothing else.
"""
import numpy as np
import pytest
import torch

import oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

GATE = 1e-4
FORGE_SEED = 0x4C455649


@pytest.fixture(scope="module")
def ctx():
    from leviathan_amd import ops
    c = ops.Context(0)
    yield c
    c.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("rows,cols,expected", [(4096, 4096, 8), (300, 2048, 8), (40000, 4096, 8),
                                                (512, 1088, 6), (64, 256, 3), (16, 8192, 3), (16, 16384, 1)])
def test_q4_0_candidates_pass_the_gate_and_agree_bitwise(ctx, rows, cols, expected):
    from leviathan_amd import capi
    w = O.synth_q4_0(rows + cols, rows * cols // 32, 0.02)
    x = O.signed_units(cols, FORGE_SEED)
    ref = O.q4_0_matvec_f64(w, rows, cols, x)
    dw, dx = dev(w), dev(x)
    cands = ctx.forge_candidates(capi.OP_Q4_0_GEMV, cols, rows)
    assert len(cands) == expected
    assert len({c.key() for c in cands}) == len(cands)
    # rows of whole 256-value tasks up to 8192 wide: the matrix-core kernel (family 1) first, with one
    # workgroup per round of row groups or a resident grid; behind it the vector-ALU kernels (family 0)
    mfma = cols % 256 == 0 and cols <= 8192
    assert [c.family for c in cands[:2]] == ([1, 1] if mfma else [0, 0][:len(cands)])
    builtin = ctx.q4_0_gemv(dw, dx, cols, rows).cpu().numpy()
    ctx.sync()
    assert O.max_rel_err(builtin, ref) < GATE
    outs = {}
    try:
        for i, s in enumerate(cands):
            ctx.forge_select(cols, rows, s)
            y = torch.full((rows,), float("nan"), device="cuda")
            ctx.q4_0_gemv(dw, dx, cols, rows, y=y)
            ctx.sync()
            got = y.cpu().numpy()
            assert O.max_rel_err(got, ref) < GATE, s.key()
            # within a family a row is summed by the same lanes in the same order whatever the tiling
            first = outs.setdefault(s.family, got)
            assert np.array_equal(got.view(np.uint32), first.view(np.uint32)), s.key()
    finally:
        ctx.forge_clear(capi.OP_Q4_0_GEMV, cols, rows)
    assert np.array_equal(builtin.view(np.uint32), outs[cands[0].family].view(np.uint32))
    if len(outs) > 1:   # two different kernels: a selection really switches
        assert not np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))


@pytest.mark.parametrize("rows,cols,ncol", [(1024, 4096, 1), (512, 1024, 3), (96, 256, 8), (256, 4096, 16)])
def test_q4_k_candidates_pass_the_gate(ctx, rows, cols, ncol):
    from leviathan_amd import capi
    w = O.synth_q4_k(rows + ncol, rows * cols // 256, 0.01)
    x = O.signed_units(cols * ncol, FORGE_SEED).reshape(ncol, cols)
    ref = np.stack([O.q4_k_matvec_f64(w, rows, cols, x[c]) for c in range(ncol)])
    dw, dx = dev(w), dev(x)
    cands = ctx.forge_candidates(capi.OP_Q4_K_GEMV, cols, rows, ncol)
    # the integer matrix-core kernel (exact sums) is the built-in choice wherever its staging fits
    assert [c.family for c in cands] == [1, 0]
    outs = []
    try:
        for s in cands:
            ctx.forge_select(cols, rows, s, ncol)
            y = torch.full((ncol, rows), float("nan"), device="cuda")
            ctx.q4_k_gemv_ncol(dw, dx, cols, rows, ncol, y=y)
            ctx.sync()
            outs.append(y.cpu().numpy())
            assert O.max_rel_err(outs[-1], ref) < GATE, s.key()
    finally:
        ctx.forge_clear(capi.OP_Q4_K_GEMV, cols, rows, ncol)
    # the two families are different kernels: a selection really switches
    assert not np.array_equal(outs[0].view(np.uint32), outs[1].view(np.uint32))
    again = ctx.q4_k_gemv_ncol(dw, dx, cols, rows, ncol).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), outs[0].view(np.uint32))   # cleared: built-in again


@pytest.mark.parametrize("rows,cols,expected", [(500, 4096, [(0, 2), (0, 1), (1, 1)]), (300, 2048, [(0, 1), (1, 1)]),
                                                (64, 8192, [(0, 1), (1, 1)]), (40, 12288, [(1, 1)])])
def test_q6_k_candidates_pass_the_gate(ctx, rows, cols, expected):
    """vk_q6k (lev-cli/src/main.rs:467): the head's candidates, the forge's own input and gate.
    With the argmax epilogue on: every candidate names the same token."""
    from leviathan_amd import capi
    w = O.synth_q6_k(rows + cols, rows * cols // 256)
    x = O.signed_units(cols, FORGE_SEED)
    ref = O.q6_k_matvec_f64(w, rows, cols, x)
    dw, dx = dev(w), dev(x)
    cands = ctx.forge_candidates(capi.OP_Q6_K_GEMV, cols, rows)
    # the matrix-core kernel first, with its built-in number of waves per row group, then with
    # 2 and 4 where those differ; behind it the kernels it replaced as the built-in choice
    listed = [(c.family, c.rows_in_flight) for c in cands]
    # rows of at most sixteen superblocks: the kernel with a wave per superblock column leads the list
    head = [(2, 0)] if cols <= 4096 else []
    assert listed[:len(head)] == head
    listed = listed[len(head):]
    assert listed[0][0] == 2 and listed[0][1] in (2, 4, 8, 16)
    assert listed == [listed[0]] + [(2, n) for n in (2, 4) if n != listed[0][1]] + expected
    outs = []
    try:
        for s in cands:
            ctx.forge_select(cols, rows, s)
            y, idx, margin = ctx.q6_k_gemv(dw, dx, cols, rows, argmax=True)
            ctx.sync()
            outs.append(y.cpu().numpy())
            assert O.max_rel_err(outs[-1], ref) < GATE, s.key()
            assert int(idx.item()) == O.argmax(outs[-1]), s.key()
    finally:
        ctx.forge_clear(capi.OP_Q6_K_GEMV, cols, rows)
    again = ctx.q6_k_gemv(dw, dx, cols, rows).cpu().numpy()
    assert np.array_equal(again.view(np.uint32), outs[0].view(np.uint32))   # cleared: built-in again
    if len(outs) > 1:   # the f64-sum kernel is a different kernel: a selection really switches
        assert not np.array_equal(outs[0].view(np.uint32), outs[-1].view(np.uint32))


@pytest.mark.parametrize("rows,cols,ncol,expected", [(200, 4096, 1, [(1, 1), (1, 0)]),
                                                      (96, 1024, 4, [(4, 1), (4, 0), (2, 1)]),
                                                      (130, 4352, 5, [(8, 1), (8, 0), (4, 1)])])
def test_q6_k_q8_candidates_pass_the_gate_and_agree_bitwise(ctx, rows, cols, ncol, expected):
    from leviathan_amd import capi
    w = O.synth_q6_k(rows + ncol, rows * cols // 256)
    x = O.signed_units(cols * ncol, FORGE_SEED).reshape(ncol, cols)
    dw = dev(w)
    xq, xs = ctx.norm_quant_q8(dev(x), cols, ncol)
    ctx.sync()
    hq, hs = xq.cpu().numpy(), xs.cpu().numpy()
    ref = np.stack([O.q6_k_matvec_q8_f64(w, rows, cols, hq[c], hs[c, :, 0]) for c in range(ncol)])
    cands = ctx.forge_candidates(capi.OP_Q6_K_GEMV_Q8, cols, rows, ncol)
    # the matrix-core kernel first (all columns in one pass), then the dot4 kernel's grids and passes
    assert [(c.family, c.rows_in_flight, c.persistent) for c in cands] == \
        [(1, ncol, 1)] + [(0, n, p) for n, p in expected]
    outs = []
    try:
        for s in cands:
            ctx.forge_select(cols, rows, s, ncol)
            y = torch.full((ncol, rows), float("nan"), device="cuda")
            ctx.q6_k_gemv_q8(dw, xq, xs, cols, rows, ncol, y=y)
            ctx.sync()
            outs.append(y.cpu().numpy())
            assert O.max_rel_err(outs[-1], ref) < GATE, s.key()
            # within a kernel family a row is summed by the same lanes in the same order whatever
            # the grid or the pass
            if s.family == 0:
                assert np.array_equal(outs[-1].view(np.uint32), outs[1].view(np.uint32)), s.key()
    finally:
        ctx.forge_clear(capi.OP_Q6_K_GEMV_Q8, cols, rows, ncol)


@pytest.mark.parametrize("hidden,inter,experts,top_k,tokens", [(2048, 768, 128, 8, 1), (512, 256, 20, 4, 3)])
def test_moe_layer_candidates_pass_the_gate_and_agree_bitwise(ctx, hidden, inter, experts, top_k, tokens):
    """MoELoweringForge.forge (MoELowering.swift:1896-1985): every candidate of the layer
    routes to the same experts and gives the same bits; the composite is gated at 1e-4."""
    from leviathan_amd import capi, ops
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=experts + tokens)
    pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                  offs["down_off"])
    dwr, dx = dev(wr), dev(x)
    g, u, d = (pool[offs["gate_off"]:], pool[offs["up_off"]:], pool[offs["down_off"]:])
    cands = ctx.forge_candidates(capi.OP_MOE_LAYER_Q4_0, hidden, inter, tokens)
    assert [(c.family, c.rows_in_flight, c.persistent) for c in cands] == [(1, 2, 0), (1, 1, 0), (1, 4, 0), (2, 2, 0),
                                                                           (0, 2, 0), (1, 2, 1)]
    outs = []
    try:
        for s in cands:
            ctx.forge_select(hidden, inter, s, tokens)
            y, ids, wts = ctx.moe_layer_q4_0(pools, dwr, dx, top_k, tokens)
            ctx.sync()
            outs.append((y.cpu().numpy(), ids.cpu().numpy(), wts.cpu().numpy()))
            for t in range(tokens):
                scores = O.f32_matvec(wr, experts, hidden, x[t])
                ref_ids, ref_w = O.router_topk(scores, top_k, None)
                H.check_moe_layer_token(outs[-1][0][t], outs[-1][1][t], outs[-1][2][t], ref_ids, ref_w, g, u, d,
                                        hidden, inter, x[t], GATE)
            # same routing whatever the schedule; the same expert kernels give the same bits; the
            # vector-ALU kernels (persistent = 1) round their sums differently
            assert np.array_equal(outs[-1][1], outs[0][1]) and np.array_equal(outs[-1][2].view(np.uint32),
                                                                              outs[0][2].view(np.uint32))
            if s.persistent == 0:
                assert np.array_equal(outs[-1][0].view(np.uint32), outs[0][0].view(np.uint32)), s.key()
    finally:
        ctx.forge_clear(capi.OP_MOE_LAYER_Q4_0, hidden, inter, tokens)
    with pytest.raises(ops.LevError):
        ctx.forge_candidates(capi.OP_MOE_LAYER_Q4_0, hidden, inter, 5)     # the grouped path has one schedule
    with pytest.raises(ops.LevError):
        ctx.forge_select(hidden, inter, capi.Schedule(capi.OP_MOE_LAYER_Q4_0, 1, 3, 0), tokens)
    with pytest.raises(ops.LevError):
        ctx.forge_select(hidden, inter, capi.Schedule(capi.OP_MOE_LAYER_Q4_0, 3, 2, 0), tokens)


def test_selection_applies_to_one_shape_only(ctx):
    from leviathan_amd import capi
    cols, ncol = 1024, 1
    w = O.synth_q4_k(9, 512 * cols // 256, 0.01)
    x = O.signed_units(cols, 3)
    dw, dx = dev(w), dev(x)
    base_256 = ctx.q4_k_gemv_ncol(dw, dx, cols, 256, ncol).cpu().numpy()
    base_512 = ctx.q4_k_gemv_ncol(dw, dx, cols, 512, ncol).cpu().numpy()
    other = ctx.forge_candidates(capi.OP_Q4_K_GEMV, cols, 256)[1]      # not the built-in choice
    ctx.forge_select(cols, 256, other)
    try:
        sel_256 = ctx.q4_k_gemv_ncol(dw, dx, cols, 256, ncol).cpu().numpy()
        sel_512 = ctx.q4_k_gemv_ncol(dw, dx, cols, 512, ncol).cpu().numpy()
    finally:
        ctx.forge_clear(capi.OP_Q4_K_GEMV, cols, 256)
    assert not np.array_equal(sel_256.view(np.uint32), base_256.view(np.uint32))
    assert np.array_equal(sel_512.view(np.uint32), base_512.view(np.uint32))


def test_selection_misuse_is_rejected(ctx):
    from leviathan_amd import capi, ops
    with pytest.raises(ops.LevError):
        ctx.forge_select(4096, 512, capi.Schedule(capi.OP_Q4_0_GEMV, 0, 3, 0))       # no such depth
    with pytest.raises(ops.LevError):
        ctx.forge_select(4096, 512, capi.Schedule(capi.OP_Q4_0_GEMV, 1, 1, 0))       # no such family
    with pytest.raises(ops.LevError):
        ctx.forge_select(4096, 512, capi.Schedule(9, 0, 1, 0))                       # no such op
    with pytest.raises(ops.LevError):
        ctx.forge_candidates(capi.OP_Q4_K_GEMV, 100, 8)                              # not a Q4_K row
    with pytest.raises(ops.LevError):
        ctx.forge_candidates(capi.OP_Q4_0_GEMV, 4096, 8, 2)                          # Q4_0 GEMV is single-column
    ctx.forge_clear(capi.OP_Q4_0_GEMV, 4096, 512)                                    # clearing nothing is fine
