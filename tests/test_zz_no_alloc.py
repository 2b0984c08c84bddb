"""GPU parity of the entry point that allocates nothing, lev_hip_moe_layer_q4_0_noalloc.

It must give the bits of lev_hip_moe_layer_q4_0 (ids, routing weights, output)
on two calls in a row, the second with a smaller input, because both calls
share one static device array that keeps the first call's contents.  Shapes
beyond the stated limits are refused before anything is launched.
"""
import numpy as np
import pytest
import torch

from tests import helpers as H

pytestmark = pytest.mark.gpu


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_both(ctx, pools, wr_d, x, top_k):
    tokens, hidden = x.shape
    x_d = dev(x)
    out = []
    for noalloc in (False, True):
        y = torch.full((tokens, hidden), float("nan"), device="cuda")
        ids = torch.full((tokens, top_k), -1, dtype=torch.int32, device="cuda")
        wts = torch.full((tokens, top_k), float("nan"), device="cuda")
        ctx.moe_layer_q4_0(pools, wr_d, x_d, top_k, tokens, y=y, ids=ids, weights=wts, noalloc=noalloc)
        ctx.sync()
        out.append((y.cpu().numpy(), ids.cpu().numpy(), wts.cpu().numpy()))
    return out


def test_noalloc_matches_allocating_entry_point_twice_in_a_row():
    from leviathan_amd import capi, ops
    ctx = ops.Context(0)
    try:
        hidden, inter, experts, top_k = 2048, 768, 128, 8
        wr, pool, offs, x = H.config5(hidden, inter, experts, 4, seed=77)
        pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"],
                                      offs["down_off"])
        wr_d = dev(wr)
        # first call: 4 tokens; second call: 1 token (a different one), smaller scratch footprint
        for xs in (x, x[2:3]):
            (y0, i0, w0), (y1, i1, w1) = run_both(ctx, pools, wr_d, xs, top_k)
            assert np.all(np.isfinite(y0))
            assert np.array_equal(i0, i1)
            assert np.array_equal(w0.view(np.uint32), w1.view(np.uint32))
            assert np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
        # a smaller layer after the larger one, and back
        wr2, pool2, offs2, x2 = H.config5(256, 128, 16, 2, seed=5)
        pools2 = ops.Context.moe_pools(dev(pool2), 256, 128, 16, offs2["gate_off"], offs2["up_off"],
                                       offs2["down_off"])
        (y0, i0, w0), (y1, i1, w1) = run_both(ctx, pools2, dev(wr2), x2, 3)
        assert np.array_equal(i0, i1) and np.array_equal(y0.view(np.uint32), y1.view(np.uint32))
        (y0, i0, w0), (y1, i1, w1) = run_both(ctx, pools, wr_d, x[:2], top_k)
        assert np.array_equal(i0, i1) and np.array_equal(y0.view(np.uint32), y1.view(np.uint32))

        # limits: more tokens than the entry point takes, and a scratch need beyond the static array
        x5 = np.concatenate([x, x[:1]])
        with pytest.raises(ops.LevError) as e:
            ctx.moe_layer_q4_0(pools, wr_d, dev(x5), top_k, 5, noalloc=True)
        assert e.value.status == capi.EXCEEDS_WORKING_SET
        wrb, poolb, offsb, xb = H.config5(64, 4096, 64, 4, seed=6)
        poolsb = ops.Context.moe_pools(dev(poolb), 64, 4096, 64, offsb["gate_off"], offsb["up_off"],
                                       offsb["down_off"])
        with pytest.raises(ops.LevError) as e:     # 4 * 64 * 4096 * 4 B of activations > 1 MiB
            ctx.moe_layer_q4_0(poolsb, dev(wrb), dev(xb), 64, 4, noalloc=True)
        assert e.value.status == capi.EXCEEDS_WORKING_SET
        ctx.sync()
    finally:
        ctx.close()


def test_noalloc_first_call_on_a_fresh_context_allocates_nothing_and_records():
    """The call is the FIRST thing a fresh context runs (its grow-on-demand scratch is still
    empty): device free memory is the same before and after; it can be recorded into a
    program on a context that never ran the shape, where the allocating entry point is
    refused (exceedsWorkingSet: scratch cannot grow under capture); every replay gives
    the bits of the allocating entry point."""
    from leviathan_amd import capi, ops
    hidden, inter, experts, top_k, tokens = 2048, 768, 128, 8, 2
    wr, pool, offs, x = H.config5(hidden, inter, experts, tokens, seed=78)
    pool_d, wr_d, x_d = dev(pool), dev(wr), dev(x)
    pools = ops.Context.moe_pools(pool_d, hidden, inter, experts, offs["gate_off"], offs["up_off"], offs["down_off"])

    def outputs():
        return (torch.full((tokens, hidden), float("nan"), device="cuda"),
                torch.full((tokens, top_k), -1, dtype=torch.int32, device="cuda"),
                torch.full((tokens, top_k), float("nan"), device="cuda"))

    ctx = ops.Context(0)
    try:
        y1, i1, w1 = outputs()
        torch.cuda.synchronize()
        free_before = torch.cuda.mem_get_info()[0]
        ctx.moe_layer_q4_0(pools, wr_d, x_d, top_k, tokens, y=y1, ids=i1, weights=w1, noalloc=True)
        ctx.sync()
        assert torch.cuda.mem_get_info()[0] == free_before
        first = (y1.cpu().numpy(), i1.cpu().numpy(), w1.cpu().numpy())
        assert np.all(np.isfinite(first[0]))
    finally:
        ctx.close()

    stream = torch.cuda.Stream()
    with torch.cuda.stream(stream):
        ctx = ops.Context(0, stream=stream)
        try:
            y2, i2, w2 = outputs()
            torch.cuda.synchronize()
            ctx.program_begin()
            with pytest.raises(ops.LevError) as e:      # its scratch would have to be allocated under capture
                ctx.moe_layer_q4_0(pools, wr_d, x_d, top_k, tokens, y=y2, ids=i2, weights=w2)
            assert e.value.status == capi.EXCEEDS_WORKING_SET
            ctx.moe_layer_q4_0(pools, wr_d, x_d, top_k, tokens, y=y2, ids=i2, weights=w2, noalloc=True)
            prog = ctx.program_end()
            for _ in range(3):
                y2.fill_(float("nan"))
                torch.cuda.synchronize()
                prog.run()
                ctx.sync()
                assert np.array_equal(y2.cpu().numpy().view(np.uint32), first[0].view(np.uint32))
                assert np.array_equal(i2.cpu().numpy(), first[1])
                assert np.array_equal(w2.cpu().numpy().view(np.uint32), first[2].view(np.uint32))
            prog.destroy()
            # the allocating entry point outside a recording: the same bits
            y3, i3, w3 = outputs()
            ctx.moe_layer_q4_0(pools, wr_d, x_d, top_k, tokens, y=y3, ids=i3, weights=w3)
            ctx.sync()
            assert np.array_equal(y3.cpu().numpy().view(np.uint32), first[0].view(np.uint32))
            assert np.array_equal(i3.cpu().numpy(), first[1])
        finally:
            ctx.close()
