"""A recorded decode-like step (record once, replay; Program / Step,
rust/crates/lev-vulkan/src/engine.rs:94-141; deferred segments,
Sources/LeviathanCore/Gemma4.swift:2313-2376) over the int8 path and the MoE
layer: every replay, with new device-resident inputs and eager work and
synchronisations in between, must reproduce the eager step bit for bit.

The step: embed(token) -> rmsnorm+quantise -> Q4_K x int8 (gate|up) ->
swiglu+quantise -> Q4_K x int8 (down) -> residual add + rmsnorm + quantise ->
MoE layer on the f32 stream -> Q6_K x int8 head -> argmax.
"""
import ctypes as C

import numpy as np
import pytest
import torch

import oracle as O

pytestmark = pytest.mark.gpu

DIM, FF, VOCAB, HEAD = 1024, 1024, 64, 96
EXPERTS, TOPK, INTER = 8, 2, 256


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def p(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def test_recorded_step_replays_bit_exact():
    from leviathan_amd import ops
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, stream=stream)
    lib, c = ctx.lib, ctx.ctx

    def must(st):
        if st:
            raise RuntimeError(lib.lev_hip_last_error(c).decode())

    table = dev(O.synth_q4_k(1, VOCAB * DIM // 256))
    w_gu = dev(O.synth_q4_k(2, 2 * FF * DIM // 256))
    w_dn = dev(O.synth_q4_k(3, DIM * FF // 256))
    w_head = dev(O.synth_q6_k(4, HEAD * DIM // 256))
    gain = dev((1.0 + 0.1 * O.normal(DIM, 5)).astype(np.float32))
    gu_bytes, dn_bytes = INTER * (DIM // 32) * 18, DIM * (INTER // 32) * 18
    pool = dev(np.concatenate([O.synth_q4_0(6, EXPERTS * gu_bytes // 18), O.synth_q4_0(7, EXPERTS * gu_bytes // 18),
                               O.synth_q4_0(8, EXPERTS * dn_bytes // 18)]))
    pools = ops.Context.moe_pools(pool, DIM, INTER, EXPERTS, 0, EXPERTS * gu_bytes, 2 * EXPERTS * gu_bytes)
    router = dev(O.normal(EXPERTS * DIM, 9, 0.0, 0.02).reshape(EXPERTS, DIM))

    with torch.cuda.stream(stream):
        tok = torch.zeros(1, dtype=torch.int32, device="cuda")
        x = torch.empty(1, DIM, device="cuda")
        xq = torch.empty(1, max(DIM, FF), dtype=torch.int8, device="cuda")
        xs = torch.empty(1, max(DIM, FF) // 32, 2, device="cuda")
        gu = torch.empty(2 * FF, device="cuda")
        dn = torch.empty(1, DIM, device="cuda")
        ymoe = torch.empty(1, DIM, device="cuda")
        ids = torch.empty(1, TOPK, dtype=torch.int32, device="cuda")
        wts = torch.empty(1, TOPK, device="cuda")
        logits = torch.empty(1, HEAD, device="cuda")
        best = torch.empty(1, dtype=torch.int32, device="cuda")
        margin = torch.empty(1, device="cuda")

    def step():
        must(lib.lev_hip_embed_q4_k(c, p(table), table.numel(), 0, p(tok), 1, p(x), x.numel(), DIM, VOCAB))
        must(lib.lev_hip_norm_quant_q8(c, p(x), DIM, None, p(gain), 1e-6, p(xq), p(xs), None, DIM, 1))
        must(lib.lev_hip_q4_k_gemv_q8(c, p(w_gu), w_gu.numel(), 0, p(xq), p(xs), DIM, p(gu), gu.numel(), DIM, 2 * FF, 1))
        must(lib.lev_hip_swiglu_quant_q8(c, p(gu), C.c_void_p(gu.data_ptr() + 4 * FF), FF, p(xq), p(xs), None))
        must(lib.lev_hip_q4_k_gemv_q8(c, p(w_dn), w_dn.numel(), 0, p(xq), p(xs), FF, p(dn), dn.numel(), FF, DIM, 1))
        must(lib.lev_hip_norm_quant_q8(c, p(x), DIM, p(dn), p(gain), 1e-6, p(xq), p(xs), None, DIM, 1))   # x += dn
        must(lib.lev_hip_moe_layer_q4_0(c, C.byref(pools), p(router), None, p(x), p(ymoe), p(ids), p(wts), TOPK, 1))
        must(lib.lev_hip_axpy(c, p(ymoe), p(x), 1.0, DIM))
        must(lib.lev_hip_q6_k_gemv_q8(c, p(w_head), w_head.numel(), 0, p(xq), p(xs), DIM, p(logits), logits.numel(),
                                      DIM, HEAD, 1))
        must(lib.lev_hip_argmax(c, p(logits), HEAD, 1, p(best), p(margin)))

    def snapshot():
        ctx.sync()
        return [t.clone() for t in (x, xq, xs, gu, dn, ymoe, ids, wts, logits, best, margin)]

    def set_token(t):
        with torch.cuda.stream(stream):
            tok.fill_(t)

    # eager runs (the first also sizes the MoE scratch, which may not grow while recording)
    eager = {}
    for t in (3, 41, 17, 63):
        set_token(t)
        step()
        eager[t] = snapshot()
    assert not torch.equal(eager[3][8], eager[41][8])           # the step depends on its token

    ctx.program_begin()
    step()
    prog = ctx.program_end()
    assert prog.node_count() >= 10
    for t in (41, 3, 63, 17, 41):
        set_token(t)
        prog.run()
        got = snapshot()
        for a, b in zip(got, eager[t]):
            assert torch.equal(a, b), t
        # the program's own eager work between replays
        set_token((t * 7) % VOCAB)
        step()
        ctx.sync()
    prog.destroy()
    ctx.close()


@pytest.mark.parametrize("experts", [12, 16])
def test_recorded_prefill_like_sequence_replays_bit_exact(experts):
    """f32 -> f16, the two prefill GEMMs (first use of the kernels happens while recording),
    grouped MoE over 24 tokens (72 pairs: over 12 experts the fp16 grouped kernels, over 16 the
    integer ones with their work items and start records), and a Q4_0 GEMV under a forge selection
    made before recording: three replays with changed inputs equal the eager results bit for bit."""
    from leviathan_amd import capi, ops
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, stream=stream)
    lib, c = ctx.lib, ctx.ctx

    def must(st):
        if st:
            raise RuntimeError(lib.lev_hip_last_error(c).decode())

    T, K, R = 24, 512, 200
    hidden, inter, top_k = 512, 256, 3
    wk = dev(O.synth_q4_k(11, R * K // 256))
    w6 = dev(O.synth_q6_k(17, R * K // 256))
    w0 = dev(O.synth_q4_0(12, 300 * 2048 // 32))
    gu_bytes, dn_bytes = inter * (hidden // 32) * 18, hidden * (inter // 32) * 18
    pool = dev(np.concatenate([O.synth_q4_0(13, experts * gu_bytes // 18), O.synth_q4_0(14, experts * gu_bytes // 18),
                               O.synth_q4_0(15, experts * dn_bytes // 18)]))
    pools = ops.Context.moe_pools(pool, hidden, inter, experts, 0, experts * gu_bytes, 2 * experts * gu_bytes)
    router = dev(O.normal(experts * hidden, 16, 0.0, 0.02).reshape(experts, hidden))
    with torch.cuda.stream(stream):
        x32 = torch.empty(T, K, device="cuda")
        x16 = torch.empty(T, K, dtype=torch.float16, device="cuda")
        yg = torch.empty(T, R, device="cuda")
        yg6 = torch.empty(T, R, device="cuda")
        ymoe = torch.empty(T, hidden, device="cuda")
        ids = torch.empty(T, top_k, dtype=torch.int32, device="cuda")
        wts = torch.empty(T, top_k, device="cuda")
        xv = torch.empty(2048, device="cuda")
        yv = torch.empty(300, device="cuda")

    def fill(seed):
        with torch.cuda.stream(stream):
            x32.copy_(dev(O.normal(T * K, seed).reshape(T, K)), non_blocking=False)
            xv.copy_(dev(O.normal(2048, seed + 1)))

    def step():
        must(lib.lev_hip_f32_to_f16(c, p(x32), p(x16), T * K))
        must(lib.lev_hip_q4_k_gemm_prefill(c, p(wk), wk.numel(), 0, p(x16), x16.numel(), p(yg), yg.numel(), K, R, T))
        must(lib.lev_hip_q6_k_gemm_prefill(c, p(w6), w6.numel(), 0, p(x16), x16.numel(), p(yg6), yg6.numel(), K, R, T))
        must(lib.lev_hip_moe_layer_q4_0(c, C.byref(pools), p(router), None, p(x32), p(ymoe), p(ids), p(wts), top_k, T))
        must(lib.lev_hip_q4_0_gemv(c, p(w0), w0.numel(), 0, p(xv), 2048, p(yv), 300, 2048, 300))

    def snapshot():
        ctx.sync()
        return [t.clone() for t in (x16, yg, yg6, ymoe, ids, wts, yv)]

    # the MoE scratch is sized by an eager MoE call (it may not grow while recording);
    # the GEMM has NOT run yet: its first launch is the recorded one
    fill(1)
    must(lib.lev_hip_moe_layer_q4_0(c, C.byref(pools), p(router), None, p(x32), p(ymoe), p(ids), p(wts), top_k, T))
    ctx.sync()
    cands = ctx.forge_candidates(capi.OP_Q4_0_GEMV, 2048, 300)
    ctx.forge_select(2048, 300, cands[-1])                       # not the built-in choice
    ctx.program_begin()
    step()
    prog = ctx.program_end()
    for seed in (5, 9, 5):
        fill(seed)
        prog.run()
        got = snapshot()
        step()                                                   # eager, same inputs
        want = snapshot()
        for a, b in zip(got, want):
            assert torch.equal(a, b), seed
    # and the results are right, not merely repeatable
    ref = O.q4_k_gemm_f16_oracle(wk.cpu().numpy(), R, K, x16.cpu().numpy().view(np.uint16), T, 0, 1)
    assert O.max_rel_err(yg.cpu().numpy(), ref) < 1e-3
    ref6 = O.q6_k_gemm_f16_oracle(w6.cpu().numpy(), R, K, x16.cpu().numpy().view(np.uint16), T, 0, 1)
    assert O.max_rel_err(yg6.cpu().numpy(), ref6) < 1e-3
    assert O.max_rel_err(yv.cpu().numpy(), O.q4_0_matvec_f64(w0.cpu().numpy(), 300, 2048, xv.cpu().numpy())) < 1e-4
    ctx.forge_clear(capi.OP_Q4_0_GEMV, 2048, 300)
    prog.destroy()
    ctx.close()


def test_scratch_growth_after_recording_keeps_the_program_valid():
    """A recorded single-token MoE program holds the context's scratch address.  A
    later eager call that needs more scratch (700 tokens, grouped path: several MiB against the first MiB) must not
    free that buffer under the program: the replay still gives the eager bits.  And a
    shape that would have to grow the scratch WHILE recording is refused, recording
    nothing for it."""
    from leviathan_amd import capi, ops
    from tests import helpers as H
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, stream=stream)
    hidden, inter, experts, top_k = 512, 256, 16, 4
    wr, pool, offs, x = H.config5(hidden, inter, experts, 700, seed=31)
    pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"], offs["down_off"])
    wr_d = dev(wr)
    with torch.cuda.stream(stream):
        x1, y1 = dev(x[:1]), torch.empty(1, hidden, device="cuda")
        ids1 = torch.empty(1, top_k, dtype=torch.int32, device="cuda")
        w1 = torch.empty(1, top_k, device="cuda")
        xb = dev(x)
        yB, idsB = torch.empty(700, hidden, device="cuda"), torch.empty(700, top_k, dtype=torch.int32, device="cuda")
        wB = torch.empty(700, top_k, device="cuda")
    ctx.moe_layer_q4_0(pools, wr_d, x1, top_k, 1, y=y1, ids=ids1, weights=w1)      # sizes the scratch for one token
    ctx.sync()
    want = y1.clone()
    ctx.program_begin()
    ctx.moe_layer_q4_0(pools, wr_d, x1, top_k, 1, y=y1, ids=ids1, weights=w1)
    # 700 tokens need far more scratch than one: refused while recording
    with pytest.raises(ops.LevError) as e:
        ctx.moe_layer_q4_0(pools, wr_d, xb, top_k, 700, y=yB, ids=idsB, weights=wB)   # nothing allocated here
    assert e.value.status == capi.EXCEEDS_WORKING_SET
    prog = ctx.program_end()
    # eager call that grows the scratch while the program is alive
    yb, _, _ = ctx.moe_layer_q4_0(pools, wr_d, xb, top_k, 700)
    ctx.sync()
    for _ in range(3):
        with torch.cuda.stream(stream):
            y1.fill_(float("nan"))
        prog.run()
        ctx.sync()
        assert torch.equal(y1, want)
        yb2, _, _ = ctx.moe_layer_q4_0(pools, wr_d, xb, top_k, 700)               # eager work on the new scratch in between
        ctx.sync()
        assert torch.equal(yb2, yb)
    prog.destroy()
    ctx.close()


def test_q4_k_eight_columns_record_with_and_without_scratch():
    """Five to eight f32 columns of Q4_K make their digit planes in the context's scratch.  Recorded on a context
    that never ran anything (no scratch yet, and nothing may be allocated while recording) the launch takes the kernel
    that stages per workgroup; recorded once the scratch exists it takes the planes kernel and the program holds the
    scratch address, which a later eager call that grows the scratch must not free.  Same bits every way."""
    from leviathan_amd import ops
    from tests import helpers as H
    rows, cols, ncol = 333, 2048, 8
    w, x, gain = H.config3(rows, cols, ncol, seed=77)
    results = []
    for warm in (False, True):
        stream = torch.cuda.Stream()
        ctx = ops.Context(0, stream=stream)
        with torch.cuda.stream(stream):
            w_d, x_d, g_d = dev(w), dev(x), dev(gain)
            y = torch.empty(ncol, rows, device="cuda")
        if warm:
            ctx.q4_k_gemv_ncol(w_d, x_d, cols, rows, ncol, gain=g_d, y=y)      # sizes the scratch
            ctx.sync()
        ctx.program_begin()
        ctx.q4_k_gemv_ncol(w_d, x_d, cols, rows, ncol, gain=g_d, y=y)
        prog = ctx.program_end()
        # an eager call that needs more scratch than the planes while the program is alive
        hidden, inter, experts, top_k = 512, 256, 16, 4
        wr, pool, offs, xm = H.config5(hidden, inter, experts, 300, seed=5)
        pools = ops.Context.moe_pools(dev(pool), hidden, inter, experts, offs["gate_off"], offs["up_off"], offs["down_off"])
        with torch.cuda.stream(stream):
            wr_d, xm_d = dev(wr), dev(xm)
        ym, _, _ = ctx.moe_layer_q4_0(pools, wr_d, xm_d, top_k, 300)
        ctx.sync()
        for _ in range(3):
            with torch.cuda.stream(stream):
                y.fill_(float("nan"))
            prog.run()
            ctx.sync()
            results.append(y.cpu().numpy().copy())
            ym2, _, _ = ctx.moe_layer_q4_0(pools, wr_d, xm_d, top_k, 300)      # eager work on the scratch in between
            ctx.sync()
            assert torch.equal(ym2, ym)
        with torch.cuda.stream(stream):
            y.fill_(float("nan"))
        ctx.q4_k_gemv_ncol(w_d, x_d, cols, rows, ncol, gain=g_d, y=y)          # eager: the planes kernel
        ctx.sync()
        results.append(y.cpu().numpy().copy())
        prog.destroy()
        ctx.close()
    xn = H.rmsnorm_rows(x, gain)
    for c in range(ncol):
        assert O.max_rel_err(results[0][c], O.q4_k_matvec_f64(w, rows, cols, xn[c])) < 1e-4, c
    for r in results[1:]:
        assert np.array_equal(r.view(np.uint32), results[0].view(np.uint32))


def test_q6_k_argmax_records_on_a_fresh_context():
    """The greedy-token epilogue needs no grow-on-demand scratch: a GEMV with argmax can be
    recorded on a context that never ran anything eagerly."""
    from leviathan_amd import ops
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, stream=stream)
    rows, cols = 640, 1024
    w = O.synth_q6_k(21, rows * cols // 256)
    xv = O.normal(cols, 22)
    with torch.cuda.stream(stream):
        w_d, x_d = dev(w), dev(xv)
        y = torch.empty(rows, device="cuda")
        idx = torch.zeros(1, dtype=torch.int32, device="cuda")
        mg = torch.zeros(1, device="cuda")
    lib, c = ctx.lib, ctx.ctx
    ctx.program_begin()
    st = lib.lev_hip_q6_k_gemv(c, p(w_d), w_d.numel(), 0, p(x_d), cols, p(y), rows, cols, rows, p(idx), p(mg))
    prog = ctx.program_end()
    assert st == 0, lib.lev_hip_last_error(c).decode()
    for _ in range(2):
        prog.run()
        ctx.sync()
        got = y.cpu().numpy()
        assert O.max_rel_err(got, O.q6_k_matvec_f64(w, rows, cols, xv)) < 1e-4
        assert int(idx.item()) == O.argmax(got)
        top = np.sort(got)[::-1]
        assert abs(float(mg.item()) - float(top[0] - top[1])) <= 1e-6 * max(1.0, abs(float(top[0])))
    prog.destroy()
    ctx.close()


def test_shared_expert_ffn_recorded_program_matches_the_cpu_chain():
    """The shared expert beside the routed ones (Gemma4.swift:3742-3773) at the model's
    sizes (hidden 2048, shared intermediate 2112): rmsnorm -> gate, up into one buffer ->
    geluUp -> down -> rmsnorm, then x += shared.  Eager against the same chain on the CPU
    (FP64 matvecs and norms, f32 between the steps) at 1e-4; recorded once and replayed
    with changed inputs, with the program's own eager work in between, bit for bit."""
    from leviathan_amd import ops
    hidden, inter = 2048, 2112
    stream = torch.cuda.Stream()
    ctx = ops.Context(0, stream=stream)
    gate = O.synth_q4_0(81, inter * hidden // 32, 0.02)
    up = O.synth_q4_0(82, inter * hidden // 32, 0.02)
    down = O.synth_q4_0(83, hidden * inter // 32, 0.02)
    ffn_norm = O.normal(hidden, 84, 1.0, 0.1)
    post_norm = O.normal(hidden, 85, 1.0, 0.1)
    xs = [O.normal(hidden, 90 + i) for i in range(4)]
    dgate, dup, ddown, dfn, dpn = dev(gate), dev(up), dev(down), dev(ffn_norm), dev(post_norm)
    x = torch.zeros(hidden, device="cuda")
    resid = torch.zeros(hidden, device="cuda")
    bufs = (torch.empty(hidden, device="cuda"), torch.empty(2 * inter, device="cuda"),
            torch.empty(inter, device="cuda"), torch.empty(hidden, device="cuda"))

    def step():
        h, shared = ctx.shared_expert_ffn(x, dfn, dgate, dup, ddown, dpn, hidden, inter, bufs=bufs)
        ctx.axpy(shared, resid, 1.0, hidden)                    # x += shared (Gemma4.swift:3115)
        return h, shared

    def load(v):
        with torch.cuda.stream(stream):
            x.copy_(torch.from_numpy(v))
            resid.copy_(torch.from_numpy(v))

    def cpu_chain(v):
        h = O.rmsnorm_f64(v, ffn_norm, 1e-6).astype(np.float32)
        g = O.q4_0_matvec_f64(gate, inter, hidden, h).astype(np.float32)
        u = O.q4_0_matvec_f64(up, inter, hidden, h).astype(np.float32)
        act = np.array([O.gelu_up_f32(float(a), float(b)) for a, b in zip(g, u)], np.float32)
        d = O.q4_0_matvec_f64(down, hidden, inter, act).astype(np.float32)
        return h, g, u, act, O.rmsnorm_f64(d, post_norm, 1e-6)

    eager = []
    for v in xs:
        load(v)
        h, shared = step()
        ctx.sync()
        ref_h, ref_g, ref_u, ref_act, ref_shared = cpu_chain(v)
        assert O.max_rel_err(h.cpu().numpy(), ref_h.astype(np.float64)) < 1e-5
        gu = bufs[1].cpu().numpy()
        assert O.max_rel_err(gu[:inter], ref_g.astype(np.float64)) < 1e-4     # gate half
        assert O.max_rel_err(gu[inter:], ref_u.astype(np.float64)) < 1e-4     # up half, at its byte offset
        assert O.max_rel_err(shared.cpu().numpy(), ref_shared) < 1e-4
        assert O.max_rel_err(resid.cpu().numpy(), v.astype(np.float64) + ref_shared) < 1e-4
        eager.append([t.clone() for t in (*bufs, resid)])

    load(xs[0])
    ctx.program_begin()
    step()
    prog = ctx.program_end()
    assert prog.node_count() >= 7                               # 2 norms, 3 matvecs, geluUp, axpy
    for i in (2, 0, 3, 1, 2):
        load(xs[i])
        prog.run()
        ctx.sync()
        for a, b in zip([*bufs, resid], eager[i]):
            assert torch.equal(a, b), i
        load(xs[(i + 1) % 4])                                   # eager work between the replays
        step()
        ctx.sync()
    prog.destroy()
    with pytest.raises(ops.LevError):
        ctx.shared_expert_ffn(x, dfn, dgate, dup, ddown, dpn, hidden, 2112 - 32, bufs=bufs)   # up half unaligned
    ctx.close()
