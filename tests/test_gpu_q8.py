"""GPU parity of the int8-activation decode path through the C ABI.

* quantiser (emit_quantize / emit_norm_quant, rust/crates/lev-forge/src/q8.rs:20-51,
  127-164): codes, scales and sums bit-exact against the oracle's quantize_q8
  (lev-cpu/src/lib.rs:306-322), also behind the RMSNorm and the residual add;
* Q4_K x int8 GEMV (emit_q4k_q8, q8.rs:191-326): gated as the reference's
  `vk-q8` command does (lev-cli/src/main.rs:1788-1868): max|got-ref|/max(1,|ref|)
  < 1e-4 against matvec_q4k_q8_f64 on the SAME quantised activations.
"""
import numpy as np
import pytest
import torch

import oracle as O
from tests import helpers as H

pytestmark = pytest.mark.gpu

GATE = 1e-4          # lev-cli/src/main.rs:12


@pytest.fixture(scope="module")
def ctx():
    from leviathan_amd import ops
    c = ops.Context(0)
    yield c
    c.close()


def dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def oracle_quant(x2d):
    qs, ds, ss = [], [], []
    for row in x2d:
        q, d, s = O.quantize_q8(row)
        qs.append(q), ds.append(d), ss.append(s)
    return np.stack(qs), np.stack(ds), np.stack(ss)


def gpu_quant(ctx, x2d, gain=None, add=None, want_y=False, eps=1e-6):
    ncol, n = x2d.shape
    xd = dev(x2d)
    out = ctx.norm_quant_q8(xd, n, ncol, gain=None if gain is None else dev(gain), eps=eps,
                            add=None if add is None else dev(add), want_y=want_y)
    ctx.sync()
    res = [t.cpu().numpy() for t in out]
    return res, xd.cpu().numpy()


def check_quant(got, x2d):
    q, d, s = oracle_quant(x2d)
    assert np.array_equal(got[0], q)
    assert np.array_equal(got[1][..., 0].view(np.uint32), d.view(np.uint32))
    assert np.array_equal(got[1][..., 1].view(np.uint32), s.view(np.uint32))


# ------------------------------------------------------------ quantiser ----

@pytest.mark.parametrize("ncol,n", [(1, 32), (1, 4096), (3, 96), (8, 4096), (2, 12288), (5, 1056)])
def test_quantize_bit_exact(ctx, ncol, n):
    x = O.signed_units(ncol * n, 0x4C455649 + n).reshape(ncol, n)
    got, _ = gpu_quant(ctx, x)
    check_quant(got, x)


def test_quantize_ties_zero_groups_and_extremes(ctx):
    x = np.zeros((2, 128), np.float32)
    # group 0: amax 127 makes id == 1: halves round to even
    x[0, :32] = np.array([127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 126.5] + [0.0] * 24, np.float32)
    # group 1 stays all zero (d = 0, codes 0)
    x[0, 64:96] = -3.0                     # every code -127
    x[0, 96:128] = np.linspace(-1e-30, 1e-30, 32, dtype=np.float32)   # tiny amax
    x[1] = O.normal(128, 9, sigma=1e4)
    got, _ = gpu_quant(ctx, x)
    check_quant(got, x)
    assert list(got[0][0, :8]) == [127, 0, 2, 2, 0, -2, -2, 126]
    assert not got[0][0, 32:64].any() and got[1][0, 1, 0] == 0.0
    assert (got[0][0, 64:96] == -127).all()


@pytest.mark.parametrize("ncol,n", [(1, 4096), (8, 4096), (3, 2048), (2, 1056)])
def test_norm_quant_matches_rmsnorm_then_quantize(ctx, ncol, n):
    x = O.normal(ncol * n, 70 + ncol, sigma=3.0).reshape(ncol, n)
    gain = (1.0 + 0.1 * O.normal(n, 71)).astype(np.float32)
    want = np.stack([O.rmsnorm(r, gain, 1e-6) for r in x])
    got, x_after = gpu_quant(ctx, x, gain=gain, want_y=True)
    assert np.array_equal(got[2].view(np.uint32), want.view(np.uint32))      # f32 output of the norm
    check_quant(got, want)
    assert np.array_equal(x_after, x)                                         # input untouched


def test_add_norm_quant_updates_the_residual_stream(ctx):
    ncol, n = 4, 4096
    x = O.normal(ncol * n, 80).reshape(ncol, n)
    delta = O.normal(ncol * n, 81, sigma=0.5).reshape(ncol, n)
    gain = (1.0 + 0.1 * O.normal(n, 82)).astype(np.float32)
    summed = (x + delta).astype(np.float32)
    want = np.stack([O.rmsnorm(r, gain, 1e-5) for r in summed])
    got, x_after = gpu_quant(ctx, x, gain=gain, add=delta, want_y=True, eps=1e-5)
    assert np.array_equal(x_after.view(np.uint32), summed.view(np.uint32))    # x += d written back
    assert np.array_equal(got[2].view(np.uint32), want.view(np.uint32))
    check_quant(got, want)


def test_fused_and_unfused_quantisation_agree_bit_for_bit(ctx):
    """docs/WINDOWS_VULKAN.md:21: the fused norm+quantize gives the activations
    of rmsnorm followed by quantize."""
    x = O.normal(2 * 4096, 90).reshape(2, 4096)
    gain = np.ones(4096, np.float32)
    fused, _ = gpu_quant(ctx, x, gain=gain)
    yd = ctx.rmsnorm(dev(x), 4096, 2, weight=dev(gain))
    ctx.sync()
    y = yd.cpu().numpy()
    # the runner's rmsnorm operator accumulates in f32; requantising ITS output
    # must agree with the oracle quantiser on those very values
    unfused, _ = gpu_quant(ctx, y)
    check_quant(unfused, y)
    same = (fused[0] == unfused[0]).mean()
    assert same > 0.999            # the two norms differ in the last bit of a few values


# ------------------------------------------------------------------ GEMV ----

def q8_gemv(ctx, w, x2d, rows, cols, gain=None):
    ncol = x2d.shape[0]
    xq, xs = ctx.norm_quant_q8(dev(x2d), cols, ncol, gain=None if gain is None else dev(gain))
    y = torch.full((ncol, rows), float("nan"), device="cuda")
    ctx.q4_k_gemv_q8(dev(w), xq, xs, cols, rows, ncol, y=y)
    ctx.sync()
    return y.cpu().numpy(), xq.cpu().numpy(), xs.cpu().numpy()


def check_gemv(got, w, rows, cols, xq, xs, tol=GATE):
    worst = 0.0
    for c in range(got.shape[0]):
        ref = O.q4_k_matvec_q8_f64(w, rows, cols, xq[c], xs[c, :, 0])
        worst = max(worst, O.max_rel_err(got[c], ref))
    assert worst < tol, worst
    return worst


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 8, 16])
def test_q4_k_q8_reference_gate_protocol(ctx, nb):
    """vk_q8 (lev-cli/src/main.rs:1788-1868): SplitMix64(0x4C455649) signed-unit
    activations, nb in {1,2,3,4,8,16}, gate 1e-4 against the q8 oracle.  The
    command reads a model tensor; here the weights are drawn from the benchmark
    distribution (d, dmin ~ |N(0, 0.01)|), whose outputs are O(1) like a model's:
    the gate divides by max(1, |ref|), so it is an absolute bound on O(1) data."""
    rows, cols = 256, 4096
    w, _, _ = H.config3(rows, cols, 1, seed=42)
    x = O.signed_units(nb * cols, 0x4C455649).reshape(nb, cols)
    got, xq, xs = q8_gemv(ctx, w, x, rows, cols)
    check_quant((xq, xs), x)
    check_gemv(got, w, rows, cols, xq, xs)
    # and the float product stays near: quantisation noise only
    for c in range(nb):
        ref = O.q4_k_matvec_f64(w, rows, cols, x[c])
        assert np.linalg.norm(got[c] - ref) < 0.02 * np.linalg.norm(ref)


@pytest.mark.parametrize("nb", [1, 16])
def test_q4_k_q8_rust_fixture_16x1024(ctx, nb):
    """The Q4_K fixture of lev-cpu/src/lib.rs:466-476 (SplitMix64(42), 16 x 1024,
    6-bit scales, d up to 0.25: outputs in the hundreds) under int8 activations."""
    rng = O.SplitMix64(42)
    w = H.rust_q4_k_blocks(rng, 16 * 4)
    x = np.array([rng.next_signed_unit() for _ in range(nb * 1024)], np.float32).reshape(nb, 1024)
    got, xq, xs = q8_gemv(ctx, w, x, 16, 1024)
    check_gemv(got, w, 16, 1024, xq, xs)


@pytest.mark.parametrize("ncol", [1, 2, 5, 7, 16])
@pytest.mark.parametrize("rows,cols", [(37, 1024), (9, 256), (20, 12288), (130, 4352)])
def test_q4_k_q8_shapes(ctx, rows, cols, ncol):
    w, x, gain = H.config3(rows, cols, ncol, seed=rows + ncol)
    got, xq, xs = q8_gemv(ctx, w, x, rows, cols, gain)
    check_gemv(got, w, rows, cols, xq, xs)


@pytest.mark.parametrize("family", [0, 1])
@pytest.mark.parametrize("rows,cols,ncol", [(37, 1024, 1), (130, 4352, 3), (20, 12288, 8), (64, 4096, 16),
                                            (5000, 4096, 12), (16, 16384, 5), (40, 28672, 4)])
def test_q4_k_q8_both_kernels_every_column_count(ctx, rows, cols, ncol, family):
    """A forge selection pins the kernel: family 1 the integer matrix-core kernels
    (built-in choice from 4 columns, and for every column count of rows up to 4096 wide, where
    a wave per superblock column serves up to four columns), 0 the dot4 kernel (built-in for
    fewer columns of wider rows); both meet the gate everywhere.  5000 rows give a wave more than three tasks (the looping
    variant); 28672 columns exceed the unrolled staging of the matrix-core kernel
    (its tail loops)."""
    from leviathan_amd import capi
    cands = ctx.forge_candidates(capi.OP_Q4_K_GEMV_Q8, cols, rows, ncol)
    assert sorted(c.family for c in cands) == [0, 1]
    assert cands[0].family == (1 if ncol >= 4 or cols <= 4096 else 0)          # candidate 0 is the built-in choice
    ctx.forge_select(cols, rows, [c for c in cands if c.family == family][0], ncol)
    try:
        w, x, gain = H.config3(rows, cols, ncol, seed=rows + ncol)
        got, xq, xs = q8_gemv(ctx, w, x, rows, cols, gain)
        check_gemv(got, w, rows, cols, xq, xs)
    finally:
        ctx.forge_clear(capi.OP_Q4_K_GEMV_Q8, cols, rows, ncol)


def test_q4_k_q8_hand_block(ctx):
    """One block, d = 1, dmin = 0.5, scales j+1, mins j, codes (i mod 16):
    with x = 1 everywhere (q = 127, d = 1/127) the product is the plain sum of
    the dequantised weights."""
    blk = np.zeros(144, np.uint8)
    blk[0:2] = np.frombuffer(np.float16(1.0).tobytes(), np.uint8)
    blk[2:4] = np.frombuffer(np.float16(0.5).tobytes(), np.uint8)
    blk[4:16] = O.q4_k_pack_scale_min(np.arange(1, 9, dtype=np.uint8), np.arange(8, dtype=np.uint8))
    lo = np.arange(32) % 16
    blk[16:] = np.tile((lo | (((lo + 3) % 16) << 4)).astype(np.uint8), 4)
    x = np.ones((1, 256), np.float32)
    got, xq, xs = q8_gemv(ctx, blk, x, 1, 256)
    want = float(O.q4_k_dequant_block_f64(blk).sum())
    assert (xq == 127).all()
    assert abs(got[0, 0] - want) <= 1e-4 * max(1.0, abs(want))
    check_gemv(got, blk, 1, 256, xq, xs)


@pytest.mark.parametrize("ncol", [1, 2, 4, 8, 16])
def test_q4_k_q8_config3_full_size(ctx, ncol):
    w, x, gain = H.config3(ncol=ncol)
    got, xq, xs = q8_gemv(ctx, w, x, 12288, 4096, gain)
    check_gemv(got, w, 12288, 4096, xq, xs)
    # columns never mix: column 0 computed alone agrees (same bits while both runs
    # use the same kernel and column count template; wider calls order the sums
    # differently)
    alone = torch.empty((1, 12288), device="cuda")
    ctx.q4_k_gemv_q8(dev(w), dev(xq[:1]), dev(xs[:1]), 4096, 12288, 1, y=alone)
    ctx.sync()
    alone = alone.cpu().numpy()[0]
    if ncol <= 2:
        assert np.array_equal(alone.view(np.uint32), got[0].view(np.uint32))
    else:   # each within the gate of the oracle, hence within twice the gate of each other
        assert O.max_rel_err(alone, O.q4_k_matvec_q8_f64(w, 12288, 4096, xq[0], xs[0, :, 0])) < GATE
        assert O.max_rel_err(alone, got[0].astype(np.float64)) < 2 * GATE


def test_q4_k_q8_weight_offset(ctx):
    rows, cols = 64, 1024
    w, x, _ = H.config3(rows, cols, 2, seed=5)
    pad = np.zeros(144 * 3, np.uint8)
    xq, xs = ctx.norm_quant_q8(dev(x), cols, 2)
    base = ctx.q4_k_gemv_q8(dev(w), xq, xs, cols, rows, 2)
    shifted = ctx.q4_k_gemv_q8(dev(np.concatenate([pad, w])), xq, xs, cols, rows, 2, w_off=pad.size)
    ctx.sync()
    assert torch.equal(base, shifted)


# ------------------------------------------------------------ Q6_K x int8 ----

def q6_q8_gemv(ctx, w, x2d, rows, cols):
    ncol = x2d.shape[0]
    xq, xs = ctx.norm_quant_q8(dev(x2d), cols, ncol)
    y = torch.full((ncol, rows), float("nan"), device="cuda")
    ctx.q6_k_gemv_q8(dev(w), xq, xs, cols, rows, ncol, y=y)
    ctx.sync()
    return y.cpu().numpy(), xq.cpu().numpy(), xs.cpu().numpy()


def check_q6(got, w, rows, cols, xq, xs):
    for c in range(got.shape[0]):
        ref = O.q6_k_matvec_q8_f64(w, rows, cols, xq[c], xs[c, :, 0])
        assert O.max_rel_err(got[c], ref) < GATE, c


@pytest.mark.parametrize("nb", [1, 2, 3, 4, 8, 16])
def test_q6_k_q8_reference_gate_protocol(ctx, nb):
    """vk_q8 on a Q6_K tensor (lev-cli/src/main.rs:1788-1868), seed and gate as above."""
    rows, cols = 200, 4096
    w = O.synth_q6_k(6, rows * cols // 256)
    x = O.signed_units(nb * cols, 0x4C455649).reshape(nb, cols)
    got, xq, xs = q6_q8_gemv(ctx, w, x, rows, cols)
    check_q6(got, w, rows, cols, xq, xs)
    for c in range(nb):
        ref = O.q6_k_matvec_f64(w, rows, cols, x[c])
        assert np.linalg.norm(got[c] - ref) < 0.02 * np.linalg.norm(ref)


@pytest.mark.parametrize("rows,cols,ncol", [(37, 1024, 1), (9, 256, 3), (20, 12288, 8), (130, 4352, 5),
                                            (11, 8192, 16)])
def test_q6_k_q8_shapes(ctx, rows, cols, ncol):
    w = O.synth_q6_k(rows + ncol, rows * cols // 256)
    x = O.normal(ncol * cols, 7 + rows).reshape(ncol, cols)
    got, xq, xs = q6_q8_gemv(ctx, w, x, rows, cols)
    check_q6(got, w, rows, cols, xq, xs)


def test_q6_k_q8_hand_block_and_saturated_codes(ctx):
    """The hand-computed -315 block of main.swift:1091-1112 (its activations are
    powers of two times +-1: every code is +-127 and q*d is x to one rounding),
    and blocks of all-ones bytes (codes 63, scales -1)."""
    blk, x = H.minus_315_block()
    got, xq, xs = q6_q8_gemv(ctx, blk, x[None], 1, 256)
    assert abs(got[0, 0] + 315.0) <= 1e-4 * 315.0
    check_q6(got, blk, 1, 256, xq, xs)
    sat = np.full(210 * 4, 0xFF, np.uint8)
    sat[208::210], sat[209::210] = 0x00, 0x3C          # d = 1.0
    x = O.signed_units(2 * 512, 3).reshape(2, 512)
    got, xq, xs = q6_q8_gemv(ctx, sat, x, 2, 512)
    check_q6(got, sat, 2, 512, xq, xs)


def test_q6_k_q8_lm_head_full_size(ctx):
    w, x = H.config2()
    x2 = np.stack([x, x[::-1].copy()])
    got, xq, xs = q6_q8_gemv(ctx, w, x2, 32000, 4096)
    check_q6(got, w, 32000, 4096, xq, xs)


# ------------------------------------------------------- SwiGLU + quantise ----

@pytest.mark.parametrize("n", [32, 4096, 3 * 11008 - 3 * 11008 % 32])
def test_swiglu_quant(ctx, n):
    g = O.normal(n, 21, sigma=2.0)
    u = O.normal(n, 22)
    g[:4] = [0.0, -100.0, 100.0, -0.0]
    xq, xs, act = ctx.swiglu_quant_q8(dev(g), dev(u), want_act=True)
    ctx.sync()
    act = act.cpu().numpy()
    g64, u64 = g.astype(np.float64), u.astype(np.float64)
    want = g64 / (1.0 + np.exp(-g64)) * u64               # silu(g) * u, lev-model/src/lib.rs:120, 240
    assert np.all(np.abs(act - want) <= 1e-6 * np.maximum(1.0, np.abs(want)))
    # the codes are the quantiser's, bit for bit, on the f32 activations the kernel formed
    check_quant((xq.cpu().numpy()[None], xs.cpu().numpy()[None]), act[None])


def test_q8_guards(ctx):
    from leviathan_amd import capi
    from leviathan_amd.ops import LevError
    x = dev(np.zeros(2 * 256, np.float32))
    for kw, status in [
        (dict(n=100, ncol=1), capi.BAD_DIMENSIONS),
        (dict(n=0, ncol=1), capi.BAD_DIMENSIONS),
        (dict(n=256, ncol=0), capi.BAD_DIMENSIONS),
        (dict(n=256, ncol=3), capi.WRONG_INPUT_COUNT),
    ]:
        with pytest.raises(LevError) as e:
            ctx.norm_quant_q8(x, **kw)
        assert e.value.status == status, kw
    w = dev(np.zeros(144 * 4, np.uint8))
    xq, xs = ctx.norm_quant_q8(x, 256, 2)
    for kw, status in [
        (dict(in_dim=100, rows=4, ncol=1), capi.BAD_DIMENSIONS),
        (dict(in_dim=256, rows=5, ncol=1), capi.BAD_DIMENSIONS),
        (dict(in_dim=256, rows=4, ncol=3), capi.WRONG_INPUT_COUNT),
        (dict(in_dim=256, rows=4, ncol=0), capi.BAD_DIMENSIONS),
        (dict(in_dim=256, rows=4, ncol=17), capi.BAD_DIMENSIONS),
    ]:
        with pytest.raises(LevError) as e:
            ctx.q4_k_gemv_q8(w, xq, xs, **kw)
        assert e.value.status == status, kw
