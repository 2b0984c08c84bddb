"""Pins the CPU oracle against the reference's own known-answer tests.

Each test cites the reference test it restates (paths relative to the
dhihm/leviathan tree).  The block bytes and expected values are the ones the
reference's tests spell out; nothing here re-types the oracle's formula.
"""
import math

import numpy as np
import pytest

import oracle as O


# --------------------------------------------------------------------------
# half precision -- rust/crates/lev-cpu/src/lib.rs:410-419, 558-567
# --------------------------------------------------------------------------

def test_half_conversion_known_values():
    assert O.f16_to_f64(0x3C00) == 1.0
    assert O.f16_to_f64(0xC000) == -2.0
    assert O.f16_to_f64(0x0001) == 2.0 ** -24
    assert O.f16_to_f64(0x7BFF) == 65504.0
    assert O.f16_to_f64(0x7C00) == math.inf
    assert math.isnan(O.f16_to_f64(0x7E00))
    assert O.f16_to_f64(0x0000) == 0.0


def test_f16_round_trips_and_rounds_to_even():
    for h in [0, 1, 0x3C00, 0xBC00, 0x7BFF, 0x0400, 0x03FF, 0x3555]:
        assert O.f32_to_f16_bits(O.f16_to_f32(h)) == h
    assert O.f32_to_f16_bits(1.0 + 1.0 / 2048.0) == 0x3C00
    assert O.f32_to_f16_bits(1.0 + 3.0 / 2048.0) == 0x3C02
    assert O.f32_to_f16_bits(1e9) == 0x7C00
    assert O.f32_to_f16_bits(-0.0) == 0x8000


def test_half_conversion_matches_numpy_for_every_bit_pattern():
    """Library cross-check: numpy.float16 is IEEE binary16."""
    bits = np.arange(65536, dtype=np.uint16)
    want = bits.view(np.float16).astype(np.float64)
    got = np.array([O.f16_to_f64(int(b)) for b in bits])
    finite = np.isfinite(want)
    assert np.array_equal(got[finite], want[finite])
    assert np.array_equal(np.isnan(got), np.isnan(want))
    assert np.array_equal(got[np.isinf(want)], want[np.isinf(want)])
    rng = np.random.default_rng(0)
    vals = np.concatenate([rng.standard_normal(4000).astype(np.float32) * s
                           for s in (1e-8, 1e-4, 1.0, 300.0, 7e4)])
    with np.errstate(over="ignore"):
        want_bits = vals.astype(np.float16).view(np.uint16)
    got_bits = np.array([O.f32_to_f16_bits(float(v)) for v in vals], dtype=np.uint16)
    assert np.array_equal(got_bits, want_bits)


# --------------------------------------------------------------------------
# SplitMix64 -- Sources/LeviathanCore/RNG.swift:12-23, lev-cpu lib.rs:357-373
# --------------------------------------------------------------------------

def test_splitmix64_published_vectors():
    """First outputs of the published SplitMix64 for seeds 0 and 1234567."""
    r = O.SplitMix64(0)
    assert [r.next() for _ in range(3)] == [
        0xE220A8397B1DCDAF, 0x6E789E6AA1B965F4, 0x06C45D188009454F]
    r = O.SplitMix64(1234567)
    assert [r.next() for _ in range(5)] == [
        6457827717110365317, 3203168211198807973, 9817491932198370423,
        4593380528125082431, 16408922859458223821]


def test_splitmix64_float_conventions():
    a, b = O.SplitMix64(99), O.SplitMix64(99)
    for _ in range(200):
        raw = a.next()
        # Swift: Float(Double(next >> 11) / 2^53) * 2 - 1
        want = np.float32(np.float32(float(raw >> 11) / 9007199254740992.0) * np.float32(2.0)
                          - np.float32(1.0))
        assert np.float32(b.next_uniform()) == want
    a, b = O.SplitMix64(7), O.SplitMix64(7)
    for _ in range(200):
        raw = a.next()
        # Rust: ((next >> 40) as f32 / 2^24) * 2 - 1
        want = np.float32(np.float32(raw >> 40) / np.float32(1 << 24)) * np.float32(2.0) \
            - np.float32(1.0)
        got = np.float32(b.next_signed_unit())
        assert got == want and -1.0 <= got < 1.0


# --------------------------------------------------------------------------
# Q4_0 -- Sources/leviathan-tests/main.swift:703-746, 5106-5117
# --------------------------------------------------------------------------

def test_q4_0_known_block():
    block = [0x00, 0x3C] + list(range(16))
    expected = [float(l) - 8 for l in range(16)] + [-8.0] * 16
    dq = O.q4_0_decode_block(block)
    assert dq.shape == (32,) and np.array_equal(dq, np.array(expected, dtype=np.float32))
    half = list(block)
    half[1] = 0x38                                  # d = 0.5
    assert abs(O.q4_0_decode_block(half)[0] - 0.5 * -8) < 1e-6
    inf = list(block)
    inf[1] = 0x7C                                   # +Inf scale rejected
    with pytest.raises(O.OracleError) as e:
        O.q4_0_decode_block(inf)
    assert e.value.status == O.NON_FINITE_SCALE


def test_q4_0_matvec_2x32():
    w = [0x00, 0x3C] + [0] * 16 + [0x00, 0xBC] + [0] * 16
    x = O.seeded_input(32, 1, 7)
    sum_x = np.float32(0)
    for v in x:
        sum_x = np.float32(sum_x + v)
    y = O.q4_0_matvec_ref(w, 2, 32, x)
    assert y.shape == (2,)
    assert abs(y[0] - (-8 * sum_x)) < 1e-3
    assert abs(y[1] - (8 * sum_x)) < 1e-3
    bad = x.copy()
    bad[0] = np.nan
    with pytest.raises(O.OracleError) as e:
        O.q4_0_matvec_ref(w, 2, 32, bad)
    assert e.value.status == O.NON_FINITE_INPUT


def test_q4_0_fp64_oracle_minus_16():
    block = [0x00, 0x3C] + [(l | ((16 + l) << 4)) & 0xFF for l in range(16)]
    y = O.q4_0_matvec_f64(block, 1, 32, np.ones(32, dtype=np.float32))
    assert y[0] == -16.0
    nan_block = [0xFF, 0x7F] + [0] * 16
    with pytest.raises(O.OracleError):
        O.q4_0_matvec_f64(nan_block, 1, 32, np.ones(32, dtype=np.float32))


def test_q4_0_geometry_guards():
    """main.swift:778-796 (same guards on the CPU twin, Q4.swift:87-101)."""
    for args, status in [
        (([], 8, 33, []), O.BAD_DIMENSIONS),
        (([], 8, 32, []), O.BAD_DIMENSIONS),
        (([0] * (8 * 18), 8, 32, [0, 0, 0]), O.WRONG_INPUT_COUNT),
    ]:
        with pytest.raises(O.OracleError) as e:
            O.q4_0_matvec_ref(*args)
        assert e.value.status == status


def _dense_q4_0(w, rows, cols):
    """Independent numpy decode used for brute-force checks."""
    b = np.asarray(w, dtype=np.uint8).reshape(rows, cols // 32, 18)
    d = b[:, :, :2].copy().view(np.float16).astype(np.float64)        # [rows, nb, 1]
    q = b[:, :, 2:]
    lo = (q & 0xF).astype(np.float64) - 8
    hi = (q >> 4).astype(np.float64) - 8
    return (np.concatenate([lo, hi], axis=2) * d).reshape(rows, cols)


def test_q4_0_matvecs_agree_with_brute_force():
    rows, cols = 35, 128
    w = O.synth_q4_0(11, rows * cols // 32, 0.02)
    x = O.seeded_input(cols, 1, 101)
    dense = _dense_q4_0(w, rows, cols)
    assert np.array_equal(O.q4_0_dequant(w).reshape(rows, cols), dense.astype(np.float32))
    want = dense @ x.astype(np.float64)
    f64 = O.q4_0_matvec_f64(w, rows, cols, x)
    assert np.allclose(f64, want, rtol=1e-13, atol=1e-13)
    for got in (O.q4_0_matvec_ref(w, rows, cols, x), O.q4_0_matvec_kernel_order(w, rows, cols, x),
                O.q4_0_matvec_ref(w, rows, cols, x, threads=3)):
        assert O.max_rel_err(got, f64) < 1e-5
    assert np.array_equal(O.q4_0_matvec_ref(w, rows, cols, x),
                          O.q4_0_matvec_ref(w, rows, cols, x, threads=4))
    # MoESIMDOracle.q4MatvecFP64 agrees with Q4Oracle.matvecFP64 (main.swift:8971-8978)
    xd = O.q4_0_matvec_f64_xd(w, 0, rows, cols, x.astype(np.float64))
    assert np.all(np.abs(xd - f64) <= 1e-12 * np.maximum(1, np.abs(f64)))
    with pytest.raises(O.OracleError):                 # out-of-extent read (main.swift:8979-8984)
        O.q4_0_matvec_f64_xd(w, 18, rows, cols, x.astype(np.float64))


# --------------------------------------------------------------------------
# Q6_K -- main.swift:993-1026, 1087-1123; lev-cpu lib.rs:495-540
# --------------------------------------------------------------------------

def test_q6_k_known_levels():
    block = [0] * 210
    block[208], block[209] = 0x00, 0x3C
    for i in range(16):
        block[192 + i] = 1
    block[0] = 0x21
    block[128] = 0x03
    dq = O.q6_k_decode_block(block)
    assert dq.shape == (256,)
    assert dq[0] == 17 and dq[32] == -32 and dq[64] == -30 and dq[96] == -32 and dq[1] == -32
    block[193] = 2
    assert O.q6_k_decode_block(block)[20] == 2 * -32
    block[209] = 0x7C
    with pytest.raises(O.OracleError) as e:
        O.q6_k_decode_block(block)
    assert e.value.status == O.NON_FINITE_SCALE


def _minus_315_block():
    block = [0] * 210
    block[208], block[209] = 0x00, 0x3C
    block[192] = 3
    block[193] = 0xFD
    block[196] = 2
    block[200] = 3
    block[204] = 2
    block[0] = 0x21
    block[128] = 0x03
    block[64] = 0x21
    block[160] = 0x01
    x = np.zeros(256, dtype=np.float32)
    x[0], x[16], x[64], x[128], x[192] = 1, -1, 2, -2, 4
    return block, x


def test_q6_k_hand_computed_minus_315():
    block, x = _minus_315_block()
    assert O.q6_k_matvec_ref(block, 1, 256, x)[0] == -315.0
    assert O.q6_k_matvec_f64(block, 1, 256, x)[0] == -315.0
    assert O.q6_k_matvec_f32(block, 1, 256, x)[0] == -315.0


def test_q6k_rust_hand_block():
    block = [0] * 210
    for i in range(128):
        block[i] = 0x55
    for i in range(16):
        block[192 + i] = (i - 8) & 0xFF
    block[208], block[209] = 0x00, 0x3C
    out = O.q6_k_dequant_block_f64(block)
    for e in range(256):
        assert out[e] == (e // 16 - 8) * -27.0
    for i in range(128, 192):
        block[i] = 0b11100100
    q = O.q6k_unpack(block)
    assert q[0] == 5 - 32 and q[32] == 5 + 16 - 32 and q[64] == 5 and q[96] == 5 + 48 - 32
    assert q[128 + 64] == 5


def test_q6k_swift_and_rust_decoders_agree_and_match_f64():
    rng = O.SplitMix64(7)
    rows, cols = 3, 512
    w = np.zeros(rows * cols // 256 * 210, dtype=np.uint8)
    for b in range(rows * cols // 256):
        for i in range(208):
            w[b * 210 + i] = rng.next() & 0xFF
        w[b * 210 + 208], w[b * 210 + 209] = 0x00, 0x2C        # d = 0.0625
    x = np.array([rng.next_signed_unit() for _ in range(cols)], dtype=np.float32)
    for b in range(rows * cols // 256):
        blk = w[b * 210:(b + 1) * 210]
        assert np.array_equal(O.q6_k_decode_block(blk), O.q6_k_dequant_block_f32(blk))
    oracle = O.q6_k_matvec_f64(w, rows, cols, x)
    assert O.max_rel_err(O.q6_k_matvec_f32(w, rows, cols, x), oracle) < 1e-4
    assert O.max_rel_err(O.q6_k_matvec_ref(w, rows, cols, x), oracle) < 1e-4
    with pytest.raises(O.OracleError):
        O.q6_k_matvec_f32(w[1:], rows, cols, x)


def _dense_q6_k(w, rows, cols):
    b = np.asarray(w, dtype=np.uint8).reshape(-1, 210)
    out = np.zeros((b.shape[0], 256))
    d = b[:, 208:210].copy().view(np.float16).astype(np.float64)[:, 0]
    sc = b[:, 192:208].view(np.int8).astype(np.float64)
    for e in range(256):
        half, r = divmod(e, 128)
        grp, l = divmod(r, 32)
        ql = b[:, half * 64 + (grp & 1) * 32 + l]
        lo = (ql & 0xF) if grp < 2 else (ql >> 4)
        hi = (b[:, 128 + half * 32 + l] >> (2 * grp)) & 3
        out[:, e] = d * sc[:, e // 16] * ((lo | (hi << 4)).astype(np.float64) - 32)
    return out.reshape(rows, cols)


def test_q6_k_brute_force():
    rows, cols = 5, 512
    w = O.synth_q6_k(2, rows * cols // 256, 0.01)
    x = O.seeded_input(cols, 1, 202)
    dense = _dense_q6_k(w, rows, cols)
    assert np.array_equal(O.q6_k_dequant(w).reshape(rows, cols), dense.astype(np.float32))
    want = dense.astype(np.float32).astype(np.float64) @ x.astype(np.float64)
    assert np.allclose(O.q6_k_matvec_f64(w, rows, cols, x), want, rtol=1e-12, atol=1e-12)
    assert np.array_equal(O.q6_k_matvec_ref(w, rows, cols, x),
                          O.q6_k_matvec_ref(w, rows, cols, x, threads=2))
    # the Rust f32 GEMV split over threads (Model::matvec, lev-model lib.rs:184-199): a row's sum does not
    # depend on which thread forms it, and stays within f32 rounding of the dense f64 product
    f32 = O.q6_k_matvec_f32(w, rows, cols, x)
    assert np.array_equal(f32, O.q6_k_matvec_f32(w, rows, cols, x, threads=3))
    assert np.allclose(f32, want, rtol=1e-4, atol=1e-4)


# --------------------------------------------------------------------------
# Q4_K -- lev-cpu lib.rs:380-493
# --------------------------------------------------------------------------

def test_q4_k_scale_min_round_trip():
    rng = O.SplitMix64(7)
    for _ in range(2000):                          # draw order: sc[j] then mn[j] per j
        sc, mn = [0] * 8, [0] * 8
        for j in range(8):
            sc[j] = rng.next() % 64
            mn[j] = rng.next() % 64
        packed = O.q4_k_pack_scale_min(sc, mn)
        for j in range(8):
            assert O.q4_k_unpack_scale_min(j, packed) == (sc[j], mn[j])


def test_q4_k_hand_block():
    block = np.zeros(144, dtype=np.uint8)
    block[0:2] = [0x00, 0x3C]                      # d = 1.0
    block[2:4] = [0x00, 0x38]                      # dmin = 0.5
    block[4:16] = O.q4_k_pack_scale_min([1] * 8, [2] * 8)
    block[16:] = 0x21
    f32 = O.q4_k_dequant_block_f32(block)
    f64 = O.q4_k_dequant_block_f64(block)
    for chunk in range(4):
        for l in range(32):
            assert f64[chunk * 64 + l] == 0.0 and f64[chunk * 64 + 32 + l] == 1.0
            assert f32[chunk * 64 + l] == 0.0 and f32[chunk * 64 + 32 + l] == 1.0


_HALVES = [0x2E66, 0x3000, 0x3266, 0x2800, 0x1C00, 0x3400]


def _rust_random_q4k_blocks(rng, n):
    out = np.zeros(n * 144, dtype=np.uint8)
    for b in range(n):
        o = b * 144
        h = _HALVES[rng.next() % 6]
        out[o], out[o + 1] = h & 0xFF, h >> 8
        h = _HALVES[rng.next() % 6]
        out[o + 2], out[o + 3] = h & 0xFF, h >> 8
        for i in range(140):
            out[o + 4 + i] = rng.next() & 0xFF
    return out


def test_q4_k_matvec_f32_matches_f64_oracle():
    rng = O.SplitMix64(42)
    rows, cols = 16, 1024
    w = _rust_random_q4k_blocks(rng, rows * cols // 256)
    x = np.array([rng.next_signed_unit() for _ in range(cols)], dtype=np.float32)
    got = O.q4_k_matvec_f32(w, rows, cols, x)
    ref = O.q4_k_matvec_f64(w, rows, cols, x)
    assert O.max_rel_err(got, ref) < 1e-4
    assert np.array_equal(got, O.q4_k_matvec_f32(w, rows, cols, x, threads=3))


def _dense_q4_k(w, rows, cols):
    b = np.asarray(w, dtype=np.uint8).reshape(-1, 144)
    d = b[:, 0:2].copy().view(np.float16).astype(np.float64)[:, 0]
    dmin = b[:, 2:4].copy().view(np.float16).astype(np.float64)[:, 0]
    s = b[:, 4:16].astype(np.int64)
    out = np.zeros((b.shape[0], 256))
    for j in range(8):
        if j < 4:
            sc, mn = s[:, j] & 63, s[:, j + 4] & 63
        else:
            sc = (s[:, j + 4] & 0xF) | ((s[:, j - 4] >> 6) << 4)
            mn = (s[:, j + 4] >> 4) | ((s[:, j] >> 6) << 4)
        q = b[:, 16 + (j // 2) * 32: 16 + (j // 2) * 32 + 32]
        nib = (q & 0xF) if j % 2 == 0 else (q >> 4)
        out[:, j * 32:(j + 1) * 32] = (d * sc)[:, None] * nib - (dmin * mn)[:, None]
    return out.reshape(rows, cols)


def test_q4_k_brute_force():
    rows, cols = 6, 512
    w = O.synth_q4_k(3, rows * cols // 256, 0.01)
    x = O.seeded_input(cols, 1, 5)
    dense = _dense_q4_k(w, rows, cols)
    got = O.q4_k_matvec_f64(w, rows, cols, x)
    assert np.allclose(got, dense @ x.astype(np.float64), rtol=1e-12, atol=1e-12)
    assert np.allclose(O.q4_k_dequant(w).reshape(rows, cols), dense, rtol=3e-7, atol=1e-9)


def test_q4_k_shape_errors():
    x = np.zeros(256, dtype=np.float32)
    for args in [([], 1, 100, x[:100]), ([0] * 10, 1, 256, x), ([0] * 144, 1, 256, x[:10])]:
        with pytest.raises(O.OracleError):
            O.q4_k_matvec_f32(*args)


# --------------------------------------------------------------------------
# int8 activations -- lev-cpu lib.rs:542-557
# --------------------------------------------------------------------------

def test_q8_round_trip():
    rng = O.SplitMix64(11)
    x = np.array([np.float32(rng.next_signed_unit()) * np.float32(3.0) for _ in range(96)],
                 dtype=np.float32)
    q, d, s = O.quantize_q8(x)
    for i, v in enumerate(x):
        assert abs(np.float32(q[i]) * d[i // 32] - v) <= d[i // 32] * 0.5001
    for g in range(3):
        assert abs(s[g] - d[g] * np.float32(int(q[g * 32:(g + 1) * 32].astype(np.int32).sum()))) < 1e-5
    q, d, s = O.quantize_q8(np.zeros(32, dtype=np.float32))
    assert not q.any() and d[0] == 0.0


def test_q8_matvec_oracle_reduces_to_the_float_oracle_on_exact_codes():
    """matvec_q4k_q8_f64 / matvec_q6k_q8_f64 (lev-cpu lib.rs:324-337) are the f64
    matvec over q*d.  With integer activations whose group maximum is 127 the
    scale is exactly 1 and q*d == x, so both oracles must give the float oracle's
    answer bit for bit; halving x halves d (a power of two) and the answer."""
    rng = np.random.default_rng(5)
    x = rng.integers(-127, 128, size=512).astype(np.float32)
    x[::32] = 127.0
    q, d, s = O.quantize_q8(x)
    assert (d == 1.0).all() and np.array_equal(q.astype(np.float32), x)
    assert np.array_equal(s, x.reshape(-1, 32).sum(axis=1))
    assert np.array_equal(O.dequantize_q8(q, d), x)
    w4 = O.synth_q4_k(3, 6 * 2)
    w6 = O.synth_q6_k(4, 6 * 2)
    assert np.array_equal(O.q4_k_matvec_q8_f64(w4, 6, 512, q, d), O.q4_k_matvec_f64(w4, 6, 512, x))
    assert np.array_equal(O.q6_k_matvec_q8_f64(w6, 6, 512, q, d), O.q6_k_matvec_f64(w6, 6, 512, x))
    qh, dh, _ = O.quantize_q8(x * np.float32(0.5))
    assert np.array_equal(qh, q) and (dh == 0.5).all()
    assert np.array_equal(O.q4_k_matvec_q8_f64(w4, 6, 512, qh, dh), 0.5 * O.q4_k_matvec_f64(w4, 6, 512, x))


# --------------------------------------------------------------------------
# RMSNorm -- lev-model lib.rs:431-435; closed form; torch cross-check
# --------------------------------------------------------------------------

def test_rmsnorm_constant_vector():
    y = O.rmsnorm(np.full(8, 2.0, np.float32), np.full(8, 0.5, np.float32), 1e-6)
    assert np.all(np.abs(y - 0.5) < 1e-5)


def test_rmsnorm_variants_agree_with_torch():
    import torch
    x = O.normal(4096, 31)
    g = O.normal(4096, 32, 1.0, 0.1)
    want = torch.nn.functional.rms_norm(torch.from_numpy(x).double(), (4096,),
                                        torch.from_numpy(g).double(), 1e-6).numpy()
    assert np.allclose(O.rmsnorm_f64(x, g, 1e-6), want, rtol=1e-12, atol=1e-12)
    assert O.max_rel_err(O.rmsnorm(x, g, 1e-6), want) < 1e-6
    assert O.max_rel_err(O.rmsnorm_f32_serial(x, g, 1e-6), want) < 1e-5
    assert O.max_rel_err(O.rmsnorm_f32_serial(x, None, 1e-6),
                         O.rmsnorm_f64(x, None, 1e-6)) < 1e-5
    # closed form: y . y / n == 1 for unit gain when eps is negligible
    y = O.rmsnorm_f64(x, None, 0.0)
    assert abs(float(y @ y) / 4096 - 1.0) < 1e-12


# --------------------------------------------------------------------------
# GELU-tanh * up -- main.swift:8947-8950, 1497-1517, 6680-6690
# --------------------------------------------------------------------------

def test_gelu_up_known_values():
    assert abs(O.gelu_up_f64(1.0, 1.0) - 0.841192) < 1e-6
    assert O.gelu_up_f64(-20.0, 3.0) == 0
    assert abs(O.gelu_up_f32(1.0, 1.0) - 0.841192) < 1e-6


def test_stable_tanh_matches_tanh():
    args = [0, 1e-8, -1e-8, 0.5, -0.5, 1, -1, 5, -5, 10, -10, 30, -30, 49, -49, 49.7, -49.7,
            100, -100, 500, -500, 1e4, -1e4, 1e6, -1e6, 30.5, 30.25]
    args += [float(np.float32(i) * np.float32(3.7) - np.float32(60)) for i in range(32)]
    assert len(args) == 59
    worst = 0.0
    for a in args:
        got = O.stable_tanh_f32(a)
        assert math.isfinite(got)
        worst = max(worst, abs(got - math.tanh(float(np.float32(a)))))
    assert worst < 1e-6


def test_gelu_up_finite_on_extreme_inputs_and_matches_torch():
    import torch
    for g, u in [(1e30, 1.0), (-1e30, 1.0), (1e-30, 2.0), (0.5, -0.25), (8.0, -9.5), (1e20, 0.0)]:
        assert math.isfinite(O.gelu_up_f32(g, u))
    g = np.linspace(-12, 12, 4001)
    want = torch.nn.functional.gelu(torch.from_numpy(g), approximate="tanh").numpy() * 1.5
    got = np.array([O.gelu_up_f64(v, 1.5) for v in g])
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)
    got32 = np.array([O.gelu_up_f32(v, 1.5) for v in g.astype(np.float32)])
    assert np.max(np.abs(got32 - want) / np.maximum(1, np.abs(want))) < 2e-6


# --------------------------------------------------------------------------
# error metric -- main.swift:8951-8955; lev-cpu lib.rs:478-485
# --------------------------------------------------------------------------

def test_max_rel_err_contract():
    assert O.max_rel_err([1001], [1000]) == 0.001
    assert O.max_rel_err([0.5], [0]) == 0.5
    assert O.max_rel_err([np.nan], [0.0]) == math.inf
    assert O.max_rel_err([1.0], [math.inf]) == math.inf
    assert O.max_rel_err([1.0, 2.0], [1.0]) == math.inf
    assert O.max_rel_err([], []) == math.inf
    assert O.max_rel_err([1.0], [1.0]) == 0.0


# --------------------------------------------------------------------------
# argmax -- tie rule lev-model lib.rs:395-403, ops.rs:508
# --------------------------------------------------------------------------

def test_argmax_ties_and_margin():
    assert O.argmax([1.0, 3.0, 3.0, 2.0]) == 1
    assert O.top_margin([1.0, 3.0, 3.0, 2.0]) == 0.0
    assert O.top_margin([1.0, 5.0, 3.0, 2.0]) == 2.0
    v = O.normal(32000, 77)
    assert O.argmax(v) == int(np.argmax(v))
    s = np.sort(v)
    assert O.top_margin(v) == s[-1] - s[-2]


# --------------------------------------------------------------------------
# MoE composite -- main.swift:8925-8946
# --------------------------------------------------------------------------

def _hand_moe():
    def block(lo, hi, q):
        return [lo, hi] + [q] * 16
    gate = sum((block(0x00, 0x3C, 0x98) for _ in range(32)), [])
    up = sum((block(0x00, 0x30, 0x98) for _ in range(32)), [])
    down = sum((block(0x00, 0x38, 0x99) for _ in range(32)), [])
    return gate, up, down


def test_moe_oracle_hand_computed():
    gate, up, down = _hand_moe()
    ones = np.ones(32, dtype=np.float32)
    ref = O.moe_experts_f64(gate, up, down, 32, 32, [0], [1.0], ones)
    assert np.array_equal(ref["gate"], np.full((1, 32), 16.0))
    assert np.array_equal(ref["up"], np.full((1, 32), 2.0))
    assert np.array_equal(ref["act"], np.full((1, 32), 32.0))
    assert np.array_equal(ref["dn"], np.full((1, 32), 512.0))
    assert np.array_equal(ref["y"], np.full(32, 512.0))
    # the reference stores gate|up fused as [2I, H]; the fused view gives the same rows
    fused = np.array(gate + up, dtype=np.uint8)
    ref2 = O.moe_experts_f64(fused, fused[len(gate):], down, 32, 32, [0], [1.0], ones)
    assert np.array_equal(ref2["dn"], ref["dn"])
    y32, act32 = O.moe_experts_f32(gate, up, down, 32, 32, [0], [0.5], ones)
    assert np.array_equal(act32, np.full((1, 32), 32.0, np.float32))
    assert np.array_equal(y32, np.full(32, 256.0, np.float32))
    bad = list(gate)
    bad[1] = 0x7C
    with pytest.raises(O.OracleError):
        O.moe_experts_f64(bad, up, down, 32, 32, [0], [1.0], ones)
    nanx = ones.copy()
    nanx[3] = np.nan
    with pytest.raises(O.OracleError):
        O.moe_experts_f64(gate, up, down, 32, 32, [0], [1.0], nanx)


def _swift_synthetic_blocks(rng, nblocks):
    """syntheticBlocks of main.swift:6560-6571 / Q4Lowering.swift:779-791."""
    out = []
    for _ in range(nblocks):
        lo, hi = rng.next() & 0xFF, rng.next() & 0xFF
        if ((lo | (hi << 8)) & 0x7C00) == 0x7C00:
            lo, hi = 0x00, 0x3C
        out += [lo, hi] + [rng.next() & 0xFF for _ in range(16)]
    return np.array(out, dtype=np.uint8)


def test_moe_tail_region_f32_inside_fp64_contract():
    """The reference's tail region (hidden 96, inter 32, topK 3) with its
    synthetic bytes: the serial f32 path must sit within 1e-4 of the FP64
    oracle (main.swift:6551-6585)."""
    hidden, inter, topk = 96, 32, 3
    gu_stride = (hidden // 32) * 18 * (2 * inter)
    dn_stride = (inter // 32) * 18 * hidden
    rng = O.SplitMix64(0x5A4C4F57)
    gu = _swift_synthetic_blocks(rng, gu_stride * topk // 18)
    dn = _swift_synthetic_blocks(rng, dn_stride * topk // 18)
    x = O.seeded_input(hidden, 1, 70004)
    ids, w = [0, 1, 2], [1.0, 1.0, 1.0]
    up_view = gu[inter * (hidden // 32) * 18:]
    strides = (gu_stride, gu_stride, dn_stride)
    y32, act32 = O.moe_experts_f32(gu, up_view, dn, hidden, inter, ids, w, x, strides)
    ref = O.moe_experts_f64(gu, up_view, dn, hidden, inter, ids, w, x, strides)
    assert O.max_rel_err(act32, ref["act"]) < 1e-4
    assert O.max_rel_err(y32, ref["y"]) < 1e-4


# --------------------------------------------------------------------------
# router -- source text Gemma4.swift:3798-3810 (no reference unit test);
# invariants, brute force and a library cross-check
# --------------------------------------------------------------------------

def test_router_f32_matvec_magnitude_gate():
    """main.swift:2615-2647: |delta| <= 1e-4 * sum|w_i x_i| + 1e-6 vs FP64."""
    for in_dim in (256, 2112, 2816, 3840):
        w = O.normal(128 * in_dim, 40 + in_dim, 0.0, 0.02).reshape(128, in_dim)
        x = O.seeded_input(in_dim, 1, in_dim)
        got = O.f32_matvec(w, 128, in_dim, x)
        ref = O.f32_matvec_f64(w, 128, in_dim, x)
        assert np.allclose(ref, w.astype(np.float64) @ x.astype(np.float64), rtol=1e-12, atol=1e-14)
        mag = np.abs(w.astype(np.float64)) @ np.abs(x.astype(np.float64))
        assert np.all(np.abs(got - ref) <= 1e-4 * mag + 1e-6)


def test_router_topk_invariants_and_cross_check():
    import torch
    for seed in range(20):
        scores = O.normal(128, 900 + seed, 0.0, 2.0)
        ids, wts = O.router_topk(scores, 8)
        assert len(set(ids.tolist())) == 8
        assert abs(float(wts.astype(np.float64).sum()) - 1.0) < 1e-6
        assert np.all(np.diff(wts) <= 0)                      # descending probability
        p = torch.softmax(torch.from_numpy(scores).double(), 0)
        tv, ti = torch.topk(p, 8)
        assert ids.tolist() == ti.tolist()
        assert np.allclose(wts, (tv / tv.sum()).numpy(), rtol=1e-6)


def test_router_topk_ties_prefer_lower_index_and_scales_apply():
    scores = np.zeros(16, dtype=np.float32)
    scores[[3, 9, 12]] = 1.0
    ids, wts = O.router_topk(scores, 5)
    assert ids.tolist() == [3, 9, 12, 0, 1]
    e = math.e
    total = 3 * e + 2
    assert np.allclose(wts, [e / total] * 3 + [1 / total] * 2, rtol=1e-6)
    scale = np.arange(16, dtype=np.float32)
    ids2, wts2 = O.router_topk(scores, 5, scale)
    assert ids2.tolist() == ids.tolist()
    assert np.allclose(wts2, wts * scale[ids], rtol=1e-7)
    with pytest.raises(O.OracleError):
        O.router_topk(np.array([0.0, np.nan], np.float32), 1)


def test_router_topk_brute_force_tiny():
    """Literal restatement of the Swift lines on tiny E with python floats."""
    rng = np.random.default_rng(5)
    for _ in range(50):
        e = int(rng.integers(2, 9))
        k = int(rng.integers(1, e + 1))
        scores = rng.integers(-3, 4, size=e).astype(np.float32) * np.float32(0.5)
        m = max(scores)
        exps = [math.exp(float(np.float32(s - m))) for s in scores]
        tot = sum(exps)
        probs = [v / tot for v in exps]
        order = sorted(range(e), key=lambda i: (-probs[i], i))[:k]
        psum = 0.0
        for i in order:
            psum += probs[i]
        want = [np.float32(probs[i] / psum) for i in order]
        ids, wts = O.router_topk(scores, k)
        assert ids.tolist() == order
        assert wts.tolist() == want


# --------------------------------------------------------------------------
# prefill GEMM oracle -- lev-cli main.rs:1201-1217, 1266-1278
# --------------------------------------------------------------------------

def test_gemm_oracle_definition():
    rows, cols, tokens = 27, 512, 3
    w = O.synth_q4_k(4, rows * cols // 256, 0.01)
    x = O.normal(tokens * cols, 4).astype(np.float16)
    got = O.q4_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 13)
    wr = O.q4_k_dequant(w).reshape(rows, cols).astype(np.float16).astype(np.float64)
    want = x.reshape(tokens, cols).astype(np.float64) @ wr[0::13].T
    assert got.shape == (tokens, 3)
    assert np.allclose(got, want, rtol=1e-12, atol=1e-12)


# --------------------------------------------------------------------------
# synthetic generators: determinism and the stated distributions
# --------------------------------------------------------------------------

def test_synthetic_generators():
    a = O.synth_q4_0(1, 4096)
    assert np.array_equal(a, O.synth_q4_0(1, 4096)) and not np.array_equal(a, O.synth_q4_0(2, 4096))
    d = a.reshape(-1, 18)[:, :2].copy().view(np.float16).astype(np.float64)
    assert np.all(np.isfinite(d)) and np.all(d >= 0)
    assert abs(d.mean() - 0.02 * math.sqrt(2 / math.pi)) < 1e-3
    codes = a.reshape(-1, 18)[:, 2:]
    assert abs(codes.mean() - 127.5) < 2.0
    b = O.synth_q6_k(2, 512).reshape(-1, 210)
    sc = b[:, 192:208].view(np.int8)
    assert sc.min() == -32 and sc.max() == 31
    assert np.all(np.isfinite(b[:, 208:210].copy().view(np.float16).astype(np.float64)))
    c = O.synth_q4_k(3, 512).reshape(-1, 144)
    assert np.all(np.isfinite(c[:, :4].copy().view(np.float16).astype(np.float64)))
    n = O.normal(200000, 9)
    assert abs(n.mean()) < 0.01 and abs(n.std() - 1.0) < 0.01


def test_q6_k_gemm_oracle_is_fp16_rounded_decode_times_x_in_f64():
    """The Q6_K prefill gate (lev-forge coopmat.rs:333-425 with lev-cli main.rs:1201-1217):
    W = fp16(decodeBlock value), X fp16, f64 accumulation -- against numpy on the
    block decode that the reference's own known answers pin, and on the -315 block
    (main.swift:1091-1120) whose weights are exact in fp16."""
    rows, cols, tokens = 7, 512, 5
    w = O.synth_q6_k(21, rows * cols // 256, 0.01)
    x = O.normal(tokens * cols, 22).astype(np.float16).reshape(tokens, cols)
    w16 = O.q6_k_dequant(w).astype(np.float16).astype(np.float64).reshape(rows, cols)
    want = x.astype(np.float64) @ w16.T
    got = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 0, 1)
    assert np.array_equal(got, want) or np.allclose(got, want, rtol=1e-13, atol=0)
    sampled = O.q6_k_gemm_f16_oracle(w, rows, cols, x.view(np.uint16), tokens, 1, 3)
    assert np.array_equal(sampled, got[:, 1::3])
    with pytest.raises(O.OracleError):
        O.q6_k_gemm_f16_oracle(w[:-1], rows, cols, x.view(np.uint16), tokens, 0, 1)
