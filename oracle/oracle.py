"""numpy view of ``liblev_oracle.so`` (the C restatement in ``lev_oracle.c``).

TEST INFRASTRUCTURE ONLY.  Every wrapper returns ``(status, value)`` or raises
``OracleError(status)`` exactly where the reference would throw; the status
numbers are those of ``lev_status`` in ``include/leviathan_hip.h``.
"""
from __future__ import annotations

import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB_PATH = os.path.join(_HERE, "liblev_oracle.so")

OK = 0
BAD_DIMENSIONS = 1
WRONG_INPUT_COUNT = 2
NON_FINITE_INPUT = 3
NON_FINITE_SCALE = 4
NON_FINITE_OUTPUT = 5
EXCEEDS_MODEL_WORKLOAD = 6
INTEGER_OVERFLOW = 7
INVALID_ARGUMENT = 14

Q4_0_BLOCK_BYTES = 18
Q4_K_BLOCK_BYTES = 144
Q6_K_BLOCK_BYTES = 210


class OracleError(Exception):
    def __init__(self, status: int):
        super().__init__(f"oracle status {status}")
        self.status = status


def build(force: bool = False) -> str:
    """Compile the C oracle with gcc (seconds)."""
    src = os.path.join(_HERE, "lev_oracle.c")
    hdr = os.path.join(_HERE, "lev_oracle.h")
    stale = (not os.path.exists(_LIB_PATH)
             or os.path.getmtime(_LIB_PATH) < max(os.path.getmtime(src), os.path.getmtime(hdr)))
    if force or stale:
        subprocess.run(["make", "-C", _HERE, "-B", "liblev_oracle.so"], check=True,
                       stdout=subprocess.DEVNULL)
    return _LIB_PATH


def _load():
    build()   # compiles only when the library is missing or older than its sources
    return C.CDLL(_LIB_PATH)


_lib = _load()

_u8p = C.POINTER(C.c_uint8)
_f32p = C.POINTER(C.c_float)
_f64p = C.POINTER(C.c_double)
_i8p = C.POINTER(C.c_int8)
_i32p = C.POINTER(C.c_int32)
_u16p = C.POINTER(C.c_uint16)
_u64p = C.POINTER(C.c_uint64)


def _sig(name, restype, *argtypes):
    fn = getattr(_lib, name)
    fn.restype = restype
    fn.argtypes = list(argtypes)
    return fn


def _u8(a):
    a = np.ascontiguousarray(a, dtype=np.uint8)
    return a, a.ctypes.data_as(_u8p)


def _f32(a):
    a = np.ascontiguousarray(a, dtype=np.float32)
    return a, a.ctypes.data_as(_f32p)


def _f64(a):
    a = np.ascontiguousarray(a, dtype=np.float64)
    return a, a.ctypes.data_as(_f64p)


def _check(st):
    if st != OK:
        raise OracleError(st)


# ---- half precision ----
_f16_to_f64 = _sig("levo_f16_to_f64", C.c_double, C.c_uint16)
_f16_to_f32 = _sig("levo_f16_to_f32", C.c_float, C.c_uint16)
_f32_to_f16 = _sig("levo_f32_to_f16_bits", C.c_uint16, C.c_float)


def f16_to_f64(h: int) -> float:
    return _f16_to_f64(h)


def f16_to_f32(h: int) -> float:
    return _f16_to_f32(h)


def f32_to_f16_bits(v: float) -> int:
    return _f32_to_f16(np.float32(v))


# ---- SplitMix64 ----
_sm_next = _sig("levo_splitmix64_next", C.c_uint64, _u64p)
_next_uniform = _sig("levo_next_uniform", C.c_float, _u64p)
_next_signed = _sig("levo_next_signed_unit", C.c_float, _u64p)
_fill_uniform = _sig("levo_fill_uniform", None, C.c_uint64, _f32p, C.c_size_t)
_fill_signed = _sig("levo_fill_signed_unit", None, C.c_uint64, _f32p, C.c_size_t)
_fill_normal = _sig("levo_fill_normal", None, C.c_uint64, C.c_float, C.c_float, _f32p, C.c_size_t)


class SplitMix64:
    """Stateful stream with both reference float conventions."""

    def __init__(self, seed: int):
        self._s = C.c_uint64(seed & 0xFFFFFFFFFFFFFFFF)

    def next(self) -> int:
        return _sm_next(C.byref(self._s))

    def next_uniform(self) -> float:          # Swift nextUniform
        return _next_uniform(C.byref(self._s))

    def next_signed_unit(self) -> float:      # Rust next_signed_unit
        return _next_signed(C.byref(self._s))


def seeded_input(dim: int, batch: int, seed: int) -> np.ndarray:
    """``seededInput`` of the reference's Swift test harness."""
    out = np.empty(dim * batch, dtype=np.float32)
    _fill_uniform(seed, out.ctypes.data_as(_f32p), out.size)
    return out


def signed_units(n: int, seed: int) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _fill_signed(seed, out.ctypes.data_as(_f32p), out.size)
    return out


def normal(n: int, seed: int, mean: float = 0.0, sigma: float = 1.0) -> np.ndarray:
    out = np.empty(n, dtype=np.float32)
    _fill_normal(seed, mean, sigma, out.ctypes.data_as(_f32p), out.size)
    return out


# ---- Q4_0 ----
_q4_decode = _sig("levo_q4_0_decode_block", C.c_int, _u8p, _f32p)
_q4_dequant = _sig("levo_q4_0_dequant", C.c_int, _u8p, C.c_size_t, _f32p)
_mv_args = (_u8p, C.c_size_t, C.c_int64, C.c_int64, _f32p, C.c_size_t)
_q4_ref = _sig("levo_q4_0_matvec_ref", C.c_int, *_mv_args, _f32p)
_q4_ref_mt = _sig("levo_q4_0_matvec_ref_mt", C.c_int, *_mv_args, _f32p, C.c_int)
_q4_ko = _sig("levo_q4_0_matvec_kernel_order", C.c_int, *_mv_args, _f32p)
_q4_f64 = _sig("levo_q4_0_matvec_f64", C.c_int, *_mv_args, _f64p)
_q4_f64_xd = _sig("levo_q4_0_matvec_f64_xd", C.c_int, _u8p, C.c_size_t, C.c_size_t, C.c_int64,
                  C.c_int64, _f64p, C.c_size_t, _f64p)


def q4_0_decode_block(block) -> np.ndarray:
    b, bp = _u8(block)
    if b.size != 18:
        raise OracleError(BAD_DIMENSIONS)
    out = np.empty(32, dtype=np.float32)
    _check(_q4_decode(bp, out.ctypes.data_as(_f32p)))
    return out


def q4_0_dequant(w) -> np.ndarray:
    b, bp = _u8(w)
    n = b.size // 18
    out = np.empty(n * 32, dtype=np.float32)
    _check(_q4_dequant(bp, n, out.ctypes.data_as(_f32p)))
    return out


def _matvec(fn, w, out_dim, in_dim, x, dtype, *extra):
    wb, wp = _u8(w)
    xa, xp = _f32(x)
    y = np.zeros(max(int(out_dim), 0), dtype=dtype)
    yp = y.ctypes.data_as(_f32p if dtype == np.float32 else _f64p)
    _check(fn(wp, wb.size, int(out_dim), int(in_dim), xp, xa.size, yp, *extra))
    return y


def q4_0_matvec_ref(w, out_dim, in_dim, x, threads: int = 0) -> np.ndarray:
    if threads > 0:
        return _matvec(_q4_ref_mt, w, out_dim, in_dim, x, np.float32, threads)
    return _matvec(_q4_ref, w, out_dim, in_dim, x, np.float32)


def q4_0_matvec_kernel_order(w, out_dim, in_dim, x) -> np.ndarray:
    return _matvec(_q4_ko, w, out_dim, in_dim, x, np.float32)


def q4_0_matvec_f64(w, out_dim, in_dim, x) -> np.ndarray:
    return _matvec(_q4_f64, w, out_dim, in_dim, x, np.float64)


def q4_0_matvec_f64_xd(w, byte_offset, out_dim, in_dim, xd) -> np.ndarray:
    wb, wp = _u8(w)
    xa, xp = _f64(xd)
    y = np.zeros(out_dim, dtype=np.float64)
    _check(_q4_f64_xd(wp, wb.size, byte_offset, out_dim, in_dim, xp, xa.size,
                      y.ctypes.data_as(_f64p)))
    return y


# ---- Q6_K ----
_q6_decode = _sig("levo_q6_k_decode_block", C.c_int, _u8p, _f32p)
_q6_unpack = _sig("levo_q6k_unpack", None, _u8p, _i8p)
_q6_dq32 = _sig("levo_q6_k_dequant_block_f32", None, _u8p, _f32p)
_q6_dq64 = _sig("levo_q6_k_dequant_block_f64", None, _u8p, _f64p)
_q6_dequant = _sig("levo_q6_k_dequant", C.c_int, _u8p, C.c_size_t, _f32p)
_q6_ref = _sig("levo_q6_k_matvec_ref", C.c_int, *_mv_args, _f32p)
_q6_ref_mt = _sig("levo_q6_k_matvec_ref_mt", C.c_int, *_mv_args, _f32p, C.c_int)
_q6_f64 = _sig("levo_q6_k_matvec_f64", C.c_int, *_mv_args, _f64p)
_q6_f32 = _sig("levo_q6_k_matvec_f32", C.c_int, *_mv_args, _f32p)
_q6_f32_mt = _sig("levo_q6_k_matvec_f32_mt", C.c_int, *_mv_args, _f32p, C.c_int)


def q6_k_decode_block(block) -> np.ndarray:
    b, bp = _u8(block)
    if b.size != 210:
        raise OracleError(BAD_DIMENSIONS)
    out = np.empty(256, dtype=np.float32)
    _check(_q6_decode(bp, out.ctypes.data_as(_f32p)))
    return out


def q6k_unpack(block) -> np.ndarray:
    b, bp = _u8(block)
    out = np.empty(256, dtype=np.int8)
    _q6_unpack(bp, out.ctypes.data_as(_i8p))
    return out


def q6_k_dequant_block_f32(block) -> np.ndarray:
    b, bp = _u8(block)
    out = np.empty(256, dtype=np.float32)
    _q6_dq32(bp, out.ctypes.data_as(_f32p))
    return out


def q6_k_dequant_block_f64(block) -> np.ndarray:
    b, bp = _u8(block)
    out = np.empty(256, dtype=np.float64)
    _q6_dq64(bp, out.ctypes.data_as(_f64p))
    return out


def q6_k_dequant(w) -> np.ndarray:
    b, bp = _u8(w)
    n = b.size // 210
    out = np.empty(n * 256, dtype=np.float32)
    _check(_q6_dequant(bp, n, out.ctypes.data_as(_f32p)))
    return out


def q6_k_matvec_ref(w, out_dim, in_dim, x, threads: int = 0) -> np.ndarray:
    if threads > 0:
        return _matvec(_q6_ref_mt, w, out_dim, in_dim, x, np.float32, threads)
    return _matvec(_q6_ref, w, out_dim, in_dim, x, np.float32)


def q6_k_matvec_f64(w, out_dim, in_dim, x) -> np.ndarray:
    return _matvec(_q6_f64, w, out_dim, in_dim, x, np.float64)


def q6_k_matvec_f32(w, rows, cols, x, threads: int = 0) -> np.ndarray:
    if threads > 0:
        return _matvec(_q6_f32_mt, w, rows, cols, x, np.float32, threads)
    return _matvec(_q6_f32, w, rows, cols, x, np.float32)


# ---- Q4_K ----
_q4k_unpack = _sig("levo_q4_k_unpack_scale_min", None, C.c_int, _u8p, _u8p, _u8p)
_q4k_pack = _sig("levo_q4_k_pack_scale_min", None, _u8p, _u8p, _u8p)
_q4k_dq32 = _sig("levo_q4_k_dequant_block_f32", None, _u8p, _f32p)
_q4k_dq64 = _sig("levo_q4_k_dequant_block_f64", None, _u8p, _f64p)
_q4k_dequant = _sig("levo_q4_k_dequant", C.c_int, _u8p, C.c_size_t, _f32p)
_q4k_f32 = _sig("levo_q4_k_matvec_f32", C.c_int, *_mv_args, _f32p)
_q4k_f32_mt = _sig("levo_q4_k_matvec_f32_mt", C.c_int, *_mv_args, _f32p, C.c_int)
_q4k_f64 = _sig("levo_q4_k_matvec_f64", C.c_int, *_mv_args, _f64p)


def q4_k_unpack_scale_min(j: int, scales12):
    s, sp = _u8(scales12)
    sc, mn = C.c_uint8(), C.c_uint8()
    _q4k_unpack(j, sp, C.byref(sc), C.byref(mn))
    return sc.value, mn.value


def q4_k_pack_scale_min(sc8, mn8) -> np.ndarray:
    a, ap = _u8(sc8)
    b, bp = _u8(mn8)
    out = np.zeros(12, dtype=np.uint8)
    _q4k_pack(ap, bp, out.ctypes.data_as(_u8p))
    return out


def q4_k_dequant_block_f32(block) -> np.ndarray:
    b, bp = _u8(block)
    out = np.empty(256, dtype=np.float32)
    _q4k_dq32(bp, out.ctypes.data_as(_f32p))
    return out


def q4_k_dequant_block_f64(block) -> np.ndarray:
    b, bp = _u8(block)
    out = np.empty(256, dtype=np.float64)
    _q4k_dq64(bp, out.ctypes.data_as(_f64p))
    return out


def q4_k_dequant(w) -> np.ndarray:
    b, bp = _u8(w)
    n = b.size // 144
    out = np.empty(n * 256, dtype=np.float32)
    _check(_q4k_dequant(bp, n, out.ctypes.data_as(_f32p)))
    return out


def q4_k_matvec_f32(w, rows, cols, x, threads: int = 0) -> np.ndarray:
    if threads > 0:
        return _matvec(_q4k_f32_mt, w, rows, cols, x, np.float32, threads)
    return _matvec(_q4k_f32, w, rows, cols, x, np.float32)


def q4_k_matvec_f64(w, rows, cols, x) -> np.ndarray:
    return _matvec(_q4k_f64, w, rows, cols, x, np.float64)


# ---- int8 activations ----
_q8 = _sig("levo_quantize_q8", C.c_int, _f32p, C.c_size_t, _i8p, _f32p, _f32p)


def quantize_q8(x):
    xa, xp = _f32(x)
    q = np.empty(xa.size, dtype=np.int8)
    d = np.empty(xa.size // 32, dtype=np.float32)
    s = np.empty(xa.size // 32, dtype=np.float32)
    _check(_q8(xp, xa.size, q.ctypes.data_as(_i8p), d.ctypes.data_as(_f32p),
               s.ctypes.data_as(_f32p)))
    return q, d, s


def dequantize_q8(q, d) -> np.ndarray:
    """xd = q as f32 * d[group], one f32 product per element (lev-cpu/src/lib.rs:327)."""
    q = np.asarray(q, dtype=np.int8).reshape(-1)
    d = np.asarray(d, dtype=np.float32).reshape(-1)
    return (q.astype(np.float32) * np.repeat(d, 32)).astype(np.float32)


def q4_k_matvec_q8_f64(w, rows, cols, q, d) -> np.ndarray:
    """matvec_q4k_q8_f64, lev-cpu/src/lib.rs:324-331."""
    return q4_k_matvec_f64(w, rows, cols, dequantize_q8(q, d))


def q6_k_matvec_q8_f64(w, rows, cols, q, d) -> np.ndarray:
    """matvec_q6k_q8_f64, lev-cpu/src/lib.rs:333-337."""
    return q6_k_matvec_f64(w, rows, cols, dequantize_q8(q, d))


# ---- RMSNorm ----
_rms = _sig("levo_rmsnorm", None, _f32p, _f32p, C.c_float, C.c_size_t, _f32p)
_rms_serial = _sig("levo_rmsnorm_f32_serial", None, _f32p, _f32p, C.c_float, C.c_size_t, _f32p)
_rms_f64 = _sig("levo_rmsnorm_f64", None, _f32p, _f32p, C.c_double, C.c_size_t, _f64p)


def rmsnorm(x, w, eps: float) -> np.ndarray:
    xa, xp = _f32(x)
    wa, wp = _f32(w)
    y = np.empty_like(xa)
    _rms(xp, wp, eps, xa.size, y.ctypes.data_as(_f32p))
    return y


def rmsnorm_f32_serial(x, w, eps: float) -> np.ndarray:
    xa, xp = _f32(x)
    wp = None
    if w is not None:
        wa, wp = _f32(w)
    y = np.empty_like(xa)
    _rms_serial(xp, wp, eps, xa.size, y.ctypes.data_as(_f32p))
    return y


def rmsnorm_f64(x, w, eps: float) -> np.ndarray:
    xa, xp = _f32(x)
    wp = None
    if w is not None:
        wa, wp = _f32(w)
    y = np.empty(xa.size, dtype=np.float64)
    _rms_f64(xp, wp, eps, xa.size, y.ctypes.data_as(_f64p))
    return y


# ---- GELU ----
stable_tanh_f32 = _sig("levo_stable_tanh_f32", C.c_float, C.c_float)
gelu_up_f32 = _sig("levo_gelu_up_f32", C.c_float, C.c_float, C.c_float)
gelu_up_f64 = _sig("levo_gelu_up_f64", C.c_double, C.c_double, C.c_double)

# ---- argmax ----
_argmax = _sig("levo_argmax", C.c_size_t, _f32p, C.c_size_t)
_margin = _sig("levo_top_margin", C.c_float, _f32p, C.c_size_t)


def argmax(logits) -> int:
    a, ap = _f32(logits)
    return int(_argmax(ap, a.size))


def top_margin(logits) -> float:
    a, ap = _f32(logits)
    return float(_margin(ap, a.size))


# ---- error metric ----
_mre = _sig("levo_max_rel_err", C.c_double, _f32p, C.c_size_t, _f64p, C.c_size_t)


def max_rel_err(got, ref) -> float:
    g, gp = _f32(np.asarray(got).ravel())
    r, rp = _f64(np.asarray(ref).ravel())
    return float(_mre(gp, g.size, rp, r.size))


# ---- router ----
_f32mv = _sig("levo_f32_matvec", None, _f32p, C.c_int64, C.c_int64, _f32p, _f32p)
_f32mv64 = _sig("levo_f32_matvec_f64", None, _f32p, C.c_int64, C.c_int64, _f32p, _f64p)
_topk = _sig("levo_router_topk", C.c_int, _f32p, C.c_int, C.c_int, _f32p, _i32p, _f32p)


def f32_matvec(w, out_dim, in_dim, x) -> np.ndarray:
    wa, wp = _f32(w)
    xa, xp = _f32(x)
    y = np.empty(out_dim, dtype=np.float32)
    _f32mv(wp, out_dim, in_dim, xp, y.ctypes.data_as(_f32p))
    return y


def f32_matvec_f64(w, out_dim, in_dim, x) -> np.ndarray:
    wa, wp = _f32(w)
    xa, xp = _f32(x)
    y = np.empty(out_dim, dtype=np.float64)
    _f32mv64(wp, out_dim, in_dim, xp, y.ctypes.data_as(_f64p))
    return y


def router_topk(scores, top_k: int, expert_scale=None):
    s, sp = _f32(scores)
    ep = None
    if expert_scale is not None:
        e, ep = _f32(expert_scale)
    ids = np.empty(top_k, dtype=np.int32)
    wts = np.empty(top_k, dtype=np.float32)
    _check(_topk(sp, s.size, top_k, ep, ids.ctypes.data_as(_i32p), wts.ctypes.data_as(_f32p)))
    return ids, wts


# ---- MoE ----
_moe32 = _sig("levo_moe_experts_f32", C.c_int, _u8p, _u8p, _u8p, C.c_size_t, C.c_size_t,
              C.c_size_t, C.c_int, C.c_int, C.c_int, _i32p, _f32p, _f32p, _f32p, _f32p)
_moe64 = _sig("levo_moe_experts_f64", C.c_int, _u8p, _u8p, _u8p, C.c_size_t, C.c_size_t,
              C.c_size_t, C.c_int, C.c_int, C.c_int, _i32p, _f32p, _f32p, _f64p, _f64p, _f64p,
              _f64p, _f64p)


def _strides(hidden, inter):
    gu = inter * (hidden // 32) * 18
    dn = hidden * (inter // 32) * 18
    return gu, dn


def moe_experts_f32(gate, up, down, hidden, inter, ids, weights, x, strides=None):
    """Reference serial per-slot loop, f32.  Returns (y[hidden], act[topk, inter])."""
    g, gp = _u8(gate)
    u, upp = _u8(up)
    d, dp = _u8(down)
    ia = np.ascontiguousarray(ids, dtype=np.int32)
    wa, wp = _f32(weights)
    xa, xp = _f32(x)
    gs, ds = _strides(hidden, inter)
    gst, ust, dst = strides if strides else (gs, gs, ds)
    k = ia.size
    y = np.empty(hidden, dtype=np.float32)
    act = np.empty((k, inter), dtype=np.float32)
    _check(_moe32(gp, upp, dp, gst, ust, dst, hidden, inter, k, ia.ctypes.data_as(_i32p), wp, xp,
                  y.ctypes.data_as(_f32p), act.ctypes.data_as(_f32p)))
    return y, act


def moe_experts_f64(gate, up, down, hidden, inter, ids, weights, x, strides=None):
    """FP64 oracle.  Returns dict(y, gate, up, act, dn)."""
    g, gp = _u8(gate)
    u, upp = _u8(up)
    d, dp = _u8(down)
    ia = np.ascontiguousarray(ids, dtype=np.int32)
    wa, wp = _f32(weights)
    xa, xp = _f32(x)
    gs, ds = _strides(hidden, inter)
    gst, ust, dst = strides if strides else (gs, gs, ds)
    k = ia.size
    out = dict(y=np.empty(hidden), gate=np.empty((k, inter)), up=np.empty((k, inter)),
               act=np.empty((k, inter)), dn=np.empty((k, hidden)))
    _check(_moe64(gp, upp, dp, gst, ust, dst, hidden, inter, k, ia.ctypes.data_as(_i32p), wp, xp,
                  *(out[n].ctypes.data_as(_f64p) for n in ("y", "gate", "up", "act", "dn"))))
    return out


# ---- prefill GEMM oracle ----
_gemm = _sig("levo_q4_k_gemm_f16_oracle", C.c_int, _u8p, C.c_size_t, C.c_int64, C.c_int64, _u16p,
             C.c_int64, C.c_int64, C.c_int64, _f64p)


def q4_k_gemm_f16_oracle(w, rows, cols, x_f16_bits, tokens, row0=0, row_step=13) -> np.ndarray:
    """f16-rounded W and X, f64 accumulate; rows row0::row_step.  [tokens, n_rows]."""
    wb, wp = _u8(w)
    xb = np.ascontiguousarray(x_f16_bits, dtype=np.uint16)
    n_rows = len(range(row0, rows, row_step))
    y = np.empty((tokens, n_rows), dtype=np.float64)
    _check(_gemm(wp, wb.size, rows, cols, xb.ctypes.data_as(_u16p), tokens, row0, row_step,
                 y.ctypes.data_as(_f64p)))
    return y


_gemm6 = _sig("levo_q6_k_gemm_f16_oracle", C.c_int, _u8p, C.c_size_t, C.c_int64, C.c_int64, _u16p,
              C.c_int64, C.c_int64, C.c_int64, _f64p)


def q6_k_gemm_f16_oracle(w, rows, cols, x_f16_bits, tokens, row0=0, row_step=13) -> np.ndarray:
    """As q4_k_gemm_f16_oracle for Q6_K weights.  [tokens, n_rows]."""
    wb, wp = _u8(w)
    xb = np.ascontiguousarray(x_f16_bits, dtype=np.uint16)
    n_rows = len(range(row0, rows, row_step))
    y = np.empty((tokens, n_rows), dtype=np.float64)
    _check(_gemm6(wp, wb.size, rows, cols, xb.ctypes.data_as(_u16p), tokens, row0, row_step,
                  y.ctypes.data_as(_f64p)))
    return y


# ---- synthetic weights ----
_sq40 = _sig("levo_synth_q4_0", None, C.c_uint64, C.c_float, _u8p, C.c_size_t)
_sq6k = _sig("levo_synth_q6_k", None, C.c_uint64, C.c_float, _u8p, C.c_size_t)
_sq4k = _sig("levo_synth_q4_k", None, C.c_uint64, C.c_float, _u8p, C.c_size_t)


def synth_q4_0(seed, nblocks, sigma_d=0.02) -> np.ndarray:
    out = np.empty(nblocks * 18, dtype=np.uint8)
    _sq40(seed, sigma_d, out.ctypes.data_as(_u8p), nblocks)
    return out


def synth_q6_k(seed, nblocks, sigma_d=0.01) -> np.ndarray:
    out = np.empty(nblocks * 210, dtype=np.uint8)
    _sq6k(seed, sigma_d, out.ctypes.data_as(_u8p), nblocks)
    return out


def synth_q4_k(seed, nblocks, sigma_d=0.01) -> np.ndarray:
    out = np.empty(nblocks * 144, dtype=np.uint8)
    _sq4k(seed, sigma_d, out.ctypes.data_as(_u8p), nblocks)
    return out
