"""Thin Python view of the C ABI for callers that hold torch tensors.

torch is used here only as a device-memory and stream provider: every method
passes ``tensor.data_ptr()`` and sizes straight to ``libleviathan_hip.so``.
Method names follow the reference's operator vocabulary
(``Gemma4Runner.matvec`` / ``rmsnorm`` / ``geluUp`` / ``axpy`` /
``runMoeBatchedRouted``; ``Builder::matvec`` / ``norm_quant`` / argmax step).
There is no CPU path: a missing library or a failed call raises.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import capi


class LevError(RuntimeError):
    """A C-ABI call returned a non-zero ``lev_status``."""

    def __init__(self, status: int, message: str):
        name = capi.load().lev_hip_status_name(status).decode()
        super().__init__(f"{name} ({status}): {message}")
        self.status = status
        self.name = name
        self.message = message


def _ptr(t):
    return C.c_void_p(t.data_ptr()) if t is not None else C.c_void_p(0)


def _dev(t, dtype, what):
    if not isinstance(t, torch.Tensor) or not t.is_cuda or t.dtype != dtype or not t.is_contiguous():
        raise TypeError(f"{what}: expected a contiguous {dtype} tensor on the GPU")
    return t


class Context:
    """``lev_ctx``: one device and one stream (torch's current stream by default)."""

    def __init__(self, device: int = 0, stream: torch.cuda.Stream | None = None,
                 own_stream: bool = False):
        self.lib = capi.load()
        if not torch.cuda.is_available():
            raise RuntimeError("no GPU visible: this library has no CPU path")
        torch.cuda.set_device(device)
        handle = C.c_void_p(-1)          # LEV_HIP_OWN_STREAM
        if not own_stream:
            s = stream if stream is not None else torch.cuda.current_stream(device)
            handle = C.c_void_p(s.cuda_stream)
        ctx = C.c_void_p()
        st = self.lib.lev_hip_ctx_create(device, handle, C.byref(ctx))
        if st != capi.OK:
            raise LevError(st, "ctx_create")
        self.ctx = ctx
        self.device = device

    def close(self):
        if getattr(self, "ctx", None):
            self.lib.lev_hip_ctx_destroy(self.ctx)
            self.ctx = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    # -- helpers ----------------------------------------------------------
    def _check(self, st: int):
        if st != capi.OK:
            raise LevError(st, self.lib.lev_hip_last_error(self.ctx).decode())

    def sync(self):
        self._check(self.lib.lev_hip_sync(self.ctx))

    def device_name(self) -> str:
        buf = C.create_string_buffer(256)
        self._check(self.lib.lev_hip_device_name(self.ctx, buf, 256))
        return buf.value.decode()

    # -- recorded programs -------------------------------------------------
    def program_begin(self):
        self._check(self.lib.lev_hip_program_begin(self.ctx))

    def program_end(self) -> "Program":
        handle = C.c_void_p()
        self._check(self.lib.lev_hip_program_end(self.ctx, C.byref(handle)))
        return Program(self, handle)

    # -- dequantise -------------------------------------------------------
    def dequant(self, qtype: int, w: torch.Tensor, nblocks: int, w_off: int = 0) -> torch.Tensor:
        _dev(w, torch.uint8, "w")
        values = 32 if qtype == capi.TYPE_Q4_0 else 256
        out = torch.empty(max(nblocks, 1) * values, dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_dequant(self.ctx, qtype, _ptr(w), w.numel(), w_off, nblocks,
                                             _ptr(out), out.numel()))
        return out[: nblocks * values]

    # -- GEMV -------------------------------------------------------------
    def q4_0_gemv(self, w, x, in_dim: int, out_rows: int, y=None, w_off: int = 0, x_count=None):
        _dev(w, torch.uint8, "w")
        _dev(x, torch.float32, "x")
        if y is None:
            y = torch.empty(max(out_rows, 1), dtype=torch.float32, device=w.device)
        xc = x.numel() if x_count is None else x_count
        self._check(self.lib.lev_hip_q4_0_gemv(self.ctx, _ptr(w), w.numel(), w_off, _ptr(x), xc,
                                               _ptr(y), y.numel(), in_dim, out_rows))
        return y

    def q6_k_gemv(self, w, x, in_dim: int, out_rows: int, y=None, w_off: int = 0, argmax=False):
        _dev(w, torch.uint8, "w")
        _dev(x, torch.float32, "x")
        if y is None:
            y = torch.empty(max(out_rows, 1), dtype=torch.float32, device=w.device)
        idx = mg = None
        if argmax:
            idx = torch.empty(1, dtype=torch.int32, device=w.device)
            mg = torch.empty(1, dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q6_k_gemv(self.ctx, _ptr(w), w.numel(), w_off, _ptr(x),
                                               x.numel(), _ptr(y), y.numel(), in_dim, out_rows,
                                               _ptr(idx), _ptr(mg)))
        return (y, idx, mg) if argmax else y

    def q4_k_gemv_ncol(self, w, x, in_dim: int, rows: int, ncol: int, gain=None, eps: float = 1e-6,
                       y=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(x, torch.float32, "x")
        if gain is not None:
            _dev(gain, torch.float32, "gain")
        if y is None:
            y = torch.empty((max(ncol, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q4_k_gemv_ncol(self.ctx, _ptr(w), w.numel(), w_off, _ptr(x),
                                                    x.numel(), _ptr(gain), eps, _ptr(y), y.numel(),
                                                    in_dim, rows, ncol))
        return y

    def q6_k_gemv_ncol(self, w, x, in_dim: int, rows: int, ncol: int, gain=None, eps: float = 1e-6,
                       y=None, w_off: int = 0):
        """Q6_K GEMV of ``ncol`` f32 columns per weight read (optional RMSNorm in front)."""
        _dev(w, torch.uint8, "w")
        _dev(x, torch.float32, "x")
        if gain is not None:
            _dev(gain, torch.float32, "gain")
        if y is None:
            y = torch.empty((max(ncol, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q6_k_gemv_ncol(self.ctx, _ptr(w), w.numel(), w_off, _ptr(x),
                                                    x.numel(), _ptr(gain), eps, _ptr(y), y.numel(),
                                                    in_dim, rows, ncol))
        return y

    def norm_quant_q8(self, x, n: int, ncol: int, gain=None, eps: float = 1e-6, add=None,
                      want_y: bool = False):
        """Int8 activations of ``x`` [ncol][n]: returns (xq int8, xs (d, s) pairs[, y f32])."""
        _dev(x, torch.float32, "x")
        if gain is not None:
            _dev(gain, torch.float32, "gain")
        if add is not None:
            _dev(add, torch.float32, "add")
        xq = torch.empty((max(ncol, 1), max(n, 1)), dtype=torch.int8, device=x.device)
        xs = torch.empty((max(ncol, 1), max(n // 32, 1), 2), dtype=torch.float32, device=x.device)
        y = torch.empty_like(x) if want_y else None
        self._check(self.lib.lev_hip_norm_quant_q8(self.ctx, _ptr(x), x.numel(), _ptr(add), _ptr(gain),
                                                   eps, _ptr(xq), _ptr(xs), _ptr(y), n, ncol))
        return (xq, xs, y) if want_y else (xq, xs)

    def q4_k_gemv_q8(self, w, xq, xs, in_dim: int, rows: int, ncol: int, y=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(xq, torch.int8, "xq")
        _dev(xs, torch.float32, "xs")
        if y is None:
            y = torch.empty((max(ncol, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q4_k_gemv_q8(self.ctx, _ptr(w), w.numel(), w_off, _ptr(xq),
                                                  _ptr(xs), xq.numel(), _ptr(y), y.numel(), in_dim,
                                                  rows, ncol))
        return y

    def q6_k_gemv_q8(self, w, xq, xs, in_dim: int, rows: int, ncol: int, y=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(xq, torch.int8, "xq")
        _dev(xs, torch.float32, "xs")
        if y is None:
            y = torch.empty((max(ncol, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q6_k_gemv_q8(self.ctx, _ptr(w), w.numel(), w_off, _ptr(xq),
                                                  _ptr(xs), xq.numel(), _ptr(y), y.numel(), in_dim,
                                                  rows, ncol))
        return y

    def swiglu_quant_q8(self, gate, up, want_act: bool = False):
        """Int8 activations of silu(gate) * up: returns (xq, xs (d, s) pairs[, act f32])."""
        _dev(gate, torch.float32, "gate")
        _dev(up, torch.float32, "up")
        n = gate.numel()
        xq = torch.empty(max(n, 1), dtype=torch.int8, device=gate.device)
        xs = torch.empty((max(n // 32, 1), 2), dtype=torch.float32, device=gate.device)
        act = torch.empty_like(gate) if want_act else None
        self._check(self.lib.lev_hip_swiglu_quant_q8(self.ctx, _ptr(gate), _ptr(up), n, _ptr(xq),
                                                     _ptr(xs), _ptr(act)))
        return (xq, xs, act) if want_act else (xq, xs)

    def embed_q4_k(self, w, tokens, dim: int, vocab: int, out=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(tokens, torch.int32, "tokens")
        n = tokens.numel()
        if out is None:
            out = torch.empty((max(n, 1), dim), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_embed_q4_k(self.ctx, _ptr(w), w.numel(), w_off, _ptr(tokens), n,
                                                _ptr(out), out.numel(), dim, vocab))
        return out

    # ---- schedule candidates and per-shape selection ----
    def forge_candidates(self, op: int, in_dim: int, rows: int, ncol: int = 1):
        buf = (capi.Schedule * 16)()
        n = C.c_uint32(0)
        self._check(self.lib.lev_hip_forge_candidates(self.ctx, op, in_dim, rows, ncol, buf, 16, C.byref(n)))
        return [capi.Schedule(*buf[i].key()) for i in range(min(n.value, 16))]

    def forge_select(self, in_dim: int, rows: int, schedule, ncol: int = 1):
        self._check(self.lib.lev_hip_forge_select(self.ctx, in_dim, rows, ncol, C.byref(schedule)))

    def forge_clear(self, op: int, in_dim: int, rows: int, ncol: int = 1):
        self._check(self.lib.lev_hip_forge_clear(self.ctx, op, in_dim, rows, ncol))

    def q4_k_gemm_prefill(self, w, x_f16, in_dim: int, rows: int, tokens: int, y=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(x_f16, torch.float16, "x")
        if y is None:
            y = torch.empty((max(tokens, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q4_k_gemm_prefill(self.ctx, _ptr(w), w.numel(), w_off,
                                                       _ptr(x_f16), x_f16.numel(), _ptr(y),
                                                       y.numel(), in_dim, rows, tokens))
        return y

    def q6_k_gemm_prefill(self, w, x_f16, in_dim: int, rows: int, tokens: int, y=None, w_off: int = 0):
        _dev(w, torch.uint8, "w")
        _dev(x_f16, torch.float16, "x")
        if y is None:
            y = torch.empty((max(tokens, 1), max(rows, 1)), dtype=torch.float32, device=w.device)
        self._check(self.lib.lev_hip_q6_k_gemm_prefill(self.ctx, _ptr(w), w.numel(), w_off,
                                                       _ptr(x_f16), x_f16.numel(), _ptr(y),
                                                       y.numel(), in_dim, rows, tokens))
        return y

    def f32_to_f16(self, x):
        _dev(x, torch.float32, "x")
        out = torch.empty(x.shape, dtype=torch.float16, device=x.device)
        self._check(self.lib.lev_hip_f32_to_f16(self.ctx, _ptr(x), _ptr(out), x.numel()))
        return out

    # -- elementwise operators -------------------------------------------
    def rmsnorm(self, x, n: int, vectors: int, weight=None, eps: float = 1e-6, y=None):
        _dev(x, torch.float32, "x")
        if y is None:
            y = torch.empty_like(x)
        self._check(self.lib.lev_hip_rmsnorm(self.ctx, _ptr(x), _ptr(y), n, vectors, _ptr(weight),
                                             eps))
        return y

    def gelu_up(self, gu, n: int, y=None):
        _dev(gu, torch.float32, "gu")
        if y is None:
            y = torch.empty(max(n, 1), dtype=torch.float32, device=gu.device)
        self._check(self.lib.lev_hip_gelu_up(self.ctx, _ptr(gu), _ptr(y), n))
        return y

    def axpy(self, x, y, c: float, n: int):
        _dev(x, torch.float32, "x")
        _dev(y, torch.float32, "y")
        self._check(self.lib.lev_hip_axpy(self.ctx, _ptr(x), _ptr(y), c, n))
        return y

    def shared_expert_ffn(self, x, ffn_norm, gate_w, up_w, down_w, post_norm, hidden: int, inter: int,
                          eps: float = 1e-6, bufs=None):
        """The shared expert that runs beside the routed ones (Gemma4.swift:3742-3773):
        h = rmsnorm(x, ffn_norm); gu = [gate h | up h] (Q4_0 matvecs, up at float offset
        `inter` of the one buffer); act = gelu_up(gu); shared = rmsnorm(down act, post_norm).
        `bufs` = (h, gu, act, shared) to reuse buffers (a recorded program needs fixed ones).
        Returns (h, shared): h also feeds the routed experts."""
        if inter % 32 or hidden % 32 or (inter * 4) % 256:
            raise LevError(capi.BAD_DIMENSIONS,
                           f"shared expert: hidden {hidden} / intermediate {inter} (blocks of 32, up half 256-byte aligned)")
        if bufs is None:
            dev = x.device
            bufs = (torch.empty(hidden, dtype=torch.float32, device=dev),
                    torch.empty(2 * inter, dtype=torch.float32, device=dev),
                    torch.empty(inter, dtype=torch.float32, device=dev),
                    torch.empty(hidden, dtype=torch.float32, device=dev))
        h, gu, act, shared = bufs
        self.rmsnorm(x, hidden, 1, weight=ffn_norm, eps=eps, y=h)
        self.q4_0_gemv(gate_w, h, hidden, inter, y=gu)
        self.q4_0_gemv(up_w, h, hidden, inter, y=gu[inter:])
        self.gelu_up(gu, inter, y=act)
        self.q4_0_gemv(down_w, act, inter, hidden, y=shared)
        self.rmsnorm(shared, hidden, 1, weight=post_norm, eps=eps, y=shared)
        return h, shared

    def argmax(self, logits, vocab: int, ncol: int = 1):
        _dev(logits, torch.float32, "logits")
        idx = torch.empty(max(ncol, 1), dtype=torch.int32, device=logits.device)
        mg = torch.empty(max(ncol, 1), dtype=torch.float32, device=logits.device)
        self._check(self.lib.lev_hip_argmax(self.ctx, _ptr(logits), vocab, ncol, _ptr(idx), _ptr(mg)))
        return idx, mg

    # -- MoE ---------------------------------------------------------------
    @staticmethod
    def moe_pools(base: torch.Tensor, hidden: int, inter: int, experts: int, gate_off: int,
                  up_off: int, down_off: int, gate_stride=None, up_stride=None, down_stride=None):
        gu = inter * (hidden // 32) * 18
        dn = hidden * (inter // 32) * 18
        pools = capi.MoEExperts(C.c_void_p(base.data_ptr()), base.numel(), gate_off, up_off, down_off,
                                gate_stride or gu, up_stride or gu, down_stride or dn, hidden, inter,
                                experts)
        pools.keepalive = base      # the struct holds a raw pointer: the tensor lives as long as it
        return pools

    def moe_route_topk(self, router_w, x, hidden: int, experts: int, top_k: int, tokens: int,
                       expert_scale=None, want_scores: bool = False):
        _dev(router_w, torch.float32, "router_w")
        _dev(x, torch.float32, "x")
        ids = torch.empty((max(tokens, 1), max(top_k, 1)), dtype=torch.int32, device=x.device)
        wts = torch.empty((max(tokens, 1), max(top_k, 1)), dtype=torch.float32, device=x.device)
        scores = (torch.empty((max(tokens, 1), max(experts, 1)), dtype=torch.float32, device=x.device)
                  if want_scores else None)
        self._check(self.lib.lev_hip_moe_route_topk(self.ctx, _ptr(router_w), _ptr(x),
                                                    _ptr(expert_scale), _ptr(ids), _ptr(wts),
                                                    _ptr(scores), hidden, experts, top_k, tokens))
        return (ids, wts, scores) if want_scores else (ids, wts)

    def moe_experts_q4_0(self, pools, x, ids, weights, top_k: int, tokens: int, want_act=False):
        _dev(x, torch.float32, "x")
        _dev(ids, torch.int32, "ids")
        _dev(weights, torch.float32, "weights")
        y = torch.empty((max(tokens, 1), pools.hidden), dtype=torch.float32, device=x.device)
        act = (torch.empty((max(tokens, 1), max(top_k, 1), pools.inter), dtype=torch.float32,
                           device=x.device) if want_act else None)
        self._check(self.lib.lev_hip_moe_experts_q4_0(self.ctx, C.byref(pools), _ptr(x), _ptr(ids),
                                                      _ptr(weights), _ptr(y), _ptr(act), top_k,
                                                      tokens))
        return (y, act) if want_act else y

    def moe_layer_q4_0(self, pools, router_w, x, top_k: int, tokens: int, expert_scale=None, y=None,
                       ids=None, weights=None, noalloc: bool = False):
        """``noalloc``: the entry point that allocates nothing inside the call (static
        device scratch; pass ``y``, ``ids`` and ``weights`` so that this wrapper
        allocates nothing either)."""
        _dev(x, torch.float32, "x")
        if y is None:
            y = torch.empty((max(tokens, 1), pools.hidden), dtype=torch.float32, device=x.device)
        if ids is None:
            ids = torch.empty((max(tokens, 1), max(top_k, 1)), dtype=torch.int32, device=x.device)
        if weights is None:
            weights = torch.empty((max(tokens, 1), max(top_k, 1)), dtype=torch.float32,
                                  device=x.device)
        fn = self.lib.lev_hip_moe_layer_q4_0_noalloc if noalloc else self.lib.lev_hip_moe_layer_q4_0
        self._check(fn(self.ctx, C.byref(pools), _ptr(router_w), _ptr(expert_scale), _ptr(x), _ptr(y),
                       _ptr(ids), _ptr(weights), top_k, tokens))
        return y, ids, weights


class Program:
    """A recorded sequence of operator calls (``lev_program``), replayed with ``run()``."""

    def __init__(self, ctx: Context, handle):
        self.ctx, self.handle = ctx, handle

    def run(self):
        self.ctx._check(self.ctx.lib.lev_hip_program_run(self.ctx.ctx, self.handle))

    def node_count(self) -> int:
        n = C.c_size_t()
        self.ctx._check(self.ctx.lib.lev_hip_program_node_count(self.handle, C.byref(n)))
        return n.value

    def destroy(self):
        if self.handle:
            self.ctx._check(self.ctx.lib.lev_hip_program_destroy(self.ctx.ctx, self.handle))
            self.handle = None


# -- host-array twins of the standalone backends --------------------------

def _reporting(fn_name, blocks, out_dim, in_dim, x):
    import numpy as np
    lib = capi.load()
    b = np.ascontiguousarray(blocks, dtype=np.uint8)
    xv = np.ascontiguousarray(x, dtype=np.float32)
    y = np.zeros(max(int(out_dim), 1), dtype=np.float32)
    ev = capi.Evidence()
    st = getattr(lib, fn_name)(b.ctypes.data_as(C.c_void_p), b.size, int(out_dim), int(in_dim),
                               xv.ctypes.data_as(C.c_void_p), xv.size,
                               y.ctypes.data_as(C.c_void_p), C.byref(ev))
    if st != capi.OK:
        raise LevError(st, fn_name)
    return y[: int(out_dim)], ev


def q4_0_matvec_reporting(blocks, out_dim, in_dim, x):
    """``Q4MetalBackend.matvecReporting`` (Q4.swift:165) on the MI355X."""
    return _reporting("lev_hip_q4_0_matvec_reporting", blocks, out_dim, in_dim, x)


def q6_k_matvec_reporting(blocks, out_dim, in_dim, x):
    """``Q6MetalBackend.matvecReporting`` (Q6.swift:199) on the MI355X."""
    return _reporting("lev_hip_q6_k_matvec_reporting", blocks, out_dim, in_dim, x)
