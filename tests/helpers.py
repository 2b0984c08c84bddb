"""Input builders shared by the tests.

The generators that carry a reference citation reproduce, draw for draw, the
synthetic inputs of the reference's own tests, so that the same bytes reach the
oracle and the HIP path.
"""
from __future__ import annotations

import struct

import numpy as np

import oracle as O


def f16_bits(v: float) -> int:
    return int(np.array([v], dtype=np.float32).astype(np.float16).view(np.uint16)[0])


def swift_q4_0_blocks(seed: int, nblocks: int) -> np.ndarray:
    """Sources/leviathan-tests/main.swift:753-761: Float16(nextUniform()*2-1)
    scale, then 16 bytes of next() & 0xFF."""
    rng = O.SplitMix64(seed)
    out = np.empty(nblocks * 18, dtype=np.uint8)
    for b in range(nblocks):
        s = np.float32(rng.next_uniform()) * np.float32(2) - np.float32(1)
        h = f16_bits(s)
        out[b * 18] = h & 0xFF
        out[b * 18 + 1] = h >> 8
        for i in range(16):
            out[b * 18 + 2 + i] = rng.next() & 0xFF
    return out


def swift_q6_k_blocks(seed: int, nblocks: int) -> np.ndarray:
    """main.swift:1032-1041: 208 random bytes then a finite Float16 d."""
    rng = O.SplitMix64(seed)
    out = np.empty(nblocks * 210, dtype=np.uint8)
    for b in range(nblocks):
        for i in range(208):
            out[b * 210 + i] = rng.next() & 0xFF
        s = np.float32(rng.next_uniform()) * np.float32(2) - np.float32(1)
        h = f16_bits(s)
        out[b * 210 + 208] = h & 0xFF
        out[b * 210 + 209] = h >> 8
    return out


def swift_synthetic_blocks(rng: "O.SplitMix64", nblocks: int) -> np.ndarray:
    """main.swift:6560-6571 / Q4Lowering.swift:779-791: two random scale bytes
    (exponent-all-ones replaced by 1.0), 16 random code bytes."""
    out = np.empty(nblocks * 18, dtype=np.uint8)
    for b in range(nblocks):
        lo, hi = rng.next() & 0xFF, rng.next() & 0xFF
        if ((lo | (hi << 8)) & 0x7C00) == 0x7C00:
            lo, hi = 0x00, 0x3C
        out[b * 18], out[b * 18 + 1] = lo, hi
        for i in range(16):
            out[b * 18 + 2 + i] = rng.next() & 0xFF
    return out


RUST_HALVES = [0x2E66, 0x3000, 0x3266, 0x2800, 0x1C00, 0x3400]


def rust_q4_k_blocks(rng: "O.SplitMix64", nblocks: int) -> np.ndarray:
    """random_blocks of rust/crates/lev-cpu/src/lib.rs:396-408."""
    out = np.zeros(nblocks * 144, dtype=np.uint8)
    for b in range(nblocks):
        o = b * 144
        h = RUST_HALVES[rng.next() % 6]
        out[o], out[o + 1] = h & 0xFF, h >> 8
        h = RUST_HALVES[rng.next() % 6]
        out[o + 2], out[o + 3] = h & 0xFF, h >> 8
        for i in range(140):
            out[o + 4 + i] = rng.next() & 0xFF
    return out


def minus_315_block():
    """The hand-computed Q6_K fixture of main.swift:1091-1112."""
    block = np.zeros(210, dtype=np.uint8)
    block[208], block[209] = 0x00, 0x3C
    block[192], block[193], block[196], block[200], block[204] = 3, 0xFD, 2, 3, 2
    block[0], block[128], block[64], block[160] = 0x21, 0x03, 0x21, 0x01
    x = np.zeros(256, dtype=np.float32)
    x[0], x[16], x[64], x[128], x[192] = 1, -1, 2, -2, 4
    return block, x


def hand_moe():
    """main.swift:8925-8938: hidden 32, inter 32, top-1; gate 16, up 2, act 32, down 512."""
    def block(lo, hi, q):
        return [lo, hi] + [q] * 16
    gate = np.array(sum((block(0x00, 0x3C, 0x98) for _ in range(32)), []), dtype=np.uint8)
    up = np.array(sum((block(0x00, 0x30, 0x98) for _ in range(32)), []), dtype=np.uint8)
    down = np.array(sum((block(0x00, 0x38, 0x99) for _ in range(32)), []), dtype=np.uint8)
    return gate, up, down


# ---- the five benchmark configurations (seeded, this build's generators) ----

def config1(rows=4096, cols=4096, seed=1):
    return O.synth_q4_0(seed, rows * cols // 32, 0.02), O.normal(cols, seed + 1000)


def config2(rows=32000, cols=4096, seed=2):
    return O.synth_q6_k(seed, rows * cols // 256, 0.01), O.normal(cols, seed + 1000)


def config3(rows=12288, cols=4096, ncol=8, seed=3):
    w = O.synth_q4_k(seed, rows * cols // 256, 0.01)
    x = O.normal(ncol * cols, seed + 1000).reshape(ncol, cols)
    gain = O.normal(cols, seed + 2000, 1.0, 0.1)
    return w, x, gain


def config4(rows=12288, cols=4096, tokens=512, seed=4):
    w = O.synth_q4_k(seed, rows * cols // 256, 0.01)
    x = O.normal(tokens * cols, seed + 1000).astype(np.float16).reshape(tokens, cols)
    return w, x


def config5(hidden=2048, inter=768, experts=128, tokens=1, seed=5):
    """Returns (router_w [E,H], pool bytes, offsets dict, x [T,H])."""
    gu = inter * (hidden // 32) * 18
    dn = hidden * (inter // 32) * 18
    gate = O.synth_q4_0(seed, experts * gu // 18, 0.02)
    up = O.synth_q4_0(seed + 1, experts * gu // 18, 0.02)
    down = O.synth_q4_0(seed + 2, experts * dn // 18, 0.02)
    pool = np.concatenate([gate, up, down])
    offs = dict(gate_off=0, up_off=gate.size, down_off=gate.size + up.size,
                gate_stride=gu, up_stride=gu, down_stride=dn)
    wr = O.normal(experts * hidden, seed + 3, 0.0, 0.02).reshape(experts, hidden)
    x = O.normal(tokens * hidden, seed + 1000).reshape(tokens, hidden)
    return wr, pool, offs, x


def rmsnorm_rows(x, gain, eps=1e-6):
    """Reference RMSNorm (lev-model/src/lib.rs:110-114) applied per row."""
    return np.stack([O.rmsnorm(r, gain, eps) for r in np.atleast_2d(x)])


# ---- GGUF files for the reader tests (the container format of the weights) ----

def gguf_str(s) -> bytes:
    raw = s if isinstance(s, bytes) else s.encode("utf-8")
    return struct.pack("<Q", len(raw)) + raw


_GGUF_FMT = {0: "<B", 1: "<b", 2: "<H", 3: "<h", 4: "<I", 5: "<i", 6: "<f", 7: "<B", 10: "<Q", 11: "<q", 12: "<d"}


def gguf_value(ty: int, v) -> bytes:
    if ty == 8:
        return gguf_str(v)
    if ty == 9:
        et, items = v
        return struct.pack("<IQ", et, len(items)) + b"".join(gguf_value(et, x) for x in items)
    return struct.pack(_GGUF_FMT[ty], v)


def write_gguf(kvs, tensors, version=3, alignment=None, pad_data_to=None) -> bytes:
    """kvs: [(key, type id, value)]; tensors: [(name, dims, type id, data bytes)].
    Tensor data is laid out in order, each at the next multiple of the alignment."""
    align = alignment or 32
    out = b"GGUF" + struct.pack("<IQQ", version, len(tensors), len(kvs))
    for key, ty, v in kvs:
        out += gguf_str(key) + struct.pack("<I", ty) + gguf_value(ty, v)
    offsets, off = [], 0
    for name, dims, ty, data in tensors:
        off = -(-off // align) * align
        offsets.append(off)
        off += len(data)
    for (name, dims, ty, data), o in zip(tensors, offsets):
        out += gguf_str(name) + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
        out += struct.pack("<IQ", ty, o)
    out += b"\0" * (-len(out) % align)
    body = b""
    for (name, dims, ty, data), o in zip(tensors, offsets):
        body += b"\0" * (o - len(body)) + bytes(data)
    out += body
    if pad_data_to is not None:
        out += b"\0" * max(0, pad_data_to - len(out))
    return out


def check_moe_layer_token(y, ids, wts, ref_ids, ref_w, gate, up, down, hidden, inter, x, tol=1e-4):
    """Parity of one token of the whole MoE block, stated as the reference states it:
    the router and the expert composite have separate contracts.
      * expert ids: bit-exact with the CPU route (F32 matvec + f64 softmax / top-k);
      * routing weights: within 2e-5 relative of the CPU route (the device accumulates
        the router scores in f64, the CPU reference in f32, so they are not bit-equal);
      * expert composite: the output against the FP64 oracle evaluated on the routing
        weights the device produced, at the reference's 1e-4 (MoESIMDOracle.contract);
      * and against the FP64 oracle on the CPU route's weights the output may differ by
        that 1e-4 plus what the weight difference itself moves it:
        sum_slot |w_dev - w_cpu| * |down_slot|.
    Returns the composite's error."""
    assert ids.tolist() == list(ref_ids), (ids, ref_ids)
    assert np.allclose(wts, ref_w, rtol=2e-5)
    ref = O.moe_experts_f64(gate, up, down, hidden, inter, ids, wts, x)
    err = O.max_rel_err(y, ref["y"])
    assert err < tol, err
    ref_cpu = O.moe_experts_f64(gate, up, down, hidden, inter, ref_ids, ref_w, x)
    moved = np.abs(wts.astype(np.float64) - np.asarray(ref_w, np.float64)) @ np.abs(ref_cpu["dn"])
    slack = tol * np.maximum(1.0, np.abs(ref_cpu["y"])) + moved
    assert np.all(np.abs(y - ref_cpu["y"]) <= slack)
    return err
