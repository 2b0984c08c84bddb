"""GGUF directory reader and MoE expert binding (host side, no GPU).

* the oracle parser (oracle/gguf.py) against the reference's own reader tests
  (rust/crates/lev-gguf/src/lib.rs:498-564: tiny file, truncated data, partial
  block, bad magic, huge counts, block sizes);
* the C++ reader of leviathan_amd/host/leviathan_gguf.hpp against the oracle's
  canonical dump, on accepted and rejected files;
* the expert binding (MoEModelBinding.swift:95-214) on a synthetic gemma4 file.
"""
import os
import struct
import subprocess

import numpy as np
import pytest

from oracle import gguf as G
from tests import helpers as H

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
TOOL = os.path.join(ROOT, "tests", "host", "build", "gguf_tool")


def tool():
    if not os.path.exists(TOOL):
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host")], check=True, stdout=subprocess.DEVNULL)
    return TOOL


def tiny_gguf(tensor_ty, dims, data_bytes):
    """tiny_gguf of lev-gguf/src/lib.rs:498-522: one string, one u32, one tensor."""
    b = b"GGUF" + struct.pack("<IQQ", 3, 1, 2)
    b += H.gguf_str("general.architecture") + struct.pack("<I", 8) + H.gguf_str("test")
    b += H.gguf_str("test.block_count") + struct.pack("<II", 4, 7)
    b += H.gguf_str("blk.0.w") + struct.pack("<I", len(dims)) + b"".join(struct.pack("<Q", d) for d in dims)
    b += struct.pack("<IQ", tensor_ty, 0)
    b += b"\0" * (-len(b) % 32)
    return b + b"\0" * data_bytes


# ---------------------------------------------------- the reference's tests ----

def test_oracle_parses_tiny_file():
    g = G.parse(tiny_gguf(12, [256, 2], 2 * 144))
    assert g["version"] == 3
    assert g["metadata"][b"general.architecture"] == (8, b"test")
    assert g["metadata"][b"test.block_count"] == (4, 7)
    assert g["tensors"][0]["type"] == 12 and g["tensors"][0]["size"] == 288
    assert g["data_offset"] % 32 == 0


def test_oracle_rejects_what_the_reference_rejects():
    for bad in (tiny_gguf(12, [256, 2], 100),            # truncated tensor data
                tiny_gguf(12, [100], 1000),              # partial block
                b"NOPE",                                  # magic
                b"GGUF" + struct.pack("<IQQ", 3, (1 << 64) - 1, 0)):   # huge tensor count
        with pytest.raises(G.GgufError):
            G.parse(bad)


def test_block_layouts_match_known_sizes():
    assert G.BLOCK_LAYOUT[2] == (32, 18) and G.BLOCK_LAYOUT[12] == (256, 144) and G.BLOCK_LAYOUT[14] == (256, 210)
    assert G.byte_size(2, [4096, 4096]) == 4096 * 4096 // 32 * 18
    assert G.byte_size(14, [4096, 32000]) == 107_520_000
    assert G.byte_size(12, [100]) is None and G.byte_size(99, [32]) is None


# ------------------------------------------------- C++ reader vs the oracle ----

def every_kind_of_value():
    kvs = [
        ("general.architecture", 8, "gemma4"),
        ("general.alignment", 4, 64),
        ("a.u8", 0, 200), ("a.i8", 1, -5), ("a.u16", 2, 60000), ("a.i16", 3, -30000),
        ("a.u32", 4, 4_000_000_000), ("a.i32", 5, -2_000_000_000), ("a.f32", 6, 1.5),
        ("a.bool", 7, 1), ("a.str", 8, "héllo wörld"), ("a.empty", 8, ""),
        ("a.u64", 10, (1 << 63) + 5), ("a.i64", 11, -(1 << 40)), ("a.f64", 12, -2.25),
        ("arr.kept", 9, (5, list(range(-3, 61)))),                       # 64 elements: kept
        ("arr.long", 9, (4, list(range(65)))),                           # 65: skipped
        ("arr.strs", 9, (8, ["a", "bc", ""])),
        ("tokenizer.ggml.tokens", 9, (8, [f"tok{i}" for i in range(100)])),   # long string array: skipped
    ]
    tensors = [
        ("token_embd.weight", [256, 10], 12, bytes(144 * 10)),
        ("blk.0.attn_q.weight", [64, 64], 2, bytes(64 * 64 // 32 * 18)),
        ("output.weight", [256, 3], 14, bytes(210 * 3)),
        ("blk.0.norm.weight", [64], 0, bytes(256)),
        ("blk.0.half.weight", [8, 2, 2], 1, bytes(64)),
    ]
    return kvs, tensors


def run_tool(tmp_path, data, mode="dump"):
    p = tmp_path / "f.gguf"
    p.write_bytes(data)
    r = subprocess.run([tool(), mode, str(p)], capture_output=True, text=True, timeout=60)
    return r.returncode, r.stdout


def test_cpp_reader_dump_equals_oracle_dump(tmp_path):
    kvs, tensors = every_kind_of_value()
    for version in (2, 3):
        data = H.write_gguf(kvs, tensors, version=version, alignment=64)
        g = G.parse(data)
        assert g["alignment"] == 64 and g["data_offset"] % 64 == 0 and len(g["skipped"]) == 2
        assert [t["offset"] % 64 for t in g["tensors"]] == [0] * 5
        rc, out = run_tool(tmp_path, data)
        assert rc == 0, out
        assert out == G.dump(g)
    # the reference's tiny file too
    data = tiny_gguf(12, [256, 2], 2 * 144)
    rc, out = run_tool(tmp_path, data)
    assert rc == 0 and out == G.dump(G.parse(data))


def test_skipped_array_offsets_point_at_the_elements():
    kvs, tensors = every_kind_of_value()
    data = H.write_gguf(kvs, tensors, alignment=64)
    g = G.parse(data)
    et, n, at = g["skipped"][b"arr.long"]
    assert (et, n) == (4, 65) and struct.unpack_from("<65I", data, at) == tuple(range(65))
    et, n, at = g["skipped"][b"tokenizer.ggml.tokens"]
    assert data[at:at + 12] == H.gguf_str("tok0")


def mutations():
    kvs, tensors = every_kind_of_value()
    good = H.write_gguf(kvs, tensors, alignment=64)
    yield "truncated file", good[:-1]
    yield "truncated directory", good[:100]
    yield "bad magic", b"GGML" + good[4:]
    yield "version 1", good[:4] + struct.pack("<I", 1) + good[8:]
    yield "version 4", good[:4] + struct.pack("<I", 4) + good[8:]
    yield "huge kv count", good[:16] + struct.pack("<Q", (1 << 16) + 1) + good[24:]
    yield "huge tensor count", good[:8] + struct.pack("<Q", (1 << 20) + 1) + good[16:]
    yield "duplicate key", H.write_gguf(kvs + [("a.u8", 0, 1)], tensors, alignment=64)
    yield "duplicate tensor", H.write_gguf(kvs, tensors + [tensors[0]], alignment=64)
    yield "nested array", H.write_gguf([("x", 9, (9, []))], [])
    yield "unknown value type", H.write_gguf([], [])[:16] + struct.pack("<Q", 1) + H.gguf_str("k") + struct.pack("<I", 13)
    yield "alignment 48", H.write_gguf([("general.alignment", 4, 48)], tensors, alignment=48)
    yield "alignment 0", H.write_gguf([("general.alignment", 4, 0)], [])
    yield "alignment as string", H.write_gguf([("general.alignment", 8, "32")], [])
    yield "partial block", H.write_gguf([], [("w", [100], 12, bytes(1000))])
    yield "unknown tensor type", H.write_gguf([], [("w", [32], 99, bytes(64))])
    yield "zero dims", H.write_gguf([], [("w", [], 0, b"")])
    yield "nine dims", H.write_gguf([], [("w", [1] * 9, 0, bytes(4))])
    yield "zero dimension", H.write_gguf([], [("w", [32, 0], 2, b"")])
    yield "element count overflows", H.write_gguf([], [("w", [1 << 40, 1 << 40], 0, bytes(4))])
    yield "invalid utf-8 key", H.write_gguf([(b"\xff\xfe", 4, 1)], [])
    yield "string beyond bound", b"GGUF" + struct.pack("<IQQ", 3, 0, 1) + struct.pack("<Q", (1 << 24) + 1)
    # tensor offset not a multiple of the alignment: patch the directory entry of a one-tensor file
    one = H.write_gguf([], [("w", [32], 2, bytes(18))], pad_data_to=4096)
    at = one.index(H.gguf_str("w")) + 9 + 4 + 8 + 4
    yield "misaligned offset", one[:at] + struct.pack("<Q", 8) + one[at + 8:]
    yield "offset beyond file", one[:at] + struct.pack("<Q", 1 << 40) + one[at + 8:]


def test_cpp_reader_rejects_exactly_what_the_oracle_rejects(tmp_path):
    n = 0
    for what, data in mutations():
        with pytest.raises(G.GgufError):
            G.parse(data)
        rc, out = run_tool(tmp_path, data)
        assert rc == 2 and out.startswith("error:"), (what, rc, out)
        n += 1
    assert n == 24


def test_directory_larger_than_the_first_read(tmp_path):
    """The reader grows its directory window (1 MiB first) until the directory fits."""
    kvs = [("tokenizer.ggml.tokens", 9, (8, ["t%07d" % i for i in range(120_000)]))]
    data = H.write_gguf(kvs, [("w", [32], 2, bytes(18))])
    assert G.parse(data)["data_offset"] > (1 << 20)
    rc, out = run_tool(tmp_path, data)
    assert rc == 0 and out == G.dump(G.parse(data))


# ------------------------------------------------------- expert binding ----

def gemma4_file(layers=2, experts=4, top_k=2, hidden=64, inter=32, **over):
    kvs = [("general.architecture", 8, over.get("arch", "gemma4")),
           ("gemma4.block_count", 4, layers), ("gemma4.expert_count", 4, experts),
           ("gemma4.expert_used_count", 4, top_k), ("gemma4.embedding_length", 4, hidden),
           ("gemma4.expert_feed_forward_length", 4, inter)]
    gu = hidden // 32 * 18 * 2 * inter * experts
    dn = inter // 32 * 18 * hidden * experts
    tensors = []
    for l in range(over.get("tensor_layers", layers)):
        tensors.append((f"blk.{l}.attn_q.weight", [hidden, hidden], 2, bytes(hidden // 32 * 18 * hidden)))
        tensors.append((f"blk.{l}.ffn_gate_up_exps.weight", [hidden, 2 * inter, over.get("gu_experts", experts)],
                        over.get("gu_type", 2), bytes(gu if "gu_experts" not in over else gu // experts * over["gu_experts"])))
        tensors.append((f"blk.{l}.ffn_down_exps.weight", [inter, hidden, experts], 2, bytes(dn)))
    return H.write_gguf(kvs, tensors), gu // experts, dn // experts


def test_moe_binding_offsets_and_strides(tmp_path):
    data, gu_stride, dn_stride = gemma4_file()
    g = G.parse(data)
    rc, out = run_tool(tmp_path, data, "bind")
    assert rc == 0, out
    lines = out.splitlines()
    assert lines[0] == f"layers 2 experts 4 topk 2 hidden 64 inter 32 gu_stride {gu_stride} dn_stride {dn_stride}"
    assert gu_stride == 64 // 32 * 18 * 64 and dn_stride == 32 // 32 * 18 * 64      # whole Q4_0 rows
    by_name = {t["name"]: g["data_offset"] + t["offset"] for t in g["tensors"]}
    for l in range(2):
        assert lines[1 + l] == (f"layer {l} gu {by_name[b'blk.%d.ffn_gate_up_exps.weight' % l]} "
                                f"dn {by_name[b'blk.%d.ffn_down_exps.weight' % l]}")
    # the route (1, 0) of the last layer: slot order kept, id * stride from the tensor start
    gu1, dn1 = by_name[b"blk.1.ffn_gate_up_exps.weight"], by_name[b"blk.1.ffn_down_exps.weight"]
    assert lines[3] == f"slot 0 id 1 gu {gu1 + gu_stride} dn {dn1 + dn_stride}"
    assert lines[4] == f"slot 1 id 0 gu {gu1} dn {dn1}"


@pytest.mark.parametrize("over", [dict(arch="llama"), dict(tensor_layers=1), dict(gu_type=12), dict(gu_experts=3),
                                  dict(top_k=5), dict(hidden=8224), dict(top_k=0)])
def test_moe_binding_rejects(tmp_path, over):
    kw = {k: v for k, v in over.items() if k in ("top_k", "hidden", "experts")}
    ov = {k: v for k, v in over.items() if k not in kw}
    if ov.get("gu_type") == 12:
        kw["hidden"] = 256                   # a whole Q4_K block per row, so that only the type is wrong
    data, _, _ = gemma4_file(**kw, **ov)
    G.parse(data)                            # a well-formed file ...
    rc, out = run_tool(tmp_path, data, "bind")
    assert rc == 2 and out.startswith("error:"), out      # ... that is not a bindable model
