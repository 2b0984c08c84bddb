"""CPU-only checks of the drop-in boundary: the shared library exists, loads,
exports every symbol ``include/leviathan_hip.h`` declares, its status codes
agree with the oracle's, and it fails loudly (no CPU fallback) without a GPU.
"""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "leviathan_hip.h")


def declared_functions():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(lev_hip_\w+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    names = declared_functions()
    for must in ["lev_hip_ctx_create", "lev_hip_sync", "lev_hip_buf_alloc", "lev_hip_dequant",
                 "lev_hip_q4_0_gemv", "lev_hip_q6_k_gemv", "lev_hip_q4_k_gemv_ncol",
                 "lev_hip_q4_k_gemm_prefill", "lev_hip_q6_k_gemm_prefill", "lev_hip_moe_route_topk", "lev_hip_moe_experts_q4_0",
                 "lev_hip_moe_layer_q4_0", "lev_hip_rmsnorm", "lev_hip_gelu_up", "lev_hip_axpy",
                 "lev_hip_argmax", "lev_hip_q4_0_matvec_reporting", "lev_hip_q6_k_matvec_reporting"]:
        assert must in names


def test_library_exports_every_declared_symbol():
    from leviathan_amd import capi
    assert os.path.exists(capi.LIB_PATH), "run `python -m leviathan_amd.build` first"
    exported = capi.exported_symbols()
    missing = [n for n in declared_functions() if n not in exported]
    assert not missing, missing


def test_ctypes_signatures_cover_the_header():
    from leviathan_amd import capi
    assert sorted(capi.SIGNATURES) == declared_functions()


def test_library_loads_and_reports_without_a_gpu():
    from leviathan_amd import capi
    lib = capi.load()
    assert lib.lev_hip_abi_version() == 2
    assert lib.lev_hip_status_name(0) == b"ok"
    assert lib.lev_hip_status_name(capi.BAD_DIMENSIONS) == b"badDimensions"
    assert lib.lev_hip_status_name(capi.NON_FINITE_SCALE) == b"nonFiniteScale"
    assert lib.lev_hip_status_name(capi.EXCEEDS_WORKING_SET) == b"exceedsWorkingSet"


def test_status_codes_agree_between_header_binding_and_oracle():
    import oracle as O
    from leviathan_amd import capi
    text = open(HEADER).read()
    enum = dict((m.group(1), int(m.group(2)))
                for m in re.finditer(r"LEV_(?:ERR_)?(\w+)\s*=\s*(\d+)", text))
    for name in ["BAD_DIMENSIONS", "WRONG_INPUT_COUNT", "NON_FINITE_INPUT", "NON_FINITE_SCALE",
                 "NON_FINITE_OUTPUT", "EXCEEDS_MODEL_WORKLOAD", "INTEGER_OVERFLOW", "INVALID_ARGUMENT"]:
        assert enum[name] == getattr(capi, name) == getattr(O, name), name
    assert enum["OK"] == 0 and enum["TYPE_Q4_0"] == 2 and enum["TYPE_Q4_K"] == 12 and enum["TYPE_Q6_K"] == 14


def test_no_cpu_fallback_without_a_gpu():
    import torch
    if torch.cuda.is_available():
        pytest.skip("GPU present")
    from leviathan_amd import capi, ops
    with pytest.raises(RuntimeError):
        ops.Context(0)
    lib = capi.load()
    ctx = C.c_void_p()
    assert lib.lev_hip_ctx_create(0, C.c_void_p(0), C.byref(ctx)) == capi.DEVICE_UNAVAILABLE
    # the host-array twin validates first, then needs the device
    import numpy as np
    x = np.zeros(32, np.float32)
    w = np.zeros(18, np.uint8)
    y = np.zeros(1, np.float32)
    st = lib.lev_hip_q4_0_matvec_reporting(w.ctypes.data_as(C.c_void_p), 18, 1, 33,
                                           x.ctypes.data_as(C.c_void_p), 32,
                                           y.ctypes.data_as(C.c_void_p), None)
    assert st == capi.BAD_DIMENSIONS
    st = lib.lev_hip_q4_0_matvec_reporting(w.ctypes.data_as(C.c_void_p), 18, 1, 32,
                                           x.ctypes.data_as(C.c_void_p), 32,
                                           y.ctypes.data_as(C.c_void_p), None)
    assert st == capi.DEVICE_UNAVAILABLE


def test_product_code_never_touches_the_oracle():
    """The shipped package must not import, load or link anything under oracle/."""
    pkg = os.path.join(ROOT, "leviathan_amd")
    for dirpath, _, files in os.walk(pkg):
        if os.path.basename(dirpath) in ("build", "lib", "__pycache__"):
            continue
        for f in files:
            if f.endswith((".py", ".hip", ".hpp", ".h", ".cpp")):
                text = open(os.path.join(dirpath, f)).read()
                assert "lev_oracle" not in text and "import oracle" not in text \
                    and "from oracle" not in text, os.path.join(dirpath, f)


def test_grouped_moe_offset_scan_writes_every_entry():
    """The per-expert offsets of the grouped MoE path (moe_group_kernel): 1024 threads,
    thread i owns experts 4i..4i+3 and writes goff[e] for e <= experts from its running
    sum; at 4096 experts the total goff[4096] lies past the last thread's share and is
    written by the thread that owns expert 4095.  Restated on the host for every expert
    count: each of the experts+1 entries is written exactly once and equals the
    exclusive prefix sum."""
    import numpy as np
    rng = np.random.default_rng(7)
    for experts in list(range(1, 70)) + [255, 256, 257, 300, 1023, 1024, 1500, 4092, 4093, 4094, 4095, 4096]:
        cnt = rng.integers(0, 5, experts)
        goff = np.full(experts + 1, -1, np.int64)
        writes = np.zeros(experts + 1, np.int64)
        padded = np.zeros(4096, np.int64)
        padded[:experts] = cnt
        local = padded.reshape(1024, 4).sum(axis=1)
        before = np.concatenate([[0], np.cumsum(local)[:-1]])            # what the shuffle scan leaves per thread
        for tid in range(1024):
            run = before[tid]
            for k in range(4):
                e = 4 * tid + k
                if e <= experts:
                    goff[e] = run
                    writes[e] += 1
                run += padded[e]
            if 4 * tid + 4 == experts and experts == 4096:
                goff[experts] = run
                writes[experts] += 1
        assert np.all(writes == 1), experts
        assert np.array_equal(goff, np.concatenate([[0], np.cumsum(cnt)])), experts
