"""ctypes binding of ``libleviathan_hip.so`` (the C ABI in ``include/leviathan_hip.h``).

This module is plumbing for tests, the benchmark and Python callers: it loads
the in-tree shared library and declares the argument types of every entry
point.  It contains no arithmetic and no fallback: if the library is missing
or an entry point fails, the caller gets an exception.
"""
from __future__ import annotations

import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "lib", "libleviathan_hip.so")

OK = 0
BAD_DIMENSIONS = 1
WRONG_INPUT_COUNT = 2
NON_FINITE_INPUT = 3
NON_FINITE_SCALE = 4
NON_FINITE_OUTPUT = 5
EXCEEDS_MODEL_WORKLOAD = 6
INTEGER_OVERFLOW = 7
DEVICE_UNAVAILABLE = 8
KERNEL_LOAD_FAILED = 9
FUNCTION_MISSING = 10
COMMAND_FAILED = 11
EXCEEDS_MAX_BUFFER_LENGTH = 12
EXCEEDS_WORKING_SET = 13
INVALID_ARGUMENT = 14

TYPE_F32, TYPE_F16, TYPE_Q4_0, TYPE_Q4_K, TYPE_Q6_K = 0, 1, 2, 12, 14


class Evidence(C.Structure):
    _fields_ = [("device_name", C.c_char * 128),
                ("device_max_buffer_length", C.c_uint64),
                ("recommended_max_working_set_size", C.c_uint64),
                ("out_dim", C.c_int64),
                ("in_dim", C.c_int64),
                ("command_status", C.c_char * 32)]


class MoEExperts(C.Structure):
    _fields_ = [("d_base", C.c_void_p), ("base_bytes", C.c_size_t),
                ("gate_off", C.c_uint64), ("up_off", C.c_uint64), ("down_off", C.c_uint64),
                ("gate_stride", C.c_uint64), ("up_stride", C.c_uint64), ("down_stride", C.c_uint64),
                ("hidden", C.c_uint32), ("inter", C.c_uint32), ("experts", C.c_uint32)]


class Schedule(C.Structure):
    _fields_ = [("op", C.c_uint32), ("family", C.c_uint32), ("rows_in_flight", C.c_uint32),
                ("persistent", C.c_uint32)]

    def key(self):
        return (self.op, self.family, self.rows_in_flight, self.persistent)


OP_Q4_0_GEMV, OP_Q4_K_GEMV, OP_Q4_K_GEMV_Q8 = 1, 2, 3
OP_Q6_K_GEMV, OP_Q6_K_GEMV_Q8, OP_MOE_LAYER_Q4_0 = 4, 5, 6

_vp, _sz, _u64, _u32, _f32, _i64, _int = (C.c_void_p, C.c_size_t, C.c_uint64, C.c_uint32, C.c_float,
                                          C.c_int64, C.c_int)

# name -> (restype, argtypes); mirrors include/leviathan_hip.h one to one.
SIGNATURES = {
    "lev_hip_abi_version": (_int, []),
    "lev_hip_status_name": (C.c_char_p, [_int]),
    "lev_hip_ctx_create": (_int, [_int, _vp, C.POINTER(_vp)]),
    "lev_hip_ctx_destroy": (_int, [_vp]),
    "lev_hip_sync": (_int, [_vp]),
    "lev_hip_last_error": (C.c_char_p, [_vp]),
    "lev_hip_device_name": (_int, [_vp, C.c_char_p, _sz]),
    "lev_hip_program_begin": (_int, [_vp]),
    "lev_hip_program_end": (_int, [_vp, C.POINTER(_vp)]),
    "lev_hip_program_run": (_int, [_vp, _vp]),
    "lev_hip_program_destroy": (_int, [_vp, _vp]),
    "lev_hip_program_node_count": (_int, [_vp, C.POINTER(_sz)]),
    "lev_hip_buf_alloc": (_int, [_vp, _sz, C.POINTER(_vp)]),
    "lev_hip_buf_free": (_int, [_vp, _vp]),
    "lev_hip_buf_upload": (_int, [_vp, _vp, _vp, _sz]),
    "lev_hip_buf_download": (_int, [_vp, _vp, _vp, _sz]),
    "lev_hip_stream_read_probe": (_int, [_vp, _vp, _sz, _vp, _u32]),
    "lev_hip_empty_launch": (_int, [_vp]),
    "lev_hip_dequant": (_int, [_vp, _int, _vp, _sz, _u64, _u64, _vp, _sz]),
    "lev_hip_q4_0_gemv": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _sz, _u32, _u32]),
    "lev_hip_q6_k_gemv": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _sz, _u32, _u32, _vp, _vp]),
    "lev_hip_q4_k_gemv_ncol": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _f32, _vp, _sz, _u32,
                                      _u32, _u32]),
    "lev_hip_q6_k_gemv_ncol": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _f32, _vp, _sz, _u32,
                                      _u32, _u32]),
    "lev_hip_norm_quant_q8": (_int, [_vp, _vp, _sz, _vp, _vp, _f32, _vp, _vp, _vp, _u32, _u32]),
    "lev_hip_q4_k_gemv_q8": (_int, [_vp, _vp, _sz, _u64, _vp, _vp, _sz, _vp, _sz, _u32, _u32, _u32]),
    "lev_hip_q6_k_gemv_q8": (_int, [_vp, _vp, _sz, _u64, _vp, _vp, _sz, _vp, _sz, _u32, _u32, _u32]),
    "lev_hip_swiglu_quant_q8": (_int, [_vp, _vp, _vp, _sz, _vp, _vp, _vp]),
    "lev_hip_embed_q4_k": (_int, [_vp, _vp, _sz, _u64, _vp, _u32, _vp, _sz, _u32, _u32]),
    "lev_hip_q4_k_gemm_prefill": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _sz, _u32, _u32, _u32]),
    "lev_hip_q6_k_gemm_prefill": (_int, [_vp, _vp, _sz, _u64, _vp, _sz, _vp, _sz, _u32, _u32, _u32]),
    "lev_hip_f32_to_f16": (_int, [_vp, _vp, _vp, _sz]),
    "lev_hip_rmsnorm": (_int, [_vp, _vp, _vp, _u32, _u32, _vp, _f32]),
    "lev_hip_gelu_up": (_int, [_vp, _vp, _vp, _u32]),
    "lev_hip_axpy": (_int, [_vp, _vp, _vp, _f32, _u32]),
    "lev_hip_argmax": (_int, [_vp, _vp, _u32, _u32, _vp, _vp]),
    "lev_hip_moe_route_topk": (_int, [_vp, _vp, _vp, _vp, _vp, _vp, _vp, _u32, _u32, _u32, _u32]),
    "lev_hip_moe_experts_q4_0": (_int, [_vp, C.POINTER(MoEExperts), _vp, _vp, _vp, _vp, _vp, _u32,
                                        _u32]),
    "lev_hip_moe_layer_q4_0": (_int, [_vp, C.POINTER(MoEExperts), _vp, _vp, _vp, _vp, _vp, _vp,
                                      _u32, _u32]),
    "lev_hip_moe_layer_q4_0_noalloc": (_int, [_vp, C.POINTER(MoEExperts), _vp, _vp, _vp, _vp, _vp, _vp,
                                              _u32, _u32]),
    "lev_hip_forge_candidates": (_int, [_vp, _u32, _u32, _u32, _u32, C.POINTER(Schedule), _u32,
                                        C.POINTER(_u32)]),
    "lev_hip_forge_select": (_int, [_vp, _u32, _u32, _u32, C.POINTER(Schedule)]),
    "lev_hip_forge_clear": (_int, [_vp, _u32, _u32, _u32, _u32]),
    "lev_hip_q4_0_matvec_reporting": (_int, [_vp, _sz, _i64, _i64, _vp, _sz, _vp,
                                             C.POINTER(Evidence)]),
    "lev_hip_q6_k_matvec_reporting": (_int, [_vp, _sz, _i64, _i64, _vp, _sz, _vp,
                                             C.POINTER(Evidence)]),
}


class LibraryMissing(RuntimeError):
    pass


_lib = None


def load(path: str = LIB_PATH) -> C.CDLL:
    """Load the in-tree library.  Raises ``LibraryMissing`` if it was not built."""
    global _lib
    if _lib is not None:
        return _lib
    if not os.path.exists(path):
        raise LibraryMissing(
            f"{path} not found: build it with `python -m leviathan_amd.build` "
            "(there is no CPU fallback)")
    try:
        # Share the HIP runtime torch already loaded, when torch is in use.
        import torch  # noqa: F401
    except Exception:
        pass
    lib = C.CDLL(path)
    for name, (res, args) in SIGNATURES.items():
        fn = getattr(lib, name)          # AttributeError if a symbol is missing
        fn.restype = res
        fn.argtypes = args
    _lib = lib
    return lib


def exported_symbols(path: str = LIB_PATH) -> set[str]:
    """Dynamic symbols of the library, read without loading it (no GPU needed)."""
    import subprocess
    out = subprocess.run(["nm", "-D", "--defined-only", path], capture_output=True, text=True,
                         check=True).stdout
    return {line.split()[-1] for line in out.splitlines() if line.strip()}
