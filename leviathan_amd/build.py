"""Builds ``libleviathan_hip.so`` (gfx950 only) from ``csrc/*.hip`` with hipcc.

Run ``python -m leviathan_amd.build``.  hipcc cross-compiles without a GPU.
Objects are compiled in parallel and linked into ``leviathan_amd/lib``.
"""
from __future__ import annotations

import os
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
OBJ_DIR = os.path.join(HERE, "build")
LIB_PATH = os.path.join(LIB_DIR, "libleviathan_hip.so")

ARCH = "gfx950"
HIPCC_FLAGS = [
    f"--offload-arch={ARCH}", "-O3", "-std=c++17", "-fPIC", "-fno-gpu-rdc",
    "-Wall", "-Wno-unused-function", "-Wno-unknown-warning-option",
    # packed FP32 VALU ops are not to be generated for this hardware pool
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
]


def hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found")
    return exe


def sources() -> list[str]:
    return sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))


def _headers_mtime() -> float:
    paths = [os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hpp")]
    paths.append(os.path.join(HERE, "..", "include", "leviathan_hip.h"))
    return max(os.path.getmtime(p) for p in paths)


def _compile(src: str, force: bool, extra: list[str]) -> str:
    obj = os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o")
    if (not force and os.path.exists(obj)
            and os.path.getmtime(obj) >= max(os.path.getmtime(src), _headers_mtime())):
        return obj
    cmd = [hipcc(), *HIPCC_FLAGS, *extra, "-c", src, "-o", obj]
    res = subprocess.run(cmd, capture_output=True, text=True)
    noise = "is not a recognized feature for this target"
    err = "\n".join(l for l in res.stderr.splitlines() if noise not in l and l.strip())
    if res.returncode != 0:
        raise RuntimeError(f"hipcc failed for {src}:\n{err}")
    if err:
        sys.stderr.write(err + "\n")
    return obj


def build(force: bool = True, jobs: int = 8, extra_flags: list[str] | None = None) -> str:
    os.makedirs(LIB_DIR, exist_ok=True)
    os.makedirs(OBJ_DIR, exist_ok=True)
    extra = list(extra_flags or [])
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        objs = list(pool.map(lambda s: _compile(s, force, extra), sources()))
    tmp = LIB_PATH + ".tmp"
    cmd = [hipcc(), f"--offload-arch={ARCH}", "-shared", "-fPIC", "-o", tmp, *objs]
    res = subprocess.run(cmd, capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError(f"link failed:\n{res.stderr}")
    os.replace(tmp, LIB_PATH)
    return LIB_PATH


if __name__ == "__main__":
    incremental = "--incremental" in sys.argv
    print(build(force=not incremental))
