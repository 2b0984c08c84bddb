"""The C++ host mirror of the Swift operator surface (leviathan_amd/host).

CPU: the parity program compiles against the in-tree headers and libraries and
lists its cases without touching a device.  GPU: every case passes.
"""
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
BIN = os.path.join(ROOT, "tests", "host", "build", "host_parity")

CASES = ["q4_backend_2x32", "q4_backend_minus_16", "q4_backend_guards", "q6_backend_minus_315",
         "q4_backend_seeded", "runner_matvec", "runner_elementwise", "runner_int8_path", "runner_f32_columns", "runner_shared_expert",
         "runner_moe",
         "runner_moe_hand_computed", "runner_gguf_file", "forge_matvec", "forge_moe_layer"]


def _built():
    if not os.path.exists(BIN):
        import oracle  # noqa: F401  (builds liblev_oracle.so if missing)
        from leviathan_amd import build as hip_build
        hip_build.build()
        subprocess.run(["make", "-C", os.path.join(ROOT, "tests", "host")], check=True,
                       stdout=subprocess.DEVNULL)
    return BIN


def test_host_mirror_compiles_and_lists_cases():
    out = subprocess.run([_built(), "--list"], check=True, capture_output=True, text=True, timeout=60)
    assert out.stdout.split() == CASES


@pytest.mark.gpu
def test_host_mirror_parity_on_gpu():
    out = subprocess.run([_built()], capture_output=True, text=True, timeout=100)
    print(out.stdout)
    print(out.stderr)
    assert out.returncode == 0, out.stdout[-2000:]
    for name in CASES:
        assert f"ok {name}" in out.stdout
