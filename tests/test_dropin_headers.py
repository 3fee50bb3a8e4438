"""The C++ front-end headers (include/turbomind/*.h) compile and link against the library in a
LlamaLinear-shaped caller (tests/cpp/llama_linear_dropin.cpp).  On a GPU box the program also runs
one GEMM through the class."""
import shutil
import subprocess

import pytest


def test_llama_linear_shaped_caller_builds_and_runs():
    if not (shutil.which("hipcc") or shutil.os.path.exists("/opt/rocm/bin/hipcc")):
        pytest.skip("hipcc not available")
    from lmdeploy_amd.build import check_headers
    exe = check_headers(verbose=False)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "drop-in GEMM ran, non-zero outputs: 0" in r.stdout or "no GPU work done" in r.stdout
