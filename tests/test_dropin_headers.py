"""The C++ front-end headers (include/turbomind/*.h) in a LlamaLinear-shaped caller
(tests/cpp/llama_linear_dropin.cpp) linked against the library and the system HIP runtime.
Without a GPU the program builds, links and reports that it did no GPU work; on a GPU box it
runs the three epilogues through `turbomind::GemmS4F16` on a case with a known closed-form answer."""
import os
import shutil
import subprocess

import pytest


def _exe():
    """The program as `__graft_entry__.build()` left it; built here only if it is missing."""
    from lmdeploy_amd import build
    exe = os.path.join(build.HERE, "build", "llama_linear_dropin")
    if os.path.exists(exe):
        return exe
    if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
        pytest.skip("hipcc not available")
    return build.check_headers(verbose=False)


def test_llama_linear_shaped_caller_builds_and_links():
    if not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")):
        pytest.skip("hipcc not available")
    from lmdeploy_amd.build import check_headers
    exe = check_headers(verbose=False)
    r = subprocess.run([exe], capture_output=True, text=True, timeout=120)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "drop-in checks passed" in r.stdout or "no GPU work done" in r.stdout


@pytest.mark.gpu
def test_llama_linear_shaped_caller_computes_the_known_answers():
    r = subprocess.run([_exe()], capture_output=True, text=True, timeout=120)
    print(r.stdout, r.stderr)
    assert r.returncode == 0, r.stdout + r.stderr
    assert "no GPU work done" not in r.stdout
    assert r.stdout.count("drop-in GEMM ran") == 2
    for T in (4, 100):
        assert ("drop-in GEMM ran, tokens %d: kGemm mismatches 0, kFusedSiluFfn mismatches 0 (+0 written past the output), "
                "kFusedAdd mismatches 0" % T) in r.stdout
    assert 'group size 256: "unsupported group size" ok' in r.stdout
    assert "tuning file: saved 1, loaded 1: ok" in r.stdout
    assert "drop-in checks passed" in r.stdout
