"""Builds libw4a16.so (HIP kernels for gfx950 + the C ABI) in-tree with hipcc.

Usage: python -m lmdeploy_amd.build            (or build_library() from Python)
"""
from __future__ import annotations

import os
import re
import shutil
import subprocess
import sys
from concurrent.futures import ThreadPoolExecutor

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libw4a16.so")

SOURCES = ["api.cpp", "repack.hip", "static_scratch.hip", "probe.hip", "gemm_decode.hip", "gemm_strip.hip", "gemm_sequence.hip", "gemm_prefill.hip"]

# -packed-fp32-ops off: hipcc must not form v_pk_*_f32 instructions for this target.
HIP_FLAGS = ["--offload-arch=gfx950", "-O3", "-std=c++17", "-fPIC", "-Wall", "-Wno-unused-function",
             "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops"]


def _hipcc() -> str:
    exe = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
    if not os.path.exists(exe):
        raise RuntimeError("hipcc not found; ROCm is required to build libw4a16.so")
    return exe


# The GEMM kernels wait for their software-pipelined loads by count.  A register spill would put
# scratch stores among those loads, and stores complete out of order with loads, so a spilling
# GEMM kernel is a wrong kernel: the build refuses it.
NO_SCRATCH = ("gemm_decode.hip", "gemm_strip.hip", "gemm_sequence.hip", "gemm_prefill.hip")


def _check_no_scratch(src: str, remarks: str) -> None:
    """The GEMM kernels issue loads from inline assembly and wait for them by count, so the compiler
    does not know when a destination register is valid.  A kernel is only safe if the compiler never
    moves such a register: no spills to scratch, and no VGPRs parked in AGPRs (the only legitimate
    AGPRs are the 4 * TTILES * NTW accumulators of a prefill kernel)."""
    name = None
    for line in remarks.splitlines():
        if "Function Name:" in line:
            name = line.split("Function Name:")[1].split("[")[0].strip()
        elif "ScratchSize [bytes/lane]:" in line:
            size = int(line.split("ScratchSize [bytes/lane]:")[1].split("[")[0])
            if size != 0:
                raise RuntimeError("%s: kernel %s spills %d bytes/lane to scratch" % (src, name, size))
        elif "AGPRs:" in line and name is not None and "_kernel" in name:
            agprs = int(line.split("AGPRs:")[1].split("[")[0])
            m = re.search(r"prefill_kernelILi(\d+)ELi(\d+)E", name)
            allowed = 4 * int(m.group(1)) * int(m.group(2)) if m else 0
            if agprs != allowed:
                raise RuntimeError("%s: kernel %s uses %d AGPRs, expected %d: the register allocator is "
                                   "parking VGPRs in AGPRs" % (src, name, agprs, allowed))


def _check_inflight(src: str, obj_dir: str) -> None:
    """Second pass over the same source to assembly text, checked by asm_lint: no compiler-generated
    instruction may touch a register whose inline-assembly load can still be in flight."""
    try:
        from .asm_lint import lint
    except ImportError:  # run as a script
        from asm_lint import lint
    asm = os.path.join(obj_dir, os.path.splitext(src)[0] + ".s")
    cmd = [_hipcc(), *HIP_FLAGS, "-S", "--cuda-device-only", os.path.join(CSRC, src), "-o", asm]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc -S failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    with open(asm) as f:
        problems = lint(f.read())
    os.remove(asm)
    if problems:
        raise RuntimeError("%s: %d uses of registers with a load in flight, e.g.\n%s"
                           % (src, len(problems), "\n".join(problems[:5])))


def _compile(src: str, obj_dir: str) -> str:
    obj = os.path.join(obj_dir, os.path.splitext(src)[0] + ".o")
    cmd = [_hipcc(), *HIP_FLAGS]
    if src.endswith(".cpp"):
        cmd += ["-x", "hip"]
    if src in NO_SCRATCH:
        cmd += ["-Rpass-analysis=kernel-resource-usage"]
    cmd += ["-c", os.path.join(CSRC, src), "-o", obj]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("hipcc failed for %s:\n%s\n%s" % (src, r.stdout, r.stderr))
    if src in NO_SCRATCH:
        _check_no_scratch(src, r.stderr)
        _check_inflight(src, obj_dir)
    return obj


def build_library(verbose: bool = True) -> str:
    """Compiles every source and links the shared library; always rebuilds."""
    obj_dir = os.path.join(HERE, "build")
    os.makedirs(obj_dir, exist_ok=True)
    os.makedirs(LIB_DIR, exist_ok=True)
    with ThreadPoolExecutor(max_workers=min(8, len(SOURCES))) as ex:
        objs = list(ex.map(lambda s: _compile(s, obj_dir), SOURCES))
    tmp = LIB_PATH + ".tmp"
    cmd = [_hipcc(), "--offload-arch=gfx950", "-shared", "-fPIC", "-o", tmp, *objs]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("link failed:\n%s\n%s" % (r.stdout, r.stderr))
    os.replace(tmp, LIB_PATH)
    if verbose:
        print("built", LIB_PATH, os.path.getsize(LIB_PATH), "bytes")
    return LIB_PATH


def check_headers(verbose: bool = True) -> str:
    """Compiles and links tests/cpp/llama_linear_dropin.cpp against the C++ front-end headers and
    the library: the proof that a LlamaLinear-shaped caller builds against them."""
    root = os.path.dirname(HERE)
    src = os.path.join(root, "tests", "cpp", "llama_linear_dropin.cpp")
    out = os.path.join(HERE, "build", "llama_linear_dropin")
    os.makedirs(os.path.dirname(out), exist_ok=True)
    cmd = [_hipcc(), "-x", "hip", "--offload-arch=gfx950", "-std=c++17", "-O1", "-Wall",
           "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
           "-I", os.path.join(root, "include"), src, "-o", out, "-L", LIB_DIR, "-lw4a16",
           "-Wl,-rpath,$ORIGIN/../lib"]
    r = subprocess.run(cmd, capture_output=True, text=True)
    if r.returncode != 0:
        raise RuntimeError("drop-in header check failed:\n%s\n%s" % (r.stdout, r.stderr))
    if verbose:
        print("built", out)
    return out


if __name__ == "__main__":
    build_library()
    check_headers()
    sys.exit(0)
