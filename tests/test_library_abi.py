"""CPU-side checks of the C ABI: the library loads, exports every symbol that include/*.h
declare, and rejects bad arguments with the documented codes before touching a GPU.
(No compute call is made here.)"""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADERS = [os.path.join(ROOT, "include", h) for h in ("w4a16.h", "w4a16_probe.h")]


@pytest.fixture(scope="module")
def L():
    from lmdeploy_amd import _lib
    return _lib


def declared_symbols():
    text = "".join(open(h).read() for h in HEADERS)
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(w4a16_[a-z0-9_]+)\s*\(", text)))


def test_header_symbols_are_exported_and_bound(L):
    names = declared_symbols()
    assert len(names) >= 15
    raw = ctypes.CDLL(L.LIB_PATH)
    for n in names:
        assert hasattr(raw, n), "library does not export %s" % n
        assert n in L.SIGNATURES, "python binding lacks %s" % n
    assert set(L.SIGNATURES) == set(names)


def test_version_and_algo_table(L):
    assert L.lib.w4a16_version().decode().startswith("w4a16-gfx950")
    assert L.lib.w4a16_algo_count() >= 10


FAKE = ctypes.c_void_p(0x1000)      # never dereferenced: every call below fails validation first
P = ctypes.c_void_p(0x2000)


def err(L):
    return L.lib.w4a16_last_error().decode()


def test_gemm_argument_validation(L):
    g = L.lib.w4a16_gemm
    assert g(None, P, P, P, P, None, 64, 4, 256, 128, 0, -1, None) == L.EARG and "null handle" in err(L)
    # gemm_s4_f16.cu:119,233: the reference's message for a group size it has no kernels for
    assert g(FAKE, P, P, P, P, None, 64, 4, 256, 256, 0, -1, None) == L.EGROUP and err(L) == "unsupported group size"
    assert g(FAKE, P, P, P, P, None, 64, 4, 256, 128, 7, -1, None) == L.EARG
    assert g(FAKE, P, P, P, P, None, -1, 4, 256, 128, 0, -1, None) == L.EARG
    assert g(FAKE, None, P, P, P, None, 64, 4, 256, 128, 0, -1, None) == L.EARG
    assert g(FAKE, P, P, P, P, None, 64, 4, 256, 128, 2, -1, None) == L.EARG and "residual" in err(L)
    assert g(FAKE, P, ctypes.c_void_p(0x2004), P, P, None, 64, 4, 256, 128, 0, -1, None) == L.EARG   # misaligned A
    # gemm_s4_f16.cu:227: shapes no kernel can run
    assert g(FAKE, P, P, P, P, None, 72, 4, 256, 128, 0, -1, None) == L.ESHAPE and err(L) == "no feasible kernel found"
    assert g(FAKE, P, P, P, P, None, 64, 4, 200, 128, 0, -1, None) == L.ESHAPE
    assert g(FAKE, P, P, P, P, None, 64, 4, 256, 128, 0, 10 ** 6, None) == L.EALGO
    # nothing to do is not an error and touches nothing
    assert g(FAKE, None, None, None, None, None, 64, 0, 256, 128, 0, -1, None) == L.OK


def test_repack_argument_validation(L):
    lib = L.lib
    assert lib.w4a16_convert_s4_k_m8(P, P, P, P, P, P, 64, 256, 16, None) == L.EGROUP
    assert lib.w4a16_convert_s4_k_m8(P, P, P, P, P, P, 24, 256, 128, None) == L.ESHAPE
    assert lib.w4a16_convert_s4_k_m8(P, P, P, P, P, P, 64, 100, 128, None) == L.ESHAPE
    assert lib.w4a16_convert_s4_k_m8(None, P, P, P, P, P, 64, 256, 128, None) == L.EARG
    assert lib.w4a16_convert_s4_k_m8(None, None, None, None, None, None, 0, 256, 128, None) == L.OK   # empty
    assert lib.w4a16_fuse_w1_w3_s4_k_m8(P, P, 12, 4, None) == L.ESHAPE
    assert lib.w4a16_fuse_w1_w3_s4_k_m8(None, P, 16, 4, None) == L.EARG
    assert lib.w4a16_transpose_qk_s4_k_m8_hf(P, P, 64, 4, 0, None) == L.ESHAPE
    assert lib.w4a16_transpose_qk_s4_k_m8_hf(P, P, 64, 4, 48, None) == L.ESHAPE      # 64 % 48 != 0
    assert lib.w4a16_dequantize_s4(None, P, 8, None) == L.EARG
    assert lib.w4a16_dequantize_s4(None, None, 0, None) == L.OK
    assert lib.w4a16_unpack_repacked(P, P, P, P, P, 64, 256, 96, None) == L.EGROUP
    assert lib.w4a16_dequantize_repacked(None, P, P, 64, 256, 128, None) == L.EARG
    assert lib.w4a16_from_reference_layout(P, P, 48, 256, None) == L.ESHAPE          # m % 32
    assert lib.w4a16_reformat_s4_k_m8(P, None, 64, 256, None) == L.EARG


def test_check_raises_with_code(L):
    rc = L.lib.w4a16_gemm(FAKE, P, P, P, P, None, 64, 4, 256, 512, 0, -1, None)
    with pytest.raises(L.W4A16Error, match="unsupported group size") as e:
        L.check(rc)
    assert e.value.code == L.EGROUP


def test_product_does_not_import_the_oracle():
    pkg = os.path.join(ROOT, "lmdeploy_amd")
    for dirpath, _, files in os.walk(pkg):
        for f in files:
            if f.endswith((".py", ".hip", ".cpp", ".h")):
                text = open(os.path.join(dirpath, f)).read()
                assert "oracle" not in text, "%s mentions the oracle" % f


def test_build_module_imports_without_the_library():
    """`python -m lmdeploy_amd.build` must work in a fresh checkout: importing the package or its build
    module must not need (or load) the shared library."""
    import subprocess
    import sys
    code = ("import sys, lmdeploy_amd, lmdeploy_amd.build; "
            "assert 'lmdeploy_amd._lib' not in sys.modules and 'lmdeploy_amd.turbomind' not in sys.modules")
    root = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
    r = subprocess.run([sys.executable, "-c", code], cwd=root, capture_output=True, text=True)
    assert r.returncode == 0, r.stderr


def test_static_and_sequence_argument_validation(L):
    lib = L.lib
    # w4a16_gemm_static: the checks of w4a16_gemm, without a handle
    s = lib.w4a16_gemm_static
    assert s(P, P, P, P, None, 64, 4, 256, 256, 0, -1, None) == L.EGROUP and err(L) == "unsupported group size"
    assert s(P, P, P, P, None, 72, 4, 256, 128, 0, -1, None) == L.ESHAPE
    assert s(None, P, P, P, None, 64, 4, 256, 128, 0, -1, None) == L.EARG
    assert s(P, P, P, P, None, 64, 4, 256, 128, 2, -1, None) == L.EARG and "residual" in err(L)
    assert s(P, P, P, P, None, 64, 4, 256, 128, 0, 10 ** 6, None) == L.EALGO
    assert s(None, None, None, None, None, 64, 0, 256, 128, 0, -1, None) == L.OK
    # w4a16_gemm_sequence: every descriptor is validated before anything is launched
    seq = lib.w4a16_gemm_sequence
    one = (L.GemmDesc * 2)()
    for d in one:
        d.C, d.A, d.X, d.Q, d.R, d.n_out, d.k, d.epilogue, d.depends = 0x2000, 0x2000, 0x2000, 0x2000, None, 64, 256, 0, 1
    assert seq(None, one, 2, 4, 128, 0, None) == L.EARG and "null handle" in err(L)
    assert seq(FAKE, None, 2, 4, 128, 0, None) == L.EARG
    assert seq(FAKE, one, 2, 4, 128, 8, None) == L.EARG and "flags" in err(L)
    assert seq(FAKE, one, 2, 4, 48, 0, None) == L.EGROUP
    one[1].n_out = 72
    assert seq(FAKE, one, 2, 4, 128, L.SEQ_PERSISTENT, None) == L.ESHAPE
    one[1].n_out, one[1].epilogue = 64, 2
    assert seq(FAKE, one, 2, 4, 128, 0, None) == L.EARG and "residual" in err(L)
    assert seq(FAKE, one, 0, 4, 128, 0, None) == L.OK            # empty list
    one[1].epilogue = 0
    assert seq(FAKE, one, 2, 0, 128, L.SEQ_PERSISTENT, None) == L.OK   # no tokens
    assert lib.w4a16_set_barrier_timeout(None, 1.0) == L.EARG
    assert lib.w4a16_sequence_status(None, None) == L.EARG
    assert lib.w4a16_save_tuning(None, b"/tmp/x") == L.EARG and lib.w4a16_load_tuning(None, b"/tmp/x") == L.EARG
    assert lib.w4a16_save_tuning(FAKE, None) == L.EARG and lib.w4a16_load_tuning(FAKE, None) == L.EARG
    assert lib.w4a16_load_tuning(FAKE, b"/nonexistent/dir/tuning.txt") == L.EARG and "cannot open" in err(L)
    assert lib.w4a16_probe_read(None, P, 1024, None) == L.EARG
    assert lib.w4a16_probe_barrier(None, 10, 1, None) == L.EARG
    assert lib.w4a16_probe_stream(None, P, 1024, 1, 4, 1, None) == L.EARG
    assert lib.w4a16_probe_stream(FAKE, P, 1024, 3, 4, 1, None) == L.EARG and "wg_per_cu" in err(L)
    assert lib.w4a16_probe_mfma(None, 8, 10, None) == L.EARG
    assert lib.w4a16_probe_mfma(FAKE, 3, 10, None) == L.EARG and "waves_per_cu" in err(L)
    assert lib.w4a16_probe_mfma(FAKE, 8, 0, None) == L.EARG and "iters" in err(L)
    assert lib.w4a16_probe_clock_begin(None, None) == L.EARG
    assert lib.w4a16_probe_clock_end(None, None, None, None, None, None) == L.EARG
    assert lib.w4a16_probe_clock_end(FAKE, None, None, None, None, None) == L.EARG and "null output" in err(L)


def test_deploy_entry_point_validation(L):
    lib = L.lib
    three = (ctypes.c_void_p * 3)(0x2000, 0x2000, 0x2000)
    q = lib.w4a16_deploy_qkv
    assert q(P, P, three, three, three, 256, 256, 256, 128, 16, None) == L.EGROUP
    assert q(P, P, three, three, three, 256, 256, 256, 96, 128, None) == L.ESHAPE      # 256 % 96
    assert q(P, P, three, three, three, 256, 256, 200, 128, 128, None) == L.ESHAPE     # k % 128
    assert q(None, P, three, three, three, 256, 256, 256, 128, 128, None) == L.EARG
    assert q(P, P, (ctypes.c_void_p * 3)(0x2000, None, 0x2000), three, three, 256, 256, 256, 128, 128, None) == L.EARG
    assert q(None, None, None, None, None, 0, 0, 256, 128, 128, None) == L.OK          # empty
    w = lib.w4a16_deploy_w13
    assert w(P, P, P, P, P, P, P, P, 64, 256, 256, None) == L.EGROUP
    assert w(P, P, P, P, P, P, P, P, 60, 256, 128, None) == L.ESHAPE                   # inter_size % 8
    assert w(P, P, P, None, P, P, P, P, 64, 256, 128, None) == L.EARG
