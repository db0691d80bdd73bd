"""The C-ABI library loads and exports every symbol include/br_hip.h declares,
and the Python binding table covers exactly that set.  No GPU needed: nothing
here launches a kernel or touches device memory."""
import ctypes
import os
import re

from conftest import ROOT

from blackriver_amd import hip


def declared_symbols(header):
    text = open(os.path.join(ROOT, "include", header)).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(br_[a-z0-9_]+)\s*\(", text)))


def test_kernel_library_exports_every_declared_symbol():
    names = declared_symbols("br_hip.h")
    assert len(names) > 30
    assert os.path.exists(hip.LIB_PATH), "build with `python -m blackriver_amd.build`"
    lib = ctypes.CDLL(hip.LIB_PATH)
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, missing


def test_python_binding_table_matches_header():
    assert sorted(hip.SIGNATURES) == declared_symbols("br_hip.h")
    hip.load()


def test_error_strings_and_host_helpers_without_gpu():
    lib = hip.load()
    assert lib.br_hip_error_string(0) == b"ok"
    assert b"input" in lib.br_hip_error_string(-2)
    slopes = (ctypes.c_double * 32)()
    assert lib.br_hip_alibi_slopes(slopes, 32) == 0
    assert abs(slopes[0] - 2.0 ** -0.25) < 1e-15 and abs(slopes[31] - 2.0 ** -8) < 1e-15
    assert lib.br_hip_alibi_slopes(slopes, 0) == -4
    # argument validation happens before any HIP call
    assert lib.br_hip_gemm(0, 0, 4, 4, 4, 1.0, None, 0, 4, 0, None, 0, 4, 0, 0, None, 0, 4, 0, None, 1, 0, None) == -2
    assert lib.br_hip_layernorm_bwd_workspace(2048, 4096) >= 2 * 4096 * 4
