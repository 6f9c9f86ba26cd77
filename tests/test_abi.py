"""The C-ABI library loads on a machine without a GPU and exports what include/sharpnet_hip.h declares."""
import os
import re

import pytest

from tests.conftest import ROOT


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "sharpnet_hip.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\bint\s+(snhip_\w+)\s*\(", text)))


def test_header_declares_the_reference_shaped_entry_points():
    syms = declared_symbols()
    for required in ("snhip_create", "snhip_destroy", "snhip_sgemm", "snhip_sgemm_strided_batched", "snhip_dot",
                     "snhip_dot_bias", "snhip_bmm"):
        assert required in syms


def test_library_exports_every_declared_symbol():
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    for name in declared_symbols():
        assert hasattr(lib, name), name + " is declared in the header but not exported"
    # and the ctypes prototype table covers the whole header
    assert sorted(hiplib.SIGNATURES) == declared_symbols()


def test_no_compute_symbols_from_vendor_blas():
    # the library must not link a vendor GEMM (hipBLAS / rocBLAS / hipBLASLt)
    import subprocess
    from sharpnet_amd import hiplib
    out = subprocess.run(["ldd", hiplib.library_path()], stdout=subprocess.PIPE, text=True).stdout.lower()
    for banned in ("hipblas", "rocblas", "libcublas", "miopen"):
        assert banned not in out


def test_status_codes_match_cublas_numbering():
    from sharpnet_amd.hiplib import CublasStatus
    text = open(os.path.join(ROOT, "include", "sharpnet_hip.h")).read()
    for name, val in re.findall(r"#define SNHIP_STATUS_(\w+) (\d+)", text):
        assert CublasStatus["CUBLAS_STATUS_" + name].value == int(val)


def test_argument_errors_without_gpu():
    """Calls that are rejected before any device work return the cuBLAS-numbered status."""
    import ctypes
    from sharpnet_amd import hiplib
    lib = hiplib.load_library()
    one = ctypes.c_float(1.0)
    # NULL handle -> NOT_INITIALIZED (1), like cuBLAS
    assert lib.snhip_sgemm(None, 0, 0, 1, 1, 1, ctypes.byref(one), None, 1, None, 1, ctypes.byref(one), None, 1) == 1
    assert lib.snhip_dot(None, None, 1, 1, 0, None, 1, 1, 0, None, 1.0, 0.0) == 1
    assert lib.snhip_destroy(None) == 1
    assert lib.snhip_create(None) == 7
    assert lib.snhip_config_count() >= 4
    d = (ctypes.c_int * 6)()
    assert lib.snhip_config_desc(0, d) == 0 and d[0] > 0 and d[1] > 0
    assert lib.snhip_config_desc(999, d) == 7


def test_missing_library_fails_loudly(tmp_path, monkeypatch):
    from sharpnet_amd import hiplib
    with pytest.raises(FileNotFoundError):
        hiplib.load_library(str(tmp_path / "libsharpnet_hip.so"))
