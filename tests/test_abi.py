"""The C ABI library loads and exports exactly what include/kmx.h declares (no GPU needed, no compute calls)."""
import ctypes
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def declared_symbols():
    text = open(os.path.join(ROOT, "include", "kmx.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(kmx_[a-z0-9_]+)\s*\(", text)))


def test_header_and_binding_list_agree(km):
    assert declared_symbols() == sorted(km.ABI_SYMBOLS)


def test_library_exports_every_declared_symbol(km):
    assert os.path.exists(km.HIP_LIB_PATH), "libkmx_hip.so must be built in-tree"
    lib = ctypes.CDLL(km.HIP_LIB_PATH)
    for name in declared_symbols():
        assert hasattr(lib, name), name


def test_header_compiles_as_c_and_cpp(tmp_path):
    import subprocess
    src = tmp_path / "t.c"
    src.write_text('#include "kmx.h"\nint main(void){ kmx_exec_params e = {256,0,0,1,1,1}; return (int)e.block_count + (int)sizeof(kmx_props) * 0; }\n')
    inc = os.path.join(ROOT, "include")
    subprocess.check_call(["gcc", "-std=c99", "-Wall", "-Werror", "-pedantic", "-I", inc, "-c", str(src), "-o", str(tmp_path / "t.o")])
    subprocess.check_call(["g++", "-std=c++14", "-Wall", "-Werror", "-I", inc, "-x", "c++", "-c", str(src), "-o", str(tmp_path / "t2.o")])


def test_exec_params_layout_matches_header(km):
    assert ctypes.sizeof(km.ExecParams) == 24
    assert [f[0] for f in km.ExecParams._fields_] == ["block_size", "block_count", "shared_mem_bytes",
                                                      "privatized_copies", "items_per_thread", "regs_cache"]


def test_argument_errors_need_no_gpu(km):
    lib = km.hip_lib()
    ex = km.ExecParams()
    # argument validation happens before any device work
    assert lib.kmx_assign_f32(km.ASSIGN_BEST, None, 0, 4, None, 0, 4, None, None, 0, 3, 10, ctypes.byref(ex)) == km.KMX_ERR_INVALID_ARGUMENT
    assert b"dim and k" in lib.kmx_last_error()
    assert lib.kmx_assign_f32(km.ASSIGN_BEST, None, 0, 4, None, 0, 4, None, None, 4, 3, 10, None) == km.KMX_ERR_INVALID_ARGUMENT
    assert lib.kmx_update_f32(7, None, 0, 4, None, None, 0, 4, None, 4, 3, 0, ctypes.byref(ex)) == km.KMX_ERR_INVALID_ARGUMENT
    assert lib.kmx_fill_zero_u32(None, 0) == km.KMX_OK
    assert lib.kmx_last_error() == b""


def test_no_device_is_reported_not_faked(km):
    if km.device_count() > 0:
        pytest.skip("a GPU is visible here")
    rc = km.hip_lib().kmx_set_device(0)
    assert rc == km.KMX_ERR_NO_DEVICE and b"No HIP devices" in km.hip_lib().kmx_last_error()
    alg = km.HipKMeansAlgorithm()
    import numpy as np
    with pytest.raises(km.KmxError):
        alg.initialize(2, 2, 4, 1, np.zeros(8, np.float32), np.zeros(4, np.float32))
