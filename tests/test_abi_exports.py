"""CPU-side checks of the C-ABI boundary: the built libraries load, export every
symbol the header declares, and reject bad calls with the reference's codes
before touching a device."""
import ctypes
import os
import re

import numpy as np
import pytest

from mycaffe_amd import cudadnn as C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "mycaffe_hip_abi.h")).read()
    return sorted(set(re.findall(r"^MCH_LONG\s+(\w+)\(", text, flags=re.M)))


def test_header_declares_reference_exports():
    decl = _declared_symbols()
    for name in C.EXPORTS + C.EXTENSION_EXPORTS:
        assert name in decl, name


def test_library_exports_every_declared_symbol():
    lib = C.load_library()
    ext = ctypes.CDLL(C.llama2_extension_path()) if os.path.exists(C.llama2_extension_path()) else None
    for name in _declared_symbols():
        owner = ext if name in C.EXTENSION_EXPORTS else lib
        if owner is None:
            pytest.skip("extension library not built")
        assert hasattr(owner, name), name


def test_double_entry_points_report_not_implemented():
    lib = C.load_library()
    err = (ctypes.c_uint16 * 256)()
    rc = lib.DLL_InvokeDouble(1, 20, None, 0, None, None, err, 256)
    assert rc == C.ERROR.NOT_IMPLEMENTED
    assert "double" in C._from_utf16(err)


def test_uninitialised_kernel_and_bad_index_codes():
    # CudaDnnDLL.cpp:296-301: a null table slot gives ERROR_PARAM_NULL; indices outside the table ERROR_PARAM_OUT_OF_RANGE
    lib = C.load_library()
    err = (ctypes.c_uint16 * 256)()
    out = (ctypes.c_float * 4)()
    pout = ctypes.cast(out, ctypes.POINTER(ctypes.c_float))
    n = ctypes.c_int32(4)
    l = np.array([16], np.int64)
    rc = lib.DLL_InvokeFloatEx2(77, 20, None, 0, l.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), 1, ctypes.byref(pout), ctypes.byref(n), err, 256)
    assert rc == C.ERROR.PARAM_NULL
    rc = lib.DLL_InvokeFloatEx2(5000, 20, None, 0, l.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), 1, ctypes.byref(pout), ctypes.byref(n), err, 256)
    assert rc == C.ERROR.PARAM_OUT_OF_RANGE
    rc = lib.DLL_InvokeFloatEx2(-1, 20, None, 0, None, 0, ctypes.byref(pout), ctypes.byref(n), err, 256)
    assert rc == C.ERROR.PARAM_OUT_OF_RANGE


def test_utf16_round_trip_helpers():
    buf = C._utf16("model.bin;tokenizer.bin é中")
    assert C._from_utf16(buf) == "model.bin;tokenizer.bin é中"
