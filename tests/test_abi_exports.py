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


def test_double_entry_points_without_a_kernel():
    # the double base type has its own kernel table (dllmain.cpp:6-14): index 1 of it is empty in a fresh process, and the
    # call says so without touching a device; the string-carrying twin (extensions, blob loaders) is not built for it
    lib = C.load_library()
    err = (ctypes.c_uint16 * 256)()
    assert lib.DLL_InvokeDouble(1, 20, None, 0, None, None, err, 256) == C.ERROR.PARAM_NULL
    assert lib.DLL_InvokeDoubleEx2(1, 20, None, 0, None, 0, None, None, err, 256) == C.ERROR.PARAM_NULL
    assert lib.DLL_InvokeDouble(5000, 20, None, 0, None, None, err, 256) == C.ERROR.PARAM_OUT_OF_RANGE
    lib.DLL_InvokeDoubleEx.restype = ctypes.c_int32
    assert lib.DLL_InvokeDoubleEx(1, 67, None, 0, None, None, None, err, 256) == C.ERROR.NOT_IMPLEMENTED
    assert "double" in C._from_utf16(err)


def test_extension_double_twins_report_not_implemented():
    # CudaExtension.llm32.11.8.def:8-11 lists the double twins; they exist and refuse
    if not os.path.exists(C.llama2_extension_path()):
        pytest.skip("extension library not built")
    ext = ctypes.CDLL(C.llama2_extension_path())
    err = (ctypes.c_uint16 * 256)()
    assert ext.DLL_InitDoubleCustomExtension(None, 1) == C.ERROR.NOT_IMPLEMENTED
    assert ext.DLL_InvokeDoubleCustomExtension(1, None, 0, None, None, err, 256) == C.ERROR.NOT_IMPLEMENTED
    assert "double" in C._from_utf16(err)
    assert ext.DLL_InvokeDoubleCustomExtensionEx(5, None, 0, None, None, None, None, 0, err, 256) == C.ERROR.NOT_IMPLEMENTED


def _def_exports(name):
    text = open(os.path.join(ROOT, "mycaffe_amd", "csrc", name)).read()
    body = text.split("EXPORTS", 1)[1]
    return [l.split()[0] for l in body.splitlines() if l.strip() and not l.strip().startswith(";")]


def test_def_files_list_what_the_libraries_export():
    # the Windows export lists name exactly the header's entry points, library by library
    decl = set(_declared_symbols())
    main, ext = _def_exports("mycaffe_hip.def"), _def_exports("mycaffe_hip_llama2.def")
    assert set(main) == decl - set(C.EXTENSION_EXPORTS)
    assert set(ext) == set(C.EXTENSION_EXPORTS)
    assert set(C.EXPORTS) == set(main)


def test_no_alloc_entry_rejects_bad_kernel_before_touching_a_device():
    lib = C.load_library()
    err = (ctypes.c_uint16 * 256)()
    l = np.zeros(12, np.int64)
    f = np.zeros(1, np.float32)
    fp, lp = f.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), l.ctypes.data_as(ctypes.POINTER(ctypes.c_int64))
    assert lib.MCH_AttnDecodeForwardNoAlloc(77, fp, 1, lp, 12, err, 256) == C.ERROR.PARAM_NULL
    assert lib.MCH_AttnDecodeForwardNoAlloc(5000, fp, 1, lp, 12, err, 256) == C.ERROR.PARAM_OUT_OF_RANGE


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


def test_call_trace_names_the_function(tmp_path):
    # MYCAFFE_HIP_TRACE=<file>: one line per dispatched call in the reference's _TRACEAPI wording (main.cu:44-55);
    # the variable is read once per process, so the traced calls run in a child process (no device needed: the
    # call fails on an uninitialised kernel and is traced all the same)
    import subprocess
    import sys
    log = tmp_path / "trace.txt"
    code = (
        "import ctypes, numpy as np\n"
        "from mycaffe_amd import cudadnn as C\n"
        "lib = C.load_library()\n"
        "err = (ctypes.c_uint16 * 256)()\n"
        "out = (ctypes.c_float * 4)()\n"
        "pout = ctypes.cast(out, ctypes.POINTER(ctypes.c_float))\n"
        "n = ctypes.c_int32(4)\n"
        "l = np.zeros(10, np.int64)\n"
        "f = np.zeros(2, np.float32)\n"
        "rc = lib.DLL_InvokeFloatEx2(77, 220, f.ctypes.data_as(ctypes.POINTER(ctypes.c_float)), 2,\n"
        "                            l.ctypes.data_as(ctypes.POINTER(ctypes.c_int64)), 10, ctypes.byref(pout), ctypes.byref(n), err, 256)\n"
        "assert rc == C.ERROR.PARAM_NULL, rc\n"
    )
    env = dict(os.environ, MYCAFFE_HIP_TRACE=str(log), PYTHONPATH=ROOT)
    subprocess.run([sys.executable, "-c", code], check=True, env=env, cwd=ROOT)
    text = log.read_text()
    assert "FLOAT calling CudaDnnDLL FunctionID (220) CUDA_FN_GEMM kernel 77 floats 2 longs 10 -> 90002" in text
