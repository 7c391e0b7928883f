"""Host-side mirror of MyCaffe's ``CudaDnn<float>`` for the attention hot path.

The reference host is C# (MyCaffe/common/CudaDnn.cs); no .NET toolchain exists in
this image, so the same wrappers are written in Python over ctypes.  Method names,
argument order and the packing of arguments into the float / long arrays follow
CudaDnn.cs (cited per method), so a call here reaches ``DLL_InvokeFloat`` /
``DLL_InvokeFloatEx2`` / ``DLL_InvokeFloatEx`` exactly as the C# host's call would
through CudaControl.  Errors come back as return codes plus a UTF-16 message and
are raised as :class:`CudaDnnError`, like the .NET exception CudaControl throws.

There is no CPU fallback: constructing :class:`CudaDnn` loads the HIP library and
fails loudly when it is missing.
"""
import ctypes
import os

import numpy as np

from . import build as _build

_HERE = os.path.dirname(os.path.abspath(__file__))


class CudaDnnError(RuntimeError):
    def __init__(self, code, message):
        super().__init__("%s [error %d]" % (message, code))
        self.code = code


class CUDAFN:
    """Function ids (CudaDnn.cs:1167-1664, CudaDnnDLL/inc/FunctionIDs.h:71-551)."""
    INITIALIZE = -2
    CLEANUP = -3
    FREEMEM_HOST = -1
    SETDEVICE = 1
    GETDEVICE = 3
    SYNCHRONIZEDEVICE = 5
    CREATE_MEMORYPOINTER = 16
    FREE_MEMORYPOINTER = 17
    ALLOCMEM_HALF = 19
    ALLOCMEM = 20
    FREEMEM = 21
    GETMEM = 22
    SETMEM = 23
    CREATE_CUDNN = 47
    FREE_CUDNN = 48
    CREATE_TENSORDESC = 50
    FREE_TENSORDESC = 51
    SET_TENSORDESC = 52
    CREATE_EXTENSION = 67
    FREE_EXTENSION = 68
    EXTENSION_RUN = 69
    SOFTMAX_FWD = 111
    SOFTMAX_BWD = 112
    CUDA_ATTN_CREATE = 160
    CUDA_ATTN_FREE = 161
    CUDA_ATTN_SET = 162
    CUDA_ATTN_FWD = 163
    CUDA_ATTN_BWD = 164
    CUDA_SET = 200
    CUDA_COPY = 202
    CUDA_GEMM2 = 219
    CUDA_GEMM = 220
    CUDA_GEMV = 221
    CUDA_AXPY = 222
    CUDA_SCAL = 224
    CUDA_SCALE = 227
    CUDA_ADD_SCALAR = 228
    CUDA_ADD = 229
    CUDA_SUB = 230
    CUDA_MUL = 231
    CUDA_DIV = 233
    CUDA_EXP = 235
    CUDA_LOG = 236
    CUDA_POWX = 237
    CUDA_SQRT = 239
    CUDA_TRANSPOSE = 261
    CUDA_MASK = 264
    CUDA_MASK_BATCH = 266
    CUDA_TRANSPOSE_HW = 267
    CUDA_INVERT = 273
    CUDA_CHANNEL_MEAN = 287
    CUDA_CHANNEL_MAX = 290
    CUDA_CHANNEL_SUB = 291
    CUDA_CHANNEL_SUM = 292
    CUDA_CHANNEL_DIV = 293
    CUDA_CHANNEL_DOT = 294
    CUDA_CHANNEL_COPY = 300
    CUDA_CHANNEL_FILLFROM = 301
    CUDA_CHANNEL_COPYALL = 302
    CUDA_CHANNEL_DUP = 303
    CUDA_CHANNEL_SUM2 = 309
    CUDA_EMBED_FWD = 390
    CUDA_RELU_FWD = 428
    CUDA_RELU_BWD = 429
    CUDA_GELU_FWD = 600
    CUDA_GELU_BWD = 601
    CUDA_SILU_FWD = 605
    CUDA_SILU_BWD = 606
    CUDA_CREATE_LAYERNORM = 970
    CUDA_FREE_LAYERNORM = 971
    CUDA_LAYERNORM_FWD = 975
    CUDA_LAYERNORM_BWD = 976
    CUDA_CREATE_ROPE = 980
    CUDA_FREE_ROPE = 981
    CUDA_ROPE_FWD = 982
    CUDA_ROPE_BWD = 983
    CUDA_CREATE_BLOBLOADER = 990
    CUDA_FREE_BLOBLOADER = 991
    CUDA_BLOBLOADER_LOAD = 992
    CUDA_BLOBLOADER_RESETOFFSET = 993
    CUDA_BLOBLOADER_ADDTOOFFSET = 994
    # additions of this library (no counterpart in the reference)
    ATTN_DECODE_FWD = 2001
    RMSNORM_FWD = 2002
    SWIGLU_FWD = 2003
    QKV_PROJ_HEADS = 2004
    LINEAR_FWD = 2005


class CUDAQRY:
    DEVICE_NAME = 1000
    EXTENSION_STRING = 1003


class DEVINIT:
    NONE = 0
    CUBLAS = 1
    CURAND = 2
    SETSEED = 4
    RESETDEVICE = 8


class DIR:
    FWD = 0
    BWD = 1


class SOFTMAX_ALGORITHM:
    FAST = 0
    ACCURATE = 1
    LOG = 2


class SOFTMAX_MODE:
    INSTANCE = 0
    CHANNEL = 1


class ERROR:
    PARAM_OUT_OF_RANGE = 90001
    PARAM_NULL = 90002
    NOT_IMPLEMENTED = 90009
    MEMORY_RANGE_EXCEEDED = 90010
    MEMORY_MIXED_HALF_TYPES = 90011
    MEMORY_HALF_TYPE_NOT_SUPPORTED = 90012
    MEMORY_NOT_FOUND = 90014
    LAYERNORM_NOT_INITIALIZED = 90161
    ROPE_NOT_INITIALIZED = 90201
    ATTN_NOT_INITIALIZED = 90281
    ATTN_INCOMPATIBLE_BLOB_SIZE = 90284
    ATTN_INVALID_BLOCK_SIZE = 90285
    BLOBLOADER_NOT_INITIALIZED = 90321
    EXTENSION_NOT_INITIALIZED = 90401
    FILE_NOT_FOUND = 2              # Win32 codes the reference's blob loader returns unchanged
    INVALID_PARAMETER = 87
    INSUFFICIENT_BUFFER = 122


_c_float_p = ctypes.POINTER(ctypes.c_float)
_c_double_p = ctypes.POINTER(ctypes.c_double)
_c_long = ctypes.c_int32
_c_longlong_p = ctypes.POINTER(ctypes.c_int64)
_c_tchar_p = ctypes.POINTER(ctypes.c_uint16)
_ERRMAX = 1024

EXPORTS = (
    "DLL_InvokeFloat", "DLL_InvokeDouble", "DLL_QueryString", "DLL_InvokeFloatEx", "DLL_InvokeDoubleEx",
    "DLL_InvokeFloatEx2", "DLL_InvokeDoubleEx2", "Internal_GetPointerFloat", "Internal_GetPointerDouble",
    "Internal_AllocHostFloat", "Internal_AllocHostDouble", "DLL_QueryStringFloatEx", "DLL_QueryStringDoubleEx",
    "MCH_TimeInvokeFloatEx2", "MCH_AttnDecodeForwardNoAlloc", "MCH_TimeInvokeFloatEx2Sets",
)
EXTENSION_EXPORTS = (
    "DLL_InitFloatCustomExtension", "DLL_InvokeFloatCustomExtension", "DLL_InvokeFloatCustomExtensionEx",
    "DLL_InitDoubleCustomExtension", "DLL_InvokeDoubleCustomExtension", "DLL_InvokeDoubleCustomExtensionEx",
)


def default_library_path():
    return os.path.join(_HERE, "libmycaffe_hip.so")


def llama2_extension_path():
    return os.path.join(_HERE, "libmycaffe_hip_llama2.so")


def load_library(path=None):
    """dlopen the HIP library (building it first only when no built file exists)."""
    path = path or default_library_path()
    if not os.path.exists(path):
        _build.build(verbose=False)
    if not os.path.exists(path):
        raise FileNotFoundError("HIP library not built: %s" % path)
    lib = ctypes.CDLL(path)
    lib.DLL_InvokeFloat.argtypes = [_c_long, _c_long, _c_float_p, _c_long, ctypes.POINTER(_c_float_p),
                                    ctypes.POINTER(_c_long), _c_tchar_p, _c_long]
    lib.DLL_InvokeFloat.restype = _c_long
    lib.DLL_InvokeFloatEx2.argtypes = [_c_long, _c_long, _c_float_p, _c_long, _c_longlong_p, _c_long,
                                       ctypes.POINTER(_c_float_p), ctypes.POINTER(_c_long), _c_tchar_p, _c_long]
    lib.DLL_InvokeFloatEx2.restype = _c_long
    lib.DLL_InvokeFloatEx.argtypes = [_c_long, _c_long, _c_float_p, _c_long, _c_tchar_p, ctypes.POINTER(_c_float_p),
                                      ctypes.POINTER(_c_long), _c_tchar_p, _c_long]
    lib.DLL_InvokeFloatEx.restype = _c_long
    lib.DLL_QueryString.argtypes = [_c_long, _c_long, ctypes.POINTER(_c_long), _c_long, ctypes.POINTER(_c_tchar_p),
                                    _c_tchar_p, _c_long]
    lib.DLL_QueryString.restype = _c_long
    lib.DLL_QueryStringFloatEx.argtypes = [_c_long, _c_long, ctypes.POINTER(_c_long), _c_long, _c_tchar_p, _c_long,
                                           _c_tchar_p, _c_long]
    lib.DLL_QueryStringFloatEx.restype = _c_long
    lib.DLL_InvokeDouble.argtypes = [_c_long, _c_long, _c_double_p, _c_long, ctypes.POINTER(_c_double_p),
                                     ctypes.POINTER(_c_long), _c_tchar_p, _c_long]
    lib.DLL_InvokeDouble.restype = _c_long
    lib.DLL_InvokeDoubleEx2.argtypes = [_c_long, _c_long, _c_double_p, _c_long, _c_longlong_p, _c_long,
                                        ctypes.POINTER(_c_double_p), ctypes.POINTER(_c_long), _c_tchar_p, _c_long]
    lib.DLL_InvokeDoubleEx2.restype = _c_long
    lib.MCH_TimeInvokeFloatEx2.argtypes = [_c_long, _c_long, _c_float_p, _c_long, _c_longlong_p, _c_long, _c_long, _c_long,
                                           _c_float_p, _c_tchar_p, _c_long]
    lib.MCH_TimeInvokeFloatEx2.restype = _c_long
    lib.MCH_TimeInvokeFloatEx2Sets.argtypes = [_c_long, _c_long, _c_float_p, _c_long, _c_longlong_p, _c_long, _c_long, _c_long, _c_long,
                                               _c_float_p, _c_tchar_p, _c_long]
    lib.MCH_TimeInvokeFloatEx2Sets.restype = _c_long
    lib.MCH_AttnDecodeForwardNoAlloc.argtypes = [_c_long, _c_float_p, _c_long, _c_longlong_p, _c_long, _c_tchar_p, _c_long]
    lib.MCH_AttnDecodeForwardNoAlloc.restype = _c_long
    return lib


def _utf16(s):
    data = s.encode("utf-16-le") + b"\0\0"
    buf = (ctypes.c_uint16 * (len(data) // 2)).from_buffer_copy(data)
    return buf


def _from_utf16(buf):
    raw = bytes(bytearray(ctypes.string_at(buf, ctypes.sizeof(buf))))
    s = raw.decode("utf-16-le", errors="replace")
    return s.split("\0", 1)[0]


class CudaDnn:
    """One kernel (device context) of the native library, float base type (``CudaDnnDouble`` below: double).

    CudaDnn.cs:1679-1760: the constructor loads the DLL at ``strPath`` and sends
    INITIALIZE with ``{deviceId, flags}`` to obtain the kernel index.
    """

    OUT_CAPACITY = 16
    # the base type T of CudaDnn<T>: element type of every array that crosses the boundary, and the entry points it uses
    DTYPE = np.float32
    _CTYPE = ctypes.c_float
    _CPTR = _c_float_p
    _INVOKE, _INVOKE_EX2 = "DLL_InvokeFloat", "DLL_InvokeFloatEx2"

    def __init__(self, nDeviceID=0, flags=DEVINIT.CUBLAS | DEVINIT.CURAND, lSeed=None, strPath=None):
        self._lib = load_library(strPath)
        self.Path = strPath or default_library_path()
        self.m_hKernel = 0
        args = [nDeviceID, flags] + ([lSeed] if lSeed is not None else [])
        rg = self.RunFloat(0, CUDAFN.INITIALIZE, args)
        self.m_hKernel = int(rg[0])
        self.m_nDeviceId = nDeviceID

    # ---- raw dispatch, the role CudaControl plays for the C# host ----------------
    def _check(self, err, errbuf):
        if err != 0:
            raise CudaDnnError(err, _from_utf16(errbuf))

    def _out(self, capacity=None):
        cap = capacity or self.OUT_CAPACITY
        buf = (self._CTYPE * cap)()
        return buf, ctypes.cast(buf, self._CPTR), _c_long(cap)

    def _collect(self, buf, pout, nout, hKernel):
        n = nout.value
        if n <= 0:
            return np.empty(0, self.DTYPE)
        addr = ctypes.addressof(pout.contents)
        if addr == ctypes.addressof(buf):
            return np.ctypeslib.as_array(buf)[:n].copy()
        # the library replaced the buffer with one of its own: copy out, hand it back (FREEMEM = -1)
        out = np.ctypeslib.as_array(pout, shape=(n,)).copy()
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        dummy_buf, dummy_p, dummy_n = self._out(4)
        getattr(self._lib, self._INVOKE)(hKernel, CUDAFN.FREEMEM_HOST, pout, 0, ctypes.byref(dummy_p), ctypes.byref(dummy_n), errbuf, _ERRMAX)
        return out

    def _farr(self, rg):
        if rg is None:
            return None, 0
        a = np.ascontiguousarray(rg, dtype=self.DTYPE).reshape(-1)
        return a, a.size

    @staticmethod
    def _larr(rg):
        if rg is None:
            return None, 0
        a = np.ascontiguousarray(rg, dtype=np.int64).reshape(-1)
        return a, a.size

    def RunFloat(self, hKernel, fn, rgf, out_capacity=None):
        a, n = self._farr(rgf)
        buf, pout, nout = self._out(out_capacity)
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = getattr(self._lib, self._INVOKE)(hKernel, fn, a.ctypes.data_as(self._CPTR) if a is not None else None, n,
                                               ctypes.byref(pout), ctypes.byref(nout), errbuf, _ERRMAX)
        self._check(err, errbuf)
        return self._collect(buf, pout, nout, hKernel)

    def RunFloatEx2(self, hKernel, fn, rgf, rgl, out_capacity=None):
        a, n = self._farr(rgf)
        l, ln = self._larr(rgl)
        buf, pout, nout = self._out(out_capacity)
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = getattr(self._lib, self._INVOKE_EX2)(hKernel, fn, a.ctypes.data_as(self._CPTR) if a is not None else None, n,
                                                   l.ctypes.data_as(_c_longlong_p) if l is not None else None, ln,
                                                   ctypes.byref(pout), ctypes.byref(nout), errbuf, _ERRMAX)
        self._check(err, errbuf)
        return self._collect(buf, pout, nout, hKernel)

    def RunFloatEx(self, hKernel, fn, rgf, strInput):
        a, n = self._farr(rgf)
        buf, pout, nout = self._out()
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        s = _utf16(strInput)
        err = self._lib.DLL_InvokeFloatEx(hKernel, fn, a.ctypes.data_as(_c_float_p) if a is not None else None, n,
                                          ctypes.cast(s, _c_tchar_p), ctypes.byref(pout), ctypes.byref(nout), errbuf, _ERRMAX)
        self._check(err, errbuf)
        return self._collect(buf, pout, nout, hKernel)

    def QueryString(self, hKernel, fn, rgArg):
        a = np.ascontiguousarray(rgArg if rgArg is not None else [], dtype=np.int32)
        pout = _c_tchar_p()
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = self._lib.DLL_QueryString(hKernel, fn, a.ctypes.data_as(ctypes.POINTER(_c_long)), a.size, ctypes.byref(pout),
                                        errbuf, _ERRMAX)
        self._check(err, errbuf)
        chars = []
        i = 0
        while pout[i] != 0:
            chars.append(pout[i])
            i += 1
        text = np.array(chars, np.uint16).tobytes().decode("utf-16-le")
        self._lib.DLL_QueryString(hKernel, CUDAFN.FREEMEM_HOST, None, 0, ctypes.byref(pout), errbuf, _ERRMAX)
        return [text]

    def QueryStringFloatEx(self, hKernel, fn, rgArg, lMax=16384):
        a = np.ascontiguousarray(rgArg, dtype=np.int32)
        out = (ctypes.c_uint16 * lMax)()
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = self._lib.DLL_QueryStringFloatEx(hKernel, fn, a.ctypes.data_as(ctypes.POINTER(_c_long)), a.size,
                                               ctypes.cast(out, _c_tchar_p), lMax, errbuf, _ERRMAX)
        self._check(err, errbuf)
        return [_from_utf16(out)]

    def _ex2(self, fn, rgf, rgl, cap=None):
        return self.RunFloatEx2(self.m_hKernel, fn, rgf, rgl, cap)

    # ---- lifetime / device ------------------------------------------------------
    def Dispose(self):
        """CudaDnn.cs:1800-1815: CLEANUP of this kernel index."""
        if self.m_hKernel > 0:
            self.RunFloat(self.m_hKernel, CUDAFN.CLEANUP, [self.m_hKernel])
            self.m_hKernel = 0

    def __del__(self):
        try:
            self.Dispose()
        except Exception:
            pass

    def SynchronizeDevice(self):
        """CudaDnn.cs:2311-2320."""
        self.RunFloat(self.m_hKernel, CUDAFN.SYNCHRONIZEDEVICE, None)

    def GetDeviceID(self):
        return int(self.RunFloat(self.m_hKernel, CUDAFN.GETDEVICE, None)[0])

    def GetDeviceName(self, nDeviceID=0):
        """CudaDnn.cs:2253-2260."""
        return self.QueryString(self.m_hKernel, CUDAQRY.DEVICE_NAME, [nDeviceID])[0]

    # ---- memory -------------------------------------------------------------------
    def AllocMemory(self, src, hStream=0, bHalfSize=False):
        """CudaDnn.cs:2584-2650 (data) / 2695-2745 (capacity).  ``src`` is either an
        element count or an array of initial values."""
        fn = CUDAFN.ALLOCMEM_HALF if bHalfSize else CUDAFN.ALLOCMEM
        if isinstance(src, (int, np.integer)):
            if src <= 0:
                raise ValueError("capacity must be positive")
            return int(self._ex2(fn, None, [int(src)])[0])
        data = np.ascontiguousarray(src, dtype=self.DTYPE).reshape(-1)
        if data.size == 0:
            raise ValueError("no data")
        head = [data.size] + ([hStream] if hStream > 0 else [])
        rgf = np.concatenate([np.array(head, self.DTYPE), data])
        return int(self._ex2(fn, rgf, head)[0])

    def FreeMemory(self, hMem):
        """CudaDnn.cs:2763-2790."""
        self._ex2(CUDAFN.FREEMEM, None, [hMem])

    def GetMemoryFloat(self, hMem, lCount=-1):
        """CudaDnn.cs:2935-2970: ``l{h, count}``; the DLL swaps in its own buffer when
        the caller's is too small."""
        cap = max(int(lCount), 1) if lCount >= 0 else self.OUT_CAPACITY
        return self._ex2(CUDAFN.GETMEM, None, [hMem, lCount], cap)

    def SetMemory(self, hMem, src, hStream=0, nCount=-1):
        """CudaDnn.cs:3027-3095: ``f{h, count, [stream,] data}``, ``l{h, count}``."""
        data = np.ascontiguousarray(src, dtype=self.DTYPE).reshape(-1)
        if nCount == -1:
            nCount = data.size
        if nCount == 0:
            raise ValueError("There are no data items to set!")
        head = [hMem, nCount] + ([hStream] if hStream > 0 else [])
        rgf = np.concatenate([np.array(head, self.DTYPE), data[:nCount]])
        self._ex2(CUDAFN.SETMEM, rgf, [hMem, nCount])

    def CreateMemoryPointer(self, hData, lOffset, lCount):
        """CudaDnn.cs:3274-3287."""
        return int(self._ex2(CUDAFN.CREATE_MEMORYPOINTER, None, [hData, lOffset, lCount])[0])

    def FreeMemoryPointer(self, hData):
        """CudaDnn.cs:3296-3304."""
        self._ex2(CUDAFN.FREE_MEMORYPOINTER, None, [hData])

    # ---- math -----------------------------------------------------------------------
    def set(self, nCount, hHandle, fVal, nIdx=-1, nXOff=0):
        """CudaDnn.cs:6739-6750."""
        self._ex2(CUDAFN.CUDA_SET, [fVal], [nCount, hHandle, 0, nIdx, nXOff])

    def copy(self, nCount, hSrc, hDst, nSrcOffset=0, nDstOffset=0, hStream=-1, bSrcHalfSizeOverride=None,
             bDstHalfSizeOverride=None):
        """CudaDnn.cs:6824-6840."""
        s = -1 if bSrcHalfSizeOverride is None else int(bSrcHalfSizeOverride)
        d = -1 if bDstHalfSizeOverride is None else int(bDstHalfSizeOverride)
        self._ex2(CUDAFN.CUDA_COPY, None, [nCount, hSrc, hDst, nSrcOffset, nDstOffset, hStream, s, d])

    def gemm(self, bTransA, bTransB, m, n, k, fAlpha, hA, hB, fBeta, hC, nAOffset=0, nBOffset=0, nCOffset=0, nGroups=1,
             nGroupOffsetA=0, nGroupOffsetB=0, nGroupOffsetC=0):
        """CudaDnn.cs:7102-7108: row-major C = alpha op(A) op(B) + beta C."""
        self._ex2(CUDAFN.CUDA_GEMM, [fAlpha, fBeta],
                  [int(bTransA), int(bTransB), m, n, k, 0, hA, hB, 0, hC, nAOffset, nBOffset, nCOffset, nGroups,
                   nGroupOffsetA, nGroupOffsetB, nGroupOffsetC])

    def gemm2(self, bTransA, bTransB, m, n, k, fAlpha, hA, hB, fBeta, hC, lda, ldb, ldc, stridea=None, strideb=None,
              stridec=None, batch_count=None):
        """The ``gemm`` overloads with leading dimensions (CudaDnn.cs:7129-7166): BLAS
        column-major semantics, optionally strided-batched."""
        rgl = [int(bTransA), int(bTransB), m, n, k, 0, hA, hB, 0, hC, lda, ldb, ldc]
        if batch_count is not None:
            rgl += [stridea, strideb, stridec, batch_count]
        self._ex2(CUDAFN.CUDA_GEMM2, [fAlpha, fBeta], rgl)

    def matmul(self, nOuterCount, m, n, k, hA, hB, hC, dfScale=1.0, bTransA=False, bTransB=False, bAccumulate=False):
        """CudaDnn.cs:7513-7524: row-major batched matmul expressed as a column-major
        gemm with swapped operands."""
        ldb = k if bTransB else n
        lda = m if bTransA else k
        self.gemm2(bTransB, bTransA, n, m, k, dfScale, hB, hA, 1.0 if bAccumulate else 0.0, hC, ldb, lda, n, k * n, m * k,
                   m * n, nOuterCount)

    def gemv(self, bTransA, m, n, fAlpha, hA, hX, fBeta, hY, nAOffset=0, nXOffset=0, nYOffset=0):
        """CudaDnn.cs:7289-7295."""
        self._ex2(CUDAFN.CUDA_GEMV, [fAlpha, fBeta], [int(bTransA), m, n, 0, hA, hX, 0, hY, nAOffset, nXOffset, nYOffset])

    def axpy(self, n, fAlpha, hX, hY, nXOff=0, nYOff=0):
        """CudaDnn.cs:7393-7399."""
        self._ex2(CUDAFN.CUDA_AXPY, [fAlpha], [n, 0, hX, hY, nXOff, nYOff])

    def scal(self, n, fAlpha, hX, nXOff=0):
        """CudaDnn.cs:7617-7623."""
        self._ex2(CUDAFN.CUDA_SCAL, [fAlpha], [n, 0, hX, nXOff])

    def scale(self, n, fAlpha, hX, hY, nXOff=0, nYOff=0):
        """CudaDnn.cs:7777-7783."""
        self._ex2(CUDAFN.CUDA_SCALE, [fAlpha], [n, 0, hX, hY, nXOff, nYOff])

    def add(self, n, hA, hB, hY, fAlpha=None):
        """CudaDnn.cs:8047-8092: Y = A + B, or Y = A + alpha * B."""
        if fAlpha is None:
            self._ex2(CUDAFN.CUDA_ADD, None, [n, hA, hB, hY])
        else:
            self._ex2(CUDAFN.CUDA_ADD, [fAlpha], [n, hA, hB, hY, 0])

    def mul(self, n, hA, hB, hY, nAOff=0, nBOff=0, nYOff=0):
        """CudaDnn.cs:8154-8160."""
        self._ex2(CUDAFN.CUDA_MUL, None, [n, hA, hB, hY, nAOff, nBOff, nYOff])

    def sub(self, n, hA, hB, hY, nAOff=0, nBOff=0, nYOff=0, nB=0):
        """CudaDnn.cs:8132-8138."""
        self._ex2(CUDAFN.CUDA_SUB, None, [n, hA, hB, hY, nAOff, nBOff, nYOff, nB])

    def div(self, n, hA, hB, hY):
        """CudaDnn.cs:8281-8287."""
        self._ex2(CUDAFN.CUDA_DIV, None, [n, hA, hB, hY])

    def add_scalar(self, n, fAlpha, hY, nYOff=0):
        """CudaDnn.cs:8010-8016."""
        self._ex2(CUDAFN.CUDA_ADD_SCALAR, [fAlpha], [n, 0, hY, nYOff])

    def powx(self, n, hA, fAlpha, hY, nAOff=0, nYOff=0):
        """CudaDnn.cs:8419-8425."""
        self._ex2(CUDAFN.CUDA_POWX, [fAlpha], [n, hA, 0, hY, nAOff, nYOff])

    def sqrt(self, n, hX, hY, dfEpsilon=0.0):
        """CudaDnn.cs:8520-8526."""
        self._ex2(CUDAFN.CUDA_SQRT, [dfEpsilon], [n, hX, hY])

    def invert(self, n, hX, hY, nXOff=0, nYOff=0, dfScaleNumerator=1.0, dfScaleDenom=1.0):
        """CudaDnn.cs:8453-8459."""
        self._ex2(CUDAFN.CUDA_INVERT, [dfScaleNumerator, dfScaleDenom], [n, hX, hY, nXOff, nYOff])

    def channel_mean(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, nXOff=0):
        """CudaDnn.cs:9030-9036."""
        self._ex2(CUDAFN.CUDA_CHANNEL_MEAN, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY, nXOff])

    def exp(self, n, hA, hY, nAOff=0, nYOff=0, dfBeta=1.0):
        """CudaDnn.cs:8332-8338: y = exp(beta a)."""
        self._ex2(CUDAFN.CUDA_EXP, [dfBeta], [n, hA, hY, nAOff, nYOff, 0])

    def log(self, n, hA, hY, dfBeta=1.0, dfAlpha=0.0):
        """CudaDnn.cs:8365-8371: y = log(beta (a + alpha))."""
        self._ex2(CUDAFN.CUDA_LOG, [dfBeta, dfAlpha], [n, hA, hY, 0, 0])

    def channel_max(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, bReturnIdx=False, bAcrossChannels=True):
        """CudaDnn.cs:9012-9018."""
        self._ex2(CUDAFN.CUDA_CHANNEL_MAX, None,
                  [nCount, nOuterNum, nChannels, nInnerNum, hX, hY, 1 if bReturnIdx else 0, 1 if bAcrossChannels else 0])

    def channel_sub(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, hA=None):
        """CudaDnn.cs:9131-9154: y = a - x (x broadcast over the channels); a = y when absent."""
        rgl = [nCount, nOuterNum, nChannels, nInnerNum, hX, hY] + ([hA] if hA is not None else [])
        self._ex2(CUDAFN.CUDA_CHANNEL_SUB, None, rgl)

    def channel_div(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, nMethod=1):
        """CudaDnn.cs:9223-9229."""
        self._ex2(CUDAFN.CUDA_CHANNEL_DIV, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY, nMethod])

    def channel_dot(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hA, hY):
        """CudaDnn.cs:9295-9301."""
        self._ex2(CUDAFN.CUDA_CHANNEL_DOT, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hA, hY])

    def channel_sum(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY):
        """CudaDnn.cs:9182-9188: y[outer, inner] = sum over the channels."""
        self._ex2(CUDAFN.CUDA_CHANNEL_SUM, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY])

    def channel_sumEx(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, bSumAcrossChannels, dir, nChannelsY=-1):
        """CudaDnn.cs:9205-9211."""
        self._ex2(CUDAFN.CUDA_CHANNEL_SUM2, None,
                  [nCount, nOuterNum, nChannels, nInnerNum, hX, hY, 1 if bSumAcrossChannels else 0, dir, nChannelsY])

    def channel_fillfrom(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY, dir):
        """CudaDnn.cs:9086-9092."""
        self._ex2(CUDAFN.CUDA_CHANNEL_FILLFROM, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY, dir])

    def channel_copyall(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY):
        """CudaDnn.cs:9443-9449."""
        self._ex2(CUDAFN.CUDA_CHANNEL_COPYALL, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY])

    def channel_duplicate(self, nCount, nOuterNum, nChannels, nInnerNum, hX, hY):
        """CudaDnn.cs:9312-9318."""
        self._ex2(CUDAFN.CUDA_CHANNEL_DUP, None, [nCount, nOuterNum, nChannels, nInnerNum, hX, hY])

    def mask(self, n, nMaskDim, fSearch, fReplace, hX, hMask, hY):
        """CudaDnn.cs:7850-7856."""
        self._ex2(CUDAFN.CUDA_MASK, [fSearch, fReplace], [n, nMaskDim, 0, 0, hX, hMask, hY])

    def mask_batch(self, n, nBatch, nMaskDim, fSearch, fReplace, hX, hMask, hY):
        """CudaDnn.cs:7899-7905."""
        self._ex2(CUDAFN.CUDA_MASK_BATCH, [fSearch, fReplace], [n, nBatch, nMaskDim, 0, 0, hX, hMask, hY])

    def transpose(self, n, hX, hY, hXCounts, hYCounts, hMapping, nNumAxes, hBuffer):
        """CudaDnn.cs:8773-8779."""
        self._ex2(CUDAFN.CUDA_TRANSPOSE, None, [n, hX, hY, hXCounts, hYCounts, hMapping, nNumAxes, hBuffer])

    def transposeHW(self, n, c, h, w, hSrc, hDst):
        """CudaDnn.cs:7536-7542."""
        self._ex2(CUDAFN.CUDA_TRANSPOSE_HW, None, [n, c, h, w, hSrc, hDst])

    def channel_copy(self, nCount, nOuterNum, nChannels, nBlocks, nInnerNum, nOffset, hX, hY, dir):
        """CudaDnn.cs:9426-9432."""
        self._ex2(CUDAFN.CUDA_CHANNEL_COPY, None, [nCount, nOuterNum, nChannels, nBlocks, nInnerNum, nOffset, hX, hY, dir])

    def embed_fwd(self, nCount, hBottomData, hWeight, nM, nN, nK, hTopData):
        """CudaDnn.cs:9751-9757."""
        self._ex2(CUDAFN.CUDA_EMBED_FWD, None, [nCount, hBottomData, hWeight, nM, nN, nK, hTopData])

    def silu_fwd(self, nCount, hBottomData, hTopData):
        """CudaDnn.cs:10152-10158."""
        self._ex2(CUDAFN.CUDA_SILU_FWD, None, [nCount, hBottomData, hTopData])

    def relu_fwd(self, nCount, hBottomData, hTopData, fNegativeSlope=0.0):
        """CudaDnn.cs:10417-10423."""
        self._ex2(CUDAFN.CUDA_RELU_FWD, [fNegativeSlope], [nCount, hBottomData, hTopData, 0])

    def relu_bwd(self, nCount, hTopDiff, hTopData, hBottomDiff, fNegativeSlope=0.0):
        """CudaDnn.cs:10438-10444."""
        self._ex2(CUDAFN.CUDA_RELU_BWD, [fNegativeSlope], [nCount, hTopDiff, hTopData, hBottomDiff, 0])

    def silu_bwd(self, nCount, hTopDiff, hTopData, hBottomDiff, hBottomData):
        """CudaDnn.cs:10174-10180."""
        self._ex2(CUDAFN.CUDA_SILU_BWD, None, [nCount, hTopDiff, hTopData, hBottomDiff, hBottomData])

    def gelu_fwd(self, nCount, hBottomData, hTopData, bEnableBertVersion):
        """CudaDnn.cs:10098-10104."""
        self._ex2(CUDAFN.CUDA_GELU_FWD, None, [nCount, hBottomData, hTopData, 1 if bEnableBertVersion else 0])

    def gelu_bwd(self, nCount, hTopDiff, hTopData, hBottomDiff, hBottomData, bEnableBertVersion):
        """CudaDnn.cs:10132-10138."""
        self._ex2(CUDAFN.CUDA_GELU_BWD, None, [nCount, hTopDiff, hTopData, hBottomDiff, hBottomData, 1 if bEnableBertVersion else 0])

    # ---- LayerNorm ------------------------------------------------------------------------------
    def CreateLayerNorm(self, nGpuID, nCount, nOuterNum, nChannels, nInnerNum, fEps=1e-10):
        """CudaDnn.cs:6307-6319."""
        return int(self._ex2(CUDAFN.CUDA_CREATE_LAYERNORM, [fEps], [nGpuID, nCount, nOuterNum, nChannels, nInnerNum])[0])

    def FreeLayerNorm(self, hLayerNorm):
        """CudaDnn.cs:6325-6331."""
        self.RunFloat(self.m_hKernel, CUDAFN.CUDA_FREE_LAYERNORM, [hLayerNorm])

    def LayerNormForward(self, hLayerNorm, hXdata, hYdata):
        """CudaDnn.cs:6339-6345."""
        self._ex2(CUDAFN.CUDA_LAYERNORM_FWD, None, [hLayerNorm, hXdata, hYdata])

    def LayerNormBackward(self, hLayerNorm, hYdata, hYdiff, hXdiff):
        """CudaDnn.cs:6354-6360."""
        self._ex2(CUDAFN.CUDA_LAYERNORM_BWD, None, [hLayerNorm, hYdata, hYdiff, hXdiff])

    # ---- cuDNN-shaped handles ---------------------------------------------------------
    def CreateCuDNN(self, hStream=0):
        """CudaDnn.cs:3509-3520."""
        return int(self.RunFloat(self.m_hKernel, CUDAFN.CREATE_CUDNN, [hStream])[0])

    def FreeCuDNN(self, h):
        """CudaDnn.cs:3527-3533."""
        self.RunFloat(self.m_hKernel, CUDAFN.FREE_CUDNN, [h])

    def CreateTensorDesc(self):
        """CudaDnn.cs:3819-3830."""
        return int(self.RunFloat(self.m_hKernel, CUDAFN.CREATE_TENSORDESC, None)[0])

    def FreeTensorDesc(self, h):
        """CudaDnn.cs:3837-3843."""
        self.RunFloat(self.m_hKernel, CUDAFN.FREE_TENSORDESC, [h])

    def SetTensorDesc(self, hHandle, n, c, h, w, bHalf=False, strides=None):
        """CudaDnn.cs:3900-3930."""
        rgl = [hHandle, int(bHalf), n, c, h, w] + (list(strides) if strides else [])
        self._ex2(CUDAFN.SET_TENSORDESC, None, rgl)

    def SoftmaxForward(self, hCuDnn, alg, mode, fAlpha, hBottomDataDesc, hBottomData, fBeta, hTopDataDesc, hTopData):
        """CudaDnn.cs:4919-4925."""
        self._ex2(CUDAFN.SOFTMAX_FWD, [fAlpha, fBeta], [hCuDnn, 0, hBottomDataDesc, hBottomData, 0, hTopDataDesc, hTopData, alg, mode])

    def SoftmaxBackward(self, hCuDnn, alg, mode, fAlpha, hTopDataDesc, hTopData, hTopDiffDesc, hTopDiff, fBeta, hBottomDiffDesc, hBottomDiff):
        """CudaDnn.cs:4941-4947."""
        self._ex2(CUDAFN.SOFTMAX_BWD, [fAlpha, fBeta],
                  [hCuDnn, 0, hTopDataDesc, hTopData, hTopDiffDesc, hTopDiff, 0, hBottomDiffDesc, hBottomDiff, alg, mode])

    # ---- attention -------------------------------------------------------------------------
    def CreateAttn(self):
        """CudaDnn.cs:5614-5626."""
        return int(self.RunFloat(self.m_hKernel, CUDAFN.CUDA_ATTN_CREATE, None)[0])

    def FreeAttn(self, hAttn):
        """CudaDnn.cs:5632-5638."""
        self.RunFloat(self.m_hKernel, CUDAFN.CUDA_ATTN_FREE, [hAttn])

    def SetAttn(self, hCuDnn, hAttn, nGpuID, bTraining, nBatch, nBlockSize, nHeads, nSize, fDropout, lSeed=0):
        """CudaDnn.cs:5653-5659."""
        self._ex2(CUDAFN.CUDA_ATTN_SET, [fDropout], [hCuDnn, hAttn, nGpuID, int(bTraining), nBatch, nBlockSize, nHeads, nSize, lSeed])

    def AttnScaledDotProductForward(self, hCuDnn, hAttn, nBlockSize, hQdata, hKdata, hVdata, hMaskdata, hYdata,
                                    bBatchMask=True, nBlockSizeK=None, bMergedY=False):
        """CudaDnn.cs:5673-5679.  ``nBlockSizeK`` (key length, when it differs from the
        query length) is an optional tenth value with no counterpart in the reference, and so
        are ``bBatchMask=2`` (a (B,T_q,T_k) mask) and ``bMergedY`` (eleventh value: Y written
        head-merged, (B,T,H,hs), instead of (B,H,T,hs))."""
        rgl = [hCuDnn, hAttn, nBlockSize, hQdata, hKdata, hVdata, hMaskdata, hYdata, int(bBatchMask)]
        if nBlockSizeK is not None or bMergedY:
            rgl.append(nBlockSizeK if nBlockSizeK is not None else nBlockSize)
        if bMergedY:
            rgl.append(1)
        self._ex2(CUDAFN.CUDA_ATTN_FWD, None, rgl)

    def QkvProjHeads(self, nBatch, nT, nHeads, nSize, hX, hWeight, hBias, hQ, hK, hV, hRope=0):
        """Fused QKV projection (no counterpart in the reference: replaces the InnerProduct, bias GEMM, three
        channel copies and three head transposes of CausalSelfAttentionLayer.cs:526-557): q, k, v written as
        (B,H,T,hs).  With hRope the two RopeForward calls on q and k (:538-545) are part of it as well."""
        rgl = [nBatch, nT, nHeads, nSize, hX, hWeight, hBias, hQ, hK, hV]
        if hRope:
            rgl.append(hRope)
        self._ex2(CUDAFN.QKV_PROJ_HEADS, None, rgl)

    def LinearForward(self, nM, nN, nK, hX, hWeight, hBias, hY):
        """y (M,N) = x (M,K) W^T (N,K) + bias in one GEMM (no counterpart in the reference: replaces the product and
        the rank-1 bias update of InnerProductLayer.cs:372-417).  hBias 0: no bias."""
        self._ex2(CUDAFN.LINEAR_FWD, None, [nM, nN, nK, hX, hWeight, hBias, hY])

    def AttnScaledDotProductBackward(self, hCuDnn, hAttn, hQdata, hQdiff, hKdata, hKdiff, hVdata, hVdiff, hMaskdata, hYData, hYdiff):
        """CudaDnn.cs:5695-5701."""
        self._ex2(CUDAFN.CUDA_ATTN_BWD, None, [hCuDnn, hAttn, hQdata, hQdiff, hKdata, hKdiff, hVdata, hVdiff, hMaskdata, hYData, hYdiff])

    def AttnDecodeForward(self, nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead,
                          nStridePos, fScale=0.0, hRope=0, hKNew=0, hVNew=0):
        """Single-call KV-cache attention for one query token per sequence (no
        counterpart in the reference: replaces the per-position loop of
        MultiheadAttentionLayer.cs:713-730,759-777)."""
        rgl = [nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead, nStridePos]
        if hRope or hKNew or hVNew:
            rgl += [hRope, hKNew, hVNew]
        self._ex2(CUDAFN.ATTN_DECODE_FWD, [fScale], rgl)

    def AttnDecodeForwardNoAlloc(self, nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead,
                                 nStridePos, fScale=0.0, hRope=0, hKNew=0, hVNew=0):
        """AttnDecodeForward through the entry point that allocates no device memory (fixed scratch inside the
        library; for callers that cannot call hipMalloc).  Same arguments, bounded problem size."""
        rgl = [nBatch, nHeads, nKvHeads, nSize, nLen, hQ, hKCache, hVCache, hY, nStrideBatch, nStrideHead, nStridePos]
        if hRope or hKNew or hVNew:
            rgl += [hRope, hKNew, hVNew]
        a, n = self._farr([fScale])
        l, ln = self._larr(rgl)
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = self._lib.MCH_AttnDecodeForwardNoAlloc(self.m_hKernel, a.ctypes.data_as(_c_float_p), n, l.ctypes.data_as(_c_longlong_p),
                                                     ln, errbuf, _ERRMAX)
        self._check(err, errbuf)

    def RmsNormForward(self, nOuter, nDim, hX, hWeight, hY, fEps=1e-5):
        """Fused RMSNorm (replaces the chain of RMSNormLayer.cs:156-180)."""
        self._ex2(CUDAFN.RMSNORM_FWD, [fEps], [nOuter, nDim, hX, hWeight, hY])

    def SwigluForward(self, n, hA, hB, hY):
        """y = silu(a) * b in one pass."""
        self._ex2(CUDAFN.SWIGLU_FWD, None, [n, hA, hB, hY])

    # ---- RoPE ---------------------------------------------------------------------------------
    def CreateRope(self, nSharedIndex, nGpuID, nCount, nBatch, nSeqLen, nHeads, nDim, fTheta=10000.0):
        """CudaDnn.cs:6375-6390."""
        return int(self._ex2(CUDAFN.CUDA_CREATE_ROPE, [fTheta], [nSharedIndex, nGpuID, nCount, nBatch, nSeqLen, nHeads, nDim])[0])

    def FreeRope(self, hRope):
        """CudaDnn.cs:6396-6402."""
        self.RunFloat(self.m_hKernel, CUDAFN.CUDA_FREE_ROPE, [hRope])

    def RopeForward(self, hRope, n, hXdata, hYdata, nFreqOffset=-1):
        """CudaDnn.cs:6409-6415."""
        self._ex2(CUDAFN.CUDA_ROPE_FWD, None, [hRope, n, hXdata, hYdata, nFreqOffset])

    def RopeBackward(self, hRope, n, hXdata, hYdiff, hXdiff):
        """CudaDnn.cs:6425-6431."""
        self._ex2(CUDAFN.CUDA_ROPE_BWD, None, [hRope, n, hXdata, hYdiff, hXdiff])

    # ---- blob loader (weights from very large files) ------------------------------------------------
    def CreateBlobLoader(self, strFile):
        """CudaDnn.cs:6438-6450."""
        return int(self.RunFloatEx(self.m_hKernel, CUDAFN.CUDA_CREATE_BLOBLOADER, None, strFile)[0])

    def FreeBlobLoader(self, hBlobLoader):
        """CudaDnn.cs:6456-6462."""
        self.RunFloat(self.m_hKernel, CUDAFN.CUDA_FREE_BLOBLOADER, [hBlobLoader])

    def LoadBlob(self, hBlobLoader, lCount, hDst, lLocalOffsetInItems):
        """CudaDnn.cs:6472-6478."""
        self._ex2(CUDAFN.CUDA_BLOBLOADER_LOAD, None, [hBlobLoader, lCount, hDst, lLocalOffsetInItems])

    def BlobLoaderResetOffset(self, hBlobLoader, lOffsetInBytes):
        """CudaDnn.cs:6485-6491."""
        self._ex2(CUDAFN.CUDA_BLOBLOADER_RESETOFFSET, None, [hBlobLoader, lOffsetInBytes])

    def BlobLoaderAddToOffset(self, hBlobLoader, lOffsetInItems):
        """CudaDnn.cs:6498-6504."""
        self._ex2(CUDAFN.CUDA_BLOBLOADER_ADDTOOFFSET, None, [hBlobLoader, lOffsetInItems])

    # ---- extensions ---------------------------------------------------------------------------------
    def CreateExtension(self, strExtensionDllPath):
        """CudaDnn.cs:3703-3715."""
        return int(self.RunFloatEx(self.m_hKernel, CUDAFN.CREATE_EXTENSION, None, strExtensionDllPath)[0])

    def FreeExtension(self, hExtension):
        """CudaDnn.cs:3721-3727."""
        self.RunFloat(self.m_hKernel, CUDAFN.FREE_EXTENSION, [hExtension])

    def RunExtension(self, hExtension, lfnIdx, rgParam, out_capacity=None):
        """CudaDnn.cs:3737-3760: ``f{hExtension, fnIdx, params...}``."""
        rgf = [hExtension, lfnIdx] + (list(np.asarray(rgParam, np.float32).reshape(-1)) if rgParam is not None else [])
        return self.RunFloat(self.m_hKernel, CUDAFN.EXTENSION_RUN, rgf, out_capacity)

    def RunExtensionEx(self, hExtension, lfnIdx, rgParam, strInput):
        """CudaDnn.cs:3771-3794."""
        rgf = [hExtension, lfnIdx] + (list(np.asarray(rgParam, np.float32).reshape(-1)) if rgParam is not None else [])
        return self.RunFloatEx(self.m_hKernel, CUDAFN.EXTENSION_RUN, rgf, strInput)

    def QueryExtensionStrings(self, hExtension, lfnIdx, rgParam):
        """CudaDnn.cs:3800-3812."""
        return self.QueryStringFloatEx(self.m_hKernel, CUDAQRY.EXTENSION_STRING, [int(hExtension), int(lfnIdx)] + [int(v) for v in rgParam])

    # ---- measurement hook --------------------------------------------------------------------------------
    def TimeFunction(self, fn, rgf, rgl, nWarmup=3, nReps=20):
        """Mean duration in ms of ``nReps`` back-to-back dispatches of one Ex2 call,
        measured by the library with HIP events on its own stream."""
        a, n = self._farr(rgf)
        l, ln = self._larr(rgl)
        ms = ctypes.c_float(0)
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = self._lib.MCH_TimeInvokeFloatEx2(self.m_hKernel, fn, a.ctypes.data_as(_c_float_p) if a is not None else None, n,
                                               l.ctypes.data_as(_c_longlong_p) if l is not None else None, ln, nWarmup, nReps,
                                               ctypes.byref(ms), errbuf, _ERRMAX)
        self._check(err, errbuf)
        return float(ms.value)

    def TimeFunctionSets(self, fn, rgf, rglSets, nWarmup=3, nReps=20):
        """As TimeFunction with one list of long arguments per set: dispatch i takes list i mod len(rglSets), so that
        the operands of one dispatch are not the ones the previous dispatches left in the caches."""
        a, n = self._farr(rgf)
        ll = len(rglSets[0])
        if any(len(r) != ll for r in rglSets):
            raise ValueError("the argument lists differ in length")
        l = np.ascontiguousarray(np.asarray(rglSets, np.int64).reshape(-1))
        ms = ctypes.c_float(0)
        errbuf = (ctypes.c_uint16 * _ERRMAX)()
        err = self._lib.MCH_TimeInvokeFloatEx2Sets(self.m_hKernel, fn, a.ctypes.data_as(_c_float_p) if a is not None else None, n,
                                                   l.ctypes.data_as(_c_longlong_p), ll, len(rglSets), nWarmup, nReps,
                                                   ctypes.byref(ms), errbuf, _ERRMAX)
        self._check(err, errbuf)
        return float(ms.value)


class CudaDnnDouble(CudaDnn):
    """One kernel of the double base type (CudaDnn<double>): every array crosses the boundary as doubles through
    DLL_InvokeDouble / DLL_InvokeDoubleEx2 (CudaDnnDLL.cpp:494-853), device memory holds doubles and the arithmetic is
    double.  The library builds the function ids of the attention path for it; any other id raises
    ``CudaDnnError`` with code NOT_IMPLEMENTED (90009)."""

    DTYPE = np.float64
    _CTYPE = ctypes.c_double
    _CPTR = _c_double_p
    _INVOKE, _INVOKE_EX2 = "DLL_InvokeDouble", "DLL_InvokeDoubleEx2"

    def RunFloatEx(self, hKernel, fn, rgf, strInput):
        raise CudaDnnError(90009, "extensions and blob loaders are float objects")
