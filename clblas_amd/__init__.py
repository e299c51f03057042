"""clblas_amd -- Python access to libclblas_amd.so, the MI355X (gfx950) xGEMM / xTRSM core
behind clBLAS's call surface.

The product is the shared library (C ABI declared in include/clblas_amd.h).  This module
only loads it with ctypes and mirrors the entry points with the reference's argument
order (src/clBLAS.h:7382-7405, 7463-7486, 7538-7561, 7622-7645, 7988-8008, 8063-8083);
matrices are passed as
torch CUDA tensors (used purely as device allocations) or as integer device addresses.

There is no CPU fallback: if the library has not been built, loading raises.
"""
import ctypes
import enum
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "libclblas_amd.so")


class Order(enum.IntEnum):
    RowMajor = 0
    ColumnMajor = 1


class Transpose(enum.IntEnum):
    NoTrans = 0
    Trans = 1
    ConjTrans = 2


class Uplo(enum.IntEnum):
    Upper = 0
    Lower = 1


class Diag(enum.IntEnum):
    Unit = 0
    NonUnit = 1


class Side(enum.IntEnum):
    Left = 0
    Right = 1


class Status(enum.IntEnum):
    Success = 0
    InvalidValue = -30
    InvalidDevice = -33
    OutOfResources = -5
    OutOfHostMemory = -6
    NotImplemented = -1024
    NotInitialized = -1023
    InvalidMatA = -1022
    InvalidMatB = -1021
    InvalidMatC = -1020
    InvalidDim = -1017
    InvalidLeadDimA = -1016
    InvalidLeadDimB = -1015
    InvalidLeadDimC = -1014
    InsufficientMemMatA = -1011
    InsufficientMemMatB = -1010
    InsufficientMemMatC = -1009


EXPORTED_SYMBOLS = (
    "clblasGetVersion",
    "clblasSetup",
    "clblasTeardown",
    "clblasSgemm",
    "clblasSgemmNoAlloc",
    "clblasDgemm",
    "clblasCgemm",
    "clblasZgemm",
    "clblasStrsm",
    "clblasDtrsm",
    "clblasCtrsm",
    "clblasZtrsm",
) + tuple("clblas%s%s" % (t, f) for f in ("syrk", "trmm", "symm", "syr2k") for t in "SDCZ") + tuple(
    "clblas%s%s" % (t, f) for f in ("herk", "her2k", "hemm") for t in "CZ") + (
    "clblasAmdReleaseStream", "clblasAmdReserveWorkspace", "clblasAmdWorkspaceStats", "clblasAmdLastDispatch",
    "clblasAmdReloadDebugEnv", "clblasAmdTrsmPollTimeouts", "clblasAmdTileModelQuery", "clblasAmdTileModelParam")

_lib = None


class FloatComplex(ctypes.Structure):
    """By-value complex scalar of clblasCgemm (two floats, one SSE register on x86-64)."""
    _fields_ = [("re", ctypes.c_float), ("im", ctypes.c_float)]


class DoubleComplex(ctypes.Structure):
    """By-value complex scalar of clblasZgemm."""
    _fields_ = [("re", ctypes.c_double), ("im", ctypes.c_double)]


def _declare(lib):
    sz, vp, i = ctypes.c_size_t, ctypes.c_void_p, ctypes.c_int
    for name, real in (("clblasSgemm", ctypes.c_float), ("clblasSgemmNoAlloc", ctypes.c_float),
                       ("clblasDgemm", ctypes.c_double)):
        fn = getattr(lib, name)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sz, real, vp, sz, sz, vp, sz, sz, real, vp, sz, sz, vp]
    for name, cplx in (("clblasCgemm", FloatComplex), ("clblasZgemm", DoubleComplex)):
        fn = getattr(lib, name)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sz, cplx, vp, sz, sz, vp, sz, sz, cplx, vp, sz, sz, vp]
    for name, real in (("clblasStrsm", ctypes.c_float), ("clblasDtrsm", ctypes.c_double)):
        fn = getattr(lib, name)
        fn.restype = i
        fn.argtypes = [i, i, i, i, i, sz, sz, real, vp, sz, sz, vp, sz, sz, vp]
    for name, cplx in (("clblasCtrsm", FloatComplex), ("clblasZtrsm", DoubleComplex)):
        fn = getattr(lib, name)
        fn.restype = i
        fn.argtypes = [i, i, i, i, i, sz, sz, cplx, vp, sz, sz, vp, sz, sz, vp]
    scalars = {"S": ctypes.c_float, "D": ctypes.c_double, "C": FloatComplex, "Z": DoubleComplex}
    for t, sc in scalars.items():
        fn = getattr(lib, "clblas%ssyrk" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sc, vp, sz, sz, sc, vp, sz, sz, vp]
        fn = getattr(lib, "clblas%strmm" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, i, i, sz, sz, sc, vp, sz, sz, vp, sz, sz, vp]
        fn = getattr(lib, "clblas%ssymm" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sc, vp, sz, sz, vp, sz, sz, sc, vp, sz, sz, vp]
        fn = getattr(lib, "clblas%ssyr2k" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sc, vp, sz, sz, vp, sz, sz, sc, vp, sz, sz, vp]
    for t, sc, real in (("C", FloatComplex, ctypes.c_float), ("Z", DoubleComplex, ctypes.c_double)):
        fn = getattr(lib, "clblas%sherk" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, real, vp, sz, sz, real, vp, sz, sz, vp]
        fn = getattr(lib, "clblas%sher2k" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sc, vp, sz, sz, vp, sz, sz, real, vp, sz, sz, vp]
        fn = getattr(lib, "clblas%shemm" % t)
        fn.restype = i
        fn.argtypes = [i, i, i, sz, sz, sc, vp, sz, sz, vp, sz, sz, sc, vp, sz, sz, vp]
    lib.clblasSetup.restype = i
    lib.clblasSetup.argtypes = []
    lib.clblasTeardown.restype = None
    lib.clblasTeardown.argtypes = []
    lib.clblasGetVersion.restype = i
    lib.clblasGetVersion.argtypes = [ctypes.POINTER(ctypes.c_uint)] * 3
    lib.clblasAmdReleaseStream.restype = i
    lib.clblasAmdReleaseStream.argtypes = [vp]
    lib.clblasAmdReserveWorkspace.restype = i
    lib.clblasAmdReserveWorkspace.argtypes = [vp, sz, sz, sz]
    lib.clblasAmdWorkspaceStats.restype = None
    lib.clblasAmdWorkspaceStats.argtypes = [ctypes.POINTER(sz), ctypes.POINTER(sz)]
    lib.clblasAmdLastDispatch.restype = sz
    lib.clblasAmdLastDispatch.argtypes = [ctypes.c_char_p, sz]
    lib.clblasAmdReloadDebugEnv.restype = None
    lib.clblasAmdReloadDebugEnv.argtypes = []
    lib.clblasAmdTileModelQuery.restype = ctypes.c_int
    lib.clblasAmdTileModelQuery.argtypes = [ctypes.c_char, sz, sz, sz, ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_int),
                                            ctypes.POINTER(ctypes.c_int), ctypes.POINTER(ctypes.c_double),
                                            ctypes.POINTER(ctypes.c_int), ctypes.c_int]
    lib.clblasAmdTileModelParam.restype = ctypes.c_int
    lib.clblasAmdTileModelParam.argtypes = [ctypes.c_char, ctypes.c_int, ctypes.c_int, ctypes.POINTER(ctypes.c_double), ctypes.c_int]
    lib.clblasAmdTrsmPollTimeouts.restype = ctypes.c_int
    lib.clblasAmdTrsmPollTimeouts.argtypes = [ctypes.POINTER(ctypes.c_uint), ctypes.c_int]


def load_library(path=None):
    """Loads libclblas_amd.so (once) and returns the ctypes handle. Raises if it is missing."""
    global _lib
    if _lib is not None and path is None:
        return _lib
    p = path or LIB_PATH
    if not os.path.exists(p):
        raise RuntimeError(
            "%s not found: build it with `python -m clblas_amd.build` (there is no fallback path)" % p)
    lib = ctypes.CDLL(p)
    _declare(lib)
    if path is None:
        _lib = lib
    return lib


def _ptr(x):
    """Device address of a torch tensor, or the integer itself."""
    if x is None:
        return None
    if isinstance(x, int):
        return ctypes.c_void_p(x)
    return ctypes.c_void_p(x.data_ptr())


def _stream(stream):
    if stream is None:
        import torch
        return ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
    if isinstance(stream, int):
        return ctypes.c_void_p(stream)
    return ctypes.c_void_p(stream.cuda_stream)


def bind(symbol, *args, stream=None):
    """A zero-argument callable that makes the call `symbol(*args, stream)` - e.g.
    bind("clblasDtrsm", order, side, uplo, trans, diag, M, N, alpha, A, offA, lda, B, offB, ldb) -
    with the arguments converted to their C types once.  For loops in which the microseconds the
    wrappers above spend per call (tensor addresses, torch's current stream) would be measured
    along with the library: benchmarks of small problems.  Tensors must stay alive and in place
    for as long as the callable is used."""
    fn = getattr(load_library(), symbol)
    types = fn.argtypes
    if len(args) + 1 != len(types):
        raise TypeError("%s takes %d arguments and a stream" % (symbol, len(types) - 1))
    conv = []
    for a, t in zip(args, types):
        if t is ctypes.c_void_p:
            conv.append(_ptr(a))
        elif t in (FloatComplex, DoubleComplex):
            z = complex(a)
            conv.append(t(z.real, z.imag))
        else:
            conv.append(t(a))
    conv.append(_stream(stream))
    conv = tuple(conv)
    return lambda: fn(*conv)


def setup():
    return load_library().clblasSetup()


def teardown():
    load_library().clblasTeardown()


def release_stream(stream=None):
    """Frees the library's scratch buffers of `stream` (its work must have completed)."""
    return load_library().clblasAmdReleaseStream(_stream(stream))


def reserve_workspace(gemm_bytes=0, trmm_bytes=0, trsm_bytes=0, stream=None):
    return load_library().clblasAmdReserveWorkspace(_stream(stream), gemm_bytes, trmm_bytes, trsm_bytes)


def workspace_stats():
    """(streams that hold scratch buffers, bytes of their current buffers)."""
    a, b = ctypes.c_size_t(), ctypes.c_size_t()
    load_library().clblasAmdWorkspaceStats(ctypes.byref(a), ctypes.byref(b))
    return a.value, b.value


TILE_PARAMS = ("eff", "alone", "k0", "tail_extra", "deep_gain", "split_gain", "streamed_gain")


def tile_model_query(type_letter, M, N, K):
    """The tile choice for a plain product, without launching: dict with the chosen tile's index, its K
    ranges and tail slices, and per tile of the table its dimensions "BMxBNxBK" and the model's cost
    (None: not offered).  type_letter: "s", "d", "c" or "z"."""
    n = 16
    tile, splits, tail = ctypes.c_int(), ctypes.c_int(), ctypes.c_int()
    costs, dims = (ctypes.c_double * n)(), (ctypes.c_int * (3 * n))()
    nt = load_library().clblasAmdTileModelQuery(type_letter.encode(), M, N, K, ctypes.byref(tile), ctypes.byref(splits),
                                                ctypes.byref(tail), costs, dims, n)
    if nt < 0:
        raise ValueError("clblasAmdTileModelQuery refused (%r, %d, %d, %d)" % (type_letter, M, N, K))
    return {"tile": tile.value, "splits": splits.value, "tail_slices": tail.value,
            "tiles": ["%dx%dx%d" % tuple(dims[3 * i:3 * i + 3]) for i in range(nt)],
            "costs": [costs[i] if costs[i] >= 0 else None for i in range(nt)]}


def tile_model_param(type_letter, tile, name, value=None):
    """Reads (value is None) or sets parameter `name` (one of TILE_PARAMS) of tile `tile`'s choice model."""
    v = ctypes.c_double(0.0 if value is None else float(value))
    if load_library().clblasAmdTileModelParam(type_letter.encode(), tile, TILE_PARAMS.index(name), ctypes.byref(v),
                                              0 if value is None else 1) != 0:
        raise ValueError("no parameter %r of tile %d for type %r" % (name, tile, type_letter))
    return v.value


def trsm_poll_timeouts(reset=False):
    """Flag waits of the TRSM substitution leaf that gave up at their poll limit on the current GPU (0 for
    a working library); blocks until the device is idle enough to be read."""
    n = ctypes.c_uint(0)
    st = load_library().clblasAmdTrsmPollTimeouts(ctypes.byref(n), 1 if reset else 0)
    if st != 0:
        raise RuntimeError("clblasAmdTrsmPollTimeouts returned %d" % st)
    return n.value


def last_dispatch():
    """(description of the last GEMM kernel this thread launched, launches issued so far)."""
    buf = ctypes.create_string_buffer(512)
    n = load_library().clblasAmdLastDispatch(buf, 512)
    return buf.value.decode(), n


def reload_debug_env():
    """Makes the library read its CLBLAS_AMD_* debugging variables again (it reads them once)."""
    load_library().clblasAmdReloadDebugEnv()


def get_version():
    a, b, c = ctypes.c_uint(), ctypes.c_uint(), ctypes.c_uint()
    load_library().clblasGetVersion(ctypes.byref(a), ctypes.byref(b), ctypes.byref(c))
    return a.value, b.value, c.value


def sgemm(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    return load_library().clblasSgemm(int(order), int(transA), int(transB), M, N, K, alpha, _ptr(A), offA, lda,
                                      _ptr(B), offB, ldb, beta, _ptr(C), offC, ldc, _stream(stream))


def sgemm_noalloc(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """clblasSgemmNoAlloc: clblasSgemm on the library's fixed scratch array (allocates nothing)."""
    return load_library().clblasSgemmNoAlloc(int(order), int(transA), int(transB), M, N, K, alpha, _ptr(A), offA, lda,
                                             _ptr(B), offB, ldb, beta, _ptr(C), offC, ldc, _stream(stream))


def dgemm(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    return load_library().clblasDgemm(int(order), int(transA), int(transB), M, N, K, alpha, _ptr(A), offA, lda,
                                      _ptr(B), offB, ldb, beta, _ptr(C), offC, ldc, _stream(stream))


def cgemm(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """alpha / beta: Python complex; A, B, C: complex64 tensors (or device addresses)."""
    a, b = complex(alpha), complex(beta)
    return load_library().clblasCgemm(int(order), int(transA), int(transB), M, N, K, FloatComplex(a.real, a.imag),
                                      _ptr(A), offA, lda, _ptr(B), offB, ldb, FloatComplex(b.real, b.imag),
                                      _ptr(C), offC, ldc, _stream(stream))


def zgemm(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """alpha / beta: Python complex; A, B, C: complex128 tensors (or device addresses)."""
    a, b = complex(alpha), complex(beta)
    return load_library().clblasZgemm(int(order), int(transA), int(transB), M, N, K, DoubleComplex(a.real, a.imag),
                                      _ptr(A), offA, lda, _ptr(B), offB, ldb, DoubleComplex(b.real, b.imag),
                                      _ptr(C), offC, ldc, _stream(stream))


def strsm(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream=None):
    return load_library().clblasStrsm(int(order), int(side), int(uplo), int(transA), int(diag), M, N, alpha,
                                      _ptr(A), offA, lda, _ptr(B), offB, ldb, _stream(stream))


def dtrsm(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream=None):
    return load_library().clblasDtrsm(int(order), int(side), int(uplo), int(transA), int(diag), M, N, alpha,
                                      _ptr(A), offA, lda, _ptr(B), offB, ldb, _stream(stream))


def ctrsm(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream=None):
    """alpha: Python complex; A, B: complex64 tensors (or device addresses)."""
    return load_library().clblasCtrsm(int(order), int(side), int(uplo), int(transA), int(diag), M, N,
                                      _scalar("C", alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb, _stream(stream))


def ztrsm(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream=None):
    """alpha: Python complex; A, B: complex128 tensors (or device addresses)."""
    return load_library().clblasZtrsm(int(order), int(side), int(uplo), int(transA), int(diag), M, N,
                                      _scalar("Z", alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb, _stream(stream))


def _scalar(prefix, x):
    """Python number -> the by-value scalar type of the S/D/C/Z routine family."""
    if prefix == "C":
        z = complex(x)
        return FloatComplex(z.real, z.imag)
    if prefix == "Z":
        z = complex(x)
        return DoubleComplex(z.real, z.imag)
    return float(x)


def syrk(prefix, order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, stream=None):
    """clblas{prefix}syrk, prefix in "SDCZ" (src/clBLAS.h:8278-8503)."""
    fn = getattr(load_library(), "clblas%ssyrk" % prefix)
    return fn(int(order), int(uplo), int(transA), N, K, _scalar(prefix, alpha), _ptr(A), offA, lda,
              _scalar(prefix, beta), _ptr(C), offC, ldc, _stream(stream))


def trmm(prefix, order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, stream=None):
    """clblas{prefix}trmm, prefix in "SDCZ" (src/clBLAS.h:7696-7928)."""
    fn = getattr(load_library(), "clblas%strmm" % prefix)
    return fn(int(order), int(side), int(uplo), int(transA), int(diag), M, N, _scalar(prefix, alpha), _ptr(A), offA,
              lda, _ptr(B), offB, ldb, _stream(stream))


def symm(prefix, order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """clblas{prefix}symm, prefix in "SDCZ" (src/clBLAS.h:8897-9145)."""
    fn = getattr(load_library(), "clblas%ssymm" % prefix)
    return fn(int(order), int(side), int(uplo), M, N, _scalar(prefix, alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb,
              _scalar(prefix, beta), _ptr(C), offC, ldc, _stream(stream))


def syr2k(prefix, order, uplo, transAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """clblas{prefix}syr2k, prefix in "SDCZ" (src/clBLAS.h:8568-8819)."""
    fn = getattr(load_library(), "clblas%ssyr2k" % prefix)
    return fn(int(order), int(uplo), int(transAB), N, K, _scalar(prefix, alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb,
              _scalar(prefix, beta), _ptr(C), offC, ldc, _stream(stream))


def herk(prefix, order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, stream=None):
    """clblas{prefix}herk, prefix in "CZ"; alpha and beta real (src/clBLAS.h:9389-9476)."""
    fn = getattr(load_library(), "clblas%sherk" % prefix)
    return fn(int(order), int(uplo), int(transA), N, K, float(alpha), _ptr(A), offA, lda, float(beta), _ptr(C), offC,
              ldc, _stream(stream))


def her2k(prefix, order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """clblas{prefix}her2k, prefix in "CZ"; alpha complex, beta real (src/clBLAS.h:9545-9644)."""
    fn = getattr(load_library(), "clblas%sher2k" % prefix)
    return fn(int(order), int(uplo), int(trans), N, K, _scalar(prefix, alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb,
              float(beta), _ptr(C), offC, ldc, _stream(stream))


def hemm(prefix, order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, stream=None):
    """clblas{prefix}hemm, prefix in "CZ" (src/clBLAS.h:9224-9326)."""
    fn = getattr(load_library(), "clblas%shemm" % prefix)
    return fn(int(order), int(side), int(uplo), M, N, _scalar(prefix, alpha), _ptr(A), offA, lda, _ptr(B), offB, ldb,
              _scalar(prefix, beta), _ptr(C), offC, ldc, _stream(stream))
