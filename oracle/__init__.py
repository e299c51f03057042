"""numpy-facing loader for the CPU oracle (oracle/liboracle.so, oracle/_ref/libnaive_ref.so).

TEST INFRASTRUCTURE ONLY: imported by tests/, by __graft_entry__.smoke() and by the
cpu_baseline leg of bench.py -- never by the product package (clblas_amd).

All matrices are 1-D numpy buffers addressed exactly as the C API addresses them
(element offsets and leading dimensions), so the tests read like the reference's own.
"""
import ctypes
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "liboracle.so")
REF_LIB_PATH = os.path.join(_HERE, "_ref", "libnaive_ref.so")

_lib = None
_ref = None

_sz = ctypes.c_size_t
_i = ctypes.c_int
_vp = ctypes.c_void_p
_u64 = ctypes.c_uint64


def build(verbose=False):
    """Compiles liboracle.so and, if the reference tree is present, _ref/libnaive_ref.so."""
    res = subprocess.run(["make", "-C", _HERE, "-B", "all"], capture_output=True, text=True)
    if res.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + res.stdout + res.stderr)
    if verbose:
        print(res.stdout.strip())


def lib():
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            build()
        L = ctypes.CDLL(LIB_PATH)
        for name, real in (("oracle_sgemm", ctypes.c_float), ("oracle_dgemm", ctypes.c_double)):
            f = getattr(L, name)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _sz, real, _vp, _sz, _sz, _vp, _sz, _sz, real, _vp, _sz, _sz]
        for name, real in (("oracle_sgemm_exact", ctypes.c_float), ("oracle_dgemm_exact", ctypes.c_double)):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_i, _i, _sz, real, _vp, _sz, _vp, _sz, real, _vp, _sz, _sz, _vp, _vp, _vp, _vp]
        for name in ("oracle_cgemm", "oracle_zgemm"):
            f = getattr(L, name)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp, _vp, _sz, _sz]
        for name in ("oracle_cgemm_exact", "oracle_zgemm_exact"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_i, _i, _i, _i, _sz, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _vp, _vp]
        for name, real in (("oracle_strsm_naive", ctypes.c_float), ("oracle_dtrsm_naive", ctypes.c_double),
                           ("oracle_strsm_blocked", ctypes.c_float), ("oracle_dtrsm_blocked", ctypes.c_double)):
            f = getattr(L, name)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _i, _i, _sz, _sz, real, _vp, _sz, _sz, _vp, _sz, _sz]
        for name in ("oracle_ctrsm_naive", "oracle_ztrsm_naive"):
            f = getattr(L, name)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz]
        for t in "sdcz":
            f = getattr(L, "oracle_%ssyrk" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _vp, _sz, _sz]
            f = getattr(L, "oracle_%strmm" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz]
            f = getattr(L, "oracle_%ssymm" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp, _vp, _sz, _sz]
            f = getattr(L, "oracle_%ssyr2k" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp, _vp, _sz, _sz]
        for t, real in (("c", ctypes.c_float), ("z", ctypes.c_double)):
            f = getattr(L, "oracle_%sherk" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, real, _vp, _sz, _sz, real, _vp, _sz, _sz]
            f = getattr(L, "oracle_%sher2k" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, real, _vp, _sz, _sz]
            f = getattr(L, "oracle_%shemm" % t)
            f.restype = _i
            f.argtypes = [_i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp, _vp, _sz, _sz]
        L.oracle_check_gemm.restype = _i
        L.oracle_check_gemm.argtypes = [_i, _i, _i, _sz, _sz, _sz, _i, _sz, _sz, _sz, _i, _sz, _sz, _sz, _i, _sz,
                                        _sz, _sz]
        L.oracle_check_trsm.restype = _i
        L.oracle_check_trsm.argtypes = [_i, _i, _i, _sz, _sz, _i, _sz, _sz, _sz, _i, _sz, _sz, _sz]
        L.oracle_num_threads.restype = _i
        for name in ("oracle_fill_uniform_f32", "oracle_fill_uniform_f64", "oracle_fill_normal_f32",
                     "oracle_fill_normal_f64"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_vp, _sz, _u64]
        for name in ("oracle_fill_int_f32", "oracle_fill_int_f64"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_vp, _sz, _u64, ctypes.c_uint32]
        for name in ("oracle_fill_tri_f32", "oracle_fill_tri_f64"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_vp, _sz, _sz, _i, _i, _u64]
        _lib = L
    return _lib


def ref_lib():
    """The reference's own naive BLAS (compiled from the reference tree), or None if absent."""
    global _ref
    if _ref is None:
        if not os.path.exists(REF_LIB_PATH):
            return None
        L = ctypes.CDLL(REF_LIB_PATH)
        for name, real in (("ref_naive_sgemm", ctypes.c_float), ("ref_naive_dgemm", ctypes.c_double)):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_i, _i, _i, _sz, _sz, _sz, real, _vp, _sz, _vp, _sz, real, _vp, _sz]
        for name in ("ref_naive_cgemm", "ref_naive_zgemm"):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_i, _i, _i, _sz, _sz, _sz, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz]
        L.ref_naive_syrk.restype = None
        L.ref_naive_syrk.argtypes = [_i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _vp, _vp, _sz]
        L.ref_naive_syr2k.restype = None
        L.ref_naive_syr2k.argtypes = [_i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _vp, _sz, _vp, _vp, _sz]
        L.ref_naive_trmm.restype = None
        L.ref_naive_trmm.argtypes = [_i, _i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _vp, _sz]
        L.ref_naive_trsm.restype = None
        L.ref_naive_trsm.argtypes = [_i, _i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _vp, _sz]
        for name, real in (("ref_naive_strsm", ctypes.c_float), ("ref_naive_dtrsm", ctypes.c_double)):
            f = getattr(L, name)
            f.restype = None
            f.argtypes = [_i, _i, _i, _i, _i, _sz, _sz, real, _vp, _sz, _vp, _sz]
        _ref = L
    return _ref


def _p(a):
    return None if a is None else a.ctypes.data_as(_vp)


def _real(a):
    return "s" if a.dtype == np.float32 else "d"


def num_threads():
    return lib().oracle_num_threads()


def _is_complex(a):
    return a.dtype in (np.complex64, np.complex128)


def _scalar(x, dtype):
    """(re, im) of a Python complex as a 2-element real array matching complex `dtype`."""
    z = complex(x)
    return np.array([z.real, z.imag], dtype=np.float32 if dtype == np.complex64 else np.float64)


def gemm(order, transA, transB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    """In-place on C (1-D buffer). Returns the clblasStatus the reference would return.
    complex64 / complex128 buffers select the complex routines (alpha, beta: Python complex)."""
    ref = C if C is not None else (A if A is not None else B)
    if _is_complex(ref):
        f = lib().oracle_cgemm if ref.dtype == np.complex64 else lib().oracle_zgemm
        al, be = _scalar(alpha, ref.dtype), _scalar(beta, ref.dtype)
        return f(int(order), int(transA), int(transB), M, N, K, _p(al), _p(A), offA, lda, _p(B), offB, ldb, _p(be),
                 _p(C), offC, ldc)
    f = lib().oracle_sgemm if ref.dtype == np.float32 else lib().oracle_dgemm
    return f(int(order), int(transA), int(transB), M, N, K, alpha, _p(A), offA, lda, _p(B), offB, ldb, beta, _p(C),
             offC, ldc)


def gemm_exact(transA, transB, K, alpha, A, lda, B, ldb, beta, C, ldc, rows, cols):
    """Column-major; A/B/C buffers start at element (0,0).  Returns (exact, magnitude) in
    float64 for the listed elements: magnitude = |alpha| sum|a b| + |beta c|."""
    rows = np.ascontiguousarray(rows, dtype=np.int64)
    cols = np.ascontiguousarray(cols, dtype=np.int64)
    mag = np.empty(rows.size, dtype=np.float64)
    if _is_complex(A):
        # transA / transB: 0 none, 1 transpose, 2 conjugate transpose; exact is complex128.
        ex = np.empty(2 * rows.size, dtype=np.float64)
        f = lib().oracle_cgemm_exact if A.dtype == np.complex64 else lib().oracle_zgemm_exact
        al, be = _scalar(alpha, A.dtype), _scalar(beta, A.dtype)
        f(int(transA != 0), int(transA == 2), int(transB != 0), int(transB == 2), K, _p(al), _p(A), lda, _p(B), ldb,
          _p(be), _p(C), ldc, rows.size, _p(rows), _p(cols), _p(ex), _p(mag))
        return ex.view(np.complex128), mag
    exact = np.empty(rows.size, dtype=np.float64)
    f = lib().oracle_sgemm_exact if A.dtype == np.float32 else lib().oracle_dgemm_exact
    f(int(bool(transA)), int(bool(transB)), K, alpha, _p(A), lda, _p(B), ldb, beta, _p(C), ldc, rows.size, _p(rows),
      _p(cols), _p(exact), _p(mag))
    return exact, mag


def trsm_naive(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    ref = B if B is not None else A
    if _is_complex(ref):
        f = lib().oracle_ctrsm_naive if ref.dtype == np.complex64 else lib().oracle_ztrsm_naive
        return f(int(order), int(side), int(uplo), int(transA), int(diag), M, N, _p(_scalar(alpha, ref.dtype)),
                 _p(A), offA, lda, _p(B), offB, ldb)
    f = lib().oracle_strsm_naive if ref.dtype == np.float32 else lib().oracle_dtrsm_naive
    return f(int(order), int(side), int(uplo), int(transA), int(diag), M, N, alpha, _p(A), offA, lda, _p(B), offB,
             ldb)


def trsm_blocked(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    ref = B if B is not None else A
    f = lib().oracle_strsm_blocked if ref.dtype == np.float32 else lib().oracle_dtrsm_blocked
    return f(int(order), int(side), int(uplo), int(transA), int(diag), M, N, alpha, _p(A), offA, lda, _p(B), offB,
             ldb)


_PREFIX = {np.dtype(np.float32): "s", np.dtype(np.float64): "d", np.dtype(np.complex64): "c",
           np.dtype(np.complex128): "z"}


def prefix(a):
    """Routine-family letter (s, d, c, z) of a buffer's dtype."""
    return _PREFIX[a.dtype]


def _sc(x, ref):
    """alpha / beta as the array the level-3 routines take by address."""
    if _is_complex(ref):
        return _scalar(x, ref.dtype)
    return np.array([x], dtype=ref.dtype)


def syrk(order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc):
    ref = C if C is not None else A
    al, be = _sc(alpha, ref), _sc(beta, ref)
    return getattr(lib(), "oracle_%ssyrk" % prefix(ref))(int(order), int(uplo), int(transA), N, K, _p(al), _p(A), offA,
                                                         lda, _p(be), _p(C), offC, ldc)


def trmm(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    ref = B if B is not None else A
    al = _sc(alpha, ref)
    return getattr(lib(), "oracle_%strmm" % prefix(ref))(int(order), int(side), int(uplo), int(transA), int(diag), M, N,
                                                         _p(al), _p(A), offA, lda, _p(B), offB, ldb)


def symm(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    ref = C if C is not None else (A if A is not None else B)
    al, be = _sc(alpha, ref), _sc(beta, ref)
    return getattr(lib(), "oracle_%ssymm" % prefix(ref))(int(order), int(side), int(uplo), M, N, _p(al), _p(A), offA,
                                                         lda, _p(B), offB, ldb, _p(be), _p(C), offC, ldc)


def syr2k(order, uplo, transAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    ref = C if C is not None else (A if A is not None else B)
    al, be = _sc(alpha, ref), _sc(beta, ref)
    return getattr(lib(), "oracle_%ssyr2k" % prefix(ref))(int(order), int(uplo), int(transAB), N, K, _p(al), _p(A),
                                                          offA, lda, _p(B), offB, ldb, _p(be), _p(C), offC, ldc)


def herk(order, uplo, transA, N, K, alpha, A, offA, lda, beta, C, offC, ldc):
    """alpha, beta real; A, C complex64 / complex128."""
    ref = C if C is not None else A
    return getattr(lib(), "oracle_%sherk" % prefix(ref))(int(order), int(uplo), int(transA), N, K, float(alpha), _p(A),
                                                         offA, lda, float(beta), _p(C), offC, ldc)


def her2k(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    """alpha complex, beta real."""
    ref = C if C is not None else (A if A is not None else B)
    return getattr(lib(), "oracle_%sher2k" % prefix(ref))(int(order), int(uplo), int(trans), N, K,
                                                          _p(_sc(alpha, ref)), _p(A), offA, lda, _p(B), offB, ldb,
                                                          float(beta), _p(C), offC, ldc)


def hemm(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc):
    ref = C if C is not None else (A if A is not None else B)
    al, be = _sc(alpha, ref), _sc(beta, ref)
    return getattr(lib(), "oracle_%shemm" % prefix(ref))(int(order), int(side), int(uplo), M, N, _p(al), _p(A), offA,
                                                         lda, _p(B), offB, ldb, _p(be), _p(C), offC, ldc)


def ref_syr2k(order, uplo, transAB, N, K, alpha, A, lda, B, ldb, beta, C, ldc):
    """Reference naive syr2k (no offsets)."""
    al, be = _sc(alpha, C), _sc(beta, C)
    ref_lib().ref_naive_syr2k("sdcz".index(prefix(C)), int(order), int(uplo), int(transAB), N, K, _p(al), _p(A), lda,
                              _p(B), ldb, _p(be), _p(C), ldc)


def ref_syrk(order, uplo, transA, N, K, alpha, A, lda, beta, C, ldc):
    """Reference naive syrk (no offsets)."""
    al, be = _sc(alpha, C), _sc(beta, C)
    ref_lib().ref_naive_syrk("sdcz".index(prefix(C)), int(order), int(uplo), int(transA), N, K, _p(al), _p(A), lda,
                             _p(be), _p(C), ldc)


def ref_trmm(order, side, uplo, transA, diag, M, N, alpha, A, lda, B, ldb):
    """Reference naive trmm (no offsets)."""
    al = _sc(alpha, B)
    ref_lib().ref_naive_trmm("sdcz".index(prefix(B)), int(order), int(side), int(uplo), int(transA), int(diag), M, N,
                             _p(al), _p(A), lda, _p(B), ldb)


def check_gemm(order, transA, transB, M, N, K, haveA, offA, lda, memA, haveB, offB, ldb, memB, haveC, offC, ldc,
               memC):
    return lib().oracle_check_gemm(int(order), int(transA), int(transB), M, N, K, int(haveA), offA, lda, memA,
                                   int(haveB), offB, ldb, memB, int(haveC), offC, ldc, memC)


def check_trsm(order, side, transA, M, N, haveA, offA, lda, memA, haveB, offB, ldb, memB):
    return lib().oracle_check_trsm(int(order), int(side), int(transA), M, N, int(haveA), offA, lda, memA,
                                   int(haveB), offB, ldb, memB)


def ref_gemm(order, transA, transB, M, N, K, alpha, A, lda, B, ldb, beta, C, ldc):
    """Reference naive gemm (no offsets: pass views that start at the first element)."""
    if _is_complex(C):
        f = ref_lib().ref_naive_cgemm if C.dtype == np.complex64 else ref_lib().ref_naive_zgemm
        al, be = _scalar(alpha, C.dtype), _scalar(beta, C.dtype)
        f(int(order), int(transA), int(transB), M, N, K, _p(al), _p(A), lda, _p(B), ldb, _p(be), _p(C), ldc)
        return
    f = ref_lib().ref_naive_sgemm if C.dtype == np.float32 else ref_lib().ref_naive_dgemm
    f(int(order), int(transA), int(transB), M, N, K, alpha, _p(A), lda, _p(B), ldb, beta, _p(C), ldc)


def ref_trsm(order, side, uplo, transA, diag, M, N, alpha, A, lda, B, ldb):
    if _is_complex(B):
        ref_lib().ref_naive_trsm(2 if B.dtype == np.complex64 else 3, int(order), int(side), int(uplo), int(transA),
                                 int(diag), M, N, _p(_scalar(alpha, B.dtype)), _p(A), lda, _p(B), ldb)
        return
    f = ref_lib().ref_naive_strsm if B.dtype == np.float32 else ref_lib().ref_naive_dtrsm
    f(int(order), int(side), int(uplo), int(transA), int(diag), M, N, alpha, _p(A), lda, _p(B), ldb)


_TYPE_CODE = {np.dtype(np.float32): 0, np.dtype(np.float64): 1, np.dtype(np.complex64): 2, np.dtype(np.complex128): 3}


def trsm_ref_inputs(dtype, order, side, uplo, diag, M, N, alpha, offA, lda, offB, ldb, seed):
    """(A, B) buffers of the reference TRSM test's input family (oracle_trsm_ref_inputs): NaN in
    every element the routine must not read, B already divided by alpha where |alpha| != 1."""
    dtype = np.dtype(dtype)
    limA = M if side == 0 else N
    rows_b, cols_b = (M, N) if order == 1 else (N, M)   # (contiguous extent, strides) of B in memory
    lenA = offA + lda * limA
    lenB = offB + ldb * cols_b
    assert lda >= limA and ldb >= rows_b
    A = np.empty(lenA, dtype=dtype)
    B = np.empty(lenB, dtype=dtype)
    al = np.array([complex(alpha).real, complex(alpha).imag], dtype=np.float64)
    f = lib().oracle_trsm_ref_inputs
    f.restype = None
    f.argtypes = [_i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _sz, _vp, _sz, _sz, _sz, _u64]
    f(_TYPE_CODE[dtype], int(order), int(side), int(uplo), int(diag), M, N, _p(al), _p(A), offA, lda, lenA, _p(B), offB,
      ldb, lenB, seed)
    return A, B


def trsm_hp(order, side, uplo, transA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, rhs):
    """Solutions of the right-hand sides `rhs` (columns of B for side left, rows for right) by
    substitution in long double, rounded to double: array (len(rhs), n), float64 or complex128."""
    n = M if side == 0 else N
    rhs = np.ascontiguousarray(rhs, dtype=np.uintp)
    X = np.empty((len(rhs), n), dtype=np.complex128)
    al = np.array([complex(alpha).real, complex(alpha).imag], dtype=np.float64)
    f = lib().oracle_trsm_hp
    f.restype = _i
    f.argtypes = [_i, _i, _i, _i, _i, _i, _sz, _sz, _vp, _vp, _sz, _sz, _vp, _sz, _sz, _vp, _sz, _vp]
    st = f(_TYPE_CODE[np.dtype(B.dtype)], int(order), int(side), int(uplo), int(transA), int(diag), M, N, _p(al), _p(A),
           offA, lda, _p(B), offB, ldb, _p(rhs), len(rhs), _p(X))
    assert st == 0, st
    return X if _is_complex(B) else np.ascontiguousarray(X.real)


# ---- seeded generators -------------------------------------------------------------------

def uniform(n, seed, dtype=np.float32):
    if dtype in (np.complex64, np.complex128):  # re and im drawn as 2n reals
        real = np.float32 if dtype == np.complex64 else np.float64
        return uniform(2 * n, seed, real).view(dtype)
    x = np.empty(n, dtype=dtype)
    (lib().oracle_fill_uniform_f32 if dtype == np.float32 else lib().oracle_fill_uniform_f64)(_p(x), n, seed)
    return x


def normal(n, seed, dtype=np.float64):
    x = np.empty(n, dtype=dtype)
    (lib().oracle_fill_normal_f32 if dtype == np.float32 else lib().oracle_fill_normal_f64)(_p(x), n, seed)
    return x


def integers(n, seed, limit, dtype=np.float32):
    if dtype in (np.complex64, np.complex128):  # Gaussian integers
        real = np.float32 if dtype == np.complex64 else np.float64
        return integers(2 * n, seed, limit, real).view(dtype)
    x = np.empty(n, dtype=dtype)
    (lib().oracle_fill_int_f32 if dtype == np.float32 else lib().oracle_fill_int_f64)(_p(x), n, seed, limit)
    return x


def triangular(n, ld, lower, seed, dtype=np.float64, poison_diag=False, tail=0):
    """ld*n (+tail) element buffer holding a conditioned triangular matrix, NaN elsewhere in the square."""
    a = np.full(ld * n + tail, np.nan, dtype=dtype)
    (lib().oracle_fill_tri_f32 if dtype == np.float32 else lib().oracle_fill_tri_f64)(_p(a), n, ld, int(lower),
                                                                                    int(poison_diag), seed)
    return a
