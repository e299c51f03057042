"""Runs the C-ABI entry points on numpy buffers: upload, call, synchronise, download.
torch is used only to hold device memory."""
import os

import numpy as np
import torch

import clblas_amd


def _dev(x):
    return torch.from_numpy(x).cuda()


def gemm(order, tA, tB, M, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, tile=None):
    fn = {np.dtype(np.float32): clblas_amd.sgemm, np.dtype(np.float64): clblas_amd.dgemm,
          np.dtype(np.complex64): clblas_amd.cgemm, np.dtype(np.complex128): clblas_amd.zgemm}[C.dtype]
    dA, dB, dC = _dev(A), _dev(B), _dev(C)
    with _forced_tile(tile):
        st = fn(order, tA, tB, M, N, K, alpha, dA, offA, lda, dB, offB, ldb, beta, dC, offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def trsm(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb):
    fn = {np.dtype(np.float32): clblas_amd.strsm, np.dtype(np.float64): clblas_amd.dtrsm,
          np.dtype(np.complex64): clblas_amd.ctrsm, np.dtype(np.complex128): clblas_amd.ztrsm}[B.dtype]
    dA, dB = _dev(A), _dev(B)
    st = fn(order, side, uplo, tA, diag, M, N, alpha, dA, offA, lda, dB, offB, ldb)
    torch.cuda.synchronize()
    return st, dB.cpu().numpy()


class debug_env:
    """Sets CLBLAS_AMD_* debugging variables for the calls inside the block.  The library reads
    its environment once, so it is told to read it again on the way in and on the way out."""

    def __init__(self, **kv):
        self.kv = {k: str(v) for k, v in kv.items() if v is not None}

    def __enter__(self):
        if self.kv:
            os.environ.update(self.kv)
            clblas_amd.reload_debug_env()

    def __exit__(self, *a):
        if self.kv:
            for k in self.kv:
                os.environ.pop(k, None)
            clblas_amd.reload_debug_env()


def _forced_tile(tile):
    return debug_env(CLBLAS_AMD_GEMM_TILE=tile)


_PREFIX = {np.dtype(np.float32): "S", np.dtype(np.float64): "D", np.dtype(np.complex64): "C",
           np.dtype(np.complex128): "Z"}


def syrk(order, uplo, tA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, tile=None):
    dA, dC = _dev(A), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.syrk(_PREFIX[C.dtype], order, uplo, tA, N, K, alpha, dA, offA, lda, beta, dC, offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def trmm(order, side, uplo, tA, diag, M, N, alpha, A, offA, lda, B, offB, ldb, tile=None):
    dA, dB = _dev(A), _dev(B)
    with _forced_tile(tile):
        st = clblas_amd.trmm(_PREFIX[B.dtype], order, side, uplo, tA, diag, M, N, alpha, dA, offA, lda, dB, offB, ldb)
        torch.cuda.synchronize()
    return st, dB.cpu().numpy()


def symm(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, tile=None):
    dA, dB, dC = _dev(A), _dev(B), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.symm(_PREFIX[C.dtype], order, side, uplo, M, N, alpha, dA, offA, lda, dB, offB, ldb, beta, dC,
                             offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def syr2k(order, uplo, tAB, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, tile=None):
    dA, dB, dC = _dev(A), _dev(B), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.syr2k(_PREFIX[C.dtype], order, uplo, tAB, N, K, alpha, dA, offA, lda, dB, offB, ldb, beta, dC,
                              offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def herk(order, uplo, tA, N, K, alpha, A, offA, lda, beta, C, offC, ldc, tile=None):
    dA, dC = _dev(A), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.herk(_PREFIX[C.dtype], order, uplo, tA, N, K, alpha, dA, offA, lda, beta, dC, offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def her2k(order, uplo, trans, N, K, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, tile=None):
    dA, dB, dC = _dev(A), _dev(B), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.her2k(_PREFIX[C.dtype], order, uplo, trans, N, K, alpha, dA, offA, lda, dB, offB, ldb, beta,
                              dC, offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()


def hemm(order, side, uplo, M, N, alpha, A, offA, lda, B, offB, ldb, beta, C, offC, ldc, tile=None):
    dA, dB, dC = _dev(A), _dev(B), _dev(C)
    with _forced_tile(tile):
        st = clblas_amd.hemm(_PREFIX[C.dtype], order, side, uplo, M, N, alpha, dA, offA, lda, dB, offB, ldb, beta, dC,
                             offC, ldc)
        torch.cuda.synchronize()
    return st, dC.cpu().numpy()
