"""Shared helpers for the parity tests: the reference tests' input generators and bounds,
restated (data generation only), and buffer layout arithmetic."""
import json
import math
import os

import numpy as np

ROW, COL = 0, 1
NOTRANS, TRANS, CONJ = 0, 1, 2
UPPER, LOWER = 0, 1
UNIT, NONUNIT = 0, 1
LEFT, RIGHT = 0, 1

GOLDEN = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "fixed_cases.json")


def golden_cases():
    with open(GOLDEN) as f:
        return json.load(f)


def mem_dims(order, trans, rows, cols):
    """(contiguous extent, number of strides) of a logical rows x cols op(X) in memory
    (reference: src/library/blas/generic/common.c:606-644)."""
    if (order == COL) == (trans == NOTRANS):
        return rows, cols
    return cols, rows


def buf_len(order, trans, rows, cols, off, ld):
    inner, outer = mem_dims(order, trans, rows, cols)
    return off + (outer - 1) * ld + inner


def elem_index(order, trans, r, c, off, ld):
    if (order == COL) == (trans == NOTRANS):
        return off + r + c * ld
    return off + r * ld + c


def logical_view(buf, order, trans, rows, cols, off, ld):
    """rows x cols numpy view (no copy) of op(X) inside a 1-D buffer."""
    isz = buf.itemsize
    if (order == COL) == (trans == NOTRANS):
        strides = (isz, ld * isz)
    else:
        strides = (ld * isz, isz)
    return np.lib.stride_tricks.as_strided(buf[off:], shape=(rows, cols), strides=strides, writeable=True)


def exact_int_limits(K, alpha, beta, dtype):
    """Bounds that make every partial sum exactly representable, so any summation order and
    any fma contraction gives identical bits (reference: src/tests/include/blas-random.h:60-93,
    test-limits.h:20-21)."""
    top = 2.0 ** 23 if dtype == np.float32 else 2.0 ** 52
    K = max(K, 2)
    ab = int(math.sqrt((K - 1) * top / (abs(alpha) * K * K))) if alpha != 0 else 100
    c = int(math.sqrt(top / (abs(beta) * K))) if beta != 0 else 100
    # keep products comfortably inside the mantissa whatever the rounding of sqrt
    return max(2, min(ab, 1 << 10)), max(2, min(c, 1 << 10))


EPS = {np.dtype(np.float32): 2.0 ** -24, np.dtype(np.float64): 2.0 ** -53,
       np.dtype(np.complex64): 2.0 ** -24, np.dtype(np.complex128): 2.0 ** -53}


def gemm_bound(K, mag, dtype, c=2.0):
    """|C - C_exact| <= c * (K+2) * eps * (|alpha| |A||B| + |beta||C|): the parity bound of the
    task with the unit roundoff; c=2 leaves room for both our result and the reference's."""
    return c * (K + 2) * EPS[np.dtype(dtype)] * mag + np.finfo(dtype).tiny


def cgemm_bound(K, mag, dtype, c=2.0):
    """Complex counterpart, applied to the real and to the imaginary part separately: each is a
    sum of 2K products (plus 2 + 2 in the epilogue), every term bounded in magnitude through
    mag = (|al.re|+|al.im|) (|A.re|+|A.im|)(|B.re|+|B.im|) + (|be.re|+|be.im|)(|C.re|+|C.im|)."""
    real = np.float32 if np.dtype(dtype) == np.dtype(np.complex64) else np.float64
    return c * (2 * K + 6) * EPS[np.dtype(dtype)] * mag + np.finfo(real).tiny


def golden_array(values, dtype):
    """A fixture buffer as a numpy array; complex buffers are stored as [re, im] pairs."""
    a = np.array(values, dtype=np.float64)
    if a.ndim == 2:
        a = a[:, 0] + 1j * a[:, 1]
    return a.astype(dtype)


def golden_scalar(v):
    return complex(v[0], v[1]) if isinstance(v, list) else v


# ---- the reference's own yardstick for TRSM --------------------------------------------------

TRSM_DELTA_0 = {np.dtype(np.float32): 2.0 ** -20, np.dtype(np.float64): 2.0 ** -50,
                np.dtype(np.complex64): 2.0 ** -20, np.dtype(np.complex128): 2.0 ** -50}


def trsm_ref_delta(dtype, side, uplo, transA, diag, alpha, abs_diag, abs_b):
    """Per-element bound of the reference's TRSM correctness test, trsmDelta
    (src/tests/correctness/trsm-delta.h:44-240), for selected right-hand sides.

    abs_diag: |a_pp|, length n (n = M for side left, N for right).  abs_b: |b| of the ORIGINAL
    right-hand sides, shape (nsel, n) (columns of B for left, rows for right).  Returns the bound
    in the same shape; the reference applies it to |reference BLAS result - clBLAS result|
    (complex: to the real and to the imaginary part, src/tests/include/matrix.h:372-400).

    Restated: s_p = |b_p / a_pp| * DELTA_0 * |alpha| (no division for a unit diagonal), summed
    along the direction of the substitution ("Gauss' method" part), plus a part for the block
    algorithm with block size 32 (16 for double complex): weights z = 1, 2, ... over the
    same-offset elements of the blocks the substitution has passed, times the block size.  For
    side right with a lower effective triangle the reference's block loop runs from block k/bs to
    (k + bs - 1)/bs, i.e. over at most one block (:216-218); that is kept as it is."""
    dtype = np.dtype(dtype)
    n = abs_b.shape[1]
    bs = 16 if dtype == np.dtype(np.complex128) else 32
    is_upper = (uplo == UPPER) == (transA == NOTRANS)
    forward = (side == LEFT) != is_upper
    s = abs_b.astype(np.float64)
    if diag == NONUNIT:
        s = s / abs_diag[None, :]
    s = s * (TRSM_DELTA_0[dtype] * abs(alpha))
    if not forward:
        s = s[:, ::-1]
    gauss = np.cumsum(s, axis=1)
    if not forward:
        gauss = gauss[:, ::-1]
    nb = (n + bs - 1) // bs
    g = np.zeros((abs_b.shape[0], nb * bs))
    g[:, :n] = gauss
    g = g.reshape(-1, nb, bs)
    if forward:
        blk = np.cumsum(np.cumsum(g, axis=1), axis=1)               # sum_{j<=pb} (pb+1-j) g[j]
    elif side == LEFT:
        blk = np.cumsum(np.cumsum(g[:, ::-1], axis=1), axis=1)[:, ::-1]   # sum_{j>=pb} (j-pb+1) g[j]
    else:
        blk = g.copy()
        blk[:, :, 0] = 0.0                                          # empty block range when k % bs == 0
    blk = blk.reshape(-1, nb * bs)[:, :n]
    return gauss + bs * blk


def trsm_ref_delta_loops(dtype, side, uplo, transA, diag, alpha, abs_diag, abs_b):
    """The same bound written as the reference's loops (one right-hand side at a time); used only
    to check the vectorised form above."""
    dtype = np.dtype(dtype)
    nsel, n = abs_b.shape
    bs = 16 if dtype == np.dtype(np.complex128) else 32
    is_upper = (uplo == UPPER) == (transA == NOTRANS)
    d0 = TRSM_DELTA_0[dtype]
    out = np.zeros((nsel, n))
    for q in range(nsel):
        delta = np.zeros(n)
        s = [(abs_b[q, p] / abs_diag[p] if diag == NONUNIT else abs_b[q, p]) * d0 * abs(alpha) for p in range(n)]
        if side == LEFT:
            order = range(n - 1, -1, -1) if is_upper else range(n)
        else:
            order = range(n) if is_upper else range(n - 1, -1, -1)
        prev = None
        for p in order:
            delta[p] = s[p] + (delta[prev] if prev is not None else 0.0)
            prev = p
        cl = np.zeros(n)
        for p in range(n):
            if side == LEFT:
                if is_upper:
                    j0, j1, z, zinc = p // bs, (n + bs - 1) // bs, 1, 1
                else:
                    j0, j1 = 0, p // bs + 1
                    z, zinc = j1 - j0, -1
            else:
                if is_upper:
                    j0, j1 = 0, p // bs + 1
                    z, zinc = j1 - j0, -1
                else:
                    j0, j1, z, zinc = p // bs, (p + bs - 1) // bs, 1, 1
            acc = 0.0
            for j in range(j0, j1):
                idx = j * bs + p % bs
                if idx >= n:
                    continue
                acc += z * delta[idx]
                z += zinc
            cl[p] = acc * bs
        out[q] = delta + cl
    return out
