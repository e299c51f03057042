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
