"""Pins the BLAS-1 part of the oracle: OpenBLAS, exact cases, ulp bounds between fused and unfused forms."""
import ctypes as C

import numpy as np
import pytest

from oracle_binding import ptr, rand_f64


def scaled_ulp(a, b, alpha, x, y0):
    """max |a - b| in units of the ulp of the largest of |alpha*x|, |y0| and the results, per element."""
    scale = np.maximum(np.maximum(np.abs(alpha * x), np.abs(y0)), np.maximum(np.abs(a), np.abs(b)))
    return float(np.max(np.abs(a - b) / np.spacing(scale)))


def test_daxpy_vs_openblas_within_one_ulp(orc, openblas):
    n, alpha = 100003, 0.7
    x, y0 = rand_f64(n, 1), rand_f64(n, 2)
    ref, fused, unfused = y0.copy(), y0.copy(), y0.copy()
    assert openblas.orc_openblas_daxpy(n, alpha, ptr(x), 1, ptr(ref), 1) == 0
    orc.orc_daxpy(n, alpha, ptr(x), 1, ptr(fused), 1)
    orc.orc_daxpy_mul_add(n, alpha, ptr(x), 1, ptr(unfused), 1)
    # One rounding (fma) against two (multiply, then add): the results differ by at most half an ulp of the
    # product plus one ulp of the sum.  Under cancellation the sum is tiny, so the distance is measured in ulps of
    # the larger operand, not of the result.
    assert scaled_ulp(fused, unfused, alpha, x, y0) <= 1.5
    # OpenBLAS picks one of the two forms per CPU kernel; it must coincide with one of them bit for bit ...
    d_f = orc.orc_max_ulp_f64(ptr(fused), ptr(ref), n)
    d_u = orc.orc_max_ulp_f64(ptr(unfused), ptr(ref), n)
    assert min(d_f, d_u) == 0
    # ... and be within the contract's 1 ulp (operand-scaled) of the fused form the GPU kernel uses
    assert scaled_ulp(fused, ref, alpha, x, y0) <= 1.5


def test_daxpy_exact_cases(orc):
    n = 1000
    x, y0 = rand_f64(n, 3), rand_f64(n, 4)
    y = y0.copy()
    orc.orc_daxpy(n, 0.5, ptr(x), 1, ptr(y), 1)  # power-of-two alpha: product exact, one rounding
    assert np.array_equal(y, 0.5 * x + y0)
    y = y0.copy()
    orc.orc_daxpy(n, 0.0, ptr(x), 1, ptr(y), 1)
    assert np.array_equal(y, y0)
    y = y0.copy()
    orc.orc_daxpy(0, 1.0, ptr(x), 1, ptr(y), 1)
    assert np.array_equal(y, y0)


def test_daxpy_strides_and_tiles(orc, openblas):
    n, incx, incy = 777, 3, -2
    x, y0 = rand_f64(n * 3, 5), rand_f64(n * 2, 6)
    ref, got = y0.copy(), y0.copy()
    assert openblas.orc_openblas_daxpy(n, 1.25, ptr(x), incx, ptr(ref), incy) == 0
    orc.orc_daxpy(n, 1.25, ptr(x), incx, ptr(got), incy)
    assert orc.orc_max_ulp_f64(ptr(got), ptr(ref), n * 2) <= 1 or \
        scaled_ulp(got[::2][:n], ref[::2][:n], 1.25, x[::3][:n][::-1], y0[::2][:n]) <= 1.5
    # tiling changes nothing: each element is touched once
    for T in (1, 100, 777, 5000):
        a, b = y0.copy(), y0.copy()
        orc.orc_daxpy(n, 0.7, ptr(x), 1, ptr(a), 1)
        tiles = orc.orc_daxpy_tiled(T, n, 0.7, ptr(x), 1, ptr(b), 1)
        assert tiles == -(-n // T) and np.array_equal(a, b)


def test_ddot(orc, openblas):
    n = 1 << 20
    x, y = rand_f64(n, 7), rand_f64(n, 8)
    exact = float(orc.orc_ddot_longdouble(n, ptr(x), 1, ptr(y), 1))
    bound = 1e-13 * float(np.linalg.norm(x) * np.linalg.norm(y))
    ob = C.c_double(0)
    assert openblas.orc_openblas_ddot(n, ptr(x), 1, ptr(y), 1, C.byref(ob)) == 0
    assert abs(ob.value - exact) <= bound
    for T in (4096, 100000, n, 3 * n):
        r = C.c_double(0.0)
        tiles = orc.orc_ddot_tiled(T, n, ptr(x), 1, ptr(y), 1, C.byref(r))
        assert tiles == -(-n // T)
        assert abs(r.value - exact) <= bound
    # the reference adds into *result (ddot.cpp:431)
    r = C.c_double(10.0)
    orc.orc_ddot_tiled(4096, n, ptr(x), 1, ptr(y), 1, C.byref(r))
    assert abs(r.value - 10.0 - exact) <= bound
    ones = np.ones(12345)
    r = C.c_double(0.0)
    orc.orc_ddot_tiled(1000, 12345, ptr(ones), 1, ptr(ones), 1, C.byref(r))
    assert r.value == 12345.0
    # permutation invariance within the bound
    p = np.random.default_rng(0).permutation(n)
    xp, yp = x[p].copy(), y[p].copy()
    r = C.c_double(0.0)
    orc.orc_ddot_tiled(8192, n, ptr(xp), 1, ptr(yp), 1, C.byref(r))
    assert abs(r.value - exact) <= bound
    # strided, negative increment pairs element i of x with element i of y counted from the far end
    m = 1000
    xs, ys = rand_f64(2 * m, 9), rand_f64(3 * m, 10)
    ld = float(orc.orc_ddot_longdouble(m, ptr(xs), 2, ptr(ys), -3))
    expect = float(np.dot(xs[::2][:m].astype(np.longdouble), ys[::3][:m][::-1].astype(np.longdouble)))
    assert abs(ld - expect) < 1e-12
