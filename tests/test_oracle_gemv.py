"""Pins the oracle's dgemv (long-double brute force and the reference's tiled schedule, dgemv.cpp:41-126) against
OpenBLAS, closed forms, exact integer data and the already pinned GEMM brute force, and its BLAS-2 model restatement
(ModelLvl2.cpp:89-259) against hand-evaluated values."""
import ctypes as C

import numpy as np
import pytest

from oracle_binding import make_table, orc_link, orc_problem, ptr, rand_f64

TILE = 1024 * 1024 * 8


def span(n, inc):
    return (n - 1) * abs(inc) + 1


@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("incx,incy", [(1, 1), (2, 3), (-1, 1), (1, -2), (-3, -1)])
def test_bruteforce_matches_openblas(orc, openblas, ta, incx, incy):
    M, N, lda = 137, 91, 150
    lx, ly = (N, M) if ta == "N" else (M, N)
    A, x, y0 = rand_f64(lda * N, 1), rand_f64(span(lx, incx), 2), rand_f64(span(ly, incy), 3)
    got, ref = y0.copy(), y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 1.23, ptr(A), lda, ptr(x), incx, 0.77, ptr(got), incy)
    assert openblas.orc_openblas_dgemv(ta.encode(), M, N, 1.23, ptr(A), lda, ptr(x), incx, 0.77, ptr(ref), incy) == 0
    scale = 1.23 * np.linalg.norm(A) * np.linalg.norm(x) + 0.77 * np.linalg.norm(y0)
    assert np.linalg.norm(got - ref) / scale < 1e-15
    touched = np.zeros(y0.size, dtype=bool)
    touched[::abs(incy)] = True
    assert np.array_equal(got[~touched], y0[~touched])  # the gaps of a strided y are not written


def test_closed_forms(orc):
    n = 64
    eye = np.eye(n).ravel()
    x, y0 = rand_f64(n, 4), rand_f64(n, 5)
    for ta in (b"N", b"T"):
        y = y0.copy()
        orc.orc_dgemv_bruteforce(ta, n, n, 2.0, ptr(eye), n, ptr(x), 1, 0.5, ptr(y), 1)
        assert np.array_equal(y, 2.0 * x + 0.5 * y0)  # exact: powers of two
    M, N = 37, 53
    ones = np.ones(M * N)
    y = np.full(M, 3.0)
    orc.orc_dgemv_bruteforce(b"N", M, N, 2.0, ptr(ones), M, ptr(np.ones(N)), 1, 4.0, ptr(y), 1)
    assert np.array_equal(y, np.full(M, 2.0 * N + 12.0))
    y = np.full(N, 3.0)
    orc.orc_dgemv_bruteforce(b"T", M, N, 2.0, ptr(ones), M, ptr(np.ones(M)), 1, 4.0, ptr(y), 1)
    assert np.array_equal(y, np.full(N, 2.0 * M + 12.0))
    # beta = 0 overwrites whatever y held, NaN included; alpha = 0 only scales
    y = np.full(M, np.nan)
    orc.orc_dgemv_bruteforce(b"N", M, N, 1.0, ptr(ones), M, ptr(np.ones(N)), 1, 0.0, ptr(y), 1)
    assert np.array_equal(y, np.full(M, float(N)))
    y = y0[:M].copy()
    orc.orc_dgemv_bruteforce(b"N", M, N, 0.0, ptr(np.full(M * N, np.nan)), M, ptr(np.ones(N)), 1, 0.5, ptr(y), 1)
    assert np.array_equal(y, 0.5 * y0[:M])  # BLAS: A and x are not referenced when alpha == 0
    # empty problems leave y alone
    y = y0.copy()
    orc.orc_dgemv_bruteforce(b"N", 0, 5, 1.0, ptr(ones), 1, ptr(x), 1, 0.0, ptr(y), 1)
    orc.orc_dgemv_bruteforce(b"N", 5, 0, 1.0, ptr(ones), 5, ptr(x), 1, 0.0, ptr(y), 1)
    assert np.array_equal(y, y0)


@pytest.mark.parametrize("ta", ["N", "T"])
def test_gemv_is_a_one_column_gemm(orc, ta):
    """The GEMM brute force is pinned separately; a matrix-vector product is its N = 1 case, bit for bit."""
    M, N, lda = 83, 59, 90
    lx, ly = (N, M) if ta == "N" else (M, N)
    A, x, y0 = rand_f64(lda * N, 6), rand_f64(lx, 7), rand_f64(ly, 8)
    y, c = y0.copy(), y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 1.1, ptr(A), lda, ptr(x), 1, 0.9, ptr(y), 1)
    orc.orc_dgemm_bruteforce(ta.encode(), b"N", ly, 1, lx, 1.1, ptr(A), lda, ptr(x), lx, 0.9, ptr(c), ly)
    assert np.array_equal(y, c)


@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("T", [16, 50, 64, 128, 1000])
@pytest.mark.parametrize("beta", [0.0, 3.0])
def test_tiled_schedule_exact_on_integers(orc, ta, T, beta):
    """Integer-valued data: every summation order gives the same bits, so the tiled schedule (beta on the first
    subkernel of a y tile, 1 afterwards; ragged edge tiles) must reproduce the untiled product exactly."""
    M, N, lda = 173, 131, 180
    lx, ly = (N, M) if ta == "N" else (M, N)
    rng = np.random.default_rng(T)
    A = rng.integers(-8, 9, lda * N).astype(np.float64)
    x = rng.integers(-8, 9, span(lx, 2)).astype(np.float64)
    y0 = rng.integers(-8, 9, span(ly, -3)).astype(np.float64)
    ref = y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 2.0, ptr(A), lda, ptr(x), 2, beta, ptr(ref), -3)
    start = y0.copy()
    if beta == 0.0:
        start[::3] = np.nan
    n = orc.orc_dgemv_tiled(T, ta.encode(), M, N, 2.0, ptr(A), lda, ptr(x), 2, beta, ptr(start), -3)
    assert n == -(-M // T) * -(-N // T)
    assert np.array_equal(start, ref)


def test_tiled_close_to_bruteforce_on_random_data(orc):
    M, N = 300, 260
    A, x, y0 = rand_f64(M * N, 9), rand_f64(N, 10), rand_f64(M, 11)
    ref = y0.copy()
    orc.orc_dgemv_bruteforce(b"N", M, N, 1.5, ptr(A), M, ptr(x), 1, 0.5, ptr(ref), 1)
    scale = 1.5 * np.linalg.norm(A) * np.linalg.norm(x) + 0.5 * np.linalg.norm(y0)
    for T in (32, 100, 512):
        y = y0.copy()
        orc.orc_dgemv_tiled(T, b"N", M, N, 1.5, ptr(A), M, ptr(x), 1, 0.5, ptr(y), 1)
        assert np.linalg.norm(y - ref) / scale < 1e-15


def blas2_problem(t1024, remote=(1, 1, 1), sl=(1.0, 1.0), D=(4096, 4096), ta=b"N"):
    Ts = [512, 1024, 2048, 4096]
    tab, keep = make_table(Ts, [t1024 * (t / 1024.0) ** 2 for t in Ts], ta.decode() * 4, "NNNN")
    p = orc_problem()
    p.D1, p.D2, p.D3, p.dtype_sz, p.ta, p.tb = D[0], D[1], 1, 8, ta, b"N"
    for i in range(3):
        p.remote[i] = p.out_remote[i] = remote[i]
    p.h2d = orc_link(0.0, 0.5e-3 / TILE, sl[0])
    p.d2h = orc_link(0.0, 0.25e-3 / TILE, sl[1])
    p.exec = C.pointer(tab)
    return p, (tab, keep)


def test_blas2_models_by_hand(orc):
    """4096 x 4096, T = 1024, everything on the host.  A vector tile of 1024 doubles (8 KiB) costs 0.48828125 us in,
    0.244140625 us out; three inputs, one output; D1/T - 1 = 3 overlapped kernels (ModelLvl2.cpp:194-259)."""
    p, keep = blas2_problem(2e-5)
    # compute-bound tile: 3 * 20 us + max(20 us, 0.244 us) + 3 * 0.48828125 us + 0.244140625 us
    assert abs(orc.orc_predict_blas2(5, p, 1024) - 8.1708984375e-5) < 1e-18
    # transfer-bound tile (1 us kernel), slowdowns 1.25 / 1.5:
    #   t_over = 0.3662109375 us * (1 - 1/1.25) + 1.46484375 us = 1.5380859375 us
    q, keep2 = blas2_problem(1e-6, sl=(1.25, 1.5))
    assert abs(orc.orc_predict_blas2(5, q, 1024) - 7.3232421875e-6) < 1e-18
    # full / zero overlap on the largest tile: exec 320 us; A 8 ms + x 1.953125 us + y 1.953125 us in; y out
    # priced like a receive
    assert abs(orc.orc_predict_blas2(9, p, 1024) - 8.00390625e-3) < 1e-15
    assert abs(orc.orc_predict_blas2(10, p, 1024) - 8.325859375e-3) < 1e-15
    # A on the device, vectors on the host: the host still holds the majority of operands
    r, keep3 = blas2_problem(2e-5, remote=(0, 1, 1))
    assert abs(orc.orc_predict_blas2(5, r, 1024) - (6e-5 + 2e-5 + 2 * 4.8828125e-7 + 2.44140625e-7)) < 1e-18
