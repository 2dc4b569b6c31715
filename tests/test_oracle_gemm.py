"""Pins the GEMM part of the CPU oracle without the reference: OpenBLAS on the same inputs, closed forms, exact
integer data, invariance under the tile size.  A dropped term, a wrong sign, a swapped or transposed operand
fails at least one of these."""
import ctypes as C

import numpy as np
import pytest

from oracle_binding import ptr, rand_f32, rand_f64

TOL64, TOL32 = 1e-13, 1e-5  # normwise relative error bounds of the build contract


def colmajor(rows, cols, ld, seed, dtype=np.float64):
    buf = (rand_f64 if dtype == np.float64 else rand_f32)(ld * cols, seed)
    return buf  # element (i, j) at buf[i + j*ld]


def view(buf, rows, cols, ld):
    return buf.reshape(cols, ld).T[:rows, :]


def denom(alpha, A, B, beta, C0):
    return abs(alpha) * np.linalg.norm(A) * np.linalg.norm(B) + abs(beta) * np.linalg.norm(C0)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(64, 48, 40), (97, 113, 71)])
def test_bruteforce_matches_numpy_and_openblas(orc, openblas, ta, tb, dims):
    M, N, K = dims
    alpha, beta = 1.2, 1.1
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 3, rb + 5, M + 2
    A, B, C0 = colmajor(ra, ca, lda, 1), colmajor(rb, cb, ldb, 2), colmajor(M, N, ldc, 3)
    opA = view(A, ra, ca, lda) if ta == "N" else view(A, ra, ca, lda).T
    opB = view(B, rb, cb, ldb) if tb == "N" else view(B, rb, cb, ldb).T
    ref = alpha * opA.astype(np.longdouble) @ opB.astype(np.longdouble) + beta * view(C0, M, N, ldc)
    C1 = C0.copy()
    orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(C1), ldc)
    d = denom(alpha, opA, opB, beta, view(C0, M, N, ldc))
    assert np.linalg.norm((view(C1, M, N, ldc) - ref).astype(np.float64)) / d < 1e-16
    # padding rows between columns are untouched
    pad = np.ones(ldc * N, dtype=bool)
    pad.reshape(N, ldc)[:, :M] = False
    assert np.array_equal(C1[pad], C0[pad])
    C2 = C0.copy()
    assert openblas.orc_openblas_dgemm(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(C2), ldc) == 0
    assert orc.orc_normwise_err_f64(ptr(C2), ptr(C1), M, N, ldc, ldc, d) < TOL64


def test_closed_forms(orc):
    n = 33
    I = np.eye(n).T.copy().ravel()
    B, C0 = rand_f64(n * n, 5), rand_f64(n * n, 6)
    C = C0.copy()
    orc.orc_dgemm_bruteforce(b"N", b"N", n, n, n, 2.0, ptr(I), n, ptr(B), n, 0.25, ptr(C), n)
    assert np.array_equal(C, 2.0 * B + 0.25 * C0)  # A = I, power-of-two scalars: products exact, one rounding
    ones = np.ones(n * 40)
    C = np.ones(n * n)
    orc.orc_dgemm_bruteforce(b"N", b"N", n, n, 40, 2.0, ptr(ones), n, ptr(ones), 40, 3.0, ptr(C), n)
    assert np.all(C == 2.0 * 40 + 3.0)  # all-ones: alpha*K + beta
    C = C0.copy()
    orc.orc_dgemm_bruteforce(b"N", b"N", n, n, n, 0.0, ptr(B), n, ptr(B), n, 0.5, ptr(C), n)
    assert np.array_equal(C, 0.5 * C0)  # alpha = 0
    C = np.full(n * n, np.nan)
    orc.orc_dgemm_bruteforce(b"N", b"N", n, n, n, 1.0, ptr(I), n, ptr(B), n, 0.0, ptr(C), n)
    assert np.array_equal(C, B)  # beta = 0 never reads C (NaN must not leak)


def test_transpose_identity(orc):
    M, N, K = 21, 17, 19
    A, B = rand_f64(M * K, 7), rand_f64(K * N, 8)
    At = view(A, M, K, M).T.copy().T.ravel()  # explicit transpose stored K x M column-major
    At = np.ascontiguousarray(view(A, M, K, M)).ravel()  # rows of A contiguous == column-major K x M of A^T
    C1, C2 = np.zeros(M * N), np.zeros(M * N)
    orc.orc_dgemm_bruteforce(b"N", b"N", M, N, K, 1.0, ptr(A), M, ptr(B), K, 0.0, ptr(C1), M)
    orc.orc_dgemm_bruteforce(b"T", b"N", M, N, K, 1.0, ptr(At), K, ptr(B), K, 0.0, ptr(C2), M)
    assert np.array_equal(C1, C2)  # same k order, same values: bit for bit


@pytest.mark.parametrize("T", [16, 24, 37, 64, 200])
@pytest.mark.parametrize("resident", [0, 1])
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "T"), ("N", "T")])
def test_tiled_schedule_exact_on_integers(orc, T, resident, ta, tb):
    """Integer-valued data: every partial sum is exact, so the tiled schedule (tile order, beta' = 0/1/beta,
    lazy reduce) must reproduce the untiled result bit for bit whatever T is."""
    M, N, K = 89, 61, 77  # not multiples of any T: edge tiles everywhere
    rng = np.random.default_rng(11)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 1, rb + 2, M + 3
    A = rng.integers(-8, 9, lda * ca).astype(np.float64)
    B = rng.integers(-8, 9, ldb * cb).astype(np.float64)
    C0 = rng.integers(-8, 9, ldc * N).astype(np.float64)
    for alpha, beta in ((2.0, 3.0), (1.0, 0.0), (-1.0, 1.0)):
        ref, got = C0.copy(), C0.copy()
        orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc)
        fired = orc.orc_dgemm_tiled(T, resident, ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(got), ldc)
        assert fired == -(-M // T) * -(-N // T) * -(-K // T)
        assert np.array_equal(ref, got)


def test_tiled_beta_zero_ignores_nan_c(orc):
    M = N = K = 40
    A, B = rand_f64(M * K, 1), rand_f64(K * N, 2)
    C = np.full(M * N, np.nan)
    orc.orc_dgemm_tiled(16, 0, b"N", b"N", M, N, K, 1.0, ptr(A), M, ptr(B), K, 0.0, ptr(C), M)
    assert not np.isnan(C).any()


@pytest.mark.parametrize("T", [64, 96, 128])
def test_tiled_T_invariance_weird_dims(orc, openblas, T):
    """Dimensions of the reference's own tester (289 / 353 / 307, dgemm_tester.cpp:133), alpha/beta from :74-75,
    sub-matrix views with ld larger than the rows (:48,78)."""
    M, N, K = 289, 353, 307
    alpha, beta = 1.23, 0.9876
    lda, ldb, ldc = 400, 400, 400
    A, B, C0 = rand_f64(lda * K, 42), rand_f64(ldb * N, 43), rand_f64(ldc * N, 44)
    ref = C0.copy()
    assert openblas.orc_openblas_dgemm(b"N", b"N", M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc) == 0
    d = denom(alpha, view(A, M, K, lda), view(B, K, N, ldb), beta, view(C0, M, N, ldc))
    for resident in (0, 1):
        got = C0.copy()
        orc.orc_dgemm_tiled(T, resident, b"N", b"N", M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(got), ldc)
        assert orc.orc_normwise_err_f64(ptr(got), ptr(ref), M, N, ldc, ldc, d) < TOL64


def test_sgemm_oracle(orc, openblas):
    M, N, K = 130, 70, 90
    alpha, beta = np.float32(1.0), np.float32(1.0)
    A, B, C0 = rand_f32(M * K, 1), rand_f32(N * K, 2), rand_f32(M * N, 3)  # B stored N x K, used transposed
    ref, bf, tl = C0.copy(), C0.copy(), C0.copy()
    assert openblas.orc_openblas_sgemm(b"N", b"T", M, N, K, alpha, ptr(A), M, ptr(B), N, beta, ptr(ref), M) == 0
    orc.orc_sgemm_bruteforce(b"N", b"T", M, N, K, alpha, ptr(A), M, ptr(B), N, beta, ptr(bf), M)
    orc.orc_sgemm_tiled(32, 0, b"N", b"T", M, N, K, alpha, ptr(A), M, ptr(B), N, beta, ptr(tl), M)
    d = float(np.linalg.norm(A.astype(np.float64)) * np.linalg.norm(B.astype(np.float64)) + np.linalg.norm(C0.astype(np.float64)))
    assert orc.orc_normwise_err_f32(ptr(bf), ptr(ref), M, N, M, M, d) < TOL32
    assert orc.orc_normwise_err_f32(ptr(tl), ptr(ref), M, N, M, M, d) < TOL32


def test_generator_known_answers(orc):
    # splitmix64, seed 1234567: first outputs of the published reference implementation
    s = C.c_uint64(1234567)
    got = [orc.orc_splitmix64(C.byref(s)) for _ in range(5)]
    assert got == [6457827717110365317, 3203168211198807973, 9817491932198370423, 4593380528125082431,
                   16408922859458223821]
    a = rand_f64(100000, 0)
    assert a.min() >= -1.0 and a.max() < 1.0 and abs(a.mean()) < 0.01 and abs(a.var() - 1 / 3) < 0.01
    assert np.array_equal(rand_f64(1000, 9)[500:], rand_f64(2000, 9)[500:1000])  # element i depends on (seed, i) only
    assert not np.array_equal(rand_f64(100, 0), rand_f64(100, 1))
    f = rand_f32(100000, 3)
    assert f.dtype == np.float32 and f.min() >= -1.0 and f.max() < 1.0 and abs(float(f.mean())) < 0.01


def test_error_metrics(orc):
    a = np.array([1.0, 2.0, 3.0])
    b = np.array([1.0, np.nextafter(2.0, 3.0), 3.0])
    assert orc.orc_max_ulp_f64(ptr(a), ptr(b), 3) == 1
    assert orc.orc_max_ulp_f64(ptr(a), ptr(a), 3) == 0
    c = np.array([-0.0, 1.0, 3.0])
    z = np.array([0.0, 1.0, 3.0])
    assert orc.orc_max_ulp_f64(ptr(c), ptr(z), 3) == 0
    assert orc.orc_digits_equal(ptr(a), ptr(np.array([1.0, 2.0, 3.0003])), 3) == 4
    assert orc.orc_digits_equal(ptr(a), ptr(a), 3) == 16
    assert abs(orc.orc_fro_norm_f64(ptr(a), 3, 1, 3) - np.sqrt(14.0)) < 1e-15
