"""Parity of the matrix-vector kernel (pl_dgemv) and of PARALiADgemv (tiling of a host-resident A, staged vectors,
beta schedule, metadata reuse) through the C ABI, against the oracle and OpenBLAS on the same seeded inputs."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import Buf, sync
from oracle_binding import ptr, rand_f64

pytestmark = pytest.mark.gpu
TOL = 1e-13


def span(n, inc):
    return (n - 1) * abs(inc) + 1


def place(pkg, arr, loc):
    return Buf(pkg, arr.size, arr.dtype, loc).set(arr)


def norm_err(got, ref, alpha, A, x, beta, y0):
    return float(np.linalg.norm(got - ref)) / (abs(alpha) * float(np.linalg.norm(A)) * float(np.linalg.norm(x)) + abs(beta) * float(np.linalg.norm(y0)) + 1e-300)


def kernel_call(pkg, L, ta, M, N, alpha, dA, lda, dx, incx, beta, dy, incy):
    ws = Buf(pkg, max(8, L.pl_dgemv_workspace_doubles(ta.encode(), M, N)), np.float64, 0)
    print("pl_dgemv", ta, M, N, alpha, beta, "lda", lda, "inc", incx, incy, flush=True)
    pkg.check(L.pl_dgemv(ta.encode(), M, N, float(alpha), dA.ptr, lda, dx.ptr, incx, float(beta), dy.ptr, incy, ws.ptr, None), "pl_dgemv")
    sync(pkg)
    return ws


@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("M,N,pad", [(137, 91, 0), (136, 90, 0), (1024, 1024, 0), (4096, 300, 1), (300, 4096, 0), (1, 1, 0), (2, 7, 0),
                                     (8192, 64, 0), (64, 8192, 2), (5000, 3000, 0), (3, 20000, 0), (20000, 3, 0)])
@pytest.mark.parametrize("incx,incy", [(1, 1), (2, 3), (-1, -2)])
def test_kernel_against_oracle(pkg, L, orc, ta, M, N, pad, incx, incy):
    """Shapes that take the 16-byte-load path (even lda; op = T: and even M) and the scalar one, single and many
    reduction chunks, fewer than four columns per wave, strided and reversed vectors."""
    lda = M + pad
    lx, ly = (N, M) if ta == "N" else (M, N)
    A, x, y0 = rand_f64(lda * N, 1), rand_f64(span(lx, incx), 2), rand_f64(span(ly, incy), 3)
    alpha, beta = 1.23, 0.9876
    ref = y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, alpha, ptr(A), lda, ptr(x), incx, beta, ptr(ref), incy)
    dA, dx, dy = place(pkg, A, 0), place(pkg, x, 0), place(pkg, y0, 0)
    kernel_call(pkg, L, ta, M, N, alpha, dA, lda, dx, incx, beta, dy, incy)
    got = dy.get()
    assert norm_err(got, ref, alpha, A, x, beta, y0) < TOL
    gaps = np.ones(y0.size, dtype=bool)
    gaps[::abs(incy)] = False
    assert np.array_equal(got[gaps], y0[gaps])


@pytest.mark.parametrize("M,N,lda", [(1001, 777, 1004), (4095, 300, 4096), (129, 5, 130), (127, 64, 128), (1, 9, 2), (3, 1, 4)])
def test_kernel_n_with_an_odd_last_row_and_16_byte_columns(pkg, L, M, N, lda):
    """op = N with an odd M and an even lda: the columns start on 16-byte boundaries, so the rows are read in pairs and
    the lane that holds the last row reads the padding element behind it along with it -- NaN here, and never part
    of y -- except in the last column, where that element does not exist: A is allocated with exactly lda * (N - 1) + M
    elements, the least BLAS asks for.  Integer data: exact."""
    rng = np.random.default_rng(M + N)
    A = np.full(lda * (N - 1) + M, np.nan)
    for n in range(N):
        A[n * lda:n * lda + M] = rng.integers(-8, 9, M)
    x = rng.integers(-8, 9, N).astype(np.float64)
    y0 = rng.integers(-8, 9, M).astype(np.float64)
    cols = np.stack([A[n * lda:n * lda + M] for n in range(N)], axis=1)
    ref = 2.0 * (cols @ x) - 3.0 * y0
    dA, dx, dy = place(pkg, A, 0), place(pkg, x, 0), place(pkg, y0, 0)
    kernel_call(pkg, L, "N", M, N, 2.0, dA, lda, dx, 1, -3.0, dy, 1)
    assert np.array_equal(dy.get(), ref)
    # the same through the entry point that brings its own scratch
    dy.set(y0)
    pkg.check(L.pl_dgemv_noalloc(b"N", M, N, 2.0, dA.ptr, lda, dx.ptr, 1, -3.0, dy.ptr, 1, None), "pl_dgemv_noalloc")
    sync(pkg)
    assert np.array_equal(dy.get(), ref)


@pytest.mark.parametrize("ta", ["N", "T"])
def test_kernel_exact_and_blas_conventions(pkg, L, orc, ta):
    M, N = 1500, 2300
    lx, ly = (N, M) if ta == "N" else (M, N)
    rng = np.random.default_rng(5)
    A = rng.integers(-8, 9, M * N).astype(np.float64)
    x = rng.integers(-8, 9, lx).astype(np.float64)
    y0 = rng.integers(-8, 9, ly).astype(np.float64)
    ref = y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 2.0, ptr(A), M, ptr(x), 1, 3.0, ptr(ref), 1)
    dA, dx, dy = place(pkg, A, 0), place(pkg, x, 0), place(pkg, y0, 0)
    kernel_call(pkg, L, ta, M, N, 2.0, dA, M, dx, 1, 3.0, dy, 1)
    assert np.array_equal(dy.get(), ref)              # integers: exact whatever the summation order
    dy.set(np.full(ly, np.nan))
    kernel_call(pkg, L, ta, M, N, 2.0, dA, M, dx, 1, 0.0, dy, 1)
    ref0 = np.zeros(ly)
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 2.0, ptr(A), M, ptr(x), 1, 0.0, ptr(ref0), 1)
    assert np.array_equal(dy.get(), ref0)             # beta = 0 never reads y
    dy.set(y0)
    dnan = place(pkg, np.full(M * N, np.nan), 0)
    kernel_call(pkg, L, ta, M, N, 0.0, dnan, M, dx, 1, 0.5, dy, 1)
    assert np.array_equal(dy.get(), 0.5 * y0)         # alpha = 0 never reads A
    kernel_call(pkg, L, ta, M, N, 0.0, dnan, M, dx, 1, 1.0, dy, 1)
    assert np.array_equal(dy.get(), 0.5 * y0)         # quick return
    ws = Buf(pkg, 64, np.float64, 0)
    assert L.pl_dgemv(ta.encode(), 0, N, 1.0, dA.ptr, 1, dx.ptr, 1, 0.0, dy.ptr, 1, ws.ptr, None) == 0
    assert L.pl_dgemv(ta.encode(), M, 0, 1.0, dA.ptr, M, dx.ptr, 1, 0.0, dy.ptr, 1, ws.ptr, None) == 0
    sync(pkg)
    assert np.array_equal(dy.get(), 0.5 * y0)         # empty problems leave y alone
    assert L.pl_dgemv(b"X", M, N, 1.0, dA.ptr, M, dx.ptr, 1, 0.0, dy.ptr, 1, ws.ptr, None) != 0
    assert L.pl_dgemv(ta.encode(), M, N, 1.0, dA.ptr, M - 1, dx.ptr, 1, 0.0, dy.ptr, 1, ws.ptr, None) != 0
    assert L.pl_dgemv(ta.encode(), M, N, 1.0, dA.ptr, M, dx.ptr, 0, 0.0, dy.ptr, 1, ws.ptr, None) != 0
    assert L.pl_dgemv(ta.encode(), M, N, 1.0, None, M, dx.ptr, 1, 0.0, dy.ptr, 1, ws.ptr, None) != 0


def call_gemv(pkg, L, ta, M, N, alpha, bA, lda, bx, incx, beta, by, incy, T=-1, cache_limit=0):
    info = pkg.atc_info()
    print("PARALiA dgemv", ta, M, N, alpha, beta, "locs", bA.loc, bx.loc, by.loc, "T", T, "inc", incx, incy, flush=True)
    pkg.check(L.PARALiA_dgemv(ta.encode(), M, N, float(alpha), bA.ptr, lda, bx.ptr, incx, float(beta), by.ptr, incy, T, cache_limit,
                              C.byref(info)), "PARALiA_dgemv")
    return info


LOCS = [(0, 0, 0), (-1, -1, -1), (-1, 0, 0), (0, -1, -1), (-2, -2, -2), (-1, -1, 0), (-1, 0, -1)]


@pytest.mark.parametrize("locs", LOCS)
@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("T", [-1, 100, 128])
def test_routine_placements(pkg, L, orc, openblas, locs, ta, T):
    """Every operand placement, both transposes, a sub-matrix view (lda > M), strided x and reversed y; T = 100 / 128
    cut A into 3 x 4 / 3 x 3 ragged tiles when it has to be streamed."""
    M, N, lda, incx, incy = 289, 353, 400, 2, -1
    lx, ly = (N, M) if ta == "N" else (M, N)
    alpha, beta = 1.23, 0.9876
    A, x, y0 = rand_f64(lda * N, 42), rand_f64(span(lx, incx), 43), rand_f64(span(ly, incy), 44)
    ref = y0.copy()
    assert openblas.orc_openblas_dgemv(ta.encode(), M, N, alpha, ptr(A), lda, ptr(x), incx, beta, ptr(ref), incy) == 0
    bA, bx, by = place(pkg, A, locs[0]), place(pkg, x, locs[1]), place(pkg, y0, locs[2])
    info = call_gemv(pkg, L, ta, M, N, alpha, bA, lda, bx, incx, beta, by, incy, T=T)
    got = by.get()
    assert norm_err(got, ref, alpha, A, x, beta, y0) < TOL
    if T > 0:
        tiled = y0.copy()
        orc.orc_dgemv_tiled(T, ta.encode(), M, N, alpha, ptr(A), lda, ptr(x), incx, beta, ptr(tiled), incy)
        assert norm_err(got, tiled, alpha, A, x, beta, y0) < TOL
        assert info.T == T and info.selected_by == b"user" and info.subkernel_num == -(-M // T) * -(-N // T)
    assert np.array_equal(bA.get(), A) and np.array_equal(bx.get(), x)  # inputs are never written


@pytest.mark.parametrize("ta", ["N", "T"])
@pytest.mark.parametrize("T", [64, 100, 512, 5000])
@pytest.mark.parametrize("beta", [0.0, 3.0])
def test_routine_streamed_exact_on_integers(pkg, L, orc, ta, T, beta):
    """Host-resident integer-valued operands: the streamed, tiled result equals the untiled one bit for bit for every
    tile size (also one larger than both dimensions), with a strided y whose gaps must survive the write-back and
    beta = 0 over NaN."""
    M, N, incy = 700, 520, 3
    lx, ly = (N, M) if ta == "N" else (M, N)
    rng = np.random.default_rng(T)
    A = rng.integers(-8, 9, M * N).astype(np.float64)
    x = rng.integers(-8, 9, lx).astype(np.float64)
    y0 = rng.integers(-8, 9, span(ly, incy)).astype(np.float64)
    ref = y0.copy()
    orc.orc_dgemv_bruteforce(ta.encode(), M, N, 2.0, ptr(A), M, ptr(x), 1, beta, ptr(ref), incy)
    start = y0.copy()
    if beta == 0.0:
        start[::incy] = np.nan
    bA, bx, by = place(pkg, A, -1), place(pkg, x, -1), place(pkg, start, -1)
    info = call_gemv(pkg, L, ta, M, N, 2.0, bA, M, bx, 1, beta, by, incy, T=T)
    assert info.T == min(T, max(M, N))
    assert np.array_equal(by.get(), ref)


def test_routine_metadata_reuse_errors_and_limits(pkg, L, orc, openblas):
    M, N, T = 384, 256, 128
    L.PARALiA_runtime_reset()
    hits, misses = C.c_long(), C.c_long()
    for seed in (1, 2, 3):
        A, x, y0 = rand_f64(M * N, seed), rand_f64(N, seed + 10), rand_f64(M, seed + 20)
        bA, bx, by = place(pkg, A, -1), place(pkg, x, -1), place(pkg, y0, -1)
        call_gemv(pkg, L, "N", M, N, 1.0, bA, M, bx, 1, 1.0, by, 1, T=T)
        ref = y0.copy()
        openblas.orc_openblas_dgemv(b"N", M, N, 1.0, ptr(A), M, ptr(x), 1, 1.0, ptr(ref), 1)
        assert norm_err(by.get(), ref, 1.0, A, x, 1.0, y0) < TOL
    L.PARALiA_runtime_stats(C.byref(hits), C.byref(misses), None, None)
    assert misses.value == 1 and hits.value == 2
    # a cache limit of two tiles still runs (ring of two blocks); less than one tile is the reference's error
    bA, bx, by = place(pkg, A, -1), place(pkg, x, -1), place(pkg, y0, -1)
    L.PARALiA_dev_cache_free(0)
    call_gemv(pkg, L, "N", M, N, 1.0, bA, M, bx, 1, 1.0, by, 1, T=T, cache_limit=2 * T * T * 8 + 512)
    assert norm_err(by.get(), ref, 1.0, A, x, 1.0, y0) < TOL
    pool = C.c_longlong()
    L.PARALiA_runtime_stats(None, None, C.byref(pool), None)
    assert 0 < pool.value <= 2 * T * T * 8 + 512
    assert L.PARALiA_dgemv(b"N", M, N, 1.0, bA.ptr, M, bx.ptr, 1, 1.0, by.ptr, 1, T, T * T * 4, None) != 0
    assert b"less memory" in L.PARALiA_last_error()
    assert L.PARALiA_dgemv(b"Q", M, N, 1.0, bA.ptr, M, bx.ptr, 1, 1.0, by.ptr, 1, -1, 0, None) != 0
    assert b"transpose" in L.PARALiA_last_error()
    assert L.PARALiA_dgemv(b"N", M, N, 1.0, bA.ptr, M - 1, bx.ptr, 1, 1.0, by.ptr, 1, -1, 0, None) != 0
    assert b"leading dimension" in L.PARALiA_last_error()
    assert L.PARALiA_dgemv(b"N", M, N, 1.0, bA.ptr, M, bx.ptr, 0, 1.0, by.ptr, 1, -1, 0, None) != 0
    assert b"increment" in L.PARALiA_last_error()
    before = by.get()
    assert L.PARALiA_dgemv(b"N", 0, N, 1.0, bA.ptr, 1, bx.ptr, 1, 0.0, by.ptr, 1, -1, 0, None) == 0   # empty: y untouched
    assert np.array_equal(by.get(), before)
    L.PARALiA_dev_cache_free(0)


def test_routine_autotuned_call(pkg, L, orc, openblas):
    """No preset: the autotuner picks T from the shipped database for a host-resident 6000 x 5000 matrix."""
    M, N = 6000, 5000
    A, x, y0 = rand_f64(M * N, 0), rand_f64(N, 1), rand_f64(M, 2)
    bA, bx, by = place(pkg, A, -1), place(pkg, x, -1), place(pkg, y0, -1)
    info = call_gemv(pkg, L, "N", M, N, 1.2, bA, M, bx, 1, 1.1, by, 1)
    assert 0 < info.T <= 6000 and info.subkernel_num >= 1
    ref = y0.copy()
    openblas.orc_openblas_dgemv(b"N", M, N, 1.2, ptr(A), M, ptr(x), 1, 1.1, ptr(ref), 1)
    assert norm_err(by.get(), ref, 1.2, A, x, 1.1, y0) < TOL


@pytest.mark.parametrize("seed", range(32))
def test_random_gemv_cases(pkg, L, orc, openblas, seed):
    """Random shapes, transposes, placements (device, pinned, pageable), tile sizes, increments of either sign, padded
    leading dimension, alpha / beta including 0, against OpenBLAS."""
    rng = np.random.default_rng(900 + seed)
    M, N = (int(x) for x in rng.integers(1, 900, 2))
    ta = str(rng.choice(["N", "T"]))
    lda = M + int(rng.integers(0, 5))
    incx, incy = (int(x) for x in rng.choice([1, 1, 2, -1, -3], 2))
    alpha = float(rng.choice([0.0, 1.0, -0.75, 1.23]))
    beta = float(rng.choice([0.0, 1.0, 0.5]))
    locs = tuple(int(x) for x in rng.choice([-2, -1, 0], 3))
    T = int(rng.choice([-1, 64, 100, 256, 2048]))
    lx, ly = (N, M) if ta == "N" else (M, N)
    A, x, y0 = rand_f64(lda * N, seed), rand_f64(span(lx, incx), seed + 100), rand_f64(span(ly, incy), seed + 200)
    ref = y0.copy()
    assert openblas.orc_openblas_dgemv(ta.encode(), M, N, alpha, ptr(A), lda, ptr(x), incx, beta, ptr(ref), incy) == 0
    bA, bx, by = place(pkg, A, locs[0]), place(pkg, x, locs[1]), place(pkg, y0, locs[2])
    call_gemv(pkg, L, ta, M, N, alpha, bA, lda, bx, incx, beta, by, incy, T=T)
    got = by.get()
    if alpha == 0.0 and beta == 0.0:
        assert np.all(got[::abs(incy)] == 0)
    else:
        assert norm_err(got, ref, alpha, A, x, beta, y0) < TOL
    gaps = np.ones(y0.size, dtype=bool)
    gaps[::abs(incy)] = False
    assert np.array_equal(got[gaps], y0[gaps])
