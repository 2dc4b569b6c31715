"""Parity of the PARALiA routines (tiling, streaming, block pool, lazy write-back, metadata reuse) called through
the C ABI, against OpenBLAS / the oracle on the same seeded inputs, for every operand placement."""
import ctypes as C
import os

import numpy as np
import pytest

from gpu_util import Buf, sync, check_daxpy_against_blas, k_tiles
from oracle_binding import ptr, rand_f32, rand_f64

pytestmark = pytest.mark.gpu
TOL64, TOL32 = 1e-13, 1e-5


def place(pkg, arr, loc):
    return Buf(pkg, arr.size, arr.dtype, loc).set(arr)


def call_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, bufA, lda, bufB, ldb, bufC, ldc, T=-1, cache_limit=0):
    info = pkg.atc_info()
    fn = L.PARALiA_dgemm if dtype == np.float64 else L.PARALiA_sgemm
    print("PARALiA gemm", np.dtype(dtype).name, ta, tb, M, N, K, alpha, beta, "locs", bufA.loc, bufB.loc, bufC.loc, "T", T,
          "limit", cache_limit, flush=True)
    pkg.check(fn(ta.encode(), tb.encode(), M, N, K, float(alpha), bufA.ptr, lda, bufB.ptr, ldb, float(beta), bufC.ptr, ldc, T,
                 cache_limit, C.byref(info)), "PARALiA gemm")
    return info


def openblas_ref(openblas, dtype, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc):
    ref = C0.copy()
    fn = openblas.orc_openblas_dgemm if dtype == np.float64 else openblas.orc_openblas_sgemm
    assert fn(ta.encode(), tb.encode(), M, N, K, float(alpha), ptr(A), lda, ptr(B), ldb, float(beta), ptr(ref), ldc) == 0
    return ref


def normwise(orc, dtype, got, ref, M, N, ldc, alpha, beta, A, ra, ca, lda, B, rb, cb, ldb, C0):
    if dtype == np.float64:
        d = abs(alpha) * orc.orc_fro_norm_f64(ptr(A), ra, ca, lda) * orc.orc_fro_norm_f64(ptr(B), rb, cb, ldb) + abs(beta) * orc.orc_fro_norm_f64(ptr(C0), M, N, ldc)
        return orc.orc_normwise_err_f64(ptr(got), ptr(ref), M, N, ldc, ldc, d)
    d = abs(alpha) * orc.orc_fro_norm_f32(ptr(A), ra, ca, lda) * orc.orc_fro_norm_f32(ptr(B), rb, cb, ldb) + abs(beta) * orc.orc_fro_norm_f32(ptr(C0), M, N, ldc)
    return orc.orc_normwise_err_f32(ptr(got), ptr(ref), M, N, ldc, ldc, d)


LOCS = [(-1, -1, -1), (0, 0, 0), (-1, -1, 0), (0, -1, -1), (-1, 0, -1), (0, 0, -1), (-2, -2, -2), (-2, 0, -1)]


@pytest.mark.parametrize("locs", LOCS)
@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
def test_dgemm_placements_and_transposes(pkg, L, orc, openblas, locs, ta, tb):
    """The reference tester's 'weird' dimensions (dgemm_tester.cpp:133), its alpha/beta (:74-75) and sub-matrix views
    with a leading dimension larger than the rows (:48,78); T = 128 gives 3 x 3 x 3 tiles with ragged edges."""
    M, N, K = 289, 353, 307
    alpha, beta = 1.23, 0.9876
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = 400, 400, 400
    A, B, C0 = rand_f64(lda * ca, 42), rand_f64(ldb * cb, 43), rand_f64(ldc * N, 44)
    bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, C0, locs[2])
    info = call_gemm(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, bA, lda, bB, ldb, bC, ldc, T=128)
    got = bC.get()
    ref = openblas_ref(openblas, np.float64, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    assert normwise(orc, np.float64, got, ref, M, N, ldc, alpha, beta, A, ra, ca, lda, B, rb, cb, ldb, C0) < TOL64
    tiled = C0.copy()
    orc.orc_dgemm_tiled(128, 1 if locs[2] >= 0 else 0, ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(tiled), ldc)
    assert normwise(orc, np.float64, got, tiled, M, N, ldc, alpha, beta, A, ra, ca, lda, B, rb, cb, ldb, C0) < TOL64
    pad = np.ones(ldc * N, dtype=bool)
    pad.reshape(N, ldc)[:, :M] = False
    assert np.array_equal(got[pad], C0[pad])
    assert info.T == 128 and info.selected_by == b"user" and info.subkernel_num == 9 * k_tiles(info, K)
    assert np.array_equal(bA.get(), A) and np.array_equal(bB.get(), B)  # inputs are never written


@pytest.mark.parametrize("T", [64, 100, 256, 512, 1000])
@pytest.mark.parametrize("beta", [0.0, 3.0])
def test_dgemm_tiled_exact_on_integers(pkg, L, orc, T, beta):
    """Integer-valued operands in pinned host memory: the streamed, tiled result must equal the untiled one bit for
    bit for every tile size, including T larger than K (tiles shallower than wide) and beta = 0 over NaN."""
    M, N, K = 700, 520, 300
    rng = np.random.default_rng(T)
    A = rng.integers(-8, 9, M * K).astype(np.float64)
    B = rng.integers(-8, 9, K * N).astype(np.float64)
    C0 = rng.integers(-8, 9, M * N).astype(np.float64)
    ref = C0.copy()
    orc.orc_dgemm_bruteforce(b"N", b"N", M, N, K, 2.0, ptr(A), M, ptr(B), K, beta, ptr(ref), M)
    start = np.full(M * N, np.nan) if beta == 0.0 else C0
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, start, -1)
    info = call_gemm(pkg, L, np.float64, "N", "N", M, N, K, 2.0, beta, bA, M, bB, K, bC, M, T=T)
    assert info.T == min(T, max(M, N, K))  # a tile larger than every dimension is the whole problem
    assert np.array_equal(bC.get(), ref)


@pytest.mark.parametrize("blocks", [3, 4, 6, 11])
def test_dgemm_block_pool_smaller_than_working_set(pkg, L, orc, openblas, blocks):
    """cache_limit (the ...Controled knob) below the working set: tiles are evicted and fetched again; the result
    does not change.  Fewer than 3 blocks is the reference's error (dgemm.cpp:41-42)."""
    M = N = K = 640
    T = 128
    A, B, C0 = rand_f64(M * K, 1), rand_f64(K * N, 2), rand_f64(M * N, 3)
    ref = openblas_ref(openblas, np.float64, "N", "T", M, N, K, 1.5, 0.5, A, M, B, N, C0, M)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    limit = blocks * T * T * 8
    L.PARALiA_dev_cache_free(0)
    info = call_gemm(pkg, L, np.float64, "N", "T", M, N, K, 1.5, 0.5, bA, M, bB, N, bC, M, T=T, cache_limit=limit)
    assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 1.5, 0.5, A, M, K, M, B, N, K, N, C0) < TOL64
    pool = C.c_longlong()
    L.PARALiA_runtime_stats(None, None, C.byref(pool), None)
    assert 0 < pool.value <= limit
    L.PARALiA_dev_cache_free(0)
    L.PARALiA_runtime_stats(None, None, C.byref(pool), None)
    assert pool.value == 0


@pytest.mark.parametrize("blocks", [5, 9, 14, 20, 33, 60, 100])
@pytest.mark.parametrize("beta", [0.0, 0.5])
def test_dgemm_pool_sweep_picks_different_orders(pkg, L, orc, openblas, blocks, beta):
    """A 6 x 5 x 7 grid of ragged tiles (138 blocks when everything fits) in pools from 5 to 100 blocks: the
    autotuner moves between the order families and the two eviction policies, the result stays the same."""
    M, N, K, T = 1436, 1180, 1700, 256
    A, B, C0 = rand_f64(M * K, 11), rand_f64(K * N, 12), rand_f64(M * N, 13)
    ref = openblas_ref(openblas, np.float64, "T", "N", M, N, K, -0.7, beta, A, K, B, K, C0, M)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    info = call_gemm(pkg, L, np.float64, "T", "N", M, N, K, -0.7, beta, bA, K, bB, K, bC, M, T=T, cache_limit=blocks * T * T * 8)
    print("  order", info.order_id, "subkernels", info.subkernel_num, flush=True)
    assert info.subkernel_num == 6 * 5 * k_tiles(info, K)
    assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 0.7, beta, A, K, M, K, B, K, N, K, C0) < TOL64


@pytest.mark.parametrize("order", [1, 10003, 20002, 30002, 40000, 60002, 70001])
def test_dgemm_with_pinned_order_family(pkg, L, orc, openblas, order, monkeypatch):
    """Every order family and both eviction policies executed for real (PARALIA_GEMM_ORDER pins the plan) in a pool of
    24 blocks for a 5 x 4 x 6 tile grid (75 blocks when everything fits); K differs per order so that each call is a
    new problem for the metadata cache."""
    monkeypatch.setenv("PARALIA_GEMM_ORDER", str(order))
    M, N, T = 1200, 1000, 256
    K = 1500 + order % 97
    A, B, C0 = rand_f64(M * K, 21), rand_f64(K * N, 22), rand_f64(M * N, 23)
    ref = openblas_ref(openblas, np.float64, "N", "N", M, N, K, 1.25, -0.5, A, M, B, K, C0, M)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    info = call_gemm(pkg, L, np.float64, "N", "N", M, N, K, 1.25, -0.5, bA, M, bB, K, bC, M, T=T, cache_limit=24 * T * T * 8)
    assert info.order_id == order
    assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 1.25, 0.5, A, M, K, M, B, K, N, K, C0) < TOL64


def test_dgemm_too_little_memory_is_an_error(pkg, L):
    M = N = K = 512
    A = rand_f64(M * K, 1)
    b = place(pkg, A, -1)
    rc = L.PARALiA_dgemm(b"N", b"N", M, N, K, 1.0, b.ptr, M, b.ptr, K, 0.0, b.ptr, M, 128, 2 * 128 * 128 * 8, None)
    assert rc != 0 and b"less memory" in L.PARALiA_last_error()
    assert L.PARALiA_dgemm(b"N", b"X", M, N, K, 1.0, b.ptr, M, b.ptr, K, 0.0, b.ptr, M, -1, 0, None) != 0
    assert b"transpose" in L.PARALiA_last_error()
    assert L.PARALiA_dgemm(b"N", b"N", M, N, K, 1.0, b.ptr, M - 1, b.ptr, K, 0.0, b.ptr, M, -1, 0, None) != 0
    assert b"leading dimension" in L.PARALiA_last_error()
    assert L.PARALiA_dgemm(b"N", b"N", 0, N, K, 1.0, b.ptr, 1, b.ptr, K, 0.0, b.ptr, 1, -1, 0, None) == 0  # empty: nothing to do


def test_dgemm_metadata_reuse(pkg, L, orc, openblas):
    """A second call with the same shape and operand locations reuses the tuned problem (the reference's PMD cache,
    dgemm.cpp:342-368) and still sees the new data."""
    M, N, K, T = 384, 256, 320, 128
    L.PARALiA_runtime_reset()
    hits, misses = C.c_long(), C.c_long()
    for seed in (1, 2, 3):
        A, B, C0 = rand_f64(M * K, seed), rand_f64(K * N, seed + 10), rand_f64(M * N, seed + 20)
        bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
        call_gemm(pkg, L, np.float64, "N", "N", M, N, K, 1.0, 1.0, bA, M, bB, K, bC, M, T=T)
        ref = openblas_ref(openblas, np.float64, "N", "N", M, N, K, 1.0, 1.0, A, M, B, K, C0, M)
        assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 1.0, 1.0, A, M, K, M, B, K, N, K, C0) < TOL64
    L.PARALiA_runtime_stats(C.byref(hits), C.byref(misses), None, None)
    assert misses.value == 1 and hits.value == 2


def test_dgemm_alpha_zero_and_k_zero(pkg, L):
    M, N = 300, 200
    C0 = rand_f64(M * N, 5)
    junk = np.full(16, np.nan)
    bJ, bC = place(pkg, junk, -1), place(pkg, C0, -1)
    call_gemm(pkg, L, np.float64, "N", "N", M, N, 50, 0.0, 0.5, bJ, M, bJ, 50, bC, M, T=128)
    assert np.array_equal(bC.get(), 0.5 * C0)  # alpha == 0: A and B are not referenced
    bC.set(C0)
    call_gemm(pkg, L, np.float64, "N", "N", M, N, 0, 1.0, 2.0, bJ, M, bJ, 1, bC, M, T=128)
    assert np.array_equal(bC.get(), 2.0 * C0)


def test_dgemm_autotuned_call(pkg, L, orc, openblas):
    """No preset: the autotuner picks T; config 1 of the benchmark set at a quarter of its size."""
    M = N = K = 1024
    alpha, beta = 1.2, 1.1
    A, B, C0 = rand_f64(M * K, 0), rand_f64(K * N, 1), rand_f64(M * N, 2)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    info = call_gemm(pkg, L, np.float64, "N", "N", M, N, K, alpha, beta, bA, M, bB, K, bC, M)
    assert 0 < info.T <= 1024 and info.subkernel_num >= 1
    ref = openblas_ref(openblas, np.float64, "N", "N", M, N, K, alpha, beta, A, M, B, K, C0, M)
    assert normwise(orc, np.float64, bC.get(), ref, M, N, M, alpha, beta, A, M, K, M, B, K, N, K, C0) < TOL64


@pytest.mark.parametrize("locs", [(-1, -1, 0), (-1, -1, -1), (0, 0, 0)])
def test_sgemm_mixed_locations(pkg, L, orc, openblas, locs):
    """Shape of benchmark config 4 in small: fp32, transA = N, transB = T, alpha = beta = 1, A and B in pinned host
    memory, C resident on the device."""
    M, N, K, T = 520, 390, 450, 128
    A, B, C0 = rand_f32(M * K, 1), rand_f32(N * K, 2), rand_f32(M * N, 3)
    bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, C0, locs[2])
    call_gemm(pkg, L, np.float32, "N", "T", M, N, K, 1.0, 1.0, bA, M, bB, N, bC, M, T=T)
    ref = openblas_ref(openblas, np.float32, "N", "T", M, N, K, 1.0, 1.0, A, M, B, N, C0, M)
    assert normwise(orc, np.float32, bC.get(), ref, M, N, M, 1.0, 1.0, A, M, K, M, B, N, K, N, C0) < TOL32


def test_dgemm_large_checksum(pkg, L):
    """4096^3 with host operands (benchmark config 1 on the GPU path): a full OpenBLAS product is replaced by the
    size-independent identity (alpha*A*B + beta*C0) v = alpha*A*(B*v) + beta*(C0*v) for a random v, evaluated in
    O(n^2) on the CPU."""
    n = 4096
    alpha, beta = 1.2, 1.1
    A, B, C0 = rand_f64(n * n, 0), rand_f64(n * n, 1), rand_f64(n * n, 2)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    info = call_gemm(pkg, L, np.float64, "N", "N", n, n, n, alpha, beta, bA, n, bB, n, bC, n)
    got = bC.get().reshape(n, n).T  # column-major
    v = rand_f64(n, 3)
    Am, Bm, Cm = A.reshape(n, n).T, B.reshape(n, n).T, C0.reshape(n, n).T
    expect = alpha * (Am @ (Bm @ v)) + beta * (Cm @ v)
    err = np.linalg.norm(got @ v - expect) / (abs(alpha) * np.linalg.norm(Am) * np.linalg.norm(Bm) * np.linalg.norm(v) + abs(beta) * np.linalg.norm(Cm) * np.linalg.norm(v))
    assert err < TOL64
    # and three random 64 x 64 panels against numpy in long double
    rng = np.random.default_rng(0)
    for _ in range(3):
        i, j = rng.integers(0, n - 64, 2)
        blk = alpha * (Am[i:i + 64, :].astype(np.longdouble) @ Bm[:, j:j + 64].astype(np.longdouble)) + beta * Cm[i:i + 64, j:j + 64]
        d = np.linalg.norm((got[i:i + 64, j:j + 64] - blk).astype(np.float64))
        assert d / (abs(alpha) * np.linalg.norm(Am[i:i + 64, :]) * np.linalg.norm(Bm[:, j:j + 64]) + abs(beta) * np.linalg.norm(Cm[i:i + 64, j:j + 64])) < TOL64


@pytest.mark.parametrize("locs", [(0, 0), (-1, -1), (-1, 0), (0, -1), (-2, -2)])
@pytest.mark.parametrize("T", [-1, 1000, 1 << 16])
def test_daxpy_routine(pkg, L, orc, openblas, locs, T):
    n, alpha = (1 << 18) + 37, 0.7
    x, y0 = rand_f64(n, 1), rand_f64(n, 2)
    bx, by = place(pkg, x, locs[0]), place(pkg, y0, locs[1])
    info = pkg.atc_info()
    print("PARALiA daxpy", n, locs, T, flush=True)
    pkg.check(L.PARALiA_daxpy(n, alpha, bx.ptr, 1, by.ptr, 1, T, C.byref(info)), "PARALiA_daxpy")
    got = by.get()
    fused = y0.copy()
    orc.orc_daxpy(n, alpha, ptr(x), 1, ptr(fused), 1)
    assert np.array_equal(got, fused)
    ref = y0.copy()
    assert openblas.orc_openblas_daxpy(n, alpha, ptr(x), 1, ptr(ref), 1) == 0
    check_daxpy_against_blas(orc, got, ref, alpha, x, y0)
    assert np.array_equal(bx.get(), x)
    if T > 0 and min(locs) < 0:
        assert info.T == T and info.subkernel_num == -(-n // T)


def test_daxpy_routine_strided_host(pkg, L, orc):
    n = 40001
    x, y0 = rand_f64(2 * n, 3), rand_f64(3 * n, 4)
    for incx, incy in ((2, 3), (-2, 3), (2, -3), (1, -1)):
        bx, by = place(pkg, x, -1), place(pkg, y0, -1)
        pkg.check(L.PARALiA_daxpy(n, -1.5, bx.ptr, incx, by.ptr, incy, 7000, None), "PARALiA_daxpy strided")
        ref = y0.copy()
        orc.orc_daxpy(n, -1.5, ptr(x), incx, ptr(ref), incy)
        assert np.array_equal(by.get(), ref), (incx, incy)


@pytest.mark.parametrize("locs", [(0, 0), (-1, -1), (-1, 0), (-2, -1)])
@pytest.mark.parametrize("T", [-1, 5000, 1 << 17])
def test_ddot_routine(pkg, L, orc, openblas, locs, T):
    n = (1 << 19) + 11
    x, y = rand_f64(n, 5), rand_f64(n, 6)
    bx, by = place(pkg, x, locs[0]), place(pkg, y, locs[1])
    res = C.c_double(0.0)
    print("PARALiA ddot", n, locs, T, flush=True)
    pkg.check(L.PARALiA_ddot(n, bx.ptr, 1, by.ptr, 1, C.byref(res), T, None), "PARALiA_ddot")
    exact = float(orc.orc_ddot_longdouble(n, ptr(x), 1, ptr(y), 1))
    bound = 1e-13 * float(np.linalg.norm(x) * np.linalg.norm(y))
    assert abs(res.value - exact) <= bound
    ob = C.c_double()
    assert openblas.orc_openblas_ddot(n, ptr(x), 1, ptr(y), 1, C.byref(ob)) == 0
    assert abs(res.value - ob.value) <= bound
    if T > 0:
        tiled = C.c_double(0.0)
        orc.orc_ddot_tiled(T, n, ptr(x), 1, ptr(y), 1, C.byref(tiled))
        assert abs(res.value - tiled.value) <= bound
    # the routine adds into *result, as the reference does (ddot.cpp:431)
    first = res.value
    pkg.check(L.PARALiA_ddot(n, bx.ptr, 1, by.ptr, 1, C.byref(res), T, None), "PARALiA_ddot again")
    assert res.value == first + first


def test_blas1_edge_cases(pkg, L):
    x = rand_f64(16, 1)
    bx = place(pkg, x, -1)
    res = C.c_double(5.0)
    assert L.PARALiA_ddot(0, bx.ptr, 1, bx.ptr, 1, C.byref(res), -1, None) == 0 and res.value == 5.0
    assert L.PARALiA_daxpy(0, 1.0, bx.ptr, 1, bx.ptr, 1, -1, None) == 0
    assert L.PARALiA_daxpy(4, 1.0, bx.ptr, 0, bx.ptr, 1, -1, None) != 0 and b"increment" in L.PARALiA_last_error()
    assert L.PARALiA_daxpy(-1, 1.0, bx.ptr, 1, bx.ptr, 1, -1, None) != 0
    assert L.PARALiA_ddot(4, bx.ptr, 1, bx.ptr, 1, None, -1, None) != 0
    ones = place(pkg, np.ones(100003), -1)
    res = C.c_double(0.0)
    assert L.PARALiA_ddot(100003, ones.ptr, 1, ones.ptr, 1, C.byref(res), 1000, None) == 0 and res.value == 100003.0


def test_vec_init_matches_oracle_generator(pkg, L):
    """The drivers' seeded fill (CoCoVecInit) produces the oracle's stream wherever the buffer lives."""
    n = 100000
    for loc in (0, -1, -2):
        b = Buf(pkg, n, np.float64, loc)
        pkg.check(L.PARALiA_vec_init_f64(b.ptr, n, 42, loc), "vec init")
        assert np.array_equal(b.get(), rand_f64(n, 42))
    b = Buf(pkg, n, np.float32, 0)
    pkg.check(L.PARALiA_vec_init_f32(b.ptr, n, 7, 0), "vec init f32")
    assert np.array_equal(b.get(), rand_f32(n, 7))


@pytest.mark.parametrize("seed", range(48))
def test_random_gemm_cases(pkg, L, orc, openblas, seed):
    """Random shapes (1 .. 600, ragged tiles), transposes, operand placements (device, pinned, pageable), tile sizes
    (autotuned or preset, also larger than a dimension), padded leading dimensions, alpha / beta including 0 and
    block-pool limits below the working set, in fp64 and fp32, against OpenBLAS on the same seeded inputs."""
    rng = np.random.default_rng(500 + seed)
    dtype = np.float64 if seed % 3 else np.float32
    gen = rand_f64 if dtype == np.float64 else rand_f32
    M, N, K = (int(x) for x in rng.integers(1, 600, 3))
    ta, tb = (str(x) for x in rng.choice(["N", "T"], 2))
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + int(rng.integers(0, 9)), rb + int(rng.integers(0, 9)), M + int(rng.integers(0, 9))
    alpha = float(rng.choice([0.0, 1.0, -0.75, 1.23]))
    beta = float(rng.choice([0.0, 1.0, 0.5, -1.1]))
    locs = tuple(int(x) for x in rng.choice([-2, -1, 0], 3))
    T = int(rng.choice([-1, 32, 64, 100, 128, 256, 1024]))
    A, B, C0 = gen(lda * ca, 3 * seed), gen(ldb * cb, 3 * seed + 1), gen(ldc * N, 3 * seed + 2)
    limit = 0
    if T > 0 and min(locs) < 0 and rng.integers(0, 3) == 0:
        limit = int(rng.integers(3, 9)) * min(T, max(M, N, K)) ** 2 * np.dtype(dtype).itemsize
        L.PARALiA_dev_cache_free(0)
    bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, C0, locs[2])
    call_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, bA, lda, bB, ldb, bC, ldc, T=T, cache_limit=limit)
    got = bC.get()
    ref = openblas_ref(openblas, dtype, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    tol = TOL64 if dtype == np.float64 else TOL32
    if alpha == 0.0 and beta == 0.0:
        assert np.all(got.reshape(N, ldc)[:, :M] == 0)
    else:
        assert normwise(orc, dtype, got, ref, M, N, ldc, alpha, beta, A, ra, ca, lda, B, rb, cb, ldb, C0) < tol
    pad = np.ones(ldc * N, dtype=bool)
    pad.reshape(N, ldc)[:, :M] = False
    assert np.array_equal(got[pad], C0[pad])
    if limit:
        L.PARALiA_dev_cache_free(0)


@pytest.mark.parametrize("seed", range(40))
def test_random_blas1_cases(pkg, L, orc, seed):
    """daxpy and ddot with random lengths, increments of either sign, placements (device, pinned, pageable) and 1-D
    tile sizes: daxpy bit for bit against the oracle's fused multiply-add (gaps of strided vectors untouched), ddot
    against the long-double sum."""
    rng = np.random.default_rng(1300 + seed)
    n = int(rng.integers(1, 300000))
    incx, incy = (int(v) for v in rng.choice([1, 1, 2, 3, -1, -2], 2))
    locs = tuple(int(v) for v in rng.choice([-2, -1, 0], 2))
    T = int(rng.choice([-1, 1000, 4096, 65536, 1 << 20]))
    alpha = float(rng.choice([0.0, 1.0, -1.5, 0.7]))
    sx, sy = (n - 1) * abs(incx) + 1, (n - 1) * abs(incy) + 1
    x, y0 = rand_f64(sx, 2 * seed), rand_f64(sy, 2 * seed + 1)
    bx, by = place(pkg, x, locs[0]), place(pkg, y0, locs[1])
    print("random blas1", n, incx, incy, locs, T, alpha, flush=True)
    res = C.c_double(0.5)
    pkg.check(L.PARALiA_ddot(n, bx.ptr, incx, by.ptr, incy, C.byref(res), T, None), "PARALiA_ddot")
    exact = float(orc.orc_ddot_longdouble(n, ptr(x), incx, ptr(y0), incy))
    bound = 1e-13 * float(np.linalg.norm(x[::abs(incx)]) * np.linalg.norm(y0[::abs(incy)])) + 1e-300
    assert abs((res.value - 0.5) - exact) <= bound
    pkg.check(L.PARALiA_daxpy(n, alpha, bx.ptr, incx, by.ptr, incy, T, None), "PARALiA_daxpy")
    ref = y0.copy()
    orc.orc_daxpy(n, alpha, ptr(x), incx, ptr(ref), incy)
    assert np.array_equal(by.get(), ref)
    assert np.array_equal(bx.get(), x)


def test_command_timeline_of_a_streamed_call(pkg, L, orc, openblas):
    """PARALiA_trace_enable: every command of the plan comes back with its stream and its start / end time.  The rows
    must be the plan (one tile GEMM per subkernel, one fetch per tile of A and B, one write-back per C tile), ordered in
    time on each stream, with every GEMM starting after the fetches of its two tiles ended; and tracing must not
    change the result."""
    M, N, K, T = 700, 600, 500, 256
    A, B, C0 = rand_f64(M * K, 1), rand_f64(K * N, 2), rand_f64(M * N, 3)
    ref = openblas_ref(openblas, np.float64, "N", "N", M, N, K, 1.0, 0.0, A, M, B, K, C0, M)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, -1)
    pkg.check(L.PARALiA_trace_enable(1), "trace on")
    try:
        info = call_gemm(pkg, L, np.float64, "N", "N", M, N, K, 1.0, 0.0, bA, M, bB, K, bC, M, T=T)
        n = int(L.PARALiA_trace_read(None, 0))
        buf = (C.c_double * (7 * n))()
        assert L.PARALiA_trace_read(buf, n) == n
    finally:
        pkg.check(L.PARALiA_trace_enable(0), "trace off")
    assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 1.0, 0.0, A, M, K, M, B, K, N, K, C0) < TOL64
    rows = [tuple(buf[7 * i:7 * i + 7]) for i in range(n)]
    Mg, Ng, Kg = -(-M // T), -(-N // T), k_tiles(info, K)
    kinds = [int(r[0]) for r in rows]
    assert kinds.count(3) == Mg * Ng * Kg == info.subkernel_num
    assert kinds.count(0) == Mg * Kg and kinds.count(1) == Kg * Ng and kinds.count(2) == 0 and kinds.count(5) == Mg * Ng
    fetch_end = {}
    last_on_stream = {}
    for kind, mi, ni, ki, stream, t0, t1 in rows:
        assert 0.0 <= t0 <= t1
        assert t0 >= last_on_stream.get(stream, 0.0) - 1e-3        # a stream runs its commands in order
        last_on_stream[stream] = t1
        if kind == 0:
            fetch_end[("A", int(mi), int(ki))] = t1
        elif kind == 1:
            fetch_end[("B", int(ki), int(ni))] = t1
        elif kind == 3:
            assert t0 >= fetch_end[("A", int(mi), int(ki))] - 1e-3 and t0 >= fetch_end[("B", int(ki), int(ni))] - 1e-3
    assert int(L.PARALiA_trace_read(None, 0)) == 0                  # switched off: the rows are gone


def test_runtime_shutdown_releases_everything_and_the_next_call_starts_cold(pkg, L, orc, openblas):
    """PARALiA_runtime_shutdown (the reference's CoCoPeLiaFreeResources + PARALiADevCacheFree): pool, streams, events and
    cached problems go; device memory returns; the routines work again afterwards, every kind of them."""
    M, N, K = 640, 512, 384
    A, B, C0 = rand_f64(M * K, 4), rand_f64(K * N, 5), rand_f64(M * N, 6)
    ref = openblas_ref(openblas, np.float64, "N", "T", M, N, K, 1.5, 0.5, A, M, B, N, C0, M)
    free0, free1, total = C.c_longlong(), C.c_longlong(), C.c_longlong()
    for rep in range(2):
        bA, bB, bC = place(pkg, A, -1), place(pkg, B, -2), place(pkg, C0, -1)
        call_gemm(pkg, L, np.float64, "N", "T", M, N, K, 1.5, 0.5, bA, M, bB, N, bC, M, T=128)
        assert normwise(orc, np.float64, bC.get(), ref, M, N, M, 1.5, 0.5, A, M, K, M, B, N, K, N, C0) < TOL64
        x, y = place(pkg, rand_f64(100000, 7), -1), place(pkg, rand_f64(100000, 8), -1)
        r = C.c_double(0.0)
        pkg.check(L.PARALiA_ddot(100000, x.ptr, 1, y.ptr, 1, C.byref(r), -1, None), "ddot")
        pool, entries = C.c_longlong(), C.c_long()
        L.PARALiA_runtime_stats(None, None, C.byref(pool), C.byref(entries))
        assert pool.value > 0 and entries.value >= 2
        pkg.check(L.pl_mem_info(C.byref(free0), C.byref(total)), "mem info")
        pkg.check(L.PARALiA_runtime_shutdown(), "shutdown")
        pkg.check(L.pl_mem_info(C.byref(free1), C.byref(total)), "mem info")
        L.PARALiA_runtime_stats(None, None, C.byref(pool), C.byref(entries))
        assert pool.value == 0 and entries.value == 0
        assert free1.value >= free0.value                            # the pool and the workspaces went back
    pkg.check(L.PARALiA_runtime_shutdown(), "shutdown twice is harmless")


def test_stream_placement_probe_and_the_schedulers_own_streams(pkg, L):
    """pl_stream_shares_queue is a functional test of "runs in order with": a stream compared with itself must be found
    to share, nine streams cannot all be independent on the hardware queues of one process (HIP's default is four), and
    the first of them must find at least one other that overlaps with it.  The scheduler builds its inventory from that
    test: after a teardown, with one to three more application streams alive than before, its four busy streams are
    again on hardware queues of their own, and the results stay exact."""
    def new_stream():
        s = C.c_void_p()
        pkg.check(L.pl_stream_create(C.byref(s)), "stream")
        return s

    def shares(cand, others):
        arr = (C.c_void_p * len(others))(*[o.value for o in others])
        out = C.c_int(-1)
        pkg.check(L.pl_stream_shares_queue(cand, arr, len(others), C.byref(out)), "placement test")
        return out.value
    streams = [new_stream() for _ in range(9)]
    assert shares(streams[0], [streams[0]]) == 1
    answers = [shares(streams[0], [s]) for s in streams[1:]]
    print("  stream 0 against streams 1..8: shares =", answers, flush=True)
    assert 0 in answers and 1 in answers
    assert shares(streams[0], streams[1:]) == 1                 # one of the eight holds its queue
    M = N = K = 768
    rng = np.random.default_rng(5)
    A, B = rng.integers(-3, 4, M * K).astype(np.float64), rng.integers(-3, 4, K * N).astype(np.float64)
    ref = (A.reshape(K, M).T @ B.reshape(N, K).T).T.ravel()
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, np.zeros(M * N), -1)
    queues = int(os.environ.get("GPU_MAX_HW_QUEUES", "4") or 4)
    extra = []
    for more in range(4):
        pkg.check(L.PARALiA_runtime_shutdown(), "shutdown")
        ind, made = C.c_int(-1), C.c_int(-1)
        pkg.check(L.PARALiA_stream_queues(C.byref(ind), C.byref(made)), "stream queues")
        assert (ind.value, made.value) == (0, 0)                  # nothing held after a teardown
        call_gemm(pkg, L, np.float64, "N", "N", M, N, K, 1.0, 0.0, bA, M, bB, K, bC, M, T=128)
        assert np.array_equal(bC.get(), ref)
        pkg.check(L.PARALiA_stream_queues(C.byref(ind), C.byref(made)), "stream queues")
        print("  %d application streams alive: %d independent scheduler streams, %d created to find them" % (9 + more, ind.value, made.value), flush=True)
        assert ind.value == min(4, queues) and 4 <= made.value <= 16
        extra.append(new_stream())
    for s in streams + extra:
        pkg.check(L.pl_stream_destroy(s), "stream destroy")
    pkg.check(L.PARALiA_runtime_shutdown(), "shutdown")


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("order", [80000, 80002, 90003, 160002, 320003, 240002, 330000, 304, 10403, 80405, 250302])
@pytest.mark.parametrize("locs", [(-1, -1, -1), (-1, -1, 0), (-2, -2, -1), (0, -1, -1)])
def test_gemm_merged_k_chains_exact_on_integers(pkg, L, orc, ta, tb, order, locs, monkeypatch):
    """Order ids of 80000 and above: the k tiles of every A row panel and B column panel lie side by side on the device
    and each K chain that the order runs back to back is ONE launch over the joined k range.  Integer-valued operands,
    ragged tiles in all three dimensions (289 x 353 x 307 at T = 64: 5 x 6 x 5 tiles), every transpose (the panel of
    an operand that is contiguous along k is a K x tile matrix, the other kind a row of dense tiles), operands pinned,
    pageable or already on the device, beta = 0 over NaN and beta != 0 (fetched C, lazy reduce): bit for bit the
    untiled result, in fp64 and fp32.  Order ids of 160000 and above add the thin start: the first k tile is cut into 2
    (160000 +) or 4 (320000 +) slabs that are fetched and multiplied as k tiles of their own (7 or 9 k tiles here), alone
    or together with merged chains (240002).  Orders whose width is rows * 100 + columns (304, 10403, with merged chains
    80405, with all three 250302) start with that block of C tiles as the k-outer panel and finish tile by tile."""
    monkeypatch.setenv("PARALIA_GEMM_ORDER", str(order))
    orders = [80000, 80002, 90003, 160002, 320003, 240002, 330000, 304, 10403, 80405, 250302]
    M, N, K, T = 289, 353, 307 + orders.index(order), 64   # a new problem for the metadata cache per order
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    rng = np.random.default_rng(order + 7 * len(ta + tb))
    for dtype, brute in ((np.float64, orc.orc_dgemm_bruteforce), (np.float32, orc.orc_sgemm_bruteforce)):
        A = rng.integers(-4, 5, ra * ca).astype(dtype)
        B = rng.integers(-4, 5, rb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, M * N).astype(dtype)
        for beta in (0.0, 2.0):
            ref = C0.copy()
            brute(ta.encode(), tb.encode(), M, N, K, 3.0, ptr(A), ra, ptr(B), rb, beta, ptr(ref), M)
            start = np.full(M * N, np.nan, dtype=dtype) if beta == 0.0 else C0
            bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, start, locs[2])
            info = call_gemm(pkg, L, dtype, ta, tb, M, N, K, 3.0, beta, bA, ra, bB, rb, bC, M, T=T)
            assert info.order_id == order and info.subkernel_num == 5 * 6 * k_tiles(info, K)
            assert k_tiles(info, K) == 5 + (1, 2, 4, 4)[order // 160000] - 1
            assert np.array_equal(bC.get(), ref), (np.dtype(dtype).name, beta)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("order", [480000, 480002, 560002, 490001, 480202])
@pytest.mark.parametrize("locs", [(-1, -1, -1), (-2, -1, 0), (0, -2, -2)])
def test_gemm_graded_start_exact_on_integers(pkg, L, orc, ta, tb, order, locs, monkeypatch):
    """Order ids of 480000 and above: the graded thin start, the first k tile cut into slabs of T/8, T/8, T/4 and T/2 (T =
    128: 16, 16, 32, 64 deep; 400 = 3 k tiles + a ragged one become 7), fetched and multiplied as k tiles of their own,
    alone, with merged K chains (560002) and with a block order (480202).  Integer data, ragged tiles, every transpose,
    pinned / pageable / device operands, beta = 0 over NaN and beta != 0, both types: bit for bit the untiled result."""
    monkeypatch.setenv("PARALIA_GEMM_ORDER", str(order))
    M, N, K, T = 289, 353, 400 + [480000, 480002, 560002, 490001, 480202].index(order), 128   # a new problem for the metadata cache per order
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    rng = np.random.default_rng(order + 5 * len(ta + tb))
    for dtype, brute in ((np.float64, orc.orc_dgemm_bruteforce), (np.float32, orc.orc_sgemm_bruteforce)):
        A = rng.integers(-4, 5, ra * ca).astype(dtype)
        B = rng.integers(-4, 5, rb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, M * N).astype(dtype)
        for beta in (0.0, -2.0):
            ref = C0.copy()
            brute(ta.encode(), tb.encode(), M, N, K, 2.0, ptr(A), ra, ptr(B), rb, beta, ptr(ref), M)
            start = np.full(M * N, np.nan, dtype=dtype) if beta == 0.0 else C0
            bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, start, locs[2])
            info = call_gemm(pkg, L, dtype, ta, tb, M, N, K, 2.0, beta, bA, ra, bB, rb, bC, M, T=T)
            assert info.order_id == order and k_tiles(info, K) == 4 + 3 and info.subkernel_num == 3 * 3 * 7
            assert np.array_equal(bC.get(), ref), (np.dtype(dtype).name, beta)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("order,T", [(160001, 100), (320002, 100), (240000, 100), (160000, 72)])
def test_gemm_thin_start_with_odd_slabs(pkg, L, orc, ta, tb, order, T, monkeypatch):
    """Thin-start slabs whose depth is not a multiple of the 16-byte vector (T = 100: slabs of 50 and of 25 elements; T =
    72: 36): the tiles that follow a slab start at an odd k, so operands contiguous along k lose their alignment and the
    tile kernel takes its element-load path.  Integer data, pinned and pageable operands, both types: exact."""
    monkeypatch.setenv("PARALIA_GEMM_ORDER", str(order))
    M, N, K = 230, 310, 275 + (order % 7)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    rng = np.random.default_rng(order + T)
    for dtype, brute in ((np.float64, orc.orc_dgemm_bruteforce), (np.float32, orc.orc_sgemm_bruteforce)):
        A = rng.integers(-4, 5, ra * ca).astype(dtype)
        B = rng.integers(-4, 5, rb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, M * N).astype(dtype)
        for locs in ((-1, -1, -1), (-2, -2, -2)):
            ref = C0.copy()
            brute(ta.encode(), tb.encode(), M, N, K, 2.0, ptr(A), ra, ptr(B), rb, -1.0, ptr(ref), M)
            bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, C0, locs[2])
            info = call_gemm(pkg, L, dtype, ta, tb, M, N, K, 2.0, -1.0, bA, ra, bB, rb, bC, M, T=T)
            assert info.order_id == order and k_tiles(info, K) == -(-K // T) + (1, 2, 4, 4)[order // 160000] - 1
            assert np.array_equal(bC.get(), ref), (np.dtype(dtype).name, locs)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("order", [720000, 720001, 880001, 1200001, 720101, 640000, 650001, 800001])
@pytest.mark.parametrize("locs", [(-1, -1, -1), (-2, -1, -2), (0, 0, -1)])
def test_gemm_strip_end_exact_on_integers(pkg, L, ta, tb, order, locs, monkeypatch):
    """Order ids of 640000 and above: the last launch of the call -- on the last C tile, 700 x 76 here at T = 1024, its
    merged K chain (720000 and above) or its last k-step -- is made in two row strips of 384 and 316 rows (the merged
    chain's splitting K two ways into the workspace), and the tile's write-back (into pinned or pageable memory), with
    beta != 0 also the fetch of the caller's C and the lazy reduce, strip by strip behind them.  Alone, with a thin and
    a graded start, after a one-tile block; every transpose, A and B pinned / pageable / on the device, fp64 and fp32,
    beta = 0 over NaN and beta != 0: bit for bit the untiled result on integer operands (exact in either type,
    whatever the order of the sums)."""
    monkeypatch.setenv("PARALIA_GEMM_ORDER", str(order))
    M, N, K, T = 1724, 1100, 1200 + [720000, 720001, 880001, 1200001, 720101, 640000, 650001, 800001].index(order), 1024
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    rng = np.random.default_rng(order + 3 * len(ta + tb))
    for dtype in (np.float64, np.float32):
        A = rng.integers(-4, 5, ra * ca).astype(dtype)
        B = rng.integers(-4, 5, rb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, M * N).astype(dtype)
        opA = A.reshape(ca, ra).T.astype(np.float64) if ta == "N" else A.reshape(ca, ra).astype(np.float64)
        opB = B.reshape(cb, rb).T.astype(np.float64) if tb == "N" else B.reshape(cb, rb).astype(np.float64)
        prod = 2.0 * (opA @ opB)                                  # integers far below 2^24: exact in both types
        for beta in (0.0, -1.0):
            ref = (prod + beta * C0.reshape(N, M).T.astype(np.float64)).T.reshape(-1).astype(dtype)
            start = np.full(M * N, np.nan, dtype=dtype) if beta == 0.0 else C0
            bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, start, locs[2])
            info = call_gemm(pkg, L, dtype, ta, tb, M, N, K, 2.0, beta, bA, ra, bB, rb, bC, M, T=T)
            assert info.order_id == order and info.T == T
            assert np.array_equal(bC.get(), ref), (np.dtype(dtype).name, beta)
            if locs[2] == -1:
                # the library's own timeline of one more call: on the last tile two write-backs, behind two reduces of two
                # fetched strips of C when there is a beta
                bC.set(start)
                L.PARALiA_trace_enable(1)
                call_gemm(pkg, L, dtype, ta, tb, M, N, K, 2.0, beta, bA, ra, bB, rb, bC, M, T=T)
                n = int(L.PARALiA_trace_read(None, 0))
                buf = (C.c_double * (7 * n))()
                L.PARALiA_trace_read(buf, n)
                L.PARALiA_trace_enable(0)
                last = [int(buf[7 * i]) for i in range(n) if (int(buf[7 * i + 1]), int(buf[7 * i + 2])) == (1, 1)]
                assert (last.count(2), last.count(4), last.count(5)) == ((0, 0, 2) if beta == 0.0 else (2, 2, 2))
                assert last.count(3) == (2 if order % 160000 >= 80000 else k_tiles(info, K) + 1)
                assert np.array_equal(bC.get(), ref)


@pytest.mark.parametrize("seed", range(60))
def test_gemm_routines_random_shapes_exact_on_integers(pkg, L, seed, monkeypatch):
    """PARALiA_dgemm / PARALiA_sgemm on random problems: shapes up to 3500 x 3500 x 3000, tile sizes 256, 512, 1024 or the
    planner's, every transpose, each operand pinned, pageable or on the device, padded leading dimensions, alpha / beta
    pairs with beta = 0 over NaN; the planner's own order, or (one case in three) a pinned strip-end order.  Integer
    operands: bit for bit numpy's fp64 result, and the padding of C untouched."""
    rng = np.random.default_rng(90000 + seed)
    dtype = np.float64 if rng.integers(2) else np.float32
    ta, tb = "NT"[rng.integers(2)], "NT"[rng.integers(2)]
    T = int([256, 512, 1024, 1024, -1][rng.integers(5)])
    M, N, K = int(rng.integers(1, 3500)), int(rng.integers(1, 3500)), int(rng.integers(1, 3000))
    locs = [int([-1, -1, -2, 0][rng.integers(4)]) for _ in range(3)]
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + int(rng.integers(0, 3)) * 2, rb + int(rng.integers(0, 3)) * 2, M + int(rng.integers(0, 3)) * 2
    A = rng.integers(-3, 4, lda * ca).astype(dtype)
    B = rng.integers(-3, 4, ldb * cb).astype(dtype)
    C0 = rng.integers(-3, 4, ldc * N).astype(dtype)
    alpha, beta = [(1.0, 0.0), (2.0, -1.0), (-1.0, 1.0), (1.0, 0.0)][rng.integers(4)]
    monkeypatch.delenv("PARALIA_GEMM_ORDER", raising=False)
    if rng.integers(3) == 0 and T > 0:
        monkeypatch.setenv("PARALIA_GEMM_ORDER", str(int([720000, 720001, 650001, 880001, 640002][rng.integers(5)])))
    a = A.reshape(ca, lda)[:, :ra].T.astype(np.float64)
    b = B.reshape(cb, ldb)[:, :rb].T.astype(np.float64)
    ref = (alpha * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T)) + beta * C0.reshape(N, ldc)[:, :M].T.astype(np.float64)).T.astype(dtype)
    start = C0.copy()
    if beta == 0.0:
        start.reshape(N, ldc)[:, :M] = np.nan
    bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, start, locs[2])
    call_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, bA, lda, bB, ldb, bC, ldc, T=T)
    got = bC.get().reshape(N, ldc)
    assert np.array_equal(got[:, :M], ref)
    assert np.array_equal(got[:, M:], C0.reshape(N, ldc)[:, M:])


@pytest.mark.parametrize("seed", range(30))
def test_gemm_routines_random_unaligned_operands_exact_on_integers(pkg, L, seed):
    """PARALiA_dgemm / PARALiA_sgemm on random problems whose operands start anywhere in a 16-byte unit and have any
    leading dimension, odd ones included: one dimension of at least 2048 (where device-resident A and B are multiplied
    from aligned copies, and where products alone on the device are cut in head and tail), two calls in three with
    every operand in HBM, the others with pinned, pageable and device operands mixed; now and then the device memory is
    given back between calls.  Integer operands: bit for bit numpy's fp64 result, nothing written outside C's M x N
    elements, A and B unchanged."""
    rng = np.random.default_rng(730000 + seed)
    dtype = np.float64 if rng.integers(2) else np.float32
    ta, tb = "NT"[rng.integers(2)], "NT"[rng.integers(2)]
    T = int([512, 1024, -1, -1][rng.integers(4)])
    dims = [int(rng.integers(2048, 4400)), int(rng.integers(1, 4400)), int(rng.integers(1, 3000))]
    rng.shuffle(dims)
    M, N, K = dims
    locs = [0, 0, 0] if rng.integers(3) > 0 else [int([-1, -2, 0][rng.integers(3)]) for _ in range(3)]
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + int(rng.integers(0, 4)), rb + int(rng.integers(0, 4)), M + int(rng.integers(0, 4))
    oa, ob, oc = int(rng.integers(0, 4)), int(rng.integers(0, 4)), int(rng.integers(0, 4))
    A = rng.integers(-3, 4, lda * ca + oa).astype(dtype)
    B = rng.integers(-3, 4, ldb * cb + ob).astype(dtype)
    C0 = rng.integers(-3, 4, ldc * N + oc).astype(dtype)
    alpha, beta = [(1.0, 0.0), (2.0, -1.0), (-1.0, 1.0), (1.0, 0.0)][rng.integers(4)]
    a = A[oa:].reshape(ca, lda)[:, :ra].T.astype(np.float64)
    b = B[ob:].reshape(cb, ldb)[:, :rb].T.astype(np.float64)
    c0 = C0[oc:].reshape(N, ldc)
    ref = (alpha * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T)) + beta * c0[:, :M].T.astype(np.float64)).T.astype(dtype)
    start = C0.copy()
    if beta == 0.0:
        start[oc:].reshape(N, ldc)[:, :M] = np.nan
    bA, bB, bC = place(pkg, A, locs[0]), place(pkg, B, locs[1]), place(pkg, start, locs[2])
    info = pkg.atc_info()
    fn = L.PARALiA_dgemm if dtype == np.float64 else L.PARALiA_sgemm
    print("gemm unaligned", np.dtype(dtype).name, ta, tb, M, N, K, "T", T, "locs", locs, "ld", lda, ldb, ldc, "offsets", oa, ob, oc, alpha, beta, flush=True)
    pkg.check(fn(ta.encode(), tb.encode(), M, N, K, alpha, bA.at(oa), lda, bB.at(ob), ldb, beta, bC.at(oc), ldc, T, 0, C.byref(info)), "gemm")
    flat = bC.get()
    got = flat[oc:].reshape(N, ldc)
    assert np.array_equal(got[:, :M], ref)
    assert np.array_equal(got[:, M:], c0[:, M:]) and np.array_equal(flat[:oc], C0[:oc])
    assert np.array_equal(bA.get(), A) and np.array_equal(bB.get(), B)
    if seed % 7 == 6:
        L.PARALiA_dev_cache_free(0)


def _strided(rng, count, inc, off):
    return rng.integers(-3, 4, off + 1 + (count - 1) * abs(inc) + int(rng.integers(0, 3))).astype(np.float64)


def _view(v, count, inc, off):
    s = v[off: off + 1 + (count - 1) * abs(inc): abs(inc)]
    return s[::-1] if inc < 0 else s


@pytest.mark.parametrize("seed", range(120))
def test_blas12_routines_random_problems_exact_on_integers(pkg, L, seed):
    """PARALiA_dgemv / PARALiA_daxpy / PARALiA_ddot on random problems: any placement of every operand, increments of
    1, 2, 3 and -1, operands that start anywhere in a cache line, odd leading dimensions, preset tile sizes or the
    library's own, alpha / beta pairs with beta = 0 over NaN and alpha = 0.  Integer operands: bit for bit numpy's
    result (ddot: added to the 5.0 the result holds), nothing else written, inputs unchanged."""
    rng = np.random.default_rng(910000 + seed)
    kind = ["gemv", "gemv", "axpy", "dot"][rng.integers(4)]
    info = pkg.atc_info()
    if kind == "gemv":
        tr = "NT"[rng.integers(2)]
        M, N = int(rng.integers(1, 5000)), int(rng.integers(1, 5000))
        lda, oa = M + int(rng.integers(0, 4)), int(rng.integers(0, 3))
        incx, incy = int([1, 1, 2, -1, 3][rng.integers(5)]), int([1, 1, 2, -1][rng.integers(4)])
        ox, oy = int(rng.integers(0, 3)), int(rng.integers(0, 3))
        nx, ny = (N, M) if tr == "N" else (M, N)
        T = int([256, 512, 1000, 2048, -1, -1][rng.integers(6)])
        locs = [int([0, 0, -1, -2][rng.integers(4)]) for _ in range(3)]
        A = rng.integers(-3, 4, lda * N + oa).astype(np.float64)
        x, y0 = _strided(rng, nx, incx, ox), _strided(rng, ny, incy, oy)
        alpha, beta = [(1.0, 0.0), (2.0, -1.0), (-1.0, 1.0), (0.0, 2.0), (1.0, 1.0)][rng.integers(5)]
        a = A[oa:].reshape(N, lda)[:, :M].T
        ref = y0.copy()
        yv = _view(ref, ny, incy, oy)
        start = y0.copy()
        if beta == 0.0:
            _view(start, ny, incy, oy)[:] = np.nan
        yv[:] = alpha * ((a if tr == "N" else a.T) @ _view(x, nx, incx, ox)) + (beta * yv if beta != 0.0 else 0.0)
        bA, bx, by = place(pkg, A, locs[0]), place(pkg, x, locs[1]), place(pkg, start, locs[2])
        print("dgemv", tr, M, N, "lda", lda, "inc", incx, incy, "offsets", oa, ox, oy, "T", T, "locs", locs, alpha, beta, flush=True)
        pkg.check(L.PARALiA_dgemv(tr.encode(), M, N, alpha, bA.at(oa), lda, bx.at(ox), incx, beta, by.at(oy), incy, T, 0, C.byref(info)), "dgemv")
        assert np.array_equal(by.get(), ref) and np.array_equal(bA.get(), A) and np.array_equal(bx.get(), x)
        return
    N = int(rng.integers(1, 3_000_000)) if rng.integers(3) else int(rng.integers(1, 3000))
    incx, incy = int([1, 1, 1, 2, -1, 3][rng.integers(6)]), int([1, 1, 1, 2, -1][rng.integers(5)])
    ox, oy = int(rng.integers(0, 17)), int(rng.integers(0, 17))
    T = int([1 << 16, 100000, -1, -1][rng.integers(4)])
    locs = [int([0, 0, -1, -2][rng.integers(4)]) for _ in range(2)]
    x, y0 = _strided(rng, N, incx, ox), _strided(rng, N, incy, oy)
    bx, by = place(pkg, x, locs[0]), place(pkg, y0, locs[1])
    print(kind, N, "inc", incx, incy, "offsets", ox, oy, "T", T, "locs", locs, flush=True)
    if kind == "axpy":
        alpha = float([2.0, -1.0, 1.0, 0.0][rng.integers(4)])
        ref = y0.copy()
        _view(ref, N, incy, oy)[:] += alpha * _view(x, N, incx, ox)
        pkg.check(L.PARALiA_daxpy(N, alpha, bx.at(ox), incx, by.at(oy), incy, T, C.byref(info)), "daxpy")
        assert np.array_equal(by.get(), ref) and np.array_equal(bx.get(), x)
    else:
        res = C.c_double(5.0)
        pkg.check(L.PARALiA_ddot(N, bx.at(ox), incx, by.at(oy), incy, C.byref(res), T, C.byref(info)), "ddot")
        assert res.value == 5.0 + float(np.dot(_view(x, N, incx, ox), _view(y0, N, incy, oy)))
        assert np.array_equal(by.get(), y0) and np.array_equal(bx.get(), x)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N"), ("N", "T"), ("T", "T")])
@pytest.mark.parametrize("M,N,K,pads,offs", [(2049, 2051, 301, (0, 0, 0), (0, 0)), (2304, 2100, 500, (1, 3, 1), (0, 0)),
                                             (2200, 2300, 260, (0, 0, 0), (1, 1)), (2048, 100, 300, (1, 1, 1), (0, 0))])
def test_gemm_device_resident_operands_that_are_not_16_byte_aligned(pkg, L, ta, tb, M, N, K, pads, offs):
    """A, B and C in HBM with odd leading dimensions or starting 8 bytes (fp32: 4) into a 16-byte unit: where the other
    dimension of the product reaches 2048 the call multiplies 16-byte aligned copies of A and B with padded leading
    dimensions (the last shape, N = 100: B is copied, A is not), C is used where it lies.  Integer operands: bit for
    bit numpy's fp64 result, the padding of C untouched, and the caller's A and B unchanged."""
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + pads[0], rb + pads[1], M + pads[2]
    rng = np.random.default_rng(M + N + K)
    for dtype in (np.float64, np.float32):
        A = rng.integers(-3, 4, lda * ca + offs[0]).astype(dtype)
        B = rng.integers(-3, 4, ldb * cb + offs[1]).astype(dtype)
        C0 = rng.integers(-3, 4, ldc * N).astype(dtype)
        a = A[offs[0]:].reshape(ca, lda)[:, :ra].T.astype(np.float64)
        b = B[offs[1]:].reshape(cb, ldb)[:, :rb].T.astype(np.float64)
        ref = (2.0 * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T)) - C0.reshape(N, ldc)[:, :M].T.astype(np.float64)).T.astype(dtype)
        bA, bB, bC = place(pkg, A, 0), place(pkg, B, 0), place(pkg, C0, 0)
        info = pkg.atc_info()
        fn = L.PARALiA_dgemm if dtype == np.float64 else L.PARALiA_sgemm
        for rep in range(3):   # the second call finds the copies' buffers in place, the third allocates them again
            if rep == 2:
                L.PARALiA_dev_cache_free(0)
            bC.set(C0)
            pkg.check(fn(ta.encode(), tb.encode(), M, N, K, 2.0, bA.at(offs[0]), lda, bB.at(offs[1]), ldb, -1.0, bC.ptr, ldc, -1, 0, C.byref(info)), "gemm")
            got = bC.get().reshape(N, ldc)
            assert np.array_equal(got[:, :M], ref)
            assert np.array_equal(got[:, M:], C0.reshape(N, ldc)[:, M:])
        assert np.array_equal(bA.get(), A) and np.array_equal(bB.get(), B)


def test_sgemm_autotuned_call_merges_k_chains(pkg, L, orc, openblas):
    """No pin: for fp32 with A and B on the host the planner is offered the merged variants and its simulator takes
    one when the product is bound by compute and the chains are long (12288 x 12288 x 16384 here); parity against
    OpenBLAS."""
    M = N = 12288
    K = 16384
    A, B, C0 = rand_f32(M * K, 1), rand_f32(N * K, 2), rand_f32(M * N, 3)
    ref = openblas_ref(openblas, np.float32, "N", "T", M, N, K, 1.0, 1.0, A, M, B, N, C0, M)
    bA, bB, bC = place(pkg, A, -1), place(pkg, B, -1), place(pkg, C0, 0)
    info = call_gemm(pkg, L, np.float32, "N", "T", M, N, K, 1.0, 1.0, bA, M, bB, N, bC, M)
    print("  T", info.T, "order", info.order_id, "predicted ms", info.pred_t * 1e3, flush=True)
    assert info.order_id >= 80000
    assert normwise(orc, np.float32, bC.get(), ref, M, N, M, 1.0, 1.0, A, M, K, M, B, N, K, N, C0) < TOL32
