"""Parity of the hand-written HIP kernels, called through the C ABI, with the CPU oracle and OpenBLAS.
Bit-exact where the arithmetic is exact (integer-valued data, daxpy against the fused form), otherwise within the
contract's tolerances: normwise relative error <= 1e-13 (fp64) / 1e-5 (fp32) for GEMM, |err| <= 1e-13 |x||y| for ddot,
<= 1 ulp per element for daxpy."""
import contextlib
import ctypes as C
import os

import numpy as np
import pytest

from gpu_util import Buf, sync, check_daxpy_against_blas
from oracle_binding import ptr, rand_f32, rand_f64

pytestmark = pytest.mark.gpu
TOL64, TOL32 = 1e-13, 1e-5


_LARGE_TILE_BITS = {}


@contextlib.contextmanager
def large_tile(pin):
    """PARALIA_GEMM_LARGE_TILE for the calls inside: "1" forces the 256 x 256 fp32 tile (every transpose), "2" the
    256 x 128 one where it exists (NN), "0" forbids both, None leaves the choice to the kernel's cost model.  The library
    reads the variable at every launch."""
    old = os.environ.pop("PARALIA_GEMM_LARGE_TILE", None)
    if pin is not None:
        os.environ["PARALIA_GEMM_LARGE_TILE"] = pin
    try:
        yield
    finally:
        os.environ.pop("PARALIA_GEMM_LARGE_TILE", None)
        if old is not None:
            os.environ["PARALIA_GEMM_LARGE_TILE"] = old


def run_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc, a_off=0, b_off=0, c_off=0):
    dA, dB, dC = Buf(pkg, A.size, dtype, 0).set(A), Buf(pkg, B.size, dtype, 0).set(B), Buf(pkg, C0.size, dtype, 0).set(C0)
    fn = L.pl_dgemm_tile if dtype == np.float64 else L.pl_sgemm_tile
    print("gemm", dtype.__name__, ta, tb, M, N, K, alpha, beta, lda, ldb, ldc, a_off, b_off, c_off, flush=True)
    pkg.check(fn(ta.encode(), tb.encode(), M, N, K, float(alpha), dA.at(a_off), lda, dB.at(b_off), ldb, float(beta), dC.at(c_off), ldc, None), "gemm tile")
    sync(pkg)
    return dC.get()


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(256, 256, 64), (289, 353, 307), (128, 128, 16), (1, 1, 1), (130, 5, 1000), (64, 700, 3)])
def test_dgemm_tile_vs_openblas(pkg, L, orc, openblas, ta, tb, dims):
    M, N, K = dims
    alpha, beta = 1.2, 1.1
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 2, M + 6  # even leading dimensions: the 16-byte vector path
    A, B, C0 = rand_f64(lda * ca, 1), rand_f64(ldb * cb, 2), rand_f64(ldc * N, 3)
    got = run_gemm(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    ref = C0.copy()
    assert openblas.orc_openblas_dgemm(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc) == 0
    d = abs(alpha) * orc.orc_fro_norm_f64(ptr(A), ra, ca, lda) * orc.orc_fro_norm_f64(ptr(B), rb, cb, ldb) + abs(beta) * orc.orc_fro_norm_f64(ptr(C0), M, N, ldc)
    assert orc.orc_normwise_err_f64(ptr(got), ptr(ref), M, N, ldc, ldc, d) < TOL64
    bf = C0.copy()
    orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(bf), ldc)
    assert orc.orc_normwise_err_f64(ptr(got), ptr(bf), M, N, ldc, ldc, d) < TOL64
    # padding between columns untouched
    pad = np.ones(ldc * N, dtype=bool)
    pad.reshape(N, ldc)[:, :M] = False
    assert np.array_equal(got[pad], C0[pad])


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "T"), ("N", "T"), ("T", "N")])
def test_dgemm_tile_unaligned_views(pkg, L, orc, ta, tb):
    """Odd leading dimensions and operand pointers offset by one element: the element-load path."""
    M, N, K = 200, 150, 77
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 3, rb + 1, M + 1
    A, B, C0 = rand_f64(lda * ca + 1, 4), rand_f64(ldb * cb + 1, 5), rand_f64(ldc * N + 1, 6)
    got = run_gemm(pkg, L, np.float64, ta, tb, M, N, K, -0.5, 2.0, A, lda, B, ldb, C0, ldc, 1, 1, 1)
    bf = C0.copy()
    orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, -0.5, ptr(A[1:]), lda, ptr(B[1:]), ldb, 2.0, ptr(bf[1:]), ldc)
    d = 0.5 * orc.orc_fro_norm_f64(ptr(A[1:]), ra, ca, lda) * orc.orc_fro_norm_f64(ptr(B[1:]), rb, cb, ldb) + 2.0 * orc.orc_fro_norm_f64(ptr(C0[1:]), M, N, ldc)
    assert orc.orc_normwise_err_f64(ptr(got[1:]), ptr(bf[1:]), M, N, ldc, ldc, d) < TOL64
    assert got[0] == C0[0]


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
def test_dgemm_tile_exact_on_integers(pkg, L, orc, ta, tb):
    """Small-integer data: every product and partial sum is exact, so any summation order gives the same bits."""
    M, N, K = 257, 131, 300
    rng = np.random.default_rng(5)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    A = rng.integers(-8, 9, ra * ca).astype(np.float64)
    B = rng.integers(-8, 9, rb * cb).astype(np.float64)
    C0 = rng.integers(-8, 9, M * N).astype(np.float64)
    for alpha, beta in ((2.0, 3.0), (1.0, 0.0), (-1.0, 1.0)):
        got = run_gemm(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, A, ra, B, rb, C0, M)
        ref = C0.copy()
        orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), ra, ptr(B), rb, beta, ptr(ref), M)
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
def test_dgemm_tile_direct_panels_exact_on_integers(pkg, L, orc, ta, tb):
    """K of 1536 and more: every fp64 panel is requested straight into LDS (interior workgroups; the ragged edge
    workgroups of the same launch take the guarded loop).  Small integers, so the result is exact in any order."""
    M, N, K = 300, 260, 1552
    rng = np.random.default_rng(11)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 2, rb + 4, M + 2
    A = rng.integers(-8, 9, lda * ca).astype(np.float64)
    B = rng.integers(-8, 9, ldb * cb).astype(np.float64)
    C0 = rng.integers(-8, 9, ldc * N).astype(np.float64)
    for alpha, beta in ((1.0, 0.0), (-2.0, 3.0)):
        got = run_gemm(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
        ref = C0.copy()
        orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc)
        assert np.array_equal(got, ref)


@pytest.mark.parametrize("operand,extra", [("A", 0), ("A", 2), ("B", 0), ("B", 2)])
def test_dgemm_tile_k_major_operand_with_a_row_stride_of_half_a_gigabyte(pkg, L, orc, operand, extra):
    """A K-major operand whose rows are exactly 2^29 bytes apart -- the largest stride whose panels the kernel still
    requests straight into LDS (eight rows per request, 32-bit lane offsets) -- and one just beyond, where the launcher
    keeps the tile that stages through registers.  The operand spans 64 GiB of device addresses; its 128 rows of K
    values are filled by the seeded generator, whose stream the oracle reproduces on the host."""
    K, ld = 1600, (1 << 26) + extra
    M, N = (128, 256) if operand == "A" else (256, 128)
    rows = 128
    big = Buf(pkg, (rows - 1) * ld + K, np.float64, 0)
    dense = np.empty((rows, K))
    for r in range(rows):
        pkg.check(L.PARALiA_vec_init_f64(big.at(r * ld), K, 100 + r, 0), "vec init")
        dense[r] = rand_f64(K, 100 + r)
    other = rand_f64(256 * K, 7)   # the MN-major partner: 256 x K (A, TransA = N) or K x 256 read as B^T (TransB = T)
    C0 = rand_f64(M * N, 8)
    dO, dC = Buf(pkg, other.size, np.float64, 0).set(other), Buf(pkg, C0.size, np.float64, 0).set(C0)
    print("gemm f64 K-major", operand, "ld", ld, flush=True)
    if operand == "A":   # C = 1.5 A^T B^T + 0.5 C: A is K x M with lda = ld, B is N x K
        pkg.check(L.pl_dgemm_tile(b"T", b"T", M, N, K, 1.5, big.ptr, ld, dO.ptr, N, 0.5, dC.ptr, M, None), "gemm tile")
    else:                # C = 1.5 A B + 0.5 C: A is M x K, B is K x N with ldb = ld
        pkg.check(L.pl_dgemm_tile(b"N", b"N", M, N, K, 1.5, dO.ptr, M, big.ptr, ld, 0.5, dC.ptr, M, None), "gemm tile")
    sync(pkg)
    got = dC.get()
    big.free()
    ref = C0.copy()
    flat = dense.ravel()
    if operand == "A":
        orc.orc_dgemm_bruteforce(b"T", b"T", M, N, K, 1.5, ptr(flat), K, ptr(other), N, 0.5, ptr(ref), M)
        d = 1.5 * np.linalg.norm(flat) * np.linalg.norm(other) + 0.5 * np.linalg.norm(C0)
    else:
        orc.orc_dgemm_bruteforce(b"N", b"N", M, N, K, 1.5, ptr(other), M, ptr(flat), K, 0.5, ptr(ref), M)
        d = 1.5 * np.linalg.norm(other) * np.linalg.norm(flat) + 0.5 * np.linalg.norm(C0)
    assert orc.orc_normwise_err_f64(ptr(got), ptr(ref), M, N, M, M, d) < TOL64


@pytest.mark.parametrize("extra,K", [(0, 96), (0, 80), (4, 96)])
def test_sgemm_small_tile_k_major_operand_with_a_row_stride_of_a_quarter_gigabyte(pkg, L, orc, extra, K):
    """The 128 x 128 fp32 tile pinned, op(A) K-major with rows exactly 2^28 bytes apart -- the largest stride its row
    requests span (sixteen rows per request) -- and just beyond, where the launcher keeps the instantiation that stages
    through registers.  K = 96 takes the 32-deep panels (eight rows per request), K = 80 the 16-deep ones (sixteen).
    32 GiB of device addresses, 128 rows of K values filled."""
    M, N, lda = 128, 256, (1 << 26) + extra
    dA = Buf(pkg, (M - 1) * lda + K, np.float32, 0)
    dense = np.empty((M, K), dtype=np.float32)
    for r in range(M):
        pkg.check(L.PARALiA_vec_init_f32(dA.at(r * lda), K, 300 + r, 0), "vec init f32")
        dense[r] = rand_f32(K, 300 + r)
    B, C0 = rand_f32(K * N, 5), rand_f32(M * N, 6)
    dB, dC = Buf(pkg, B.size, np.float32, 0).set(B), Buf(pkg, C0.size, np.float32, 0).set(C0)
    print("gemm f32 small tile, K-major A, lda", lda, flush=True)
    with large_tile("0"):
        pkg.check(L.pl_sgemm_tile(b"T", b"N", M, N, K, 1.0, dA.ptr, lda, dB.ptr, K, 1.0, dC.ptr, M, None), "gemm tile")
    sync(pkg)
    got = dC.get()
    dA.free()
    ref = C0.copy()
    flat = dense.ravel()
    orc.orc_sgemm_bruteforce(b"T", b"N", M, N, K, 1.0, ptr(flat), K, ptr(B), K, 1.0, ptr(ref), M)
    d = float(np.linalg.norm(flat.astype(np.float64)) * np.linalg.norm(B.astype(np.float64)) + np.linalg.norm(C0.astype(np.float64)))
    assert orc.orc_normwise_err_f32(ptr(got), ptr(ref), M, N, M, M, d) < TOL32


def test_sgemm_large_tile_gives_way_to_a_row_stride_beyond_its_lane_offsets(pkg, L, orc):
    """The 256 x 256 fp32 tile pinned, op(A) K-major with rows more than 2^29 bytes apart: the launcher takes the
    small tile (and its grid), whatever the pin says."""
    M, N, K, lda = 3, 300, 600, (1 << 27) + 4
    dA = Buf(pkg, (M - 1) * lda + K, np.float32, 0)
    dense = np.empty((M, K), dtype=np.float32)
    for r in range(M):
        pkg.check(L.PARALiA_vec_init_f32(dA.at(r * lda), K, 40 + r, 0), "vec init f32")
        dense[r] = rand_f32(K, 40 + r)
    B, C0 = rand_f32(K * N, 5), rand_f32(M * N, 6)
    dB, dC = Buf(pkg, B.size, np.float32, 0).set(B), Buf(pkg, C0.size, np.float32, 0).set(C0)
    with large_tile("1"):
        pkg.check(L.pl_sgemm_tile(b"T", b"N", M, N, K, 1.0, dA.ptr, lda, dB.ptr, K, 1.0, dC.ptr, M, None), "gemm tile")
    sync(pkg)
    got = dC.get()
    ref = C0.copy()
    flat = dense.ravel()
    orc.orc_sgemm_bruteforce(b"T", b"N", M, N, K, 1.0, ptr(flat), K, ptr(B), K, 1.0, ptr(ref), M)
    d = float(np.linalg.norm(flat.astype(np.float64)) * np.linalg.norm(B.astype(np.float64)) + np.linalg.norm(C0.astype(np.float64)))
    assert orc.orc_normwise_err_f32(ptr(got), ptr(ref), M, N, M, M, d) < TOL32


@pytest.mark.parametrize("seed", range(40))
def test_gemm_tile_random_shapes_exact_on_integers(pkg, L, orc, seed):
    """Random shapes, transposes, leading dimensions, operand offsets and scalars through the tile kernels of both types,
    with whatever macro tile the launcher picks or a pinned one: k extents that are multiples of 32, of 16 only, or of
    neither, so that the 32-deep and 16-deep direct panels and the guarded loop all come up, next to ragged edge
    workgroups in the same launch.  Small integers, so the brute-force oracle must be matched bit for bit."""
    rng = np.random.default_rng(1000 + seed)
    dtype = np.float64 if seed % 2 == 0 else np.float32
    ta, tb = "NT"[rng.integers(2)], "NT"[rng.integers(2)]
    M, N = int(rng.integers(1, 420)), int(rng.integers(1, 420))
    K = int([32 * rng.integers(1, 40), 16 * (2 * rng.integers(1, 30) + 1), rng.integers(1, 700)][rng.integers(3)])
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    aligned = bool(rng.integers(2))
    pad = (lambda: 4 * int(rng.integers(0, 4))) if aligned else (lambda: int(rng.integers(0, 7)))
    lda, ldb, ldc = ra + pad(), rb + pad(), M + pad()
    off = 0 if aligned else int(rng.integers(0, 2))
    A = rng.integers(-4, 5, lda * ca + off).astype(dtype)
    B = rng.integers(-4, 5, ldb * cb + off).astype(dtype)
    C0 = rng.integers(-4, 5, ldc * N + off).astype(dtype)
    alpha, beta = [(1.0, 0.0), (2.0, -1.0), (-1.0, 1.0), (0.5, 2.0)][rng.integers(4)]
    pin = [None, "0", "1", "2"][rng.integers(4)] if dtype == np.float32 else None
    with large_tile(pin):
        got = run_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc, off, off, off)
    ref = C0.copy()
    brute = orc.orc_dgemm_bruteforce if dtype == np.float64 else orc.orc_sgemm_bruteforce
    brute(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A[off:]), lda, ptr(B[off:]), ldb, beta, ptr(ref[off:]), ldc)
    assert np.array_equal(got, ref), (dtype.__name__, ta, tb, M, N, K, lda, ldb, ldc, off, alpha, beta, pin)


def test_dgemm_tile_special_scalars(pkg, L):
    M, N, K = 100, 90, 50
    A, B, C0 = rand_f64(M * K, 1), rand_f64(K * N, 2), rand_f64(M * N, 3)
    nan_c = np.full(M * N, np.nan)
    got = run_gemm(pkg, L, np.float64, "N", "N", M, N, K, 1.0, 0.0, A, M, B, K, nan_c, M)
    assert not np.isnan(got).any()  # beta == 0 never reads C
    nan_a = np.full(M * K, np.nan)
    got = run_gemm(pkg, L, np.float64, "N", "N", M, N, K, 0.0, 0.5, nan_a, M, B, K, C0, M)
    assert np.array_equal(got, 0.5 * C0)  # alpha == 0: A and B are not referenced
    got = run_gemm(pkg, L, np.float64, "N", "N", M, N, 0, 1.0, 0.0, A, M, B, 1, C0, M)
    assert np.array_equal(got, np.zeros(M * N))  # K == 0, beta == 0: C is cleared
    got = run_gemm(pkg, L, np.float64, "N", "N", M, N, 0, 1.0, 1.0, A, M, B, 1, C0, M)
    assert np.array_equal(got, C0)
    # identity: C = alpha*B + beta*C0 with power-of-two scalars is exact
    n = 160
    I = np.eye(n).ravel()
    Bn, Cn = rand_f64(n * n, 8), rand_f64(n * n, 9)
    got = run_gemm(pkg, L, np.float64, "N", "N", n, n, n, 2.0, 0.25, I, n, Bn, n, Cn, n)
    assert np.array_equal(got, 2.0 * Bn + 0.25 * Cn)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(256, 256, 64), (289, 353, 307), (33, 1000, 129)])
def test_sgemm_tile_vs_openblas(pkg, L, orc, openblas, ta, tb, dims):
    M, N, K = dims
    alpha, beta = np.float32(1.0), np.float32(1.0)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 8, M + 4
    A, B, C0 = rand_f32(lda * ca, 1), rand_f32(ldb * cb, 2), rand_f32(ldc * N, 3)
    got = run_gemm(pkg, L, np.float32, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    ref = C0.copy()
    assert openblas.orc_openblas_sgemm(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc) == 0
    d = orc.orc_fro_norm_f32(ptr(A), ra, ca, lda) * orc.orc_fro_norm_f32(ptr(B), rb, cb, ldb) + orc.orc_fro_norm_f32(ptr(C0), M, N, ldc)
    assert orc.orc_normwise_err_f32(ptr(got), ptr(ref), M, N, ldc, ldc, d) < TOL32
    bf = C0.copy()
    orc.orc_sgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(bf), ldc)
    assert orc.orc_normwise_err_f32(ptr(got), ptr(bf), M, N, ldc, ldc, d) < TOL32


def test_sgemm_tile_exact_and_unaligned(pkg, L, orc):
    M, N, K = 150, 97, 210
    rng = np.random.default_rng(6)
    A = rng.integers(-4, 5, (M + 1) * K + 3).astype(np.float32)
    B = rng.integers(-4, 5, (N + 3) * K + 3).astype(np.float32)
    C0 = rng.integers(-4, 5, (M + 1) * N + 3).astype(np.float32)
    got = run_gemm(pkg, L, np.float32, "N", "T", M, N, K, 1.0, 1.0, A, M + 1, B, N + 3, C0, M + 1, 3, 1, 2)
    ref = C0.copy()
    orc.orc_sgemm_bruteforce(b"N", b"T", M, N, K, 1.0, ptr(A[3:]), M + 1, ptr(B[1:]), N + 3, 1.0, ptr(ref[2:]), M + 1)
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("ta,tb,pin", [("N", "N", "1"), ("N", "T", "1"), ("T", "N", "1"), ("T", "T", "1"), ("N", "N", "2")])
@pytest.mark.parametrize("dims,off", [((4096, 4096, 64), 0), ((4000, 4100, 77), 0), ((8192 + 256, 2048, 33), 0), ((4096, 4096, 40), 1),
                                      ((2048, 2304, 1056), 0)])
def test_sgemm_large_tile_exact_on_integers(pkg, L, openblas, ta, tb, dims, off, pin):
    """The 256 x 256 macro tile of fp32 (pin "1": all panels loaded straight into LDS, K-major ones in the swizzled layout
    and read in the permuted k order) and the 256 x 128 one (pin "2", NN), forced for shapes the cost model would give to
    the small tile: interior tiles, partial tiles on both edges, k not a multiple of the panel depth (the guarded loop
    writes the same LDS layouts through registers), a long k with whole panels (the pipelined loop), and operands one
    element off the 16-byte alignment (the element-load path).  Small-integer data, so OpenBLAS gives the exact bits."""
    M, N, K = dims
    rng = np.random.default_rng(11)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4 * (1 - off) + off, rb + off, M + 8 * (1 - off) + off
    A = rng.integers(-4, 5, lda * ca + off).astype(np.float32)
    B = rng.integers(-4, 5, ldb * cb + off).astype(np.float32)
    C0 = rng.integers(-4, 5, ldc * N + off).astype(np.float32)
    with large_tile(pin):
        got = run_gemm(pkg, L, np.float32, ta, tb, M, N, K, 2.0, -1.0, A, lda, B, ldb, C0, ldc, off, off, off)
    ref = C0.copy()
    assert openblas.orc_openblas_sgemm(ta.encode(), tb.encode(), M, N, K, 2.0, ptr(A[off:]), lda, ptr(B[off:]), ldb, -1.0, ptr(ref[off:]), ldc) == 0
    assert np.array_equal(got, ref)  # includes the padding between columns, which both leave alone


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("K,off", [(1536, 0), (1552, 0), (1536, 1), (96, 0), (32, 0)])
def test_sgemm_small_tile_direct_panels_exact_on_integers(pkg, L, openblas, ta, tb, K, off):
    """The 128 x 128 fp32 tile pinned: panels requested straight into LDS, 32 deep where K is a multiple of 32 (1536, 96,
    32), 16 deep otherwise (1552); interior workgroups take the pipelined loop, the ragged edge workgroups of the same
    launch and operands that are not 16-byte aligned (off = 1) the guarded one over the same LDS layouts.  Small
    integers: exact in any order, so the result must equal OpenBLAS bit for bit."""
    M, N = 300, 260
    rng = np.random.default_rng(21)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 8, M + 4
    A = rng.integers(-4, 5, lda * ca + off).astype(np.float32)
    B = rng.integers(-4, 5, ldb * cb + off).astype(np.float32)
    C0 = rng.integers(-4, 5, ldc * N + off).astype(np.float32)
    with large_tile("0"):
        got = run_gemm(pkg, L, np.float32, ta, tb, M, N, K, 2.0, -1.0, A, lda, B, ldb, C0, ldc, off, off, off)
    ref = C0.copy()
    assert openblas.orc_openblas_sgemm(ta.encode(), tb.encode(), M, N, K, 2.0, ptr(A[off:]), lda, ptr(B[off:]), ldb, -1.0, ptr(ref[off:]), ldc) == 0
    assert np.array_equal(got, ref)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("beta", [0.5, 0.0])
@pytest.mark.parametrize("pin", ["1", "2", "0", None])
def test_sgemm_large_tile_vs_openblas(pkg, L, orc, openblas, ta, tb, pin, beta):
    """Random data at 4096 x 4096 x 8192, where the kernel's cost model picks the large tile by itself (pin None).  Every
    tile is held to OpenBLAS within the fp32 tolerance.  Tiles that multiply k in the same order give the same bits:
    for NT (no K-major operand) all of them; with a K-major operand the 256 x 256 and the 128 x 128 tile both walk each
    16-deep group of k in the permuted order of their direct panels and agree, the 256 x 128 tile (NN only, panels
    staged through registers) keeps the plain order."""
    M, N, K = 4096, 4096, 8192
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    A, B, C0 = rand_f32(ra * ca, 1), rand_f32(rb * cb, 2), rand_f32(M * N, 3)
    with large_tile(pin):
        got = run_gemm(pkg, L, np.float32, ta, tb, M, N, K, 1.5, beta, A, ra, B, rb, C0, M)
    ref = C0.copy()
    assert openblas.orc_openblas_sgemm(ta.encode(), tb.encode(), M, N, K, 1.5, ptr(A), ra, ptr(B), rb, beta, ptr(ref), M) == 0
    d = 1.5 * orc.orc_fro_norm_f32(ptr(A), ra, ca, ra) * orc.orc_fro_norm_f32(ptr(B), rb, cb, rb) + beta * orc.orc_fro_norm_f32(ptr(C0), M, N, M)
    assert orc.orc_normwise_err_f32(ptr(got), ptr(ref), M, N, M, M, d) < TOL32
    same_order = "all" if (ta, tb) == ("N", "T") else ("plain" if (pin == "2" and (ta, tb) == ("N", "N")) else "permuted")
    key = (ta, tb, beta, same_order)
    if key in _LARGE_TILE_BITS:
        assert np.array_equal(got, _LARGE_TILE_BITS[key])
    _LARGE_TILE_BITS[key] = got


@pytest.mark.parametrize("n", [1, 2, 3, 1000, 100003, 1 << 22, (1 << 22) + 1])
def test_daxpy(pkg, L, orc, openblas, n):
    alpha = 0.7
    x, y0 = rand_f64(n, 1), rand_f64(n, 2)
    dx, dy = Buf(pkg, n, np.float64, 0).set(x), Buf(pkg, n, np.float64, 0).set(y0)
    print("daxpy", n, flush=True)
    pkg.check(L.pl_daxpy(n, alpha, dx.ptr, 1, dy.ptr, 1, None), "daxpy")
    sync(pkg)
    got = dy.get()
    fused = y0.copy()
    orc.orc_daxpy(n, alpha, ptr(x), 1, ptr(fused), 1)
    assert np.array_equal(got, fused)  # the kernel computes fma(alpha, x, y): one rounding, bit for bit
    ref = y0.copy()
    assert openblas.orc_openblas_daxpy(n, alpha, ptr(x), 1, ptr(ref), 1) == 0
    # contract: within 1 ulp per element of OpenBLAS (ulp of the larger operand: the sum may cancel)
    check_daxpy_against_blas(orc, got, ref, alpha, x, y0)


def test_daxpy_strided_unaligned_and_alpha_zero(pkg, L, orc):
    n = 5001
    x, y0 = rand_f64(3 * n + 1, 3), rand_f64(2 * n + 1, 4)
    dx, dy = Buf(pkg, x.size, np.float64, 0).set(x), Buf(pkg, y0.size, np.float64, 0).set(y0)
    pkg.check(L.pl_daxpy(n, 1.25, dx.at(1), 3, dy.at(1), -2, None), "daxpy strided")
    sync(pkg)
    ref = y0.copy()
    orc.orc_daxpy(n, 1.25, ptr(x[1:]), 3, ptr(ref[1:]), -2)
    assert np.array_equal(dy.get(), ref)
    dy.set(y0)
    pkg.check(L.pl_daxpy(n, 1.0, dx.at(1), 1, dy.at(1), 1, None), "daxpy unaligned")  # 8-byte aligned only
    sync(pkg)
    ref = y0.copy()
    orc.orc_daxpy(n, 1.0, ptr(x[1:]), 1, ptr(ref[1:]), 1)
    assert np.array_equal(dy.get(), ref)
    dy.set(y0)
    pkg.check(L.pl_daxpy(n, 0.0, dx.ptr, 1, dy.ptr, 1, None), "daxpy alpha 0")
    sync(pkg)
    assert np.array_equal(dy.get(), y0)


@pytest.mark.parametrize("n", [1, 2, 5, 4097, 1 << 20, (1 << 23) + 3])
def test_ddot(pkg, L, orc, openblas, n):
    x, y = rand_f64(n, 5), rand_f64(n, 6)
    dx, dy = Buf(pkg, n, np.float64, 0).set(x), Buf(pkg, n, np.float64, 0).set(y)
    ws = Buf(pkg, L.pl_ddot_workspace_doubles(), np.float64, 0)
    res = Buf(pkg, 1, np.float64, 0).set(np.array([123.0]))
    print("ddot", n, flush=True)
    pkg.check(L.pl_ddot(n, dx.ptr, 1, dy.ptr, 1, res.ptr, 0, ws.ptr, None), "ddot")
    sync(pkg)
    got = res.get()[0]
    exact = float(orc.orc_ddot_longdouble(n, ptr(x), 1, ptr(y), 1))
    bound = 1e-13 * float(np.linalg.norm(x) * np.linalg.norm(y))
    assert abs(got - exact) <= bound
    ob = C.c_double()
    assert openblas.orc_openblas_ddot(n, ptr(x), 1, ptr(y), 1, C.byref(ob)) == 0
    assert abs(got - ob.value) <= bound
    # accumulate flag adds to what is there; same input twice gives the same bits (fixed summation order)
    pkg.check(L.pl_ddot(n, dx.ptr, 1, dy.ptr, 1, res.ptr, 1, ws.ptr, None), "ddot acc")
    sync(pkg)
    assert res.get()[0] == got + got
    pkg.check(L.pl_ddot(n, dx.ptr, 1, dy.ptr, 1, res.ptr, 0, ws.ptr, None), "ddot again")
    sync(pkg)
    assert res.get()[0] == got


def test_ddot_exact_and_strided(pkg, L, orc):
    n = 123457
    ones = np.ones(n)
    d1 = Buf(pkg, n, np.float64, 0).set(ones)
    ws = Buf(pkg, L.pl_ddot_workspace_doubles(), np.float64, 0)
    res = Buf(pkg, 1, np.float64, 0)
    pkg.check(L.pl_ddot(n, d1.ptr, 1, d1.ptr, 1, res.ptr, 0, ws.ptr, None), "ddot ones")
    sync(pkg)
    assert res.get()[0] == float(n)
    m = 7001
    x, y = rand_f64(2 * m + 1, 7), rand_f64(3 * m + 1, 8)
    dx, dy = Buf(pkg, x.size, np.float64, 0).set(x), Buf(pkg, y.size, np.float64, 0).set(y)
    pkg.check(L.pl_ddot(m, dx.at(1), 2, dy.at(1), -3, res.ptr, 0, ws.ptr, None), "ddot strided")
    sync(pkg)
    exact = float(orc.orc_ddot_longdouble(m, ptr(x[1:]), 2, ptr(y[1:]), -3))
    assert abs(res.get()[0] - exact) <= 1e-13 * float(np.linalg.norm(x) * np.linalg.norm(y))
    pkg.check(L.pl_ddot(0, dx.ptr, 1, dy.ptr, 1, res.ptr, 0, ws.ptr, None), "ddot empty")
    sync(pkg)
    assert res.get()[0] == 0.0


@pytest.mark.parametrize("ox,oy", [(1, 1), (3, 3), (15, 15), (5, 21), (16, 16), (2, 4), (1, 0), (0, 7)])
@pytest.mark.parametrize("n", [1, 2, 7, 14, 15, 16, 40, 1000003])
def test_daxpy_ddot_vectors_that_start_inside_a_cache_line(pkg, L, ox, oy, n):
    """x and y starting at element ox / oy of 256-byte aligned arrays.  When both sit at the same place in their 16 bytes
    the elements in front of y's next cache line are handled one by one and the 16-byte pairs start on that line (also
    when the vector ends before it); otherwise the element kernels run.  Integer data: exact, and nothing outside the
    n elements of y is written."""
    rng = np.random.default_rng(n + 31 * ox + oy)
    X = rng.integers(-9, 10, n + 64).astype(np.float64)
    Y = rng.integers(-9, 10, n + 64).astype(np.float64)
    dx, dy = Buf(pkg, X.size, np.float64, 0).set(X), Buf(pkg, Y.size, np.float64, 0).set(Y)
    pkg.check(L.pl_daxpy(n, 3.0, dx.at(ox), 1, dy.at(oy), 1, None), "daxpy")
    sync(pkg)
    ref = Y.copy()
    ref[oy:oy + n] += 3.0 * X[ox:ox + n]
    assert np.array_equal(dy.get(), ref)
    res = Buf(pkg, 1, np.float64, 0).set(np.array([5.0]))
    ws = Buf(pkg, int(L.pl_ddot_workspace_doubles()), np.float64, 0)
    pkg.check(L.pl_ddot(n, dx.at(ox), 1, dy.at(oy), 1, res.ptr, 1, ws.ptr, None), "ddot")
    sync(pkg)
    assert res.get()[0] == 5.0 + float(np.dot(X[ox:ox + n], ref[oy:oy + n]))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_geadd(pkg, L, dtype):
    M, N = 1001, 77
    lds, lda, ldo = M + 1, M + 2, M + 3  # odd strides among them: mixed vector / element paths
    rng = np.random.default_rng(9)
    src = rng.integers(-50, 50, lds * N).astype(dtype)
    acc = rng.integers(-50, 50, lda * N).astype(dtype)
    out0 = rng.integers(-50, 50, ldo * N).astype(dtype)
    ds, da, do = Buf(pkg, src.size, dtype, 0).set(src), Buf(pkg, acc.size, dtype, 0).set(acc), Buf(pkg, out0.size, dtype, 0).set(out0)
    fn = L.pl_dgeadd_tile if dtype == np.float64 else L.pl_sgeadd_tile
    pkg.check(fn(M, N, 3.0, ds.ptr, lds, da.ptr, lda, do.ptr, ldo, None), "geadd")
    sync(pkg)
    got = do.get().reshape(N, ldo)
    ref = out0.copy().reshape(N, ldo)
    ref[:, :M] = 3.0 * src.reshape(N, lds)[:, :M] + acc.reshape(N, lda)[:, :M]
    assert np.array_equal(got, ref)
    # in place (out aliases acc), even strides: the vector path
    M2 = 1000
    acc2 = rng.integers(-50, 50, M2 * N).astype(dtype)
    src2 = rng.integers(-50, 50, M2 * N).astype(dtype)
    da2, ds2 = Buf(pkg, acc2.size, dtype, 0).set(acc2), Buf(pkg, src2.size, dtype, 0).set(src2)
    pkg.check(fn(M2, N, -2.0, ds2.ptr, M2, da2.ptr, M2, da2.ptr, M2, None), "geadd in place")
    sync(pkg)
    assert np.array_equal(da2.get(), -2.0 * src2 + acc2)


def run_gemm_ws(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc, ws_elems=None):
    """The workspace entry point; returns (result, workspace bytes the shape asked for)."""
    esz = np.dtype(dtype).itemsize
    need = int(L.pl_gemm_tile_workspace_bytes(M, N, K, esz))
    n_ws = max(1, need // esz) if ws_elems is None else ws_elems
    dA, dB, dC = Buf(pkg, A.size, dtype, 0).set(A), Buf(pkg, B.size, dtype, 0).set(B), Buf(pkg, C0.size, dtype, 0).set(C0)
    dW = Buf(pkg, n_ws, dtype, 0).set(np.full(n_ws, np.nan, dtype=dtype))      # stale workspace content must not matter
    fn = L.pl_dgemm_tile_ws if dtype == np.float64 else L.pl_sgemm_tile_ws
    print("gemm_ws", np.dtype(dtype).name, ta, tb, M, N, K, alpha, beta, lda, ldb, ldc, "workspace", need, flush=True)
    pkg.check(fn(ta.encode(), tb.encode(), M, N, K, float(alpha), dA.ptr, lda, dB.ptr, ldb, float(beta), dC.ptr, ldc, dW.ptr, n_ws * esz, None), "gemm tile ws")
    sync(pkg)
    return dC.get(), need


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(256, 256, 1024), (300, 200, 777), (128, 128, 4096), (1000, 1000, 1000), (64, 1500, 513), (130, 2, 300)])
def test_dgemm_tile_split_k_vs_openblas(pkg, L, orc, openblas, ta, tb, dims):
    """Few C tiles and a long K: K is split over several workgroups per tile and the partial products are added by a
    second kernel.  Ragged chunks (K not a multiple of the chunk), beta != 0, padded leading dimensions."""
    M, N, K = dims
    alpha, beta = 1.2, 1.1
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 2, M + 6
    A, B, C0 = rand_f64(lda * ca, 1), rand_f64(ldb * cb, 2), rand_f64(ldc * N, 3)
    got, need = run_gemm_ws(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    assert need > 0 and need % (M * N * 8) == 0 and need // (M * N * 8) >= 2
    ref = C0.copy()
    assert openblas.orc_openblas_dgemm(ta.encode(), tb.encode(), M, N, K, alpha, ptr(A), lda, ptr(B), ldb, beta, ptr(ref), ldc) == 0
    d = abs(alpha) * orc.orc_fro_norm_f64(ptr(A), ra, ca, lda) * orc.orc_fro_norm_f64(ptr(B), rb, cb, ldb) + abs(beta) * orc.orc_fro_norm_f64(ptr(C0), M, N, ldc)
    assert orc.orc_normwise_err_f64(ptr(got), ptr(ref), M, N, ldc, ldc, d) < TOL64
    pad = np.ones(ldc * N, dtype=bool)
    pad.reshape(N, ldc)[:, :M] = False
    assert np.array_equal(got[pad], C0[pad])
    # twice the same call: the slices are added in a fixed order, so the bits repeat
    again, _ = run_gemm_ws(pkg, L, np.float64, ta, tb, M, N, K, alpha, beta, A, lda, B, ldb, C0, ldc)
    assert np.array_equal(got, again)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims,splits", [((512, 700, 4096), 8), ((512, 700, 4096), 3), ((384, 76, 1201), 2), ((1024, 1024, 700), 5),
                                         ((2048, 2048, 600), 2), ((200, 300, 100), 4), ((256, 256, 2048), 1)])
def test_gemm_tile_with_the_callers_split_count(pkg, L, ta, tb, dims, splits):
    """pl_dgemm_tile_split / pl_sgemm_tile_split: K goes to the number of workgroups per tile the caller names, also for
    shapes the launcher's own model would not split (2048 x 2048 tiles fill the device), in whole panels per chunk with
    a ragged last chunk, with beta = 0 over NaN and beta != 0, padded leading dimensions; a count of 1, a K too short
    for two chunks, or a workspace under splits * M * N elements run the unsplit kernel; a count below 1 is refused.
    Integer operands (sums far below 2^24): bit for bit numpy's fp64 product, whichever way K is cut."""
    M, N, K = dims
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 8, M + 4
    rng = np.random.default_rng(M + N + K + splits)
    for dtype in (np.float64, np.float32):
        esz = np.dtype(dtype).itemsize
        fn = L.pl_dgemm_tile_split if dtype == np.float64 else L.pl_sgemm_tile_split
        A = rng.integers(-4, 5, lda * ca).astype(dtype)
        B = rng.integers(-4, 5, ldb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, ldc * N).astype(dtype)
        a = A.reshape(ca, lda)[:, :ra].T.astype(np.float64)        # the column-major operands as matrices
        b = B.reshape(cb, ldb)[:, :rb].T.astype(np.float64)
        prod = 3.0 * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T))
        dA, dB = Buf(pkg, A.size, dtype, 0).set(A), Buf(pkg, B.size, dtype, 0).set(B)
        for beta, ws_slices in ((0.0, splits), (-2.0, splits), (0.0, splits - 1)):
            n_ws = max(1, ws_slices * M * N)
            dW = Buf(pkg, n_ws, dtype, 0).set(np.full(n_ws, np.nan, dtype=dtype))
            start = np.full(ldc * N, np.nan, dtype=dtype) if beta == 0.0 else C0
            dC = Buf(pkg, start.size, dtype, 0).set(start)
            ref = (prod + beta * C0.reshape(N, ldc)[:, :M].T.astype(np.float64)).T.astype(dtype)
            print("gemm_split", np.dtype(dtype).name, ta, tb, M, N, K, "splits", splits, "workspace slices", ws_slices, "beta", beta, flush=True)
            pkg.check(fn(ta.encode(), tb.encode(), M, N, K, 3.0, dA.ptr, lda, dB.ptr, ldb, beta, dC.ptr, ldc, dW.ptr, n_ws * esz, splits, None), "gemm tile split")
            sync(pkg)
            got = dC.get().reshape(N, ldc)
            assert np.array_equal(got[:, :M], ref), (np.dtype(dtype).name, beta, ws_slices)
            if beta != 0.0:
                assert np.array_equal(got[:, M:], C0.reshape(N, ldc)[:, M:])      # the padding of C is never written
        assert fn(ta.encode(), tb.encode(), M, N, K, 3.0, dA.ptr, lda, dB.ptr, ldb, 0.0, dC.ptr, ldc, dW.ptr, n_ws * esz, 0, None) == 7      # PL_ERR_ARG, refused before any launch
        sync(pkg)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(2560, 2560, 4096), (3072, 1400, 2048), (1537, 1500, 1100), (600, 500, 700), (2560, 2560, 1200)])
def test_gemm_tile_alone_on_the_device(pkg, L, ta, tb, dims):
    """pl_dgemm_tile_alone / pl_sgemm_tile_alone: the launcher's choice for a product that has the device to itself (K
    split so that whole rounds of workgroups are filled: every shape here but the last, whose K is too short to pay),
    with the workspace it asks for, with none (unsplit), beta = 0 over NaN and beta != 0, ragged edges.  Integer operands: bit for bit numpy's
    fp64 product."""
    M, N, K = dims
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 8, M + 4
    rng = np.random.default_rng(M + N + K)
    for dtype in (np.float64, np.float32):
        esz = np.dtype(dtype).itemsize
        fn = L.pl_dgemm_tile_alone if dtype == np.float64 else L.pl_sgemm_tile_alone
        A = rng.integers(-4, 5, lda * ca).astype(dtype)
        B = rng.integers(-4, 5, ldb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, ldc * N).astype(dtype)
        a = A.reshape(ca, lda)[:, :ra].T.astype(np.float64)
        b = B.reshape(cb, ldb)[:, :rb].T.astype(np.float64)
        prod = -2.0 * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T))
        dA, dB = Buf(pkg, A.size, dtype, 0).set(A), Buf(pkg, B.size, dtype, 0).set(B)
        for beta in (0.0, 3.0):
            need = int(L.pl_gemm_tile_alone_workspace_bytes(ta.encode(), tb.encode(), M, N, K, 1 if beta == 0.0 else 0, esz))
            tm, tn, sp = C.c_int(), C.c_int(), C.c_int()
            assert L.pl_gemm_tile_choice_alone(esz, ta.encode(), tb.encode(), M, N, K, 1 if beta == 0.0 else 0, need, C.byref(tm), C.byref(tn), C.byref(sp)) == 0
            assert need == (sp.value * M * N * esz if sp.value > 1 else 0) and (sp.value > 1) == (K != 1200)
            for ws_bytes in (need, 0):
                n_ws = max(1, ws_bytes // esz)
                dW = Buf(pkg, n_ws, dtype, 0).set(np.full(n_ws, np.nan, dtype=dtype))
                start = np.full(ldc * N, np.nan, dtype=dtype) if beta == 0.0 else C0
                dC = Buf(pkg, start.size, dtype, 0).set(start)
                ref = (prod + beta * C0.reshape(N, ldc)[:, :M].T.astype(np.float64)).T.astype(dtype)
                print("gemm_alone", np.dtype(dtype).name, ta, tb, M, N, K, "splits", sp.value, "workspace", ws_bytes, "beta", beta, flush=True)
                pkg.check(fn(ta.encode(), tb.encode(), M, N, K, -2.0, dA.ptr, lda, dB.ptr, ldb, beta, dC.ptr, ldc, dW.ptr if ws_bytes else None, ws_bytes, None), "gemm tile alone")
                sync(pkg)
                assert np.array_equal(dC.get().reshape(N, ldc)[:, :M], ref), (np.dtype(dtype).name, beta, ws_bytes)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("dims", [(3072, 3072, 1024), (3000, 3010, 2050), (2816, 3534, 2048), (1408, 7222, 512)])
def test_gemm_tile_alone_cut_in_head_and_tail(pkg, L, ta, tb, dims):
    """pl_dgemm_tile_alone / pl_sgemm_tile_alone on products whose tiles do not fill whole rounds and whose K is too short
    for an even split: the first tile columns of C go out as one unsplit launch, the rest as a second launch that splits
    K (pl_gemm_tile_cut_alone says where and how).  Leading dimensions with padding, ragged M, N and K, beta = 0 over
    NaN and beta != 0, the workspace full of NaN and exactly as large as asked for.  Integer operands: bit for bit
    numpy's fp64 product, the padding of C untouched."""
    M, N, K = dims
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    lda, ldb, ldc = ra + 4, rb + 8, M + 4
    rng = np.random.default_rng(M + N + K)
    for dtype in (np.float64, np.float32):
        esz = np.dtype(dtype).itemsize
        fn = L.pl_dgemm_tile_alone if dtype == np.float64 else L.pl_sgemm_tile_alone
        A = rng.integers(-4, 5, lda * ca).astype(dtype)
        B = rng.integers(-4, 5, ldb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, ldc * N).astype(dtype)
        a = A.reshape(ca, lda)[:, :ra].T.astype(np.float64)
        b = B.reshape(cb, ldb)[:, :rb].T.astype(np.float64)
        prod = -2.0 * ((a if ta == "N" else a.T) @ (b if tb == "N" else b.T))
        dA, dB = Buf(pkg, A.size, dtype, 0).set(A), Buf(pkg, B.size, dtype, 0).set(B)
        for beta in (0.0, 3.0):
            need = int(L.pl_gemm_tile_alone_workspace_bytes(ta.encode(), tb.encode(), M, N, K, 1 if beta == 0.0 else 0, esz))
            nh, ts = C.c_long(), C.c_int()
            assert L.pl_gemm_tile_cut_alone(esz, ta.encode(), tb.encode(), M, N, K, 1 if beta == 0.0 else 0, need, C.byref(nh), C.byref(ts)) == 0
            assert ts.value > 1 and 0 < nh.value < N and nh.value % 128 == 0 and need == ts.value * M * (N - nh.value) * esz
            n_ws = need // esz
            dW = Buf(pkg, n_ws, dtype, 0).set(np.full(n_ws, np.nan, dtype=dtype))
            start = C0.copy()
            if beta == 0.0:
                start.reshape(N, ldc)[:, :M] = np.nan
            dC = Buf(pkg, start.size, dtype, 0).set(start)
            ref = (prod + beta * C0.reshape(N, ldc)[:, :M].T.astype(np.float64)).T.astype(dtype)
            print("gemm_alone_cut", np.dtype(dtype).name, ta, tb, M, N, K, "head", nh.value, "tail splits", ts.value, "beta", beta, flush=True)
            pkg.check(fn(ta.encode(), tb.encode(), M, N, K, -2.0, dA.ptr, lda, dB.ptr, ldb, beta, dC.ptr, ldc, dW.ptr, need, None), "gemm tile alone")
            sync(pkg)
            got = dC.get().reshape(N, ldc)
            assert np.array_equal(got[:, :M], ref), (np.dtype(dtype).name, beta)
            assert np.array_equal(got[:, M:], C0.reshape(N, ldc)[:, M:])


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("N", "T"), ("T", "N"), ("T", "T")])
@pytest.mark.parametrize("M,N,K,splits", [(1000, 900, 520, 0), (2047, 2047, 777, 0), (130, 140, 2000, 0), (511, 2048, 4000, 4), (300, 257, 64, 1), (129, 1, 33, 0),
                                          (2500, 2400, 1100, -1)])
def test_gemm_tile_on_operands_that_live_in_larger_blocks(pkg, L, ta, tb, M, N, K, splits):
    """pl_dgemm_tile_padded / pl_sgemm_tile_padded: the operands lie in blocks that reach up to the next multiple of 128 rows
    of op(A) and columns of op(B), and the caller says so, so the workgroups on the ragged edge of C load like interior
    ones.  What lies beyond M and N is NaN here and must not reach C; C itself has no room to spare (ldc = M, exactly
    M x N elements, NaN where beta = 0), and its result is exact on integer operands.  Also with the launcher's and the
    caller's split counts and its count for a product alone on the device (-1), a ragged K, and extents that promise less
    than M or N (refused)."""
    Mr, Nr = -(-M // 128) * 128, -(-N // 128) * 128
    rng = np.random.default_rng(M + N + K)
    for dtype in (np.float64, np.float32):
        esz = np.dtype(dtype).itemsize
        fn = L.pl_dgemm_tile_padded if dtype == np.float64 else L.pl_sgemm_tile_padded
        # op(A): Mr x K readable, M x K valid; stored M-major (ta = N: Mr x K, ld Mr) or K-major (ta = T: K x Mr, ld K + 16)
        a = rng.integers(-4, 5, (M, K)).astype(np.float64)
        b = rng.integers(-4, 5, (K, N)).astype(np.float64)
        if ta == "N":
            lda = Mr
            A = np.full((K, lda), np.nan); A[:, :M] = a.T
        else:
            lda = K + 16
            A = np.full((Mr, lda), np.nan); A[:M, :K] = a
        if tb == "N":
            ldb = K + 16
            B = np.full((Nr, ldb), np.nan); B[:N, :K] = b.T
        else:
            ldb = Nr
            B = np.full((K, ldb), np.nan); B[:, :N] = b
        C0 = rng.integers(-4, 5, (N, M)).astype(np.float64)
        dA, dB = Buf(pkg, A.size, dtype, 0).set(A.reshape(-1).astype(dtype)), Buf(pkg, B.size, dtype, 0).set(B.reshape(-1).astype(dtype))
        n_ws = max(1, max(splits, 16) * M * N)
        dW = Buf(pkg, n_ws, dtype, 0)
        for beta in (0.0, 2.0):
            start = np.full(M * N, np.nan) if beta == 0.0 else C0.reshape(-1)
            dC = Buf(pkg, M * N, dtype, 0).set(start.astype(dtype))
            print("gemm_padded", np.dtype(dtype).name, ta, tb, M, N, K, "readable", Mr, Nr, "splits", splits, "beta", beta, flush=True)
            pkg.check(fn(ta.encode(), tb.encode(), M, N, K, 3.0, dA.ptr, lda, dB.ptr, ldb, beta, dC.ptr, M, dW.ptr, n_ws * esz, splits, Mr, Nr, None), "gemm tile padded")
            sync(pkg)
            ref = (3.0 * (a @ b) + beta * C0.T).T.astype(dtype)
            assert np.array_equal(dC.get().reshape(N, M), ref), (np.dtype(dtype).name, beta)
        assert fn(ta.encode(), tb.encode(), M, N, K, 3.0, dA.ptr, lda, dB.ptr, ldb, 0.0, dC.ptr, M, dW.ptr, n_ws * esz, splits, M - 1, Nr, None) != 0
        assert fn(ta.encode(), tb.encode(), M, N, K, 3.0, dA.ptr, lda, dB.ptr, ldb, 0.0, dC.ptr, M, dW.ptr, n_ws * esz, -2, Mr, Nr, None) == 7
        sync(pkg)


@pytest.mark.parametrize("ta,tb", [("N", "N"), ("T", "N")])
def test_gemm_tile_split_k_exact_and_fallback(pkg, L, orc, ta, tb):
    """Integer-valued data: the split result equals the unsplit one bit for bit, for fp64 and fp32; beta = 0 with a
    NaN-filled C; a workspace that is too small falls back to the unsplit kernel."""
    M, N, K = 257, 131, 2048
    rng = np.random.default_rng(6)
    ra, ca = (M, K) if ta == "N" else (K, M)
    rb, cb = (K, N) if tb == "N" else (N, K)
    for dtype in (np.float64, np.float32):
        A = rng.integers(-4, 5, ra * ca).astype(dtype)
        B = rng.integers(-4, 5, rb * cb).astype(dtype)
        C0 = rng.integers(-4, 5, M * N).astype(dtype)
        for alpha, beta in ((2.0, 3.0), (1.0, 0.0)):
            Cin = np.full(M * N, np.nan, dtype=dtype) if beta == 0.0 else C0
            got, need = run_gemm_ws(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, ra, B, rb, Cin, M)
            assert need > 0
            plain = run_gemm(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, ra, B, rb, Cin, M)
            assert np.array_equal(got, plain)
            small, _ = run_gemm_ws(pkg, L, dtype, ta, tb, M, N, K, alpha, beta, A, ra, B, rb, Cin, M, ws_elems=16)
            assert np.array_equal(small, plain)
    ref = C0.astype(np.float64)
    A64, B64 = A.astype(np.float64), B.astype(np.float64)
    orc.orc_dgemm_bruteforce(ta.encode(), tb.encode(), M, N, K, 1.0, ptr(A64), ra, ptr(B64), rb, 0.0, ptr(ref), M)
    assert np.array_equal(got.astype(np.float64), ref)


def test_sgemm_tile_split_k_vs_openblas(pkg, L, orc, openblas):
    M, N, K = 384, 200, 3001
    A, B, C0 = rand_f32(M * K, 1), rand_f32(N * K, 2), rand_f32(M * N, 3)
    got, need = run_gemm_ws(pkg, L, np.float32, "N", "T", M, N, K, 0.75, -1.5, A, M, B, N, C0, M)
    assert need > 0
    ref = C0.copy()
    assert openblas.orc_openblas_sgemm(b"N", b"T", M, N, K, 0.75, ptr(A), M, ptr(B), N, -1.5, ptr(ref), M) == 0
    d = 0.75 * float(np.linalg.norm(A.astype(np.float64))) * float(np.linalg.norm(B.astype(np.float64))) + 1.5 * float(np.linalg.norm(C0.astype(np.float64)))
    assert float(np.linalg.norm(got.astype(np.float64) - ref.astype(np.float64))) / d < TOL32
