"""The stand-in that parity tests use on a machine without OpenBLAS (conftest._HostReferenceBlas): its five entry
points must agree with OpenBLAS where OpenBLAS exists, so that falling back to it weakens nothing."""
import ctypes as C

import numpy as np

import conftest
from oracle_binding import ptr, rand_f32, rand_f64


def test_stand_in_agrees_with_openblas(orc):
    ref = conftest._HostReferenceBlas(orc)
    have = orc.orc_openblas_open(None) == 0
    M, N, K = 37, 29, 53
    for ta, tb in ((b"N", b"N"), (b"T", b"N"), (b"N", b"T"), (b"T", b"T")):
        ra, ca = (M, K) if ta == b"N" else (K, M)
        rb, cb = (K, N) if tb == b"N" else (N, K)
        A, B, C0 = rand_f64(ra * ca, 1), rand_f64(rb * cb, 2), rand_f64(M * N, 3)
        c1 = C0.copy()
        assert ref.orc_openblas_dgemm(ta, tb, M, N, K, 1.2, ptr(A), ra, ptr(B), rb, 1.1, ptr(c1), M) == 0
        Am = A.reshape(ca, ra).T if ta == b"N" else A.reshape(ca, ra)
        Bm = B.reshape(cb, rb).T if tb == b"N" else B.reshape(cb, rb)
        want = 1.2 * (Am @ Bm) + 1.1 * C0.reshape(N, M).T
        assert np.allclose(c1.reshape(N, M).T, want, rtol=0, atol=1e-13)
        if have:
            c2 = C0.copy()
            assert orc.orc_openblas_dgemm(ta, tb, M, N, K, 1.2, ptr(A), ra, ptr(B), rb, 1.1, ptr(c2), M) == 0
            assert np.allclose(c1, c2, rtol=0, atol=1e-13)
        Af, Bf, Cf = rand_f32(ra * ca, 4), rand_f32(rb * cb, 5), rand_f32(M * N, 6)
        s1 = Cf.copy()
        assert ref.orc_openblas_sgemm(ta, tb, M, N, K, 0.5, ptr(Af), ra, ptr(Bf), rb, 2.0, ptr(s1), M) == 0
        if have:
            s2 = Cf.copy()
            assert orc.orc_openblas_sgemm(ta, tb, M, N, K, 0.5, ptr(Af), ra, ptr(Bf), rb, 2.0, ptr(s2), M) == 0
            assert np.allclose(s1, s2, rtol=0, atol=1e-4)
    A, x, y0 = rand_f64(M * N, 7), rand_f64(N, 8), rand_f64(M, 9)
    y1 = y0.copy()
    assert ref.orc_openblas_dgemv(b"N", M, N, 0.7, ptr(A), M, ptr(x), 1, 0.3, ptr(y1), 1) == 0
    assert np.allclose(y1, 0.7 * (A.reshape(N, M).T @ x) + 0.3 * y0, rtol=0, atol=1e-13)
    a, b = rand_f64(1001, 10), rand_f64(1001, 11)
    r = C.c_double()
    assert ref.orc_openblas_ddot(1001, ptr(a), 1, ptr(b), 1, C.byref(r)) == 0
    assert abs(r.value - float(np.dot(a.astype(np.longdouble), b.astype(np.longdouble)))) <= 1e-15 * 1001
    y = b.copy()
    assert ref.orc_openblas_daxpy(1001, 0.7, ptr(a), 1, ptr(y), 1) == 0
    if have:
        y2 = b.copy()
        assert orc.orc_openblas_daxpy(1001, 0.7, ptr(a), 1, ptr(y2), 1) == 0
        assert orc.orc_max_ulp_f64(ptr(y), ptr(y2), 1001) <= 1
    assert b"host reference" in ref.orc_openblas_path()
