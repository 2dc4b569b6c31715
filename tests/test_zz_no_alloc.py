"""pl_dgemv_noalloc, the entry point that allocates nothing: its partial sums live in a fixed per-device array instead
of a caller-provided workspace.  Checked through the C ABI against pl_dgemv (same kernels and summation order, so the
outputs must be bitwise equal) on two calls in a row, the second on a smaller input, so that whatever the first call
left in the shared array cannot leak into the second result."""
import ctypes as C

import numpy as np
import pytest

from gpu_util import Buf, sync

pytestmark = pytest.mark.gpu


def _case(pkg, L, trans, M, N, lda, incx, incy, alpha, beta, seed, stream):
    rng = np.random.default_rng(seed)
    len_x, len_y = (N, M) if trans == b"N" else (M, N)
    A = rng.uniform(-1, 1, lda * N)
    x = rng.uniform(-1, 1, (len_x - 1) * abs(incx) + 1)
    y0 = rng.uniform(-1, 1, (len_y - 1) * abs(incy) + 1)
    dA, dx = Buf(pkg, A.size, np.float64, 0).set(A), Buf(pkg, x.size, np.float64, 0).set(x)
    y_ref, y_new = Buf(pkg, y0.size, np.float64, 0).set(y0), Buf(pkg, y0.size, np.float64, 0).set(y0)
    need = int(L.pl_dgemv_workspace_doubles(trans, M, N))
    assert need <= int(L.pl_dgemv_noalloc_max_doubles())
    ws = Buf(pkg, max(need, 8), np.float64, 0)
    print("dgemv_noalloc case", trans, M, N, lda, incx, incy, alpha, beta, "seed", seed, flush=True)
    pkg.check(L.pl_dgemv(trans, M, N, alpha, dA.ptr, lda, dx.ptr, incx, beta, y_ref.ptr, incy, ws.ptr, stream), "pl_dgemv")
    pkg.check(L.pl_dgemv_noalloc(trans, M, N, alpha, dA.ptr, lda, dx.ptr, incx, beta, y_new.ptr, incy, stream), "pl_dgemv_noalloc")
    pkg.check(L.pl_stream_sync(stream), "sync")
    ref, got = y_ref.get(), y_new.get()
    assert np.array_equal(ref, got), float(np.abs(ref - got).max())
    # and the reference face itself is right (loose check; its own parity tests are elsewhere)
    Am = A.reshape(N, lda).T[:M, :]
    xs, ys = x[::abs(incx)], y0[::abs(incy)]
    if incx < 0:
        xs = xs[::-1]
    want = alpha * ((Am @ xs) if trans == b"N" else (Am.T @ xs)) + beta * (ys[::-1] if incy < 0 else ys)
    out = got[::abs(incy)]
    if incy < 0:
        out = out[::-1]
    assert np.allclose(out, want, rtol=0, atol=1e-11 * max(M, N))


def test_noalloc_matches_workspace_face_on_consecutive_calls(pkg, L):
    s = C.c_void_p()
    pkg.check(L.pl_stream_create(C.byref(s)), "stream")
    try:
        # large first (64 chunks x 4097 partial sums in the shared array), then smaller shapes of both kinds
        _case(pkg, L, b"N", 4096, 8192, 4100, 1, 1, 1.2, 1.1, 1, s)
        _case(pkg, L, b"N", 1000, 777, 1000, 1, 1, -0.5, 0.0, 2, s)
        _case(pkg, L, b"T", 8192, 2048, 8192, 1, 1, 1.2, 1.1, 3, s)
        _case(pkg, L, b"T", 513, 130, 515, 2, -3, 0.7, 0.3, 4, s)
        _case(pkg, L, b"N", 129, 65, 129, -1, 2, 2.0, 1.0, 5, s)
    finally:
        sync(pkg)
        pkg.check(L.pl_stream_destroy(s), "stream destroy")


def test_noalloc_refuses_shapes_beyond_its_scratch(pkg, L):
    M, N = 1 << 20, 512                       # one chunk of 2^20 + 1 partial sums: twice the fixed array
    assert int(L.pl_dgemv_workspace_doubles(b"N", M, N)) > int(L.pl_dgemv_noalloc_max_doubles())
    one = Buf(pkg, 8, np.float64, 0)
    rc = L.pl_dgemv_noalloc(b"N", M, N, 1.0, one.ptr, M, one.ptr, 1, 0.0, one.ptr, 1, None)
    assert rc == 2                            # PL_ERR_DIM, refused on the host before any launch
    assert b"pl_dgemv_noalloc" in L.pl_last_error()
    sync(pkg)
