"""Buffers that live where the library put them (device, pinned host, pageable host) for the GPU tests."""
import ctypes as C

import numpy as np


class Buf:
    """n elements of dtype at location loc (0 device, -1 pinned host, -2 pageable host), allocated through the C ABI."""

    def __init__(self, pkg, n, dtype, loc):
        self.pkg, self.L, self.n, self.dtype, self.loc = pkg, pkg.lib(), int(n), np.dtype(dtype), loc
        self.nbytes = self.n * self.dtype.itemsize
        p = C.c_void_p()
        pkg.check(self.L.PARALiA_malloc(C.byref(p), max(self.nbytes, 8), loc), "PARALiA_malloc")
        self.ptr = p.value

    def host_view(self):
        assert self.loc < 0
        raw = (C.c_char * self.nbytes).from_address(self.ptr)
        return np.frombuffer(raw, dtype=self.dtype, count=self.n)

    def set(self, arr):
        arr = np.ascontiguousarray(arr, dtype=self.dtype).ravel()
        assert arr.size == self.n
        if self.loc < 0:
            self.host_view()[:] = arr
        else:
            self.pkg.check(self.L.pl_copy(self.ptr, arr.ctypes.data, self.nbytes), "pl_copy h2d")
        return self

    def get(self):
        if self.loc < 0:
            return self.host_view().copy()
        out = np.empty(self.n, dtype=self.dtype)
        self.pkg.check(self.L.pl_copy(out.ctypes.data, self.ptr, self.nbytes), "pl_copy d2h")
        return out

    def at(self, elem_offset):
        return self.ptr + elem_offset * self.dtype.itemsize

    def free(self):
        if self.ptr:
            self.L.PARALiA_free(self.ptr, self.loc)
            self.ptr = None

    def __del__(self):
        try:
            self.free()
        except Exception:
            pass


def sync(pkg):
    pkg.check(pkg.lib().pl_device_sync(), "device sync")


def gemm_denominator(alpha, opA_norm, opB_norm, beta, c0_norm):
    return abs(alpha) * opA_norm * opB_norm + abs(beta) * c0_norm


def check_daxpy_against_blas(orc, got, blas_result, alpha, x, y0):
    """The daxpy contract: every element within 1 ulp of the host BLAS.  A BLAS whose kernel uses a fused multiply-add
    (the builds on these machines do) is held to that plainly.  Only a BLAS that is shown, bit for bit, to round
    alpha*x before adding may differ more where the sum cancels; then the bound is 1.5 units in the last place of the
    larger operand (half a unit for the rounded product, half for each final rounding).  Prints which case applied."""
    import oracle_binding as ob
    worst = int(orc.orc_max_ulp_f64(ob.ptr(got), ob.ptr(blas_result), got.size))
    if worst <= 1:
        print("  daxpy vs host BLAS: worst distance %d ulp (plain 1-ulp contract)" % worst, flush=True)
        return worst
    unfused = y0.copy()
    orc.orc_daxpy_mul_add(got.size, alpha, ob.ptr(x), 1, ob.ptr(unfused), 1)
    assert np.array_equal(blas_result, unfused), "host BLAS result is neither within 1 ulp nor the unfused evaluation: %d ulp" % worst
    scale = np.maximum(np.maximum(np.abs(alpha * x), np.abs(y0)), np.maximum(np.abs(got), np.abs(blas_result)))
    scaled = float(np.max(np.abs(got - blas_result) / np.spacing(scale)))
    print("  daxpy vs host BLAS without fused multiply-add: worst %d ulp of the result, %.2f units of the larger operand" % (worst, scaled), flush=True)
    assert scaled <= 1.5
    return worst


def k_tiles(info, K, T=None):
    """k tiles of a streamed GEMM plan: ceil(K / T), plus the extra slabs of a thin start (order id 160000 * s + ...:
    the first k tile is cut into 2 (s = 1) or 4 (s = 2: equal, s = 3: graded) slabs that are fetched and multiplied
    separately)."""
    T = T or info.T
    return -(-K // T) + (1, 2, 4, 4)[info.order_id % 640000 // 160000] - 1
