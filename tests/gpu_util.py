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
