import ctypes as C

import numpy as np

TOL = 1e-5   # the reference's tolerance: max|a-b| / max|ref| (mom6_zb/zb_host.f90:118-120, README.md:25)


def maxrel(a, ref):
    ref = np.asarray(ref, dtype=np.float64)
    return float(np.abs(np.asarray(a, dtype=np.float64) - ref).max() / np.abs(ref).max())


def bits_equal(a, b):
    a = np.ascontiguousarray(a, dtype=np.float32)
    b = np.ascontiguousarray(b, dtype=np.float32)
    return a.shape == b.shape and np.array_equal(a.view(np.uint32), b.view(np.uint32))


class DevBuf:
    """A device buffer from fortis_alloc filled from a numpy array."""

    def __init__(self, L, array=None, nbytes=None):
        self.L = L
        self.nbytes = array.nbytes if array is not None else nbytes
        self.ptr = L.fortis_alloc(self.nbytes)
        assert self.ptr, "fortis_alloc failed"
        if array is not None:
            a = np.ascontiguousarray(array)
            L.fortis_h2d(self.ptr, a.ctypes.data, a.nbytes)

    def get(self, shape, dtype=np.float32):
        out = np.empty(shape, dtype=dtype)
        self.L.fortis_d2h(out.ctypes.data, self.ptr, out.nbytes)
        return out

    def free(self):
        self.L.fortis_free(self.ptr)


def ptrs(bufs):
    return (C.c_void_p * len(bufs))(*[b.ptr for b in bufs])
