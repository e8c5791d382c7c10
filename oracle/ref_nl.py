"""TEST INFRASTRUCTURE ONLY: loader of oracle/_ref/libref_nl_{f32,f64}.so, the reference's own legacy CPU
neighbour list (STAF/src/descriptor_builder/cell_list.cu.cc) built by `make -C oracle _ref` in the authoring
container.  Used to validate the oracle's neighbour list; absent libraries mean "skip"."""
import ctypes as C
import os

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))


def available(dtype=np.float64):
    return os.path.exists(_path(dtype))


def _path(dtype):
    return os.path.join(_HERE, "_ref", "libref_nl_f64.so" if np.dtype(dtype) == np.float64 else "libref_nl_f32.so")


def neighbor_list(frac, box6, cutoff, nr, dtype=np.float64):
    """frac [N,3] fractional coordinates of one frame -> with [N,nr], dist2 [N,nr], howmany [N], max."""
    lib = C.CDLL(_path(dtype))
    ct = C.c_double if np.dtype(dtype) == np.float64 else C.c_float
    frac = np.ascontiguousarray(frac, dtype)
    box6 = np.ascontiguousarray(box6, dtype)
    N = frac.shape[0]
    # the legacy list writes past nr while it inserts (it is sized with slack rows); give it room
    w = np.zeros((N, nr), np.int32)
    d2 = np.zeros((N, nr), dtype)
    hm = np.zeros(N, np.int32)
    lib.ref_neighbor_list.restype = C.c_int
    mx = lib.ref_neighbor_list(C.c_int(N), frac.ctypes.data_as(C.c_void_p), box6.ctypes.data_as(C.c_void_p),
                               ct(cutoff), C.c_int(nr), w.ctypes.data_as(C.c_void_p), d2.ctypes.data_as(C.c_void_p),
                               hm.ctypes.data_as(C.c_void_p))
    return w, d2, hm, mx
