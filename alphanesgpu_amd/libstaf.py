"""Host-side mirror of the MD entry (include/staf.h): what LAMMPS' pair_style staf calls through libstaf.

    model = StafModel(model_dir, precision=0)           # staf_load
    e, f, virial = model.compute(x, box, types)         # staf_compute, own minimum-image neighbour list
    e, f, virial = model.compute(x_all, box, types_all, nlocal=n, howmany=h, neigh=w)   # caller's list, ghosts

numpy in / numpy out (host pointers, as the reference's entry takes them); the GPU work happens inside the library.
"""
import ctypes as C

import numpy as np

from . import _lib

STAF_MLP_ORT, STAF_MLP_NATIVE = 0, 1

RETURN_CODES = {
    -1: "null model or pointer",
    -3: "nlocal <= 0",
    -4: "maxneigh exceeds the radial buffer",
    -7: "zero box diagonal",
    -8: "unsupported atom type",
    -9: "neighbour index out of range",
    -10: "an atom has more neighbours than Buffer_radial_descriptors",
    -11: "an atom of the caller's list is named by more than 4 x the radial buffer centres",
    -20: "GPU runtime error",
}


class StafOptions(C.Structure):
    _fields_ = [("mlp_backend", C.c_int), ("device_id", C.c_int), ("precision", C.c_int), ("reserved", C.c_int)]


class StafComputeError(RuntimeError):
    def __init__(self, code):
        self.code = code
        super().__init__(f"staf_compute returned {code}: {RETURN_CODES.get(code, 'error')}")


def _bind():
    L = _lib.lib()
    if getattr(L, "_libstaf_bound", False):
        return L
    L.staf_options_default.argtypes = [C.POINTER(StafOptions)]
    L.staf_options_default.restype = None
    L.staf_cuda_set_device.argtypes = [C.c_int]
    L.staf_load.argtypes = [C.c_char_p, C.POINTER(StafOptions)]
    L.staf_load.restype = C.c_void_p
    L.staf_free.argtypes = [C.c_void_p]
    L.staf_free.restype = None
    L.staf_compute.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                               C.c_void_p, C.c_int, C.c_void_p, C.c_void_p, C.c_void_p]
    L._libstaf_bound = True
    return L


def options_default():
    o = StafOptions()
    _bind().staf_options_default(C.byref(o))
    return o


class StafModel:
    def __init__(self, model_dir, precision=0, device_id=0, mlp_backend=STAF_MLP_NATIVE, full_virial=False,
                 host_mlp=False, eager=False):
        L = _bind()
        o = options_default()
        o.mlp_backend, o.device_id, o.precision = mlp_backend, device_id, precision
        # reserved bit 0: all six virial components; bit 1: evaluate the MLP on the host instead of on the GPU;
        # bit 2: launch every call's kernels eagerly instead of replaying a recorded HIP graph
        o.reserved = (1 if full_virial else 0) | (2 if host_mlp else 0) | (4 if eager else 0)
        self._L = L
        self._h = L.staf_load(str(model_dir).encode(), C.byref(o))
        if not self._h:
            raise RuntimeError(f"staf_load failed for {model_dir}")

    def compute(self, x, box, types=None, nlocal=None, howmany=None, neigh=None, want_virial=True):
        """x [nall,3] float64, box [6] = (Lx, xy, xz, Ly, yz, Lz), types [nall] int32 (0-based).
        Returns (energy of the owned atoms, forces [nall,3], virial [6] = xx yy zz xy xz yz); want_virial=False
        passes a null virial pointer (the virial kernels are skipped) and returns None for it."""
        x = np.ascontiguousarray(x, np.float64).reshape(-1, 3)
        box = np.ascontiguousarray(box, np.float64).reshape(6)
        nall = x.shape[0]
        nlocal = nall if nlocal is None else int(nlocal)
        nghost = nall - nlocal
        tp = None if types is None else np.ascontiguousarray(types, np.int32)
        hm = w = None
        maxneigh = 0
        if howmany is not None:
            hm = np.ascontiguousarray(howmany, np.int32)
            w = np.ascontiguousarray(neigh, np.int32).reshape(nlocal, -1)
            maxneigh = w.shape[1]
        f = np.zeros((nall, 3), np.float64)
        vir = np.zeros(6, np.float64) if want_virial else None
        e = C.c_double(0.0)
        p = lambda a: None if a is None else a.ctypes.data_as(C.c_void_p)
        rc = self._L.staf_compute(self._h, nlocal, nghost, p(x), p(box), p(tp), p(hm), p(w), maxneigh, C.byref(e),
                                  p(f), p(vir))
        if rc != 0:
            raise StafComputeError(rc)
        return e.value, f, vir

    def close(self):
        if self._h:
            self._L.staf_free(self._h)
            self._h = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass
