"""ctypes loader of libstaf_hip.so (the C-ABI library declared in include/staf_ops.h).

The product path has no fallback: if the library is missing or a call fails,
an exception is raised.
"""
import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# STAF_HIP_LIB selects another build of the same library (e.g. an experimental variant)
LIB_PATH = os.environ.get("STAF_HIP_LIB") or os.path.join(_HERE, "lib", "libstaf_hip.so")

STAF_OK = 0
ERRORS = {
    -1: "STAF_E_NOT_CONSTRUCTED: compute called before construct_descriptors_light",
    -2: "STAF_E_BAD_ARG: null pointer or bad dimension",
    -3: "STAF_E_HIP: a HIP runtime call failed",
    -10: "STAF_E_RADIAL_OVERFLOW: an atom has more neighbours than radial_buffer",
    -11: "STAF_E_SCATTER_OVERFLOW: an atom is listed by more centres than the force scatter holds",
    -12: "STAF_E_LIMIT: dimension beyond the kernels' limits, or feature not built",
    -13: "STAF_E_CAPTURE: the stream is being captured into a graph and the call would have to allocate; run the "
         "same call once outside the capture first",
    -14: "STAF_E_STALE_MAP: a force op was handed a view of a descriptor output whose intmap2b no longer holds what "
         "the descriptor op wrote, or whose first row is not the first atom of the centre species",
}


class StafError(RuntimeError):
    def __init__(self, code, where):
        self.code = code
        super().__init__(f"{where}: {ERRORS.get(code, 'error')} (code {code})")


_lib = None


def lib():
    """The loaded library.  Raises if it has not been built (python -m alphanesgpu_amd.build)."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                f"{LIB_PATH} not found: build it with `python -m alphanesgpu_amd.build` "
                "(there is no CPU or PyTorch fallback for the STAF kernels)")
        # One process holds one HIP runtime.  PyTorch ships its own copy of it under the same library name: when
        # PyTorch is going to be used in this process its copy has to be the one loaded first (this library then
        # binds to it); loaded in the other order, PyTorch finds no GPU.
        try:
            import torch  # noqa: F401
        except ImportError:
            pass
        _lib = C.CDLL(LIB_PATH)
        _lib.staf_ops_version.restype = C.c_char_p
    return _lib


def sfx(dtype):
    import torch
    if dtype == torch.float32:
        return "f32", C.c_float
    if dtype == torch.float64:
        return "f64", C.c_double
    raise TypeError(f"STAF ops support float32/float64, got {dtype}")


def call(name, *args):
    fn = getattr(lib(), name)
    fn.restype = C.c_int
    rc = fn(*args)
    if rc != STAF_OK:
        raise StafError(rc, name)
    return rc


def ptr(t):
    """Device pointer of a contiguous torch tensor (None -> NULL)."""
    if t is None:
        return C.c_void_p(0)
    if not t.is_contiguous():
        raise ValueError("STAF ops need contiguous tensors")
    return C.c_void_p(t.data_ptr())
