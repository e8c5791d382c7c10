"""TEST INFRASTRUCTURE ONLY: numpy front end of the CPU oracle (oracle/staf_oracle.cpp).

Loads oracle/libstaf_oracle.so with ctypes and exposes one function per
reference op on host numpy arrays.  Nothing in the product package imports
this module; only tests/, the smoke entry and the benchmark's cpu_baseline leg do.
"""
import ctypes as C
import os
import subprocess

import numpy as np

_HERE = os.path.dirname(os.path.abspath(__file__))
_LIB = None


def build(force=False):
    """Compile the oracle with g++ (see oracle/Makefile)."""
    so = os.path.join(_HERE, "libstaf_oracle.so")
    if force and os.path.exists(so):
        os.remove(so)
    subprocess.check_call(["make", "-s", "-C", _HERE, so])
    return so


def lib():
    global _LIB
    if _LIB is None:
        so = os.path.join(_HERE, "libstaf_oracle.so")
        if not os.path.exists(so):
            build()
        _LIB = C.CDLL(so)
    return _LIB


def _sfx(dtype):
    dtype = np.dtype(dtype)
    if dtype == np.float32:
        return "f32", C.c_float
    if dtype == np.float64:
        return "f64", C.c_double
    raise TypeError(dtype)


def _p(a):
    return None if a is None else a.ctypes.data_as(C.c_void_p)


def _r(a, dtype):
    return np.ascontiguousarray(a, dtype=dtype)


def _i(a):
    return np.ascontiguousarray(a, dtype=np.int32)


def _call(name, dtype, *args):
    sfx, _ = _sfx(dtype)
    fn = getattr(lib(), f"oracle_{name}_{sfx}")
    fn.restype = C.c_int
    return fn(*args)


def fill_repulsion(rc, rs, dtype=np.float64):
    """-> array [A, B, C, alpha, beta] (reforce.cc:101-141)."""
    _, ct = _sfx(dtype)
    out = np.zeros(5, dtype)
    _call("fill_repulsion", dtype, ct(rc), ct(rs), _p(out))
    return out


def cutoff_curve(rc, rs, dtype=np.float64, n=1000):
    _, ct = _sfx(dtype)
    c5 = fill_repulsion(rc, rs, dtype)
    xs = np.zeros(n, dtype)
    ys = np.zeros(n, dtype)
    _call("cutoff_curve", dtype, ct(rc), ct(rs), _p(c5), C.c_int(n), _p(xs), _p(ys))
    return xs, ys


def inverse_box(box6, dtype=np.float64):
    b = _r(box6, dtype)
    inv = np.zeros(6, dtype)
    _call("inverse_box", dtype, _p(b), _p(inv))
    return inv


def cart_to_frac(pos, box, dtype=np.float64):
    """pos [nf,3N] cart, box [nf,6] -> frac [nf,N,3]."""
    pos = _r(pos, dtype)
    box = _r(box, dtype)
    nf = box.shape[0]
    N = pos.shape[1] // 3
    frac = np.zeros((nf, N, 3), dtype)
    _call("cart_to_frac", dtype, C.c_int(nf), C.c_int(N), _p(pos), _p(box), _p(frac))
    return frac


def cell_dims(box6, cutoff, N, dtype=np.float64):
    _, ct = _sfx(dtype)
    b = _r(box6, dtype)
    out = np.zeros(3, np.int32)
    _call("cell_dims", dtype, _p(b), ct(cutoff), C.c_int(N), _p(out))
    return out


def neighbor_list(frac, box, cutoff, nr, fma_mode=0, cells=False, dtype=np.float64):
    """frac [nf,N,3], box [nf,6] -> with [nf,N,nr], dist2 [nf,N,nr], howmany [nf,N], max."""
    _, ct = _sfx(dtype)
    frac = _r(frac, dtype)
    box = _r(box, dtype)
    nf, N = frac.shape[0], frac.shape[1]
    w = np.zeros((nf, N, nr), np.int32)
    d2 = np.zeros((nf, N, nr), dtype)
    hm = np.zeros((nf, N), np.int32)
    name = "neighbor_list_cells" if cells else "neighbor_list"
    mx = _call(name, dtype, C.c_int(nf), C.c_int(N), _p(frac), _p(box), ct(cutoff), C.c_int(nr),
               C.c_int(fma_mode), _p(w), _p(d2), _p(hm))
    return w, d2, hm, mx


def compute_descriptors_light(pos, box, Rc, Ra, Rs, nr, na, fma_mode=0, dtype=np.float64):
    """The whole descriptor op.  pos [nf,3N], box [nf,6] -> dict of the 9 op outputs
    (+ 'with', 'howmany', 'max_neigh')."""
    _, ct = _sfx(dtype)
    pos = _r(pos, dtype)
    box = _r(box, dtype)
    nf = box.shape[0]
    N = pos.shape[1] // 3
    o = dict(
        raddescr=np.zeros((nf, N, nr), dtype), angdescr=np.zeros((nf, N, na), dtype),
        des3bsupp=np.zeros((nf, N, nr), dtype), intmap2b=np.zeros((nf, N, nr + 1), np.int32),
        intmap3b=np.zeros((nf, N, na * 2), np.int32), der2b=np.zeros((nf, N, 3, nr), dtype),
        der3b=np.zeros((nf, N, 3, na * 2), dtype), der3bsupp=np.zeros((nf, N, 3, nr), dtype),
        numtriplet=np.zeros((nf, N), np.int32))
    o["with"] = np.zeros((nf, N, nr), np.int32)
    o["howmany"] = np.zeros((nf, N), np.int32)
    mx = _call("compute_descriptors_light", dtype, C.c_int(nf), C.c_int(N), C.c_int(nr), C.c_int(na), _p(pos),
               _p(box), ct(Rc), ct(Ra), ct(Rs), C.c_int(fma_mode), _p(o["raddescr"]), _p(o["angdescr"]),
               _p(o["des3bsupp"]), _p(o["intmap2b"]), _p(o["intmap3b"]), _p(o["der2b"]), _p(o["der3b"]),
               _p(o["der3bsupp"]), _p(o["numtriplet"]), _p(o["with"]), _p(o["howmany"]))
    o["max_neigh"] = mx
    return o


def descriptors_from_list(frac, box, howmany, with_, Rc, Ra, Rs, nr, na, n_centres=None, skip_pbc=0,
                          dtype=np.float64):
    """Radial + angular fill from a given neighbour list (also the libstaf injected-list form:
    frac holds Npos >= n_centres atoms per frame)."""
    _, ct = _sfx(dtype)
    frac = _r(frac, dtype)
    box = _r(box, dtype)
    nf, Npos = frac.shape[0], frac.shape[1]
    N = Npos if n_centres is None else n_centres
    hm = _i(howmany)
    w = _i(with_)
    c5 = fill_repulsion(Rc, Rs, dtype)
    o = dict(
        raddescr=np.zeros((nf, N, nr), dtype), angdescr=np.zeros((nf, N, na), dtype),
        des3bsupp=np.zeros((nf, N, nr), dtype), intmap2b=np.zeros((nf, N, nr + 1), np.int32),
        intmap3b=np.zeros((nf, N, na * 2), np.int32), der2b=np.zeros((nf, N, 3, nr), dtype),
        der3b=np.zeros((nf, N, 3, na * 2), dtype), der3bsupp=np.zeros((nf, N, 3, nr), dtype),
        numtriplet=np.zeros((nf, N), np.int32))
    _call("descriptors_radial", dtype, C.c_int(nf), C.c_int(N), C.c_int(Npos), C.c_int(nr), _p(frac), _p(box),
          _p(hm), _p(w), ct(Rc), ct(Ra), ct(Rs), ct(c5[0]), ct(c5[1]), ct(c5[2]), ct(c5[3]), ct(c5[4]),
          C.c_int(skip_pbc), _p(o["raddescr"]), _p(o["intmap2b"]), _p(o["der2b"]), _p(o["des3bsupp"]),
          _p(o["der3bsupp"]), _p(o["numtriplet"]))
    _call("descriptors_angular", dtype, C.c_int(nf), C.c_int(N), C.c_int(Npos), C.c_int(nr), C.c_int(na), _p(frac),
          _p(box), _p(w), ct(Ra), _p(o["numtriplet"]), C.c_int(skip_pbc), _p(o["angdescr"]), _p(o["intmap3b"]),
          _p(o["der3b"]))
    return o


def radial_afs(raddescr, intmap2b, alpha2b, emb2b_sq, type_map):
    dtype = raddescr.dtype
    nf, Nl, nr = raddescr.shape
    Ar = alpha2b.shape[1]
    out = np.zeros((nf, Nl, Ar), dtype)
    _call("radial_afs", dtype, C.c_int(nf), C.c_int(Nl), C.c_int(nr), C.c_int(Ar), _p(_r(raddescr, dtype)),
          _p(_i(intmap2b)), _p(_r(alpha2b, dtype)), _p(_r(emb2b_sq, dtype)), _p(_i(type_map)), _p(out))
    return out


def angular_afs(angdescr, des3bsupp, intmap3b, alpha3b, emb3b_sq, type_map, numtriplet):
    dtype = angdescr.dtype
    nf, Nl, na = angdescr.shape
    nr = des3bsupp.shape[2]
    Aa = alpha3b.shape[1] // 3
    out = np.zeros((nf, Nl, Aa), dtype)
    _call("angular_afs", dtype, C.c_int(nf), C.c_int(Nl), C.c_int(nr), C.c_int(na), C.c_int(Aa),
          _p(_r(des3bsupp, dtype)), _p(_r(angdescr, dtype)), _p(_i(intmap3b)), _p(_r(alpha3b, dtype)),
          _p(_r(emb3b_sq, dtype)), _p(_i(type_map)), _p(_i(numtriplet)), _p(out))
    return out


def force_radial(netderiv, der2b, intmap2b, raddescr, alpha2b, emb2b_sq, type_map, tipos, actual_type,
                 pos=None, box=None):
    """ComputeForceRadial (pos/box None) or ComputeForceRadialVirial -> force [nf,3N] (, virial [nf,9])."""
    dtype = raddescr.dtype
    nf, Nl, nr = raddescr.shape
    N = len(type_map)
    Ar = alpha2b.shape[1]
    force = np.zeros((nf, 3 * N), dtype)
    vir = np.zeros((nf, 9), dtype) if pos is not None else None
    _call("force_doublets", dtype, C.c_int(nf), C.c_int(N), C.c_int(nr), C.c_int(Ar), _p(_r(netderiv, dtype)),
          _p(_r(raddescr, dtype)), _p(_r(der2b, dtype)), _p(_i(intmap2b)), _p(_r(alpha2b, dtype)),
          _p(_r(emb2b_sq, dtype)), _p(_i(type_map)), _p(_i(tipos)), C.c_int(actual_type), _p(force), _p(vir),
          _p(None if pos is None else _r(pos, dtype)), _p(None if box is None else _r(box, dtype)))
    return force if pos is None else (force, vir)


def force_tripl(netderiv, des3bsupp, angdescr, der3bsupp, der3b, intmap2b, intmap3b, alpha3b, emb3b_sq, type_map,
                tipos, actual_type, numtriplet, pos=None, box=None):
    dtype = angdescr.dtype
    nf, Nl, na = angdescr.shape
    nr = des3bsupp.shape[2]
    N = len(type_map)
    Aa = alpha3b.shape[1] // 3
    force = np.zeros((nf, 3 * N), dtype)
    vir = np.zeros((nf, 9), dtype) if pos is not None else None
    _call("force_tripl", dtype, C.c_int(nf), C.c_int(N), C.c_int(nr), C.c_int(na), C.c_int(Aa),
          _p(_r(netderiv, dtype)), _p(_r(des3bsupp, dtype)), _p(_r(angdescr, dtype)), _p(_r(der3bsupp, dtype)),
          _p(_r(der3b, dtype)), _p(_i(intmap3b)), _p(_r(alpha3b, dtype)), _p(_r(emb3b_sq, dtype)), _p(_i(type_map)),
          _p(_i(tipos)), C.c_int(actual_type), _p(_i(numtriplet)), _p(force), _p(vir),
          _p(None if pos is None else _r(pos, dtype)), _p(None if box is None else _r(box, dtype)))
    return force if pos is None else (force, vir)


def two_body_par_grad(prevgrad, raddescr, intmap2b, alpha2b, emb2b_sq, type_map):
    dtype = raddescr.dtype
    nf, Nl, nr = raddescr.shape
    nt, Ar = alpha2b.shape
    ga = np.zeros((nt, Ar), dtype)
    ge = np.zeros((nt, Ar), dtype)
    _call("alphagrad_dist", dtype, C.c_int(nf), C.c_int(Nl), C.c_int(nr), C.c_int(Ar), C.c_int(nt),
          _p(_r(prevgrad, dtype)), _p(_r(raddescr, dtype)), _p(_i(intmap2b)), _p(_r(alpha2b, dtype)),
          _p(_r(emb2b_sq, dtype)), _p(_i(type_map)), _p(ga), _p(ge))
    return ga, ge


def sort_proj3body_grad(prevgrad, angdescr, des3bsupp, intmap3b, intmap2b, alpha3b, emb3b_sq, type_map, numtriplet):
    dtype = angdescr.dtype
    nf, Nl, na = angdescr.shape
    nr = des3bsupp.shape[2]
    ntc = alpha3b.shape[0]
    Aa = alpha3b.shape[1] // 3
    ga = np.zeros((ntc, 3 * Aa), dtype)
    ge = np.zeros((ntc, Aa), dtype)
    _call("alphagrad_ang", dtype, C.c_int(nf), C.c_int(Nl), C.c_int(nr), C.c_int(na), C.c_int(Aa), C.c_int(ntc),
          _p(_r(prevgrad, dtype)), _p(_r(angdescr, dtype)), _p(_r(des3bsupp, dtype)), _p(_i(intmap3b)),
          _p(_r(alpha3b, dtype)), _p(_r(emb3b_sq, dtype)), _p(_i(type_map)), _p(_i(numtriplet)), _p(ga), _p(ge))
    return ga, ge


def force_radial_grad(prevgrad, netderiv, der2b, intmap2b, raddescr, alpha2b, emb2b_sq, type_map, tipos, actual_type,
                      prevgrad_virial=None, pos=None, box=None):
    dtype = raddescr.dtype
    nf, Nl, nr = raddescr.shape
    N = len(type_map)
    nt = len(tipos)
    Ar = alpha2b.shape[1]
    gn = np.zeros((nf, Nl, Ar), dtype)
    ga = np.zeros((nt, Ar), dtype)
    ge = np.zeros((nt, Ar), dtype)
    _call("gradforce_2b", dtype, C.c_int(nf), C.c_int(N), C.c_int(nr), C.c_int(Ar), C.c_int(nt),
          _p(_r(prevgrad, dtype)), _p(_r(netderiv, dtype)), _p(_r(raddescr, dtype)), _p(_r(der2b, dtype)),
          _p(_i(intmap2b)), _p(_r(alpha2b, dtype)), _p(_r(emb2b_sq, dtype)), _p(_i(type_map)), _p(_i(tipos)),
          C.c_int(actual_type), _p(gn), _p(ga), _p(ge),
          _p(None if prevgrad_virial is None else _r(prevgrad_virial, dtype)),
          _p(None if pos is None else _r(pos, dtype)), _p(None if box is None else _r(box, dtype)))
    return gn, ga, ge


def force_tripl_grad(prevgrad, netderiv, des3bsupp, angdescr, der3bsupp, der3b, intmap2b, intmap3b, alpha3b, emb3b_sq,
                     type_map, tipos, actual_type, numtriplet, prevgrad_virial=None, pos=None, box=None):
    dtype = angdescr.dtype
    nf, Nl, na = angdescr.shape
    nr = des3bsupp.shape[2]
    N = len(type_map)
    nt = len(tipos)
    ntc = nt * (nt + 1) // 2
    Aa = alpha3b.shape[1] // 3
    gn = np.zeros((nf, Nl, Aa), dtype)
    ga = np.zeros((ntc, 3 * Aa), dtype)
    ge = np.zeros((ntc, Aa), dtype)
    _call("gradforce_tripl", dtype, C.c_int(nf), C.c_int(N), C.c_int(nr), C.c_int(na), C.c_int(Aa), C.c_int(nt),
          _p(_r(prevgrad, dtype)), _p(_r(netderiv, dtype)), _p(_r(des3bsupp, dtype)), _p(_r(angdescr, dtype)),
          _p(_r(der3bsupp, dtype)), _p(_r(der3b, dtype)), _p(_i(intmap3b)), _p(_r(alpha3b, dtype)),
          _p(_r(emb3b_sq, dtype)), _p(_i(type_map)), _p(_i(tipos)), C.c_int(actual_type), _p(_i(numtriplet)), _p(gn),
          _p(ga), _p(ge), _p(None if prevgrad_virial is None else _r(prevgrad_virial, dtype)),
          _p(None if pos is None else _r(pos, dtype)), _p(None if box is None else _r(box, dtype)))
    return gn, ga, ge
