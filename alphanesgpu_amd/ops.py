"""Host-side mirror of the reference's custom ops, on torch (ROCm) tensors.

Every function here has the name, argument order and output shapes of the
TensorFlow op it replaces (snake_case, as tf.load_op_library exposes them) and
forwards to the C-ABI library libstaf_hip.so.  torch is used for device memory
and the current stream only; all arithmetic happens in the HIP kernels.

Per-centre inputs [nf, Nl, ...] may be contiguous tensors (what tf.split gives
the reference ops) or dim-1 slices of the descriptor op's [nf, N, ...] outputs;
slices are passed through without a copy (the library takes the frame stride).
"""
import ctypes as C

import torch

from . import _lib
from ._lib import call, ptr, sfx

_I = C.c_int


def _stream():
    return C.c_void_p(torch.cuda.current_stream().cuda_stream)


def _row(t):
    n = 1
    for d in t.shape[2:]:
        n *= d
    return n


def _view_ptr(t, ld_ref=None):
    """Pointer + frame stride (in atoms) of a per-centre tensor that is contiguous or a dim-1 slice."""
    row = _row(t)
    st = t.stride()
    inner_ok = True
    acc = 1
    for d in range(t.dim() - 1, 1, -1):
        if t.shape[d] != 1 and st[d] != acc:
            inner_ok = False
        acc *= t.shape[d]
    if not inner_ok or (t.shape[1] > 1 and st[1] != row):
        raise ValueError("STAF ops need per-centre tensors that are contiguous or sliced along dim 1 only")
    if t.shape[0] > 1:
        if st[0] % row:
            raise ValueError("bad frame stride")
        ld = st[0] // row
        if ld_ref is not None and ld != ld_ref:
            raise ValueError("per-centre tensors of one call must share the frame stride")
    else:
        # one frame: the stride is never used to step, but it still tells whether the tensor is a slice of a
        # descriptor output [1, N, ...] (frame stride N), which lets the library find what it keeps for that tensor
        ld = st[0] // row if (st[0] % row == 0 and st[0] // row >= t.shape[1]) else t.shape[1]
        if ld_ref is not None:
            ld = ld_ref
    return C.c_void_p(t.data_ptr()), ld


class _Views:
    """Collects the per-centre tensors of one call and checks that they share one frame stride."""

    def __init__(self):
        self.ld = None

    def __call__(self, t):
        p, ld = _view_ptr(t, self.ld)
        self.ld = ld
        return p


def _dense(t):
    return t if t.is_contiguous() else t.contiguous()


def _i32(t):
    if t.dtype != torch.int32:
        raise TypeError("index tensors must be int32")
    return t


# --------------------------------------------------------------------------- library state


def set_sync_errors(on=True):
    """True (default): ops that can detect a device-side error synchronise and raise.  False: errors
    accumulate and are raised by poll_status()."""
    _lib.lib().staf_ops_set_sync_errors(_I(1 if on else 0))


def poll_status():
    call("staf_ops_poll_status", _stream())


def kernel_timing(on=True):
    """Brackets every kernel the library launches with HIP events on its launch stream (measurement aid)."""
    _lib.lib().staf_ops_kernel_timing(_I(1 if on else 0))


def kernel_time(kernel):
    """(summed milliseconds, launches) of the named kernel since the last call for that name; waits for the device."""
    ms, n = C.c_double(0.0), C.c_int(0)
    call("staf_ops_kernel_time", C.c_char_p(kernel.encode()), C.byref(ms), C.byref(n))
    return ms.value, n.value


def release():
    """Frees every work area the library holds on the current device (after waiting for it); the next call sizes
    them again.  Graphs captured before hold pointers into the freed areas and must not be replayed afterwards."""
    _lib.lib().staf_ops_release()


def version():
    return _lib.lib().staf_ops_version().decode()


# --------------------------------------------------------------------------- descriptor op

_constructed = {}


def construct_descriptors_light(radial_cutoff, radial_buffer, angular_buffer, numpar, boxer, rs, ra, max_batch,
                                dtype=torch.float64, cutoff_curve_path=None):
    """ConstructDescriptorsLight (STAF/src/descriptor_builder/reforce.cc:182-238).  `boxer` is accepted and
    ignored, as in the reference.  Returns the exit code tensor [0]."""
    s, ct = sfx(dtype)
    path = None if cutoff_curve_path is None else str(cutoff_curve_path).encode()
    call(f"staf_op_construct_descriptors_light_{s}", ct(float(radial_cutoff)), _I(int(radial_buffer)),
         _I(int(angular_buffer)), _I(int(numpar)), ct(float(rs)), ct(float(ra)), _I(int(max_batch)),
         C.c_char_p(path))
    _constructed[dtype] = (int(radial_buffer), int(angular_buffer))
    return torch.zeros(1, dtype=torch.int32)


def descriptor_options(dist2_fma=False, zero_padding=False):
    call("staf_op_descriptor_options", _I(int(bool(dist2_fma))), _I(int(bool(zero_padding))))


def descriptor_cell_threshold(n_atoms=4096):
    """Frames of at least n_atoms atoms search their neighbours through a cell list (same outputs)."""
    call("staf_op_descriptor_cell_threshold", _I(int(n_atoms)))


def add_n(tensors, out=None):
    """Sum of same-shaped tensors in one launch per four inputs, ((a + b) + c) + d in that order: the callers' sum of
    the per-op force arrays (force_radial + force_angular, tf.math.add_n over the species)."""
    ts = [_dense(t) for t in tensors]
    if len(ts) == 1:
        return ts[0].clone() if out is None else out.copy_(ts[0])
    s, _ = sfx(ts[0].dtype)
    out = torch.empty_like(ts[0]) if out is None else out
    acc = None
    while ts:
        group = ([acc] if acc is not None else []) + ts[:4 - (acc is not None)]
        ts = ts[4 - (acc is not None):]
        group += [None] * (4 - len(group))
        call(f"staf_op_add_n_{s}", ptr(out), ptr(group[0]), ptr(group[1]), ptr(group[2]), ptr(group[3]),
             _I(out.numel()), _stream())
        acc = out
    return out


def descriptor_coefficients(dtype=torch.float64):
    s, ct = sfx(dtype)
    out = (ct * 5)()
    call(f"staf_op_descriptor_coefficients_{s}", out)
    return [float(v) for v in out]


def compute_descriptors_light(positions, boxer, out=None):
    """ComputeDescriptorsLight (reforce.cc:241-444): positions [nf,3N], boxer [nf,6] ->
    (raddescr, angdescr, des3bsupp, intmap2b, intmap3b, der2b, der3b, der3bsupp, numtriplet)."""
    dtype = positions.dtype
    s, _ = sfx(dtype)
    if dtype not in _constructed:
        raise _lib.StafError(-1, "compute_descriptors_light")
    nr, na = _constructed[dtype]
    positions = _dense(positions)
    boxer = _dense(boxer)
    nf = boxer.shape[0]
    N = positions.shape[1] // 3
    dev = positions.device
    if out is None:
        e = lambda *sh: torch.empty(sh, dtype=dtype, device=dev)
        ei = lambda *sh: torch.empty(sh, dtype=torch.int32, device=dev)
        out = (e(nf, N, nr), e(nf, N, na), e(nf, N, nr), ei(nf, N, nr + 1), ei(nf, N, 2 * na), e(nf, N, 3, nr),
               e(nf, N, 3, 2 * na), e(nf, N, 3, nr), ei(nf, N))
    raddescr, angdescr, des3bsupp, intmap2b, intmap3b, der2b, der3b, der3bsupp, numtriplet = out
    call(f"staf_op_compute_descriptors_light_{s}", ptr(positions), ptr(boxer), _I(nf), _I(N), ptr(raddescr),
         ptr(angdescr), ptr(des3bsupp), ptr(intmap2b), ptr(intmap3b), ptr(der2b), ptr(der3b), ptr(der3bsupp),
         ptr(numtriplet), _stream())
    return out


def compute_descriptors_fingerprints(positions, boxer, type_map, n_local, alpha3b_parameters, type_emb3b_parameters,
                                     alpha2b_parameters=None, type_emb2b_parameters=None, out=None, species=None):
    """Descriptors and the fingerprints of every centre species in one launch (no counterpart as one op in the
    reference): what compute_descriptors_light(positions, boxer) returns, then, per species k (n_local[k] atoms,
    species-sorted, summing to N), three_body_afs[k] [nf,n_local[k],Aa] as compute_sort_proj3body gives it for the
    species' rows with alpha3b_parameters[k], type_emb3b_parameters[k] and -- if the 2-body parameter lists are
    given -- radial_afs[k] [nf,n_local[k],Ar] as compute_sort_proj gives it, same bits.
    species = (first, count): only the centres of these species (the descriptor rows of the others are not touched
    and their entries of the returned lists are None): one call per species, each on a stream of its own, lets the ops that follow a species'
    fingerprints start when that species is through.
    -> (descriptor tuple, [three_body_afs[k]], [radial_afs[k]] or None)."""
    dtype = positions.dtype
    s, _ = sfx(dtype)
    if dtype not in _constructed:
        raise _lib.StafError(-1, "compute_descriptors_fingerprints")
    nr, na = _constructed[dtype]
    positions = _dense(positions)
    boxer = _dense(boxer)
    nf = boxer.shape[0]
    N = positions.shape[1] // 3
    dev = positions.device
    nt = len(n_local)
    e = lambda *sh: torch.empty(sh, dtype=dtype, device=dev)
    ei = lambda *sh: torch.empty(sh, dtype=torch.int32, device=dev)
    if out is None:
        out = (e(nf, N, nr), e(nf, N, na), e(nf, N, nr), ei(nf, N, nr + 1), ei(nf, N, 2 * na), e(nf, N, 3, nr),
               e(nf, N, 3, 2 * na), e(nf, N, 3, nr), ei(nf, N))
    raddescr, angdescr, des3bsupp, intmap2b, intmap3b, der2b, der3b, der3bsupp, numtriplet = out
    a3 = [_dense(t) for t in alpha3b_parameters]
    e3 = [_dense(t) for t in type_emb3b_parameters]
    Aa = e3[0].shape[1]
    first, count = (0, nt) if species is None else species
    mine = lambda k: first <= k < first + count
    af3 = [e(nf, int(n), Aa) if mine(k) else None for k, n in enumerate(n_local)]   # (None: not one of `species`)
    with2 = alpha2b_parameters is not None
    a2 = [_dense(t) for t in alpha2b_parameters] if with2 else []
    e2 = [_dense(t) for t in type_emb2b_parameters] if with2 else []
    Ar = e2[0].shape[1] if with2 else 0
    af2 = [e(nf, int(n), Ar) if mine(k) else None for k, n in enumerate(n_local)] if with2 else None
    arr = lambda ts: (C.c_void_p * nt)(*[None if t is None else t.data_ptr() for t in ts]) if ts else None
    tm = _i32(type_map)
    call(f"staf_op_descriptors_fingerprints_{s}", ptr(positions), ptr(boxer), _I(nf), _I(N), ptr(raddescr),
         ptr(angdescr), ptr(des3bsupp), ptr(intmap2b), ptr(intmap3b), ptr(der2b), ptr(der3b), ptr(der3bsupp),
         ptr(numtriplet), _I(nt), (C.c_int * nt)(*[int(n) for n in n_local]), _I(first), _I(count), ptr(tm), _I(Aa), arr(a3), arr(e3),
         arr(af3), _I(Ar), arr(a2), arr(e2), arr(af2 or []), _stream())
    return out, af3, af2


# --------------------------------------------------------------------------- fingerprints


def compute_sort_proj(radial_descriptor, interaction_map_rad, alpha2b_parameters, type_emb2b_parameters, type_map):
    """ComputeSortProj (STAF/src/fingerprint/rad/reforce.cc:13-19) -> two_body_afs [nf,Nl,Ar]."""
    dtype = radial_descriptor.dtype
    s, _ = sfx(dtype)
    nf, Nl, nr = radial_descriptor.shape
    nt, Ar = alpha2b_parameters.shape
    v = _Views()
    pD = v(radial_descriptor)
    pI = v(_i32(interaction_map_rad))
    out = torch.empty((nf, Nl, Ar), dtype=dtype, device=radial_descriptor.device)
    call(f"staf_op_radial_afs_{s}", pD, _I(nr), ptr(_dense(alpha2b_parameters)), _I(Ar), ptr(out), _I(nf), _I(Nl),
         pI, ptr(_dense(type_emb2b_parameters)), ptr(_i32(type_map)), _I(nt), _I(v.ld), _stream())
    return out


def compute_sort_proj3body(angular_descriptor, radial_descriptor, interaction_map_angular, interaction_map_rad,
                           alpha3b_parameters, type_emb3b_parameters, type_map, num_triplet, nt=None):
    """ComputeSortProj3body (STAF/src/fingerprint/ang/reforce.cc:15-24) -> three_body_afs [nf,Nl,Aa].
    radial_descriptor is des3bsupp.  nt defaults to the number of species implied by the rows of alpha3b."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    ntc = alpha3b_parameters.shape[0]
    Aa = alpha3b_parameters.shape[1] // 3
    nt = _nt_from_ntc(ntc) if nt is None else nt
    v = _Views()
    pT = v(angular_descriptor)
    pD = v(radial_descriptor)
    pI3 = v(_i32(interaction_map_angular))
    pI2 = v(_i32(interaction_map_rad))
    pN = v(_i32(num_triplet))
    out = torch.empty((nf, Nl, Aa), dtype=dtype, device=angular_descriptor.device)
    call(f"staf_op_angular_afs_{s}", pD, pT, _I(nr), _I(na), ptr(out), _I(nf), _I(Nl), pI3, pI2,
         ptr(_dense(alpha3b_parameters)), _I(Aa), ptr(_dense(type_emb3b_parameters)), ptr(_i32(type_map)), pN,
         _I(nt), _I(v.ld), _stream())
    return out


def _nt_from_ntc(ntc):
    nt = 1
    while nt * (nt + 1) // 2 < ntc:
        nt += 1
    if nt * (nt + 1) // 2 != ntc:
        raise ValueError(f"{ntc} rows is not nt(nt+1)/2 for any nt")
    return nt


# --------------------------------------------------------------------------- forces


def init_force_radial(buffdim):
    call("staf_op_init_force_radial", _I(int(buffdim)))
    return torch.zeros(1, dtype=torch.int32)


def init_force_tripl(buffdim):
    call("staf_op_init_force_tripl", _I(int(buffdim)))
    return torch.zeros(1, dtype=torch.int32)


def init_grad_force_radial(buffdim):
    call("staf_op_init_grad_force_radial", _I(int(buffdim)))
    return torch.zeros(1, dtype=torch.int32)


def init_grad_force_tripl(buffdim):
    call("staf_op_init_grad_force_tripl", _I(int(buffdim)))
    return torch.zeros(1, dtype=torch.int32)


def _scalar_dev(x, device):
    if torch.is_tensor(x):
        return _i32(x).reshape(-1).to(device)
    return torch.tensor([int(x)], dtype=torch.int32, device=device)


def compute_force_radial(netderiv, descriptor_derivative_rad, interaction_map_rad, radial_descriptor,
                         alpha2b_parameters, type_emb2b_parameters, type_map, tipos, actual_type, pos=None, box=None):
    """ComputeForceRadial (STAF/src/force/rad/reforce.cc:39-49) -> force [nf,3N]; with pos/box:
    ComputeForceRadialVirial (:133-146) -> (force, virial [nf,9])."""
    dtype = radial_descriptor.dtype
    s, _ = sfx(dtype)
    dev = radial_descriptor.device
    nf, Nl, nr = radial_descriptor.shape
    N = type_map.shape[0]
    nt, Ar = alpha2b_parameters.shape
    v = _Views()
    pdD = v(descriptor_derivative_rad)
    pI = v(_i32(interaction_map_rad))
    pD = v(radial_descriptor)
    force = torch.empty((nf, 3 * N), dtype=dtype, device=dev)
    virial = torch.empty((nf, 9), dtype=dtype, device=dev) if pos is not None else None
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_force_doublets_{s}", ptr(_dense(netderiv)), pD, pdD, pI, _I(nr), _I(N), _I(nf), _I(Ar),
         ptr(_dense(alpha2b_parameters)), ptr(_dense(type_emb2b_parameters)), _I(nt), ptr(_i32(tipos)), ptr(at),
         ptr(force), ptr(_i32(type_map)), _I(Nl), ptr(virial), ptr(None if pos is None else _dense(pos)),
         ptr(None if box is None else _dense(box)), _I(v.ld), _stream())
    return force if pos is None else (force, virial)


def compute_force_radial_virial(netderiv, descriptor_derivative_rad, interaction_map_rad, radial_descriptor,
                                alpha2b_parameters, type_emb2b_parameters, type_map, tipos, actual_type, pos, box):
    return compute_force_radial(netderiv, descriptor_derivative_rad, interaction_map_rad, radial_descriptor,
                                alpha2b_parameters, type_emb2b_parameters, type_map, tipos, actual_type, pos, box)


def compute_force_tripl(netderiv, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                        descriptor_derivative_ang, interaction_map_rad, interaction_map_ang, alpha3b_parameters,
                        type_emb3b_parameters, type_map, tipos, actual_type, num_triplets, pos=None, box=None):
    """ComputeForceTripl (STAF/src/force/ang/reforce.cc:44-58) -> force [nf,3N]; with pos/box:
    ComputeForceTriplVirial (:159-176).  radial_descriptor = des3bsupp, descriptor_derivative_rad = der3bsupp."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    dev = angular_descriptor.device
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    N = type_map.shape[0]
    nt = tipos.shape[0]
    Aa = alpha3b_parameters.shape[1] // 3
    v = _Views()
    pD = v(radial_descriptor)
    pT = v(angular_descriptor)
    pdD = v(descriptor_derivative_rad)
    pd3 = v(descriptor_derivative_ang)
    pI2 = v(_i32(interaction_map_rad))
    pI3 = v(_i32(interaction_map_ang))
    pN = v(_i32(num_triplets))
    force = torch.empty((nf, 3 * N), dtype=dtype, device=dev)
    virial = torch.empty((nf, 9), dtype=dtype, device=dev) if pos is not None else None
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_force_tripl_{s}", ptr(_dense(netderiv)), pD, pT, pdD, pd3, pI2, pI3, _I(nr), _I(na), _I(N), _I(nf),
         _I(Aa), ptr(_dense(type_emb3b_parameters)), _I(nt), ptr(_i32(tipos)), ptr(at), ptr(force), pN,
         ptr(_dense(alpha3b_parameters)), ptr(_i32(type_map)), _I(Nl), ptr(virial),
         ptr(None if pos is None else _dense(pos)), ptr(None if box is None else _dense(box)), _I(v.ld), _stream())
    return force if pos is None else (force, virial)


def compute_force_tripl_slots(netderiv, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                              descriptor_derivative_ang, interaction_map_rad, interaction_map_ang, alpha3b_parameters,
                              type_emb3b_parameters, type_map, tipos, actual_type, num_triplets):
    """First half of ComputeForceTripl: the 3-body forces of one centre species as they act on each centre's
    neighbour slots, (slot_forces [nf,Nl,nr,3], self_forces [nf,Nl,3]), not yet collected by the atoms that receive
    them.  force_total() collects them for all species, and adds the 2-body forces, in one launch."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    dev = angular_descriptor.device
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    N = type_map.shape[0]
    nt = tipos.shape[0]
    Aa = alpha3b_parameters.shape[1] // 3
    v = _Views()
    pD = v(radial_descriptor)
    pT = v(angular_descriptor)
    pdD = v(descriptor_derivative_rad)
    pd3 = v(descriptor_derivative_ang)
    pI2 = v(_i32(interaction_map_rad))
    pI3 = v(_i32(interaction_map_ang))
    pN = v(_i32(num_triplets))
    slots = torch.empty((nf, Nl, nr, 3), dtype=dtype, device=dev)
    own = torch.empty((nf, Nl, 3), dtype=dtype, device=dev)
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_force_tripl_slots_{s}", ptr(_dense(netderiv)), pD, pT, pdD, pd3, pI2, pI3, _I(nr), _I(na), _I(N),
         _I(nf), _I(Aa), ptr(_dense(type_emb3b_parameters)), _I(nt), ptr(_i32(tipos)), ptr(at), ptr(slots), ptr(own),
         pN, ptr(_dense(alpha3b_parameters)), ptr(_i32(type_map)), _I(Nl), _I(v.ld), _stream())
    return slots, own


def compute_forces_slots(netderiv3b, netderiv2b, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                         descriptor_derivative_ang, radial_descriptor_2b, descriptor_derivative_rad_2b,
                         interaction_map_rad, interaction_map_ang, alpha3b_parameters, type_emb3b_parameters,
                         alpha2b_parameters, type_emb2b_parameters, type_map, tipos, actual_type, num_triplets):
    """compute_force_tripl_slots with the 2-body pair forces of the same centres (what ComputeForceRadial computes
    from netderiv2b, raddescr = radial_descriptor_2b and der2b = descriptor_derivative_rad_2b) added to the slot
    forces in the same launch: (slot_forces [nf,Nl,nr,3], self_forces [nf,Nl,3]) of 2-body + 3-body.  force_total()
    then gives the total force without any per-op force array."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    dev = angular_descriptor.device
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    N = type_map.shape[0]
    nt = tipos.shape[0]
    Aa = alpha3b_parameters.shape[1] // 3
    Ar = alpha2b_parameters.shape[1]
    v = _Views()
    pD = v(radial_descriptor)
    pT = v(angular_descriptor)
    pdD = v(descriptor_derivative_rad)
    pd3 = v(descriptor_derivative_ang)
    pD2 = v(radial_descriptor_2b)
    pdD2 = v(descriptor_derivative_rad_2b)
    pI2 = v(_i32(interaction_map_rad))
    pI3 = v(_i32(interaction_map_ang))
    pN = v(_i32(num_triplets))
    slots = torch.empty((nf, Nl, nr, 3), dtype=dtype, device=dev)
    own = torch.empty((nf, Nl, 3), dtype=dtype, device=dev)
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_forces_slots_{s}", ptr(_dense(netderiv3b)), ptr(_dense(netderiv2b)), pD, pT, pdD, pd3, pD2, pdD2,
         pI2, pI3, _I(nr), _I(na), _I(N), _I(nf), _I(Aa), _I(Ar), ptr(_dense(type_emb3b_parameters)),
         ptr(_dense(alpha3b_parameters)), ptr(_dense(alpha2b_parameters)), ptr(_dense(type_emb2b_parameters)), _I(nt),
         ptr(_i32(tipos)), ptr(at), ptr(slots), ptr(own), pN, ptr(_i32(type_map)), _I(Nl), _I(v.ld), _stream())
    return slots, own


def force_total(interaction_map_rad_full, n_local, slot_forces, self_forces, forces2b=None, out=None):
    """Total force [nf,3N] in one launch: for every species k, in this order, forces2b[k] (a per-op force array,
    e.g. what compute_force_radial returned for centre species k; None to skip) plus the 3-body forces of species k
    collected from slot_forces[k] / self_forces[k] (compute_force_tripl_slots; None to skip).  Same bits as adding
    the per-op force arrays in that order.  interaction_map_rad_full is the whole intmap2b tensor [nf,N,nr+1] the
    descriptor op wrote; n_local the atoms per species (host integers)."""
    im = _i32(interaction_map_rad_full)
    if not im.is_contiguous():
        raise ValueError("force_total needs the descriptor op's whole intmap2b tensor")
    nf, N, nr1 = im.shape
    nt = len(n_local)
    some = next(t for t in list(slot_forces) + list(forces2b or []) if t is not None)
    dtype, dev = some.dtype, some.device
    s, _ = sfx(dtype)
    arr = lambda ts: (C.c_void_p * nt)(*[None if t is None else _dense(t).data_ptr() for t in ts])
    keep = [None if t is None else _dense(t) for t in list(slot_forces) + list(self_forces) + list(forces2b or [])]
    total = torch.empty((nf, 3 * N), dtype=dtype, device=dev) if out is None else out
    call(f"staf_op_force_total_{s}", ptr(im), _I(nr1 - 1), _I(N), _I(nf), _I(nt), (C.c_int * nt)(*[int(n) for n in n_local]),
         arr(slot_forces), arr(self_forces), arr(forces2b if forces2b is not None else [None] * nt), ptr(total),
         _stream())
    del keep
    return total


def compute_force_tripl_virial(netderiv, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                               descriptor_derivative_ang, interaction_map_rad, interaction_map_ang,
                               alpha3b_parameters, type_emb3b_parameters, type_map, tipos, actual_type, num_triplets,
                               pos, box):
    return compute_force_tripl(netderiv, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                               descriptor_derivative_ang, interaction_map_rad, interaction_map_ang,
                               alpha3b_parameters, type_emb3b_parameters, type_map, tipos, actual_type, num_triplets,
                               pos, box)


# --------------------------------------------------------------------------- parameter gradients (energy branch)


def compute_two_body_par_grad(prev_grad, radial_descriptor, interaction_map_rad, alpha2b_parameters,
                              type_emb2b_parameters, type_map):
    """ComputeTwoBodyParGrad (STAF/src/grad_finger/rad/reforce.cc:14-22) -> (nextgrad_alpha2b, nextgrad_emb2b)."""
    dtype = radial_descriptor.dtype
    s, _ = sfx(dtype)
    dev = radial_descriptor.device
    nf, Nl, nr = radial_descriptor.shape
    nt, Ar = alpha2b_parameters.shape
    v = _Views()
    pD = v(radial_descriptor)
    pI = v(_i32(interaction_map_rad))
    ga = torch.empty((nt, Ar), dtype=dtype, device=dev)
    ge = torch.empty((nt, Ar), dtype=dtype, device=dev)
    call(f"staf_op_alpha_dist_grad_{s}", pD, _I(nr), ptr(_dense(alpha2b_parameters)), _I(Ar), ptr(ga), _I(nf), _I(Nl),
         pI, ptr(_dense(prev_grad)), ptr(_dense(type_emb2b_parameters)), ptr(_i32(type_map)), ptr(ge), _I(nt),
         _I(v.ld), _stream())
    return ga, ge


def compute_sort_proj3body_grad(previous_gradient, angular_desciptors, radial_descriptors, intmap3b, intmap2b,
                                alpha3b_parameters, type_emb3b, type_map, num_triplets, nt=None):
    """ComputeSortProj3bodyGrad (STAF/src/grad_finger/ang/reforce.cc:12-23) -> (alphagrad3body [ntc,3Aa],
    nextgrad_emb3b [ntc,Aa] == 0)."""
    dtype = angular_desciptors.dtype
    s, _ = sfx(dtype)
    dev = angular_desciptors.device
    nf, Nl, na = angular_desciptors.shape
    nr = radial_descriptors.shape[2]
    ntc = alpha3b_parameters.shape[0]
    Aa = alpha3b_parameters.shape[1] // 3
    nt = _nt_from_ntc(ntc) if nt is None else nt
    v = _Views()
    pT = v(angular_desciptors)
    pD = v(radial_descriptors)
    pI3 = v(_i32(intmap3b))
    pI2 = v(_i32(intmap2b))
    pN = v(_i32(num_triplets))
    ga = torch.empty((ntc, 3 * Aa), dtype=dtype, device=dev)
    ge = torch.empty((ntc, Aa), dtype=dtype, device=dev)
    call(f"staf_op_alphagrad_ang_{s}", pD, pT, _I(nr), _I(na), ptr(_dense(previous_gradient)), _I(nf), _I(Nl), pI3,
         pI2, ptr(_dense(alpha3b_parameters)), _I(Aa), ptr(ga), ptr(_dense(type_emb3b)), ptr(_i32(type_map)), ptr(ge),
         pN, _I(ntc), _I(nt), _I(v.ld), _stream())
    return ga, ge


# --------------------------------------------------------------------------- gradients of the force ops


def compute_force_radial_grad(prevgrad, netderiv, descriptor_derivative_rad, interaction_map_rad, radial_descriptor,
                              alpha2b_parameters, type_emb2b_parameters, type_map, tipos, actual_type,
                              prevgrad_virial=None, pos=None, box=None):
    """ComputeForceRadialGrad (STAF/src/grad_force/rad/reforce.cc:42-55) -> (gradnet [nf,Nl,Ar], grad_alpha2b,
    grad_emb2b [nt,Ar]); with prevgrad_virial/pos/box: ComputeForceRadialVirialGrad (:160-176)."""
    dtype = radial_descriptor.dtype
    s, _ = sfx(dtype)
    dev = radial_descriptor.device
    nf, Nl, nr = radial_descriptor.shape
    N = type_map.shape[0]
    nt, Ar = alpha2b_parameters.shape
    v = _Views()
    pdD = v(descriptor_derivative_rad)
    pI = v(_i32(interaction_map_rad))
    pD = v(radial_descriptor)
    gn = torch.empty((nf, Nl, Ar), dtype=dtype, device=dev)
    ga = torch.empty((nt, Ar), dtype=dtype, device=dev)
    ge = torch.empty((nt, Ar), dtype=dtype, device=dev)
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_gradforce_2b_{s}", ptr(_dense(prevgrad)), pD, _I(nr), ptr(_dense(alpha2b_parameters)), _I(Ar), pdD,
         pI, _I(nf), _I(N), _I(Nl), ptr(_dense(netderiv)), ptr(_dense(type_emb2b_parameters)), _I(nt),
         ptr(_i32(type_map)), ptr(_i32(tipos)), ptr(at), ptr(gn), ptr(ga), ptr(ge),
         ptr(None if prevgrad_virial is None else _dense(prevgrad_virial)),
         ptr(None if pos is None else _dense(pos)), ptr(None if box is None else _dense(box)), _I(v.ld), _stream())
    return gn, ga, ge


def compute_force_tripl_grad(prevgrad, netderiv, radial_descriptor, angular_descriptor, descriptor_derivative_rad,
                             descriptor_derivative_ang, interaction_map_rad, interaction_map_ang, alpha3b_parameters,
                             type_emb3b_parameters, type_map, tipos, actual_type, num_triplets, prevgrad_virial=None,
                             pos=None, box=None):
    """ComputeForceTriplGrad (STAF/src/grad_force/ang/reforce.cc:39-56) -> (gradnet [nf,Nl,Aa], gradalpha
    [ntc,3Aa], gradck [ntc,Aa] == 0); with prevgrad_virial/pos/box: ComputeForceTriplVirialGrad (:186-206)."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    dev = angular_descriptor.device
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    N = type_map.shape[0]
    nt = tipos.shape[0]
    ntc = nt * (nt + 1) // 2
    Aa = alpha3b_parameters.shape[1] // 3
    v = _Views()
    pD = v(radial_descriptor)
    pT = v(angular_descriptor)
    pdD = v(descriptor_derivative_rad)
    pd3 = v(descriptor_derivative_ang)
    pI2 = v(_i32(interaction_map_rad))
    pI3 = v(_i32(interaction_map_ang))
    pN = v(_i32(num_triplets))
    gn = torch.empty((nf, Nl, Aa), dtype=dtype, device=dev)
    ga = torch.empty((ntc, 3 * Aa), dtype=dtype, device=dev)
    ge = torch.empty((ntc, Aa), dtype=dtype, device=dev)
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_gradforce_tripl_{s}", ptr(_dense(prevgrad)), ptr(_dense(netderiv)), pD, pT, pdD, pd3, pI2, pI3,
         _I(nr), _I(na), _I(N), _I(nf), _I(Aa), ptr(_dense(type_emb3b_parameters)), _I(nt), ptr(_i32(tipos)), ptr(at),
         pN, ptr(_dense(alpha3b_parameters)), ptr(_i32(type_map)), _I(Nl), ptr(gn), ptr(ga), ptr(ge),
         ptr(None if prevgrad_virial is None else _dense(prevgrad_virial)),
         ptr(None if pos is None else _dense(pos)), ptr(None if box is None else _dense(box)), _I(v.ld), _stream())
    return gn, ga, ge


def compute_tripl_grads_fused(prevgrad_force, netderiv, prevgrad_energy, radial_descriptor, angular_descriptor,
                              descriptor_derivative_rad, descriptor_derivative_ang, interaction_map_rad,
                              interaction_map_ang, alpha3b_parameters, type_emb3b_parameters, type_map, tipos,
                              actual_type, num_triplets, prevgrad_virial=None, pos=None, box=None):
    """Both 3-body parameter gradients of a training step in one launch (no counterpart as one op in the reference):
    what compute_force_tripl_grad(prevgrad_force, netderiv, ...) and compute_sort_proj3body_grad(prevgrad_energy,
    ...) return, as (gradnet [nf,Nl,Aa], gradalpha_force [ntc,3Aa], gradalpha_energy [ntc,3Aa], gradck [ntc,Aa] == 0).
    The two ops share everything but a few accumulations per (triplet, channel), so this costs about what the
    force-branch op costs alone."""
    dtype = angular_descriptor.dtype
    s, _ = sfx(dtype)
    dev = angular_descriptor.device
    nf, Nl, na = angular_descriptor.shape
    nr = radial_descriptor.shape[2]
    N = type_map.shape[0]
    nt = tipos.shape[0]
    ntc = nt * (nt + 1) // 2
    Aa = alpha3b_parameters.shape[1] // 3
    v = _Views()
    pD = v(radial_descriptor)
    pT = v(angular_descriptor)
    pdD = v(descriptor_derivative_rad)
    pd3 = v(descriptor_derivative_ang)
    pI2 = v(_i32(interaction_map_rad))
    pI3 = v(_i32(interaction_map_ang))
    pN = v(_i32(num_triplets))
    gn = torch.empty((nf, Nl, Aa), dtype=dtype, device=dev)
    gaf = torch.empty((ntc, 3 * Aa), dtype=dtype, device=dev)
    gae = torch.empty((ntc, 3 * Aa), dtype=dtype, device=dev)
    ge = torch.empty((ntc, Aa), dtype=dtype, device=dev)
    at = _scalar_dev(actual_type, dev)
    call(f"staf_op_grads_tripl_fused_{s}", ptr(_dense(prevgrad_force)), ptr(_dense(netderiv)),
         ptr(_dense(prevgrad_energy)), pD, pT, pdD, pd3, pI2, pI3, _I(nr), _I(na), _I(N), _I(nf), _I(Aa),
         ptr(_dense(type_emb3b_parameters)), _I(nt), ptr(_i32(tipos)), ptr(at), pN, ptr(_dense(alpha3b_parameters)),
         ptr(_i32(type_map)), _I(Nl), ptr(gn), ptr(gaf), ptr(gae), ptr(ge),
         ptr(None if prevgrad_virial is None else _dense(prevgrad_virial)),
         ptr(None if pos is None else _dense(pos)), ptr(None if box is None else _dense(box)), _I(v.ld), _stream())
    return gn, gaf, gae, ge


def compute_force_radial_virial_grad(prevgrad, prevgrad_virial, netderiv, descriptor_derivative_rad,
                                     interaction_map_rad, radial_descriptor, alpha2b_parameters,
                                     type_emb2b_parameters, type_map, tipos, actual_type, pos, box):
    """ComputeForceRadialVirialGrad (STAF/src/grad_force/rad/reforce.cc:160-176)."""
    return compute_force_radial_grad(prevgrad, netderiv, descriptor_derivative_rad, interaction_map_rad,
                                     radial_descriptor, alpha2b_parameters, type_emb2b_parameters, type_map, tipos,
                                     actual_type, prevgrad_virial, pos, box)


def compute_force_tripl_virial_grad(prevgrad, prevgrad_virial, netderiv, radial_descriptor, angular_descriptor,
                                    descriptor_derivative_rad, descriptor_derivative_ang, interaction_map_rad,
                                    interaction_map_ang, alpha3b_parameters, type_emb3b_parameters, type_map, tipos,
                                    actual_type, num_triplets, pos, box):
    """ComputeForceTriplVirialGrad (STAF/src/grad_force/ang/reforce.cc:186-206)."""
    return compute_force_tripl_grad(prevgrad, netderiv, radial_descriptor, angular_descriptor,
                                    descriptor_derivative_rad, descriptor_derivative_ang, interaction_map_rad,
                                    interaction_map_ang, alpha3b_parameters, type_emb3b_parameters, type_map, tipos,
                                    actual_type, num_triplets, prevgrad_virial, pos, box)
