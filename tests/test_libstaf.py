"""The MD-facing entry (include/staf.h, include/staf_mlp.h): staf_load / staf_compute / staf_free and the MLP plug-in.

CPU tests cover the host-only parts (MLP plug-in against the numpy Dense stack, option defaults, null handling);
GPU tests call staf_compute through the C ABI and compare with the oracle pipeline, the reference's recorded
energies, and the two neighbour-list modes against each other."""
import ctypes as C
import json
import os

import numpy as np
import pytest

from util import GOLDEN, load_frame_mbpol, load_model, load_water_smoke, mlp_energy_and_grad, nerr

KNOWN = json.load(open(os.path.join(GOLDEN, "known_answers.json")))
RC = 4.5


# ----------------------------------------------------------------------------- host-only

class _Eval(C.Structure):
    _fields_ = [("n_type", C.c_int), ("n_atoms", C.POINTER(C.c_int)), ("n_af", C.POINTER(C.c_int)),
                ("af_f32", C.POINTER(C.c_float)), ("af_f64", C.POINTER(C.c_double)),
                ("energy_f32", C.POINTER(C.c_float)), ("energy_f64", C.POINTER(C.c_double)),
                ("dE_daf_f32", C.POINTER(C.c_float)), ("dE_daf_f64", C.POINTER(C.c_double))]


@pytest.mark.parametrize("prec", ["float", "double"])
def test_mlp_plugin_matches_numpy_dense_stack(prec):
    """staf_mlp_eval on the exported mlp_type*.bin against the numpy evaluation of the same weights read from the
    .npz export: energy = 1/2 sum of atomic energies, dE_daf = d(sum atomic)/d af."""
    from alphanesgpu_amd import _lib
    L = _lib.lib()
    L.staf_mlp_create.restype = C.c_void_p
    L.staf_mlp_create.argtypes = [C.c_int, C.c_char_p, C.c_int, C.c_int]
    L.staf_mlp_eval.argtypes = [C.c_void_p, C.POINTER(_Eval)]
    L.staf_mlp_destroy.argtypes = [C.c_void_p]
    L.staf_mlp_ntypes.argtypes = [C.c_void_p]
    L.staf_mlp_n_af.argtypes = [C.c_void_p, C.c_int]
    L.staf_mlp_precision.argtypes = [C.c_void_p]
    p = 0 if prec == "float" else 1
    dt, ct = (np.float32, C.c_float) if p == 0 else (np.float64, C.c_double)
    tipos, model = load_model(prec)
    h = L.staf_mlp_create(1, os.path.join(GOLDEN, f"model_{prec}").encode(), p, 0)
    assert h
    assert L.staf_mlp_ntypes(h) == 2 and L.staf_mlp_precision(h) == p
    rng = np.random.default_rng(5)
    n_atoms = np.array([7, 12], np.int32)
    n_af = np.array([L.staf_mlp_n_af(h, k) for k in range(2)], np.int32)
    assert list(n_af) == [m["mu"].size for m in model]
    afs = [rng.uniform(0.05, 3.0, (n_atoms[k], n_af[k])).astype(dt) for k in range(2)]
    flat = np.concatenate([a.reshape(-1) for a in afs])
    grad = np.zeros_like(flat)
    e = ct(0)
    ev = _Eval()
    ev.n_type = 2
    ev.n_atoms = n_atoms.ctypes.data_as(C.POINTER(C.c_int))
    ev.n_af = n_af.ctypes.data_as(C.POINTER(C.c_int))
    if p == 0:
        ev.af_f32, ev.dE_daf_f32 = (flat.ctypes.data_as(C.POINTER(C.c_float)), grad.ctypes.data_as(C.POINTER(C.c_float)))
        ev.energy_f32 = C.pointer(e)
    else:
        ev.af_f64, ev.dE_daf_f64 = (flat.ctypes.data_as(C.POINTER(C.c_double)),
                                    grad.ctypes.data_as(C.POINTER(C.c_double)))
        ev.energy_f64 = C.pointer(e)
    assert L.staf_mlp_eval(h, C.byref(ev)) == 0
    want_e, want_g = 0.0, []
    for k in range(2):
        ek, gk = mlp_energy_and_grad(afs[k].astype(np.float64), model[k]["mu"].astype(np.float64),
                                     [(W.astype(np.float64), b.astype(np.float64), a) for W, b, a in model[k]["layers"]])
        want_e += 0.5 * float(ek)
        want_g.append(gk.reshape(-1))
    want_g = np.concatenate(want_g)
    tol = 2e-5 if p == 0 else 1e-12
    assert abs(e.value - want_e) <= tol * max(1.0, abs(want_e))
    assert nerr(grad, want_g) <= tol
    # wrong fingerprint width is refused
    bad = n_af.copy()
    bad[1] += 1
    ev.n_af = bad.ctypes.data_as(C.POINTER(C.c_int))
    assert L.staf_mlp_eval(h, C.byref(ev)) == -3
    L.staf_mlp_destroy(h)
    assert L.staf_mlp_create(1, b"/nonexistent_model_dir", p, 0) is None


def test_options_default_and_null_model():
    from alphanesgpu_amd import libstaf
    o = libstaf.options_default()
    assert (o.mlp_backend, o.device_id, o.precision) == (libstaf.STAF_MLP_ORT, 0, 0)
    L = libstaf._bind()
    x = np.zeros(3)
    assert L.staf_compute(None, 1, 0, x.ctypes.data, x.ctypes.data, None, None, None, 0, None, None, None) == -1


# ----------------------------------------------------------------------------- GPU

def _wrap(pos, box6):
    """Positions folded into the primary cell of box6 = (Lx, xy, xz, Ly, yz, Lz)."""
    H = np.array([[box6[0], box6[1], box6[2]], [0, box6[3], box6[4]], [0, 0, box6[5]]])
    s = np.linalg.solve(H, pos.T).T
    s -= np.floor(s)
    return s @ H.T, H


def _ghost_configuration(pos, box6, types, rc):
    """What an MD code hands over: owned atoms plus explicit periodic images (ghosts) within rc of an owned atom,
    and per owned atom the neighbours within rc sorted by distance (indices into owned+ghost)."""
    pos, H = _wrap(pos, box6)
    n = len(pos)
    shifts = [np.array([a, b, c]) for a in (-1, 0, 1) for b in (-1, 0, 1) for c in (-1, 0, 1) if (a, b, c) != (0, 0, 0)]
    gx, gowner = [], []
    for sh in shifts:
        img = pos + H @ sh
        d2 = ((img[:, None, :] - pos[None, :, :]) ** 2).sum(-1)
        keep = np.where((d2 < rc * rc).any(axis=1))[0]
        gx.append(img[keep])
        gowner.append(keep)
    gx = np.concatenate(gx)
    gowner = np.concatenate(gowner)
    allx = np.concatenate([pos, gx])
    alltypes = np.concatenate([types, types[gowner]]).astype(np.int32)
    d2 = ((pos[:, None, :] - allx[None, :, :]) ** 2).sum(-1)
    lists = []
    for i in range(n):
        c = np.where((d2[i] < rc * rc) & (d2[i] > 1e-24))[0]
        lists.append(c[np.argsort(d2[i, c], kind="stable")])
    maxneigh = max(len(l) for l in lists)
    howmany = np.array([len(l) for l in lists], np.int32)
    neigh = np.zeros((n, maxneigh), np.int32)
    for i, l in enumerate(lists):
        neigh[i, :len(l)] = l
    return pos, allx, alltypes, gowner, howmany, neigh


def _as64(model):
    return [{k: (v.astype(np.float64) if isinstance(v, np.ndarray) else
                 [(W.astype(np.float64), b.astype(np.float64), a) for W, b, a in v]) for k, v in m.items()}
            for m in model]


@pytest.mark.gpu
def test_compute_matches_oracle_pipeline_fp64_model(oracle):
    """float64 model: energy, forces and virial diagonal of the reference frame against the oracle ops wired in the
    reference's order; tolerance 1e-10 (fp64 kernels, sums of ~1e3 terms in different orders)."""
    from alphanesgpu_amd import libstaf
    from test_oracle_pins import energy_and_forces
    tipos, model = load_model("double")
    pos, box, tp, type_map = load_frame_mbpol(np.float64)
    E, F, W, _, _ = energy_and_forces(oracle, pos, box, tp, type_map, _as64(model), virial=True)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1, full_virial=True)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], type_map)
    assert abs(e - float(E[0])) <= 1e-10 * abs(float(E[0]))
    assert nerr(f.reshape(-1), F[0]) <= 1e-10
    Wm = W[0].reshape(3, 3)
    want = np.array([Wm[0, 0], Wm[1, 1], Wm[2, 2], 0.5 * (Wm[0, 1] + Wm[1, 0]), 0.5 * (Wm[0, 2] + Wm[2, 0]),
                     0.5 * (Wm[1, 2] + Wm[2, 1])])
    assert nerr(vir, want) <= 1e-10
    # second call on the same handle (buffers reused) gives the same bits
    e2, f2, vir2 = m.compute(pos.reshape(-1, 3), box[0], type_map)
    assert e2 == e and np.array_equal(f2, f) and np.array_equal(vir2, vir)
    m.close()


@pytest.mark.gpu
def test_compute_6144_atom_box_matches_oracle_pipeline(oracle):
    """The large-box configuration through the MD entry: 2048 water molecules, one call, neighbour list rebuilt by the library
    (cell list: 6144 >= 4096 atoms), no tensor of the angular buffer's width on the device; energy and forces against
    the oracle ops wired in the reference's order (all-pairs neighbour search there), 1e-10."""
    from alphanesgpu_amd import libstaf, synth
    from test_oracle_pins import energy_and_forces
    tipos, model = load_model("double")
    b = synth.water_batch("water6144")
    pos, box = b["pos"].astype(np.float64), b["box"].astype(np.float64)
    E, F, W, _, _ = energy_and_forces(oracle, pos, box, b["tipos"], b["type_map"], _as64(model), virial=True)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1, full_virial=True)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], b["type_map"])
    assert abs(e - float(E[0])) <= 1e-10 * abs(float(E[0]))
    assert nerr(f.reshape(-1), F[0]) <= 1e-10
    Wm = W[0].reshape(3, 3)
    assert nerr(vir[:3], np.array([Wm[0, 0], Wm[1, 1], Wm[2, 2]])) <= 1e-10
    m.close()


@pytest.mark.gpu
def test_compute_is_invariant_under_periodic_replication():
    """A size-independent property at a size the oracle does not reach: the 6144-atom box replicated 2x2x2 (49152
    atoms, species-sorted, box edges doubled) has the same local environments, so the energy and the virial are
    eight times those of the single box and every replica carries the single box's forces (1e-12; the sums are
    the same, only the neighbour search runs over other cells)."""
    from alphanesgpu_amd import libstaf, synth
    b = synth.water_batch("water6144")
    x = b["pos"][0].reshape(-1, 3).astype(np.float64)
    box = b["box"][0].astype(np.float64)
    tm = b["type_map"]
    L = box[0]
    n_o = int((tm == 0).sum())
    shifts = np.array([[i, j, k] for i in range(2) for j in range(2) for k in range(2)], float) * L
    xo = np.concatenate([x[:n_o] + s for s in shifts])
    xh = np.concatenate([x[n_o:] + s for s in shifts])
    big_x = np.concatenate([xo, xh]) - L / 2
    big_tm = np.array([0] * len(xo) + [1] * len(xh), np.int32)
    big_box = box.copy()
    big_box[[0, 3, 5]] *= 2
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1)
    e, f, v = m.compute(x, box, tm)
    E, F, V = m.compute(big_x, big_box, big_tm)
    m.close()
    assert abs(E - 8 * e) <= 1e-12 * abs(8 * e)
    want = np.concatenate([np.concatenate([f[:n_o]] * 8), np.concatenate([f[n_o:]] * 8)])
    assert nerr(F.reshape(-1), want.reshape(-1)) <= 1e-12
    assert nerr(V, 8 * v) <= 1e-12


@pytest.mark.gpu
def test_compute_reproduces_recorded_energies_fp32_model(oracle):
    """float32 MLP (the reference's default build): E and rms(F) recorded by the reference for its 768-atom frame
    (test/test-lammps-STAF-inference-STAF-comp/results/frames.csv:2) and PE of data.water_smoke
    (test/B_ARCHITECTURE.md:167).  The water_smoke atoms come in file order (O H H ...), so this also covers the
    species-sorted packing and un-packing."""
    from alphanesgpu_amd import libstaf
    from test_oracle_pins import energy_and_forces
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_float"), precision=0)
    pos, box, tp, type_map = load_frame_mbpol(np.float64)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], type_map)
    ka = KNOWN["frame0_model_float"]
    assert abs(e - ka["E_lammps"]) < 1.5e-4 and abs(e - ka["E_python"]) < 1.5e-4
    assert abs(float(np.sqrt(np.mean(f ** 2))) - ka["rms_F_python"]) < 5e-6
    assert np.all(vir[3:] == 0.0)          # diagonal only unless asked otherwise

    pos, box, types = load_water_smoke(np.float64)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], types)
    assert abs(e - KNOWN["water_smoke_model_float"]["PE"]) < 2e-4
    # forces in the caller's order against the oracle on the species-sorted arrangement (float64 MLP there:
    # the float32 MLP's rounding is ~1e-6 of the force scale)
    tipos, model = load_model("float")
    order = np.argsort(types, kind="stable")
    ps = pos.reshape(-1, 3)[order].reshape(1, -1)
    E, F, _, _, _ = energy_and_forces(oracle, ps, box, np.bincount(types).astype(np.int32),
                                      types[order].astype(np.int32), _as64(model))
    Fo = np.zeros_like(f)
    Fo[order] = F[0].reshape(-1, 3)
    assert nerr(f, Fo) < 2e-5
    # permuting the caller's atom order permutes the forces and nothing else
    rng = np.random.default_rng(11)
    perm = rng.permutation(len(types))
    e_p, f_p, vir_p = m.compute(pos.reshape(-1, 3)[perm], box[0], types[perm])
    assert abs(e_p - e) < 1e-5 * abs(e)
    assert nerr(f_p, f[perm]) < 2e-5
    m.close()


@pytest.mark.gpu
def test_compute_with_injected_list_and_ghosts_matches_own_list():
    """The MD code's neighbour list (explicit periodic images as ghost atoms, no wrap inside the kernels) against
    the library's own minimum-image list: same energy and virial, and the ghost forces folded back onto their
    owners give the same forces.  float64 model, tolerance 1e-10."""
    from alphanesgpu_amd import libstaf
    pos, box, types = load_water_smoke(np.float64)
    pos = pos.reshape(-1, 3)
    n = len(pos)
    wrapped, allx, alltypes, gowner, howmany, neigh = _ghost_configuration(pos, box[0], types, RC)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1, full_virial=True)
    e0, f0, v0 = m.compute(wrapped, box[0], types)
    e1, f1, v1 = m.compute(allx, box[0], alltypes, nlocal=n, howmany=howmany, neigh=neigh)
    folded = f1[:n].copy()
    np.add.at(folded, gowner, f1[n:])
    assert abs(e1 - e0) <= 1e-10 * abs(e0)
    assert nerr(folded, f0) <= 1e-10
    assert nerr(v1, v0) <= 1e-10
    # and back: the own-list mode is not left in no-wrap mode by the previous call
    e2, f2, v2 = m.compute(wrapped, box[0], types)
    assert e2 == e0 and np.array_equal(f2, f0)
    m.close()


@pytest.mark.gpu
@pytest.mark.parametrize("prec,tol", [("double", 1e-11), ("float", 2e-5)])
def test_device_mlp_matches_host_mlp(prec, tol):
    """The MLP evaluated on the GPU between the kernels (default) against the host evaluation of the same weights
    (reserved bit 1): energy, forces, virial.  float64 nets: 1e-11; float32 nets: the two evaluations sum in
    different orders, 2e-5 of the largest force."""
    from alphanesgpu_amd import libstaf
    pos, box, types = load_water_smoke(np.float64)
    pos = pos.reshape(-1, 3)
    p = 1 if prec == "double" else 0
    host = libstaf.StafModel(os.path.join(GOLDEN, f"model_{prec}"), precision=p, full_virial=True, host_mlp=True)
    e0, f0, v0 = host.compute(pos, box[0], types)
    host.close()
    # the kernel the library picks by itself, then each of its two device kernels (a handle of its own each: a
    # handle replays what its first calls recorded)
    for force in (None, "STAF_MLP_MATRIX", "STAF_MLP_VECTOR"):
        if force:
            os.environ[force] = "1"
        try:
            dev = libstaf.StafModel(os.path.join(GOLDEN, f"model_{prec}"), precision=p, full_virial=True)
            e1, f1, v1 = dev.compute(pos, box[0], types)
            dev.close()
        finally:
            if force:
                os.environ.pop(force, None)
        assert abs(e1 - e0) <= max(tol, 1e-6 if p == 0 else 0) * abs(e0), force
        assert nerr(f1, f0) <= tol, force
        assert nerr(v1, v0) <= tol, force


@pytest.mark.gpu
@pytest.mark.parametrize("prec,tol", [("double", 1e-11), ("float", 2e-5)])
def test_device_mlp_kernels_on_small_widths_and_ragged_atom_counts(tmp_path, prec, tol):
    """Both device kernels of the network (the matrix-core one, 16 atoms per workgroup, and the vector one) against
    the host evaluation on a written three-species model whose widths (fingerprints 9/7/11, hidden 20) are no
    multiples of the tile sizes and whose atom counts (7, 9, 3) leave every workgroup partly empty: a wrong row
    layout of the matrix tiles or a padding row entering a sum shows here, not on the 256/512-atom frames."""
    from alphanesgpu_amd import libstaf, model_dir
    from test_oracle_pins import cluster, small_model
    ps = small_model(3, (5, 4, 6), (4, 3, 5, 3, 4, 3), seed=5, hidden=20, dense=True)
    pos, box, tipos, type_map = cluster([7, 9, 3], seed=9)
    model_dir.write_model_dir(str(tmp_path), ps, rc=4.5, rc_ang=3.2, rs=1.6, radial_buffer=24, angular_buffer=276,
                              tipos=tipos, precision=prec)
    p = 1 if prec == "double" else 0
    host = libstaf.StafModel(str(tmp_path), precision=p, full_virial=True, host_mlp=True)
    e0, f0, v0 = host.compute(pos.reshape(-1, 3), box[0], type_map)
    host.close()
    for force in ("STAF_MLP_MATRIX", "STAF_MLP_VECTOR"):      # the library picks by size and precision otherwise
        os.environ[force] = "1"
        try:
            dev = libstaf.StafModel(str(tmp_path), precision=p, full_virial=True)
            e1, f1, v1 = dev.compute(pos.reshape(-1, 3), box[0], type_map)
            dev.close()
        finally:
            os.environ.pop(force, None)
        assert abs(e1 - e0) <= max(tol, 1e-6 if p == 0 else 0) * abs(e0), force
        assert nerr(f1, f0) <= tol and nerr(v1, v0) <= tol, force


@pytest.mark.gpu
def test_compute_without_virial_gives_the_same_energy_and_forces():
    """A null virial pointer skips the virial kernels; energy and forces keep their bits."""
    from alphanesgpu_amd import libstaf
    pos, box, tp, type_map = load_frame_mbpol(np.float64)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], type_map)
    e2, f2, vir2 = m.compute(pos.reshape(-1, 3), box[0], type_map, want_virial=False)
    assert vir2 is None and np.all(np.isfinite(vir))
    assert e2 == e and np.array_equal(f2, f)
    m.close()


@pytest.mark.gpu
def test_replayed_calls_give_the_bits_of_eager_calls_and_follow_shape_changes():
    """From the second call of a shape the library replays a recorded HIP graph.  A handle that replays and one that
    launches eagerly walk through the same sequence of configurations -- the 768-atom frame moving from call to
    call, then the water_smoke frame (other atom count and order), then the first one again, with and without
    virial -- and must agree bit for bit on every call (all sums have a fixed order)."""
    from alphanesgpu_amd import libstaf
    d = os.path.join(GOLDEN, "model_double")
    a = libstaf.StafModel(d, precision=1, full_virial=True)
    b = libstaf.StafModel(d, precision=1, full_virial=True, eager=True)
    posA, boxA, _, tmA = load_frame_mbpol(np.float64)
    posB, boxB, typB = load_water_smoke(np.float64)
    rng = np.random.default_rng(17)
    # (a shape is recorded after 2 calls in a row at first, after 4 and 8 once graphs have been dropped young: the
    # runs below are long enough to be recorded and replayed each time)
    plan = [("A", True)] * 4 + [("B", True)] * 3 + [("A", True)] * 7 + [("A", False)] * 10 + [("B", False)] * 2
    first = {}
    for step, (which, want_w) in enumerate(plan):
        pos, box, types = (posA, boxA[0], tmA) if which == "A" else (posB, boxB[0], typB)
        x = pos.reshape(-1, 3) + 0.02 * rng.standard_normal((pos.shape[1] // 3, 3))   # the atoms move every step
        ea, fa, wa = a.compute(x, box, types, want_virial=want_w)
        eb, fb, wb = b.compute(x, box, types, want_virial=want_w)
        assert ea == eb and np.array_equal(fa, fb), (step, which)
        assert (wa is None and wb is None) or np.array_equal(wa, wb), (step, which)
        assert np.isfinite(ea) and np.abs(fa).max() > 0
        first.setdefault(which, ea)
        if step and plan[step - 1][0] == which:
            assert ea != prev_e          # the inputs did change: a replay that re-used old inputs would show here
        prev_e = ea
    a.close()
    b.close()


@pytest.mark.gpu
def test_release_of_the_ops_state_between_replayed_calls():
    """staf_ops_release (the op interface's call that frees the library's work areas) while a handle of the MD entry
    holds a recorded graph: the graph points into freed memory, so the handle drops it, evaluates eagerly and
    records again -- same bits on every call."""
    from alphanesgpu_amd import libstaf, ops
    pos, box, _, type_map = load_frame_mbpol(np.float64)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1, full_virial=True)
    x = pos.reshape(-1, 3)
    ref = [m.compute(x, box[0], type_map) for _ in range(4)][-1]      # recorded and replayed by now
    for _ in range(2):
        ops.release()
        for _ in range(4):
            e, f, w = m.compute(x, box[0], type_map)
            assert e == ref[0] and np.array_equal(f, ref[1]) and np.array_equal(w, ref[2])
    m.close()


@pytest.mark.gpu
def test_three_handles_on_three_host_threads():
    """Three handles, each used by a host thread of its own at the same time (every handle records and replays its
    own graph on its own streams): every call returns the bits a single handle returned for the same positions."""
    import threading
    from alphanesgpu_amd import libstaf
    pos, box, _, type_map = load_frame_mbpol(np.float64)
    x = pos.reshape(-1, 3)
    d = os.path.join(GOLDEN, "model_double")
    rng = np.random.default_rng(1)
    xs = [x + 0.02 * rng.standard_normal(x.shape) for _ in range(8)]
    ref = libstaf.StafModel(d, precision=1, full_virial=True)
    want = [ref.compute(xx, box[0], type_map) for xx in xs]
    ref.close()
    bad = []

    def worker(t):
        try:
            m = libstaf.StafModel(d, precision=1, full_virial=True)
            for rep in range(2):
                for i, xx in enumerate(xs):
                    e, f, w = m.compute(xx, box[0], type_map)
                    if e != want[i][0] or not np.array_equal(f, want[i][1]) or not np.array_equal(w, want[i][2]):
                        bad.append((t, rep, i))
            m.close()
        except Exception as ex:   # a thread's exception would otherwise be lost
            bad.append((t, repr(ex)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not bad, bad[:10]


@pytest.mark.gpu
def test_compute_return_codes():
    """Validation order and codes of libstaf/src/staf_api.cpp:196-337."""
    from alphanesgpu_amd import libstaf
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_float"), precision=0)
    pos, box, types = load_water_smoke(np.float64)
    pos = pos.reshape(-1, 3)
    code = lambda **kw: pytest.raises(libstaf.StafComputeError, m.compute, **kw).value.code
    assert code(x=pos[:0], box=box[0], types=types[:0]) == -3
    zb = box[0].copy()
    zb[3] = 0.0
    assert code(x=pos, box=zb, types=types) == -7
    bt = types.copy()
    bt[5] = 2
    assert code(x=pos, box=box[0], types=bt) == -8
    hm = np.ones(len(pos), np.int32)
    w = np.zeros((len(pos), 4), np.int32)
    w[3, 0] = len(pos)
    assert code(x=pos, box=box[0], types=types, howmany=hm, neigh=w) == -9
    # one atom named by more centres than the force gather holds keys for (4 x the radial buffer): every other atom
    # of the frame lists atom 0.  Detected on the device, returned by the host; every kernel runs to its end.
    w[:] = 0
    w[0, 0] = 1
    assert len(pos) - 1 > 4 * 60
    assert code(x=pos, box=box[0], types=types, howmany=hm, neigh=w) == -11
    # a valid call still works afterwards
    e, f, v = m.compute(pos, box[0], types)
    assert abs(e - KNOWN["water_smoke_model_float"]["PE"]) < 2e-4
    m.close()
    with pytest.raises(RuntimeError):
        libstaf.StafModel("/nonexistent_model_dir")


# ----------------------------------------------------------------------------- a caller written in C

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
MD_STEP = os.path.join(ROOT, "tests", "c_consumer", "md_step")


def test_headers_are_plain_c_and_the_c_caller_is_built():
    """include/*.h compile as C99 and as C++11 with -pedantic (they are what a C or C++ host includes), and the C
    caller built against include/staf.h alone links the library and reports a usage error without touching a GPU."""
    import subprocess
    for h in ("staf.h", "staf_mlp.h", "staf_ops.h"):
        path = os.path.join(ROOT, "include", h)
        for cc, std, lang in (("gcc", "-std=c99", "c"), ("g++", "-std=c++11", "c++")):
            r = subprocess.run([cc, std, "-Wall", "-Wextra", "-pedantic", "-Werror", "-fsyntax-only", "-x", lang, path],
                               capture_output=True, text=True)
            assert r.returncode == 0, (h, cc, r.stderr)
    assert os.path.exists(MD_STEP), "run __graft_entry__.build() first"
    r = subprocess.run([MD_STEP], capture_output=True, text=True)
    assert r.returncode == 100 and "usage" in r.stderr


@pytest.mark.gpu
def test_c_caller_reproduces_recorded_energy():
    """The plain-C program (tests/c_consumer/md_step.c: staf_load, staf_compute with the library's own neighbour
    list, staf_free) on the reference's 768-atom frame with its float32 model: E and rms(F) recorded by the
    reference (test/test-lammps-STAF-inference-STAF-comp/results/frames.csv:2); a second step on rigidly shifted
    coordinates gives the same energy and forces to rounding."""
    import subprocess
    d = os.path.join(GOLDEN, "frame_mbpol")
    r = subprocess.run([MD_STEP, os.path.join(GOLDEN, "model_float"), os.path.join(d, "pos_0"),
                        os.path.join(d, "box_0"), os.path.join(d, "type.dat"), "0", "2"],
                       capture_output=True, text=True, timeout=110)
    assert r.returncode == 0, (r.stdout, r.stderr)
    lines = [l.split() for l in r.stdout.splitlines() if l.startswith("step")]
    assert len(lines) == 2 and all(l[3] == "0" for l in lines)
    e = [float(l[5]) for l in lines]
    rms = [float(l[7]) for l in lines]
    ka = KNOWN["frame0_model_float"]
    assert abs(e[0] - ka["E_lammps"]) < 1.5e-4 and abs(rms[0] - ka["rms_F_python"]) < 5e-6
    # float32 network: the shifted coordinates round differently (same bounds as the permutation check above)
    assert abs(e[1] - e[0]) < 1e-5 * abs(e[0]) and abs(rms[1] - rms[0]) < 2e-5
    vir = [float(x) for x in lines[0][9:15]]
    assert vir[3] == vir[4] == vir[5] == 0.0 and all(v != 0.0 for v in vir[:3])
