"""Descriptors and fingerprints of all species in one launch (staf_op_descriptors_fingerprints) against the ops it
stands for, on a real MI355X: every descriptor tensor and every fingerprint array bit for bit (the launch runs the
same code per centre as staf_op_compute_descriptors_light, staf_op_angular_afs and staf_op_radial_afs; those are
held to the oracle in test_gpu_parity.py), and one case directly against the oracle."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _separate(ops, torch, pos, box, tm, tipos, P, with2):
    d = ops.compute_descriptors_light(pos, box)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = d
    af3, af2, o = [], [], 0
    nt = len(tipos)
    for k, n in enumerate(tipos):
        s = slice(o, o + n)
        o += n
        af3.append(ops.compute_sort_proj3body(ang[:, s], sup[:, s], im3[:, s], im2[:, s], P[k]["alpha3b"],
                                              P[k]["emb3b"], tm, ntr[:, s], nt=nt))
        if with2:
            af2.append(ops.compute_sort_proj(rad[:, s], im2[:, s], P[k]["alpha2b"], P[k]["emb2b"], tm))
    return d, af3, af2


def _check(ops, torch, pos, box, tm, tipos, P, with2=True):
    want_d, want3, want2 = _separate(ops, torch, pos, box, tm, tipos, P, with2)
    got_d, got3, got2 = ops.compute_descriptors_fingerprints(
        pos, box, tm, tipos, [p["alpha3b"] for p in P], [p["emb3b"] for p in P],
        [p["alpha2b"] for p in P] if with2 else None, [p["emb2b"] for p in P] if with2 else None)
    ops.poll_status()
    names = ("raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp", "numtriplet")
    for name, a, b in zip(names, want_d, got_d):
        if name == "der3b":   # beyond an atom's triplets der3b is left as it was: compare what is written
            ntr = want_d[8].to(torch.int64)
            m = torch.clamp(ntr * (ntr - 1) // 2, max=a.shape[-1] // 2)
            idx = torch.arange(a.shape[-1] // 2, device=a.device)
            live = (idx[None, None, :] < m[:, :, None])[:, :, None, :, None].expand(a.shape[0], a.shape[1], 3, -1, 2)
            a = torch.where(live, a.view(a.shape[0], a.shape[1], 3, -1, 2), torch.zeros((), dtype=a.dtype, device=a.device))
            b = torch.where(live, b.view(b.shape[0], b.shape[1], 3, -1, 2), torch.zeros((), dtype=b.dtype, device=b.device))
        assert torch.equal(a, b), name
    for k in range(len(tipos)):
        assert got3[k].shape == want3[k].shape and torch.equal(got3[k], want3[k]), f"three_body_afs[{k}]"
        if with2:
            assert got2[k].shape == want2[k].shape and torch.equal(got2[k], want2[k]), f"radial_afs[{k}]"
    if not with2:
        assert got2 is None
    return got_d, got3, got2


def _water(name, dtype, nf=None, dense=False):
    import torch
    from alphanesgpu_amd import ops, synth
    b = synth.water_batch(name)
    nf = b["nf"] if nf is None else nf
    tdt = torch.float32 if np.dtype(dtype) == np.float32 else torch.float64
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box = T(b["pos"][:nf].astype(dtype)), T(b["box"][:nf].astype(dtype))
    params = synth.fingerprint_params(dtype=np.dtype(dtype), dense_embedding=dense)
    P = [{k: T(v) for k, v in m.items()} for m in params]
    ops.construct_descriptors_light(synth.RC, synth.NR, synth.NA, b["N"], box, synth.RS, synth.RA, nf, dtype=tdt)
    return ops, torch, pos, box, T(b["type_map"]), [int(x) for x in b["tipos"]], P, b, params


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_one_launch_gives_the_bits_of_the_three_ops(dtype):
    ops, torch, pos, box, tm, tipos, P, _, _ = _water("water768_f64", dtype, nf=2)
    _check(ops, torch, pos, box, tm, tipos, P)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_dense_embeddings_and_no_two_body_part(dtype):
    ops, torch, pos, box, tm, tipos, P, _, _ = _water("water96", dtype, dense=True)
    _check(ops, torch, pos, box, tm, tipos, P, with2=False)
    _check(ops, torch, pos, box, tm, tipos, P, with2=True)


def test_cell_list_frames():
    """6144 atoms: the neighbour search of the launch goes through the cell list."""
    ops, torch, pos, box, tm, tipos, P, _, _ = _water("water6144", np.float64)
    _check(ops, torch, pos, box, tm, tipos, P)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_three_species_one_of_them_empty(dtype):
    import torch
    from alphanesgpu_amd import ops, synth
    rng = np.random.default_rng(8)
    tip = [6, 0, 7]
    n = sum(tip)
    pts = []
    while len(pts) < n:
        c = rng.uniform(-3.0, 3.0, 3)
        if all(np.linalg.norm(c - q) > 0.9 for q in pts):
            pts.append(c)
    dev = torch.device("cuda:0")
    tdt = torch.float32 if np.dtype(dtype) == np.float32 else torch.float64
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos = T(np.array(pts).reshape(1, -1).astype(dtype))
    box = T(np.array([[13.0, 0, 0, 14.0, 0, 15.0]]).astype(dtype))
    params = synth.fingerprint_params(nt=3, ar_map=(3, 2, 4), aa_map=(2, 3, 2, 2, 3, 2), dtype=np.dtype(dtype),
                                      dense_embedding=True)
    P = [{k: T(v) for k, v in m.items()} for m in params]
    tm = T(np.repeat(np.arange(3), tip).astype(np.int32))
    ops.construct_descriptors_light(4.5, 16, 60, n, box, 1.5, 3.5, 1, dtype=tdt)
    _, af3, af2 = _check(ops, torch, pos, box, tm, tip, P)
    assert af3[1].shape == (1, 0, 14) and af2[1].shape == (1, 0, 9)


def test_against_the_oracle(oracle):
    """fp64, two 768-atom frames: fingerprints of the launch within 1e-12 of the oracle's."""
    import pipeline
    from util import nerr
    ops, torch, pos, box, tm, tipos, P, b, params = _water("water768_f64", np.float64, nf=2)
    _, af3, af2 = ops.compute_descriptors_fingerprints(pos, box, tm, tipos, [p["alpha3b"] for p in P],
                                                       [p["emb3b"] for p in P], [p["alpha2b"] for p in P],
                                                       [p["emb2b"] for p in P])
    ops.poll_status()
    from alphanesgpu_amd import synth
    up = synth.synthetic_upstream(2, b["tipos"], params, 11, np.float64)
    ref = pipeline.run_oracle(oracle, b["pos"][:2], b["box"][:2], b["tipos"], b["type_map"], params, up, synth.NR,
                              synth.NA, np.float64)
    for k in range(2):
        assert nerr(af3[k].cpu().numpy(), ref["af3"][k]) < 1e-12
        assert nerr(af2[k].cpu().numpy(), ref["af2"][k]) < 1e-12


def test_bad_arguments_are_refused():
    from alphanesgpu_amd import _lib
    ops, torch, pos, box, tm, tipos, P, _, _ = _water("water96", np.float64)
    with pytest.raises(_lib.StafError):   # species counts that do not sum to the number of atoms
        ops.compute_descriptors_fingerprints(pos, box, tm, [tipos[0], tipos[1] - 1], [p["alpha3b"] for p in P],
                                             [p["emb3b"] for p in P])


def test_layer_gives_the_outputs_and_gradients_of_the_separate_layers():
    """layers.descriptor_physics_layer against descriptor_layer + one physics_layer per species: same descriptor
    tensors, same fingerprints, and the same parameter gradients of a loss that is linear in the fingerprints."""
    import torch
    from alphanesgpu_amd import layers, synth
    dev = torch.device("cuda:0")
    b = synth.water_batch("water96")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box, tm = T(b["pos"]), T(b["box"]), T(b["type_map"])
    tipos = [int(x) for x in b["tipos"]]
    params = synth.fingerprint_params(dtype=np.float64, dense_embedding=True)
    desc = layers.descriptor_layer(synth.RC, synth.NR, synth.RA, synth.NA, b["N"], box, synth.RS, b["nf"])

    def physics():
        return [layers.physics_layer(T(m["alpha2b"]), T(m["alpha3b"]), [T(np.sqrt(m["emb2b"])), T(np.sqrt(m["emb3b"]))])
                for m in params]

    rng = np.random.default_rng(3)
    weights = [T(rng.standard_normal((b["nf"], n, params[0]["alpha2b"].shape[1] + params[0]["alpha3b"].shape[1] // 3)))
               for n in tipos]
    # the separate layers
    ph = physics()
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = desc(pos, box)
    want, first = [], 0
    for k, n in enumerate(tipos):
        s = slice(first, first + n)
        first += n
        want.append(ph[k](rad[:, s], sup[:, s], im2[:, s], ang[:, s], im3[:, s], ntr[:, s], tm))
    sum((w * a).sum() for w, a in zip(weights, want)).backward()
    # one launch
    ph1 = physics()
    both = layers.descriptor_physics_layer(desc, ph1, tipos)
    d1, got = both(pos, box, tm)
    sum((w * a).sum() for w, a in zip(weights, got)).backward()
    for a, c in zip((rad, ang, sup, im2, im3, d2, d3s, ntr), (d1[0], d1[1], d1[2], d1[3], d1[4], d1[5], d1[7], d1[8])):
        assert torch.equal(a, c)
    for k in range(len(tipos)):
        assert torch.equal(want[k], got[k])
        for name in ("alpha2b", "alpha3b", "type_emb_2b", "type_emb_3b"):
            g0, g1 = getattr(ph[k], name).grad, getattr(ph1[k], name).grad
            assert g0 is not None and g1 is not None and torch.equal(g0, g1), (k, name)


def test_random_configurations():
    """Twelve seeded random configurations through the one-launch entry and the three ops: 1-3 species with 1-13
    atoms each, 1-3 frames, orthorhombic and triclinic boxes with the cluster shifted far outside the cell, random
    cutoffs Rs < Ra <= Rc, 1-6 channels per block, an angular buffer anywhere between the atom count and the full
    triangle (truncated triplet lists included), either precision, block or dense embeddings; once per case the
    species are also computed by one call each."""
    import torch
    from alphanesgpu_amd import ops, synth
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(20250307)
    for case in range(12):
        nt = int(rng.integers(1, 4))
        tip = [int(x) for x in rng.integers(1, 14, nt)]
        n = sum(tip)
        nf = int(rng.integers(1, 4))
        L = float(rng.uniform(9.5, 16.0))
        spread = float(rng.uniform(2.2, 4.5))
        tric = float(rng.random() < 0.5)
        pos, box = np.zeros((nf, 3 * n)), np.zeros((nf, 6))
        for b in range(nf):
            pts = []
            while len(pts) < n:
                c = rng.uniform(-spread, spread, 3)
                if all(np.linalg.norm(c - q) > 0.85 for q in pts):
                    pts.append(c)
            pos[b] = (np.array(pts) + rng.uniform(-30, 30, 3)).reshape(-1)
            box[b] = [L, 0.6 * tric, -0.3 * tric, L + 0.7, 0.4 * tric, L + 1.3]
        rc = float(rng.uniform(3.0, 4.6))
        ra = float(rng.uniform(2.0, rc))
        rs = float(rng.uniform(0.9, 0.5 * rc))
        nr = n + 2
        na = int(rng.integers(max(3, n), nr * (nr - 1) // 2 + 1))
        ar = tuple(int(x) for x in rng.integers(1, 7, nt))
        aa = tuple(int(x) for x in rng.integers(1, 7, nt * (nt + 1) // 2))
        dtype = np.float64 if rng.random() < 0.6 else np.float32
        dense = bool(rng.random() < 0.5)
        tdt = torch.float32 if dtype == np.float32 else torch.float64
        params = synth.fingerprint_params(nt=nt, ar_map=ar, aa_map=aa, seed=case + 1, dtype=np.dtype(dtype),
                                          dense_embedding=dense)
        P = [{k: T(v) for k, v in m.items()} for m in params]
        tpos, tbox = T(pos.astype(dtype)), T(box.astype(dtype))
        tm = T(np.repeat(np.arange(nt), tip).astype(np.int32))
        ops.construct_descriptors_light(rc, nr, na, n, tbox, rs, ra, nf, dtype=tdt)
        try:
            _check(ops, torch, tpos, tbox, tm, tip, P)
            # species by species into one set of tensors
            want_d, want3, want2 = _separate(ops, torch, tpos, tbox, tm, tip, P, True)
            out = None
            for k in range(nt):
                out, af3, af2 = ops.compute_descriptors_fingerprints(
                    tpos, tbox, tm, tip, [p["alpha3b"] for p in P], [p["emb3b"] for p in P],
                    [p["alpha2b"] for p in P], [p["emb2b"] for p in P], out=out, species=(k, 1))
                assert torch.equal(af3[k], want3[k]) and torch.equal(af2[k], want2[k])
            ops.poll_status()
            for idx in (0, 1, 2, 3, 4, 5, 7, 8):
                assert torch.equal(out[idx], want_d[idx]), idx
        except AssertionError as e:
            raise AssertionError(f"case {case}: nt={nt} tipos={tip} nf={nf} rc={rc:.2f} ra={ra:.2f} rs={rs:.2f} "
                                 f"nr={nr} na={na} ar={ar} aa={aa} {np.dtype(dtype).name} dense={dense}: {e}") from e


def test_radial_overflow_is_reported_by_the_launch_too():
    """More neighbours than radial_buffer: STAF_E_RADIAL_OVERFLOW as from the descriptor op, every kernel exits
    normally, and a call with a large enough buffer right afterwards gives the bits of the three ops."""
    import torch
    from alphanesgpu_amd import ops, synth, _lib
    b = synth.water_batch("water96")
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box, tm = T(b["pos"]), T(b["box"]), T(b["type_map"])
    tipos = [int(x) for x in b["tipos"]]
    params = synth.fingerprint_params(dtype=np.float64)
    P = [{k: T(v) for k, v in m.items()} for m in params]
    ops.construct_descriptors_light(4.5, 20, 190, b["N"], None, 2.25, 4.5, 1, dtype=torch.float64)
    with pytest.raises(_lib.StafError) as e:
        ops.compute_descriptors_fingerprints(pos, box, tm, tipos, [p["alpha3b"] for p in P], [p["emb3b"] for p in P],
                                             [p["alpha2b"] for p in P], [p["emb2b"] for p in P])
    assert e.value.code == -10
    ops.construct_descriptors_light(synth.RC, synth.NR, synth.NA, b["N"], box, synth.RS, synth.RA, 1, dtype=torch.float64)
    _check(ops, torch, pos, box, tm, tipos, P)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_wide_channel_sets(dtype):
    """Three species with 141 three-body and 57 two-body channels (classes of up to 42 active channels: three table
    chunks, and in double precision an LDS request beyond what a launch gets without asking)."""
    import torch
    from alphanesgpu_amd import ops, synth
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    rng = np.random.default_rng(21)
    tip = [18, 15, 13]
    n = sum(tip)
    pts = []
    while len(pts) < n:
        c = rng.uniform(-3.2, 3.2, 3)
        if all(np.linalg.norm(c - q) > 0.75 for q in pts):
            pts.append(c)
    pos = T((np.array(pts) + rng.uniform(-5, 5, 3)).reshape(1, -1).astype(dtype))
    box = T(np.array([[16.0, 0.5, -0.3, 16.7, 0.4, 17.3]]).astype(dtype))
    params = synth.fingerprint_params(nt=3, ar_map=(11, 16, 30), aa_map=(12, 5, 40, 4, 42, 38), seed=2,
                                      dtype=np.dtype(dtype))
    P = [{k: T(v) for k, v in m.items()} for m in params]
    tm = T(np.repeat(np.arange(3), tip).astype(np.int32))
    tdt = torch.float32 if np.dtype(dtype) == np.float32 else torch.float64
    ops.construct_descriptors_light(5.4, n + 2, 938, n, box, 1.5, 4.9, 1, dtype=tdt)
    _check(ops, torch, pos, box, tm, tip, P)


def test_hip_graph_replay_of_the_species_launches_matches_eager():
    """One launch per species, each followed by the species' slot forces, on the species' own stream, the collecting
    launch on the step's stream; captured once into a HIP graph: every replay, with eager steps and
    synchronisations in between, gives the eager single-stream result bit for bit."""
    import torch
    from alphanesgpu_amd import ops, synth
    dev = torch.device("cuda:0")
    b = synth.water_batch("water96")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box, tm, tp = T(b["pos"]), T(b["box"]), T(b["type_map"]), T(b["tipos"])
    tipos = [int(x) for x in b["tipos"]]
    nt, nf, N = len(tipos), b["nf"], b["N"]
    params = synth.fingerprint_params(dtype=np.float64)
    P = [{k: T(v) for k, v in m.items()} for m in params]
    up = synth.synthetic_upstream(nf, b["tipos"], params, 3, np.float64)
    G2, G3 = [T(x) for x in up["G2"]], [T(x) for x in up["G3"]]
    at = [torch.tensor([k], dtype=torch.int32, device=dev) for k in range(nt)]
    nr, na = synth.NR, synth.NA
    ops.construct_descriptors_light(synth.RC, nr, na, N, box, synth.RS, synth.RA, nf, dtype=torch.float64)
    e = lambda *sh: torch.empty(sh, dtype=torch.float64, device=dev)
    ei = lambda *sh: torch.empty(sh, dtype=torch.int32, device=dev)
    dbuf = (e(nf, N, nr), e(nf, N, na), e(nf, N, nr), ei(nf, N, nr + 1), ei(nf, N, 2 * na), e(nf, N, 3, nr),
            e(nf, N, 3, 2 * na), e(nf, N, 3, nr), ei(nf, N))
    side = [torch.cuda.Stream() for _ in range(nt)]
    lists = ([p["alpha3b"] for p in P], [p["emb3b"] for p in P], [p["alpha2b"] for p in P], [p["emb2b"] for p in P])
    first = [sum(tipos[:k]) for k in range(nt)]

    def species(k):
        d, af3, af2 = ops.compute_descriptors_fingerprints(pos, box, tm, tipos, *lists, out=dbuf, species=(k, 1))
        rad, ang, sup, im2, im3, d2, d3, d3s, ntr = [x[:, first[k]:first[k] + tipos[k]] for x in d]
        p = P[k]
        slots = ops.compute_forces_slots(G3[k], G2[k], sup, ang, d3s, d3, rad, d2, im2, im3, p["alpha3b"], p["emb3b"],
                                         p["alpha2b"], p["emb2b"], tm, tp, at[k], ntr)
        return af3[k], af2[k], slots

    def step(streams):
        outs = [None] * nt
        if streams is None:
            for k in range(nt):
                outs[k] = species(k)
        else:
            main = torch.cuda.current_stream()
            ready = main.record_event()
            done = []
            for k in sorted(range(nt), key=lambda k: -tipos[k]):
                with torch.cuda.stream(streams[k]):
                    streams[k].wait_event(ready)
                    outs[k] = species(k)
                    done.append(streams[k].record_event())
            for ev in done:
                main.wait_event(ev)
        total = ops.force_total(dbuf[3], tipos, [o[2][0] for o in outs], [o[2][1] for o in outs])
        return [o[0] for o in outs] + [o[1] for o in outs] + [total]

    ops.set_sync_errors(False)
    try:
        want = [t.clone() for t in step(None)]
        step(side)                      # sizes the per-stream work areas before the capture
        ops.poll_status()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            held = step(side)
        for rep in range(3):
            g.replay()
            torch.cuda.synchronize()
            for x, y in zip(held, want):
                assert torch.equal(x, y), f"replay {rep}"
            again = step(None)          # eager work between the replays
            ops.poll_status()
            torch.cuda.synchronize()
            for x, y in zip(again, want):
                assert torch.equal(x, y)
    finally:
        ops.set_sync_errors(True)
