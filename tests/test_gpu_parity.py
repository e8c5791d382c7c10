"""Parity of the HIP library against the CPU oracle, through the C ABI, on a real MI355X.

Bars: neighbour lists and every other integer output bit-exact over the whole arrays, padding included;
floating-point outputs within 1e-12 (fp64) / 1e-5 (fp32) of the oracle, in two measures that both have to hold:
the normalised error max|a-b| / max|b| per tensor, and element by element |a-b| <= tol |b| + tol rms(b)
(util.eerr).  der3b is compared on active slots (its padding is unspecified in the reference); every other
padding must be exactly 0.
"""
import numpy as np
import pytest

from util import eerr, load_frame_mbpol, load_model, nerr, radial_mask, triplet_mask
import pipeline

pytestmark = pytest.mark.gpu

TOL = {np.dtype(np.float32): 1e-5, np.dtype(np.float64): 1e-12}
NR, NA = 60, 1770


def _synth(name, nf=None):
    from alphanesgpu_amd import synth
    b = synth.water_batch(name)
    if nf is not None:
        b["pos"] = b["pos"][:nf]
        b["box"] = b["box"][:nf]
        b["nf"] = nf
    return b


def _params(dtype, dense=False, seed=7):
    from alphanesgpu_amd import synth
    return synth.fingerprint_params(dtype=dtype, dense_embedding=dense, seed=seed)


def compare(ref, got, dtype, nr=NR, na=NA, truth=None):
    """ref: oracle in `dtype`; got: HIP library in `dtype`.  For fp32, `truth` is the fp64 oracle evaluated on the
    fp32 oracle's descriptor tensors, i.e. the exactly rounded value of every downstream op on the same fp32 inputs:
    the library must be within 1e-5 of it.  (Its distance from the fp32 oracle is then at most 1e-5 plus the fp32
    oracle's own sequential-summation error; the reference accumulates these sums with float atomics in arbitrary
    order and is itself only defined to that level.  Where the fp32 oracle's own error is below 1e-5 -- everything
    but the parameter gradients, which are sums over all atoms of all frames -- the library is also held to
    1e-5 of the fp32 oracle directly.)"""
    tol = TOL[np.dtype(dtype)]
    d0, d1 = ref["desc"], got["desc"]
    # integer outputs: bit-exact, whole arrays
    for k in ("intmap2b", "intmap3b", "numtriplet"):
        assert np.array_equal(d0[k], d1[k]), f"{k} differs"
    rm = radial_mask(d0["intmap2b"], nr)
    tm = triplet_mask(d0["numtriplet"], na)
    errs = {}
    for k in ("raddescr", "des3bsupp"):
        errs[k] = max(nerr(d1[k] * rm, d0[k] * rm), eerr(d1[k], d0[k], where=rm))
        assert np.all(d1[k][~rm] == 0), f"{k} padding not zero"
    rm3 = np.broadcast_to(rm[:, :, None, :], d0["der2b"].shape)
    for k in ("der2b", "der3bsupp"):
        errs[k] = max(nerr(d1[k] * rm3, d0[k] * rm3), eerr(d1[k], d0[k], where=rm3))
        assert np.all(d1[k][~rm3] == 0)
    errs["angdescr"] = max(nerr(d1["angdescr"], d0["angdescr"]), eerr(d1["angdescr"], d0["angdescr"], where=tm))
    assert np.all(d1["angdescr"][~tm] == 0)
    nf, N = d0["numtriplet"].shape
    m3 = np.repeat(tm[:, :, None, :], 3, axis=2)
    m3 = np.repeat(m3[..., None], 2, axis=-1).reshape(nf, N, 3, 2 * na)
    errs["der3b"] = max(nerr(np.where(m3, d1["der3b"], 0), np.where(m3, d0["der3b"], 0)),
                        eerr(d1["der3b"], d0["der3b"], where=m3))

    def check(name, x, y, z, long_sum=False):
        if z is None:
            errs[name] = max(nerr(x, y), eerr(x, y))
        else:
            errs[name] = max(nerr(x, z), eerr(x, z))   # library vs exact value: must meet the tolerance
            own = nerr(y, z)                             # fp32 oracle's own distance from the exact value
            lim = tol + own if long_sum else tol
            assert nerr(x, y) <= lim, f"{name}: {nerr(x, y)} from the fp32 oracle (its own error {own})"

    for key in ("af2", "af3", "f2", "f3"):
        for k, (a, b) in enumerate(zip(got[key], ref[key])):
            check(f"{key}[{k}]", a, b, None if truth is None else truth[key][k])
    for key, names in (("g2", ("alpha", "emb")), ("g3", ("alpha", "emb")), ("gf2", ("net", "alpha", "emb")),
                       ("gf3", ("net", "alpha", "emb"))):
        for k, (a, b) in enumerate(zip(got[key], ref[key])):
            for i, (nm, x, y) in enumerate(zip(names, a, b)):
                if key in ("g3", "gf3") and nm == "emb":
                    assert np.all(x == 0) and np.all(y == 0), "emb3b gradients must be identically zero"
                else:
                    check(f"{key}[{k}].{nm}", x, y, None if truth is None else truth[key][k][i], long_sum=nm != "net")
    bad = {k: v for k, v in errs.items() if not (v <= tol)}
    assert not bad, f"beyond {tol}: {bad}"
    return errs


def _truth(oracle, ref, b_tipos, type_map, params, up, dtype):
    if np.dtype(dtype) != np.float32:
        return None
    d, p, u = pipeline.promote(ref, params, up)
    return pipeline.run_oracle(oracle, None, None, b_tipos, type_map, p, u, NR, NA, np.float64, desc=d)


def _run_case(oracle, b, dtype, dense=False, fma_mode=0, views=True, seed=11):
    dtype = np.dtype(dtype)
    params = _params(dtype, dense)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    up = pipeline.synthetic_upstream(box.shape[0], b["tipos"], params, seed, dtype)
    ref = pipeline.run_oracle(oracle, pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype, fma_mode)
    got = pipeline.run_hip(pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype, fma_mode, views)
    return compare(ref, got, dtype, truth=_truth(oracle, ref, b["tipos"], b["type_map"], params, up, dtype))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_water96_all_ops(oracle, dtype):
    """Config 1 (96 atoms, box 9.86 < 3 Rc: every cell is a neighbour cell) -- all ops, both precisions."""
    print(_run_case(oracle, _synth("water96"), dtype))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_water96_dense_embedding(oracle, dtype):
    """Non-block embeddings: every channel active for every species pair."""
    _run_case(oracle, _synth("water96"), dtype, dense=True)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_water768_two_frames(oracle, dtype):
    """768-atom generator, two frames in one batch (frame stride paths), views of the descriptor outputs."""
    _run_case(oracle, _synth("water768_f64", nf=2), dtype)


def test_water768_contiguous_splits(oracle):
    """Per-species tensors passed as contiguous copies (what tf.split hands the reference ops)."""
    _run_case(oracle, _synth("water768_f64", nf=2), np.float32, views=False)


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_dist2_fma_mode(oracle, dtype):
    """Neighbour test evaluated as fma(z,z,fma(y,y,x*x)) in both oracle and kernel: still bit-exact."""
    _run_case(oracle, _synth("water96"), dtype, fma_mode=1)


@pytest.mark.parametrize("prec,dtype", [("float", np.float32), ("double", np.float64)])
def test_reference_frame_and_model(oracle, prec, dtype):
    """The reference's own 768-atom MB-pol frame with its exported trained parameters."""
    pos, box, tipos, type_map = load_frame_mbpol(dtype)
    _, model = load_model(prec)
    params = [{k: m[k] for k in ("alpha2b", "alpha3b", "emb2b", "emb3b")} for m in model]
    up = pipeline.synthetic_upstream(1, tipos, params, 5, dtype)
    ref = pipeline.run_oracle(oracle, pos, box, tipos, type_map, params, up, NR, NA, dtype)
    got = pipeline.run_hip(pos, box, tipos, type_map, params, up, NR, NA, dtype)
    compare(ref, got, dtype, truth=_truth(oracle, ref, tipos, type_map, params, up, dtype))
    assert ref["desc"]["intmap2b"][..., 0].max() == 48


def test_bit_reproducible(oracle):
    """Two runs of the whole sequence give identical bits (no float atomics anywhere)."""
    b = _synth("water768_f32", nf=1)
    dtype = np.dtype(np.float32)
    params = _params(dtype)
    up = pipeline.synthetic_upstream(1, b["tipos"], params, 3, dtype)
    r1 = pipeline.run_hip(b["pos"], b["box"], b["tipos"], b["type_map"], params, up, NR, NA, dtype)
    r2 = pipeline.run_hip(b["pos"], b["box"], b["tipos"], b["type_map"], params, up, NR, NA, dtype)
    for key in ("af2", "af3", "f2", "f3", "g2", "g3", "gf2", "gf3"):
        for a, c in zip(r1[key], r2[key]):
            if isinstance(a, tuple):
                for x, y in zip(a, c):
                    assert np.array_equal(x, y), key
            else:
                assert np.array_equal(a, c), key


def test_radial_overflow_is_reported():
    """More neighbours than radial_buffer: the reference exits; the library returns STAF_E_RADIAL_OVERFLOW."""
    import torch
    from alphanesgpu_amd import ops, _lib
    b = _synth("water96")
    dev = torch.device("cuda:0")
    ops.construct_descriptors_light(4.5, 20, 190, b["N"], None, 2.25, 4.5, 1, dtype=torch.float64)
    with pytest.raises(_lib.StafError) as e:
        ops.compute_descriptors_light(torch.as_tensor(b["pos"]).to(dev), torch.as_tensor(b["box"]).to(dev))
    assert e.value.code == -10
    # deferred mode: nothing raised by the op, the poll reports it
    ops.set_sync_errors(False)
    try:
        ops.compute_descriptors_light(torch.as_tensor(b["pos"]).to(dev), torch.as_tensor(b["box"]).to(dev))
        with pytest.raises(_lib.StafError) as e2:
            ops.poll_status()
        assert e2.value.code == -10
        ops.poll_status()  # cleared
    finally:
        ops.set_sync_errors(True)


def test_condition_stays_with_the_stream_that_raised_it():
    """Each stream has its own error word: an overflow raised (and left unfetched) on a side stream does not
    make a later, valid op on another stream return it; the poll, which reads every word, still reports it."""
    import torch
    from alphanesgpu_amd import ops, _lib
    b = _synth("water96")
    dev = torch.device("cuda:0")
    pos, box = torch.as_tensor(b["pos"]).to(dev), torch.as_tensor(b["box"]).to(dev)
    side = torch.cuda.Stream()
    torch.cuda.synchronize()
    ops.set_sync_errors(False)
    try:
        ops.construct_descriptors_light(4.5, 20, 190, b["N"], None, 2.25, 4.5, 1, dtype=torch.float64)
        with torch.cuda.stream(side):
            ops.compute_descriptors_light(pos, box)
        side.synchronize()
        ops.set_sync_errors(True)
        ops.construct_descriptors_light(4.5, 60, 1770, b["N"], None, 2.25, 4.5, 1, dtype=torch.float64)
        ops.compute_descriptors_light(pos, box)   # valid, on the default stream: returns STAF_OK
        with pytest.raises(_lib.StafError) as e:
            ops.poll_status()
        assert e.value.code == -10
        ops.poll_status()  # cleared
    finally:
        ops.set_sync_errors(True)


def test_compute_before_construct_other_precision():
    import torch
    from alphanesgpu_amd import ops, _lib
    ops._constructed.pop(torch.float32, None)
    with pytest.raises(_lib.StafError) as e:
        ops.compute_descriptors_light(torch.zeros(1, 9, device="cuda:0"), torch.ones(1, 6, device="cuda:0"))
    assert e.value.code == -1


def test_full_size_properties(oracle):
    """The benchmark's headline configuration at full size (768 atoms, 4 frames, fp32): size-independent checks.
    Newton's third law (sum of forces = 0 per frame), linearity of the force ops in G, and the exact
    adjoint relation between the force op and its gradient: sum(Q * F(G)) == sum(G * dG(Q))."""
    import torch
    from alphanesgpu_amd import ops
    b = _synth("water768_f32")
    dtype = np.dtype(np.float64)  # properties checked in fp64 for sharp thresholds
    params = _params(dtype)
    nf = b["nf"]
    up = pipeline.synthetic_upstream(nf, b["tipos"], params, 9, dtype)
    got = pipeline.run_hip(b["pos"].astype(dtype), b["box"].astype(dtype), b["tipos"], b["type_map"], params, up, NR,
                           NA, dtype)
    for k in range(2):
        for key, G in (("f2", up["G2"][k]), ("f3", up["G3"][k])):
            F = got[key][k].reshape(nf, -1, 3)
            assert np.abs(F.sum(1)).max() < 1e-10 * np.abs(F).max() * F.shape[1]
            gnet = got["gf2" if key == "f2" else "gf3"][k][0]
            lhs = float((up["Q"] * got[key][k]).sum())
            rhs = float((G * gnet).sum())
            assert abs(lhs - rhs) <= 1e-10 * max(abs(lhs), 1.0), (key, k, lhs, rhs)
    ntr = got["desc"]["numtriplet"]
    assert got["desc"]["intmap2b"][..., 0].max() <= NR and (ntr * (ntr - 1) // 2).max() <= NA


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_virial_forms(oracle, dtype):
    """ComputeForce{Radial,Tripl}Virial and their *VirialGrad ops against the oracle: forces unchanged, W [nf,9],
    and gradients with a non-zero dL/dW.  Two frames of the 768-atom generator (periodic images matter)."""
    import torch
    from alphanesgpu_amd import ops
    from util import species_slices
    dtype = np.dtype(dtype)
    tol = TOL[dtype]
    b = _synth("water768_f64", nf=2)
    params = _params(dtype, dense=True)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    nf = 2
    up = pipeline.synthetic_upstream(nf, b["tipos"], params, 21, dtype)
    rng = np.random.Generator(np.random.Philox(5))
    Wg = rng.standard_normal((nf, 9)).astype(dtype)
    d = oracle.compute_descriptors_light(pos, box, 4.5, 4.5, 2.25, NR, NA, dtype=dtype)
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    ops.construct_descriptors_light(4.5, NR, NA, b["N"], None, 2.25, 4.5, nf, dtype=tdt)
    ops.descriptor_options(False, True)
    names = ["raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp", "numtriplet"]
    g = dict(zip(names, ops.compute_descriptors_light(T(pos), T(box))))
    tm, tp = T(b["type_map"]), T(b["tipos"])
    Q, tWg, tpos, tbox = T(up["Q"]), T(Wg), T(pos), T(box)
    f64 = lambda x: x.astype(np.float64) if isinstance(x, np.ndarray) and x.dtype == np.float32 else x
    for k, s in enumerate(species_slices(b["tipos"])):
        m = params[k]
        c = lambda a: np.ascontiguousarray(a[:, s])
        v = lambda key: g[key][:, s]
        tk = {kk: T(vv) for kk, vv in m.items()}
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        a2 = (c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]), m["alpha2b"], m["emb2b"], b["type_map"], b["tipos"], k)
        a3 = (c(d["des3bsupp"]), c(d["angdescr"]), c(d["der3bsupp"]), c(d["der3b"]), c(d["intmap2b"]),
              c(d["intmap3b"]), m["alpha3b"], m["emb3b"], b["type_map"], b["tipos"], k, c(d["numtriplet"]))

        def oracle_all(G2, G3, Q, W, a2, a3, pos, box):
            f2r, w2r = oracle.force_radial(G2, *a2, pos=pos, box=box)
            f3r, w3r = oracle.force_tripl(G3, *a3, pos=pos, box=box)
            g2r = oracle.force_radial_grad(Q, G2, *a2, prevgrad_virial=W, pos=pos, box=box)
            g3r = oracle.force_tripl_grad(Q, G3, *a3, prevgrad_virial=W, pos=pos, box=box)
            return dict(f2=f2r, w2=w2r, f3=f3r, w3=w3r, **{"g2.net": g2r[0], "g2.alpha": g2r[1], "g2.emb": g2r[2],
                                                           "g3.net": g3r[0], "g3.alpha": g3r[1]})

        ref = oracle_all(up["G2"][k], up["G3"][k], up["Q"], Wg, a2, a3, pos, box)
        # fp32: the exactly rounded values on the same fp32 inputs (fp64 oracle on promoted copies), see compare()
        exact = None
        if dtype == np.float32:
            exact = oracle_all(f64(up["G2"][k]), f64(up["G3"][k]), f64(up["Q"]), f64(Wg), tuple(f64(x) for x in a2),
                               tuple(f64(x) for x in a3), f64(pos), f64(box))
        f2, w2 = ops.compute_force_radial_virial(T(up["G2"][k]), v("der2b"), v("intmap2b"), v("raddescr"),
                                                 tk["alpha2b"], tk["emb2b"], tm, tp, at, tpos, tbox)
        f3, w3 = ops.compute_force_tripl_virial(T(up["G3"][k]), v("des3bsupp"), v("angdescr"), v("der3bsupp"),
                                                v("der3b"), v("intmap2b"), v("intmap3b"), tk["alpha3b"], tk["emb3b"],
                                                tm, tp, at, v("numtriplet"), tpos, tbox)
        g2 = ops.compute_force_radial_virial_grad(Q, tWg, T(up["G2"][k]), v("der2b"), v("intmap2b"), v("raddescr"),
                                                  tk["alpha2b"], tk["emb2b"], tm, tp, at, tpos, tbox)
        g3 = ops.compute_force_tripl_virial_grad(Q, tWg, T(up["G3"][k]), v("des3bsupp"), v("angdescr"),
                                                 v("der3bsupp"), v("der3b"), v("intmap2b"), v("intmap3b"),
                                                 tk["alpha3b"], tk["emb3b"], tm, tp, at, v("numtriplet"), tpos, tbox)
        got = dict(f2=f2, w2=w2, f3=f3, w3=w3, **{"g2.net": g2[0], "g2.alpha": g2[1], "g2.emb": g2[2],
                                                  "g3.net": g3[0], "g3.alpha": g3[1]})
        for name, x in got.items():
            x = x.cpu().numpy()
            if exact is None:
                e = max(nerr(x, ref[name]), eerr(x, ref[name]))
                assert e <= tol, (name, k, e)
            else:
                # sums over all centres of a frame (virial) or of the batch (parameter gradients): the fp32
                # oracle's own sequential-summation error is allowed on top when comparing with it
                e = max(nerr(x, exact[name]), eerr(x, exact[name]))
                assert e <= tol, (name, k, e)
                own = nerr(ref[name], exact[name])
                long_sum = name.startswith("w") or name.endswith((".alpha", ".emb"))
                assert nerr(x, ref[name]) <= tol + (own if long_sum else 0.0), (name, k, nerr(x, ref[name]), own)
        assert torch.all(g3[2] == 0)


def _generic_case(oracle, pos, box, tipos, dtype, nr, na, rc, ra, rs, nt, seed=5, dense=False, maps=None):
    """All ops on an arbitrary configuration: oracle and library with the same synthetic parameters."""
    from alphanesgpu_amd import synth
    dtype = np.dtype(dtype)
    tipos = np.asarray(tipos, np.int32)
    type_map = np.concatenate([np.full(n, k, np.int32) for k, n in enumerate(tipos)])
    kw = {} if maps is None else dict(ar_map=maps[0], aa_map=maps[1])   # one block per species / species pair
    params = synth.fingerprint_params(nt=nt, dtype=dtype, dense_embedding=dense, seed=seed, **kw)
    pos, box = pos.astype(dtype), box.astype(dtype)
    up = pipeline.synthetic_upstream(box.shape[0], tipos, params, seed, dtype)
    ref = pipeline.run_oracle(oracle, pos, box, tipos, type_map, params, up, nr, na, dtype, rc=rc, ra=ra, rs=rs)
    got = pipeline.run_hip(pos, box, tipos, type_map, params, up, nr, na, dtype, rc=rc, ra=ra, rs=rs)
    truth = None
    if dtype == np.float32:
        d, p, u = pipeline.promote(ref, params, up)
        truth = pipeline.run_oracle(oracle, None, None, tipos, type_map, p, u, nr, na, np.float64, desc=d)
    return compare(ref, got, dtype, nr=nr, na=na, truth=truth), ref


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_single_species_example(oracle, dtype):
    """The reference's single-species example (STAF/example_inference: 50 atoms, Rc = Ra = 22, Rs = 11, nr = 50,
    na = 1225): nt = 1, one parameter row, Ra = Rc so every neighbour is an angular one."""
    import os
    from util import GOLDEN
    d = os.path.join(GOLDEN, "frame_single_species")
    pos = np.loadtxt(os.path.join(d, "pos_0")).reshape(1, -1)
    box = np.loadtxt(os.path.join(d, "box_0")).reshape(1, 6)
    _generic_case(oracle, pos, box, [pos.shape[1] // 3], dtype, nr=50, na=1225, rc=22.0, ra=22.0, rs=11.0, nt=1,
                  maps=((20,), (40,)))


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_three_species_with_isolated_atoms(oracle, dtype):
    """nt = 3 (five parameter rows sigma, six species classes), dense embeddings, Ra < Rc, a triclinic box, and the
    ragged cases: an atom with no neighbour at all, a pair that only sees each other (no triplet), an atom with
    neighbours but fewer than two inside Ra."""
    rng = np.random.default_rng(2)
    tip = [7, 9, 8]
    n = sum(tip)
    L = 14.0
    pts = []
    while len(pts) < n - 4:                      # a loose cluster around the origin
        c = rng.uniform(-3.2, 3.2, 3)
        if all(np.linalg.norm(c - q) > 1.0 for q in pts):
            pts.append(c)
    pts += [np.array([6.5, 6.5, 6.5]),            # isolated
            np.array([-6.0, 6.0, 0.0]), np.array([-6.0, 6.0, 1.1]),   # a dimer far from everything
            np.array([0.0, -6.2, -6.2])]          # sees the cluster only beyond Ra, if at all
    pos = np.array(pts)
    order = rng.permutation(n)                    # species assigned at random, then stored species-sorted
    pos = pos[order].reshape(1, -1)
    box = np.array([[L, 0.7, -0.4, L + 1.0, 0.5, L + 2.0]])
    errs, ref = _generic_case(oracle, pos, box, tip, dtype, nr=24, na=276, rc=4.5, ra=3.2, rs=1.6, nt=3, dense=True,
                              maps=((5, 4, 6), (4, 3, 5, 3, 4, 3)))
    hm = ref["desc"]["intmap2b"][0, :, 0]
    ntr = ref["desc"]["numtriplet"][0]
    assert hm.min() == 0 and (hm == 1).sum() >= 2 and (ntr < hm).any()


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_angular_buffer_smaller_than_triplet_count(oracle, dtype):
    """angular_buffer below m(m-1)/2: the reference silently drops the triplets beyond it (its kernels span only na
    storage indices); the library must drop exactly the same ones in every op."""
    b = _synth("water96")
    ntr = None
    errs, ref = _generic_case(oracle, b["pos"], b["box"], b["tipos"], dtype, nr=60, na=400, rc=4.5, ra=4.5, rs=2.25,
                              nt=2)
    m = ref["desc"]["numtriplet"].astype(np.int64)
    assert ((m * (m - 1)) // 2 > 400).any()


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_cell_list_gives_the_same_descriptors(dtype):
    """Large frames find their neighbours through a cell list, small ones test every atom: every output of the
    descriptor op must have the same bits either way.  768 atoms (4 x 4 x 4 cells at Rc = 4.5), an orthorhombic and
    a sheared box, some atoms moved by whole lattice vectors (positions outside the box); boxes divided along no or
    one axis only; a frame with a cell that holds more atoms than the list has places for."""
    import torch
    from alphanesgpu_amd import ops, synth
    b = _synth("water768_f32")
    N, nf = b["N"], 2
    pos0 = b["pos"][:nf].astype(dtype).reshape(nf, N, 3)
    L = float(b["box"][0][0])
    tdt = torch.float64 if dtype == np.float64 else torch.float32
    rng = np.random.default_rng(5)
    try:
        for box6 in ([L, 0, 0, L, 0, L], [L, 0.3 * L, -0.2 * L, L, 0.25 * L, L]):
            a, bv, c = np.array([box6[0], 0, 0]), np.array([box6[1], box6[3], 0]), np.array([box6[2], box6[4], box6[5]])
            pos = pos0.copy()
            k = rng.integers(-2, 3, size=(nf, N, 3))
            moved = rng.random((nf, N)) < 0.2
            pos += (moved[..., None] * (k[..., :1] * a + k[..., 1:2] * bv + k[..., 2:] * c)).astype(dtype)
            box = np.tile(np.array(box6, dtype), (nf, 1))
            tp, tb = torch.as_tensor(pos.reshape(nf, -1)).cuda(), torch.as_tensor(box).cuda()
            ops.construct_descriptors_light(synth.RC, 80, NA, N, tb, synth.RS, synth.RA, nf, dtype=tdt)
            ops.descriptor_options(dist2_fma=False, zero_padding=True)
            ops.descriptor_cell_threshold(0)
            every = [x.clone() for x in ops.compute_descriptors_light(tp, tb)]
            ops.descriptor_cell_threshold(1)
            cells = ops.compute_descriptors_light(tp, tb)
            assert int(every[3][..., 0].min()) > 10      # intmap2b counts: a real neighbourhood everywhere
            for x, y in zip(every, cells):
                assert torch.equal(x, y)
        # a box too small to be divided (9.86 / 4.5 < 3: one cell per axis) and one divided along one axis only
        b96 = _synth("water96")
        p96 = b96["pos"][:1].astype(dtype)
        L9 = float(b96["box"][0][0])
        for box6, reps in (([L9, 0, 0, L9, 0, L9], 1), ([L9, 0, 0, L9, 0, 2 * L9], 2)):
            pos = p96.reshape(1, -1, 3)
            if reps == 2:
                pos = np.concatenate([pos, pos + np.array([0, 0, L9], dtype)], axis=1)
            n96 = pos.shape[1]
            box = np.array([box6], dtype)
            tp, tb = torch.as_tensor(np.ascontiguousarray(pos.reshape(1, -1))).cuda(), torch.as_tensor(box).cuda()
            ops.construct_descriptors_light(synth.RC, 80, NA, n96, tb, synth.RS, synth.RA, 1, dtype=tdt)
            ops.descriptor_options(dist2_fma=False, zero_padding=True)   # construct has reset the options
            ops.descriptor_cell_threshold(0)
            every = [x.clone() for x in ops.compute_descriptors_light(tp, tb)]
            ops.descriptor_cell_threshold(1)
            cells = ops.compute_descriptors_light(tp, tb)
            for x, y in zip(every, cells):
                assert torch.equal(x, y)
        # a cell with more atoms than it has places (nr = 80: 96 places): two clumps of 49 atoms in opposite corners of
        # one cell, out of each other's reach, in a thin gas.  The centres in and around that cell test every atom.
        Lg, ncell = 19.72, 4
        side = Lg / ncell
        lo = np.array([1.0, 2.0, 1.0]) * side
        ca, cb = lo + 0.45, lo + side - 0.45
        clump = lambda centre: centre + (rng.random((49, 3)) - 0.5) * 0.6
        gas = rng.random((160, 3)) * Lg
        far = lambda c: np.linalg.norm(gas - c - Lg * np.round((gas - c) / Lg), axis=1) > synth.RC + 0.6
        gas = gas[far(ca) & far(cb)]   # (an atom between the clumps would have both for neighbours)
        pos = np.concatenate([clump(ca), clump(cb), gas])
        pos = pos[rng.permutation(len(pos))]
        ng = len(pos)
        tp = torch.as_tensor(pos.reshape(1, -1).astype(dtype)).cuda()
        tb = torch.as_tensor(np.array([[Lg, 0, 0, Lg, 0, Lg]], dtype)).cuda()
        ops.construct_descriptors_light(synth.RC, 80, NA, ng, tb, synth.RS, synth.RA, 1, dtype=tdt)
        ops.descriptor_options(dist2_fma=False, zero_padding=True)
        ops.descriptor_cell_threshold(0)
        every = [x.clone() for x in ops.compute_descriptors_light(tp, tb)]
        ops.descriptor_cell_threshold(1)
        for _ in range(3):   # (the counters of the cells alternate between two sets from call to call)
            cells = ops.compute_descriptors_light(tp, tb)
            assert 48 <= int(every[3][..., 0].max()) < 80
            for x, y in zip(every, cells):
                assert torch.equal(x, y)
        # a thin frame: the 96-atom box 3 x 3 x 3 times, stretched by 1.3 -- 8 cells of width Rc fit along an axis, but
        # the grid has at most N / 8 = 324 cells: a coarser one (6 x 7 x 7) serves
        t = np.array([[x, y, z] for x in range(3) for y in range(3) for z in range(3)], dtype)
        pos = (1.3 * (p96.reshape(1, -1, 3) + L9 * t[:, None, :])).reshape(1, -1)
        nthin = pos.shape[1] // 3
        tp = torch.as_tensor(np.ascontiguousarray(pos.astype(dtype))).cuda()
        tb = torch.as_tensor(np.array([[3.9 * L9, 0, 0, 3.9 * L9, 0, 3.9 * L9]], dtype)).cuda()
        ops.construct_descriptors_light(synth.RC, 80, NA, nthin, tb, synth.RS, synth.RA, 1, dtype=tdt)
        ops.descriptor_options(dist2_fma=False, zero_padding=True)
        ops.descriptor_cell_threshold(0)
        every = [x.clone() for x in ops.compute_descriptors_light(tp, tb)]
        ops.descriptor_cell_threshold(1)
        cells = ops.compute_descriptors_light(tp, tb)
        assert nthin == 2592 and int(every[3][..., 0].min()) > 5
        for x, y in zip(every, cells):
            assert torch.equal(x, y)
    finally:
        ops.descriptor_cell_threshold(4096)


def test_cell_list_in_a_replayed_graph():
    """The descriptor op with the cell list, captured once in a HIP graph: the cells' counters alternate between two
    sets from call to call, also from replay to replay and across eager calls on the same stream in between.  Every
    replay, on new positions each time, gives what the search over all atoms gives for them, bit for bit."""
    import torch
    from alphanesgpu_amd import ops, synth
    b = _synth("water768_f32")
    N, nf = b["N"], 2
    pos0 = b["pos"][:nf].astype(np.float64).reshape(nf, -1)
    tb = torch.as_tensor(np.ascontiguousarray(b["box"][:nf]).astype(np.float64)).cuda()
    rng = np.random.default_rng(11)
    frames = [torch.as_tensor(pos0 + rng.normal(0, 0.05, pos0.shape)).cuda() for _ in range(5)]
    ops.construct_descriptors_light(synth.RC, 80, NA, N, tb, synth.RS, synth.RA, nf, dtype=torch.float64)
    ops.descriptor_options(dist2_fma=False, zero_padding=True)
    try:
        ops.descriptor_cell_threshold(0)
        want = [[x.clone() for x in ops.compute_descriptors_light(f, tb)] for f in frames]
        ops.descriptor_cell_threshold(1)
        tp = frames[0].clone()
        side = torch.cuda.Stream()                       # the library keeps its work areas, cells included, per stream
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            held = ops.compute_descriptors_light(tp, tb)     # sizes the work areas before the capture
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g, stream=side):
            held = ops.compute_descriptors_light(tp, tb, out=held)
        for rep, (f, w) in enumerate(zip(frames, want)):
            tp.copy_(f)
            torch.cuda.synchronize()
            g.replay()
            torch.cuda.synchronize()
            for x, y in zip(held, w):
                assert torch.equal(x, y), f"replay {rep}"
            with torch.cuda.stream(side):
                for _ in range(rep % 2 + 1):             # one or two eager calls: the next replay starts on either set
                    eager = ops.compute_descriptors_light(f, tb)
            torch.cuda.synchronize()
            for x, y in zip(eager, w):
                assert torch.equal(x, y)
    finally:
        ops.descriptor_cell_threshold(4096)


def test_hip_graph_replay_with_two_streams_matches_eager():
    """The whole op sequence captured once in a HIP graph, the two per-species chains forked onto their own streams
    (per-stream scratch inside the library): every replay, with eager calls and synchronisations in between, gives
    the eager result bit for bit."""
    import torch
    from alphanesgpu_amd import ops, synth
    import pipeline
    dev = torch.device("cuda:0")
    batch = synth.water_batch("water96")
    dt = batch["dtype"]
    tdt = torch.float64
    nr, na = synth.NR, synth.NA
    nf, N = batch["nf"], batch["N"]
    tipos = [int(x) for x in batch["tipos"]]
    nt = len(tipos)
    params = synth.fingerprint_params(dtype=dt)
    up = pipeline.synthetic_upstream(nf, batch["tipos"], params, 3, dt)
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box, tm, tp = T(batch["pos"]), T(batch["box"]), T(batch["type_map"]), T(batch["tipos"])
    P = [{k: T(v) for k, v in m.items()} for m in params]
    G2, G3 = [T(x) for x in up["G2"]], [T(x) for x in up["G3"]]
    Q = T(up["Q"])
    at = [torch.tensor([k], dtype=torch.int32, device=dev) for k in range(nt)]
    ops.construct_descriptors_light(synth.RC, nr, na, N, box, synth.RS, synth.RA, nf, dtype=tdt)
    ops.set_sync_errors(False)
    side = [torch.cuda.Stream() for _ in range(nt)]
    sl, o = [], 0
    for n in tipos:
        sl.append(slice(o, o + n))
        o += n

    def chain(k, d):
        rad, ang, sup, im2, im3, d2, d3, d3s, ntr = [x[:, sl[k]] for x in d]
        p = P[k]
        a3 = ops.compute_sort_proj3body(ang, sup, im3, im2, p["alpha3b"], p["emb3b"], tm, ntr, nt=nt)
        f2 = ops.compute_force_radial(G2[k], d2, im2, rad, p["alpha2b"], p["emb2b"], tm, tp, at[k])
        f3 = ops.compute_force_tripl(G3[k], sup, ang, d3s, d3, im2, im3, p["alpha3b"], p["emb3b"], tm, tp, at[k], ntr)
        ga = ops.compute_force_tripl_grad(Q, G3[k], sup, ang, d3s, d3, im2, im3, p["alpha3b"], p["emb3b"], tm, tp,
                                          at[k], ntr)
        return [a3, f2 + f3, ga[0], ga[1]]

    def step(streams):
        d = ops.compute_descriptors_light(pos, box)
        if streams is None:
            return [chain(k, d) for k in range(nt)]
        main = torch.cuda.current_stream()
        ready = main.record_event()
        outs, done = [], []
        for k in range(nt):
            with torch.cuda.stream(streams[k]):
                streams[k].wait_event(ready)
                r = chain(k, d)
                # eager steps tell the allocator that the step's stream reads these; under capture the graph's
                # private pool keeps them and the returned list holds the references: no allocator event is
                # queued inside the captured region
                if not torch.cuda.is_current_stream_capturing():
                    for t in r:
                        t.record_stream(main)
                outs.append(r)
                done.append(streams[k].record_event())
        for ev in done:
            main.wait_event(ev)
        return outs

    try:
        want = step(None)
        step(side)                      # grows the per-stream scratch before the capture
        ops.poll_status()
        torch.cuda.synchronize()
        g = torch.cuda.CUDAGraph()
        with torch.cuda.graph(g):
            held = step(side)
        for rep in range(3):
            g.replay()
            torch.cuda.synchronize()
            for a, b in zip(held, want):
                for x, y in zip(a, b):
                    assert torch.equal(x, y), f"replay {rep}"
            again = step(None)          # eager work between the replays, on the default stream
            ops.poll_status()
            torch.cuda.synchronize()
            for a, b in zip(again, want):
                for x, y in zip(a, b):
                    assert torch.equal(x, y)
    finally:
        ops.set_sync_errors(True)



@pytest.mark.gpu
def test_capture_with_synchronising_error_returns_left_on():
    """With the default error mode (every op waits for its stream to return a device-detected condition) an op that is
    being captured must not wait: the capture succeeds, the replay gives the eager result, and the condition is read
    with poll_status afterwards."""
    import torch
    from alphanesgpu_amd import ops, synth
    dev = torch.device("cuda:0")
    batch = synth.water_batch("water96")
    nr, na = synth.NR, synth.NA
    nf, N = batch["nf"], batch["N"]
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box, tm = T(batch["pos"]), T(batch["box"]), T(batch["type_map"])
    p = {k: T(v) for k, v in synth.fingerprint_params(dtype=batch["dtype"])[0].items()}
    ops.construct_descriptors_light(synth.RC, nr, na, N, box, synth.RS, synth.RA, nf, dtype=torch.float64)
    ops.set_sync_errors(True)

    def step(out=None):
        d = ops.compute_descriptors_light(pos, box, out=out)
        return d, ops.compute_sort_proj(d[0], d[3], p["alpha2b"], p["emb2b"], tm)

    d_want, af_want = step()
    s = torch.cuda.Stream()
    with torch.cuda.stream(s):
        d_held, _ = step()              # the stream's work areas exist before the capture
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=s):
        _, af_held = step(out=d_held)
    for rep in range(2):
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(af_held, af_want), f"replay {rep}"
        assert torch.equal(d_held[3], d_want[3])
    ops.poll_status()


@pytest.mark.gpu
def test_random_configurations(oracle):
    """Twelve seeded random configurations through every op: 1-3 species with 1-13 atoms each (parameter rows and
    classes of every shape), 1-3 frames, orthorhombic and triclinic boxes with the cluster shifted far outside the
    cell, random cutoffs Rs < Ra <= Rc, channel counts 1-6 per block, an angular buffer anywhere between the atom
    count and the full triangle (truncated triplet lists included), either precision, block or dense embeddings."""
    rng = np.random.default_rng(20240611)
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
        try:
            _generic_case(oracle, pos, box, tip, dtype, nr=nr, na=na, rc=rc, ra=ra, rs=rs, nt=nt, seed=case + 1,
                          dense=dense, maps=(ar, aa))
        except AssertionError as e:
            raise AssertionError(f"case {case}: nt={nt} tipos={tip} nf={nf} rc={rc:.2f} ra={ra:.2f} rs={rs:.2f} "
                                 f"nr={nr} na={na} ar={ar} aa={aa} {np.dtype(dtype).name} dense={dense}: {e}") from e


@pytest.mark.gpu
def test_random_dense_clusters(oracle):
    """Eleven seeded dense clusters through every op: 1-3 species with 8-33 atoms each inside a cutoff of 5-6.5, so
    that an atom has up to ~85 neighbours inside the angular cutoff -- several sweeps of the 3-body force kernel, more
    than 64 slots to group by species, up to 19 channels per species pair (more than one table chunk), angular
    buffers that cut the triplet list, either precision, block or dense embeddings."""
    rng = np.random.default_rng(7)
    seen_wide = seen_chunks = False
    for case in range(11):
        nt = int(rng.integers(1, 4))
        tip = [int(x) for x in rng.integers(8, 34, nt)]
        n = sum(tip)
        nf = int(rng.integers(1, 3))
        L = float(rng.uniform(14.0, 18.0))
        spread = float(rng.uniform(2.6, 3.6))
        pos, box = np.zeros((nf, 3 * n)), np.zeros((nf, 6))
        for b in range(nf):
            pts = []
            while len(pts) < n:
                c = rng.uniform(-spread, spread, 3)
                if all(np.linalg.norm(c - q) > 0.75 for q in pts):
                    pts.append(c)
            pos[b] = (np.array(pts) + rng.uniform(-5, 5, 3)).reshape(-1)
            box[b] = [L, 0.5, -0.3, L + 0.7, 0.4, L + 1.3]
        rc = float(rng.uniform(5.0, 6.5))
        ra = float(rng.uniform(0.8 * rc, rc))
        rs = float(rng.uniform(0.9, 2.0))
        nr = n + 2
        na = int(rng.integers(nr * (nr - 1) // 4, nr * (nr - 1) // 2 + 1))
        ar = tuple(int(x) for x in rng.integers(1, 7, nt))
        aa = tuple(int(x) for x in rng.integers(1, 20, nt * (nt + 1) // 2))
        dtype = np.float64 if rng.random() < 0.5 else np.float32
        dense = bool(rng.random() < 0.5)
        seen_wide |= nr > 64
        seen_chunks |= max(aa) > 16
        try:
            _generic_case(oracle, pos, box, tip, dtype, nr=nr, na=na, rc=rc, ra=ra, rs=rs, nt=nt, seed=case + 1,
                          dense=dense, maps=(ar, aa))
        except AssertionError as e:
            raise AssertionError(f"case {case}: nt={nt} tipos={tip} nf={nf} rc={rc:.2f} ra={ra:.2f} rs={rs:.2f} "
                                 f"nr={nr} na={na} ar={ar} aa={aa} {np.dtype(dtype).name} dense={dense}: {e}") from e
    assert seen_wide and seen_chunks   # the draws cover what the test is for


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_tiny_systems(oracle, dtype):
    """One atom (no neighbour at all), two atoms of one or two species, one water molecule, three atoms: every op,
    one and three frames, buffers larger and smaller than the neighbour counts."""
    cases = [([1], [[0.1, 0.2, 0.3]]),
             ([2], [[0, 0, 0], [1.1, 0.2, 0.1]]),
             ([1, 1], [[0, 0, 0], [1.0, 0.3, 0.2]]),
             ([1, 2], [[0, 0, 0], [0.96, 0, 0], [-0.24, 0.93, 0]]),
             ([3], [[0, 0, 0], [1.0, 0, 0], [0, 1.2, 0]])]
    for tip, pts in cases:
        n = sum(tip)
        for nf in (1, 3):
            pos = np.tile(np.array(pts, float).reshape(1, -1), (nf, 1)) + np.arange(nf)[:, None] * 0.01
            box = np.tile(np.array([[12.0, 0.3, -0.2, 12.5, 0.1, 13.0]]), (nf, 1))
            for nr, na in ((n + 2, 3), (4, 6)):
                _generic_case(oracle, pos, box, tip, dtype, nr=nr, na=na, rc=4.5, ra=4.5, rs=2.25, nt=len(tip),
                              seed=2)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_wide_channel_sets(oracle, dtype):
    """Three species with 141 three-body and 57 two-body channels: the parameter tables and gradient accumulators of
    the triplet kernels then take more than the 64 KB of LDS a launch gets without asking (the library requests up to
    the CU's 160 KB per kernel), and a class has up to 42 active channels (three table chunks)."""
    rng = np.random.default_rng(21)
    tip = [18, 15, 13]
    n = sum(tip)
    pts = []
    while len(pts) < n:
        c = rng.uniform(-3.2, 3.2, 3)
        if all(np.linalg.norm(c - q) > 0.75 for q in pts):
            pts.append(c)
    pos = (np.array(pts) + rng.uniform(-5, 5, 3)).reshape(1, -1)
    box = np.array([[16.0, 0.5, -0.3, 16.7, 0.4, 17.3]])
    _generic_case(oracle, pos, box, tip, dtype, nr=n + 2, na=938, rc=5.4, ra=4.9, rs=1.5, nt=3, seed=2,
                  maps=((11, 16, 30), (12, 5, 40, 4, 42, 38)))


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_add_n_is_the_sequential_sum(dtype):
    """ops.add_n (the callers' sum of per-op force arrays) against adding the arrays one after the other: same
    order, same bits, for 1 to 9 inputs, also in place."""
    import torch
    from alphanesgpu_amd import ops
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    g = torch.Generator(device="cpu").manual_seed(3)
    xs = [torch.randn(2, 3001, generator=g, dtype=tdt).cuda() for _ in range(9)]
    for n in range(1, 10):
        want = xs[0].clone()
        for x in xs[1:n]:
            want = want + x
        assert torch.equal(ops.add_n(xs[:n]), want), n
    acc = xs[0].clone()
    ops.add_n([acc, xs[1], xs[2]], out=acc)
    assert torch.equal(acc, (xs[0] + xs[1]) + xs[2])


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_species_without_atoms(oracle, dtype):
    """A three-species parameter set on frames that hold no atom of the middle species: its ops are called with an
    empty centre range, write nothing (fingerprints), zeros (forces, virial, parameter gradients), and the other
    species' results are those of the oracle."""
    import torch
    from alphanesgpu_amd import ops
    rng = np.random.default_rng(8)
    tip = [6, 0, 7]
    n = sum(tip)
    pts = []
    while len(pts) < n:
        c = rng.uniform(-3.0, 3.0, 3)
        if all(np.linalg.norm(c - q) > 0.9 for q in pts):
            pts.append(c)
    pos = np.array(pts).reshape(1, -1)
    box = np.array([[13.0, 0, 0, 14.0, 0, 15.0]])
    errs, ref = _generic_case(oracle, pos, box, tip, dtype, nr=16, na=60, rc=4.5, ra=3.5, rs=1.5, nt=3, dense=True,
                              maps=((3, 2, 4), (2, 3, 2, 2, 3, 2)))
    assert ref["af2"][1].shape[1] == 0 and not ref["f2"][1].any() and not ref["gf3"][1][1].any()


@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_default_options_write_the_reference_padding(oracle, dtype):
    """The descriptor op with the options construct leaves (no descriptor_options call), into buffers pre-filled
    with NaN / garbage: intmap2b, intmap3b, numtriplet and angdescr must equal the oracle's over the WHOLE arrays --
    the reference zeroes them before its kernels run (STAF/src/descriptor_builder/reforce.cc:357-358,375-376,
    385-386) and its own gate compares int3b over all padded elements (comparison_summary.txt:32-33).  The
    nr-wide outputs carry zeros in their padding; only der3b beyond the triplets stays as it was."""
    import torch
    from alphanesgpu_amd import ops
    dtype = np.dtype(dtype)
    tol = TOL[dtype]
    b = _synth("water768_f64", nf=2)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    nf, N = 2, b["N"]
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    dev = torch.device("cuda:0")
    d = oracle.compute_descriptors_light(pos, box, 4.5, 4.5, 2.25, NR, NA, dtype=dtype)
    ops.construct_descriptors_light(4.5, NR, NA, N, None, 2.25, 4.5, nf, dtype=tdt)   # resets the options
    nan = lambda *sh: torch.full(sh, float("nan"), dtype=tdt, device=dev)
    junk = lambda *sh: torch.full(sh, -123456789, dtype=torch.int32, device=dev)
    out = (nan(nf, N, NR), nan(nf, N, NA), nan(nf, N, NR), junk(nf, N, NR + 1), junk(nf, N, 2 * NA), nan(nf, N, 3, NR),
           nan(nf, N, 3, 2 * NA), nan(nf, N, 3, NR), junk(nf, N))
    ops.compute_descriptors_light(torch.as_tensor(pos).to(dev), torch.as_tensor(box).to(dev), out=out)
    names = ["raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp", "numtriplet"]
    g = {k: v.cpu().numpy() for k, v in zip(names, out)}
    for k in ("intmap2b", "intmap3b", "numtriplet"):
        assert np.array_equal(g[k], d[k]), k
    assert g["intmap3b"].size == nf * N * 2 * NA
    tm = triplet_mask(d["numtriplet"], NA)
    assert np.all(g["angdescr"][~tm] == 0) and not np.isnan(g["angdescr"]).any()
    assert max(nerr(g["angdescr"], d["angdescr"]), eerr(g["angdescr"], d["angdescr"], where=tm)) <= tol
    for k in ("raddescr", "des3bsupp", "der2b", "der3bsupp"):
        assert not np.isnan(g[k]).any(), k
    m3 = np.repeat(np.repeat(tm[:, :, None, :], 3, axis=2)[..., None], 2, axis=-1).reshape(nf, N, 3, 2 * NA)
    assert np.isnan(g["der3b"][~m3]).all() and not np.isnan(g["der3b"][m3]).any()
    assert nerr(np.where(m3, g["der3b"], 0), np.where(m3, d["der3b"], 0)) <= tol


def test_config2_full_size_fp32(oracle):
    """The headline configuration as benchmarked: 768 atoms, 4 frames, fp32, every op against the oracle."""
    print(_run_case(oracle, _synth("water768_f32"), np.float32))


def test_config3_full_size_fp64(oracle):
    """The double-precision training configuration: 768 atoms, 4 frames, fp64, full training step (all eight ops)."""
    print(_run_case(oracle, _synth("water768_f64"), np.float64))


def test_config4_train8_fp32(oracle):
    """The eight-frame training configuration: eight 768-atom frames, fp32, all eight ops of a training step."""
    print(_run_case(oracle, _synth("water768_train8"), np.float32))


def test_config5_water6144_fp64(oracle):
    """The large-box configuration: 6144 atoms, one frame, fp64; above the library's default threshold, so the neighbours are
    found through the cell list (8 x 8 x 8 cells) while the oracle tests all pairs."""
    from alphanesgpu_amd import ops
    ops.descriptor_cell_threshold(4096)
    b = _synth("water6144")
    assert b["N"] == 6144 and b["N"] >= 4096
    print(_run_case(oracle, b, np.float64))


def test_stale_neighbour_map_is_reported():
    """A force op handed a view of a descriptor output that was overwritten afterwards: the transposed map the
    library kept for that tensor no longer matches it, and the op says so instead of returning wrong forces."""
    import torch
    from alphanesgpu_amd import ops, _lib
    b = _synth("water96")
    dev = torch.device("cuda:0")
    dtype = np.dtype(np.float64)
    params = _params(dtype)
    N = b["N"]
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    ops.construct_descriptors_light(4.5, NR, NA, N, None, 2.25, 4.5, 1, dtype=torch.float64)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = ops.compute_descriptors_light(T(b["pos"]), T(b["box"]))
    tm, tp = T(b["type_map"]), T(b["tipos"])
    at = torch.tensor([0], dtype=torch.int32, device=dev)
    n0 = int(b["tipos"][0])
    G2 = torch.ones(1, n0, params[0]["alpha2b"].shape[1], dtype=torch.float64, device=dev)
    args = lambda: (G2, d2[:, :n0], im2[:, :n0], rad[:, :n0], T(params[0]["alpha2b"]), T(params[0]["emb2b"]), tm, tp, at)
    ops.compute_force_radial(*args())          # fine
    im2[0, 0, 1] = (int(im2[0, 0, 1]) + 1) % N  # slot 0 of atom 0 now names another atom
    with pytest.raises(_lib.StafError) as e:
        ops.compute_force_radial(*args())
    assert e.value.code == -14
    # once a remembered map has failed its check the library forgets what it remembered: the same view is now
    # transposed by the op itself, like the private copy below, and gives that copy's forces
    f_view = ops.compute_force_radial(*args())
    f_copy = ops.compute_force_radial(G2, d2[:, :n0].clone(), im2[:, :n0].clone(), rad[:, :n0].clone(),
                                      T(params[0]["alpha2b"]), T(params[0]["emb2b"]), tm, tp, at)
    assert torch.equal(f_view, f_copy)
    # a private copy of the modified map is transposed by the op itself: no complaint
    # (clone: a leading slice of a one-frame tensor already is contiguous, .contiguous() would hand back the view)
    ops.compute_force_radial(G2, d2[:, :n0].clone(), im2[:, :n0].clone(), rad[:, :n0].clone(),
                             T(params[0]["alpha2b"]), T(params[0]["emb2b"]), tm, tp, at)


@pytest.mark.parametrize("dtype,case", [(np.float64, "water96"), (np.float64, "water768"), (np.float32, "water768"),
                                        (np.float64, "dense"), (np.float64, "virial")])
def test_fused_tripl_grads(oracle, dtype, case):
    """staf_op_grads_tripl_fused: the gradient of the 3-body force op and the gradient of the 3-body fingerprint op
    in one launch, against the oracle's two ops (fp64: 1e-12) and against the library's two separate ops (fp32: the
    separate ops are held to the oracle by the other tests; the fused sums differ from theirs by rounding only)."""
    import torch
    from alphanesgpu_amd import ops
    from util import species_slices
    dtype = np.dtype(dtype)
    b = _synth("water96") if case == "water96" else _synth("water768_f64", nf=2)
    params = _params(dtype, dense=case == "dense")
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    nf = box.shape[0]
    up = pipeline.synthetic_upstream(nf, b["tipos"], params, 17, dtype)
    Wg = np.random.Generator(np.random.Philox(8)).standard_normal((nf, 9)).astype(dtype) if case == "virial" else None
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    ops.construct_descriptors_light(4.5, NR, NA, b["N"], None, 2.25, 4.5, nf, dtype=tdt)
    ops.descriptor_options(False, False)
    names = ["raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp", "numtriplet"]
    g = dict(zip(names, ops.compute_descriptors_light(T(pos), T(box))))
    d = oracle.compute_descriptors_light(pos, box, 4.5, 4.5, 2.25, NR, NA, dtype=dtype) if dtype == np.float64 else None
    tm, tp, Q = T(b["type_map"]), T(b["tipos"]), T(up["Q"])
    vir = {} if Wg is None else dict(prevgrad_virial=T(Wg), pos=T(pos), box=T(box))
    tol = TOL[dtype]
    for k, s in enumerate(species_slices(b["tipos"])):
        m = params[k]
        v = lambda key: g[key][:, s]
        al, em = T(m["alpha3b"]), T(m["emb3b"])
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        G3, P3 = T(up["G3"][k]), T(up["P3"][k])
        common = (v("des3bsupp"), v("angdescr"), v("der3bsupp"), v("der3b"), v("intmap2b"), v("intmap3b"), al, em, tm,
                  tp, at, v("numtriplet"))
        gn, gaf, gae, ge = ops.compute_tripl_grads_fused(Q, G3, P3, *common, **vir)
        sn, saf, _ = ops.compute_force_tripl_grad(Q, G3, *common, **vir)
        sae, _ = ops.compute_sort_proj3body_grad(P3, v("angdescr"), v("des3bsupp"), v("intmap3b"), v("intmap2b"), al,
                                                 em, tm, v("numtriplet"), nt=len(b["tipos"]))
        torch.cuda.synchronize()
        assert torch.all(ge == 0)
        n = lambda t: t.cpu().numpy()
        pair_tol = 1e-13 if dtype == np.float64 else 3e-6
        for name, x, y in (("net", gn, sn), ("alpha_force", gaf, saf), ("alpha_energy", gae, sae)):
            assert nerr(n(x), n(y)) <= pair_tol, (name, k, nerr(n(x), n(y)))
            assert eerr(n(x), n(y)) <= 10 * pair_tol, (name, k, eerr(n(x), n(y)))
        if d is not None:
            c = lambda a: np.ascontiguousarray(a[:, s])
            a3 = (c(d["des3bsupp"]), c(d["angdescr"]), c(d["der3bsupp"]), c(d["der3b"]), c(d["intmap2b"]),
                  c(d["intmap3b"]), m["alpha3b"], m["emb3b"], b["type_map"], b["tipos"], k, c(d["numtriplet"]))
            okw = {} if Wg is None else dict(prevgrad_virial=Wg, pos=pos, box=box)
            on, oaf, _ = oracle.force_tripl_grad(up["Q"], up["G3"][k], *a3, **okw)
            oae, _ = oracle.sort_proj3body_grad(up["P3"][k], c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]),
                                                c(d["intmap2b"]), m["alpha3b"], m["emb3b"], b["type_map"],
                                                c(d["numtriplet"]))
            for name, x, y in (("net", gn, on), ("alpha_force", gaf, oaf), ("alpha_energy", gae, oae)):
                assert max(nerr(n(x), y), eerr(n(x), y)) <= tol, (name, k, nerr(n(x), y), eerr(n(x), y))


@pytest.mark.parametrize("dtype,case", [(np.float64, "water96"), (np.float32, "water768"), (np.float64, "three")])
def test_force_total_has_the_bits_of_the_per_op_forces_added(dtype, case):
    """staf_op_force_tripl_slots + staf_op_force_total: the total force in one launch equals, bit for bit, the sum
    (staf_op_add_n order: 2-body of species 0, 3-body of species 0, 2-body of species 1, ...) of the per-op force
    arrays, which the other tests hold to the oracle.  Also with terms left out, and for a species without atoms."""
    import torch
    from alphanesgpu_amd import ops, synth
    from util import species_slices
    dtype = np.dtype(dtype)
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    if case == "three":
        # three species, the last one without atoms: its terms are skipped
        b = _synth("water96")
        tipos = np.array([32, 64, 0], np.int32)
        type_map = b["type_map"]
        params = synth.fingerprint_params(dtype=dtype, nt=3, dense_embedding=True, ar_map=(5, 4, 6),
                                          aa_map=(4, 3, 5, 3, 4, 3))
    else:
        b = _synth("water96") if case == "water96" else _synth("water768_f32", nf=2)
        tipos, type_map = b["tipos"], b["type_map"]
        params = _params(dtype)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    nf, N, nt = box.shape[0], b["N"], len(tipos)
    up = pipeline.synthetic_upstream(nf, tipos, params, 31, dtype)
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    ops.construct_descriptors_light(4.5, NR, NA, N, None, 2.25, 4.5, nf, dtype=tdt)
    ops.descriptor_options(False, False)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = ops.compute_descriptors_light(T(pos), T(box))
    tm, tp = T(type_map), T(tipos)
    f2, f3, slots, own = [], [], [], []
    for k, s in enumerate(species_slices(tipos)):
        p = {kk: T(vv) for kk, vv in params[k].items()}
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        G2, G3 = T(up["G2"][k]), T(up["G3"][k])
        f2.append(ops.compute_force_radial(G2, d2[:, s], im2[:, s], rad[:, s], p["alpha2b"], p["emb2b"], tm, tp, at))
        a3 = (G3, sup[:, s], ang[:, s], d3s[:, s], d3[:, s], im2[:, s], im3[:, s], p["alpha3b"], p["emb3b"], tm, tp, at,
              ntr[:, s])
        f3.append(ops.compute_force_tripl(*a3))
        if int(tipos[k]) > 0:
            sl, ow = ops.compute_force_tripl_slots(*a3)
        else:
            sl, ow = None, None
        slots.append(sl)
        own.append(ow)
    n_local = [int(n) for n in tipos]
    want = ops.add_n([x for k in range(nt) for x in (f2[k], f3[k])])
    got = ops.force_total(im2, n_local, slots, own, f2)
    torch.cuda.synchronize()
    assert torch.equal(got, want)
    # 2-body pair forces folded into the slot forces by the same launch: the total without any per-op force array,
    # equal to the sum of the per-op arrays to rounding
    slots23, own23 = [], []
    for k, s in enumerate(species_slices(tipos)):
        if int(tipos[k]) == 0:
            slots23.append(None)
            own23.append(None)
            continue
        p = {kk: T(vv) for kk, vv in params[k].items()}
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        sl, ow = ops.compute_forces_slots(T(up["G3"][k]), T(up["G2"][k]), sup[:, s], ang[:, s], d3s[:, s], d3[:, s],
                                          rad[:, s], d2[:, s], im2[:, s], im3[:, s], p["alpha3b"], p["emb3b"],
                                          p["alpha2b"], p["emb2b"], tm, tp, at, ntr[:, s])
        slots23.append(sl)
        own23.append(ow)
    got23 = ops.force_total(im2, n_local, slots23, own23).cpu().numpy()
    tol = TOL[dtype]
    assert max(nerr(got23, want.cpu().numpy()), eerr(got23, want.cpu().numpy())) <= tol
    # 3-body terms alone, and with the first species' terms left out
    assert torch.equal(ops.force_total(im2, n_local, slots, own), ops.add_n(f3))
    some2 = [None] + f2[1:]
    some3 = [None] + slots[1:]
    want2 = ops.add_n([x for k in range(1, nt) for x in (f2[k], f3[k])])
    assert torch.equal(ops.force_total(im2, n_local, some3, [None] + own[1:], some2), want2)
    # a private copy of the map is not one the library remembers: refused, not guessed at
    from alphanesgpu_amd import _lib
    with pytest.raises(_lib.StafError) as e:
        ops.force_total(im2.clone(), n_local, slots, own, f2)
    assert e.value.code == -2


def test_scatter_overflow_is_reported():
    """A neighbour map of unknown origin in which one atom is listed by more centres than the force op's transposed
    map holds keys for (4 x nr): the op returns STAF_E_SCATTER_OVERFLOW (detected on the device, returned by the
    host after the op's synchronisation; every kernel runs to its end) and the next valid call is not affected."""
    import torch
    from alphanesgpu_amd import ops, _lib
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(5)
    nf, Nl, N, nr, nt, Ar = 1, 40, 64, 8, 2, 6
    assert Nl > 4 * nr
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    im = np.zeros((nf, Nl, nr + 1), np.int32)
    im[..., 0] = 2
    im[..., 1] = 63                                    # every centre names atom 63 in its first slot
    im[..., 2] = np.arange(Nl)[None, :] % 20 + 40      # and one of atoms 40..59 in its second
    D = T(rng.uniform(0.1, 1.0, (nf, Nl, nr)))
    dD = T(rng.standard_normal((nf, Nl, 3, nr)))
    G = T(rng.standard_normal((nf, Nl, Ar)))
    al, em = T(rng.uniform(0.5, 2.0, (nt, Ar))), T(rng.uniform(0.2, 1.0, (nt, Ar)))
    tm = T((np.arange(N) >= Nl).astype(np.int32))
    tp = T(np.array([Nl, N - Nl], np.int32))
    at = torch.tensor([0], dtype=torch.int32, device=dev)
    with pytest.raises(_lib.StafError) as e:
        ops.compute_force_radial(G, dD, T(im), D, al, em, tm, tp, at)
    assert e.value.code == -11
    ops.poll_status()                                  # reported once, then cleared: a second read finds nothing
    im[:, 4 * nr:, 1] = 62                             # 32 centres name atom 63: exactly what the map holds
    f = ops.compute_force_radial(G, dD, T(im), D, al, em, tm, tp, at)
    assert torch.isfinite(f).all()


def test_release_frees_the_work_areas_and_the_next_calls_rebuild_them():
    """staf_ops_release between two runs of every op: same bits before and after.  A force op handed descriptor
    outputs from before the release no longer finds them among the maps the library remembers and transposes the
    map itself: same forces to rounding (its sums run in another order)."""
    import torch
    from alphanesgpu_amd import ops
    b = _synth("water96")
    dtype = np.dtype(np.float64)
    params = _params(dtype)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    up = pipeline.synthetic_upstream(1, b["tipos"], params, 3, dtype)
    r1 = pipeline.run_hip(pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype)
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = ops.compute_descriptors_light(T(pos), T(box))
    n0 = int(b["tipos"][0])
    tm, tp = T(b["type_map"]), T(b["tipos"])
    at = torch.tensor([0], dtype=torch.int32, device=dev)
    args = (T(up["G2"][0]), d2[:, :n0], im2[:, :n0], rad[:, :n0], T(params[0]["alpha2b"]), T(params[0]["emb2b"]),
            tm, tp, at)
    before = ops.compute_force_radial(*args).cpu().numpy()
    ops.release()
    after = ops.compute_force_radial(*args).cpu().numpy()
    assert nerr(after, before) <= 1e-13
    r2 = pipeline.run_hip(pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype)
    for key in ("af2", "af3", "f2", "f3"):
        for x, y in zip(r1[key], r2[key]):
            assert np.array_equal(x, y), key
    for key in ("g2", "g3", "gf2", "gf3"):
        for x, y in zip(r1[key], r2[key]):
            for u, v in zip(x, y):
                assert np.array_equal(u, v), key


def test_three_host_threads_on_their_own_streams(monkeypatch):
    """The library's state is per device and per stream behind one lock: three host threads, each on a stream of its
    own, run the whole op sequence at the same time (a framework's executor calls ops from several threads), and
    every result has the bits of the single-threaded run."""
    import threading
    import torch
    from alphanesgpu_amd import ops
    b = _synth("water96")
    dtype = np.dtype(np.float64)
    params = _params(dtype)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    up = pipeline.synthetic_upstream(1, b["tipos"], params, 3, dtype)
    want = pipeline.run_hip(pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype)
    # the geometry and the options stay as the call above set them: threads only compute
    monkeypatch.setattr(ops, "construct_descriptors_light", lambda *a, **k: None)
    monkeypatch.setattr(ops, "descriptor_options", lambda *a, **k: None)
    bad = []

    def same(x, y):
        if isinstance(x, tuple):
            return all(same(u, v) for u, v in zip(x, y))
        return np.array_equal(x, y)

    def worker(t):
        try:
            with torch.cuda.stream(torch.cuda.Stream()):
                for it in range(3):
                    got = pipeline.run_hip(pos, box, b["tipos"], b["type_map"], params, up, NR, NA, dtype)
                    for key in ("af2", "af3", "f2", "f3", "g2", "g3", "gf2", "gf3"):
                        for x, y in zip(got[key], want[key]):
                            if not same(x, y):
                                bad.append((t, it, key))
                    for k in ("intmap2b", "intmap3b", "numtriplet", "raddescr", "angdescr", "der2b"):
                        if not np.array_equal(got["desc"][k], want["desc"][k]):
                            bad.append((t, it, k))
        except Exception as e:   # a thread's exception would otherwise be lost
            bad.append((t, repr(e)))

    threads = [threading.Thread(target=worker, args=(t,)) for t in range(3)]
    for th in threads:
        th.start()
    for th in threads:
        th.join()
    assert not bad, bad[:10]


def test_growth_under_capture_is_refused():
    """An op that meets a shape it has no work area for while its stream is being captured returns STAF_E_CAPTURE
    and launches nothing; after one eager call of the same shape the capture goes through and replays correctly."""
    import torch
    from alphanesgpu_amd import ops, _lib
    dev = torch.device("cuda:0")
    dtype = np.dtype(np.float64)
    params = _params(dtype)
    rng = np.random.default_rng(1)
    nf, Nl, nr, Ar, N = 3, 700, 60, params[0]["alpha2b"].shape[1], 1400
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    D = T(rng.uniform(0.1, 1.0, (nf, Nl, nr)))
    im = np.zeros((nf, Nl, nr + 1), np.int32)
    im[..., 0] = 20
    im[..., 1:21] = rng.integers(0, N, (nf, Nl, 20))
    im2, P2 = T(im), T(rng.standard_normal((nf, Nl, Ar)))
    tm = T(rng.integers(0, 2, N).astype(np.int32))
    al, em = T(params[0]["alpha2b"]), T(params[0]["emb2b"])
    cap = torch.cuda.Stream()          # a stream the library has never seen: no work area yet
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=cap):
        keep = D + 1.0                 # the refused call adds no node: the graph holds this one
        with pytest.raises(_lib.StafError) as e:
            ops.compute_two_body_par_grad(P2, D, im2, al, em, tm)
        assert e.value.code == -13
    with torch.cuda.stream(cap):
        want = ops.compute_two_body_par_grad(P2, D, im2, al, em, tm)
    torch.cuda.synchronize()
    g2 = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g2, stream=cap):
        held = ops.compute_two_body_par_grad(P2, D, im2, al, em, tm)
    for _ in range(2):
        g2.replay()
        torch.cuda.synchronize()
        for x, y in zip(held, want):
            assert torch.equal(x, y)


@pytest.mark.gpu
@pytest.mark.parametrize("dtype", [np.float64, np.float32])
def test_triplet_counts_out_of_range_are_clamped(dtype):
    """A caller's numtriplet tensor with entries below zero or above the radial buffer: the 3-body ops clamp them to
    0 .. nr (a negative count means no triplet, a count above nr the whole row), so the outputs are those of the
    clamped tensor, bit for bit, and no kernel reads outside its rows."""
    import torch
    from alphanesgpu_amd import ops
    from util import species_slices
    dtype = np.dtype(dtype)
    b = _synth("water96")
    params = _params(dtype)
    pos, box = b["pos"].astype(dtype), b["box"].astype(dtype)
    nf = box.shape[0]
    up = pipeline.synthetic_upstream(nf, b["tipos"], params, 23, dtype)
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    ops.construct_descriptors_light(4.5, NR, NA, b["N"], None, 2.25, 4.5, nf, dtype=tdt)
    ops.descriptor_options(False, True)   # every padded slot zero: a count above the row's own is well defined
    names = ["raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp", "numtriplet"]
    g = dict(zip(names, ops.compute_descriptors_light(T(pos), T(box))))
    tm, tp, Q = T(b["type_map"]), T(b["tipos"]), T(up["Q"])
    bad = g["numtriplet"].clone()
    bad[:, 0::3] = -7
    bad[:, 1::3] = NR + 1000
    good = bad.clamp(0, NR)
    for k, s in enumerate(species_slices(b["tipos"])):
        m = params[k]
        v = lambda key: g[key][:, s]
        al, em = T(m["alpha3b"]), T(m["emb3b"])
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        G3, P3 = T(up["G3"][k]), T(up["P3"][k])

        def run(ntr):
            common = (v("des3bsupp"), v("angdescr"), v("der3bsupp"), v("der3b"), v("intmap2b"), v("intmap3b"), al,
                      em, tm, tp, at, ntr[:, s])
            out = [ops.compute_sort_proj3body(v("angdescr"), v("des3bsupp"), v("intmap3b"), v("intmap2b"), al, em, tm,
                                              ntr[:, s], nt=len(b["tipos"])),
                   ops.compute_force_tripl(G3, *common)]
            out += list(ops.compute_tripl_grads_fused(Q, G3, P3, *common))
            torch.cuda.synchronize()
            return [o.clone() for o in out]

        for x, y in zip(run(bad), run(good)):
            assert torch.isfinite(x).all()
            assert torch.equal(x, y), k
    ops.descriptor_options(False, False)
    ops.poll_status()


@pytest.mark.gpu
def test_changed_row_of_a_remembered_map_is_reported_by_its_checksum():
    """A remembered (symmetric) map whose content changes in a way the reciprocity check cannot see: two slots of a
    row of an atom OUTSIDE the op's species swapped (every listed pair is still listed both ways, only the slot
    order no longer matches the descriptor rows).  The atom that collects through that row recomputes the row's
    checksum, which differs from the one the descriptor op stored: stale map, for the per-op force kernels and for
    the collecting launch of the step-level path."""
    import torch
    from alphanesgpu_amd import ops, _lib
    b = _synth("water96")
    dev = torch.device("cuda:0")
    dtype = np.dtype(np.float64)
    params = _params(dtype)
    N = b["N"]
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    tm, tp = T(b["type_map"]), T(b["tipos"])
    at = torch.tensor([0], dtype=torch.int32, device=dev)
    n0 = int(b["tipos"][0])
    p0 = params[0]
    G2 = torch.ones(1, n0, p0["alpha2b"].shape[1], dtype=torch.float64, device=dev)
    G3 = torch.ones(1, n0, p0["alpha3b"].shape[1] // 3, dtype=torch.float64, device=dev)

    def fresh():
        ops.construct_descriptors_light(4.5, NR, NA, N, None, 2.25, 4.5, 1, dtype=torch.float64)
        out = ops.compute_descriptors_light(T(b["pos"]), T(b["box"]))
        im2 = out[3]
        victim = N - 1                      # an atom of the other species
        assert int(im2[0, victim, 0]) >= 2
        a, c = int(im2[0, victim, 1]), int(im2[0, victim, 2])
        im2[0, victim, 1], im2[0, victim, 2] = c, a
        return out

    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = fresh()
    with pytest.raises(_lib.StafError) as e:
        ops.compute_force_radial(G2, d2[:, :n0], im2[:, :n0], rad[:, :n0], T(p0["alpha2b"]), T(p0["emb2b"]), tm, tp, at)
    assert e.value.code == -14
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = fresh()
    with pytest.raises(_lib.StafError) as e:
        ops.compute_force_tripl(G3, sup[:, :n0], ang[:, :n0], d3s[:, :n0], d3[:, :n0], im2[:, :n0], im3[:, :n0],
                                T(p0["alpha3b"]), T(p0["emb3b"]), tm, tp, at, ntr[:, :n0])
    assert e.value.code == -14
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = fresh()
    slots, selfs = ops.compute_force_tripl_slots(G3, sup[:, :n0], ang[:, :n0], d3s[:, :n0], d3[:, :n0], im2[:, :n0],
                                                 im3[:, :n0], T(p0["alpha3b"]), T(p0["emb3b"]), tm, tp, at,
                                                 ntr[:, :n0])
    with pytest.raises(_lib.StafError) as e:
        ops.force_total(im2, [int(x) for x in b["tipos"]], [slots, None], [selfs, None])
    assert e.value.code == -14
    # an untouched map of a new descriptor call is remembered afresh and collects without complaint
    ops.construct_descriptors_light(4.5, NR, NA, N, None, 2.25, 4.5, 1, dtype=torch.float64)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = ops.compute_descriptors_light(T(b["pos"]), T(b["box"]))
    ops.compute_force_radial(G2, d2[:, :n0], im2[:, :n0], rad[:, :n0], T(p0["alpha2b"]), T(p0["emb2b"]), tm, tp, at)
    ops.poll_status()
