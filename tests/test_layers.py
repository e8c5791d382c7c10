"""PyTorch layer shells (alphanesgpu_amd/layers.py) with the reference's gradient routing.

A small two-species model is assembled from the layers the way the reference's training step assembles its TF
modules (STAF/staf_models/staf_model.py:168-208: descriptor tensors split per species -> physics layer, lognorm,
Dense stack -> dE/dAF by differentiation of the network -> force layer), a loss
L = sum_b cE_b E_b + sum Q.F (+ sum Qw.W) is back-propagated with torch.autograd, and every kind of trainable parameter is checked against central finite
differences of the same loss evaluated through the CPU oracle pipeline.  That pins the routing (which gradient op
feeds which input, the second-order path through the network, the squared embeddings), not the ops themselves,
which have their own parity tests."""
import numpy as np
import pytest


def _two_frames():
    from test_oracle_pins import cluster
    a = cluster([4, 5], seed=21)
    b = cluster([4, 5], seed=22)
    return np.concatenate([a[0], b[0]]), np.concatenate([a[1], b[1]]), a[2], a[3]


def _oracle_loss(oracle, frames, model, cE, Q, Qw, nr, na, rc, ra, rs):
    from test_oracle_pins import energy_and_forces
    pos, box, tipos, type_map = frames
    E, F, W, _, _ = energy_and_forces(oracle, pos, box, tipos, type_map, model, nr=nr, na=na, rc=rc, ra=ra, rs=rs,
                                      virial=Qw is not None)
    L = float(np.dot(cE, E) + np.sum(Q * F))
    if Qw is not None:
        L += float(np.sum(Qw * W))
    return L


@pytest.mark.gpu
@pytest.mark.parametrize("virial", [False, True])
def test_autograd_through_the_layers_matches_finite_differences_of_the_oracle(oracle, virial):
    import torch
    from alphanesgpu_amd import layers
    from test_oracle_pins import small_model
    dev = torch.device("cuda:0")
    nr, na, rc, ra, rs = 16, 45, 4.5, 3.4, 1.6
    frames = _two_frames()
    pos, box, tipos, type_map = frames
    nf, nt = pos.shape[0], len(tipos)
    model = small_model(nt, (3, 2), (2, 2, 3), seed=13, hidden=5, dense=True)
    rng = np.random.default_rng(4)
    cE = rng.standard_normal(nf)
    Q = rng.standard_normal((nf, pos.shape[1]))
    Qw = rng.standard_normal((nf, 9)) if virial else None

    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    tpos, tbox, ttm, ttp = T(pos), T(box), T(type_map), T(tipos)
    desc = layers.descriptor_layer(rc, nr, ra, na, pos.shape[1] // 3, tbox, rs, nf)
    rad, ang, sup, im2, im3, d2, d3, d3s, ntr = desc(tpos, tbox)
    flayer = layers.force_virial_layer(nr, na) if virial else layers.force_layer(nr, na)
    phys, logn, dense = [], [], []
    for m in model:
        phys.append(layers.physics_layer(T(m["alpha2b"]), T(m["alpha3b"]),
                                         [T(np.sqrt(m["emb2b"])), T(np.sqrt(m["emb3b"]))]))
        logn.append(layers.lognorm_layer(T(m["mu"])))
        dense.append([(torch.nn.Parameter(T(W)), torch.nn.Parameter(T(b)), act) for W, b, act in m["layers"]])

    E = torch.zeros(nf, dtype=torch.float64, device=dev)
    F = torch.zeros((nf, pos.shape[1]), dtype=torch.float64, device=dev)
    Wv = torch.zeros((nf, 9), dtype=torch.float64, device=dev)
    o = 0
    for k, n in enumerate(tipos):
        s = slice(o, o + int(n))
        o += int(n)
        c = lambda a: a[:, s]
        af = phys[k](c(rad), c(sup), c(im2), c(ang), c(im3), c(ntr), ttm)
        x = logn[k](af)
        for W, b, act in dense[k]:
            x = x @ W + b
            if act == "tanh":
                x = torch.tanh(x)
        e_atoms = x[..., 0]
        E = E + 0.5 * e_atoms.sum(dim=1)
        net_der, = torch.autograd.grad(e_atoms.sum(), af, create_graph=True)
        Ar = phys[k].nalpha_r
        args = (net_der[..., :Ar].contiguous(), c(rad), c(d2), c(im2), phys[k].alpha2b,
                net_der[..., Ar:].contiguous(), c(ang), c(sup), c(d3), c(d3s), c(im3), c(ntr), phys[k].alpha3b,
                phys[k].type_emb_2b, phys[k].type_emb_3b, ttm, ttp, k)
        if virial:
            f, w = flayer(*args, tpos, tbox)
            Wv = Wv + w
        else:
            f = flayer(*args)
        F = F + f
    L = (T(cE) * E).sum() + (T(Q) * F).sum()
    if virial:
        L = L + (T(Qw) * Wv).sum()
    L.backward()

    L0 = _oracle_loss(oracle, frames, model, cE, Q, Qw, nr, na, rc, ra, rs)
    assert abs(L.item() - L0) <= 1e-10 * max(1.0, abs(L0))

    def fd(k, key, idx, layer=None, h=1e-5):
        """central difference of the oracle loss in one entry of one parameter array"""
        vals = []
        for sgn in (+1, -1):
            mm = [dict(m, layers=[(W.copy(), b.copy(), a) for W, b, a in m["layers"]]) for m in model]
            if layer is None:
                arr = mm[k][key].copy()
                if key in ("emb2b", "emb3b"):        # the trainable quantity is the unsquared embedding
                    r = np.sqrt(arr)
                    r[idx] += sgn * h
                    arr = r * r
                else:
                    arr[idx] += sgn * h
                mm[k][key] = arr
            else:
                mm[k]["layers"][layer][key][idx] += sgn * h
            vals.append(_oracle_loss(oracle, frames, mm, cE, Q, Qw, nr, na, rc, ra, rs))
        return (vals[0] - vals[1]) / (2 * h)

    g = lambda p: p.grad.detach().cpu().numpy()
    checks = []
    for k in range(nt):
        Aa = phys[k].nalpha_a
        checks += [(g(phys[k].alpha2b)[1, 0], fd(k, "alpha2b", (1, 0))),
                   (g(phys[k].alpha2b)[0, 1], fd(k, "alpha2b", (0, 1))),
                   (g(phys[k].alpha3b)[0, 1], fd(k, "alpha3b", (0, 1))),               # alpha1
                   (g(phys[k].alpha3b)[1, Aa], fd(k, "alpha3b", (1, Aa))),             # alpha2
                   (g(phys[k].alpha3b)[2, 2 * Aa + 1], fd(k, "alpha3b", (2, 2 * Aa + 1))),   # beta
                   (g(phys[k].type_emb_2b)[1, 1], fd(k, "emb2b", (1, 1))),
                   (g(logn[k].mu)[2], fd(k, "mu", (2,))),
                   (g(dense[k][0][0])[1, 2], fd(k, 0, (1, 2), layer=0)),
                   (g(dense[k][1][1])[3], fd(k, 1, (3,), layer=1))]
        # the reference's gradient ops return zeros for the 3-body embedding (its kernels never fill that output):
        # the routing hands exactly that on
        assert not g(phys[k].type_emb_3b).any()
    got = np.array([a for a, _ in checks])
    want = np.array([b for _, b in checks])
    scale = np.abs(want).max()
    # finite differences with h = 1e-5 on a smooth function of O(1) curvature: ~1e-9 absolute
    assert np.all(np.abs(got - want) <= 2e-7 * scale), (got, want)
    assert np.count_nonzero(np.abs(want) > 1e-6 * scale) >= len(want) - 4


def test_layer_classes_have_the_reference_signatures():
    """Names and argument lists of STAF/source_routine/*.py (descriptor_builder.py:16,31, physics_layer_mod.py:10,33,
    55,59, force_layer_mod.py:9,25-27,78,90-92)."""
    import inspect
    from alphanesgpu_amd import layers
    sig = lambda f: [p for p in inspect.signature(f).parameters if p != "self"]
    assert sig(layers.descriptor_layer.__init__)[:8] == ["rc", "rad_buff", "rc_ang", "ang_buff", "N", "box_example",
                                                         "Rs", "maxbatch"]
    assert sig(layers.descriptor_layer.forward) == ["pos", "box"]
    assert sig(layers.physics_layer.__init__) == ["init_alpha2b", "init_alpha3b", "initial_type_emb"]
    assert sig(layers.physics_layer.forward) == ["x2b", "x3bsupp", "intmap2b", "x3b", "intmap3b", "numtriplet",
                                                 "type_map"]
    assert sig(layers.lognorm_layer.__init__) == ["mu"] and sig(layers.lognorm_layer.forward) == ["restot"]
    call = ["net_der_r", "x2b", "intder2b", "int2b", "alpha2b", "net_der_a", "x3b", "x3bsupp", "intder3b",
            "intder3bsupp", "int3b", "numtriplet", "alpha3b", "type_emb_2b", "type_emb_3b", "type_map", "tipos",
            "type_now"]
    assert sig(layers.force_layer.__init__) == ["radbuff", "angbuff"] and sig(layers.force_layer.forward) == call
    assert sig(layers.force_virial_layer.__init__) == ["radbuff", "angbuff", "with_grad"]
    assert sig(layers.force_virial_layer.forward) == call + ["pos", "box"]
