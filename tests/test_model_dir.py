"""Model-directory files (alphanesgpu_amd/model_dir.py): the writer against the files the reference exported
(tests/golden/model_float, model_double: copies of test/test-lammps-smoke/model_onnx_*), the reader against the
test suite's own loader, and a written three-species model through staf_load / staf_compute against the oracle."""
import os

import numpy as np
import pytest

from util import GOLDEN, load_model, nerr

DAT = ("alpha_2body", "alpha_3body", "alpha_mu", "type_emb_2b_sq", "type_emb_3b_sq", "type_emb_2b", "type_emb_3b")


@pytest.mark.parametrize("prec", ["float", "double"])
def test_writer_reproduces_the_exported_model_files(tmp_path, prec):
    """Binary MLP files byte for byte, text files value for value, from the parameters as the tests load them."""
    from alphanesgpu_amd import model_dir
    tipos, model = load_model(prec)
    gold = os.path.join(GOLDEN, f"model_{prec}")
    species = [dict(m, mu=m["mu_dat"]) for m in model]
    for m, sp in zip(model, species):
        assert np.array_equal(m["mu"], m["mu_dat"].astype(m["mu"].dtype))
    model_dir.write_model_dir(str(tmp_path), species, tipos=tipos, precision=prec)
    for k in range(len(tipos)):
        a = open(os.path.join(gold, f"mlp_type{k}.bin"), "rb").read()
        b = open(os.path.join(tmp_path, f"mlp_type{k}.bin"), "rb").read()
        assert a == b
        for name in DAT:
            want = np.loadtxt(os.path.join(gold, f"type{k}_{name}.dat"))
            got = np.loadtxt(os.path.join(tmp_path, f"type{k}_{name}.dat"))
            assert np.array_equal(want, got), name
    for name in ("cutoff_info", "type.dat"):
        assert np.array_equal(np.loadtxt(os.path.join(gold, name)), np.loadtxt(os.path.join(tmp_path, name)))
    keys = lambda p: {l.split("=")[0].strip(): l.split("=")[1].strip() for l in open(p) if "=" in l}
    assert keys(os.path.join(gold, "staf_jmd.cfg")) == keys(os.path.join(tmp_path, "staf_jmd.cfg"))


@pytest.mark.parametrize("prec", ["float", "double"])
def test_reader_agrees_with_the_test_loader(prec):
    from alphanesgpu_amd import model_dir
    tipos, model = load_model(prec)
    settings, species = model_dir.read_model_dir(os.path.join(GOLDEN, f"model_{prec}"))
    assert settings == dict(rc=4.5, rc_ang=4.5, rs=2.25, radial_buffer=60, angular_buffer=1770, number_of_types=2)
    for m, sp in zip(model, species):
        assert sp["precision"] == prec
        for key in ("alpha2b", "alpha3b", "emb2b", "emb3b"):
            assert np.array_equal(sp[key].astype(m[key].dtype), m[key])
        assert np.array_equal(sp["mu"], m["mu"])
        assert len(sp["layers"]) == len(m["layers"])
        for (W, b, act), (W0, b0, act0) in zip(sp["layers"], m["layers"]):
            assert act == act0 and np.array_equal(W, W0) and np.array_equal(b, b0.reshape(-1))


def test_mlp_bin_rejects_what_it_cannot_hold(tmp_path):
    from alphanesgpu_amd import model_dir
    with pytest.raises(ValueError):
        model_dir.write_mlp_bin(str(tmp_path / "a.bin"), np.zeros(3), [(np.zeros((3, 1)), np.zeros(1), "gelu")])
    with pytest.raises(ValueError):
        model_dir.write_mlp_bin(str(tmp_path / "b.bin"), np.zeros(3), [(np.zeros((3, 2)), np.zeros(1), "tanh")])
    (tmp_path / "c.bin").write_bytes(b"NOTAMODEL")
    with pytest.raises(ValueError):
        model_dir.read_mlp_bin(str(tmp_path / "c.bin"))


@pytest.mark.gpu
def test_compute_with_a_written_three_species_model(oracle, tmp_path):
    """A random three-species model (Ra < Rc, dense embeddings, species of different fingerprint widths) written
    to disk, loaded by staf_load and evaluated on a cluster given in mixed atom order: energy, forces and the six
    virial components against the oracle pipeline; tolerance 1e-10 (fp64 kernels, other summation orders)."""
    from alphanesgpu_amd import libstaf, model_dir
    from test_oracle_pins import cluster, energy_and_forces, small_model
    nr, na, rc, ra, rs = 24, 276, 4.5, 3.2, 1.6
    ps = small_model(3, (5, 4, 6), (4, 3, 5, 3, 4, 3), seed=5, dense=True)
    pos, box, tipos, type_map = cluster([5, 6, 4], seed=9)
    E, F, W, _, _ = energy_and_forces(oracle, pos, box, tipos, type_map, ps, nr=nr, na=na, rc=rc, ra=ra, rs=rs,
                                      virial=True)
    model_dir.write_model_dir(str(tmp_path), ps, rc=rc, rc_ang=ra, rs=rs, radial_buffer=nr, angular_buffer=na,
                              tipos=tipos)
    m = libstaf.StafModel(str(tmp_path), precision=1, full_virial=True)
    perm = np.random.default_rng(3).permutation(len(type_map))
    e, f, vir = m.compute(pos.reshape(-1, 3)[perm], box[0], type_map[perm])
    m.close()
    assert abs(e - float(E[0])) <= 1e-10 * max(1.0, abs(float(E[0])))
    assert nerr(f, F[0].reshape(-1, 3)[perm]) <= 1e-10
    Wm = W[0].reshape(3, 3)
    want = np.array([Wm[0, 0], Wm[1, 1], Wm[2, 2], 0.5 * (Wm[0, 1] + Wm[1, 0]), 0.5 * (Wm[0, 2] + Wm[2, 0]),
                     0.5 * (Wm[1, 2] + Wm[2, 1])])
    assert nerr(vir, want) <= 1e-10
