"""Batch inference class (alphanesgpu_amd/inference.py, the reference's staf_full_inference.full_test) on the
reference's exported models and its 768-atom frame: against the energies the reference recorded, and against the MD
entry of the library (staf_compute), which reaches the same numbers through different host code."""
import json
import os

import numpy as np
import pytest

from util import GOLDEN, load_frame_mbpol, nerr

KNOWN = json.load(open(os.path.join(GOLDEN, "known_answers.json")))


@pytest.mark.gpu
def test_full_test_matches_the_md_entry():
    import torch
    from alphanesgpu_amd import inference, libstaf
    pos, box, tipos, type_map = load_frame_mbpol(np.float64)
    N = len(type_map)
    # two frames in one batch: the recorded one and the same atoms shifted rigidly and wrapped differently
    pos2 = np.concatenate([pos, pos + 1.75])
    box2 = np.concatenate([box, box])
    inf = inference.staf_full_inference(os.path.join(GOLDEN, "model_double"), max_batch=2)
    E, F, W = inf.full_test(pos2, box2)
    E, F, W = E.cpu().numpy(), F.cpu().numpy(), W.cpu().numpy()
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1, full_virial=True)
    e, f, vir = m.compute(pos.reshape(-1, 3), box[0], type_map)
    m.close()
    # fp64 everywhere; the two paths sum in different orders
    assert abs(E[0] - e) <= 1e-10 * abs(e) and abs(E[1] - e) <= 1e-9 * abs(e)
    assert nerr(F[0], f.reshape(-1)) <= 1e-10 and nerr(F[1], f.reshape(-1)) <= 1e-8
    Wm = W[0].reshape(3, 3)
    sym = np.array([Wm[0, 0], Wm[1, 1], Wm[2, 2], 0.5 * (Wm[0, 1] + Wm[1, 0]), 0.5 * (Wm[0, 2] + Wm[2, 0]),
                    0.5 * (Wm[1, 2] + Wm[2, 1])])
    assert nerr(sym, vir) <= 1e-10
    # energy only: same energies, zero forces and virial
    E0, F0, W0 = inf.full_test(pos2, box2, energy_only=True)
    assert np.array_equal(E0.cpu().numpy(), E) and not F0.any() and not W0.any()
    assert F.shape == (2, 3 * N) and W.shape == (2, 9)


@pytest.mark.gpu
def test_float32_model_and_cluster_energy():
    """The float32 export against the energy the reference recorded for it (fp64 kernels with the float32 network:
    to the network's rounding; everything in float32: to float32 accumulation over 768 atoms), and energy_of_n_atoms on a water trimer
    given in mixed atom order against the MD entry on the same cluster."""
    import torch
    from alphanesgpu_amd import inference, libstaf
    pos, box, tipos, type_map = load_frame_mbpol(np.float64)
    ka = KNOWN["frame0_model_float"]
    inf = inference.staf_full_inference(os.path.join(GOLDEN, "model_float"))
    E, F, W = inf.full_test(pos, box)
    assert abs(float(E[0]) - ka["E_python"]) < 1.5e-4
    assert abs(float(torch.sqrt(torch.mean(F[0] ** 2))) - ka["rms_F_python"]) < 5e-6
    inf = inference.staf_full_inference(os.path.join(GOLDEN, "model_float"), dtype=torch.float32)
    E, F, W = inf.full_test(pos, box)
    # float32 descriptors and fingerprints as well (the recorded value is the reference's float32 Python pipeline)
    assert abs(float(E[0]) - ka["E_python"]) < 2e-3
    assert abs(float(torch.sqrt(torch.mean(F[0].double() ** 2))) - ka["rms_F_python"]) < 1e-4

    inf64 = inference.staf_full_inference(os.path.join(GOLDEN, "model_double"))
    p = pos.reshape(-1, 3)
    nO = int(tipos[0])
    # three molecules of the frame: oxygens 0..2 with their nearest two hydrogens each (minimum image), unwrapped
    L = box[0, [0, 3, 5]]
    atoms, types = [], []
    for o in range(3):
        d = p[nO:] - p[o]
        d -= L * np.round(d / L)
        near = np.argsort(np.linalg.norm(d, axis=1))[:2]
        atoms += [p[o], p[o] + d[near[0]], p[o] + d[near[1]]]
        types += [0, 1, 1]
    atoms, types = np.array(atoms), np.array(types, np.int32)
    big = np.array([60.0, 0, 0, 60.0, 0, 60.0])
    e_n = inf64.energy_of_n_atoms(atoms, types, big)
    m = libstaf.StafModel(os.path.join(GOLDEN, "model_double"), precision=1)
    e, _, _ = m.compute(atoms, big, types)
    m.close()
    assert abs(e_n - e) <= 1e-10 * max(1.0, abs(e))
