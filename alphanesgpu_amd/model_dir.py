"""Model directory of the MD entry (`staf_load`): writer and reader of the files the reference exports.

A model directory holds, per centre species k (formats as written by the reference's exporters,
STAF/save_models/export_mlp_grad_onnx.py:73-89 for the binary MLP, numpy.savetxt text for the rest, and read by
libstaf/src/staf_api.cpp:139-148 and libstaf/src/mlp/staf_mlp_ort.cc):

    type{k}_alpha_2body.dat     [nt, Ar]        text
    type{k}_alpha_3body.dat     [ntc, 3*Aa]     text, ntc = nt(nt+1)/2
    type{k}_type_emb_2b.dat     [nt, Ar]        text, the embedding as trained
    type{k}_type_emb_2b_sq.dat  [nt, Ar]        text, its square (what the kernels take)
    type{k}_type_emb_3b.dat     [ntc, Aa]       text
    type{k}_type_emb_3b_sq.dat  [ntc, Aa]       text
    type{k}_alpha_mu.dat        [n_af]          text, one value per line
    mlp_type{k}.bin             "STAFMLP1", int32 {precision, n_af, n_layers}, mu[n_af], then per layer
                                int32 {activation, in, out}, W[in, out] row-major, b[out]
    cutoff_info                 "Rc nr" / "Rc_ang na" / "Rs 0"
    staf_jmd.cfg                "key = value" lines
    type.dat                    atoms per species of the training frames (optional)

`species` below is a list with one dict per centre species: alpha2b, alpha3b, emb2b, emb3b (the squared
embeddings, as the ops take them), mu, layers = [(W[in, out], b[out], activation name), ...].
"""
import os

import numpy as np

ACTIVATIONS = {"linear": 0, "tanh": 1, "relu": 2}
_ACT_NAMES = {v: k for k, v in ACTIVATIONS.items()}


def write_mlp_bin(path, mu, layers, precision="double"):
    """One species' MLP in the "STAFMLP1" layout."""
    dt = np.float64 if precision == "double" else np.float32
    mu = np.asarray(mu, dtype=dt).reshape(-1)
    with open(path, "wb") as f:
        f.write(b"STAFMLP1")
        f.write(np.array([1 if dt == np.float64 else 0, mu.shape[0], len(layers)], dtype=np.int32).tobytes())
        f.write(mu.tobytes())
        for W, b, act in layers:
            if act not in ACTIVATIONS:
                raise ValueError(f"unsupported activation {act!r}")
            W = np.ascontiguousarray(W, dtype=dt)
            b = np.ascontiguousarray(b, dtype=dt).reshape(-1)
            if W.ndim != 2 or b.shape[0] != W.shape[1]:
                raise ValueError("layer shapes: W[in, out], b[out]")
            f.write(np.array([ACTIVATIONS[act], W.shape[0], W.shape[1]], dtype=np.int32).tobytes())
            f.write(W.tobytes())
            f.write(b.tobytes())


def read_mlp_bin(path):
    """Returns (precision name, mu, layers) of a "STAFMLP1" file."""
    raw = open(path, "rb").read()
    if raw[:8] != b"STAFMLP1":
        raise ValueError(f"{path}: not a STAFMLP1 file")
    prec, n_af, n_layers = np.frombuffer(raw, dtype=np.int32, count=3, offset=8)
    dt = np.float64 if prec == 1 else np.float32
    o = 20
    mu = np.frombuffer(raw, dtype=dt, count=n_af, offset=o).copy()
    o += n_af * dt().itemsize
    layers = []
    for _ in range(n_layers):
        act, nin, nout = np.frombuffer(raw, dtype=np.int32, count=3, offset=o)
        o += 12
        W = np.frombuffer(raw, dtype=dt, count=nin * nout, offset=o).reshape(nin, nout).copy()
        o += nin * nout * dt().itemsize
        b = np.frombuffer(raw, dtype=dt, count=nout, offset=o).copy()
        o += nout * dt().itemsize
        layers.append((W, b, _ACT_NAMES[int(act)]))
    if o != len(raw):
        raise ValueError(f"{path}: {len(raw) - o} trailing bytes")
    return ("double" if prec == 1 else "float"), mu, layers


def write_model_dir(path, species, rc=4.5, rc_ang=4.5, rs=2.25, radial_buffer=60, angular_buffer=1770, tipos=None,
                    precision="double"):
    """Writes every file `staf_load` reads.  Embeddings are given squared; the unsquared files hold their roots."""
    os.makedirs(path, exist_ok=True)
    nt = len(species)
    ntc = nt * (nt + 1) // 2
    for k, sp in enumerate(species):
        a2 = np.atleast_2d(np.asarray(sp["alpha2b"], dtype=np.float64))
        a3 = np.atleast_2d(np.asarray(sp["alpha3b"], dtype=np.float64))
        e2 = np.atleast_2d(np.asarray(sp["emb2b"], dtype=np.float64))
        e3 = np.atleast_2d(np.asarray(sp["emb3b"], dtype=np.float64))
        if a2.shape[0] != nt or e2.shape != a2.shape:
            raise ValueError(f"species {k}: alpha2b and emb2b are [nt, Ar]")
        if a3.shape[0] != ntc or a3.shape[1] % 3 or e3.shape != (ntc, a3.shape[1] // 3):
            raise ValueError(f"species {k}: alpha3b is [ntc, 3*Aa], emb3b [ntc, Aa]")
        if (e2 < 0).any() or (e3 < 0).any():
            raise ValueError(f"species {k}: the embeddings are squares")
        pre = os.path.join(path, f"type{k}_")
        np.savetxt(pre + "alpha_2body.dat", a2)
        np.savetxt(pre + "alpha_3body.dat", a3)
        np.savetxt(pre + "type_emb_2b_sq.dat", e2)
        np.savetxt(pre + "type_emb_3b_sq.dat", e3)
        np.savetxt(pre + "type_emb_2b.dat", np.sqrt(e2))
        np.savetxt(pre + "type_emb_3b.dat", np.sqrt(e3))
        np.savetxt(pre + "alpha_mu.dat", np.asarray(sp["mu"], dtype=np.float64).reshape(-1))
        write_mlp_bin(os.path.join(path, f"mlp_type{k}.bin"), sp["mu"], sp["layers"], precision)
    with open(os.path.join(path, "cutoff_info"), "w") as f:
        f.write(f"{rc:g} {radial_buffer}\n{rc_ang:g} {angular_buffer}\n{rs:g} 0\n")
    with open(os.path.join(path, "staf_jmd.cfg"), "w") as f:
        f.write(f"Buffer_radial_descriptors = {radial_buffer}\nBuffer_angular_descriptors = {angular_buffer}\n"
                f"Cutoff = {rc:g}\nCutoff_Angular = {rc_ang:g}\nHardcore_Cutoff = {rs:g}\n"
                f"number_of_types = {nt}\nfile_of_tipos = type.dat\nnn_export_dir = .\n")
    if tipos is not None:
        np.savetxt(os.path.join(path, "type.dat"), np.asarray(tipos, dtype=np.int64).reshape(-1), fmt="%d")


def read_model_dir(path):
    """Returns (settings dict, species list) of a model directory, the MLP taken from mlp_type{k}.bin."""
    cfg = {}
    p = os.path.join(path, "staf_jmd.cfg")
    if os.path.exists(p):
        for line in open(p):
            if "=" in line:
                key, val = (x.strip() for x in line.split("=", 1))
                cfg[key] = val
    nt = int(cfg["number_of_types"]) if "number_of_types" in cfg else \
        sum(1 for f in os.listdir(path) if f.startswith("mlp_type") and f.endswith(".bin"))
    species = []
    for k in range(nt):
        g = lambda name: np.atleast_2d(np.loadtxt(os.path.join(path, f"type{k}_{name}.dat")))
        sq = lambda name: g(name + "_sq") if os.path.exists(os.path.join(path, f"type{k}_{name}_sq.dat")) \
            else g(name) ** 2
        prec, mu, layers = read_mlp_bin(os.path.join(path, f"mlp_type{k}.bin"))
        species.append(dict(alpha2b=g("alpha_2body"), alpha3b=g("alpha_3body"), emb2b=sq("type_emb_2b"),
                            emb3b=sq("type_emb_3b"), mu=mu, layers=layers, precision=prec))
    settings = dict(rc=float(cfg.get("Cutoff", 4.5)), rc_ang=float(cfg.get("Cutoff_Angular", 4.5)),
                    rs=float(cfg.get("Hardcore_Cutoff", 2.25)),
                    radial_buffer=int(cfg.get("Buffer_radial_descriptors", 60)),
                    angular_buffer=int(cfg.get("Buffer_angular_descriptors", 1770)), number_of_types=nt)
    return settings, species
