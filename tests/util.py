"""Shared helpers of the tests: fixture loaders, the reference-shaped model glue on numpy, comparison metrics."""
import os
import sys

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
GOLDEN = os.path.join(ROOT, "tests", "golden")
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def load_frame_mbpol(dtype=np.float64):
    """The reference's 768-atom MB-pol water frame (test/test-inference-pipeline/frames)."""
    d = os.path.join(GOLDEN, "frame_mbpol")
    pos = np.loadtxt(os.path.join(d, "pos_0")).astype(dtype).reshape(1, -1)
    box = np.loadtxt(os.path.join(d, "box_0")).astype(dtype).reshape(1, 6)
    tipos = np.loadtxt(os.path.join(d, "type.dat")).astype(np.int32).reshape(-1)
    type_map = np.concatenate([np.full(n, k, np.int32) for k, n in enumerate(tipos)])
    return pos, box, tipos, type_map


def load_water_smoke(dtype=np.float64):
    """test/test-lammps-smoke/data.water_smoke (LAMMPS atomic data file) -> pos [1,3N] in file order, box, types."""
    path = os.path.join(GOLDEN, "frame_mbpol", "data.water_smoke")
    lines = open(path).read().splitlines()
    n = int([l for l in lines if l.strip().endswith("atoms")][0].split()[0])
    lo_hi = [l.split() for l in lines if l.strip().endswith(("xlo xhi", "ylo yhi", "zlo zhi"))]
    L = [float(x[1]) - float(x[0]) for x in lo_hi]
    start = [i for i, l in enumerate(lines) if l.startswith("Atoms")][0] + 2
    rows = np.array([[float(v) for v in lines[start + i].split()] for i in range(n)])
    rows = rows[np.argsort(rows[:, 0])]
    types = rows[:, 1].astype(np.int32) - 1
    pos = rows[:, 2:5].astype(dtype).reshape(1, -1)
    box = np.array([[L[0], 0, 0, L[1], 0, L[2]]], dtype)
    return pos, box, types


def load_model(prec="float"):
    """Exported model parameters (test/test-lammps-smoke/model_onnx_*): per species dict with alpha2b, alpha3b,
    emb2b (squared), emb3b (squared), mu, and the MLP layers [(W, b, act), ...]."""
    d = os.path.join(GOLDEN, f"model_{prec}")
    dt = np.float32 if prec == "float" else np.float64
    tipos = np.loadtxt(os.path.join(d, "type.dat")).astype(np.int32).reshape(-1)
    out = []
    for k in range(len(tipos)):
        g = lambda f: np.atleast_2d(np.loadtxt(os.path.join(d, f"type{k}_{f}.dat"))).astype(dt)
        z = np.load(os.path.join(d, f"mlp_type{k}.npz"))
        nl = int(z["n_layers"][0]) if z["n_layers"][0] > 1 else sum(1 for f in z.files if f.startswith("W"))
        layers = [(z[f"W{i}"].astype(dt), z[f"b{i}"].astype(dt), str(z["activations"][i])) for i in range(nl)]
        out.append(dict(alpha2b=g("alpha_2body"), alpha3b=g("alpha_3body"), emb2b=g("type_emb_2b_sq"),
                        emb3b=g("type_emb_3b_sq"), mu=z["mu"].astype(dt), mu_dat=g("alpha_mu").reshape(-1),
                        layers=layers))
    return tipos, out


def mlp_energy_and_grad(af, mu, layers):
    """Native Dense of libstaf (libstaf/src/mlp/staf_mlp_ort.cc:186-233): x = log(af+1e-3)-mu, Dense stack,
    returns (sum of atomic energies, d(sum atomic)/d af).  af [n, n_af]."""
    dt = af.dtype
    x = np.log(af + dt.type(1e-3)) - mu
    acts = [x]
    for W, b, act in layers:
        y = acts[-1] @ W + b
        if act == "tanh":
            y = np.tanh(y)
        elif act == "relu":
            y = np.maximum(y, 0)
        acts.append(y.astype(dt))
    e = acts[-1].sum(dtype=dt)
    delta = np.ones_like(acts[-1])
    for li in range(len(layers) - 1, -1, -1):
        W, b, act = layers[li]
        g = delta
        if act == "tanh":
            g = g * (1 - acts[li + 1] ** 2)
        elif act == "relu":
            g = g * (acts[li + 1] > 0)
        delta = (g @ W.T).astype(dt)
    return e, (delta / (af + dt.type(1e-3))).astype(dt)


def species_slices(tipos):
    o = 0
    out = []
    for n in tipos:
        out.append(slice(o, o + int(n)))
        o += int(n)
    return out


def nerr(a, b):
    """max|a-b| / max|b|: the normalised error all floating-point tolerances in the tests refer to."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    if b.size == 0:
        assert a.shape == b.shape
        return 0.0
    s = np.max(np.abs(b))
    return float(np.max(np.abs(a - b)) / (s if s > 0 else 1.0))


def eerr(a, b, where=None):
    """Element-wise error max_e |a_e - b_e| / (|b_e| + rms(b)): `eerr <= tol` is the statement
    |a - b| <= tol |b| + tol rms(b) for every element, so small entries are held to the scale of the typical
    entry and not to that of the largest one.  where: boolean mask of the elements that count (rms over them)."""
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    if where is not None:
        a, b = a[where], b[where]
    if b.size == 0:
        return 0.0
    rms = float(np.sqrt(np.mean(b * b)))
    if rms == 0.0:
        return float(np.max(np.abs(a - b)))
    return float(np.max(np.abs(a - b) / (np.abs(b) + rms)))


def radial_mask(intmap2b, nr):
    """[nf,N,nr] True on active neighbour slots."""
    return np.arange(nr)[None, None, :] < intmap2b[:, :, :1]


def triplet_mask(numtriplet, na):
    ntr = numtriplet * (numtriplet - 1) // 2
    return np.arange(na)[None, None, :] < ntr[:, :, None]
