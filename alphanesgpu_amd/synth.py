"""Seeded synthetic inputs of the benchmark configurations: rigid-water frames and
fingerprint parameters of the reference's shapes.  numpy only (Philox counter RNG),
so the same (config, seed) gives the same arrays on every machine with this image.
"""
import numpy as np

OH = 0.9572            # O-H bond, Angstrom
HOH = 104.52           # H-O-H angle, degrees
MIN_INTER = 1.3        # closest allowed intermolecular contact

CONFIGS = {
    # name: molecules lattice, box edge, thermal jitter sigma, frames, dtype, buffers
    "water96": dict(lattice=(4, 4, 2), L=9.86, sigma=0.0, nf=1, dtype="float64"),
    "water768_f32": dict(lattice=(8, 8, 4), L=19.6, sigma=0.05, nf=4, dtype="float32"),
    "water768_f64": dict(lattice=(8, 8, 4), L=19.6, sigma=0.05, nf=4, dtype="float64"),
    "water768_train8": dict(lattice=(8, 8, 4), L=19.6, sigma=0.05, nf=8, dtype="float32"),
    "water6144": dict(lattice=(16, 16, 8), L=39.1, sigma=0.05, nf=1, dtype="float64"),
}
CONFIG_INDEX = {"water96": 0, "water768_f32": 1, "water768_f64": 2, "water768_train8": 3, "water6144": 4}
RC, RA, RS, NR = 4.5, 4.5, 2.25, 60
NA = NR * (NR - 1) // 2
AR_MAP = (10, 10)        # radial channels per neighbour species
AA_MAP = (14, 13, 13)    # angular channels per species pair (OO, OH, HH)


def _rng(seed):
    return np.random.Generator(np.random.Philox(int(seed)))


def _rot(q):
    w, x, y, z = q
    return np.array([[1 - 2 * (y * y + z * z), 2 * (x * y - z * w), 2 * (x * z + y * w)],
                     [2 * (x * y + z * w), 1 - 2 * (x * x + z * z), 2 * (y * z - x * w)],
                     [2 * (x * z - y * w), 2 * (y * z + x * w), 1 - 2 * (x * x + y * y)]])


def water_frame(lattice, L, sigma, seed, jitter=0.5):
    """One frame: -> pos [3N] (all O then all H, unwrapped, centred on 0), box6.
    Molecule centres are stratified: one per lattice cell, uniform inside `jitter` x the cell edge around
    the cell centre (0.5 = anywhere in its own cell), which gives the ~38 neighbours within 4.5 A of liquid water.
    A molecule is accepted when none of its atoms is closer than MIN_INTER to an atom placed before it (minimum
    image); otherwise its orientation and its place in the cell are drawn again, and after every 50 failures the
    part of the cell it may fall in shrinks towards the cell centre, where a fitting orientation always exists."""
    rng = _rng(seed)
    nx, ny, nz = lattice
    nmol = nx * ny * nz
    half = np.deg2rad(HOH) / 2
    h_local = OH * np.array([[np.sin(half), 0.0, np.cos(half)], [-np.sin(half), 0.0, np.cos(half)]])
    sp = np.array([L / nx, L / ny, L / nz])
    placed = np.zeros((3 * nmol, 3))
    O = np.zeros((nmol, 3))
    H = np.zeros((nmol, 2, 3))
    m = 0
    for iz in range(nz):
        for iy in range(ny):
            for ix in range(nx):
                centre = (np.array([ix, iy, iz]) + 0.5) * sp
                for attempt in range(4000):
                    jit = jitter * 0.8 ** (attempt // 50)
                    c = centre + rng.uniform(-jit, jit, 3) * sp
                    q = rng.standard_normal(4)
                    q /= np.linalg.norm(q)
                    hs = c + h_local @ _rot(q).T
                    mol = np.vstack([c[None], hs])
                    if m:
                        d = mol[:, None, :] - placed[None, :3 * m, :]
                        d -= L * np.rint(d / L)
                        if np.min(np.einsum("abc,abc->ab", d, d)) < MIN_INTER ** 2:
                            continue
                    break
                else:
                    raise RuntimeError(f"water_frame: molecule {m} does not fit (seed {seed})")
                O[m] = c
                H[m] = hs
                placed[3 * m:3 * m + 3] = mol
                m += 1
    pos = np.vstack([O, H.reshape(-1, 3)])
    if sigma > 0:
        pos = pos + rng.normal(0.0, sigma, pos.shape)
    pos -= L / 2
    box = np.array([L, 0.0, 0.0, L, 0.0, L])
    return pos.reshape(-1), box


def water_batch(name, seed=None):
    """-> dict(pos [nf,3N], box [nf,6], type_map [N] int32, tipos [2] int32, dtype, nf, N)."""
    cfg = CONFIGS[name]
    base = 1000 + CONFIG_INDEX[name] if seed is None else seed
    nf = cfg["nf"]
    ps, bs = [], []
    for f in range(nf):
        p, b = water_frame(cfg["lattice"], cfg["L"], cfg["sigma"], base * 1000 + f)
        ps.append(p)
        bs.append(b)
    dtype = np.dtype(cfg["dtype"])
    nmol = int(np.prod(cfg["lattice"]))
    N = 3 * nmol
    return dict(pos=np.stack(ps).astype(dtype), box=np.stack(bs).astype(dtype),
                type_map=np.array([0] * nmol + [1] * (2 * nmol), np.int32), tipos=np.array([nmol, 2 * nmol], np.int32),
                dtype=dtype, nf=nf, N=N)


def block_embedding(widths):
    """0/1 block matrix [len(widths), sum(widths)]: row k is 1 on its own block of channels
    (the reference's initial type embeddings, STAF/init_params/init_AFs_param.py:14-22); squaring leaves it unchanged."""
    m = np.zeros((len(widths), sum(widths)))
    o = 0
    for k, w in enumerate(widths):
        m[k, o:o + w] = 1.0
        o += w
    return m


def fingerprint_params(nt=2, ar_map=AR_MAP, aa_map=AA_MAP, seed=7, dtype=np.float64, dense_embedding=False):
    """Per centre species k: alpha2b [nt,Ar], alpha3b [ntc,3*Aa] (alpha1,alpha2,beta ~ U(0.5,2)),
    squared embeddings emb2b [nt,Ar], emb3b [ntc,Aa], mu [Ar+Aa] ~ U(-1,1)."""
    rng = _rng(seed)
    ntc = nt * (nt + 1) // 2
    Ar, Aa = sum(ar_map), sum(aa_map)
    out = []
    for _ in range(nt):
        e2 = block_embedding(ar_map)
        e3 = block_embedding(aa_map)
        if dense_embedding:
            e2 = rng.uniform(0.2, 1.0, e2.shape)
            e3 = rng.uniform(0.2, 1.0, e3.shape)
        out.append(dict(
            alpha2b=rng.uniform(0.5, 2.0, (nt, Ar)).astype(dtype),
            alpha3b=rng.uniform(0.5, 2.0, (ntc, 3 * Aa)).astype(dtype),
            emb2b=e2.astype(dtype), emb3b=e3.astype(dtype),
            mu=rng.uniform(-1.0, 1.0, Ar + Aa).astype(dtype)))
    return out


def synthetic_upstream(nf, tipos, params, seed, dtype):
    """Stand-ins for what the MLP and the loss feed into the ops: G = d(sum e)/dAF ~ N(0,1), P = dL/dAF ~ N(0,1),
    Q = dL/dF ~ N(0,1)."""
    rng = np.random.Generator(np.random.Philox(seed))
    N = int(np.sum(tipos))
    up = dict(Q=rng.standard_normal((nf, 3 * N)).astype(dtype), G2=[], G3=[], P2=[], P3=[])
    for k, n in enumerate(tipos):
        Ar = params[k]["alpha2b"].shape[1]
        Aa = params[k]["alpha3b"].shape[1] // 3
        up["G2"].append(rng.standard_normal((nf, int(n), Ar)).astype(dtype))
        up["G3"].append(rng.standard_normal((nf, int(n), Aa)).astype(dtype))
        up["P2"].append(rng.standard_normal((nf, int(n), Ar)).astype(dtype))
        up["P3"].append(rng.standard_normal((nf, int(n), Aa)).astype(dtype))
    return up
