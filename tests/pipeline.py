"""Runs the full op sequence of one training-shaped step -- descriptor op, fingerprints, forces, parameter
gradients -- once through the CPU oracle and once through the HIP library, with the reference's Python-layer
argument mapping (STAF/source_routine/*.py, STAF/gradient_utility/*.py), and returns every tensor of both."""
import numpy as np

from alphanesgpu_amd.synth import synthetic_upstream  # noqa: F401  (the tests call it through this module)
from util import species_slices

RC, RA, RS = 4.5, 4.5, 2.25


def promote(ref, params, up):
    """fp64 copies of an fp32 run's descriptor tensors, parameters and upstream gradients: feeding them to the fp64
    oracle gives the exactly-rounded value of every downstream op on the very same fp32 inputs."""
    f64 = lambda a: a.astype(np.float64) if a.dtype == np.float32 else a
    d = {k: (f64(v) if isinstance(v, np.ndarray) else v) for k, v in ref["desc"].items()}
    p = [{k: f64(v) for k, v in m.items()} for m in params]
    u = {k: (f64(v) if isinstance(v, np.ndarray) else [f64(x) for x in v]) for k, v in up.items()}
    return d, p, u


def run_oracle(O, pos, box, tipos, type_map, params, up, nr, na, dtype, fma_mode=0, rc=RC, ra=RA, rs=RS, desc=None):
    d = desc if desc is not None else O.compute_descriptors_light(pos, box, rc, ra, rs, nr, na, fma_mode=fma_mode,
                                                                  dtype=dtype)
    out = dict(desc=d, af2=[], af3=[], f2=[], f3=[], g2=[], g3=[], gf2=[], gf3=[])
    if d["max_neigh"] > nr:
        return out
    for k, s in enumerate(species_slices(tipos)):
        m = params[k]
        c = lambda a: np.ascontiguousarray(a[:, s])
        out["af2"].append(O.radial_afs(c(d["raddescr"]), c(d["intmap2b"]), m["alpha2b"], m["emb2b"], type_map))
        out["af3"].append(O.angular_afs(c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]), m["alpha3b"],
                                        m["emb3b"], type_map, c(d["numtriplet"])))
        out["f2"].append(O.force_radial(up["G2"][k], c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]), m["alpha2b"],
                                        m["emb2b"], type_map, tipos, k))
        out["f3"].append(O.force_tripl(up["G3"][k], c(d["des3bsupp"]), c(d["angdescr"]), c(d["der3bsupp"]),
                                       c(d["der3b"]), c(d["intmap2b"]), c(d["intmap3b"]), m["alpha3b"], m["emb3b"],
                                       type_map, tipos, k, c(d["numtriplet"])))
        out["g2"].append(O.two_body_par_grad(up["P2"][k], c(d["raddescr"]), c(d["intmap2b"]), m["alpha2b"],
                                             m["emb2b"], type_map))
        out["g3"].append(O.sort_proj3body_grad(up["P3"][k], c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]),
                                               c(d["intmap2b"]), m["alpha3b"], m["emb3b"], type_map,
                                               c(d["numtriplet"])))
        out["gf2"].append(O.force_radial_grad(up["Q"], up["G2"][k], c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]),
                                              m["alpha2b"], m["emb2b"], type_map, tipos, k))
        out["gf3"].append(O.force_tripl_grad(up["Q"], up["G3"][k], c(d["des3bsupp"]), c(d["angdescr"]),
                                             c(d["der3bsupp"]), c(d["der3b"]), c(d["intmap2b"]), c(d["intmap3b"]),
                                             m["alpha3b"], m["emb3b"], type_map, tipos, k, c(d["numtriplet"])))
    return out


def run_hip(pos, box, tipos, type_map, params, up, nr, na, dtype, fma_mode=0, views=True, zero_padding=True,
            rc=RC, ra=RA, rs=RS):
    """Same sequence through libstaf_hip.so on cuda:0.  views=True passes dim-1 slices of the descriptor outputs
    (no copies); views=False passes contiguous per-species copies like tf.split."""
    import torch
    from alphanesgpu_amd import ops
    tdt = torch.float32 if np.dtype(dtype) == np.float32 else torch.float64
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    nf = box.shape[0]
    N = pos.shape[1] // 3
    ops.construct_descriptors_light(rc, nr, na, N, T(box), rs, ra, nf, dtype=tdt)
    ops.descriptor_options(dist2_fma=bool(fma_mode), zero_padding=zero_padding)
    ops.init_force_radial(nr)
    ops.init_force_tripl(na)
    ops.init_grad_force_radial(nr)
    ops.init_grad_force_tripl(na)
    names = ["raddescr", "angdescr", "des3bsupp", "intmap2b", "intmap3b", "der2b", "der3b", "der3bsupp",
             "numtriplet"]
    outs = ops.compute_descriptors_light(T(pos.astype(dtype)), T(box.astype(dtype)))
    d = dict(zip(names, outs))
    tm = T(type_map.astype(np.int32))
    tp = T(np.asarray(tipos, np.int32))
    res = dict(desc={k: v.cpu().numpy() for k, v in d.items()}, af2=[], af3=[], f2=[], f3=[], g2=[], g3=[], gf2=[],
               gf3=[])
    Q = T(up["Q"])
    for k, s in enumerate(species_slices(tipos)):
        m = {kk: T(vv) for kk, vv in params[k].items() if kk in ("alpha2b", "alpha3b", "emb2b", "emb3b")}
        sl = (lambda a: a[:, s]) if views else (lambda a: a[:, s].contiguous())
        G2, G3, P2, P3 = T(up["G2"][k]), T(up["G3"][k]), T(up["P2"][k]), T(up["P3"][k])
        at = torch.tensor([k], dtype=torch.int32, device=dev)
        res["af2"].append(ops.compute_sort_proj(sl(d["raddescr"]), sl(d["intmap2b"]), m["alpha2b"], m["emb2b"], tm))
        res["af3"].append(ops.compute_sort_proj3body(sl(d["angdescr"]), sl(d["des3bsupp"]), sl(d["intmap3b"]),
                                                     sl(d["intmap2b"]), m["alpha3b"], m["emb3b"], tm,
                                                     sl(d["numtriplet"]), nt=len(tipos)))
        res["f2"].append(ops.compute_force_radial(G2, sl(d["der2b"]), sl(d["intmap2b"]), sl(d["raddescr"]),
                                                  m["alpha2b"], m["emb2b"], tm, tp, at))
        res["f3"].append(ops.compute_force_tripl(G3, sl(d["des3bsupp"]), sl(d["angdescr"]), sl(d["der3bsupp"]),
                                                 sl(d["der3b"]), sl(d["intmap2b"]), sl(d["intmap3b"]), m["alpha3b"],
                                                 m["emb3b"], tm, tp, at, sl(d["numtriplet"])))
        res["g2"].append(ops.compute_two_body_par_grad(P2, sl(d["raddescr"]), sl(d["intmap2b"]), m["alpha2b"],
                                                       m["emb2b"], tm))
        res["g3"].append(ops.compute_sort_proj3body_grad(P3, sl(d["angdescr"]), sl(d["des3bsupp"]), sl(d["intmap3b"]),
                                                         sl(d["intmap2b"]), m["alpha3b"], m["emb3b"], tm,
                                                         sl(d["numtriplet"]), nt=len(tipos)))
        res["gf2"].append(ops.compute_force_radial_grad(Q, G2, sl(d["der2b"]), sl(d["intmap2b"]), sl(d["raddescr"]),
                                                        m["alpha2b"], m["emb2b"], tm, tp, at))
        res["gf3"].append(ops.compute_force_tripl_grad(Q, G3, sl(d["des3bsupp"]), sl(d["angdescr"]),
                                                       sl(d["der3bsupp"]), sl(d["der3b"]), sl(d["intmap2b"]),
                                                       sl(d["intmap3b"]), m["alpha3b"], m["emb3b"], tm, tp, at,
                                                       sl(d["numtriplet"])))
    torch.cuda.synchronize()
    to_np = lambda x: tuple(t.cpu().numpy() for t in x) if isinstance(x, tuple) else x.cpu().numpy()
    for key in ("af2", "af3", "f2", "f3", "g2", "g3", "gf2", "gf3"):
        res[key] = [to_np(x) for x in res[key]]
    return res
