#!/usr/bin/env python3
"""Benchmark of the STAF fingerprint hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W] [--workload water768_f32] [--mode fwd_force|full_step]

One step = one pass of the op sequence over one synthetic batch that is already resident in HBM:
descriptor op (neighbour list + radial/angular descriptors), then per centre species the 2-body and
3-body fingerprint ops and the 2-body and 3-body force ops (mode fwd_force); mode full_step adds the four
parameter-gradient ops (dL/dalpha from the energy branch and from the force branch).  Upstream gradients
(dE/dAF, dL/dAF, dL/dF) are fixed synthetic tensors: the per-species MLP is not part of this path.

Prints ONE JSON line (metric, value = frames/s, roofline of the dominant kernel, CPU baseline).
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK_GBS = 8000.0  # MI355X HBM3E, published
# Vector-ALU roof: 256 CUs x 4 SIMDs, each issuing one 64-lane instruction per 4 cycles at the published 2.4 GHz
# (= the published 78.6 TFLOP/s of fp64, and of non-packed fp32, when every instruction is an FMA)
VALU_PEAK_WAVE_INST = 256 * 4 * 2.4e9 / 4
# Vector instructions the formulas of a 3-body op need per (triplet, active channel) item, fp32 / fp64, counted on
# the inner loops of csrc/staf_tri.hpp and csrc/staf_force3.hpp (pair factors from the exponential tables, exp(beta T),
# the op's accumulations; fp64 carries the written-out exponential instead of the hardware exp2: 15 instructions and a
# table read in the reduce kernels, 18 in the force kernel).
# Set-up, triplet decoding, table building, staging and reductions are overhead and not counted.
ALGORITHMIC_INST = {"af3_kernel": (7, 21), "desc_fp_kernel": (7, 21), "force3_kernel": (13, 30), "grad3_kernel": (14, 28),
                    "gradforce3_kernel": (36, 50), "grads3_kernel": (40, 54)}

SETTLE_STEPS = 300   # untimed graph replays of the set-up, see run_workload()
REPEATS = 5          # timed blocks of --steps steps each; the median block is reported

PROFILES = os.path.join(ROOT, "profiles")
# bench.py's kernel names (the library's timing names) -> the names the profiler prints
PROFILED_NAME = {
    ("force3_kernel", "f32"): "staf::force3_kernel<float, false, 4, true>",      # 2-body + 3-body slot forces
    ("force3_kernel", "f64"): "staf::force3_kernel<double, false, 4, true>",
    ("force3_kernel_3b_only", "f32"): "staf::force3_kernel<float, false, 4, false>",   # the reference's op sequence
    ("force3_kernel_3b_only", "f64"): "staf::force3_kernel<double, false, 4, false>",
    ("gradforce3_kernel", "f32"): "staf::tri_reduce_kernel<float, 2, false>",
    ("gradforce3_kernel", "f64"): "staf::tri_reduce_kernel<double, 2, false>",
    ("af3_kernel", "f32"): "staf::tri_reduce_kernel<float, 0, false>",
    ("af3_kernel", "f64"): "staf::tri_reduce_kernel<double, 0, false>",
    ("grad3_kernel", "f32"): "staf::tri_reduce_kernel<float, 1, false>",
    ("grad3_kernel", "f64"): "staf::tri_reduce_kernel<double, 1, false>",
    ("grads3_kernel", "f32"): "staf::tri_reduce_kernel<float, 3, false>",
    ("grads3_kernel", "f64"): "staf::tri_reduce_kernel<double, 3, false>",
    ("desc_fp_kernel", "f32"): "staf::desc_fingerprints_kernel<float>",     # descriptors + fingerprints, one launch
    ("desc_fp_kernel", "f64"): "staf::desc_fingerprints_kernel<double>",
    ("desc_kernel", "f32"): "staf::desc_kernel<float>",
    ("desc_kernel", "f64"): "staf::desc_kernel<double>",
    ("af3_fused", "f64"): "staf::tri_reduce_kernel<double, 0, true>",
    ("force3_fused", "f64"): "staf::force3_kernel<double, true, 4, true>",
}


class ProfileMissing(RuntimeError):
    pass


def profile_traffic(kernel, workload, prec):
    """HBM bytes per launch of `kernel` in `workload` from the committed rocprofv3 --pmc summary
    profiles/<kernel>_<workload>_hbm_counters.txt: (FETCH_SIZE x f + WRITE_SIZE x w) KiB averaged over the kernel's
    launches of a step, f and w = 1 GiB over what the same counter reads for the 1 GiB device copies of the same run.
    Raises ProfileMissing when the file, the kernel or the calibration copy is not in it."""
    import re
    path = os.path.join(PROFILES, f"{kernel}_{workload}_hbm_counters.txt")
    if not os.path.exists(path):
        raise ProfileMissing(f"{path} not found: no measured HBM traffic for {kernel} in {workload}")
    want = PROFILED_NAME[(kernel, prec)]
    vals = {"FETCH_SIZE": {}, "WRITE_SIZE": {}}
    copy = {}
    for line in open(path):
        m = re.match(r"^(.*?)\s+(\d+)\s+(FETCH_SIZE|WRITE_SIZE)=([0-9.eE+-]+)\(n=(\d+)\)\s*$", line)
        if not m:
            continue
        name, grid, ctr, v, n = m.group(1), int(m.group(2)), m.group(3), float(m.group(4)), int(m.group(5))
        inst = re.search(r"staf::(force3_kernel|tri_reduce_kernel|desc_kernel|desc_fingerprints_kernel)<[^>]*>", name)
        if inst and inst.group(0) not in PROFILED_NAME.values():
            # a row of an instantiation this library no longer builds: the file mixes runs of several builds
            raise ProfileMissing(f"{path} holds rows of {inst.group(0)}, which the current library does not build: "
                                 "regenerate it from one run")
        if name.startswith("__amd_rocclr_copyBuffer") and v > 1e5:
            copy[ctr] = v
        elif want in name:
            vals[ctr][grid] = (v, n)
    if len(copy) != 2 or not vals["FETCH_SIZE"] or set(vals["FETCH_SIZE"]) != set(vals["WRITE_SIZE"]):
        raise ProfileMissing(f"{path}: no rows for {want} (or no 1 GiB calibration copy) in both counters")
    kib = 0.0
    for grid, (f, _) in vals["FETCH_SIZE"].items():
        w, _ = vals["WRITE_SIZE"][grid]
        kib += f * (1048576.0 / copy["FETCH_SIZE"]) + w * (1048576.0 / copy["WRITE_SIZE"])
    return kib / len(vals["FETCH_SIZE"]) * 1024.0, os.path.relpath(path, ROOT)


def profile_valu_share(kernel, workload, mode, prec):
    """Share of the GPU's vector-issue slots that `kernel` fills when launched alone (column `issue` of
    profiles/step_<mode>_<workload>_sq_counters.txt, time-weighted over the kernel's launches of a step)."""
    tag = {"fwd_force": "step_fwd_force", "full_step": "step_full"}[mode]
    path = os.path.join(PROFILES, f"{tag}_{workload}_sq_counters.txt")
    if not os.path.exists(path):
        raise ProfileMissing(f"{path} not found: no SQ counters for {workload} ({mode})")
    want = PROFILED_NAME[(kernel, prec)].replace("staf::", "")
    num = den = 0.0
    for line in open(path):
        if not line.startswith(want):
            continue
        rest = line[len(want):].split()
        # grid waves avg_us VALU LDS issue ...
        us, issue = float(rest[2]), float(rest[5])
        num += us * issue
        den += us
    if den == 0.0:
        raise ProfileMissing(f"{path}: no row for {want}")
    return num / den, os.path.relpath(path, ROOT)


def algorithmic_bytes(N, tipos, nr, na, Ar, Aa, nt, s):
    """Bytes each op's signature forces through HBM once per frame (inputs read once, outputs written once),
    per-species calls summed.  Keys are the kernels that do the op's work."""
    ntc = nt * (nt + 1) // 2
    out = dict(desc_kernel=(N * (8 * nr + 7 * na)) * s + N * (nr + 1 + 2 * na + 1) * 4 + (3 * N + 6) * s)
    for k in ("af2", "af3", "force2", "force3", "grad2", "grad3", "gradforce2", "gradforce3", "grads3"):
        out[k + "_kernel"] = 0
    for Nl in tipos:
        par2 = 2 * nt * Ar * s
        par3 = (3 * ntc * Aa + ntc * Aa) * s
        tm = N * 4
        out["af2_kernel"] += Nl * nr * s + Nl * (nr + 1) * 4 + par2 + tm + Nl * Ar * s            # ComputeSortProj
        out["af3_kernel"] += (Nl * (na + nr) * s + Nl * (2 * na + nr + 1 + 1) * 4 + par3 + tm
                              + Nl * Aa * s)                                                      # ComputeSortProj3body
        out["force2_kernel"] += (Nl * (Ar + nr + 3 * nr) * s + Nl * (nr + 1) * 4 + par2 + tm
                                 + 3 * N * s)                                                     # ComputeForceRadial
        out["force3_kernel"] += (Nl * (Aa + nr + na + 3 * nr + 6 * na) * s + Nl * (nr + 1 + 2 * na + 1) * 4 + par3
                                 + tm + 3 * N * s)                                                # ComputeForceTripl
        out["grad2_kernel"] += (Nl * (Ar + nr) * s + Nl * (nr + 1) * 4 + par2 + tm
                                + 2 * nt * Ar * s)                                                # ComputeTwoBodyParGrad
        out["grad3_kernel"] += (Nl * (Aa + na + nr) * s + Nl * (2 * na + nr + 1 + 1) * 4 + par3 + tm
                                + (3 * ntc * Aa + ntc * Aa) * s)                                  # ...3bodyGrad
        out["gradforce2_kernel"] += (3 * N * s + Nl * (Ar + nr + 3 * nr) * s + Nl * (nr + 1) * 4 + par2 + tm
                                     + Nl * Ar * s + 2 * nt * Ar * s)                             # ComputeForceRadialGrad
        out["gradforce3_kernel"] += (3 * N * s + Nl * (Aa + nr + na + 3 * nr + 6 * na) * s
                                     + Nl * (nr + 1 + 2 * na + 1) * 4 + par3 + tm + Nl * Aa * s
                                     + (3 * ntc * Aa + ntc * Aa) * s)                             # ComputeForceTriplGrad
        # both 3-body parameter gradients in one pass: the inputs of ComputeForceTriplGrad, dL/dAF3 beside them, and
        # one more parameter-gradient array out
        out["grads3_kernel"] += (3 * N * s + Nl * (2 * Aa + nr + na + 3 * nr + 6 * na) * s
                                 + Nl * (nr + 1 + 2 * na + 1) * 4 + par3 + tm + Nl * Aa * s
                                 + (2 * 3 * ntc * Aa + ntc * Aa) * s)
    return out


def host_threads():
    """(threads the CPU legs use, cores the host shows).  The job's CPU share is what OMP_NUM_THREADS says where it
    is set (a GPU box hands a one-GPU job 16 of its cores), else every core."""
    cores = os.cpu_count() or 1
    try:
        share = int(os.environ.get("OMP_NUM_THREADS", cores))
    except ValueError:
        share = cores
    return max(1, min(share, cores)), cores


def cpu_baseline(batch, params, up, mode, nr, na, max_frames=2):
    """Times the CPU oracle on the first frames of the same batch: one thread (the reported value), and one frame per
    thread on all threads of the job's CPU share (frames are independent; ctypes releases the GIL inside the
    oracle's C++ calls)."""
    from concurrent.futures import ThreadPoolExecutor

    from oracle import staf_oracle as O
    dt = batch["dtype"]
    tipos, type_map = batch["tipos"], batch["type_map"]

    def frames(lo, hi):
        pos, box = batch["pos"][lo:hi], batch["box"][lo:hi]
        d = O.compute_descriptors_light(pos, box, 4.5, 4.5, 2.25, nr, na, dtype=dt)
        o = 0
        for k, n in enumerate(tipos):
            s = slice(o, o + int(n))
            o += int(n)
            m = params[k]
            c = lambda a: np.ascontiguousarray(a[:, s])
            u = lambda name: up[name][k][lo:hi]
            O.radial_afs(c(d["raddescr"]), c(d["intmap2b"]), m["alpha2b"], m["emb2b"], type_map)
            O.angular_afs(c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]), m["alpha3b"], m["emb3b"], type_map,
                          c(d["numtriplet"]))
            O.force_radial(u("G2"), c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]), m["alpha2b"], m["emb2b"],
                           type_map, tipos, k)
            O.force_tripl(u("G3"), c(d["des3bsupp"]), c(d["angdescr"]), c(d["der3bsupp"]), c(d["der3b"]),
                          c(d["intmap2b"]), c(d["intmap3b"]), m["alpha3b"], m["emb3b"], type_map, tipos, k,
                          c(d["numtriplet"]))
            if mode == "full_step":
                O.two_body_par_grad(u("P2"), c(d["raddescr"]), c(d["intmap2b"]), m["alpha2b"], m["emb2b"], type_map)
                O.sort_proj3body_grad(u("P3"), c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]),
                                      c(d["intmap2b"]), m["alpha3b"], m["emb3b"], type_map, c(d["numtriplet"]))
                O.force_radial_grad(up["Q"][lo:hi], u("G2"), c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]),
                                    m["alpha2b"], m["emb2b"], type_map, tipos, k)
                O.force_tripl_grad(up["Q"][lo:hi], u("G3"), c(d["des3bsupp"]), c(d["angdescr"]), c(d["der3bsupp"]),
                                   c(d["der3b"]), c(d["intmap2b"]), c(d["intmap3b"]), m["alpha3b"], m["emb3b"],
                                   type_map, tipos, k, c(d["numtriplet"]))

    nfs = min(max_frames, batch["nf"])
    reps = 3 if mode == "full_step" else 5

    def median_time(fn):
        fn()   # warm-up
        ts = []
        for _ in range(reps):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return float(np.median(ts))

    el = median_time(lambda: frames(0, nfs))
    threads, cores_visible = host_threads()
    nfr = batch["nf"]
    with ThreadPoolExecutor(threads) as ex:
        elm = median_time(lambda: list(ex.map(lambda i: frames(i % nfr, i % nfr + 1), range(threads))))
    return dict(value=nfs / el, unit="frames/s", cores=1, kind="port", host_cores=cores_visible,
                sample=f"{nfs} frame(s) of the same batch, same ops, scalar C++ oracle (-O2 -ffp-contract=off), 1 thread, "
                       f"median of {reps} after a warm-up; the host shows {cores_visible} cores",
                multicore=dict(value=threads / elm, unit="frames/s", cores=threads, host_cores=cores_visible,
                               sample=f"{threads} frames, one per thread on the {threads} threads of the job's CPU "
                                      f"share ({cores_visible} cores visible), same oracle, median of {reps}"))


def triplet_channel_items(desc_out, type_map_dev, tipos, params, nr, na):
    """Per centre species: sum over its centres and over the species pairs (ta <= tb) of the centre's triplets of
    (triplets of that pair) x (channels with non-zero squared embedding in parameter row ta + tb).  From the
    descriptor op's own outputs (numtriplet = neighbours inside the angular cutoff, the first of the sorted row)."""
    import torch
    im2, ntr = desc_out[3], desc_out[8]
    nt = len(tipos)
    nbr = im2[..., 1:].long()
    inside = torch.arange(nr, device=im2.device)[None, None, :] < ntr[..., None]
    sp = type_map_dev.long()[nbr]
    counts = [((sp == t) & inside).sum(-1).double() for t in range(nt)]   # [nf, N] each
    out = []
    o = 0
    for k, n in enumerate(tipos):
        nact = [(np.asarray(params[k]["emb3b"])[sg] != 0).sum() for sg in range(2 * nt - 1)]
        tot = 0.0
        for ta in range(nt):
            ca = counts[ta][:, o:o + n]
            for tb in range(ta, nt):
                cb = counts[tb][:, o:o + n]
                size = ca * (ca - 1) / 2 if ta == tb else ca * cb
                tot += float(size.sum()) * float(nact[ta + tb])
        out.append(tot)
        o += n
    return out


def numpy_mlp(af, mu, layers):
    """The per-species network of the MD entry on the host (Dense stack on log(af + 1e-3) - mu, as
    libstaf/src/mlp/staf_mlp_ort.cc:186-233): (sum of atomic energies, d sum / d af)."""
    x = np.log(af + 1e-3) - mu
    acts = [x]
    for W, b, act in layers:
        z = acts[-1] @ W + b
        acts.append(np.tanh(z) if act == "tanh" else (np.maximum(z, 0) if act == "relu" else z))
    g = np.ones_like(acts[-1])
    for (W, b, act), a_out in zip(reversed(layers), reversed(acts[1:])):
        if act == "tanh":
            g = g * (1 - a_out * a_out)
        elif act == "relu":
            g = g * (a_out > 0)
        g = g @ W.T
    return float(acts[-1].sum()), g / (af + 1e-3)


def run_md(args, workload):
    """The MD entry end to end: staf_compute on the workload's first frame, host arrays in and out, the library's
    own neighbour list rebuilt on every call, fingerprints -> device MLP -> forces without leaving the GPU.  The
    model is a random-initialised one of the reference's architecture (60 fingerprints -> 140 -> 140 -> 1, tanh),
    written as a model directory and loaded with staf_load."""
    import tempfile

    import torch
    from alphanesgpu_amd import libstaf, model_dir, ops, synth
    batch = synth.water_batch(workload)
    N, tipos, type_map = batch["N"], [int(x) for x in batch["tipos"]], batch["type_map"]
    nt = len(tipos)
    nr, na = synth.NR, synth.NA
    x = np.ascontiguousarray(batch["pos"][0].astype(np.float64).reshape(-1, 3))
    box = np.ascontiguousarray(batch["box"][0].astype(np.float64))
    params = synth.fingerprint_params(dtype=np.float64, dense_embedding=args.dense_embedding)
    rng = np.random.Generator(np.random.Philox(23))
    species = []
    for p in params:
        n_af = p["alpha2b"].shape[1] + p["alpha3b"].shape[1] // 3
        dims = [n_af, 140, 140, 1]
        layers = [(rng.standard_normal((a, b)) / np.sqrt(a), 0.1 * rng.standard_normal(b), "tanh" if b > 1 else "linear")
                  for a, b in zip(dims[:-1], dims[1:])]
        species.append(dict(p, layers=layers))
    Ar, Aa = params[0]["alpha2b"].shape[1], params[0]["alpha3b"].shape[1] // 3
    tmp = tempfile.mkdtemp(prefix="staf_bench_model_")
    model_dir.write_model_dir(tmp, species, rc=synth.RC, rc_ang=synth.RA, rs=synth.RS, radial_buffer=nr,
                              angular_buffer=na, tipos=tipos, precision="double")
    m = libstaf.StafModel(tmp, precision=1)
    for _ in range(8):     # sizes every buffer; the shape repeats, so the call's kernel sequence is recorded and replayed
        e, f, vir = m.compute(x, box, type_map)
    for _ in range(args.warmup):
        m.compute(x, box, type_map)
    block_s = []
    for _ in range(REPEATS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            m.compute(x, box, type_map)
        torch.cuda.synchronize()     # every call ends with its own synchronisation; this one finds nothing to wait for
        block_s.append(time.perf_counter() - t0)
    el = float(np.median(block_s))
    # per-kernel times from the library's events: a handle that launches every call eagerly (replayed graphs hold no events)
    me = libstaf.StafModel(tmp, precision=1, eager=True)
    for _ in range(3):
        e2, f2, _ = me.compute(x, box, type_map)
    if not (e2 == e and np.array_equal(f2, f)):
        print("bench.py: replayed and eager calls of staf_compute differ", file=sys.stderr)
        sys.exit(1)
    nprof = max(3, min(args.steps, 20))
    t1 = time.perf_counter()
    ops.kernel_timing(True)
    for _ in range(nprof):
        me.compute(x, box, type_map)
    ops.kernel_timing(False)
    el_eager = (time.perf_counter() - t1) / nprof
    kern = {}
    for name in ("cell_build_kernel", "desc_kernel", "af2_kernel", "af3_kernel", "force2_kernel", "force3_kernel",
                 "gather_kernel", "force_total_kernel"):
        ms, n = ops.kernel_time(name)
        if n:
            kern[name] = dict(ms_per_step=ms / nprof, launches_per_step=n // nprof, avg_launch_ms=ms / n)
    me.close()
    # items of the 3-body kernels, from an operator-level descriptor call on the same frame
    dev = torch.device("cuda:0")
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    ops.construct_descriptors_light(synth.RC, nr, na, N, None, synth.RS, synth.RA, 1, dtype=torch.float64)
    d_ = ops.compute_descriptors_light(T(batch["pos"][:1].astype(np.float64)), T(batch["box"][:1].astype(np.float64)))
    items = float(sum(triplet_channel_items(d_, T(type_map), tipos, params, nr, na)))
    pairs = float(d_[3][..., 0].clamp(max=nr).double().sum())
    del d_
    torch.cuda.empty_cache()
    # Bytes the call's kernels move once through HBM by their signatures (no tensor of the angular buffer's width
    # exists on this path).  In rows of N x nr doubles: the radial-only descriptor kernel writes 12 (raddescr,
    # des3bsupp, der2b x3, der3bsupp x3, unit x4) and the neighbour map; the 2-body fingerprints read 1 and the map,
    # the fused 3-body fingerprints 5 (des3bsupp, unit), the force launch 12 (raddescr, der2b, des3bsupp, der3bsupp,
    # unit) -- counted as 4 + 8 below; the slot forces are written and read once (3 rows); fingerprints and their
    # gradients are written and read once each; positions in, forces out (and the virial pass over the slot forces).
    s = 8
    row = N * nr * s
    imap = N * (nr + 1) * 4
    md_bytes = (12 * row + imap) + (row + imap) + (5 * row + imap) + (4 * row + imap) + (8 * row + imap) \
        + 2 * 3 * row + 4 * N * (Ar + Aa) * s + 10 * N * 3 * s
    dom = max(kern, key=lambda k: kern[k]["ms_per_step"])
    alg = {"af3_kernel": ALGORITHMIC_INST["af3_kernel"][1], "force3_kernel": ALGORITHMIC_INST["force3_kernel"][1]}
    valu_frac = {k: items * alg[k] / 64.0 / (kern[k]["ms_per_step"] * 1e-3) / VALU_PEAK_WAVE_INST for k in alg if k in kern}
    try:
        valu_share, valu_src = profile_valu_share_md(dom, workload)
    except ProfileMissing as ex:
        valu_share, valu_src = None, str(ex)
    t_dom = kern[dom]["ms_per_step"] * 1e-3
    out = {
        "metric": "frames/s descriptor fwd+force/alpha bwd, 768-atom water fp32/fp64; % HBM roofline",
        "value": args.steps / el,
        "unit": "frames/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": el / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "f64",
        "data": "synthetic",
        "config": {"workload": workload, "entry": "staf_compute (MD entry, include/staf.h)", "mode": "energy + forces + virial",
                   "atoms": N, "frames_per_step": 1, "Rc": synth.RC, "radial_buffer": nr, "angular_buffer": na,
                   "Ar": Ar, "Aa": Aa, "mlp": "60-140-140-1 tanh per species, float64, random init, on the GPU",
                   "neighbour_list": "the library's own, rebuilt on every call (cell list from 4096 atoms on)",
                   "boundary": "host arrays in (positions, box, species) and out (energy, forces, virial): the PCIe "
                               "copies and the call's one synchronisation are inside the timed region",
                   "launch": "the call's kernel sequence recorded once as a HIP graph and replayed",
                   "timing": f"median of {REPEATS} blocks of {args.steps} calls"},
        "block_ms_per_step": [b / args.steps * 1e3 for b in block_s],
        "eager_ms_per_step": el_eager * 1e3,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": md_bytes / (el / args.steps) / 1e9,
                     "peak": HBM_PEAK_GBS, "unit": "GB/s", "frac": md_bytes / (el / args.steps) / 1e9 / HBM_PEAK_GBS,
                     "frac_is": "bytes of the whole call (nr-wide tensors only: this path holds no tensor of the angular "
                                "buffer's width) over the call's time over peak: low by construction, the call is bound "
                                "by vector-ALU issue and by the latency of its ~25 dependent launches",
                     "traffic": None, "algorithmic_bytes_per_call": md_bytes,
                     "valu": {"bound": "valu", "unit": "wave instructions/s", "kernel": dom,
                              "algorithmic_inst_per_item": alg.get(dom), "items_per_call": items,
                              "achieved": (items * alg[dom] / 64.0 / t_dom) if dom in alg else None,
                              "peak": VALU_PEAK_WAVE_INST,
                              "frac": valu_frac.get(dom), "exp_per_s": (items / t_dom) if dom in alg else None,
                              "executed_issue_share": valu_share, "executed_issue_share_source": valu_src,
                              "note": "per (triplet, active channel) item as in the operator chain; the fused kernels "
                                      "also rebuild the angular descriptor and its Jacobian per triplet, which "
                                      "executed_issue_share includes"}},
        "kernel_valu_frac_algorithmic": valu_frac,
        "kernel_ms_per_step": {k: v["ms_per_step"] for k, v in kern.items()},
        "kernels_sum_ms": sum(v["ms_per_step"] for v in kern.values()),
        "active_slots": {"pairs_per_atom": pairs / N, "triplet_channel_items": items},
        "ms_per_frame": el / args.steps * 1e3,
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = md_cpu_baseline(x, box, tipos, type_map, species, nr, na)
    m.close()
    return out


def profile_valu_share_md(kernel, workload):
    """Issue share of the MD call's dominant kernel from profiles/md_step_<workload>_sq_counters.txt."""
    path = os.path.join(PROFILES, f"md_step_{workload}_sq_counters.txt")
    if not os.path.exists(path):
        raise ProfileMissing(f"{path} not found")
    want = PROFILED_NAME[({"af3_kernel": "af3_fused", "force3_kernel": "force3_fused"}.get(kernel, kernel), "f64")]
    want = want.replace("staf::", "")
    num = den = 0.0
    for line in open(path):
        if not line.startswith(want):
            continue
        rest = line[len(want):].split()
        us, issue = float(rest[2]), float(rest[5])
        num += us * issue
        den += us
    if den == 0.0:
        raise ProfileMissing(f"{path}: no row for {want}")
    return num / den, os.path.relpath(path, ROOT)


def md_cpu_baseline(x, box, tipos, type_map, species, nr, na):
    """The same call on the host: the CPU oracle's ops wired in the order of the reference's inference
    (STAF/staf_models/staf_model_inference_full.py:89-144) with the network as numpy matrix products, one thread
    for the oracle; one call, median of 3 after a warm-up."""
    from oracle import staf_oracle as O
    pos = x.reshape(1, -1)
    bx = box.reshape(1, 6)

    def call():
        d = O.compute_descriptors_light(pos, bx, 4.5, 4.5, 2.25, nr, na, dtype=np.float64)
        o = 0
        E = 0.0
        F = np.zeros_like(pos)
        for k, n in enumerate(tipos):
            sl = slice(o, o + n)
            o += n
            m = species[k]
            c = lambda a: np.ascontiguousarray(a[:, sl])
            af2 = O.radial_afs(c(d["raddescr"]), c(d["intmap2b"]), m["alpha2b"], m["emb2b"], type_map)
            af3 = O.angular_afs(c(d["angdescr"]), c(d["des3bsupp"]), c(d["intmap3b"]), m["alpha3b"], m["emb3b"],
                                type_map, c(d["numtriplet"]))
            af = np.concatenate([af2, af3], axis=2)
            e, g = numpy_mlp(af[0], m["mu"], m["layers"])
            E += 0.5 * e
            A2 = af2.shape[2]
            G = g[None]
            F += O.force_radial(np.ascontiguousarray(G[:, :, :A2]), c(d["der2b"]), c(d["intmap2b"]), c(d["raddescr"]),
                                m["alpha2b"], m["emb2b"], type_map, np.asarray(tipos, np.int32), k)
            F += O.force_tripl(np.ascontiguousarray(G[:, :, A2:]), c(d["des3bsupp"]), c(d["angdescr"]),
                               c(d["der3bsupp"]), c(d["der3b"]), c(d["intmap2b"]), c(d["intmap3b"]), m["alpha3b"],
                               m["emb3b"], type_map, np.asarray(tipos, np.int32), k, c(d["numtriplet"]))
        return E, F

    call()
    ts = []
    for _ in range(3):
        t0 = time.perf_counter()
        call()
        ts.append(time.perf_counter() - t0)
    _, cores_visible = host_threads()
    return dict(value=1.0 / float(np.median(ts)), unit="frames/s", cores=1, kind="port", host_cores=cores_visible,
                sample="one call on the same frame: scalar C++ oracle ops (-O2 -ffp-contract=off, 1 thread; all-pairs "
                       "neighbour search) and the network as numpy matrix products, median of 3 after a warm-up; "
                       f"the host shows {cores_visible} cores")


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=5)
    ap.add_argument("--workload", default=None,
                    help="one workload only (water96, water768_f32, water768_f64, water768_train8, water6144); "
                         "default: the headline water768_f32 fwd_force with the water768_f64 full_step record nested "
                         "under \"also\"")
    ap.add_argument("--mode", default=None, choices=[None, "fwd_force", "full_step"])
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--profiling-run", action="store_true",
                    help="the run that writes the profiles: figures read from profiles/ may be absent (null in the "
                         "line) instead of ending the run")
    ap.add_argument("--streams", type=int, default=3, choices=[1, 2, 3],
                    help="2: the per-species op chains (independent until the forces are summed) are issued on one "
                         "HIP stream per species; 3: in addition the 2-body ops of the species with the most centres "
                         "and the 2-body force ops of the other species run on the step's own stream; 1: everything "
                         "on one stream")
    ap.add_argument("--no-graph", action="store_true",
                    help="launch every op of every step from Python instead of replaying one captured HIP graph")
    ap.add_argument("--reference-op-sequence", action="store_true",
                    help="call the ops one by one as the reference's layers and gradient registry do: a force array per "
                         "force op (ComputeForceRadial, ComputeForceTripl) summed by one more launch, and the 3-body "
                         "parameter gradients as two ops (ComputeSortProj3bodyGrad, ComputeForceTriplGrad).  Default: "
                         "the library's step-level entry points -- the 3-body slot forces of all species collected "
                         "and added to the 2-body forces in one launch (staf_op_force_tripl_slots + "
                         "staf_op_force_total), both 3-body parameter gradients in one pass "
                         "(staf_op_grads_tripl_fused); same results")
    ap.add_argument("--first-stage", choices=["auto", "fused", "separate"], default="auto",
                    help="descriptors and fingerprints of a species in one launch (staf_op_descriptors_fingerprints) "
                         "or as the descriptor op and the fingerprint ops; auto: fused for single-precision "
                         "forward+force steps of at most 4096 atoms")
    ap.add_argument("--dense-embedding", action="store_true",
                    help="type embeddings without zeros: every 3-body channel is active for every species pair "
                         "(default: the 0/1 block embeddings the reference trains with, a third of them active)")
    ap.add_argument("--entry", default="ops", choices=["ops", "md"],
                    help="ops: the operator chain (default).  md: the MD entry staf_compute end to end on the workload's "
                         "first frame (host arrays in and out, own neighbour list rebuilt each call, device MLP)")
    ap.add_argument("--contiguous-splits", action="store_true",
                    help="copy per-species tensors like tf.split instead of passing views")
    args = ap.parse_args()
    if args.gpus != 1:
        print("bench.py: this build measures one GPU only (frames are independent: a data-parallel run gives each GPU its share of the frame batch); "
              "run with --gpus 1", file=sys.stderr)
        sys.exit(2)
    import torch
    if not torch.cuda.is_available():
        print("bench.py: no GPU visible", file=sys.stderr)
        sys.exit(1)
    if args.entry == "md":
        out = run_md(args, args.workload or "water6144")
    elif args.workload is not None:
        out = run_workload(args, args.workload, args.mode)
    else:
        # The metric names both halves: fp32 descriptor fwd + force (the headline line) and the fp64 full step with
        # the parameter-gradient ops, measured in the same process right behind it.
        out = run_workload(args, "water768_f32", "fwd_force")
        out["also"] = [run_workload(args, "water768_f64", "full_step"), run_md(args, "water6144")]
        if not args.reference_op_sequence:
            # the same two steps launched op by op as the reference's layers call them (drop-in sequence), for comparison
            import copy
            ref_args = copy.copy(args)
            ref_args.reference_op_sequence = True
            ref_args.no_cpu_baseline = True
            ref_args.profiling_run = True
            for rec, (wl, md) in zip([out, out["also"][0]], [("water768_f32", "fwd_force"), ("water768_f64", "full_step")]):
                r = run_workload(ref_args, wl, md)
                rec["reference_op_sequence"] = {"value": r["value"], "unit": r["unit"], "ms_per_step": r["ms_per_step"],
                                                "block_ms_per_step": r["block_ms_per_step"],
                                                "op_sequence": r["config"]["op_sequence"],
                                                "kernel_ms_per_step": r["kernel_ms_per_step"]}
    print(json.dumps(out))


def run_workload(args, workload, mode):
    import torch
    from alphanesgpu_amd import ops, synth

    dev = torch.device("cuda:0")
    batch = synth.water_batch(workload)
    mode = mode or ("fwd_force" if workload in ("water768_f32", "water6144") else "full_step")
    dtype = batch["dtype"]
    tdt = torch.float32 if dtype == np.float32 else torch.float64
    nr, na = synth.NR, synth.NA
    nf, N = batch["nf"], batch["N"]
    tipos = [int(x) for x in batch["tipos"]]
    nt = len(tipos)
    params = synth.fingerprint_params(dtype=dtype, dense_embedding=args.dense_embedding)
    Ar, Aa = params[0]["alpha2b"].shape[1], params[0]["alpha3b"].shape[1] // 3
    up = synth.synthetic_upstream(nf, batch["tipos"], params, 11, dtype)

    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    pos, box = T(batch["pos"]), T(batch["box"])
    tm, tp = T(batch["type_map"]), T(batch["tipos"])
    P = [{k: T(v) for k, v in m.items()} for m in params]
    G2, G3 = [T(x) for x in up["G2"]], [T(x) for x in up["G3"]]
    P2, P3 = [T(x) for x in up["P2"]], [T(x) for x in up["P3"]]
    Q = T(up["Q"])
    at = [torch.tensor([k], dtype=torch.int32, device=dev) for k in range(nt)]
    ops.construct_descriptors_light(synth.RC, nr, na, N, box, synth.RS, synth.RA, nf, dtype=tdt)
    ops.descriptor_options(dist2_fma=False, zero_padding=False)
    for f, b in ((ops.init_force_radial, nr), (ops.init_force_tripl, na), (ops.init_grad_force_radial, nr),
                 (ops.init_grad_force_tripl, na)):
        f(b)
    ops.set_sync_errors(False)
    e = lambda *sh: torch.empty(sh, dtype=tdt, device=dev)
    ei = lambda *sh: torch.empty(sh, dtype=torch.int32, device=dev)
    dbuf = (e(nf, N, nr), e(nf, N, na), e(nf, N, nr), ei(nf, N, nr + 1), ei(nf, N, 2 * na), e(nf, N, 3, nr),
            e(nf, N, 3, 2 * na), e(nf, N, 3, nr), ei(nf, N))
    slices = []
    o = 0
    for n in tipos:
        slices.append(slice(o, o + n))
        o += n
    if args.contiguous_splits:
        sl = lambda a, s: a[:, s].contiguous()
    else:
        sl = lambda a, s: a[:, s]

    timers = {}

    def timed(name, fn, record):
        if not record:
            return fn()
        a, b = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        a.record()
        r = fn()
        b.record()
        timers.setdefault(name, []).append((a, b))
        return r

    side = [torch.cuda.Stream() for _ in range(nt)] if args.streams > 1 else None

    # The ops of one centre species, by body order (2 / 3) and phase: 0 fingerprints, 1 forces, 2 parameter gradient
    # of the energy branch, 3 gradient of the force op.  In a real step the network sits between phase 0 and 1
    # and the loss between 1 and 2, so an op of a phase depends on both ops of the species' previous phase.
    n_phase = 4 if mode == "full_step" else 2

    def species_views(k, d):
        return [sl(x, slices[k]) for x in d]

    def body_op(k, v, body, phase, record):
        radk, angk, supk, im2k, im3k, d2k, d3k, d3sk, ntrk = v
        p = P[k]
        if phase == 0 and one_launch:
            return None    # the fingerprints come out of the step's first launch
        if body == 2:
            if phase == 0:
                return timed("af2", lambda: ops.compute_sort_proj(radk, im2k, p["alpha2b"], p["emb2b"], tm), record)
            if phase == 1 and not args.reference_op_sequence:
                return None    # the pair forces are added to the slot forces by the 3-body force launch
            if phase == 1:
                return timed("force2", lambda: ops.compute_force_radial(G2[k], d2k, im2k, radk, p["alpha2b"],
                                                                        p["emb2b"], tm, tp, at[k]), record)
            if phase == 2:
                return timed("grad2", lambda: ops.compute_two_body_par_grad(P2[k], radk, im2k, p["alpha2b"],
                                                                            p["emb2b"], tm), record)
            return timed("gradforce2", lambda: ops.compute_force_radial_grad(Q, G2[k], d2k, im2k, radk, p["alpha2b"],
                                                                             p["emb2b"], tm, tp, at[k]), record)
        if phase == 0:
            return timed("af3", lambda: ops.compute_sort_proj3body(angk, supk, im3k, im2k, p["alpha3b"], p["emb3b"],
                                                                   tm, ntrk, nt=nt), record)
        if phase == 1 and not args.reference_op_sequence:
            # slot forces of 2-body + 3-body only: the atoms collect them, for all species at once, in the step's
            # last launch
            return timed("force3", lambda: ops.compute_forces_slots(G3[k], G2[k], supk, angk, d3sk, d3k, radk, d2k,
                                                                    im2k, im3k, p["alpha3b"], p["emb3b"],
                                                                    p["alpha2b"], p["emb2b"], tm, tp, at[k], ntrk),
                         record)
        if phase == 1:
            return timed("force3", lambda: ops.compute_force_tripl(G3[k], supk, angk, d3sk, d3k, im2k, im3k,
                                                                   p["alpha3b"], p["emb3b"], tm, tp, at[k], ntrk),
                         record)
        if phase == 2 and not args.reference_op_sequence:
            # both 3-body parameter gradients (energy branch and force branch) in one pass
            return timed("grads3", lambda: ops.compute_tripl_grads_fused(Q, G3[k], P3[k], supk, angk, d3sk, d3k, im2k,
                                                                         im3k, p["alpha3b"], p["emb3b"], tm, tp,
                                                                         at[k], ntrk), record)
        if phase == 3 and not args.reference_op_sequence:
            return None
        if phase == 2:
            return timed("grad3", lambda: ops.compute_sort_proj3body_grad(P3[k], angk, supk, im3k, im2k,
                                                                          p["alpha3b"], p["emb3b"], tm, ntrk, nt=nt),
                         record)
        return timed("gradforce3", lambda: ops.compute_force_tripl_grad(Q, G3[k], supk, angk, d3sk, d3k, im2k, im3k,
                                                                        p["alpha3b"], p["emb3b"], tm, tp, at[k],
                                                                        ntrk), record)

    def species_chain(k, d, record, forces):
        """af2, af3, force2, force3, (grad2, grad3, gradforce2, gradforce3) of species k on the current stream."""
        v = species_views(k, d)
        for phase in range(n_phase):
            for body in (2, 3):
                out = body_op(k, v, body, phase, record)
                if phase == 1:
                    forces[(k, body)] = out

    big = int(np.argmax(tipos))   # the species with the most centres: its 3-body chain is the longest in the step

    # The library's step-level entry points: descriptors and the fingerprints of every species in one launch
    # (a workgroup per centre goes from the neighbour search to the centre's fingerprints), then per species the
    # slot forces (and the fused gradient pass), then the collecting launch.
    # It pays where the centres of a step number about what the GPU holds at once (2048 workgroups of the
    # single-precision kernels: the three launches it replaces each leave the GPU half empty while their last
    # workgroups run); with several rounds of workgroups per launch the separate launches, which walk over the
    # centres with persistent workgroups and run the species' fingerprint launches side by side, are faster.
    one_launch = (not args.reference_op_sequence and
                  (args.first_stage == "fused" or
                   (args.first_stage == "auto" and dtype == np.float32 and nf * N <= 4096 and mode == "fwd_force")))
    par_a3, par_e3 = [p["alpha3b"] for p in P], [p["emb3b"] for p in P]
    par_a2, par_e2 = [p["alpha2b"] for p in P], [p["emb2b"] for p in P]

    def first_stage(record, species=None):
        return timed("descriptor+fingerprints",
                     lambda: ops.compute_descriptors_fingerprints(pos, box, tm, tipos, par_a3, par_e3, par_a2, par_e2,
                                                                  out=dbuf, species=species)[0], record)

    def step(record=False, streams=side):
        if one_launch and streams is not None:
            d = dbuf   # written species by species below
        elif one_launch:
            d = first_stage(record)
        else:
            d = timed("descriptor", lambda: ops.compute_descriptors_light(pos, box, out=dbuf), record)
        forces = {}
        if streams is None:
            for k in range(nt):
                species_chain(k, d, record, forces)
        else:
            main_stream = torch.cuda.current_stream()   # the capture stream while a graph is recorded
            ready = main_stream.record_event()
            done = []
            forces_done = []   # events behind the force op of a side chain: all the total force waits for
            if one_launch:
                # Nothing of a species depends on another species before the total force: each species' chain on
                # its own stream, from its first launch (descriptors and fingerprints of its centres) on, the species
                # with the most centres first; the small 2-body gradient ops of all on the step's stream.
                order = sorted(range(nt), key=lambda k: -tipos[k])
                views = {k: species_views(k, d) for k in order}
                fingerprints = {}
                for k in order:
                    with torch.cuda.stream(streams[k]):
                        streams[k].wait_event(ready)
                        first_stage(record, (k, 1))
                        fingerprints[k] = streams[k].record_event()
                        forces[(k, 3)] = body_op(k, views[k], 3, 1, record)
                        forces_done.append(streams[k].record_event())
                        for phase in range(2, n_phase):
                            body_op(k, views[k], 3, phase, record)
                        for phase in range(2, n_phase):
                            body_op(k, views[k], 2, phase, record)
                        if n_phase > 2:
                            done.append(streams[k].record_event())
            else:

                def small_species():
                    for k in sorted(range(nt), key=lambda k: -tipos[k]):
                        if k == big and args.streams == 3:
                            continue
                        if args.streams == 3:
                            # Fingerprints and 3-body ops on the species' stream; its 2-body force (and the 2-body ops
                            # after it) on the step's stream, behind the largest species' 2-body ops and after both
                            # fingerprint ops of the species: that stream is idle by then, and the species' own chain,
                            # the last one to end otherwise, is shorter by those ops (126.0 -> 122.8 us per fp32 step).
                            vk = species_views(k, d)
                            with torch.cuda.stream(streams[k]):
                                streams[k].wait_event(ready)
                                body_op(k, vk, 2, 0, record)
                                body_op(k, vk, 3, 0, record)
                                fingerprints = streams[k].record_event()
                                forces[(k, 3)] = body_op(k, vk, 3, 1, record)
                                forces_done.append(streams[k].record_event())
                                for phase in range(2, n_phase):
                                    body_op(k, vk, 3, phase, record)
                                if n_phase > 2:
                                    done.append(streams[k].record_event())
                            main_stream.wait_event(fingerprints)
                            forces[(k, 2)] = body_op(k, vk, 2, 1, record)
                            for phase in range(2, n_phase):
                                body_op(k, vk, 2, phase, record)
                            continue
                        with torch.cuda.stream(streams[k]):
                            streams[k].wait_event(ready)
                            species_chain(k, d, record, forces)
                            forces_done.append(streams[k].record_event())

                if args.streams == 3:
                    # The largest species in two chains: its 3-body ops on its own stream, its 2-body ops on the
                    # step's stream (idle otherwise until the forces are summed).  Each chain's force op waits for the
                    # other's fingerprint op, the dependency the network creates in a real step.  (The gradient ops take
                    # their upstream gradients as given, here as in the per-species chains: no wait between them.)
                    # Issue order = the order in which a graph replay submits the chains: the longest one (the 3-body ops
                    # of the largest species) goes first, so that it starts right behind the descriptors, the other
                    # species' chains last (issued between the two, they held back the large species' 2-body ops
                    # until they were through).
                    sb = streams[big]
                    v = species_views(big, d)
                    for phase in range(2):
                        with torch.cuda.stream(sb):
                            if phase == 0:
                                sb.wait_event(ready)
                            out3 = body_op(big, v, 3, phase, record)
                            e3 = sb.record_event()
                        out2 = body_op(big, v, 2, phase, record)
                        e2 = main_stream.record_event()
                        if phase == 0:
                            main_stream.wait_event(e3)
                            sb.wait_event(e2)
                        else:
                            forces[(big, 2)], forces[(big, 3)] = out2, out3
                    with torch.cuda.stream(sb):
                        forces_done.append(e3)
                        for phase in range(2, n_phase):
                            body_op(big, v, 3, phase, record)
                        if n_phase > 2:
                            done.append(sb.record_event())
                    for phase in range(2, n_phase):
                        body_op(big, v, 2, phase, record)
                small_species()
            for ev in forces_done:
                main_stream.wait_event(ev)
            # eager steps: the force arrays were allocated on the side streams and are consumed on this one.  Under
            # capture the graph's private pool keeps them (and `forces` holds them until the sum is recorded): no
            # allocator event is queued inside the captured region.
            if not torch.cuda.is_current_stream_capturing():
                for f in forces.values():
                    for t in (f if isinstance(f, tuple) else (f,)):
                        if t is not None:
                            t.record_stream(main_stream)
        # Total force, one launch, always in the same order (2-body of species 0, 3-body of species 0, 2-body of
        # species 1, ...): the sum of the per-op force arrays (the reference's force_radial + force_angular and add_n
        # over the species) or, with the library's step-level entry points, the same sum with the 3-body slot forces
        # of all species collected by the receiving atoms inside that launch.
        if args.reference_op_sequence:
            total = timed("total", lambda: ops.add_n([forces[(k, body)] for k in range(nt) for body in (2, 3)]), record)
        else:
            total = timed("total", lambda: ops.force_total(d[3], tipos, [forces[(k, 3)][0] for k in range(nt)],
                                                           [forces[(k, 3)][1] for k in range(nt)]), record)
        if streams is not None:
            for ev in done:
                main_stream.wait_event(ev)   # the side chains' gradient ops end the step
        return total

    # One step = one replay of a HIP graph that holds the whole op sequence (the ops run on the stream they are
    # called on, so stream capture records their kernels; scratch is grown by the eager warm-up steps first).
    graph = None
    run = step
    for _ in range(2):
        step()
    ops.poll_status()
    if not args.no_graph:
        # the library keeps its scratch per stream and cannot grow it while a stream is captured: the step runs
        # once eagerly on the very streams the capture uses
        cap = torch.cuda.Stream()
        with torch.cuda.stream(cap):
            step()
        ops.poll_status()
        torch.cuda.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=cap):
            graph_out = step()
        run = graph.replay
    # A fresh process finds the GPU at idle clocks, and a few steps of 0.15-0.5 ms do not bring it to its working
    # clocks (the first fifty steps run 4-5 % slower than the steady state a training run is in): part of the set-up
    # is a run of untimed steps, beside the caller's own warm-up steps.
    for _ in range(SETTLE_STEPS if graph is not None else 20):
        run()
    for _ in range(args.warmup):
        run()
    ops.poll_status()
    # REPEATS blocks of exactly --steps steps, each between two device synchronisations; the median block is the
    # figure reported (a single block of 20 steps lasts under 3 ms and picks up whatever else the host does)
    block_s = []
    for _ in range(REPEATS):
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for _ in range(args.steps):
            run()
        torch.cuda.synchronize()
        block_s.append(time.perf_counter() - t0)
    el = float(np.median(block_s))
    ops.poll_status()
    if graph is not None:
        # the replayed graph must reproduce the eager step bit for bit (all reductions have a fixed order)
        graph.replay()
        torch.cuda.synchronize()
        got = graph_out.clone()
        want = step(streams=None)
        torch.cuda.synchronize()
        if not torch.equal(got, want):
            print("bench.py: HIP graph replay differs from the eager step", file=sys.stderr)
            sys.exit(1)

    # the same step with everything on one stream (reported beside the main figure)
    nprof = max(3, min(args.steps, 20))
    el1 = el
    if side is not None:
        torch.cuda.synchronize()
        # (three untimed steps first: the eager tensors of this arrangement are new to the allocator, whose first
        # device allocations after a capture have taken tens of milliseconds)
        for _ in range(3):
            step(streams=None)
        torch.cuda.synchronize()
        t1 = time.perf_counter()
        for _ in range(nprof):
            step(streams=None)
        torch.cuda.synchronize()
        el1 = (time.perf_counter() - t1) * args.steps / nprof

    # per-op GPU time with events on the launch stream, one stream (separate pass: events perturb the pipeline)
    for _ in range(nprof):
        step(record=True, streams=None)
    torch.cuda.synchronize()
    op_ms = {k: float(np.mean([a.elapsed_time(b) for a, b in v])) for k, v in timers.items()}
    calls = {k: len(v) // nprof for k, v in timers.items()}

    # what a plain device copy reaches on this GPU (bytes read + bytes written per second): second roofline denominator
    # (measured after the timed steps: six GiB of copies just before them would not leave the GPU as it was);
    # the six 1 GiB copies (__amd_rocclr_copyBuffer) are also the reference point of the HBM traffic counters
    src = torch.ones(1 << 28, dtype=torch.float32, device=dev)
    dst = torch.empty_like(src)
    dst.copy_(src)
    ev = [torch.cuda.Event(enable_timing=True) for _ in range(2)]
    ev[0].record()
    for _ in range(5):
        dst.copy_(src)
    ev[1].record()
    torch.cuda.synchronize()
    copy_gbs = 5 * 2 * src.numel() * 4 / (ev[0].elapsed_time(ev[1]) * 1e-3) / 1e9
    del src, dst

    # per-kernel GPU time from the library's own HIP events, recorded on the stream each kernel is launched on
    ops.kernel_timing(True)
    for _ in range(nprof):
        step(streams=None)
    ops.kernel_timing(False)
    s = np.dtype(dtype).itemsize
    ab = algorithmic_bytes(N, tipos, nr, na, Ar, Aa, nt, s)
    if not args.reference_op_sequence:
        # the 3-body force launch also does the 2-body force op's work: it is priced on the bytes of both signatures
        # less the force arrays neither op writes here, plus the slot forces it writes instead
        ab["force3_kernel"] += ab["force2_kernel"] - 2 * nt * 3 * N * s + N * (nr + 1) * 3 * s
        # the step's first launch does the work of the descriptor op and of both fingerprint ops of every species:
        # it is priced on what the three signatures hold less the descriptor tensors the fingerprint ops would
        # read back (here they come out of the cache of the CU that wrote them)
        ab["desc_fp_kernel"] = (ab["desc_kernel"] + N * (Ar + Aa) * s
                                + nt * ((2 * nt * Ar) + (nt * (nt + 1) // 2) * 4 * Aa) * s + N * 4)
    kern = {}
    for name in list(ab) + ["gather_kernel", "force_total_kernel", "transpose_sort_kernel", "cell_build_kernel"]:
        ms, n = ops.kernel_time(name)
        if n:
            kern[name] = dict(ms_per_step=ms / nprof, launches_per_step=n // nprof, avg_launch_ms=ms / n)
    per_step = {k: op_ms[k] * calls[k] for k in op_ms}
    step_bytes = sum(ab[k] for k in kern if k in ab)
    # the same byte count over the active slots only (pairs and triplets that exist), reported beside the padded one
    d_ = ops.compute_descriptors_light(pos, box, out=dbuf)
    torch.cuda.synchronize()
    cnt2 = d_[3][..., 0].clamp(max=nr).double()
    mtr = d_[8].double()
    nr_act = float(cnt2.mean())
    na_act = float(torch.clamp(mtr * (mtr - 1) / 2, max=na).mean())
    ab_act = algorithmic_bytes(N, tipos, nr_act, na_act, Ar, Aa, nt, s)
    if not args.reference_op_sequence:
        ab_act["force3_kernel"] += ab_act["force2_kernel"] - 2 * nt * 3 * N * s + N * (nr_act + 1) * 3 * s
    step_bytes_act = sum(ab_act[k] for k in kern if k in ab_act)
    # (triplet, active channel) items of the 3-body ops per centre species: the triplets of a centre by the species
    # pair of their two neighbours, times the channels whose squared embedding is not zero for that pair
    items = triplet_channel_items(d_, tm, tipos, params, nr, na)
    total_items = float(sum(items))
    col = 0 if dtype == np.float32 else 1
    valu_frac = {k: total_items * ALGORITHMIC_INST[k][col] / 64.0 / (kern[k]["ms_per_step"] * 1e-3) / VALU_PEAK_WAVE_INST
                 for k in kern if k in ALGORITHMIC_INST}
    step_alg_inst = sum(total_items * ALGORITHMIC_INST[k][col] / 64.0 for k in kern if k in ALGORITHMIC_INST)
    # the kernel the step spends most of its time in, priced against HBM with the bytes its op signature moves
    dom = max((k for k in kern if k in ab), key=lambda k: kern[k]["ms_per_step"])
    dom_bytes_per_launch = ab[dom] * nf / kern[dom]["launches_per_step"]
    achieved = dom_bytes_per_launch / (kern[dom]["avg_launch_ms"] * 1e-3) / 1e9
    prec = "f32" if dtype == np.float32 else "f64"
    try:
        traffic, traffic_src = profile_traffic(dom, workload, prec)
    except ProfileMissing as e:
        if workload in ("water768_f32", "water768_f64") and not args.profiling_run:
            raise SystemExit(f"bench.py: {e}")      # the configurations the metric is quoted on must be profiled
        traffic, traffic_src = None, str(e)
    try:
        valu_share, valu_src = profile_valu_share(dom, workload, mode, prec)
    except ProfileMissing as e:
        if workload in ("water768_f32", "water768_f64") and not args.profiling_run:
            raise SystemExit(f"bench.py: {e}")
        valu_share, valu_src = None, str(e)
    valu = None
    if dom in ALGORITHMIC_INST:
        per_launch = total_items / kern[dom]["launches_per_step"]
        t_launch = kern[dom]["avg_launch_ms"] * 1e-3
        valu = {"bound": "valu", "unit": "wave instructions/s",
                "algorithmic_inst_per_item": ALGORITHMIC_INST[dom][col],
                "items_per_launch": per_launch,
                "achieved": per_launch * ALGORITHMIC_INST[dom][col] / 64.0 / t_launch,
                "peak": VALU_PEAK_WAVE_INST,
                "frac": per_launch * ALGORITHMIC_INST[dom][col] / 64.0 / t_launch / VALU_PEAK_WAVE_INST,
                "exp_per_s": per_launch / t_launch,
                "executed_issue_share": valu_share, "executed_issue_share_source": valu_src,
                "note": "algorithmic = the instructions the op's formulas need per (triplet, active channel) item; "
                        "executed_issue_share = all vector instructions the kernel issues (SQ_INSTS_VALU x 4 cycles "
                        "over the launch's SIMD-cycles, rocprofv3): the difference is set-up, decoding, tables, "
                        "staging and reductions"
                        + ("; this launch also holds the descriptor op's work (neighbour search, descriptor rows and "
                           "their Jacobians), for which no per-item count is defined: the algorithmic figure counts the "
                           "3-body fingerprint items only" if dom == "desc_fp_kernel" else "")}
    # bytes desc_kernel really writes: the nr-wide tensors, angdescr and intmap3b over their whole rows (padding is
    # written as 0 like the reference's memsets), der3b over the triplets that exist only
    desc_written = N * (8 * nr + na) * s + N * (nr + 1 + 2 * na + 1) * 4 + N * 6 * na_act * s + (3 * N + 6) * s
    out = {
        "metric": "frames/s descriptor fwd+force/alpha bwd, 768-atom water fp32/fp64; % HBM roofline",
        "value": nf * args.steps / el,
        "unit": "frames/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": el / args.steps * 1e3,
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": prec,
        "data": "synthetic",
        "config": {"workload": workload, "mode": mode, "atoms": N, "frames_per_step": nf, "Rc": synth.RC,
                   "radial_buffer": nr, "angular_buffer": na, "Ar": Ar, "Aa": Aa,
                   "type_embeddings": ("dense: every channel active for every species pair" if args.dense_embedding
                                       else "0/1 blocks as the reference trains with: 14/13/13 of the 40 3-body "
                                            "channels active per species pair"),
                   "descriptor_padding": "library default = the reference op's: angdescr, intmap2b, intmap3b, "
                                         "numtriplet zero beyond the active slots; der3b padding left untouched",
                   "species_tensors": "contiguous copies" if args.contiguous_splits else "views",
                   "species_streams": args.streams,
                   "schedule": ({1: "one stream", 2: "one stream per species",
                                 3: "one stream per species; on the step's stream the 2-body ops of the largest "
                                    "species and the 2-body force ops of the others"}[args.streams]
                                if args.reference_op_sequence or args.streams == 1 else
                                "first launch on the step's stream, then one stream per species for its 3-body ops; "
                                "the 2-body gradient ops on the step's stream"),
                   "op_sequence": ("the reference's: one force array per force op and one launch that adds them; "
                                   "one op per parameter gradient" if args.reference_op_sequence else
                                   "the library's step-level entry points: descriptors and the fingerprints of all "
                                   "species in one launch (staf_op_descriptors_fingerprints), per species one launch for the 2-body and "
                                   "3-body slot forces (staf_op_forces_slots), collected by the receiving atoms of all "
                                   "species in one launch (staf_op_force_total)" + ("; both 3-body parameter gradients in one pass "
                                                             "(staf_op_grads_tripl_fused)" if mode == "full_step"
                                                             else "")),
                   "launch": "python per op" if graph is None else "hip graph replay",
                   "timing": f"median of {REPEATS} blocks of {args.steps} steps"},
        "block_ms_per_step": [b / args.steps * 1e3 for b in block_s],
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved, "peak": HBM_PEAK_GBS,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK_GBS,
                     "frac_is": "algorithmic bytes of the op's signature (padded slots included) over launch time "
                                "over peak; hbm_frac_measured prices the bytes the counters saw",
                     "traffic": traffic, "traffic_source": traffic_src,
                     "hbm_frac_measured": (None if traffic is None else
                                           traffic / (kern[dom]["avg_launch_ms"] * 1e-3) / 1e9 / HBM_PEAK_GBS),
                     "valu": valu,
                     "valu_issue_share": valu_share, "valu_issue_share_source": valu_src,
                     "measured_copy_GBs": copy_gbs, "frac_of_measured_copy": achieved / copy_gbs,
                     "algorithmic_bytes_per_launch": dom_bytes_per_launch,
                     "avg_launch_ms": kern[dom]["avg_launch_ms"],
                     "launches_per_step": kern[dom]["launches_per_step"]},
        "kernel_hbm_frac": {k: ab[k] * nf / (kern[k]["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS
                            for k in kern if k in ab},
        # desc_kernel against the bytes it writes (its signature's bytes include der3b padding it leaves alone)
        "desc_kernel_hbm_frac_of_written_bytes": (
            desc_written * nf / (kern["desc_kernel"]["ms_per_step"] * 1e-3) / 1e9 / HBM_PEAK_GBS
            if "desc_kernel" in kern else None),
        "kernel_valu_frac_algorithmic": valu_frac,
        "whole_step_valu_frac_algorithmic": step_alg_inst / (el / args.steps) / VALU_PEAK_WAVE_INST,
        "triplet_channel_items_per_step": total_items,
        "kernel_ms_per_step": {k: v["ms_per_step"] for k, v in kern.items()},
        "whole_step_hbm_frac": step_bytes * nf / (el / args.steps) / 1e9 / HBM_PEAK_GBS,
        "whole_step_frac_of_measured_copy": step_bytes * nf / (el / args.steps) / 1e9 / copy_gbs,
        "whole_step_hbm_frac_active_slots": step_bytes_act * nf / (el / args.steps) / 1e9 / HBM_PEAK_GBS,
        "active_slots": {"pairs_per_atom": nr_act, "triplets_per_atom": na_act},
        "op_ms_per_step": per_step,
        "ms_per_frame": el / args.steps * 1e3 / nf,
        "single_stream": {"value": nf * args.steps / el1, "ms_per_step": el1 / args.steps * 1e3},
    }
    if not args.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(batch, params, up, mode, nr, na)
    # leave the device as the next workload of this process expects to find it
    ops.set_sync_errors(True)
    return out


if __name__ == "__main__":
    main()
