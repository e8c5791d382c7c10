"""The op-level C ABI driven by a program that is neither Python nor torch: tests/c_consumer/ops_chain.cpp
(hipMalloc, one stream, every staf_op_*_f64 in the reference's call order) against a fixture the CPU oracle writes."""
import os
import struct
import subprocess

import numpy as np
import pytest

from util import ROOT, species_slices
import pipeline

BIN = os.path.join(ROOT, "tests", "c_consumer", "ops_chain")


def _record(f, name, a):
    a = np.ascontiguousarray(a)
    kind = 0 if a.dtype == np.int32 else 1
    assert a.dtype in (np.int32, np.float64), (name, a.dtype)
    f.write(name.encode().ljust(32, b"\0")[:32])
    f.write(struct.pack("<iq", kind, a.size))
    f.write(a.tobytes())


def write_fixture(path, oracle, nf=2, nr=60, na=1770):
    from alphanesgpu_amd import synth
    b = synth.water_batch("water96")
    rng = np.random.Generator(np.random.Philox(77))
    pos = np.concatenate([b["pos"]] + [b["pos"] + rng.normal(0, 0.03, b["pos"].shape) for _ in range(nf - 1)])
    box = np.repeat(b["box"], nf, axis=0)
    tipos, type_map = b["tipos"], b["type_map"]
    dtype = np.dtype(np.float64)
    params = synth.fingerprint_params(dtype=dtype, dense_embedding=True, seed=12)
    up = pipeline.synthetic_upstream(nf, tipos, params, 13, dtype)
    ref = pipeline.run_oracle(oracle, pos, box, tipos, type_map, params, up, nr, na, dtype)
    d = ref["desc"]
    with open(path, "wb") as f:
        _record(f, "dims", np.array([nf, b["N"], len(tipos), nr, na], np.int32))
        _record(f, "geom", np.array([pipeline.RC, pipeline.RS, pipeline.RA]))
        _record(f, "pos", pos)
        _record(f, "box", box)
        _record(f, "tipos", tipos.astype(np.int32))
        _record(f, "type_map", type_map.astype(np.int32))
        _record(f, "Q", up["Q"])
        for k in ("raddescr", "angdescr", "des3bsupp", "der2b", "der3b", "der3bsupp"):
            _record(f, k, d[k])     # the oracle leaves zeros in every padded slot
        for k in ("intmap2b", "intmap3b", "numtriplet"):
            _record(f, k, d[k].astype(np.int32))
        ftot = None     # the callers' sum of the per-op force arrays, in the order of staf_op_force_total
        for k in range(len(tipos)):
            for part in (ref["f2"][k], ref["f3"][k]):
                ftot = part.copy() if ftot is None else ftot + part
        _record(f, "ftot", ftot)
        for k in range(len(tipos)):
            m = params[k]
            for name in ("alpha2b", "emb2b", "alpha3b", "emb3b"):
                _record(f, f"{name}_{k}", m[name])
            for name in ("G2", "G3", "P2", "P3"):
                _record(f, f"{name}_{k}", up[name][k])
            _record(f, f"af2_{k}", ref["af2"][k])
            _record(f, f"af3_{k}", ref["af3"][k])
            _record(f, f"f2_{k}", ref["f2"][k])
            _record(f, f"f3_{k}", ref["f3"][k])
            _record(f, f"g2a_{k}", ref["g2"][k][0])
            _record(f, f"g2e_{k}", ref["g2"][k][1])
            _record(f, f"g3a_{k}", ref["g3"][k][0])
            _record(f, f"g3e_{k}", ref["g3"][k][1])
            for i, nm in enumerate(("n", "a", "e")):
                _record(f, f"gf2{nm}_{k}", ref["gf2"][k][i])
                _record(f, f"gf3{nm}_{k}", ref["gf3"][k][i])


@pytest.mark.gpu
def test_cpp_caller_of_every_op_matches_the_oracle(oracle, tmp_path):
    assert os.path.exists(BIN), "tests/c_consumer/ops_chain is built by __graft_entry__.build()"
    path = str(tmp_path / "ops_chain.fixture")
    write_fixture(path, oracle)
    r = subprocess.run([BIN, path], capture_output=True, text=True, timeout=120)
    print(r.stdout)
    print(r.stderr)
    assert r.returncode == 0, r.stdout[-3000:] + r.stderr[-2000:]
    assert "ops_chain: OK" in r.stdout and "FAIL" not in r.stdout


def test_fixture_writer_round_trip(oracle, tmp_path):
    """The fixture format as the C++ reader expects it: name[32], kind, count, data; every expected array present."""
    path = str(tmp_path / "fx.bin")
    write_fixture(path, oracle, nf=1)
    names = {}
    with open(path, "rb") as f:
        while True:
            h = f.read(32)
            if not h:
                break
            kind, count = struct.unpack("<iq", f.read(12))
            names[h.rstrip(b"\0").decode()] = (kind, count)
            f.seek(count * (4 if kind == 0 else 8), 1)
    assert names["ftot"] == (1, 3 * 96) and names["dims"] == (0, 5) and names["der3b"] == (1, 96 * 3 * 2 * 1770)
    for k in range(2):
        for nm in ("af2", "af3", "f2", "f3", "g2a", "g2e", "g3a", "g3e", "gf2n", "gf2a", "gf2e", "gf3n", "gf3a", "gf3e"):
            assert f"{nm}_{k}" in names
