"""bench.py's command-line contract where no GPU is needed: more than one GPU is refused with a message, a host
without a GPU is reported (no CPU fallback), and the byte accounting of the roofline matches the per-frame figures
the measurement is specified with (768 atoms, nr = 60, na = 1770, Ar = 20, Aa = 40)."""
import os
import subprocess
import sys

import pytest

from util import ROOT

BENCH = os.path.join(ROOT, "bench.py")


def test_more_than_one_gpu_is_refused():
    r = subprocess.run([sys.executable, BENCH, "--gpus", "2"], capture_output=True, text=True, timeout=120)
    assert r.returncode != 0 and "one GPU" in r.stderr and r.stdout.strip() == ""


def test_no_gpu_is_an_error_not_a_fallback():
    import torch
    if torch.cuda.is_available():
        pytest.skip("a GPU is visible")
    r = subprocess.run([sys.executable, BENCH, "--steps", "1", "--warmup", "0"], capture_output=True, text=True,
                       timeout=300)
    assert r.returncode != 0 and "no GPU" in r.stderr and r.stdout.strip() == ""


def test_algorithmic_bytes_match_the_specified_per_frame_figures():
    """Descriptor op 50.6 / 90.2 MB, fingerprints 17.2 / 23.2, forces 51.0 / 90.7, energy-branch gradients 17.2 / 23.2,
    force gradients 51.2 / 91.1 MB per frame in fp32 / fp64; 118.9 MB (fwd + force, fp32) and 318.5 MB (full step,
    fp64) in total."""
    sys.path.insert(0, ROOT)
    import bench
    tot = {}
    for s, want in ((4, dict(desc=50.6, af=17.2, force=51.0, grad=17.2, gradforce=51.2)),
                    (8, dict(desc=90.2, af=23.2, force=90.7, grad=23.2, gradforce=91.1))):
        ab = bench.algorithmic_bytes(768, [256, 512], 60, 1770, 20, 40, 2, s)
        got = dict(desc=ab["desc_kernel"], af=ab["af2_kernel"] + ab["af3_kernel"],
                   force=ab["force2_kernel"] + ab["force3_kernel"], grad=ab["grad2_kernel"] + ab["grad3_kernel"],
                   gradforce=ab["gradforce2_kernel"] + ab["gradforce3_kernel"])
        for k, v in want.items():
            assert abs(got[k] / 1e6 - v) < 0.1, (s, k, got[k] / 1e6, v)     # the figures are given to 0.1 MB
        tot[s] = got
    assert abs(sum(tot[4][k] for k in ("desc", "af", "force")) / 1e6 - 118.9) < 0.15
    assert abs(sum(tot[8].values()) / 1e6 - 318.5) < 0.15
