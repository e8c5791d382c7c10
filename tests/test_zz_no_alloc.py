"""The entry point that allocates nothing, staf_op_alpha_dist_grad_noalloc_f64, through the C ABI: same results as
staf_op_alpha_dist_grad_f64 bit for bit (same kernels, same partial-sum layout; the bar for this floating-point
output is 1e-12, bit equality is stronger), on two calls in a row, the second with a smaller input, so that what the
first call left in the shared work area must not leak into the second.  Also: the size limit is refused."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def _inputs(rng, nf, Nl, N, nr, nt, Ar, dev):
    import torch
    T = lambda a: torch.as_tensor(np.ascontiguousarray(a)).to(dev)
    D = rng.uniform(0.05, 1.0, (nf, Nl, nr))
    im = np.zeros((nf, Nl, nr + 1), np.int32)
    cnt = rng.integers(0, nr + 1, (nf, Nl))
    im[..., 0] = cnt
    im[..., 1:] = rng.integers(0, N, (nf, Nl, nr))
    im[..., 1:][np.arange(nr)[None, None, :] >= cnt[..., None]] = 0
    return dict(D=T(D), im=T(im), P=T(rng.standard_normal((nf, Nl, Ar))), al=T(rng.uniform(0.5, 2.0, (nt, Ar))),
                em=T(rng.uniform(0.2, 1.0, (nt, Ar))), tm=T(rng.integers(0, nt, N).astype(np.int32)),
                dims=(nf, Nl, nr, nt, Ar))


def _call(name, x):
    import torch
    from alphanesgpu_amd import _lib
    nf, Nl, nr, nt, Ar = x["dims"]
    ga = torch.full((nt, Ar), float("nan"), dtype=torch.float64, device=x["D"].device)
    ge = torch.full((nt, Ar), float("nan"), dtype=torch.float64, device=x["D"].device)
    p = lambda t: C.c_void_p(t.data_ptr())
    fn = getattr(_lib.lib(), name)
    fn.restype = C.c_int
    rc = fn(p(x["D"]), C.c_int(nr), p(x["al"]), C.c_int(Ar), p(ga), C.c_int(nf), C.c_int(Nl), p(x["im"]), p(x["P"]),
            p(x["em"]), p(x["tm"]), p(ge), C.c_int(nt), C.c_int(Nl),
            C.c_void_p(torch.cuda.current_stream().cuda_stream))
    torch.cuda.synchronize()
    return rc, ga, ge


def test_noalloc_entry_matches_the_allocating_one_twice_in_a_row():
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(17)
    big = _inputs(rng, 4, 512, 768, 60, 2, 20, dev)      # 2048 centres: more than the 1024 partial rows
    small = _inputs(rng, 1, 37, 96, 24, 3, 7, dev)       # a smaller call right behind it, other dims throughout
    for x in (big, small):
        rc, ga, ge = _call("staf_op_alpha_dist_grad_noalloc_f64", x)
        assert rc == 0
        rc0, ga0, ge0 = _call("staf_op_alpha_dist_grad_f64", x)
        assert rc0 == 0
        assert not torch.isnan(ga).any() and not torch.isnan(ge).any()
        assert torch.equal(ga, ga0) and torch.equal(ge, ge0)
        scale = float(ga0.abs().max())
        assert float((ga - ga0).abs().max()) <= 1e-12 * scale
    # and the big one again after the small one
    rc, ga, ge = _call("staf_op_alpha_dist_grad_noalloc_f64", big)
    rc0, ga0, ge0 = _call("staf_op_alpha_dist_grad_f64", big)
    assert rc == 0 and rc0 == 0 and torch.equal(ga, ga0) and torch.equal(ge, ge0)


def test_noalloc_entry_refuses_what_its_work_area_cannot_hold():
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(3)
    # 4096 centres -> 1024 partial rows (+ 32) of 2 * nt * Ar = 160 doubles: 1.35 MB > 1 MiB
    x = _inputs(rng, 8, 512, 768, 20, 4, 20, dev)
    rc, ga, ge = _call("staf_op_alpha_dist_grad_noalloc_f64", x)
    assert rc == -12
    assert torch.isnan(ga).all()                          # nothing was written
    rc0, _, _ = _call("staf_op_alpha_dist_grad_f64", x)
    assert rc0 == 0


def test_noalloc_entry_empty_species():
    import torch
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(4)
    x = _inputs(rng, 2, 1, 10, 8, 2, 5, dev)
    x["dims"] = (2, 0, 8, 2, 5)
    rc, ga, ge = _call("staf_op_alpha_dist_grad_noalloc_f64", x)
    assert rc == 0 and torch.all(ga == 0) and torch.all(ge == 0)
