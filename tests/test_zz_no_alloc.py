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


def _raw_call(name, x, ga, ge, stream):
    """The C call alone: no tensor is created and nothing is waited for here."""
    from alphanesgpu_amd import _lib
    nf, Nl, nr, nt, Ar = x["dims"]
    p = lambda t: C.c_void_p(t.data_ptr())
    fn = getattr(_lib.lib(), name)
    fn.restype = C.c_int
    return fn(p(x["D"]), C.c_int(nr), p(x["al"]), C.c_int(Ar), p(ga), C.c_int(nf), C.c_int(Nl), p(x["im"]), p(x["P"]),
              p(x["em"]), p(x["tm"]), p(ge), C.c_int(nt), C.c_int(Nl), C.c_void_p(stream.cuda_stream))


def test_noalloc_entry_against_the_oracle():
    """Directly against the CPU oracle's 2-body parameter gradient (not only through the allocating twin)."""
    import torch
    from oracle import staf_oracle as O
    from util import eerr
    dev = torch.device("cuda:0")
    x = _inputs(np.random.default_rng(23), 2, 96, 160, 40, 2, 20, dev)
    rc, ga, ge = _call("staf_op_alpha_dist_grad_noalloc_f64", x)
    assert rc == 0
    h = lambda k: x[k].cpu().numpy()
    ga0, ge0 = O.two_body_par_grad(h("P"), h("D"), h("im"), h("al"), h("em"), h("tm"))
    for got, want in ((ga, ga0), (ge, ge0)):
        assert eerr(got.cpu().numpy(), want) <= 1e-12   # |a - b| <= 1e-12 (|b| + rms(b)) element by element


def test_noalloc_entry_leaves_device_memory_alone_and_captures_on_a_stream_never_seen():
    """What the entry exists for: free device memory is the same before and after eager calls (also on a stream the
    library has never been called on), and the call can be captured on a fresh stream that never ran it eagerly;
    every replay reproduces the eager bits."""
    import torch
    dev = torch.device("cuda:0")
    x = _inputs(np.random.default_rng(29), 4, 512, 768, 60, 2, 20, dev)
    nt, Ar = x["dims"][3], x["dims"][4]
    new = lambda: torch.full((nt, Ar), float("nan"), dtype=torch.float64, device=dev)
    ga0, ge0 = new(), new()
    cur = torch.cuda.current_stream()
    assert _raw_call("staf_op_alpha_dist_grad_noalloc_f64", x, ga0, ge0, cur) == 0   # resolves the symbol's address
    torch.cuda.synchronize()
    # eager calls on the current stream and on a brand-new one: hipMemGetInfo must not move
    fresh = torch.cuda.Stream()
    ga1, ge1 = new(), new()
    torch.cuda.synchronize()
    free_before = torch.cuda.mem_get_info()[0]
    assert _raw_call("staf_op_alpha_dist_grad_noalloc_f64", x, ga1, ge1, cur) == 0
    torch.cuda.synchronize()
    fresh.wait_stream(cur)
    assert _raw_call("staf_op_alpha_dist_grad_noalloc_f64", x, ga1, ge1, fresh) == 0
    torch.cuda.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before
    assert torch.equal(ga1, ga0) and torch.equal(ge1, ge0)
    # capture on a stream no call of the library has seen, without an eager run on it
    cap = torch.cuda.Stream()
    ga2, ge2 = new(), new()
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g, stream=cap):
        rc = _raw_call("staf_op_alpha_dist_grad_noalloc_f64", x, ga2, ge2, torch.cuda.current_stream())
    assert rc == 0
    for rep in range(3):
        ga2.fill_(float("nan"))
        ge2.fill_(float("nan"))
        torch.cuda.synchronize()
        g.replay()
        torch.cuda.synchronize()
        assert torch.equal(ga2, ga0) and torch.equal(ge2, ge0), f"replay {rep}"
        # eager work of the same entry between the replays (it shares the work area, in stream order)
        assert _raw_call("staf_op_alpha_dist_grad_noalloc_f64", x, ga1, ge1, cur) == 0
        torch.cuda.synchronize()
        assert torch.equal(ga1, ga0)
