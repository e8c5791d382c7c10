"""The C-ABI library loads without a GPU and exports every entry point that include/*.h declares."""
import ctypes
import glob
import os
import re

from util import ROOT


def _declared():
    names = set()
    for h in glob.glob(os.path.join(ROOT, "include", "*.h")):
        src = re.sub(r"/\*.*?\*/", "", open(h).read(), flags=re.S)
        names |= set(re.findall(r"\b(staf_[a-z0-9_]+)\s*\(", src))
    return sorted(names)


def test_library_exports_every_declared_symbol():
    from alphanesgpu_amd import _lib
    assert os.path.exists(_lib.LIB_PATH), "build the library first: python -m alphanesgpu_amd.build"
    lib = ctypes.CDLL(_lib.LIB_PATH)
    names = _declared()
    assert len(names) >= 31
    missing = [n for n in names if not hasattr(lib, n)]
    assert not missing, f"declared in include/*.h but not exported: {missing}"


def test_host_only_entry_points():
    """Calls that need no device: version, the Init* ops and argument validation of construct."""
    from alphanesgpu_amd import _lib
    lib = _lib.lib()
    assert lib.staf_ops_version().decode() == "0.1"
    for f in ("staf_op_init_force_radial", "staf_op_init_force_tripl", "staf_op_init_grad_force_radial",
              "staf_op_init_grad_force_tripl"):
        assert getattr(lib, f)(ctypes.c_int(60)) == 0
        assert getattr(lib, f)(ctypes.c_int(0)) == -2
    rc = lib.staf_op_construct_descriptors_light_f64(ctypes.c_double(4.5), ctypes.c_int(0), ctypes.c_int(1770),
                                                     ctypes.c_int(768), ctypes.c_double(2.25), ctypes.c_double(4.5),
                                                     ctypes.c_int(4), ctypes.c_char_p(None))
    assert rc == -2


def test_construct_coefficients_and_cutoff_curve(tmp_path, oracle):
    """construct_descriptors_light computes A, B, C on the host like fill_repulsion and writes the same curve file."""
    import numpy as np
    from alphanesgpu_amd import _lib
    lib = _lib.lib()
    for sfx, ct, dt, tol in (("f64", ctypes.c_double, np.float64, 1e-13), ("f32", ctypes.c_float, np.float32, 2e-6)):
        path = str(tmp_path / f"curve_{sfx}.dat")
        rc = getattr(lib, f"staf_op_construct_descriptors_light_{sfx}")(ct(4.5), ctypes.c_int(60), ctypes.c_int(1770),
                                                                       ctypes.c_int(768), ct(2.25), ct(4.5),
                                                                       ctypes.c_int(4), ctypes.c_char_p(path.encode()))
        assert rc == 0
        out = (ct * 5)()
        assert getattr(lib, f"staf_op_descriptor_coefficients_{sfx}")(out) == 0
        want = oracle.fill_repulsion(4.5, 2.25, dt)
        got = np.array(list(out), np.float64)
        assert np.all(np.abs(got - want) <= tol * np.maximum(np.abs(want), 1e-30) + (1e-18 if sfx == "f32" else 0))
        ref = np.loadtxt(os.path.join(ROOT, "tests", "golden",
                                      "cutoff_curve_double.dat" if sfx == "f64" else "cutoff_curve_float.dat"))
        mine = np.loadtxt(path)
        ulp6 = lambda v: 10.0 ** (np.floor(np.log10(np.maximum(np.abs(v), 1e-300))) - 5)
        assert mine.shape == (1000, 2)
        assert np.all(np.abs(mine - ref) <= 1.6 * ulp6(ref) + 1e-12)


def test_library_depends_on_the_hip_runtime_only():
    """The boundary carries no framework types and the library no framework dependency: its dynamic section names
    the HIP runtime and the C/C++ runtimes, nothing of torch (a C or C++ host links it as it is), and it exports no
    oracle symbol."""
    import subprocess
    from alphanesgpu_amd import _lib
    dyn = subprocess.run(["readelf", "-d", _lib.LIB_PATH], capture_output=True, text=True, check=True).stdout
    needed = re.findall(r"\(NEEDED\)\s+Shared library: \[([^\]]+)\]", dyn)
    assert any(n.startswith("libamdhip64") for n in needed)
    allowed = ("libamdhip64", "libstdc++", "libm.", "libgcc_s", "libc.", "ld-linux", "libpthread", "libdl", "librt")
    assert all(n.startswith(allowed) for n in needed), needed
    syms = subprocess.run(["nm", "-D", "--defined-only", _lib.LIB_PATH], capture_output=True, text=True,
                          check=True).stdout
    assert "oracle" not in syms.lower()
