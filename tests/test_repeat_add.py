"""flyvec_amd/csrc/fv_repeat_add.h on the host: n sequential fp32 additions done in O(binades)
steps must equal the plain loop bit for bit (the kernels rely on it for the sparse Hebbian term)."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("repeat_add") / "librepeat_add.so"
    subprocess.run(["gcc", "-O2", "-ffp-contract=off", "-shared", "-fPIC",
                    "-I", os.path.join(ROOT, "flyvec_amd", "csrc"),
                    os.path.join(ROOT, "tests", "native", "repeat_add_shim.c"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.fvt_count_mismatches.restype = C.c_uint64
    lib.fvt_count_mismatches.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64]
    lib.fvt_add_repeat.restype = C.c_float
    lib.fvt_add_repeat.argtypes = [C.c_float, C.c_float, C.c_uint32]
    return lib


def mismatches(lib, v, f, n):
    v = np.ascontiguousarray(v, dtype=np.float32)
    f = np.ascontiguousarray(f, dtype=np.float32)
    n = np.ascontiguousarray(n, dtype=np.uint32)
    return lib.fvt_count_mismatches(v.ctypes.data, f.ctypes.data, n.ctypes.data, len(v))


def test_training_like_values(shim):
    rng = np.random.default_rng(0)
    N = 300000
    v = -rng.normal(0, 1, N) * rng.normal(0, 0.02, N)      # -xx * W
    f = 1.0 / rng.integers(1, 2_000_000, N)                # 1 / count
    assert mismatches(shim, v, f, rng.integers(0, 6000, N)) == 0


def test_wild_magnitudes_and_signs(shim):
    rng = np.random.default_rng(1)
    N = 300000
    v = rng.normal(0, 1, N) * 10.0 ** rng.uniform(-12, 6, N)
    f = rng.normal(0, 1, N) * 10.0 ** rng.uniform(-12, 6, N)
    assert mismatches(shim, v, f, rng.integers(0, 3000, N)) == 0


def test_exact_ties_and_binade_edges(shim):
    rng = np.random.default_rng(2)
    N = 300000
    v = rng.integers(0x3f000000, 0x41000000, N).astype(np.uint32).view(np.float32)
    ulp = np.spacing(v)
    for scale in (64, 3):
        f = (rng.integers(1, scale, N) + 0.5) * ulp * rng.choice([-1, 1], N)   # fraction exactly 1/2 ulp
        n = rng.integers(0, 3000 if scale == 64 else 100000, N)
        assert mismatches(shim, v, f, n) == 0
        assert mismatches(shim, -v, f, n) == 0
    # walks that end exactly on a power of two from above and below
    v = np.float32(1.0) + np.arange(1, 2000, dtype=np.float32) * np.spacing(np.float32(1.0))
    f = -np.spacing(np.float32(1.0)) * np.ones_like(v)
    assert mismatches(shim, v, f, np.arange(1, 2000) + 5) == 0


def test_zero_denormal_absorbed(shim):
    rng = np.random.default_rng(3)
    v = np.concatenate([np.zeros(1000), rng.normal(0, 1e-40, 1000), np.full(1000, 1e8)])
    f = np.concatenate([rng.normal(0, 1e-42, 1000), rng.normal(0, 1e-41, 1000), np.full(1000, 0.5)])
    assert mismatches(shim, v, f, rng.integers(0, 5000, 3000)) == 0
    assert shim.fvt_add_repeat(1.0, 0.25, 0) == 1.0
    assert shim.fvt_add_repeat(1.0, 0.25, 8) == 3.0
