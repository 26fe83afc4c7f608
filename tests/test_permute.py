"""flyvec_amd/csrc/fv_permute.h on the host: the per-index window shuffle must be a bijection of
[0, n) for every n, depend on the seed, and look like a random permutation."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("permute") / "libpermute.so"
    subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "flyvec_amd", "csrc"),
                    os.path.join(ROOT, "tests", "native", "permute_shim.c"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.fvt_permutation.restype = None
    lib.fvt_permutation.argtypes = [C.c_uint64, C.c_uint64, C.c_void_p]
    lib.fvt_half_bits.restype = C.c_uint32
    lib.fvt_half_bits.argtypes = [C.c_uint64]
    return lib


def permutation(lib, n, seed):
    out = np.empty(n, dtype=np.uint64)
    lib.fvt_permutation(n, seed, out.ctypes.data)
    return out


@pytest.mark.parametrize("n", [1, 2, 3, 4, 5, 7, 8, 9, 15, 16, 17, 100, 255, 256, 257, 1000, 4095, 4097,
                               65536, 100003, 1 << 20, 3_000_001])
def test_bijection(shim, n):
    p = permutation(shim, n, seed=12345)
    assert np.array_equal(np.sort(p), np.arange(n, dtype=np.uint64))


def test_domain_is_below_four_n(shim):
    for n in [1, 2, 3, 5, 17, 1000, 66_500_000, (1 << 31) + 5, (1 << 62)]:
        hb = shim.fvt_half_bits(n)
        assert 2 ** (2 * hb) >= n
        assert n <= 2 or 2 ** (2 * hb) < 4 * n


def test_seed_changes_the_order_and_is_repeatable(shim):
    n = 50000
    a, b, a2 = permutation(shim, n, 1), permutation(shim, n, 2), permutation(shim, n, 1)
    assert np.array_equal(a, a2)
    assert np.mean(a == b) < 0.001
    assert np.mean(a == np.arange(n)) < 0.001


def test_looks_random(shim):
    # bucket counts of where each tenth of the indices lands: chi-square against uniform, and the
    # correlation between neighbours' images
    n = 1_000_000
    p = permutation(shim, n, 99).astype(np.int64)
    table = np.zeros((10, 10))
    src = (np.arange(n) * 10) // n
    dst = (p * 10) // n
    np.add.at(table, (src, dst), 1)
    expected = n / 100
    chi2 = ((table - expected) ** 2 / expected).sum()
    assert chi2 < 160        # 81 degrees of freedom; 160 is far in the tail (p < 1e-6)
    d = np.diff(p).astype(np.float64)
    # for a random permutation |p[i+1] - p[i]| averages n / 3
    assert abs(np.abs(d).mean() / n - 1 / 3) < 0.005
    r = np.corrcoef(p[:-1], p[1:])[0, 1]
    assert abs(r) < 0.005
