"""flyvec_amd/csrc/fv_layout.h on the host: for every accepted K the farthest element a window gather
reads lies inside the allocation of the token-major matrix.

The gather (fv_gather_batch in fv_internal.h) loads Wt[row * ldk + lane + 64 * j] for all 64 lanes and
j < ceil(K / 64), rows 0 .. N (row N = the zero row a masked position reads). The bound is evaluated
here independently of the header's own arithmetic."""
import ctypes as C
import os
import subprocess

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
FV_MAX_HID = 2048


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("layout") / "liblayout.so"
    subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "flyvec_amd", "csrc"),
                    os.path.join(ROOT, "tests", "native", "layout_shim.c"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.fvt_ldk.restype = C.c_uint32
    lib.fvt_ldk.argtypes = [C.c_uint32]
    for name in ("fvt_alloc_elems", "fvt_gather_reach"):
        getattr(lib, name).restype = C.c_uint64
        getattr(lib, name).argtypes = [C.c_uint32, C.c_uint64]
    lib.fvt_pad_elems.restype = C.c_uint64
    lib.fvt_pad_elems.argtypes = [C.c_uint32]
    return lib


def farthest_read(K, N, ldk):
    """Largest element index the gather touches: last lane, last register, row N."""
    nv = -(-K // 64)
    return max(row * ldk + 63 + 64 * (nv - 1) for row in (0, N - 1, N))


def test_every_accepted_hid_reads_inside_the_allocation(shim):
    for K in range(1, FV_MAX_HID + 1):
        ldk = shim.fvt_ldk(K)
        assert ldk >= K and ldk % 4 == 0 and ldk - K < 4
        for N in (1, 2, 10, 254, 40000, 100000):
            elems = shim.fvt_alloc_elems(K, N)
            assert farthest_read(K, N, ldk) < elems, (K, N)
            assert shim.fvt_gather_reach(K, N) == farthest_read(K, N, ldk) + 1
            assert elems >= (N + 1) * ldk  # the whole zero row is there
            assert elems == N * ldk + shim.fvt_pad_elems(K)


def test_small_hid_needs_more_than_two_pad_rows(shim):
    # two rows behind the matrix cover the overrun only while 64 * ceil(K / 64) <= 2 * ldk
    for K in (1, 2, 3, 5, 28):
        assert shim.fvt_pad_elems(K) == 64 > 2 * shim.fvt_ldk(K)
    for K in (29, 32, 64, 400, 1000, 2048):
        assert shim.fvt_pad_elems(K) == 2 * shim.fvt_ldk(K) >= 64 * -(-K // 64)
    # the case a page-aligned allocation exposes: K = 4, V = 127 (N = 254)
    assert shim.fvt_alloc_elems(4, 254) * 4 > (254 * 4 + 63 + 1) * 4 - 1


def test_slot_records_of_all_blocks_have_places_of_their_own_inside_the_allocation(shim):
    """fv_slot_place: record `number` of block `blk` when every block of the sparse launch has a region of `region`
    records. Every (block, number) gets a place of its own below region * n_blocks, and the first records of all
    blocks lie side by side at the front."""
    shim.fvt_slot_place.restype = C.c_uint64
    shim.fvt_slot_place.argtypes = [C.c_uint32] * 4
    shim.fvt_slot_regions_records.restype = C.c_uint64
    shim.fvt_slot_regions_records.argtypes = [C.c_uint32] * 2
    shim.fvt_slot_primary.restype = C.c_uint32
    primary = shim.fvt_slot_primary()
    for region, n_blocks in ((1, 4), (7, 8), (primary - 1, 12), (primary, 12), (primary + 1, 12), (3 * primary + 5, 20)):
        total = shim.fvt_slot_regions_records(region, n_blocks)
        assert total == region * n_blocks
        seen = set()
        for blk in range(n_blocks):
            for number in range(region):
                place = shim.fvt_slot_place(blk, number, region, n_blocks)
                assert place < total
                seen.add(place)
                if number < min(region, primary):
                    assert place == blk * min(region, primary) + number
        assert len(seen) == total          # no two records share a place
    # the shapes the trainer meets: 1600 blocks of 10000 records, 8192 blocks of 2^23 - 2 (beyond 32 bits)
    assert shim.fvt_slot_place(1599, 9999, 10000, 1600) == 1600 * 10000 - 1
    big = (1 << 23) - 2
    assert shim.fvt_slot_place(8191, big - 1, big, 8192) == 8192 * big - 1
