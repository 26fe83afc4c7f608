"""What the compiler made of the kernels, read from the built library's own metadata (no GPU needed).

A kernel whose arrays or long-lived values end up in scratch memory still computes the right results, only
several times slower (a scratch access is a trip to memory, and a reload waits for every load in flight before
it): the parity tests cannot see that.  The code objects inside libflyvec_hip.so carry, per kernel, the size of
its scratch frame and the registers it spills; this test holds them to what the hot kernels were built with.
"""
import re
import struct

import pytest

msgpack = pytest.importorskip("msgpack")

# kernels allowed a scratch frame: a small evaluation stack by design, and one spilled LDS address on a cold path
ALLOWED_SCRATCH_BYTES = {
    "fv_combine_leaves_kernel": 256,
    "fv_sparse_grouping_kernel": 16,
}
# the launches of a training step and the hashing kernel must fit their blocks' share of the register file
MAX_VGPRS = {
    "fv_dense_onepass_kernel": 128,   # 1024 threads: four waves per SIMD
    "fv_dense_stream_kernel": 128,
    "fv_sparse_grouping_kernel": 80,  # six waves per SIMD
    "fv_gather_winner_kernel": 128,
    "fv_hash_kernel": 128,
}


def _code_objects(blob):
    """The device code objects of every translation unit (clang offload bundles inside the shared library)."""
    for m in re.finditer(b"__CLANG_OFFLOAD_BUNDLE__", blob):
        start = m.start()
        (n_entries,) = struct.unpack_from("<Q", blob, start + 24)
        p = start + 32
        for _ in range(n_entries):
            off, size, triple_len = struct.unpack_from("<QQQ", blob, p)
            p += 24
            triple = blob[p:p + triple_len].decode()
            p += triple_len
            if "amdgcn" in triple and size:
                yield triple, blob[start + off:start + off + size]


def _kernels(elf):
    """amdhsa.kernels of one code object: the msgpack document in its AMDGPU note."""
    assert elf[:4] == b"\x7fELF"
    (shoff,) = struct.unpack_from("<Q", elf, 0x28)
    shentsize, shnum, _ = struct.unpack_from("<HHH", elf, 0x3A)
    found = []
    for i in range(shnum):
        sh = struct.unpack_from("<IIQQQQIIQQ", elf, shoff + i * shentsize)
        if sh[1] != 7:  # SHT_NOTE
            continue
        p, end = sh[4], sh[4] + sh[5]
        while p < end:
            namesz, descsz, typ = struct.unpack_from("<III", elf, p)
            p += 12
            name = elf[p:p + namesz]
            p += (namesz + 3) & ~3
            desc = elf[p:p + descsz]
            p += (descsz + 3) & ~3
            if typ == 32 and name.startswith(b"AMDGPU"):  # NT_AMDGPU_METADATA
                found += msgpack.unpackb(desc, raw=False, strict_map_key=False).get("amdhsa.kernels", [])
    return found


def _plain_name(mangled):
    """fv_x_kernel from _Z<length>fv_x_kernel<template arguments and parameter types>."""
    m = re.match(r"_Z(\d+)", mangled)
    if not m:
        return mangled
    return mangled[m.end():m.end() + int(m.group(1))]


@pytest.fixture(scope="module")
def kernels():
    from flyvec_amd import _lib
    assert _lib.LIB_PATH.exists(), "run `python -m flyvec_amd.build` (or __graft_entry__.build()) first"
    blob = _lib.LIB_PATH.read_bytes()
    out = []
    for triple, elf in _code_objects(blob):
        assert "gfx950" in triple
        out += _kernels(elf)
    assert len(out) > 100, "the library's kernels were not found"
    return out


def test_names_are_read(kernels):
    names = {_plain_name(k[".name"]) for k in kernels}
    for must in list(MAX_VGPRS) + ["fv_sparse_kernel", "fv_group_kernel", "fv_slot_update_kernel"]:
        assert must in names, f"{must} not among {sorted(names)[:8]} ..."


def test_no_kernel_keeps_arrays_in_scratch_memory(kernels):
    over = []
    for k in kernels:
        name = _plain_name(k[".name"])
        if k[".private_segment_fixed_size"] > ALLOWED_SCRATCH_BYTES.get(name, 0):
            over.append((k[".name"], k[".private_segment_fixed_size"], k[".vgpr_spill_count"]))
    assert not over, f"kernels with a scratch frame (name, bytes, spilled registers): {over}"


def test_hot_kernels_fit_their_register_budget(kernels):
    for k in kernels:
        limit = MAX_VGPRS.get(_plain_name(k[".name"]))
        if limit is not None:
            assert k[".vgpr_count"] <= limit, (k[".name"], k[".vgpr_count"])
