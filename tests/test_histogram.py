"""flyvec_amd/csrc/fv_histogram.h on the host: the token histogram behind 1/frequency counts a corpus of any
length the device can hold. The reference indexes its corpus with uint64_t (flyvec/src/model_arrays.cu:396-424)
and was run on 5,785,895,233 and 8.07 G tokens (flyvec/src/test_inv.cpp:10-11, test_preprocess.cpp:9, 67); the
arithmetic that decides whether such a corpus is counted right -- grid size, what one block's 32-bit LDS counters
can receive, counters in HBM that stop instead of wrapping, the clamp at the fp32 counter's 2^24 -- is evaluated
here without a GPU."""
import ctypes as C
import os
import subprocess

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


@pytest.fixture(scope="module")
def shim(tmp_path_factory):
    out = tmp_path_factory.mktemp("histogram") / "libhistogram.so"
    subprocess.run(["gcc", "-O2", "-shared", "-fPIC", "-I", os.path.join(ROOT, "flyvec_amd", "csrc"),
                    os.path.join(ROOT, "tests", "native", "histogram_shim.c"), "-o", str(out)], check=True)
    lib = C.CDLL(str(out))
    lib.fvt_hist_blocks.restype = C.c_uint32
    lib.fvt_hist_blocks.argtypes = [C.c_uint64]
    lib.fvt_hist_block_tokens.restype = C.c_uint64
    lib.fvt_hist_block_tokens.argtypes = [C.c_uint64, C.c_uint32]
    lib.fvt_hist_saturated_sum.restype = C.c_uint32
    lib.fvt_hist_saturated_sum.argtypes = [C.c_uint32, C.c_uint32]
    lib.fvt_hist_invert.restype = C.c_float
    lib.fvt_hist_invert.argtypes = [C.c_uint32]
    lib.fvt_hist_max_tokens.restype = C.c_uint64
    lib.fvt_hist_thread_span.restype = C.c_uint64
    lib.fvt_hist_thread_span.argtypes = [C.c_uint64, C.c_uint32, C.c_uint32, C.c_uint32, C.c_void_p]
    return lib


CORPORA = [1, 255, 4096, 4097, 10_000_000, 200_000_000, (1 << 32) - 1, 1 << 32, 5_785_895_233, 8_070_000_000,
           72 * (1 << 30), (1 << 42) - 1]


def test_every_token_is_visited_once_with_64_bit_indices(shim):
    out = (C.c_uint64 * 2)()
    for n in CORPORA:
        blocks = shim.fvt_hist_blocks(n)
        assert 1 <= blocks <= 2048
        total, last = 0, -1
        # first and last block in full, a sample of the others: the counts of all threads add up to n
        for b in sorted(set([0, blocks - 1, blocks // 2, blocks // 3])):
            for t in (0, 1, 63, 255):
                c = shim.fvt_hist_thread_span(n, blocks, b, t, out)
                if c:
                    assert out[0] == b * 256 + t and out[1] < n and out[1] + blocks * 256 >= n
                    last = max(last, out[1])
        stride = blocks * 256
        # closed form of the sum over every thread of the launch
        full, rest = divmod(n, stride)
        assert full * stride + rest == n
        per_thread = [full + (1 if i < rest else 0) for i in (0, rest - 1 if rest else 0, rest, stride - 1)]
        for i, want in zip((0, rest - 1 if rest else 0, rest, stride - 1), per_thread):
            c = shim.fvt_hist_thread_span(n, blocks, i // 256, i % 256, out)
            assert c == want, (n, i)


def test_lds_counters_of_a_block_cannot_wrap(shim):
    assert shim.fvt_hist_max_tokens() == 1 << 42
    for n in CORPORA:
        blocks = shim.fvt_hist_blocks(n)
        most = shim.fvt_hist_block_tokens(n, blocks)
        assert most < 1 << 32, n                      # every token of the block could be the same id
        assert most * blocks >= n


def test_counters_in_hbm_stop_instead_of_wrapping(shim):
    rng = np.random.default_rng(0)
    stop = 0x80000000
    for seen, add in [(0, 0), (0, 1), (stop - 1, 1), (stop - 1, 2), (stop, 1), (stop, 0xffffffff), (0xffffffff, 0xffffffff),
                      (123, 0xffffffff), (stop - 5, 4)] + [tuple(int(x) for x in rng.integers(0, 1 << 32, 2)) for _ in range(2000)]:
        got = shim.fvt_hist_saturated_sum(seen, add)
        assert got == min(seen + add, stop) if seen <= stop else got == stop
    # 2048 blocks that have each seen the same id 2^31 times: the sum passes 2^32 many times over, the counter stops
    c = 0
    for _ in range(2048):
        c = shim.fvt_hist_saturated_sum(c, (1 << 31) + 7)
    assert c == stop


def test_result_is_the_fp32_counters(shim):
    """1 / count with the count as a float32 accumulator of += 1.0 would hold it: exact up to 2^24, stuck there."""
    for count in [0, 1, 2, 3, 34, 1000, (1 << 24) - 1, 1 << 24, (1 << 24) + 1, 17_545_497, 1 << 31, 0xffffffff]:
        got = shim.fvt_hist_invert(count)
        if count == 0:
            assert got == 0.0
            continue
        acc = np.float32(min(count, 1 << 24))           # += 1.0 is exact below 2^24 and changes nothing from there on
        assert np.float32(acc + np.float32(1.0)) == acc or count < 1 << 24
        assert got == np.float32(1.0 / np.float64(acc))
