"""fv_inverse_frequency_static, the entry point that allocates nothing (its counters live in an array
built into the library), against fv_inverse_frequency, the entry point it is a variant of: bit for bit,
on two calls in a row, the second on a smaller corpus and a smaller vocabulary -- whatever the first
call left in the shared array must not reach the second result."""
import ctypes as C

import numpy as np
import pytest

from flyvec_amd import engine
from flyvec_amd._lib import DeviceBuffer, FlyvecError, FV_ERR_DATA, FV_ERR_INVALID, check, device_memory, load

pytestmark = pytest.mark.gpu

STATIC_MAX_VOCAB = 1 << 20


def static_inverse_frequency(corpus, vocab):
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    d_corpus = DeviceBuffer.from_numpy(corpus) if len(corpus) else None
    d_out = DeviceBuffer(4 * vocab)
    try:
        check(load().fv_inverse_frequency_static(d_corpus.ptr if d_corpus else None, len(corpus), vocab, d_out.ptr))
        return d_out.to_numpy(np.float32, (vocab,))
    finally:
        if d_corpus:
            d_corpus.free()
        d_out.free()


def zipf_corpus(n, vocab, seed, masked):
    rng = np.random.default_rng(seed)
    p = 1.0 / np.arange(1, vocab + 1) ** 1.07
    tokens = rng.choice(vocab, size=n, p=p / p.sum()).astype(np.int32)
    tokens[rng.integers(0, n, masked)] = -1
    return tokens


def test_two_calls_in_a_row_match_the_allocating_entry_point(gpu, oracle_lib):
    big = zipf_corpus(400_000, 30_000, seed=11, masked=500)
    small = zipf_corpus(50_000, 700, seed=12, masked=50)
    for tokens, vocab in ((big, 30_000), (small, 700)):
        got = static_inverse_frequency(tokens, vocab)
        want = engine.inverse_frequency(tokens, vocab)
        assert got.dtype == np.float32 and np.array_equal(got, want)
        assert np.array_equal(got, oracle_lib.inverse_frequency(tokens, vocab))
    # the small vocabulary's ids were the big corpus's most frequent ones: stale counters would show
    assert static_inverse_frequency(small, 700).max() <= 1.0


def test_the_call_leaves_the_device_memory_as_it_found_it(gpu):
    """Free device memory, as the runtime reports it, is the same before and after the call (its buffers are the
    caller's, allocated before the first reading; the first call on a device has already happened above or happens
    in the warm-up here, so that the library's code object and its array are resident)."""
    tokens = zipf_corpus(300_000, 5_000, seed=13, masked=100)
    d_corpus, d_out = DeviceBuffer.from_numpy(tokens), DeviceBuffer(4 * 5_000)
    try:
        check(load().fv_inverse_frequency_static(d_corpus.ptr, len(tokens), 5_000, d_out.ptr))   # warm-up
        before = device_memory()[0]
        for _ in range(3):
            check(load().fv_inverse_frequency_static(d_corpus.ptr, len(tokens), 5_000, d_out.ptr))
            assert device_memory()[0] == before
        assert np.array_equal(d_out.to_numpy(np.float32, (5_000,)), engine.inverse_frequency(tokens, 5_000))
    finally:
        d_corpus.free()
        d_out.free()


def test_empty_corpus_and_absent_ids(gpu):
    assert np.array_equal(static_inverse_frequency(np.zeros(0, np.int32), 17), np.zeros(17, np.float32))
    got = static_inverse_frequency(np.array([3, 3, -1, 5], np.int32), 8)
    assert np.array_equal(got, np.array([0, 0, 0, 0.5, 0, 1, 0, 0], np.float32))


def test_limits_are_refused_with_a_message(gpu):
    lib = load()
    out = DeviceBuffer(16)
    try:
        assert lib.fv_inverse_frequency_static(None, 0, STATIC_MAX_VOCAB + 1, out.ptr) == FV_ERR_INVALID
        assert b"at most" in lib.fv_last_error()
        assert lib.fv_inverse_frequency_static(None, 0, 0, out.ptr) == FV_ERR_INVALID
        assert lib.fv_inverse_frequency_static(None, 5, 4, out.ptr) == FV_ERR_INVALID
        assert lib.fv_inverse_frequency_static(None, 0, 4, None) == FV_ERR_INVALID
    finally:
        out.free()
    with pytest.raises(FlyvecError) as e:
        static_inverse_frequency(np.array([1, 9, 2], np.int32), 4)
    assert e.value.code == FV_ERR_DATA
    # the largest vocabulary the array serves
    tokens = np.array([0, STATIC_MAX_VOCAB - 1, STATIC_MAX_VOCAB - 1], np.int32)
    got = static_inverse_frequency(tokens, STATIC_MAX_VOCAB)
    assert got[0] == 1.0 and got[-1] == 0.5 and np.count_nonzero(got) == 2
