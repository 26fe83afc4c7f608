"""The device-side window table and 1/frequency against the checker and the golden fixture."""
import os

import numpy as np
import pytest

from conftest import small_corpus

pytestmark = pytest.mark.gpu


def offsets_from_lengths(lengths, first=0):
    return np.concatenate([[first], first + np.cumsum(lengths)]).astype(np.uint64)


def test_golden_window_tables(gpu):
    from flyvec_amd import count_windows, window_starts
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "window_table.npz"))
    for k in range(int(z["n_cases"])):
        off, w = z[f"offsets_{k}"], int(z[f"w_{k}"])
        assert count_windows(off, w) == int(z[f"count_{k}"])
        assert np.array_equal(window_starts(off, w), z[f"starts_{k}"])


@pytest.mark.parametrize("seed,w,n_chunks", [(0, 11, 5000), (1, 15, 70000), (2, 1, 3000), (3, 64, 9000), (4, 3, 1)])
def test_window_table_against_checker(gpu, oracle_lib, seed, w, n_chunks):
    from flyvec_amd import count_windows, window_starts
    rng = np.random.default_rng(seed)
    lengths = rng.geometric(1 / 25, size=n_chunks)
    lengths[rng.integers(0, n_chunks, max(1, n_chunks // 100))] = rng.integers(200, 400)
    lengths[rng.integers(0, n_chunks, max(1, n_chunks // 100))] = 0
    off = offsets_from_lengths(lengths, first=int(seed % 2) * 9)
    assert count_windows(off, w) == oracle_lib.count_windows(off, w)
    assert np.array_equal(window_starts(off, w), oracle_lib.window_starts(off, w))


def test_empty_and_degenerate_offsets(gpu):
    from flyvec_amd import count_windows, window_starts
    assert count_windows(np.array([0], dtype=np.uint64), 11) == 0
    assert count_windows(np.array([], dtype=np.uint64), 11) == 0
    assert window_starts(np.array([0, 5], dtype=np.uint64), 11).size == 0
    assert window_starts(np.array([0, 11], dtype=np.uint64), 11).tolist() == [0]


def test_inverse_frequency(gpu, oracle_lib):
    from flyvec_amd import inverse_frequency
    rng = np.random.default_rng(5)
    for V in (7, 300, 20000):
        corpus = rng.integers(-1, V, size=200000).astype(np.int32)
        corpus[corpus == 3] = 4        # an absent id
        assert np.array_equal(inverse_frequency(corpus, V), oracle_lib.inverse_frequency(corpus, V))


def test_inverse_frequency_saturation(gpu, oracle_lib):
    from flyvec_amd import inverse_frequency
    n = (1 << 24) + 5000               # the reference's fp32 counter stops at 2^24
    corpus = np.zeros(n, dtype=np.int32)
    corpus[:7] = 1
    got = inverse_frequency(corpus, 2)
    assert got[0] == np.float32(1.0 / float(1 << 24)) and got[1] == np.float32(1.0 / 7.0)


def test_inverse_frequency_in_the_form_whose_counters_stop(gpu, oracle_lib):
    """A corpus of 2^31 tokens or more is counted by a kernel whose counters in HBM stop instead of wrapping; the test
    hook sends a small corpus through it: same result as the plain form and as the oracle, ids above and below
    the part of the vocabulary a block counts in LDS."""
    from flyvec_amd import inverse_frequency, _lib
    lib = _lib.load()
    V = 30000
    rng = np.random.default_rng(11)
    corpus = np.minimum(rng.zipf(1.2, size=1_500_000) - 1, V - 1).astype(np.int32)
    corpus[::7] = V - 1 - (np.arange(len(corpus[::7])) % 9000).astype(np.int32)   # counted in HBM directly
    corpus[5::1001] = -1
    plain = inverse_frequency(corpus, V)
    try:
        assert lib.fv_histogram_stops_from(1) == 0
        stops = inverse_frequency(corpus, V)
    finally:
        assert lib.fv_histogram_stops_from(0) == 0
    want = oracle_lib.inverse_frequency(corpus, V)
    assert np.array_equal(plain, want) and np.array_equal(stops, want)


def test_trainer_tables_match_the_standalone_functions(gpu, oracle_lib):
    from flyvec_amd import Trainer
    V = 300
    tokens, offsets = small_corpus(50000, V)
    t = Trainer(V, 32, 11, 64)
    t.set_corpus(tokens, offsets)
    assert np.array_equal(t.window_starts(), oracle_lib.window_starts(offsets, 11))
    assert np.array_equal(t.inverse_frequency(), oracle_lib.inverse_frequency(tokens, V))
    assert np.array_equal(t.get_permutation(), np.arange(t.num_windows, dtype=np.uint64))
    t.close()
