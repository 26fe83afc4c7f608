"""Pins the window-table and 1/frequency restatements (oracle/flyvec_oracle.c).

fvo_count_windows / fvo_window_starts are checked against the reference's own prune_input.cpp
compiled into oracle/_ref (flyvec/src/prune_input.cpp:64-122) on random and edge-case offsets, and
against hand-computed tables; fvo_inverse_frequency against a numpy bincount and the fp32 counter's
saturation at 2^24 (flyvec/src/model_arrays.cu:396-424)."""
import numpy as np
import pytest

from oracle import train_oracle as to


def offsets_from_lengths(lengths, first=0):
    return np.concatenate([[first], first + np.cumsum(lengths)]).astype(np.uint64)


def test_hand_computed_table():
    # chunks of length 3, 5, 2, 4 with w = 3: windows 1 + 3 + 0 + 2; starts are running sums + i
    off = offsets_from_lengths([3, 5, 2, 4])
    assert to.count_windows(off, 3) == 6
    assert to.window_starts(off, 3).tolist() == [0, 3, 4, 5, 10, 11]


def test_maxlen_cut_and_short_chunks():
    # chunks of 213 tokens are kept, 214 and longer are dropped (MAXLEN = 214, prune_input.cpp:7, 76)
    off = offsets_from_lengths([213, 214, 300, 10, 11])
    w = 11
    assert to.count_windows(off, w) == (213 - w + 1) + 0 + 0 + 0 + 1
    st = to.window_starts(off, w)
    assert st[0] == 0 and st[-1] == 213 + 214 + 300 + 10


def test_offsets_not_starting_at_zero_are_rebased():
    # the reference accumulates lengths from 0 and never reads offsets[s] as a position
    a = to.window_starts(offsets_from_lengths([12, 30, 11]), 11)
    b = to.window_starts(offsets_from_lengths([12, 30, 11], first=1000), 11)
    assert np.array_equal(a, b)


def test_missing_sentinel_drops_last_chunk():
    lengths = [20, 15, 30]
    full = offsets_from_lengths(lengths)
    assert to.count_windows(full[:-1], 11) == to.count_windows(full, 11) - (30 - 11 + 1)


@pytest.mark.skipif(to.ref_lib() is None, reason="oracle/_ref was not built (reference tree absent)")
@pytest.mark.parametrize("seed,w", [(0, 11), (1, 15), (2, 3), (3, 1), (4, 64)])
def test_against_reference_build(seed, w):
    rng = np.random.default_rng(seed)
    lengths = rng.geometric(1 / 25, size=5000)
    lengths[rng.integers(0, 5000, 30)] = rng.integers(200, 400, 30)  # around and above MAXLEN
    lengths[rng.integers(0, 5000, 30)] = 0                           # empty chunks
    off = offsets_from_lengths(lengths, first=int(rng.integers(0, 2)) * 17)
    assert to.count_windows(off, w) == to.ref_count_windows(off, w)
    assert np.array_equal(to.window_starts(off, w), to.ref_window_starts(off, w))


@pytest.mark.skipif(to.ref_lib() is None, reason="oracle/_ref was not built (reference tree absent)")
def test_against_reference_build_edge_cases():
    for lengths in ([], [5], [11], [10], [213], [214], [11] * 7, [0, 0, 12, 0]):
        off = offsets_from_lengths(lengths)
        assert to.count_windows(off, 11) == to.ref_count_windows(off, 11), lengths
        assert np.array_equal(to.window_starts(off, 11), to.ref_window_starts(off, 11)), lengths


def test_golden_fixture_from_reference_build():
    """tests/golden/window_table.npz was written by tests/golden/make_window_table.py from the
    reference's own prune_input.cpp; it travels to machines where the reference is absent."""
    import os
    path = os.path.join(os.path.dirname(__file__), "golden", "window_table.npz")
    z = np.load(path)
    for k in range(int(z["n_cases"])):
        off, w = z[f"offsets_{k}"], int(z[f"w_{k}"])
        assert to.count_windows(off, w) == int(z[f"count_{k}"])
        assert np.array_equal(to.window_starts(off, w), z[f"starts_{k}"])


def test_inverse_frequency_matches_bincount():
    rng = np.random.default_rng(5)
    V = 300
    corpus = rng.integers(-1, V, size=20000).astype(np.int32)
    corpus[corpus == 7] = 8  # id 7 absent -> 0
    got = to.inverse_frequency(corpus, V)
    cnt = np.bincount(corpus[corpus >= 0], minlength=V)
    want = np.where(cnt > 0, (1.0 / np.maximum(cnt, 1).astype(np.float64)).astype(np.float32), 0).astype(np.float32)
    assert np.array_equal(got, want)
    assert got[7] == 0.0


def test_inverse_frequency_saturates_like_an_fp32_counter():
    n = (1 << 24) + 1000
    corpus = np.zeros(n, dtype=np.int32)
    corpus[:5] = 1
    got = to.inverse_frequency(corpus, 2)
    assert got[0] == np.float32(1.0 / float(1 << 24))  # the counter stopped at 2^24
    assert got[1] == np.float32(0.2)
