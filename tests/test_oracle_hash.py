"""Pins the numpy restatement of the hashing rule (oracle/hash_oracle.py; flyvec/core.py:23-36, 153-158).

The reference's own golden values need its downloaded model, which is not available, so they pin
only shape, dtype and popcount (README.md:41-61: 400 long, int8, exactly 50 ones for k = 50).  The
restatement is therefore checked against a sort-free definition by brute force, the invariants of a
threshold code, hand-made ties and adjacent floats, and numpy itself for the normalisation sums."""
import numpy as np
import pytest

from oracle import hash_oracle as ho

f32 = np.float32


def brute_code(act, k):
    """Definition without sorting: a_k = the value with at least k elements >= it and fewer than k
    elements > it (k-th largest with multiplicity); same for k+1."""
    def kth(j):
        for x in act:
            if (act >= x).sum() >= j and (act > x).sum() < j:
                return x
        raise AssertionError
    thr = f32(f32(kth(k) + kth(k + 1)) / f32(2))
    return np.array([1 if x > thr else 0 for x in act], dtype=np.int8)


@pytest.mark.parametrize("seed", range(6))
def test_sparse_code_against_brute_force(seed):
    rng = np.random.default_rng(seed)
    for K in (2, 3, 5, 8):
        for _ in range(20):
            act = rng.integers(-3, 4, size=K).astype(f32) if seed % 2 else rng.standard_normal(K).astype(f32)
            for k in range(1, K):
                want = brute_code(act, k)
                assert np.array_equal(ho.sparse_code(act, k), want)
                assert np.array_equal(ho.threshold_codes(act[None, :], k)[0], want)


def test_shape_dtype_popcount_of_the_reference_readme():
    # README.md:41-61 prints a 400-long int8 vector with exactly 50 ones for the default k = 50
    rng = np.random.default_rng(0)
    code = ho.sparse_code(rng.standard_normal(400).astype(f32), 50)
    assert code.shape == (400,) and code.dtype == np.int8 and code.sum() == 50
    assert ho.sparse_code(rng.standard_normal(400).astype(f32), 4).sum() == 4  # README.md:69-75


def test_threshold_semantics_on_ties_and_adjacent_floats():
    act = np.array([5, 4, 4, 4, 1], dtype=f32)
    assert ho.sparse_code(act, 2).tolist() == [1, 0, 0, 0, 0]      # tie at the k / k+1 boundary: 1 bit, not 2
    assert ho.sparse_code(act, 1).tolist() == [1, 0, 0, 0, 0]
    assert ho.sparse_code(act, 4).tolist() == [1, 1, 1, 1, 0]
    assert ho.sparse_code(np.full(6, 2.5, dtype=f32), 3).sum() == 0  # all equal: empty code
    a = f32(1.0)
    b = np.nextafter(a, f32(2.0))                                     # adjacent floats: fl32(a+b)/2 rounds to even
    code = ho.sparse_code(np.array([b, a, 0], dtype=f32), 1)
    thr = f32(f32(a + b) / f32(2))
    assert code.tolist() == [int(b > thr), int(a > thr), 0]
    with pytest.raises(IndexError):
        ho.sparse_code(np.arange(4, dtype=f32), 4)                    # k >= K reads act_sort[k]
    with pytest.raises(IndexError):
        ho.threshold_codes(np.zeros((1, 4), dtype=f32), 4)


def test_invariants():
    rng = np.random.default_rng(3)
    act = rng.standard_normal((64, 100)).astype(f32)
    prev = np.zeros_like(act, dtype=np.int8)
    for k in (1, 5, 20, 50, 99):
        code = ho.threshold_codes(act, k)
        assert (code.sum(axis=1) == k).all()                          # no ties in random data
        assert (code >= prev).all()                                   # codes nest as k grows
        order = np.argsort(-act, axis=1)
        assert all(set(np.flatnonzero(code[r])) == set(order[r, :k]) for r in range(len(act)))
        prev = code


def test_batch_forms_agree_with_the_per_word_loop():
    rng = np.random.default_rng(4)
    K, V = 64, 50
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    ids = rng.integers(1, V, size=40)
    loop = ho.hash_targets_loop(W, ids, 10)
    assert np.array_equal(ho.hash_targets(W, ids, 10), loop)
    assert np.array_equal(ho.hash_windows(W, (V + ids)[:, None].astype(np.int32), 10), loop)  # w = 1


def test_window_sum_is_sequential_fp32_in_window_order():
    rng = np.random.default_rng(5)
    K, V, w = 16, 20, 6
    W = (rng.standard_normal((K, 2 * V)) * 10.0 ** rng.integers(-3, 4, size=(K, 2 * V))).astype(f32)
    idx = rng.integers(0, 2 * V, size=(30, w)).astype(np.int32)
    idx[rng.random(idx.shape) < 0.2] = -1
    act = ho.window_activations(W, idx)
    for r in range(len(idx)):
        for h in range(K):
            s = f32(0)
            for c in range(w):
                if idx[r, c] >= 0:
                    s = f32(s + W[h, idx[r, c]])
            assert act[r, h] == s


def test_pack_unpack():
    rng = np.random.default_rng(6)
    for K in (1, 63, 64, 65, 400):
        codes = (rng.random((10, K)) < 0.3).astype(np.int8)
        words = ho.pack_codes(codes)
        assert words.shape == (10, (K + 63) // 64) and words.dtype == np.uint64
        for r in range(10):
            for h in np.flatnonzero(codes[r]):
                assert (int(words[r, int(h) >> 6]) >> (int(h) & 63)) & 1
        assert np.array_equal(ho.unpack_codes(words, K), codes)
        assert int(sum(bin(int(x)).count("1") for x in words.ravel())) == int(codes.sum())


def test_numpy_buffer_size_is_the_default():
    assert np.getbufsize() == ho.NUMPY_BUFSIZE


@pytest.mark.parametrize("n", [1, 7, 8, 9, 127, 128, 129, 255, 256, 1000, 4096, 8192, 8193, 16384, 40000, 100001])
def test_row_sum_restatement_against_numpy_sum(n):
    rng = np.random.default_rng(n)
    a = (rng.standard_normal((4, n)) * 10.0 ** rng.integers(-2, 3, size=(4, n))).astype(f32)
    sq = a ** 2
    want = np.sum(sq, axis=1)                                        # what normalize_synapses calls
    got = np.array([ho.numpy_row_sum_f32(row) for row in sq], dtype=f32)
    assert np.array_equal(got, want)


def test_normalize_synapses_statement():
    rng = np.random.default_rng(8)
    syn = rng.standard_normal((5, 300)).astype(f32)
    out = ho.normalize_synapses(syn)
    assert out.dtype == f32
    assert np.allclose(np.sqrt((out.astype(np.float64) ** 2).sum(axis=1)), 1.0, atol=1e-6)
    assert np.array_equal(np.power(np.sum(syn ** 2, axis=1), 1 / 2), np.sqrt(np.sum(syn ** 2, axis=1)))
