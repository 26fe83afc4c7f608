"""Parity of the HIP hashing path against the numpy restatement of flyvec/core.py:153-158,
through the C ABI.  Codes are compared bit for bit."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

f32 = np.float32


def test_config1_target_ids(gpu):
    """K = 400, V = 20000, 4096 Zipf target ids, k = 50, int8 codes (the reference's per-word path)."""
    from flyvec_amd import Hasher, synthetic
    from oracle import hash_oracle as ho
    W = synthetic.synapses(400, 20000, seed=1)
    ids = synthetic.zipf_ids(4096, 20000, seed=2)
    h = Hasher(W)
    got = h.hash_targets(ids, 50)
    assert got.dtype == np.int8 and got.shape == (4096, 400)
    assert np.array_equal(got, ho.hash_targets_loop(W, ids, 50))
    assert (got.sum(axis=1) == 50).all()
    h.close()


def test_config3_window_batch(gpu):
    """K = 400, V = 20000, 1,048,576 windows of w = 11, k = 32, 7 packed words per window: every window of the
    batch is compared with the numpy oracle bit for bit (the oracle's chunks are dealt over a few threads; numpy
    releases the interpreter lock inside its loops)."""
    from concurrent.futures import ThreadPoolExecutor
    from flyvec_amd import Hasher, synthetic
    from oracle import hash_oracle as ho
    K, V, w, k, n = 400, 20000, 11, 32, 1 << 20
    W = synthetic.synapses(K, V, seed=1)
    idx = synthetic.window_indices(n, w, V, seed=7)
    h = Hasher(W)
    bits = h.hash_windows(idx, k, packed=True)
    assert bits.shape == (n, 7) and bits.dtype == np.uint64
    part = 1 << 15
    with ThreadPoolExecutor(max_workers=8) as pool:
        want = list(pool.map(lambda s: ho.pack_codes(ho.hash_windows(W, idx[s:s + part], k)), range(0, n, part)))
    want = np.concatenate(want)
    assert want.shape == bits.shape
    assert np.array_equal(bits, want)
    pop = np.unpackbits(bits.view(np.uint8), axis=1).sum(axis=1)
    assert pop.max() <= k and (pop == k).mean() > 0.999          # exactly k bits unless fp32 ties
    assert not (bits[:, 6] >> np.uint64(16)).any()                  # no bit beyond neuron 399
    sub = slice(n - 50000, n)
    b2, c2 = h.hash_windows(idx[sub], k, packed=True, codes=True)
    assert np.array_equal(b2, bits[sub]) and np.array_equal(ho.pack_codes(c2), b2)
    h.close()


@pytest.mark.parametrize("K,V,w,k", [(2, 10, 1, 1), (5, 20, 3, 2), (63, 50, 11, 10), (64, 50, 11, 63), (65, 50, 5, 1),
                                     (130, 40, 64, 50), (400, 300, 15, 399), (1000, 200, 15, 32), (2048, 30, 7, 100)])
def test_shapes(gpu, K, V, w, k):
    from flyvec_amd import Hasher
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(K + w)
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, 2 * V, size=(700, w)).astype(np.int32)
    idx[rng.random(idx.shape) < 0.1] = -1
    idx[3] = -1                                                     # a fully masked window: all activations 0
    h = Hasher(W)
    bits, codes = h.hash_windows(idx, k, packed=True, codes=True)
    want = ho.hash_windows(W, idx, k)
    assert np.array_equal(codes, want)
    assert np.array_equal(bits, ho.pack_codes(want))
    assert codes[3].sum() == 0
    h.close()


def test_ties_adjacent_floats_and_equal_activations(gpu):
    from flyvec_amd import Hasher
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(3)
    K, V = 100, 40
    W = rng.integers(-2, 3, size=(K, 2 * V)).astype(f32)           # coarse grid: ties at the k / k+1 boundary
    W[:, 5] = 1.0
    W[: K // 2, 5] = np.nextafter(f32(1.0), f32(2.0))               # two adjacent floats only
    W[:, 6] = 0.25                                                  # all equal
    idx = rng.integers(0, 2 * V, size=(2000, 3)).astype(np.int32)
    idx[0] = [5, -1, -1]
    idx[1] = [6, -1, -1]
    h = Hasher(W)
    for k in (1, 7, 50, 99):
        codes = h.hash_windows(idx, k, packed=False, codes=True)
        want = ho.hash_windows(W, idx, k)
        assert np.array_equal(codes, want)
        assert (codes.sum(axis=1) <= k).all() and (codes.sum(axis=1) < k).any()
        assert codes[1].sum() == 0
    h.close()


def test_argument_and_data_errors(gpu):
    from flyvec_amd import Hasher, _lib
    rng = np.random.default_rng(4)
    K, V = 16, 10
    h = Hasher(rng.standard_normal((K, 2 * V)).astype(f32))
    with pytest.raises(IndexError):
        h.hash_targets([1, 2], K)                                   # the reference reads act_sort[k]
    with pytest.raises(IndexError):
        h.hash_targets([1, 2], 0)
    with pytest.raises(_lib.FlyvecError) as e:
        h.hash_targets([1, V], 4)
    assert e.value.code == _lib.FV_ERR_DATA
    with pytest.raises(_lib.FlyvecError) as e:
        h.hash_windows(np.array([[0, 2 * V, 1]], dtype=np.int32), 4)
    assert e.value.code == _lib.FV_ERR_DATA
    assert h.hash_windows(np.array([[0, 1, 2]], dtype=np.int32), 4).shape == (1, 1)   # still usable
    assert h.hash_targets(np.array([], dtype=np.int32), 4).shape == (0, K)            # empty batch
    assert np.array_equal(h.weights(), h.weights())
    h.close()


def test_normalize_matches_numpy(gpu):
    from flyvec_amd import Hasher
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(5)
    for K, N in ((400, 40000), (37, 2 * 4097), (8, 6), (64, 2 * 8192)):
        W = (rng.standard_normal((K, N)) * 10.0 ** rng.integers(-2, 2, size=(K, 1))).astype(f32)
        h = Hasher(W)
        assert np.array_equal(h.weights(), W)
        h.normalize()
        assert np.array_equal(h.weights(), ho.normalize_synapses(W)), (K, N)
        h.close()


@pytest.mark.parametrize("p", [1, 2, 3, 4, 7])
def test_normalize_with_another_exponent(gpu, p):
    """flyvec/core.py:23 takes the exponent of the norm. p = 1 and p = 2 are numpy's fast paths (the value, the
    fp32 product) and the device restates them exactly; from p = 3 on numpy's float32 power is the C library's
    powf, whose last bit is not pinned by anything the reference holds (parity unpinned for that case): the device
    takes the product in double, rounded once, and the normalised matrix agrees to rounding."""
    from flyvec_amd import Hasher
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(50 + p)
    for K, N in ((37, 2 * 4097), (400, 2000)):
        W = (rng.standard_normal((K, N)) * 10.0 ** rng.integers(-1, 2, size=(K, 1))).astype(f32)
        if p % 2:
            W = np.abs(W)                     # an odd power of a mixed-sign row sums to anything, its root to NaN
        h = Hasher(W)
        h.normalize(p=p)
        got, want = h.weights(), ho.normalize_synapses(W, p=p)
        assert np.isfinite(want).all()
        if p <= 2:
            assert np.array_equal(got, want), (K, N)
        else:
            assert np.allclose(got, want, rtol=2e-6, atol=0.0), (K, N)
        h.close()
    h = Hasher(W)
    for bad in (0, -2, 1.5, 65):
        with pytest.raises(ValueError):
            h.normalize(p=bad)
    h.close()


def test_code_table_serves_the_per_word_calls(gpu):
    """FlyVec.get_sparse_embedding reads a table of the whole vocabulary's codes, computed on the device by one
    batched launch per hash length: its rows equal the launches per id and the numpy oracle's per-word path
    (flyvec/core.py:153-158) bit for bit, and it is computed again when the resident matrix changes."""
    from flyvec_amd import FlyVec
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(12)
    K, V = 400, 700
    vocab = ["<UNK>"] + [f"t{i}" for i in range(1, V)]
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    model = FlyVec(W, tokenizer=vocab, normalize_synapses=False)
    for k in (50, 32, 1, 399):
        table = model.code_table(k)
        assert table.shape == (V, K) and table.dtype == np.int8 and not table.flags.writeable
        assert model.code_table(k) is table                                    # kept, not computed again
        assert np.array_equal(table, ho.hash_targets_loop(W, np.arange(V), k))
        for i in (1, 2, 17, V - 1):
            one = model.hasher.hash_targets([i], k)[0]                         # a launch of its own
            emb = model.get_sparse_embedding(f"t{i}", k)
            assert emb["id"] == i and emb["token"] == f"t{i}" and emb["embedding"].flags.writeable
            assert np.array_equal(emb["embedding"], one) and np.array_equal(one, table[i])
            assert np.array_equal(model.get_sparse_embedding(i, k)["embedding"], one)   # by id
    with pytest.raises(IndexError):
        model.code_table(K)                                                    # the reference reads act_sort[k]
    with pytest.raises(IndexError):
        model.get_sparse_embedding(V, 50)
    assert len(model._code_tables) <= FlyVec.CODE_TABLES_KEPT
    # a change of the resident matrix makes the tables stale
    before = model.code_table(50)
    model.hasher.normalize()
    Wn = ho.normalize_synapses(W)
    after = model.code_table(50)
    assert after is not before and np.array_equal(after, ho.hash_targets_loop(Wn, np.arange(V), 50))
    assert np.array_equal(model.synapses, Wn)
    assert np.array_equal(model.get_sparse_embedding("t5")["embedding"], ho.sparse_code(Wn[:, V + 5], 50))


def test_flyvec_wrapper_semantics(gpu, tmp_path):
    """The behaviours the reference's notebook asserts (nbs/00_core.ipynb:333-350) on a synthetic model."""
    from flyvec_amd import FlyVec
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(6)
    vocab = ["<UNK>", "hello", "world", "market", "fly"] + [f"tok{i}" for i in range(95)]
    K, V = 400, len(vocab)
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    path = tmp_path / "model.npy"
    np.save(path, W)
    (tmp_path / "config.yaml").write_text("synapses: model.npy\nnormalize_synapses: true\ntokenizer: tok.pkl\n")
    model = FlyVec.from_config(tmp_path / "config.yaml", tokenizer=vocab)
    Wn = ho.normalize_synapses(W)
    emb = model.get_sparse_embedding("market")
    assert emb["token"] == "market" and emb["id"] == 3
    assert emb["embedding"].dtype == np.int8 and emb["embedding"].shape == (400,) and emb["embedding"].sum() == 50
    assert np.array_equal(emb["embedding"], ho.sparse_code(Wn[:, V + 3], 50))
    assert np.array_equal(model.get_sparse_embedding("hello world")["embedding"],
                          model.get_sparse_embedding("hello")["embedding"])              # first token only
    assert np.array_equal(model.get_sparse_embedding("HeLLo")["embedding"],
                          model.get_sparse_embedding("hello")["embedding"])              # case-insensitive
    assert model.get_sparse_embedding("market", 4)["embedding"].sum() == 4
    unk = model.get_sparse_embedding("DefNotAWord")
    assert unk["id"] == 0 and unk["token"] == "<UNK>" and not unk["embedding"].any()
    assert unk["embedding"].dtype == np.uint8
    with pytest.raises(ValueError, match="empty string"):
        model.get_sparse_embedding("")
    assert np.array_equal(model.get_dense_embedding("fly")["embedding"], Wn[:, V + 4])
    vecs = model.simple_word_vectors(k=20)
    assert set(vecs) == set(vocab) and all(v.shape == (400,) for v in vecs.values())
    assert np.array_equal(vecs["world"], ho.sparse_code(Wn[:, V + 2], 20)) and not vecs["<UNK>"].any()
    win = np.array([[1, 2, V + 3, 4, -1]], dtype=np.int32)
    assert np.array_equal(model.get_context_embeddings(win, 30), ho.hash_windows(Wn, win, 30))


def test_flyvec_wrapper_stop_words_and_export(gpu, tmp_path):
    """stop_word_ids / stop_words are attributes as in the reference (flyvec/core.py:109-117);
    exclude_stop_words drops them from the whole-vocabulary table; the table exports as JSON."""
    import json
    from flyvec_amd import FlyVec
    from oracle import hash_oracle as ho
    rng = np.random.default_rng(9)
    vocab = ["<UNK>", "the", "of", "fly", "brain"] + [f"tok{i}" for i in range(45)]
    K, V = 128, len(vocab)
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    np.save(tmp_path / "model.npy", W)
    np.save(tmp_path / "stop.npy", np.array([1, 2], dtype=np.int64))
    (tmp_path / "config.yaml").write_text("synapses: model.npy\nstop_words: stop.npy\ntokenizer: tok.pkl\n")
    model = FlyVec.from_config(tmp_path / "config.yaml", tokenizer=vocab)       # normalize_synapses defaults to False
    assert model.stop_word_ids == {1, 2} and model.stop_words == {"the", "of"}
    assert model.vocab == vocab and model.n_vocab == V and model.n_neurons == K
    assert np.array_equal(model.synapses, W)
    kept = model.simple_word_vectors(k=10, exclude_stop_words=True)
    assert set(kept) == set(vocab) - {"the", "of"}
    n = model.export_simple_embeddings(tmp_path / "simple.json", k=10)
    table = json.loads((tmp_path / "simple.json").read_text())
    assert n == V and set(table) == set(vocab)
    assert table["brain"] == ho.sparse_code(W[:, V + 4], 10).astype(int).tolist() and sum(table["brain"]) == 10
    with pytest.raises(NotImplementedError):
        FlyVec.load()


def test_host_batches_in_chunks_on_two_streams(gpu):
    """Host-buffer batches larger than one chunk (131072 windows) alternate between two streams: ragged sizes
    around the chunk boundaries, pageable and page-locked buffers, both outputs, the device-resident entry point
    as the reference, and an index out of range in a late chunk."""
    from flyvec_amd import Hasher, _lib, synthetic
    from flyvec_amd._lib import DeviceBuffer
    from oracle import hash_oracle as ho
    K, V, w, k = 200, 3000, 7, 24
    W = synthetic.synapses(K, V, seed=3)
    h = Hasher(W)
    chunk = 1 << 17
    for n in (chunk - 1, chunk, chunk + 1, 2 * chunk + 77, 3 * chunk + 5):
        idx = synthetic.window_indices(n, w, V, seed=n % 97)
        idx[::1001, 2] = -1
        bits, codes = h.hash_windows(idx, k, packed=True, codes=True)
        d_idx, d_bits = DeviceBuffer.from_numpy(idx), DeviceBuffer(n * h.words * 8)
        h.hash_windows_dev(d_idx, n, w, k, bits_buf=d_bits)
        h.sync()
        assert np.array_equal(bits, d_bits.to_numpy(np.uint64, (n, h.words)))
        assert np.array_equal(ho.pack_codes(codes), bits)
        for sl in (slice(0, 3000), slice(chunk - 1500, chunk + 1500), slice(n - 3000, n)):
            assert np.array_equal(codes[sl], ho.hash_windows(W, idx[sl], k))
        d_idx.free()
        d_bits.free()
    # page-locked buffers in and out
    n = 2 * chunk + 9
    idx = synthetic.window_indices(n, w, V, seed=5)
    pin_idx = _lib.pinned_empty(idx.shape, np.int32)
    pin_idx[:] = idx
    pin_bits = _lib.pinned_empty((n, h.words), np.uint64)
    pin_bits[:] = 0
    out = h.hash_windows(pin_idx, k, out_bits=pin_bits)
    assert out is pin_bits and np.array_equal(pin_bits, h.hash_windows(idx, k))
    # a smaller batch afterwards (the lanes' buffers are kept), and target ids beyond one chunk
    assert np.array_equal(h.hash_windows(idx[:1000], k), pin_bits[:1000])
    ids = synthetic.zipf_ids(chunk + 300, V, seed=8)
    got = h.hash_targets(ids, k)
    assert np.array_equal(got[-500:], ho.hash_targets_loop(W, ids[-500:], k))
    # an index out of range in the last chunk is reported, the call returns, the hasher stays usable
    bad = idx.copy()
    bad[n - 3, 1] = 2 * V
    with pytest.raises(_lib.FlyvecError) as e:
        h.hash_windows(bad, k)
    assert e.value.code == _lib.FV_ERR_DATA
    assert np.array_equal(h.hash_windows(idx[:1000], k), pin_bits[:1000])
    h.close()
