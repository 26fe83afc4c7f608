"""Device half of flyvec_amd/corpus.py: stop-word masking (flyvec/src/remove_words.cpp:28-37) against
numpy, and the encoder's shards carried through merge -> flyvec_train."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu


def test_mask_tokens_equals_numpy(gpu):
    from flyvec_amd import corpus
    rng = np.random.default_rng(0)
    V = 5000
    tokens = rng.integers(-1, V, size=300_001).astype(np.int32)
    remove = rng.choice(V, size=419, replace=False).astype(np.int32)   # the reference's list has 419 ids
    want = tokens.copy()
    want[np.isin(want, remove)] = -1
    got = corpus.mask_tokens(tokens.copy(), remove, vocab=V)
    assert np.array_equal(got, want)
    assert np.array_equal(corpus.mask_tokens(got.copy(), remove, vocab=V), want)          # idempotent
    assert np.array_equal(corpus.mask_tokens(tokens.copy(), np.zeros(0, np.int32), vocab=V), tokens)
    assert np.array_equal(corpus.mask_tokens(tokens.copy(), np.repeat(remove[:3], 5), vocab=V),
                          np.where(np.isin(tokens, remove[:3]), -1, tokens))               # duplicates in the list


def test_mask_tokens_errors(gpu):
    from flyvec_amd import _lib, corpus
    tokens = np.arange(10, dtype=np.int32)
    with pytest.raises(_lib.FlyvecError) as e:
        corpus.mask_tokens(tokens, np.array([3, 99], dtype=np.int32), vocab=10)
    assert e.value.code == _lib.FV_ERR_DATA
    with pytest.raises(ValueError):
        corpus.mask_tokens(tokens.astype(np.int64), [1])


def test_shards_to_checkpoint(gpu, tmp_path):
    from flyvec_amd import corpus
    from flyvec_amd.train_flyvec import main as train_main
    rng = np.random.default_rng(3)
    V = 200
    shard_dir = tmp_path / "shards"
    shard_dir.mkdir()
    for stem in ("part0", "part1", "part2"):
        lens = rng.integers(5, 40, size=150)
        ids = rng.integers(1, V, size=int(lens.sum())).astype(np.int32)
        ids[-1] = V - 1
        np.save(shard_dir / f"{stem}.npy", ids)
        np.save(shard_dir / f"{stem}_offsets.npy", np.cumsum(lens).astype(np.uint64))   # ends, no leading 0
    stop = np.array([1, 2, 3], dtype=np.int32)
    np.save(tmp_path / "stop.npy", stop)
    corpus.main(["merge", str(shard_dir), "-o", str(tmp_path / "merged"), "--stop-ids", str(tmp_path / "stop.npy")])
    tokens = np.load(tmp_path / "merged" / "encodings.npy")
    offsets = np.load(tmp_path / "merged" / "offsets.npy")
    assert not np.isin(tokens, stop).any() and (tokens == -1).any()
    assert offsets[0] == 0 and offsets[-1] == len(tokens) and len(offsets) == 3 * 150 + 1
    out = tmp_path / "ckpt"
    assert train_main([str(tmp_path / "merged" / "encodings.npy"), str(tmp_path / "merged" / "offsets.npy"),
                       "-o", str(out), "--hid", "32", "-b", "128", "--Nep", "1", "--seed", "0"]) == 0
    (ckpt,) = list(out.iterdir())
    W = np.load(ckpt)
    assert W.shape == (32, 2 * V) and np.isfinite(W).all()
    # masked ids never enter a window: their context and target columns keep their initial spread
    assert np.abs(W[:, stop]).max() < 0.2


def test_prune_windows_equals_the_checker_and_the_reference_tool(gpu, oracle_lib):
    """fv_prune_windows against the CPU restatement, which tests/test_oracle_train.py holds against the
    reference's own prune_input_data; here also directly against that build where it travelled."""
    from flyvec_amd import _lib, corpus
    to = oracle_lib
    rng = np.random.default_rng(0)
    for rows, cols, hi in [(1, 1, 3), (7, 2, 2), (1000, 3, 4), (5000, 11, 8), (300, 16, 5), (257, 64, 30), (4, 11, 1)]:
        data = rng.integers(-1, hi, size=(rows, cols)).astype(np.int32)
        want = to.prune_windows(data)
        got = corpus.prune_windows(data.copy())
        assert np.array_equal(got, want), (rows, cols)
        if to.ref_lib() is not None:
            assert np.array_equal(got, to.ref_prune_windows(data)), (rows, cols)
        assert np.array_equal(corpus.prune_windows(got.copy()), got)          # idempotent
        assert np.array_equal(got[:, cols // 2], data[:, cols // 2])           # the centre is never touched
    empty = np.zeros((0, 11), dtype=np.int32)
    assert corpus.prune_windows(empty).shape == (0, 11)
    with pytest.raises(_lib.FlyvecError) as e:
        corpus.prune_windows(np.zeros((2, 65), dtype=np.int32))
    assert e.value.code == _lib.FV_ERR_INVALID
    with pytest.raises(ValueError):
        corpus.prune_windows(np.zeros((2, 3), dtype=np.int64))


def test_prune_windows_golden_fixture(gpu):
    """The reference's own prune_input_data output (tests/golden/prune_windows.npz) through the C ABI."""
    import os
    from flyvec_amd import corpus
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "prune_windows.npz"))
    for k in range(int(z["n_cases"])):
        assert np.array_equal(corpus.prune_windows(z[f"in_{k}"].copy()), z[f"out_{k}"]), k
