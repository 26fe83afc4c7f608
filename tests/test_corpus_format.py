"""Host half of flyvec_amd/corpus.py: the encoder's shard format (sentence ends per shard,
flyvec/tokenizer.py:199-227) turned into the trainer's (chunk starts with a leading 0 and the
closing sentinel, flyvec/train_flyvec.py:172-173)."""
import numpy as np
import pytest

from flyvec_amd import corpus
from oracle import train_oracle as to


def encoder_like(rng, n_sent, vocab):
    """What encode_sentences_from_fname returns for a shard: ids, cumulative sentence ends."""
    lens = rng.integers(0, 30, size=n_sent)
    ids = rng.integers(0, vocab, size=int(lens.sum())).astype(np.int32)
    return ids, np.cumsum(lens).astype(np.uint64)


def test_ends_to_offsets():
    off = corpus.chunk_ends_to_offsets(np.array([3, 7, 7, 12], dtype=np.uint64))
    assert off.dtype == np.uint64 and off.tolist() == [0, 3, 7, 7, 12]           # last end is the sentinel
    assert corpus.chunk_ends_to_offsets([3, 7], n_tokens=9).tolist() == [0, 3, 7, 9]   # trailing tokens: one more chunk
    assert corpus.chunk_ends_to_offsets([], n_tokens=0).tolist() == [0, 0]
    with pytest.raises(ValueError):
        corpus.chunk_ends_to_offsets([5, 3])
    with pytest.raises(ValueError):
        corpus.chunk_ends_to_offsets([5, 30], n_tokens=20)


def test_concatenation_keeps_every_sentence_and_window():
    rng = np.random.default_rng(0)
    shards = [encoder_like(rng, n, 500) for n in (40, 1, 0, 75)]
    tokens, offsets = corpus.concatenate_shards(shards)
    assert tokens.dtype == np.int32 and offsets.dtype == np.uint64
    assert np.array_equal(tokens, np.concatenate([s[0] for s in shards]))
    assert offsets[0] == 0 and offsets[-1] == len(tokens) and np.all(np.diff(offsets.astype(np.int64)) >= 0)
    # the sentences are the same token runs, in order
    want = [ids[a:b].tolist() for ids, ends in shards for a, b in zip(np.r_[0, ends[:-1]].astype(int), ends.astype(int))]
    got = [tokens[a:b].tolist() for a, b in zip(offsets[:-1].astype(int), offsets[1:].astype(int))]
    assert [g for g in got if g] == [w for w in want if w]
    # and the window count is the sum over the shards
    w = 11
    per_shard = sum(to.count_windows(corpus.chunk_ends_to_offsets(ends, len(ids)), w) for ids, ends in shards)
    assert to.count_windows(offsets, w) == per_shard
    assert corpus.validate(tokens, offsets) == int(tokens.max()) + 1


def test_validate_rejects_what_the_trainer_rejects():
    tokens = np.array([1, 2, -1, 3], dtype=np.int32)
    good = np.array([0, 2, 4], dtype=np.uint64)
    assert corpus.validate(tokens, good) == 4
    with pytest.raises(ValueError):
        corpus.validate(tokens, np.array([2, 4], dtype=np.uint64))        # the encoder's raw ends: no leading 0
    with pytest.raises(ValueError):
        corpus.validate(tokens, np.array([0, 3, 2], dtype=np.uint64))
    with pytest.raises(ValueError):
        corpus.validate(tokens, np.array([0, 9], dtype=np.uint64))
    with pytest.raises(ValueError):
        corpus.validate(tokens.astype(np.int64), good)
    with pytest.raises(ValueError):
        corpus.validate(np.array([1, -2], dtype=np.int32), np.array([0, 2], dtype=np.uint64))
    with pytest.raises(ValueError):
        corpus.validate(tokens, good, vocab=3)


def test_shard_pairs(tmp_path):
    rng = np.random.default_rng(1)
    for stem in ("b_part", "a_part"):
        ids, ends = encoder_like(rng, 5, 50)
        np.save(tmp_path / f"{stem}.npy", ids)
        np.save(tmp_path / f"{stem}_offsets.npy", ends)
    pairs = corpus.shard_pairs(tmp_path)
    assert [p[0].name for p in pairs] == ["a_part.npy", "b_part.npy"]
    (tmp_path / "a_part.npy").unlink()
    with pytest.raises(FileNotFoundError):
        corpus.shard_pairs(tmp_path)
