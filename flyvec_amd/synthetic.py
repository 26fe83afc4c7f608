"""Synthetic corpora and index batches of the benchmark configurations.

The reference ships no data (its corpus and pretrained matrix are downloads), so the bench and
the tests draw inputs of the same shape: bounded-Zipf token ids, geometric chunk lengths,
standard-normal synapses, all from fixed seeds.
"""
import numpy as np


def zipf_ids(n, vocab, s=1.07, seed=0, dtype=np.int32):
    """n ids with P(id = r) proportional to r^-s over r in [1, vocab); id 0 (<UNK>) is never drawn."""
    rng = np.random.default_rng(seed)
    p = np.arange(1, vocab, dtype=np.float64) ** (-s)
    cdf = np.cumsum(p / p.sum())
    ids = 1 + np.searchsorted(cdf, rng.random(n), side="right")
    return np.minimum(ids, vocab - 1).astype(dtype)


def corpus(n_tokens, vocab, s=1.07, mean_chunk=25, seed_tokens=3, seed_chunks=4):
    """(tokens int32, offsets uint64): offsets start at 0 and end with the n_tokens sentinel
    (flyvec/train_flyvec.py:172-173 takes len(offsets) - 1 chunks); the vocabulary inferred as
    max + 1 (flyvec/train_flyvec.py:168) is exactly `vocab`."""
    tokens = zipf_ids(n_tokens, vocab, s=s, seed=seed_tokens)
    if tokens.max() != vocab - 1:
        tokens[-1] = vocab - 1
    rng = np.random.default_rng(seed_chunks)
    n_draw = int(n_tokens / mean_chunk * 1.2) + 16
    ends = np.cumsum(rng.geometric(1.0 / mean_chunk, size=n_draw).astype(np.uint64))
    while ends[-1] < n_tokens:
        more = np.cumsum(rng.geometric(1.0 / mean_chunk, size=n_draw).astype(np.uint64)) + ends[-1]
        ends = np.concatenate([ends, more])
    ends = ends[ends < n_tokens]
    offsets = np.concatenate([[0], ends, [n_tokens]]).astype(np.uint64)
    return tokens, offsets


def synapses(hid, vocab, seed=5, mu=0.0, sigma=1.0):
    """K x 2V fp32; sigma = 1 is the benchmark's standard normal, (mu, sigma) = (0, 0.02) the
    trainer's default initialisation (flyvec/train_flyvec.py:41-42, 241)."""
    rng = np.random.default_rng(seed)
    W = rng.standard_normal((hid, 2 * vocab), dtype=np.float32)
    if sigma != 1.0:
        W *= np.float32(sigma)
    if mu != 0.0:
        W += np.float32(mu)
    return W


def window_indices(n, w, vocab, s=1.07, seed=7, centre_to_target=True):
    """(n, w) int32 column indices of a K x 2V matrix: Zipf ids, centre column shifted into the
    target block as the trainer's sampler does (flyvec/src/cuda_funcs.cu:929-932)."""
    idx = zipf_ids(n * w, vocab, s=s, seed=seed).reshape(n, w)
    if centre_to_target:
        idx[:, w // 2] += vocab
    return idx
