"""The corpus files either side of the trainer: what the reference's encoder writes, what
``flyvec_train`` reads, and the steps between.

The reference's tokenizer writes one pair of files per text shard (flyvec/tokenizer.py:199-227):
``<stem>.npy`` -- int32 token ids -- and ``<stem>_offsets.npy`` -- uint64 *ends* of the sentences,
cumulative inside the shard, without a leading 0.  The trainer wants one ``encodings.npy`` and one
``offsets.npy`` of chunk *starts*: ``offsets[0] = 0``, and the final chunk is only used when the
array ends with the number of tokens (flyvec/train_flyvec.py:172-173).  Stop words are removed from
an encoded corpus by overwriting their ids with -1 (flyvec/src/remove_words.cpp:28-37).

    python -m flyvec_amd.corpus merge SHARD_DIR -o OUT_DIR [--stop-ids ids.npy]
"""
import argparse
import ctypes as C
from pathlib import Path

import numpy as np

from . import _lib
from ._lib import check, ptr


def chunk_ends_to_offsets(ends, n_tokens=None):
    """Sentence ends as flyvec/tokenizer.py:199-215 returns them -> the trainer's chunk starts:
    a leading 0, the ends, and (once) the number of tokens as the closing sentinel."""
    ends = np.asarray(ends, dtype=np.uint64).reshape(-1)
    if len(ends) and np.any(ends[1:] < ends[:-1]):
        raise ValueError("sentence ends must be non-decreasing")
    if n_tokens is None:
        n_tokens = int(ends[-1]) if len(ends) else 0
    if len(ends) and int(ends[-1]) > n_tokens:
        raise ValueError(f"last sentence ends at {int(ends[-1])}, the shard holds {n_tokens} tokens")
    parts = [np.zeros(1, dtype=np.uint64), ends]
    if not len(ends) or int(ends[-1]) != n_tokens:
        parts.append(np.array([n_tokens], dtype=np.uint64))
    return np.concatenate(parts)


def concatenate_shards(shards):
    """[(ids, sentence_ends), ...] in corpus order -> (tokens int32, offsets uint64) for the trainer.
    Tokens of a shard that follow its last sentence end form one more chunk."""
    tokens, offsets, shift = [], [np.zeros(1, dtype=np.uint64)], 0
    for ids, ends in shards:
        ids = np.asarray(ids)
        if ids.dtype != np.int32:
            if ids.size and (ids.min() < -1 or ids.max() > np.iinfo(np.int32).max):
                raise ValueError("token ids do not fit int32")
            ids = ids.astype(np.int32)
        off = chunk_ends_to_offsets(ends, len(ids))
        tokens.append(ids.reshape(-1))
        offsets.append(off[1:] + np.uint64(shift))
        shift += len(ids)
    tok = np.concatenate(tokens) if tokens else np.zeros(0, dtype=np.int32)
    off = np.concatenate(offsets)
    return np.ascontiguousarray(tok, dtype=np.int32), np.ascontiguousarray(off, dtype=np.uint64)


def shard_pairs(directory):
    """The (<stem>.npy, <stem>_offsets.npy) pairs of a directory, sorted by stem."""
    directory = Path(directory)
    pairs = []
    for off in sorted(directory.glob("*_offsets.npy")):
        ids = off.with_name(off.name[: -len("_offsets.npy")] + ".npy")
        if not ids.exists():
            raise FileNotFoundError(f"{off.name} has no {ids.name} beside it")
        pairs.append((ids, off))
    return pairs


def validate(tokens, offsets, vocab=None):
    """The checks ``fv_trainer_set_corpus`` makes, on the host: dtype, ids in [-1, vocab), offsets
    starting at 0, non-decreasing, inside the corpus. Returns the vocabulary size the trainer infers
    (max + 1, flyvec/train_flyvec.py:168)."""
    tokens, offsets = np.asarray(tokens), np.asarray(offsets)
    if tokens.dtype != np.int32 or tokens.ndim != 1:
        raise ValueError("encodings must be a 1-D int32 array")
    if offsets.dtype != np.uint64 or offsets.ndim != 1 or len(offsets) < 1:
        raise ValueError("offsets must be a non-empty 1-D uint64 array")
    if int(offsets[0]) != 0:
        raise ValueError("offsets must start with 0 (flyvec/src/prune_input.cpp:88-122 sums chunk lengths from 0)")
    if np.any(offsets[1:] < offsets[:-1]) or int(offsets[-1]) > len(tokens):
        raise ValueError("offsets must be non-decreasing and end inside the corpus")
    inferred = int(tokens.max()) + 1 if len(tokens) else 0
    if len(tokens) and int(tokens.min()) < -1:
        raise ValueError("token ids below -1")
    if vocab is not None and inferred > vocab:
        raise ValueError(f"token id {inferred - 1} is outside the vocabulary of {vocab}")
    return inferred


def mask_tokens(tokens, remove_ids, vocab=None):
    """In place: every occurrence of an id of `remove_ids` becomes -1, in one pass on the device
    (flyvec/src/remove_words.cpp:28-37 makes one pass over the corpus per id)."""
    if tokens.dtype != np.int32 or not tokens.flags.c_contiguous or not tokens.flags.writeable:
        raise ValueError("tokens must be a writable C-contiguous int32 array")
    remove_ids = np.ascontiguousarray(remove_ids, dtype=np.int32).reshape(-1)
    if vocab is None:
        vocab = max(int(tokens.max()) + 1 if len(tokens) else 1, int(remove_ids.max()) + 1 if len(remove_ids) else 1, 1)
    check(_lib.load().fv_mask_tokens(ptr(tokens), tokens.size, ptr(remove_ids), len(remove_ids), int(vocab)))
    return tokens


def prune_windows(windows):
    """In place: in every row of an int32 (rows, cols) window matrix a value that an earlier column holds
    becomes -1; the centre column takes no part and keeps its value (flyvec/src/prune_input.cpp:14
    prune_input_data, a tool the reference exports but never calls)."""
    if windows.dtype != np.int32 or windows.ndim != 2 or not windows.flags.c_contiguous or not windows.flags.writeable:
        raise ValueError("windows must be a writable C-contiguous int32 matrix")
    check(_lib.load().fv_prune_windows(ptr(windows), windows.shape[0], windows.shape[1]))
    return windows


def merge_directory(shard_dir, out_dir, stop_ids=None):
    """Shards of the reference's encoder -> encodings.npy + offsets.npy for ``flyvec_train``."""
    pairs = shard_pairs(shard_dir)
    if not pairs:
        raise FileNotFoundError(f"no <stem>_offsets.npy in {shard_dir}")
    tokens, offsets = concatenate_shards((np.load(i), np.load(o)) for i, o in pairs)
    if stop_ids is not None:
        mask_tokens(tokens, np.load(stop_ids) if isinstance(stop_ids, (str, Path)) else stop_ids)
    validate(tokens, offsets)
    out_dir = Path(out_dir)
    out_dir.mkdir(parents=True, exist_ok=True)
    np.save(out_dir / "encodings.npy", tokens)
    np.save(out_dir / "offsets.npy", offsets)
    return tokens, offsets


def main(argv=None):
    ap = argparse.ArgumentParser(prog="python -m flyvec_amd.corpus")
    sub = ap.add_subparsers(dest="cmd", required=True)
    m = sub.add_parser("merge", help="join the encoder's shards into encodings.npy + offsets.npy")
    m.add_argument("shard_dir")
    m.add_argument("-o", "--output_dir", default=".")
    m.add_argument("--stop-ids", default=None, help=".npy of token ids to overwrite with -1")
    args = ap.parse_args(argv)
    tokens, offsets = merge_directory(args.shard_dir, args.output_dir, args.stop_ids)
    print(f"{len(tokens)} tokens, {len(offsets) - 1} chunks, vocabulary {int(tokens.max()) + 1 if len(tokens) else 0}, "
          f"{int((tokens < 0).sum())} masked")


if __name__ == "__main__":
    main()
