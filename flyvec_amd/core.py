"""``FlyVec``: the reference's inference wrapper (flyvec/core.py:39-211) over the device hasher.

Same method names, arguments, return dictionaries and error behaviour for the hashing path:
``get_sparse_embedding`` / ``get_dense_embedding`` / ``simple_word_vectors`` / ``tokenize`` /
``is_unknown_token`` / ``from_config``.  The synapse matrix lives in HBM; every embedding is
computed by libflyvec_hip.so (there is no numpy fallback).  The gensim tokenizer of the reference
(flyvec/tokenizer.py) is a text front-end outside this package: any object with ``tokenize``,
``token2id``, ``id2token`` and ``n_vocab`` can be passed, or a plain vocabulary list (id = position,
id 0 = ``<UNK>``), in which case words are lower-cased and split on whitespace.
"""
from pathlib import Path
from typing import Dict, Optional, Sequence, Union

import numpy as np

from .engine import Hasher


class VocabTokenizer:
    """Minimal stand-in for the tokenizer interface FlyVec uses (flyvec/tokenizer.py:146-197)."""

    def __init__(self, vocab: Sequence[str]):
        self.vocab = list(vocab)
        self._ids = {t: i for i, t in enumerate(self.vocab)}

    def tokenize(self, sentence: str):
        return sentence.lower().split()

    def token2id(self, token: str) -> int:
        return self._ids.get(token, 0)

    def id2token(self, idx: int) -> str:
        return self.vocab[idx]

    def n_vocab(self) -> int:
        return len(self.vocab)


class FlyVec:
    """A tokenizer plus synapse weights resident on the GPU, for hashing words."""

    def __init__(self, synapse_file: Union[Path, str, np.ndarray], tokenizer=None,
                 stopword_file: Optional[Union[Path, str]] = None, normalize_synapses: bool = True):
        self.synapse_file = synapse_file
        self.stopword_file = str(stopword_file) if stopword_file is not None else None
        self.normalize_synapses = normalize_synapses
        if tokenizer is not None and not hasattr(tokenizer, "token2id"):
            tokenizer = VocabTokenizer(tokenizer)
        self.tokenizer = tokenizer
        syn = synapse_file if isinstance(synapse_file, np.ndarray) else np.load(str(synapse_file))
        if syn.ndim != 2 or syn.shape[1] % 2:
            raise ValueError(f"synapses must be (K, 2V), got {syn.shape}")
        self.hasher = Hasher(syn)
        if normalize_synapses:
            self.hasher.normalize()  # flyvec/core.py:87
        self._synapses = None
        self._stop_ids = None
        # hash_length -> (version of the resident matrix, codes of every token id): what the per-word calls read
        self._code_tables = {}

    @classmethod
    def load(cls, force_redownload=False):
        """flyvec/core.py:50-60 downloads the pretrained model from a bucket; this package fetches
        nothing. Unpack the model directory yourself and use ``from_config``."""
        raise NotImplementedError("FlyVec.load() downloads data in the reference; use FlyVec.from_config("
                                  "'<model dir>/config.yaml', tokenizer=...) on a local copy")

    @classmethod
    def from_config(cls, fname: Union[Path, str], tokenizer=None):
        """flyvec/core.py:62-77: keys ``synapses``, ``normalize_synapses``, ``stop_words``; the
        ``tokenizer`` / ``phrases`` entries name gensim pickles and are not opened here."""
        import yaml
        fpath = Path(fname)
        ref_dir = fpath.parent
        with open(fname, "r") as fp:
            conf = yaml.safe_load(fp)
        stop = ref_dir / conf["stop_words"] if "stop_words" in conf else None
        return cls(ref_dir / conf["synapses"], tokenizer=tokenizer, stopword_file=stop,
                   normalize_synapses=conf.get("normalize_synapses", False))

    # -- properties of the reference class -------------------------------------------------------
    @property
    def n_neurons(self):
        return self.hasher.hid

    @property
    def n_vocab(self):
        return self.hasher.n_columns // 2

    @property
    def synapses(self):
        """The (normalised) matrix as the device holds it, K x 2V."""
        if self._synapses is None or self._synapses[0] != self.hasher.version:
            self._synapses = (self.hasher.version, self.hasher.weights())
        return self._synapses[1]

    @property
    def token_vocab(self):
        return list(self.tokenizer.vocab) if hasattr(self.tokenizer, "vocab") else \
            [self.tokenizer.id2token(i) for i in range(self.tokenizer.n_vocab())]

    @property
    def vocab(self):
        return self.tokenizer.vocab

    @property
    def dictionary(self):
        return self.tokenizer.dictionary

    @property
    def stop_word_ids(self):
        """Token ids the model should not respond to (flyvec/core.py:109-112); empty without a file."""
        if self._stop_ids is None:
            self._stop_ids = set(int(i) for i in np.load(self.stopword_file)) if self.stopword_file else set()
        return self._stop_ids

    @property
    def stop_words(self):
        """flyvec/core.py:114-117."""
        return set(self.tokenizer.id2token(t) for t in self.stop_word_ids)

    @property
    def unknown_embedding_info(self):
        # flyvec/core.py:119-125 (note the uint8 dtype of this one vector)
        return {"token": "<UNK>", "id": 0, "embedding": np.zeros(self.n_neurons).astype(np.uint8)}

    def tokenize(self, sentence: str):
        return self.tokenizer.tokenize(sentence)

    def _first_token_id(self, word):
        if isinstance(word, (int, np.integer)):
            return None, int(word)
        if len(word) == 0:
            raise ValueError("Token cannot be the empty string")  # flyvec/core.py:132-133
        tok = self.tokenizer.tokenize(word)[0]
        return tok, self.tokenizer.token2id(tok)

    def is_unknown_token(self, token) -> bool:
        return self._first_token_id(token)[1] == 0

    # -- embeddings --------------------------------------------------------------------------------
    CODE_TABLES_KEPT = 4  # hash lengths whose whole-vocabulary tables are kept (8 MB each at K = 400, V = 20000)

    def code_table(self, hash_length: int = 50) -> np.ndarray:
        """(n_vocab, K) int8: the code of every token id for this hash length, computed on the device by one
        batched launch the first time the length is asked for and kept until the resident matrix changes.
        The reference's API hashes one word per call (flyvec/core.py:139-163, looped at :187-211); a launch, two
        copies and a synchronisation per word cost more than the arithmetic, so the per-word calls read here."""
        entry = self._code_tables.get(hash_length)
        if entry is None or entry[0] != self.hasher.version:
            codes = self.hasher.hash_targets(np.arange(self.n_vocab, dtype=np.int32), hash_length)
            codes.setflags(write=False)
            self._code_tables.pop(hash_length, None)
            while len(self._code_tables) >= self.CODE_TABLES_KEPT:
                self._code_tables.pop(next(iter(self._code_tables)))
            entry = self._code_tables[hash_length] = (self.hasher.version, codes)
        return entry[1]

    def get_sparse_embedding(self, word, hash_length: int = 50):
        """flyvec/core.py:139-163; ``word`` may also be a token id."""
        tok, tok_id = self._first_token_id(word)
        if tok_id == 0:
            return self.unknown_embedding_info
        if not 0 <= tok_id < self.n_vocab:
            raise IndexError(f"token id {tok_id} is outside the vocabulary of {self.n_vocab}")
        code = self.code_table(hash_length)[tok_id].copy()  # the caller's own array, as the reference returns
        return {"token": tok if tok is not None else self._id2token(tok_id), "id": tok_id, "embedding": code}

    def get_dense_embedding(self, word):
        """flyvec/core.py:165-185: the target-block column of the token."""
        tok, tok_id = self._first_token_id(word)
        if tok_id == 0:
            return self.unknown_embedding_info
        return {"token": tok if tok is not None else self._id2token(tok_id), "id": tok_id,
                "embedding": self.synapses[:, self.n_vocab + tok_id]}

    def get_sparse_embeddings(self, ids, hash_length: int = 50) -> np.ndarray:
        """Batched form: (n, K) int8 codes of the given token ids in one launch."""
        return self.hasher.hash_targets(ids, hash_length)

    def get_context_embeddings(self, windows, hash_length: int = 50, packed=False) -> np.ndarray:
        """Codes of (n, w) windows of column indices (context ids, centre id + n_vocab, -1 = masked)."""
        return self.hasher.hash_windows(windows, hash_length, packed=packed, codes=not packed)

    def _id2token(self, i):
        return self.tokenizer.id2token(i) if self.tokenizer is not None else str(i)

    def simple_word_vectors(self, k: int = 50, exclude_stop_words=False, output_list=False) -> Dict[str, np.ndarray]:
        """flyvec/core.py:187-211 in one batch: token -> code for the whole vocabulary. Tokens whose
        id is 0 get the unknown embedding, as the reference's per-word call returns."""
        vocab = self.token_vocab
        ids = np.array([self.tokenizer.token2id(self.tokenizer.tokenize(t)[0]) if len(t) else -1
                        for t in vocab], dtype=np.int64)
        stop = self.stop_word_ids if exclude_stop_words else set()
        good = ids > 0
        codes = self.hasher.hash_targets(ids[good].astype(np.int32), k) if good.any() else None
        out = {}
        row = 0
        for t, i, g in zip(vocab, ids, good):
            if g:
                vec = codes[row]
                row += 1
            elif i == 0:
                vec = self.unknown_embedding_info["embedding"]
            else:
                print(f"Invalid token: `{t}`. Continuing.")
                continue
            if exclude_stop_words and int(i) in stop:
                continue
            out[t] = list(vec) if output_list else vec
        return out

    def export_simple_embeddings(self, path, k: int = 50, exclude_stop_words=False):
        """Writes ``simple_word_vectors(k, output_list=True)`` as JSON: token -> list of 0/1, the
        context-independent artefact the reference's README describes (README.md:132-138)."""
        import json
        vecs = self.simple_word_vectors(k, exclude_stop_words=exclude_stop_words, output_list=True)
        with open(path, "w") as fp:
            json.dump({t: [int(x) for x in v] for t, v in vecs.items()}, fp)
        return len(vecs)
