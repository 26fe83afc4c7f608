"""Python handles over the C ABI: ``Trainer`` (the minibatch step) and ``Hasher`` (top-k codes).

These are thin: every operation is one call into libflyvec_hip.so; numpy is used only for the
host buffers that cross the boundary.
"""
import ctypes as C

import numpy as np

from . import _lib
from ._lib import check, ptr


def count_windows(offsets, w):
    """flyvec/src/prune_input.cpp:64 getnum_samples."""
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    out = C.c_uint64(0)
    check(_lib.load().fv_count_windows(ptr(offsets), max(len(offsets) - 1, 0), w, C.byref(out)))
    return out.value


def window_starts(offsets, w):
    """flyvec/src/prune_input.cpp:88 compute_offset_phrases."""
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    n = count_windows(offsets, w)
    out = np.empty(n, dtype=np.uint64)
    check(_lib.load().fv_build_window_starts(ptr(offsets), max(len(offsets) - 1, 0), w, ptr(out), n))
    return out


def inverse_frequency(corpus, vocab):
    """flyvec/src/model_arrays.cu:396 compute_inverse_word_frequency."""
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    out = np.empty(int(vocab), dtype=np.float32)
    check(_lib.load().fv_inverse_frequency(ptr(corpus), len(corpus), int(vocab), ptr(out)))
    return out


class Trainer:
    """Owns the synapse matrix, the corpus and the window table in HBM."""

    def __init__(self, vocab, hid=400, window=11, batch=10000, initial_learning_rate=0.002,
                 delta=0.0, prec=1.0e-30, tie_rule=0, lmid=1.0, lbase=1.0, prune_duplicates=False):
        self.lib = _lib.load()
        self.vocab, self.hid, self.window, self.batch = int(vocab), int(hid), int(window), int(batch)
        cfg = _lib.TrainConfig(vocab=self.vocab, hid=self.hid, window=self.window, batch=self.batch,
                               tie_rule=int(tie_rule), initial_learning_rate=initial_learning_rate,
                               delta=delta, prec=prec, lmid=lmid, lbase=lbase,
                               prune_duplicates=int(bool(prune_duplicates)))
        h = C.c_void_p()
        check(self.lib.fv_trainer_create(C.byref(cfg), C.byref(h)))
        self.handle = h

    def close(self):
        if getattr(self, "handle", None) is not None and self.handle.value:
            self.lib.fv_trainer_destroy(self.handle)
        self.handle = None
        self._checkpoint = None  # the page-locked buffer of save_weights

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def __enter__(self):
        return self

    def __exit__(self, *exc):
        self.close()

    # -- set-up ---------------------------------------------------------------------------
    def set_corpus(self, tokens, offsets):
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
        check(self.lib.fv_trainer_set_corpus(self.handle, ptr(tokens), len(tokens), ptr(offsets), len(offsets)))

    def set_corpus_starts(self, tokens, starts):
        """The corpus with a window-start table built elsewhere (what the reference's driver passes)."""
        tokens = np.ascontiguousarray(tokens, dtype=np.int32)
        starts = np.ascontiguousarray(starts, dtype=np.uint64)
        check(self.lib.fv_trainer_set_corpus_starts(self.handle, ptr(tokens), len(tokens), ptr(starts), len(starts)))

    @property
    def num_windows(self):
        out = C.c_uint64(0)
        check(self.lib.fv_trainer_num_windows(self.handle, C.byref(out)))
        return out.value

    def window_starts(self):
        out = np.empty(self.num_windows, dtype=np.uint64)
        check(self.lib.fv_trainer_get_window_starts(self.handle, ptr(out), len(out)))
        return out

    def inverse_frequency(self):
        out = np.empty(self.vocab, dtype=np.float32)
        check(self.lib.fv_trainer_get_inverse_frequency(self.handle, ptr(out)))
        return out

    def set_weights(self, W):
        W = np.ascontiguousarray(W, dtype=np.float32)
        if W.shape != (self.hid, 2 * self.vocab):
            raise ValueError(f"weights must be ({self.hid}, {2 * self.vocab}), got {W.shape}")
        check(self.lib.fv_trainer_set_weights(self.handle, ptr(W)))

    def get_weights(self, out=None):
        """The K x 2V matrix in the checkpoint's layout. `out`: a C-contiguous float32 array of that shape to
        fill (page-locked memory from _lib.pinned_empty is copied by DMA, five times as fast)."""
        if out is None:
            out = np.empty((self.hid, 2 * self.vocab), dtype=np.float32)
        if out.shape != (self.hid, 2 * self.vocab) or out.dtype != np.float32 or not out.flags.c_contiguous:
            raise ValueError(f"out must be a C-contiguous float32 array of shape {(self.hid, 2 * self.vocab)}")
        check(self.lib.fv_trainer_get_weights(self.handle, ptr(out)))
        return out

    def save_weights(self, path):
        """Writes the matrix as a .npy checkpoint (flyvec/train_flyvec.py:262: np.save of the K x 2V fp32
        matrix) through a page-locked buffer the trainer keeps for this."""
        if getattr(self, "_checkpoint", None) is None:
            self._checkpoint = _lib.pinned_empty((self.hid, 2 * self.vocab), np.float32)
        np.save(path, self.get_weights(self._checkpoint))

    def shuffle(self, seed=0):
        check(self.lib.fv_trainer_shuffle(self.handle, int(seed)))

    def set_permutation(self, perm):
        perm = np.ascontiguousarray(perm, dtype=np.uint64)
        check(self.lib.fv_trainer_set_permutation(self.handle, ptr(perm), len(perm)))

    def get_permutation(self):
        out = np.empty(self.num_windows, dtype=np.uint64)
        check(self.lib.fv_trainer_get_permutation(self.handle, ptr(out), len(out)))
        return out

    # -- the hot path ------------------------------------------------------------------------
    def step(self, first_window, n_windows, eps, delta=0.0):
        """One minibatch; delta != 0 adds the anti-Hebbian term on the second neuron of every window."""
        if delta:
            check(self.lib.fv_trainer_step_delta(self.handle, int(first_window), int(n_windows), float(eps),
                                                 float(delta)))
        else:
            check(self.lib.fv_trainer_step(self.handle, int(first_window), int(n_windows), float(eps)))

    def epoch_delta(self, epoch_id, n_epochs):
        out = C.c_float(0)
        check(self.lib.fv_trainer_epoch_delta(self.handle, int(epoch_id), int(n_epochs), C.byref(out)))
        return out.value

    def second_winners(self, n):
        out = np.empty(int(n), dtype=np.int32)
        check(self.lib.fv_trainer_get_second_winners(self.handle, ptr(out), len(out)))
        return out

    def run_epoch(self, epoch_id, n_epochs):
        check(self.lib.fv_trainer_run_epoch(self.handle, int(epoch_id), int(n_epochs)))

    def set_stale_tail(self, on):
        """True: run_epoch trains a final partial minibatch with the previous minibatch's rows behind its own,
        as the reference does (flyvec/src/cuda_funcs.cu:1679 against :1700-1732); False (default): the
        remainder only."""
        check(self.lib.fv_trainer_set_stale_tail(self.handle, 1 if on else 0))

    def epoch_eps(self, epoch_id, n_epochs):
        out = C.c_float(0)
        check(self.lib.fv_trainer_epoch_eps(self.handle, int(epoch_id), int(n_epochs), C.byref(out)))
        return out.value

    def sync(self):
        check(self.lib.fv_trainer_sync(self.handle))

    @property
    def giveups_recovered(self):
        """Epochs in which run_epoch took up again behind a single dense launch that gave up."""
        out = C.c_uint64(0)
        check(self.lib.fv_trainer_get_giveups_recovered(self.handle, C.byref(out)))
        return out.value

    def set_dense_launches(self, launches):
        """1: both passes over the matrix in one launch (kept in registers between them where it fits,
        its rows streamed otherwise), 3: the streaming form whatever the size, 2: separate launches,
        0: as chosen at creation.  Same results either way."""
        check(self.lib.fv_trainer_set_dense_launches(self.handle, int(launches)))

    def set_grouping_launch(self, separate):
        """True: the windows are grouped by winner in a launch of its own; False: inside the
        sparse-element launch where the step allows it.  Same results either way."""
        check(self.lib.fv_trainer_set_grouping_launch(self.handle, 1 if separate else 0))

    def set_slot_regions(self, per_block):
        """True (the default): every block of the sparse-element launch that groups for itself keeps its
        records in room of its own; False: in its class's region, behind the lower neurons' records.
        Same results either way."""
        check(self.lib.fv_trainer_set_slot_regions(self.handle, 1 if per_block else 0))

    def set_light_blocks(self, on):
        """True (the default): a neuron with few windows is finished by one block of the sparse-element launch
        that groups for itself, an entry per thread; False: by its four class blocks like the others.
        Same results either way."""
        check(self.lib.fv_trainer_set_light_blocks(self.handle, 1 if on else 0))

    def set_sentinel_list(self, entries):
        """Test hook: the single dense launch's LDS list of sparse elements counts as full after `entries`
        (0: its real size); the elements beyond are finished where they are met.  Same results."""
        check(self.lib.fv_trainer_set_sentinel_list(self.handle, int(entries)))

    @property
    def grouping_launch(self):
        """True when a step without the anti-Hebbian term groups in a launch of its own."""
        out = C.c_uint32(0)
        check(self.lib.fv_trainer_get_grouping_launch(self.handle, C.byref(out)))
        return bool(out.value)

    @property
    def dense_launches(self):
        out = C.c_uint32(0)
        check(self.lib.fv_trainer_get_dense_launches(self.handle, C.byref(out)))
        return out.value

    @property
    def dense_path_counts(self):
        """(single dense launches that knew max|ds| when they started, launches that made the pass for it)."""
        known, made = C.c_uint64(0), C.c_uint64(0)
        check(self.lib.fv_trainer_get_dense_path_counts(self.handle, C.byref(known), C.byref(made)))
        return known.value, made.value

    def _set_wait_limit(self, rounds):
        check(self.lib.fv_trainer_set_wait_limit(self.handle, int(rounds)))

    def winners(self, n):
        out = np.empty(int(n), dtype=np.int32)
        check(self.lib.fv_trainer_get_winners(self.handle, ptr(out), len(out)))
        return out

    def step_stats(self):
        xx = np.empty(self.hid, dtype=np.float32)
        nc = C.c_float(0)
        check(self.lib.fv_trainer_get_step_stats(self.handle, ptr(xx), C.byref(nc)))
        return xx, nc.value

    def row_norms(self, n_rows=10):
        n_rows = min(int(n_rows), self.hid)
        out = np.empty(n_rows, dtype=np.float64)
        check(self.lib.fv_trainer_row_norms(self.handle, n_rows, ptr(out)))
        return out

    def time_steps(self, first_window, n_steps, eps, per_kernel=True):
        total = C.c_float(0)
        kern = (C.c_float * _lib.FV_TRAIN_KERNELS)()
        check(self.lib.fv_trainer_time_steps(self.handle, int(first_window), int(n_steps), float(eps),
                                             C.byref(total), kern if per_kernel else None))
        return total.value, dict(zip(_lib.TRAIN_KERNEL_NAMES, list(kern))) if per_kernel else None

    def time_steps_graph(self, first_window, n_steps, eps, steps_per_graph=1):
        """The same steps enqueued as HIP graphs of `steps_per_graph` steps each; milliseconds for all."""
        total = C.c_float(0)
        check(self.lib.fv_trainer_time_steps_graph(self.handle, int(first_window), int(n_steps), float(eps),
                                                   int(steps_per_graph), C.byref(total)))
        return total.value

    def _time_kernel(self, index, reps):
        ms = C.c_float(0)
        check(self.lib.fv_trainer_time_kernel(self.handle, index, reps, C.byref(ms)))
        return ms.value

    def time_kernels(self, reps=20):
        """Mean duration (ms) of each kernel of the last step, launched back to back `reps` times.
        Leaves W good for timing only."""
        return {name: self._time_kernel(i, reps) for i, name in enumerate(_lib.TRAIN_KERNEL_NAMES)}


class Hasher:
    """A checkpoint matrix resident in HBM plus the batched top-k threshold code."""

    def __init__(self, W):
        self.lib = _lib.load()
        W = np.ascontiguousarray(W, dtype=np.float32)
        if W.ndim != 2:
            raise ValueError("synapse matrix must be 2-D (K, N)")
        self.hid, self.n_columns = W.shape
        self.words = (self.hid + 63) // 64
        h = C.c_void_p()
        check(self.lib.fv_hasher_create(ptr(W), self.hid, self.n_columns, C.byref(h)))
        self.handle = h
        self.version = 0  # counts the changes of the resident matrix (what is derived from it goes stale)

    def close(self):
        if getattr(self, "handle", None) is not None and self.handle.value:
            self.lib.fv_hasher_destroy(self.handle)
        self.handle = None

    def __del__(self):
        try:
            self.close()
        except Exception:
            pass

    def normalize(self, prec=1.0e-32, p=2):
        """flyvec/core.py:23-36 on the resident matrix, p a positive integer: the two passes over the
        matrix run on the device; the p-th root of the K row sums is numpy's, as in the reference. Equal to the
        reference bit for bit for p = 1 and p = 2 (its default, all its own code uses); from p = 3 on numpy's
        float32 power is the C library's powf and the result agrees to rounding."""
        if int(p) != p or not 1 <= p <= 64:
            raise ValueError(f"p = {p}: the norm's exponent must be an integer from 1 to 64")
        p = int(p)
        sums = np.empty(self.hid, dtype=np.float32)
        check(self.lib.fv_hasher_row_sum_pow(self.handle, p, ptr(sums)))
        nc = np.power(sums, 1 / p).reshape(self.hid, 1)
        div = np.ascontiguousarray((nc + prec).reshape(-1), dtype=np.float32)
        check(self.lib.fv_hasher_scale_rows(self.handle, ptr(div)))
        self.version += 1

    def weights(self):
        out = np.empty((self.hid, self.n_columns), dtype=np.float32)
        check(self.lib.fv_hasher_get_weights(self.handle, ptr(out)))
        return out

    def _check_k(self, k):
        if not 0 < k < self.hid:
            # the reference reads act_sort[k] (flyvec/core.py:157)
            raise IndexError(f"hash length {k} is out of bounds for {self.hid} neurons")

    def hash_targets(self, ids, k=50):
        self._check_k(k)
        ids = np.ascontiguousarray(ids, dtype=np.int32).reshape(-1)
        out = np.empty((len(ids), self.hid), dtype=np.int8)
        check(self.lib.fv_hash_targets(self.handle, ptr(ids), len(ids), k, ptr(out)))
        return out

    def hash_windows(self, idx, k=50, packed=True, codes=False, out_bits=None, out_codes=None):
        """idx (n, w) int32 column indices (-1 = masked). Returns packed uint64 words, int8 codes,
        or both as a tuple. out_bits / out_codes: arrays to fill instead of new ones (page-locked ones
        from flyvec_amd._lib.pinned_empty, like a page-locked idx, are copied without staging)."""
        self._check_k(k)
        idx = np.ascontiguousarray(idx, dtype=np.int32)
        if idx.ndim != 2:
            raise ValueError("idx must be (n, w)")
        n, w = idx.shape
        for out, shape, dt in ((out_bits, (n, self.words), np.uint64), (out_codes, (n, self.hid), np.int8)):
            if out is not None and (out.shape != shape or out.dtype != dt or not out.flags.c_contiguous):
                raise ValueError(f"output must be a C-contiguous {np.dtype(dt).name} array of shape {shape}")
        packed, codes = packed or out_bits is not None, codes or out_codes is not None
        bits = (out_bits if out_bits is not None else np.empty((n, self.words), dtype=np.uint64)) if packed else None
        cds = (out_codes if out_codes is not None else np.empty((n, self.hid), dtype=np.int8)) if codes else None
        check(self.lib.fv_hash_windows(self.handle, ptr(idx), n, w, k, ptr(bits), ptr(cds)))
        if packed and codes:
            return bits, cds
        return bits if packed else cds

    def hash_windows_dev(self, idx_buf, n, w, k, bits_buf=None, codes_buf=None):
        self._check_k(k)
        check(self.lib.fv_hash_windows_dev(self.handle, idx_buf.ptr, n, w, k,
                                           bits_buf.ptr if bits_buf else None,
                                           codes_buf.ptr if codes_buf else None))

    def sync(self):
        check(self.lib.fv_hasher_sync(self.handle))

    def time_windows(self, idx_buf, n, w, k, bits_buf=None, codes_buf=None, reps=10):
        ms = C.c_float(0)
        check(self.lib.fv_hasher_time_windows(self.handle, idx_buf.ptr, n, w, k,
                                              bits_buf.ptr if bits_buf else None,
                                              codes_buf.ptr if codes_buf else None, reps, C.byref(ms)))
        return ms.value
