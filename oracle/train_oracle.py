"""ctypes view of flyvec_oracle.c and of the reference's prune_input.cpp.

TEST INFRASTRUCTURE ONLY (see the package docstring).  ``build()`` runs the
Makefile next to this file; ``lib()`` / ``ref_lib()`` load what it produced.
"""
import ctypes as C
import os
import subprocess
from pathlib import Path

import numpy as np

HERE = Path(__file__).resolve().parent
LIB_PATH = HERE / "_build" / "libflyvec_oracle.so"
REF_PATH = HERE / "_ref" / "libprune_input_ref.so"

_lib = None
_ref = None


def build(quiet=True):
    out = subprocess.run(["make", "-C", str(HERE)], capture_output=True, text=True)
    if out.returncode != 0:
        raise RuntimeError("oracle build failed:\n" + out.stdout + out.stderr)
    if not quiet:
        print(out.stdout)


def _p(a):
    return a.ctypes.data_as(C.c_void_p)


def lib():
    global _lib
    if _lib is None:
        if not LIB_PATH.exists():
            build()
        L = C.CDLL(str(LIB_PATH))
        L.fvo_num_threads.restype = C.c_int
        L.fvo_count_windows.restype = C.c_uint64
        L.fvo_count_windows.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        L.fvo_window_starts.restype = None
        L.fvo_window_starts.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p]
        L.fvo_inverse_frequency.restype = None
        L.fvo_inverse_frequency.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64, C.c_void_p]
        L.fvo_inflate.restype = None
        L.fvo_inflate.argtypes = [C.c_void_p, C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64,
                                  C.c_int, C.c_uint64, C.c_void_p]
        L.fvo_activations.restype = None
        L.fvo_activations.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_uint64, C.c_int,
                                      C.c_void_p, C.c_uint64, C.c_void_p, C.c_void_p]
        L.fvo_argmax_reference.restype = C.c_int
        L.fvo_argmax_reference.argtypes = [C.c_void_p, C.c_int]
        L.fvo_argmax_lowest.restype = C.c_int
        L.fvo_argmax_lowest.argtypes = [C.c_void_p, C.c_int]
        L.fvo_epoch_eps.restype = C.c_float
        L.fvo_epoch_eps.argtypes = [C.c_float, C.c_uint64, C.c_uint64]
        L.fvo_xx_sums.restype = None
        L.fvo_xx_sums.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_int, C.c_int, C.c_void_p]
        L.fvo_train_step.restype = None
        L.fvo_train_step.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_void_p, C.c_uint64,
                                     C.c_int, C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_void_p,
                                     C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fvo_epoch_delta.restype = C.c_float
        L.fvo_epoch_delta.argtypes = [C.c_float, C.c_uint64, C.c_uint64]
        L.fvo_train_step_delta.restype = None
        L.fvo_train_step_delta.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_void_p, C.c_uint64,
                                           C.c_int, C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_float,
                                           C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_void_p, C.c_void_p]
        L.fvo_train_step_weighted.restype = None
        L.fvo_train_step_weighted.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_uint64, C.c_void_p, C.c_uint64,
                                              C.c_int, C.c_void_p, C.c_float, C.c_float, C.c_int, C.c_float,
                                              C.c_float, C.c_float, C.c_void_p, C.c_void_p, C.c_void_p,
                                              C.c_void_p, C.c_void_p, C.c_void_p, C.c_void_p]
        L.fvo_train_steps_weighted.restype = C.c_uint64
        L.fvo_train_steps_weighted.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p,
                                               C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p,
                                               C.c_float, C.c_float, C.c_int, C.c_float, C.c_float, C.c_float,
                                               C.c_int, C.c_void_p]
        L.fvo_train_steps_tail.restype = C.c_uint64
        L.fvo_train_steps_tail.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p,
                                           C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p,
                                           C.c_float, C.c_float, C.c_int, C.c_float, C.c_float, C.c_float,
                                           C.c_int, C.c_int, C.c_void_p]
        L.fvo_inflate_prune.restype = None
        L.fvo_inflate_prune.argtypes = L.fvo_inflate.argtypes
        L.fvo_prune_windows.restype = None
        L.fvo_prune_windows.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        L.fvo_train_steps_delta.restype = C.c_uint64
        L.fvo_train_steps_delta.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p,
                                            C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p,
                                            C.c_float, C.c_float, C.c_int, C.c_float, C.c_void_p]
        L.fvo_train_steps.restype = C.c_uint64
        L.fvo_train_steps.argtypes = [C.c_void_p, C.c_int, C.c_uint64, C.c_void_p, C.c_void_p, C.c_void_p,
                                      C.c_uint64, C.c_uint64, C.c_uint64, C.c_uint64, C.c_int, C.c_void_p,
                                      C.c_float, C.c_float, C.c_int, C.c_void_p]
        _lib = L
    return _lib


def ref_lib():
    """The reference's own prune_input.cpp (None when oracle/_ref was never built)."""
    global _ref
    if _ref is None and REF_PATH.exists():
        R = C.CDLL(str(REF_PATH))
        R.getnum_samples.restype = C.c_uint64
        R.getnum_samples.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        R.compute_offset_phrases.restype = None
        R.compute_offset_phrases.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint64]
        R.prune_input_data.restype = None
        R.prune_input_data.argtypes = [C.c_void_p, C.c_uint64, C.c_uint64]
        _ref = R
    return _ref


def num_threads():
    return lib().fvo_num_threads()


def count_windows(offsets, w):
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    return int(lib().fvo_count_windows(_p(offsets), max(len(offsets) - 1, 0), w))


def window_starts(offsets, w):
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    n = count_windows(offsets, w)
    out = np.empty(n, dtype=np.uint64)
    lib().fvo_window_starts(_p(offsets), max(len(offsets) - 1, 0), w, _p(out))
    return out


def ref_count_windows(offsets, w):
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    with _quiet_stderr():
        return int(ref_lib().getnum_samples(_p(offsets), max(len(offsets) - 1, 0), w))


def ref_window_starts(offsets, w):
    offsets = np.ascontiguousarray(offsets, dtype=np.uint64)
    n = ref_count_windows(offsets, w)
    out = np.empty(n + 1, dtype=np.uint64)
    with _quiet_stderr():
        ref_lib().compute_offset_phrases(_p(out), _p(offsets), max(len(offsets) - 1, 0), w)
    return out[:n]


class _quiet_stderr:
    """The reference prints progress to stderr from C; keep test logs readable."""

    def __enter__(self):
        self._saved = os.dup(2)
        self._null = os.open(os.devnull, os.O_WRONLY)
        os.dup2(self._null, 2)

    def __exit__(self, *exc):
        os.dup2(self._saved, 2)
        os.close(self._null)
        os.close(self._saved)


def inverse_frequency(corpus, V):
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    out = np.empty(V, dtype=np.float32)
    lib().fvo_inverse_frequency(_p(corpus), len(corpus), V, _p(out))
    return out


def inflate(corpus, starts, perm, first, n, w, V):
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    starts = np.ascontiguousarray(starts, dtype=np.uint64)
    perm = np.ascontiguousarray(perm, dtype=np.uint64)
    out = np.empty((n, w), dtype=np.int32)
    lib().fvo_inflate(_p(corpus), _p(starts), _p(perm), first, n, w, V, _p(out))
    return out


def inflate_prune(corpus, starts, perm, first, n, w, V):
    """inflate() with the in-window duplicate pruning of the reference's (switched-off) device kernel."""
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    starts = np.ascontiguousarray(starts, dtype=np.uint64)
    perm = np.ascontiguousarray(perm, dtype=np.uint64)
    out = np.empty((n, w), dtype=np.int32)
    lib().fvo_inflate_prune(_p(corpus), _p(starts), _p(perm), first, n, w, V, _p(out))
    return out


def prune_windows(data):
    """The reference's host tool prune_input_data on a copy of an int32 (rows, cols) window matrix."""
    out = np.array(data, dtype=np.int32, order="C", copy=True)
    rows, cols = out.shape
    lib().fvo_prune_windows(_p(out), rows, cols)
    return out


def ref_prune_windows(data):
    """The same through the reference's own prune_input.cpp (oracle/_ref)."""
    out = np.array(data, dtype=np.int32, order="C", copy=True)
    rows, cols = out.shape
    ref_lib().prune_input_data(_p(out), rows, cols)
    return out


def activations(W, idx, invf):
    W = np.ascontiguousarray(W, dtype=np.float32)
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    invf = np.ascontiguousarray(invf, dtype=np.float32)
    K, N = W.shape
    n, w = idx.shape
    raw = np.empty((n, K), dtype=np.float32)
    sc = np.empty((n, K), dtype=np.float32)
    lib().fvo_activations(_p(W), K, N, _p(idx), n, w, _p(invf), len(invf), _p(raw), _p(sc))
    return raw, sc


def argmax_reference(row):
    row = np.ascontiguousarray(row, dtype=np.float32)
    return int(lib().fvo_argmax_reference(_p(row), len(row)))


def argmax_lowest(row):
    row = np.ascontiguousarray(row, dtype=np.float32)
    return int(lib().fvo_argmax_lowest(_p(row), len(row)))


def xx_sums(winners, sc, K, order_kind=0):
    """Per-neuron totals of the scaled activations; order_kind 0 = the step's order (64 interleaved
    partial sums), 1 = plain window order."""
    winners = np.ascontiguousarray(winners, dtype=np.int32)
    sc = np.ascontiguousarray(sc, dtype=np.float32)
    xx = np.empty(K, dtype=np.float32)
    lib().fvo_xx_sums(_p(winners), _p(sc), len(winners), K, order_kind, _p(xx))
    return xx


def epoch_eps(lr0, epoch, n_epochs):
    return float(lib().fvo_epoch_eps(lr0, epoch, n_epochs))


def epoch_delta(delta, epoch, n_epochs):
    return float(lib().fvo_epoch_delta(delta, epoch, n_epochs))


def train_step(W, idx, invf, eps, prec=1e-30, tie_rule=0, delta=0.0, lmid=1.0, lbase=1.0):
    """In-place step on W (K, 2V) fp32 C-order.  Returns dict(winners, sc, seconds, sc2, xx, nc, ds);
    delta is the anti-Hebbian strength of the step (0 = none), lmid / lbase weigh the centre and the
    context positions of a window (1 = the reference's command line)."""
    assert W.dtype == np.float32 and W.flags.c_contiguous
    idx = np.ascontiguousarray(idx, dtype=np.int32)
    invf = np.ascontiguousarray(invf, dtype=np.float32)
    K, N = W.shape
    n, w = idx.shape
    ds = np.empty((K, N), dtype=np.float32)
    win = np.empty(n, dtype=np.int32)
    sc = np.empty(n, dtype=np.float32)
    xx = np.empty(K, dtype=np.float32)
    nc = np.zeros(1, dtype=np.float32)
    win2 = np.empty(n, dtype=np.int32)
    sc2 = np.empty(n, dtype=np.float32)
    lib().fvo_train_step_weighted(_p(W), K, N, len(invf), _p(idx), n, w, _p(invf), eps, prec, tie_rule, delta,
                                  lmid, lbase, _p(ds), _p(win), _p(sc), _p(win2), _p(sc2), _p(xx), _p(nc))
    return dict(winners=win, sc=sc, seconds=win2, sc2=sc2, xx=xx, nc=float(nc[0]), ds=ds)


def train_steps(W, corpus, starts, perm, first, B, n_steps, w, invf, eps, prec=1e-30, tie_rule=0, delta=0.0,
                lmid=1.0, lbase=1.0, prune=False, stale_tail=False):
    """In-place n_steps minibatches; returns the winners of all processed windows. stale_tail: a final partial
    minibatch is trained with the previous minibatch's rows behind its own, as the reference does."""
    assert W.dtype == np.float32 and W.flags.c_contiguous
    corpus = np.ascontiguousarray(corpus, dtype=np.int32)
    starts = np.ascontiguousarray(starts, dtype=np.uint64)
    perm = np.ascontiguousarray(perm, dtype=np.uint64)
    invf = np.ascontiguousarray(invf, dtype=np.float32)
    K, N = W.shape
    V = N // 2
    nwin = len(perm)
    cap = max(0, min(n_steps * B, nwin - first))
    win = np.empty(cap, dtype=np.int32)
    done = lib().fvo_train_steps_tail(_p(W), K, V, _p(corpus), _p(starts), _p(perm), nwin, first, B, n_steps,
                                      w, _p(invf), eps, prec, tie_rule, delta, lmid, lbase, int(bool(prune)),
                                      int(bool(stale_tail)), _p(win))
    return win[:done]
