"""numpy restatement of the reference's hashing arithmetic.  TEST INFRASTRUCTURE ONLY.

The single-word rule is ``flyvec/core.py:153-158``:

    i_sorted = np.argsort(-act); act_sort = act[i_sorted]
    thr = (act_sort[k - 1] + act_sort[k]) / 2.0
    binary = (act > thr).astype(np.int8)

with ``act = synapses[:, n_vocab + tok_id]`` (``core.py:179``).  It is a
*threshold* code: with ties at the k / k+1 boundary fewer than k bits are set.

The windowed form (no counterpart in the reference, which only hashes one
target column) sums the window's columns sequentially in fp32, in window
order, skipping masked ids (-1), and applies the same threshold rule.

Pinned by tests/test_oracle_hash.py: brute force on small K against a
sort-free definition, popcount / nesting invariants, hand-made tie and
adjacent-float cases, and w = 1 reducing to the single-word rule.

Bit packing is this build's own definition: neuron h -> word h >> 6, bit
h & 63 (== ``np.packbits(code, bitorder="little")`` padded to whole uint64).
"""
import numpy as np


def sparse_code(act: np.ndarray, k: int) -> np.ndarray:
    """flyvec/core.py:155-158 on one activation vector (K,) fp32 -> (K,) int8."""
    act = np.asarray(act)
    i_sorted = np.argsort(-act)
    act_sort = act[i_sorted]
    thr = (act_sort[k - 1] + act_sort[k]) / 2.0  # IndexError when k >= K, as the reference
    return (act > thr).astype(np.int8)


def hash_targets_loop(W: np.ndarray, ids, k: int) -> np.ndarray:
    """The reference's only batch form (core.py:187-211): one Python call per id."""
    V = W.shape[1] // 2
    out = np.empty((len(ids), W.shape[0]), dtype=np.int8)
    for n, t in enumerate(ids):
        out[n] = sparse_code(W[:, V + int(t)], k)
    return out


def threshold_codes(act: np.ndarray, k: int) -> np.ndarray:
    """Vectorised form of the same rule on rows of act (n, K) fp32 -> (n, K) int8."""
    act = np.ascontiguousarray(act, dtype=np.float32)
    K = act.shape[1]
    if not 0 < k < K:
        raise IndexError("hash length must satisfy 0 < k < K")
    # descending order statistics k-1 and k (with multiplicity)
    part = np.partition(act, (K - k - 1, K - k), axis=1)
    a_k = part[:, K - k]
    a_k1 = part[:, K - k - 1]
    thr = (a_k + a_k1).astype(np.float32) * np.float32(0.5)
    return (act > thr[:, None]).astype(np.int8)


def hash_targets(W: np.ndarray, ids, k: int) -> np.ndarray:
    V = W.shape[1] // 2
    ids = np.asarray(ids, dtype=np.int64)
    return threshold_codes(W[:, V + ids].T, k)


def window_activations(W: np.ndarray, idx: np.ndarray) -> np.ndarray:
    """act[r] = sum over window positions in order of W[:, idx[r, c]], fp32, -1 skipped."""
    idx = np.asarray(idx)
    Wt = np.ascontiguousarray(W.T)  # (N, K): a column of W becomes a contiguous row
    act = np.zeros((idx.shape[0], W.shape[0]), dtype=np.float32)
    for c in range(idx.shape[1]):
        col = idx[:, c]
        ok = col >= 0
        rows = Wt[np.where(ok, col, 0)]
        rows[~ok] = 0.0
        act += rows  # elementwise fp32 add: one rounding per position, window order
    return act


def hash_windows(W: np.ndarray, idx: np.ndarray, k: int, chunk: int = 16384) -> np.ndarray:
    idx = np.asarray(idx)
    out = np.empty((idx.shape[0], W.shape[0]), dtype=np.int8)
    for s in range(0, idx.shape[0], chunk):
        out[s:s + chunk] = threshold_codes(window_activations(W, idx[s:s + chunk]), k)
    return out


def pack_codes(codes: np.ndarray) -> np.ndarray:
    """(n, K) 0/1 -> (n, ceil(K/64)) uint64, neuron h at word h>>6 bit h&63."""
    codes = np.asarray(codes, dtype=np.uint8)
    n, K = codes.shape
    words = (K + 63) // 64
    padded = np.zeros((n, words * 64), dtype=np.uint8)
    padded[:, :K] = codes
    by = np.packbits(padded, axis=1, bitorder="little")
    return np.ascontiguousarray(by).view("<u8").reshape(n, words)


def unpack_codes(words: np.ndarray, K: int) -> np.ndarray:
    words = np.ascontiguousarray(words, dtype="<u8")
    bits = np.unpackbits(words.view(np.uint8).reshape(words.shape[0], -1), axis=1, bitorder="little")
    return bits[:, :K].astype(np.int8)


def normalize_synapses(syn: np.ndarray, prec=1.0e-32, p=2) -> np.ndarray:
    """flyvec/core.py:23-36, statement for statement (numpy does the arithmetic)."""
    K, N = syn.shape
    nc = np.power(np.sum(syn ** p, axis=1), 1 / p).reshape(K, 1)
    return syn / np.tile(nc + prec, (1, N))


def pairwise_sum_f32(a: np.ndarray) -> np.float32:
    """numpy's float32 pairwise summation of one contiguous run, restated: blocks of at most 128
    elements are summed with 8 interleaved accumulators combined as ((r0+r1)+(r2+r3))+((r4+r5)+
    (r6+r7)) plus a sequential tail; longer ranges split at n/2 rounded down to a multiple of 8."""
    a = np.asarray(a, dtype=np.float32)
    n = len(a)
    if n < 8:
        res = np.float32(-0.0)
        for x in a:
            res = np.float32(res + x)
        return res
    if n <= 128:
        r = [np.float32(a[k]) for k in range(8)]
        i = 8
        while i < n - (n % 8):
            for k in range(8):
                r[k] = np.float32(r[k] + a[i + k])
            i += 8
        res = np.float32(np.float32(np.float32(r[0] + r[1]) + np.float32(r[2] + r[3])) +
                         np.float32(np.float32(r[4] + r[5]) + np.float32(r[6] + r[7])))
        while i < n:
            res = np.float32(res + a[i])
            i += 1
        return res
    n2 = n // 2
    n2 -= n2 % 8
    return np.float32(pairwise_sum_f32(a[:n2]) + pairwise_sum_f32(a[n2:]))


NUMPY_BUFSIZE = 8192  # numpy.getbufsize() default: add.reduce hands the inner loop runs of this many elements


def numpy_row_sum_f32(a: np.ndarray) -> np.float32:
    """numpy.sum of one contiguous float32 row, restated: starting from 0, the pairwise sum of each
    run of 8192 elements is added in order.  The device kernels of fv_hasher_row_sumsq follow this
    plan; the test-suite checks it against numpy.sum itself."""
    out = np.float32(0)
    for s in range(0, len(a), NUMPY_BUFSIZE):
        out = np.float32(out + pairwise_sum_f32(a[s:s + NUMPY_BUFSIZE]))
    return out
