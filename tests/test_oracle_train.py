"""Pins the training-step restatement (oracle/flyvec_oracle.c) without any import of the reference.

Nothing in the reference tests the trainer, so the C restatement is checked against
  * a from-scratch brute force of the same rule in Python scalars on tiny shapes,
  * numpy restatements of the sampler and the activations,
  * closed forms: one-window batch, W = 0 fixed point, invariance to rescaling 1/frequency by a
    power of two, max|dW| == eps, rows changed == distinct winners with a non-zero total, masked
    ids contribute nothing,
  * for the reference's argmax reduction order, a second derivation (closed-form priority key)
    of what the literal 64-thread simulation in C computes.
"""
import numpy as np
import pytest

from oracle import train_oracle as to

f32 = np.float32


# ---- brute force ---------------------------------------------------------------------------------

def brute_argmax_lowest(raw):
    best = 0
    for i in range(1, len(raw)):
        if raw[i] > raw[best]:
            best = i
    return best


def brute_step(W, idx, invf, eps, prec, argmax=brute_argmax_lowest, delta=0.0, lmid=1.0, lbase=1.0):
    """flyvec/src/cuda_funcs.cu:1662-1803 (sparse, frequency scaling) in Python scalars. With
    delta != 0 the second neuron of every window (the search repeated with the winner's activation
    overwritten by -9999.9999, :495-548) receives the anti-Hebbian terms (:668, :726-734); their
    place in the order of additions: after the Hebbian ones. lmid / lbase weigh the centre position and
    the others (:266-286, :307-327, :675-697)."""
    W = W.copy()
    K, N = W.shape
    V = N // 2
    n, w = idx.shape
    delta = f32(delta)
    L = [f32(lmid) if c == w // 2 else f32(lbase) for c in range(w)]

    def scaled(h, r):
        ss = 0.0
        for c in range(w):
            i = idx[r, c]
            if i != -1:
                ss += float(f32(f32(W[h, i] * L[c]) * invf[i % V]))  # fp32 products, double sum
        return f32(ss)

    win, sc, win2, sc2 = [], [], [], []
    for r in range(n):
        raw = []
        for h in range(K):
            s = 0.0  # double accumulator
            for c in range(w):
                i = idx[r, c]
                if i != -1:
                    s += float(f32(W[h, i] * L[c]))
            raw.append(f32(s))
        b = argmax(raw)
        win.append(b)
        sc.append(scaled(b, r))
        if delta != 0:
            raw[b] = f32(-9999.9999)
            b2 = argmax(raw)
            win2.append(b2)
            sc2.append(scaled(b2, r))
    xx = [f32(0)] * K
    for r in range(n):
        xx[win[r]] = f32(xx[win[r]] + sc[r])
    if delta != 0:
        xx2 = [f32(0)] * K
        for r in range(n):
            xx2[win2[r]] = f32(xx2[win2[r]] + f32(-delta * sc2[r]))
        xx = [f32(a + b) for a, b in zip(xx, xx2)]
    ds = np.zeros((K, N), dtype=f32)
    for h in range(K):
        if xx[h] != 0:
            for c in range(N):
                ds[h, c] = f32(-xx[h]) * W[h, c]
    for r in range(n):
        for c in range(w):
            i = idx[r, c]
            if i != -1:
                ds[win[r], i] = f32(ds[win[r], i] + f32(float(L[c]) * float(invf[i % V])))  # double product
    if delta != 0:
        for r in range(n):
            for c in range(w):
                i = idx[r, c]
                if i != -1:
                    ds[win2[r], i] = f32(ds[win2[r], i] + f32(f32(-delta * L[c]) * invf[i % V]))
    nc = f32(0)
    for h in range(K):
        if xx[h] != 0:
            nc = max(nc, f32(np.max(np.abs(ds[h]))))
        else:
            ds[h] = 0
    s = f32(eps) / f32(prec) if f32(prec) > nc else f32(eps) / nc
    for h in range(K):
        if xx[h] != 0:
            for c in range(N):
                v = f32(s * ds[h, c])
                if abs(float(v)) > 1.0e-10:
                    W[h, c] = f32(W[h, c] + v)
    if delta != 0:
        return W, np.array(win, dtype=np.int32), np.array(xx, dtype=f32), float(nc), np.array(win2, dtype=np.int32)
    return W, np.array(win, dtype=np.int32), np.array(xx, dtype=f32), float(nc)


@pytest.mark.parametrize("seed", range(8))
def test_step_against_brute_force(seed):
    rng = np.random.default_rng(seed)
    K, V, w, n = int(rng.integers(2, 5)), int(rng.integers(3, 7)), 3, int(rng.integers(1, 9))
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, V, size=(n, w)).astype(np.int32)
    idx[:, w // 2] += V
    idx[rng.random((n, w)) < 0.15] = -1
    invf = (1.0 / rng.integers(1, 50, size=V)).astype(f32)
    eps, prec = 2e-2, 1e-30
    want_W, want_win, want_xx, want_nc = brute_step(W, idx, invf, eps, prec)
    got_W = W.copy()
    res = to.train_step(got_W, idx, invf, eps, prec, tie_rule=0)
    assert np.array_equal(res["winners"], want_win)
    assert np.array_equal(res["xx"], want_xx)
    assert res["nc"] == want_nc
    assert np.array_equal(got_W, want_W)


# ---- stages against numpy ----------------------------------------------------------------------------

def test_inflate_against_numpy():
    rng = np.random.default_rng(1)
    V, w = 50, 5
    corpus = rng.integers(0, V, size=2000).astype(np.int32)
    corpus[rng.integers(0, 2000, 50)] = -1
    starts = np.sort(rng.integers(0, 2000 - w, size=300)).astype(np.uint64)
    perm = rng.permutation(300).astype(np.uint64)
    got = to.inflate(corpus, starts, perm, 20, 100, w, V)
    want = np.stack([corpus[int(starts[p]):int(starts[p]) + w] for p in perm[20:120]]).copy()
    mid = want[:, w // 2]
    want[:, w // 2] = np.where(mid == -1, -1, mid + V)  # centre column goes to the target block
    assert np.array_equal(got, want)


def test_activations_against_numpy():
    rng = np.random.default_rng(2)
    K, V, w, n = 37, 40, 7, 64
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, 2 * V, size=(n, w)).astype(np.int32)
    idx[rng.random((n, w)) < 0.1] = -1
    invf = rng.random(V).astype(f32)
    raw, sc = to.activations(W, idx, invf)
    ok = idx >= 0
    cols = np.where(ok, idx, 0)
    g = W[:, cols]                                  # (K, n, w) fp32
    want_raw = np.zeros((K, n))
    want_sc = np.zeros((K, n))
    for c in range(w):                               # double accumulation in window order
        want_raw += np.where(ok[:, c], g[:, :, c].astype(np.float64), 0.0)
        prod = (g[:, :, c] * invf[cols[:, c] % V]).astype(f32)   # fp32 product
        want_sc += np.where(ok[:, c], prod.astype(np.float64), 0.0)
    assert np.array_equal(raw, want_raw.T.astype(f32))
    assert np.array_equal(sc, want_sc.T.astype(f32))


def test_eps_schedule():
    # flyvec/src/cuda_funcs.cu:1229: fp32 ratio, double product, one rounding
    for lr0, ep, nep in [(2e-4, 0, 15), (2e-4, 7, 15), (0.002, 14, 15), (0.002, 3, 7)]:
        want = f32(float(f32(lr0)) * (1.0 - float(f32(f32(ep) / f32(nep)))))
        assert to.epoch_eps(lr0, ep, nep) == want


# ---- argmax tie rules ------------------------------------------------------------------------------------

def reference_priority(h):
    """Closed form of the reduction order of flyvec/src/cuda_funcs.cu:488-561: thread t = h % 64
    scans h = t, t+64, ...; warp 0 beats warp 1; inside a warp the shuffle-down tree with a strict
    comparison prefers lanes in bit-reversed order; index 0 seeds every thread."""
    if h == 0:
        return (-1, 0, 0)
    t, q = h % 64, h // 64
    rev = int(f"{t % 32:05b}"[::-1], 2)
    return (t // 32, rev, q)


def argmax_by_priority(row):
    m = max(row)
    return min((h for h in range(len(row)) if row[h] == m), key=reference_priority)


def test_reference_tie_rule_examples():
    K = 400
    row = np.zeros(K, dtype=f32)
    assert to.argmax_reference(row) == 0          # all equal
    row[:] = -1
    row[1] = row[2] = 5                              # lane 2 (bit-reversed 8) beats lane 1 (16)
    assert to.argmax_reference(row) == 2 and to.argmax_lowest(row) == 1
    row[:] = -1
    row[67] = row[5] = 5                             # lane 5 (reversed 20) beats lane 3 (24)
    assert to.argmax_reference(row) == 5
    row[:] = -1
    row[40] = row[33] = 5                            # warp 1 lanes: 8 -> 2, 1 -> 16
    assert to.argmax_reference(row) == 40
    row[:] = -1
    row[0] = row[17] = 5                             # the seed (data[0], 0) is never replaced by an equal
    assert to.argmax_reference(row) == 0
    row[:] = -1
    row[64 + 9] = row[9] = 5                         # same thread: the lower index is met first
    assert to.argmax_reference(row) == 9


@pytest.mark.parametrize("K", [1, 5, 63, 64, 65, 130, 400, 1000])
def test_reference_tie_rule_against_closed_form(K):
    rng = np.random.default_rng(K)
    for _ in range(200):
        row = rng.integers(0, 4, size=K).astype(f32)  # few distinct values: ties everywhere
        assert to.argmax_reference(row) == argmax_by_priority(list(row))
        assert to.argmax_lowest(row) == int(np.argmax(row))
    for _ in range(50):
        row = rng.standard_normal(K).astype(f32)      # no ties: every rule is plain argmax
        assert to.argmax_reference(row) == int(np.argmax(row)) == to.argmax_lowest(row)


# ---- closed forms ---------------------------------------------------------------------------------------------

def setup_small(seed, K=16, V=30, w=5, n=40):
    rng = np.random.default_rng(seed)
    W = (0.1 * rng.standard_normal((K, 2 * V))).astype(f32)
    idx = rng.integers(0, V, size=(n, w)).astype(np.int32)
    idx[:, w // 2] += V
    invf = (1.0 / rng.integers(1, 200, size=V)).astype(f32)
    return W, idx, invf


def test_single_window_closed_form():
    W, idx, invf = setup_small(0, n=1)
    V = W.shape[1] // 2
    W0 = W.copy()
    res = to.train_step(W, idx, invf, 1e-3)
    mu = int(res["winners"][0])
    raw = W0[:, idx[0]].astype(np.float64).sum(axis=1).astype(f32)
    assert mu == int(np.argmax(raw))
    sc = f32((W0[mu, idx[0]] * invf[idx[0] % V]).astype(f32).astype(np.float64).sum())
    assert res["xx"][mu] == sc and np.count_nonzero(res["xx"]) == 1
    ds = f32(-sc) * W0[mu]
    for i in idx[0]:
        ds[i] = f32(ds[i] + invf[i % V])
    assert np.array_equal(res["ds"][mu], ds)
    changed = np.flatnonzero((W != W0).any(axis=1))
    assert changed.tolist() == [mu]                  # every other row untouched


def test_zero_matrix_is_a_fixed_point():
    W, idx, invf = setup_small(1)
    W[:] = 0
    res = to.train_step(W, idx, invf, 1e-3)
    assert not W.any() and res["nc"] == 0.0 and not res["xx"].any()
    assert (res["winners"] == 0).all()               # all-equal activations: index 0 under both rules


def test_rows_changed_are_the_winners_and_step_size_is_eps():
    W, idx, invf = setup_small(2)
    W0 = W.copy()
    eps = 1e-3
    res = to.train_step(W, idx, invf, eps)
    won = np.unique(res["winners"])
    won = won[res["xx"][won] != 0]
    assert np.flatnonzero((W != W0).any(axis=1)).tolist() == won.tolist()
    assert res["nc"] == np.abs(res["ds"]).max()
    assert abs(np.abs(W - W0).max() - eps) <= 2e-7 * max(1.0, np.abs(W0).max())  # s * nc == eps up to rounding


def test_invariant_to_power_of_two_rescale_of_inverse_frequency():
    # xx and the sparse term are both linear in 1/f and max|ds| divides the scale out; a power of
    # two makes every intermediate scale exactly
    W, idx, invf = setup_small(3)
    Wa, Wb = W.copy(), W.copy()
    ra = to.train_step(Wa, idx, invf, 1e-3)
    rb = to.train_step(Wb, idx, (invf * f32(8)).astype(f32), 1e-3)
    assert np.array_equal(ra["winners"], rb["winners"])
    assert np.array_equal(rb["xx"], ra["xx"] * f32(8)) and rb["nc"] == ra["nc"] * 8
    assert np.array_equal(Wa, Wb)


def test_masked_positions_contribute_nothing():
    W, idx, invf = setup_small(4)
    V = W.shape[1] // 2
    # a column nobody else uses, then mask it: same result as if those windows were shorter
    idx2 = idx.copy()
    idx2[:, 0] = -1
    Wa = W.copy()
    ra = to.train_step(Wa, idx2, invf, 1e-3)
    Wz = W.copy()
    Wz[:, V - 1] = 0                                   # a zero column adds exactly 0 to every sum ...
    idx3 = idx.copy()
    idx3[:, 0] = V - 1
    invf3 = invf.copy()
    invf3[V - 1] = 0                                   # ... and a zero 1/f adds 0 to ds
    idx3[idx3 == V - 1] = V - 1
    keep = ~(idx[:, 1:] == V - 1).any(axis=1)          # windows that do not otherwise use that column
    Wb = Wz.copy()
    rb = to.train_step(Wb, idx3[keep], invf3, 1e-3)
    Wc = Wz.copy()
    rc = to.train_step(Wc, idx2[keep], invf3, 1e-3)
    assert np.array_equal(rb["winners"], rc["winners"]) and np.array_equal(Wb, Wc)
    assert ra["winners"].shape[0] == idx.shape[0]


def test_multi_step_driver_matches_single_steps():
    rng = np.random.default_rng(7)
    V, K, w, B = 40, 12, 5, 16
    corpus = rng.integers(0, V, size=3000).astype(np.int32)
    off = np.concatenate([[0], np.cumsum(rng.geometric(1 / 20, size=200))]).astype(np.uint64)
    off = off[off <= 3000]
    starts = to.window_starts(off, w)
    perm = rng.permutation(len(starts)).astype(np.uint64)
    invf = to.inverse_frequency(corpus, V)
    W = (0.1 * rng.standard_normal((K, 2 * V))).astype(f32)
    Wa, Wb = W.copy(), W.copy()
    wins = to.train_steps(Wa, corpus, starts, perm, 0, B, 3, w, invf, 1e-3)
    got = []
    for s in range(3):
        idx = to.inflate(corpus, starts, perm, s * B, B, w, V)
        got.append(to.train_step(Wb, idx, invf, 1e-3)["winners"])
    assert np.array_equal(wins, np.concatenate(got)) and np.array_equal(Wa, Wb)
    # last partial batch: only the remainder is processed
    tail = len(perm) - (len(perm) // B) * B
    if tail:
        wt = to.train_steps(Wa, corpus, starts, perm, (len(perm) // B) * B, B, 1, w, invf, 1e-3)
        assert len(wt) == tail


# ---- order of the per-neuron totals ---------------------------------------------------------------

def xx_numpy(winners, sc, K):
    """The step's order, restated: the rows in groups of 64; a neuron's values of a group are added in row order
    (np.cumsum in float32 adds strictly left to right), and the array of group sums, padded with zeros to a power
    of two, is halved by adding neighbours until one value is left."""
    n = len(winners)
    G = max(1, -(-n // 64))
    size = 1
    while size < G:
        size *= 2
    out = np.zeros(K, dtype=f32)
    for h in range(K):
        P = np.zeros(size, dtype=f32)
        for g in range(G):
            rows = slice(64 * g, min(64 * g + 64, n))
            v = sc[rows][winners[rows] == h]
            if len(v):
                P[g] = np.cumsum(v, dtype=f32)[-1]
        while len(P) > 1:
            P = (P[0::2] + P[1::2]).astype(f32)
        out[h] = P[0]
    return out


@pytest.mark.parametrize("n,K", [(1, 3), (50, 4), (64, 1), (65, 1), (129, 2), (5000, 7), (10000, 400), (40000, 3), (65537, 2)])
def test_xx_order_against_numpy(n, K):
    rng = np.random.default_rng(n + K)
    winners = rng.integers(0, K, size=n).astype(np.int32)
    sc = (rng.standard_normal(n) * 10.0 ** rng.uniform(-3, 1, n)).astype(f32)
    assert np.array_equal(to.xx_sums(winners, sc, K, 0), xx_numpy(winners, sc, K))
    seq = np.zeros(K, dtype=f32)
    for r in range(n):
        seq[winners[r]] = f32(seq[winners[r]] + sc[r])
    assert np.array_equal(to.xx_sums(winners, sc, K, 1), seq)


def test_xx_order_is_row_order_where_the_tree_is_a_chain_and_close_elsewhere():
    rng = np.random.default_rng(5)
    # one group: the plain sum in row order
    winners = rng.integers(0, 5, size=64).astype(np.int32)
    sc = rng.standard_normal(64).astype(f32)
    assert np.array_equal(to.xx_sums(winners, sc, 5, 0), to.xx_sums(winners, sc, 5, 1))
    # two groups, and a neuron that wins the whole first group and one window of the second: P_0 + P_1 is the sum
    # in row order
    winners = np.ones(128, dtype=np.int32)
    winners[:64] = 0
    winners[64 + 5] = 0
    sc = rng.standard_normal(128).astype(f32)
    assert to.xx_sums(winners, sc, 2, 0)[0] == to.xx_sums(winners, sc, 2, 1)[0]
    # one value per group in groups 0, 1, 2, 4: ((a + b) + (c + 0)) + ((d + 0) + 0) = ((a + b) + c) + d
    winners = np.ones(5 * 64, dtype=np.int32)
    winners[[3, 64 + 9, 128 + 63, 256]] = 0
    sc = rng.standard_normal(len(winners)).astype(f32)
    a, b, c, d = sc[[3, 64 + 9, 128 + 63, 256]]
    want = f32(f32(f32(a + b) + c) + d)
    assert to.xx_sums(winners, sc, 2, 0)[0] == want == to.xx_sums(winners, sc, 2, 1)[0]
    # one value per group in groups 1, 2, 3: (0 + a) + (b + c), which is not the sum in row order
    winners = np.ones(4 * 64, dtype=np.int32)
    winners[[64, 128, 192]] = 0
    sc = np.array([0.1] * 256, dtype=f32)
    sc[[64, 128, 192]] = [f32(1.0), f32(2.0 ** -24), f32(2.0 ** -24)]
    assert to.xx_sums(winners, sc, 2, 0)[0] == f32(f32(1.0) + f32(2.0 ** -23))       # b + c first: it survives
    assert to.xx_sums(winners, sc, 2, 1)[0] == f32(1.0)                               # one by one both are lost
    # a sum that starts at +0 is never -0, whatever it adds
    winners = np.zeros(70, dtype=np.int32)
    sc = np.full(70, -0.0, dtype=f32)
    assert not np.signbit(to.xx_sums(winners, sc, 1, 0)[0])
    # many windows: the two orders differ, by rounding only
    winners = rng.integers(0, 3, size=30000).astype(np.int32)
    sc = np.abs(rng.standard_normal(30000)).astype(f32)
    a, b = to.xx_sums(winners, sc, 3, 0), to.xx_sums(winners, sc, 3, 1)
    exact = np.array([sc[winners == h].astype(np.float64).sum() for h in range(3)])
    assert not np.array_equal(a, b)                              # the orders do differ ...
    assert np.all(np.abs(a - exact) <= 2e-5 * exact)             # ... by rounding only
    assert np.all(np.abs(b - exact) <= 2e-5 * exact)


def test_step_uses_the_grouped_order():
    rng = np.random.default_rng(8)
    K, V, w, n = 3, 30, 5, 2000
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, V, size=(n, w)).astype(np.int32)
    idx[:, w // 2] += V
    invf = (1.0 / rng.integers(1, 50, size=V)).astype(f32)
    res = to.train_step(W.copy(), idx, invf, 1e-3)
    assert np.bincount(res["winners"], minlength=K).max() > 64
    assert np.array_equal(res["xx"], xx_numpy(res["winners"], res["sc"], K))


# ---- anti-Hebbian term (delta != 0) -----------------------------------------------------------------

@pytest.mark.parametrize("seed", range(8))
def test_delta_step_against_brute_force(seed):
    rng = np.random.default_rng(100 + seed)
    K, V, w, n = int(rng.integers(1, 5)), int(rng.integers(3, 7)), 3, int(rng.integers(1, 9))
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, V, size=(n, w)).astype(np.int32)
    idx[:, w // 2] += V
    idx[rng.random((n, w)) < 0.15] = -1
    invf = (1.0 / rng.integers(1, 50, size=V)).astype(f32)
    eps, prec, delta = 2e-2, 1e-30, 0.4
    want_W, want_win, want_xx, want_nc, want_win2 = brute_step(W, idx, invf, eps, prec, delta=delta)
    got_W = W.copy()
    res = to.train_step(got_W, idx, invf, eps, prec, tie_rule=0, delta=delta)
    assert np.array_equal(res["winners"], want_win) and np.array_equal(res["seconds"], want_win2)
    assert np.array_equal(res["xx"], want_xx)
    assert res["nc"] == want_nc
    assert np.array_equal(got_W, want_W)


def test_delta_single_window_closed_form():
    W, idx, invf = setup_small(0, n=1)
    V = W.shape[1] // 2
    W0 = W.copy()
    delta = f32(0.25)
    res = to.train_step(W, idx, invf, 1e-3, delta=float(delta))
    mu, nu = int(res["winners"][0]), int(res["seconds"][0])
    raw = W0[:, idx[0]].astype(np.float64).sum(axis=1).astype(f32)
    assert mu == int(np.argmax(raw)) and mu != nu
    assert nu == int(np.argsort(-raw, kind="stable")[1])          # the runner-up of the window
    sc = lambda h: f32((W0[h, idx[0]] * invf[idx[0] % V]).astype(f32).astype(np.float64).sum())
    assert res["xx"][mu] == sc(mu) and res["xx"][nu] == f32(-delta * sc(nu)) and np.count_nonzero(res["xx"]) == 2
    ds_nu = f32(-res["xx"][nu]) * W0[nu]
    for i in idx[0]:
        ds_nu[i] = f32(ds_nu[i] + f32(-delta * invf[i % V]))
    assert np.array_equal(res["ds"][nu], ds_nu)
    changed = np.flatnonzero((W != W0).any(axis=1))
    assert sorted(changed.tolist()) == sorted([mu, nu])


def test_delta_zero_is_the_plain_step_and_one_neuron_meets_itself():
    W, idx, invf = setup_small(5)
    Wa, Wb = W.copy(), W.copy()
    ra = to.train_step(Wa, idx, invf, 1e-3)
    rb = to.train_step(Wb, idx, invf, 1e-3, delta=0.0)
    assert np.array_equal(Wa, Wb) and np.array_equal(ra["winners"], rb["winners"])
    # with a single neuron the second search finds the same neuron again: it receives both terms
    rng = np.random.default_rng(2)
    W1 = rng.standard_normal((1, 12)).astype(f32)
    idx1 = np.array([[1, 8, 3]], dtype=np.int32)
    invf1 = np.full(6, 0.5, dtype=f32)
    want = brute_step(W1, idx1, invf1, 1e-2, 1e-30, delta=0.3)
    got = W1.copy()
    res = to.train_step(got, idx1, invf1, 1e-2, delta=0.3)
    assert res["seconds"][0] == 0 and np.array_equal(got, want[0])


def test_epoch_delta_schedule():
    # flyvec/src/cuda_funcs.cu:1230: delta * 0.5 * (1 + tanh((ep - 0.125 Nep) / 10)), rounded to fp32 once
    import math
    for delta, ep, nep in [(0.4, 0, 15), (0.4, 7, 15), (0.4, 14, 15), (1.0, 100, 200), (0.0, 3, 15)]:
        want = f32(float(f32(delta)) * 0.5 * (1.0 + math.tanh((float(f32(ep)) - 0.125 * nep) / 10.0)))
        assert to.epoch_delta(delta, ep, nep) == want


# ---- position weights Lmid / Lbase -------------------------------------------------------------------

@pytest.mark.parametrize("seed", range(8))
def test_weighted_step_against_brute_force(seed):
    rng = np.random.default_rng(300 + seed)
    K, V, w, n = int(rng.integers(1, 5)), int(rng.integers(3, 7)), int(rng.choice([1, 3, 4])), int(rng.integers(1, 9))
    W = rng.standard_normal((K, 2 * V)).astype(f32)
    idx = rng.integers(0, V, size=(n, w)).astype(np.int32)
    idx[:, w // 2] += V
    idx[rng.random((n, w)) < 0.15] = -1
    invf = (1.0 / rng.integers(1, 50, size=V)).astype(f32)
    delta = 0.0 if seed % 2 == 0 else 0.3
    lmid, lbase = float(f32(rng.uniform(0.2, 3.0))), float(f32(rng.uniform(0.2, 3.0)))
    want = brute_step(W, idx, invf, 2e-2, 1e-30, delta=delta, lmid=lmid, lbase=lbase)
    got_W = W.copy()
    res = to.train_step(got_W, idx, invf, 2e-2, 1e-30, tie_rule=0, delta=delta, lmid=lmid, lbase=lbase)
    assert np.array_equal(res["winners"], want[1])
    assert np.array_equal(res["xx"], want[2]) and res["nc"] == want[3]
    assert np.array_equal(got_W, want[0])
    if delta:
        assert np.array_equal(res["seconds"], want[4])


def test_unit_weights_are_the_plain_step_and_a_power_of_two_changes_nothing():
    W, idx, invf = setup_small(3)
    Wa, Wb, Wc = W.copy(), W.copy(), W.copy()
    ra = to.train_step(Wa, idx, invf, 1e-3, delta=0.2)
    rb = to.train_step(Wb, idx, invf, 1e-3, delta=0.2, lmid=1.0, lbase=1.0)
    assert np.array_equal(Wa, Wb) and np.array_equal(ra["xx"], rb["xx"])
    # Lmid = Lbase = 4: activations, xx and ds are all 4x (exactly: a power of two), max|ds| is 4x, the
    # scale eps / max|ds| is a quarter: the same update bit for bit
    rc = to.train_step(Wc, idx, invf, 1e-3, delta=0.2, lmid=4.0, lbase=4.0)
    assert np.array_equal(rc["winners"], ra["winners"]) and np.array_equal(rc["seconds"], ra["seconds"])
    assert np.array_equal(rc["xx"], ra["xx"] * f32(4)) and rc["nc"] == ra["nc"] * 4
    assert np.array_equal(Wc, Wa)


def test_a_zero_weight_is_a_masked_position():
    """Lmid = 0 removes the centre from both activations and adds 0 to ds there: the step on the same
    windows with the centre masked (-1).  Lbase = 0: the step with every context position masked."""
    W, idx, invf = setup_small(7, n=6)
    w = idx.shape[1]
    mid = w // 2
    for lmid, lbase in [(0.0, 1.0), (1.0, 0.0)]:
        masked = idx.copy()
        if lmid == 0.0:
            masked[:, mid] = -1
        else:
            keep = masked[:, mid].copy()
            masked[:] = -1
            masked[:, mid] = keep
        Wa, Wb = W.copy(), W.copy()
        ra = to.train_step(Wa, idx, invf, 1e-3, lmid=lmid, lbase=lbase)
        rb = to.train_step(Wb, masked, invf, 1e-3)
        assert np.array_equal(ra["winners"], rb["winners"])
        assert np.array_equal(ra["xx"], rb["xx"]) and ra["nc"] == rb["nc"]
        assert np.array_equal(Wa, Wb)


def test_weights_reach_the_centre_and_the_context_separately():
    """One window: the winner is the argmax of Lmid * W[:, centre] + Lbase * sum of W[:, context];
    weights chosen so that the winner differs between (Lmid, Lbase) = (8, 1) and (1, 8)."""
    K, V = 2, 4
    W = np.zeros((K, 2 * V), dtype=f32)
    idx = np.array([[0, V + 1, 2]], dtype=np.int32)       # context 0, centre 1 (target block), context 2
    W[0, V + 1] = 1.0                                     # neuron 0 likes the centre token
    W[1, 0] = 0.75; W[1, 2] = 0.75                        # neuron 1 likes the context
    invf = np.full(V, 0.5, dtype=f32)
    for lmid, lbase, want in [(8.0, 1.0, 0), (1.0, 8.0, 1), (1.0, 1.0, 1)]:
        Wc = W.copy()
        res = to.train_step(Wc, idx, invf, 1e-3, lmid=lmid, lbase=lbase)
        assert int(res["winners"][0]) == want
        raw = lmid * W[:, V + 1] + lbase * (W[:, 0] + W[:, 2])
        assert want == int(np.argmax(raw))
        # the sparse term of the winner's row: L * 1/f per position, on top of -xx * W
        h = want
        ds = f32(-res["xx"][h]) * W[h]
        for c, i in enumerate(idx[0]):
            ds[i] = f32(ds[i] + f32((lmid if c == 1 else lbase) * 0.5))
        assert np.array_equal(res["ds"][h], ds)


# ---- in-window duplicate pruning ---------------------------------------------------------------------

def first_occurrence_mask(tokens_row, include_centre, mid):
    """True where a position holds a token that no EARLIER position holds (the centre counted among the
    earlier ones or not), written with sets, not with the reference's nested scan."""
    seen, keep = set(), []
    for c, t in enumerate(tokens_row):
        keep.append(t not in seen)
        if c != mid or include_centre:
            seen.add(t)
    return keep


def test_prune_windows_matches_the_reference_tool():
    """fvo_prune_windows against the reference's own prune_input_data (compiled into oracle/_ref)."""
    if to.ref_lib() is None:
        pytest.skip("oracle/_ref not built")
    rng = np.random.default_rng(0)
    for cols in (1, 2, 3, 4, 11, 16):
        data = rng.integers(-1, 6, size=(200, cols)).astype(np.int32)
        assert np.array_equal(to.prune_windows(data), to.ref_prune_windows(data)), cols
    data = rng.integers(0, 3, size=(50, 11)).astype(np.int32)     # many duplicates
    assert np.array_equal(to.prune_windows(data), to.ref_prune_windows(data))


def test_prune_windows_golden_fixture_from_reference_build():
    """tests/golden/prune_windows.npz was written by tests/golden/make_prune_windows.py from the reference's own
    prune_input_data; it travels to machines where neither the reference nor its build is present."""
    import os
    z = np.load(os.path.join(os.path.dirname(__file__), "golden", "prune_windows.npz"))
    for k in range(int(z["n_cases"])):
        assert np.array_equal(to.prune_windows(z[f"in_{k}"]), z[f"out_{k}"]), k
    assert z["out_7"].tolist() == [[7, -1, 7, -1, -1], [1, 2, 1, -1, -1], [-1, 3, -1, -1, -1], [4, 5, 6, -1, -1]]


def test_prune_windows_keeps_first_occurrences():
    rng = np.random.default_rng(1)
    for cols in (1, 5, 11):
        data = rng.integers(0, 7, size=(100, cols)).astype(np.int32)
        out = to.prune_windows(data)
        mid = cols // 2
        for row, got in zip(data, out):
            keep = first_occurrence_mask(row.tolist(), False, mid)
            want = [t if (k or c == mid) else -1 for c, (t, k) in enumerate(zip(row.tolist(), keep))]
            assert got.tolist() == want


def test_inflate_prune_keeps_first_occurrences_and_the_centre():
    rng = np.random.default_rng(2)
    V, w = 6, 7
    corpus = rng.integers(0, V, size=400).astype(np.int32)
    corpus[rng.random(400) < 0.1] = -1
    starts = np.arange(0, 400 - w, dtype=np.uint64)
    perm = rng.permutation(len(starts)).astype(np.uint64)
    got = to.inflate_prune(corpus, starts, perm, 3, 200, w, V)
    plain = to.inflate(corpus, starts, perm, 3, 200, w, V)
    mid = w // 2
    for r in range(200):
        row = corpus[int(starts[perm[3 + r]]):][:w].tolist()
        keep = first_occurrence_mask(row, True, mid)
        for c in range(w):
            if c == mid:
                assert got[r, c] == plain[r, c]                   # the centre always survives
            elif row[c] != -1 and keep[c]:
                assert got[r, c] == plain[r, c]
            else:
                assert got[r, c] == -1
    # a window without repeated tokens is untouched
    corpus2 = np.arange(50, dtype=np.int32) % 40
    st2 = np.arange(0, 30, dtype=np.uint64)
    assert np.array_equal(to.inflate_prune(corpus2, st2, st2, 0, 30, w, 40), to.inflate(corpus2, st2, st2, 0, 30, w, 40))


@pytest.mark.parametrize("prune", [False, True])
def test_stale_tail_reuses_the_previous_minibatch_rows(prune):
    """flyvec/src/cuda_funcs.cu:1679 samples only the remainder of a final partial minibatch while :1700-1732
    run on all Num rows: the rows behind the remainder are the previous minibatch's. The multi-step driver's
    stale_tail mode must equal the single step run on that index matrix assembled by hand; without a full
    minibatch before it, and with the mode off, the remainder alone is trained."""
    from flyvec_amd import synthetic
    V, K, w, B = 60, 9, 5, 64
    tokens, offsets = synthetic.corpus(4000, V if not prune else 12, mean_chunk=14)
    tokens[-1] = min(V, tokens.max() + 1) - 1
    starts = to.window_starts(offsets, w)
    invf = to.inverse_frequency(tokens, V)
    perm = np.random.default_rng(2).permutation(len(starts)).astype(np.uint64)
    n_win = 2 * B + 23                                   # two full minibatches and a remainder of 23
    perm = perm[:n_win].copy()
    W0 = synthetic.synapses(K, V, seed=3, sigma=0.3)
    inflate = to.inflate_prune if prune else to.inflate
    # by hand: two full steps, then the last on [23 new rows ; rows 23.. of the second minibatch]
    Wh = W0.copy()
    for j in range(2):
        to.train_step(Wh, inflate(tokens, starts, perm, j * B, B, w, V), invf, 1e-2)
    plain = Wh.copy()
    idx = inflate(tokens, starts, perm, B, B, w, V).copy()
    idx[:23] = inflate(tokens, starts, perm, 2 * B, 23, w, V)
    ref = to.train_step(Wh, idx, invf, 1e-2)
    to.train_step(plain, idx[:23], invf, 1e-2)
    Ws = W0.copy()
    win = to.train_steps(Ws, tokens, starts, perm, 0, B, 3, w, invf, 1e-2, prune=prune, stale_tail=True)
    assert np.array_equal(Ws.view(np.uint32), Wh.view(np.uint32)) and not np.array_equal(Ws, plain)
    assert len(win) == n_win and np.array_equal(win[2 * B:], ref["winners"][:23])
    Wp = W0.copy()
    to.train_steps(Wp, tokens, starts, perm, 0, B, 3, w, invf, 1e-2, prune=prune)
    assert np.array_equal(Wp.view(np.uint32), plain.view(np.uint32))
    # no full minibatch before the partial one: the remainder alone, in both modes
    a, b = W0.copy(), W0.copy()
    to.train_steps(a, tokens, starts, perm[:23].copy(), 0, B, 1, w, invf, 1e-2, prune=prune, stale_tail=True)
    to.train_step(b, inflate(tokens, starts, perm, 0, 23, w, V), invf, 1e-2)
    assert np.array_equal(a.view(np.uint32), b.view(np.uint32))
