"""Parity of the HIP training step against the CPU checker, through the C ABI.

The step is deterministic by construction (window-ordered xx, count-based sparse term), so the
comparison is bit for bit: identical winners and identical W.  The bars the task states
(winners >= 99.9 %, relative L2 of W <= 1e-4 after 100 steps) are asserted as well, at the
benchmark's full size."""
import functools

import numpy as np
import pytest

from conftest import small_corpus

pytestmark = pytest.mark.gpu

f32 = np.float32


def make_trainer(tokens, offsets, V, K, w, B, W0, tie=0, lr0=2e-4, perm_seed=6, prec=1e-30, launches=0):
    from flyvec_amd import Trainer
    t = Trainer(V, K, w, B, initial_learning_rate=lr0, tie_rule=tie, prec=prec)
    t.set_dense_launches(launches)  # 0: as chosen at creation, 1 / 2: both passes over W in one launch / in two
    t.set_corpus(tokens, offsets)
    perm = np.random.default_rng(perm_seed).permutation(t.num_windows).astype(np.uint64)
    t.set_permutation(perm)
    t.set_weights(W0)
    return t, perm


def oracle_inputs(to, tokens, offsets, V, w):
    return to.window_starts(offsets, w), to.inverse_frequency(tokens, V)


def run_both(gpu, oracle_lib, V, K, w, B, steps, tie=0, sigma=0.02, n_tokens=60000, W0=None, lr0=2e-4,
             mean_chunk=25, n_masked=40, seed=0, launches=0):
    from flyvec_amd import synthetic
    to = oracle_lib
    tokens, offsets = small_corpus(n_tokens, V, seed=seed, mean_chunk=mean_chunk, n_masked=n_masked)
    if W0 is None:
        W0 = synthetic.synapses(K, V, seed=5 + seed, sigma=sigma)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, tie=tie, lr0=lr0, launches=launches)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    assert t.num_windows == len(starts)
    eps = t.epoch_eps(0, 15)
    assert eps == to.epoch_eps(lr0, 0, 15)
    wins = []
    steps = min(steps, t.num_windows // B)
    for s in range(steps):
        t.step(s * B, B, eps)
        wins.append(t.winners(B))
    Wg = t.get_weights()
    Wo = W0.copy()
    wo = to.train_steps(Wo, tokens, starts, perm, 0, B, steps, w, invf, eps, tie_rule=tie)
    t.close()
    return np.concatenate(wins), wo, Wg, Wo


@pytest.mark.parametrize("launches", [1, 2, 3])
@pytest.mark.parametrize("tie", [0, 1])
def test_small_config_bit_exact(gpu, oracle_lib, tie, launches):
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=500, K=400, w=11, B=512, steps=30, tie=tie, launches=launches)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("K,w,V,B", [(1, 1, 5, 1), (3, 2, 7, 3), (5, 3, 40, 64), (63, 1, 100, 128), (64, 5, 100, 100), (65, 15, 200, 256),
                                     (130, 64, 300, 64), (1000, 15, 300, 512), (2048, 7, 64, 128),
                                     (30, 11, 20000, 700), (30, 11, 30000, 700), (3, 5, 400000, 300)])
def test_shapes_bit_exact(gpu, oracle_lib, K, w, V, B):
    # K not a multiple of 64 / 4, every lane-count template, w from 1 to 64; the last cases have more
    # columns per class than one pass over the LDS counters of the sparse kernel holds (2V / 4 > 10240)
    n_tokens = 40000 if V < 20000 else 120000
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=w, B=B, steps=6, n_tokens=n_tokens, mean_chunk=40)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("K,w,V,B", [(1, 1, 5, 1), (65, 15, 200, 256), (1000, 15, 300, 512), (2048, 7, 64, 128),
                                     (30, 11, 30000, 700), (200, 11, 20000, 2000), (400, 11, 20000, 3000),
                                     (400, 11, 20970, 3000), (3, 5, 400000, 300)])
def test_shapes_bit_exact_with_two_dense_launches(gpu, oracle_lib, K, w, V, B):
    # the shapes above take the single launch wherever the matrix fits the registers of the device;
    # here the same step with the maximum pass and the update as two launches, on matrices of every
    # size class of the single launch (4, 8, 12, 16 groups of 16 bytes per thread, and the largest that fits)
    n_tokens = 40000 if V < 20000 else 120000
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=w, B=B, steps=4, n_tokens=n_tokens, mean_chunk=40,
                              launches=2)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("K,w,V,B", [(1, 1, 5, 1), (65, 15, 200, 256), (1000, 15, 300, 512), (2048, 7, 64, 128),
                                     (30, 11, 30000, 700), (400, 11, 20970, 3000), (3, 5, 400000, 300),
                                     (600, 11, 40000, 2000)])
def test_shapes_bit_exact_with_the_rows_streamed_through_one_dense_launch(gpu, oracle_lib, K, w, V, B):
    # the single launch that keeps nothing in registers between its passes: rows of 1 to 2048 neurons, one round
    # of rows and many, matrices that fit the register form and one (192 MB) that does not
    n_tokens = 40000 if V < 20000 else 120000
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=w, B=B, steps=4, n_tokens=n_tokens, mean_chunk=40,
                              launches=3)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("K,V", [(200, 20000), (300, 20000), (400, 20000), (400, 20480)])
def test_single_dense_launch_size_classes(gpu, oracle_lib, K, V):
    # 32, 48, 64 and 65.5 MB of W: a thread of the single launch keeps 8, 12, 16 and 16 groups (40960 rows are the most: 256 blocks x 10 rows x 16)
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=11, B=3000, steps=4, n_tokens=120000, mean_chunk=40,
                              launches=1)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


def test_dense_launch_forms(gpu):
    from flyvec_amd import Trainer, _lib, synthetic
    V, K, w, B = 300, 64, 7, 128
    tokens, offsets = small_corpus(20000, V)
    W0 = synthetic.synapses(K, V)
    got = {}
    for launches in (1, 2, 3):
        t, _ = make_trainer(tokens, offsets, V, K, w, B, W0, launches=launches)
        assert t.dense_launches == min(launches, 2) or launches == 3 and t.dense_launches == 1
        for s in range(5):
            t.step(s * B, B, 1e-3)
        got[launches] = (t.get_weights(), t.step_stats()[1])
        t.close()
    assert np.array_equal(got[1][0], got[2][0]) and got[1][1] == got[2][1]
    assert np.array_equal(got[3][0], got[2][0]) and got[3][1] == got[2][1]
    # a matrix beyond the registers of the device: its single launch streams the rows
    big = Trainer(400000, 64, 5, 32)
    assert big.dense_launches == 1
    big.set_dense_launches(2)
    assert big.dense_launches == 2
    big.set_dense_launches(1)
    assert big.dense_launches == 1
    big.close()
    with pytest.raises(_lib.FlyvecError):
        Trainer(V, K, w, B).set_dense_launches(4)


@pytest.mark.parametrize("form", [1, 3])  # the matrix kept in registers between the passes / its rows streamed
def test_single_dense_launch_gives_up_cleanly(gpu, oracle_lib, form):
    """The wait between the two passes of the single launch is bounded. With a limit of zero rounds every block
    gives up at once (all kernels still run to their end): the step leaves W alone, the next synchronisation
    reports it, and the trainer carries on with two launches."""
    from flyvec_amd import _lib, synthetic
    to = oracle_lib
    V, K, w, B = 300, 64, 7, 128
    tokens, offsets = small_corpus(20000, V)
    W0 = synthetic.synapses(K, V)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, launches=form)
    t._set_wait_limit(0)
    t.step(0, B, 1e-3)
    with pytest.raises(_lib.FlyvecError) as e:
        t.sync()
    assert e.value.code == _lib.FV_ERR_STATE
    assert t.dense_launches == 2
    t.sync()                                   # reported once
    assert np.array_equal(t.get_weights(), W0)
    # the measurement hooks report it too: a figure over launches that neither waited nor updated is no figure
    t.set_dense_launches(form)
    with pytest.raises(_lib.FlyvecError) as e:
        t.time_steps(0, 3, 1e-3, per_kernel=False)
    assert e.value.code == _lib.FV_ERR_STATE
    t.set_dense_launches(form)
    with pytest.raises(_lib.FlyvecError) as e:
        t.time_steps_graph(0, 2, 1e-3, 1)
    assert e.value.code == _lib.FV_ERR_STATE
    assert np.array_equal(t.get_weights(), W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    for launches in (2, form):                 # usable afterwards, in either form
        t._set_wait_limit(1 << 14)
        t.set_dense_launches(launches)
        t.set_weights(W0)
        for s in range(3):
            t.step(s * B, B, 1e-3)
        Wo = W0.copy()
        to.train_steps(Wo, tokens, starts, perm, 0, B, 3, w, invf, 1e-3)
        assert np.array_equal(t.get_weights(), Wo)
    t.close()


@pytest.mark.parametrize("tie", [0, 1])
def test_ties_follow_the_selected_rule(gpu, oracle_lib, tie):
    # weights on a coarse grid: exact ties among raw activations in most windows
    rng = np.random.default_rng(11)
    V, K = 60, 200
    W0 = (rng.integers(-2, 3, size=(K, 2 * V)) * 0.25).astype(f32)
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=5, B=256, steps=8, tie=tie, W0=W0, n_masked=0)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)
    if tie == 1:
        lowest = run_both(gpu, oracle_lib, V=V, K=K, w=5, B=256, steps=1, tie=0, W0=W0, n_masked=0)[0]
        assert not np.array_equal(lowest[:256], wg[:256])  # the two rules really differ on this input


def test_zero_matrix_is_a_fixed_point(gpu, oracle_lib):
    V, K = 100, 64
    W0 = np.zeros((K, 2 * V), dtype=f32)
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=11, B=128, steps=3, W0=W0)
    assert (wg == 0).all() and np.array_equal(wg, wo)
    assert not Wg.any()


def test_one_neuron_wins_everything(gpu, oracle_lib):
    # every window goes to neuron 3: one owner block takes the whole batch (more windows than its
    # LDS staging holds at once, counts in the thousands on the frequent tokens)
    from flyvec_amd import synthetic
    V, K, B = 300, 70, 5000
    W0 = synthetic.synapses(K, V, sigma=0.01)
    W0[3] = np.abs(W0[3]) + 1.0
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=11, B=B, steps=3, W0=W0, n_tokens=100000)
    assert (wg == 3).all() and np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("V", [300, 12000])
def test_heavy_neuron_uses_32_bit_counters(gpu, oracle_lib, V):
    # one neuron wins 7000 windows of 11: 77000 window positions, past what 16-bit counters hold;
    # with V = 12000 its column classes also need more than one counting pass (2V / 4 > 5120)
    from flyvec_amd import synthetic
    K, B = 6, 7000
    W0 = synthetic.synapses(K, V, sigma=0.01)
    W0[2] = np.abs(W0[2]) + 1.0
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=V, K=K, w=11, B=B, steps=2, W0=W0, n_tokens=120000)
    assert (wg == 2).all() and np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


def test_minibatch_larger_than_the_match_masks(gpu, oracle_lib):
    # 70000 windows per step: the grouping kernel's threads take runs of more than 64 windows
    wg, wo, Wg, Wo = run_both(gpu, oracle_lib, V=200, K=5, w=3, B=70000, steps=2, n_tokens=200000, mean_chunk=40)
    assert np.array_equal(wg, wo)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("launches", [1, 2])
def test_timing_hooks(gpu, launches):
    from flyvec_amd import _lib, synthetic
    V, K, w, B = 300, 64, 11, 256
    tokens, offsets = small_corpus(20000, V)
    t, _ = make_trainer(tokens, offsets, V, K, w, B, synthetic.synapses(K, V, sigma=0.02), launches=launches)
    t.step(0, B, 1e-3)
    # as one launch the max pass, the update and the slot update are timed under the first of their names
    empty = {"update", "slot_update"} if launches == 1 else set()
    total, per = t.time_steps(B, 3, 1e-3)
    assert total > 0 and set(per) == set(_lib.TRAIN_KERNEL_NAMES)
    assert all(v > 0 for k, v in per.items() if k not in empty) and all(v >= 0 for v in per.values())
    single = t.time_kernels(reps=3)
    assert set(single) == set(_lib.TRAIN_KERNEL_NAMES)
    assert all(v > 0 for k, v in single.items() if k not in empty) and all(v >= 0 for v in single.values())
    assert _lib.calibration_copy(1 << 20, 3) > 0
    t.close()


@pytest.mark.parametrize("launches,per_graph", [(1, 1), (1, 4), (2, 3), (3, 2)])
def test_steps_enqueued_as_graphs_train_like_any_others(gpu, launches, per_graph):
    """Seven steps from HIP graphs (the last graph shorter than the others), steps launched the ordinary way
    before and after them: the matrix is the one that ordinary steps alone leave."""
    from flyvec_amd import synthetic
    V, K, w, B = 300, 64, 11, 256
    tokens, offsets = small_corpus(30000, V)
    W0 = synthetic.synapses(K, V, sigma=0.02)
    t, _ = make_trainer(tokens, offsets, V, K, w, B, W0, launches=launches)
    for s in range(12):
        t.step(s * B, B, 1e-3)
    want = t.get_weights()
    t.set_weights(W0)
    for s in range(2):
        t.step(s * B, B, 1e-3)
    assert t.time_steps_graph(2 * B, 7, 1e-3, per_graph) > 0
    for s in range(9, 12):
        t.step(s * B, B, 1e-3)
    got = t.get_weights()
    assert t.dense_launches == min(launches, 2) or launches == 3
    t.close()
    assert np.array_equal(got, want)


def test_partial_last_batch_and_epoch_driver(gpu, oracle_lib):
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B = 200, 96, 11, 300
    tokens, offsets = small_corpus(9000, V, n_masked=10)
    W0 = synthetic.synapses(K, V, sigma=0.02)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, lr0=2e-3)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    nwin = t.num_windows
    assert nwin % B != 0
    Wo = W0.copy()
    for ep in (0, 1, 14):
        t.run_epoch(ep, 15)
        eps = to.epoch_eps(2e-3, ep, 15)
        assert t.epoch_eps(ep, 15) == eps
        to.train_steps(Wo, tokens, starts, perm, 0, B, nwin // B + 1, w, invf, eps)
        assert np.array_equal(t.get_weights(), Wo), f"epoch {ep}"
    assert len(t.winners(nwin % B)) == nwin % B  # the last step took only the remainder
    t.close()


def test_step_statistics_and_size_independent_properties(gpu, oracle_lib):
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B = 400, 128, 11, 1000
    tokens, offsets = small_corpus(80000, V)
    W0 = synthetic.synapses(K, V, sigma=0.02)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    eps = 2e-4
    t.step(0, B, eps)
    xx, nc = t.step_stats()
    win = t.winners(B)
    W1 = t.get_weights()
    idx = to.inflate(tokens, starts, perm, 0, B, w, V)
    Wc = W0.copy()
    ref = to.train_step(Wc, idx, invf, eps)
    assert np.array_equal(xx, ref["xx"]) and nc == ref["nc"] and np.array_equal(win, ref["winners"])
    # rows that changed are exactly the winners with a non-zero total; the largest change is eps
    changed = np.flatnonzero((W1 != W0).any(axis=1))
    won = np.unique(win)
    assert changed.tolist() == won[xx[won] != 0].tolist()
    assert abs(np.abs(W1 - W0).max() - eps) < 1e-9
    t.close()


def test_repeatable_and_permutation_round_trip(gpu):
    from flyvec_amd import synthetic
    V, K, w, B = 300, 100, 11, 400
    tokens, offsets = small_corpus(30000, V)
    W0 = synthetic.synapses(K, V, sigma=0.02)
    outs = []
    for _ in range(2):
        t, perm = make_trainer(tokens, offsets, V, K, w, B, W0)
        assert np.array_equal(t.get_permutation(), perm)
        for s in range(5):
            t.step(s * B, B, 1e-3)
        outs.append(t.get_weights())
        t.shuffle(7)
        p2 = t.get_permutation()
        assert sorted(p2.tolist()) == list(range(len(perm))) and not np.array_equal(p2, perm)
        t.close()
    assert np.array_equal(outs[0], outs[1])


@pytest.mark.parametrize("launches", [1, 2, 3])
def test_steps_in_any_order_and_across_order_changes(gpu, oracle_lib, launches):
    """The single dense launch samples the column indices of the windows that follow its step; the next
    step uses them only if it takes exactly those windows in an unchanged order.  Sequential steps, jumps,
    partial batches, a new permutation, a device reshuffle and a new corpus in between: always the oracle's W."""
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B = 300, 64, 7, 128
    tokens, offsets = small_corpus(20000, V)
    W0 = synthetic.synapses(K, V)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, launches=launches)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    nwin = t.num_windows
    Wo = W0.copy()

    def both(first, n, corpus=tokens, st=starts, f=invf):
        t.step(first, n, 1e-3)
        wo = to.train_steps(Wo, corpus, st, perm, first, n, 1, w, f, 1e-3)
        assert np.array_equal(t.winners(n), wo), (first, n)

    both(0, B); both(B, B); both(2 * B, B)        # the windows that follow: sampled ahead
    both(7 * B, B)                                  # a jump
    both(8 * B, 100)                                # fewer windows than were sampled ahead
    both(8 * B + 100, B); both(9 * B + 100, B)      # following a partial batch
    both(0, B)                                      # backwards
    both(nwin - B - 40, B); both(nwin - 40, 40)     # the last, partial batch of the order (sampled ahead as such)
    assert np.array_equal(t.get_weights(), Wo)
    both(B, B)
    perm = np.random.default_rng(9).permutation(nwin).astype(np.uint64)
    t.set_permutation(perm)                         # the windows that follow are other windows now
    both(2 * B, B); both(3 * B, B)
    t.shuffle(5)
    perm = t.get_permutation()
    both(4 * B, B); both(5 * B, B)
    assert np.array_equal(t.get_weights(), Wo)
    tokens2, offsets2 = small_corpus(15000, V, seed=3)
    t.set_corpus(tokens2, offsets2)                 # identity order over another corpus
    starts2, invf2 = oracle_inputs(to, tokens2, offsets2, V, w)
    perm = np.arange(t.num_windows, dtype=np.uint64)
    both(6 * B, B, tokens2, starts2, invf2); both(7 * B, B, tokens2, starts2, invf2)
    assert np.array_equal(t.get_weights(), Wo)
    t.close()


def test_two_trainers_side_by_side(gpu, oracle_lib):
    """Where the single dense launch has to make the pass for max|ds| its blocks exchange their maxima inside the
    launch and want every compute unit, so while a process holds two trainers a step enqueues the launch twice in
    the form that waits for nobody (steps of both are enqueued without a synchronisation in between here). Both
    trainers, the first steps on a new matrix (the pass) and the later ones (max|ds| known) included, train to the
    checker's bits; alone again, a trainer returns to the one launch."""
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B = 300, 64, 7, 128
    tokens, offsets = small_corpus(20000, V)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    Wa, Wb = synthetic.synapses(K, V, seed=1), synthetic.synapses(K, V, seed=2)
    a, perm_a = make_trainer(tokens, offsets, V, K, w, B, Wa, perm_seed=6)
    assert a.dense_launches == 1
    b, perm_b = make_trainer(tokens, offsets, V, K, w, B, Wb, perm_seed=7)
    assert a.dense_launches == 1 and b.dense_launches == 1
    for s in range(6):
        a.step(s * B, B, 1e-3)
        b.step(s * B, B, 1e-3)
    b.sync()
    known, made = b.dense_path_counts
    assert known + made == 6 and made >= 1 and known >= 3
    Wo = Wb.copy()
    to.train_steps(Wo, tokens, starts, perm_b, 0, B, 6, w, invf, 1e-3)
    assert np.array_equal(b.get_weights(), Wo)
    b.close()
    assert a.dense_launches == 1
    for s in range(6, 9):
        a.step(s * B, B, 1e-3)
    Wo = Wa.copy()
    to.train_steps(Wo, tokens, starts, perm_a, 0, B, 9, w, invf, 1e-3)
    assert np.array_equal(a.get_weights(), Wo)
    assert sum(a.dense_path_counts) == 9
    a.close()


@pytest.mark.parametrize("launches", [1, 3])
def test_second_trainer_alive_while_the_pass_for_the_maximum_is_needed(gpu, oracle_lib, launches):
    """The form of the single dense launch that waits for nobody (a second trainer exists in the process), on
    weights whose largest entries sit on the most frequent tokens: nearly every step has to make the pass for
    max|ds|, which the first of the two launches then makes and the second follows with the update. Step by
    step against the checker, in the register and in the streaming form, run_epoch's partial last minibatch
    included."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 800, 96, 9, 2000
    tokens, offsets = small_corpus(80000, V, seed=2)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    perm = np.random.default_rng(3).permutation(len(starts)).astype(np.uint64)
    hot = np.argsort(-np.bincount(tokens[tokens >= 0], minlength=V))[:6]
    planted = synthetic.synapses(K, V, seed=9)
    planted[:, hot[:3]] = np.float32(7.0)
    other = Trainer(50, 8, 3, 16)                    # idle, but alive
    t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
    t.set_dense_launches(launches)
    t.set_corpus(tokens, offsets)
    t.set_permutation(perm)
    t.set_weights(planted)
    assert t.dense_launches == 1
    Wo = planted.copy()
    for s in range(8):
        t.step(s * B, B, 1e-3)
        ref = to.train_step(Wo, to.inflate(tokens, starts, perm, s * B, B, w, V), invf, 1e-3)
        xx, nc = t.step_stats()
        assert np.array_equal(t.winners(B), ref["winners"]) and np.array_equal(xx, ref["xx"]), s
        assert nc == ref["nc"], s
    assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32))
    known, made = t.dense_path_counts
    assert known + made == 8 and made >= 4
    t.set_weights(planted)
    t.run_epoch(3, 15)
    Wo = planted.copy()
    to.train_steps(Wo, tokens, starts, perm, 0, B, len(starts) // B + 1, w, invf, to.epoch_eps(1e-3, 3, 15))
    assert len(starts) % B != 0 and np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32))
    assert t.giveups_recovered == 0
    t.close()
    other.close()


def test_device_shuffle_is_a_cumulative_bijection(gpu):
    from flyvec_amd import Trainer
    V, w = 300, 11
    tokens, offsets = small_corpus(200000, V)
    a, b = Trainer(V, 8, w, 64), Trainer(V, 8, w, 64)
    a.set_corpus(tokens, offsets)
    b.set_corpus(tokens, offsets)
    n = a.num_windows
    assert np.array_equal(a.get_permutation(), np.arange(n, dtype=np.uint64))   # identity after set_corpus
    a.shuffle(3)
    sigma = a.get_permutation()
    assert np.array_equal(np.sort(sigma), np.arange(n, dtype=np.uint64))
    assert np.mean(sigma == np.arange(n)) < 0.01
    p0 = np.random.default_rng(1).permutation(n).astype(np.uint64)
    b.set_permutation(p0)
    b.shuffle(3)                                   # same seed, same call number: the same sigma
    assert np.array_equal(b.get_permutation(), p0[sigma])
    a.shuffle(3)                                   # a later call under the same seed draws another sigma
    again = a.get_permutation()
    assert np.array_equal(np.sort(again), np.arange(n, dtype=np.uint64))
    assert not np.array_equal(again, sigma[sigma])
    a.close()
    b.close()


def test_errors_are_reported_not_fatal(gpu):
    from flyvec_amd import Trainer, _lib, synthetic
    V, K = 50, 16
    tokens, offsets = small_corpus(3000, V, n_masked=0)
    t = Trainer(V, K, 5, 32)
    with pytest.raises(_lib.FlyvecError) as e:
        t.step(0, 32, 1e-3)
    assert e.value.code == _lib.FV_ERR_STATE
    bad = tokens.copy()
    bad[10] = V + 3
    with pytest.raises(_lib.FlyvecError) as e:
        t.set_corpus(bad, offsets)
    assert e.value.code == _lib.FV_ERR_DATA
    bad[10] = -2
    with pytest.raises(_lib.FlyvecError) as e:
        t.set_corpus(bad, offsets)
    assert e.value.code == _lib.FV_ERR_DATA
    off_bad = offsets.copy()
    off_bad[-1] = len(tokens) + 100
    with pytest.raises(_lib.FlyvecError) as e:
        t.set_corpus(tokens, off_bad)
    assert e.value.code == _lib.FV_ERR_DATA
    t.set_corpus(tokens, offsets)
    t.set_weights(synthetic.synapses(K, V))
    with pytest.raises(_lib.FlyvecError):
        t.step(0, 33, 1e-3)                      # more than the batch
    with pytest.raises(_lib.FlyvecError):
        t.step(t.num_windows - 5, 32, 1e-3)      # past the end
    with pytest.raises(ValueError):
        t.set_weights(np.zeros((K, V), dtype=f32))
    t.step(0, 32, 1e-3)                          # still usable after the errors
    t.sync()
    t.close()


def test_row_norms(gpu):
    from flyvec_amd import Trainer, synthetic
    V, K = 300, 40
    tokens, offsets = small_corpus(5000, V)
    W0 = synthetic.synapses(K, V)
    t = Trainer(V, K, 11, 64)
    t.set_corpus(tokens, offsets)
    t.set_weights(W0)
    want = np.sqrt((W0[:10].astype(np.float64) ** 2).sum(axis=1))
    assert np.allclose(t.row_norms(10), want, rtol=1e-12)
    t.close()


@functools.lru_cache(maxsize=1)
def headline_corpus():
    """The 10,000,000-token Zipf(1.07) corpus of the headline configuration (geometric chunks, mean 25), with what
    the checker derives from it."""
    from flyvec_amd import synthetic
    from oracle import train_oracle as to
    tokens, offsets = synthetic.corpus(10_000_000, 20000)
    return tokens, offsets, to.window_starts(offsets, 11), to.inverse_frequency(tokens, 20000)


def test_headline_config_100_steps(gpu, oracle_lib):
    """K = 400, V = 20000, w = 11, B = 10000 on the 10 M-token corpus, 100 steps from one seed: the stated bars
    (winners >= 99.9 %, relative L2 <= 1e-4) and, stronger, bit equality."""
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B, steps = 20000, 400, 11, 10000, 100
    tokens, offsets, starts, invf = headline_corpus()
    assert len(tokens) == 10_000_000 and 6_500_000 < len(starts) < 6_800_000
    W0 = synthetic.synapses(K, V, seed=5)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0)
    assert t.num_windows == len(starts)
    eps = t.epoch_eps(0, 15)
    wins = []
    for s in range(steps):
        t.step(s * B, B, eps)
        wins.append(t.winners(B))
    Wg = t.get_weights()
    t.close()
    Wo = W0.copy()
    wo = to.train_steps(Wo, tokens, starts, perm, 0, B, steps, w, invf, eps)
    wg = np.concatenate(wins)
    agree = float(np.mean(wg == wo))
    rel = float(np.linalg.norm(Wg - Wo) / np.linalg.norm(Wo))
    assert agree >= 0.999, agree
    assert rel <= 1e-4, rel
    assert np.array_equal(wg, wo) and np.array_equal(Wg, Wo)


def test_large_config_shape(gpu, oracle_lib):
    """K = 1000, V = 50000, w = 15, B = 50000 (W = 400 MB) on the 200 M-token Zipf(1.0) corpus the configuration
    names: the most frequent token occurs more than 2^24 times, so its 1/frequency is the saturated one of the
    reference's fp32 counter (flyvec/src/model_arrays.cu:396-424). Two steps, bit for bit."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B, steps = 50000, 1000, 15, 50000, 2
    tokens, offsets = synthetic.corpus(200_000_000, V, s=1.0, mean_chunk=40)
    head = int(np.count_nonzero(tokens == 1))
    assert head > 1 << 24, head
    W0 = synthetic.synapses(K, V, seed=5, sigma=0.02)
    t = Trainer(V, K, w, B, initial_learning_rate=2e-4)
    t.set_corpus(tokens, offsets)
    nwin = t.num_windows
    # a bijection of [0, nwin) that is cheap to write down at this size: i -> (a i + b) mod nwin, gcd(a, nwin) = 1
    a = 1_000_003
    while np.gcd(a, nwin) != 1:
        a += 2
    perm = (np.arange(nwin, dtype=np.uint64) * np.uint64(a) + np.uint64(12345)) % np.uint64(nwin)
    t.set_permutation(perm)
    t.set_weights(W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    assert nwin == len(starts) and 0.6 * len(tokens) < nwin < 0.75 * len(tokens)
    assert invf[1] == np.float32(1.0) / np.float32(1 << 24) and invf[1] > 1.0 / head   # saturated, not 1 / count
    assert np.array_equal(t.inverse_frequency(), invf)
    eps = t.epoch_eps(0, 15)
    wins = []
    for s in range(steps):
        t.step(s * B, B, eps)
        wins.append(t.winners(B))
    Wg = t.get_weights()
    t.close()
    Wo = W0.copy()
    wo = to.train_steps(Wo, tokens, starts, perm, 0, B, steps, w, invf, eps)
    assert np.array_equal(np.concatenate(wins), wo)
    assert np.array_equal(Wg, Wo)


# ---- anti-Hebbian term (delta != 0) -----------------------------------------------------------------

def run_both_delta(to, V, K, w, B, steps, delta, tie=0, n_tokens=60000, W0=None, sigma=0.02, seed=0, separate=False,
                   launches=0, mixed=False):
    """separate: the two lists of a neuron's windows grouped by launches of their own (else inside the sparse launch
    wherever the trainer has the bit rows and the regions for it); mixed: every third step without the term."""
    from flyvec_amd import synthetic
    tokens, offsets = small_corpus(n_tokens, V, seed=seed)
    if W0 is None:
        W0 = synthetic.synapses(K, V, seed=5 + seed, sigma=sigma)
    t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, tie=tie, launches=launches)
    t.set_grouping_launch(separate)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    eps = t.epoch_eps(0, 15)
    steps = min(steps, t.num_windows // B)
    Wo = W0.copy()
    for s in range(steps):
        d = 0.0 if mixed and s % 3 == 1 else delta
        t.step(s * B, B, eps, delta=d)
        idx = to.inflate(tokens, starts, perm, s * B, B, w, V)
        ref = to.train_step(Wo, idx, invf, eps, tie_rule=tie, delta=d)
        assert np.array_equal(t.winners(B), ref["winners"]), f"winners, step {s}"
        if d:
            assert np.array_equal(t.second_winners(B), ref["seconds"]), f"second neurons, step {s}"
        xx, nc = t.step_stats()
        assert np.array_equal(xx, ref["xx"]) and nc == ref["nc"], f"xx / max|ds|, step {s}"
    Wg = t.get_weights()
    t.close()
    return Wg, Wo


@pytest.mark.parametrize("separate", [False, True])
@pytest.mark.parametrize("tie", [0, 1])
def test_delta_small_config_bit_exact(gpu, oracle_lib, tie, separate):
    Wg, Wo = run_both_delta(oracle_lib, V=500, K=400, w=11, B=512, steps=10, delta=0.4, tie=tie, separate=separate)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("separate", [False, True])
@pytest.mark.parametrize("K,w,V,B", [(1, 1, 5, 1), (2, 3, 9, 7), (65, 15, 200, 256), (130, 64, 300, 64),
                                     (30, 11, 30000, 700), (20, 7, 22000, 500),   # the wider counter arrays
                                     (400, 11, 3000, 4000), (96, 9, 500, 16384)])
def test_delta_shapes_bit_exact(gpu, oracle_lib, K, w, V, B, separate):
    n_tokens = 40000 if V < 20000 else 120000
    n_tokens = max(n_tokens, 8 * B)
    Wg, Wo = run_both_delta(oracle_lib, V=V, K=K, w=w, B=B, steps=4, delta=0.25, n_tokens=n_tokens, separate=separate)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("launches", [1, 2, 3])
def test_delta_grouped_inside_the_sparse_launch(gpu, oracle_lib, launches):
    """The anti-Hebbian step whose sparse launch takes both of a neuron's window lists from bit rows (no grouping
    launches), at a shape where every block of that launch has a slot region of its own: every dense-launch form,
    steps with and without the term in turn (the second neurons' bit rows keep a parity of their own), and the
    epoch driver with the schedule."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 1500, 130, 11, 3000
    Wg, Wo = run_both_delta(to, V=V, K=K, w=w, B=B, steps=7, delta=0.4, n_tokens=90000, launches=launches, mixed=True)
    assert np.array_equal(Wg, Wo)
    tokens, offsets = small_corpus(30000, V, seed=4)
    W0 = synthetic.synapses(K, V, seed=2, sigma=0.02)
    t = Trainer(V, K, w, B, initial_learning_rate=1e-3, delta=0.3)
    t.set_dense_launches(launches)
    t.set_corpus(tokens, offsets)
    t.set_weights(W0)
    t.shuffle(3)
    perm = t.get_permutation()
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    assert len(starts) % B != 0 and len(starts) > 2 * B
    Wo = W0.copy()
    for ep in (0, 9):
        t.run_epoch(ep, 15)
        to.train_steps(Wo, tokens, starts, perm, 0, B, len(starts) // B + 1, w, invf, to.epoch_eps(1e-3, ep, 15),
                       delta=to.epoch_delta(0.3, ep, 15))
        assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32)), ep
    t.close()


def test_delta_with_ties_and_heavy_neurons(gpu, oracle_lib):
    # coarse weights: ties in both searches; then two neurons that take every first and second place
    # of 7000 windows (32-bit counters in both counter arrays)
    from flyvec_amd import synthetic
    rng = np.random.default_rng(11)
    V, K = 60, 200
    W0 = (rng.integers(-2, 3, size=(K, 2 * V)) * 0.25).astype(f32)
    for tie in (0, 1):
        Wg, Wo = run_both_delta(oracle_lib, V=V, K=K, w=5, B=256, steps=4, delta=0.5, tie=tie, W0=W0)
        assert np.array_equal(Wg, Wo)
    # (V = 12000: each of the two neurons' class blocks has more records than the first part of its slot region holds)
    for V in (300, 12000):
        K, B = 6, 7000
        W0 = synthetic.synapses(K, V, sigma=0.01)
        W0[2] = np.abs(W0[2]) + 1.0
        W0[4] = np.abs(W0[4]) + 0.5
        Wg, Wo = run_both_delta(oracle_lib, V=V, K=K, w=11, B=B, steps=2, delta=0.3, W0=W0, n_tokens=120000)
        assert np.array_equal(Wg, Wo)


def test_delta_epoch_schedule_and_driver(gpu, oracle_lib):
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 200, 96, 11, 300
    tokens, offsets = small_corpus(9000, V, n_masked=10)
    W0 = synthetic.synapses(K, V, sigma=0.02)
    t = Trainer(V, K, w, B, initial_learning_rate=2e-3, delta=0.4)
    t.set_corpus(tokens, offsets)
    perm = np.random.default_rng(6).permutation(t.num_windows).astype(np.uint64)
    t.set_permutation(perm)
    t.set_weights(W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    nwin = t.num_windows
    Wo = W0.copy()
    for ep in (0, 7, 14):
        delta = to.epoch_delta(0.4, ep, 15)
        assert t.epoch_delta(ep, 15) == delta and delta > 0
        t.run_epoch(ep, 15)
        to.train_steps(Wo, tokens, starts, perm, 0, B, nwin // B + 1, w, invf, to.epoch_eps(2e-3, ep, 15),
                       delta=delta)
        assert np.array_equal(t.get_weights(), Wo), f"epoch {ep}"
    t.step(0, B, 1e-3)                       # a plain step afterwards still works
    with pytest.raises(Exception):
        t.second_winners(B)                  # and has no second neurons to show
    t.close()


# ---- position weights (Lmid, Lbase) and in-window duplicate pruning --------------------------------------

def run_both_variant(to, V, K, w, B, steps, delta=0.0, lmid=1.0, lbase=1.0, prune=False, tie=0, launches=0,
                     n_tokens=60000, sigma=0.02, seed=0, vocab_for_tokens=None):
    """Steps with the rule's dormant variants switched on, against the checker step by step."""
    from flyvec_amd import Trainer, synthetic
    # pruning only matters when tokens repeat inside a window: draw them from a small vocabulary then
    tokens, offsets = small_corpus(n_tokens, vocab_for_tokens or V, seed=seed)
    tokens[-1] = V - 1
    W0 = synthetic.synapses(K, V, seed=5 + seed, sigma=sigma)
    t = Trainer(V, K, w, B, initial_learning_rate=2e-4, tie_rule=tie, lmid=lmid, lbase=lbase, prune_duplicates=prune)
    t.set_dense_launches(launches)
    t.set_corpus(tokens, offsets)
    perm = np.random.default_rng(6).permutation(t.num_windows).astype(np.uint64)
    t.set_permutation(perm)
    t.set_weights(W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    eps = t.epoch_eps(0, 15)
    steps = min(steps, t.num_windows // B)
    Wo = W0.copy()
    inflate = to.inflate_prune if prune else to.inflate
    for s in range(steps):
        t.step(s * B, B, eps, delta=delta)
        idx = inflate(tokens, starts, perm, s * B, B, w, V)
        ref = to.train_step(Wo, idx, invf, eps, tie_rule=tie, delta=delta, lmid=lmid, lbase=lbase)
        assert np.array_equal(t.winners(B), ref["winners"]), f"winners, step {s}"
        if delta:
            assert np.array_equal(t.second_winners(B), ref["seconds"]), f"second neurons, step {s}"
        xx, nc = t.step_stats()
        assert np.array_equal(xx, ref["xx"]) and nc == ref["nc"], f"xx / max|ds|, step {s}"
    Wg = t.get_weights()
    t.close()
    return Wg, Wo


@pytest.mark.parametrize("launches", [1, 2, 3])
@pytest.mark.parametrize("lmid,lbase,delta", [(2.5, 0.75, 0.0), (0.3, 1.0, 0.0), (1.0, 3.0, 0.4), (0.0, 1.0, 0.0),
                                              (1.0, 0.0, 0.4), (-1.5, 0.5, 0.0)])
def test_position_weights_bit_exact(gpu, oracle_lib, lmid, lbase, delta, launches):
    Wg, Wo = run_both_variant(oracle_lib, V=500, K=400, w=11, B=512, steps=6, delta=delta, lmid=lmid, lbase=lbase,
                              launches=launches)
    assert np.array_equal(Wg, Wo)


@pytest.mark.parametrize("K,w,V,B,tie", [(1, 1, 5, 1, 0), (3, 2, 7, 3, 1), (65, 15, 200, 256, 0), (130, 64, 300, 64, 1),
                                         (1000, 4, 300, 512, 0), (30, 11, 30000, 700, 0)])
def test_position_weights_shapes(gpu, oracle_lib, K, w, V, B, tie):
    n_tokens = 40000 if V < 20000 else 120000
    Wg, Wo = run_both_variant(oracle_lib, V=V, K=K, w=w, B=B, steps=4, delta=0.25, lmid=1.75, lbase=0.6, tie=tie,
                              n_tokens=n_tokens)
    assert np.array_equal(Wg, Wo)


def test_unit_weights_take_the_unweighted_kernels(gpu, oracle_lib):
    # Lmid = Lbase = 1 is the default path: same bits as a trainer created without the fields
    Wa, Wo = run_both_variant(oracle_lib, V=300, K=64, w=7, B=128, steps=5)
    Wb = run_both(gpu, oracle_lib, V=300, K=64, w=7, B=128, steps=5, n_tokens=60000)[2]
    assert np.array_equal(Wa, Wo) and np.array_equal(Wa, Wb)


@pytest.mark.parametrize("launches", [1, 2, 3])
@pytest.mark.parametrize("w,small_vocab", [(11, 12), (7, 5), (64, 40), (2, 3), (1, 4)])
def test_duplicate_pruning_bit_exact(gpu, oracle_lib, w, small_vocab, launches):
    # tokens drawn from a handful of ids, so most windows hold repeats; V stays larger (unused columns)
    Wg, Wo = run_both_variant(oracle_lib, V=300, K=96, w=w, B=256, steps=6, prune=True, vocab_for_tokens=small_vocab,
                              launches=launches, delta=0.2 if w == 7 else 0.0)
    assert np.array_equal(Wg, Wo)


def test_duplicate_pruning_with_weights_and_epoch_driver(gpu, oracle_lib):
    """Everything at once through run_epoch: pruning, weights, the anti-Hebbian schedule, a partial last batch."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 200, 96, 11, 300
    tokens, offsets = small_corpus(9000, 25, n_masked=10)
    tokens[-1] = V - 1
    W0 = synthetic.synapses(K, V, sigma=0.02)
    t = Trainer(V, K, w, B, initial_learning_rate=2e-4, delta=0.3, lmid=1.5, lbase=0.8, prune_duplicates=True)
    t.set_corpus(tokens, offsets)
    perm = np.random.default_rng(6).permutation(t.num_windows).astype(np.uint64)
    t.set_permutation(perm)
    t.set_weights(W0)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    t.run_epoch(3, 15)
    eps, delta = t.epoch_eps(3, 15), t.epoch_delta(3, 15)
    Wo = W0.copy()
    n_steps = (t.num_windows + B - 1) // B
    to.train_steps(Wo, tokens, starts, perm, 0, B, n_steps, w, invf, eps, delta=delta, lmid=1.5, lbase=0.8, prune=True)
    assert np.array_equal(t.get_weights(), Wo)
    t.close()


def test_an_epoch_of_the_headline_configuration_in_every_launch_form(gpu, oracle_lib):
    """K = 400, V = 20000, w = 11, B = 10000 over the whole 10 M-token corpus: one epoch through run_epoch behind a
    device shuffle (663 full minibatches and the partial one) equals the checker's epoch over the same order bit for
    bit, as one dense launch per step, as separate launches, and with the grouping launch of its own; every block
    exchange, slot record and ahead-sampled minibatch of the single launch has to come out right for that."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 20000, 400, 11, 10000
    tokens, offsets, starts, invf = headline_corpus()
    W0 = synthetic.synapses(K, V, seed=5)
    got, perms = {}, []
    for launches, separate in ((1, False), (2, False), (1, True)):
        t = Trainer(V, K, w, B, initial_learning_rate=2e-4)
        t.set_dense_launches(launches)
        t.set_grouping_launch(separate)      # grouped inside the sparse launch, or by a launch of its own
        t.set_corpus(tokens, offsets)
        nwin = t.num_windows
        assert nwin == len(starts) and nwin // B >= 650 and nwin % B != 0
        t.set_weights(W0)
        t.shuffle(11)
        perms.append(t.get_permutation())
        t.run_epoch(0, 15)
        got[launches, separate] = t.get_weights()
        assert len(t.winners(nwin % B)) == nwin % B      # the last step took the remainder only
        if launches == 1:
            known, made = t.dense_path_counts
            assert known + made == nwin // B + 1 and t.giveups_recovered == 0
        t.close()
    assert np.array_equal(perms[0], perms[1]) and np.array_equal(perms[0], perms[2])
    assert np.array_equal(np.sort(perms[0]), np.arange(nwin, dtype=np.uint64))
    Wo = W0.copy()
    wo = to.train_steps(Wo, tokens, starts, perms[0], 0, B, nwin // B + 1, w, invf, to.epoch_eps(2e-4, 0, 15))
    assert len(wo) == nwin
    assert np.isfinite(Wo).all() and not np.array_equal(Wo, W0)
    for form, Wg in got.items():
        assert np.array_equal(Wg, Wo), form


@pytest.mark.parametrize("V,K,w,B,steps", [
    (300, 64, 7, 128, 6),        # a few windows per neuron
    (500, 2, 5, 6000, 3),        # two neurons: each wins more windows than LDS stages at once
    (800, 8, 11, 4096, 3),       # hundreds of windows per neuron: activations fetched by rank
    (2000, 400, 11, 16384, 2),   # the largest batch the sparse launch groups for itself
    (300, 70, 64, 200, 3),       # the widest window
])
def test_grouping_forms_agree_and_match_the_oracle(gpu, oracle_lib, V, K, w, B, steps):
    """Grouping by winner inside the sparse launch (bit rows left by the winner kernel) and as a launch of
    its own give the same matrix, xx and winners, bit for bit, and both equal the oracle's; a shorter
    last step and a switch of form between steps are part of the run."""
    from flyvec_amd import synthetic
    to = oracle_lib
    tokens, offsets = small_corpus(max(40000, 3 * B * steps), V, seed=3)
    W0 = synthetic.synapses(K, V, seed=9)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    got = {}
    for form in ("inside", "separate", "alternating"):
        t, perm = make_trainer(tokens, offsets, V, K, w, B, W0)
        assert t.grouping_launch is False
        t.set_grouping_launch(form == "separate")
        assert t.grouping_launch is (form == "separate")
        first = 0
        for s in range(steps):
            if form == "alternating":
                t.set_grouping_launch(s % 2 == 1)
            n = B if s + 1 < steps else max(1, B // 3 + 1)
            t.step(first, n, 1e-3)
            first += n
        got[form] = (t.get_weights(), t.winners(n).copy(), t.step_stats())
        t.close()
    for form in ("separate", "alternating"):
        assert np.array_equal(got["inside"][0], got[form][0])
        assert np.array_equal(got["inside"][1], got[form][1])
        assert np.array_equal(got["inside"][2][0], got[form][2][0]) and got["inside"][2][1] == got[form][2][1]
    Wo = W0.copy()
    first = 0
    for s in range(steps):
        n = B if s + 1 < steps else max(1, B // 3 + 1)
        to.train_steps(Wo, tokens, starts, perm, first, n, 1, w, invf, 1e-3, 1e-30)
        first += n
    assert np.array_equal(got["inside"][0], Wo)


def test_batches_beyond_the_grouping_limit_take_the_separate_launch(gpu):
    from flyvec_amd import Trainer, _lib
    t = Trainer(300, 16, 5, 16385)
    assert t.grouping_launch is True
    t.set_grouping_launch(False)            # the rule, not a promise
    assert t.grouping_launch is True
    with pytest.raises(_lib.FlyvecError) as e:
        _lib.check(t.lib.fv_trainer_set_grouping_launch(t.handle, 2))
    assert e.value.code == _lib.FV_ERR_INVALID
    t.close()


def test_measurement_launches_leave_the_grouping_buffers_consistent(gpu, oracle_lib):
    """time_kernels repeats single kernels of the last step (the winner kernel many times over the same bit
    rows); the steps that follow still equal the oracle's from the matrix the measurement left."""
    from flyvec_amd import synthetic
    to = oracle_lib
    V, K, w, B = 600, 96, 9, 1500
    tokens, offsets = small_corpus(60000, V, seed=4)
    W0 = synthetic.synapses(K, V, seed=2)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    for launches in (1, 2):
        t, perm = make_trainer(tokens, offsets, V, K, w, B, W0, launches=launches)
        for s in range(3):
            t.step(s * B, B, 1e-3)
        t.time_kernels(reps=3)                 # leaves W in a state of its own
        W1 = t.get_weights()
        finite = np.isfinite(W1).all()
        if not finite:                         # sentinels planted by the repeated sparse launch: start afresh
            t.set_weights(W0)
            W1 = W0.copy()
        for s in range(3, 6):
            t.step(s * B, B, 1e-3)
        Wg = t.get_weights()
        t.close()
        Wo = W1.copy()
        to.train_steps(Wo, tokens, starts, perm, 3 * B, B, 3, w, invf, 1e-3, 1e-30)
        assert np.array_equal(Wg, Wo)


def _random_case(case):
    rng = np.random.default_rng(1000 + case)
    c = dict(V=int(rng.integers(50, 3000)), K=int(rng.integers(1, 600)), w=int(rng.integers(1, 33)) | 1,
             B=int(rng.integers(1, 9000)), steps=int(rng.integers(1, 4)), tie=int(rng.integers(0, 2)),
             lmid=float(rng.choice([1.0, 1.0, 0.5, 2.0])), lbase=float(rng.choice([1.0, 1.0, 1.5])),
             prune=bool(rng.integers(0, 2)), launches=int(rng.integers(1, 3)),
             zipf_s=1.0 + float(rng.random()) * 0.3, sigma=float(rng.choice([0.02, 0.02, 1e-6, 0.0])))
    c["mean_chunk"] = int(rng.integers(c["w"] + 2, 60))
    c["last_n"] = int(rng.integers(1, c["B"] + 1))
    return c


@pytest.mark.parametrize("case", range(30))
def test_random_configurations_match_the_oracle(gpu, oracle_lib, case):
    """Seeded random combinations of shape (K, V, w, B), tie rule, position weights, duplicate pruning, dense-launch
    form and a partial last minibatch: both grouping forms against the checker, step by step, bit for bit."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    c = _random_case(case)
    V, K, w, B = c["V"], c["K"], c["w"], c["B"]
    n_tokens = max(20000, 3 * B * c["steps"] + 1000)
    tokens, offsets = synthetic.corpus(n_tokens, V, s=c["zipf_s"], mean_chunk=c["mean_chunk"],
                                       seed_tokens=case + 3, seed_chunks=case + 4)
    W0 = synthetic.synapses(K, V, seed=case, sigma=c["sigma"])
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    if len(starts) < B * c["steps"]:
        pytest.skip(f"{len(starts)} windows for {c}")
    perm = np.random.default_rng(case).permutation(len(starts)).astype(np.uint64)
    inflate = to.inflate_prune if c["prune"] else to.inflate
    sizes = [B] * (c["steps"] - 1) + [c["last_n"]]
    Wo, ref = W0.copy(), []
    first = 0
    for n in sizes:
        idx = inflate(tokens, starts, perm, first, n, w, V)
        ref.append(to.train_step(Wo, idx, invf, 1e-3, tie_rule=c["tie"], lmid=c["lmid"], lbase=c["lbase"]))
        first += n
    for separate in (False, True):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3, tie_rule=c["tie"], lmid=c["lmid"], lbase=c["lbase"],
                    prune_duplicates=c["prune"])
        t.set_dense_launches(3 if c["launches"] == 1 and case % 3 == 0 else c["launches"])  # 3: one launch, rows streamed
        t.set_grouping_launch(separate)
        t.set_slot_regions(case % 2 == 0)  # odd cases: the blocks of the launch that groups for itself share class regions
        t.set_corpus(tokens, offsets)
        t.set_permutation(perm)
        t.set_weights(W0)
        first = 0
        for s, n in enumerate(sizes):
            t.step(first, n, 1e-3)
            first += n
            assert np.array_equal(t.winners(n), ref[s]["winners"]), f"winners, step {s}, {c}"
            xx, nc = t.step_stats()
            assert np.array_equal(xx, ref[s]["xx"]) and nc == ref[s]["nc"], f"xx / max|ds|, step {s}, {c}"
        Wg = t.get_weights()
        t.close()
        assert np.array_equal(Wg.view(np.uint32), Wo.view(np.uint32)), f"W, separate grouping {separate}, {c}"


@pytest.mark.parametrize("K,w,V,B", [(50, 5, 2000, 20000), (300, 11, 800, 40000), (7, 3, 50, 65535)])
def test_minibatches_beyond_16384_windows(gpu, oracle_lib, K, w, V, B):
    """More than 16384 windows per minibatch (the grouping launch is a launch of its own there, up to 64 windows
    per thread of its blocks; the last case is the largest batch whose window ids fit 16 bits): three steps against
    the checker, the last one partial, in both forms of the single dense launch and as separate launches."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    tokens, offsets = small_corpus(3 * B * 2 + 40000, V, seed=12)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    assert len(starts) >= 3 * B
    perm = np.random.default_rng(13).permutation(len(starts)).astype(np.uint64)
    W0 = synthetic.synapses(K, V, seed=4, sigma=0.02)
    sizes = [B, B, B // 3 + 1]
    Wo, ref, first = W0.copy(), [], 0
    for n in sizes:
        ref.append(to.train_step(Wo, to.inflate(tokens, starts, perm, first, n, w, V), invf, 1e-3))
        first += n
    for launches in (1, 2, 3):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
        t.set_dense_launches(launches)
        t.set_corpus(tokens, offsets)
        t.set_permutation(perm)
        t.set_weights(W0)
        first = 0
        for s, n in enumerate(sizes):
            t.step(first, n, 1e-3)
            first += n
            assert np.array_equal(t.winners(n), ref[s]["winners"]), f"winners, step {s}, launches {launches}"
            xx, nc = t.step_stats()
            assert np.array_equal(xx, ref[s]["xx"]) and nc == ref[s]["nc"], f"xx / max|ds|, step {s}, launches {launches}"
        Wg = t.get_weights()
        t.close()
        assert np.array_equal(Wg.view(np.uint32), Wo.view(np.uint32)), f"W, launches {launches}"


@pytest.mark.parametrize("launches", [1, 2, 3])
@pytest.mark.parametrize("V,K,w,B", [(20000, 400, 11, 3000), (700, 130, 9, 2500), (300, 500, 64, 600), (900, 40, 1, 900),
                                     (60, 300, 15, 200), (5000, 7, 5, 4000), (3000, 2048, 3, 1000)])
def test_neurons_with_few_windows_are_finished_by_one_block(gpu, oracle_lib, V, K, w, B, launches):
    """The sparse-element launch that groups for itself gives a neuron with no more window positions than a block
    has threads to one block, an entry per thread, for all four column classes (the other three blocks end at
    once). With that form and without it, against the checker step by step: many neurons (most are such), few
    (every neuron heavy), w = 64 (four windows fill a block) and w = 1, repeated tokens inside a window, ties."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    tokens, offsets = small_corpus(max(40000, 12 * B), V, seed=V % 7, mean_chunk=max(25, w + 8))
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    perm = np.random.default_rng(V).permutation(len(starts)).astype(np.uint64)
    W0 = synthetic.synapses(K, V, seed=3, sigma=0.02)
    if K == 300:
        W0 = np.round(W0 * 100) / np.float32(100)            # a coarse grid: ties among the activations
    steps = min(4, len(starts) // B)
    assert steps >= 2
    Wo, ref = W0.copy(), []
    for s in range(steps):
        ref.append(to.train_step(Wo, to.inflate(tokens, starts, perm, s * B, B, w, V), invf, 1e-3))
    counts = np.bincount(ref[0]["winners"], minlength=K)
    stride = (w + 3) & ~3
    few = np.count_nonzero((counts > 0) & (counts * stride <= 256))
    assert few > 0 or K <= 7, "no neuron of this case takes the form under test"
    for light in (True, False):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
        t.set_dense_launches(launches)
        t.set_light_blocks(light)
        t.set_corpus(tokens, offsets)
        t.set_permutation(perm)
        t.set_weights(W0)
        assert t.grouping_launch is False
        for s in range(steps):
            t.step(s * B, B, 1e-3)
            assert np.array_equal(t.winners(B), ref[s]["winners"]), (light, s)
            xx, nc = t.step_stats()
            assert np.array_equal(xx, ref[s]["xx"]) and nc == ref[s]["nc"], (light, s)
        assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32)), light
        t.close()


@pytest.mark.parametrize("launches,entries", [(1, 1), (1, 37), (3, 1), (3, 300)])
def test_sparse_elements_beyond_the_sentinel_list_are_finished_where_they_are_met(gpu, oracle_lib, launches, entries):
    """The single dense launch with a sentinel list that counts as full after a few entries: nearly every sparse
    element takes the path of an element that finds the list full."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 700, 130, 9, 2500
    tokens, offsets = small_corpus(70000, V, seed=8)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    perm = np.random.default_rng(9).permutation(len(starts)).astype(np.uint64)
    W0 = synthetic.synapses(K, V, seed=2, sigma=0.02)
    Wo = W0.copy()
    t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
    t.set_dense_launches(launches)
    t.set_sentinel_list(entries)
    t.set_corpus(tokens, offsets)
    t.set_permutation(perm)
    t.set_weights(W0)
    for s in range(4):
        ref = to.train_step(Wo, to.inflate(tokens, starts, perm, s * B, B, w, V), invf, 1e-3)
        t.step(s * B, B, 1e-3)
        xx, nc = t.step_stats()
        assert np.array_equal(xx, ref["xx"]) and nc == ref["nc"]
    Wg = t.get_weights()
    known, made = t.dense_path_counts
    t.close()
    assert known >= 1 and made >= 1   # both ways through the launch
    assert np.array_equal(Wg.view(np.uint32), Wo.view(np.uint32))


@pytest.mark.parametrize("launches", [1, 2, 3])
@pytest.mark.parametrize("per_block", [True, False])
def test_slot_records_per_block_or_per_class(gpu, oracle_lib, launches, per_block):
    """The records of a step's sparse elements in a region per block of the sparse launch, or in one region per
    class behind the lower neurons' records: three steps against the checker, with one neuron winning most windows
    (its records are many) and most neurons winning none."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 500, 70, 7, 3000
    tokens, offsets = small_corpus(60000, V, seed=4)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    perm = np.random.default_rng(5).permutation(len(starts)).astype(np.uint64)
    W0 = synthetic.synapses(K, V, seed=3, sigma=0.02)
    W0[11] += 0.05  # neuron 11 wins nearly everything
    Wo = W0.copy()
    t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
    t.set_dense_launches(launches)
    t.set_slot_regions(per_block)
    t.set_corpus(tokens, offsets)
    t.set_permutation(perm)
    t.set_weights(W0)
    for s in range(3):
        ref = to.train_step(Wo, to.inflate(tokens, starts, perm, s * B, B, w, V), invf, 1e-3)
        t.step(s * B, B, 1e-3)
        assert np.array_equal(t.winners(B), ref["winners"])
        assert np.bincount(ref["winners"], minlength=K)[11] > B // 2
        xx, nc = t.step_stats()
        assert np.array_equal(xx, ref["xx"]) and nc == ref["nc"]
    Wg = t.get_weights()
    t.close()
    assert np.array_equal(Wg.view(np.uint32), Wo.view(np.uint32))


@pytest.mark.parametrize("launches", [1, 2, 3])
def test_dense_launch_knows_the_maximum_from_the_rows_largest_weights(gpu, oracle_lib, launches):
    """The single dense launch carries every row's two largest |W| and, with what the sparse launch reports on
    them, knows max|ds| before it reads the matrix; where the largest weights of the deciding row are sparse
    elements of the step it makes the pass instead. Both ways, step by step, against the checker: random weights
    (the maximum is nearly always known), and weights whose largest entries sit on the most frequent tokens
    (they are sparse elements of nearly every row in every step: the pass has to be made)."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 800, 96, 9, 2000
    tokens, offsets = small_corpus(80000, V, seed=2)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    perm = np.random.default_rng(3).permutation(len(starts)).astype(np.uint64)
    hot = np.argsort(-np.bincount(tokens[tokens >= 0], minlength=V))[:6]
    plain = synthetic.synapses(K, V, seed=9)
    planted = plain.copy()
    # the same largest value three times in every row, on tokens that nearly every window holds; being positive,
    # the dense term of such an element (-xx * 7, xx > 0) is partly cancelled by its sparse term, so no sparse
    # element reaches the bound |xx| * 7 that the row would have if one of the three were dense
    planted[:, hot[:3]] = np.float32(7.0)
    tied = plain.copy()
    tied[:, hot[0]] = np.float32(6.0)                # one sparse element and one dense element hold the row's
    tied[:, 5] = np.float32(-6.0) if 5 not in hot else tied[:, 5]   # largest value: the dense one decides
    counts = {}
    for name, W0 in (("plain", plain), ("planted", planted), ("tied", tied)):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
        t.set_dense_launches(launches)   # as separate launches the pass for the maximum ends at once when it is known
        t.set_corpus(tokens, offsets)
        t.set_permutation(perm)
        t.set_weights(W0)
        Wo = W0.copy()
        for s in range(8):
            t.step(s * B, B, 1e-3)
            ref = to.train_step(Wo, to.inflate(tokens, starts, perm, s * B, B, w, V), invf, 1e-3)
            xx, nc = t.step_stats()
            assert np.array_equal(t.winners(B), ref["winners"]) and np.array_equal(xx, ref["xx"]), (name, s)
            assert nc == ref["nc"], (name, s)
        assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32)), name
        counts[name] = t.dense_path_counts
        t.close()
    assert all(known + made == 8 and made >= 1 for known, made in counts.values())   # the first step makes the pass
    assert counts["plain"][0] >= 5
    assert counts["planted"][1] >= 4


@pytest.mark.parametrize("launches,prune", [(1, False), (2, False), (1, True), (3, False)])
def test_stale_tail_of_the_last_minibatch(gpu, oracle_lib, launches, prune):
    """The reference trains a final partial minibatch on all Num rows, the ones behind the remainder being the
    previous minibatch's (flyvec/src/cuda_funcs.cu:1679 against :1700-1732). Switched on, run_epoch does the same,
    over two epochs with a reshuffled order in between, bit for bit with the checker's mode; switched off it
    trains the remainder only."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 400, 70, 7, 900
    tokens, offsets = small_corpus(9000, V if not prune else 30, seed=6)
    tokens[-1] = V - 1
    W0 = synthetic.synapses(K, V, seed=4)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    assert len(starts) % B not in (0,) and len(starts) > 3 * B
    for stale in (True, False):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3, prune_duplicates=prune)
        t.set_dense_launches(launches)
        t.set_stale_tail(stale)
        t.set_corpus(tokens, offsets)
        t.set_weights(W0)
        Wo = W0.copy()
        for ep in range(2):
            t.shuffle(ep)
            perm = t.get_permutation()
            t.run_epoch(ep, 15)
            to.train_steps(Wo, tokens, starts, perm, 0, B, len(starts) // B + 1, w, invf, to.epoch_eps(1e-3, ep, 15),
                           prune=prune, stale_tail=stale)
        assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32)), stale
        t.close()


@pytest.mark.parametrize("planted", [False, True])
def test_run_epoch_takes_up_again_behind_a_launch_that_gave_up(gpu, oracle_lib, planted):
    """The reference's minibatch loop never skips a step (flyvec/src/cuda_funcs.cu:1662-1812). With the wait of
    the single dense launch forced to zero rounds (every kernel still runs to its end) the first launch that has
    to make the pass for max|ds| gives up -- the epoch's first step on a fresh matrix, or, with the rows' largest
    weights planted on the most frequent tokens, the first step whose deciding row has them among its sparse
    elements although they are known from the epoch before -- and so do the launches behind it; run_epoch redoes the epoch from that step with two launches per step and the matrix
    equals the checker's."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, K, w, B = 800, 96, 9, 2000
    tokens, offsets = small_corpus(80000, V, seed=2)
    starts, invf = oracle_inputs(to, tokens, offsets, V, w)
    W0 = synthetic.synapses(K, V, seed=9)
    if planted:
        hot = np.argsort(-np.bincount(tokens[tokens >= 0], minlength=V))[:3]
        W0[:, hot] = np.float32(7.0)
    t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
    t.set_dense_launches(1)
    t.set_corpus(tokens, offsets)
    t.set_weights(W0)
    Wo = W0.copy()
    n_steps = len(starts) // B + 1
    for ep in range(2):
        t.shuffle(ep)
        perm = t.get_permutation()
        if ep == 1 or not planted:
            t.set_dense_launches(1)
            t._set_wait_limit(0)
        t.run_epoch(ep, 15)
        to.train_steps(Wo, tokens, starts, perm, 0, B, n_steps, w, invf, to.epoch_eps(1e-3, ep, 15))
        assert np.array_equal(t.get_weights().view(np.uint32), Wo.view(np.uint32)), ep
    # one recovery each: on a fresh matrix in the first epoch (the separate launches it falls back to keep the rows'
    # largest weights too, so the second epoch's single launches know the maximum and have nothing to wait for);
    # with the planted weights in the second epoch
    assert t.giveups_recovered == 1
    assert t.dense_launches == (2 if planted else 1)
    t.sync()                   # nothing left to report
    t.close()
