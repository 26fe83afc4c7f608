"""The reference's own C ABI (flyvec/train_flyvec.py:62-263), served by libflyvec_hip.so under the reference's
five library names: driven here in the order and with the argument types the reference's driver uses, the
matrix it leaves after every epoch must equal, bit for bit, what the CPU checker computes over the same window
orders (the reference's tie rule, its treatment of the last minibatch), and what this library's own interface
computes with the same settings."""
import ctypes as C

import numpy as np
import pytest

from conftest import small_corpus

pytestmark = pytest.mark.gpu


def _bind(tmp_path):
    from flyvec_amd import build
    links = {p.name: C.CDLL(str(p)) for p in build.install_legacy_names(tmp_path / "src")}
    links["prune_input.so"].getnum_samples.restype = C.c_uint64
    links["model_descriptor.so"].model_create_descriptor.restype = C.c_void_p
    links["model_arrays.so"].model_create_arrays.restype = C.c_void_p
    links["cuda_helpers.so"].do_gpu_cudaHostAlloc.restype = C.c_void_p
    links["model_arrays.so"].get_data_pointer.restype = C.c_void_p
    return links


def test_reference_driver_call_sequence(gpu, oracle_lib, tmp_path):
    from flyvec_amd import Trainer, build, synthetic
    to = oracle_lib
    V, hid, W, batch, Nep = 300, 48, 11, 700, 3
    tokens, offsets = small_corpus(30000, V, seed=1)
    R = synthetic.synapses(hid, V, seed=2, sigma=0.02)

    links = _bind(tmp_path)
    model_descriptor, model_arrays = links["model_descriptor.so"], links["model_arrays.so"]
    cuda_helpers, model, prune_input = links["cuda_helpers.so"], links["cuda_funcs.so"], links["prune_input.so"]

    num_gpus = cuda_helpers.get_cuda_num_devices()
    assert num_gpus == 1
    DSCR = model_descriptor.model_create_descriptor(C.c_int32(num_gpus))
    DATA = model_arrays.model_create_arrays(C.c_int32(num_gpus))
    n_tok = len(tokens)
    INPUT = cuda_helpers.do_gpu_cudaHostAlloc(C.c_uint64(n_tok * 4))
    INPUT_np = np.ctypeslib.as_array(C.cast(INPUT, C.POINTER(C.c_int32)), shape=(n_tok,))
    np.copyto(INPUT_np, tokens)
    vocabulary_size = np.uint64(np.max(INPUT_np) + 1)
    assert vocabulary_size == V
    n_sent = len(offsets) - 1
    n_phr = prune_input.getnum_samples(C.c_void_p(offsets.ctypes.data), C.c_uint64(n_sent), C.c_uint64(W))
    PHR = cuda_helpers.do_gpu_cudaHostAlloc(C.c_uint64((n_phr + 1) * 8))
    prune_input.compute_offset_phrases(C.c_void_p(PHR), C.c_void_p(offsets.ctypes.data), C.c_uint64(n_sent), C.c_uint64(W))
    d = C.c_void_p(DSCR)
    for value, key in ((1, b"IM_HEIGHT"), (11, b"IM_WIDTH"), (1, b"Nchannels"), (C.c_uint64(n_phr), b"Ns_1"), (W, b"W"),
                       (1, b"ST"), (hid, b"hid"), (batch, b"Num"), (C.c_uint64(int(vocabulary_size)), b"vocabulary_size"),
                       (1, b"sparse_input"), (1, b"frequency_scaling")):
        model_descriptor.set_model_param_int(value, key, d)
    for value, key in ((1e-3, b"initial_learning_rate"), (0.0, b"delta"), (1e-30, b"prec"), (0.0, b"mu"), (0.02, b"sigma"),
                       (1.0, b"Lmid"), (1.0, b"Lbase")):
        model_descriptor.set_model_param_float(C.c_float(value), key, d)
    model_descriptor.compute_model_derived_parameters(d)
    model_descriptor.print_model_params(d)
    model_arrays.model_arrays_allocate_memory(d, C.c_void_p(DATA), C.c_int32(num_gpus))
    model_arrays.set_up_INPUT_pointer(b"INPUT", C.c_void_p(DATA), d, C.c_void_p(INPUT), C.c_void_p(PHR), b"i4", C.c_int32(0))
    model_arrays.compute_inverse_word_frequency(C.c_void_p(DATA), d, C.c_void_p(INPUT), C.c_uint64(n_tok), C.c_int32(0))
    SYN = C.cast(model_arrays.get_data_pointer(b"synapses", C.c_void_p(DATA), C.c_int32(0)), C.POINTER(C.c_float))
    SYN_np = np.ctypeslib.as_array(SYN, shape=(hid, 2 * V))
    np.copyto(SYN_np, R)
    saved = []
    for ep in range(Nep):
        model_arrays.do_reshuffle_indices(d, C.c_void_p(DATA), C.c_int32(0))
        model.launch_epoch_INPUT_AS_INT(d, C.c_void_p(DATA), C.c_int32(num_gpus), C.c_uint64(ep), C.c_uint64(Nep))
        saved.append(SYN_np.copy())

    model_arrays.flyvec_legacy_release(d, C.c_void_p(DATA))   # not in the reference: frees what the handles hold
    t = Trainer(V, hid, W, batch, initial_learning_rate=1e-3, tie_rule=1)
    t.set_stale_tail(True)
    t.set_corpus(tokens, offsets)
    assert t.num_windows == n_phr
    starts = np.ctypeslib.as_array(C.cast(PHR, C.POINTER(C.c_uint64)), shape=(n_phr,))
    assert np.array_equal(starts, t.window_starts())
    assert t.dense_launches == 1        # the released model no longer counts as a second trainer
    t.set_weights(R)
    invf = to.inverse_frequency(tokens, V)
    assert np.array_equal(starts, to.window_starts(offsets, W))
    Wo = R.copy()
    t.shuffle(0)                        # the shuffle model_arrays_allocate_memory makes (flyvec/src/model_arrays.cu:180-198)
    assert n_phr % batch != 0 and n_phr > batch   # the last minibatch is a partial one behind a full one
    for ep in range(Nep):
        t.shuffle(ep + 1)
        perm = t.get_permutation()
        assert np.array_equal(np.sort(perm), np.arange(n_phr, dtype=np.uint64))
        t.run_epoch(ep, Nep)
        assert np.array_equal(t.get_weights().view(np.uint32), saved[ep].view(np.uint32)), ep
        to.train_steps(Wo, tokens, starts, perm, 0, batch, n_phr // batch + 1, W, invf, to.epoch_eps(1e-3, ep, Nep),
                       tie_rule=1, stale_tail=True)
        assert np.array_equal(Wo.view(np.uint32), saved[ep].view(np.uint32)), f"checker, epoch {ep}"
    t.close()
    assert not np.array_equal(saved[0], R) and np.isfinite(saved[-1]).all()


def test_window_matrix_through_set_data_pointer(gpu, oracle_lib, tmp_path):
    """flyvec/src/model_arrays.cu:320 set_data_pointer("INPUT", arrays, descriptor, ptr, "i4", device), the
    reference's six arguments: ptr is a matrix of Ns_1 windows already cut out, IM_HEIGHT * IM_WIDTH * Nchannels
    ids per row. One epoch over it equals the checker's over the same windows; the matrix can be the caller's own
    memory (flyvec_legacy_set_synapses, an addition)."""
    from flyvec_amd import Trainer, synthetic
    to = oracle_lib
    V, hid, W, batch = 120, 32, 11, 256
    rng = np.random.default_rng(5)
    n_win = 3 * batch + 57
    links = _bind(tmp_path)
    model_descriptor, model_arrays, cuda_helpers, model = (links["model_descriptor.so"], links["model_arrays.so"],
                                                           links["cuda_helpers.so"], links["cuda_funcs.so"])
    INPUT = cuda_helpers.do_gpu_cudaHostAlloc(C.c_uint64(n_win * W * 4))
    windows = np.ctypeslib.as_array(C.cast(INPUT, C.POINTER(C.c_int32)), shape=(n_win, W))
    windows[:] = synthetic.zipf_ids(n_win * W, V, seed=9).reshape(n_win, W)
    windows[rng.random(windows.shape) < 0.02] = -1
    windows[-1, -1] = V - 1
    DSCR = model_descriptor.model_create_descriptor(C.c_int32(1))
    DATA = model_arrays.model_create_arrays(C.c_int32(1))
    d, a = C.c_void_p(DSCR), C.c_void_p(DATA)
    for value, key in ((1, b"IM_HEIGHT"), (W, b"IM_WIDTH"), (1, b"Nchannels"), (C.c_uint64(n_win), b"Ns_1"), (W, b"W"),
                       (1, b"ST"), (hid, b"hid"), (batch, b"Num"), (C.c_uint64(V), b"vocabulary_size"),
                       (1, b"sparse_input"), (1, b"frequency_scaling")):
        model_descriptor.set_model_param_int(value, key, d)
    for value, key in ((2e-3, b"initial_learning_rate"), (0.0, b"delta"), (1e-30, b"prec")):
        model_descriptor.set_model_param_float(C.c_float(value), key, d)
    model_descriptor.compute_model_derived_parameters(d)
    model_arrays.model_arrays_allocate_memory(d, a, C.c_int32(1))
    model_arrays.set_data_pointer(b"INPUT", a, d, C.c_void_p(INPUT), b"i4", C.c_int32(0))
    model_arrays.set_data_pointer(b"no such array", a, d, C.c_void_p(INPUT), b"i4", C.c_int32(0))   # reported, ignored
    R = synthetic.synapses(hid, V, seed=3, sigma=0.02)
    mine = R.copy()
    model_arrays.flyvec_legacy_set_synapses(a, C.c_void_p(mine.ctypes.data))
    assert model_arrays.get_data_pointer(b"synapses", a, C.c_int32(0)) == mine.ctypes.data
    model.launch_epoch_INPUT_AS_INT(d, a, C.c_int32(1), C.c_uint64(0), C.c_uint64(5))
    model_arrays.flyvec_legacy_release(d, a)

    flat = windows.reshape(-1).copy()
    starts = np.arange(n_win, dtype=np.uint64) * np.uint64(W)
    t = Trainer(V, hid, W, batch, initial_learning_rate=2e-3, tie_rule=1)
    t.set_corpus_starts(flat, starts)
    t.shuffle(0)
    perm = t.get_permutation()
    t.close()
    Wo = R.copy()
    to.train_steps(Wo, flat, starts, perm, 0, batch, n_win // batch + 1, W, to.inverse_frequency(flat, V),
                   to.epoch_eps(2e-3, 0, 5), tie_rule=1, stale_tail=True)
    assert np.array_equal(mine.view(np.uint32), Wo.view(np.uint32)) and not np.array_equal(mine, R)


def test_corpus_with_a_given_window_table(gpu, oracle_lib):
    """fv_trainer_set_corpus_starts: the table built elsewhere gives the same training as the offsets; a window
    that does not fit the corpus is refused."""
    from flyvec_amd import Trainer, _lib, synthetic
    V, K, w, B = 200, 32, 5, 300
    tokens, offsets = small_corpus(8000, V, seed=3)
    starts = oracle_lib.window_starts(offsets, w)
    W0 = synthetic.synapses(K, V, seed=1)
    got = []
    for given in (False, True):
        t = Trainer(V, K, w, B, initial_learning_rate=1e-3)
        if given:
            t.set_corpus_starts(tokens, starts)
        else:
            t.set_corpus(tokens, offsets)
        t.set_weights(W0)
        t.shuffle(5)
        t.run_epoch(0, 4)
        got.append((t.get_weights(), t.inverse_frequency(), t.window_starts()))
        if given:
            bad = starts.copy()
            bad[7] = len(tokens) - w + 1
            with pytest.raises(_lib.FlyvecError) as e:
                t.set_corpus_starts(tokens, bad)
            assert e.value.code == _lib.FV_ERR_DATA
        t.close()
    assert all(np.array_equal(a, b) for a, b in zip(*got))
