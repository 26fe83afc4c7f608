"""The reference's own C ABI (flyvec/train_flyvec.py:62-263), served by libflyvec_hip.so under the reference's
five library names: driven here in the order and with the argument types the reference's driver uses, the
matrix it leaves must equal, bit for bit, what this library's own interface computes with the same settings
(the reference's tie rule, its treatment of the last minibatch, the same shuffle seeds)."""
import ctypes as C

import numpy as np
import pytest

from conftest import small_corpus

pytestmark = pytest.mark.gpu


def test_reference_driver_call_sequence(gpu, tmp_path):
    from flyvec_amd import Trainer, build, synthetic
    V, hid, W, batch, Nep = 300, 48, 11, 700, 3
    tokens, offsets = small_corpus(30000, V, seed=1)
    R = synthetic.synapses(hid, V, seed=2, sigma=0.02)

    links = {p.name: C.CDLL(str(p)) for p in build.install_legacy_names(tmp_path / "src")}
    model_descriptor, model_arrays = links["model_descriptor.so"], links["model_arrays.so"]
    cuda_helpers, model, prune_input = links["cuda_helpers.so"], links["cuda_funcs.so"], links["prune_input.so"]
    prune_input.getnum_samples.restype = C.c_uint64
    model_descriptor.model_create_descriptor.restype = C.c_void_p
    model_arrays.model_create_arrays.restype = C.c_void_p
    cuda_helpers.do_gpu_cudaHostAlloc.restype = C.c_void_p
    model_arrays.get_data_pointer.restype = C.c_void_p

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
    for ep in range(Nep):
        t.shuffle(ep)
        t.run_epoch(ep, Nep)
        assert np.array_equal(t.get_weights().view(np.uint32), saved[ep].view(np.uint32)), ep
    t.close()
    assert not np.array_equal(saved[0], R) and np.isfinite(saved[-1]).all()


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
