"""The C-ABI library: builds, loads, exports every symbol include/flyvec_hip.h declares, and its
Python mirror declares the same set.  No compute call is made (this suite runs without a GPU)."""
import ctypes as C
import os
import re

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
HEADER = os.path.join(ROOT, "include", "flyvec_hip.h")


def declared_symbols():
    text = open(HEADER).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fv_[a-z0-9_]+)\s*\(", text)))


def test_header_declares_the_expected_surface():
    syms = declared_symbols()
    for must in ("fv_last_error", "fv_count_windows", "fv_build_window_starts", "fv_inverse_frequency",
                 "fv_trainer_create", "fv_trainer_set_corpus", "fv_trainer_step", "fv_trainer_run_epoch",
                 "fv_hash_targets", "fv_hash_windows", "fv_hash_windows_dev"):
        assert must in syms
    assert len(syms) >= 40


def test_library_exports_every_declared_symbol():
    from flyvec_amd import _lib
    assert _lib.LIB_PATH.exists(), "run `python -m flyvec_amd.build` (or __graft_entry__.build()) first"
    lib = C.CDLL(str(_lib.LIB_PATH))
    missing = [s for s in declared_symbols() if not hasattr(lib, s)]
    assert not missing, f"declared in the header but not exported: {missing}"


def test_python_binding_covers_the_header():
    from flyvec_amd import _lib
    bound = set(_lib.SIGNATURES) | {"fv_last_error"}
    assert bound == set(declared_symbols())
    _lib.load()  # sets argtypes on every symbol; raises if one is absent


def test_struct_layout_matches_the_header():
    from flyvec_amd._lib import TrainConfig
    # uint64 + 4 x uint32 + 5 x float + uint32 = 48 bytes, no padding
    assert C.sizeof(TrainConfig) == 48
    assert TrainConfig.vocab.offset == 0 and TrainConfig.hid.offset == 8 and TrainConfig.prec.offset == 32
    assert TrainConfig.lmid.offset == 36 and TrainConfig.lbase.offset == 40 and TrainConfig.prune_duplicates.offset == 44


def test_argument_errors_need_no_device():
    from flyvec_amd import _lib
    lib = _lib.load()
    out = C.c_void_p()
    assert lib.fv_trainer_create(None, C.byref(out)) == _lib.FV_ERR_INVALID
    assert b"null" in lib.fv_last_error()
    cfg = _lib.TrainConfig(vocab=10, hid=4000, window=11, batch=10, tie_rule=0, initial_learning_rate=1e-3,
                           delta=0.0, prec=1e-30, lmid=1.0, lbase=1.0, prune_duplicates=0)
    assert lib.fv_trainer_create(C.byref(cfg), C.byref(out)) == _lib.FV_ERR_INVALID
    assert b"hid" in lib.fv_last_error()
    cfg.hid, cfg.delta = 400, float("nan")
    assert lib.fv_trainer_create(C.byref(cfg), C.byref(out)) == _lib.FV_ERR_INVALID
    assert b"delta" in lib.fv_last_error()
    cfg.delta, cfg.lmid = 0.0, float("nan")
    assert lib.fv_trainer_create(C.byref(cfg), C.byref(out)) == _lib.FV_ERR_INVALID
    assert b"Lmid" in lib.fv_last_error()
    cfg.lmid, cfg.prune_duplicates = 1.0, 2
    assert lib.fv_trainer_create(C.byref(cfg), C.byref(out)) == _lib.FV_ERR_INVALID
    assert b"prune_duplicates" in lib.fv_last_error()


def test_missing_library_fails_loudly(monkeypatch, tmp_path):
    from flyvec_amd import _lib
    monkeypatch.setattr(_lib, "_lib", None)
    monkeypatch.setattr(_lib, "LIB_PATH", tmp_path / "nope.so")
    with pytest.raises(FileNotFoundError, match="no CPU implementation"):
        _lib.load()


def test_without_a_gpu_the_product_raises_instead_of_falling_back():
    from flyvec_amd import _lib, Trainer
    try:
        n = _lib.device_count()
    except _lib.FlyvecError:
        n = 0
    if n > 0:
        pytest.skip("a GPU is present")
    with pytest.raises(_lib.FlyvecError):
        Trainer(vocab=100, hid=16, window=3, batch=8)


LEGACY_HEADER = os.path.join(ROOT, "include", "flyvec_legacy.h")
LEGACY_SYMBOLS = ["do_gpu_cudaMallocManaged", "do_cpu_malloc", "do_gpu_cudaHostAlloc", "get_cuda_num_devices",
                  "prune_input_data", "getnum_samples", "compute_offset_phrases", "model_create_descriptor",
                  "set_model_param_int", "set_model_param_float", "compute_model_derived_parameters",
                  "copy_model_params", "print_model_params", "model_create_arrays", "model_arrays_allocate_memory",
                  "push_INPUT_memory_to_GPU", "get_data_pointer", "set_data_pointer", "set_up_INPUT_pointer",
                  "compute_inverse_word_frequency", "do_reshuffle_indices", "launch_epoch_INPUT_AS_INT",
                  "launch_epoch_INPUT_AS_IMAGE", "launch_epoch_INPUT_AS_FLOAT"]


def test_legacy_surface_is_declared_and_exported(tmp_path):
    """The 24 symbols the reference's driver binds from its five shared objects (flyvec/train_flyvec.py:62-139)."""
    from flyvec_amd import _lib, build
    text = re.sub(r"/\*.*?\*/", "", open(LEGACY_HEADER).read(), flags=re.S)
    declared = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*)\s*\(", text))
    assert set(LEGACY_SYMBOLS) <= declared
    lib = C.CDLL(str(_lib.LIB_PATH))
    assert not [s for s in LEGACY_SYMBOLS if not hasattr(lib, s)]
    for extra in ("flyvec_legacy_release", "flyvec_legacy_set_synapses"):                # the two additions
        assert hasattr(lib, extra) and extra in declared
    links = build.install_legacy_names(tmp_path / "bin")
    assert sorted(p.name for p in links) == sorted(build.LEGACY_NAMES)
    for p in links:                                    # each name opens the one library
        assert hasattr(C.CDLL(str(p)), "launch_epoch_INPUT_AS_INT")
    # the descriptor needs no device
    lib.model_create_descriptor.restype = C.c_void_p
    d = lib.model_create_descriptor(C.c_int32(1))
    lib.set_model_param_int(C.c_uint64(123), b"vocabulary_size", C.c_void_p(d))
    lib.set_model_param_int(C.c_uint64(1), b"sparse_input", C.c_void_p(d))
    lib.set_model_param_float(C.c_float(0.5), b"delta", C.c_void_p(d))
    lib.compute_model_derived_parameters(C.c_void_p(d))
    lib.print_model_params(C.c_void_p(d))
