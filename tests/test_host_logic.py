"""Host-side mirror of the reference's driver and wrapper: CLI surface, checkpoint naming,
synthetic generators, byte model, bench argument handling.  No GPU needed."""
import os
import subprocess
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_cli_defaults_match_the_reference_console_script():
    # flyvec/train_flyvec.py:31-47
    from flyvec_amd.train_flyvec import build_parser
    a = build_parser().parse_args(["enc.npy", "off.npy"])
    assert (a.output_dir, a.save_every, a.ckpt_prefix, a.starting_checkpoint) == (".", 1, "flyvec_model", None)
    assert (a.W, a.hid, a.initial_learning_rate, a.delta, a.mu, a.sigma) == (11, 400, 0.002, 0.0, 0.0, 0.02)
    assert (a.Nep, a.batch_size, a.prec) == (15, 10000, 1.0e-30)
    b = build_parser().parse_args(["e", "o", "-o", "out", "-s", "3", "-b", "64"])  # short flags of the twin
    assert (b.output_dir, b.save_every, b.batch_size) == ("out", 3, 64)


def test_checkpoint_epoch_parsing():
    from flyvec_amd.train_flyvec import checkpoint_epoch
    assert checkpoint_epoch("out/flyvec_model_H_400_W_11_LR_0.002_7") == 7      # the reference's form
    assert checkpoint_epoch("out/flyvec_model_H_400_W_11_LR_0.002_12.npy") == 12  # and the file numpy.save wrote


def test_console_scripts_are_registered():
    text = open(os.path.join(ROOT, "setup.py")).read()
    assert "flyvec_train=flyvec_amd.train_flyvec:main" in text
    assert "flyvec_compile=flyvec_amd.train_flyvec:init" in text


def test_synthetic_corpus_contract():
    from flyvec_amd import synthetic
    tokens, offsets = synthetic.corpus(50000, 300)
    assert tokens.dtype == np.int32 and offsets.dtype == np.uint64
    assert tokens.min() >= 1 and tokens.max() == 299           # V is inferred as max + 1
    assert offsets[0] == 0 and offsets[-1] == 50000 and (np.diff(offsets.astype(np.int64)) >= 1).all()
    assert 15 < np.diff(offsets.astype(np.int64)).mean() < 35  # geometric, mean 25
    counts = np.bincount(tokens)
    assert counts[1] > counts[2] > counts[5] > counts[50]      # Zipf head
    idx = synthetic.window_indices(100, 11, 300)
    assert idx.shape == (100, 11) and (idx[:, 5] >= 300).all() and (np.delete(idx, 5, axis=1) < 300).all()
    t2, o2 = synthetic.corpus(50000, 300)
    assert np.array_equal(tokens, t2) and np.array_equal(offsets, o2)  # seeded


def test_byte_model_matches_the_baseline_figures():
    sys.path.insert(0, ROOT)
    import bench
    assert bench.step_byte_model(400, 40000, 11, 10000) == 369_760_000
    assert bench.step_byte_model(1000, 100000, 15, 50000) == 4_212_000_000
    assert bench.hash_bytes_per_window(400, 11) == 17_700
    per = bench.kernel_bytes(400, 40000, 11, 10000)
    # the kernels of the step as six launches move the model's bytes; the single dense launch moves the matrix once each way
    six = sum(per[k] for k in ("gather_winner", "group_xx", "sparse_owners", "absmax_ds", "update", "slot_update"))
    assert 369_760_000 - 200_000 <= six <= 369_760_000 + 200_000
    assert per["dense_update"] == 8 * 400 * 40000 + 8 * 10000 * 11
    # with the single dense launch the sparse launch is held to the model's whole sparse term, 16 B w
    assert bench.kernel_bytes(400, 40000, 11, 10000, single_dense_launch=True)["sparse_owners"] == 16 * 10000 * 11 == 1_760_000
    # the bytes the scheme has to move: the matrix once each way
    assert bench.step_moved_model(400, 40000, 11, 10000) == 176_000_000 + 128_000_000 + 1_760_000 == 305_760_000
    assert bench.frac_fields("x", 8.0e12, 2.0) == {"x_frac": 0.5}
    assert bench.frac_fields("x", 8.0e12, 0.5) == {"x_frac": None, "x_byte_model_comparison": 2.0}


def test_bench_reads_counters_from_the_profile_summaries():
    sys.path.insert(0, ROOT)
    import bench
    for which in ("step", "large"):
        c = bench.profile_counters(which)
        assert {"gather_winner", "sparse_owners"} <= set(c), which
        assert bench.traffic_bytes(c, "gather_winner") > 0
        assert c["gather_winner"]["valu_insts"] > 0
    assert bench.traffic_bytes({}, "gather_winner") is None


def test_bench_refuses_more_than_one_gpu():
    out = subprocess.run([sys.executable, os.path.join(ROOT, "bench.py"), "--gpus", "2"], capture_output=True, text=True)
    assert out.returncode != 0 and "one GPU" in (out.stderr + out.stdout)


def test_vocab_tokenizer():
    from flyvec_amd.core import VocabTokenizer
    tok = VocabTokenizer(["<UNK>", "hello", "world"])
    assert tok.tokenize("Hello World") == ["hello", "world"]
    assert tok.token2id("hello") == 1 and tok.token2id("nope") == 0 and tok.id2token(2) == "world"
    assert tok.n_vocab() == 3
