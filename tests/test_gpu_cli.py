"""flyvec_train end to end: .npy in, checkpoints out, same names and layout as the reference
(flyvec/train_flyvec.py:151-152, 262-263), resumable, and usable by the hashing wrapper."""
import numpy as np
import pytest

from conftest import small_corpus

pytestmark = pytest.mark.gpu


def test_cli_trains_saves_resumes(gpu, oracle_lib, tmp_path):
    from flyvec_amd import FlyVec
    from flyvec_amd.train_flyvec import main
    V, K, w, B = 300, 64, 11, 256
    tokens, offsets = small_corpus(20000, V)
    np.save(tmp_path / "encodings.npy", tokens)
    np.save(tmp_path / "offsets.npy", offsets)
    out = tmp_path / "ckpt"
    argv = [str(tmp_path / "encodings.npy"), str(tmp_path / "offsets.npy"), "-o", str(out), "--hid", str(K),
            "--W", str(w), "-b", str(B), "--Nep", "3", "--save_every", "2", "--seed", "1",
            "--initial_learning_rate", "0.002"]
    assert main(argv) == 0
    names = sorted(p.name for p in out.iterdir())
    # epochs 0..2, saved when (i+1) % 2 == 0 or i == Nep - 1
    assert names == ["flyvec_model_H_64_W_11_LR_0.002_1.npy", "flyvec_model_H_64_W_11_LR_0.002_2.npy"]
    W2 = np.load(out / names[1])
    assert W2.shape == (K, 2 * V) and W2.dtype == np.float32 and W2.flags.c_contiguous
    assert np.isfinite(W2).all()

    # the checker over the same initial matrix and the same window orders (flyvec/train_flyvec.py:241, 253-263:
    # normal(mu, sigma) weights, a reshuffle before every epoch, eps = lr0 (1 - ep / Nep)) gives the same checkpoints
    from flyvec_amd import Trainer
    to = oracle_lib
    Wo = np.float32(np.random.default_rng(1).normal(0.0, 0.02, (K, 2 * V)))
    t = Trainer(V, K, w, B)
    t.set_corpus(tokens, offsets)
    starts, invf = to.window_starts(offsets, w), to.inverse_frequency(tokens, V)
    assert t.num_windows == len(starts) and len(starts) % B != 0
    t.shuffle(1)
    for ep in range(3):
        t.shuffle(1 + 1 + ep)
        to.train_steps(Wo, tokens, starts, t.get_permutation(), 0, B, len(starts) // B + 1, w, invf,
                       to.epoch_eps(0.002, ep, 3))
        if ep >= 1:
            assert np.array_equal(np.load(out / names[ep - 1]).view(np.uint32), Wo.view(np.uint32)), f"epoch {ep}"
    t.close()

    # same seed: same checkpoints
    out2 = tmp_path / "ckpt2"
    argv2 = list(argv)
    argv2[3] = str(out2)
    assert main(argv2) == 0
    assert np.array_equal(np.load(out2 / names[1]), W2)

    # resume from the epoch-1 checkpoint: runs epoch 1 and 2 again from that matrix
    out3 = tmp_path / "ckpt3"
    argv3 = list(argv)
    argv3[3] = str(out3)
    argv3 += ["--starting_checkpoint", str(out / names[0])]
    assert main(argv3) == 0
    assert sorted(p.name for p in out3.iterdir()) == ["flyvec_model_H_64_W_11_LR_0.002_2.npy"]

    # a trained checkpoint feeds the hashing wrapper
    model = FlyVec(out / names[1], tokenizer=["<UNK>"] + [f"t{i}" for i in range(1, V)], normalize_synapses=False)
    assert model.get_sparse_embedding("t5", 10)["embedding"].sum() <= 10


def test_cli_with_anti_hebbian_term(gpu, tmp_path):
    """--delta reaches the trainer and follows the epoch schedule of flyvec/src/cuda_funcs.cu:1230."""
    from flyvec_amd.train_flyvec import main
    V = 300
    tokens, offsets = small_corpus(20000, V)
    np.save(tmp_path / "encodings.npy", tokens)
    np.save(tmp_path / "offsets.npy", offsets)
    outs = {}
    for name, delta in (("plain", "0"), ("anti", "0.4")):
        out = tmp_path / name
        assert main([str(tmp_path / "encodings.npy"), str(tmp_path / "offsets.npy"), "-o", str(out), "--hid", "64",
                     "-b", "256", "--Nep", "2", "--save_every", "2", "--seed", "1", "--delta", delta]) == 0
        (ckpt,) = list(out.iterdir())
        outs[name] = np.load(ckpt)
        assert np.isfinite(outs[name]).all()
    assert not np.array_equal(outs["plain"], outs["anti"])
