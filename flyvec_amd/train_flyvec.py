"""``flyvec_train`` / ``flyvec_compile``: the reference's training CLI over libflyvec_hip.so.

Mirrors flyvec/train_flyvec.py:30-263 (and its argparse twin flyvec/flyvec_train.py:93-114):
same positional arguments, same options and defaults, same set-up order (corpus -> vocabulary
size -> window table -> 1/frequency -> initial or resumed weights), same epoch loop (reshuffle,
run epoch, checkpoint) and the same checkpoint name
``{prefix}_H_{hid}_W_{W}_LR_{lr}_{epoch}.npy`` holding the K x 2V fp32 matrix.

Differences, all supersets: ``-o/-s/-b`` short flags (the twin has them, the README uses ``-o``);
``--starting_checkpoint`` accepts a path ending in ``.npy`` (the reference's
``int(path.split("_")[-1])`` raises on it); ``--seed`` makes a run repeatable.
"""
import argparse
import sys
import time
from pathlib import Path

import numpy as np


def init(argv=None):
    """``flyvec_compile``: build the native library (flyvec/train_flyvec.py:25-27 runs short_make)."""
    from . import build
    path = build.build(verbose=True)
    print(f"built {path}")
    return 0


def build_parser():
    p = argparse.ArgumentParser(prog="flyvec_train", description="Train FlyVec synapses on one MI355X")
    p.add_argument("encodings_source", type=str,
                   help="Path to the tokens encoded as an ID. (eltype should be np.int32)")
    p.add_argument("offsets_source", type=str,
                   help="Path to the offsets array indicating where each chunk of text starts "
                        "(eltype should be np.uint64, first value should be 0)")
    p.add_argument("--output_dir", "-o", default=".", type=str,
                   help="Directory in which to save the checkpoints. Created if it does not exist")
    p.add_argument("--save_every", "-s", type=int, default=1, help="How many epochs to run before saving a checkpoint")
    p.add_argument("--ckpt_prefix", default="flyvec_model", type=str, help="Prefix to name each checkpoint")
    p.add_argument("--starting_checkpoint", type=str, default=None, help="Path to .npy file of saved checkpoint")
    p.add_argument("--W", default=11, type=int, help="Size of the W-gram sliding window")
    p.add_argument("--hid", default=400, type=int, help="Number of hidden units (neurons)")
    p.add_argument("--initial_learning_rate", default=0.002, type=float, help="Initial learning rate")
    p.add_argument("--delta", default=0.0, type=float, help="Anti-Hebbian strength on the second neuron of a window (flyvec/src/cuda_funcs.cu:1230 schedules it over the epochs)")
    p.add_argument("--Lmid", default=1.0, type=float, help="Weight of a window's centre position (the reference holds 1.0 and has no flag for it; flyvec/src/cuda_funcs.cu:266-327, 675-697)")
    p.add_argument("--Lbase", default=1.0, type=float, help="Weight of the other window positions (likewise)")
    p.add_argument("--prune_duplicates", action="store_true", help="Drop a token that an earlier position of its window holds (the sampler variant the reference has switched off, flyvec/src/cuda_funcs.cu:938-979)")
    p.add_argument("--stale_last_batch", action="store_true", help="Train an epoch's final partial minibatch with the previous minibatch's rows behind its own, as the reference's launch sizes do (flyvec/src/cuda_funcs.cu:1679 against :1700-1732); default: the remainder only")
    p.add_argument("--mu", default=0.0, type=float, help="Mean of the random normal initialisation")
    p.add_argument("--sigma", default=0.02, type=float, help="Stdev of the random normal initialisation")
    p.add_argument("--Nep", default=15, type=int, help="Maximum number of epochs, fewer if starting from a checkpoint")
    p.add_argument("--batch_size", "-b", default=10000, type=int, help="Minibatch size")
    p.add_argument("--prec", default=1.0e-30, type=float, help="Precision, avoid dividing by 0")
    p.add_argument("--seed", default=None, type=int, help="Seed of the weight initialisation and the shuffles")
    p.add_argument("--tie_rule", default="lowest", choices=["lowest", "reference"],
                   help="argmax tie-break: lowest neuron index, or the reference kernel's reduction order")
    return p


def checkpoint_epoch(path):
    """Epoch number at the end of a checkpoint name (flyvec/train_flyvec.py:239), '.npy' allowed."""
    stem = str(path)
    if stem.endswith(".npy"):
        stem = stem[:-4]
    return int(stem.split("_")[-1])


def train(args, log=print):
    from .engine import Trainer

    output_dir = Path(args.output_dir)
    output_dir.mkdir(parents=True, exist_ok=True)
    output = str(output_dir / f"{args.ckpt_prefix}_H_{args.hid}_W_{args.W}_LR_{args.initial_learning_rate}_")

    tokens = np.load(args.encodings_source, mmap_mode="r")
    offsets = np.load(args.offsets_source, mmap_mode="r")
    vocabulary_size = int(np.max(tokens) + 1)  # flyvec/train_flyvec.py:168
    log(f"Determined a vocabulary size of {vocabulary_size}")
    N = 2 * vocabulary_size

    trainer = Trainer(vocab=vocabulary_size, hid=args.hid, window=args.W, batch=args.batch_size,
                      initial_learning_rate=args.initial_learning_rate, delta=args.delta, prec=args.prec,
                      tie_rule=1 if args.tie_rule == "reference" else 0, lmid=args.Lmid, lbase=args.Lbase,
                      prune_duplicates=args.prune_duplicates)
    trainer.set_stale_tail(args.stale_last_batch)
    log("Copying input...")
    trainer.set_corpus(tokens, offsets)
    log(f"Number of phrases:  {trainer.num_windows}")

    log("Setting initial weights...")
    epoch_start = 0
    if args.starting_checkpoint is not None:
        R = np.load(args.starting_checkpoint, mmap_mode="r")
        epoch_start = checkpoint_epoch(args.starting_checkpoint)
    else:
        rng = np.random.default_rng(args.seed)
        R = np.float32(rng.normal(args.mu, args.sigma, (args.hid, N)))
    trainer.set_weights(R)

    seed = args.seed if args.seed is not None else int(time.time_ns() & 0xFFFFFFFF)
    trainer.shuffle(seed)  # the reference shuffles once at allocation (flyvec/src/model_arrays.cu:184-197)
    saved = []
    for i, ep in enumerate(range(epoch_start, args.Nep)):
        log(f"epoch ID =  {ep}")
        for r, nrm in enumerate(trainer.row_norms(10)):
            print(f"Lp_norm(syn[{r}]) = {nrm:g}", file=sys.stderr)
        t1 = time.time()
        trainer.shuffle(seed + 1 + ep)
        t11 = time.time()
        trainer.run_epoch(ep, args.Nep)
        t2 = time.time()
        log(f"time per epoch =  {t2 - t1} [s]   py_model_arrays_reshuffle_indices time =  {t11 - t1} [s]")
        if ((i + 1) % args.save_every) == 0 or i == (args.Nep - 1):
            trainer.save_weights(output + str(ep))
            saved.append(output + str(ep) + ".npy")
    trainer.close()
    return saved


def main(argv=None):
    args = build_parser().parse_args(argv)
    train(args)
    return 0


if __name__ == "__main__":
    sys.exit(main())
