#!/usr/bin/env python3
"""Benchmark of the FlyVec hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one training minibatch (sampler -> gather-sum -> winner -> xx -> max|ds| -> update)
at the headline configuration: K = 400 neurons, V = 20000, w = 11, B = 10000 windows, on a
synthetic 10 M-token Zipf(1.07) corpus with geometric chunk lengths, fp32, everything resident in
HBM before the timed region.  One JSON line is printed:

  value              training windows / s over the K timed steps
  roofline           the dominant kernel of the step against the 8 TB/s HBM peak: achieved =
                     algorithmic bytes of that kernel per launch / its mean duration, measured with
                     HIP events on the trainer's stream
  step_roofline_frac (algorithmic bytes of the whole step / 8 TB/s) / measured time per step
  cpu_baseline       the CPU restatement of the same step (oracle/, C + OpenMP) timed on this host
  hash               the batched top-k hash (1,048,576 windows, k = 32, bit-packed) the same way,
                     with the reference's numpy per-word path as its CPU baseline
"""
import argparse
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

HBM_PEAK = 8.0e12  # B/s, MI355X

TRAIN = dict(K=400, V=20000, w=11, B=10000, n_tokens=10_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.07, mean_chunk=25)
# the 400 MB matrix that exceeds the 256 MB Infinity Cache; the corpus is shortened from 200 M to
# 20 M tokens (the step does not depend on its length)
LARGE = dict(K=1000, V=50000, w=15, B=50000, n_tokens=20_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.0, mean_chunk=40)
EPOCH = dict(K=400, V=20000, w=11, B=10000, n_tokens=100_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.07, mean_chunk=25)
HASH = dict(K=400, V=20000, w=11, k=32, n=1 << 20)


# HBM-side bytes per launch at the headline configuration, from two rocprofv3 --pmc runs of this
# script (FETCH_SIZE, then WRITE_SIZE; KiB per dispatch), each scaled by what the same counter reads
# for the plain copy kernel of --copy-calibration (FETCH_SIZE reads half the bytes copied: x2.0;
# WRITE_SIZE reads them all: x1.0). Traffic below the algorithmic bytes means the rest was served
# by the L2 caches.
MEASURED_TRAFFIC = {
    "dense_max_update": (33303.5 * 2.0 + 65249.7) * 1024,
    "gather_winner": (28514.5 * 2.0 + 817.5) * 1024,
    "sparse_owners": (5819.5 * 2.0 + 2993.3) * 1024,  # grouping by winner included
    "hash": (2478239.7 * 2.0 + 82381.6) * 1024,
    # the step as six launches (--dense-launches 2 --separate-grouping)
    "update": (32309.5 * 2.0 + 62498.2) * 1024,
    "absmax_ds": (31275.5 * 2.0 + 64.0) * 1024,
    "slot_update": (621.9 * 2.0 + 1501.2) * 1024,
    "group_xx": (312.9 * 2.0 + 87.2) * 1024,
}

# the same for --workload large-step (profiles/train_step_K1000_V50000_B50000.txt)
MEASURED_TRAFFIC_LARGE = {
    "gather_winner": (760768.6 * 2.0 + 5100.7) * 1024,
    "group_xx": (1249.9 * 2.0 + 316.0) * 1024,
    "sparse_owners": (30823.7 * 2.0 + 17905.1) * 1024,
    "absmax_ds": (195347.6 * 2.0 + 67.9) * 1024,
    "update": (195624.6 * 2.0 + 390612.4) * 1024,
    "slot_update": (3550.7 * 2.0 + 11373.4) * 1024,
}

# the two passes over W of a step (and the sparse elements' update) as one launch: W stays in
# registers between them, so the launch moves 8*K*N bytes of W while the byte model of the step
# counts the two passes' 12*K*N
DENSE_ONE = "dense_max_update"


def train_bytes(K, N, w, B):
    """Algorithmic HBM bytes per step and per kernel: every window gathers w rows of K floats once;
    W is read once for max|ds| and read + written once by the update; ds is never stored; token
    ids, 1/f lookups and the sparse count updates are 16 bytes per window position."""
    per = {
        "gather_winner": 4 * B * w * K,
        "group_xx": 8 * B,
        "sparse_owners": 8 * B * w,
        "absmax_ds": 4 * K * N,
        "update": 8 * K * N,
        "slot_update": 8 * B * w,
    }
    return 4 * B * w * K + 12 * K * N + 16 * B * w, per


def hash_bytes_per_window(K, w):
    return 4 * w * K + 4 * w + 8 * ((K + 63) // 64)


def bench_train(steps, warmup, cpu_seconds, c=TRAIN, dense_launches=0, separate_grouping=False):
    from flyvec_amd import Trainer, synthetic
    tokens, offsets = synthetic.corpus(c["n_tokens"], c["V"], s=c["zipf_s"], mean_chunk=c["mean_chunk"])
    W0 = synthetic.synapses(c["K"], c["V"], seed=5)
    t = Trainer(c["V"], c["K"], c["w"], c["B"], initial_learning_rate=c["lr0"], prec=c["prec"])
    t.set_dense_launches(dense_launches)
    t.set_grouping_launch(separate_grouping)
    t.set_corpus(tokens, offsets)
    nwin = t.num_windows
    perm = np.random.default_rng(6).permutation(nwin).astype(np.uint64)
    t.set_permutation(perm)
    t.set_weights(W0)
    eps = t.epoch_eps(0, c["n_epochs"])
    need = (warmup + 2 * steps) * c["B"]
    if need > nwin:
        raise SystemExit(f"{warmup}+2x{steps} steps need {need} windows, the corpus has {nwin}")

    for s in range(warmup):
        t.step(s * c["B"], c["B"], eps)
    t.sync()
    # timed region: exactly `steps` steps, device idle before and after
    t0 = time.perf_counter()
    for s in range(steps):
        t.step((warmup + s) * c["B"], c["B"], eps)
    t.sync()
    wall = time.perf_counter() - t0
    # the same number of steps again, timed by two HIP events on the trainer's stream
    total_ms, _ = t.time_steps((warmup + steps) * c["B"], steps, eps, per_kernel=False)
    ev_ms_per_step = total_ms / steps
    # per-kernel durations: each kernel of the last step launched back to back between two HIP
    # events on that stream (bracketing every kernel inside a step would add ~3 us of event
    # overhead to each); this destroys W, so it comes last
    kern_ms = t.time_kernels(reps=50)
    launches = t.dense_launches
    grouping_separate = t.grouping_launch
    t.close()

    N = 2 * c["V"]
    step_bytes, per_kernel = train_bytes(c["K"], N, c["w"], c["B"])
    if launches == 1:
        # max|ds|, the update and the slot update ran as one launch (timed under the first name;
        # the others are empty)
        parts = ("absmax_ds", "update", "slot_update")
        kern_ms[DENSE_ONE] = sum(kern_ms.pop(k) for k in parts)
        per_kernel[DENSE_ONE] = sum(per_kernel.pop(k) for k in parts)
    if not grouping_separate:
        # the sparse launch has grouped the windows by winner itself: no grouping launch ran
        kern_ms["sparse_owners"] += kern_ms.pop("group_xx")
        per_kernel["sparse_owners"] += per_kernel.pop("group_xx")
    dom = max(kern_ms, key=kern_ms.get)
    achieved = per_kernel[dom] / (kern_ms[dom] * 1e-3)
    ms_per_step = wall / steps * 1e3
    out = {
        "value": steps * c["B"] / wall,
        "ms_per_step": ms_per_step,
        "event_ms_per_step": ev_ms_per_step,
        "kernel_ms": kern_ms,
        "roofline": {"bound": "hbm", "kernel": dom, "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9,
                     "unit": "GB/s", "frac": achieved / HBM_PEAK,
                     "traffic": (MEASURED_TRAFFIC if c is TRAIN else MEASURED_TRAFFIC_LARGE).get(dom),
                     "algorithmic_bytes": per_kernel[dom]},
        "dense_launches": launches,
        "grouping_launch": "own" if grouping_separate else "in sparse_owners",
        "step_roofline_frac": (step_bytes / HBM_PEAK) / (ms_per_step * 1e-3),
        "step_algorithmic_bytes": step_bytes,
        "n_windows": nwin,
    }

    if dom == DENSE_ONE:
        # what the launch has to move (W read once, written once) and the rate on that count
        moved = 8 * c["K"] * N + 8 * c["B"] * c["w"]
        out["roofline"]["moved_bytes"] = moved
        out["roofline"]["frac_of_moved"] = moved / (kern_ms[dom] * 1e-3) / HBM_PEAK

    if cpu_seconds > 0:
        from oracle import train_oracle as to
        starts = to.window_starts(offsets, c["w"])
        invf = to.inverse_frequency(tokens, c["V"])
        Wc = W0.copy()
        to.train_steps(Wc, tokens, starts, perm, 0, c["B"], 2, c["w"], invf, eps, c["prec"])  # warm caches
        done, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < cpu_seconds and (done + 8) * c["B"] <= nwin:
            to.train_steps(Wc, tokens, starts, perm, done * c["B"], c["B"], 8, c["w"], invf, eps, c["prec"])
            done += 8
        dt = time.perf_counter() - t0
        out["cpu_baseline"] = {"value": done * c["B"] / dt, "unit": "windows/s", "cores": to.num_threads(),
                               "kind": "port",
                               "sample": f"{done} steps of the same workload (B={c['B']}) by the C/OpenMP "
                                         f"restatement of the reference step, {dt:.1f} s"}
    return out


def bench_epoch(c=EPOCH):
    """One full epoch as flyvec_train runs it (flyvec/train_flyvec.py:253-263): reshuffle, every
    minibatch of the corpus, then one checkpoint written as .npy; set-up is timed beside it."""
    import tempfile
    from flyvec_amd import Trainer, synthetic
    t0 = time.perf_counter()
    tokens, offsets = synthetic.corpus(c["n_tokens"], c["V"], s=c["zipf_s"], mean_chunk=c["mean_chunk"])
    W0 = synthetic.synapses(c["K"], c["V"], seed=5)
    t_gen = time.perf_counter() - t0
    t = Trainer(c["V"], c["K"], c["w"], c["B"], initial_learning_rate=c["lr0"], prec=c["prec"])
    t0 = time.perf_counter()
    t.set_corpus(tokens, offsets)      # upload, window table, 1/frequency, identity order: all on the device
    t.set_weights(W0)
    t.sync()
    t_setup = time.perf_counter() - t0
    nwin = t.num_windows
    t.shuffle(1)
    t.run_epoch(0, c["n_epochs"])      # warm-up epoch: first-touch of every buffer
    t0 = time.perf_counter()
    t.shuffle(2)
    t.sync()
    t_shuffle = time.perf_counter() - t0
    t1 = time.perf_counter()
    t.run_epoch(1, c["n_epochs"])      # returns when the device has finished
    t_steps = time.perf_counter() - t1
    t2 = time.perf_counter()
    W = t.get_weights()
    with tempfile.TemporaryDirectory() as d:
        np.save(os.path.join(d, "flyvec_model_1.npy"), W)
    t_ckpt = time.perf_counter() - t2
    total = time.perf_counter() - t0
    t.close()
    n_steps = (nwin + c["B"] - 1) // c["B"]
    step_bytes, _ = train_bytes(c["K"], 2 * c["V"], c["w"], c["B"])
    return {"value": nwin / total, "seconds_per_epoch": total, "n_windows": nwin, "n_steps": n_steps,
            "ms_per_step": t_steps / n_steps * 1e3,
            "breakdown_s": {"shuffle": t_shuffle, "minibatch_loop": t_steps, "checkpoint": t_ckpt,
                            "setup_once": t_setup, "synthetic_corpus_generation": t_gen},
            "step_roofline_frac": (step_bytes * (nwin / c["B"]) / HBM_PEAK) / t_steps}


def bench_hash(reps, cpu_seconds):
    from flyvec_amd import Hasher, synthetic
    from flyvec_amd._lib import DeviceBuffer
    c = HASH
    W = synthetic.synapses(c["K"], c["V"], seed=1)
    idx = synthetic.window_indices(c["n"], c["w"], c["V"], seed=7)
    h = Hasher(W)
    d_idx = DeviceBuffer.from_numpy(idx)
    d_bits = DeviceBuffer(c["n"] * h.words * 8)
    h.time_windows(d_idx, c["n"], c["w"], c["k"], bits_buf=d_bits, reps=2)  # warm-up
    ms = h.time_windows(d_idx, c["n"], c["w"], c["k"], bits_buf=d_bits, reps=reps)
    h.sync()
    bpw = hash_bytes_per_window(c["K"], c["w"])
    achieved = bpw * c["n"] / (ms * 1e-3)
    out = {"metric": "hash codes/s", "value": c["n"] / (ms * 1e-3), "unit": "codes/s", "ms_per_batch": ms,
           "config": {"workload": f"batched contextual hash: K={c['K']} V={c['V']} w={c['w']} k={c['k']} "
                                  f"n={c['n']} windows, 7 uint64 words out"},
           "dtype": "f32",
           "roofline": {"bound": "hbm", "kernel": "hash", "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9,
                        "unit": "GB/s", "frac": achieved / HBM_PEAK, "traffic": MEASURED_TRAFFIC["hash"],
                        "algorithmic_bytes": bpw * c["n"]}}
    if cpu_seconds > 0:
        from oracle import hash_oracle as ho
        ids = synthetic.zipf_ids(4096, c["V"], seed=2)
        n_done, t0 = 0, time.perf_counter()
        while time.perf_counter() - t0 < cpu_seconds:
            ho.hash_targets_loop(W, ids, 50)
            n_done += len(ids)
        dt = time.perf_counter() - t0
        sample = idx[:32768]
        t1 = time.perf_counter()
        ho.hash_windows(W, sample, c["k"])
        dtw = time.perf_counter() - t1
        out["cpu_baseline"] = {"value": n_done / dt, "unit": "codes/s", "cores": 1, "kind": "port",
                               "sample": f"numpy per-word path (argsort, k=50) on 4096 Zipf target ids, "
                                         f"repeated for {dt:.1f} s",
                               "windows_vectorised_numpy": {"value": len(sample) / dtw, "unit": "codes/s",
                                                            "sample": f"{len(sample)} windows of the same batch"}}
    h.close()
    d_idx.free()
    d_bits.free()
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline sample length (0 = skip)")
    ap.add_argument("--no-hash", action="store_true")
    ap.add_argument("--separate-grouping", action="store_true",
                    help="group the windows by winner in a launch of its own (the default does it inside the sparse launch)")
    ap.add_argument("--dense-launches", type=int, choices=[0, 1, 2], default=0,
                    help="the passes over W of a step as one launch (1), two (2), or as the library chooses (0)")
    ap.add_argument("--workload", choices=["step", "large-step", "epoch"], default="step",
                    help="step: the headline minibatch step (default); large-step: K=1000, V=50000, w=15, "
                         "B=50000 (400 MB matrix); epoch: one full epoch over 100 M tokens with shuffle and "
                         "checkpoint")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB copy kernel (yardstick for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    from flyvec_amd import _lib
    info = _lib.device_info()
    if args.workload == "epoch":
        c = EPOCH
        ep = bench_epoch(c)
        print(json.dumps({
            "metric": "train windows/s over one full epoch", "value": ep["value"], "unit": "windows/s",
            "n_gpus": 1, "steps": ep["n_steps"], "warmup": ep["n_steps"], "ms_per_step": ep["ms_per_step"],
            "higher_is_better": True, "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
            "config": {"workload": f"full training epoch: {c['n_tokens']} Zipf(1.07) tokens, K={c['K']} "
                                   f"Nvoc={c['V']} w={c['w']} B={c['B']}, {ep['n_windows']} windows, device "
                                   f"shuffle before and one .npy checkpoint after"},
            "device": info["name"].strip(), "seconds_per_epoch": ep["seconds_per_epoch"],
            "breakdown_s": ep["breakdown_s"], "step_roofline_frac": ep["step_roofline_frac"]}))
        return
    c = LARGE if args.workload == "large-step" else TRAIN
    if args.workload == "large-step":
        args.steps, args.warmup, args.no_hash = min(args.steps, 50), min(args.warmup, 5), True
    tr = bench_train(args.steps, args.warmup, args.cpu_seconds, c, args.dense_launches, args.separate_grouping)
    line = {
        "metric": f"train windows/s at K={c['K']},Nvoc={c['V'] // 1000}k",
        "value": tr["value"], "unit": "windows/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": tr["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"single training minibatch step: K={c['K']} Nvoc={c['V']} w={c['w']} B={c['B']}, "
                               f"{c['n_tokens']} Zipf({c['zipf_s']}) tokens, geometric chunks (mean {c['mean_chunk']}), "
                               f"{tr['n_windows']} windows, lr 2e-4, fp32"},
        "device": info["name"].strip(),
        "roofline": tr["roofline"],
        "step_roofline_frac": tr["step_roofline_frac"],
        "step_algorithmic_bytes": tr["step_algorithmic_bytes"],
        "event_ms_per_step": tr["event_ms_per_step"],
        "kernel_ms": tr["kernel_ms"],
        "dense_launches": tr["dense_launches"],
        "grouping_launch": tr["grouping_launch"],
    }
    if "cpu_baseline" in tr:
        line["cpu_baseline"] = tr["cpu_baseline"]
    if not args.no_hash:
        line["hash"] = bench_hash(reps=10, cpu_seconds=min(args.cpu_seconds, 5.0))
    if args.copy_calibration:
        nbytes = 1 << 30
        ms = _lib.calibration_copy(nbytes, reps=5)
        line["copy_calibration"] = {"bytes_read": nbytes, "bytes_written": nbytes, "ms": ms,
                                    "GB/s": 2 * nbytes / (ms * 1e-3) / 1e9}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
