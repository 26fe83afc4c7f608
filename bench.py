#!/usr/bin/env python3
"""Benchmark of the FlyVec hot path on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

A "step" is one training minibatch (sampler -> gather-sum -> winner -> xx -> max|ds| -> update)
at the headline configuration: K = 400 neurons, V = 20000, w = 11, B = 10000 windows, on a
synthetic 10 M-token Zipf(1.07) corpus with geometric chunk lengths, fp32, everything resident in
HBM before the timed region.  One JSON line is printed:

  value              training windows / s over the K timed steps
  roofline           the dominant kernel of the step against the 8 TB/s HBM peak: achieved = the bytes
                     that kernel has to move per launch / its mean duration, measured with HIP events
                     on the trainer's stream; traffic = HBM-side bytes per launch from the rocprofv3
                     counter runs summarised under profiles/ (read from that file, not from this run)
  kernels            the same for every kernel of the step; the window gathers, whose bytes are largely
                     served by the L2 caches, are held against measured HBM-side traffic and against the
                     vector-ALU issue rate instead of against their algorithmic bytes
  step_roofline_frac (byte model of the whole step, 4BwK + 12KN + 16Bw, / 8 TB/s) / measured time per step
  step_moved_frac    the same with the bytes the step's scheme has to move, 4BwK + 8KN + 16Bw: max|ds| comes from
                     the carried row maxima, so the matrix is read once and written once (null, and the figure
                     under step_moved_byte_model_comparison, where it exceeds 1 because caches serve the gathers)
  cpu_baseline       the CPU restatement of the same step (oracle/, C + OpenMP) timed on this host
  hash               the batched top-k hash (1,048,576 windows, k = 32, bit-packed), device-resident,
                     with the reference's numpy per-word path as its CPU baseline; targets_4096 and per_word_us:
                     the reference-shaped calls (4096 target ids in one call; one word per call)
  hash_host          the same batch through the host-buffer entry point (copies included)
  large_step         K = 1000, V = 50000, w = 15, B = 50000 on a 200 M-token corpus (400 MB matrix)
  epoch              one full epoch over a 100 M-token corpus with device shuffle and one checkpoint
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
# vector-ALU issue rate: 256 compute units x 4 SIMDs, one wave64 instruction per SIMD every 4 cycles
# (16 lanes per SIMD), at the 2.4 GHz peak engine clock
VALU_ISSUE_PEAK = 256 * 4 * 2.4e9 / 4
# L2 request throughput: 8 XCDs x 16 channels, one 128-byte request per channel and clock (the per-channel rate
# of the CDNA 3 L2; no figure is published for this part), at the same clock
L2_REQUEST_BYTES = 128
L2_PEAK = 8 * 16 * L2_REQUEST_BYTES * 2.4e9

TRAIN = dict(K=400, V=20000, w=11, B=10000, n_tokens=10_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.07, mean_chunk=25)
LARGE = dict(K=1000, V=50000, w=15, B=50000, n_tokens=200_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.0, mean_chunk=40)
EPOCH = dict(K=400, V=20000, w=11, B=10000, n_tokens=100_000_000, lr0=2e-4, n_epochs=15, prec=1e-30,
             zipf_s=1.07, mean_chunk=25)
HASH = dict(K=400, V=20000, w=11, k=32, n=1 << 20)

# rocprofv3 summaries of the command lines below them; their lines "@ <kernel> name=value ..." carry the
# per-launch counter means this script quotes (HBM-side KiB fetched / written, wave-level VALU instructions)
PROFILE = {"step": "profiles/train_step_and_hash_K400_V20000_B10000.txt",
           "large": "profiles/train_step_K1000_V50000_B50000.txt"}
FETCH_SCALE, WRITE_SCALE = 2.0, 1.0  # what the counters read for a plain copy kernel of known size


def profile_counters(which):
    """{kernel: {name: value}} from the '@' lines of a profiles/ summary ({} if the file is absent)."""
    out = {}
    try:
        with open(os.path.join(ROOT, PROFILE[which])) as f:
            for line in f:
                if line.startswith("@ "):
                    parts = line.split()
                    out[parts[1]] = {k: float(v) for k, v in (p.split("=") for p in parts[2:])}
    except OSError:
        pass
    return out


def traffic_bytes(counters, kernel):
    c = counters.get(kernel)
    if not c or "fetch_kib" not in c or "write_kib" not in c:
        return None
    return (c["fetch_kib"] * FETCH_SCALE + c["write_kib"] * WRITE_SCALE) * 1024


def kernel_bytes(K, N, w, B, single_dense_launch=False):
    """Bytes every kernel of a step has to move. The window gather reads w rows of K floats per window
    (largely from L2: the rows repeat); the dense passes read the matrix for max|ds| and read + write it
    for the update -- the single launch keeps it in registers or knows max|ds| beforehand and so moves it
    once each way. The sparse term is 16 bytes per window position in the byte model (token id, 1/f look-up,
    read and write of the element): as six launches half of it falls to the sparse launch and half to the slot
    update; with the single dense launch the sparse launch is held to all 16 (it reads the ids and 1/f, reads the
    elements and writes the sentinels) and the dense launch's share is the records it reads back."""
    return {
        "gather_winner": 4 * B * w * K,
        "group_xx": 8 * B,
        "sparse_owners": (16 if single_dense_launch else 8) * B * w,
        "absmax_ds": 4 * K * N,
        "update": 8 * K * N,
        "slot_update": 8 * B * w,
        "dense_update": 8 * K * N + 8 * B * w,
    }


def step_byte_model(K, N, w, B):
    """The byte model the step is held to: gathers counted in full, the matrix read for max|ds| and read +
    written for the update (12 K N), 16 bytes per window position. A scheme that skips one of those
    passes scores above its share of this model; that is said where it applies."""
    return 4 * B * w * K + 12 * K * N + 16 * B * w


def step_moved_model(K, N, w, B):
    """The bytes the step's own scheme has to move: as step_byte_model, but max|ds| is taken from the carried two
    largest weights of every row, so the matrix is read once and written once (8 K N)."""
    return 4 * B * w * K + 8 * K * N + 16 * B * w


def frac_fields(prefix, model, seconds):
    """{prefix_frac: model time at 8 TB/s / measured time}; a figure above 1 is no fraction of a roof (caches
    served bytes the model counts): it goes under a key that says so and the fraction reads null."""
    value = (model / HBM_PEAK) / seconds
    if value <= 1.0:
        return {prefix + "_frac": value}
    return {prefix + "_frac": None, prefix + "_byte_model_comparison": value}


def hash_bytes_per_window(K, w):
    return 4 * w * K + 4 * w + 8 * ((K + 63) // 64)


def hbm_entry(kernel, nbytes, ms, traffic, source):
    achieved = nbytes / (ms * 1e-3)
    return {"bound": "hbm", "kernel": kernel, "achieved": achieved / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
            "frac": achieved / HBM_PEAK, "traffic": traffic, "traffic_source": source if traffic else None,
            "algorithmic_bytes": nbytes}


def gather_entry(kernel, nbytes, ms, counters, source):
    """A window-gather kernel: its algorithmic bytes mostly hit in L2, so it is held against the HBM-side
    traffic the counters saw and against the rate at which the vector ALUs can issue."""
    traffic = traffic_bytes(counters, kernel)
    out = {"kernel": kernel, "algorithmic_bytes": nbytes, "algorithmic_rate_GBps": nbytes / (ms * 1e-3) / 1e9,
           "traffic": traffic, "traffic_source": source if traffic else None}
    if traffic:
        out["hbm"] = {"bound": "hbm", "achieved": traffic / (ms * 1e-3) / 1e9, "peak": HBM_PEAK / 1e9, "unit": "GB/s",
                      "frac": traffic / (ms * 1e-3) / HBM_PEAK, "basis": "measured HBM-side traffic / duration"}
    insts = counters.get(kernel, {}).get("valu_insts")
    if insts:
        out["valu_issue"] = {"bound": "valu_issue", "achieved": insts / (ms * 1e-3) / 1e9, "peak": VALU_ISSUE_PEAK / 1e9,
                             "unit": "G wave-instructions/s", "frac": insts / (ms * 1e-3) / VALU_ISSUE_PEAK,
                             "insts_per_launch": insts, "insts_source": source}
    reqs = counters.get(kernel, {}).get("tcc_req")
    if reqs:
        out["l2_requests"] = {"bound": "l2", "achieved": reqs * L2_REQUEST_BYTES / (ms * 1e-3) / 1e9, "peak": L2_PEAK / 1e9,
                              "unit": "GB/s", "frac": reqs * L2_REQUEST_BYTES / (ms * 1e-3) / L2_PEAK,
                              "requests_per_launch": reqs, "requests_source": source,
                              "basis": "TCC_REQ_sum x 128 B / duration against 8 XCDs x 16 channels x 128 B per clock "
                                       "at 2.4 GHz"}
    return out


def bench_train(steps, warmup, cpu_seconds, c=TRAIN, which="step", dense_launches=0, separate_grouping=False,
                graphs=False):
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
    known0, made0 = t.dense_path_counts
    # timed region: exactly `steps` steps, device idle before and after
    t0 = time.perf_counter()
    for s in range(steps):
        t.step((warmup + s) * c["B"], c["B"], eps)
    t.sync()
    wall = time.perf_counter() - t0
    known1, made1 = t.dense_path_counts
    # the same number of steps again, timed by two HIP events on the trainer's stream
    total_ms, _ = t.time_steps((warmup + steps) * c["B"], steps, eps, per_kernel=False)
    ev_ms_per_step = total_ms / steps
    # per-kernel durations: each kernel of the last step launched back to back between two HIP
    # events on that stream (bracketing every kernel inside a step would add 3 to 5 us of event
    # overhead to each); this destroys W, so it is the last thing this trainer does
    kern_ms = t.time_kernels(reps=50)
    launches = t.dense_launches
    grouping_separate = t.grouping_launch
    t.close()
    # the same steps as HIP graphs (a graph per step, then one graph for all) against stream launches, in a trainer
    # of its own: the three forms on one matrix in one state, one after the other
    graph = None
    g_steps = min(steps, (nwin // c["B"] - warmup) // 3)
    if graphs and g_steps >= 5:
        g = Trainer(c["V"], c["K"], c["w"], c["B"], initial_learning_rate=c["lr0"], prec=c["prec"])
        g.set_dense_launches(dense_launches)
        g.set_grouping_launch(separate_grouping)
        g.set_corpus(tokens, offsets)
        g.set_permutation(perm)
        g.set_weights(W0)
        for s in range(warmup):
            g.step(s * c["B"], c["B"], eps)
        g.sync()
        stream_ms = g.time_steps(warmup * c["B"], g_steps, eps, per_kernel=False)[0] / g_steps
        per_step_ms = g.time_steps_graph((warmup + g_steps) * c["B"], g_steps, eps, 1) / g_steps
        whole_ms = g.time_steps_graph((warmup + 2 * g_steps) * c["B"], g_steps, eps, g_steps) / g_steps
        g.close()
        graph = {"steps": g_steps, "stream_launches_ms_per_step": stream_ms,
                 "graph_per_step_ms_per_step": per_step_ms, "one_graph_ms_per_step": whole_ms,
                 "note": "a trainer of its own, the three forms one after the other on consecutive windows: the same "
                         "kernels with the same arguments, as stream launches and captured into HIP graphs that are "
                         "instantiated before the clock starts; HIP events on the trainer's stream"}

    N = 2 * c["V"]
    per_kernel = kernel_bytes(c["K"], N, c["w"], c["B"], single_dense_launch=launches == 1)
    if launches == 1:
        # max|ds|, the update and the slot update ran as one launch (timed under the first name; the others are empty)
        kern_ms["dense_update"] = sum(kern_ms.pop(k) for k in ("absmax_ds", "update", "slot_update"))
        for k in ("absmax_ds", "update", "slot_update"):
            per_kernel.pop(k)
    else:
        per_kernel.pop("dense_update")
    if not grouping_separate:
        # the sparse launch has grouped the windows by winner itself: no grouping launch ran
        kern_ms["sparse_owners"] += kern_ms.pop("group_xx")
        per_kernel["sparse_owners"] += per_kernel.pop("group_xx")
    counters = profile_counters(which)
    source = PROFILE[which]
    kernels = {}
    for k, ms in kern_ms.items():
        if k == "gather_winner":
            kernels[k] = gather_entry(k, per_kernel[k], ms, counters, source)
        else:
            kernels[k] = hbm_entry(k, per_kernel[k], ms, traffic_bytes(counters, k), source)
        kernels[k]["ms"] = ms
    dom = max(kern_ms, key=kern_ms.get)
    if dom == "gather_winner":
        g = kernels[dom]
        roofline = dict(g.get("hbm") or {"bound": "hbm", "achieved": None, "peak": HBM_PEAK / 1e9, "unit": "GB/s", "frac": None})
        roofline.update(kernel=dom, traffic=g["traffic"], traffic_source=g["traffic_source"],
                        algorithmic_bytes=g["algorithmic_bytes"])
    else:
        roofline = {k: v for k, v in kernels[dom].items() if k != "ms"}
    model = step_byte_model(c["K"], N, c["w"], c["B"])
    ms_per_step = wall / steps * 1e3
    out = {
        "value": steps * c["B"] / wall,
        "ms_per_step": ms_per_step,
        "event_ms_per_step": ev_ms_per_step,
        "roofline": roofline,
        "kernels": kernels,
        "dense_launches": launches,
        "grouping_launch": "own" if grouping_separate else "in sparse_owners",
        "step_roofline_frac": (model / HBM_PEAK) / (ms_per_step * 1e-3),
        "step_byte_model": model,
        "step_moved_model": step_moved_model(c["K"], N, c["w"], c["B"]),
        "n_windows": nwin,
    }
    out.update(frac_fields("step_moved", out["step_moved_model"], ms_per_step * 1e-3))
    if graph:
        out["hip_graph"] = graph
    if launches == 1:
        out["dense_launch_paths"] = {"knew_max_ds": known1 - known0, "made_the_pass": made1 - made0,
                                     "note": "timed steps whose single dense launch took max|ds| from the carried "
                                             "row maxima / read the matrix for it first"}
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


def bench_delta_step(steps, warmup, plain_ms_per_step, c=TRAIN, delta=0.4):
    """The same step with the anti-Hebbian term of the reference switched on (delta != 0 at
    flyvec/src/cuda_funcs.cu:870-935: the neuron that came second in a window is pushed away from it), which the
    reference's driver leaves at 0: the second neuron's window lists are grouped and summed beside the winner's."""
    from flyvec_amd import Trainer, synthetic
    tokens, offsets = synthetic.corpus(c["n_tokens"], c["V"], s=c["zipf_s"], mean_chunk=c["mean_chunk"])
    t = Trainer(c["V"], c["K"], c["w"], c["B"], initial_learning_rate=c["lr0"], prec=c["prec"])
    t.set_corpus(tokens, offsets)
    t.set_permutation(np.random.default_rng(6).permutation(t.num_windows).astype(np.uint64))
    t.set_weights(synthetic.synapses(c["K"], c["V"], seed=5))
    eps = t.epoch_eps(0, c["n_epochs"])
    for s in range(warmup):
        t.step(s * c["B"], c["B"], eps, delta=delta)
    t.sync()
    t0 = time.perf_counter()
    for s in range(steps):
        t.step((warmup + s) * c["B"], c["B"], eps, delta=delta)
    t.sync()
    ms = (time.perf_counter() - t0) / steps * 1e3
    kern_ms = {k: v for k, v in t.time_kernels(reps=20).items() if v > 1e-3}  # empty launches take 0.2 us
    t.close()
    return {"delta": delta, "value": c["B"] / (ms * 1e-3), "unit": "windows/s", "steps": steps, "warmup": warmup,
            "ms_per_step": ms, "us_over_the_step_without_the_term": (ms - plain_ms_per_step) * 1e3,
            "kernel_ms": kern_ms,
            "note": "same corpus, order, matrix and batch as the headline step; wall clock over the timed steps, device "
                    "idle before and after; kernel_ms from replays of the last step's launches between HIP events"}


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
    with tempfile.TemporaryDirectory() as d:
        t.save_weights(os.path.join(d, "flyvec_model_0.npy"))  # and of the checkpoint's page-locked buffer
    known0, made0 = t.dense_path_counts
    t0 = time.perf_counter()
    t.shuffle(2)
    t.sync()
    t_shuffle = time.perf_counter() - t0
    t1 = time.perf_counter()
    t.run_epoch(1, c["n_epochs"])      # returns when the device has finished
    t_steps = time.perf_counter() - t1
    t2 = time.perf_counter()
    with tempfile.TemporaryDirectory() as d:
        t.save_weights(os.path.join(d, "flyvec_model_1.npy"))
    t_ckpt = time.perf_counter() - t2
    total = time.perf_counter() - t0
    known1, made1 = t.dense_path_counts
    t.close()
    n_steps = (nwin + c["B"] - 1) // c["B"]
    model = step_byte_model(c["K"], 2 * c["V"], c["w"], c["B"])
    moved = frac_fields("step_moved", step_moved_model(c["K"], 2 * c["V"], c["w"], c["B"]) * (nwin / c["B"]), t_steps)
    return {**moved, "metric": "train windows/s over one full epoch", "value": nwin / total, "unit": "windows/s",
            "config": {"workload": f"full training epoch: {c['n_tokens']} Zipf({c['zipf_s']}) tokens, K={c['K']} "
                                   f"Nvoc={c['V']} w={c['w']} B={c['B']}, {nwin} windows, device shuffle before "
                                   f"and one .npy checkpoint after (second epoch of a run)"},
            "seconds_per_epoch": total, "n_windows": nwin, "n_steps": n_steps,
            "ms_per_step": t_steps / n_steps * 1e3,
            "breakdown_s": {"shuffle": t_shuffle, "minibatch_loop": t_steps, "checkpoint": t_ckpt,
                            "setup_once": t_setup, "synthetic_corpus_generation": t_gen},
            "step_roofline_frac": (model * (nwin / c["B"]) / HBM_PEAK) / t_steps,
            "dense_launch_paths": {"knew_max_ds": known1 - known0, "made_the_pass": made1 - made0}}


def bench_reference_shaped_calls(h, W, c):
    """The calls in the shape the reference's API has (flyvec/core.py:139-163, 187-211): the 4096 Zipf target ids
    of the CPU-runnable configuration (k = 50, int8 codes) in one fv_hash_targets call from host memory, and one
    word per Python call -- through FlyVec.get_sparse_embedding, which reads a whole-vocabulary table that one
    device launch fills on first use, and, for comparison, as one launch per word."""
    from flyvec_amd import FlyVec, synthetic
    ids = synthetic.zipf_ids(4096, c["V"], seed=2)
    h.hash_targets(ids, 50)
    best = float("inf")
    for _ in range(20):
        t0 = time.perf_counter()
        h.hash_targets(ids, 50)
        best = min(best, time.perf_counter() - t0)
    vocab = ["<UNK>"] + [f"t{i}" for i in range(1, c["V"])]
    words = [vocab[i] for i in ids]
    model = FlyVec(W, tokenizer=vocab, normalize_synapses=False)
    t0 = time.perf_counter()
    model.code_table(50)
    table_ms = (time.perf_counter() - t0) * 1e3
    for word in words[:64]:
        model.get_sparse_embedding(word)
    t0 = time.perf_counter()
    for word in words:
        model.get_sparse_embedding(word)
    per_word = (time.perf_counter() - t0) / len(words)
    t0 = time.perf_counter()
    for i in ids[:512]:
        model.hasher.hash_targets([int(i)], 50)
    per_launch = (time.perf_counter() - t0) / 512
    model.hasher.close()
    return {"targets_4096": {"value": len(ids) / best, "unit": "codes/s", "ms_per_call": best * 1e3,
                             "workload": "fv_hash_targets: 4096 Zipf(1.07) target ids in host memory -> int8 codes of "
                                         "length 400 in host memory, k = 50, one call (copies and launch included)"},
            "per_word_us": per_word * 1e6,
            "per_word": {"us_per_word": per_word * 1e6, "codes_per_s": 1.0 / per_word,
                         "workload": "FlyVec.get_sparse_embedding(word) in a Python loop over the same 4096 words "
                                     "(tokenizer look-up included), served from the whole-vocabulary table",
                         "table_fill_ms": table_ms,
                         "table": f"{c['V']} x {c['K']} int8 per hash length, one fv_hash_targets call on first use",
                         "one_launch_per_word_us": per_launch * 1e6}}


def bench_hash(reps, cpu_seconds, host_reps=5, host=True):
    from flyvec_amd import Hasher, synthetic, _lib
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
    counters = profile_counters("step")
    workload = (f"batched contextual hash: K={c['K']} V={c['V']} w={c['w']} k={c['k']} n={c['n']} windows, "
                f"{h.words} uint64 words out")
    out = {"metric": "hash codes/s", "value": c["n"] / (ms * 1e-3), "unit": "codes/s", "ms_per_batch": ms,
           "config": {"workload": workload + ", indices and codes resident in HBM"}, "dtype": "f32",
           "roofline": gather_entry("hash", bpw * c["n"], ms, counters, PROFILE["step"]),
           "byte_model_frac": (bpw * c["n"] / HBM_PEAK) / (ms * 1e-3),
           "byte_model_note": "time the algorithmic bytes would take at 8 TB/s / measured time; above 1 because the "
                              "64 MB matrix is served by the L2 and Infinity caches"}
    if host:
        out.update(bench_reference_shaped_calls(h, W, c))
    if not host:
        h.close()
        d_idx.free()
        d_bits.free()
        return out, None
    # the same batch from host buffers through fv_hash_windows: copies included
    host = {}
    bits = np.empty((c["n"], h.words), dtype=np.uint64)
    pin_idx = _lib.pinned_empty(idx.shape, np.int32)
    pin_idx[:] = idx
    pin_bits = _lib.pinned_empty(bits.shape, np.uint64)
    pin_bits[:] = 0
    for name, i, o in (("pageable", idx, bits), ("page_locked", pin_idx, pin_bits)):
        h.hash_windows(i, c["k"], out_bits=o)
        best = float("inf")
        for _ in range(host_reps):
            t0 = time.perf_counter()
            h.hash_windows(i, c["k"], out_bits=o)
            best = min(best, time.perf_counter() - t0)
        host[name] = {"value": c["n"] / best, "unit": "codes/s", "ms_per_batch": best * 1e3}
    moved = idx.nbytes + bits.nbytes
    out_host = {"metric": "hash codes/s from host buffers (PCIe-inclusive)", "config": {"workload": workload + ", numpy "
                "buffers in host memory through fv_hash_windows (chunks on two streams)"},
                "bytes_over_the_link": moved, "buffers": host,
                "link_GBps_page_locked": moved / (host["page_locked"]["ms_per_batch"] * 1e-3) / 1e9}
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
    return out, out_host


def train_line(c, tr, steps, warmup):
    line = {
        "metric": f"train windows/s at K={c['K']},Nvoc={c['V'] // 1000}k",
        "value": tr["value"], "unit": "windows/s", "n_gpus": 1, "steps": steps, "warmup": warmup,
        "ms_per_step": tr["ms_per_step"], "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f32", "data": "synthetic",
        "config": {"workload": f"single training minibatch step: K={c['K']} Nvoc={c['V']} w={c['w']} B={c['B']}, "
                               f"{c['n_tokens']} Zipf({c['zipf_s']}) tokens, geometric chunks (mean {c['mean_chunk']}), "
                               f"{tr['n_windows']} windows, lr 2e-4, fp32"},
    }
    for k in ("roofline", "step_roofline_frac", "step_byte_model", "step_moved_frac", "step_moved_byte_model_comparison",
              "step_moved_model", "event_ms_per_step", "kernels", "dense_launches",
              "grouping_launch", "dense_launch_paths", "hip_graph", "cpu_baseline"):
        if k in tr:
            line[k] = tr[k]
    return line


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--cpu-seconds", type=float, default=12.0, help="CPU baseline sample length (0 = skip)")
    ap.add_argument("--no-hash", action="store_true")
    ap.add_argument("--no-hash-host", action="store_true", help="skip the hash timings from host buffers and the calls "
                    "shaped like the reference's API (profiling runs: their small launches would mix into the "
                    "per-kernel means)")
    ap.add_argument("--no-graph", action="store_true", help="skip the steps enqueued as HIP graphs")
    ap.add_argument("--no-large", action="store_true", help="skip the K=1000, V=50000 step")
    ap.add_argument("--no-epoch", action="store_true", help="skip the full epoch over 100 M tokens")
    ap.add_argument("--separate-grouping", action="store_true",
                    help="group the windows by winner in a launch of its own (the default does it inside the sparse launch)")
    ap.add_argument("--dense-launches", type=int, choices=[0, 1, 2, 3], default=0,
                    help="the passes over W of a step as one launch (1; 3: its streaming form), separate launches (2), or as the "
                         "library chooses (0)")
    ap.add_argument("--workload", choices=["all", "step", "large-step", "epoch"], default="all",
                    help="all: the headline step with the hash batch, the large step and the epoch as sub-objects "
                         "(default); step / large-step / epoch: that workload alone as the line")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="also run a plain 1 GiB copy kernel (yardstick for rocprofv3 byte counters)")
    args = ap.parse_args()
    if args.gpus != 1:
        raise SystemExit("bench.py measures one GPU: this build has no multi-GPU path (--gpus must be 1)")

    from flyvec_amd import _lib
    info = _lib.device_info()
    if args.workload == "epoch":
        ep = bench_epoch(EPOCH)
        ep.update({"n_gpus": 1, "steps": ep["n_steps"], "warmup": ep["n_steps"], "higher_is_better": True,
                   "scaling": "weak", "vs_baseline": None, "dtype": "f32", "data": "synthetic",
                   "device": info["name"].strip()})
        print(json.dumps(ep))
        return
    if args.workload == "large-step":
        steps, warmup = min(args.steps, 50), min(args.warmup, 5)
        tr = bench_train(steps, warmup, args.cpu_seconds, LARGE, "large", args.dense_launches, args.separate_grouping)
        line = train_line(LARGE, tr, steps, warmup)
        line["device"] = info["name"].strip()
        print(json.dumps(line))
        return
    tr = bench_train(args.steps, args.warmup, args.cpu_seconds, TRAIN, "step", args.dense_launches,
                     args.separate_grouping, graphs=not args.no_graph)
    line = train_line(TRAIN, tr, args.steps, args.warmup)
    line["device"] = info["name"].strip()
    if not args.no_hash:
        line["hash"], line["hash_host"] = bench_hash(reps=10, cpu_seconds=min(args.cpu_seconds, 5.0),
                                                     host=not args.no_hash_host)
    if args.workload == "all":
        line["delta_step"] = bench_delta_step(args.steps, args.warmup, tr["ms_per_step"])
        if not args.no_large:
            steps, warmup = min(args.steps, 30), min(args.warmup, 5)
            lt = bench_train(steps, warmup, 0.0, LARGE, "large", args.dense_launches, args.separate_grouping)
            line["large_step"] = train_line(LARGE, lt, steps, warmup)
        if not args.no_epoch:
            line["epoch"] = bench_epoch(EPOCH)
    if args.copy_calibration:
        nbytes = 1 << 30
        ms = _lib.calibration_copy(nbytes, reps=5)
        line["copy_calibration"] = {"bytes_read": nbytes, "bytes_written": nbytes, "ms": ms,
                                    "GB/s": 2 * nbytes / (ms * 1e-3) / 1e9}
    print(json.dumps(line))


if __name__ == "__main__":
    main()
