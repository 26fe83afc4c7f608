"""Writes tests/golden/window_table.npz with the reference's own window table.

Runs in the build container only: it calls oracle/_ref/libprune_input_ref.so, i.e.
flyvec/src/prune_input.cpp compiled from the mounted reference tree (getnum_samples :64-84,
compute_offset_phrases :88-122).  The fixture is data (offsets in, count and starts out)."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
from oracle import train_oracle as to  # noqa: E402


def main():
    assert to.ref_lib() is not None, "build oracle/_ref first (make -C oracle)"
    out = {}
    cases = []
    rng = np.random.default_rng(2024)
    for w in (11, 15, 3):
        lengths = rng.geometric(1 / 25, size=400)
        lengths[rng.integers(0, 400, 6)] = rng.integers(205, 230, 6)
        lengths[rng.integers(0, 400, 6)] = 0
        cases.append((np.concatenate([[0], np.cumsum(lengths)]).astype(np.uint64), w))
    cases.append((np.array([5, 30, 30, 60, 300, 311], dtype=np.uint64), 11))  # offsets[0] != 0
    cases.append((np.array([0], dtype=np.uint64), 11))                        # no chunk at all
    for k, (off, w) in enumerate(cases):
        out[f"offsets_{k}"] = off
        out[f"w_{k}"] = np.int64(w)
        out[f"count_{k}"] = np.int64(to.ref_count_windows(off, w))
        out[f"starts_{k}"] = to.ref_window_starts(off, w)
    out["n_cases"] = np.int64(len(cases))
    path = os.path.join(os.path.dirname(__file__), "window_table.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, {k: int(out[f"count_{k}"]) for k in range(len(cases))})


if __name__ == "__main__":
    main()
