"""Writes tests/golden/prune_windows.npz with the output of the reference's own prune_input_data.

Runs in the build container only: it calls oracle/_ref/libprune_input_ref.so, i.e.
flyvec/src/prune_input.cpp compiled from the mounted reference tree (prune_input_data :14-60).
The fixture is data: window matrices in, pruned matrices out."""
import os
import sys

import numpy as np

sys.path.insert(0, os.path.join(os.path.dirname(__file__), "..", ".."))
from oracle import train_oracle as to  # noqa: E402


def main():
    assert to.ref_lib() is not None, "build oracle/_ref first (make -C oracle)"
    rng = np.random.default_rng(77)
    out = {}
    cases = [rng.integers(-1, hi, size=(rows, cols)).astype(np.int32)
             for rows, cols, hi in [(40, 11, 6), (40, 11, 3), (25, 15, 9), (30, 4, 3), (20, 2, 2), (20, 1, 4), (12, 64, 20)]]
    cases.append(np.array([[7, 7, 7, 7, 7], [1, 2, 1, 2, 1], [-1, 3, -1, 3, -1], [4, 5, 6, 4, 5]], dtype=np.int32))
    for k, data in enumerate(cases):
        out[f"in_{k}"] = data
        out[f"out_{k}"] = to.ref_prune_windows(data)
    out["n_cases"] = np.int64(len(cases))
    path = os.path.join(os.path.dirname(__file__), "prune_windows.npz")
    np.savez_compressed(path, **out)
    print("wrote", path, [tuple(c.shape) for c in cases])


if __name__ == "__main__":
    main()
