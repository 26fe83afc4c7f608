import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs an MI355X (run with -m gpu on the GPU box)")


def _gpu_available():
    try:
        from flyvec_amd import _lib
        return _lib.device_count() > 0
    except Exception:
        return False


@pytest.fixture(scope="session")
def gpu():
    """The native library on a machine with a GPU; GPU tests fail (not skip) if it is missing."""
    from flyvec_amd import _lib
    _lib.load()
    assert _lib.device_count() > 0, "no HIP device visible"
    return _lib


@pytest.fixture(autouse=True)
def _no_trainer_left_over():
    """A trainer that an earlier test left to the garbage collector (inside an exception's traceback, say)
    still counts as alive in the library, and a second live trainer switches the single dense launch off."""
    import gc
    gc.collect()
    yield


@pytest.fixture(scope="session")
def oracle_lib():
    from oracle import train_oracle
    train_oracle.lib()
    return train_oracle


def small_corpus(n_tokens=60000, vocab=500, seed=0, mean_chunk=25, n_masked=40):
    from flyvec_amd import synthetic
    tokens, offsets = synthetic.corpus(n_tokens, vocab, mean_chunk=mean_chunk, seed_tokens=seed + 3,
                                       seed_chunks=seed + 4)
    if n_masked:
        rng = np.random.default_rng(seed + 99)
        tokens[rng.integers(0, n_tokens - 1, n_masked)] = -1
        tokens[-1] = vocab - 1
    return tokens, offsets
