"""flyvec_amd: the FlyVec training step and top-k hashing on one AMD MI355X.

``Trainer`` / ``Hasher`` are handles over libflyvec_hip.so (see include/flyvec_hip.h);
``FlyVec`` mirrors the reference's inference class; ``flyvec_amd.train_flyvec:main`` is the
``flyvec_train`` command. Importing the package does not load the native library; the first
handle does, and raises if it has not been built.
"""
__version__ = "0.1.0"

from .core import FlyVec  # noqa: F401
from .engine import Hasher, Trainer, count_windows, inverse_frequency, window_starts  # noqa: F401
