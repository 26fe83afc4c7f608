"""CPU checker for the FlyVec hot path.  TEST INFRASTRUCTURE ONLY.

Only tests, the smoke check and the bench's CPU-baseline leg may import this
package; the shipped library never does.  Two parts:

* ``hash_oracle`` -- numpy restatement of ``flyvec/core.py:23-36, 153-158``
  (normalisation, top-k threshold code) and its windowed generalisation.
* ``train_oracle`` -- ctypes view of ``flyvec_oracle.c`` (the training step and
  its host set-up, restated from ``flyvec/src/*.cu``), plus the reference's own
  ``prune_input.cpp`` when ``oracle/_ref`` was built.
"""
from . import hash_oracle, train_oracle  # noqa: F401
