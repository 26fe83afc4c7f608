"""Builds libflyvec_hip.so for gfx950 with hipcc (cross-compiles without a GPU).

The reference's counterpart is ``flyvec_compile`` -> ``sh short_make``
(flyvec/train_flyvec.py:25-27, flyvec/src/short_make): five nvcc invocations producing
five shared objects.  Here one hipcc invocation produces one library, in-tree.
"""
import shutil
import subprocess
import sys
from pathlib import Path

PKG = Path(__file__).resolve().parent
CSRC = PKG / "csrc"
INCLUDE = PKG.parent / "include"
LIB_DIR = PKG / "lib"
LIB_PATH = LIB_DIR / "libflyvec_hip.so"
SOURCES = ["fv_runtime.hip", "fv_corpus.hip", "fv_train.hip", "fv_hash.hip"]

HIPCC_FLAGS = [
    "-O3", "-std=c++17", "--offload-arch=gfx950", "-fPIC", "-shared",
    # bit-exact parity with the CPU checker needs separate multiplies and adds
    "-ffp-contract=off",
    # packed fp32 instructions are kept out of the generated code
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall", "-Wno-unused-function",
]


def hipcc_path():
    for cand in (shutil.which("hipcc"), "/opt/rocm/bin/hipcc"):
        if cand and Path(cand).exists():
            return cand
    raise RuntimeError("hipcc not found (looked on PATH and in /opt/rocm/bin)")


def build(verbose=False, extra_flags=()):
    """Compile every HIP source into flyvec_amd/lib/libflyvec_hip.so. Returns its path."""
    LIB_DIR.mkdir(exist_ok=True)
    cmd = [hipcc_path(), *HIPCC_FLAGS, *extra_flags, f"-I{INCLUDE}", f"-I{CSRC}",
           *[str(CSRC / s) for s in SOURCES], "-o", str(LIB_PATH)]
    if verbose:
        print(" ".join(cmd), flush=True)
    out = subprocess.run(cmd, capture_output=True, text=True)
    if out.returncode != 0:
        raise RuntimeError("hipcc failed:\n" + out.stdout + out.stderr)
    if verbose and out.stderr.strip():
        print(out.stderr, file=sys.stderr)
    return LIB_PATH


def main():
    path = build(verbose=True)
    print(f"built {path}")


if __name__ == "__main__":
    main()
