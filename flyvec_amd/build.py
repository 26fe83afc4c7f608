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
SOURCES = ["fv_runtime.hip", "fv_corpus.hip", "fv_train.hip", "fv_hash.hip", "fv_legacy.hip"]
# the five shared objects the reference's driver opens (flyvec/train_flyvec.py:62-66)
LEGACY_NAMES = ["model_descriptor.so", "model_arrays.so", "cuda_helpers.so", "cuda_funcs.so", "prune_input.so"]

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


def install_legacy_names(directory):
    """Links the reference's five library names in `directory` to libflyvec_hip.so, which exports their
    symbols as well (include/flyvec_legacy.h): the reference's driver then runs on this library."""
    directory = Path(directory)
    directory.mkdir(parents=True, exist_ok=True)
    for name in LEGACY_NAMES:
        link = directory / name
        if link.is_symlink() or link.exists():
            link.unlink()
        link.symlink_to(LIB_PATH)
    return [directory / n for n in LEGACY_NAMES]


def main():
    import argparse
    ap = argparse.ArgumentParser(description=__doc__)
    ap.add_argument("--legacy-names", metavar="DIR", help="also link the reference's five library names in DIR")
    args = ap.parse_args()
    path = build(verbose=True)
    print(f"built {path}")
    if args.legacy_names:
        for link in install_legacy_names(args.legacy_names):
            print(f"linked {link}")


if __name__ == "__main__":
    main()
