"""Builds the HIP library (gfx950) in-tree: vet_amd/lib/libvetrast.so.

Run as `python -m vet_amd.build`. hipcc cross-compiles, so no GPU is needed.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
CSRC = os.path.join(HERE, "csrc")
LIB_DIR = os.path.join(HERE, "lib")
LIB_PATH = os.path.join(LIB_DIR, "libvetrast.so")

# -ffp-contract=off: the projection must round every operation on its own so that pixel assignment is reproducible.
# -munsafe-fp-atomics: float atomicAdd becomes the hardware global_atomic_add_f32 instead of a compare-and-swap loop.
HIPCC_FLAGS = [
    "--offload-arch=gfx950",
    "-O3",
    "-std=c++17",
    "-fPIC",
    "-shared",
    "-ffp-contract=off",
    "-munsafe-fp-atomics",
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-Wall",
    "-Wno-unused-function",
]


def build_library(verbose=True):
    os.makedirs(LIB_DIR, exist_ok=True)
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + [os.path.join(CSRC, "vetrast.hip"), "-o", LIB_PATH]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return LIB_PATH


if __name__ == "__main__":
    build_library()
    print("built", LIB_PATH)
    sys.exit(0)
