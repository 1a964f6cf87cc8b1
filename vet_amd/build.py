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


TORCH_EXT_PATH = os.path.join(LIB_DIR, "vetrast_torch.so")


def build_torch_extension(verbose=True):
    """libtorch shim (vet_amd/torch_ext) as a Python extension module vet_amd/lib/vetrast_torch.so, linked against
    libvetrast.so. Plain host C++: g++ against the torch headers, no device code."""
    import sysconfig

    import torch
    from torch.utils import cpp_extension

    os.makedirs(LIB_DIR, exist_ok=True)
    inc = cpp_extension.include_paths()
    torch_lib = os.path.join(os.path.dirname(torch.__file__), "lib")
    cmd = [os.environ.get("CXX", "g++"), "-O2", "-std=c++17", "-fPIC", "-shared", "-Wall", "-Wno-unused-function",
           "-D__HIP_PLATFORM_AMD__=1", "-DUSE_ROCM=1", "-DTORCH_EXTENSION_NAME=vetrast_torch",
           "-DTORCH_API_INCLUDE_EXTENSION_H", f"-D_GLIBCXX_USE_CXX11_ABI={int(torch._C._GLIBCXX_USE_CXX11_ABI)}"]
    for i in inc + ["/opt/rocm/include", sysconfig.get_paths()["include"]]:
        cmd += ["-isystem", i]
    cmd += [os.path.join(HERE, "torch_ext", "point_render.cpp"), "-o", TORCH_EXT_PATH,
            f"-L{torch_lib}", f"-L{LIB_DIR}", "-lvetrast", "-lc10", "-lc10_hip", "-ltorch_cpu", "-ltorch_hip", "-ltorch",
            "-ltorch_python", "-Wl,-rpath,$ORIGIN", f"-Wl,-rpath,{torch_lib}"]
    if verbose:
        print(" ".join(cmd), flush=True)
    subprocess.run(cmd, check=True)
    return TORCH_EXT_PATH


if __name__ == "__main__":
    build_library()
    print("built", LIB_PATH)
    if "--lib-only" not in sys.argv:
        build_torch_extension()
        print("built", TORCH_EXT_PATH)
    sys.exit(0)
