"""Builds libfp8bs.so (hipcc, gfx950 only) next to this file.

Replaces the import-time JIT of the reference (torch.utils.cpp_extension.load_inline for gfx942,
1-amd-fp8-mm/amd-fp8-mm-submission.py:582-592) with an explicit ahead-of-time build: no pybind, no
torch headers, one shared library with a C ABI.
"""
import os
import subprocess
import sys

HERE = os.path.dirname(os.path.abspath(__file__))
ROOT = os.path.dirname(HERE)
LIB_PATH = os.path.join(HERE, "libfp8bs.so")
SOURCES = [os.path.join(HERE, "csrc", f) for f in ("fp8bs_kernels.hip", "fp8bs_api.hip", "fp8bs_quant.hip", "fp8bs_route.hip")]

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-shared", "-fPIC",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + os.path.join(HERE, "csrc"),
]


def build(verbose: bool = False) -> str:
    """Compile the library (always recompiles) and return its path."""
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    cmd = [hipcc] + HIPCC_FLAGS + ["-o", LIB_PATH] + SOURCES
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    if res.returncode != 0:
        sys.stderr.write(res.stdout)
        raise RuntimeError("hipcc failed building libfp8bs.so (exit %d)" % res.returncode)
    return LIB_PATH


if __name__ == "__main__":
    print(build(verbose=True))
