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
PYCALL_PATH = os.path.join(HERE, "_fp8bs_pycall.so")
CSRC = os.path.join(HERE, "csrc")
SOURCES = sorted(os.path.join(CSRC, f) for f in os.listdir(CSRC) if f.endswith(".hip"))
OBJ_DIR = os.path.join(HERE, "csrc", "_obj")          # git-ignored build products

HIPCC_FLAGS = [
    "--offload-arch=gfx950", "-O3", "-std=c++20", "-fPIC",
    # keep the compiler from forming packed-fp32 VALU instructions
    "-Xclang", "-target-feature", "-Xclang", "-packed-fp32-ops",
    "-I" + os.path.join(ROOT, "include"), "-I" + CSRC,
]


def _run(cmd, verbose):
    if verbose:
        print(" ".join(cmd), flush=True)
    res = subprocess.run(cmd, stdout=subprocess.PIPE, stderr=subprocess.STDOUT, text=True)
    return res.returncode, res.stdout


def build(verbose: bool = False, jobs: int = 0) -> str:
    """Compile the library (always recompiles) and return its path.  The tiled kernel is instantiated per
    tile shape in a translation unit of its own (csrc/fp8bs_tile_*.hip): the files compile side by side."""
    from concurrent.futures import ThreadPoolExecutor
    hipcc = os.environ.get("HIPCC", "/opt/rocm/bin/hipcc")
    os.makedirs(OBJ_DIR, exist_ok=True)
    jobs = jobs or min(len(SOURCES), int(os.environ.get("MAX_JOBS", os.cpu_count() or 4)), 16)
    objs = [os.path.join(OBJ_DIR, os.path.basename(src)[:-4] + ".o") for src in SOURCES]
    cmds = [[hipcc] + HIPCC_FLAGS + ["-c", "-o", obj, src] for src, obj in zip(SOURCES, objs)]
    with ThreadPoolExecutor(max_workers=jobs) as pool:
        results = list(pool.map(lambda c: _run(c, verbose), cmds))
    for (rc, out), src in zip(results, SOURCES):
        if rc != 0:
            sys.stderr.write(out)
            raise RuntimeError("hipcc failed compiling %s (exit %d)" % (os.path.basename(src), rc))
    rc, out = _run([hipcc, "--offload-arch=gfx950", "-shared", "-fPIC", "-o", LIB_PATH] + objs, verbose)
    if rc != 0:
        sys.stderr.write(out)
        raise RuntimeError("hipcc failed linking libfp8bs.so (exit %d)" % rc)
    try:
        build_pycall(verbose)
    except (RuntimeError, OSError) as ex:
        # no Python.h or no host compiler: the package then binds the same functions through ctypes
        sys.stderr.write("warning: %s; continuing without the CPython binding\n" % ex)
        if os.path.exists(PYCALL_PATH):
            os.remove(PYCALL_PATH)                    # a stale binding must not shadow the library just built
    return LIB_PATH


def build_pycall(verbose: bool = False) -> str:
    """The CPython binding of the two GEMM entry points (csrc/fp8bs_pycall.c): host compiler, linked against
    libfp8bs.so next to it.  Replaces ctypes' argument marshalling on the hot call path only."""
    import sysconfig
    cc = os.environ.get("CC", "gcc")
    cmd = [cc, "-O2", "-shared", "-fPIC", "-I" + sysconfig.get_paths()["include"], "-I" + os.path.join(ROOT, "include"),
           "-o", PYCALL_PATH, os.path.join(CSRC, "fp8bs_pycall.c"), "-L" + HERE, "-lfp8bs", "-Wl,-rpath,$ORIGIN"]
    rc, out = _run(cmd, verbose)
    if rc != 0:
        sys.stderr.write(out)
        raise RuntimeError("%s failed building _fp8bs_pycall.so (exit %d)" % (cc, rc))
    return PYCALL_PATH


if __name__ == "__main__":
    print(build(verbose=True))
