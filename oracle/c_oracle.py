"""TEST INFRASTRUCTURE ONLY - ctypes access to oracle/libfp8bs_oracle.so (built by oracle/Makefile)."""
import ctypes
import os
import subprocess

import numpy as np
import torch

HERE = os.path.dirname(os.path.abspath(__file__))
LIB = os.path.join(HERE, "libfp8bs_oracle.so")


PROBE_LIB = os.path.join(HERE, "libmfma_probe.so")


def build() -> str:
    """Both checker libraries: the C restatement (host compiler) and the MFMA probe (hipcc, gfx950)."""
    subprocess.run(["make", "-s", "-B", "-C", HERE, "all"], check=True, stdout=subprocess.DEVNULL if os.environ.get("ORACLE_QUIET") else None)
    return LIB


_probe = None


def load_probe() -> ctypes.CDLL:
    """oracle/libmfma_probe.so (built ahead of time by build(); GPU runs load what is there)."""
    global _probe
    if _probe is None:
        if not os.path.exists(PROBE_LIB):
            raise RuntimeError("oracle/libmfma_probe.so is not built: run `make -C oracle` (needs hipcc)")
        lib = ctypes.CDLL(PROBE_LIB)
        lib.mfma_probe_chain_16x16x32.restype = ctypes.c_int
        lib.mfma_probe_chain_16x16x32.argtypes = [ctypes.c_void_p, ctypes.c_void_p, ctypes.c_int, ctypes.c_void_p, ctypes.c_void_p]
        _probe = lib
    return _probe


_lib = None


def load() -> ctypes.CDLL:
    global _lib
    if _lib is None:
        if not os.path.exists(LIB):
            subprocess.run(["make", "-s", "-C", HERE, "libfp8bs_oracle.so"], check=True)
        lib = ctypes.CDLL(LIB)
        lib.fp8bs_ref_e4m3fn_to_float.restype = ctypes.c_float
        lib.fp8bs_ref_e4m3fn_to_float.argtypes = [ctypes.c_uint8]
        lib.fp8bs_ref_float_to_bf16.restype = ctypes.c_uint16
        lib.fp8bs_ref_float_to_bf16.argtypes = [ctypes.c_float]
        vp, i32 = ctypes.c_void_p, ctypes.c_int
        lib.fp8bs_ref_gemm.restype = i32
        lib.fp8bs_ref_gemm.argtypes = [vp, vp, vp, vp, vp, i32, i32, i32]
        lib.fp8bs_ref_gemm_grouped.restype = i32
        lib.fp8bs_ref_gemm_grouped.argtypes = [vp, vp, vp, vp, vp, vp, i32, i32, i32, i32]
        _lib = lib
    return _lib


def _storage(t: torch.Tensor) -> np.ndarray:
    """Contiguous numpy copy of a K-major tensor's storage order (the transpose)."""
    tt = t.cpu()
    tt = tt.transpose(-1, -2).contiguous()
    if tt.dtype == torch.float8_e4m3fn:
        tt = tt.view(torch.uint8)
    return tt.numpy()


def ref_gemm(data) -> torch.Tensor:
    """C restatement on a (a, b, a_scale, b_scale, c) tuple; returns bf16 [M, N]."""
    a, b, a_scale, b_scale = data[:4]
    m, k = a.shape
    n = b.shape[0]
    sa, sb, ssa, ssb = _storage(a), _storage(b), _storage(a_scale), _storage(b_scale)
    out = np.empty((m, n), dtype=np.uint16)
    rc = load().fp8bs_ref_gemm(sa.ctypes.data, sb.ctypes.data, ssa.ctypes.data, ssb.ctypes.data,
                               out.ctypes.data, m, n, k)
    assert rc == 0
    return torch.from_numpy(out.view(np.int16)).view(torch.bfloat16)


def ref_gemm_grouped(data) -> torch.Tensor:
    a, b, a_scale, b_scale, row_offsets = data[:5]
    rows, k = a.shape
    e, n = b.shape[0], b.shape[1]
    sa, sb, ssa, ssb = _storage(a), _storage(b), _storage(a_scale), _storage(b_scale)
    ro = row_offsets.cpu().numpy().astype(np.int32)
    out = np.zeros((rows, n), dtype=np.uint16)
    rc = load().fp8bs_ref_gemm_grouped(sa.ctypes.data, sb.ctypes.data, ssa.ctypes.data, ssb.ctypes.data,
                                       out.ctypes.data, ro.ctypes.data, e, rows, n, k)
    assert rc == 0
    return torch.from_numpy(out.view(np.int16)).view(torch.bfloat16)
