"""GPU block quantisers: row-major fp32/bf16 matrices -> the operands ``custom_kernel`` takes.

The reference has no quantiser (its operands arrive quantised, 1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:66-77);
these wrap ``fp8bs_quantize_a`` / ``fp8bs_quantize_b`` / ``fp8bs_gather_a`` of libfp8bs.so and return tensors with exactly
the shapes, dtypes and K-major strides of that contract.  The rule is the one of ``inputs.quantize_a`` /
``inputs.quantize_b`` (the host-side quantisers), bit for bit.  No fallback: without the library the
import of ``_lib`` raises.
"""
from typing import Optional, Tuple

import torch

from . import _lib

_DTYPES = {torch.float32: 0, torch.bfloat16: 1}


def _check_input(x: torch.Tensor, name: str) -> None:
    if x.dtype not in _DTYPES:
        raise TypeError("%s must be float32 or bfloat16, got %s" % (name, x.dtype))
    if x.dim() != 2 or not x.is_cuda:
        raise ValueError("%s must be a 2-D tensor on the GPU" % name)
    if x.shape[1] % 128 != 0:
        raise ValueError("%s: K = %d is not a multiple of 128" % (name, x.shape[1]))
    if x.shape[1] > 0 and x.stride(1) != 1:
        raise ValueError("%s must be row-major (stride 1 along K), got strides %s" % (name, tuple(x.stride())))


def quantize_a(x: torch.Tensor, row_map: Optional[torch.Tensor] = None, fused: Optional[bool] = None) -> Tuple[torch.Tensor, torch.Tensor]:
    """x [T, K] -> (a e4m3fn [M, K] stride (1, M), a_scale fp32 [M, K/128] stride (1, M)).

    Without ``row_map`` M = T.  With ``row_map`` (int32 [M] on the GPU) output row i is input row
    ``row_map[i]``: the expert-contiguous gather of routed tokens.  Two routes, the same bytes: with at most as many
    output rows as tokens the gather is fused into the quantiser (one kernel); with more (every token routed to
    several experts, so rows repeat) every token is quantised once and the bytes are gathered by ``gather_a`` (two
    kernels: 4096 -> 32768 rows x 7168 take 91-97 us that way against 154 us fused, which quantises each token once
    per copy), provided the gather's fast path applies (T and M multiples of 4, T <= 40960).  ``fused`` = True / False
    forces the one-kernel / two-kernel route.
    """
    _check_input(x, "x")
    t, k = x.shape
    if row_map is not None:
        if row_map.dtype != torch.int32 or row_map.dim() != 1 or row_map.device != x.device or not row_map.is_contiguous():
            raise ValueError("row_map must be a contiguous int32 vector on x's device")
        m = row_map.numel()
        if fused is None:
            fused = not (m > t and t % 4 == 0 and m % 4 == 0 and 0 < t <= 40960)
        if not fused:
            return gather_a(*quantize_a(x), row_map)
    else:
        m = t
    a_store = torch.empty(k, m, dtype=torch.float8_e4m3fn, device=x.device)
    s_store = torch.empty(k // 128, m, dtype=torch.float32, device=x.device)
    with torch.cuda.device(x.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(_lib.load().fp8bs_quantize_a(
            x.data_ptr(), _DTYPES[x.dtype], x.stride(0) if t > 1 else max(k, 1),
            row_map.data_ptr() if row_map is not None else None, t,
            a_store.data_ptr(), s_store.data_ptr(), m, k, stream))
    return a_store.t(), s_store.t()


def quantize_b(w: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """w [N, K] -> (b e4m3fn [N, K] stride (1, N), b_scale fp32 [ceil(N/128), K/128] stride (1, NB))."""
    _check_input(w, "w")
    n, k = w.shape
    nb = (n + 127) // 128
    b_store = torch.empty(k, n, dtype=torch.float8_e4m3fn, device=w.device)
    s_store = torch.empty(k // 128, nb, dtype=torch.float32, device=w.device)
    with torch.cuda.device(w.device):
        stream = torch.cuda.current_stream().cuda_stream
        _lib.check(_lib.load().fp8bs_quantize_b(
            w.data_ptr(), _DTYPES[w.dtype], w.stride(0) if n > 1 else max(k, 1),
            b_store.data_ptr(), s_store.data_ptr(), n, k, stream))
    return b_store.t(), s_store.t()


def gather_a(a: torch.Tensor, a_scale: torch.Tensor, row_map: torch.Tensor) -> Tuple[torch.Tensor, torch.Tensor]:
    """Rows ``row_map`` of quantised activations: (a [T, K], a_scale [T, K/128]) K-major -> the same for M rows.

    ``gather_a(*quantize_a(x), row_map)`` returns exactly what ``quantize_a(x, row_map)`` returns, but
    quantises every token once instead of once per routed copy (the reference copies rows into expert
    order, 2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:174-191).  Entries of ``row_map`` outside [0, T) give
    zero rows with scale 1e-12.
    """
    if a.dtype != torch.float8_e4m3fn or a_scale.dtype != torch.float32 or a.dim() != 2 or a_scale.dim() != 2 or not a.is_cuda:
        raise TypeError("a must be a float8_e4m3fn and a_scale a float32 2-D tensor on the GPU")
    t, k = a.shape
    if k % 128 != 0 or tuple(a_scale.shape) != (t, k // 128):
        raise ValueError("a [T, K] needs K %% 128 == 0 and a_scale [T, K/128]; got %s and %s" % (tuple(a.shape), tuple(a_scale.shape)))
    if not a.t().is_contiguous() or not a_scale.t().is_contiguous():
        raise ValueError("a and a_scale must be K-major (stride 1 along rows)")
    if row_map.dtype != torch.int32 or row_map.dim() != 1 or row_map.device != a.device or not row_map.is_contiguous():
        raise ValueError("row_map must be a contiguous int32 vector on a's device")
    m = row_map.numel()
    a_store = torch.empty(k, m, dtype=torch.float8_e4m3fn, device=a.device)
    s_store = torch.empty(k // 128, m, dtype=torch.float32, device=a.device)
    with torch.cuda.device(a.device):
        _lib.check(_lib.load().fp8bs_gather_a(a.data_ptr(), a_scale.data_ptr(), t, row_map.data_ptr(),
                                              a_store.data_ptr(), s_store.data_ptr(), m, k,
                                              torch.cuda.current_stream().cuda_stream))
    return a_store.t(), s_store.t()
