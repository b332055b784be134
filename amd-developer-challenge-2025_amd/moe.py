"""MoE routing on the GPU: top-k selection, row_offsets and the expert-contiguous row order.

Wraps ``fp8bs_moe_topk`` / ``fp8bs_moe_route`` of libfp8bs.so.  Roles in the reference
(2-amd-moe/amd-moe-submission.py): ``top4_nre32`` / ``topk`` (:32-105), ``calculate_index`` (:107-156)
and the host read of the counts (:230-234); here nothing synchronises with the host and the row order is
deterministic (by expert, then token id).  The outputs plug into ``quant.quantize_a(x, row_map)`` and
``grouped_kernel``.  No fallback: without the library the import of ``_lib`` raises.
"""
from typing import Optional, Tuple

import torch

from . import _lib
from .submission import _check_operands, _is_kmajor, _stream_ptr


_route_ws = {}     # (device index, stream) -> uint8 tensor: the routing kernels' scratch, grown on demand, reused across
                   # calls on that stream (calls that overlap on two streams of one GPU must not share the count tables)


def topk(scores: torch.Tensor, k: int, out: Optional[torch.Tensor] = None) -> torch.Tensor:
    """scores fp32 [T, E] row-major on the GPU -> int32 [T, k], best first, lowest index first among equals.
    ``out`` (contiguous int32 [T, k] on the same GPU) is filled and returned if given: no allocation."""
    if scores.dtype != torch.float32 or scores.dim() != 2 or not scores.is_cuda or not scores.is_contiguous():
        raise ValueError("scores must be a contiguous float32 [tokens, experts] tensor on the GPU")
    t, e = scores.shape
    if out is None:
        out = torch.empty(t, k, dtype=torch.int32, device=scores.device)
    elif out.dtype != torch.int32 or tuple(out.shape) != (t, k) or out.device != scores.device or not out.is_contiguous():
        raise ValueError("out must be a contiguous int32 [tokens, k] tensor on the scores' device")
    with torch.cuda.device(scores.device):
        _lib.check(_lib.load().fp8bs_moe_topk(scores.data_ptr(), t, e, k, out.data_ptr(), _stream_ptr(scores.device)))
    return out


def route(top_idx: torch.Tensor, experts: int, out: Optional[Tuple[torch.Tensor, torch.Tensor, torch.Tensor]] = None
          ) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """top_idx int32 [T, k] -> (row_offsets int32 [E+1], row_map int32 [T*k], slot_of int32 [T, k]).

    Expert e owns rows [row_offsets[e], row_offsets[e+1]); ``row_map[row]`` is the token of that row
    (rows of an expert ordered by token id); ``slot_of[t, j]`` is the row of token t's j-th choice.
    Rows beyond ``row_offsets[E]`` (only if some entries of ``top_idx`` are outside [0, E)) are -1.
    ``out`` = the three tensors of a previous call (or any of those shapes, contiguous int32 on the same GPU)
    are filled and returned: a layer that routes every step then allocates nothing per call.
    """
    if top_idx.dtype != torch.int32 or top_idx.dim() != 2 or not top_idx.is_cuda or not top_idx.is_contiguous():
        raise ValueError("top_idx must be a contiguous int32 [tokens, topk] tensor on the GPU")
    t, k = top_idx.shape
    dev = top_idx.device
    if out is None:
        row_offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
        row_map = torch.empty(t * k, dtype=torch.int32, device=dev)
        slot_of = torch.empty(t, k, dtype=torch.int32, device=dev)
    else:
        row_offsets, row_map, slot_of = out
        for name, x, shape in (("row_offsets", row_offsets, (experts + 1,)), ("row_map", row_map, (t * k,)), ("slot_of", slot_of, (t, k))):
            if x.dtype != torch.int32 or tuple(x.shape) != shape or x.device != dev or not x.is_contiguous():
                raise ValueError("out: %s must be a contiguous int32 tensor of shape %s on top_idx's device" % (name, shape))
    lib = _lib.load()
    need = lib.fp8bs_moe_route_workspace_bytes(t, experts)
    with torch.cuda.device(dev):
        stream = _stream_ptr(dev)
        key = (dev.index, stream)
        ws = _route_ws.get(key)
        if ws is None or ws.numel() < need:
            # A buffer that is outgrown stays alive until this stream's earlier kernels are done with it: the caching
            # allocator hands a freed block only to later work of the stream it was allocated on.
            if ws is None and len(_route_ws) >= 16:      # streams come and go: keep the table bounded (oldest entry out)
                _route_ws.pop(next(iter(_route_ws)))
            ws = torch.empty(max(need, 4096), dtype=torch.uint8, device=dev)
            _route_ws[key] = ws
        _lib.check(lib.fp8bs_moe_route(top_idx.data_ptr(), t, experts, k, row_offsets.data_ptr(), row_map.data_ptr(),
                                       slot_of.data_ptr(), ws.data_ptr(), ws.numel(), stream))
    return row_offsets, row_map, slot_of


def gate_up_silu(data):
    """Gate/up projection with silu(gate) * up fused into the GEMM: ``data = (a, b, a_scale, b_scale, row_offsets, h)``.

    ``b`` holds gate and up weights interleaved by row (row 2i = gate_i, row 2i+1 = up_i), [E, n, k] with
    every expert K-major (or [n, k] K-major with ``row_offsets=None`` for one dense weight); ``h`` is
    bf16 [rows, n/2].  Role of re_silu_mul_kernel (2-amd-moe/amd-moe-submission.py:366-407) fused as in
    2-amd-moe/5-amd-fp8-moe-hip-fuse.py:366-408.  Fills and returns ``h``.
    """
    a, b, a_scale, b_scale, row_offsets, h = data
    if a.dim() != 2:
        raise ValueError("a must be a [rows, k] tensor")
    rows, k = a.shape
    grouped = row_offsets is not None
    if b.dim() != (3 if grouped else 2):
        raise ValueError("b must be [E, n, k] with row_offsets and [n, k] without")
    num_experts = b.shape[0] if grouped else 0
    n = b.shape[1] if grouped else b.shape[0]
    if n % 2:
        raise ValueError("n must be even: gate and up rows come in pairs")
    nb, kb = (n + 127) // 128, k // 128
    if grouped:
        if tuple(b.shape) != (num_experts, n, k) or tuple(b_scale.shape) != (num_experts, nb, kb):
            raise ValueError("b / b_scale shapes do not match [E, n, k] / [E, ceil(n/128), k/128]")
        if not b.transpose(1, 2).is_contiguous() or not b_scale.transpose(1, 2).is_contiguous():
            raise ValueError("every expert of b and b_scale must be K-major")
        if row_offsets.dtype != torch.int32 or tuple(row_offsets.shape) != (num_experts + 1,) or row_offsets.device != a.device:
            raise ValueError("row_offsets must be an int32 tensor with num_experts+1 entries on the operands' GPU")
    else:
        if tuple(b.shape) != (n, k) or tuple(b_scale.shape) != (nb, kb):
            raise ValueError("b / b_scale shapes do not match [n, k] / [ceil(n/128), k/128]")
        if not _is_kmajor(b) or not _is_kmajor(b_scale):
            raise ValueError("b and b_scale must be K-major")
    # dtypes, devices, shapes and K-major strides of a, a_scale and h ([rows, n/2]) as for the plain GEMM's c
    _check_operands(a, b, a_scale, b_scale, h, rows, n // 2, k)
    with torch.cuda.device(a.device):
        _lib.check(_lib.load().fp8bs_gemm_silu_mul(
            a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), h.data_ptr(),
            row_offsets.data_ptr() if grouped else None, num_experts, rows, n, k, _stream_ptr(a.device)))
    return h


def combine(y: torch.Tensor, slot_of: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """out[t] = sum_j weights[t, j] * y[slot_of[t, j]]  (y bf16 [rows, d], weights fp32 [T, k]) -> bf16 [T, d].

    Role of pack_output (2-amd-moe/amd-moe-submission.py:239-301); fp32 accumulation in the order of j.
    """
    if y.dtype != torch.bfloat16 or y.dim() != 2 or not y.is_contiguous() or not y.is_cuda:
        raise ValueError("y must be a contiguous bfloat16 [rows, d] tensor on the GPU")
    if slot_of.dtype != torch.int32 or not slot_of.is_contiguous() or weights.dtype != torch.float32 \
            or not weights.is_contiguous() or slot_of.shape != weights.shape or slot_of.dim() != 2:
        raise ValueError("slot_of (int32) and weights (float32) must be contiguous [tokens, topk] tensors")
    t, k = slot_of.shape
    d = y.shape[1]
    out = torch.empty(t, d, dtype=torch.bfloat16, device=y.device)
    with torch.cuda.device(y.device):
        _lib.check(_lib.load().fp8bs_moe_combine(y.data_ptr(), y.shape[0], slot_of.data_ptr(), weights.data_ptr(), out.data_ptr(),
                                                 t, k, d, _stream_ptr(y.device)))
    return out
