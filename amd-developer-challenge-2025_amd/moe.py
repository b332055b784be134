"""MoE routing on the GPU: top-k selection, row_offsets and the expert-contiguous row order.

Wraps ``fp8bs_moe_topk`` / ``fp8bs_moe_route`` of libfp8bs.so.  Roles in the reference
(2-amd-moe/amd-moe-submission.py): ``top4_nre32`` / ``topk`` (:32-105), ``calculate_index`` (:107-156)
and the host read of the counts (:230-234); here nothing synchronises with the host and the row order is
deterministic (by expert, then token id).  The outputs plug into ``quant.quantize_a(x, row_map)`` and
``grouped_kernel``.  No fallback: without the library the import of ``_lib`` raises.
"""
from typing import Tuple

import torch

from . import _lib


def topk(scores: torch.Tensor, k: int) -> torch.Tensor:
    """scores fp32 [T, E] row-major on the GPU -> int32 [T, k], best first, lowest index first among equals."""
    if scores.dtype != torch.float32 or scores.dim() != 2 or not scores.is_cuda or not scores.is_contiguous():
        raise ValueError("scores must be a contiguous float32 [tokens, experts] tensor on the GPU")
    t, e = scores.shape
    out = torch.empty(t, k, dtype=torch.int32, device=scores.device)
    with torch.cuda.device(scores.device):
        _lib.check(_lib.load().fp8bs_moe_topk(scores.data_ptr(), t, e, k, out.data_ptr(),
                                              torch.cuda.current_stream().cuda_stream))
    return out


def route(top_idx: torch.Tensor, experts: int) -> Tuple[torch.Tensor, torch.Tensor, torch.Tensor]:
    """top_idx int32 [T, k] -> (row_offsets int32 [E+1], row_map int32 [T*k], slot_of int32 [T, k]).

    Expert e owns rows [row_offsets[e], row_offsets[e+1]); ``row_map[row]`` is the token of that row
    (rows of an expert ordered by token id); ``slot_of[t, j]`` is the row of token t's j-th choice.
    Rows beyond ``row_offsets[E]`` (only if some entries of ``top_idx`` are outside [0, E)) are -1.
    """
    if top_idx.dtype != torch.int32 or top_idx.dim() != 2 or not top_idx.is_cuda or not top_idx.is_contiguous():
        raise ValueError("top_idx must be a contiguous int32 [tokens, topk] tensor on the GPU")
    t, k = top_idx.shape
    dev = top_idx.device
    row_offsets = torch.empty(experts + 1, dtype=torch.int32, device=dev)
    row_map = torch.full((t * k,), -1, dtype=torch.int32, device=dev)
    slot_of = torch.empty(t, k, dtype=torch.int32, device=dev)
    with torch.cuda.device(dev):
        lib = _lib.load()
        need = lib.fp8bs_moe_route_workspace_bytes(t, experts)
        ws = torch.empty(max(need, 4), dtype=torch.uint8, device=dev)
        _lib.check(lib.fp8bs_moe_route(top_idx.data_ptr(), t, experts, k, row_offsets.data_ptr(), row_map.data_ptr(),
                                       slot_of.data_ptr(), ws.data_ptr(), ws.numel(), torch.cuda.current_stream().cuda_stream))
    return row_offsets, row_map, slot_of
