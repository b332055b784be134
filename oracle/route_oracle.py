"""TEST INFRASTRUCTURE ONLY - CPU restatement (numpy) of the MoE routing in front of the grouped GEMM.

Nothing in the product path imports this file: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may, and only as the checker.

What it restates, citing the reference's fp16 MoE layer (2-amd-moe/amd-moe-submission.py):
  * topk_ref    the selection rule of `topk` (:32-56) and `top4_nre32` (:58-105): per token, k times
                the strictly greatest score not yet taken; the scan runs over ascending expert index
                with a strict comparison, so the lowest index wins among equal scores; results are
                best-first; a score that is not greater than -inf (-inf itself, NaN) is never taken
                and leaves index -1
  * route_ref   the bookkeeping of `calculate_index` (:107-156) + the exclusive prefix of
                `calculate_offset` (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:142-148), with the total
                appended, and with the one freedom the reference leaves (its positions come from
                atomicAdd and vary between runs) fixed: rows of an expert are ordered by token id

How each function is pinned (tests/test_route_oracle.py; the reference has no tests or fixtures):
  * topk_ref    torch.topk on rows of distinct scores (a library routine); a hand-written tie
                fixture; sortedness of the selected scores; -inf / NaN rows
  * route_ref   the permutation and row_offsets that inputs.make_grouped derives independently with
                torch.sort / bincount / cumsum; invariants: row_map restricted to an expert is strictly
                increasing, slot_of inverts row_map, row_offsets is the prefix sum of the histogram
"""
import numpy as np


def topk_ref(scores: np.ndarray, k: int) -> np.ndarray:
    """scores float32 [T, E] -> int32 [T, k] following amd-moe-submission.py:32-56 literally."""
    scores = np.asarray(scores, dtype=np.float32)
    t, e = scores.shape
    out = np.full((t, k), -1, dtype=np.int32)
    for row in range(t):
        for i in range(k):
            best, best_j = -np.inf, -1
            for j in range(e):
                if scores[row, j] > best and j not in out[row, :i]:
                    best, best_j = scores[row, j], j
            out[row, i] = best_j
    return out


def route_ref(top_idx: np.ndarray, experts: int):
    """top_idx int [T, k] -> (row_offsets int32 [E+1], row_map int32 [T*k] (-1 beyond the total), slot_of int32 [T, k]).

    Entries outside [0, experts) are ignored; an expert repeated inside one token's list keeps one row
    (its first occurrence).
    """
    top_idx = np.asarray(top_idx)
    t, k = top_idx.shape
    per_expert = [[] for _ in range(experts)]
    for tok in range(t):
        for j in range(k):
            e = int(top_idx[tok, j])
            if 0 <= e < experts and e not in top_idx[tok, :j]:
                per_expert[e].append((tok, j))
    row_offsets = np.zeros(experts + 1, dtype=np.int32)
    row_map = np.full(t * k, -1, dtype=np.int32)
    slot_of = np.full((t, k), -1, dtype=np.int32)
    row = 0
    for e in range(experts):
        row_offsets[e] = row
        for tok, j in per_expert[e]:          # appended in token order
            row_map[row] = tok
            slot_of[tok, j] = row
            row += 1
    row_offsets[experts] = row
    return row_offsets, row_map, slot_of
