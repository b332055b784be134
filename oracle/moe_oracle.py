"""TEST INFRASTRUCTURE ONLY - CPU restatement (torch/numpy) of the expert-FFN pieces around the grouped GEMM.

Nothing in the product path imports this file: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may, and only as the checker.

What it restates, citing the reference's fp16 MoE layer (2-amd-moe/amd-moe-submission.py):
  * silu_mul_ref   re_silu_mul_kernel (:366-407): silu(gate) * up with silu(x) = x / (1 + exp(-x)).
                   Here gate_i / up_i are columns 2i / 2i+1 of the fp32 block-scaled product (the layout
                   the fused epilogue needs) and the result is rounded once to bf16; the reference
                   rounds silu to fp16 before an fp16 multiply, a difference far inside the bar
                   (rtol 2e-2, atol 1e-3) the outputs are held to.
  * combine_ref    pack_output (:239-301): out[t] = sum_j weight[t][j] * y[row of (t, j)], accumulated
                   in the order j = 0..topk-1 (fp32 here, fp16 there), entries without a row skipped.

How each function is pinned (tests/test_moe_oracle.py; the reference has no tests or fixtures):
  * silu_mul_ref   torch.nn.functional.silu (a library routine) on de-interleaved columns; the values
                   silu(0) = 0, silu(x) -> x for large x, -> 0 for very negative x; a hand-checked 2x4 case
  * combine_ref    an explicit Python triple loop; torch.index_add_ on the flattened (token, choice)
                   list; one-hot weights return rows of y; linearity in the weights
"""
import torch


def silu_mul_ref(c_fp32: torch.Tensor) -> torch.Tensor:
    """fp32 [rows, n] (n even, columns gate0, up0, gate1, up1, ...) -> bf16 [rows, n/2]."""
    c = c_fp32.float()
    gate, up = c[:, 0::2], c[:, 1::2]
    return (gate / (1.0 + torch.exp(-gate)) * up).to(torch.bfloat16)


def combine_ref(y: torch.Tensor, slot_of: torch.Tensor, weights: torch.Tensor) -> torch.Tensor:
    """y bf16 [rows, d], slot_of int [T, k], weights fp32 [T, k] -> bf16 [T, d]."""
    t, k = slot_of.shape
    yf = y.float()
    acc = torch.zeros(t, y.shape[1], dtype=torch.float32)
    for j in range(k):                                   # fixed order of accumulation
        s = slot_of[:, j].long()
        ok = s >= 0
        term = torch.zeros_like(acc)
        term[ok] = weights[ok, j].unsqueeze(1) * yf[s[ok]]
        # fused multiply-add in fp32 is what the kernel does; the difference to mul+add is below bf16 resolution
        acc = acc + term
    return acc.to(torch.bfloat16)
