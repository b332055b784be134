"""TEST INFRASTRUCTURE ONLY - CPU restatement of the reference's FP8 block-scaled GEMM semantics.

Nothing in the product path imports this file: only tests/, __graft_entry__.smoke() and the
cpu_baseline leg of bench.py may, and only as the checker.

What it restates (each function cites the reference lines it follows):
  * dequantisation   A32[i,kk] = float(a[i,kk]) * a_scale[i, kk/128]
                     B32[j,kk] = float(b[j,kk]) * b_scale[j/128, kk/128]
                     (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:17-25, 34-42)
  * product          C = A32 @ B32^T in fp32  (0-amd-fp8-mm-new-begins.py:85-89)
  * output cast      bf16, round to nearest even (1-amd-fp8-mm/amd-fp8-mm-submission.py:364)
  * grouped walk     expert e owns rows [row_offsets[e], row_offsets[e+1])
                     (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:142-148, 328-336)
The FP8 type is OCP e4m3fn (gfx950), not the reference's e4m3fnuz (gfx942); the decode used here is
the closed form  (-1)^s * 2^(e-7) * (1 + m/8),  subnormals m * 2^-9,  NaN at 0x7F / 0xFF.

How each function is pinned (the reference ships no tests, golden vectors or fixtures, and its
harness `task`/`reference` modules are not vendored, so nothing from the reference itself can pin
these; the checks below are in tests/test_oracle.py):
  * e4m3fn_table      all 256 codes against torch's own float8_e4m3fn -> float32 conversion and
                      against the independent C decoder in oracle/fp8bs_ref.c
  * dequant_a/b       brute-force gather with explicit Python loops over the storage order
                      a[kk*M+i], b[kk*N+j], as[(kk/128)*M+i], bs[(kk/128)*NB+j/128]
                      (amd-fp8-mm-submission.py:66-75) on shapes with N tails
  * ref_kernel        float64 triple loop on tiny inputs; all-ones scales reduce it to a plain
                      matmul; one-hot A rows return dequantised B rows; scaling one a_scale column
                      scales exactly that K block's contribution; the committed power-of-two fixture
                      tests/golden/gemm_16x32x256.json (exact in fp32); and bit-for-bit (<= 1 bf16
                      ulp) agreement with the independent C restatement on configuration 1
  * ref_grouped       equals a loop of ref_kernel over row_offsets slices; empty experts
  * parity_report     the strict per-element bar; what it excuses is decided by oracle/mfma_model, which is
                      pinned on its own (tests/test_mfma_model.py: hand-built cases, two implementations,
                      dot products recorded on MI355X)
"""
import numpy as np
import torch

BLOCK = 128


def e4m3fn_table() -> np.ndarray:
    """float32[256]: value of every OCP e4m3fn code, closed form (bias 7, no inf, NaN = S.1111.111)."""
    out = np.empty(256, dtype=np.float32)
    for code in range(256):
        s, e, m = code >> 7, (code >> 3) & 15, code & 7
        if e == 0:
            v = m * 2.0 ** -9
        elif e == 15 and m == 7:
            v = float("nan")
        else:
            v = 2.0 ** (e - 7) * (1.0 + m / 8.0)
        out[code] = -v if s else v
    return out


def dequant_a(a: torch.Tensor, a_scale: torch.Tensor) -> torch.Tensor:
    """fp32 [M, K] = float(a) * a_scale broadcast over each 1x128 block
    (dqa_kernel, 1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:17-25)."""
    return a.float() * a_scale.float().repeat_interleave(BLOCK, dim=1)


def dequant_b(b: torch.Tensor, b_scale: torch.Tensor) -> torch.Tensor:
    """fp32 [N, K] = float(b) * b_scale broadcast over each 128x128 block, NB = ceil(N/128) scale rows
    (dqb_kernel, 1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:34-42)."""
    n = b.shape[0]
    s = b_scale.float().repeat_interleave(BLOCK, dim=0)[:n].repeat_interleave(BLOCK, dim=1)
    return b.float() * s


def ref_kernel(data):
    """Oracle of custom_kernel: dequantise, fp32 matmul, cast to bf16; returns a new [M, N] bf16 tensor
    (1-amd-fp8-mm/0-amd-fp8-mm-new-begins.py:85-89 plus the bf16 store of amd-fp8-mm-submission.py:364)."""
    a, b, a_scale, b_scale = (t.cpu() for t in data[:4])
    c32 = dequant_a(a, a_scale) @ dequant_b(b, b_scale).t()
    return c32.to(torch.bfloat16)


def ref_kernel_fp32(data) -> torch.Tensor:
    """Same as ref_kernel without the final bf16 rounding (what the reference's NB script returns)."""
    a, b, a_scale, b_scale = (t.cpu() for t in data[:4])
    return dequant_a(a, a_scale) @ dequant_b(b, b_scale).t()


def ref_grouped(data, rows=None):
    """Oracle of grouped_kernel: data = (a, b, a_scale, b_scale, row_offsets, c); b is [E, N, K].
    Expert e multiplies rows [row_offsets[e], row_offsets[e+1]) by its own weight
    (2-amd-moe/3-amd-fp8-moe-hip-myhgemm.py:328-336).  ``rows``: optional 1-D LongTensor of row
    indices to evaluate (a sample, to bound CPU time); returns bf16 [len(rows) or total, N]."""
    a, b, a_scale, b_scale, row_offsets = (t.cpu() for t in data[:5])
    offs = row_offsets.tolist()
    n = b.shape[1]
    if rows is None:
        rows = torch.arange(a.shape[0])
    out = torch.empty(len(rows), n, dtype=torch.bfloat16)
    for e in range(len(offs) - 1):
        sel = ((rows >= offs[e]) & (rows < offs[e + 1])).nonzero().flatten()
        if sel.numel() == 0:
            continue
        r = rows[sel]
        a32 = dequant_a(a[r], a_scale[r])
        out[sel] = (a32 @ dequant_b(b[e], b_scale[e]).t()).to(torch.bfloat16)
    return out


def within_tolerance(out: torch.Tensor, ref: torch.Tensor, rtol: float = 2e-2, atol: float = 1e-3):
    """Per-element check |out - ref| <= atol + rtol*|ref| (the bar the build is held to).
    Returns (ok, number of violating elements, max abs error)."""
    o, r = out.float().cpu(), ref.float().cpu()
    err = (o - r).abs()
    bad = ~(err <= atol + rtol * r.abs())
    return (not bool(bad.any())), int(bad.sum()), float(err.max()) if err.numel() else 0.0


def parity_report(out: torch.Tensor, ref: torch.Tensor, data, split_k: int = 1, rtol: float = 2e-2, atol: float = 1e-3):
    """The bar of the build with every exception accounted for.

    Every element must satisfy |out - ref| <= atol + rtol*|ref| against the exact-fp32 oracle `ref`, or be
    bit-identical to what the instruction-level model of the FP8 matrix cores (oracle/mfma_model) gives for
    the kernel's arithmetic on `data` with this K split: then the deviation is the instruction's rounding,
    reproduced on the CPU, not the kernel's.  (On N(0,1) x N(0,1) operands the outputs are large against
    atol and a few heavily cancelled near-zero outputs land beyond the bar that way.)
    Returns (ok, strict_violations, violations_not_reproduced_by_the_model)."""
    from . import mfma_model
    o, r = out.float().cpu(), ref.float().cpu()
    bad = ~((o - r).abs() <= atol + rtol * r.abs())
    nstrict = int(bad.sum())
    if nstrict == 0:
        return True, 0, 0
    idx = bad.nonzero().numpy()
    modelled, _ = mfma_model.model_kernel_at(data, idx, split_k)
    got = out.cpu()[bad]
    unexplained = int((got.view(torch.int16) != modelled.view(torch.int16)).sum())
    return unexplained == 0, nstrict, unexplained
