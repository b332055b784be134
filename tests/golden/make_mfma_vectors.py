"""Records what gfx950's FP8 matrix cores return for crafted and random 128-element dot products.

    python tests/golden/make_mfma_vectors.py [--out tests/golden/mfma_hw_vectors.npz]      (needs an MI355X)

Every vector pair (a row of A, a row of B: 128 e4m3fn codes each, in k-row order of one K block) goes
through the library's C ABI as a GEMM with K = 256 whose second K block is all zero, all scales 1 and a K
split of 2: the first fp32 partial plane of the caller's workspace then holds the raw result of one
v_mfma_f32_16x16x128_f8f6f4 with C = 0 for that pair, before any rounding to bf16.  The fixture holds the
codes and those fp32 results; tests/test_mfma_model.py checks oracle/mfma_model against it on the CPU and
tests/test_gpu_mfma_model.py measures the same vectors again on the GPU it runs on.

The reference ships no vectors for this (it has no tests at all); these are measurements of the hardware,
not outputs of the reference.
"""
import argparse
import importlib
import os
import sys

import numpy as np
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.dirname(os.path.abspath(__file__))))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def code(sig: int, ex: int, neg: int = 0) -> int:
    """e4m3fn code of sig * 2^(ex-3): sig 8..15 with ex -6..8 (normal), sig 0..7 with ex == -6 (subnormal)."""
    if sig >= 8:
        c = ((ex + 7) << 3) | (sig - 8)
    else:
        assert ex == -6
        c = sig
    assert (c & 0x7F) != 0x7F
    return c | (0x80 if neg else 0)


def pow2(p: int) -> int:
    """e4m3fn code of 2^p, -9 <= p <= 8 (subnormal below 2^-6)."""
    return ((p + 7) << 3) if p >= -6 else (1 << (p + 9))


def pow2_pair(v: int, neg: int = 0):
    """(a code, b code) whose product is +-2^v, -18 <= v <= 16."""
    ea = max(-9, min(8, v // 2))
    return pow2(ea) | (0x80 if neg else 0), pow2(v - ea)


def vectors():
    """(A, B, tag): uint8 [count, 128] in k-row order, and what each case is for."""
    rng = np.random.default_rng(20250)
    valid = np.array([c for c in range(256) if (c & 0x7F) != 0x7F], dtype=np.uint8)
    cases, tags = [], []

    def add(items, tag):
        cases.append(items)
        tags.append(tag)

    # a product of 2^16 next to one of 2^e in the same run of 8 / another run of the same lane group / another lane group
    for pos, where in ((1, "same run"), (32, "paired run"), (8, "next lane group"), (64, "second half")):
        for e in range(-2, 9):
            for neg in (0, 1):
                add([(0,) + pow2_pair(16), (pos,) + pow2_pair(e, neg)], "2^16 and 2^%d, %s" % (e, where))
    # subnormal operands: the window hangs on the exponent sum, not on the value
    for e in range(-18, -6):
        add([(0, 0x78, 0x01), (1,) + pow2_pair(e)], "2^8 x 2^-9 (subnormal) and 2^%d" % e)
    # every ordered pair of runs: 2^16 in run q1, 165 * 2^-13 (2.58 output ulps) in run q2
    for q1 in range(16):
        for q2 in range(16):
            if q1 != q2:
                for neg in (0, 1):
                    add([(8 * q1,) + pow2_pair(16), (8 * q2, code(11, -3, neg), code(15, -4))], "order of runs %d %d" % (q1, q2))
    # a small accumulator under a large pair: floored, or dropped when more than 25 binades below
    for d in range(20, 31):
        for neg in (0, 1):
            for sig in (8, 11, 15):
                v = 16 - d
                ea = max(-6, min(8, v // 2))
                add([(0, code(sig, ea, neg), pow2(v - ea)), (8,) + pow2_pair(16)], "accumulator %d binades below the next pair" % d)
    # ties of the final rounding broken (or not) by a term far below the accumulator
    for t in range(1, 11):
        for hs in (0, 1):
            for ts in (0, 1):
                for where in (9, 40, 16, 72):
                    add([(0,) + pow2_pair(16), (8,) + pow2_pair(-8, hs), (where,) + pow2_pair(-8 - t, ts)], "half an ulp and 2^-%d of it" % t)
    # the same against an accumulator with an odd last bit (2^16 + 2^-7), where a tie moves the result
    for t in range(1, 11):
        for hs in (0, 1):
            for ts in (0, 1):
                add([(0,) + pow2_pair(16), (32,) + pow2_pair(-7), (8,) + pow2_pair(-8, hs), (9,) + pow2_pair(-8 - t, ts)], "odd accumulator, half an ulp and 2^-%d of it" % t)
    # a pair whose products cancel to zero still floors the accumulator
    add([(24, code(13, -5, 1), code(12, -5)), (120, code(15, 4), code(8, 7)), (121, code(15, 4, 1), code(8, 7))], "cancelling pair")
    # NaN
    add([(0, 0x7F, 0x00), (1,) + pow2_pair(3)], "NaN x 0")
    add([(100, 0x38, 0xFF), (1,) + pow2_pair(3)], "1 x NaN")
    # random sparse
    for t in range(1400):
        items = []
        for q in rng.choice(16, int(rng.integers(1, 9)), replace=False):
            for r in rng.choice(8, int(rng.integers(1, 4)), replace=False):
                items.append((8 * int(q) + int(r), int(valid[rng.integers(0, len(valid))]), int(valid[rng.integers(0, len(valid))])))
        add(items, "random sparse")
    # dense: quantised N(0,1) rows as the benchmark configurations have them, narrow exponent bands (heavy
    # cancellation), and uniformly random codes
    for t in range(400):
        x = rng.standard_normal((2, 128)).astype(np.float32)
        x = x / np.abs(x).max(axis=1, keepdims=True) * 448.0
        q = torch.from_numpy(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
        add([(k, int(q[0, k]), int(q[1, k])) for k in range(128)], "dense gaussian")
    for t in range(200):
        lo = int(rng.integers(0, 9))
        a = (((rng.integers(lo, lo + 3, 128) + 4) << 3) | rng.integers(0, 8, 128) | (rng.integers(0, 2, 128) << 7)).astype(np.uint8)
        b = (((rng.integers(lo, lo + 3, 128) + 2) << 3) | rng.integers(0, 8, 128) | (rng.integers(0, 2, 128) << 7)).astype(np.uint8)
        add([(k, int(a[k]), int(b[k])) for k in range(128)], "dense narrow band")
    for t in range(200):
        a, b = valid[rng.integers(0, len(valid), 128)], valid[rng.integers(0, len(valid), 128)]
        add([(k, int(a[k]), int(b[k])) for k in range(128)], "dense random codes")
    A = np.zeros((len(cases), 128), dtype=np.uint8)
    B = np.zeros((len(cases), 128), dtype=np.uint8)
    for i, items in enumerate(cases):
        for k, ca, cb in items:
            A[i, k], B[i, k] = ca, cb
    return A, B, np.array(tags)


def measure(A: np.ndarray, B: np.ndarray, variant: int = 3, chunk: int = 2048) -> np.ndarray:
    """fp32 [count]: the matrix cores' result for every (A[i], B[i]) pair, through the C ABI (see module docstring)."""
    pkg = importlib.import_module("amd-developer-challenge-2025_amd")
    lib = pkg._lib.load()
    dev = torch.device("cuda:0")
    out = np.zeros(A.shape[0], dtype=np.float32)
    for lo in range(0, A.shape[0], chunk):
        a_, b_ = A[lo:lo + chunk], B[lo:lo + chunk]
        m = a_.shape[0]
        n = (m + 7) // 8 * 8
        a = torch.zeros(256, m, dtype=torch.uint8)
        a[:128] = torch.from_numpy(np.ascontiguousarray(a_.T))
        b = torch.zeros(256, n, dtype=torch.uint8)
        b[:128, :m] = torch.from_numpy(np.ascontiguousarray(b_.T))
        a, b = a.to(dev), b.to(dev)
        a_scale = torch.ones(2, m, dtype=torch.float32, device=dev)
        b_scale = torch.ones(2, (n + 127) // 128, dtype=torch.float32, device=dev)
        c = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
        ws = torch.zeros(2, m, n, dtype=torch.float32, device=dev)
        pkg._lib.check(lib.fp8bs_gemm_ex(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(),
                                         ws.data_ptr(), ws.numel() * 4, m, n, 256, variant, 2, None))
        torch.cuda.synchronize()
        out[lo:lo + m] = torch.diagonal(ws[0][:, :m]).cpu().numpy()
    return out


def measure_16x16x32(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """fp32 [count]: the same pairs through the FP8 MFMA of the reference's kernel, v_mfma_f32_16x16x32_fp8_fp8,
    four chained per 128 k with the fp32 accumulator carried through
    (1-amd-fp8-mm/amd-fp8-mm-submission.py:345-352), measured by the checker's probe kernel
    (oracle/mfma_16x16x32_probe.hip)."""
    from oracle import c_oracle
    lib = c_oracle.load_probe()
    dev = torch.device("cuda:0")
    a = torch.from_numpy(np.ascontiguousarray(A)).to(dev)
    b = torch.from_numpy(np.ascontiguousarray(B)).to(dev)
    out = torch.zeros(A.shape[0], dtype=torch.float32, device=dev)
    assert lib.mfma_probe_chain_16x16x32(a.data_ptr(), b.data_ptr(), A.shape[0], out.data_ptr(), None) == 0
    torch.cuda.synchronize()
    return out.cpu().numpy()


def exact_sums(A: np.ndarray, B: np.ndarray) -> np.ndarray:
    """float64 [count]: the exact value of every dot product (every product is a multiple of 2^-18 below 2^18,
    so 128 of them add up without rounding in a double); NaN where an operand holds a NaN code."""
    def dec(c):
        c = c.astype(np.int64)
        e, m = (c >> 3) & 15, c & 7
        v = np.where(e == 0, m * 2.0 ** -9, (8 + m) * 2.0 ** (e - 10.0))
        return np.where(c >> 7, -v, v)
    s = (dec(A) * dec(B)).sum(axis=1)
    nan = ((A & 0x7F) == 0x7F).any(axis=1) | ((B & 0x7F) == 0x7F).any(axis=1)
    return np.where(nan, np.nan, s)


if __name__ == "__main__":
    ap = argparse.ArgumentParser()
    ap.add_argument("--out", default=os.path.join(ROOT, "tests", "golden", "mfma_hw_vectors.npz"))
    ap.add_argument("--out32", default=os.path.join(ROOT, "tests", "golden", "mfma_16x16x32_hw_vectors.npz"),
                    help="results of the reference's instruction on the same vectors (D32 only; the codes are in --out)")
    ap.add_argument("--only32", action="store_true", help="leave --out as it is")
    args = ap.parse_args()
    A, B, tags = vectors()
    os.makedirs(os.path.dirname(os.path.abspath(args.out)), exist_ok=True)
    if not args.only32:
        D = measure(A, B)
        np.savez_compressed(args.out, A=A, B=B, D=D, tags=tags)
        print("recorded %d dot products -> %s" % (len(D), args.out), flush=True)
    D32 = measure_16x16x32(A, B)
    np.savez_compressed(args.out32, D32=D32)
    print("recorded %d chained 16x16x32 results -> %s" % (len(D32), args.out32), flush=True)
