"""Pins the oracle (oracle/fp8bs_oracle.py, oracle/fp8bs_ref.c) without the HIP code: closed forms,
library routines, brute force on tiny inputs and the committed fixtures.  CPU only."""
import json
import os
from fractions import Fraction

import numpy as np
import pytest
import torch

from conftest import GOLDEN


def test_e4m3fn_table_matches_fixture_torch_and_c(oracle, c_oracle):
    tab = oracle.e4m3fn_table()
    with open(os.path.join(GOLDEN, "e4m3fn_table.json")) as f:
        fix = json.load(f)["values"]
    via_torch = torch.arange(256, dtype=torch.int32).to(torch.uint8).view(torch.float8_e4m3fn).float().numpy()
    lib = c_oracle.load()
    for code in range(256):
        if fix[code] == "nan":
            assert np.isnan(tab[code]) and np.isnan(via_torch[code]) and np.isnan(lib.fp8bs_ref_e4m3fn_to_float(code))
            continue
        exact = Fraction(fix[code])
        assert Fraction(float(tab[code])) == exact
        assert Fraction(float(via_torch[code])) == exact          # torch's own conversion routine
        assert Fraction(lib.fp8bs_ref_e4m3fn_to_float(code)) == exact
    assert fix[0x7E] == "448/1" and fix[0x08] == "1/64" and fix[0x01] == "1/512" and fix[0x38] == "1/1"
    assert np.signbit(tab[0x80]) and tab[0x80] == 0.0            # e4m3fn keeps a negative zero


def test_c_bf16_rounding_is_rne(c_oracle):
    lib = c_oracle.load()
    g = torch.Generator().manual_seed(1)
    x = torch.randn(20000, generator=g) * torch.logspace(-20, 20, 20000)
    x = torch.cat([x, torch.tensor([0.0, -0.0, 1.0, 1.00390625, 1.01171875, 3.3895314e38, 65280.0, 1e-40])])
    want = x.to(torch.bfloat16).view(torch.int16).numpy().astype(np.uint16)
    got = np.array([lib.fp8bs_ref_float_to_bf16(float(v)) for v in x.tolist()], dtype=np.uint16)
    assert np.array_equal(got, want)
    # ties go to even: 1 + 2^-8 is exactly between 1.0 and 1 + 2^-7
    assert lib.fp8bs_ref_float_to_bf16(1.00390625) == 0x3F80
    assert lib.fp8bs_ref_float_to_bf16(1.01171875) == 0x3F82


def _rand_case(pkg, m, n, k, seed):
    g = torch.Generator().manual_seed(seed)
    a, a_scale = pkg.inputs.quantize_a(torch.randn(m, k, generator=g))
    b, b_scale = pkg.inputs.quantize_b(torch.randn(n, k, generator=g) * 0.05)
    return a, b, a_scale, b_scale, torch.zeros(m, n, dtype=torch.bfloat16)


def test_dequant_indexing_brute_force_with_tails(pkg, oracle):
    """Storage order a[kk*M+i], b[kk*N+j], as[(kk/128)*M+i], bs[(kk/128)*NB+j/128]
    (reference: 1-amd-fp8-mm/amd-fp8-mm-submission.py:66-75), N = 192 has a partial scale block."""
    m, n, k = 10, 192, 256
    a, b, a_scale, b_scale, _ = _rand_case(pkg, m, n, k, 3)
    tab = oracle.e4m3fn_table()
    nb = (n + 127) // 128
    # flat storage, exactly as the kernels see it
    sa = a.t().contiguous().view(torch.uint8).flatten().tolist()
    sb = b.t().contiguous().view(torch.uint8).flatten().tolist()
    sas = a_scale.t().contiguous().flatten().tolist()
    sbs = b_scale.t().contiguous().flatten().tolist()
    assert len(sbs) == nb * (k // 128)
    da, db = oracle.dequant_a(a, a_scale), oracle.dequant_b(b, b_scale)
    for i in range(m):
        for kk in range(0, k, 7):
            want = np.float32(tab[sa[kk * m + i]]) * np.float32(sas[(kk // 128) * m + i])
            assert da[i, kk].item() == want
    for j in list(range(0, n, 5)) + [127, 128, 191]:
        for kk in range(0, k, 11):
            want = np.float32(tab[sb[kk * n + j]]) * np.float32(sbs[(kk // 128) * nb + j // 128])
            assert db[j, kk].item() == want


def test_ref_kernel_vs_float64_triple_loop(pkg, oracle, c_oracle):
    m, n, k = 5, 7, 256
    data = _rand_case(pkg, m, n, k, 4)
    a, b, a_scale, b_scale, _ = data
    tab = oracle.e4m3fn_table().astype(np.float64)
    av = tab[a.view(torch.uint8).numpy()]
    bv = tab[b.view(torch.uint8).numpy()]
    want = np.zeros((m, n))
    for i in range(m):
        for j in range(n):
            s = 0.0
            for kk in range(k):
                s += av[i, kk] * float(a_scale[i, kk // 128]) * bv[j, kk] * float(b_scale[j // 128, kk // 128])
            want[i, j] = s
    got32 = oracle.ref_kernel_fp32(data).double().numpy()
    assert np.allclose(got32, want, rtol=1e-5, atol=1e-6)
    want_bf16 = torch.from_numpy(want).float().to(torch.bfloat16)
    for got in (oracle.ref_kernel(data), c_oracle.ref_gemm(data)):
        # at most one bf16 ulp apart (fp32 accumulation order can flip a rounding tie)
        assert (got.float() - want_bf16.float()).abs().max() <= want_bf16.float().abs().max() * 2 ** -7


def test_all_ones_scales_reduce_to_plain_matmul(pkg, oracle):
    a, b, a_scale, b_scale, c = _rand_case(pkg, 16, 24, 384, 5)
    ones_a, ones_b = torch.ones_like(a_scale), torch.ones_like(b_scale)
    got = oracle.ref_kernel_fp32((a, b, ones_a, ones_b, c))
    assert torch.equal(got, a.float() @ b.float().t())


def test_one_hot_rows_return_dequantised_b(pkg, oracle):
    m, n, k = 4, 130, 256
    _, b, _, b_scale, c = _rand_case(pkg, m, n, k, 6)
    x = torch.zeros(m, k)
    hot = [3, 127, 128, 255]
    for i, kk in enumerate(hot):
        x[i, kk] = 1.0
    a = x.to(torch.float8_e4m3fn).t().contiguous().t()
    a_scale = torch.full((m, k // 128), 2.0).t().contiguous().t()
    got = oracle.ref_kernel_fp32((a, b, a_scale, b_scale, c))
    db = oracle.dequant_b(b, b_scale)
    for i, kk in enumerate(hot):
        assert torch.equal(got[i], 2.0 * db[:, kk])


def test_scaling_one_a_scale_column_scales_that_block_only(pkg, oracle):
    data = _rand_case(pkg, 8, 256, 384, 7)
    a, b, a_scale, b_scale, c = data
    base = oracle.ref_kernel_fp32(data).double()
    # contribution of K block 1 alone: zero the other blocks' scales
    only1 = a_scale.clone(); only1[:, 0] = 0; only1[:, 2] = 0
    part1 = oracle.ref_kernel_fp32((a, b, only1, b_scale, c)).double()
    doubled = a_scale.clone(); doubled[:, 1] *= 2
    got = oracle.ref_kernel_fp32((a, b, doubled, b_scale, c)).double()
    assert torch.allclose(got, base + part1, rtol=1e-5, atol=1e-6)
    # b_scale picks the right 128-row block: doubling row-block 1 doubles columns 128..255 only
    bs2 = b_scale.clone(); bs2[1, :] *= 2
    got = oracle.ref_kernel_fp32((a, b, a_scale, bs2, c))
    assert torch.equal(got[:, :128], base[:, :128].float()) and torch.equal(got[:, 128:], 2 * base[:, 128:].float())


def test_golden_power_of_two_fixture(golden_gemm, oracle, c_oracle):
    data, expected, expected_fp32 = golden_gemm
    assert torch.equal(oracle.ref_kernel_fp32(data), expected_fp32)        # exact: no rounding freedom
    assert torch.equal(oracle.ref_kernel(data).view(torch.int16), expected.view(torch.int16))
    assert torch.equal(c_oracle.ref_gemm(data).view(torch.int16), expected.view(torch.int16))


def test_torch_and_c_restatements_agree_on_config1(pkg, oracle, c_oracle):
    data = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0])
    r_t, r_c = oracle.ref_kernel(data), c_oracle.ref_gemm(data)
    diff = (r_t.float() - r_c.float()).abs()
    # never more than one bf16 ulp, plus the fp32-vs-double accumulation slack that shows on
    # heavily cancelled (near-zero) outputs
    ulp = r_t.float().abs() * 2 ** -7 + 2e-6 * r_t.float().abs().max()
    assert bool((diff <= ulp).all())
    assert (diff > 0).float().mean() < 0.01          # and almost always identical
    ok, nbad, _ = oracle.within_tolerance(r_c, r_t)
    assert ok and nbad == 0


def test_fold_per_block_equals_dequant_then_matmul(pkg, oracle):
    """sum_kb (sum_k a*b) * as * bs  ==  dequantise-then-matmul, to fp32 rounding (the kernels fold per
    K block, amd-fp8-mm-submission.py:350-352; the oracle dequantises first)."""
    data = _rand_case(pkg, 12, 140, 512, 8)
    a, b, a_scale, b_scale, _ = data
    af, bf = a.double(), b.double()
    folded = torch.zeros(12, 140, dtype=torch.float64)
    for kb in range(4):
        p = af[:, kb * 128:(kb + 1) * 128] @ bf[:, kb * 128:(kb + 1) * 128].t()
        s = a_scale[:, kb].double()[:, None] * b_scale[:, kb].double().repeat_interleave(128)[:140][None, :]
        folded += p * s
    assert torch.allclose(oracle.ref_kernel_fp32(data).double(), folded, rtol=1e-5, atol=1e-5 * float(folded.abs().max()))


def test_grouped_equals_loop_of_dense_and_handles_empty_experts(pkg, oracle, c_oracle):
    cfg = pkg.inputs.CONFIGS[4]
    data = pkg.inputs.make_grouped(cfg, tokens=6, n=136, k=256, experts=8, topk=2)   # some experts get no rows
    a, b, a_scale, b_scale, row_offsets, c = data
    offs = row_offsets.tolist()
    assert offs[0] == 0 and offs[-1] == a.shape[0] == 12 and any(offs[e] == offs[e + 1] for e in range(8))
    got = oracle.ref_grouped(data)
    for e in range(8):
        lo, hi = offs[e], offs[e + 1]
        if hi > lo:
            dense = oracle.ref_kernel((a[lo:hi], b[e], a_scale[lo:hi], b_scale[e], None))
            assert torch.equal(got[lo:hi].view(torch.int16), dense.view(torch.int16))
    sample = torch.tensor([0, 5, 11])
    assert torch.equal(oracle.ref_grouped(data, rows=sample).view(torch.int16), got[sample].view(torch.int16))
    gc = c_oracle.ref_gemm_grouped(data)
    assert oracle.within_tolerance(gc, got)[0]


def test_within_tolerance_rule(oracle):
    ref = torch.tensor([0.0, 1.0, -100.0])
    assert oracle.within_tolerance(torch.tensor([0.0009, 1.02, -101.9]), ref)[0]
    ok, nbad, _ = oracle.within_tolerance(torch.tensor([0.0011, 1.0, -100.0]), ref)
    assert not ok and nbad == 1
    assert not oracle.within_tolerance(torch.tensor([float("nan"), 1.0, -100.0]), ref)[0]
