"""Pins oracle/moe_oracle.py without the reference (which ships no tests)."""
import importlib

import pytest
import torch


@pytest.fixture(scope="module")
def mo():
    return importlib.import_module("oracle.moe_oracle")


def test_silu_mul_against_torch_silu_and_closed_values(mo):
    g = torch.Generator().manual_seed(1)
    c = torch.randn(37, 64, generator=g) * 3
    want = (torch.nn.functional.silu(c[:, 0::2]) * c[:, 1::2]).to(torch.bfloat16)
    got = mo.silu_mul_ref(c)
    assert got.shape == (37, 32)
    assert torch.allclose(got.float(), want.float(), rtol=2 ** -7, atol=1e-30)        # <= 1 bf16 ulp
    hand = torch.tensor([[0.0, 5.0, 2.0, 3.0], [50.0, 2.0, -50.0, 7.0]])
    out = mo.silu_mul_ref(hand).float()
    assert out[0, 0] == 0.0                                                             # silu(0) = 0
    assert abs(out[0, 1] - 2.0 / (1 + 2.718281828 ** -2) * 3.0) < 0.02                  # 5.2848
    assert out[1, 0] == 100.0 and abs(out[1, 1]) < 1e-15                                # silu(50) = 50, silu(-50) ~ 0


def test_combine_against_loops_and_index_add(mo):
    g = torch.Generator().manual_seed(2)
    rows, d, t, k = 40, 24, 13, 3
    y = torch.randn(rows, d, generator=g).to(torch.bfloat16)
    slot = torch.stack([torch.randperm(rows, generator=g)[:k] for _ in range(t)]).to(torch.int32)
    slot[2, 1] = -1
    w = torch.rand(t, k, generator=g)
    got = mo.combine_ref(y, slot, w).float()
    loop = torch.zeros(t, d)
    for tok in range(t):
        for j in range(k):
            if slot[tok, j] >= 0:
                for c in range(d):
                    loop[tok, c] += w[tok, j] * float(y[slot[tok, j], c])
    assert torch.allclose(got, loop, rtol=2 ** -7, atol=1e-6)
    flat_ok = (slot >= 0).reshape(-1)
    ia = torch.zeros(t, d).index_add_(0, torch.arange(t).repeat_interleave(k)[flat_ok],
                                      (w.reshape(-1, 1) * y.float()[slot.reshape(-1).clamp(min=0).long()])[flat_ok])
    assert torch.allclose(got, ia, rtol=2 ** -7, atol=1e-6)


def test_combine_one_hot_and_linearity(mo):
    g = torch.Generator().manual_seed(3)
    y = torch.randn(10, 16, generator=g).to(torch.bfloat16)
    slot = torch.tensor([[3, 7], [0, 9]], dtype=torch.int32)
    one_hot = torch.tensor([[1.0, 0.0], [0.0, 1.0]])
    out = mo.combine_ref(y, slot, one_hot)
    assert torch.equal(out[0], y[3]) and torch.equal(out[1], y[9])
    w = torch.rand(2, 2, generator=g)
    a = mo.combine_ref(y, slot, w).float()
    b = mo.combine_ref(y, slot, 2 * w).float()
    assert torch.allclose(b, 2 * a, rtol=2 ** -7)
