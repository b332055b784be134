"""Parity of the fused silu-mul GEMM epilogue and the weighted un-permute with oracle/moe_oracle.py on a
real MI355X (bar: |out - ref| <= 1e-3 + 2e-2*|ref| on every element), and the whole expert FFN chain.
Run with:  python -u -m pytest tests -m gpu
"""
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu
RTOL, ATOL = 2e-2, 1e-3


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def mo():
    return importlib.import_module("oracle.moe_oracle")


@pytest.fixture(scope="module")
def ro():
    return importlib.import_module("oracle.route_oracle")


@pytest.fixture(scope="module")
def moe(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.moe")


@pytest.fixture(scope="module")
def quant(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.quant")


def _within(oracle, out, ref, what):
    ok, nbad, maxerr = oracle.within_tolerance(out, ref, RTOL, ATOL)
    assert ok, "%s: %d elements outside the bar (max abs err %g)" % (what, nbad, maxerr)


@pytest.mark.parametrize("m,n,k", [(256, 512, 512), (272, 288, 256), (100, 70, 128), (512, 4096, 1024),
                                   (257, 512, 256), (1023, 288, 384), (3, 64, 128), (130, 4096, 128),      # rows off the 4-row grid
                                   (300, 380, 256), (129, 2002, 128), (64, 6, 128), (513, 1038, 384),      # n/2 off the 8-column grid: rows of h stored in pieces
                                   (128, 72, 128), (300, 296, 256), (257, 1080, 384), (64, 8, 128)])       # n on the 8-column grid, n/2 four columns off it
def test_dense_silu_mul(pkg, moe, oracle, mo, dev, m, n, k):
    """std 0.02 weights keep gate/up at O(1) so that silu is exercised around its bend"""
    g = torch.Generator().manual_seed(m + n)
    a, a_scale = pkg.inputs.quantize_a(torch.randn(m, k, generator=g))
    b, b_scale = pkg.inputs.quantize_b(torch.randn(n, k, generator=g) * (2.0 / k ** 0.5))
    h = torch.full((m, n // 2), 7.0, dtype=torch.bfloat16, device=dev)
    out = moe.gate_up_silu((a.to(dev), b.to(dev), a_scale.to(dev), b_scale.to(dev), None, h))
    assert out is h
    ref = mo.silu_mul_ref(oracle.ref_kernel_fp32((a, b, a_scale, b_scale, None)))
    _within(oracle, out.cpu(), ref, "dense silu_mul %dx%dx%d" % (m, n, k))


@pytest.mark.parametrize("tokens,n", [(160, 512), (161, 512), (67, 512),        # 480 rows; 483 and 201: totals off the 4-row grid
                                      (160, 380), (67, 2002), (161, 262),       # n/2 off the 8-column grid, n off the 4-byte grid of b's rows
                                      (160, 104), (161, 1336), (67, 584)])      # n a multiple of 8 but not of 16
def test_grouped_silu_mul(pkg, moe, oracle, mo, dev, tokens, n):
    cfg = pkg.inputs.CONFIGS[4]
    data = pkg.inputs.make_grouped(cfg, tokens=tokens, n=n, k=256, experts=6, topk=3)
    a, b, a_scale, b_scale, row_offsets, c = data
    rows = a.shape[0]
    h = torch.zeros(rows, n // 2, dtype=torch.bfloat16, device=dev)
    out = moe.gate_up_silu((a.to(dev), b.to(dev), a_scale.to(dev), b_scale.to(dev), row_offsets.to(dev), h))
    offs = row_offsets.tolist()
    ref = torch.empty(rows, n // 2, dtype=torch.bfloat16)
    for e in range(6):
        if offs[e + 1] > offs[e]:
            sl = slice(offs[e], offs[e + 1])
            # scale so that the pre-activations are O(1)
            ref[sl] = mo.silu_mul_ref(oracle.ref_kernel_fp32((a[sl], b[e], a_scale[sl], b_scale[e], None)))
    _within(oracle, out.cpu(), ref, "grouped silu_mul")


@pytest.mark.parametrize("tokens,k,d", [(100, 4, 256), (33, 8, 7168), (1, 1, 8)])
def test_combine(moe, oracle, mo, dev, tokens, k, d):
    g = torch.Generator().manual_seed(tokens + d)
    rows = tokens * k
    y = torch.randn(rows, d, generator=g).to(torch.bfloat16)
    slot = torch.randperm(rows, generator=g).reshape(tokens, k).to(torch.int32)
    if tokens > 2:
        slot[2, 0] = -1
    w = torch.rand(tokens, k, generator=g)
    out = moe.combine(y.to(dev), slot.to(dev), w.to(dev))
    _within(oracle, out.cpu(), mo.combine_ref(y, slot, w), "combine")


def test_expert_ffn_chain(pkg, moe, quant, oracle, mo, ro, dev):
    """scores -> top-k -> route -> quantise+gather -> gate/up GEMM with fused silu-mul -> quantise ->
    down GEMM -> weighted un-permute, against the same chain built from the oracles on the host."""
    tokens, experts, topk, dh, di = 192, 4, 2, 256, 128
    g = torch.Generator().manual_seed(5)
    x = torch.randn(tokens, dh, generator=g)
    scores = torch.softmax(torch.randn(tokens, experts, generator=g), dim=1)
    w13 = [torch.randn(2 * di, dh, generator=g) * (2.0 / dh ** 0.5) for _ in range(experts)]     # gate/up interleaved by row
    w2 = [torch.randn(dh, di, generator=g) * (1.0 / di ** 0.5) for _ in range(experts)]

    def stack(ws, qfn, n, k, device=None):
        bs = torch.empty(experts, k, n, dtype=torch.float8_e4m3fn, device=device)
        ss = torch.empty(experts, k // 128, (n + 127) // 128, dtype=torch.float32, device=device)
        for e in range(experts):
            qb, sb = qfn(ws[e] if device is None else ws[e].to(device))
            bs[e], ss[e] = qb.t(), sb.t()
        return bs.transpose(1, 2), ss.transpose(1, 2)

    # ---- device chain ----
    sc = scores.to(dev)
    top = moe.topk(sc, topk)
    row_offsets, row_map, slot_of = moe.route(top, experts)
    a1, a1s = quant.quantize_a(x.to(dev), row_map)
    b13, b13s = stack(w13, quant.quantize_b, 2 * di, dh, dev)
    rows = tokens * topk
    h = moe.gate_up_silu((a1, b13, a1s, b13s, row_offsets, torch.empty(rows, di, dtype=torch.bfloat16, device=dev)))
    a2, a2s = quant.quantize_a(h)
    b2, b2s = stack(w2, quant.quantize_b, dh, di, dev)
    y = pkg.grouped_kernel((a2, b2, a2s, b2s, row_offsets, torch.empty(rows, dh, dtype=torch.bfloat16, device=dev)))
    weights = torch.gather(sc, 1, top.long())
    out = moe.combine(y, slot_of, weights)

    # ---- host chain from the oracles ----
    top_r = ro.topk_ref(scores.numpy(), topk)
    offs_r, map_r, slot_r = ro.route_ref(top_r, experts)
    assert np.array_equal(top.cpu().numpy(), top_r) and np.array_equal(slot_of.cpu().numpy(), slot_r)
    ha1, ha1s = pkg.inputs.quantize_a(x[torch.from_numpy(map_r).long()])
    hb13, hb13s = stack(w13, pkg.inputs.quantize_b, 2 * di, dh)
    hb2, hb2s = stack(w2, pkg.inputs.quantize_b, dh, di)
    h_r = torch.empty(rows, di, dtype=torch.bfloat16)
    for e in range(experts):
        sl = slice(int(offs_r[e]), int(offs_r[e + 1]))
        if sl.stop > sl.start:
            h_r[sl] = mo.silu_mul_ref(oracle.ref_kernel_fp32((ha1[sl], hb13[e], ha1s[sl], hb13s[e], None)))
    _within(oracle, h.cpu(), h_r, "chain: gate/up + silu_mul")
    # the second half is checked from the device's own h (bit-identical operands on both sides)
    ha2, ha2s = pkg.inputs.quantize_a(h.cpu().float())
    assert torch.equal(a2.cpu().view(torch.uint8), ha2.view(torch.uint8)) and torch.equal(a2s.cpu(), ha2s)
    y_r = oracle.ref_grouped((ha2, hb2, ha2s, hb2s, torch.from_numpy(offs_r), None))
    _within(oracle, y.cpu(), y_r, "chain: down projection")
    out_r = mo.combine_ref(y.cpu(), torch.from_numpy(slot_r), torch.gather(scores, 1, torch.from_numpy(top_r).long()))
    _within(oracle, out.cpu(), out_r, "chain: combine")


def test_out_of_range_tables_are_ignored(pkg, moe, dev):
    """row offsets beyond the matrix and slots beyond y must not write or read outside the tensors"""
    g = torch.Generator().manual_seed(9)
    y = torch.randn(32, 64, generator=g).to(torch.bfloat16).to(dev)
    slot = torch.tensor([[0, 31], [5, 32], [-7, 4], [1000000, 2]], dtype=torch.int32, device=dev)
    w = torch.ones(4, 2, device=dev)
    out = moe.combine(y, slot, w).float().cpu()
    yf = y.float().cpu()
    assert torch.allclose(out[0], (yf[0] + yf[31]).to(torch.bfloat16).float())
    assert torch.equal(out[1], yf[5]) and torch.equal(out[2], yf[4]) and torch.equal(out[3], yf[2])
    data = pkg.inputs.make_grouped(pkg.inputs.CONFIGS[4], tokens=64, n=256, k=128, experts=4, topk=2)
    a, b, a_scale, b_scale, row_offsets, c = (t.to(dev) for t in data)
    good = pkg.grouped_kernel((a, b, a_scale, b_scale, row_offsets, torch.zeros_like(c))).clone()
    bad = row_offsets.clone()
    bad[-1] = 10 ** 6                                          # last expert claims rows far beyond the matrix
    guard = torch.full((c.shape[0] + 64, c.shape[1]), 5.0, dtype=torch.bfloat16, device=dev)
    out = pkg.grouped_kernel((a, b, a_scale, b_scale, bad, guard[:c.shape[0]]))
    torch.cuda.synchronize()
    assert torch.equal(out.view(torch.int16), good.view(torch.int16))
    assert bool((guard[c.shape[0]:] == 5.0).all())
