"""Parity of the HIP routing kernels (through the C ABI) with oracle/route_oracle.py on a real MI355X:
index outputs bit for bit, and the whole chain scores -> top-k -> row_offsets/row_map -> gathered
quantisation -> grouped GEMM against the oracle's grouped product.  Run with:  python -u -m pytest tests -m gpu
"""
import importlib

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    return torch.device("cuda:0")


@pytest.fixture(scope="module")
def ro():
    return importlib.import_module("oracle.route_oracle")


@pytest.fixture(scope="module")
def moe(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.moe")


@pytest.fixture(scope="module")
def quant(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.quant")


@pytest.mark.parametrize("tokens,experts,k", [(300, 32, 4), (1000, 32, 8), (257, 5, 2), (64, 256, 6), (1, 8, 8)])
def test_topk_bit_exact(moe, ro, dev, tokens, experts, k):
    g = torch.Generator().manual_seed(tokens + experts)
    s = torch.rand(tokens, experts, generator=g)
    s[::7, 1] = s[::7, 0]                                       # ties
    if experts > 4:
        s[::11, 3] = float("-inf")
        s[::13, 2] = float("nan")
    got = moe.topk(s.to(dev), k).cpu().numpy()
    assert np.array_equal(got, ro.topk_ref(s.numpy(), k))


def test_topk_rows_of_minus_inf(moe, ro, dev):
    s = torch.full((3, 6), float("-inf"))
    s[1, 4] = 2.0
    got = moe.topk(s.to(dev), 3).cpu().numpy()
    assert np.array_equal(got, ro.topk_ref(s.numpy(), 3))
    assert got[0].tolist() == [-1, -1, -1] and got[1].tolist() == [4, -1, -1]


@pytest.mark.parametrize("experts", [8, 32, 64, 100])          # the wave-per-token kernel (<= 64 experts) and the per-thread scan
def test_topk_signed_zeros_compare_equal(moe, ro, dev, experts):
    """+0.0 and -0.0 are equal scores (the reference compares with __hgt, 2-amd-moe/amd-moe-submission.py:32-56):
    among them the lowest index wins, whatever their sign bits, in both kernels."""
    s = torch.full((6, experts), -1.0)
    s[0, 5], s[0, 2] = -0.0, 0.0                                 # +0 at the lower index
    s[1, 2], s[1, 5] = -0.0, 0.0                                 # -0 at the lower index: still index 2 first
    s[2, 1], s[2, 3], s[2, 6] = 0.0, -0.0, 0.0
    s[3, :] = -0.0
    s[4, :] = 0.0
    s[4, 1::2] = -0.0
    s[5, 7], s[5, 0], s[5, 4] = 1.0, -0.0, 0.0
    got = moe.topk(s.to(dev), 4).cpu().numpy()
    assert np.array_equal(got, ro.topk_ref(s.numpy(), 4))
    assert got[0, :2].tolist() == [2, 5] and got[1, :2].tolist() == [2, 5] and got[2, :3].tolist() == [1, 3, 6]
    assert got[3].tolist() == [0, 1, 2, 3] and got[4].tolist() == [0, 1, 2, 3] and got[5, :3].tolist() == [7, 0, 4]


def test_route_into_caller_tensors_and_rows_beyond_the_total(moe, ro, dev):
    """`out=`: the three outputs of an earlier call are filled again, no allocation; rows beyond
    row_offsets[E] (choices outside [0, E)) read -1 although the tensors held other values before."""
    rng = np.random.default_rng(5)
    tokens, experts, k = 700, 16, 4
    top = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
    first = moe.route(torch.from_numpy(top).to(dev), experts)
    ptrs = [t.data_ptr() for t in first]
    top2 = top.copy()
    top2[::3, 1] = experts + 5                                   # ignored choices: fewer rows than tokens * k
    top2[::5, 2] = -1
    for t in first:
        t.fill_(12345)
    again = moe.route(torch.from_numpy(top2).to(dev), experts, out=first)
    assert [t.data_ptr() for t in again] == ptrs
    wo, wm, ws = ro.route_ref(top2, experts)
    assert np.array_equal(again[0].cpu().numpy(), wo) and np.array_equal(again[1].cpu().numpy(), wm) and np.array_equal(again[2].cpu().numpy(), ws)
    assert int(wo[-1]) < tokens * k and bool((again[1][int(wo[-1]):] == -1).all())
    idx = moe.topk(torch.rand(tokens, experts, device=dev), k)
    assert moe.topk(torch.rand(tokens, experts, device=dev), k, out=idx).data_ptr() == idx.data_ptr()
    with pytest.raises(ValueError):
        moe.route(torch.from_numpy(top).to(dev), experts, out=(first[0], first[1][:-1], first[2]))


@pytest.mark.parametrize("tokens,experts,k", [(300, 8, 3), (4096, 32, 8), (255, 1, 1), (1025, 1000, 4), (5, 32, 8), (20000, 16, 2)])
def test_route_bit_exact(moe, ro, dev, tokens, experts, k):
    rng = np.random.default_rng(tokens * 31 + experts)
    top = np.stack([rng.permutation(experts)[:k] for _ in range(tokens)]).astype(np.int32)
    row_offsets, row_map, slot_of = moe.route(torch.from_numpy(top).to(dev), experts)
    wo, wm, ws = ro.route_ref(top, experts)
    assert np.array_equal(row_offsets.cpu().numpy(), wo)
    assert np.array_equal(row_map.cpu().numpy(), wm)
    assert np.array_equal(slot_of.cpu().numpy(), ws)


def test_route_ignores_bad_and_repeated_entries(moe, ro, dev):
    rng = np.random.default_rng(9)
    top = np.stack([rng.permutation(6)[:3] for _ in range(700)]).astype(np.int32)
    top[3, 1] = -1
    top[4, 2] = 6
    top[5, 1] = top[5, 0]
    top[300, 2] = top[300, 0]
    row_offsets, row_map, slot_of = moe.route(torch.from_numpy(top).to(dev), 6)
    wo, wm, ws = ro.route_ref(top, 6)
    assert np.array_equal(row_offsets.cpu().numpy(), wo)
    assert np.array_equal(row_map.cpu().numpy(), wm)
    assert np.array_equal(slot_of.cpu().numpy(), ws)
    assert int(row_offsets[-1]) == 700 * 3 - 4


def test_route_is_deterministic_and_empty_experts(moe, dev):
    top = torch.tensor([[0, 2], [2, 0], [0, 2]] * 100, dtype=torch.int32, device=dev)     # expert 1, 3 unused
    a = moe.route(top, 4)
    b = moe.route(top, 4)
    for x, y in zip(a, b):
        assert torch.equal(x, y)
    assert a[0].tolist() == [0, 300, 300, 600, 600]


def test_scores_to_grouped_gemm_chain(moe, quant, pkg, oracle, ro, dev):
    """router scores -> top-k -> route -> quantise-with-gather -> grouped GEMM, against the oracle's
    grouped product of host-permuted, host-quantised operands."""
    tokens, experts, k, n, kk = 384, 8, 3, 256, 512
    g = torch.Generator().manual_seed(31)
    x = torch.randn(tokens, kk, generator=g)
    scores = torch.rand(tokens, experts, generator=g)
    ws = [torch.randn(n, kk, generator=g) * 0.02 for _ in range(experts)]
    # device chain
    top = moe.topk(scores.to(dev), k)
    row_offsets, row_map, slot_of = moe.route(top, experts)
    a, a_scale = quant.quantize_a(x.to(dev), row_map)
    b_store = torch.empty(experts, kk, n, dtype=torch.float8_e4m3fn, device=dev)
    bs_store = torch.empty(experts, kk // 128, n // 128, dtype=torch.float32, device=dev)
    for e in range(experts):
        qb, sb = quant.quantize_b(ws[e].to(dev))
        b_store[e] = qb.t()
        bs_store[e] = sb.t()
    rows = tokens * k
    c = torch.zeros(rows, n, dtype=torch.bfloat16, device=dev)
    out = pkg.grouped_kernel((a, b_store.transpose(1, 2), a_scale, bs_store.transpose(1, 2), row_offsets, c))
    # host chain
    top_ref = ro.topk_ref(scores.numpy(), k)
    wo, wm, _ = ro.route_ref(top_ref, experts)
    assert np.array_equal(row_offsets.cpu().numpy(), wo) and np.array_equal(row_map.cpu().numpy(), wm)
    ha, has = pkg.inputs.quantize_a(x[torch.from_numpy(wm).long()])
    hb = torch.empty(experts, kk, n, dtype=torch.float8_e4m3fn)
    hbs = torch.empty(experts, kk // 128, n // 128, dtype=torch.float32)
    for e in range(experts):
        qb, sb = pkg.inputs.quantize_b(ws[e])
        hb[e] = qb.t()
        hbs[e] = sb.t()
    ref = oracle.ref_grouped((ha, hb.transpose(1, 2), has, hbs.transpose(1, 2), torch.from_numpy(wo),
                              torch.zeros(rows, n, dtype=torch.bfloat16)))
    ok, nbad, maxerr = oracle.within_tolerance(out.cpu(), ref, 2e-2, 1e-3)
    assert ok, "%d outside the bar, max err %g" % (nbad, maxerr)


def test_routing_calls_that_overlap_on_two_streams(pkg, dev):
    """moe.route keeps one scratch buffer per device and stream: two different routing problems issued
    alternately on two streams, without waiting in between, each give their serial result (one buffer shared by
    both streams would let one call's count tables overwrite the other's)."""
    moe = importlib.import_module("amd-developer-challenge-2025_amd.moe")
    probs = []
    for tokens, experts, k, seed in ((4096, 32, 8, 1), (3000, 48, 6, 2)):
        g = torch.Generator(device=dev).manual_seed(seed)
        idx = moe.topk(torch.rand(tokens, experts, generator=g, device=dev), k)
        serial = tuple(t.clone() for t in moe.route(idx, experts))
        probs.append((idx, experts, serial))
    torch.cuda.synchronize()
    streams = [torch.cuda.Stream(), torch.cuda.Stream()]
    outs = [[], []]
    for rep in range(20):
        for i, (idx, experts, _) in enumerate(probs):
            with torch.cuda.stream(streams[i]):
                outs[i].append(moe.route(idx, experts))
    torch.cuda.synchronize()
    for i, (_, _, serial) in enumerate(probs):
        for rep, got in enumerate(outs[i]):
            for name, x, y in zip(("row_offsets", "row_map", "slot_of"), got, serial):
                assert torch.equal(x, y), "stream %d call %d: %s" % (i, rep, name)
