"""Pins oracle/route_oracle.py without the reference (which ships no tests): torch.topk, a tie fixture,
the independent torch derivation in inputs.make_grouped, and invariants."""
import importlib

import numpy as np
import pytest
import torch


@pytest.fixture(scope="module")
def ro():
    return importlib.import_module("oracle.route_oracle")


def test_topk_matches_torch_on_distinct_scores(ro):
    g = torch.Generator().manual_seed(3)
    s = torch.rand(200, 32, generator=g)                      # distinct with probability ~1
    assert all(len(set(r.tolist())) == 32 for r in s)
    for k in (1, 4, 8):
        want = s.topk(k, dim=1).indices.numpy().astype(np.int32)
        assert np.array_equal(ro.topk_ref(s.numpy(), k), want)


def test_topk_tie_fixture_and_special_values(ro):
    s = np.array([[1, 3, 3, 2, 3, 0],                         # ties: lowest index first
                  [5, 5, 5, 5, 5, 5],
                  [-np.inf, 1, np.nan, -np.inf, 0, np.nan]], dtype=np.float32)
    got = ro.topk_ref(s, 4)
    assert got[0].tolist() == [1, 2, 4, 3]
    assert got[1].tolist() == [0, 1, 2, 3]
    assert got[2].tolist() == [1, 4, -1, -1]                  # -inf and NaN are never selected
    sel = np.take_along_axis(s[:2], got[:2], axis=1)
    assert np.all(np.diff(sel, axis=1) <= 0)                  # best first
    # +0.0 and -0.0 are equal scores: the lowest index wins whatever the sign bits
    z = np.array([[-1, -1, 0.0, -1, -1, -0.0], [-1, -1, -0.0, -1, -1, 0.0], [-0.0, 0.0, -0.0, 0.0, 1.0, -1]], dtype=np.float32)
    assert ro.topk_ref(z, 2)[0].tolist() == [2, 5] and ro.topk_ref(z, 2)[1].tolist() == [2, 5]
    assert ro.topk_ref(z, 4)[2].tolist() == [4, 0, 1, 2]


def test_route_matches_the_independent_torch_derivation(ro, pkg):
    cfg = pkg.inputs.CONFIGS[4]
    tokens, experts, topk = 300, 8, 3
    gen = torch.Generator().manual_seed(cfg.seed)
    torch.randn(tokens, 128, generator=gen)                    # same stream position as make_grouped
    route = torch.rand(tokens, experts, generator=gen).topk(topk, dim=1).indices
    data = pkg.inputs.make_grouped(cfg, tokens=tokens, n=128, k=128, experts=experts, topk=topk)
    row_offsets, row_map, slot_of = ro.route_ref(route.numpy(), experts)
    assert np.array_equal(row_offsets, data[4].numpy())
    # make_grouped's row order: sort by expert, then token id
    token_ids = torch.arange(tokens).repeat_interleave(topk)
    order = torch.sort(route.reshape(-1) * tokens + token_ids).indices
    assert np.array_equal(row_map, token_ids[order].numpy())


def test_route_invariants(ro):
    rng = np.random.default_rng(5)
    tokens, experts, topk = 257, 5, 2
    top = np.stack([rng.permutation(experts)[:topk] for _ in range(tokens)]).astype(np.int32)
    top[3, 1] = -1                                             # ignored
    top[4, 1] = experts                                        # ignored
    top[5, 1] = top[5, 0]                                      # repeated expert: one row
    row_offsets, row_map, slot_of = ro.route_ref(top, experts)
    total = row_offsets[-1]
    assert total == tokens * topk - 3 and np.all(row_map[total:] == -1)
    for e in range(experts):
        rows = row_map[row_offsets[e]:row_offsets[e + 1]]
        assert np.all(np.diff(rows) > 0)                       # by token id, no token twice
        assert all(e in top[t] for t in rows)
    assert slot_of[3, 1] == -1 and slot_of[4, 1] == -1 and slot_of[5, 1] == -1
    valid = slot_of >= 0
    assert np.array_equal(row_map[slot_of[valid]], np.nonzero(valid)[0])
    hist = np.bincount(top[valid], minlength=experts)
    assert np.array_equal(np.diff(row_offsets), hist)
