"""Host logic: the block quantisers and the synthetic-input factory.  CPU only."""
import pytest
import torch


def test_quantize_a_layout_and_invariants(pkg, oracle):
    g = torch.Generator().manual_seed(0)
    x = torch.randn(48, 384, generator=g) * 3
    x[5, 128:256] = 0                                   # an all-zero block
    a, a_scale = pkg.inputs.quantize_a(x)
    assert a.dtype == torch.float8_e4m3fn and a.shape == (48, 384) and a.stride() == (1, 48)
    assert a_scale.dtype == torch.float32 and a_scale.shape == (48, 3) and a_scale.stride() == (1, 48)
    q = a.float()
    assert q.abs().max() <= 448 and not q.isnan().any()
    deq = oracle.dequant_a(a, a_scale)
    blocks = x.reshape(48, 3, 128)
    amax = blocks.abs().amax(2)
    # the block maximum maps to +-448 exactly, so dequantising recovers amax
    assert torch.allclose(deq.reshape(48, 3, 128).abs().amax(2), amax, rtol=1e-6, atol=0)
    # e4m3 has 3 mantissa bits: relative error <= 2^-4 for values in the normal range
    normal = x.abs() > (amax / 448 * 2 ** -6).repeat_interleave(128, 1)
    rel = ((deq - x).abs() / x.abs().clamp_min(1e-30))[normal]
    assert rel.max() <= 2 ** -4 + 1e-6
    assert torch.equal(deq[5, 128:256], torch.zeros(128)) and a_scale[5, 1] > 0
    # idempotence: quantising the dequantised tensor reproduces the codes
    a2, s2 = pkg.inputs.quantize_a(deq)
    assert torch.equal(a2.view(torch.uint8), a.view(torch.uint8)) and torch.allclose(s2, a_scale, rtol=1e-6)


def test_quantize_b_partial_last_block(pkg, oracle):
    g = torch.Generator().manual_seed(1)
    w = torch.randn(192, 256, generator=g) * 0.02
    b, b_scale = pkg.inputs.quantize_b(w)
    assert b.shape == (192, 256) and b.stride() == (1, 192)
    assert b_scale.shape == (2, 2) and b_scale.stride() == (1, 2)
    assert torch.allclose(b_scale[1, 0], w[128:192, :128].abs().max() / 448)
    deq = oracle.dequant_b(b, b_scale)
    assert ((deq - w).abs() <= w.abs() * 2 ** -4 + b_scale.max() * 2 ** -9 + 1e-12).all()


def test_clamp_guards_against_cast_overflow(pkg):
    x = torch.full((1, 128), 1.0); x[0, 0] = 1e30      # ratio far beyond 448 for the small entries is fine
    a, s = pkg.inputs.quantize_a(x)
    assert not a.float().isnan().any() and a.float()[0, 0] == 448


@pytest.mark.parametrize("idx", [0, 2, 3])
def test_dense_configs_shapes(pkg, idx):
    cfg = pkg.inputs.CONFIGS[idx]
    a, b, a_scale, b_scale, c = pkg.inputs.make_dense(cfg, m=min(cfg.m, 64), n=min(cfg.n, 272), k=256)
    m, n = a.shape[0], b.shape[0]
    assert a.stride() == (1, m) and b.stride() == (1, n)
    assert a_scale.shape == (m, 2) and a_scale.stride() == (1, m)
    nb = (n + 127) // 128
    assert b_scale.shape == (nb, 2) and b_scale.stride() == (1, nb)
    assert c.shape == (m, n) and c.is_contiguous() and c.dtype == torch.bfloat16
    # same seed, same bytes
    a2 = pkg.inputs.make_dense(cfg, m=min(cfg.m, 64), n=min(cfg.n, 272), k=256)[0]
    assert torch.equal(a.view(torch.uint8), a2.view(torch.uint8))


def test_config_table_matches_the_published_sizes(pkg):
    sizes = [(c.m, c.n, c.k, c.experts, c.topk) for c in pkg.inputs.CONFIGS]
    assert sizes == [(256, 512, 1024, 0, 0), (4096, 4096, 4096, 0, 0), (4096, 2112, 7168, 0, 0),
                     (64, 18432, 7168, 0, 0), (4096, 4096, 7168, 32, 8)]


def test_grouped_inputs_routing_and_layout(pkg, oracle):
    cfg = pkg.inputs.CONFIGS[4]
    tokens, e, tk, n, k = 40, 8, 3, 144, 256
    a, b, a_scale, b_scale, row_offsets, c = pkg.inputs.make_grouped(cfg, tokens=tokens, n=n, k=k, experts=e, topk=tk)
    rows = tokens * tk
    assert a.shape == (rows, k) and a.stride() == (1, rows) and a_scale.stride() == (1, rows)
    assert b.shape == (e, n, k) and b.stride() == (n * k, 1, n)
    assert b_scale.shape == (e, 2, 2) and b_scale.stride() == (4, 1, 2)
    assert row_offsets.dtype == torch.int32 and row_offsets[0] == 0 and row_offsets[-1] == rows
    assert (row_offsets[1:] >= row_offsets[:-1]).all() and c.shape == (rows, n)
    # every token appears exactly topk times, in distinct experts
    x = torch.randn(tokens, k, generator=torch.Generator().manual_seed(cfg.seed))
    qa, _ = pkg.inputs.quantize_a(x)
    rows_u8 = a.view(torch.uint8)
    counts = torch.zeros(tokens, dtype=torch.int64)
    for t in range(tokens):
        hits = (rows_u8 == qa.view(torch.uint8)[t]).all(1).nonzero().flatten()
        counts[t] = hits.numel()
        experts = torch.bucketize(hits, row_offsets[1:].long(), right=True)
        assert experts.unique().numel() == hits.numel()
    assert (counts == tk).all()
