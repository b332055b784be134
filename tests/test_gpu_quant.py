"""Parity of the HIP block quantisers (through the C ABI) with oracle/quant_oracle.py on a real MI355X.

Byte and scale outputs are compared bit for bit.  Run with:  python -u -m pytest tests -m gpu
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
def qo():
    return importlib.import_module("oracle.quant_oracle")


@pytest.fixture(scope="module")
def quant(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.quant")


def _store(q, s):
    """K-major views -> storage-order numpy arrays (what the C ABI wrote)."""
    return q.t().contiguous().view(torch.uint8).cpu().numpy(), s.t().contiguous().cpu().numpy()


def _draw(seed, rows, k, std=1.0):
    g = torch.Generator().manual_seed(seed)
    x = torch.randn(rows, k, generator=g) * std
    x = torch.where(torch.rand(rows, k, generator=g) < 0.01, x * 20, x)
    if rows > 2 and k >= 256:
        x[1, :128] = 0
        x[2, 128:256] *= 1e-20
    return x


def test_conversion_on_every_critical_value(quant, qo, oracle, dev):
    """Blocks whose maximum is exactly 448 have scale 1, so the kernel's fp32 -> e4m3fn conversion is
    checked directly on every representable value, every rounding midpoint and their fp32 neighbours."""
    table = oracle.e4m3fn_table().astype(np.float64)
    pos = np.sort(table[:127])
    mids = (pos[:-1] + pos[1:]) / 2
    crit = np.concatenate([pos, mids]).astype(np.float32)
    crit = np.concatenate([crit, np.nextafter(crit, np.float32(np.inf)), np.nextafter(crit, np.float32(-np.inf))])
    crit = crit[(crit >= 0) & (crit <= 448)]
    crit = np.concatenate([crit, -crit])
    nblk = (crit.size + 126) // 127
    x = np.zeros((1, nblk * 128), dtype=np.float32)
    for b in range(nblk):
        chunk = crit[b * 127:(b + 1) * 127]
        x[0, b * 128] = 448.0
        x[0, b * 128 + 1:b * 128 + 1 + chunk.size] = chunk
    x = np.repeat(x, 16, axis=0)
    q, s = _store(*quant.quantize_a(torch.from_numpy(x).to(dev)))
    assert np.all(s == 1.0)
    want, _ = qo.quantize_a_ref(x)
    assert np.array_equal(q, want)
    assert np.array_equal(q[:, 0], torch.from_numpy(x[0]).to(torch.float8_e4m3fn).view(torch.uint8).numpy())


@pytest.mark.parametrize("rows,k", [(128, 128), (130, 384), (16, 1024), (257, 256), (1, 128)])
def test_quantize_a_fp32_bit_exact(quant, qo, dev, rows, k):
    x = _draw(100 + rows, rows, k)
    q, s = _store(*quant.quantize_a(x.to(dev)))
    wq, ws = qo.quantize_a_ref(x.numpy())
    assert np.array_equal(s, ws)
    assert np.array_equal(q, wq)


def test_quantize_a_bf16_and_row_stride(quant, qo, dev):
    x = _draw(5, 192, 512).to(torch.bfloat16)
    q, s = _store(*quant.quantize_a(x.to(dev)))
    wq, ws = qo.quantize_a_ref(x.float().numpy())
    assert np.array_equal(s, ws) and np.array_equal(q, wq)
    # a K slice of a wider matrix: rows 640 elements apart
    wide = _draw(6, 96, 640)
    q, s = _store(*quant.quantize_a(wide.to(dev)[:, 128:512]))
    wq, ws = qo.quantize_a_ref(wide[:, 128:512].contiguous().numpy())
    assert np.array_equal(s, ws) and np.array_equal(q, wq)


def test_quantize_a_returns_the_contract_layout(quant, dev):
    a, a_scale = quant.quantize_a(_draw(8, 64, 256).to(dev))
    assert a.dtype == torch.float8_e4m3fn and a.shape == (64, 256) and a.stride() == (1, 64)
    assert a_scale.dtype == torch.float32 and a_scale.shape == (64, 2) and a_scale.stride() == (1, 64)


def test_quantize_a_row_map(quant, qo, dev):
    x = _draw(9, 50, 256)
    row_map = torch.tensor([7, 7, 0, 49, 3, 12, 12, 12, 30] * 20, dtype=torch.int32)
    q, s = _store(*quant.quantize_a(x.to(dev), row_map.to(dev)))
    wq, ws = qo.quantize_a_ref(x.numpy(), row_map.numpy())
    assert q.shape == (256, 180)
    assert np.array_equal(s, ws) and np.array_equal(q, wq)


@pytest.mark.parametrize("tokens,rows,k", [(64, 256, 128),          # 16 k rows per workgroup
                                           (4096, 8192 + 4, 256),   # two row chunks, the second 4 rows
                                           (4100, 512, 128),        # 8 k rows per workgroup
                                           (8200, 256, 128),        # 4 k rows per workgroup
                                           (50, 180, 256),          # tokens not a multiple of 4: byte-wise kernel
                                           (64, 90, 128),           # rows not a multiple of 4: byte-wise kernel
                                           (4, 4, 128)])
def test_gather_a_bit_exact(quant, qo, dev, tokens, rows, k):
    g = torch.Generator().manual_seed(tokens * 7 + rows)
    q_src = torch.randint(0, 256, (k, tokens), dtype=torch.uint8, generator=g)
    s_src = torch.rand(k // 128, tokens, generator=g) + 0.01
    row_map = torch.randint(0, tokens, (rows,), dtype=torch.int32, generator=g)
    row_map[::17] = -1
    row_map[3::29] = tokens
    row_map[-1] = tokens - 1
    a = q_src.to(dev).view(torch.float8_e4m3fn).t()
    q, s = _store(*quant.gather_a(a, s_src.to(dev).t(), row_map.to(dev)))
    wq, ws = qo.gather_a_ref(q_src.numpy(), s_src.numpy(), row_map.numpy())
    assert q.shape == (k, rows) and s.shape == (k // 128, rows)
    assert np.array_equal(q, wq) and np.array_equal(s, ws)


def test_gather_after_quantise_equals_fused_gather(quant, dev):
    """Full MoE size: 4096 tokens routed 8 ways, K = 7168; both routes to the same 32768-row operand."""
    g = torch.Generator().manual_seed(77)
    x = (torch.randn(4096, 7168, generator=g) * 3).to(dev)
    row_map = torch.randint(0, 4096, (32768,), dtype=torch.int32, generator=g).to(dev)
    a1, s1 = quant.quantize_a(x, row_map, fused=True)
    a2, s2 = quant.gather_a(*quant.quantize_a(x), row_map)
    assert a2.shape == a1.shape and a2.stride() == a1.stride() and s2.stride() == s1.stride()
    assert torch.equal(a1.view(torch.uint8), a2.view(torch.uint8)) and torch.equal(s1, s2)
    a3, s3 = quant.quantize_a(x, row_map)                        # more rows than tokens: the two-kernel route by default
    assert torch.equal(a1.view(torch.uint8), a3.view(torch.uint8)) and torch.equal(s1, s3) and a3.stride() == a1.stride()


def test_gather_a_argument_errors(quant, dev):
    a, s = quant.quantize_a(torch.randn(8, 128, device=dev))
    with pytest.raises(ValueError):
        quant.gather_a(a, s, torch.zeros(4, dtype=torch.int64, device=dev))
    with pytest.raises(ValueError):
        quant.gather_a(a, s[:, :0], torch.zeros(4, dtype=torch.int32, device=dev))
    with pytest.raises(TypeError):
        quant.gather_a(a.view(torch.uint8), s, torch.zeros(4, dtype=torch.int32, device=dev))
    q0, s0 = quant.gather_a(a, s, torch.zeros(0, dtype=torch.int32, device=dev))
    assert q0.shape == (0, 128) and s0.shape == (0, 1)


@pytest.mark.parametrize("n,k,dtype", [(256, 256, torch.float32), (2112, 512, torch.float32), (200, 256, torch.float32),
                                       (384, 384, torch.bfloat16)])
def test_quantize_b_bit_exact(quant, qo, dev, n, k, dtype):
    w = (_draw(200 + n, n, k, std=0.02)).to(dtype)
    b, b_scale = quant.quantize_b(w.to(dev))
    nb = (n + 127) // 128
    assert b.shape == (n, k) and b.stride() == (1, n) and b_scale.shape == (nb, k // 128) and b_scale.stride() == (1, nb)
    q, s = _store(b, b_scale)
    wq, ws = qo.quantize_b_ref(w.float().numpy())
    assert np.array_equal(s, ws) and np.array_equal(q, wq)


def test_full_size_cfg3_activations(quant, qo, dev):
    """4096 x 7168 fp32, the activations of configuration 3 (1 % outliers x 20)."""
    x = _draw(20253, 4096, 7168)
    q, s = _store(*quant.quantize_a(x.to(dev)))
    wq, ws = qo.quantize_a_ref(x.numpy())
    assert np.array_equal(s, ws)
    assert np.array_equal(q, wq)


def test_gpu_quantised_operands_feed_the_gemm(quant, pkg, oracle, dev):
    """quantise on the GPU -> custom_kernel == host-quantised operands -> custom_kernel, bit for bit,
    and both within the bar of the oracle."""
    g = torch.Generator().manual_seed(77)
    x, w = torch.randn(256, 512, generator=g), torch.randn(384, 512, generator=g) * 0.02
    a, a_scale = quant.quantize_a(x.to(dev))
    b, b_scale = quant.quantize_b(w.to(dev))
    c = torch.zeros(256, 384, dtype=torch.bfloat16, device=dev)
    out = pkg.custom_kernel((a, b, a_scale, b_scale, c))
    ha, has = pkg.inputs.quantize_a(x)
    hb, hbs = pkg.inputs.quantize_b(w)
    c2 = torch.zeros(256, 384, dtype=torch.bfloat16, device=dev)
    out2 = pkg.custom_kernel((ha.to(dev), hb.to(dev), has.to(dev), hbs.to(dev), c2))
    assert torch.equal(out.view(torch.int16), out2.view(torch.int16))
    ref = oracle.ref_kernel((ha, hb, has, hbs, torch.zeros(256, 384, dtype=torch.bfloat16)))
    ok, nbad, maxerr = oracle.within_tolerance(out.cpu(), ref, 2e-2, 1e-3)
    assert ok, "%d outside the bar, max err %g" % (nbad, maxerr)


def test_quantiser_argument_errors(quant, dev):
    with pytest.raises(ValueError):
        quant.quantize_a(torch.zeros(16, 100, device=dev))
    with pytest.raises(TypeError):
        quant.quantize_a(torch.zeros(16, 128, device=dev, dtype=torch.float16))
    with pytest.raises(ValueError):
        quant.quantize_a(torch.zeros(128, 16, device=dev).t())
    a, s = quant.quantize_a(torch.zeros(0, 128, device=dev))
    assert a.shape == (0, 128) and s.shape == (0, 1)
