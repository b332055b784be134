"""fnuz operands and the 18 leaderboard shapes on a real MI355X.  Run with:  python -u -m pytest tests -m gpu"""
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
def harness(pkg):
    return importlib.import_module("amd-developer-challenge-2025_amd.harness")


@pytest.fixture(scope="module")
def qo():
    return importlib.import_module("oracle.quant_oracle")


def test_fnuz_to_fn_kernel_bit_exact(harness, qo, dev):
    rng = np.random.default_rng(1)
    codes = np.concatenate([np.arange(256, dtype=np.uint8), rng.integers(0, 256, 100_003, dtype=np.uint8)])
    t = torch.from_numpy(codes).to(dev).view(torch.float8_e4m3fnuz)
    got = harness.fnuz_to_fn(t).view(torch.uint8).cpu().numpy()
    assert np.array_equal(got, qo.fnuz_to_fn_ref(codes))


def test_custom_kernel_fnuz(harness, pkg, oracle, qo, dev):
    """operands quantised for the reference's hardware (max 240, fnuz codes): same scales, same result
    as the oracle on the fnuz-decoded values"""
    m, n, k = 256, 384, 512
    g = torch.Generator().manual_seed(3)
    x, w = torch.randn(m, k, generator=g), torch.randn(n, k, generator=g) * 0.02

    def quant_fnuz(t, block_rows):
        rows = t.shape[0]
        tb = t.reshape(rows // block_rows, block_rows, k // 128, 128)
        scale = (tb.abs().amax(dim=(1, 3)) / 240.0).clamp_min(1e-12)
        q = (tb / scale[:, None, :, None]).clamp(-240, 240).reshape(rows, k).to(torch.float8_e4m3fnuz)
        return q.t().contiguous().t(), scale.repeat_interleave(1, 0).t().contiguous().t()

    a, a_scale = quant_fnuz(x, 1)
    b, b_scale = quant_fnuz(w, 128)
    c = torch.zeros(m, n, dtype=torch.bfloat16, device=dev)
    out = harness.custom_kernel_fnuz((a.to(dev), b.to(dev), a_scale.to(dev), b_scale.to(dev), c))
    assert out is c
    a32 = a.float() * a_scale.repeat_interleave(128, 1)
    b32 = b.float() * b_scale.repeat_interleave(128, 0).repeat_interleave(128, 1)
    ref = (a32 @ b32.t()).to(torch.bfloat16)
    ok, nbad, maxerr = oracle.within_tolerance(out.cpu(), ref, RTOL, ATOL)
    assert ok, "%d outside the bar, max err %g" % (nbad, maxerr)


@pytest.mark.parametrize("case", range(18))
def test_leaderboard_shape(harness, pkg, oracle, dev, case):
    """Each of the 18 shapes of the upstream benchmark (README.md:65-82), full size.  Inputs are
    N(0,1) x N(0,1): outputs are large against atol, so the FP8 matrix cores' truncated accumulation
    shows on a few near-zero outputs; as for configurations 1 and 2, every element beyond the strict bar
    must be bit-identical to the instruction-level model."""
    s = harness.LEADERBOARD_SHAPES[case]
    data = harness.generate_input(s["m"], s["n"], s["k"], s["seed"], dev)
    out = pkg.custom_kernel(data)
    cpu = tuple(t.cpu() for t in data)
    ref = oracle.ref_kernel(cpu)
    ok, nstrict, nunexplained = oracle.parity_report(out.cpu(), ref, cpu, pkg.plan(s["m"], s["n"], s["k"]).split_k, RTOL, ATOL)
    print("%s: %d elements beyond the strict bar, %d not reproduced by the instruction model" % (s, nstrict, nunexplained))
    assert ok, "%s: %d strict violations, %d not reproduced by the instruction model" % (s, nstrict, nunexplained)
