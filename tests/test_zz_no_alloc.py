"""fp8bs_gemm_noalloc (the entry point that allocates nothing: K-split partial planes in a device array that is
part of the library) against fp8bs_gemm with a caller workspace, through the C ABI.
Run with:  python -u -m pytest tests -m gpu"""
import pytest
import torch

pytestmark = pytest.mark.gpu
SCRATCH_LIMIT = 32 * 1024 * 1024


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    return torch.device("cuda:0")


def _call_both(pkg, dev, cfg, m, n, k):
    lib = pkg._lib.load()
    cpu = pkg.inputs.make_dense(cfg, m=m, n=n, k=k)
    a, b, a_scale, b_scale, _ = (t.to(dev) for t in cpu)
    plan = pkg.plan(m, n, k)
    ws = torch.empty(max(int(plan.workspace_bytes), 16), dtype=torch.uint8, device=dev)
    want = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    got = torch.full((m, n), float("nan"), dtype=torch.bfloat16, device=dev)
    stream = torch.cuda.current_stream().cuda_stream
    pkg._lib.check(lib.fp8bs_gemm(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), want.data_ptr(),
                                  ws.data_ptr(), ws.numel(), m, n, k, stream))
    pkg._lib.check(lib.fp8bs_gemm_noalloc(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), got.data_ptr(),
                                          m, n, k, stream))
    torch.cuda.synchronize()
    return plan, want, got


def test_two_calls_in_a_row_the_second_smaller(pkg, dev):
    """both shapes are planned with a K split, so the built-in array carries the partial planes; the second call
    finds the first call's planes in it and must not be disturbed by them"""
    cfg = pkg.inputs.CONFIGS[3]                                   # skinny-M distributions
    first = second = None
    for m, n, k in ((64, 18432, 7168), (32, 2048, 4096)):
        plan, want, got = _call_both(pkg, dev, cfg, m, n, k)
        assert plan.split_k > 1 and 0 < plan.workspace_bytes <= SCRATCH_LIMIT
        assert not torch.isnan(got.float()).any()
        assert torch.equal(got.view(torch.int16), want.view(torch.int16)), "%dx%dx%d" % (m, n, k)
        first, second = second, got
    assert first is not None and second is not None


def test_without_a_split_and_beyond_the_limit(pkg, dev):
    lib = pkg._lib.load()
    plan, want, got = _call_both(pkg, dev, pkg.inputs.CONFIGS[0], 256, 512, 1024)          # no K split planned: the array is not touched
    assert plan.split_k == 1 and torch.equal(got.view(torch.int16), want.view(torch.int16))
    # a shape whose planned K split needs more partial-plane bytes than the array holds is refused, nothing is launched
    m, n, k = 2048, 2048, 32768
    plan = pkg.plan(m, n, k)
    assert plan.split_k > 1 and plan.workspace_bytes > SCRATCH_LIMIT
    a = torch.zeros(k, m, dtype=torch.uint8, device=dev)
    b = torch.zeros(k, n, dtype=torch.uint8, device=dev)
    a_scale = torch.ones(k // 128, m, device=dev)
    b_scale = torch.ones(k // 128, n // 128, device=dev)
    c = torch.full((m, n), 7.0, dtype=torch.bfloat16, device=dev)
    st = lib.fp8bs_gemm_noalloc(a.data_ptr(), b.data_ptr(), a_scale.data_ptr(), b_scale.data_ptr(), c.data_ptr(), m, n, k,
                                torch.cuda.current_stream().cuda_stream)
    torch.cuda.synchronize()
    assert st == 8 and b"scratch" in lib.fp8bs_strerror(st)
    assert bool((c == 7.0).all())


def test_under_graph_capture(pkg, dev):
    """what the entry point is for: a call with a K split captured into a HIP graph (no allocation, no workspace
    argument) and replayed with other inputs, eager work and synchronisation in between - every replay equals the
    eager result of fp8bs_gemm bit for bit"""
    lib = pkg._lib.load()
    cfg = pkg.inputs.CONFIGS[3]
    m, n, k = 64, 2304, 2048
    assert pkg.plan(m, n, k).split_k > 1
    sets = [tuple(t.to(dev) for t in pkg.inputs.make_dense(pkg.inputs.Config("capture", m, n, k, cfg.a_outlier_frac, cfg.a_outlier_mul, cfg.b_std, 0, 0, s)))
            for s in (1, 2)]
    eager = [pkg.custom_kernel(tuple(s[:4]) + (torch.empty_like(s[4]),)).clone() for s in sets]
    static = tuple(t.clone() for t in sets[0])

    def call():
        pkg._lib.check(lib.fp8bs_gemm_noalloc(static[0].data_ptr(), static[1].data_ptr(), static[2].data_ptr(), static[3].data_ptr(),
                                              static[4].data_ptr(), m, n, k, torch.cuda.current_stream().cuda_stream))
    call()                                                        # outside capture: the array's address is looked up here
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        call()
    for rep in range(4):
        src, want = sets[rep % 2], eager[rep % 2]
        for dst, s in zip(static[:4], src[:4]):
            dst.copy_(s)
        static[4].fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static[4].view(torch.int16), want.view(torch.int16)), "replay %d" % rep
        pkg.custom_kernel(sets[(rep + 1) % 2])                    # eager work between replays
        torch.cuda.synchronize()
