"""K blocks, not tiles, dealt to the workgroups (fp8bs_gemm_ex with split_k < 0): one launch, partial tiles
exchanged through the workspace, summed by the tile's owner in a fixed order.

Held to the same bar as every other path (|out - ref| <= 1e-3 + 2e-2*|ref| on every element against the
oracle), and - because the order of the sums is fixed by the shape, the tile and the number of workgroups -
to the instruction-level model bit for bit.  The reference splits K with a second kernel that merges the
planes (1-amd-fp8-mm/amd-fp8-mm-submission.py:371-511); this is the same work in one launch.
"""
import ctypes
import importlib
import os
import subprocess
import sys

import numpy as np
import pytest
import torch

pytestmark = pytest.mark.gpu

RTOL, ATOL = 2e-2, 1e-3
ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))

# variant -> (tile rows, tile columns, workgroups that fit one CU)
TILES = {2: (256, 256, 1), 3: (128, 128, 2), 4: (64, 128, 3), 5: (256, 128, 1), 9: (256, 192, 1), 10: (256, 128, 1),
         11: (192, 192, 1), 12: (64, 256, 1)}


@pytest.fixture(scope="module")
def dev():
    assert torch.cuda.is_available(), "these tests need the GPU box"
    return torch.device("cuda:0")


def _to(data, dev):
    return tuple(t.to(dev) if isinstance(t, torch.Tensor) else t for t in data)


def _dealt(dev, m, n, k, variant):
    """The cuts the library makes for this shape and tile on this device."""
    mm = importlib.import_module("oracle.mfma_model")
    tm, tn, per_cu = TILES[variant]
    pairs = -(-m // tm) * -(-n // tn) * (k // 128)
    grid = min(torch.cuda.get_device_properties(dev).multi_processor_count * per_cu, pairs)
    return mm.DealtKBlocks(m, n, k, tm, tn, grid)


@pytest.mark.parametrize("variant", sorted(TILES))
def test_config1_every_element_equals_the_model(pkg, oracle, dev, variant):
    """256 x 512 x 1024: more workgroups than tiles, so every tile is cut into several pieces.  All 131072
    outputs must be the modelled kernel's bits: the pieces, their order and the one rounding."""
    mm = importlib.import_module("oracle.mfma_model")
    cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0])
    out = pkg.custom_kernel(_to(cpu, dev), variant=variant, split_k=-1).cpu()
    cuts = _dealt(dev, 256, 512, 1024, variant)
    assert cuts.max_pieces > 1
    idx = np.stack(np.meshgrid(np.arange(256), np.arange(512), indexing="ij"), -1).reshape(-1, 2)
    want, _ = mm.model_kernel_at(cpu, idx, cuts)
    assert torch.equal(out.reshape(-1).view(torch.int16), want.view(torch.int16)), "variant %d" % variant
    ok, nstrict, nun = oracle.parity_report(out, oracle.ref_kernel(cpu), cpu, cuts, RTOL, ATOL)
    assert ok, "variant %d: %d beyond the bar, %d not reproduced" % (variant, nstrict, nun)


@pytest.mark.parametrize("m,n,k", [(272, 2112, 512), (304, 400, 384), (64, 1024, 1024), (512, 144, 1280), (1, 7, 128), (33, 129, 384),
                                   (516, 264, 384), (4095, 512, 256), (1021, 264, 384), (61, 2048, 1024), (3, 18432, 512),
                                   (2050, 136, 384), (257, 192, 384), (513, 136, 1024), (300, 1001, 128), (255, 383, 256),
                                   (1024, 512, 7168), (1000, 1536, 2304), (130, 4100, 1536)])
def test_ragged_shapes(pkg, oracle, dev, m, n, k):
    """Tails in m and n (rows off the 4-row grid, columns off the 8-column grid: the instantiation that repairs
    the last bytes of a and b, which must happen in the segment that holds the last K block), tiles larger than
    the matrix, one K block, more workgroups than (tile, K block) pairs."""
    cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[2], m=m, n=n, k=k)
    ref = oracle.ref_kernel(cpu)
    for variant in (2, 3, 4, 9, 10, 11, 12):
        out = pkg.custom_kernel(_to(cpu, dev), variant=variant, split_k=-1)
        ok, nbad, maxerr = oracle.within_tolerance(out, ref, RTOL, ATOL)
        assert ok, "%dx%dx%d variant %d: %d elements outside the bar (max abs err %g)" % (m, n, k, variant, nbad, maxerr)


@pytest.mark.parametrize("cfg_index,variant", [(3, 2), (3, 9), (3, 11), (4, 12), (4, 10)])
def test_full_size_configurations(pkg, oracle, dev, cfg_index, variant):
    """Configuration 3 (4096 x 2112 x 7168: fewer tiles than CUs, every tile shared by two or three workgroups)
    and configuration 4 (64 x 18432 x 7168: every tile shared by four or five) at full size, every element."""
    cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[cfg_index - 1])
    out = pkg.custom_kernel(_to(cpu, dev), variant=variant, split_k=-1)
    ok, nbad, maxerr = oracle.within_tolerance(out, oracle.ref_kernel(cpu), RTOL, ATOL)
    assert ok, "config %d variant %d: %d elements outside the bar (max abs err %g)" % (cfg_index, variant, nbad, maxerr)


def test_many_tiles_per_workgroup(pkg, oracle, dev):
    """More tiles than workgroups: a run holds the end of one tile, whole tiles and the start of another; the
    whole tiles take the plain path (next tile's first block sent ahead of the output stores)."""
    cfg = pkg.inputs.CONFIGS[2]
    for (m, n, k, variant) in ((4100, 4096, 384, 2), (2049, 4104, 256, 3), (4096, 4232, 512, 11), (8192, 2048, 640, 10)):
        cpu = pkg.inputs.make_dense(cfg, m=m, n=n, k=k)
        data = _to(cpu, dev)
        out = pkg.custom_kernel(data, variant=variant, split_k=-1)
        exact = pkg.custom_kernel((data[0], data[1], data[2], data[3], torch.zeros_like(out)), variant=1, split_k=1)
        torch.cuda.synchronize()
        err = (out.float() - exact.float()).abs()
        bad = int((err > ATOL + RTOL * exact.float().abs()).sum())
        assert bad == 0, "%dx%dx%d variant %d: %d elements differ from the scalar kernel" % (m, n, k, variant, bad)


def test_repeated_calls_and_graph_replays_find_the_flags_down(pkg, dev):
    """The owner takes every flag down after reading it, so a second call - and a replay of a captured call,
    which carries the same flag value as the first - never mistakes the earlier call's flags for its own."""
    cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[3], m=64, n=2304, k=2048)
    data = _to(cpu, dev)
    first = pkg.custom_kernel(data, variant=12, split_k=-1).clone()
    for _ in range(3):
        data[4].fill_(5.0)
        assert torch.equal(pkg.custom_kernel(data, variant=12, split_k=-1).view(torch.int16), first.view(torch.int16))
    other = _to(pkg.inputs.make_dense(pkg.inputs.CONFIGS[2], m=64, n=2304, k=2048), dev)
    want_other = pkg.custom_kernel(other, variant=12, split_k=-1).clone()
    static = tuple(t.clone() for t in data)
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        pkg.custom_kernel(static, variant=12, split_k=-1)        # the capture stream's workspace exists from here on
    torch.cuda.current_stream().wait_stream(side)
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph):
        pkg.custom_kernel(static, variant=12, split_k=-1)
    for rep in range(4):
        src, want = (data, first) if rep % 2 == 0 else (other, want_other)
        for dst, s in zip(static[:4], src[:4]):
            dst.copy_(s)
        static[4].fill_(3.0)
        graph.replay()
        torch.cuda.synchronize()
        assert torch.equal(static[4].view(torch.int16), want.view(torch.int16)), "replay %d" % rep
        pkg.custom_kernel(data)                                  # eager work between replays
        torch.cuda.synchronize()


def test_workspace_too_small_is_refused(pkg, dev):
    lib = pkg._lib.load()
    cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0])
    a, b, sa, sb, c = _to(cpu, dev)
    ws = torch.empty(1 << 20, dtype=torch.uint8, device=dev)
    st = lib.fp8bs_gemm_ex(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), ws.data_ptr(), ws.numel(),
                           256, 512, 1024, 2, -1, None)
    assert st == 3                                               # FP8BS_ERR_WORKSPACE
    st = lib.fp8bs_gemm_ex(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), None, 0, 256, 512, 1024, 2, -1, None)
    assert st == 3
    for variant in (1, 6):                                       # the scalar and the streaming kernels deal no K blocks
        st = lib.fp8bs_gemm_ex(a.data_ptr(), b.data_ptr(), sa.data_ptr(), sb.data_ptr(), c.data_ptr(), ws.data_ptr(), ws.numel(),
                               256, 512, 1024, variant, -1, None)
        assert st == 7                                           # FP8BS_ERR_BAD_VARIANT


def test_a_wait_that_gives_up_ends_the_kernel_and_sets_the_status_word():
    """FP8BS_STREAMK_SPIN < 0 makes every owner's wait give up at once (set from the host, in a process of its
    own because the library reads it once): the kernel runs to its end, the first word of the workspace holds
    FP8BS_ERR_TIMEOUT, and a later call with the limit back in place is right again."""
    code = r"""
import importlib, os, sys, torch
sys.path.insert(0, %r)
pkg = importlib.import_module("amd-developer-challenge-2025_amd")
sub = importlib.import_module("amd-developer-challenge-2025_amd.submission")
dev = torch.device("cuda:0")
cpu = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0])
data = tuple(t.to(dev) for t in cpu)
stream = torch.cuda.current_stream().cuda_stream
ws = sub._workspace(dev, (64 << 20) + 16384, stream)
ws[:16].zero_()
pkg.custom_kernel(data, variant=2, split_k=-1)
torch.cuda.synchronize()
print("status", int(ws[:4].view(torch.int32)[0]))
""" % ROOT
    env = dict(os.environ, FP8BS_STREAMK_SPIN="-1")
    res = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert "status 9" in res.stdout, res.stdout + res.stderr[-1000:]
    env = dict(os.environ)
    env.pop("FP8BS_STREAMK_SPIN", None)
    res = subprocess.run([sys.executable, "-c", code], env=env, stdout=subprocess.PIPE, stderr=subprocess.PIPE, text=True, timeout=300)
    assert res.returncode == 0, res.stderr[-2000:]
    assert "status 0" in res.stdout, res.stdout + res.stderr[-1000:]
