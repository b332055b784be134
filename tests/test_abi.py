"""The C-ABI library loads without a GPU, exports every symbol include/fp8bs.h declares, and its
host-only entry points (planner, argument checks, error strings) behave.  No GPU compute here."""
import ctypes
import importlib
import os
import re

import pytest
import torch

from conftest import ROOT


def _declared_symbols():
    text = open(os.path.join(ROOT, "include", "fp8bs.h")).read()
    text = re.sub(r"/\*.*?\*/", "", text, flags=re.S)
    return sorted(set(re.findall(r"\b(fp8bs_[a-z_]+)\s*\(", text)))


def test_library_exports_every_declared_symbol(pkg):
    lib = pkg._lib.load()
    declared = _declared_symbols()
    assert set(declared) == set(pkg._lib.EXPORTS)
    for name in declared:
        assert getattr(lib, name) is not None
    assert lib.fp8bs_version() >= pkg._lib.MIN_VERSION


def test_every_variant_has_a_name_and_the_plan_struct_matches_the_header(pkg):
    text = open(os.path.join(ROOT, "include", "fp8bs.h")).read()
    count = int(re.search(r"FP8BS_VARIANT_COUNT\s*=\s*(\d+)", text).group(1))
    assert set(pkg._lib.VARIANT_NAMES) == set(range(count))
    body = re.search(r"typedef struct fp8bs_plan_t \{(.*?)\} fp8bs_plan_t;", text, flags=re.S).group(1)
    body = re.sub(r"/\*.*?\*/", "", body, flags=re.S)
    fields = [f.strip() for decl in re.findall(r"(?:int32_t|uint64_t)\s+([^;]+);", body) for f in decl.split(",")]
    assert fields == [name for name, _ in pkg._lib.Plan._fields_]
    shift = int(re.search(r"#define FP8BS_SPLIT_SUM_IN_KERNEL \(1 << (\d+)\)", text).group(1))
    assert pkg._lib.SPLIT_SUM_IN_KERNEL == 1 << shift
    assert ctypes.sizeof(pkg._lib.Plan) == 4 * 12 + 8                # twelve int32, then the 8-byte workspace size


def test_plan_with_the_devices_cu_count(pkg):
    """num_cus <= 0 asks the current device (256 where there is none), the count fp8bs_gemm plans with."""
    lib = pkg._lib.load()
    a, b = pkg._lib.Plan(), pkg._lib.Plan()
    cus = torch.cuda.get_device_properties(0).multi_processor_count if torch.cuda.is_available() else 256
    for shape in ((4096, 2112, 7168), (64, 18432, 7168), (1024, 512, 7168)):
        assert lib.fp8bs_plan(*shape, 0, ctypes.byref(a)) == 0 and lib.fp8bs_plan(*shape, cus, ctypes.byref(b)) == 0
        assert bytes(a) == bytes(b)
        assert a.stream_k == 0 and a.workspace_bytes == pkg.workspace_bytes(*shape)


def _planned_workspace(p, m, n):
    """What a plan's K split needs: counters and one fp32 tile per (tile, partition) when the partitions are summed in
    the kernel, whole fp32 planes when a reduce kernel follows."""
    if p.split_k == 1:
        return 0
    if p.sum_in_kernel:
        return 16384 + -(-m // p.tile_m) * -(-n // p.tile_n) * p.split_k * p.tile_m * p.tile_n * 4
    return p.split_k * m * n * 4


def test_plan_shape_families(pkg):
    p = pkg.plan(4096, 4096, 4096)
    assert p.variant == 2 and (p.tile_m, p.tile_n) == (256, 256) and p.split_k == 1 and p.workspace_bytes == 0
    assert p.grid_x == 256 and p.block_threads == 512 and p.lds_bytes == 2 * (128 * 512 + 1024 + 256)     # A + B + a_scale row + b_scale values, two stages
    p = pkg.plan(64, 18432, 7168)                       # skinny-M: the 64x256 tile with three stages, 72 tiles x a K split of 3
    assert p.variant == 12 and (p.tile_m, p.tile_n) == (64, 256) and p.split_k == 3 and p.grid_x == 216
    assert p.block_threads == 512 and p.lds_bytes == 3 * (128 * 320 + 1024 + 256)
    assert p.sum_in_kernel == 1                          # three partitions: summed by the last workgroup of each tile, one launch
    assert p.workspace_bytes == 16384 + 72 * 3 * 64 * 256 * 4 == pkg.workspace_bytes(64, 18432, 7168)
    p = pkg.plan(130, 190, 256)                         # n not a multiple of 8, short K -> a tiled kernel without a K split
    assert p.variant in (2, 3, 4, 9, 10, 11, 12) and p.split_k == 1
    p, q = pkg.plan(1024, 190, 7168), pkg.plan(1024, 192, 7168)   # long K, few tiles: a K split, also with n off the 8-column grid
    assert p.variant == q.variant and p.variant in (2, 3, 4, 9, 10, 11, 12) and p.split_k == q.split_k > 1
    assert p.workspace_bytes == _planned_workspace(p, 1024, 190) and (p.sum_in_kernel == 1) == (p.split_k in (2, 3))
    for m in (130, 4095, 3, 1):                               # any m: the tiled kernels, one launch, nothing extra in the workspace
        p, q = pkg.plan(m, 192, 256), pkg.plan((m + 3) & ~3, 192, 256)
        assert p.variant == q.variant and p.variant not in (1, 6, 7, 8) and p.split_k == q.split_k
        assert p.workspace_bytes == _planned_workspace(p, m, 192)
    p, q = pkg.plan(3, 18432, 7168), pkg.plan(4, 18432, 7168) # a few rows against a large b: the same skinny plan for any m
    assert p.variant == q.variant == 12 and p.split_k == q.split_k and p.workspace_bytes == _planned_workspace(p, 3, 18432) and q.workspace_bytes == _planned_workspace(q, 4, 18432)
    assert pkg.plan(3, 190, 256).variant in (3, 4, 12)
    p = pkg.plan(256, 512, 1024)                        # small: one of the sub-256 tiles, never the scalar kernel
    assert p.variant in (3, 4, 10, 12) and p.split_k >= 1 and p.split_k <= 8
    p = pkg.plan(1024, 512, 7168)                       # few tiles, long K: the planner splits K
    assert p.variant in (3, 4, 10, 12) and p.split_k > 1
    p = pkg.plan(6144, 4608, 7168)                      # large: the 256x256 tile, no split
    assert p.variant == 2 and p.split_k == 1
    p = pkg.plan(4096, 2112, 7168)                      # 2112 = 11 x 192: 242 tiles of 192x192 instead of 144 of 256x256, 16 of them a quarter full
    assert p.variant == 11 and (p.tile_m, p.tile_n) == (192, 192) and p.grid_x == 242 and p.lds_bytes == 3 * (128 * 384 + 1024 + 256)
    p = pkg.plan(4096, 3072, 8192)                      # 256 tiles of 256x192
    assert p.variant == 9 and (p.tile_m, p.tile_n) == (256, 192) and p.grid_x == 256 and p.lds_bytes == 2 * (128 * 448 + 1024 + 256)
    p = pkg.plan(4096, 2048, 8192)                      # 256 tiles of 256x128, three stages
    assert p.variant == 10 and (p.tile_m, p.tile_n) == (256, 128) and p.lds_bytes == 3 * (128 * 384 + 1024 + 256)


def test_plan_skinny_rule_and_the_streaming_kernels(pkg):
    """At most 64 rows against a B of 24 MB or more: always the 64x256 three-stage tile, with the K split of the
    streaming model.  Everything else goes through the cost model of all the tiles (the 64x256 tile among them).
    The streaming kernels are never planned (forced variants only)."""
    for m, n, k, skinny in [(64, 18432, 7168, True), (16, 18432, 7168, True), (4, 18432, 7168, True), (64, 7168, 7168, True),
                            (1, 28672, 4096, True), (64, 18440, 7168, True), (63, 18429, 7168, True),
                            (65, 18432, 7168, False), (128, 18432, 7168, False), (64, 2048, 7168, False),
                            (64, 7168, 2048, False), (32, 512, 2048, False), (1536, 1536, 4096, False)]:
        p = pkg.plan(m, n, k)
        if skinny:
            assert p.variant == 12 and p.grid_x == -(-n // 256) * p.split_k, (m, n, k, p.variant)
        assert p.variant not in (1, 6, 7, 8)
        assert 1 <= p.split_k <= 8 and p.workspace_bytes == _planned_workspace(p, m, n)
        assert p.sum_in_kernel == 0 or p.split_k in (2, 3)              # only two or three partitions are summed in the kernel
    assert pkg.plan(1536, 1536, 4096).variant == 12           # the cost model's pick for a few hundred rows per tile column
    # few rows: summed in the kernel only where the planes are large enough for the reduce launch to cost more
    assert pkg.plan(64, 18432, 7168).sum_in_kernel == 1 and pkg.plan(1, 18432, 7168).sum_in_kernel == 0
    for m in (1, 5, 63):                                      # rows that are not a multiple of four: the same plan
        p, q = pkg.plan(m, 18432, 7168), pkg.plan((m + 3) & ~3, 18432, 7168)
        assert p.variant == q.variant == 12 and p.split_k == q.split_k


def test_plan_rejects_bad_shapes(pkg):
    lib = pkg._lib.load()
    out = pkg._lib.Plan()
    assert lib.fp8bs_plan(16, 16, 100, 0, ctypes.byref(out)) == 2      # k not a multiple of 128
    assert lib.fp8bs_plan(0, 16, 128, 0, ctypes.byref(out)) == 2
    assert lib.fp8bs_plan(16, 16, 128, 0, None) == 1
    assert pkg.workspace_bytes(16, 16, 100) == 0


def test_argument_errors_are_reported_before_any_launch(pkg):
    lib = pkg._lib.load()
    one = ctypes.c_void_p(16)      # never dereferenced: the checks fail first
    assert lib.fp8bs_gemm(one, one, one, one, one, None, 0, 16, 16, 100, None) == 2
    assert lib.fp8bs_gemm(None, one, one, one, one, None, 0, 16, 16, 128, None) == 1
    assert lib.fp8bs_gemm(one, one, one, one, one, None, 0, -1, 16, 128, None) == 2
    assert lib.fp8bs_gemm(one, one, one, one, one, None, 0, 0, 16, 128, None) == 0       # empty: nothing to do
    assert lib.fp8bs_gemm(one, one, one, one, one, None, 0, 1 << 20, 16, 1 << 13, None) == 4   # 2^33 bytes of a
    assert lib.fp8bs_gemm_ex(one, one, one, one, one, None, 0, 16, 16, 128, 99, 1, None) == 7
    assert lib.fp8bs_gemm_ex(one, one, one, one, one, None, 0, 128, 20, 512, 2, 2, None) == 3  # a K split takes any n, but needs its workspace
    assert lib.fp8bs_gemm_ex(one, one, one, one, one, None, 0, 128, 20, 128, 6, 1, None) == 7  # the streaming kernels need n % 8 == 0
    assert lib.fp8bs_gemm_ex(one, one, one, one, one, None, 0, 130, 16, 128, 7, 1, None) == 7  # the wider streaming kernels need m % 4 == 0
    assert lib.fp8bs_gemm_ex(one, one, one, one, one, None, 0, 64, 256, 1024, 4, 4, None) == 3 # split-K without workspace
    assert lib.fp8bs_gemm_grouped(one, one, one, one, one, None, 4, 16, 16, 128, None) == 1
    assert lib.fp8bs_gemm_grouped(one, one, one, one, one, one, 0, 16, 16, 128, None) == 6
    for code in range(0, 9):
        assert len(lib.fp8bs_strerror(code)) > 0
    with pytest.raises(RuntimeError, match="multiple of 128"):
        pkg._lib.check(2)


def test_custom_kernel_validates_its_operands(pkg):
    a, b, a_scale, b_scale, c = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0], m=32, n=128, k=128)
    with pytest.raises(ValueError, match="GPU tensor"):
        pkg.custom_kernel((a, b, a_scale, b_scale, c))           # CPU tensors: no CPU path exists
    with pytest.raises(TypeError):
        pkg.custom_kernel((a.float(), b, a_scale, b_scale, c))
    with pytest.raises(TypeError):
        pkg.custom_kernel((a, b, a_scale, b_scale, c.float()))


def test_gate_up_silu_validates_its_operands(pkg):
    """Wrong shapes and layouts are refused on the host: the kernel sizes its buffer descriptors from the
    arguments, so a mismatched b or b_scale would be read past its allocation."""
    moe = importlib.import_module("amd-developer-challenge-2025_amd.moe")
    a, b, a_scale, b_scale, c = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0], m=32, n=128, k=256)
    h = torch.empty(32, 64, dtype=torch.bfloat16)
    with pytest.raises(ValueError, match="GPU tensor"):
        moe.gate_up_silu((a, b, a_scale, b_scale, None, h))                       # everything right but the device
    wrong_k = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0], m=32, n=128, k=128)
    with pytest.raises(ValueError, match="shapes do not match"):
        moe.gate_up_silu((a, wrong_k[1], a_scale, b_scale, None, h))              # b's K differs from a's
    with pytest.raises(ValueError, match="shapes do not match"):
        moe.gate_up_silu((a, b, a_scale, wrong_k[3], None, h))                    # b_scale of another K
    with pytest.raises(ValueError, match="shapes do not match"):
        moe.gate_up_silu((a, b, wrong_k[2], b_scale, None, h))                    # a_scale of another K
    with pytest.raises(ValueError, match="K-major"):
        moe.gate_up_silu((a, b.contiguous(), a_scale, b_scale, None, h))          # row-major b
    with pytest.raises(ValueError, match=r"\[rows, n\]"):
        moe.gate_up_silu((a, b, a_scale, b_scale, None, torch.empty(32, 128, dtype=torch.bfloat16)))   # h must have n/2 columns
    with pytest.raises(ValueError, match="E, n, k"):
        moe.gate_up_silu((a, b, a_scale, b_scale, torch.zeros(2, dtype=torch.int32), h))   # grouped call with a 2-D b
    with pytest.raises(TypeError):
        moe.gate_up_silu((a.float(), b, a_scale, b_scale, None, h))


def test_custom_kernel_without_version_counters(pkg):
    """Tensors made under inference_mode have no version counter: the checked-once cache must step aside,
    not raise (the call then fails on the operands being CPU tensors, like any other CPU call)."""
    with torch.inference_mode():
        data = pkg.inputs.make_dense(pkg.inputs.CONFIGS[0], m=32, n=128, k=128)
        with pytest.raises(ValueError, match="GPU tensor"):
            pkg.custom_kernel(data)


def test_cpython_binding_returns_what_ctypes_returns(pkg):
    """csrc/fp8bs_pycall.c binds fp8bs_gemm_ex / fp8bs_gemm_grouped_ex without ctypes' marshalling: built by build(),
    same status codes for the argument errors that are reported before any launch, type errors raised."""
    lib, fast = pkg._lib.load(), pkg._lib.pycall()
    assert fast is not None, "the CPython binding was not built (amd-developer-challenge-2025_amd/build.py)"
    one = 16
    for args in ((one, one, one, one, one, None, 0, 16, 16, 100, 0, 0, None),          # k not a multiple of 128
                 (None, one, one, one, one, None, 0, 16, 16, 128, 0, 0, None),         # null pointer
                 (one, one, one, one, one, None, 0, 0, 16, 128, 0, 0, None),           # empty
                 (one, one, one, one, one, None, 0, 1 << 20, 16, 1 << 13, 0, 0, None), # too large
                 (one, one, one, one, one, None, 0, 16, 16, 128, 99, 1, None),         # unknown variant
                 (one, one, one, one, one, None, 0, 64, 256, 1024, 4, 4, None)):       # forced K split without a workspace
        assert fast.gemm_ex(*args) == lib.fp8bs_gemm_ex(*args)
    g = (one, one, one, one, one, None, 4, 16, 16, 128, 0, None)
    assert fast.gemm_grouped_ex(*g) == lib.fp8bs_gemm_grouped(*(g[:10] + g[11:])) == 1
    assert fast.gemm_grouped_ex(one, one, one, one, one, one, 0, 16, 16, 128, 0, None) == 6
    with pytest.raises(TypeError):
        fast.gemm_ex(1, 2, 3)
    with pytest.raises(TypeError):
        fast.gemm_ex("a", one, one, one, one, None, 0, 16, 16, 128, 0, 0, None)
    with pytest.raises(OverflowError):
        fast.gemm_ex(one, one, one, one, one, None, 0, 1 << 40, 16, 128, 0, 0, None)


def test_root_submission_module_reexports_entry_point(pkg):
    import submission
    assert submission.custom_kernel is pkg.custom_kernel
