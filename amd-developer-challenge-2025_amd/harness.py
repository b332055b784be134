"""Compatibility with the upstream harness the reference was written for (gpu-mode/reference-kernels,
problems/amd/fp8-mm; reference README.md:54-101): its tests-file format, the 18 leaderboard shapes, its
fnuz operands, and `test` / `benchmark` style runs.

The upstream `task.py` / `reference.py` / `eval.py` are not part of the reference repository and are
not reproduced here; what this module offers is what a maintainer needs on the submission side:
  * parse_tests           the `m: ..; n: ..; k: ..; seed: ..` lines of a tests file (README.md:65-82)
  * LEADERBOARD_SHAPES    the 18 benchmark shapes listed there
  * custom_kernel_fnuz    custom_kernel for operands in float8_e4m3fnuz (the type the harness generates
                          for gfx942, 1-amd-fp8-mm/amd-fp8-mm-submission.py:20-21): bytes are converted to
                          e4m3fn of the same value on the GPU, scales are used unchanged
  * generate_input        inputs of the contract's shapes/strides for (m, n, k, seed) from this build's
                          own seeded generator (the upstream CUDA-generator stream cannot be reproduced)
  * benchmark             per-shape times and their geometric mean, the leaderboard's figure of merit
"""
import math
import re
from typing import Dict, Iterable, List

import torch

from . import _lib, inputs, quant
from .submission import custom_kernel

LEADERBOARD_TESTS = """
m: 1024; n: 1536; k: 7168; seed: 8135
m: 1024; n: 3072; k: 1536; seed: 6251
m: 1024; n: 576 ; k: 7168; seed: 12346
m: 1024; n: 7168; k: 256 ; seed: 5364
m: 1024; n: 7168; k: 2048; seed: 6132
m: 1024; n: 4608; k: 7168; seed: 7531
m: 1024; n: 7168; k: 2304; seed: 12345
m: 1024; n: 512 ; k: 7168; seed: 6563
m: 1024; n: 4096; k: 512 ; seed: 17512
m: 6144; n: 1536; k: 7168; seed: 6543
m: 6144; n: 3072; k: 1536; seed: 234
m: 6144; n: 576 ; k: 7168; seed: 9863
m: 6144; n: 7168; k: 256 ; seed: 764243
m: 6144; n: 7168; k: 2048; seed: 76547
m: 6144; n: 4608; k: 7168; seed: 65436
m: 6144; n: 7168; k: 2304; seed: 452345
m: 6144; n: 512 ; k: 7168; seed: 12341
m: 6144; n: 4096; k: 512 ; seed: 45245
"""


def parse_tests(text: str) -> List[Dict[str, int]]:
    """Lines of `key: value; key: value; ...` -> list of dicts of ints; blank lines and `#` comments are skipped."""
    cases = []
    for ln, line in enumerate(text.splitlines(), 1):
        line = line.split("#", 1)[0].strip()
        if not line:
            continue
        case = {}
        for part in line.split(";"):
            part = part.strip()
            if not part:
                continue
            m = re.fullmatch(r"([A-Za-z_]\w*)\s*:\s*(-?\d+)", part)
            if not m:
                raise ValueError("tests file line %d: cannot parse %r" % (ln, part))
            case[m.group(1)] = int(m.group(2))
        for key in ("m", "n", "k", "seed"):
            if key not in case:
                raise ValueError("tests file line %d: missing %r" % (ln, key))
        cases.append(case)
    return cases


LEADERBOARD_SHAPES = parse_tests(LEADERBOARD_TESTS)


def generate_input(m: int, n: int, k: int, seed: int, device="cuda"):
    """(a, b, a_scale, b_scale, c) of the contract's dtypes, shapes and K-major strides, quantised on the GPU."""
    dev = torch.device(device)
    g = torch.Generator(device=dev).manual_seed(seed)
    a, a_scale = quant.quantize_a(torch.randn(m, k, generator=g, device=dev))
    b, b_scale = quant.quantize_b(torch.randn(n, k, generator=g, device=dev))
    return a, b, a_scale, b_scale, torch.zeros(m, n, dtype=torch.bfloat16, device=dev)


def fnuz_to_fn(t: torch.Tensor) -> torch.Tensor:
    """float8_e4m3fnuz tensor -> float8_e4m3fn tensor of the same values, shape and strides (GPU)."""
    if t.dtype != torch.float8_e4m3fnuz or not t.is_cuda:
        raise TypeError("expected a float8_e4m3fnuz tensor on the GPU")
    if not (t.is_contiguous() or (t.dim() == 2 and t.t().is_contiguous())):
        raise ValueError("expected a contiguous or K-major tensor")
    out = torch.empty_strided(t.shape, t.stride(), dtype=torch.float8_e4m3fn, device=t.device)
    with torch.cuda.device(t.device):
        _lib.check(_lib.load().fp8bs_convert_fnuz_to_fn(t.data_ptr(), out.data_ptr(), t.numel(),
                                                        torch.cuda.current_stream().cuda_stream))
    return out


def custom_kernel_fnuz(data):
    """custom_kernel for operands in float8_e4m3fnuz: same tuple, same scales, fills and returns ``c``."""
    a, b, a_scale, b_scale, c = data
    return custom_kernel((fnuz_to_fn(a), fnuz_to_fn(b), a_scale, b_scale, c))


def benchmark(cases: Iterable[Dict[str, int]] = LEADERBOARD_SHAPES, steps: int = 50, warmup: int = 5, device="cuda"):
    """Per-case mean time in microseconds (HIP events around `steps` calls) and the geometric mean."""
    out = []
    for case in cases:
        data = generate_input(case["m"], case["n"], case["k"], case["seed"], device)
        for _ in range(warmup):
            custom_kernel(data)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        for _ in range(steps):
            custom_kernel(data)
        e1.record()
        e1.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        out.append(dict(case, us=us, tflops=2.0 * case["m"] * case["n"] * case["k"] / us * 1e-6))
    geomean = math.exp(sum(math.log(r["us"]) for r in out) / len(out)) if out else float("nan")
    return out, geomean
