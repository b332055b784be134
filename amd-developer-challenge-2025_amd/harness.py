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
  * run_tests             `test` mode (README.md:37-43, 85-101: `eval.py test ./fp8-mm/tests`): every case of a tests
                          file is generated, run through custom_kernel and handed to a checker that the caller
                          injects (the upstream flow compares with its reference.py; this package ships no CPU
                          implementation, so the comparison is the caller's - the test-suite passes its oracle)
  * benchmark             `benchmark` mode: per-shape times and their geometric mean, the leaderboard's figure of merit
  * main                  `python -m amd-developer-challenge-2025_amd.harness test|benchmark <tests file> [--checker module:function]`
"""
import importlib
import math
import re
import sys
from typing import Callable, Dict, Iterable, List, Optional, Tuple

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


def run_tests(text: str, check: Callable[[tuple, torch.Tensor], Tuple[bool, str]], device="cuda",
              kernel: Optional[Callable] = None) -> List[Dict]:
    """`test` mode over a tests file's text: for every case generate the inputs, call ``kernel`` (default
    custom_kernel) and ask ``check(data, output) -> (passed, message)``.  ``data`` is the input tuple as
    generated (on the GPU), ``output`` the returned tensor.  Returns one dict per case: the case's keys plus
    ``passed`` and ``message``; an exception raised by the kernel or the checker fails the case with its text."""
    kernel = kernel or custom_kernel
    results = []
    for case in parse_tests(text):
        try:
            data = generate_input(case["m"], case["n"], case["k"], case["seed"], device)
            out = kernel(data)
            torch.cuda.synchronize()
            passed, message = check(data, out)
        except Exception as ex:       # noqa: BLE001 - a failing case must not end the run
            passed, message = False, "%s: %s" % (type(ex).__name__, ex)
        results.append(dict(case, passed=bool(passed), message=str(message)))
    return results


def benchmark(cases: Iterable[Dict[str, int]] = LEADERBOARD_SHAPES, steps: int = 50, warmup: int = 5, device="cuda", preheat_s: float = 0.02):
    """Per-case mean time in microseconds (HIP events around `steps` back-to-back calls, after `warmup` calls
    and at least `preheat_s` seconds of untimed calls so that the clocks have settled) and the geometric mean."""
    out = []
    for case in cases:
        data = generate_input(case["m"], case["n"], case["k"], case["seed"], device)
        for _ in range(warmup):
            custom_kernel(data)
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        n = 16
        while True:
            for _ in range(n):
                custom_kernel(data)
            e1.record()
            e1.synchronize()
            if e0.elapsed_time(e1) * 1e-3 >= preheat_s or n > (1 << 20):
                break
            n *= 2
        e0.record()
        for _ in range(steps):
            custom_kernel(data)
        e1.record()
        e1.synchronize()
        us = e0.elapsed_time(e1) * 1e3 / steps
        out.append(dict(case, us=us, tflops=2.0 * case["m"] * case["n"] * case["k"] / us * 1e-6))
    geomean = math.exp(sum(math.log(r["us"]) for r in out) / len(out)) if out else float("nan")
    return out, geomean


def main(argv: Optional[List[str]] = None) -> int:
    """`test <tests file> --checker module:function` or `benchmark <tests file>`, the two modes of the upstream
    eval.py (README.md:99-101).  Prints one line per case and a summary; returns 0 if every case passed."""
    argv = list(sys.argv[1:] if argv is None else argv)
    if len(argv) < 2 or argv[0] not in ("test", "benchmark"):
        print("usage: harness test <tests file> --checker module:function | harness benchmark <tests file>", file=sys.stderr)
        return 2
    with open(argv[1]) as f:
        text = f.read()
    if argv[0] == "benchmark":
        rows, geo = benchmark(parse_tests(text))
        for r in rows:
            print("m: %d; n: %d; k: %d; seed: %d  %.1f us  %.0f TFLOP/s" % (r["m"], r["n"], r["k"], r["seed"], r["us"], r["tflops"]))
        print("geometric mean: %.2f us" % geo)
        return 0
    if len(argv) < 4 or argv[2] != "--checker" or ":" not in argv[3]:
        print("test mode needs --checker module:function (check(data, output) -> (passed, message)): this package has no CPU implementation to compare with", file=sys.stderr)
        return 2
    mod, fn = argv[3].split(":", 1)
    check = getattr(importlib.import_module(mod), fn)
    results = run_tests(text, check)
    for r in results:
        print("m: %d; n: %d; k: %d; seed: %d  %s  %s" % (r["m"], r["n"], r["k"], r["seed"], "pass" if r["passed"] else "FAIL", r["message"]))
    failed = sum(not r["passed"] for r in results)
    print("%d of %d cases passed" % (len(results) - failed, len(results)))
    return 0 if failed == 0 else 1


if __name__ == "__main__":
    sys.exit(main())
