import importlib
import json
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def pkg():
    return importlib.import_module("amd-developer-challenge-2025_amd")


@pytest.fixture(scope="session")
def oracle():
    return importlib.import_module("oracle.fp8bs_oracle")


@pytest.fixture(scope="session")
def c_oracle():
    mod = importlib.import_module("oracle.c_oracle")
    mod.load()
    return mod


@pytest.fixture(scope="session")
def golden_gemm():
    """The committed 16x32x256 power-of-two fixture as a (a, b, a_scale, b_scale, c) CPU tuple + expected bits."""
    with open(os.path.join(GOLDEN, "gemm_16x32x256.json")) as f:
        g = json.load(f)
    m, n, k = g["m"], g["n"], g["k"]
    kb, nb = k // 128, (n + 127) // 128
    a = torch.tensor(g["a"], dtype=torch.uint8).reshape(k, m).view(torch.float8_e4m3fn).t()
    b = torch.tensor(g["b"], dtype=torch.uint8).reshape(k, n).view(torch.float8_e4m3fn).t()
    a_scale = torch.tensor(g["a_scale"], dtype=torch.float32).reshape(kb, m).t()
    b_scale = torch.tensor(g["b_scale"], dtype=torch.float32).reshape(kb, nb).t()
    c = torch.zeros(m, n, dtype=torch.bfloat16)
    expected = torch.tensor(g["expected_bf16_bits"], dtype=torch.int32).to(torch.int16).view(torch.bfloat16).reshape(m, n)
    expected_fp32 = torch.tensor(g["expected_fp32"], dtype=torch.float32).reshape(m, n)
    return (a, b, a_scale, b_scale, c), expected, expected_fp32
