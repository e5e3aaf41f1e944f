"""Test configuration: the `gpu` marker, import path, and helpers shared by the suites.

`-m "not gpu"` runs the oracle pins, host logic and C-ABI export checks (no device needed);
`-m gpu` runs the parity tests proper, which call the HIP kernels through the C ABI.
"""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a gfx950 device (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


@pytest.fixture(autouse=True)
def _seed_everything():
    torch.manual_seed(9999)
    yield


def rel_err(actual, expected):
    """max |a - e| / max |e| -- the relative error the parity bar is stated in."""
    a = actual.detach().double().cpu()
    e = expected.detach().double().cpu()
    return ((a - e).abs().max() / e.abs().max().clamp_min(1e-30)).item()


def max_abs_err(actual, expected):
    return (actual.detach().double().cpu() - expected.detach().double().cpu()).abs().max().item()


# Parity bars: fp32 max-abs 1e-5; bf16 / fp16 relative 2e-2 (dropout off).
FP32_ATOL = 1e-5
HALF_RTOL = 2e-2


def assert_parity(actual, expected, dtype, what=""):
    if dtype == torch.float32:
        err = max_abs_err(actual, expected)
        assert err <= FP32_ATOL, f"{what}: max-abs {err:.3e} > {FP32_ATOL}"
    else:
        # relative to the largest reference magnitude; the floor only matters when the
        # reference is identically zero (e.g. dQ for a single key)
        err = max_abs_err(actual, expected)
        bound = HALF_RTOL * expected.detach().double().abs().max().item() + 1e-5
        assert err <= bound, f"{what}: max-abs {err:.3e} > {bound:.3e} (= {HALF_RTOL} relative)"
