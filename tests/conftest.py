"""Shared test plumbing.

`-m "not gpu"` tests run without a GPU: the oracle against the reference's own
CPU flavor / golden vectors / closed forms, the host logic, and that the C-ABI
library loads and exports what include/paras_hip.h declares.
`-m gpu` tests are the parity tests proper and call the HIP kernels through the
C ABI (tests/capi.py) or through the `paras` PyTorch device.
"""
import os
import sys
from pathlib import Path

import pytest

ROOT = Path(__file__).resolve().parent.parent
for p in (ROOT / "tests", ROOT / "oracle", ROOT / "framework-torch-paras_amd"):
    if str(p) not in sys.path:
        sys.path.insert(0, str(p))


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


@pytest.fixture(autouse=True)
def _seed():
    import torch
    torch.manual_seed(0)   # the reference's runner seeds before every test (tests/common.py:52)
    yield


def bits(t):
    """Integer view of a floating tensor for bit-exact comparison (NaNs canonicalised)."""
    import torch
    t = t.detach().cpu().contiguous()
    if t.dtype.is_floating_point:
        t = torch.where(t.isnan(), torch.full_like(t, float("nan")), t)
        return t.view({2: torch.int16, 4: torch.int32, 8: torch.int64}[t.element_size()])
    return t


def assert_bit_exact(actual, expected, what=""):
    import torch
    a, e = bits(actual), bits(expected)
    assert a.shape == e.shape, f"{what}: shape {tuple(a.shape)} vs {tuple(e.shape)}"
    assert actual.dtype == expected.dtype, f"{what}: dtype {actual.dtype} vs {expected.dtype}"
    bad = int((a != e).sum())
    assert bad == 0, f"{what}: {bad}/{a.numel()} elements differ bitwise"
