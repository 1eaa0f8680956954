import os
import sys

import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


@pytest.fixture(scope="session")
def oracle():
    from oracle import oracle as o
    o.lib()
    return o


def bits(t):
    """torch bf16 tensor -> numpy uint16 bit patterns."""
    import torch
    return t.detach().cpu().contiguous().view(torch.int16).numpy().view("uint16")


def np_of(t):
    return t.detach().cpu().contiguous().numpy()


def bf16_close(a_bits, b_bits, atol=2e-3, rtol=1e-2):
    """The path's tolerance: every element passes if |d| <= atol OR |d|/max(|a|,|b|) <= rtol
    (abs-or-rel, as the reference's checker, tests/gtest_utils.h:47-61).  Returns (ok, max_abs, n_bad)."""
    import numpy as np
    a = (a_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    b = (b_bits.astype(np.uint32) << 16).view(np.float32).astype(np.float64)
    d = np.abs(a - b)
    rel = d / np.maximum(np.maximum(np.abs(a), np.abs(b)), 1e-30)
    bad = (d > atol) & (rel > rtol)
    bad |= ~np.isfinite(a) | ~np.isfinite(b)
    return (not bad.any()), float(d.max() if d.size else 0.0), int(bad.sum())
