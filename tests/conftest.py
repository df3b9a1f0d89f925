import os
import sys

import numpy as np
import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)

GOLDEN_DIR = os.path.join(ROOT, "tests", "golden")


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def load_golden(name):
    """Returns (params, inputs, out, meta) of tests/golden/<name>.npz as torch tensors / python scalars."""
    z = np.load(os.path.join(GOLDEN_DIR, name + ".npz"), allow_pickle=False)
    params, inputs, meta, out = {}, {}, {}, None
    for key in z.files:
        arr = z[key]
        if key.startswith("param/"):
            params[key[6:]] = torch.from_numpy(arr)
        elif key.startswith("in/"):
            inputs[key[3:]] = torch.from_numpy(arr)
        elif key.startswith("meta/"):
            meta[key[5:]] = arr.item() if arr.ndim == 0 else arr
        elif key == "out":
            out = torch.from_numpy(arr)
    return params, inputs, out, meta


def max_rel(a, b):
    """max|a-b| / max|b| (the attention parity measure)."""
    return ((a - b).abs().max() / b.abs().max().clamp_min(1e-30)).item()


def max_rel_elementwise(a, b, floor=1e-3):
    """max |a-b| / |b| over the entries with |b| > floor * max|b|."""
    keep = b.abs() > floor * b.abs().max()
    return ((a - b).abs()[keep] / b.abs()[keep]).max().item()


def rel_l2(a, b):
    return ((a - b).norm() / b.norm().clamp_min(1e-30)).item()


@pytest.fixture(scope="session")
def gpu():
    if not torch.cuda.is_available():
        pytest.skip("no GPU visible")
    return torch.device("cuda:0")
