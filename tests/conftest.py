import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")
    config.addinivalue_line("markers", "slow: takes more than a few seconds on CPU")


def has_gpu():
    try:
        import torch
        return torch.cuda.is_available()
    except Exception:
        return False


def pytest_collection_modifyitems(config, items):
    if has_gpu():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def make_qkv(Sq, Hq, Hkv, D, seed=0, scaled=True):
    """Seeded synthetic inputs as the benchmark draws them: fp32 N(0,1) (times
    D^-0.5 when `scaled`), rounded to bf16 so CPU oracle and GPU see equal values."""
    import torch
    g = torch.Generator().manual_seed(seed)
    s = D ** -0.5 if scaled else 1.0
    q = (torch.randn(Sq, Hq, D, generator=g) * s).to(torch.bfloat16)
    k = (torch.randn(Sq, Hkv, D, generator=g) * s).to(torch.bfloat16)
    v = (torch.randn(Sq, Hkv, D, generator=g) * s).to(torch.bfloat16)
    return q, k, v


def to_np(t):
    return t.detach().float().cpu().numpy()
