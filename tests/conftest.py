import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this environment")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def make_qkv(B, H, Lq, Lk, d, seed, amp=1.0):
    """Seeded fp32 tensors generated on the CPU and rounded to bf16 once, so that the oracle and
    the HIP path see identical bits."""
    g = torch.Generator().manual_seed(seed)
    q = (torch.randn(B, H, Lq, d, generator=g) * amp).to(torch.bfloat16)
    k = (torch.randn(B, H, Lk, d, generator=g) * amp).to(torch.bfloat16)
    v = (torch.randn(B, H, Lk, d, generator=g) * amp).to(torch.bfloat16)
    return q, k, v
