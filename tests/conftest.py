import os
import random
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
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def make_case(batch, seqlen, heads, head_dim=128, dtype=torch.bfloat16, seed=0, device="cpu"):
    """The reference test's data recipe (tests/test_moba_attn.py:8-34): seeded
    N(0,1) q/k/v in bf16 and batch-1 sorted random sequence boundaries.  Data is
    drawn on the CPU so that the oracle and the GPU path see identical bits."""
    random.seed(seed)
    g = torch.Generator().manual_seed(seed)
    q = torch.randn((seqlen, heads, head_dim), generator=g, dtype=torch.float32).to(dtype)
    k = torch.randn((seqlen, heads, head_dim), generator=g, dtype=torch.float32).to(dtype)
    v = torch.randn((seqlen, heads, head_dim), generator=g, dtype=torch.float32).to(dtype)
    do = torch.randn((seqlen, heads, head_dim), generator=g, dtype=torch.float32).to(dtype)
    cuts = sorted(random.sample(range(1, seqlen - 1), batch - 1)) if batch > 1 else []
    cu = [0] + cuts + [seqlen]
    max_seqlen = max(b - a for a, b in zip(cu[:-1], cu[1:]))
    if device != "cpu":
        q, k, v, do = (x.to(device) for x in (q, k, v, do))
    return q, k, v, do, cu, max_seqlen
