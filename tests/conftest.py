"""Shared test plumbing: import paths, the `gpu` marker, seeded inputs."""
import os
import sys

import pytest
import torch

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
for p in (ROOT, os.path.join(ROOT, "longcat-video_amd")):
    if p not in sys.path:
        sys.path.insert(0, p)


def pytest_configure(config):
    config.addinivalue_line("markers", "gpu: needs a real MI355X (run with -m gpu on the GPU box)")


def pytest_collection_modifyitems(config, items):
    if torch.cuda.is_available():
        return
    skip = pytest.mark.skip(reason="no GPU in this process")
    for item in items:
        if "gpu" in item.keywords:
            item.add_marker(skip)


def seeded_qkv(seed, B, H, Sq, Sk, D, dtype, rms_norm=False):
    """q,k,v ~ N(0,1) drawn in fp32 on the CPU from one generator (device
    independent), optionally RMS-normalised per head over D, cast to dtype."""
    g = torch.Generator().manual_seed(seed)
    q = torch.randn(B, H, Sq, D, generator=g)
    k = torch.randn(B, H, Sk, D, generator=g)
    v = torch.randn(B, H, Sk, D, generator=g)
    if rms_norm:
        q = q * torch.rsqrt(q.pow(2).mean(-1, keepdim=True) + 1e-6)
        k = k * torch.rsqrt(k.pow(2).mean(-1, keepdim=True) + 1e-6)
    return q.to(dtype), k.to(dtype), v.to(dtype)
