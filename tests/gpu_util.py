"""Helpers shared by the GPU parity tests."""

import sys

import pytest
import torch


def require_gpu():
    if not torch.cuda.is_available():
        pytest.skip("needs a ROCm GPU")
    return torch.device("cuda:0")


def announce(*what):
    """Name the case before launching, so a faulting run still tells which case it was."""
    print("[case]", *what, flush=True)
    sys.stdout.flush()


def spiked_logits(n, v, scale, dtype, seed, device):
    g = torch.Generator(device="cpu").manual_seed(seed)
    x = torch.randn(n, v, generator=g) * scale
    rows = torch.rand(n, generator=g) < 0.05
    cols = torch.randint(0, v, (n,), generator=g)
    x[rows, cols[rows]] += 15.0
    return x.to(dtype).to(device)
