"""Shared helpers of the GPU parity tests (imported by tests only)."""
import sys

import numpy as np
import torch


def announce(*a):
    """name the case before touching the GPU, so a fault still tells which case ran"""
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def rel_l2(a, b):
    a = np.asarray(a, dtype=np.float64)
    b = np.asarray(b, dtype=np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))


def to_dev(a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def bf16_dev(bits):
    """uint16 bf16 bit patterns -> torch.bfloat16 tensor on the GPU"""
    return torch.from_numpy(np.ascontiguousarray(bits).view(np.int16)).cuda().view(torch.bfloat16)
