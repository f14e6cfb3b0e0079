"""Shared helpers of the GPU parity tests."""
import sys

import numpy as np
import torch


def say(*a):
    """Names the case before it touches the GPU, so a fault can be traced to it."""
    print("[case]", *a, flush=True)
    sys.stdout.flush()


def draw_roles(seed, B, H, S, p=(0.2, 0.3, 0.5), first_global=True):
    rng = np.random.default_rng(seed)
    r = rng.choice(3, size=(B, H, S), p=p).astype(np.uint8)
    if first_global:
        r[:, :, 0] = 0
    return r


def to_dev(x, dtype=None):
    t = torch.as_tensor(x)
    if dtype is not None:
        t = t.to(dtype)
    return t.cuda()
