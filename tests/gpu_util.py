"""Shared helpers of the GPU parity tests."""
import os

import numpy as np
import torch

from oracle import glq_oracle as O

DEV = "cuda"


def t(a, dtype=None):
    x = torch.from_numpy(np.ascontiguousarray(a))
    if dtype is not None:
        x = x.to(dtype)
    return x.to(DEV)


def rel(a, b):
    a = a.detach().float().cpu().numpy() if isinstance(a, torch.Tensor) else a
    b = b.detach().float().cpu().numpy() if isinstance(b, torch.Tensor) else b
    return O.rel_fro(a, b)


def e8_table_f16():
    return t(O.e8_table().astype(np.float16))


def say(*a):
    print(*a, flush=True)
