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


_KEPT = {}


def td(a):
    """Device copy of a numpy array, one per array object: every call returns the same tensor, so
    that what the load-time step derived from its memory (folded E8 streams) is found again."""
    hit = _KEPT.get(id(a))
    if hit is None or hit[0] is not a:
        hit = _KEPT[id(a)] = (a, t(a))
    return hit[1]


def e8_prepared(ext, cb, q1, q2=None, q3=None, q4=None, cb2=None):
    """The index arrays on the device, through the library's load-time step (ext.e8_prepare)."""
    qs = [None if q is None else td(q) for q in (q1, q2, q3, q4)]
    ext.e8_prepare(qs[0], cb, qs[1], cb2 if cb2 is not None else cb, qs[2], qs[3])
    return qs


def rel(a, b):
    a = a.detach().float().cpu().numpy() if isinstance(a, torch.Tensor) else a
    b = b.detach().float().cpu().numpy() if isinstance(b, torch.Tensor) else b
    return O.rel_fro(a, b)


_E8_TABLE = []


def e8_table_f16():
    """The shell table on the device, one tensor per process (layers share their table)."""
    if not _E8_TABLE:
        _E8_TABLE.append(t(O.e8_table().astype(np.float16)))
    return _E8_TABLE[0]


def say(*a):
    print(*a, flush=True)
