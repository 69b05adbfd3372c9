"""The Viterbi add-compare-select step under the reference's name
(glq/trellis_step_kernel.py:98-109), on `viterbi_acs_step_kernel`.

`cb` is the reference's `bitshift_codebook` (or anything with its attributes `L`, `K`, `V`
and `recons_state` (V, 1, 2^L) fp32).  Only the 3INST geometry is served: L = 16, V = 1,
K = 1..4; any other raises KeyError, which is what the reference's table lookup raises
for a configuration it has no kernel for, so its caller's loud fallback
(glq/trellis.py:275-293) keeps working.
"""
from __future__ import annotations

import torch

from . import ext


def fused_update(cb, cost, thing, out_row):
    """Drop-in for `bitshift_codebook.update(cost, thing, out_row)`: returns the new cost
    (B, 2^L) fp32 and writes the int32 predecessors into out_row (B, 2^(L-K))."""
    if cb.L != 16 or cb.V != 1 or not 1 <= cb.K <= 4:
        raise KeyError((cb.V, cb.K * cb.V))
    lut = cb.recons_state.reshape(-1)
    x = thing.reshape(-1).to(torch.float16)
    return ext.viterbi_acs_step(cost, x.contiguous(), lut.to(torch.float32).contiguous(), cb.K, out_row)
