"""Nearest-codeword search under the reference's names (glq/codebook_kernel.py:169-256).

One HIP kernel (`e8_quantize_kernel`) serves both: argmin_k(|c_k|^2 - 2<x, c_k>) in fp32 in
coordinate order with the lowest index on ties, i.e. the arithmetic of the reference's CPU
branch (glq/codebook.py:253-278), which its tensor-core search approximates in fp16.
"""
from __future__ import annotations

import torch

from . import ext


def triton_codebook_nn(x, codebook, codebook_norms, _block_n: int = 0, _block_k: int = 0, out=None):
    """(N, D=8) rows -> (N,) int64 indices of the nearest rows of `codebook` (K, 8).  The tile
    arguments are accepted and ignored; `out`, if given, receives the indices."""
    _, idx = ext.e8_quantize(x, codebook, codebook_norms, return_decoded=False)
    if out is not None:
        out.copy_(idx)
        return out
    return idx


def triton_codebook_nn_decode(x, codebook, codebook_norms, decoded_out=None, idx_out=None):
    """Search and gather in one launch: (decoded (N, 8) fp16, indices (N,) int64)."""
    dec, idx = ext.e8_quantize(x, codebook, codebook_norms, return_decoded=True)
    if idx_out is not None:
        idx_out.copy_(idx)
        idx = idx_out
    if decoded_out is not None:
        decoded_out.copy_(dec)
        dec = decoded_out
    else:
        dec = dec.to(torch.float16)
    return dec, idx
