"""Host-side block-diagonal Hadamard bookkeeping (integers only, no compute).

Mirrors glq/hadamard.py:133-163 (_block_decompose) and
glq/quantized_linear.py:36-76 (_pack_block_meta, _pack_shard_meta).
"""
from __future__ import annotations

import math
import struct

import torch


def block_decompose(n: int) -> list[int]:
    """n -> descending powers of two summing to n (2688 -> [2048, 512, 128])."""
    blocks = []
    while n > 0:
        p = 1 << (n.bit_length() - 1)
        blocks.append(p)
        n -= p
    return blocks


def next_pow2(n: int) -> int:
    return 1 << (n - 1).bit_length() if n > 0 else 1


def pack_block_meta(block_sizes) -> torch.Tensor:
    """CPU int32 (N, 4): {column offset, bs, log2 bs, 0} per sub-block."""
    meta = torch.zeros((len(block_sizes), 4), dtype=torch.int32, device="cpu")
    off = 0
    for i, bs in enumerate(block_sizes):
        meta[i, 0] = off
        meta[i, 1] = bs
        meta[i, 2] = int(math.log2(bs))
        off += bs
    return meta


def pack_shard_meta(shard_blocks) -> torch.Tensor:
    """Sub-blocks of several output shards with global offsets.  Column 3 holds the
    bit pattern of the host fp32 1/sqrt(bs) for single-block shards (the value the
    per-shard path multiplies by), 0 otherwise."""
    rows = []
    off = 0
    for blocks in shard_blocks:
        single = len(blocks) == 1
        for bs in blocks:
            w = 0
            if single:
                r = torch.tensor(1.0, dtype=torch.float32) / torch.sqrt(
                    torch.tensor(float(bs), dtype=torch.float32))
                w = struct.unpack("<i", struct.pack("<f", float(r)))[0]
            rows.append([off, bs, int(math.log2(bs)), w])
            off += bs
    return torch.tensor(rows, dtype=torch.int32, device="cpu").reshape(-1, 4)


# ---- transforms under the reference's names (glq/hadamard.py:77-131, 166-178) ----------
_block_decompose = block_decompose
_ONES = {}


def _ones(n, device):
    key = (n, str(device))
    t = _ONES.get(key)
    if t is None:
        t = _ONES[key] = torch.ones(n, dtype=torch.float16, device=device)
    return t


def _fht_rows(x: torch.Tensor, block_sizes) -> torch.Tensor:
    """Normalised Walsh-Hadamard transform of every block of the last dim, computed in fp32
    by the output-transform kernel with unit signs; the result has x's dtype and shape."""
    if not x.is_cuda:
        raise RuntimeError("the Hadamard transforms are GPU only here; there is no CPU fallback")
    from . import ext
    n = x.shape[-1]
    rows = x.reshape(-1, n).to(torch.float32).contiguous()
    out = torch.empty_like(rows)
    blocks = [int(b) for b in block_sizes]
    if rows.shape[0]:
        meta = pack_block_meta(blocks).to(x.device) if len(blocks) > 1 else None
        ext.glq_output_rht_blockdiag_cuda(rows, _ones(n, x.device), out, n, n,
                                          torch.tensor(blocks, dtype=torch.int64), meta)
    return out.to(x.dtype).reshape(x.shape)


def fast_hadamard_transform(x: torch.Tensor) -> torch.Tensor:
    """H_n x / sqrt(n) along the last dim, n a power of two (glq/hadamard.py:77-131)."""
    n = x.shape[-1]
    assert n > 0 and (n & (n - 1)) == 0, f"Last dim {n} must be power of 2"
    return _fht_rows(x, [n])


def block_diagonal_fht(x: torch.Tensor, block_sizes) -> torch.Tensor:
    """Independent transforms of consecutive power-of-two blocks of the last dim, written
    back into x, which is also returned (glq/hadamard.py:166-178)."""
    assert sum(int(b) for b in block_sizes) == x.shape[-1], (list(block_sizes), x.shape[-1])
    x.copy_(_fht_rows(x, block_sizes))
    return x
