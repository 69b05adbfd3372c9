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
