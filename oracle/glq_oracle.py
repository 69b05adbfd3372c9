"""CPU restatement of GLQ's quantized-linear forward -- TEST INFRASTRUCTURE ONLY.

This module is the checker for the HIP kernels.  It is imported by ``tests/``,
``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of ``bench.py`` and by
nothing else: the product package never imports it and has no CPU fallback.

Everything is numpy (integer/byte work) with fp32 arithmetic in the same order as
the reference's CPU path.  Each function cites the reference lines it restates
(paths are relative to the reference checkout).

Pinned by (see tests/test_oracle_*.py):
  fht / block_diag_fht   Sylvester closed form H[i,j]=(-1)^popcount(i&j)/sqrt(n) by
                         brute-force matmul, involution, Parseval, [3,1]->[4,2]/sqrt2
                         (reference tests/test_hadamard.py:15-41)
  block_decompose, meta  doctest values 2688->[2048,512,128], 5376->[4096,1024,256]
                         (glq/hadamard.py:136-139,156-159), tests/test_rht.py:50-57
  e8 table               sha256 of the fp32 bytes, shell counts, lattice membership
  e8_dequant_matmul      naive gather+GEMM, indices 0 / 65535, inv_rs=0 == 1 stage
                         (tests/test_inference_kernel.py:36-47,133-147,245-254)
  decode_3inst           six known answers + sha256 of the whole 65536-entry LUT
  trellis layout/decode  golden vectors written from the reference's pack_layer /
                         decode_layer (tests/golden/), plus a second, independent
                         lane-walk formulation in the tests
  viterbi / e8 nearest   golden state/index sequences from the reference encoders
  e8_embedding_rows      closed form: brute-force Sylvester matrix product on small n, and
                         equality with row-by-row (one-hot) use of e8_dequant + fht
  linear forwards        golden end-to-end outputs from E8RHTLinear.forward (CPU)
  moe_trellis_forward    no golden vector exists (the reference tests only the op's schema,
                         tests/test_glq_vllm.py:595-640): pinned as a composition -- one expert
                         with weight 1 equals down(act(gate) * up) built from the pinned
                         trellis_linear_forward and activation values computed with math.exp /
                         math.tanh in the test, linearity in the routing weights, invariance
                         under reordering a token's choices, out-of-range expert ids
                         contributing nothing, known activation values (silu(1), gelu(1), relu2)
"""
from __future__ import annotations

import math
import os

import numpy as np

TD = 16                      # trellis tile edge (glq/trellis.py:39)
L_STATE = 16                 # trellis state width in bits

_DATA = os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "glq_amd", "data")


# --------------------------------------------------------------------------- #
# Hadamard                                                                     #
# --------------------------------------------------------------------------- #
def block_decompose(n: int) -> list[int]:
    """n -> descending powers of two summing to n (glq/hadamard.py:133-146)."""
    out = []
    while n > 0:
        p = 1 << (n.bit_length() - 1)
        out.append(p)
        n -= p
    return out


def next_pow2(n: int) -> int:
    """glq/rht.py:10-11."""
    return 1 << (n - 1).bit_length() if n > 0 else 1


def pack_block_meta(blocks) -> np.ndarray:
    """(N,4) int32 rows {offset, bs, log2 bs, 0} (glq/quantized_linear.py:36-51)."""
    meta = np.zeros((len(blocks), 4), dtype=np.int32)
    off = 0
    for i, bs in enumerate(blocks):
        meta[i] = (off, bs, int(math.log2(bs)), 0)
        off += bs
    return meta


def pack_shard_meta(shard_blocks) -> np.ndarray:
    """Rows for several output shards with global offsets; column 3 holds the
    bit pattern of the host fp32 1/sqrt(bs) for single-block shards, else 0
    (glq/quantized_linear.py:54-76)."""
    rows = []
    off = 0
    for blocks in shard_blocks:
        single = len(blocks) == 1
        for bs in blocks:
            w = 0
            if single:
                r = np.float32(1.0) / np.sqrt(np.float32(bs))
                w = int(np.array([r], dtype=np.float32).view(np.int32)[0])
            rows.append([off, bs, int(math.log2(bs)), w])
            off += bs
    return np.array(rows, dtype=np.int32).reshape(-1, 4)


def fht(x: np.ndarray) -> np.ndarray:
    """Normalised Walsh-Hadamard transform along the last axis, fp32, butterflies
    in ascending distance, one division by sqrt(n) at the end
    (glq/hadamard.py:10-28)."""
    x = np.array(x, dtype=np.float32, copy=True)
    n = x.shape[-1]
    assert n > 0 and (n & (n - 1)) == 0, n
    lead = x.shape[:-1]
    h = 1
    while h < n:
        v = x.reshape(*lead, n // (2 * h), 2, h)
        a = v[..., 0, :].copy()
        b = v[..., 1, :].copy()
        v[..., 0, :] = a + b
        v[..., 1, :] = a - b
        x = v.reshape(*lead, n)
        h *= 2
    return (x / np.float32(math.sqrt(n))).astype(np.float32)


def block_diag_fht(x: np.ndarray, blocks) -> np.ndarray:
    """Independent FHT per power-of-two block (glq/hadamard.py:166-178)."""
    x = np.array(x, dtype=np.float32, copy=True)
    off = 0
    for bs in blocks:
        x[..., off:off + bs] = fht(x[..., off:off + bs])
        off += bs
    return x


def rht_signs(m_pad: int, n_pad: int, seed: int = 42):
    """Seeded +-1 vectors, SU drawn first then SV (glq/rht.py:81-88).  The draw is
    torch's CPU generator; there is no other definition of it."""
    import torch
    gen = torch.Generator(device="cpu").manual_seed(seed)
    su = (torch.randint(0, 2, (m_pad,), generator=gen).float() * 2 - 1).numpy()
    sv = (torch.randint(0, 2, (n_pad,), generator=gen).float() * 2 - 1).numpy()
    return su.astype(np.float32), sv.astype(np.float32)


def rht_transform_weights(W: np.ndarray, su, sv, blocks_m, blocks_n) -> np.ndarray:
    """W~ = H_m diag(su) W diag(sv) H_n on the zero-padded matrix
    (glq/rht.py:102-122)."""
    m_pad, n_pad = sum(blocks_m), sum(blocks_n)
    Wp = np.zeros((m_pad, n_pad), dtype=np.float32)
    Wp[:W.shape[0], :W.shape[1]] = W
    Wt = block_diag_fht(Wp * sv[None, :], blocks_n)
    Wt = Wt.T.copy() * su[None, :]
    Wt = block_diag_fht(Wt, blocks_m).T.copy()
    return Wt


# --------------------------------------------------------------------------- #
# E8 shell codebook                                                            #
# --------------------------------------------------------------------------- #
def e8_nibbles() -> np.ndarray:
    """The 65536-entry table as shipped data: one uint32 per row, nibble i holds
    round(2 v_i)+6 (glq/codebook.py:102-115).  Row order is data, not derivable
    (glq/codebook.py:156 sorts with an unstable argsort)."""
    return np.load(os.path.join(_DATA, "e8_shell_nibbles.npy"))


def e8_unpack_nibbles(packed: np.ndarray) -> np.ndarray:
    """uint32 rows -> (K,8) fp32, v_i = nibble_i*0.5-3 (glq/codebook.py:107)."""
    p = packed.astype(np.uint32)
    cols = [((p >> np.uint32(4 * i)) & np.uint32(15)).astype(np.float32) * np.float32(0.5)
            - np.float32(3.0) for i in range(8)]
    return np.stack(cols, axis=1)


_E8 = None


def e8_table() -> np.ndarray:
    global _E8
    if _E8 is None:
        _E8 = e8_unpack_nibbles(e8_nibbles())
    return _E8


def e8_decode(idx: np.ndarray, table: np.ndarray | None = None) -> np.ndarray:
    """Gather rows by the unsigned 16-bit pattern of the stored int16
    (glq/codebook.py:280-282, glq/inference_kernel.py:1207-1208)."""
    t = e8_table() if table is None else table
    return t[np.asarray(idx).astype(np.int64) & 0xFFFF]


def e8_quantize(x: np.ndarray, table: np.ndarray | None = None, chunk: int = 4096):
    """Nearest row by argmin(-2<x,c>+|c|^2), lowest index on ties, fp32
    (glq/codebook.py:253-278, CPU branch).  Returns (decoded, idx int64)."""
    t = e8_table() if table is None else table
    tt = np.ascontiguousarray(t.T)
    norms = (t * t).sum(-1).astype(np.float32)
    x = np.asarray(x, dtype=np.float32)
    out = np.empty(x.shape[0], dtype=np.int64)
    for s in range(0, x.shape[0], chunk):
        d = np.float32(-2.0) * (x[s:s + chunk] @ tt) + norms
        out[s:s + chunk] = d.argmin(-1)
    return t[out], out


def e8_dequant(Qidxs, Qidxs2=None, inv_rs=0.0, Qidxs3=None, inv_rs2=0.0,
               Qidxs4=None, inv_rs3=0.0, table=None, table2=None) -> np.ndarray:
    """RHT-domain weight (m_pad, n_pad) before Wscale:
    cb[i1] + cb2[i2]*inv_rs [+ cb[i3]*inv_rs2 + cb[i4]*inv_rs3], fp32
    (glq/quantized_linear.py:1177-1194)."""
    m, nb = Qidxs.shape
    W = e8_decode(Qidxs.reshape(-1), table).reshape(m, nb * 8)
    if Qidxs2 is not None and inv_rs != 0.0:
        t2 = table if table2 is None else table2
        W = W + e8_decode(Qidxs2.reshape(-1), t2).reshape(m, nb * 8) * np.float32(inv_rs)
        for q, s in ((Qidxs3, inv_rs2), (Qidxs4, inv_rs3)):
            if q is None or s == 0.0:
                break
            W = W + e8_decode(q.reshape(-1), table).reshape(m, nb * 8) * np.float32(s)
    return W.astype(np.float32)


def e8_dequant_matmul(x_rht, Qidxs, wscale, Qidxs2=None, inv_rs=0.0, table=None,
                      table2=None) -> np.ndarray:
    """y_rht = x_rht @ W^T * Wscale (glq/inference_kernel.py:1194-1216)."""
    W = e8_dequant(Qidxs, Qidxs2, inv_rs, table=table, table2=table2)
    return (np.asarray(x_rht, dtype=np.float32) @ W.T * np.float32(wscale)).astype(np.float32)


def e8_embedding_rows(ids, Qidxs, sv, wscale_rows, Qidxs2=None, inv_rs_rows=None, embedding_dim=None,
                      embed_scale=1.0, table=None, table2=None) -> np.ndarray:
    """Quantized-embedding lookup, fp32 (glq/quantized_linear.py:1277-1340):
    deq = cb[q1[id]] (+ cb2[q2[id]] * inv_rs[id]); deq *= Wscale[id]; FHT over the padded
    row; * sv; * embed_scale; trimmed to embedding_dim."""
    ids = np.asarray(ids, dtype=np.int64)
    flat = ids.reshape(-1)
    nb = Qidxs.shape[1]
    n_pad = nb * 8
    deq = e8_decode(Qidxs[flat].reshape(-1), table).reshape(flat.shape[0], n_pad).astype(np.float32)
    if Qidxs2 is not None and inv_rs_rows is not None:
        t2 = table if table2 is None else table2
        deq2 = e8_decode(Qidxs2[flat].reshape(-1), t2).reshape(flat.shape[0], n_pad).astype(np.float32)
        deq = deq + deq2 * np.asarray(inv_rs_rows, dtype=np.float32)[flat][:, None]
    deq = deq * np.asarray(wscale_rows, dtype=np.float32)[flat][:, None]
    deq = fht(deq) * np.asarray(sv, dtype=np.float32)
    if embed_scale != 1.0:
        deq = deq * np.float32(embed_scale)
    d = n_pad if embedding_dim is None else embedding_dim
    return deq[:, :d].reshape(*ids.shape, d).astype(np.float32)


def e8_quantize_layer(W, bpw=2, seed=42, block_diagonal=True):
    """RHT + nearest-E8 rounding with an identity Hessian, i.e.
    quantize_layer_e8_shell_rht with H=I, where the LDLQ feedback term is zero
    (glq/quantize_model.py:445-651, glq/ldlq.py:90-197).  Returns the artifact
    dict {Qidxs[,Qidxs2,inv_resid_scale],SU,SV,Wscale} and the RHT-domain W_hat."""
    m, n = W.shape
    if block_diagonal:
        bm, bn = block_decompose(m), block_decompose(n)
    else:
        bm, bn = [next_pow2(m)], [next_pow2(n)]
    su, sv = rht_signs(sum(bm), sum(bn), seed)
    Wt = rht_transform_weights(np.asarray(W, np.float32), su, sv, bm, bn)
    rms = float(np.sqrt((Wt.astype(np.float32) ** 2).mean(dtype=np.float32)))
    wscale = rms * 1.0 if rms > 1e-10 else 1.0           # opt_scale = 1.0 (table file)
    Wr = (Wt / np.float32(wscale)).astype(np.float32)
    mp, npad = Wr.shape
    v = Wr.reshape(mp * npad // 8, 8)
    dec1, i1 = e8_quantize(v)
    art = {"Qidxs": i1.reshape(mp, npad // 8).astype(np.uint16).view(np.int16),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
           "Wscale": np.float32(wscale), "blocks_m": bm, "blocks_n": bn}
    hat = dec1
    if bpw == 4:
        rs = 3.0                                           # resid_scale (table file)
        dec2, i2 = e8_quantize((v - dec1) * np.float32(rs))
        art["Qidxs2"] = i2.reshape(mp, npad // 8).astype(np.uint16).view(np.int16)
        art["inv_resid_scale"] = np.float32(1.0 / rs)
        hat = dec1 + dec2 / np.float32(rs)
    elif bpw != 2:
        raise ValueError(bpw)
    return art, hat.reshape(mp, npad)


# --------------------------------------------------------------------------- #
# Trellis 3INST                                                                #
# --------------------------------------------------------------------------- #
def decode_3inst(states: np.ndarray) -> np.ndarray:
    """16-bit state -> fp16 weight: h = s*89226354+64248484 (mod 2^32),
    r = (h & 0x8FFF8FFF) ^ 0x3B603B60, w = fp16(r>>16) + fp16(r&0xFFFF) with the
    sum rounded once to fp16 (glq/trellis.py:122-134)."""
    s = np.asarray(states).astype(np.uint64) & np.uint64(0xFFFFFFFF)
    h = (s * np.uint64(89226354) + np.uint64(64248484)) & np.uint64(0xFFFFFFFF)
    r = (h & np.uint64(0x8FFF8FFF)) ^ np.uint64(0x3B603B60)
    hi = (r >> np.uint64(16)).astype(np.uint16).view(np.float16)
    lo = (r & np.uint64(0xFFFF)).astype(np.uint16).view(np.float16)
    return (hi + lo).astype(np.float16)


_LUT = None


def lut_3inst() -> np.ndarray:
    global _LUT
    if _LUT is None:
        _LUT = decode_3inst(np.arange(1 << L_STATE))
    return _LUT


def trellis_opt_scale() -> float:
    """1/(0.9*rms(lut)) (glq/trellis.py:561)."""
    lut = lut_3inst().astype(np.float64)
    return 1.0 / (math.sqrt((lut * lut).mean()) * 0.9)


# step t of a tile's trellis -> position in the 16x16 tile (row-major).
# glq/trellis.py:99-101: arange(256).reshape(2,8,2,4,2).permute(1,3,2,0,4)
PERMUTE = np.arange(256).reshape(2, 8, 2, 4, 2).transpose(1, 3, 2, 0, 4).reshape(-1)
INV_PERMUTE = np.zeros(256, dtype=np.int64)
INV_PERMUTE[PERMUTE] = np.arange(256)


def trellis_bits_from_packed(packed: np.ndarray) -> int:
    """K = packed width / 16 (glq/csrc/glq_trellis.cu:862-869)."""
    w = packed.shape[-1]
    if w % 16 != 0 or not 1 <= w // 16 <= 4:
        raise ValueError(f"packed width {w} is not 16*K with K in 1..4 bits/weight")
    return w // 16


def kernel_to_stream_bytes(packed: np.ndarray, m: int, n: int, K: int) -> np.ndarray:
    """Kernel-layout int16 blob -> (num_tiles, 32K) bytes, row s of a tile holding
    stream bits [8s, 8s+8) MSB first; tiles row-major over (m/16, n/16).
    Inverse of kernel_tile_flip(forward=True) composed with the big-endian int16
    packing of pack_trellis (glq/trellis.py:486-505, 580-602)."""
    b = np.ascontiguousarray(packed).view(np.uint8).reshape(m // 32, n // 32, 32, 2, 2, K)
    b = b[..., ::-1]                                   # chunk is little-endian
    # (mp, kp, lane, ks, ms, c) -> (mp, ms, kp, ks, lane, c)
    b = b.transpose(0, 4, 1, 3, 2, 5)
    return np.ascontiguousarray(b).reshape((m // 16) * (n // 16), 32 * K)


def stream_bytes_to_kernel(sb: np.ndarray, m: int, n: int, K: int) -> np.ndarray:
    """Inverse of kernel_to_stream_bytes -> int16 ((m/16)(n/16), 16K)."""
    b = sb.reshape(m // 32, 2, n // 32, 2, 32, K).transpose(0, 2, 4, 3, 1, 5)[..., ::-1]
    return np.ascontiguousarray(b).reshape(-1).view(np.int16).reshape((m // 16) * (n // 16), 16 * K)


def unpack_states(sb: np.ndarray, K: int) -> np.ndarray:
    """(T, 32K) stream bytes -> (T, 256) states; state t = cyclic stream bits
    [K t, K t + 16) MSB first (glq/trellis.py:507-523)."""
    bits = np.unpackbits(sb, axis=1)                              # MSB first
    bits = np.concatenate([bits, bits[:, :L_STATE]], axis=1).astype(np.int64)
    T = sb.shape[0]
    idx = (np.arange(256)[:, None] * K + np.arange(L_STATE)[None, :])   # (256,16)
    w = (1 << np.arange(L_STATE - 1, -1, -1)).astype(np.int64)
    return (bits[:, idx] * w).sum(-1).reshape(T, 256)


def unpack_states_fast(sb: np.ndarray, K: int) -> np.ndarray:
    """Same result as unpack_states, computed with 32-bit byte windows instead of a
    bit array (an order of magnitude faster; used for full-size layers).  State t
    starts at stream bit K t = 8 q + r: take bytes q..q+2 as a 24-bit big-endian
    window and drop the 8 - r low bits."""
    T, nbytes = sb.shape
    ext = np.concatenate([sb, sb[:, :3]], axis=1).astype(np.uint32)
    start = np.arange(256) * K
    q, r = start >> 3, start & 7
    win = (ext[:, q] << np.uint32(16)) | (ext[:, q + 1] << np.uint32(8)) | ext[:, q + 2]
    return ((win >> (8 - r).astype(np.uint32)[None, :]) & np.uint32(0xFFFF)).astype(np.int64)


def pack_states(states: np.ndarray, K: int) -> np.ndarray:
    """(T,256) states of a valid tail-biting path -> (T, 32K) stream bytes.
    Bit K t + i of the stream is bit (15-i) of state t; consecutive states must
    overlap (glq/trellis.py:486-505, the assert at 495-496, and cyclically)."""
    s = np.asarray(states).astype(np.int64)
    nxt = np.roll(s, -1, axis=1)
    if not np.array_equal(s & ((1 << (L_STATE - K)) - 1), nxt >> K):
        raise ValueError("states are not a cyclic shift-register path")
    top = (s >> (L_STATE - K)) & ((1 << K) - 1)                   # first K bits of each window
    bits = ((top[:, :, None] >> np.arange(K - 1, -1, -1)[None, None, :]) & 1).astype(np.uint8)
    return np.packbits(bits.reshape(s.shape[0], 256 * K), axis=1)


def tiles_to_matrix(tiles: np.ndarray, m: int, n: int) -> np.ndarray:
    """(T,256) per-step values -> (m,n): undo PERMUTE, re-tile
    (glq/trellis.py:641-643)."""
    nat = tiles[:, INV_PERMUTE]
    return nat.reshape(m // 16, n // 16, 16, 16).transpose(0, 2, 1, 3).reshape(m, n)


def matrix_to_tiles(W: np.ndarray) -> np.ndarray:
    """(m,n) -> (T,256) in trellis-step order (glq/trellis.py:679-681)."""
    m, n = W.shape
    nat = W.reshape(m // 16, 16, n // 16, 16).transpose(0, 2, 1, 3).reshape(-1, 256)
    return nat[:, PERMUTE]


def trellis_states(packed: np.ndarray, m: int, n: int, fast: bool = False) -> np.ndarray:
    K = trellis_bits_from_packed(packed)
    if packed.shape[0] != (m // 16) * (n // 16):
        raise ValueError("packed rows != (m/16)*(n/16)")
    sb = kernel_to_stream_bytes(packed, m, n, K)
    return unpack_states_fast(sb, K) if fast else unpack_states(sb, K)


def decode_layer(packed: np.ndarray, m: int, n: int, fast: bool = False) -> np.ndarray:
    """Kernel-layout packed int16 -> normalised hatW (m,n) fp16-exact values in
    fp32 (glq/trellis.py:629-643).  fast=True uses unpack_states_fast and works in
    strips of 32 rows to bound memory on full-size layers."""
    if not fast:
        st = trellis_states(packed, m, n)
        return tiles_to_matrix(lut_3inst()[st].astype(np.float32), m, n)
    lut = lut_3inst().astype(np.float32)
    out = np.empty((m, n), dtype=np.float32)
    per_strip = 2 * (n // 16)
    rows = 256                                                   # strip height per pass
    for r0 in range(0, m, rows):
        h = min(rows, m - r0)
        sub = packed[(r0 // 32) * per_strip:((r0 + h) // 32) * per_strip]
        st = trellis_states(sub, h, n, fast=True)
        out[r0:r0 + h] = tiles_to_matrix(lut[st], h, n)
    return out


def decode_layer_nstage(packed_list, cum_inv_rs, m, n) -> np.ndarray:
    """sum_s decode(stage_s)*cum_inv_rs[s], fp32 (glq/trellis.py:923-933)."""
    out = None
    for p, s in zip(packed_list, cum_inv_rs):
        d = decode_layer(p, m, n) * np.float32(s)
        out = d if out is None else out + d
    return out


def pack_layer_from_states(states: np.ndarray, m: int, n: int, K: int) -> np.ndarray:
    """(T,256) step-ordered states -> kernel-layout int16 (glq/trellis.py:608-619)."""
    return stream_bytes_to_kernel(pack_states(states, K), m, n, K)


def random_packed(m: int, n: int, K: int, seed: int = 0) -> np.ndarray:
    """Uniform random bits: every bit pattern is a valid tail-biting stream."""
    rng = np.random.default_rng(seed)
    return rng.integers(-32768, 32768, size=((m // 16) * (n // 16), 16 * K), dtype=np.int16)


# ---- Viterbi encoder (inputs for realistic-quantization tests) ------------- #
def _viterbi(X: np.ndarray, K: int, lut: np.ndarray, overlap=None) -> np.ndarray:
    """X (T, B) fp32 -> states (T, B).  glq/trellis.py:253-296: cost over all 2^16
    states, predecessor group min with lowest-k tie-break, optional tail-biting
    constraint on the first and last state."""
    T, B = X.shape
    S = 1 << L_STATE
    G = 1 << (L_STATE - K)
    lutf = lut.astype(np.float32)[None, :]
    cost = (lutf - X[0][:, None]) ** 2
    inf = np.float32(np.inf)
    if overlap is not None:
        mask = np.full((B, S), inf, dtype=np.float32)
        allow = (overlap[:, None].astype(np.int64) << K) + np.arange(1 << K)[None, :]
        np.put_along_axis(mask, allow, 0.0, axis=1)
        cost = np.minimum(cost + mask, inf)
    from_state = np.empty((T, B, G), dtype=np.int32)
    base = np.arange(G, dtype=np.int64)[None, :]
    for i in range(1, T):
        c = cost.reshape(B, 1 << K, G)
        k = c.argmin(axis=1)                                   # first minimum = lowest k
        best = np.take_along_axis(c, k[:, None, :], axis=1)[:, 0, :]
        from_state[i] = (base + (k.astype(np.int64) << (L_STATE - K))).astype(np.int32)
        err = (lutf - X[i][:, None]) ** 2
        cost = err + np.repeat(best, 1 << K, axis=1)
    if overlap is not None:
        mask = np.full((B, S), inf, dtype=np.float32)
        allow = overlap[:, None].astype(np.int64) + (np.arange(1 << K)[None, :] << (L_STATE - K))
        np.put_along_axis(mask, allow, 0.0, axis=1)
        cost = np.minimum(cost + mask, inf)
    final = np.empty((T, B), dtype=np.int64)
    final[T - 1] = cost.argmin(-1)
    for i in range(T - 1, 0, -1):
        final[i - 1] = np.take_along_axis(from_state[i], (final[i] >> K)[:, None], axis=1)[:, 0]
    return final


def trellis_quantize_tiles(tiles: np.ndarray, K: int, chunk: int = 64):
    """(B,256) fp32 tiles (already in step order) -> (hat (B,256) fp32, states (B,256)).
    Two-pass tail-biting search of glq/trellis.py:467-484 with the fp16 cast of
    line 468."""
    lut = lut_3inst()
    outs, outh = [], []
    for s in range(0, tiles.shape[0], chunk):
        X = tiles[s:s + chunk].astype(np.float16).astype(np.float32).T.copy()   # (256, b)
        T = X.shape[0]
        rolled = np.roll(X, T // 2, axis=0)
        st1 = _viterbi(rolled, K, lut)
        overlap = st1[T // 2] >> K
        st = _viterbi(X, K, lut, overlap=overlap)
        outs.append(st.T.copy())
        outh.append(lut[st].astype(np.float32).T.copy())
    return np.concatenate(outh), np.concatenate(outs)


def trellis_quantize_layer(W, K=4, seed=42, K2=None, resid_scale=None):
    """RHT + tile-trellis quantisation with an identity Hessian (LDLQ feedback is
    zero), glq/trellis.py:649-688, 832-914, 936-993.  Returns artifacts and the
    normalised RHT-domain reconstruction."""
    m, n = W.shape
    bm, bn = block_decompose(m), block_decompose(n)
    su, sv = rht_signs(m, n, seed)
    Wt = rht_transform_weights(np.asarray(W, np.float32), su, sv, bm, bn)
    rms = float(np.sqrt((Wt ** 2).mean(dtype=np.float32)))
    wscale = rms * trellis_opt_scale()
    Wr = (Wt / np.float32(wscale)).astype(np.float32)
    tiles = matrix_to_tiles(Wr)
    hat, st = trellis_quantize_tiles(tiles, K)
    art = {"trellis_packed": pack_layer_from_states(st, m, n, K),
           "SU": su.astype(np.float16), "SV": sv.astype(np.float16),
           "Wscale": np.float32(wscale), "blocks_m": bm, "blocks_n": bn}
    recon = hat
    if K2 is not None:
        resid = tiles - hat
        if resid_scale is None:
            cal = {1: 1.29, 2: 1.06, 3: 0.94, 4: 0.74}[K2]     # glq/trellis.py:829
            # the reference fits the ratio on the first column block it visits
            # (the last 16 columns); with H = I any block is an equally valid
            # estimate, and the value is stored, so decode does not depend on it
            r_t = float(np.sqrt((tiles.astype(np.float32) ** 2).mean()))
            r_r = max(float(np.sqrt((resid.astype(np.float32) ** 2).mean())), 1e-12)
            resid_scale = r_t / r_r * cal
        hat2, st2 = trellis_quantize_tiles(resid * np.float32(resid_scale), K2)
        art["trellis_packed2"] = pack_layer_from_states(st2, m, n, K2)
        art["inv_resid_scale2"] = np.float32(1.0 / resid_scale)
        recon = hat + hat2 * np.float32(1.0 / resid_scale)
    return art, tiles_to_matrix(recon, m, n)


# --------------------------------------------------------------------------- #
# Layer forwards (the reference's CPU dequantize-then-matmul path)             #
# --------------------------------------------------------------------------- #
def linear_forward_rht(x, W_rht, su, sv, blocks_n, blocks_m, in_features, out_features,
                       bias=None):
    """y = (H_m(H_n(pad(x)*sv) @ W_rht^T)) * su, sliced (glq/quantized_linear.py:
    1003-1010 and 1149-1154, 1195, 1225-1231).  W_rht already carries Wscale."""
    x = np.asarray(x, dtype=np.float32).reshape(-1, in_features)
    n_pad, m_pad = sum(blocks_n), sum(blocks_m)
    xp = np.zeros((x.shape[0], n_pad), dtype=np.float32)
    xp[:, :in_features] = x
    x_rht = block_diag_fht(xp * np.asarray(sv, np.float32)[None, :], blocks_n)
    y_rht = (x_rht @ W_rht.T).astype(np.float32)
    y = block_diag_fht(y_rht, blocks_m) * np.asarray(su, np.float32)[None, :]
    y = y[:, :out_features]
    if bias is not None:
        y = y + np.asarray(bias, np.float32)[None, :]
    return y.astype(np.float32)


def dense_weight(W_rht, su, sv, blocks_m, blocks_n, out_features, in_features):
    """Weight-domain matrix of an RHT-domain weight that already carries Wscale:
    `su * H_m( (H_n(rows) * sv) columns )`, cut to (out, in)  (E8RHTLinear.dequantize,
    glq/quantized_linear.py:1250-1265; dequantize_glq_weight, glq_vllm/dequant.py:46-55;
    the reference has it for whole power-of-two transforms only, block-diagonal follows
    glq/hadamard.py:166-178)."""
    A = block_diag_fht(np.asarray(W_rht, np.float32), blocks_n) * np.asarray(sv, np.float32)[None, :]
    B = block_diag_fht(np.ascontiguousarray(A.T), blocks_m).T * np.asarray(su, np.float32)[:, None]
    return np.ascontiguousarray(B[:out_features, :in_features]).astype(np.float32)


def trellis_linear_forward(x, art, in_features, out_features):
    """E8RHTLinear._forward_trellis CPU fallback (glq/quantized_linear.py:986-1010)."""
    m, n = out_features, in_features
    if "trellis_packed2" in art:
        Wn = decode_layer_nstage([art["trellis_packed"], art["trellis_packed2"]],
                                 [1.0, float(art["inv_resid_scale2"])], m, n)
    else:
        Wn = decode_layer(art["trellis_packed"], m, n)
    W = (Wn.astype(np.float32) * np.float32(art["Wscale"])).astype(np.float32)
    return linear_forward_rht(x, W, art["SU"].astype(np.float32), art["SV"].astype(np.float32),
                              art["blocks_n"], art["blocks_m"], n, m)


def e8_linear_forward(x, art, in_features, out_features, table=None):
    """E8RHTLinear.forward CPU path: the weight is re-decoded on every call and
    Wscale multiplies the product (glq/quantized_linear.py:1149-1154, 1175-1195,
    1225-1231)."""
    W = e8_dequant(art["Qidxs"], art.get("Qidxs2"), float(art.get("inv_resid_scale", 0.0)),
                   table=table)
    x = np.asarray(x, dtype=np.float32).reshape(-1, in_features)
    bn, bm = art["blocks_n"], art["blocks_m"]
    n_pad, m_pad = sum(bn), sum(bm)
    xp = np.zeros((x.shape[0], n_pad), dtype=np.float32)
    xp[:, :in_features] = x
    x_rht = block_diag_fht(xp * art["SV"].astype(np.float32)[None, :], bn)
    y_rht = (x_rht @ W.T * np.float32(art["Wscale"])).astype(np.float32)
    y = block_diag_fht(y_rht, bm) * art["SU"].astype(np.float32)[None, :]
    return y[:, :out_features].astype(np.float32)


# --------------------------------------------------------------------------- #
# Routed experts of a mixture-of-experts layer                                 #
# --------------------------------------------------------------------------- #
def gated_activation(h, intermediate, act):
    """act(gate) * up with gate = h[:, :intermediate], up = h[:, intermediate:2*intermediate]:
    0 SiLU, 1 GELU (tanh form), 2 squared ReLU (glq/csrc/glq_cuda.cu:4540-4559)."""
    h = np.asarray(h, np.float32)
    g, up = h[:, :intermediate], h[:, intermediate:2 * intermediate]
    if act == 0:
        a = g / (np.float32(1.0) + np.exp(-g))
    elif act == 1:
        a = np.float32(0.5) * g * (np.float32(1.0) + np.tanh(np.float32(0.7978845608028654)
                                                           * (g + np.float32(0.044715) * g * g * g)))
    elif act == 2:
        r = np.maximum(g, np.float32(0.0))
        a = r * r
    else:
        raise ValueError(act)
    return (a * up).astype(np.float32)


def moe_dense_experts(arts, out_features, in_features):
    """RHT-domain fp32 weight (with Wscale) of every expert of one projection, decoded once."""
    out = []
    for art in arts:
        if "trellis_packed2" in art:
            Wn = decode_layer_nstage([art["trellis_packed"], art["trellis_packed2"]],
                                     [1.0, float(art["inv_resid_scale2"])], out_features, in_features)
        else:
            Wn = decode_layer(art["trellis_packed"], out_features, in_features, fast=True)
        out.append((Wn.astype(np.float32) * np.float32(art["Wscale"])).astype(np.float32))
    return out


def moe_trellis_forward(x, topk_ids, topk_weights, w13_arts, w2_arts, hidden, intermediate, act,
                        w13_dense=None, w2_dense=None):
    """glq_fused_moe_trellis_3inst_cuda restated token by token (glq/csrc/glq_cuda.cu:5030-5250):
    out[t] = sum_j w[t, j] * w2_e(act(gate) * up), (gate | up) = w13_e(x[t]), e = ids[t, j]; the
    per-slot results are rounded to fp16 after each output transform and after the activation
    (h_w13, h_act, expert_out are fp16 tensors there), the weighted sum runs over j in order
    in fp32 (glq_moe_weighted_scatter_reduce_kernel, :4520-4537) and is rounded to fp16.
    Expert ids outside [0, E) contribute nothing (pad slots, m_indices = -1).  *_arts: one
    artifact dict per expert, as for trellis_linear_forward."""
    x = np.asarray(x, np.float32).reshape(-1, hidden)
    ids = np.asarray(topk_ids).reshape(x.shape[0], -1)
    w = np.asarray(topk_weights, np.float32).reshape(ids.shape)
    E = len(w13_arts)
    if w13_dense is None:
        w13_dense = moe_dense_experts(w13_arts, 2 * intermediate, hidden)
    if w2_dense is None:
        w2_dense = moe_dense_experts(w2_arts, hidden, intermediate)
    f16 = lambda a: a.astype(np.float16).astype(np.float32)
    out = np.zeros((x.shape[0], hidden), np.float32)
    for t in range(x.shape[0]):
        acc = np.zeros(hidden, np.float32)
        for j in range(ids.shape[1]):
            e = int(ids[t, j])
            if e < 0 or e >= E:
                continue
            a13, a2 = w13_arts[e], w2_arts[e]
            h = f16(linear_forward_rht(x[t:t + 1], w13_dense[e], a13["SU"].astype(np.float32),
                                       a13["SV"].astype(np.float32), a13["blocks_n"], a13["blocks_m"],
                                       hidden, 2 * intermediate))
            a = f16(gated_activation(h, intermediate, act))
            y = f16(linear_forward_rht(a, w2_dense[e], a2["SU"].astype(np.float32),
                                       a2["SV"].astype(np.float32), a2["blocks_n"], a2["blocks_m"],
                                       intermediate, hidden))
            acc = acc + w[t, j] * y[0]
        out[t] = acc
    return f16(out)


def rel_fro(a, b) -> float:
    a = np.asarray(a, np.float64)
    b = np.asarray(b, np.float64)
    return float(np.linalg.norm(a - b) / max(np.linalg.norm(b), 1e-30))
