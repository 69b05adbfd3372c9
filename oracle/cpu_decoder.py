"""CPU restatement of batch-1 decode through trellis-quantized linears: TEST AND BASELINE
INFRASTRUCTURE ONLY (imported by tests/ and by bench.py's cpu_baseline leg, never by glq_amd/).

Every linear runs the reference's CPU path for a trellis layer -- weight decoded once and cached in
the transform domain, then per call fp32 FHT of x * SV -> fp32 matmul -> FHT -> * SU
(glq/quantized_linear.py:986-1010) -- through `glq_oracle.linear_forward_rht`.  The glue around the
linears is the SmolLM3 decoder layer as transformers' SmolLM3Config describes it (RMSNorm, rotary
embedding skipped on every n-th layer, grouped-query attention on a KV cache, SiLU-gated MLP, tied
output head); the reference has no decoder of its own, its callers are HF models
(glq/hf_integration.py, benchmarks/run_model.py:8).

Pinned by tests/test_oracle_cpu_decoder.py: one-token steps on the cache against a full causal
recompute with dense weight-domain matrices (`glq_oracle.dense_weight`) written out in the test.
"""
from __future__ import annotations

import numpy as np

from . import glq_oracle as O

LINEAR_NAMES = ("q", "k", "v", "o", "gate", "up", "down")


def linear_shapes(hidden, heads, kv_heads, head_dim, ffn):
    """(out, in) of the seven linears of one layer."""
    return {"q": (heads * head_dim, hidden), "k": (kv_heads * head_dim, hidden), "v": (kv_heads * head_dim, hidden),
            "o": (hidden, heads * head_dim), "gate": (ffn, hidden), "up": (ffn, hidden), "down": (hidden, ffn)}


def make_layer(shapes, bits, seed, wscale=0.02 * 0.8933837):
    """One layer's linears from random code bits (every bit pattern is a valid stream): name ->
    (W_rht * Wscale fp32 (m, n), su, sv, blocks_n, blocks_m)."""
    layer = {}
    for j, name in enumerate(LINEAR_NAMES):
        m, n = shapes[name]
        packed = O.random_packed(m, n, bits, seed=seed * 16 + j)
        su, sv = O.rht_signs(m, n, 42 + seed * 16 + j)
        W = (O.decode_layer(packed, m, n, fast=True) * np.float32(wscale)).astype(np.float32)
        layer[name] = (W, su.astype(np.float32), sv.astype(np.float32), O.block_decompose(n), O.block_decompose(m))
    return layer


class CpuDecoder:
    def __init__(self, layers, emb, hidden, heads, kv_heads, head_dim, max_len=64, rms_eps=1e-6, rope_theta=2e6,
                 no_rope_interval=4):
        self.layers, self.emb = layers, np.asarray(emb, np.float32)
        self.hidden, self.heads, self.kv_heads, self.head_dim = hidden, heads, kv_heads, head_dim
        self.eps, self.no_rope_interval = np.float32(rms_eps), no_rope_interval
        inv = 1.0 / (rope_theta ** (np.arange(0, head_dim, 2, dtype=np.float32) / head_dim))
        ang = np.arange(max_len, dtype=np.float32)[:, None] * inv[None]
        ang = np.concatenate([ang, ang], -1)
        self.cos, self.sin = np.cos(ang).astype(np.float32), np.sin(ang).astype(np.float32)
        L = len(layers)
        self.kc = np.zeros((L, kv_heads, max_len, head_dim), np.float32)
        self.vc = np.zeros_like(self.kc)
        self.pos = 0

    def _lin(self, li, name, x):
        W, su, sv, bn, bm = self.layers[li][name]
        return O.linear_forward_rht(x, W, su, sv, bn, bm, W.shape[1], W.shape[0])

    def _norm(self, x):                                       # norm weights are ones (random-init decoder)
        return x / np.sqrt((x * x).mean(-1, keepdims=True, dtype=np.float32) + self.eps)

    def _rope(self, x, pos):                                  # x (H, D)
        d = self.head_dim // 2
        rot = np.concatenate([-x[:, d:], x[:, :d]], -1)
        return x * self.cos[pos][None] + rot * self.sin[pos][None]

    def step(self, tok):
        """Feed one token at the next position; returns the logits (vocab,) fp32."""
        H, KV, D = self.heads, self.kv_heads, self.head_dim
        p = self.pos
        x = self.emb[tok][None].copy()
        for li in range(len(self.layers)):
            h = self._norm(x)
            q = self._lin(li, "q", h).reshape(H, D)
            k = self._lin(li, "k", h).reshape(KV, D)
            v = self._lin(li, "v", h).reshape(KV, D)
            if (li + 1) % self.no_rope_interval != 0:
                q, k = self._rope(q, p), self._rope(k, p)
            self.kc[li, :, p], self.vc[li, :, p] = k, v
            rep = H // KV
            kk = np.repeat(self.kc[li, :, :p + 1], rep, axis=0)          # (H, T, D)
            vv = np.repeat(self.vc[li, :, :p + 1], rep, axis=0)
            s = np.einsum("hd,htd->ht", q, kk) / np.float32(D ** 0.5)
            s = np.exp(s - s.max(-1, keepdims=True))
            a = np.einsum("ht,htd->hd", s / s.sum(-1, keepdims=True), vv).reshape(1, H * D).astype(np.float32)
            x = x + self._lin(li, "o", a)
            h = self._norm(x)
            g, u = self._lin(li, "gate", h), self._lin(li, "up", h)
            x = x + self._lin(li, "down", (g / (1.0 + np.exp(-g)) * u).astype(np.float32))
        self.pos += 1
        return (self._norm(x) @ self.emb.T)[0]
