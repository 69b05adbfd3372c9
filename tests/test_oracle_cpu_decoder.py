"""The CPU decoder of the baseline leg (oracle/cpu_decoder.py): one-token steps on the KV cache
against a full causal recompute through dense weight-domain matrices, written out here."""
import numpy as np

from oracle import cpu_decoder as D
from oracle import glq_oracle as O


def _full_recompute(layers, emb, ids, heads, kv_heads, head_dim, no_rope_interval, cos, sin, eps=1e-6):
    T = len(ids)
    x = emb[ids].astype(np.float32)
    dense = [{n: O.dense_weight(W, su, sv, bm, bn, W.shape[0], W.shape[1]) for n, (W, su, sv, bn, bm) in L.items()}
             for L in layers]
    norm = lambda t: t / np.sqrt((t * t).mean(-1, keepdims=True) + eps)   # noqa: E731
    causal = np.tril(np.ones((T, T), bool))
    d = head_dim // 2
    for li, L in enumerate(dense):
        h = norm(x)
        q = (h @ L["q"].T).reshape(T, heads, head_dim)
        k = (h @ L["k"].T).reshape(T, kv_heads, head_dim)
        v = (h @ L["v"].T).reshape(T, kv_heads, head_dim)
        if (li + 1) % no_rope_interval != 0:
            rope = lambda t: t * cos[:T, None] + np.concatenate([-t[..., d:], t[..., :d]], -1) * sin[:T, None]  # noqa: E731
            q, k = rope(q), rope(k)
        rep = heads // kv_heads
        kk, vv = np.repeat(k, rep, 1), np.repeat(v, rep, 1)
        s = np.einsum("thd,shd->hts", q, kk) / head_dim ** 0.5
        s = np.where(causal[None], s, -np.inf)
        s = np.exp(s - s.max(-1, keepdims=True))
        a = np.einsum("hts,shd->thd", s / s.sum(-1, keepdims=True), vv).reshape(T, heads * head_dim)
        x = x + a @ L["o"].T
        h = norm(x)
        g = h @ L["gate"].T
        x = x + (g / (1 + np.exp(-g)) * (h @ L["up"].T)) @ L["down"].T
    return norm(x[-1:]) @ emb.T


def test_cached_steps_equal_full_recompute():
    hidden, heads, kv, hd, ffn, vocab = 128, 2, 1, 64, 192, 50
    shapes = D.linear_shapes(hidden, heads, kv, hd, ffn)
    assert shapes["q"] == (128, 128) and shapes["k"] == (64, 128) and shapes["down"] == (128, 192)
    layers = [D.make_layer(shapes, 4, s) for s in range(2)]
    emb = (np.random.default_rng(0).standard_normal((vocab, hidden)) * 0.5).astype(np.float32)
    dec = D.CpuDecoder(layers, emb, hidden, heads, kv, hd, max_len=16, no_rope_interval=2)
    ids = [3, 17, 44, 8, 20]
    for t, tok in enumerate(ids):
        logits = dec.step(tok)
        ref = _full_recompute(layers, emb, ids[:t + 1], heads, kv, hd, 2, dec.cos, dec.sin)[0]
        assert O.rel_fro(logits, ref) < 1e-4, (t, O.rel_fro(logits, ref))
    assert dec.pos == 5
