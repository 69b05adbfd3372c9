"""The decoder of configs[4] against an independent fp32 model (needs an MI355X).

The reference model is plain torch on the CPU in fp32: every quantized linear is replaced by a
dense matrix W_hat = diag(su) H_m (Wscale * decode(packed)) H_n diag(sv) built by the ORACLE
(numpy dequantizer and numpy Hadamard transforms), and the glue (RMSNorm, rotary embedding on
all but every n-th layer, causal grouped-query attention, SiLU gate, residuals, tied output head)
is written out from the SmolLM3 architecture.  Compared: the logits of a prompt, the logits of
one-token steps on the cache, and the greedy tokens wherever the reference's own top-2 margin
is larger than the observed logit error (a tie in the reference decides nothing).
"""
import numpy as np
import pytest
import torch
import torch.nn.functional as F

from oracle import glq_oracle as O
from tests.gpu_util import DEV, rel, say

pytestmark = pytest.mark.gpu


def _dense(lin):
    """Weight-domain fp32 matrix of one quantized linear, through the oracle only."""
    m, n = lin.m, lin.n
    W = O.decode_layer(lin.packed.cpu().numpy(), m, n, fast=True) * np.float32(lin.wscale)
    bm, bn = O.block_decompose(m), O.block_decompose(n)
    A = O.block_diag_fht(W, bn)
    A = O.block_diag_fht(A.T.copy(), bm).T
    su, sv = lin.su.float().cpu().numpy(), lin.sv.float().cpu().numpy()
    return torch.from_numpy(np.ascontiguousarray(A * su[:, None] * sv[None, :]))


class RefModel:
    def __init__(self, dec):
        self.cfg = dec.cfg
        self.emb = dec.emb.float().cpu()
        self.layers = [{k: (_dense(v) if k in ("q", "k", "v", "o", "gate", "up", "down") else v.float().cpu())
                        for k, v in L.items()} for L in dec.layers]
        self.ln_f = dec.ln_f.float().cpu()
        # the decoder keeps its rotation tables in bf16: part of the model, not of the kernels
        self.cos, self.sin = dec.cos.float().cpu(), dec.sin.float().cpu()

    def _norm(self, x, w):
        return x * torch.rsqrt(x.pow(2).mean(-1, keepdim=True) + self.cfg.rms_eps) * w

    def _rope(self, x, pos):                                 # x (T, H, D)
        d = x.shape[-1] // 2
        rot = torch.cat((-x[..., d:], x[..., :d]), -1)
        return x * self.cos[pos][:, None] + rot * self.sin[pos][:, None]

    def logits(self, ids):
        """Logits (1, vocab) of the last position of the sequence `ids` (full causal recompute)."""
        cfg = self.cfg
        T, D = len(ids), cfg.head_dim
        pos = torch.arange(T)
        x = self.emb[ids]
        causal = torch.ones(T, T, dtype=torch.bool).tril()
        for li, L in enumerate(self.layers):
            h = self._norm(x, L["ln1"])
            q = (h @ L["q"].T).view(T, cfg.heads, D)
            k = (h @ L["k"].T).view(T, cfg.kv_heads, D)
            v = (h @ L["v"].T).view(T, cfg.kv_heads, D)
            if (li + 1) % cfg.no_rope_interval != 0:
                q, k = self._rope(q, pos), self._rope(k, pos)
            rep = cfg.heads // cfg.kv_heads
            kk, vv = k.repeat_interleave(rep, 1), v.repeat_interleave(rep, 1)
            s = torch.einsum("thd,shd->hts", q, kk) / D ** 0.5
            s = s.masked_fill(~causal[None], float("-inf"))
            a = torch.einsum("hts,shd->thd", s.softmax(-1), vv).reshape(T, cfg.heads * D)
            x = x + a @ L["o"].T
            h = self._norm(x, L["ln2"])
            x = x + (F.silu(h @ L["gate"].T) * (h @ L["up"].T)) @ L["down"].T
        return self._norm(x[-1:], self.ln_f) @ self.emb.T


def _check_against_reference(dec, prompt, n_new, tol):
    ref = RefModel(dec)
    ids = prompt.tolist()
    # prompt: logits of the last prompt position
    lg = dec.prefill(prompt.to(DEV)).float().cpu()
    rl = ref.logits(ids)
    e0 = rel(lg, rl.numpy())
    say("prefill logits rel err", e0)
    assert e0 < tol, e0
    # greedy decode on the cache, eager one-token steps, teacher-forced reference
    toks, errs, decided = [], [], 0
    for _ in range(n_new):
        tok = int(dec.tok.item())
        toks.append(tok)
        ids.append(tok)
        lg = dec._step().float().cpu()
        rl = ref.logits(ids)
        errs.append(rel(lg, rl.numpy()))
        err_abs = float((lg - rl).abs().max())
        top2 = rl[0].topk(2).values
        if float(top2[0] - top2[1]) > 2 * err_abs:           # the reference itself is decided
            decided += 1
            assert int(dec.tok.item()) == int(rl.argmax()), (len(toks), float(top2[0] - top2[1]), err_abs)
    say("step logits rel err max", max(errs), "decided steps", decided, "of", n_new)
    assert max(errs) < tol, errs
    assert decided >= n_new // 2, decided
    # the captured graph produces the same tokens as the eager steps
    out, _, _ = dec.generate(prompt.to(DEV), n_new, use_graph=True)
    assert out.tolist() == toks


def test_small_decoder_end_to_end_against_fp32_reference():
    from glq_amd.decoder import DecoderConfig, TrellisDecoder
    say("decoder reference: small")
    cfg = DecoderConfig(hidden=256, layers=3, heads=2, kv_heads=1, head_dim=128, ffn=512, vocab=1000,
                        no_rope_interval=2, bits=4)
    dec = TrellisDecoder(cfg, device=DEV, seed=3, max_len=64)
    prompt = torch.randint(0, cfg.vocab, (20,), generator=torch.Generator().manual_seed(0))
    _check_against_reference(dec, prompt, 16, 3e-2)


def test_full_shape_decoder_layers_against_fp32_reference():
    """The SmolLM3-3B shapes of configs[4] (hidden 2048, 16 / 4 heads of 128, FFN 11008, vocab
    128256) with two layers, the second without rotary embedding: prompt logits, one-token steps
    through the fused finishing launches and the output head with its arg-max."""
    from glq_amd.decoder import DecoderConfig, TrellisDecoder
    say("decoder reference: full shape, 2 layers")
    cfg = DecoderConfig(layers=2, no_rope_interval=2)
    dec = TrellisDecoder(cfg, device=DEV, seed=1, max_len=64)
    prompt = torch.randint(0, cfg.vocab, (24,), generator=torch.Generator().manual_seed(5))
    _check_against_reference(dec, prompt, 6, 3e-2)
