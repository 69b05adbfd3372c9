"""A SmolLM3-shaped decoder whose seven linears per layer are trellis-3INST quantized, used
to measure end-to-end batch-1 decode (the caller of the quantized-linear forward in the
reference's HF path, glq/hf_integration.py and benchmarks/run_model.py:8).

Random initialisation only: every bit pattern is a valid tail-biting trellis stream, so the
packed weights are random bits with Wscale = 0.02 * opt_scale (weights of rms 0.02), the
sign vectors are seeded, norms are ones and the tied bf16 embedding is N(0, 0.02).  The
architecture follows transformers' SmolLM3Config defaults: grouped-query attention, RMSNorm,
SiLU-gated MLP, rotary embeddings skipped on every fourth layer, tied lm_head.

The whole decode step (embedding row -> 36 layers -> logits -> argmax -> position + 1) is
captured once in a HIP graph and replayed per token; position and token live on the device.
"""
from __future__ import annotations

import ctypes as C
import os
import time
from dataclasses import dataclass

import torch
import torch.nn.functional as F

from . import _lib, ext, hadamard
from ._lib import check


@dataclass
class DecoderConfig:
    hidden: int = 2048
    layers: int = 36
    heads: int = 16
    kv_heads: int = 4
    head_dim: int = 128
    ffn: int = 11008
    vocab: int = 128256
    rms_eps: float = 1e-6
    rope_theta: float = 2e6
    no_rope_interval: int = 4          # every 4th layer skips the rotary embedding
    bits: int = 4


class _Linear:
    """One quantized linear: the buffers E8RHTLinear registers for a trellis layer."""

    def __init__(self, out_f, in_f, bits, gen, dev):
        self.m, self.n = out_f, in_f
        self.packed = torch.randint(-32768, 32768, ((out_f // 16) * (in_f // 16), 16 * bits),
                                    generator=gen, device=dev, dtype=torch.int16)
        self.su = (torch.randint(0, 2, (out_f,), generator=gen, device=dev) * 2 - 1).to(torch.float16)
        self.sv = (torch.randint(0, 2, (in_f,), generator=gen, device=dev) * 2 - 1).to(torch.float16)
        self.wscale = 0.02 * 0.8933837
        bn, bm = hadamard.block_decompose(in_f), hadamard.block_decompose(out_f)
        self.bn, self.bm = torch.tensor(bn, dtype=torch.int64), torch.tensor(bm, dtype=torch.int64)
        self.bn_meta = hadamard.pack_block_meta(bn).to(dev)
        self.bm_meta = hadamard.pack_block_meta(bm).to(dev)

    def __call__(self, x):                                   # (B, in) bf16 -> (B, out) bf16
        return ext.glq_fused_linear_trellis_3inst_cuda(
            x, self.sv, self.su, self.packed, self.bn, self.bm, self.bn_meta, self.bm_meta,
            self.wscale, self.n, self.m, self.n, self.m, out_dtype=torch.bfloat16)

    @property
    def packed_bytes(self):
        return self.packed.numel() * 2


def _group(x, lins, separate=False):
    """Layers that read the same activations: one decode launch (1..4 tokens; 5..16: one per layer) or one launch of the many-token
    kernel (more than 64 tokens, separate=True: one contiguous tensor per layer) for all of them."""
    a = lins[0]
    return ext.glq_fused_linear_trellis_3inst_group(
        x, [(l.sv, l.su, l.packed, l.wscale, l.m, l.m) for l in lins], a.bn, a.bn_meta, a.n, a.n,
        out_dtype=torch.bfloat16, separate=separate)


def _shard_array(lins):
    arr = (ext._TrellisShard * len(lins))()
    for i, l in enumerate(lins):
        arr[i] = ext._TrellisShard(l.sv.data_ptr(), l.su.data_ptr(), l.packed.data_ptr(), l.packed.shape[0],
                                   l.packed.shape[1], float(l.wscale), l.m, l.m, None)
    return arr


def _group_ws(lins, dev):
    lib = _lib.load()
    nb = lib.glqh_fused_linear_trellis_group_workspace_bytes(1, lins[0].n, sum(l.m for l in lins), len(lins))
    return torch.empty(max(int(nb), 256), dtype=torch.uint8, device=dev)


def _linear_add_rms_norm(lin, a, x, w, eps):
    """x_out = x + lin(a); h = RMSNorm(x_out) * w: decode launch + one finishing launch."""
    x_out, h = torch.empty_like(x), torch.empty_like(x)
    ws = _group_ws((lin,), x.device)
    bn, nbn = ext._host_i64(lin.bn)
    arr = _shard_array((lin,))                                   # kept alive across the call
    check(_lib.load().glqh_trellis_linear_add_rmsnorm_bf16(
        a.data_ptr(), lin.n, C.addressof(arr), bn, nbn,
        lin.bn_meta.data_ptr() if nbn > 1 else None, lin.n, x.data_ptr(), w.data_ptr(), float(eps),
        x_out.data_ptr(), h.data_ptr(), ws.data_ptr(), ws.numel(), _stream()))
    return x_out, h


def _gate_up_silu(gate, up, h):
    """act = silu(gate(h)) * up(h): decode launch + one finishing launch."""
    act = torch.empty(1, gate.m, dtype=torch.bfloat16, device=h.device)
    ws = _group_ws((gate, up), h.device)
    bn, nbn = ext._host_i64(gate.bn)
    arr = _shard_array((gate, up))                               # kept alive across the call
    check(_lib.load().glqh_trellis_gate_up_silu_bf16(
        h.data_ptr(), gate.n, C.addressof(arr), bn, nbn,
        gate.bn_meta.data_ptr() if nbn > 1 else None, gate.n, act.data_ptr(), ws.data_ptr(), ws.numel(),
        _stream()))
    return act


def _qkv_rope_store(q, k, v, h, pos, cos, sin, qr, kc, vc, head_dim, max_len, apply_rope):
    """q/k/v projections of one token, rotated and stored: decode launch + one finishing launch."""
    ws = _group_ws((q, k, v), h.device)
    bn, nbn = ext._host_i64(q.bn)
    arr = _shard_array((q, k, v))                                # kept alive across the call
    check(_lib.load().glqh_trellis_qkv_rope_store_bf16(
        h.data_ptr(), q.n, C.addressof(arr), bn, nbn, q.bn_meta.data_ptr() if nbn > 1 else None, q.n,
        pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), qr.data_ptr(), kc.data_ptr(), vc.data_ptr(), head_dim,
        max_len, int(apply_rope), ws.data_ptr(), ws.numel(), _stream()))


def attn_state(heads, max_len, device):
    """Zeroed state buffer of the attention launch that shares a long context's keys between workgroups
    (one per decoder: calls that overlap on one GPU need one each); None when max_len is too short for shares."""
    if os.environ.get("GLQ_ATTN_SHARED_KEYS", "1") == "0":
        return None
    nbytes = int(_lib.load().glqh_attn_split_state_bytes(heads, max_len))
    return torch.zeros(nbytes, dtype=torch.uint8, device=device) if nbytes else None


def _qkv_rope_attn(q, k, v, h, pos, cos, sin, kc, vc, out, heads, kv_heads, head_dim, max_len, apply_rope,
                   state=None):
    """q/k/v projections of one token, rotated, appended to the cache and attended over:
    decode launch + one finishing launch.  state (attn_state): from 1024 cached positions on the keys are
    shared by several workgroups per head."""
    ws = _group_ws((q, k, v), h.device)
    bn, nbn = ext._host_i64(q.bn)
    arr = _shard_array((q, k, v))                                # kept alive across the call
    check(_lib.load().glqh_trellis_qkv_rope_attn_shared_bf16(
        h.data_ptr(), q.n, C.addressof(arr), bn, nbn, q.bn_meta.data_ptr() if nbn > 1 else None, q.n,
        pos.data_ptr(), cos.data_ptr(), sin.data_ptr(), kc.data_ptr(), vc.data_ptr(), out.data_ptr(), heads,
        kv_heads, head_dim, max_len, int(apply_rope), ws.data_ptr(), ws.numel(),
        state.data_ptr() if state is not None else None, state.numel() if state is not None else 0, _stream()))


def _rms_norm(x, w, eps):
    out = torch.empty_like(x)
    check(_lib.load().glqh_rmsnorm_bf16(x.data_ptr(), w.data_ptr(), out.data_ptr(), x.shape[0], x.shape[1],
                                        float(eps), _stream()))
    return out


def _add_rms_norm(x, delta, w, eps):
    x_out, h = torch.empty_like(x), torch.empty_like(x)
    check(_lib.load().glqh_add_rmsnorm_bf16(x.data_ptr(), delta.data_ptr(), w.data_ptr(), x_out.data_ptr(),
                                            h.data_ptr(), x.shape[0], x.shape[1], float(eps), _stream()))
    return x_out, h


def _rms_norm_torch(x, w, eps):
    xf = x.float()
    return (xf * torch.rsqrt(xf.pow(2).mean(-1, keepdim=True) + eps)).to(x.dtype) * w


def _stream():
    return torch.cuda.current_stream().cuda_stream


def _rope(x, cos, sin):                                      # x (T, H, D); cos/sin (T, D)
    d = x.shape[-1] // 2
    rot = torch.cat((-x[..., d:], x[..., :d]), dim=-1)
    return x * cos[:, None, :] + rot * sin[:, None, :]


class TrellisDecoder:
    def __init__(self, cfg: DecoderConfig | None = None, device="cuda:0", seed=0, max_len=1024,
                 fuse_epilogues=True):
        self.cfg = cfg = cfg or DecoderConfig()
        # one-token steps finish o / gate+up / down inside the launch that transforms their output
        self.fuse_epilogues = fuse_epilogues and cfg.hidden <= 6144
        self.dev = dev = torch.device(device)
        self.max_len = max_len
        g = torch.Generator(device=dev).manual_seed(seed)
        H, D = cfg.hidden, cfg.head_dim
        self.emb = (torch.randn(cfg.vocab, H, generator=g, device=dev) * 0.02).to(torch.bfloat16)
        self.layers = []
        for _ in range(cfg.layers):
            self.layers.append(dict(
                q=_Linear(cfg.heads * D, H, cfg.bits, g, dev), k=_Linear(cfg.kv_heads * D, H, cfg.bits, g, dev),
                v=_Linear(cfg.kv_heads * D, H, cfg.bits, g, dev), o=_Linear(H, cfg.heads * D, cfg.bits, g, dev),
                gate=_Linear(cfg.ffn, H, cfg.bits, g, dev), up=_Linear(cfg.ffn, H, cfg.bits, g, dev),
                down=_Linear(H, cfg.ffn, cfg.bits, g, dev),
                ln1=torch.ones(H, dtype=torch.bfloat16, device=dev),
                ln2=torch.ones(H, dtype=torch.bfloat16, device=dev)))
        self.ln_f = torch.ones(H, dtype=torch.bfloat16, device=dev)
        inv = 1.0 / (cfg.rope_theta ** (torch.arange(0, D, 2, device=dev, dtype=torch.float32) / D))
        ang = torch.arange(max_len, device=dev, dtype=torch.float32)[:, None] * inv[None]
        ang = torch.cat((ang, ang), dim=-1)
        self.cos, self.sin = ang.cos().to(torch.bfloat16), ang.sin().to(torch.bfloat16)
        self.kc = torch.zeros(cfg.layers, cfg.kv_heads, max_len, D, dtype=torch.bfloat16, device=dev)
        self.vc = torch.zeros_like(self.kc)
        self.pos = torch.zeros(1, dtype=torch.int64, device=dev)     # next position to write
        self.tok = torch.zeros(1, dtype=torch.int64, device=dev)     # token to feed next
        self.arange = torch.arange(max_len, device=dev)
        self.graph = None
        self.attn_state = attn_state(cfg.heads, max_len, dev)        # long contexts: keys shared between workgroups
        # one-token steps: output head and arg-max in the library (table streamed once)
        self.fast_head = H in (2048, 4096)
        if self.fast_head:
            self.logits = torch.empty(1, cfg.vocab, dtype=torch.float32, device=dev)
            self.head_ws = torch.empty(max(int(_lib.load().glqh_lm_head_workspace_bytes()), 256), dtype=torch.uint8,
                                       device=dev)

    @property
    def packed_bytes_per_token(self):
        return sum(l[k].packed_bytes for l in self.layers for k in ("q", "k", "v", "o", "gate", "up", "down"))

    # ---- one block over T tokens at positions pos (T,) ----------------------------------
    # The residual stream travels as (x, delta): the pending branch output is added by the
    # kernel that also computes the next RMSNorm.
    def _block(self, li, x, delta, pos, mask):
        cfg, L = self.cfg, self.layers[li]
        T, D = x.shape[0], cfg.head_dim
        lib = _lib.load()
        if delta is None:
            h = _rms_norm(x, L["ln1"], cfg.rms_eps)
        elif isinstance(delta, tuple):                           # (layer, its input): not applied yet
            x, h = _linear_add_rms_norm(delta[0], delta[1], x, L["ln1"], cfg.rms_eps)
        else:
            x, h = _add_rms_norm(x, delta, L["ln1"], cfg.rms_eps)
        apply_rope = int((li + 1) % cfg.no_rope_interval != 0)
        if T == 1 and self.fuse_epilogues and D == 128:
            a = torch.empty(1, cfg.heads * D, dtype=torch.bfloat16, device=x.device)
            _qkv_rope_attn(L["q"], L["k"], L["v"], h, pos, self.cos, self.sin, self.kc[li], self.vc[li], a,
                           cfg.heads, cfg.kv_heads, D, self.max_len, apply_rope, self.attn_state)
            x, h = _linear_add_rms_norm(L["o"], a, x, L["ln2"], cfg.rms_eps)
            return x, (L["down"], _gate_up_silu(L["gate"], L["up"], h))
        if T <= 4:
            qkv = _group(h, (L["q"], L["k"], L["v"]))
            nq, nk = L["q"].m, L["k"].m
            q, k, v = qkv[:, :nq], qkv[:, nq:nq + nk], qkv[:, nq + nk:]
            if T > 1:
                q, k, v = q.contiguous(), k.contiguous(), v.contiguous()
        elif T > 64:
            q, k, v = _group(h, (L["q"], L["k"], L["v"]), separate=True)
        else:
            q, k, v = L["q"](h), L["k"](h), L["v"](h)
        qr = torch.empty_like(q)
        check(lib.glqh_rope_kv_store_bf16(
            q.data_ptr(), k.data_ptr(), v.data_ptr(), pos.data_ptr(), self.cos.data_ptr(), self.sin.data_ptr(),
            qr.data_ptr(), self.kc[li].data_ptr(), self.vc[li].data_ptr(), T, cfg.heads, cfg.kv_heads, D,
            self.max_len, apply_rope, _stream()))
        if T == 1 and D == 128:
            a = torch.empty(1, cfg.heads * D, dtype=torch.bfloat16, device=x.device)
            check(lib.glqh_attn_decode_bf16(qr.data_ptr(), self.kc[li].data_ptr(), self.vc[li].data_ptr(),
                                            pos.data_ptr(), a.data_ptr(), cfg.heads, cfg.kv_heads, D,
                                            self.max_len, _stream()))
        else:
            a = F.scaled_dot_product_attention(qr.view(T, cfg.heads, D).transpose(0, 1)[None], self.kc[li][None],
                                               self.vc[li][None], attn_mask=mask, enable_gqa=True)
            a = a[0].transpose(0, 1).reshape(T, cfg.heads * D)
        if T == 1 and self.fuse_epilogues:
            # the output transforms of o / gate+up / down run in the launch that consumes them
            x, h = _linear_add_rms_norm(L["o"], a, x, L["ln2"], cfg.rms_eps)
            return x, (L["down"], _gate_up_silu(L["gate"], L["up"], h))
        x, h = _add_rms_norm(x, L["o"](a), L["ln2"], cfg.rms_eps)
        if T == 1:
            gu = _group(h, (L["gate"], L["up"]))
            gate, up = gu[:, :cfg.ffn], gu[:, cfg.ffn:]               # one row: both halves contiguous
        elif T > 64:
            gate, up = _group(h, (L["gate"], L["up"]), separate=True)
        else:
            gate, up = L["gate"](h), L["up"](h)
        act = torch.empty(T, cfg.ffn, dtype=torch.bfloat16, device=x.device)
        check(lib.glqh_silu_mul_bf16(gate.data_ptr(), up.data_ptr(), act.data_ptr(), act.numel(), _stream()))
        return x, L["down"](act)

    def _forward(self, ids, pos, tok_out=None):
        """ids, pos: (T,) int64 on the device.  Returns the logits of the last token; with
        tok_out (one-token steps) their arg-max is written there as well."""
        T = ids.numel()
        mask = None
        if not (T == 1 and self.cfg.head_dim == 128):
            mask = (self.arange[None, :] <= pos[:, None])[None, None]   # (1,1,T,max_len): causal over the cache
        x, delta = self.emb.index_select(0, ids), None
        for li in range(self.cfg.layers):
            x, delta = self._block(li, x, delta, pos, mask)
        if isinstance(delta, tuple):
            _, h = _linear_add_rms_norm(delta[0], delta[1], x, self.ln_f, self.cfg.rms_eps)
        else:
            _, h = _add_rms_norm(x[-1:], delta[-1:], self.ln_f, self.cfg.rms_eps)
        if tok_out is not None and T == 1 and self.fast_head:
            check(_lib.load().glqh_lm_head_argmax_bf16(
                h.data_ptr(), self.emb.data_ptr(), self.cfg.vocab, self.cfg.hidden, self.logits.data_ptr(),
                tok_out.data_ptr(), self.head_ws.data_ptr(), self.head_ws.numel(), _stream()))
            return self.logits
        logits = torch.matmul(h, self.emb.t()).float()
        if tok_out is not None:
            tok_out.copy_(logits.argmax(-1))
        return logits

    def prefill(self, prompt_ids):
        T = prompt_ids.numel()
        if not 0 < T < self.max_len:
            raise RuntimeError(f"prefill: prompt of {T} tokens does not fit max_len = {self.max_len}")
        logits = self._forward(prompt_ids.to(self.dev), self.arange[:T])
        self.tok.copy_(logits.argmax(-1))
        self.pos.fill_(T)
        return logits

    def _step(self):
        logits = self._forward(self.tok, self.pos, tok_out=self.tok)
        self.pos.add_(1)
        return logits

    def capture(self):
        """Capture the decode step.  State (pos, tok, caches) is restored afterwards."""
        pos0, tok0 = self.pos.clone(), self.tok.clone()
        self._step()                                              # eager warm-up outside capture
        torch.cuda.synchronize()
        s = torch.cuda.Stream()
        s.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(s):
            self.graph = torch.cuda.CUDAGraph()
            with torch.cuda.graph(self.graph, stream=s):
                self._logits = self._step()
        torch.cuda.current_stream().wait_stream(s)
        self.pos.copy_(pos0)
        self.tok.copy_(tok0)
        torch.cuda.synchronize()

    def generate(self, prompt_ids, n_new, use_graph=True):
        """Greedy decode.  Returns (tokens (n_new,), prefill seconds, decode seconds)."""
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        self.prefill(prompt_ids)
        torch.cuda.synchronize()
        t_prefill = time.perf_counter() - t0
        if use_graph and self.graph is None:
            self.capture()
        out = torch.empty(n_new, dtype=torch.int64, device=self.dev)
        if int(self.pos.item()) + n_new > self.max_len:
            raise RuntimeError(f"generate: {int(self.pos.item())} cached + {n_new} new tokens exceed "
                               f"max_len = {self.max_len}")
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(n_new):
            out[i:i + 1].copy_(self.tok)
            if use_graph:
                self.graph.replay()
            else:
                self._step()
        torch.cuda.synchronize()
        return out, t_prefill, time.perf_counter() - t0
