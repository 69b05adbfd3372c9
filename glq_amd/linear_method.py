"""Serving-side twin of the reference's vLLM linear method for trellis layers, without vLLM.

`GLQLinearMethod` (glq_vllm/linear_method.py) does three things around the ops of this
library: it keeps the separately quantized shards of a merged linear (fused q/k/v, gate/up)
side by side (`GLQShardedParameter`, :289-391), it hoists every host read and every derived
tensor into a load-time step (`process_weights_after_loading` / `_setup_trellis_weights`,
:1031-1110, 1308-1464), and it applies a layer as one fused op per shard -- or, for merged
3INST layers, as one `fused_linear_trellis_3inst_yrht[_rvq2]` per shard into a shared
`(B, total_m)` fp32 buffer followed by a single `output_rht_shards` (`_glq_apply_trellis`,
:643-741; the switch is `GLQ_TRELLIS_BATCH_OUT_RHT`).  vLLM is not a dependency of this build, so
that call sequence lives here on plain tensors: the same op names, argument order, load-time
invariants and error messages, resolved through `torch.ops.glq.*` when the ops are registered
and through `glq_amd.ext` otherwise.  `apply` allocates with torch only and reads nothing back
to the host, so it can be captured in a HIP graph.
"""
from __future__ import annotations

import os

import torch

from .hadamard import block_decompose, pack_block_meta, pack_shard_meta
from .quantized_linear import E8RHTLinear, _MAX_TOKENS_PER_CALL

# GLQ_TRELLIS_BATCH_OUT_RHT=0 gives every shard its own output transform and concatenates
# (glq_vllm/linear_method.py:616).
_GLQ_BATCH_OUT_RHT = os.environ.get("GLQ_TRELLIS_BATCH_OUT_RHT", "1") != "0"
# Merged single-stage shards go through the library's grouped call (one decode or many-token launch for all
# shards at 1-4 and at more than 64 tokens, one decode launch per shard between one transform launch per sign
# vector and one finishing launch at 5-64), merged two-stage shards at 1-64 tokens through its two-stage form:
# same result up to the rounding of another K split.  Whole merged linear, reference op sequence / grouped call,
# us: q/k/v of a 2048-wide model 39.5 / 31.3 at one token, 52.5 / 36.0 at 4, 68.5 / 45.4 at 128, 95.3 / 52.7 at
# 512; gate/up 2048 -> 2 x 11008 39.9 / 33.7, 43.7 / 37.7, 122 / 74, 277 / 108 (756 / 279 at 2048 tokens); q/k/v
# of a 4096-wide 6 bpw model at one token 55.1 / 36.7.  GLQ_MERGED_GROUPED=0 keeps the reference's per-shard
# sequence (fused_linear_trellis_3inst_yrht per shard + output_rht_shards, glq_vllm/linear_method.py:664-710)
# at every token count; otherwise, up to 63 tokens, shards the grouped call does not take
# (mixed, more than four) take it, and from 64 tokens on those run as whole fused
# linears, concatenated.
_GLQ_MERGED_GROUPED = os.environ.get("GLQ_MERGED_GROUPED", "1") != "0"
_GROUP_MAX_SHARDS = 4                                          # layers per grouped call (GLQH_MAX_SHARDS)

# Largest output block of the shard-batched transform.  The reference stops at 8192 (shared-memory
# budget of its kernel, glq_vllm/linear_method.py:618-623); the kernel here cuts blocks into
# 1024-point slices and takes every block size the per-shard transform takes.
_S4B_MAX_OUT_BLOCK = 32768


def trellis_rvq_recipe(bpw):
    """Rates of the trellis stages at integer `bpw` 2..8: one stage up to 4, above that a 4-bit
    stage plus a residual stage of bpw - 4 bits (glq/trellis.py:788-808)."""
    bpw = int(bpw)
    if not 2 <= bpw <= 8:
        raise ValueError(f"trellis supports integer bpw 2-8, got {bpw}")
    return [bpw] if bpw <= 4 else [4, bpw - 4]


class GLQShards:
    """Per-shard tensors of one buffer of a merged layer; `get_shard(i)` as
    `GLQShardedParameter.get_shard` (glq_vllm/linear_method.py:289-391)."""

    def __init__(self, tensors):
        self._shard_data = list(tensors)

    def get_shard(self, i):
        return self._shard_data[i]

    def __len__(self):
        return len(self._shard_data)


def _op(name):
    """`torch.ops.glq.<name>` when registered, else the extension function of the same name
    (the reference resolves its entries the same way, glq_vllm/linear_method.py:625-641, 676-688)."""
    if hasattr(torch.ops, "glq") and hasattr(torch.ops.glq, name):
        return getattr(torch.ops.glq, name)
    from . import inference_kernel as ik
    return getattr(ik.require_cuda_ext(f"glq_{name}_cuda"), f"glq_{name}_cuda")


class MergedTrellisLinear:
    """Separately quantized trellis-3INST shards that read the same activations and whose outputs
    are concatenated (fused q/k/v, gate/up), or a single layer (one shard).

    Attributes follow the reference's layer object: `SV`, `SU`, `trellis_packed`,
    `trellis_packed2`, `tlut`, `Wscale`, `inv_resid_scale2` (`GLQShards`), `glq_in_features`,
    `glq_n_pad`, `glq_shard_sizes`, `glq_num_shards`, `glq_bpw`, `glq_is_fused`; after
    `process_weights_after_loading()` also `_glq_trellis_meta` and `_glq_s4b`.  A shard that was
    never loaded (numel-0 `trellis_packed`) yields exact-zero columns, as the reference's
    KV-shared layers do."""

    glq_is_trellis = True

    def __init__(self, in_features, shard_sizes, bpw=4):
        self.glq_in_features = int(in_features)
        self.glq_n_pad = int(in_features)                    # trellis layers are never padded
        self.glq_shard_sizes = [int(s) for s in shard_sizes]
        self.glq_num_shards = len(self.glq_shard_sizes)
        self.glq_is_fused = self.glq_num_shards > 1
        self.glq_bpw = int(bpw)
        n = self.glq_num_shards
        i16 = lambda: torch.zeros(0, dtype=torch.int16)      # noqa: E731
        self.trellis_packed = GLQShards(i16() for _ in range(n))
        self.trellis_packed2 = GLQShards(i16() for _ in range(n))
        self.tlut = GLQShards(torch.zeros(0, dtype=torch.float16) for _ in range(n))
        self.SU = GLQShards(torch.ones(s, dtype=torch.float16) for s in self.glq_shard_sizes)
        self.SV = GLQShards(torch.ones(self.glq_n_pad, dtype=torch.float16) for _ in range(n))
        self.Wscale = GLQShards(torch.zeros((), dtype=torch.float32) for _ in range(n))
        self.inv_resid_scale2 = GLQShards(torch.zeros((), dtype=torch.float32) for _ in range(n))
        self._glq_trellis_meta = None
        self._glq_s4b = None

    @classmethod
    def from_linears(cls, linears, bpw=None):
        """Merge trellis `E8RHTLinear` modules that share `in_features` (shards keep their own
        sign vectors and scales: they were quantized separately)."""
        linears = list(linears)
        if not linears or any(not l._is_trellis for l in linears):
            raise RuntimeError("MergedTrellisLinear.from_linears needs trellis layers")
        if len({l.in_features for l in linears}) != 1:
            raise RuntimeError("merged shards must share in_features")
        if bpw is None:
            bpw = sum(t.shape[1] // 16 for t in (linears[0].trellis_packed, linears[0].trellis_packed2)
                      if t.numel() > 0)
        self = cls(linears[0].in_features, [l.out_features for l in linears], bpw)
        for name in ("trellis_packed", "trellis_packed2", "tlut", "SU", "SV", "Wscale", "inv_resid_scale2"):
            setattr(self, name, GLQShards(getattr(l, name) for l in linears))
        return self

    # ------------------------------------------------------------------ load time
    def process_weights_after_loading(self, device=None):
        """Everything that reads the host or allocates, once, before any capture
        (glq_vllm/linear_method.py:1308-1464): buffers to the device, scalars to Python floats,
        the load-time invariants between the recipe and what the checkpoint carries, block lists
        and device metas per shard, and for a merged 3INST layer the shard-batched output
        transform's concatenated sign vector and sub-block table."""
        if device is None:
            device = next(t.device for t in self.trellis_packed._shard_data + self.SV._shard_data
                          if t.device.type == "cuda")
        device = torch.device(device)
        for name in ("trellis_packed", "trellis_packed2", "inv_resid_scale2", "tlut", "SU", "SV", "Wscale"):
            sh = getattr(self, name)
            for i, t in enumerate(sh._shard_data):
                if t.device != device:
                    sh._shard_data[i] = t.to(device)
        n = self.glq_num_shards
        self._glq_trellis_meta = []
        for i in range(n):
            p2 = self.trellis_packed2.get_shard(i)
            has2 = p2.numel() > 0
            self._glq_trellis_meta.append({
                "wscale": float(self.Wscale.get_shard(i).item()),
                "in": self.glq_in_features,
                "out": self.glq_shard_sizes[i],
                "n_pad": self.glq_n_pad,
                "m_pad": self.glq_shard_sizes[i],
                "loaded": self.trellis_packed.get_shard(i).numel() > 0,
                "has_s2": has2,
                "inv_rs2": float(self.inv_resid_scale2.get_shard(i).item()) if has2 else 0.0,
            })
        want_s2 = len(trellis_rvq_recipe(self.glq_bpw)) > 1
        for i, meta in enumerate(self._glq_trellis_meta):
            if not meta["loaded"]:
                continue
            if self.tlut.get_shard(i).numel() > 0:
                raise NotImplementedError("HYB (tlut) trellis checkpoints are not served by this build; "
                                          "re-quantize with variant 3inst")
            if want_s2 and not meta["has_s2"]:
                raise RuntimeError(f"GLQ trellis {self.glq_bpw} bpw shard {i}: trellis_packed2 is missing, so the "
                                   "residual stage would be dropped and the layer would serve 4 bpw quality.")
            if want_s2 and meta["inv_rs2"] == 0.0:
                raise RuntimeError(f"GLQ trellis {self.glq_bpw} bpw shard {i}: trellis_packed2 is present but "
                                   "inv_resid_scale2 is 0.0 -- the residual would decode to nothing. The "
                                   "checkpoint is half-written.")
            if not want_s2 and meta["has_s2"]:
                raise RuntimeError(f"GLQ trellis {self.glq_bpw} bpw shard {i}: the checkpoint carries a "
                                   "trellis_packed2 the recipe has no stage for.")
        for meta in self._glq_trellis_meta:
            bn, bm = block_decompose(meta["n_pad"]), block_decompose(meta["m_pad"])
            meta["_bn"] = torch.tensor(bn, dtype=torch.int64, device="cpu")
            meta["_bm"] = torch.tensor(bm, dtype=torch.int64, device="cpu")
            meta["_bnm"] = pack_block_meta(bn).to(device)
            meta["_bmm"] = pack_block_meta(bm).to(device)
        self._glq_s4b = None
        if self.glq_is_fused:
            shard_blocks = [block_decompose(m["m_pad"]) for m in self._glq_trellis_meta]
            max_bs = max(max(b) for b in shard_blocks)
            if max_bs <= _S4B_MAX_OUT_BLOCK:
                self._glq_s4b = {
                    "shard_meta": pack_shard_meta(shard_blocks).to(device),
                    "su_cat": torch.cat([self.SU.get_shard(i)[:m["m_pad"]].contiguous()
                                         for i, m in enumerate(self._glq_trellis_meta)]).to(device),
                    "total_m": sum(m["m_pad"] for m in self._glq_trellis_meta),
                    "max_bs": max_bs,
                    "has_s2": any(m["has_s2"] for m in self._glq_trellis_meta),
                }
        return self

    # ------------------------------------------------------------------ apply
    def apply(self, x, bias=None):
        """(.., in_features) -> (.., sum(shard_sizes)) in x's dtype: the call sequence of
        `_glq_apply_trellis` plus the bias add of `GLQLinearMethod.apply`."""
        if self._glq_trellis_meta is None:
            raise RuntimeError("process_weights_after_loading() must run before apply()")
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.shape[0] == 0:                                   # no tokens: nothing to launch
            return x.new_empty(*shape[:-1], sum(self.glq_shard_sizes))
        if x2.shape[0] > _MAX_TOKENS_PER_CALL:                 # the kernels' grids carry the token index in 16 bits
            y = torch.cat([self._apply_2d(c) for c in x2.split(_MAX_TOKENS_PER_CALL)])
        else:
            y = self._apply_2d(x2)
        if bias is not None:
            y = y + bias.to(y.dtype)
        return y.reshape(*shape[:-1], y.shape[-1])

    def _grouped_ok(self, B):
        metas = self._glq_trellis_meta
        if not (self.glq_is_fused and all(m["loaded"] and not m["has_s2"] for m in metas)):
            return False
        if len({self.trellis_packed.get_shard(i).shape[1] for i in range(len(metas))}) != 1:
            return False
        return len(metas) <= _GROUP_MAX_SHARDS

    def _grouped_rvq2_ok(self, B):
        """Up to 64 tokens of merged stacked shards (first stages of 4 bpw, second stages of one rate): the
        library's grouped two-stage call."""
        metas = self._glq_trellis_meta
        if B < 1 or B > 64 or len(metas) > _GROUP_MAX_SHARDS or \
                not (self.glq_is_fused and all(m["loaded"] and m["has_s2"] for m in metas)):
            return False
        n = range(len(metas))
        return ({self.trellis_packed.get_shard(i).shape[1] for i in n} == {64} and
                len({self.trellis_packed2.get_shard(i).shape[1] for i in n}) == 1)

    def _apply_2d(self, x):
        _apply = E8RHTLinear._trellis_linear_apply
        metas = self._glq_trellis_meta
        if _GLQ_MERGED_GROUPED and x.dtype in (torch.float16, torch.bfloat16) and self._grouped_rvq2_ok(x.shape[0]):
            from . import ext
            m0 = metas[0]
            return ext.glq_fused_linear_trellis_3inst_group_rvq2(
                x.contiguous(), [(self.SV.get_shard(i), self.SU.get_shard(i), self.trellis_packed.get_shard(i),
                                  self.trellis_packed2.get_shard(i), m["wscale"], m["inv_rs2"], m["out"], m["m_pad"])
                                 for i, m in enumerate(metas)],
                m0["_bn"], m0["_bnm"], m0["in"], m0["n_pad"], out_dtype=x.dtype)
        if _GLQ_MERGED_GROUPED and x.dtype in (torch.float16, torch.bfloat16) and self._grouped_ok(x.shape[0]):
            from . import ext
            m0 = metas[0]
            return ext.glq_fused_linear_trellis_3inst_group(
                x.contiguous(), [(self.SV.get_shard(i), self.SU.get_shard(i), self.trellis_packed.get_shard(i),
                                  m["wscale"], m["out"], m["m_pad"]) for i, m in enumerate(metas)],
                m0["_bn"], m0["_bnm"], m0["in"], m0["n_pad"], out_dtype=x.dtype)
        if self.glq_is_fused:
            s4b = self._glq_s4b
            # from 64 tokens on, shards the grouped call does not take (stacked, mixed, more than four) run as
            # whole fused linears, concatenated: their sums stay fp16 between the tile kernel and the output
            # transform and stacked shards take the library route above 2048 tokens, which a shared fp32 y_rht
            # rules out (gate/up 4096 -> 2 x 14336 at 6 bpw, 512 / 2048 / 4096 tokens: 334 / 1262 / 2407 -> 251 /
            # 935 / 1509 us; q/k/v 160 / 339 / 634 -> 116 / 247 / 436)
            whole = _GLQ_MERGED_GROUPED and x.shape[0] >= 64
            if s4b is not None and _GLQ_BATCH_OUT_RHT and not whole:
                yrht = _op("fused_linear_trellis_3inst_yrht")
                yrht2 = _op("fused_linear_trellis_3inst_yrht_rvq2") if s4b["has_s2"] else None
                shards_rht = _op("output_rht_shards")
                xh = x.half().contiguous()
                total_m = s4b["total_m"]
                y_rht = torch.empty((x.shape[0], total_m), dtype=torch.float32, device=x.device)
                col = 0
                for i, meta in enumerate(metas):
                    if not meta["loaded"]:
                        y_rht[:, col:col + meta["m_pad"]].zero_()
                        col += meta["m_pad"]
                        continue
                    if meta["has_s2"]:
                        yrht2(xh, self.SV.get_shard(i), self.trellis_packed.get_shard(i),
                              self.trellis_packed2.get_shard(i), meta["_bn"], meta["_bnm"], meta["wscale"],
                              meta["inv_rs2"], meta["in"], meta["n_pad"], meta["m_pad"], y_rht, col)
                    else:
                        yrht(xh, self.SV.get_shard(i), self.trellis_packed.get_shard(i), meta["_bn"],
                             meta["_bnm"], meta["wscale"], meta["in"], meta["n_pad"], meta["m_pad"], y_rht, col)
                    col += meta["m_pad"]
                y = torch.empty((x.shape[0], total_m), dtype=torch.float16, device=x.device)
                shards_rht(y_rht, s4b["su_cat"], y, total_m, s4b["shard_meta"], s4b["max_bs"])
                return y.to(x.dtype)
            outs = []
            for i, meta in enumerate(metas):
                if not meta["loaded"]:
                    outs.append(torch.zeros(x.shape[0], meta["out"], dtype=x.dtype, device=x.device))
                    continue
                outs.append(_apply(x, self.SV.get_shard(i), self.SU.get_shard(i), self.trellis_packed.get_shard(i),
                                   self.tlut.get_shard(i), meta["_bn"], meta["_bm"], meta["_bnm"], meta["_bmm"],
                                   meta["wscale"], meta["in"], meta["out"], meta["n_pad"], meta["m_pad"], bias=None,
                                   out_dtype=x.dtype, trellis_packed2=self.trellis_packed2.get_shard(i),
                                   inv_resid_scale2=meta["inv_rs2"]))
            return torch.cat(outs, dim=-1)
        meta = metas[0]
        return _apply(x, self.SV.get_shard(0), self.SU.get_shard(0), self.trellis_packed.get_shard(0),
                      self.tlut.get_shard(0), meta["_bn"], meta["_bm"], meta["_bnm"], meta["_bmm"], meta["wscale"],
                      meta["in"], meta["out"], meta["n_pad"], meta["m_pad"], bias=None, out_dtype=x.dtype,
                      trellis_packed2=self.trellis_packed2.get_shard(0), inv_resid_scale2=meta["inv_rs2"])


class MergedShellLinear:
    """Separately quantized E8-shell shards that read the same activations and whose outputs are
    concatenated (fused q/k/v, gate/up), or a single layer (one shard): the shell side of
    `GLQLinearMethod.apply` (glq_vllm/linear_method.py:1490-1522) with `_glq_apply_shard` per shard
    (:394-522).

    Attributes follow the reference's layer object: `Qidxs`, `Qidxs2`, `Qidxs3`, `Qidxs4`, `SU`, `SV`, `Wscale`,
    `inv_resid_scale`, `inv_resid_scale2`, `inv_resid_scale3` (`GLQShards`), `glq_in_features`,
    `glq_shard_sizes`, `glq_num_shards`, `glq_is_fused`; after `process_weights_after_loading()` also
    `_glq_shard_meta` (per shard: `wscale`, `has_stage2`, `n_stages`, `inv_rs`, `inv_rs2`, `inv_rs3`, `out`,
    `in`, `m_pad`, `n_pad`, `log_n`, `log_m`, `bd_meta`).  Block-diagonal shards (buffers of the layer's own
    sizes) run as one `fused_linear_block_diag` each, legacy shards (buffers padded to powers of two) as one
    `fused_linear` each (the reference issues `input_rht`, `dequant_matmul`, `output_rht` there); activations
    keep their dtype (fp16 or bf16) where the reference casts to fp16 and back."""

    glq_is_trellis = False

    def __init__(self, in_features, shard_sizes, codebook, codebook2=None):
        self.glq_in_features = int(in_features)
        self.glq_shard_sizes = [int(s) for s in shard_sizes]
        self.glq_num_shards = len(self.glq_shard_sizes)
        self.glq_is_fused = self.glq_num_shards > 1
        self.codebook, self.codebook2 = codebook, codebook2    # (65536, 8) table; stage 2's own table if it has one
        n = self.glq_num_shards
        i16 = lambda: torch.zeros(0, dtype=torch.int16)      # noqa: E731
        f32 = lambda: torch.zeros((), dtype=torch.float32)   # noqa: E731
        for name in ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4"):
            setattr(self, name, GLQShards(i16() for _ in range(n)))
        for name in ("Wscale", "inv_resid_scale", "inv_resid_scale2", "inv_resid_scale3"):
            setattr(self, name, GLQShards(f32() for _ in range(n)))
        self.SU = GLQShards(torch.ones(s, dtype=torch.float16) for s in self.glq_shard_sizes)
        self.SV = GLQShards(torch.ones(self.glq_in_features, dtype=torch.float16) for _ in range(n))
        self._glq_shard_meta = None

    @classmethod
    def from_linears(cls, linears):
        """Merge shell `E8RHTLinear` modules that share `in_features` and tables."""
        linears = list(linears)
        if not linears or any(l._is_trellis for l in linears):
            raise RuntimeError("MergedShellLinear.from_linears needs E8-shell layers")
        if len({l.in_features for l in linears}) != 1:
            raise RuntimeError("merged shards must share in_features")
        if any(l.codebook is None for l in linears):
            raise RuntimeError("set_codebook() must be called on every layer before merging")
        self = cls(linears[0].in_features, [l.out_features for l in linears], linears[0].codebook,
                   linears[0].codebook2)
        for name in ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4", "SU", "SV", "Wscale", "inv_resid_scale",
                     "inv_resid_scale2", "inv_resid_scale3"):
            setattr(self, name, GLQShards(getattr(l, name) for l in linears))
        return self

    def process_weights_after_loading(self, device=None):
        """Everything that reads the host or allocates, once, before any capture
        (glq_vllm/linear_method.py:1031-1110): buffers and tables to the device, scalars to Python floats,
        block lists and their device copies, and the library's load-time step per shard (packed tables,
        folded index streams: `ext.e8_prepare`)."""
        from . import ext
        from .hadamard import next_pow2
        dev = torch.device(device) if device is not None else self.Qidxs.get_shard(0).device
        names = ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4", "SU", "SV", "Wscale", "inv_resid_scale",
                 "inv_resid_scale2", "inv_resid_scale3")
        for name in names:
            sh = getattr(self, name)
            sh._shard_data = [t.to(dev) for t in sh._shard_data]
        half = lambda t: None if t is None else t.to(dev).half().contiguous()   # noqa: E731
        self._cb, self._cb2 = half(self.codebook), half(self.codebook2)
        self._empty_i16 = torch.zeros(0, dtype=torch.int16, device=dev)
        self._empty_f16 = torch.zeros(0, dtype=torch.float16, device=dev)
        metas = []
        for i, out in enumerate(self.glq_shard_sizes):
            q = self.Qidxs.get_shard(i)
            if q.dim() != 2 or q.dtype != torch.int16:
                raise RuntimeError(f"shard {i}: Qidxs must be a 2-D int16 tensor")
            m_pad, n_pad = int(q.shape[0]), int(q.shape[1]) * 8
            inv = [float(getattr(self, nm).get_shard(i).item())
                   for nm in ("inv_resid_scale", "inv_resid_scale2", "inv_resid_scale3")]
            n_stages = 1
            for s, nm in enumerate(("Qidxs2", "Qidxs3", "Qidxs4")):
                present = getattr(self, nm).get_shard(i).numel() > 0
                if present != (inv[s] != 0.0):
                    raise RuntimeError(f"shard {i}: stage {s + 2} is half-configured: {nm} is "
                                       f"{'present' if present else 'absent'} but its scale is {inv[s]}")
                if present:
                    if n_stages != s + 1:
                        raise RuntimeError(f"shard {i}: stage {s + 2} without stage {s + 1}")
                    n_stages = s + 2
            legacy = (m_pad, n_pad) == (next_pow2(out), next_pow2(self.glq_in_features)) and \
                (m_pad, n_pad) != (out, self.glq_in_features)
            if not legacy and (m_pad < out or n_pad < self.glq_in_features):
                raise RuntimeError(f"shard {i}: buffers of {m_pad} x {n_pad} for a {out} x {self.glq_in_features} layer")
            bd = None
            if not legacy:
                bn, bm = block_decompose(n_pad), block_decompose(m_pad)
                bd = dict(blocks_n_tensor=torch.tensor(bn, dtype=torch.int64), blocks_m_tensor=torch.tensor(bm, dtype=torch.int64),
                          blocks_n_meta_gpu=pack_block_meta(bn).to(dev), blocks_m_meta_gpu=pack_block_meta(bm).to(dev))
            cb2 = self._cb2 if self._cb2 is not None else self._cb
            ext.e8_prepare(q, self._cb, self.Qidxs2.get_shard(i) if n_stages >= 2 else None, cb2 if n_stages >= 2 else None,
                           self.Qidxs3.get_shard(i) if n_stages >= 3 else None,
                           self.Qidxs4.get_shard(i) if n_stages >= 4 else None)
            metas.append(dict(wscale=float(self.Wscale.get_shard(i).item()), has_stage2=n_stages >= 2, n_stages=n_stages,
                              inv_rs=inv[0], inv_rs2=inv[1], inv_rs3=inv[2], out=out, **{"in": self.glq_in_features},
                              m_pad=m_pad, n_pad=n_pad, log_n=n_pad.bit_length() - 1, log_m=m_pad.bit_length() - 1,
                              bd_meta=bd))
        self._glq_shard_meta = metas
        return self

    def _apply_shard(self, x, i):
        """`_glq_apply_shard` (glq_vllm/linear_method.py:394-522) for shard i."""
        meta = self._glq_shard_meta[i]
        n = meta["n_stages"]
        cb2 = self._cb2 if self._cb2 is not None else self._cb
        q2 = self.Qidxs2.get_shard(i) if n >= 2 else self._empty_i16
        q3 = self.Qidxs3.get_shard(i) if n >= 3 else self._empty_i16
        q4 = self.Qidxs4.get_shard(i) if n >= 4 else self._empty_i16
        stages = (q2, cb2 if n >= 2 else self._empty_f16, meta["inv_rs"] if n >= 2 else 0.0,
                  q3, self._cb if n >= 3 else self._empty_f16, meta["inv_rs2"] if n >= 3 else 0.0,
                  q4, self._cb if n >= 4 else self._empty_f16, meta["inv_rs3"] if n >= 4 else 0.0)
        bd = meta["bd_meta"]
        if bd is not None:
            return _op("fused_linear_block_diag")(
                x, self.SV.get_shard(i), self.SU.get_shard(i), self.Qidxs.get_shard(i), self._cb, meta["wscale"],
                meta["in"], meta["out"], meta["n_pad"], meta["m_pad"], bd["blocks_n_tensor"], bd["blocks_m_tensor"],
                bd["blocks_n_meta_gpu"], bd["blocks_m_meta_gpu"], *stages)
        return _op("fused_linear")(
            x, self.SV.get_shard(i), self.SU.get_shard(i), self.Qidxs.get_shard(i), self._cb, meta["wscale"],
            meta["in"], meta["out"], meta["n_pad"], meta["m_pad"], meta["log_n"], meta["log_m"], *stages)

    def apply(self, x, bias=None):
        """(.., in_features) -> (.., sum(shard_sizes)) in x's dtype: every shard on its own, concatenated,
        plus the bias add of `GLQLinearMethod.apply`."""
        if self._glq_shard_meta is None:
            raise RuntimeError("process_weights_after_loading() must run before apply()")
        shape = x.shape
        x2 = x.reshape(-1, shape[-1])
        if x2.shape[0] == 0:                                   # no tokens: nothing to launch
            return x.new_empty(*shape[:-1], sum(self.glq_shard_sizes))
        xin = (x2 if x2.dtype in (torch.float16, torch.bfloat16) else x2.half()).contiguous()
        chunks = xin.split(_MAX_TOKENS_PER_CALL)               # the kernels' grids carry the token index in 16 bits
        rows = []
        for c in chunks:
            outs = [self._apply_shard(c, i) for i in range(self.glq_num_shards)]
            rows.append(outs[0] if len(outs) == 1 else torch.cat(outs, dim=-1))
        y = rows[0] if len(rows) == 1 else torch.cat(rows)
        if y.dtype != x.dtype:
            y = y.to(x.dtype)
        if bias is not None:
            y = y + bias.unsqueeze(0).to(y.dtype)
        return y.reshape(*shape[:-1], y.shape[-1])


def process_weights_after_loading(layer, device=None):
    """Load-time step for any kind of layer: `MergedTrellisLinear`, `MergedShellLinear` (above) or an `E8RHTLinear`
    module (`prepare()`: scalars, metas, packed tables and folded index streams)."""
    if isinstance(layer, (MergedTrellisLinear, MergedShellLinear)):
        return layer.process_weights_after_loading(device)
    if isinstance(layer, E8RHTLinear):
        if device is not None and layer.SV.device != torch.device(device):
            layer.to(device)
        layer.prepare()
        return layer
    raise TypeError(f"cannot prepare a {type(layer).__name__}")
