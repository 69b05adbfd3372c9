"""E8RHTLinear -- quantized linear layer (E8 shell or trellis-3INST) on the HIP path.

Mirrors the reference module's contract (glq/quantized_linear.py:165-1265): constructor
arguments, buffer names / shapes / dtypes (so reference checkpoints load with
``load_state_dict``), ``set_codebook``, shape adaption on load, and the dispatch to one
fused op per forward.  What it does not carry over is the reference's pure-torch
fallback: on a CPU tensor or without the built library ``forward`` raises.

Buffers
  shell   Qidxs, Qidxs2, Qidxs3, Qidxs4  (m_pad, n_pad/8) int16 (bit pattern = uint16 index)
          inv_resid_scale, inv_resid_scale2, inv_resid_scale3  () fp32, 0 = stage absent
  trellis trellis_packed, trellis_packed2  ((m/16)(n/16), 16K) int16, tlut (0,) for 3INST,
          inv_resid_scale2 () fp32
  both    SU (m_pad,) fp16, SV (n_pad,) fp16, Wscale () fp32, optional bias (out,) fp16
"""
from __future__ import annotations

import math
import os

import torch
import torch.nn as nn

from .hadamard import block_decompose, next_pow2, pack_block_meta


def _codebook_tensor(cb):
    """Accept the reference's codebook object (``.codebook_half``), or a plain tensor."""
    if cb is None:
        return None
    if isinstance(cb, torch.Tensor):
        return cb
    for attr in ("codebook_half", "codebook"):
        t = getattr(cb, attr, None)
        if isinstance(t, torch.Tensor):
            return t
    raise TypeError(f"cannot take an E8 table from {type(cb).__name__}")


_MAX_TOKENS_PER_CALL = 32768

# GLQ_FUSED_TRELLIS=0 replaces the single fused trellis call by its three parts, each an op of
# its own (input transform, one decode matmul per stage, output transform): the reference's
# kill-switch of the same name (glq/quantized_linear.py:23-30), there for A/B runs.  The parts
# are still HIP kernels; there is no torch decode in this build.
_GLQ_FUSED_TRELLIS_ENABLED = os.environ.get("GLQ_FUSED_TRELLIS", "1") != "0"

class E8RHTLinear(nn.Module):
    def __init__(self, in_features: int, out_features: int, bias: bool = False,
                 block_diagonal: bool = False, codebook_type: str = "e8_shell"):
        super().__init__()
        if codebook_type not in ("e8_shell", "trellis"):
            raise NotImplementedError(f"codebook_type {codebook_type!r}: only the E8 shell and "
                                      "trellis codebooks are served by this build")
        self.in_features, self.out_features = in_features, out_features
        self._is_trellis = codebook_type == "trellis"
        if self._is_trellis:
            block_diagonal = True
        if block_diagonal:
            self.blocks_m, self.blocks_n = block_decompose(out_features), block_decompose(in_features)
        else:                                           # legacy checkpoints: pad to a power of two
            self.blocks_m, self.blocks_n = [next_pow2(out_features)], [next_pow2(in_features)]
        self.m_pad, self.n_pad = sum(self.blocks_m), sum(self.blocks_n)
        self.block_diagonal = block_diagonal

        i16 = dict(dtype=torch.int16)
        if self._is_trellis:
            self.register_buffer("trellis_packed", torch.zeros(0, **i16))
            self.register_buffer("trellis_packed2", torch.zeros(0, **i16))
            self.register_buffer("inv_resid_scale2", torch.zeros((), dtype=torch.float32))
            self.register_buffer("tlut", torch.zeros(0, dtype=torch.float16))
        else:
            shape = (self.m_pad, self.n_pad // 8)
            self.register_buffer("Qidxs", torch.zeros(shape, **i16))
            self.register_buffer("Qidxs2", torch.zeros(shape, **i16))
            self.register_buffer("inv_resid_scale", torch.zeros((), dtype=torch.float32))
            self.register_buffer("Qidxs3", torch.zeros(shape, **i16))
            self.register_buffer("inv_resid_scale2", torch.zeros((), dtype=torch.float32))
            self.register_buffer("Qidxs4", torch.zeros(shape, **i16))
            self.register_buffer("inv_resid_scale3", torch.zeros((), dtype=torch.float32))
        self.register_buffer("SU", torch.ones(self.m_pad, dtype=torch.float16))
        self.register_buffer("SV", torch.ones(self.n_pad, dtype=torch.float16))
        self.register_buffer("Wscale", torch.ones((), dtype=torch.float32))
        if bias:
            self.register_buffer("bias", torch.zeros(out_features, dtype=torch.float16))
        else:
            self.bias = None

        self.codebook = None
        self.codebook2 = None
        self._scalars = None                 # host copies of Wscale / residual scales
        self._prepared_for = None            # identity of the buffers the load-time step last saw
        self._trellis_has_kernel = True
        self._rebuild_meta()

    # ------------------------------------------------------------------ bookkeeping
    def _rebuild_meta(self):
        self._blocks_n_tensor = torch.tensor(self.blocks_n, dtype=torch.int64, device="cpu")
        self._blocks_m_tensor = torch.tensor(self.blocks_m, dtype=torch.int64, device="cpu")
        self._blocks_n_meta_cpu = pack_block_meta(self.blocks_n)
        self._blocks_m_meta_cpu = pack_block_meta(self.blocks_m)
        self._blocks_n_meta_gpu = None
        self._blocks_m_meta_gpu = None

    @property
    def weight(self):
        """Zero-element proxy so that ``layer.weight.device`` works."""
        return torch.empty(0, dtype=torch.float16, device=self.SV.device)

    def set_codebook(self, codebook, codebook2=None):
        """Attach the shared table(s) after loading; host copies of the scalars are
        re-read on the next forward."""
        self.codebook, self.codebook2 = codebook, codebook2
        if self._is_trellis:
            self._trellis_has_kernel = getattr(codebook, "has_kernel", True)
        self._scalars = None
        self._prepared_for = None

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        if self._is_trellis:
            for suffix in ("trellis_packed", "trellis_packed2", "tlut"):
                key = prefix + suffix
                if key in state_dict:
                    buf = getattr(self, suffix)
                    if buf.device.type != "meta" and buf.shape != state_dict[key].shape:
                        buf.resize_(state_dict[key].shape)
            # optional buffers of a single-stage checkpoint
            if prefix + "trellis_packed" in state_dict:
                for suffix, fn in (("trellis_packed2", lambda: torch.zeros(0, dtype=torch.int16)),
                                   ("inv_resid_scale2", lambda: torch.zeros((), dtype=torch.float32)),
                                   ("tlut", lambda: torch.zeros(0, dtype=torch.float16))):
                    if prefix + suffix not in state_dict:
                        state_dict[prefix + suffix] = fn()
                        getattr(self, suffix).resize_(state_dict[prefix + suffix].shape)
        else:
            qkey = prefix + "Qidxs"
            if qkey in state_dict:
                self._adopt_shape(*state_dict[qkey].shape)
                shape = (self.m_pad, self.n_pad // 8)
                for suffix in ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4"):
                    buf = getattr(self, suffix)
                    if buf.device.type != "meta" and tuple(buf.shape) != shape:
                        buf.resize_(shape).zero_()
                for suffix, n in (("SU", self.m_pad), ("SV", self.n_pad)):
                    buf = getattr(self, suffix)
                    if buf.device.type != "meta" and buf.shape[0] != n:
                        buf.resize_(n).fill_(1)
                    t = state_dict.get(prefix + suffix)
                    if t is not None and t.shape[0] < n:      # legacy: shorter sign vectors
                        padded = torch.ones(n, dtype=t.dtype, device=t.device)
                        padded[:t.shape[0]] = t
                        state_dict[prefix + suffix] = padded
                for suffix in ("Qidxs2", "Qidxs3", "Qidxs4"):
                    if prefix + suffix not in state_dict:
                        state_dict[prefix + suffix] = torch.zeros(shape, dtype=torch.int16)
                for suffix in ("inv_resid_scale", "inv_resid_scale2", "inv_resid_scale3"):
                    if prefix + suffix not in state_dict:
                        state_dict[prefix + suffix] = torch.zeros((), dtype=torch.float32)
        self._scalars = None
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys,
                                      unexpected_keys, error_msgs)

    def _adopt_shape(self, rows, blocks8):
        """The checkpoint is authoritative for the padded dims: non-power-of-two shapes mean
        a block-diagonal transform (glq/quantized_linear.py:542-572)."""
        m_pad, n_pad = int(rows), int(blocks8) * 8
        if (m_pad, n_pad) == (self.m_pad, self.n_pad):
            return
        pow2 = lambda v: v > 0 and (v & (v - 1)) == 0  # noqa: E731
        if pow2(m_pad) and pow2(n_pad) and m_pad >= self.out_features and n_pad >= self.in_features \
                and (m_pad, n_pad) == (next_pow2(self.out_features), next_pow2(self.in_features)):
            self.block_diagonal = False
            self.blocks_m, self.blocks_n = [m_pad], [n_pad]
        else:
            self.block_diagonal = True
            self.blocks_m, self.blocks_n = block_decompose(m_pad), block_decompose(n_pad)
        self.m_pad, self.n_pad = m_pad, n_pad
        self._rebuild_meta()

    def prepare(self):
        """Load-time step, to be called once the buffers are on the GPU and the table is attached,
        before any stream capture: host copies of the scalars, block meta on the device and, for an
        E8 layer, the packed table(s) and the folded index streams the small-batch and tile kernels
        read (1.5 x the index bytes; `GLQ_E8_FOLD=0` / `GLQ_E8_FOLD_MAX_BYTES` bound them).  The
        reference's place for this work is `GLQLinearMethod.process_weights_after_loading`
        (glq_vllm/linear_method.py:1031-1110).  A forward call outside capture runs it if the
        caller did not; a layer first seen under capture is served on its indices and warns.
        Returns the bytes of folded streams the layer holds."""
        from . import ext
        dev = self.SV.device
        if dev.type != "cuda":
            raise RuntimeError("E8RHTLinear.prepare() needs the buffers on the GPU")
        self._scalars = None
        sc = self._resolve(dev, prepare=False)
        held = 0
        if not self._is_trellis:
            if self.codebook is None:
                raise RuntimeError("set_codebook() must be called before prepare()")
            n = sc["n_stages"]
            cb, cb2 = self._tables(dev, n)
            held = ext.e8_prepare(self.Qidxs, cb, self.Qidxs2 if n >= 2 else None, cb2,
                                  self.Qidxs3 if n >= 3 else None, self.Qidxs4 if n >= 4 else None)
        self._prepared_for = self._buffer_identity()
        return held

    def _buffer_identity(self):
        names = ("trellis_packed", "trellis_packed2") if self._is_trellis else ("Qidxs", "Qidxs2", "Qidxs3", "Qidxs4")
        return tuple((getattr(self, n).data_ptr(), getattr(self, n)._version) for n in names) + (str(self.SV.device),)

    def _tables(self, device, n_stages):
        """The attached table(s) as fp16 tensors on `device`, converted once."""
        cb = _codebook_tensor(self.codebook)
        if cb.device != device or cb.dtype != torch.float16:
            cb = cb.to(device=device, dtype=torch.float16)
            self.codebook = cb
        cb2 = None
        if n_stages >= 2:
            cb2 = _codebook_tensor(self.codebook2)
            if cb2.device != device or cb2.dtype != torch.float16:
                cb2 = cb2.to(device=device, dtype=torch.float16)
                self.codebook2 = cb2
        return cb, cb2

    def dequantize(self) -> torch.Tensor:
        """The dense (out_features, in_features) fp32 weight, for validation
        (glq/quantized_linear.py:1237-1265): every stage decoded and combined in fp32, scaled, both
        transforms undone.  `forward(x)` equals `x @ dequantize().T` up to the fp16 rounding of the
        forward path."""
        from . import dequant
        dev = self.SV.device
        if dev.type != "cuda":
            raise RuntimeError("E8RHTLinear.dequantize() (glq_amd) runs on the GPU only")
        sc = self._resolve(dev, prepare=False)
        if self._is_trellis:
            W_rht = dequant.trellis_rht_domain_weight(self.trellis_packed, self.m_pad, self.n_pad,
                                                      self.trellis_packed2 if sc["has2"] else None, sc["inv2"])
        else:
            if self.codebook is None:
                raise RuntimeError("set_codebook() must be called before dequantize()")
            n, inv = sc["n_stages"], sc["inv"]
            cb, cb2 = self._tables(dev, n)
            W_rht = dequant.e8_rht_domain_weight(self.Qidxs, cb, self.Qidxs2 if n >= 2 else None, cb2, inv[0],
                                                 self.Qidxs3 if n >= 3 else None, inv[1],
                                                 self.Qidxs4 if n >= 4 else None, inv[2])
        return dequant.weight_from_rht_domain(W_rht, self.SU, self.SV, sc["wscale"], self.out_features,
                                              self.in_features, self.blocks_m, self.blocks_n)

    def _resolve(self, device, prepare=True):
        """One-time host reads (scalars) and device copies (block meta) per device; outside stream
        capture also the load-time step of `prepare()` if the caller has not run it."""
        if prepare and not self._is_trellis and self._prepared_for != self._buffer_identity():
            if torch.cuda.is_current_stream_capturing():
                if self._scalars is None:
                    raise RuntimeError("E8RHTLinear: first forward under stream capture; call prepare() "
                                       "(or run one forward) before capturing")
            else:
                self.prepare()
        if self._scalars is None:
            if self._is_trellis:
                has2 = self.trellis_packed2.numel() > 0
                self._scalars = dict(wscale=float(self.Wscale.item()), has2=has2,
                                     inv2=float(self.inv_resid_scale2.item()) if has2 else 0.0)
            else:
                inv = [float(self.inv_resid_scale.item()), float(self.inv_resid_scale2.item()),
                       float(self.inv_resid_scale3.item())]
                n = 1
                if self.codebook2 is not None and inv[0] != 0.0:
                    n = 2
                    if inv[1] != 0.0:
                        n = 3
                        if inv[2] != 0.0:
                            n = 4
                inv = [v if i + 2 <= n else 0.0 for i, v in enumerate(inv)]
                self._scalars = dict(wscale=float(self.Wscale.item()), inv=inv, n_stages=n)
        if self._blocks_n_meta_gpu is None or self._blocks_n_meta_gpu.device != device:
            self._blocks_n_meta_gpu = self._blocks_n_meta_cpu.to(device)
            self._blocks_m_meta_gpu = self._blocks_m_meta_cpu.to(device)
        return self._scalars

    # ------------------------------------------------------------------ forward
    @staticmethod
    def _trellis_linear_apply(x2d, SV, SU, trellis_packed, tlut, blocks_n, blocks_m,
                              blocks_n_meta, blocks_m_meta, wscale, in_features, out_features,
                              n_pad, m_pad, bias=None, out_dtype=torch.float16,
                              trellis_packed2=None, inv_resid_scale2=0.0):
        """One fused op per call: input RHT -> trellis decode/matmul -> x Wscale -> output
        RHT.  Same signature as the reference's static method
        (glq/quantized_linear.py:837-899), shared by the module and by serving code."""
        from . import ext
        if tlut is not None and tlut.numel() > 0:
            raise NotImplementedError("HYB (tlut) trellis checkpoints are not served by this "
                                      "build; re-quantize with variant 3inst")
        x = x2d if x2d.dtype in (torch.float16, torch.bfloat16) else x2d.half()
        x = x.contiguous()
        has_s2 = trellis_packed2 is not None and trellis_packed2.numel() > 0
        ops = torch.ops.glq if hasattr(torch.ops, "glq") else None
        if not _GLQ_FUSED_TRELLIS_ENABLED:
            x_rht = torch.empty((x.shape[0], n_pad), dtype=torch.float16, device=x.device)
            ext.glq_input_rht_blockdiag_cuda(x, SV, x_rht, in_features, n_pad, blocks_n, blocks_n_meta)
            y_rht = ext.glq_decode_matmul_trellis_3inst_cuda(x_rht, trellis_packed, m_pad, n_pad, float(wscale))
            if has_s2:
                ext.glq_decode_matmul_trellis_3inst_cuda(
                    x_rht, trellis_packed2, m_pad, n_pad, float(wscale) * float(inv_resid_scale2),
                    out=y_rht, accum=True)
            y = torch.empty((x.shape[0], out_features), dtype=x.dtype, device=x.device)
            ext.glq_output_rht_blockdiag_cuda(y_rht, SU, y, out_features, m_pad, blocks_m, blocks_m_meta)
        elif has_s2:
            fn = getattr(ops, "fused_linear_trellis_3inst_rvq2", None) if ops is not None else None
            args = (x, SV, SU, trellis_packed, trellis_packed2, blocks_n, blocks_m, blocks_n_meta,
                    blocks_m_meta, float(wscale), float(inv_resid_scale2), in_features, out_features,
                    n_pad, m_pad)
            y = fn(*args) if fn is not None else \
                ext.glq_fused_linear_trellis_3inst_rvq2_cuda(*args, out_dtype=x.dtype)
        else:
            fn = getattr(ops, "fused_linear_trellis_3inst", None) if ops is not None else None
            args = (x, SV, SU, trellis_packed, blocks_n, blocks_m, blocks_n_meta, blocks_m_meta,
                    float(wscale), in_features, out_features, n_pad, m_pad)
            y = fn(*args) if fn is not None else \
                ext.glq_fused_linear_trellis_3inst_cuda(*args, out_dtype=x.dtype)
        if y.dtype != out_dtype:
            y = y.to(out_dtype)
        if bias is not None:
            y = y + bias.unsqueeze(0).to(out_dtype)
        return y

    def forward(self, x: torch.Tensor) -> torch.Tensor:
        if not x.is_cuda:
            raise RuntimeError("E8RHTLinear (glq_amd) runs on the GPU only: there is no CPU path")
        from . import ext
        if not self._is_trellis and self.codebook is None:
            raise RuntimeError("set_codebook() must be called before forward")
        sc = self._resolve(x.device)
        shape = x.shape
        x2d = x.reshape(-1, self.in_features)
        if x2d.shape[0] == 0:                      # no tokens: nothing to launch
            return x.new_empty(*shape[:-1], self.out_features)
        if x2d.shape[0] > _MAX_TOKENS_PER_CALL:    # the kernels' grids carry the token index in 16 bits
            parts = [self.forward(c) for c in x2d.split(_MAX_TOKENS_PER_CALL)]
            return torch.cat(parts).reshape(*shape[:-1], self.out_features)
        if self._is_trellis:
            if not self._trellis_has_kernel:
                raise RuntimeError("natural-layout trellis checkpoints cannot be decoded by the "
                                   "kernel; re-quantize with the kernel layout")
            if not ext.glq_trellis_kernel_supported(self.m_pad, self.n_pad):
                raise RuntimeError(f"trellis kernel needs m % 32 == 0 and k % 64 == 0, got "
                                   f"{self.m_pad}x{self.n_pad}")
            y = E8RHTLinear._trellis_linear_apply(
                x2d, self.SV, self.SU, self.trellis_packed, self.tlut, self._blocks_n_tensor,
                self._blocks_m_tensor, self._blocks_n_meta_gpu, self._blocks_m_meta_gpu,
                sc["wscale"], self.in_features, self.out_features, self.n_pad, self.m_pad,
                bias=self.bias, out_dtype=x.dtype, trellis_packed2=self.trellis_packed2,
                inv_resid_scale2=sc["inv2"])
            return y.reshape(*shape[:-1], self.out_features)

        n = sc["n_stages"]
        cb, cb2 = self._tables(x.device, n)
        xin = x2d if x2d.dtype in (torch.float16, torch.bfloat16) else x2d.half()
        xin = xin.contiguous()
        inv = sc["inv"]
        q2 = self.Qidxs2 if n >= 2 else None
        q3 = self.Qidxs3 if n >= 3 else None
        q4 = self.Qidxs4 if n >= 4 else None
        common = (xin, self.SV, self.SU, self.Qidxs, cb, sc["wscale"], self.in_features,
                  self.out_features, self.n_pad, self.m_pad)
        tail = (q2, cb2, inv[0], q3, cb if q3 is not None else None, inv[1], q4,
                cb if q4 is not None else None, inv[2])
        if self.block_diagonal:
            y = ext.glq_fused_linear_block_diag_cuda(
                *common, self._blocks_n_tensor, self._blocks_m_tensor, self._blocks_n_meta_gpu,
                self._blocks_m_meta_gpu, *tail, out_dtype=xin.dtype)
        else:
            y = ext.glq_fused_linear_cuda(*common, int(math.log2(self.n_pad)),
                                          int(math.log2(self.m_pad)), *tail, out_dtype=xin.dtype)
        if y.dtype != x.dtype:
            y = y.to(x.dtype)
        if self.bias is not None:
            y = y + self.bias.unsqueeze(0).to(x.dtype)
        return y.reshape(*shape[:-1], self.out_features)

    def extra_repr(self) -> str:
        kind = "trellis" if self._is_trellis else "e8_shell"
        return (f"in_features={self.in_features}, out_features={self.out_features}, "
                f"bias={self.bias is not None}, m_pad={self.m_pad}, n_pad={self.n_pad}, {kind}")


class E8RHTEmbedding(nn.Module):
    """nn.Embedding equivalent over per-row E8-quantized weights with a right-side transform.

    Mirrors the reference module (glq/quantized_linear.py:1343-1452): buffers ``Qidxs``
    (vocab, n_pad/8) int16, ``SV`` (n_pad,) fp16, ``SU`` (1,) fp16 (never read), ``Wscale``
    (vocab,) fp32, ``Qidxs2`` and ``inv_resid_scale`` (vocab,) fp32 for the residual stage;
    ``n_pad`` is the next power of two of ``embedding_dim``; ``embed_scale`` multiplies the
    looked-up rows.  ``forward`` is one kernel launch (gather, decode, transform, scale).
    """

    def __init__(self, num_embeddings: int, embedding_dim: int, embed_scale: float = 1.0):
        super().__init__()
        self.num_embeddings = num_embeddings
        self.embedding_dim = embedding_dim
        self.embed_scale = float(embed_scale)
        self.n_pad = next_pow2(embedding_dim) if embedding_dim > 0 else 1
        self.register_buffer("Qidxs", torch.zeros(num_embeddings, self.n_pad // 8, dtype=torch.int16))
        self.register_buffer("SV", torch.ones(self.n_pad, dtype=torch.float16))
        self.register_buffer("SU", torch.ones(1, dtype=torch.float16))
        self.register_buffer("Wscale", torch.ones(num_embeddings, dtype=torch.float32))
        self.register_buffer("Qidxs2", torch.zeros(num_embeddings, self.n_pad // 8, dtype=torch.int16))
        self.register_buffer("inv_resid_scale", torch.zeros(num_embeddings, dtype=torch.float32))
        self.codebook = None
        self.codebook2 = None
        self._n_stages = 1

    def set_codebook(self, codebook, codebook2=None):
        self.codebook, self.codebook2 = codebook, codebook2
        if self.Wscale.device.type == "meta":
            return
        self._n_stages = 1
        if codebook2 is not None and bool(self.inv_resid_scale.abs().any().item()):
            self._n_stages = 2

    def _load_from_state_dict(self, state_dict, prefix, local_metadata, strict, missing_keys,
                              unexpected_keys, error_msgs):
        # 2-bpw checkpoints omit the residual-stage keys
        if prefix + "Qidxs" in state_dict:
            if prefix + "Qidxs2" not in state_dict:
                state_dict[prefix + "Qidxs2"] = torch.zeros(self.num_embeddings, self.n_pad // 8,
                                                            dtype=torch.int16)
            if prefix + "inv_resid_scale" not in state_dict:
                state_dict[prefix + "inv_resid_scale"] = torch.zeros(self.num_embeddings, dtype=torch.float32)
            elif state_dict[prefix + "inv_resid_scale"].dim() == 0:
                state_dict[prefix + "inv_resid_scale"] = (
                    state_dict[prefix + "inv_resid_scale"].reshape(1).expand(self.num_embeddings).clone())
        super()._load_from_state_dict(state_dict, prefix, local_metadata, strict, missing_keys,
                                      unexpected_keys, error_msgs)

    def forward(self, input_ids: torch.Tensor) -> torch.Tensor:
        if self.codebook is None:
            raise RuntimeError("E8RHTEmbedding.set_codebook() must be called first")
        from . import ext
        out_dtype = getattr(self, "_compute_dtype", self.SV.dtype)
        two = self._n_stages >= 2 and self.codebook2 is not None
        return ext.glq_embedding_dequant(
            input_ids, self.Qidxs, self.SV, self.Wscale, _codebook_tensor(self.codebook),
            self.Qidxs2 if two else None, self.inv_resid_scale if two else None,
            _codebook_tensor(self.codebook2) if two else None, n_pad=self.n_pad,
            embedding_dim=self.embedding_dim, embed_scale=self.embed_scale, out_dtype=out_dtype)

    def extra_repr(self) -> str:
        return (f"num_embeddings={self.num_embeddings}, embedding_dim={self.embedding_dim}, "
                f"n_pad={self.n_pad}")
