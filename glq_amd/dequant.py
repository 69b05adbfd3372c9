"""Dense weights from quantized layers, for validation and for hosts that want a plain matrix.

Mirrors `E8RHTLinear.dequantize` (glq/quantized_linear.py:1237-1265) and
`dequantize_glq_weight` (glq_vllm/dequant.py:31-57): decode every stage in the transform
domain, combine in fp32, scale, then undo the two randomized Hadamard transforms
(`W = su * H_m( (H_n(W_rht rows) * sv) columns )`) and cut the padding away.  The decode and
both transforms are the HIP kernels of the forward path; the reference does the same with its
table lookups and `fast_hadamard_transform`.  Unlike the reference (whole power-of-two
transforms only) block-diagonal layers are handled too, and trellis layers as well.
"""
from __future__ import annotations

import ctypes as C

import torch

from . import _lib, ext
from ._lib import GLQH_F32, check
from .hadamard import block_decompose, pack_block_meta

_ROWS_PER_CALL = 16384          # the transforms carry the row index in 16 bits


def _inverse_transform_rows(R, signs, keep, blocks, scale=1.0):
    """(rows, pad) fp32 -> (rows, keep) fp32: per row `scale * signs * H_blocks(row)`, cut to
    the first `keep` columns."""
    rows, pad = R.shape
    lib = _lib.load()
    out = torch.empty((rows, keep), dtype=torch.float32, device=R.device)
    arr, nb = ext._host_i64(blocks)
    meta = pack_block_meta(blocks).to(R.device) if nb > 1 else None
    with torch.cuda.device(R.device):
        for r0 in range(0, rows, _ROWS_PER_CALL):
            r1 = min(rows, r0 + _ROWS_PER_CALL)
            check(lib.glqh_output_rht_scaled(
                C.c_void_p(R[r0:r1].data_ptr()), float(scale), ext._p(signs), C.c_void_p(out[r0:r1].data_ptr()),
                GLQH_F32, keep, r1 - r0, keep, pad, ext._meta_ptr(meta) if nb > 1 else None, arr, nb,
                ext._stream()))
    return out


def weight_from_rht_domain(W_rht, SU, SV, wscale, out_features, in_features, blocks_m=None, blocks_n=None):
    """(m_pad, n_pad) fp32 transform-domain weight (before Wscale) -> (out, in) fp32 weight."""
    m_pad, n_pad = W_rht.shape
    blocks_m = block_decompose(m_pad) if blocks_m is None else [int(b) for b in blocks_m]
    blocks_n = block_decompose(n_pad) if blocks_n is None else [int(b) for b in blocks_n]
    ext._chk(W_rht, "W_rht", torch.float32)
    ext._chk(SU, "SU", torch.float16)
    ext._chk(SV, "SV", torch.float16)
    if SU.numel() != m_pad or SV.numel() != n_pad:
        raise RuntimeError(f"sign vectors of {SU.numel()} / {SV.numel()} entries for a {m_pad} x {n_pad} weight")
    A = _inverse_transform_rows(W_rht, SV, int(in_features), blocks_n)                # rows: H_n, * sv
    At = A.t().contiguous()                                                           # (in, m_pad)
    Wt = _inverse_transform_rows(At, SU, int(out_features), blocks_m, float(wscale))  # columns: H_m, * su
    return Wt.t().contiguous()


def e8_rht_domain_weight(Qidxs, codebook, Qidxs2=None, codebook2=None, inv_resid_scale=0.0, Qidxs3=None,
                         inv_resid_scale2=0.0, Qidxs4=None, inv_resid_scale3=0.0):
    """(m_pad, n_pad) fp32: cb[Qidxs] + inv_rs * cb2[Qidxs2] + ... (no Wscale)."""
    lib = _lib.load()
    dev = Qidxs.device
    cb = ext._half_table(ext._on_device(codebook, dev))
    cb2 = None if codebook2 is None else ext._half_table(ext._on_device(codebook2, dev))
    t1, q2, t2, n2, q3, q4 = ext._e8_args(Qidxs, cb, Qidxs2, cb2, inv_resid_scale, Qidxs3, inv_resid_scale2,
                                          Qidxs4, inv_resid_scale3)
    M, nblk = Qidxs.shape
    W = torch.empty((M, nblk * 8), dtype=torch.float32, device=dev)
    with torch.cuda.device(dev):
        check(lib.glqh_e8_decompress_f32(ext._p(Qidxs), ext._p(q2), ext._p(q3), ext._p(q4), ext._p(t1), ext._p(t2),
                                         n2, float(inv_resid_scale), float(inv_resid_scale2),
                                         float(inv_resid_scale3), M, nblk * 8, ext._p(W), ext._stream()))
    return W


def trellis_rht_domain_weight(trellis_packed, m_pad, n_pad, trellis_packed2=None, inv_resid_scale2=0.0):
    """(m_pad, n_pad) fp32: decode(stage 1) + inv_rs2 * decode(stage 2), each stage's values exact
    fp16, the sum in fp32 (glq/trellis.py:923-933)."""
    W = ext.glq_decompress_trellis_3inst_cuda(trellis_packed, m_pad, n_pad).float()
    if trellis_packed2 is not None and trellis_packed2.numel() > 0 and float(inv_resid_scale2) != 0.0:
        W.add_(ext.glq_decompress_trellis_3inst_cuda(trellis_packed2, m_pad, n_pad, allow_r1=True).float(),
               alpha=float(inv_resid_scale2))
    return W


def dequantize_glq_weight(Qidxs, SU, SV, Wscale, codebook, Qidxs2=None, inv_resid_scale=0.0, codebook2=None,
                          out_features=None, in_features=None):
    """Argument order and result of the reference's helper (glq_vllm/dequant.py:31-57): the dense
    fp16 weight of an E8 layer, cut to (out_features, in_features) when both are given."""
    if not Qidxs.is_cuda:
        raise RuntimeError("dequantize_glq_weight runs on the GPU only: there is no CPU path")
    m_pad, n_pad = Qidxs.shape[0], Qidxs.shape[1] * 8
    cb = codebook if isinstance(codebook, torch.Tensor) else getattr(codebook, "codebook_half", None)
    cb2 = codebook2 if codebook2 is None or isinstance(codebook2, torch.Tensor) else codebook2.codebook_half
    two = Qidxs2 is not None and float(inv_resid_scale) != 0.0 and cb2 is not None
    W_rht = e8_rht_domain_weight(Qidxs.contiguous(), cb, Qidxs2.contiguous() if two else None, cb2 if two else None,
                                 float(inv_resid_scale) if two else 0.0)
    cut = out_features is not None and in_features is not None
    W = weight_from_rht_domain(W_rht, SU.to(torch.float16).contiguous(), SV.to(torch.float16).contiguous(),
                               float(Wscale), out_features if cut else m_pad, in_features if cut else n_pad)
    return W.half()
