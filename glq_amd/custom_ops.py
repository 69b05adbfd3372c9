"""``torch.ops.glq.*`` for the quantized-linear path, backed by libglq_hip.so.

Same op names and schemas as the reference's registration
(glq_vllm/custom_ops.py:56-131, 359-428), so the call sites that prefer
``torch.ops.glq.<op>`` when it exists (glq/quantized_linear.py:863-896, 1079-1120,
glq_vllm/linear_method.py:451, 664-710) run unchanged, and torch.compile / graph capture
see one opaque node per linear.  Fake (meta) implementations give shapes and dtypes
without touching data.  On ROCm the dispatch key of GPU tensors is "CUDA".

One widening: the fused ops accept bf16 activations and then return bf16 (the reference
only ever passes fp16 and gets fp16 back, which is unchanged).
"""
from __future__ import annotations

import torch
from torch.library import Library

_lib = Library("glq", "FRAGMENT")
_registered = False

SCHEMAS = {
    "dequant_matvec": "dequant_matvec(Tensor x, Tensor qidxs, Tensor codebook, float wscale, "
                      "Tensor qidxs2, Tensor codebook2, float inv_resid_scale, "
                      "Tensor codebook_abs) -> Tensor",
    "dequant_matmul": "dequant_matmul(Tensor x, Tensor qidxs, Tensor codebook, float wscale, "
                      "Tensor qidxs2, Tensor codebook2, float inv_resid_scale, "
                      "Tensor codebook_abs, "
                      "Tensor qidxs3, Tensor codebook3, float inv_resid_scale2, "
                      "Tensor qidxs4, Tensor codebook4, float inv_resid_scale3) -> Tensor",
    "dequant_matvec_packed": "dequant_matvec_packed(Tensor x, Tensor qidxs, Tensor codebook_packed, "
                             "float wscale) -> Tensor",
    "dequant_matmul_packed": "dequant_matmul_packed(Tensor x, Tensor qidxs, Tensor codebook_packed, "
                             "float wscale) -> Tensor",
    "input_rht": "input_rht(Tensor x, Tensor sv, Tensor(a!) out, int in_features, "
                 "int stride_x, float rsqrt_n, int n_pad, int log_n) -> ()",
    "output_rht": "output_rht(Tensor y_rht, Tensor su, Tensor(a!) out, int out_features, "
                  "int m_pad, int log_m, float rsqrt_m) -> ()",
    # Same schemas under the names the reference gives its transforms of more than 16384
    # points (glq_vllm/custom_ops.py:132-148, callers glq_vllm/linear_method.py:473, 518);
    # here one set of kernels serves every size.
    "input_rht_triton": "input_rht_triton(Tensor x, Tensor sv, Tensor(a!) out, int in_features, "
                        "int stride_x, float rsqrt_n, int n_pad, int log_n) -> ()",
    "output_rht_triton": "output_rht_triton(Tensor y_rht, Tensor su, Tensor(a!) out, "
                         "int out_features, int m_pad, int log_m, float rsqrt_m) -> ()",
    "fused_linear": "fused_linear(Tensor x, Tensor sv, Tensor su, "
                    "Tensor qidxs, Tensor codebook, float wscale, "
                    "int in_features, int out_features, "
                    "int n_pad, int m_pad, int log_n, int log_m, "
                    "Tensor qidxs2, Tensor codebook2, float inv_resid_scale, "
                    "Tensor qidxs3, Tensor codebook3, float inv_resid_scale2, "
                    "Tensor qidxs4, Tensor codebook4, float inv_resid_scale3) -> Tensor",
    "fused_linear_block_diag": "fused_linear_block_diag(Tensor x, Tensor sv, Tensor su, "
                               "Tensor qidxs, Tensor codebook, float wscale, "
                               "int in_features, int out_features, int n_pad, int m_pad, "
                               "Tensor blocks_n, Tensor blocks_m, "
                               "Tensor blocks_n_meta, Tensor blocks_m_meta, "
                               "Tensor qidxs2, Tensor codebook2, float inv_resid_scale, "
                               "Tensor qidxs3, Tensor codebook3, float inv_resid_scale2, "
                               "Tensor qidxs4, Tensor codebook4, float inv_resid_scale3) -> Tensor",
    "fused_linear_trellis_3inst": "fused_linear_trellis_3inst(Tensor x, Tensor sv, Tensor su, "
                                  "Tensor trellis_packed, "
                                  "Tensor blocks_n, Tensor blocks_m, Tensor blocks_n_meta, "
                                  "Tensor blocks_m_meta, "
                                  "float wscale, int in_features, int out_features, "
                                  "int n_pad, int m_pad) -> Tensor",
    "fused_linear_trellis_3inst_yrht": "fused_linear_trellis_3inst_yrht(Tensor x, Tensor sv, "
                                       "Tensor trellis_packed, "
                                       "Tensor blocks_n, Tensor blocks_n_meta, float wscale, "
                                       "int in_features, int n_pad, int m_pad, "
                                       "Tensor(a!) y_rht_out, int col) -> ()",
    "fused_linear_trellis_3inst_rvq2": "fused_linear_trellis_3inst_rvq2(Tensor x, Tensor sv, Tensor su, "
                                       "Tensor trellis_packed, Tensor trellis_packed2, "
                                       "Tensor blocks_n, Tensor blocks_m, Tensor blocks_n_meta, "
                                       "Tensor blocks_m_meta, "
                                       "float wscale, float inv_resid_scale2, int in_features, "
                                       "int out_features, int n_pad, int m_pad) -> Tensor",
    "fused_linear_trellis_3inst_yrht_rvq2": "fused_linear_trellis_3inst_yrht_rvq2(Tensor x, Tensor sv, "
                                            "Tensor trellis_packed, Tensor trellis_packed2, "
                                            "Tensor blocks_n, Tensor blocks_n_meta, float wscale, "
                                            "float inv_resid_scale2, "
                                            "int in_features, int n_pad, int m_pad, "
                                            "Tensor(a!) y_rht_out, int col) -> ()",
    "output_rht_shards": "output_rht_shards(Tensor y_rht, Tensor su, Tensor(a!) y, "
                         "int out_features, Tensor shard_meta, int max_bs) -> ()",
    # glq_vllm/custom_ops.py:22-36: the routed-expert step of a mixture-of-experts layer
    "fused_moe_trellis_3inst": "fused_moe_trellis_3inst(Tensor x, Tensor topk_ids, Tensor topk_weights, "
                               "Tensor w13_trellis_packed, Tensor w13_trellis_packed2, "
                               "Tensor w13_SU, Tensor w13_SV, Tensor w13_Wscale, "
                               "Tensor w13_inv_resid_scale2, "
                               "Tensor w2_trellis_packed, Tensor w2_trellis_packed2, "
                               "Tensor w2_SU, Tensor w2_SV, Tensor w2_Wscale, "
                               "Tensor w2_inv_resid_scale2, "
                               "int hidden_size, int intermediate_size, int w13_out_features, "
                               "int n_pad_w13, int m_pad_w13, int n_pad_w2, int m_pad_w2, "
                               "Tensor blocks_n_w13, Tensor blocks_m_w13, "
                               "Tensor blocks_n_w13_meta, Tensor blocks_m_w13_meta, "
                               "Tensor blocks_n_w2, Tensor blocks_m_w2, "
                               "Tensor blocks_n_w2_meta, Tensor blocks_m_w2_meta, "
                               "int activation_type) -> Tensor",
    # glq_vllm/custom_ops.py:301-308
    "embedding_dequant": "embedding_dequant(Tensor input_ids, Tensor qidxs, Tensor sv, "
                         "Tensor wscale, Tensor codebook, Tensor? qidxs2, "
                         "Tensor? inv_resid_scale, Tensor? codebook2, int n_pad, "
                         "int embedding_dim, float embed_scale, ScalarType? out_dtype) -> Tensor",
}


def _act_dtype(x):
    return x.dtype if x.dtype in (torch.float16, torch.bfloat16) else torch.float16


# ---- fake implementations (shapes / dtypes only) ---------------------------------------
def _dequant_matvec_fake(x, qidxs, codebook, wscale, qidxs2, codebook2, inv_resid_scale, codebook_abs):
    return x.new_empty((qidxs.shape[0],), dtype=torch.float32)


def _dequant_matmul_fake(x, qidxs, codebook, wscale, qidxs2, codebook2, inv_resid_scale, codebook_abs,
                         qidxs3, codebook3, inv_resid_scale2, qidxs4, codebook4, inv_resid_scale3):
    return x.new_empty((x.shape[0], qidxs.shape[0]), dtype=torch.float32)


def _dequant_matvec_packed_fake(x, qidxs, codebook_packed, wscale):
    return x.new_empty((qidxs.shape[0],), dtype=torch.float32)


def _dequant_matmul_packed_fake(x, qidxs, codebook_packed, wscale):
    return x.new_empty((x.shape[0], qidxs.shape[0]), dtype=torch.float32)


def _none_fake(*args):
    return None


def _fused_linear_fake(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad, m_pad,
                       log_n, log_m, qidxs2, codebook2, inv_resid_scale, qidxs3, codebook3,
                       inv_resid_scale2, qidxs4, codebook4, inv_resid_scale3):
    return x.new_empty((x.shape[0], out_features), dtype=_act_dtype(x))


def _fused_linear_block_diag_fake(x, sv, su, qidxs, codebook, wscale, in_features, out_features, n_pad,
                                  m_pad, blocks_n, blocks_m, blocks_n_meta, blocks_m_meta, qidxs2,
                                  codebook2, inv_resid_scale, qidxs3, codebook3, inv_resid_scale2,
                                  qidxs4, codebook4, inv_resid_scale3):
    return x.new_empty((x.shape[0], out_features), dtype=_act_dtype(x))


def _fused_linear_trellis_3inst_fake(x, sv, su, trellis_packed, blocks_n, blocks_m, blocks_n_meta,
                                     blocks_m_meta, wscale, in_features, out_features, n_pad, m_pad):
    return x.new_empty((x.shape[0], out_features), dtype=_act_dtype(x))


def _fused_linear_trellis_3inst_rvq2_fake(x, sv, su, trellis_packed, trellis_packed2, blocks_n,
                                          blocks_m, blocks_n_meta, blocks_m_meta, wscale,
                                          inv_resid_scale2, in_features, out_features, n_pad, m_pad):
    return x.new_empty((x.shape[0], out_features), dtype=_act_dtype(x))


def _fused_moe_trellis_3inst_fake(x, topk_ids, topk_weights,
                                  w13_trellis_packed, w13_trellis_packed2,
                                  w13_SU, w13_SV, w13_Wscale, w13_inv_resid_scale2,
                                  w2_trellis_packed, w2_trellis_packed2,
                                  w2_SU, w2_SV, w2_Wscale, w2_inv_resid_scale2,
                                  hidden_size, intermediate_size, w13_out_features,
                                  n_pad_w13, m_pad_w13, n_pad_w2, m_pad_w2,
                                  blocks_n_w13, blocks_m_w13, blocks_n_w13_meta, blocks_m_w13_meta,
                                  blocks_n_w2, blocks_m_w2, blocks_n_w2_meta, blocks_m_w2_meta,
                                  activation_type):
    # (num_tokens, hidden) in the activation dtype (glq_vllm/custom_ops.py:701-718 returns fp16)
    return x.new_empty((*x.shape[:-1], hidden_size), dtype=_act_dtype(x))


def _embedding_dequant_fake(input_ids, qidxs, sv, wscale, codebook, qidxs2, inv_resid_scale, codebook2,
                            n_pad, embedding_dim, embed_scale, out_dtype):
    dt = out_dtype if out_dtype is not None else sv.dtype
    return input_ids.new_empty((*input_ids.shape, embedding_dim), dtype=dt)


FAKES = {
    "dequant_matvec": _dequant_matvec_fake,
    "dequant_matmul": _dequant_matmul_fake,
    "dequant_matvec_packed": _dequant_matvec_packed_fake,
    "dequant_matmul_packed": _dequant_matmul_packed_fake,
    "input_rht": _none_fake,
    "input_rht_triton": _none_fake,
    "output_rht_triton": _none_fake,
    "output_rht": _none_fake,
    "fused_linear": _fused_linear_fake,
    "fused_linear_block_diag": _fused_linear_block_diag_fake,
    "fused_linear_trellis_3inst": _fused_linear_trellis_3inst_fake,
    "fused_linear_trellis_3inst_yrht": _none_fake,
    "fused_linear_trellis_3inst_rvq2": _fused_linear_trellis_3inst_rvq2_fake,
    "fused_linear_trellis_3inst_yrht_rvq2": _none_fake,
    "output_rht_shards": _none_fake,
    "embedding_dequant": _embedding_dequant_fake,
    "fused_moe_trellis_3inst": _fused_moe_trellis_3inst_fake,
}


def _impls():
    from . import ext

    def fused_linear(x, *a):
        return ext.glq_fused_linear_cuda(x, *a, out_dtype=_act_dtype(x))

    def fused_linear_block_diag(x, *a):
        return ext.glq_fused_linear_block_diag_cuda(x, *a, out_dtype=_act_dtype(x))

    def fused_linear_trellis_3inst(x, *a):
        return ext.glq_fused_linear_trellis_3inst_cuda(x, *a, out_dtype=_act_dtype(x))

    def fused_linear_trellis_3inst_rvq2(x, *a):
        return ext.glq_fused_linear_trellis_3inst_rvq2_cuda(x, *a, out_dtype=_act_dtype(x))

    return {
        "dequant_matvec": ext.glq_dequant_matvec_cuda,
        "dequant_matmul": ext.glq_dequant_matmul_cuda,
        "dequant_matvec_packed": ext.glq_dequant_matvec_packed_cuda,
        "dequant_matmul_packed": ext.glq_dequant_matmul_packed_cuda,
        "input_rht": ext.glq_input_rht_cuda,
        "input_rht_triton": ext.glq_input_rht_cuda,
        "output_rht_triton": ext.glq_output_rht_cuda,
        "output_rht": ext.glq_output_rht_cuda,
        "fused_linear": fused_linear,
        "fused_linear_block_diag": fused_linear_block_diag,
        "fused_linear_trellis_3inst": fused_linear_trellis_3inst,
        "fused_linear_trellis_3inst_yrht": ext.glq_fused_linear_trellis_3inst_yrht_cuda,
        "fused_linear_trellis_3inst_rvq2": fused_linear_trellis_3inst_rvq2,
        "fused_linear_trellis_3inst_yrht_rvq2": ext.glq_fused_linear_trellis_3inst_yrht_rvq2_cuda,
        "output_rht_shards": ext.glq_output_rht_shards_cuda,
        "embedding_dequant": ext.glq_embedding_dequant,
        "fused_moe_trellis_3inst": ext.glq_fused_moe_trellis_3inst_cuda,
    }


def register():
    """Define the ops and attach the HIP implementations.  Idempotent; raises if the
    library cannot be loaded (there is nothing to fall back to)."""
    global _registered
    if _registered:
        return
    from . import _lib as loader
    loader.load()
    impls = _impls()
    for name, schema in SCHEMAS.items():
        _lib.define(schema)
        _lib.impl(name, impls[name], "CUDA")
        _lib._register_fake(name, FAKES[name])
    _registered = True


def is_registered() -> bool:
    return _registered
