"""ctypes binding of libglq_hip.so (declared in include/glq_hip.h)."""
from __future__ import annotations

import ctypes as C
import os

_HERE = os.path.dirname(os.path.abspath(__file__))
# GLQ_HIP_LIB overrides the in-tree library (e.g. to try another build of the same ABI)
LIB_PATH = os.environ.get("GLQ_HIP_LIB") or os.path.join(_HERE, "libglq_hip.so")

_lib = None
_load_error = None

c_i64, c_int, c_dbl, c_vp, c_sz = C.c_int64, C.c_int, C.c_double, C.c_void_p, C.c_size_t

# name -> (restype, argtypes); one entry per declaration in include/glq_hip.h
SIGNATURES = {
    "glqh_version": (c_int, []),
    "glqh_last_error": (C.c_char_p, []),
    "glqh_init": (c_int, []),
    "glqh_trellis_kernel_supported": (c_int, [c_i64, c_i64]),
    "glqh_decompress_trellis_3inst": (c_int, [c_vp, c_i64, c_i64, c_i64, c_i64, c_int, c_vp, c_vp]),
    "glqh_trellis_gemv_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64]),
    "glqh_decode_matmul_trellis_3inst": (
        c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_i64, c_i64, c_dbl, c_vp, c_i64, c_int,
                c_vp, c_sz, c_vp]),
    "glqh_trellis_gemv_partials": (
        c_int, [c_vp, c_i64, c_vp, c_i64, c_i64, c_i64, c_i64, c_vp, c_sz, c_vp, c_vp]),
    "glqh_input_rht": (
        c_int, [c_vp, c_int, c_i64, c_vp, c_vp, c_int, c_i64, c_i64, c_i64, c_vp, c_vp, c_i64,
                c_dbl, c_vp]),
    "glqh_output_rht": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_vp, c_vp, c_i64,
                c_dbl, c_vp]),
    "glqh_output_rht_scaled": (
        c_int, [c_vp, c_dbl, c_vp, c_vp, c_int, c_i64, c_i64, c_i64, c_i64, c_vp, c_vp, c_i64, c_vp]),
    "glqh_output_rht_shards": (
        c_int, [c_vp, c_vp, c_vp, c_int, c_i64, c_i64, c_i64, c_vp, c_i64, c_i64, c_vp]),
    "glqh_fused_linear_trellis_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64]),
    "glqh_fused_linear_trellis_3inst": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp,
                c_vp, c_i64, c_i64, c_vp, c_i64, c_i64,
                c_vp, c_i64, c_vp, c_i64, c_vp, c_vp,
                c_dbl, c_dbl, c_i64, c_i64, c_i64, c_i64,
                c_vp, c_int, c_i64, c_vp, c_i64, c_vp, c_sz, c_vp]),
    "glqh_noalloc_scratch_bytes": (c_sz, []),
    "glqh_fused_linear_trellis_3inst_noalloc": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp,
                c_vp, c_i64, c_i64, c_vp, c_i64, c_i64,
                c_vp, c_i64, c_vp, c_i64, c_vp, c_vp,
                c_dbl, c_dbl, c_i64, c_i64, c_i64, c_i64,
                c_vp, c_int, c_i64, c_vp, c_i64, c_vp]),
    "glqh_e8_pack_table": (c_int, [c_vp, c_i64, c_vp, c_vp, c_vp]),
    "glqh_e8_repack_table": (c_int, [c_vp, c_i64, c_vp, c_vp, c_vp]),
    "glqh_e8_matmul_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64]),
    "glqh_e8_dequant_matmul": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64,
                c_dbl, c_dbl, c_dbl, c_dbl, c_i64, c_i64, c_vp, c_vp, c_sz, c_vp]),
    "glqh_e8_dequant_matmul_folded": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64,
                c_dbl, c_dbl, c_dbl, c_dbl, c_i64, c_i64, c_vp, c_vp, c_sz, c_vp, c_vp]),
    "glqh_e8_fold_table": (c_int, [c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp]),
    "glqh_e8_fold_indices": (c_int, [c_vp, c_i64, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp]),
    "glqh_e8_folded_count": (c_i64, [c_i64, c_i64]),
    "glqh_e8_fold_eligible": (c_int, [c_i64, c_i64, c_i64]),
    "glqh_e8_decompress": (
        c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_dbl, c_dbl, c_dbl, c_i64, c_i64,
                c_vp, c_vp]),
    "glqh_e8_decompress_f32": (
        c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_dbl, c_dbl, c_dbl, c_i64, c_i64,
                c_vp, c_vp]),
    "glqh_e8_embedding_rows": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_i64, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64,
                c_dbl, c_vp, c_int, c_i64, c_vp]),
    "glqh_fused_linear_e8_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64]),
    "glqh_fused_linear_e8": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
                c_vp, c_vp, c_i64, c_dbl, c_dbl, c_dbl, c_dbl,
                c_vp, c_i64, c_vp, c_i64, c_vp, c_vp,
                c_i64, c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_vp, c_sz, c_vp]),
    "glqh_fused_linear_e8_folded": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
                c_vp, c_vp, c_i64, c_dbl, c_dbl, c_dbl, c_dbl,
                c_vp, c_i64, c_vp, c_i64, c_vp, c_vp,
                c_i64, c_i64, c_i64, c_i64, c_vp, c_int, c_i64, c_vp, c_sz, c_vp, c_vp]),
    "glqh_fused_linear_trellis_group_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64, c_int]),
    "glqh_fused_linear_trellis_3inst_group": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_int, c_vp, c_i64, c_vp, c_i64, c_i64, c_int, c_i64,
                c_vp, c_sz, c_vp]),
    "glqh_fused_linear_trellis_3inst_group_rvq2": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp, c_int, c_vp, c_i64, c_vp, c_i64, c_i64, c_int, c_i64,
                c_vp, c_sz, c_vp]),
    "glqh_fused_moe_trellis_workspace_bytes": (c_sz, [c_i64, c_i64, c_i64, c_vp, c_vp]),
    "glqh_fused_moe_trellis_3inst": (
        c_int, [c_vp, c_int, c_i64, c_i64, c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_i64, c_int, c_vp, c_int,
                c_i64, c_vp, c_sz, c_vp]),
    "glqh_e8_quantize": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp]),
    "glqh_trellis_quantize_workspace_bytes": (c_sz, [c_int, c_i64]),
    "glqh_trellis_quantize_tiles": (c_int, [c_vp, c_i64, c_int, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "glqh_trellis_pack_states": (c_int, [c_vp, c_i64, c_i64, c_int, c_vp, c_vp]),
    "glqh_viterbi_acs_step": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_int, c_vp]),
    # include/glq_decoder_ops.h
    "glqh_rmsnorm_bf16": (c_int, [c_vp, c_vp, c_vp, c_i64, c_i64, c_dbl, c_vp]),
    "glqh_add_rmsnorm_bf16": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_dbl, c_vp]),
    "glqh_rope_kv_store_bf16": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp,
                                        c_i64, c_i64, c_i64, c_i64, c_i64, c_int, c_vp]),
    "glqh_attn_decode_bf16": (c_int, [c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64, c_i64, c_i64, c_vp]),
    "glqh_silu_mul_bf16": (c_int, [c_vp, c_vp, c_vp, c_i64, c_vp]),
    "glqh_lm_head_workspace_bytes": (c_sz, []),
    "glqh_lm_head_argmax_bf16": (c_int, [c_vp, c_vp, c_i64, c_i64, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "glqh_trellis_linear_add_rmsnorm_bf16": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_dbl, c_vp, c_vp, c_vp, c_sz, c_vp]),
    "glqh_trellis_qkv_rope_store_bf16": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                c_int, c_vp, c_sz, c_vp]),
    "glqh_trellis_qkv_rope_attn_bf16": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                c_i64, c_i64, c_int, c_vp, c_sz, c_vp]),
    "glqh_trellis_qkv_rope_attn_shared_bf16": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_vp, c_vp, c_vp, c_vp, c_i64, c_i64,
                c_i64, c_i64, c_int, c_vp, c_sz, c_vp, c_sz, c_vp]),
    "glqh_attn_split_state_bytes": (c_sz, [c_i64, c_i64]),
    "glqh_trellis_gate_up_silu_bf16": (
        c_int, [c_vp, c_i64, c_vp, c_vp, c_i64, c_vp, c_i64, c_vp, c_vp, c_sz, c_vp]),
}

GLQH_F16, GLQH_BF16, GLQH_F32 = 0, 1, 2


def load():
    """Load the shared library once; raise with the build hint if it is missing."""
    global _lib, _load_error
    if _lib is not None:
        return _lib
    if _load_error is not None:
        raise RuntimeError(_load_error)
    if not os.path.exists(LIB_PATH):
        _load_error = (f"{LIB_PATH} is missing: build it with glq_amd/csrc/build.sh "
                       "(hipcc --offload-arch=gfx950). There is no CPU fallback.")
        raise RuntimeError(_load_error)
    try:
        lib = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(lib, name)
            fn.restype = res
            fn.argtypes = args
    except (OSError, AttributeError) as e:
        _load_error = f"failed to load {LIB_PATH}: {type(e).__name__}: {e}"
        raise RuntimeError(_load_error) from e
    _lib = lib
    return lib


def status():
    """(loaded, error) without raising -- for diagnostics, like the reference's
    cuda_ext_status() (glq/inference_kernel.py:185-196)."""
    try:
        load()
        return True, None
    except RuntimeError as e:
        return False, str(e)


def check(rc: int):
    if rc != 0:
        raise RuntimeError(load().glqh_last_error().decode("utf-8", "replace"))
