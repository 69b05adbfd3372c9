/* libglq_hip.so -- glue operators of the batch-1 decode loop (bf16 in, bf16 out).
 *
 * None of these has a counterpart in the reference's native extension: the reference leaves
 * RMSNorm, rotary embedding, the KV cache and attention to the host model code
 * (transformers' modeling files, driven by glq/hf_integration.py and
 * benchmarks/run_model.py).  They exist here so that the end-to-end decode measurement of
 * the 3B-shape model times the quantized linears rather than dozens of small framework
 * kernels per layer.  Callers: glq_amd/decoder.py only.  Same conventions as glq_hip.h:
 * device pointers, launch on `stream`, no allocation, nonzero return + glqh_last_error().
 */
#ifndef GLQ_DECODER_OPS_H
#define GLQ_DECODER_OPS_H

#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* out[t] = bf16(bf16(x[t] * rsqrt(mean(x[t]^2) + eps)) * w); x, out (T, H), w (H). */
int glqh_rmsnorm_bf16(const void *x, const void *w, void *out, int64_t T, int64_t H, double eps,
                      void *stream);

/* x_out = bf16(x + delta); h_out = RMSNorm(x_out) * w, as glqh_rmsnorm_bf16 (residual add and the
 * next norm in one launch). */
int glqh_add_rmsnorm_bf16(const void *x, const void *delta, const void *w, void *x_out, void *h_out,
                          int64_t T, int64_t H, double eps, void *stream);

/* Rotate q (T, heads, D) and k (T, kv_heads, D) by the angle rows pos[t] of cos_t / sin_t
 * (max_len, D; halves (i, i + D/2) paired) when apply_rope != 0, write q to q_out and append
 * k, v to the caches (kv_heads, max_len, D) at positions pos[t]. */
int glqh_rope_kv_store_bf16(const void *q, const void *k, const void *v, const int64_t *pos,
                            const void *cos_t, const void *sin_t, void *q_out, void *k_cache,
                            void *v_cache, int64_t T, int64_t heads, int64_t kv_heads,
                            int64_t head_dim, int64_t max_len, int apply_rope, void *stream);

/* One query token against cache positions 0..*pos (grouped-query attention, softmax in
 * fp32): q (heads, D) -> out (heads, D); D = 128, max_len <= 12288. */
int glqh_attn_decode_bf16(const void *q, const void *k_cache, const void *v_cache,
                          const int64_t *pos, void *out, int64_t heads, int64_t kv_heads,
                          int64_t head_dim, int64_t max_len, void *stream);

/* out = bf16(bf16(silu(gate)) * up), n elements. */
int glqh_silu_mul_bf16(const void *gate, const void *up, void *out, int64_t n, void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GLQ_DECODER_OPS_H */
