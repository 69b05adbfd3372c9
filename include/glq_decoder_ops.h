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

#include <stddef.h>
#include <stdint.h>

#include "glq_hip.h"

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

/* Positions live on the device (`pos`), so the host cannot check them: every kernel below that
 * takes `pos` compares it with max_len itself.  Precondition: 0 <= pos[t] < max_len, and cos_t /
 * sin_t hold at least max_len rows.  A position outside [0, max_len) makes the kernels skip that
 * token entirely -- no cache row, no q_out / out row is written and nothing is read through the
 * position -- instead of overrunning the caches or the score buffer; the caller's output rows
 * then keep what they held before the call. */

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

/* One token through a trellis linear whose output is a residual branch (o_proj, down_proj),
 * finished in the launch that transforms the output:
 *   y = linear(x);  x_out = bf16(resid + bf16(y));  h_out = RMSNorm(x_out) * norm_w
 * (the results of glqh_fused_linear_trellis_3inst_group + glqh_add_rmsnorm_bf16 up to fp32
 * summation order, in two launches instead of three).  x (in_features) bf16; shard as in
 * glqh_fused_linear_trellis_3inst_group with out_features == m_pad <= ~7000 (its y is
 * ignored); ws: glqh_fused_linear_trellis_group_workspace_bytes(1, n_pad, m_pad, 1) bytes. */
int glqh_trellis_linear_add_rmsnorm_bf16(const void *x, int64_t in_features,
                                         const glqh_trellis_shard *shard, const int64_t *blocks_n,
                                         int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                                         int64_t n_pad, const void *resid, const void *norm_w,
                                         double eps, void *x_out, void *h_out, void *ws,
                                         size_t ws_bytes, void *stream);

/* One token through gate_proj and up_proj (gate_up[0], gate_up[1], same shape) and the gate:
 *   act = bf16(bf16(silu(bf16 gate(x))) * bf16 up(x)),  act (out_features) bf16
 * bit-identical to glqh_fused_linear_trellis_3inst_group + glqh_silu_mul_bf16, in two launches
 * instead of three.  ws: ...group_workspace_bytes(1, n_pad, 2 * m_pad, 2) bytes. */
int glqh_trellis_gate_up_silu_bf16(const void *x, int64_t in_features,
                                   const glqh_trellis_shard *gate_up, const int64_t *blocks_n,
                                   int64_t n_blocks_n, const glqh_block_meta *bn_meta_dev,
                                   int64_t n_pad, void *act_out, void *ws, size_t ws_bytes,
                                   void *stream);

/* One token through q_proj, k_proj, v_proj (qkv[0..2], out_features == m_pad, rows = whole heads of
 * head_dim, every Hadamard block of m_pad at least one head) and glqh_rope_kv_store_bf16 in the
 * launch that transforms their outputs: q rotated -> q_out (heads, D); k rotated and v -> cache
 * row *pos.  Bit-identical to glqh_fused_linear_trellis_3inst_group + glqh_rope_kv_store_bf16.
 * ws: ...group_workspace_bytes(1, n_pad, sum of m_pad, 3) bytes. */
int glqh_trellis_qkv_rope_store_bf16(const void *x, int64_t in_features, const glqh_trellis_shard *qkv,
                                     const int64_t *blocks_n, int64_t n_blocks_n,
                                     const glqh_block_meta *bn_meta_dev, int64_t n_pad,
                                     const int64_t *pos, const void *cos_t, const void *sin_t,
                                     void *q_out, void *k_cache, void *v_cache, int64_t head_dim,
                                     int64_t max_len, int apply_rope, void *ws, size_t ws_bytes,
                                     void *stream);

/* The same with the attention of the token in that launch as well: q / k / v projections,
 * rotary, cache append at *pos and single-query attention over positions 0..*pos ->
 * out (heads, D) bf16.  Bit-identical to glqh_trellis_qkv_rope_store_bf16 +
 * glqh_attn_decode_bf16; head_dim = 128, max_len <= ~11000. */
int glqh_trellis_qkv_rope_attn_bf16(const void *x, int64_t in_features, const glqh_trellis_shard *qkv,
                                    const int64_t *blocks_n, int64_t n_blocks_n,
                                    const glqh_block_meta *bn_meta_dev, int64_t n_pad,
                                    const int64_t *pos, const void *cos_t, const void *sin_t,
                                    void *k_cache, void *v_cache, void *out, int64_t heads,
                                    int64_t kv_heads, int64_t head_dim, int64_t max_len,
                                    int apply_rope, void *ws, size_t ws_bytes, void *stream);

/* The same with the keys of a long context shared by several workgroups per head.  state:
 * glqh_attn_split_state_bytes(heads, max_len) bytes that the caller sets to zero once and then leaves to
 * this entry (every call returns them to zero; calls that overlap on one GPU need a state buffer each).
 * Up to min(8, (max_len - 1) / 512) workgroups per head take a share of the keys once the context holds 512 keys for
 * each (from 1024 positions on), write (maximum, sum, weighted rows) of their share, and the one that finishes
 * last merges the shares in ascending order: no workgroup waits for another.  Below 1024 positions, and with
 * state == NULL, one workgroup per head finishes alone, bit-identical to the entry above; with shares the row
 * differs from it by rounding (another order of summation).  max_len <= ~90000; at most 256 heads. */
size_t glqh_attn_split_state_bytes(int64_t heads, int64_t max_len);
int glqh_trellis_qkv_rope_attn_shared_bf16(const void *x, int64_t in_features, const glqh_trellis_shard *qkv,
                                           const int64_t *blocks_n, int64_t n_blocks_n,
                                           const glqh_block_meta *bn_meta_dev, int64_t n_pad,
                                           const int64_t *pos, const void *cos_t, const void *sin_t,
                                           void *k_cache, void *v_cache, void *out, int64_t heads,
                                           int64_t kv_heads, int64_t head_dim, int64_t max_len,
                                           int apply_rope, void *ws, size_t ws_bytes, void *state,
                                           size_t state_bytes, void *stream);

size_t glqh_lm_head_workspace_bytes(void);

/* Output head of a decode step: logits[r] = <h, table[r, :]> for a (vocab, hidden) bf16 table and
 * one bf16 activation row (fp32 sums), *token_out = the row of the largest logit (lowest row on
 * ties).  logits_out (vocab fp32) may be NULL.  hidden = 2048 or 4096; ws:
 * glqh_lm_head_workspace_bytes() bytes.  Two launches; the table is streamed once. */
int glqh_lm_head_argmax_bf16(const void *h, const void *table, int64_t vocab, int64_t hidden,
                             float *logits_out, int64_t *token_out, void *ws, size_t ws_bytes,
                             void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GLQ_DECODER_OPS_H */
