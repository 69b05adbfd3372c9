/* libglq_hip.so -- C ABI of the MI355X (gfx950) quantized-linear forward.
 *
 * Every entry point takes plain device pointers, sizes and a hipStream_t (passed
 * as void*), launches on that stream, never synchronises and never allocates.
 * Scratch memory is supplied by the caller (`ws`, sized by the matching
 * *_workspace_bytes function).  Return value: 0 on success, non-zero on a refused
 * call; glqh_last_error() then returns the reason (thread-local, valid until the
 * next call on the same thread).
 *
 * Each declaration names the reference interface it stands in for; paths are
 * relative to the reference checkout (cnygaard/glq v0.8.8).
 */
#ifndef GLQ_HIP_H
#define GLQ_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* element types of activation / output buffers */
#define GLQH_F16  0
#define GLQH_BF16 1
#define GLQH_F32  2

/* block meta row: {offset, bs, log2(bs), w}; w != 0 is the bit pattern of an fp32
 * normalisation factor that overrides 1/sqrt(bs).
 * glq/quantized_linear.py:36-76 (_pack_block_meta, _pack_shard_meta). */
typedef struct { int32_t offset, bs, log_bs, w; } glqh_block_meta;

int         glqh_version(void);
const char *glqh_last_error(void);
/* One-time per-process setup (kernel attributes, device limits); idempotent and
 * called implicitly by every entry point.  glq/csrc/glq_trellis.cu:823-853. */
int         glqh_init(void);

/* ---- trellis 3INST ------------------------------------------------------ */

/* m % 32 == 0 && k % 64 == 0.  glq/csrc/glq_trellis.cu:979-981. */
int glqh_trellis_kernel_supported(int64_t m, int64_t k);

/* packed ((m/16)(k/16), 16R) int16 -> dense (m,k) fp16, bit-exact with the
 * reference dequantizer.  R = packed_cols/16 in 2..4 (1 only with allow_r1).
 * glq_decompress_trellis_3inst_cuda, glq/csrc/glq_trellis.cu:1064-1085. */
int glqh_decompress_trellis_3inst(const void *packed, int64_t packed_rows, int64_t packed_cols,
                                  int64_t m, int64_t k, int allow_r1,
                                  void *out_f16, void *stream);

/* Scratch bytes needed by the matvec / matmul below for B tokens. */
size_t glqh_trellis_gemv_workspace_bytes(int64_t m, int64_t k, int64_t B);

/* out[b, :] (fp32, row stride out_stride) = (accum ? out : 0) + wscale * W @ x[b, :]
 * with x (B,k) fp16 already in the RHT domain.  B == 1 is the GEMV
 * (glq_decode_matvec_trellis_3inst_cuda, glq/csrc/glq_trellis.cu:1087-1126), B > 1 the
 * batched form that keeps the weights compressed
 * (glq_decode_matmul_trellis_3inst_cuda, glq/csrc/glq_trellis.cu:1192-1232).
 * R == 1 is accepted only with accum (a residual stage). */
int glqh_decode_matmul_trellis_3inst(const void *x_f16, int64_t B,
                                     const void *packed, int64_t packed_rows, int64_t packed_cols,
                                     int64_t m, int64_t k, double wscale,
                                     float *out, int64_t out_stride, int accum,
                                     void *ws, size_t ws_bytes, void *stream);

/* First of the two launches of glqh_decode_matmul_trellis_3inst, on its own: raw fp32
 * split-K partial sums part[(slot*B + token)*m + row], slot < *ksplit_out, unscaled.
 * For callers that fold the fixed-order reduction into their own consumer (as the fused
 * linear does) and for timing the decode kernel in isolation.  The reference has no
 * separate entry for this step (its GEMV reduces inside the block,
 * glq/csrc/glq_trellis.cu:485-510).  From 17 tokens on (GLQ_TRELLIS_TILE_MIN) the many-token kernels keep their repacked
 * activations behind the partial sums: part_bytes must then cover
 * glqh_trellis_gemv_workspace_bytes(m, k, B) (the sums rounded up to 256 bytes + that copy). */
int glqh_trellis_gemv_partials(const void *x_f16, int64_t B,
                               const void *packed, int64_t packed_rows, int64_t packed_cols,
                               int64_t m, int64_t k, float *part, size_t part_bytes,
                               int *ksplit_out, void *stream);

/* ---- randomized Hadamard transforms ------------------------------------- */

/* out[b, 0:n_pad] = blockFHT(pad(x[b, 0:in_features]) * sv), per block 1/sqrt(bs).
 * x is f16 or bf16 with row stride x_stride; out is f32 or f16, contiguous rows of
 * n_pad.  meta (device, n_blocks rows) may be NULL when n_blocks == 1 (one block of
 * n_pad, normalised by rsqrt_n if non-zero).
 * glq_input_rht_cuda / glq_input_rht_blockdiag_cuda, glq/csrc/glq_cuda.cu:2385-2441,
 * 2774-2823. */
int glqh_input_rht(const void *x, int x_dtype, int64_t x_stride, const void *sv_f16,
                   void *out, int out_dtype, int64_t B, int64_t in_features, int64_t n_pad,
                   const glqh_block_meta *meta_dev, const int64_t *blocks_host, int64_t n_blocks,
                   double rsqrt_n, void *stream);

/* y[b, 0:out_features] = (blockFHT(y_rht[b, 0:m_pad]) * su)[0:out_features], cast to
 * f16 / bf16 / f32.  y_rht has row stride y_rht_stride (a slice of a wider buffer is
 * allowed), y has row stride y_stride.
 * glq_output_rht_cuda / glq_output_rht_blockdiag_cuda, glq/csrc/glq_cuda.cu:2444-2499,
 * 2825-2874. */
int glqh_output_rht(const float *y_rht, int64_t y_rht_stride, const void *su_f16,
                    void *y, int y_dtype, int64_t y_stride, int64_t B,
                    int64_t out_features, int64_t m_pad,
                    const glqh_block_meta *meta_dev, const int64_t *blocks_host, int64_t n_blocks,
                    double rsqrt_m, void *stream);

/* The same transform of scale * y_rht, y_rht contiguous (B, m_pad) fp32.  No counterpart in
 * the reference's binding list: it finishes the many-token route (dequantize once, one
 * library GEMM with fp32 output, glq/csrc/glq_trellis.cu:1322-1334), where Wscale has not been
 * applied yet, without a separate pass over y_rht. */
int glqh_output_rht_scaled(const float *y_rht, double scale, const void *su_f16,
                           void *y, int y_dtype, int64_t y_stride, int64_t B,
                           int64_t out_features, int64_t m_pad,
                           const glqh_block_meta *meta_dev, const int64_t *blocks_host, int64_t n_blocks,
                           void *stream);

/* One launch over every sub-block of every output shard of a fused qkv / gate_up
 * linear: shard_meta rows carry global offsets into y_rht (B, total_m); su and y are
 * indexed with the same offsets (y is (B, out_features), out_features == total_m).
 * glq_output_rht_shards_cuda, glq/csrc/glq_cuda.cu:2882-2916. */
int glqh_output_rht_shards(const float *y_rht, const void *su_f16, void *y, int y_dtype,
                           int64_t B, int64_t out_features, int64_t total_m,
                           const glqh_block_meta *shard_meta_dev, int64_t n_rows, int64_t max_bs,
                           void *stream);

/* ---- fused trellis linear ------------------------------------------------ */

size_t glqh_fused_linear_trellis_workspace_bytes(int64_t B, int64_t n_pad, int64_t m_pad);

/* y (B,out_features) = outRHT( wscale * W1 @ inRHT(x) [+ wscale*inv_rs2 * W2 @ inRHT(x)] ).
 * packed2 == NULL with inv_resid_scale2 == 0 is the single-stage layer; any other
 * mismatch of the two is refused ("half-configured").  x is f16 or bf16, y f16 or bf16.
 * glq_fused_linear_trellis_3inst_cuda / ..._rvq2_cuda, glq/csrc/glq_trellis.cu:1339-1366,
 * 1407-1440.  When y_rht_out != NULL the call stops at the RHT-domain product and
 * writes fp32 into y_rht_out[b*y_rht_stride + 0 .. m_pad) (the caller passes the column
 * offset folded into the pointer) and y may be NULL:
 * glq_fused_linear_trellis_3inst_yrht_cuda / ..._yrht_rvq2_cuda, :1373-1397, 1443-1473. */
int glqh_fused_linear_trellis_3inst(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                    const void *sv_f16, const void *su_f16,
                                    const void *packed, int64_t packed_rows, int64_t packed_cols,
                                    const void *packed2, int64_t packed2_rows, int64_t packed2_cols,
                                    const int64_t *blocks_n, int64_t n_blocks_n,
                                    const int64_t *blocks_m, int64_t n_blocks_m,
                                    const glqh_block_meta *bn_meta_dev,
                                    const glqh_block_meta *bm_meta_dev,
                                    double wscale, double inv_resid_scale2,
                                    int64_t in_features, int64_t out_features,
                                    int64_t n_pad, int64_t m_pad,
                                    void *y, int y_dtype, int64_t y_stride,
                                    float *y_rht_out, int64_t y_rht_stride,
                                    void *ws, size_t ws_bytes, void *stream);

/* glqh_fused_linear_trellis_3inst without the workspace argument, for callers that cannot
 * allocate device memory (code under HIP-graph capture, tight serving loops, harnesses that
 * forbid hipMalloc).  No counterpart in the reference.  The scratch (x_rht and the split-K
 * partial sums) lives in a device array built into the library, glqh_noalloc_scratch_bytes()
 * = 8 MiB per GPU.  Its address is resolved once per device by glqh_init() -- which every entry
 * of the library runs -- with that device current: call glqh_init() (or any entry) once on each
 * device before capturing, and the captured call has nothing left to set up.  The
 * call allocates nothing and is refused with a message when
 * glqh_fused_linear_trellis_workspace_bytes(B, n_pad, m_pad) exceeds that size.  Results are
 * bit-identical to glqh_fused_linear_trellis_3inst.  All calls on one GPU share the array:
 * calls that overlap on one GPU (different streams, different threads) race; calls on one
 * stream are ordered and safe. */
size_t glqh_noalloc_scratch_bytes(void);
int glqh_fused_linear_trellis_3inst_noalloc(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                            const void *sv_f16, const void *su_f16,
                                            const void *packed, int64_t packed_rows, int64_t packed_cols,
                                            const void *packed2, int64_t packed2_rows, int64_t packed2_cols,
                                            const int64_t *blocks_n, int64_t n_blocks_n,
                                            const int64_t *blocks_m, int64_t n_blocks_m,
                                            const glqh_block_meta *bn_meta_dev,
                                            const glqh_block_meta *bm_meta_dev,
                                            double wscale, double inv_resid_scale2,
                                            int64_t in_features, int64_t out_features,
                                            int64_t n_pad, int64_t m_pad,
                                            void *y, int y_dtype, int64_t y_stride,
                                            float *y_rht_out, int64_t y_rht_stride, void *stream);

/* ---- several trellis layers on the same activations, two launches ------------- */

#define GLQH_MAX_SHARDS 4

typedef struct {
    const void *sv_f16;          /* (n_pad) input signs of this layer */
    const void *su_f16;          /* (m_pad) output signs */
    const void *packed;          /* ((m_pad/16)(n_pad/16), 16R) int16 */
    int64_t packed_rows, packed_cols;
    double wscale;
    int64_t out_features, m_pad; /* m_pad's block sizes are block_decompose(m_pad) */
    void *y;                     /* this layer's first output element, row stride y_stride;
                                    NULL in every shard: stop after the decode launch (the
                                    split-K partial sums stay in the workspace) */
} glqh_trellis_shard;

size_t glqh_fused_linear_trellis_group_workspace_bytes(int64_t B, int64_t n_pad, int64_t total_m_pad,
                                                       int n_shards);

/* Separately quantized layers that consume the same x (fused q/k/v, gate/up of a merged
 * linear): one decode launch and one output-transform launch for all of them instead of
 * two or three per layer.  Replaces the per-shard loop of the vLLM linear method
 * (glq_vllm/linear_method.py:664-710: fused_linear_trellis_3inst_yrht per shard, then
 * output_rht_shards; glq/csrc/glq_trellis.cu:1373-1397, glq/csrc/glq_cuda.cu:2882-2916) and
 * gives, per shard, the result of glqh_fused_linear_trellis_3inst on that shard up to the
 * rounding of a different K split.  Single-stage layers of one rate R, at most 4 tokens,
 * canonical (block_decompose) output block sizes; anything else is refused and the caller
 * falls back to per-layer calls.
 * 5..64 tokens: one input transform per distinct sign vector, one decode launch per layer (the small-batch
 * kernel under the K plan of the tallest up to 16 tokens, the small-tile kernel under its own plan above)
 * and one output-transform launch for all layers, or one per layer where their K plans differ (no K-slot
 * sum launches, no shared fp32 buffer in between).
 * More than 64 tokens (up to four layers, every y given): one input transform per distinct sign
 * vector, ONE launch of the many-token kernel over the row tiles of all layers (small layers do not
 * fill the chip one by one) and one output transform per layer.  y_stride 0 there: every layer's rows
 * are packed (row stride = its out_features), so that each layer's output is a contiguous matrix.
 */
int glqh_fused_linear_trellis_3inst_group(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                          const glqh_trellis_shard *shards, int n_shards,
                                          const int64_t *blocks_n, int64_t n_blocks_n,
                                          const glqh_block_meta *bn_meta_dev,
                                          int64_t in_features, int64_t n_pad,
                                          int y_dtype, int64_t y_stride,
                                          void *ws, size_t ws_bytes, void *stream);

/* Second stage of a stacked (two-stage, 5-8 bits/weight) shard: the residual stream and its
 * scale, trellis_packed2 / inv_resid_scale2 of glq/quantized_linear.py:986-1010. */
typedef struct {
    const void *packed2;      /* ((m_pad/16) * (n_pad/16), 16 * R2) int16 */
    int64_t packed2_rows, packed2_cols;
    double inv_resid_scale2;
} glqh_trellis_stage2;

/* The grouped call for stacked layers at 1..64 tokens (at one token the decode step of fused q/k/v and gate/up of a
 * 5-8 bits/weight checkpoint; the reference runs fused_linear_trellis_3inst_yrht_rvq2 per shard,
 * glq_vllm/linear_method.py:664-710): one decode launch reads both streams of every layer (first
 * stages of 4 bits/weight, second stages of one common rate, stage2[i] belongs to shards[i]) and one
 * launch finishes them.  2..64 tokens: one input transform per distinct sign vector, one launch per layer
 * that decodes both streams (the small-batch kernel to 16 tokens, the small-tile kernel above), one
 * finishing launch.  Workspace:
 * glqh_fused_linear_trellis_group_workspace_bytes(B, ...).  Every shard's y must be given; other token
 * counts and rates are refused (per-layer calls serve them). */
int glqh_fused_linear_trellis_3inst_group_rvq2(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                               const glqh_trellis_shard *shards,
                                               const glqh_trellis_stage2 *stage2, int n_shards,
                                               const int64_t *blocks_n, int64_t n_blocks_n,
                                               const glqh_block_meta *bn_meta_dev,
                                               int64_t in_features, int64_t n_pad,
                                               int y_dtype, int64_t y_stride,
                                               void *ws, size_t ws_bytes, void *stream);

/* One projection (gate/up "w13" or down "w2") of the routed experts of a mixture-of-experts
 * layer, the experts stacked along the first dimension (glq/csrc/glq_cuda.cu:5043-5064). */
typedef struct {
    const void *packed;          /* (E, (m/16)(k/16), 16 R1) int16, stage 1, R1 = 2..4 */
    int64_t packed_rows;         /* per expert: (m_pad/16)(n_pad/16) */
    int64_t packed_cols;         /* 16 R1 */
    const void *packed2;         /* (E, same rows, 16 R2) int16, R2 = 1..4, or NULL */
    int64_t packed2_cols;
    const void *su_f16;          /* (E, m_pad) */
    const void *sv_f16;          /* (n_pad,) shared by the experts */
    const float *wscale_dev;     /* (E,) fp32, device */
    const float *inv_rs2_dev;    /* (E,) fp32, device; read only with a second stage */
    const int64_t *blocks_n;     /* host */
    int64_t n_blocks_n;
    const glqh_block_meta *bn_meta_dev;
    const int64_t *blocks_m;     /* host; must be the block_decompose sizes of m_pad */
    int64_t n_blocks_m;
    int64_t in_features, out_features, n_pad, m_pad;
} glqh_moe_proj;

size_t glqh_fused_moe_trellis_workspace_bytes(int64_t num_tokens, int64_t top_k, int64_t num_experts,
                                              const glqh_moe_proj *w13, const glqh_moe_proj *w2);

/* The routed-expert step of a mixture-of-experts layer on trellis-3INST weights,
 * out[t] = sum_j topk_weights[t][j] * w2_e( act(gate) * up ),  (gate | up) = w13_e(x[t]),
 * e = topk_ids[t][j], as one host call with the routing read on the device (no host
 * synchronisation, no allocation: capturable).  Replaces glq_fused_moe_trellis_3inst_cuda
 * (glq/csrc/glq_cuda.cu:5030-5250; grouped matmul glq/csrc/glq_trellis.cu:1475-1540) behind
 * torch.ops.glq.fused_moe_trellis_3inst (glq_vllm/custom_ops.py:22-36).  With few (token,
 * choice) slots every slot is one fused-input GEMV on its expert's stream; from
 * max(16, 3/4 num_experts) slots on a routing launch groups the slots by expert and every
 * expert's stream is read once per 16 of its rows (GLQ_MOE_GROUP_MIN sets that count), once
 * per up to 64 rows from an average of 12 rows per expert on (GLQ_MOE_WIDE_MIN_ROWS); from an
 * average of 24 rows per expert on (GLQ_MOE_TILE_MIN_ROWS, 0 = never) the expert-sorted slots go
 * through the many-token tile kernel in runs of up to 128-512 rows of one expert, the decoded
 * weights of a 128-row tile meeting the whole run on the matrix cores.  From 1024 slots on the
 * launches between the two projections (output transform, activation, input transform) and after
 * them (output transform, weighted sum) are one launch each (GLQ_MOE_FUSE=0: separate), with the
 * same roundings and the same bits.  Intermediate results are rounded to
 * fp16 where the reference rounds them (after each output transform and after the
 * activation), the weighted sum runs over the choices in order in fp32.  activation_type:
 * 0 SiLU, 1 GELU (tanh form), 2 squared ReLU, each times the up half.  Expert ids outside
 * [0, num_experts) contribute nothing.  x f16 or bf16, out f16 or bf16. */
int glqh_fused_moe_trellis_3inst(const void *x, int x_dtype, int64_t x_stride, int64_t num_tokens,
                                 const int64_t *topk_ids, const float *topk_weights, int64_t top_k,
                                 int64_t num_experts, const glqh_moe_proj *w13, const glqh_moe_proj *w2,
                                 int64_t intermediate_size, int activation_type, void *out, int out_dtype,
                                 int64_t out_stride, void *ws, size_t ws_bytes, void *stream);

/* ---- E8 shell codebook ---------------------------------------------------- */

/* (n_entries, 8) fp16 table -> n_entries uint32 of eight 4-bit codes round(2 v) + 6, the
 * codes of glq/codebook.py:102-115 in the kernels' own nibble order (nibble p = column 2p,
 * nibble p + 4 = column 2p + 1).  *bad_dev (device int32, zeroed by the caller) counts the
 * rows with a coordinate outside {-3, -2.5, ..., 3}; if it is nonzero afterwards the packed
 * table must not be used. */
int glqh_e8_pack_table(const void *codebook_f16, int64_t n_entries, uint32_t *packed_out,
                       int32_t *bad_dev, void *stream);

/* The reference's `codebook_packed` buffer (n_entries int32, nibble c = code of column c,
 * glq/codebook.py:102-115, consumed by glq_dequant_matvec_packed_cuda /
 * glq_dequant_matmul_packed_cuda, glq/csrc/glq_bindings.cpp:38-50) -> the kernels' nibble
 * order.  *bad_dev counts words holding a code above 12. */
int glqh_e8_repack_table(const uint32_t *codebook_packed, int64_t n_entries, uint32_t *packed_out,
                         int32_t *bad_dev, void *stream);

/* ---- folded form of the E8 streams (no counterpart in the reference) ---------------------
 * The 65536 codewords of the shell table are built from only 1286 distinct half codewords
 * (columns 0..3 or 4..7, signs included).  A table of those as finished fp16 values (8 bytes
 * each) fits LDS whole, so the small-batch kernel (1..16 tokens) and the many-token tile kernel
 * (17 tokens and more, n_pad a multiple of 256) look every index up without leaving the CU and
 * without expanding anything -- at the price of a second, on-device copy of the index streams:
 * per index two 11-bit half numbers, stored as a 16-bit word plus a byte (3 bytes instead of
 * 2).  Made once per table and per layer at load time; the original indices stay in use for
 * every other route (small or ragged layers, decompress + library GEMM, the embedding). */
typedef struct {
    const uint16_t *lo16[4];     /* per stage, tile order: first half number | (second & 31) << 11 */
    const uint8_t *hi8[4];       /* per stage, tile order: second half number >> 5 */
    const void *halves1;         /* half-codeword table of stage 1 (and of stages 3, 4): 4 fp16 per entry */
    int64_t n_halves1;
    const void *halves2;         /* the same for stage 2 when it has a table of its own, else NULL */
    int64_t n_halves2;
} glqh_e8_folded;

/* table: n_entries nibble-packed words (glqh_e8_pack_table / glqh_e8_repack_table), device.
 * halves_out (device, room for `capacity` entries of 8 bytes; the kernels take up to 2048): the
 * distinct half codewords in order of first appearance (first half of an entry before its
 * second), as 4 fp16 values; map_out (device, n_entries words): entry k = number of its first
 * half | number of its second half << 16.  *n_halves_out (host) = the count; fails if it
 * exceeds `capacity`.  Copies the table to the host and the results back: synchronizes the
 * stream, not capturable. */
int glqh_e8_fold_table(const uint32_t *table, int64_t n_entries, void *halves_out, int64_t capacity,
                       uint32_t *map_out, int64_t *n_halves_out, void *stream);

/* 1 when a product of this shape and token count reads the folded streams (the LDS-table
 * kernel or, above 16 tokens, the tile kernel serves it), 0 when they would go unused. */
int glqh_e8_fold_eligible(int64_t m_pad, int64_t n_pad, int64_t B);

/* Entries of a folded stream of a (rows, cols) index matrix: rows padded to 16, cols to 32. */
int64_t glqh_e8_folded_count(int64_t rows, int64_t cols);

/* q: (rows, cols) int16 indices read as unsigned (clamped to n_entries - 1) -> lo16_out and
 * hi8_out, glqh_e8_folded_count(rows, cols) entries each, through `map` of glqh_e8_fold_table,
 * in the tile order the kernel reads (16 rows x 32 indices per tile, the 8 consecutive indices
 * of row i, group g at entry 8 * (16 g + i) of the tile; padding holds half number 0).
 * Asynchronous. */
int glqh_e8_fold_indices(const void *q, int64_t rows, int64_t cols, const uint32_t *map, int64_t n_entries,
                         uint16_t *lo16_out, uint8_t *hi8_out, void *stream);

size_t glqh_e8_matmul_workspace_bytes(int64_t m_pad, int64_t n_pad, int64_t B);

/* out[b, :] (fp32, stride m_pad) = wscale * (cb[q1] + inv_rs*cb2[q2] + inv_rs2*cb3[q3]
 * + inv_rs3*cb4[q4]) @ x[b, :], x (B, n_pad) fp16 in the RHT domain, q* (m_pad, n_pad/8)
 * int16 read as unsigned.  A stage is absent when its index pointer is NULL or its scale
 * is 0.  Tables are nibble-packed (glqh_e8_pack_table); table1 must hold all 65536 rows
 * (it is indexed with the full 16-bit pattern and its low-norm prefix is copied to LDS),
 * table2 has n_entries2 rows (65536, or 256 for the 3-bit recipe), stages 3-4 use table 1.
 * glq_dequant_matvec_cuda / glq_dequant_matmul_cuda, glq/csrc/glq_cuda.cu:1384-1637. */
int glqh_e8_dequant_matmul(const void *x_f16, int64_t B,
                           const void *q1, const void *q2, const void *q3, const void *q4,
                           const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                           double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                           int64_t m_pad, int64_t n_pad,
                           float *out, void *ws, size_t ws_bytes, void *stream);

/* The same with the layer's folded streams beside the indices: up to 16 tokens on shapes
 * the LDS-table kernel serves, the product reads `folded` instead of q1..q4 / the tables;
 * every other case ignores it.  Same workspace.  The decoded values are the same; the K plan
 * may differ (on folded streams K can stay inside a workgroup, and one- and two-stage
 * products are then written finished, without a reduction launch), so results agree with
 * glqh_e8_dequant_matmul to fp32 summation order (1e-5 relative), bit for bit where the plans
 * coincide.  folded == NULL is glqh_e8_dequant_matmul. */
int glqh_e8_dequant_matmul_folded(const void *x_f16, int64_t B,
                                  const void *q1, const void *q2, const void *q3, const void *q4,
                                  const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                  double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                                  int64_t m_pad, int64_t n_pad,
                                  float *out, void *ws, size_t ws_bytes, void *stream,
                                  const glqh_e8_folded *folded);

/* Dense fp16 (m_pad, n_pad) RHT-domain weight before Wscale: cb[q1] + inv_rs*cb2[q2] + ...
 * combined in fp32 and rounded once.  First half of the many-token path of
 * glq_dequant_matmul_cuda (glq/csrc/glq_cuda.cu:1519-1637): dequantize once, then one
 * library GEMM, as the reference's trellis prefill does (glq/csrc/glq_trellis.cu:1322-1334). */
int glqh_e8_decompress(const void *q1, const void *q2, const void *q3, const void *q4,
                       const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                       double inv_rs, double inv_rs2, double inv_rs3,
                       int64_t m_pad, int64_t n_pad, void *out_f16, void *stream);

/* The same weight as unrounded fp32 sums: the RHT-domain half of E8RHTLinear.dequantize
 * (glq/quantized_linear.py:1237-1249) and dequantize_glq_weight (glq_vllm/dequant.py:31-44),
 * which decode every stage and combine them in fp32. */
int glqh_e8_decompress_f32(const void *q1, const void *q2, const void *q3, const void *q4,
                           const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                           double inv_rs, double inv_rs2, double inv_rs3,
                           int64_t m_pad, int64_t n_pad, float *out_f32, void *stream);

/* Quantized embedding lookup: rows `ids` of a (num_embeddings, n_pad/8) index matrix are decoded,
 * scaled per row, inverse-transformed (one power-of-two block of n_pad <= 8192 values) and
 * written as (n_ids, embedding_dim) rows of `out`:
 *   out[t] = embed_scale * sv * H(Wscale[id] * (cb[q1[id]] + inv_rs[id] * cb2[q2[id]])) / sqrt(n_pad).
 * ids: int64 on the device; an id outside [0, num_embeddings) yields a zero row.  q2 / table2 /
 * inv_rs may be NULL (single stage); wscale and inv_rs hold one fp32 per row.
 * _dequant_embedding_rows / E8RHTEmbedding.forward, glq/quantized_linear.py:1277-1340, 1427-1446;
 * op schema glq_vllm/custom_ops.py:301-308. */
int glqh_e8_embedding_rows(const int64_t *ids, int64_t n_ids,
                           const void *q1, const void *q2,
                           const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                           const float *wscale_rows, const float *inv_rs_rows, const void *sv_f16,
                           int64_t n_pad, int64_t embedding_dim, int64_t num_embeddings,
                           double embed_scale, void *out, int out_dtype, int64_t out_stride,
                           void *stream);

size_t glqh_fused_linear_e8_workspace_bytes(int64_t B, int64_t n_pad, int64_t m_pad);

/* Whole E8 linear: input RHT -> gather-matmul -> output RHT.
 * glq_fused_linear_cuda (pow2, one block each side) and
 * glq_fused_linear_block_diag_cuda, glq/csrc/glq_cuda.cu:2533-2742, 3038-3266. */
int glqh_fused_linear_e8(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                         const void *sv_f16, const void *su_f16,
                         const void *q1, const void *q2, const void *q3, const void *q4,
                         const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                         double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                         const int64_t *blocks_n, int64_t n_blocks_n,
                         const int64_t *blocks_m, int64_t n_blocks_m,
                         const glqh_block_meta *bn_meta_dev, const glqh_block_meta *bm_meta_dev,
                         int64_t in_features, int64_t out_features, int64_t n_pad, int64_t m_pad,
                         void *y, int y_dtype, int64_t y_stride,
                         void *ws, size_t ws_bytes, void *stream);

/* glqh_fused_linear_e8 with the layer's folded streams (see glqh_e8_dequant_matmul_folded). */
int glqh_fused_linear_e8_folded(const void *x, int x_dtype, int64_t x_stride, int64_t B,
                                const void *sv_f16, const void *su_f16,
                                const void *q1, const void *q2, const void *q3, const void *q4,
                                const uint32_t *table1, const uint32_t *table2, int64_t n_entries2,
                                double wscale, double inv_rs, double inv_rs2, double inv_rs3,
                                const int64_t *blocks_n, int64_t n_blocks_n,
                                const int64_t *blocks_m, int64_t n_blocks_m,
                                const glqh_block_meta *bn_meta_dev, const glqh_block_meta *bm_meta_dev,
                                int64_t in_features, int64_t out_features, int64_t n_pad, int64_t m_pad,
                                void *y, int y_dtype, int64_t y_stride,
                                void *ws, size_t ws_bytes, void *stream,
                                const glqh_e8_folded *folded);

/* ---- encode side --------------------------------------------------------------- */

/* Nearest row of an (n_entries, 8) fp32 table for each of N fp32 vectors:
 * argmin_k( norms[k] - 2 <x, table[k]> ) with the lowest index winning ties; idx_out (N) int64,
 * decoded_out (N, 8) fp32 or NULL.  E8ShellCodebook.quantize / _quantize_pytorch
 * (glq/codebook.py:227-278), triton_codebook_nn(_decode) (glq/codebook_kernel.py:169-256).
 * norms = |table[k]|^2 (fp32), as the reference's codebook_norms buffer. */
int glqh_e8_quantize(const float *x, const float *table_f32, const float *norms_f32, int64_t N,
                     int64_t n_entries, int64_t *idx_out, float *decoded_out, void *stream);

size_t glqh_trellis_quantize_workspace_bytes(int K, int64_t n_tiles);

/* Tail-biting Viterbi search of the 3INST trellis for n_tiles sequences of 256 fp32 values
 * (a 16x16 tile in step order): states_out (n_tiles, 256) int32, hat_out (n_tiles, 256) fp32 =
 * decode_3inst(state).  Inputs are rounded to fp16 first, costs are fp32, ties go to the
 * lowest predecessor / lowest final state; two passes tie the ends together.
 * bitshift_codebook.quantize / viterbi (glq/trellis.py:253-296, 467-484) and the Triton
 * add-compare-select step (glq/trellis_step_kernel.py:30-109).  K = 1..4. */
int glqh_trellis_quantize_tiles(const float *tiles, int64_t n_tiles, int K, int32_t *states_out,
                                float *hat_out, void *ws, size_t ws_bytes, void *stream);

/* One add-compare-select step of that search on cost rows in memory, for callers that
 * drive the search step by step: cost (B, 65536) fp32 -> cost_out (B, 65536) fp32 and
 * prev_out (B, 2^(16-K)) int32, with x (B) fp16 the step's inputs and lut (65536) fp32 the
 * state values.  prev_out[b, j] = j + (k* << (16-K)), k* = first minimum over ascending k of
 * cost[b, k*2^(16-K) + j] (a NaN displaces a number); cost_out[b, j*2^K + r] =
 * (lut[j*2^K + r] - x[b])^2 + that minimum, separate subtract, multiply and add.
 * bitshift_codebook.update (glq/trellis.py:230-251) = fused_update
 * (glq/trellis_step_kernel.py:30-109) at V = 1, L = 16.  cost_out must not alias cost. */
int glqh_viterbi_acs_step(const float *cost, const void *x_f16, const float *lut_f32, float *cost_out,
                          int32_t *prev_out, int64_t B, int K, void *stream);

/* Trellis states of an (m, n) layer (tiles in row-major tile order, 256 steps each, int32)
 * -> packed ((m/16)(n/16), 16K) int16 in the kernel layout, K = 1..4.
 * bitshift_codebook.pack_trellis + pack_layer (glq/trellis.py:486-510, 580-619). */
int glqh_trellis_pack_states(const int32_t *states, int64_t m, int64_t n, int K, void *packed_out,
                             void *stream);

#ifdef __cplusplus
}
#endif
#endif /* GLQ_HIP_H */
