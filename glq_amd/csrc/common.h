// Shared host/device helpers for libglq_hip (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <hip/hip_fp16.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/glq_hip.h"

typedef _Float16 f16;
typedef _Float16 f16x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x2 __attribute__((ext_vector_type(2)));
typedef uint32_t u32x4 __attribute__((ext_vector_type(4)));
typedef float f32x4 __attribute__((ext_vector_type(4)));
typedef float f32x2 __attribute__((ext_vector_type(2)));

#define GLQH_WAVE 64
#define GLQH_MAX_GROUP GLQH_MAX_SHARDS      // layers per grouped launch
#define GLQH_MAX_LDS_BYTES (160 * 1024)

// ---- error reporting (host) -------------------------------------------------
int glqh_fail(const char *fmt, ...);             // sets the thread-local message, returns 1
int glqh_check_hip(hipError_t e, const char *what);
int glqh_device_cus(void);                       // cached compute-unit count

// Named host-side range around the launches of one phase of a linear, under the reference's
// three names (glq/quantized_linear.py:1132-1233: "input_rht", "dequant_matmul", "output_rht"),
// for rocprofv3 --marker-trace.  Uses the roctx library when the process already has one loaded
// (torch does) or GLQ_ROCTX=1 asks to load it; GLQ_ROCTX=0 switches the ranges off.
struct glqh_range {
    bool on;
    explicit glqh_range(const char *name);
    ~glqh_range();
    glqh_range(const glqh_range &) = delete;
    glqh_range &operator=(const glqh_range &) = delete;
};

#define GLQH_REQUIRE(cond, ...)            \
    do {                                   \
        if (!(cond)) return glqh_fail(__VA_ARGS__); \
    } while (0)

#define GLQH_LAUNCH_CHECK(what)                                   \
    do {                                                          \
        int rc_ = glqh_check_hip(hipGetLastError(), what);        \
        if (rc_) return rc_;                                      \
    } while (0)

// ---- small device helpers -----------------------------------------------------
__device__ __forceinline__ float bf16_bits_to_f32(uint16_t b) {
    return __builtin_bit_cast(float, (uint32_t)b << 16);
}

__device__ __forceinline__ uint16_t f32_to_bf16_bits(float f) {   // round-to-nearest-even
    uint32_t u = __builtin_bit_cast(uint32_t, f);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40);   // NaN
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}

__device__ __forceinline__ float load_act(const void *p, int dtype, int64_t i) {
    if (dtype == GLQH_F16) return (float)((const f16 *)p)[i];
    if (dtype == GLQH_BF16) return bf16_bits_to_f32(((const uint16_t *)p)[i]);
    return ((const float *)p)[i];
}

__device__ __forceinline__ void store_act(void *p, int dtype, int64_t i, float v) {
    if (dtype == GLQH_F16) ((f16 *)p)[i] = (f16)v;
    else if (dtype == GLQH_BF16) ((uint16_t *)p)[i] = f32_to_bf16_bits(v);
    else ((float *)p)[i] = v;
}

// Block meta carried in the kernel arguments (no dependent global load at the start of a
// latency-bound kernel).  When the block sizes are the descending power-of-two decomposition
// of their total (what block_decompose yields), the total alone determines every row:
// block j is the j-th set bit of `canon` from the top and its offset is the sum of the bits
// above it.  canon == 0 means "read the device array".
struct glqh_meta_args {
    int canon;
};

__device__ __forceinline__ glqh_block_meta glqh_meta_row(const glqh_meta_args a,
                                                         const glqh_block_meta *dev, int j) {
    if (a.canon == 0) return dev[j];
    uint32_t rem = (uint32_t)a.canon;
    for (int i = 0; i < j; ++i) rem &= ~(0x80000000u >> __builtin_clz(rem));   // j is uniform
    const int l = 31 - __builtin_clz(rem);
    glqh_block_meta r;
    r.offset = a.canon - (int)rem;
    r.bs = 1 << l;
    r.log_bs = l;
    r.w = 0;
    return r;
}

// canon from host block sizes; 0 when they are not the canonical decomposition
inline int glqh_fill_meta_args(glqh_meta_args *out, const int64_t *blocks, int64_t n_blocks,
                               int64_t single_size) {
    out->canon = 0;
    if (n_blocks <= 1) {
        if (single_size <= 0 || single_size > 0x40000000ll || (single_size & (single_size - 1))) return 0;
        out->canon = (int)single_size;
        return 1;
    }
    if (!blocks) return 0;
    int64_t sum = 0, prev = 0x7fffffffffffffffll;
    for (int64_t i = 0; i < n_blocks; ++i) {
        const int64_t b = blocks[i];
        if (b <= 0 || (b & (b - 1)) || b >= prev) return 0;
        prev = b;
        sum += b;
    }
    if (sum > 0x7fffffffll) return 0;
    out->canon = (int)sum;
    return 1;
}

// internal kernels' host launchers (defined in fht.hip / trellis.hip / e8.hip)
struct glqh_ysrc {                 // where the output RHT reads its RHT-domain input
    const float *direct;           // (B, stride) fp32, or NULL when partials are used
    int64_t stride;                // row stride of `direct`
    const float *part;             // split-K partial sums: element (stage, k, b, row) at
                                   // part[stage * part_sstride + k * part_kstride + b * m_pad + row]
    int64_t part_sstride;
    int64_t part_kstride;
    int ksplit;
    float scale[4];                // wscale per stage (already multiplied by inv_rs)
    int nparts;
    float *copy_out;               // optional: also write the combined fp32 row here
    int64_t copy_stride;
    int part_f16;                  // the partial sums are fp16 (same strides, in elements); served by the
                                   // whole-block kernels only (glqh_output_rht_wide_eligible)
};

// 1 when glqh_launch_output_rht serves this call with the whole-block kernels (many tokens,
// canonical blocks of 8..8192 rows), the only ones that read fp16 partial sums.
int glqh_output_rht_wide_eligible(int64_t B, const int64_t *blocks_host, int64_t n_blocks, int64_t m_pad);

int glqh_launch_input_rht(const void *x, int x_dtype, int64_t x_stride, const void *sv,
                          void *out, int out_dtype, int64_t B, int64_t in_features, int64_t n_pad,
                          const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                          int64_t n_blocks, float rsqrt_n, hipStream_t stream);

int glqh_launch_output_rht(const glqh_ysrc &src, const void *su, void *y, int y_dtype,
                           int64_t y_stride, int64_t B, int64_t out_features, int64_t m_pad,
                           const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                           int64_t n_blocks, int64_t max_bs_hint, float rsqrt_m,
                           hipStream_t stream);

int glqh_launch_output_rht_canon_wide(const glqh_ysrc &src, const void *su, void *y, int y_dtype, int64_t y_stride,
                                      int64_t B, int64_t out_features, int64_t m_pad, hipStream_t stream);

// out[tok, row] = (accum ? out : 0) + scale * sum_s part[s * kstride + tok * m + row]
int glqh_launch_reduce_splits(const float *part, int ksplit, int64_t kstride, int64_t B, int64_t m,
                              float scale, float *out, int64_t out_stride, int accum,
                              hipStream_t stream);

// E8 gather matmul into per-stage split-K partials:
// part[((slot * nstages + stage) * B + tok) * m_pad + row]
int glqh_e8_pick_ksplit(int64_t m_pad, int64_t n_pad, int64_t B, int fold = 0);
int glqh_e8_mma_direct_ok(int64_t m_pad, int64_t n_pad, int64_t B, int nstages);
int glqh_launch_e8_pack_table(const void *cb, int64_t n_entries, uint32_t *out, int32_t *bad,
                              hipStream_t stream);
int glqh_launch_e8_repack_table(const uint32_t *in, int64_t n_entries, uint32_t *out, int32_t *bad,
                                hipStream_t stream);
// pscale: per-stage factors applied to the partial sums as they are written (NULL: ones)
struct glqh_e8_pscale {
    float v[4];
};
int glqh_launch_e8_partial(const void *x, int64_t B, const void *const q[4], int nstages,
                           const uint32_t *t1, const uint32_t *t2, int64_t n2, int64_t m_pad,
                           int64_t n_pad, int ksplit, float *part, hipStream_t stream,
                           const float *pscale = nullptr, const glqh_e8_folded *fold = nullptr, int direct = 0);
int glqh_launch_e8_fold_indices(const void *q, int64_t rows, int64_t cols, const uint32_t *map, int64_t n_entries,
                                uint16_t *lo16_out, uint8_t *hi8_out, hipStream_t stream);
int glqh_launch_e8_decompress(const void *const q[4], int nstages, const uint32_t *t1,
                              const uint32_t *t2, int64_t n2, float s2, float s3, float s4,
                              int64_t m_pad, int64_t n_pad, void *out, hipStream_t stream);
int glqh_launch_e8_decompress_f32(const void *const q[4], int nstages, const uint32_t *t1,
                                  const uint32_t *t2, int64_t n2, float s2, float s3, float s4,
                                  int64_t m_pad, int64_t n_pad, float *out, hipStream_t stream);

int glqh_launch_e8_embedding(const int64_t *ids, int64_t n_ids, const void *q1, const void *q2,
                             const uint32_t *t1, const uint32_t *t2, int64_t n2, const float *wscale,
                             const float *inv_rs, const void *sv, int64_t n_pad, int64_t embedding_dim,
                             int64_t num_embeddings, float embed_scale, void *out, int out_dtype,
                             int64_t out_stride, hipStream_t stream);

// fused-input trellis GEMV (B <= 4): plan returns 0 when the shape/batch is not eligible
int glqh_trellis_fusein_plan(int64_t m, int64_t k, int64_t B, int *steps_out, int *ksplit_out);
size_t glqh_trellis_fusein_lds(int steps, int NB);
int glqh_launch_trellis_fusein(const void *packed, int R, const void *x, int x_dtype, int64_t x_stride,
                               const void *sv, int64_t B, int64_t m, int64_t k, int64_t in_features,
                               int steps, int ksplit, const glqh_block_meta *bn_meta,
                               const int64_t *blocks_host, int n_blocks, float *part,
                               hipStream_t stream);
int glqh_launch_trellis_fusein_group(const void *const packed[], const void *const sv[], float *const part[],
                                     const int64_t m[], int n_shards, int R, const void *x, int x_dtype,
                                     int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int steps,
                                     int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                     int n_blocks, hipStream_t stream);
// one output transform per shard from its split-K partials, all in one launch
int glqh_launch_output_rht_group(const float *const part[], const void *const su[], void *const y[],
                                 const float scale[], const int64_t m_pad[], const int64_t out_features[],
                                 int n_shards, int y_dtype, int64_t y_stride, int64_t B, int ksplit,
                                 hipStream_t stream);
// decode-loop epilogues (decoder_ops.hip): one token, split-K partials -> output transform -> ...
int glqh_launch_out_add_rmsnorm(const float *part, int ksplit, float scale, const void *su, int64_t m,
                                const void *resid, const void *norm_w, float eps, void *x_out, void *h_out,
                                hipStream_t stream);
int glqh_launch_out_silu_mul(const float *part_gate, const float *part_up, int ksplit, float scale_gate,
                             float scale_up, const void *su_gate, const void *su_up, int64_t m_pad,
                             int64_t out_features, void *act_out, hipStream_t stream);
int glqh_launch_out_rope_store(const float *const part[3], const void *const su[3], const float scale[3],
                               const int64_t m[3], int ksplit, const int64_t *pos, const void *cos_t,
                               const void *sin_t, void *q_out, void *k_cache, void *v_cache, int64_t head_dim,
                               int64_t max_len, int apply_rope, hipStream_t stream);
int glqh_launch_out_rope_attn(const float *const part[3], const void *const su[3], const float scale[3],
                              const int64_t m[3], int ksplit, const int64_t *pos, const void *cos_t,
                              const void *sin_t, void *k_cache, void *v_cache, void *out, int64_t heads,
                              int64_t kv_heads, int64_t head_dim, int64_t max_len, int apply_rope,
                              void *split_state, size_t split_state_bytes, hipStream_t stream);
int glqh_attn_split_shares(int64_t max_len);
int glqh_trellis_init(void);
