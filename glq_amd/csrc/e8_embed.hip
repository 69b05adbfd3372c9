// Quantized embedding lookup: gather the requested rows' E8 indices, decode them, undo the
// right-side transform and scale -- the per-row path of E8RHTEmbedding
// (glq/quantized_linear.py:1277-1340, 1427-1446):
//
//     out[t, :] = embed_scale * sv * H_n( Wscale[id] * (cb[q1[id]] + inv_rs[id] * cb2[q2[id]]) ) / sqrt(n)
//
// One workgroup per token: the row's n_pad/8 indices are read once (2 bytes per 8 values,
// coalesced), each looked up in the 4-bit-coded table (256 KB, L2 resident), the decoded row
// is staged in LDS, transformed there and written out in the caller's dtype.  The bound is
// the HBM read of the indices: 2 (or 4) bytes per 8 output values.
#include "common.h"
#include "fht_device.h"

namespace {

constexpr int EMB_THREADS = 256;
constexpr int EMB_MAX_LOG_N = 13;                                // 8192 values: 33 KB of LDS

// value of coordinate c (0..7) of a table word (codes 0..12 -> -3..3 step 1/2; nibble
// (c >> 1) + 4 * (c & 1) holds coordinate c)
__device__ __forceinline__ float emb_coord(uint32_t word, int c) {
    const int pos = (c >> 1) + 4 * (c & 1);
    return (float)((word >> (4 * pos)) & 15u) * 0.5f - 3.0f;
}

template <typename OT>
__global__ void __launch_bounds__(EMB_THREADS)
e8_embedding_kernel(const int64_t *__restrict__ ids, const uint16_t *__restrict__ q1,
                    const uint16_t *__restrict__ q2, const uint32_t *__restrict__ t1,
                    const uint32_t *__restrict__ t2, uint32_t n2, const float *__restrict__ wscale,
                    const float *__restrict__ inv_rs, const f16 *__restrict__ sv, int log_n,
                    int embedding_dim, int64_t num_embeddings, float embed_scale, OT *__restrict__ out,
                    int64_t out_stride) {
#pragma clang fp contract(off)                                   // (v1 + v2 * inv) * ws, each step rounded
    extern __shared__ float s[];
    const int n = 1 << log_n;
    const int nblk = n >> 3;
    const int64_t tok = blockIdx.x;
    const int64_t id = ids[tok];
    const bool valid = id >= 0 && id < num_embeddings;           // uniform over the workgroup
    OT *orow = out + tok * out_stride;
    if (!valid) {                                                // an id outside the table yields a zero row
        for (int i = threadIdx.x; i < embedding_dim; i += EMB_THREADS) orow[i] = f32_to_act<OT>(0.0f);
        return;
    }
    const float ws = wscale[id];
    const float inv = q2 ? inv_rs[id] : 0.0f;
    const uint16_t *r1 = q1 + id * nblk;
    const uint16_t *r2 = q2 ? q2 + id * nblk : nullptr;
    for (int j = threadIdx.x; j < nblk; j += EMB_THREADS) {
        const uint32_t w1 = t1[r1[j]];
        uint32_t w2 = 0x66666666u;                               // the zero vector (code 6 = 0.0)
        if (r2) {
            const uint32_t i2 = r2[j];
            w2 = t2[i2 < n2 ? i2 : n2 - 1];
        }
#pragma unroll
        for (int c = 0; c < 8; ++c) {
            float v = emb_coord(w1, c);
            if (r2) v = v + emb_coord(w2, c) * inv;
            s[lds_pad(8 * j + c)] = v * ws;
        }
    }
    __syncthreads();
    struct {
        OT *orow;
        const f16 *sv;
        int embedding_dim;
        float norm, scale;
        __device__ float aux(int i) const { return (float)sv[i]; }
        __device__ void put(int i, float v, float f) const {
            if (i < embedding_dim) orow[i] = f32_to_act<OT>(v * norm * f * scale);
        }
    } store = {orow, sv, embedding_dim, rsqrt_pow2(log_n), embed_scale};
    fht_staged(s, log_n, store);
}

}  // namespace

int glqh_launch_e8_embedding(const int64_t *ids, int64_t n_ids, const void *q1, const void *q2,
                             const uint32_t *t1, const uint32_t *t2, int64_t n2, const float *wscale,
                             const float *inv_rs, const void *sv, int64_t n_pad, int64_t embedding_dim,
                             int64_t num_embeddings, float embed_scale, void *out, int out_dtype,
                             int64_t out_stride, hipStream_t stream) {
    GLQH_REQUIRE(ids && q1 && t1 && wscale && sv && out, "e8 embedding: null pointer");
    GLQH_REQUIRE(n_pad >= 8 && (n_pad & (n_pad - 1)) == 0, "e8 embedding: n_pad=%lld is not a power of two >= 8",
                 (long long)n_pad);
    GLQH_REQUIRE(n_pad <= (1ll << EMB_MAX_LOG_N), "e8 embedding: n_pad=%lld exceeds %d", (long long)n_pad,
                 1 << EMB_MAX_LOG_N);
    GLQH_REQUIRE(embedding_dim >= 1 && embedding_dim <= n_pad, "e8 embedding: embedding_dim %lld must be in 1..n_pad",
                 (long long)embedding_dim);
    GLQH_REQUIRE(!q2 || (t2 && n2 >= 1 && inv_rs), "e8 embedding: second stage needs its table and scales");
    GLQH_REQUIRE(n_ids >= 0 && n_ids <= 0x7fffffffll, "e8 embedding: %lld ids out of range", (long long)n_ids);
    GLQH_REQUIRE(out_stride >= embedding_dim, "e8 embedding: output stride %lld < embedding_dim", (long long)out_stride);
    if (n_ids == 0) return 0;
    int log_n = 0;
    while ((1ll << log_n) < n_pad) ++log_n;
    const size_t lds = (size_t)(n_pad + n_pad / 32 + 32) * sizeof(float);
    dim3 grid((unsigned)n_ids);
#define GLQH_EMB(OT)                                                                                         \
    hipLaunchKernelGGL((e8_embedding_kernel<OT>), grid, dim3(EMB_THREADS), lds, stream, ids,               \
                       (const uint16_t *)q1, (const uint16_t *)q2, t1, t2, (uint32_t)n2, wscale, inv_rs,    \
                       (const f16 *)sv, log_n, (int)embedding_dim, num_embeddings, embed_scale, (OT *)out,  \
                       out_stride)
    switch (out_dtype) {
    case GLQH_F16: GLQH_EMB(f16); break;
    case GLQH_BF16: GLQH_EMB(uint16_t); break;
    case GLQH_F32: GLQH_EMB(float); break;
    default: return glqh_fail("e8 embedding: bad output dtype %d", out_dtype);
    }
#undef GLQH_EMB
    GLQH_LAUNCH_CHECK("e8 embedding launch");
    return 0;
}
