// Randomized Hadamard transforms around the quantized matmul.
//
// One workgroup transforms one power-of-two sub-block of one token.  The block is
// staged in LDS as fp32 and the log2(bs) butterfly stages run in place in ascending
// distance with (lo, hi) <- (a + b, a - b), the order the reference's CPU and CUDA
// paths use (glq/hadamard.py:10-28, glq/csrc/glq_fht.cuh:14-21), followed by one
// multiplication with 1/sqrt(bs).
#include "common.h"

namespace {

constexpr int RHT_THREADS = 256;

struct rht_block {
    int off, bs, log_bs;
    float norm;
};

__device__ __forceinline__ rht_block rht_get_block(const glqh_block_meta *meta, glqh_block_meta single,
                                                   float single_norm) {
    glqh_block_meta mrow = meta ? meta[blockIdx.x] : single;
    rht_block b;
    b.off = mrow.offset;
    b.bs = mrow.bs;
    b.log_bs = mrow.log_bs;
    if (mrow.w != 0) b.norm = __builtin_bit_cast(float, mrow.w);
    else if (!meta && single_norm != 0.0f) b.norm = single_norm;
    else  // 1/sqrt(2^L) exactly rounded: a power of two, times 1/sqrt(2) when L is odd
        b.norm = ldexpf((mrow.log_bs & 1) ? 0.70710678118654752f : 1.0f, -(mrow.log_bs >> 1));
    return b;
}

// In-place Walsh-Hadamard butterflies over s[0..bs) held in LDS.  All threads of the
// workgroup must call it; ends with a barrier.
__device__ __forceinline__ void fht_lds(float *s, int bs) {
    const int tid = threadIdx.x;
    const int nthr = blockDim.x;
    for (int h = 1; h < bs; h <<= 1) {
        __syncthreads();
        for (int p = tid; p < (bs >> 1); p += nthr) {
            int i = ((p & ~(h - 1)) << 1) | (p & (h - 1));
            int j = i | h;
            float a = s[i], b = s[j];
            s[i] = a + b;
            s[j] = a - b;
        }
    }
    __syncthreads();
}

__global__ void __launch_bounds__(RHT_THREADS)
input_rht_kernel(const void *__restrict__ x, int x_dtype, int64_t x_stride,
                 const f16 *__restrict__ sv, void *__restrict__ out, int out_dtype,
                 int in_features, int n_pad, const glqh_block_meta *__restrict__ meta,
                 glqh_block_meta single, float single_norm) {
    extern __shared__ float s[];
    const rht_block blk = rht_get_block(meta, single, single_norm);
    const int64_t b = blockIdx.y;
    for (int i = threadIdx.x; i < blk.bs; i += blockDim.x) {
        int col = blk.off + i;
        float v = 0.0f;
        if (col < in_features) v = load_act(x, x_dtype, b * x_stride + col) * (float)sv[col];
        s[i] = v;
    }
    fht_lds(s, blk.bs);
    for (int i = threadIdx.x; i < blk.bs; i += blockDim.x)
        store_act(out, out_dtype, b * (int64_t)n_pad + blk.off + i, s[i] * blk.norm);
}

__global__ void __launch_bounds__(RHT_THREADS)
output_rht_kernel(glqh_ysrc src, const f16 *__restrict__ su, void *__restrict__ y, int y_dtype,
                  int64_t y_stride, int out_features, int m_pad,
                  const glqh_block_meta *__restrict__ meta, glqh_block_meta single,
                  float single_norm) {
    extern __shared__ float s[];
    const rht_block blk = rht_get_block(meta, single, single_norm);
    const int64_t b = blockIdx.y;
    for (int i = threadIdx.x; i < blk.bs; i += blockDim.x) {
        int row = blk.off + i;
        float v;
        if (src.nparts == 0) {
            v = src.direct[b * src.stride + row];
        } else {
            // fixed-order sum of the split-K partials of each stage: deterministic
            v = 0.0f;
            for (int st = 0; st < src.nparts; ++st) {
                const float *p = src.part[st] + b * (int64_t)m_pad + row;
                float acc = 0.0f;
                for (int k = 0; k < src.ksplit; ++k) acc += p[(int64_t)k * src.part_kstride];
                v += src.scale[st] * acc;
            }
            if (src.copy_out) src.copy_out[b * src.copy_stride + row] = v;
        }
        s[i] = v;
    }
    if (y == nullptr) return;                 // caller only wanted the RHT-domain row
    fht_lds(s, blk.bs);
    for (int i = threadIdx.x; i < blk.bs; i += blockDim.x) {
        int row = blk.off + i;
        if (row < out_features)
            store_act(y, y_dtype, b * y_stride + row, s[i] * blk.norm * (float)su[row]);
    }
}

int check_blocks(const int64_t *blocks_host, int64_t n_blocks, int64_t total, int64_t *max_bs,
                 const char *what) {
    int64_t sum = 0, mx = 0;
    for (int64_t i = 0; i < n_blocks; ++i) {
        int64_t bs = blocks_host[i];
        GLQH_REQUIRE(bs > 0 && (bs & (bs - 1)) == 0, "%s: block size %lld is not a power of two",
                     what, (long long)bs);
        sum += bs;
        mx = bs > mx ? bs : mx;
    }
    GLQH_REQUIRE(sum == total, "%s: block sizes sum to %lld, expected %lld", what, (long long)sum,
                 (long long)total);
    *max_bs = mx;
    return 0;
}

int ilog2(int64_t v) {
    int l = 0;
    while ((1ll << l) < v) ++l;
    return l;
}

}  // namespace

int glqh_launch_input_rht(const void *x, int x_dtype, int64_t x_stride, const void *sv,
                          void *out, int out_dtype, int64_t B, int64_t in_features, int64_t n_pad,
                          const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                          int64_t n_blocks, float rsqrt_n, hipStream_t stream) {
    GLQH_REQUIRE(x && sv && out, "input_rht: null pointer");
    GLQH_REQUIRE(B >= 1 && B <= 65535, "input_rht: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(in_features >= 1 && in_features <= n_pad,
                 "input_rht: in_features %lld must be in 1..n_pad=%lld", (long long)in_features,
                 (long long)n_pad);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16 || x_dtype == GLQH_F32,
                 "input_rht: bad x dtype");
    GLQH_REQUIRE(out_dtype == GLQH_F32 || out_dtype == GLQH_F16, "input_rht: out must be f32 or f16");
    int64_t max_bs = n_pad;
    glqh_block_meta single = {0, (int32_t)n_pad, ilog2(n_pad), 0};
    if (n_blocks > 1) {
        GLQH_REQUIRE(meta_dev && blocks_host, "input_rht: block-diagonal call needs meta and sizes");
        if (check_blocks(blocks_host, n_blocks, n_pad, &max_bs, "input_rht")) return 1;
    } else {
        GLQH_REQUIRE((n_pad & (n_pad - 1)) == 0, "input_rht: single block n_pad=%lld is not a power of two",
                     (long long)n_pad);
        meta_dev = nullptr;
        n_blocks = 1;
    }
    GLQH_REQUIRE(max_bs * 4 <= GLQH_MAX_LDS_BYTES, "input_rht: block of %lld exceeds LDS", (long long)max_bs);
    dim3 grid((unsigned)n_blocks, (unsigned)B);
    hipLaunchKernelGGL(input_rht_kernel, grid, dim3(RHT_THREADS), (size_t)max_bs * 4, stream, x, x_dtype,
                       x_stride, (const f16 *)sv, out, out_dtype, (int)in_features, (int)n_pad,
                       meta_dev, single, rsqrt_n);
    GLQH_LAUNCH_CHECK("input_rht launch");
    return 0;
}

int glqh_launch_output_rht(const glqh_ysrc &src, const void *su, void *y, int y_dtype,
                           int64_t y_stride, int64_t B, int64_t out_features, int64_t m_pad,
                           const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                           int64_t n_blocks, int64_t max_bs_hint, float rsqrt_m,
                           hipStream_t stream) {
    GLQH_REQUIRE(B >= 1 && B <= 65535, "output_rht: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(y == nullptr || su != nullptr, "output_rht: null su");
    GLQH_REQUIRE(out_features >= 1 && out_features <= m_pad,
                 "output_rht: out_features %lld must be in 1..m_pad=%lld", (long long)out_features,
                 (long long)m_pad);
    GLQH_REQUIRE(y_dtype == GLQH_F16 || y_dtype == GLQH_BF16 || y_dtype == GLQH_F32,
                 "output_rht: bad y dtype");
    int64_t max_bs = m_pad;
    glqh_block_meta single = {0, (int32_t)m_pad, ilog2(m_pad), 0};
    if (n_blocks > 1 || (meta_dev && !blocks_host)) {
        GLQH_REQUIRE(meta_dev, "output_rht: block-diagonal call needs meta");
        if (blocks_host) {
            if (check_blocks(blocks_host, n_blocks, m_pad, &max_bs, "output_rht")) return 1;
        } else {
            GLQH_REQUIRE(max_bs_hint > 0 && (max_bs_hint & (max_bs_hint - 1)) == 0,
                         "output_rht: max_bs %lld is not a power of two", (long long)max_bs_hint);
            max_bs = max_bs_hint;
        }
    } else {
        GLQH_REQUIRE((m_pad & (m_pad - 1)) == 0, "output_rht: single block m_pad=%lld is not a power of two",
                     (long long)m_pad);
        meta_dev = nullptr;
        n_blocks = 1;
    }
    GLQH_REQUIRE(max_bs * 4 <= GLQH_MAX_LDS_BYTES, "output_rht: block of %lld exceeds LDS", (long long)max_bs);
    dim3 grid((unsigned)n_blocks, (unsigned)B);
    hipLaunchKernelGGL(output_rht_kernel, grid, dim3(RHT_THREADS), (size_t)max_bs * 4, stream, src,
                       (const f16 *)su, y, y_dtype, y_stride, (int)out_features, (int)m_pad,
                       meta_dev, single, rsqrt_m);
    GLQH_LAUNCH_CHECK("output_rht launch");
    return 0;
}

int glqh_rht_init(void) {
    int rc = glqh_check_hip(hipFuncSetAttribute((const void *)input_rht_kernel,
                                                hipFuncAttributeMaxDynamicSharedMemorySize,
                                                GLQH_MAX_LDS_BYTES), "input_rht attribute");
    if (rc) return rc;
    return glqh_check_hip(hipFuncSetAttribute((const void *)output_rht_kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize,
                                              GLQH_MAX_LDS_BYTES), "output_rht attribute");
}
