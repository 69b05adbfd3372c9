// Randomized Hadamard transforms around the quantized matmul.
//
// One workgroup transforms one power-of-two sub-block of one token in fp32 and
// multiplies once with 1/sqrt(bs) (glq/hadamard.py:10-28, glq/csrc/glq_fht.cuh:14-21,
// glq/csrc/glq_cuda.cu:1756-1839, 2005-2079, 2092-2208).
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

// ---------------------------------------------------------------------------------
// Block transform in a few register-radix passes.
//
// The log2(bs) index bits are split into fields of at most RMAX bits, taken from the top
// bit down.  In one pass a thread owns groups of 2^r elements that differ only in the
// field's bits, runs the field's r butterfly stages in registers and puts the group
// back.  The first pass reads its elements through `load` (global memory: consecutive
// lanes touch consecutive addresses), the last pass hands them to `store`; in between
// the block lives in LDS with one pad word per 32 so that the strided accesses of the
// low fields stay conflict-free.  A butterfly stage is (lo, hi) <- (a + b, a - b); the
// stages of different bits commute, so the result is the Walsh-Hadamard transform of
// the block (summation order differs from the ascending-distance order of
// glq/hadamard.py:10-28 by fp32 rounding only).
// ---------------------------------------------------------------------------------
constexpr int RMAX = 5;

__device__ __forceinline__ int lds_pad(int i) { return i + (i >> 5); }

template <int R, bool FIRST, bool LAST, class Load, class Store>
__device__ __forceinline__ void fht_pass(float *lds, int bs, int s, Load &load, Store &store) {
    constexpr int N = 1 << R;
    const int ngroups = bs >> R;
    for (int g = threadIdx.x; g < ngroups; g += blockDim.x) {
        const int lo = g & ((1 << s) - 1);
        const int base = ((g >> s) << (s + R)) | lo;
        float v[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {                       // N independent loads in flight
            const int idx = base + (j << s);
            if constexpr (FIRST) v[j] = load(idx);
            else v[j] = lds[lds_pad(idx)];
        }
#pragma unroll
        for (int h = 1; h < N; h <<= 1) {
#pragma unroll
            for (int j = 0; j < N; ++j) {
                if ((j & h) == 0) {
                    const float a = v[j], b = v[j | h];
                    v[j] = a + b;
                    v[j | h] = a - b;
                }
            }
        }
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = base + (j << s);
            if constexpr (LAST) store(idx, v[j]);
            else lds[lds_pad(idx)] = v[j];
        }
    }
}

template <bool FIRST, bool LAST, class Load, class Store>
__device__ __forceinline__ void fht_pass_r(int r, float *lds, int bs, int s, Load &load, Store &store) {
    switch (r) {
    case 1: fht_pass<1, FIRST, LAST>(lds, bs, s, load, store); break;
    case 2: fht_pass<2, FIRST, LAST>(lds, bs, s, load, store); break;
    case 3: fht_pass<3, FIRST, LAST>(lds, bs, s, load, store); break;
    case 4: fht_pass<4, FIRST, LAST>(lds, bs, s, load, store); break;
    default: fht_pass<5, FIRST, LAST>(lds, bs, s, load, store); break;
    }
}

// All threads of the workgroup must call it.  lds needs bs + bs/32 floats.  With
// STAGED the block is already in LDS (padded layout) and `load` is not used.
template <bool STAGED, class Load, class Store>
__device__ __forceinline__ void fht_block(float *lds, int log_bs, Load load, Store store) {
    const int bs = 1 << log_bs;
    if (log_bs == 0) {
        if (threadIdx.x == 0) store(0, STAGED ? lds[0] : load(0));
        return;
    }
    const int npass = (log_bs + RMAX - 1) / RMAX;
    int s = log_bs;
    for (int p = 0; p < npass; ++p) {
        const int left = npass - p;
        const int r = (s + left - 1) / left;              // balanced field widths
        s -= r;
        const bool first = p == 0 && !STAGED, last = p == npass - 1;
        if (first && last) fht_pass_r<true, true>(r, lds, bs, s, load, store);
        else if (first) fht_pass_r<true, false>(r, lds, bs, s, load, store);
        else if (last) fht_pass_r<false, true>(r, lds, bs, s, load, store);
        else fht_pass_r<false, false>(r, lds, bs, s, load, store);
        if (!last) __syncthreads();
    }
}

template <typename T> __device__ __forceinline__ float act_to_f32(T v);
template <> __device__ __forceinline__ float act_to_f32<f16>(f16 v) { return (float)v; }
template <> __device__ __forceinline__ float act_to_f32<uint16_t>(uint16_t v) { return bf16_bits_to_f32(v); }
template <> __device__ __forceinline__ float act_to_f32<float>(float v) { return v; }
template <typename T> __device__ __forceinline__ T f32_to_act(float v);
template <> __device__ __forceinline__ f16 f32_to_act<f16>(float v) { return (f16)v; }
template <> __device__ __forceinline__ uint16_t f32_to_act<uint16_t>(float v) { return f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ float f32_to_act<float>(float v) { return v; }

// XT / OT: element types (bf16 travels as uint16_t)
template <typename XT, typename OT>
__global__ void __launch_bounds__(RHT_THREADS)
input_rht_kernel(const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv,
                 OT *__restrict__ out, int in_features, int n_pad,
                 const glqh_block_meta *__restrict__ meta, glqh_block_meta single,
                 float single_norm) {
    extern __shared__ float s[];
    const rht_block blk = rht_get_block(meta, single, single_norm);
    const XT *xr = x + (int64_t)blockIdx.y * x_stride;
    OT *orow = out + (int64_t)blockIdx.y * n_pad + blk.off;
    auto load = [&](int i) -> float {
        const int col = blk.off + i;
        return col < in_features ? act_to_f32<XT>(xr[col]) * (float)sv[col] : 0.0f;
    };
    auto store = [&](int i, float v) { orow[i] = f32_to_act<OT>(v * blk.norm); };
    fht_block<false>(s, blk.log_bs, load, store);
}

template <typename YT, bool PARTS>
__global__ void __launch_bounds__(RHT_THREADS)
output_rht_kernel(glqh_ysrc src, const f16 *__restrict__ su, YT *__restrict__ y, int64_t y_stride,
                  int out_features, int m_pad, const glqh_block_meta *__restrict__ meta,
                  glqh_block_meta single, float single_norm) {
    extern __shared__ float s[];
    const rht_block blk = rht_get_block(meta, single, single_norm);
    const int64_t b = blockIdx.y;
    YT *yrow = y + b * y_stride;
    auto store = [&](int i, float v) {
        const int row = blk.off + i;
        if (row < out_features) yrow[row] = f32_to_act<YT>(v * blk.norm * (float)su[row]);
    };
    if constexpr (!PARTS) {
        const float *__restrict__ d = src.direct + b * src.stride + blk.off;
        auto load = [&](int i) -> float { return d[i]; };
        fht_block<false>(s, blk.log_bs, load, store);
    } else {
        // Stage the block into LDS while summing the split-K partials of each stage in a
        // fixed order (deterministic).  Eight rows per thread are in flight at once.
        constexpr int U = 8;
        const int bs = blk.bs;
        for (int i0 = threadIdx.x; i0 < bs; i0 += U * RHT_THREADS) {
            float tot[U];
#pragma unroll
            for (int u = 0; u < U; ++u) tot[u] = 0.0f;
            for (int st = 0; st < src.nparts; ++st) {
                const float *__restrict__ p = src.part[st] + b * (int64_t)m_pad + blk.off;
                float acc[U];
#pragma unroll
                for (int u = 0; u < U; ++u) acc[u] = 0.0f;
#pragma unroll 4
                for (int k = 0; k < src.ksplit; ++k) {
#pragma unroll
                    for (int u = 0; u < U; ++u) {
                        const int i = i0 + u * RHT_THREADS;
                        acc[u] += i < bs ? p[(int64_t)k * src.part_kstride + i] : 0.0f;
                    }
                }
#pragma unroll
                for (int u = 0; u < U; ++u) tot[u] += src.scale[st] * acc[u];
            }
#pragma unroll
            for (int u = 0; u < U; ++u) {
                const int i = i0 + u * RHT_THREADS;
                if (i < bs) {
                    s[lds_pad(i)] = tot[u];
                    if (src.copy_out) src.copy_out[b * src.copy_stride + blk.off + i] = tot[u];
                }
            }
        }
        __syncthreads();
        auto load = [&](int i) -> float { return 0.0f; };
        fht_block<true>(s, blk.log_bs, load, store);
    }
}

size_t rht_lds_bytes(int64_t max_bs) { return (size_t)(max_bs + max_bs / 32 + 32) * sizeof(float); }

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
    GLQH_REQUIRE(rht_lds_bytes(max_bs) <= GLQH_MAX_LDS_BYTES, "input_rht: block of %lld exceeds LDS", (long long)max_bs);
    dim3 grid((unsigned)n_blocks, (unsigned)B);
    const size_t lds = rht_lds_bytes(max_bs);
#define GLQH_IN_LAUNCH(XT, OT)                                                                      \
    hipLaunchKernelGGL((input_rht_kernel<XT, OT>), grid, dim3(RHT_THREADS), lds, stream,            \
                       (const XT *)x, x_stride, (const f16 *)sv, (OT *)out, (int)in_features,       \
                       (int)n_pad, meta_dev, single, rsqrt_n)
    if (out_dtype == GLQH_F32) {
        if (x_dtype == GLQH_F16) GLQH_IN_LAUNCH(f16, float);
        else if (x_dtype == GLQH_BF16) GLQH_IN_LAUNCH(uint16_t, float);
        else GLQH_IN_LAUNCH(float, float);
    } else {
        if (x_dtype == GLQH_F16) GLQH_IN_LAUNCH(f16, f16);
        else if (x_dtype == GLQH_BF16) GLQH_IN_LAUNCH(uint16_t, f16);
        else GLQH_IN_LAUNCH(float, f16);
    }
#undef GLQH_IN_LAUNCH
    GLQH_LAUNCH_CHECK("input_rht launch");
    return 0;
}

int glqh_launch_output_rht(const glqh_ysrc &src, const void *su, void *y, int y_dtype,
                           int64_t y_stride, int64_t B, int64_t out_features, int64_t m_pad,
                           const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                           int64_t n_blocks, int64_t max_bs_hint, float rsqrt_m,
                           hipStream_t stream) {
    GLQH_REQUIRE(B >= 1 && B <= 65535, "output_rht: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(y != nullptr && su != nullptr, "output_rht: null y or su");
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
    GLQH_REQUIRE(rht_lds_bytes(max_bs) <= GLQH_MAX_LDS_BYTES, "output_rht: block of %lld exceeds LDS", (long long)max_bs);
    dim3 grid((unsigned)n_blocks, (unsigned)B);
    const size_t lds = rht_lds_bytes(max_bs);
#define GLQH_OUT_LAUNCH(YT, PARTS)                                                                  \
    hipLaunchKernelGGL((output_rht_kernel<YT, PARTS>), grid, dim3(RHT_THREADS), lds, stream, src,   \
                       (const f16 *)su, (YT *)y, y_stride, (int)out_features, (int)m_pad, meta_dev, \
                       single, rsqrt_m)
    if (src.nparts == 0) {
        if (y_dtype == GLQH_F16) GLQH_OUT_LAUNCH(f16, false);
        else if (y_dtype == GLQH_BF16) GLQH_OUT_LAUNCH(uint16_t, false);
        else GLQH_OUT_LAUNCH(float, false);
    } else {
        if (y_dtype == GLQH_F16) GLQH_OUT_LAUNCH(f16, true);
        else if (y_dtype == GLQH_BF16) GLQH_OUT_LAUNCH(uint16_t, true);
        else GLQH_OUT_LAUNCH(float, true);
    }
#undef GLQH_OUT_LAUNCH
    GLQH_LAUNCH_CHECK("output_rht launch");
    return 0;
}

template <typename K>
static int set_max_lds(K kernel, const char *what) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize,
                                              GLQH_MAX_LDS_BYTES), what);
}

int glqh_rht_init(void) {
    return set_max_lds(input_rht_kernel<f16, float>, "input_rht attribute") ||
           set_max_lds(input_rht_kernel<uint16_t, float>, "input_rht attribute") ||
           set_max_lds(input_rht_kernel<float, float>, "input_rht attribute") ||
           set_max_lds(input_rht_kernel<f16, f16>, "input_rht attribute") ||
           set_max_lds(input_rht_kernel<uint16_t, f16>, "input_rht attribute") ||
           set_max_lds(input_rht_kernel<float, f16>, "input_rht attribute") ||
           set_max_lds(output_rht_kernel<f16, false>, "output_rht attribute") ||
           set_max_lds(output_rht_kernel<uint16_t, false>, "output_rht attribute") ||
           set_max_lds(output_rht_kernel<float, false>, "output_rht attribute") ||
           set_max_lds(output_rht_kernel<f16, true>, "output_rht attribute") ||
           set_max_lds(output_rht_kernel<uint16_t, true>, "output_rht attribute") ||
           set_max_lds(output_rht_kernel<float, true>, "output_rht attribute");
}
