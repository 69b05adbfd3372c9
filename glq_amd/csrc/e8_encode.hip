// E8 shell codebook encoder: nearest table row by argmin_k( |c_k|^2 - 2 <x, c_k> ), strict "<"
// so that the lowest index wins ties (glq/codebook.py:253-278; glq/codebook_kernel.py:12-83).
//
// One lane owns VPT vectors (8 fp32 each, in registers) and every wave walks the whole table:
// the table row is uniform over the wave, so it arrives through the scalar data path (one
// 32-byte scalar load per row) and feeds the multiply-adds as a scalar operand -- no LDS, no
// expansion, 8 FMAs + 1 FMA + compare + 2 selects per (vector, row).  The dot product is
// summed in coordinate order in fp32 with fused multiply-adds and the distance is
// fma(-2, dot, norm): for fp32 inputs this is the arithmetic of the reference's CPU branch.
#include "common.h"

namespace {

typedef float f32x4v __attribute__((ext_vector_type(4)));

constexpr int EQ_THREADS = 256;
constexpr int EQ_VPT = 4;

__global__ void __launch_bounds__(EQ_THREADS)
e8_quantize_kernel(const float *__restrict__ x, const float *__restrict__ table,
                   const float *__restrict__ norms, int64_t N, int K, int64_t *__restrict__ idx_out,
                   float *__restrict__ dec_out) {
    const int64_t v0 = ((int64_t)blockIdx.x * EQ_THREADS + threadIdx.x) * EQ_VPT;
    float xv[EQ_VPT][8], best[EQ_VPT];
    int bi[EQ_VPT];
#pragma unroll
    for (int u = 0; u < EQ_VPT; ++u) {
        const int64_t v = v0 + u < N ? v0 + u : N - 1;
        const f32x4v a = *(const f32x4v *)(x + v * 8), b = *(const f32x4v *)(x + v * 8 + 4);
        xv[u][0] = a.x; xv[u][1] = a.y; xv[u][2] = a.z; xv[u][3] = a.w;
        xv[u][4] = b.x; xv[u][5] = b.y; xv[u][6] = b.z; xv[u][7] = b.w;
        best[u] = __builtin_inff();
        bi[u] = 0;
    }
#pragma unroll 4
    for (int k = 0; k < K; ++k) {
        const float *c = table + (int64_t)k * 8;               // uniform: scalar loads
        const float nk = norms[k];
#pragma unroll
        for (int u = 0; u < EQ_VPT; ++u) {
            float dot = 0.0f;
#pragma unroll
            for (int d = 0; d < 8; ++d) dot = __builtin_fmaf(xv[u][d], c[d], dot);
            const float dist = __builtin_fmaf(-2.0f, dot, nk);
            const bool better = dist < best[u];
            best[u] = better ? dist : best[u];
            bi[u] = better ? k : bi[u];
        }
    }
#pragma unroll
    for (int u = 0; u < EQ_VPT; ++u) {
        if (v0 + u < N) {
            idx_out[v0 + u] = bi[u];
            if (dec_out) {
                const float *c = table + (int64_t)bi[u] * 8;
#pragma unroll
                for (int d = 0; d < 8; ++d) dec_out[(v0 + u) * 8 + d] = c[d];
            }
        }
    }
}

}  // namespace

int glqh_launch_e8_quantize(const float *x, const float *table, const float *norms, int64_t N, int K,
                            int64_t *idx_out, float *dec_out, hipStream_t stream) {
    const int64_t per_wg = (int64_t)EQ_THREADS * EQ_VPT;
    const int64_t wgs = (N + per_wg - 1) / per_wg;
    GLQH_REQUIRE(wgs <= 2147483647ll, "e8 quantize: too many vectors");
    hipLaunchKernelGGL(e8_quantize_kernel, dim3((unsigned)wgs), dim3(EQ_THREADS), 0, stream, x, table, norms, N,
                       K, idx_out, dec_out);
    GLQH_LAUNCH_CHECK("e8 quantize launch");
    return 0;
}
