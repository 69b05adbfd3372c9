// E8 shell codebook: table packing and gather GEMV / small-batch GEMM (gfx950).
//
// Weight row i, columns 8j..8j+7 = table[u16(Qidxs[i,j])] (+ residual stages scaled by
// cumulative 1/resid_scale), glq/codebook.py:280-282, glq/quantized_linear.py:1177-1194.
// Every table coordinate is one of the 13 values -3, -2.5, ..., 3, so a row packs into
// eight 4-bit codes n = 2v + 6 (glq/codebook.py:102-115).  The packed word used here
// interleaves the codes so that one mask yields two adjacent columns:
//     nibble p     = code of column 2p
//     nibble p + 4 = code of column 2p + 1            (p = 0..3)
// and (word >> 4p) & 0x000F000F | 0x60006000 is the fp16 pair (512 + n/2) of columns
// (2p, 2p+1); subtracting 515 gives the exact coordinates.
//
// Work split: eight lanes share a row (one 16-byte run of 8 indices = 64 columns per
// lane and step), a wave covers 8 rows, a workgroup 32.  K is split over gridDim.y; the
// partial sums of each stage go to a scratch array and are combined in a fixed order by
// the consumer, so outputs are bit-identical from run to run.
#include "common.h"

namespace {

constexpr int E8_THREADS = 256;
constexpr int E8_ROWS_PER_WG = 32;

__global__ void __launch_bounds__(256)
e8_pack_table_kernel(const f16 *__restrict__ cb, int n_entries, uint32_t *__restrict__ out,
                     int32_t *__restrict__ bad) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_entries) return;
    uint32_t word = 0;
    bool ok = true;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        float v = (float)cb[(int64_t)i * 8 + c];
        float n = 2.0f * v + 6.0f;
        int code = (int)n;
        ok = ok && (n == (float)code) && code >= 0 && code <= 12;
        const int pos = (c >> 1) + 4 * (c & 1);
        word |= (uint32_t)(code & 15) << (4 * pos);
    }
    out[i] = word;
    if (!ok) atomicAdd(bad, 1);
}

// Words in the reference's own packing (nibble c = code of column c,
// glq/codebook.py:102-115, the `codebook_packed` buffer) -> the interleaved order above.
__global__ void __launch_bounds__(256)
e8_repack_table_kernel(const uint32_t *__restrict__ in, int n_entries, uint32_t *__restrict__ out,
                       int32_t *__restrict__ bad) {
    const int i = blockIdx.x * 256 + threadIdx.x;
    if (i >= n_entries) return;
    const uint32_t w = in[i];
    uint32_t word = 0;
    bool ok = true;
#pragma unroll
    for (int c = 0; c < 8; ++c) {
        const uint32_t code = (w >> (4 * c)) & 15u;
        ok = ok && code <= 12u;
        word |= code << (4 * ((c >> 1) + 4 * (c & 1)));
    }
    out[i] = word;
    if (!ok) atomicAdd(bad, 1);
}

__device__ __forceinline__ f16x2 e8_pair(uint32_t word, int p) {
    uint32_t u = ((word >> (4 * p)) & 0x000F000Fu) | 0x60006000u;
    f16x2 v = __builtin_bit_cast(f16x2, u);
    const f16x2 off = {(f16)515.0f, (f16)515.0f};
    return v - off;
}

// grid = (ceil(m_pad/32), ksplit, ceil(B/NB)).  part[((slot*NS + stage)*B + tok)*m_pad + row]
template <int NS, int NB>
__global__ void __launch_bounds__(E8_THREADS)
e8_gemv_kernel(const uint16_t *__restrict__ q1, const uint16_t *__restrict__ q2,
               const uint16_t *__restrict__ q3, const uint16_t *__restrict__ q4,
               const uint32_t *__restrict__ t1, const uint32_t *__restrict__ t2, uint32_t n2,
               const f16 *__restrict__ x, int B, int m_pad, int n_pad, float *__restrict__ part,
               glqh_e8_pscale ps) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int c = lane & 7;
    const int row = blockIdx.x * E8_ROWS_PER_WG + wave * 8 + (lane >> 3);
    const bool row_ok = row < m_pad;
    const int nblk = n_pad >> 3;                      // 8-column blocks per row
    const int nchunks = (nblk + 7) >> 3;              // 64-column chunks (last may be ragged)
    const int tok0 = blockIdx.z * NB;
    const bool vec_ok = (nblk & 7) == 0;              // rows are 16-byte aligned runs

    float acc[NB][NS];
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[t][s] = 0.0f;

    const uint16_t *qs[4] = {q1, q2, q3, q4};
    const int64_t rbase = (int64_t)(row_ok ? row : 0) * nblk;

    for (int ch = blockIdx.y * 8 + c; ch < nchunks; ch += gridDim.y * 8) {
        uint32_t idxw[NS][4];                          // 8 indices per stage, two per word
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            const uint16_t *qp = qs[s] + rbase + 8 * ch;
            if (vec_ok) {
                u32x4 v = __builtin_nontemporal_load((const u32x4 *)qp);
                idxw[s][0] = v.x; idxw[s][1] = v.y; idxw[s][2] = v.z; idxw[s][3] = v.w;
            } else {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const int b0 = 8 * ch + 2 * e;
                    uint32_t lo = b0 < nblk ? qp[2 * e] : 0u;
                    uint32_t hi = b0 + 1 < nblk ? qp[2 * e + 1] : 0u;
                    idxw[s][e] = lo | (hi << 16);
                }
            }
        }
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const int blk = 8 * ch + e;
            const bool live_blk = blk < nblk;          // only the ragged tail can be false
            uint32_t word[NS];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                uint32_t idx = (idxw[s][e >> 1] >> (16 * (e & 1))) & 0xFFFFu;
                if (s == 1) {
                    idx = idx < n2 ? idx : n2 - 1;
                    word[s] = t2[idx];
                } else {
                    word[s] = t1[idx];
                }
            }
#pragma unroll
            for (int t = 0; t < NB; ++t) {
                const int tok = tok0 + t;
                u32x4 xv = {0u, 0u, 0u, 0u};
                if (tok < B && live_blk) xv = *(const u32x4 *)(x + (int64_t)tok * n_pad + 8 * blk);
                const uint32_t xw[4] = {xv.x, xv.y, xv.z, xv.w};
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int p = 0; p < 4; ++p)
                        acc[t][s] = __builtin_amdgcn_fdot2(e8_pair(word[s], p),
                                                           __builtin_bit_cast(f16x2, xw[p]),
                                                           acc[t][s], false);
            }
        }
    }

#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int s = 0; s < NS; ++s) {
            float v = acc[t][s];
            v += __shfl_xor(v, 1, GLQH_WAVE);
            v += __shfl_xor(v, 2, GLQH_WAVE);
            v += __shfl_xor(v, 4, GLQH_WAVE);
            const int tok = tok0 + t;
            if (c == 0 && row_ok && tok < B)
                part[(((int64_t)blockIdx.y * NS + s) * B + tok) * m_pad + row] = ps.v[s] * v;
        }
}

// Dense fp16 weight (m_pad, n_pad) in the RHT domain, before Wscale: stages combined in
// fp32 and rounded once (the reference's batched path rounds the combined weight to fp16
// as well, glq/csrc/glq_cuda.cu:868-899).  One thread per 8-column block.
template <typename OT>
__global__ void __launch_bounds__(256)
e8_decompress_kernel(const uint16_t *__restrict__ q1, const uint16_t *__restrict__ q2,
                     const uint16_t *__restrict__ q3, const uint16_t *__restrict__ q4,
                     const uint32_t *__restrict__ t1, const uint32_t *__restrict__ t2, uint32_t n2,
                     float s2, float s3, float s4, int nstages, int64_t total_blocks,
                     OT *__restrict__ out) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= total_blocks) return;
    float w[8];
    {
        const uint32_t word = t1[q1[i]];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            f16x2 v = e8_pair(word, p);
            w[2 * p] = (float)v.x;
            w[2 * p + 1] = (float)v.y;
        }
    }
    const uint16_t *qs[3] = {q2, q3, q4};
    const float sc[3] = {s2, s3, s4};
    for (int st = 1; st < nstages; ++st) {
        uint32_t idx = qs[st - 1][i];
        uint32_t word;
        if (st == 1) word = t2[idx < n2 ? idx : n2 - 1];
        else word = t1[idx];
#pragma unroll
        for (int p = 0; p < 4; ++p) {
            f16x2 v = e8_pair(word, p);
            w[2 * p] += sc[st - 1] * (float)v.x;
            w[2 * p + 1] += sc[st - 1] * (float)v.y;
        }
    }
    if constexpr (sizeof(OT) == 4) {                            // the unrounded fp32 sums (dequantize)
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float4 o = {w[4 * h], w[4 * h + 1], w[4 * h + 2], w[4 * h + 3]};
            *(float4 *)(out + i * 8 + 4 * h) = o;
        }
    } else {
        f16 o[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (f16)w[c];
        *(u32x4 *)(out + i * 8) = *(const u32x4 *)o;
    }
}

// The same for large layers: the table's first P entries (the low-norm shells that Gaussian
// weights mostly hit) live in LDS, one persistent 1024-thread workgroup per CU; only the
// tail goes to L2 (random 4-byte L2 gathers run at 0.5 per clock per CU, LDS ones at ~10).
// Every lookup issues both loads, the unused one aimed at a shared entry, so that all loads
// stay unconditional.  Values and rounding are those of e8_decompress_kernel.
constexpr int E8D_THREADS = 1024;
constexpr int E8D_LDS_ENTRIES = 39936;                         // 156 KB of the 160 KB LDS

__global__ void __launch_bounds__(E8D_THREADS)
e8_decompress_lds_kernel(const uint16_t *__restrict__ q1, const uint16_t *__restrict__ q2,
                         const uint16_t *__restrict__ q3, const uint16_t *__restrict__ q4,
                         const uint32_t *__restrict__ t1, const uint32_t *__restrict__ t2, uint32_t n2,
                         int t2_is_t1, float s2, float s3, float s4, int nstages, int64_t total_blocks,
                         int P, f16 *__restrict__ out) {
    extern __shared__ uint32_t tab[];
    for (int j = threadIdx.x; j < P / 4; j += E8D_THREADS) ((u32x4 *)tab)[j] = ((const u32x4 *)t1)[j];
    __syncthreads();
    const uint32_t pre = (uint32_t)P, pre2 = t2_is_t1 ? (uint32_t)P : 0u;
    const uint16_t *qs[3] = {q2, q3, q4};
    const float sc[3] = {s2, s3, s4};
    for (int64_t i = (int64_t)blockIdx.x * E8D_THREADS + threadIdx.x; i < total_blocks;
         i += (int64_t)gridDim.x * E8D_THREADS) {
        float w[8];
        {
            const uint32_t idx = q1[i];
            const uint32_t wl = tab[min(idx, pre - 1)], wg = t1[max(idx, pre)];
            const uint32_t word = idx < pre ? wl : wg;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                f16x2 v = e8_pair(word, p);
                w[2 * p] = (float)v.x;
                w[2 * p + 1] = (float)v.y;
            }
        }
        for (int st = 1; st < nstages; ++st) {
            uint32_t idx = qs[st - 1][i];
            const uint32_t *tg = st == 1 ? t2 : t1;
            const uint32_t pp = st == 1 ? pre2 : pre;
            if (st == 1) idx = idx < n2 ? idx : n2 - 1;
            const uint32_t wl = tab[min(idx, pre - 1)], wg = tg[max(idx, pp)];
            const uint32_t word = idx < pp ? wl : wg;
#pragma unroll
            for (int p = 0; p < 4; ++p) {
                f16x2 v = e8_pair(word, p);
                w[2 * p] += sc[st - 1] * (float)v.x;
                w[2 * p + 1] += sc[st - 1] * (float)v.y;
            }
        }
        f16 o[8];
#pragma unroll
        for (int c = 0; c < 8; ++c) o[c] = (f16)w[c];
        *(u32x4 *)(out + i * 8) = *(const u32x4 *)o;
    }
}

template <int NS>
int launch_e8_NS(const void *x, int64_t B, const void *const q[4], const uint32_t *t1,
                 const uint32_t *t2, int64_t n2, int64_t m_pad, int64_t n_pad, int ksplit,
                 float *part, hipStream_t stream, glqh_e8_pscale ps) {
    const unsigned gx = (unsigned)((m_pad + E8_ROWS_PER_WG - 1) / E8_ROWS_PER_WG);
    const uint16_t *q1 = (const uint16_t *)q[0], *q2 = (const uint16_t *)q[1];
    const uint16_t *q3 = (const uint16_t *)q[2], *q4 = (const uint16_t *)q[3];
    const f16 *xp = (const f16 *)x;
    if (B == 1) {
        hipLaunchKernelGGL((e8_gemv_kernel<NS, 1>), dim3(gx, ksplit, 1), dim3(E8_THREADS), 0, stream, q1,
                           q2, q3, q4, t1, t2, (uint32_t)n2, xp, (int)B, (int)m_pad, (int)n_pad, part, ps);
    } else if (B <= 2) {
        hipLaunchKernelGGL((e8_gemv_kernel<NS, 2>), dim3(gx, ksplit, 1), dim3(E8_THREADS), 0, stream, q1,
                           q2, q3, q4, t1, t2, (uint32_t)n2, xp, (int)B, (int)m_pad, (int)n_pad, part, ps);
    } else {
        hipLaunchKernelGGL((e8_gemv_kernel<NS, 4>), dim3(gx, ksplit, (unsigned)((B + 3) / 4)),
                           dim3(E8_THREADS), 0, stream, q1, q2, q3, q4, t1, t2, (uint32_t)n2, xp, (int)B,
                           (int)m_pad, (int)n_pad, part, ps);
    }
    GLQH_LAUNCH_CHECK("e8 gemv launch");
    return 0;
}

}  // namespace

int glqh_e8_mma_init(void);
int glqh_e8_mma_ksplit(int64_t m_pad, int64_t n_pad, int64_t B, int64_t n1, int fold);
int glqh_launch_e8_mma(const void *x, int64_t B, const void *const q[4], int nstages, const uint32_t *t1,
                       int64_t n1, const uint32_t *t2, int64_t n2, int64_t m_pad, int64_t n_pad, float *part,
                       hipStream_t stream, const float *pscale, const glqh_e8_folded *fold, int direct);

int glqh_e8_init(void) {
    if (glqh_check_hip(hipFuncSetAttribute((const void *)e8_decompress_lds_kernel,
                                           hipFuncAttributeMaxDynamicSharedMemorySize, E8D_LDS_ENTRIES * 4),
                       "e8 decompress attribute"))
        return 1;
    return glqh_e8_mma_init();
}

// K-split of the kernel that will serve the call.
int glqh_e8_pick_ksplit(int64_t m_pad, int64_t n_pad, int64_t B, int fold) {
    // large layers at up to 16 tokens go to the LDS-table kernel, which has its own slots
    const int mma_ks = glqh_e8_mma_ksplit(m_pad, n_pad, B, 65536, fold);
    if (mma_ks > 0) return mma_ks;
    const int64_t wgs = (m_pad + E8_ROWS_PER_WG - 1) / E8_ROWS_PER_WG;
    const int64_t target = (int64_t)glqh_device_cus() * 4;
    int64_t ks = (target + wgs - 1) / wgs;
    int64_t cap = (((n_pad / 8 + 7) / 8) + 7) / 8;       // one chunk per lane at the most slots (a last slot may be ragged)
    if (cap < 1) cap = 1;
    if (ks > cap) ks = cap;
    if (ks > 32) ks = 32;
    if (ks < 1) ks = 1;
    return (int)ks;
}

namespace {
// index -> (16-bit word, byte) of its two half numbers through the map of glqh_e8_fold_table, written
// in the order the small-batch kernel reads: tiles of 16 rows x 32 indices, inside a tile the 8
// consecutive indices of lane 16 g + i (row i of the tile, indices 8 g .. 8 g + 7) at entry 8 * lane,
// so that a wave's load of a step is one contiguous kilobyte.  Rows and columns are padded to whole
// tiles with half number 0; indices past the table are clamped as the kernels clamp them.
__global__ void __launch_bounds__(256)
e8_fold_indices_kernel(const uint16_t *__restrict__ q, int rows, int cols, const uint32_t *__restrict__ map,
                       uint32_t n_entries, uint16_t *__restrict__ lo16, uint8_t *__restrict__ hi8, int64_t count) {
    const int64_t o = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (o >= count) return;
    const int col_tiles = (cols + 31) >> 5;
    const int64_t tile = o >> 9;
    const int lane = (int)(o >> 3) & 63, e = (int)o & 7;
    const int row = (int)(tile / col_tiles) * 16 + (lane & 15);
    const int col = (int)(tile % col_tiles) * 32 + 8 * (lane >> 4) + e;
    uint32_t first = 0, second = 0;
    if (row < rows && col < cols) {
        const uint32_t m = map[min((uint32_t)q[(int64_t)row * cols + col], n_entries - 1u)];
        first = m & 0xFFFFu;
        second = m >> 16;
    }
    lo16[o] = (uint16_t)(first | (second & 31u) << 11);
    hi8[o] = (uint8_t)(second >> 5);
}
}  // namespace

int glqh_launch_e8_fold_indices(const void *q, int64_t rows, int64_t cols, const uint32_t *map, int64_t n_entries,
                                uint16_t *lo16_out, uint8_t *hi8_out, hipStream_t stream) {
    const int64_t count = ((rows + 15) / 16) * ((cols + 31) / 32) * 512;
    GLQH_REQUIRE(rows <= 2147483647ll && cols <= 2147483647ll && (count + 255) / 256 <= 2147483647ll,
                 "e8 fold: too many indices");
    hipLaunchKernelGGL(e8_fold_indices_kernel, dim3((unsigned)((count + 255) / 256)), dim3(256), 0, stream,
                       (const uint16_t *)q, (int)rows, (int)cols, map, (uint32_t)n_entries, lo16_out, hi8_out, count);
    GLQH_LAUNCH_CHECK("e8 fold indices launch");
    return 0;
}

int glqh_launch_e8_pack_table(const void *cb, int64_t n_entries, uint32_t *out, int32_t *bad,
                              hipStream_t stream) {
    hipLaunchKernelGGL(e8_pack_table_kernel, dim3((unsigned)((n_entries + 255) / 256)), dim3(256), 0,
                       stream, (const f16 *)cb, (int)n_entries, out, bad);
    GLQH_LAUNCH_CHECK("e8 pack table launch");
    return 0;
}

int glqh_launch_e8_repack_table(const uint32_t *in, int64_t n_entries, uint32_t *out, int32_t *bad,
                                hipStream_t stream) {
    hipLaunchKernelGGL(e8_repack_table_kernel, dim3((unsigned)((n_entries + 255) / 256)), dim3(256), 0,
                       stream, in, (int)n_entries, out, bad);
    GLQH_LAUNCH_CHECK("e8 repack table launch");
    return 0;
}

int glqh_launch_e8_partial(const void *x, int64_t B, const void *const q[4], int nstages,
                           const uint32_t *t1, const uint32_t *t2, int64_t n2, int64_t m_pad,
                           int64_t n_pad, int ksplit, float *part, hipStream_t stream, const float *pscale,
                           const glqh_e8_folded *fold, int direct) {
    glqh_range range("dequant_matmul");
    glqh_e8_pscale ps = {{1.0f, 1.0f, 1.0f, 1.0f}};
    if (pscale)
        for (int i = 0; i < 4; ++i) ps.v[i] = pscale[i];
    // the folded streams serve the LDS-table kernel only; every other route reads the indices themselves
    if (glqh_e8_mma_ksplit(m_pad, n_pad, B, 65536, fold != nullptr) > 0)
        return glqh_launch_e8_mma(x, B, q, nstages, t1, 65536, t2, n2, m_pad, n_pad, part, stream, pscale, fold, direct);
    GLQH_REQUIRE(!direct, "e8 matmul: finished sums are an option of the LDS-table kernel");
    switch (nstages) {
    case 1: return launch_e8_NS<1>(x, B, q, t1, t2, n2, m_pad, n_pad, ksplit, part, stream, ps);
    case 2: return launch_e8_NS<2>(x, B, q, t1, t2, n2, m_pad, n_pad, ksplit, part, stream, ps);
    case 3: return launch_e8_NS<3>(x, B, q, t1, t2, n2, m_pad, n_pad, ksplit, part, stream, ps);
    case 4: return launch_e8_NS<4>(x, B, q, t1, t2, n2, m_pad, n_pad, ksplit, part, stream, ps);
    }
    return glqh_fail("e8 matmul: %d stages unsupported (1-4)", nstages);
}

int glqh_launch_e8_decompress(const void *const q[4], int nstages, const uint32_t *t1,
                              const uint32_t *t2, int64_t n2, float s2, float s3, float s4,
                              int64_t m_pad, int64_t n_pad, void *out, hipStream_t stream) {
    const int64_t total = m_pad * (n_pad / 8);
    if (total >= ((int64_t)1 << 19)) {                           // the table load pays from 4 M weights up
        const int P = E8D_LDS_ENTRIES;
        hipLaunchKernelGGL(e8_decompress_lds_kernel, dim3((unsigned)glqh_device_cus()), dim3(E8D_THREADS),
                           (size_t)P * 4, stream, (const uint16_t *)q[0], (const uint16_t *)q[1],
                           (const uint16_t *)q[2], (const uint16_t *)q[3], t1, t2, (uint32_t)n2,
                           (int)(t1 == t2 && n2 == 65536), s2, s3, s4, nstages, total, P, (f16 *)out);
        GLQH_LAUNCH_CHECK("e8 decompress launch");
        return 0;
    }
    hipLaunchKernelGGL(e8_decompress_kernel<f16>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       (const uint16_t *)q[0], (const uint16_t *)q[1], (const uint16_t *)q[2],
                       (const uint16_t *)q[3], t1, t2, (uint32_t)n2, s2, s3, s4, nstages, total,
                       (f16 *)out);
    GLQH_LAUNCH_CHECK("e8 decompress launch");
    return 0;
}

int glqh_launch_e8_decompress_f32(const void *const q[4], int nstages, const uint32_t *t1,
                                  const uint32_t *t2, int64_t n2, float s2, float s3, float s4,
                                  int64_t m_pad, int64_t n_pad, float *out, hipStream_t stream) {
    const int64_t total = m_pad * (n_pad / 8);
    hipLaunchKernelGGL(e8_decompress_kernel<float>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                       (const uint16_t *)q[0], (const uint16_t *)q[1], (const uint16_t *)q[2],
                       (const uint16_t *)q[3], t1, t2, (uint32_t)n2, s2, s3, s4, nstages, total, out);
    GLQH_LAUNCH_CHECK("e8 decompress (fp32) launch");
    return 0;
}
