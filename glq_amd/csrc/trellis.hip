// Trellis-3INST decode, GEMV and small-batch GEMM for gfx950 (wave64).
//
// Storage (one layer (m,k), R bits per weight, R = packed width / 16):
//   * 16x16 tiles; a tile is a cyclic stream of 256*R bits; trellis step t has the
//     16-bit state = stream bits [R t, R t + 16) and the weight decode_3inst(state)
//     (glq/trellis.py:122-134, 486-523).
//   * step t = 8 l + j sits at row (l>>2) + 8*((j>>1)&1), col 2*(l&3) + 8*(j>>2) + (j&1)
//     of its tile (glq/trellis.py:99-101).
//   * tiles are stored in 2x2 blocks (m-pair mp, k-pair kp), blocks ordered mp-major.
//     Inside a block, "stream lane" l in [0,32) owns one 4R-byte record holding its
//     8R-bit chunk of the four tiles in the order (k0,m0),(k0,m1),(k1,m0),(k1,m1), each
//     chunk little-endian with its most significant bit first in the stream
//     (glq/trellis.py:580-602).  A lane needs 16 more bits: the top of lane l+1's chunk
//     (R = 1: lanes l+1 and l+2), wrapping at 32.
//
// Mapping to the hardware: one wave64 step covers two adjacent blocks of the same
// m-pair -- lanes 0..31 take block (mp, 2q), lanes 32..63 block (mp, 2q+1) -- so a wave
// reads 256*R contiguous bytes with one load instruction per lane, rotates the
// continuation bits inside each 32-lane half with one cross-lane permute per two
// chunks, decodes 32 weights per lane in registers and multiplies them against the
// activations with fp32 accumulation.  Every output row is owned by one workgroup per
// K-split slot and summed in a fixed order, so results are bit-identical run to run.
#include "common.h"
#include "fht_device.h"
#include "trellis_device.h"

namespace {

// ---------------------------------------------------------------------------------
// decompress: packed -> dense fp16 (m,k), bit-exact with the reference dequantizer
// ---------------------------------------------------------------------------------
template <int R>
__global__ void __launch_bounds__(TR_THREADS)
tr_decompress_kernel(const uint8_t *__restrict__ packed, f16 *__restrict__ W, int m, int k) {
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int nsteps = k >> 6;
    const int q = blockIdx.x * TR_WAVES + wave;
    if (q >= nsteps) return;                               // whole wave exits together
    const int mp = blockIdx.y;
    const int l = lane & 31;
    const int kp = 2 * q + (lane >> 5);
    const int64_t rec = ((int64_t)mp * (k >> 5) + kp) * 32 + l;
    tr_record<R> r = tr_load_record<R>(packed + rec * (4 * R));
    uint32_t cont[4];
    tr_continuation<R>(r, lane, cont);
    const int a = l >> 2, b = l & 3;
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
            const int ci = ks * 2 + ms;
            const int row0 = 32 * mp + 16 * ms + a;
            const int col0 = 32 * kp + 16 * ks + 2 * b;
#pragma unroll
            for (int jp = 0; jp < 4; ++jp) {               // states 2jp, 2jp+1: adjacent columns
                f16x2 w;
                w.x = tr_weight(tr_state<R>(r.c[ci], cont[ci], 2 * jp));
                w.y = tr_weight(tr_state<R>(r.c[ci], cont[ci], 2 * jp + 1));
                const int row = row0 + 8 * (jp & 1);
                const int col = col0 + 8 * (jp >> 1);
                *(f16x2 *)(W + (int64_t)row * k + col) = w;
            }
        }
    }
}

// Decode the 32 weights of one record and accumulate them against the lane's activations.
// xa[t][ks] = (x[2b], x[2b+1]) and xb[t][ks] = (x[2b+8], x[2b+9]) of k-tile ks, token t;
// acc[t][ms*2 + rh] is the fp32 sum of row 16*ms + 8*rh + a.
template <int NB>
struct tr_xfrag {
    uint32_t a[NB][2], b[NB][2];
};

template <int NB>
struct tr_acc {
    float v[NB][4];
};

template <int R, int NB>
__device__ __forceinline__ tr_acc<NB> tr_accumulate(const tr_record<R> r, int lane, const tr_xfrag<NB> xf,
                                                    tr_acc<NB> acc) {
    uint32_t cont[4];
    tr_continuation<R>(r, lane, cont);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
            const int ci = ks * 2 + ms;
#pragma unroll
            for (int j = 0; j < 8; ++j) {
                // both fp16 halves of the state multiply the same activation
                f16x2 w = __builtin_bit_cast(f16x2, tr_hash(tr_state<R>(r.c[ci], cont[ci], j)));
                const int rh = (j >> 1) & 1;
#pragma unroll
                for (int t = 0; t < NB; ++t) {
                    const uint32_t xw = (j >> 2) ? xf.b[t][ks] : xf.a[t][ks];
                    // splat the selected half: (lo,lo) or (hi,hi)
                    const uint32_t sp = (j & 1) ? __builtin_amdgcn_perm(xw, xw, 0x07060706u)
                                                : __builtin_amdgcn_perm(xw, xw, 0x05040504u);
                    acc.v[t][ms * 2 + rh] = __builtin_amdgcn_fdot2(w, __builtin_bit_cast(f16x2, sp),
                                                                   acc.v[t][ms * 2 + rh], false);
                }
            }
        }
    }
    return acc;
}

// Workgroup reduction shared by the GEMV kernels: lanes -> waves -> 32 rows per token.
// Returns through `red` (LDS, [TR_WAVES][NB][32]); ends with a barrier.
template <int NB>
__device__ __forceinline__ void tr_reduce_to_lds(tr_acc<NB> acc, float (*red)[NB][32], int lane,
                                                 int wave) {
    const int l = lane & 31, a = l >> 2, b = l & 3, hf = lane >> 5;
#pragma unroll
    for (int t = 0; t < NB; ++t)
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            float v = acc.v[t][i];
            v += __shfl_xor(v, 1, GLQH_WAVE);
            v += __shfl_xor(v, 2, GLQH_WAVE);
            v += __shfl_xor(v, 32, GLQH_WAVE);
            acc.v[t][i] = v;
        }
    if (hf == 0 && b == 0) {
#pragma unroll
        for (int t = 0; t < NB; ++t)
#pragma unroll
            for (int i = 0; i < 4; ++i) red[wave][t][(i >> 1) * 16 + (i & 1) * 8 + a] = acc.v[t][i];
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------------
// GEMV with the input transform folded in (B <= NB tokens).
//
// grid = (m/32, ksplit).  K slot s owns the `steps` consecutive wave-steps starting at
// s*steps, i.e. the Ls = 64*steps columns [s*Ls, (s+1)*Ls) of the transformed activations
// (Ls a power of two).  A Hadamard block of size bs >= Ls that contains the slice factors as
// H_bs = H_(bs/Ls) (x) H_Ls, so the slice r of its output is
//     H_Ls( sum_h (-1)^popcount(r & h) * xs[h*Ls + j] ) / sqrt(bs),   xs = sv * x,
// which costs one pass over the block's inputs (they sit in L2) and a short transform;
// blocks smaller than the slice are transformed whole.  The slice is kept in LDS as fp16
// and feeds the decode loop.  The first record of every wave is requested before the
// prologue so that the HBM latency overlaps it.
// ---------------------------------------------------------------------------------
template <int R, typename XT, int NB>
__device__ __forceinline__ void
tr_gemv_fusein_body(const uint8_t *__restrict__ packed, const XT *__restrict__ x, int64_t x_stride,
                    const f16 *__restrict__ sv, int B, int m, int k, int in_features, int steps,
                    const glqh_block_meta *__restrict__ bn_meta, int n_blocks,
                    glqh_meta_args margs, float *__restrict__ part, float *smem, float (*red)[NB][32]) {
    const int Ls = steps << 6;
    float *fbuf = smem;                                         // Ls + Ls/32 floats
    f16 *xh = (f16 *)(smem + Ls + (Ls >> 5) + 32);              // [NB][Ls] fp16
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int l = lane & 31;
    const int hf = lane >> 5;
    const int b = l & 3;
    const int mp = blockIdx.x;
    const int slot = blockIdx.y;
    const int nsteps = k >> 6;
    const int q0 = slot * steps;
    const int q1 = min(q0 + steps, nsteps);
    const int c0 = q0 << 6;

    // This wave's first TR_PRE records are requested right behind its first activation loads
    // (loads complete in order: the transform then waits for the activations only, and the
    // packed stream arrives from HBM while it runs).
    const uint8_t *row_base = packed + (int64_t)mp * (k >> 5) * 32 * (4 * R);
    const uint8_t *lane_base = row_base + ((int64_t)hf * 32 + l) * (4 * R);   // + q * 64 * 4R
    constexpr int64_t STEP_BYTES = 64 * 4 * R;
    int q = q0 + wave;
    tr_record<R> cur[TR_PRE];
    bool requested = false;
    auto request = [&]() {
        if (requested) return;
        requested = true;
#pragma unroll
        for (int i = 0; i < TR_PRE; ++i) {
            cur[i] = tr_record<R>{};
            if (q + i * TR_WAVES < q1) cur[i] = tr_load_record<R>(lane_base + (q + i * TR_WAVES) * STEP_BYTES);
        }
    };

    // 8-byte loads of four activations / signs are possible (uniform over the launch)
    const bool quads = (((uintptr_t)x | (uintptr_t)sv) & 7) == 0 && (x_stride & 3) == 0;
    // ---- prologue: transformed activations of this slot's columns -> xh ----
    for (int jb = 0; jb < n_blocks; ++jb) {
        const glqh_block_meta bm = glqh_meta_row(margs, bn_meta, jb);
        const int lo = max(bm.offset, c0), hi = min(bm.offset + bm.bs, c0 + Ls);
        if (lo >= hi) continue;                                  // uniform over the workgroup
        const int len = hi - lo;                                 // min(bs, Ls), a power of two
        const int log_len = 31 - __builtin_clz(len);
        const int nsub = bm.bs >> log_len;
        const int r = (lo - bm.offset) >> log_len;
        const float norm = bm.w != 0 ? __builtin_bit_cast(float, bm.w) : rsqrt_pow2(bm.log_bs);
        for (int t = 0; t < NB; ++t) {
            if (t >= B) break;
            const XT *xr = x + (int64_t)t * x_stride;
            fht_barrier<true>();                                 // fbuf free again (record loads stay in flight)
            f16 *xo = xh + t * Ls + (lo - c0);
            const bool quad_rows = quads && (bm.offset & 3) == 0 && log_len >= 2 && bm.offset + bm.bs <= in_features;
            if (quad_rows && log_len <= fht_wave_max_log<4>()) {  // the slice in registers
                const unsigned tid = threadIdx.x;
                float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
                const bool live = 4 * tid < (1u << log_len);
                if (live) signed_input_quad_n<XT>(z, 4 * tid, log_len, nsub, r, xr + bm.offset, sv + bm.offset, request);
                else request();                                  // waves without elements load nothing
                fht_wave<4, false, true>(z, log_len, fbuf, tid);
                if (live) {
#pragma unroll
                    for (int qq = 0; qq < 4; ++qq) xo[fht_wave_index<4>(log_len, tid, qq)] = (f16)(z[qq] * norm);
                }
                continue;
            }
            if (quad_rows)
                stage_signed_input_quads<TR_THREADS, XT, 8, true>(fbuf, log_len, nsub, r, xr + bm.offset, sv + bm.offset,
                                                                  request);
            else
                stage_signed_slices<TR_THREADS>(fbuf, log_len, nsub, r, [&](int h, int j) -> float {
                    const int col = bm.offset + (h << log_len) + j;
                    const float v = act_to_f32<XT>(xr[min(col, in_features - 1)]) * (float)sv[col];
                    return col < in_features ? v : 0.0f;
                });
            request();
            struct {
                f16 *xo;
                float norm;
                __device__ float aux(int) const { return norm; }
                __device__ void put(int i, float v, float f) const { xo[i] = (f16)(v * f); }
            } store = {xo, norm};
            fht_staged<true>(fbuf, log_len, store);             // barriers that leave the record loads in flight
        }
    }
    request();                                                   // a slot without columns of its own
    __syncthreads();

    // ---- decode loop ----
    tr_acc<NB> acc = {};
    for (; q < q1; q += TR_PRE * TR_WAVES) {
        tr_record<R> nxt[TR_PRE];
#pragma unroll
        for (int i = 0; i < TR_PRE; ++i) {
            const int qn = q + (TR_PRE + i) * TR_WAVES;
            nxt[i] = cur[i];
            if (qn < q1) nxt[i] = tr_load_record<R>(lane_base + qn * STEP_BYTES);
        }
#pragma unroll
        for (int i = 0; i < TR_PRE; ++i) {
            const int qi = q + i * TR_WAVES;
            if (qi < q1) {                                       // uniform over the wave
                const int kp = 2 * qi + hf;
                tr_xfrag<NB> xf;
#pragma unroll
                for (int t = 0; t < NB; ++t) {
                    const uint32_t *xp = (const uint32_t *)(xh + t * Ls + (32 * kp - c0) + 2 * b);
#pragma unroll
                    for (int ks = 0; ks < 2; ++ks) {
                        xf.a[t][ks] = t < B ? xp[8 * ks] : 0u;
                        xf.b[t][ks] = t < B ? xp[8 * ks + 4] : 0u;
                    }
                }
                acc = tr_accumulate<R, NB>(cur[i], lane, xf, acc);
            }
        }
#pragma unroll
        for (int i = 0; i < TR_PRE; ++i) cur[i] = nxt[i];
    }
    tr_reduce_to_lds<NB>(acc, red, lane, wave);
    for (int idx = threadIdx.x; idx < NB * 32; idx += TR_THREADS) {
        const int t = idx >> 5, row = idx & 31;
        if (t >= B) continue;
        float v = red[0][t][row];
#pragma unroll
        for (int w = 1; w < TR_WAVES; ++w) v += red[w][t][row];
        part[((int64_t)slot * B + t) * m + 32 * mp + row] = v;
    }
}

template <int R, typename XT, int NB>
__global__ void __launch_bounds__(TR_THREADS)
tr_gemv_fusein_kernel(const uint8_t *__restrict__ packed, const XT *__restrict__ x, int64_t x_stride,
                      const f16 *__restrict__ sv, int B, int m, int k, int in_features, int steps,
                      const glqh_block_meta *__restrict__ bn_meta, int n_blocks,
                      glqh_meta_args margs, float *__restrict__ part) {
    extern __shared__ float smem[];
    __shared__ float red[TR_WAVES][NB][32];
    tr_gemv_fusein_body<R, XT, NB>(packed, x, x_stride, sv, B, m, k, in_features, steps, bn_meta, n_blocks,
                                   margs, part, smem, red);
}

// Several layers that read the same activations (fused q/k/v, gate/up:
// glq_vllm/linear_method.py:664-710) in one launch: blockIdx.z picks the shard, each with
// its own packed stream, input signs and partial-sum buffer; workgroups past a shard's
// rows retire.
struct tr_fusein_group {
    const uint8_t *packed[GLQH_MAX_GROUP];
    const f16 *sv[GLQH_MAX_GROUP];
    float *part[GLQH_MAX_GROUP];
    int m[GLQH_MAX_GROUP];
};

template <int R, typename XT, int NB>
__global__ void __launch_bounds__(TR_THREADS)
tr_gemv_fusein_group_kernel(tr_fusein_group g, const XT *__restrict__ x, int64_t x_stride, int B, int k,
                            int in_features, int steps, const glqh_block_meta *__restrict__ bn_meta,
                            int n_blocks, glqh_meta_args margs) {
    extern __shared__ float smem[];
    __shared__ float red[TR_WAVES][NB][32];
    const int z = blockIdx.z;
    const uint8_t *packed = g.packed[0];
    const f16 *sv = g.sv[0];
    float *part = g.part[0];
    int m = g.m[0];
#pragma unroll
    for (int i = 1; i < GLQH_MAX_GROUP; ++i)
        if (i == z) { packed = g.packed[i]; sv = g.sv[i]; part = g.part[i]; m = g.m[i]; }
    if ((int)blockIdx.x * 32 >= m) return;
    tr_gemv_fusein_body<R, XT, NB>(packed, x, x_stride, sv, B, m, k, in_features, steps, bn_meta, n_blocks,
                                   margs, part, smem, red);
}

__global__ void __launch_bounds__(256)
reduce_splits_kernel(const float *__restrict__ part, int ksplit, int64_t kstride, int m, float scale,
                     float *__restrict__ out, int64_t out_stride, int accum) {
    const int row = blockIdx.x * 256 + threadIdx.x;
    const int tok = blockIdx.y;
    if (row >= m) return;
    float v = 0.0f;
    for (int s = 0; s < ksplit; ++s) v += part[(int64_t)s * kstride + (int64_t)tok * m + row];
    float *o = out + (int64_t)tok * out_stride + row;
    *o = accum ? (*o + scale * v) : scale * v;
}

}  // namespace

int glqh_launch_reduce_splits(const float *part, int ksplit, int64_t kstride, int64_t B, int64_t m,
                              float scale, float *out, int64_t out_stride, int accum,
                              hipStream_t stream) {
    dim3 grid((unsigned)((m + 255) / 256), (unsigned)B);
    hipLaunchKernelGGL(reduce_splits_kernel, grid, dim3(256), 0, stream, part, ksplit, kstride, (int)m,
                       scale, out, out_stride, accum);
    GLQH_LAUNCH_CHECK("reduce_splits launch");
    return 0;
}

int glqh_launch_trellis_decompress(const void *packed, int R, int64_t m, int64_t k, void *out,
                                   hipStream_t stream) {
    const uint8_t *p = (const uint8_t *)packed;
    f16 *W = (f16 *)out;
    dim3 grid((unsigned)((k / 64 + TR_WAVES - 1) / TR_WAVES), (unsigned)(m / 32));
    switch (R) {
    case 1: hipLaunchKernelGGL(tr_decompress_kernel<1>, grid, dim3(TR_THREADS), 0, stream, p, W, (int)m, (int)k); break;
    case 2: hipLaunchKernelGGL(tr_decompress_kernel<2>, grid, dim3(TR_THREADS), 0, stream, p, W, (int)m, (int)k); break;
    case 3: hipLaunchKernelGGL(tr_decompress_kernel<3>, grid, dim3(TR_THREADS), 0, stream, p, W, (int)m, (int)k); break;
    case 4: hipLaunchKernelGGL(tr_decompress_kernel<4>, grid, dim3(TR_THREADS), 0, stream, p, W, (int)m, (int)k); break;
    default: return glqh_fail("trellis kernel supports R (bits/weight) 1-4, got %d", R);
    }
    GLQH_LAUNCH_CHECK("trellis decompress launch");
    return 0;
}

// ---- fused-input GEMV: plan and launch ----------------------------------------------
// steps per K slot: a power of two >= TR_WAVES chosen so that about four workgroups per CU
// are in flight; the slice 64*steps is capped at 8192 columns (LDS).
int glqh_trellis_fusein_plan(int64_t m, int64_t k, int64_t B, int *steps_out, int *ksplit_out) {
    if (B < 1 || B > 4) return 0;
    const int64_t nsteps = k / 64;
    const int64_t wgs = m / 32;
    const int64_t target = (int64_t)glqh_device_cus() * 4;
    int64_t ks_target = (target + wgs - 1) / wgs;
    if (ks_target < 1) ks_target = 1;
    int64_t want = (nsteps + ks_target - 1) / ks_target;
    int64_t steps = TR_WAVES;
    // Every workgroup first sums the (block / slice) sub-slices of its Hadamard block: keep
    // that to eight terms for the largest block (1024 x 4096: 10.1 -> 8.7 us per linear,
    // 1024 x 8192: 18.5 -> 9.9 us, four tokens 42.8 -> 17.8 us).
    int64_t bs = 1;
    while (2 * bs <= k) bs <<= 1;
    while (steps * 64 * 8 < bs && steps < 128) steps <<= 1;
    while (steps < want) steps <<= 1;
    if (steps > 128) steps = 128;
    *steps_out = (int)steps;
    *ksplit_out = (int)((nsteps + steps - 1) / steps);
    return 1;
}

size_t glqh_trellis_fusein_lds(int steps, int NB) {
    const size_t Ls = (size_t)steps * 64;
    return (Ls + Ls / 32 + 32) * sizeof(float) + (size_t)NB * Ls * sizeof(f16);
}

template <int R, typename XT, int NB>
static int launch_fusein(const void *packed, const void *x, int64_t x_stride, const void *sv, int64_t B,
                         int64_t m, int64_t k, int64_t in_features, int steps, int ksplit,
                         const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                         float *part, hipStream_t stream) {
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    dim3 grid((unsigned)(m / 32), (unsigned)ksplit, 1);
    hipLaunchKernelGGL((tr_gemv_fusein_kernel<R, XT, NB>), grid, dim3(TR_THREADS),
                       glqh_trellis_fusein_lds(steps, NB), stream, (const uint8_t *)packed, (const XT *)x,
                       x_stride, (const f16 *)sv, (int)B, (int)m, (int)k, (int)in_features, steps,
                       n_blocks > 1 ? bn_meta : nullptr, n_blocks > 1 ? n_blocks : 1, margs, part);
    GLQH_LAUNCH_CHECK("trellis fused-input gemv launch");
    return 0;
}

template <int R>
static int launch_fusein_R(const void *packed, const void *x, int x_dtype, int64_t x_stride,
                           const void *sv, int64_t B, int64_t m, int64_t k, int64_t in_features,
                           int steps, int ksplit, const glqh_block_meta *bn_meta,
                           const int64_t *blocks_host, int n_blocks, float *part, hipStream_t stream) {
#define GLQH_FI(XT, NB) launch_fusein<R, XT, NB>(packed, x, x_stride, sv, B, m, k, in_features, steps, \
                                                 ksplit, bn_meta, blocks_host, n_blocks, part, stream)
    if (B == 1) return x_dtype == GLQH_F16 ? GLQH_FI(f16, 1) : GLQH_FI(uint16_t, 1);
    return x_dtype == GLQH_F16 ? GLQH_FI(f16, 4) : GLQH_FI(uint16_t, 4);
#undef GLQH_FI
}

int glqh_launch_trellis_fusein(const void *packed, int R, const void *x, int x_dtype, int64_t x_stride,
                               const void *sv, int64_t B, int64_t m, int64_t k, int64_t in_features,
                               int steps, int ksplit, const glqh_block_meta *bn_meta,
                               const int64_t *blocks_host, int n_blocks, float *part,
                               hipStream_t stream) {
    glqh_range range("dequant_matmul");
    switch (R) {
    case 2: return launch_fusein_R<2>(packed, x, x_dtype, x_stride, sv, B, m, k, in_features, steps, ksplit, bn_meta, blocks_host, n_blocks, part, stream);
    case 3: return launch_fusein_R<3>(packed, x, x_dtype, x_stride, sv, B, m, k, in_features, steps, ksplit, bn_meta, blocks_host, n_blocks, part, stream);
    case 4: return launch_fusein_R<4>(packed, x, x_dtype, x_stride, sv, B, m, k, in_features, steps, ksplit, bn_meta, blocks_host, n_blocks, part, stream);
    }
    return glqh_fail("fused-input trellis kernel supports R (bits/weight) 2-4, got %d", R);
}

template <int R, typename XT, int NB>
static int launch_fusein_group(const tr_fusein_group &g, int64_t max_m, int n_shards, const void *x,
                               int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int steps,
                               int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                               int n_blocks, hipStream_t stream) {
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    dim3 grid((unsigned)(max_m / 32), (unsigned)ksplit, (unsigned)n_shards);
    hipLaunchKernelGGL((tr_gemv_fusein_group_kernel<R, XT, NB>), grid, dim3(TR_THREADS),
                       glqh_trellis_fusein_lds(steps, NB), stream, g, (const XT *)x, x_stride, (int)B, (int)k,
                       (int)in_features, steps, n_blocks > 1 ? bn_meta : nullptr, n_blocks > 1 ? n_blocks : 1,
                       margs);
    GLQH_LAUNCH_CHECK("trellis fused-input group launch");
    return 0;
}

int glqh_launch_trellis_fusein_group(const void *const packed[], const void *const sv[], float *const part[],
                                     const int64_t m[], int n_shards, int R, const void *x, int x_dtype,
                                     int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int steps,
                                     int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                     int n_blocks, hipStream_t stream) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(n_shards >= 1 && n_shards <= GLQH_MAX_GROUP, "trellis group: 1..%d shards", GLQH_MAX_GROUP);
    tr_fusein_group g = {};
    int64_t max_m = 0;
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        const int j = i < n_shards ? i : 0;
        g.packed[i] = (const uint8_t *)packed[j];
        g.sv[i] = (const f16 *)sv[j];
        g.part[i] = part[j];
        g.m[i] = (int)m[j];
        if (m[j] > max_m) max_m = m[j];
    }
#define GLQH_FG(RR, XT, NB) launch_fusein_group<RR, XT, NB>(g, max_m, n_shards, x, x_stride, B, k, in_features, \
                                                            steps, ksplit, bn_meta, blocks_host, n_blocks, stream)
#define GLQH_FG_R(RR)                                                                   \
    (B == 1 ? (x_dtype == GLQH_F16 ? GLQH_FG(RR, f16, 1) : GLQH_FG(RR, uint16_t, 1))     \
            : (x_dtype == GLQH_F16 ? GLQH_FG(RR, f16, 4) : GLQH_FG(RR, uint16_t, 4)))
    switch (R) {
    case 2: return GLQH_FG_R(2);
    case 3: return GLQH_FG_R(3);
    case 4: return GLQH_FG_R(4);
    }
#undef GLQH_FG_R
#undef GLQH_FG
    return glqh_fail("fused-input trellis kernel supports R (bits/weight) 2-4, got %d", R);
}

template <typename K>
static int tr_set_max_lds(K kernel, int NB) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel,
                                              hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)glqh_trellis_fusein_lds(128, NB)),
                          "trellis fused-input attribute");
}

int glqh_trellis_init(void) {
    int rc = 0;
#define GLQH_ATTR(R) rc = rc || tr_set_max_lds(tr_gemv_fusein_kernel<R, f16, 1>, 1) ||         \
                          tr_set_max_lds(tr_gemv_fusein_kernel<R, uint16_t, 1>, 1) ||          \
                          tr_set_max_lds(tr_gemv_fusein_kernel<R, f16, 4>, 4) ||               \
                          tr_set_max_lds(tr_gemv_fusein_kernel<R, uint16_t, 4>, 4) ||          \
                          tr_set_max_lds(tr_gemv_fusein_group_kernel<R, f16, 1>, 1) ||         \
                          tr_set_max_lds(tr_gemv_fusein_group_kernel<R, uint16_t, 1>, 1) ||    \
                          tr_set_max_lds(tr_gemv_fusein_group_kernel<R, f16, 4>, 4) ||         \
                          tr_set_max_lds(tr_gemv_fusein_group_kernel<R, uint16_t, 4>, 4)
    GLQH_ATTR(2);
    GLQH_ATTR(3);
    GLQH_ATTR(4);
#undef GLQH_ATTR
    return rc;
}
