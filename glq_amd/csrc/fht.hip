// Randomized Hadamard transforms around the quantized matmul.
//
// One workgroup transforms one power-of-two sub-block of one token in fp32 and
// multiplies once with 1/sqrt(bs) (glq/hadamard.py:10-28, glq/csrc/glq_fht.cuh:14-21,
// glq/csrc/glq_cuda.cu:1756-1839, 2005-2079, 2092-2208).
#include <algorithm>
#include "common.h"
#include "fht_device.h"

namespace {

#ifndef GLQH_RHT_THREADS
#define GLQH_RHT_THREADS 256
#endif
constexpr int RHT_THREADS = GLQH_RHT_THREADS;

// XT / OT: element types (bf16 travels as uint16_t)
template <typename XT, typename OT>
__device__ __forceinline__ void
input_rht_body(const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv,
               OT *__restrict__ out, int in_features, int n_pad,
               const glqh_block_meta *__restrict__ meta, const glqh_meta_args &margs,
               float single_norm, int spb, int log_slice, float *s) {
    const rht_slice blk = rht_get_slice(meta, margs, single_norm, spb, log_slice);
    if (!blk.live) return;
    const XT *xr = x + (int64_t)blockIdx.y * x_stride;
    struct {
        OT *orow;
        float norm;
        __device__ float aux(int) const { return norm; }
        __device__ void put(int i, float v, float f) const { orow[i] = f32_to_act<OT>(v * f); }
    } store = {out + (int64_t)blockIdx.y * n_pad + blk.off + (blk.r << blk.log_len), blk.norm};
    if constexpr (sizeof(XT) == 2) {
        // 16-bit activations, block wholly inside the row, 8-byte aligned: the slice in registers
        if (blk.log_len >= 2 && blk.log_len <= fht_wave_max_log<4>() && blk.off + blk.bs <= in_features &&
            (((uintptr_t)(xr + blk.off) | (uintptr_t)(sv + blk.off)) & 7) == 0) {   // uniform
            const int tid = threadIdx.x;
            const bool live = 4 * tid < (1 << blk.log_len);
            float z[4] = {0.0f, 0.0f, 0.0f, 0.0f};
            if (live) signed_input_quad_n<XT>(z, 4u * tid, blk.log_len, blk.nsub, blk.r, xr + blk.off, sv + blk.off);
            fht_wave<4>(z, blk.log_len, s, tid);
            if (live) {
#pragma unroll
                for (int q = 0; q < 4; ++q) store.put(fht_wave_index<4>(blk.log_len, tid, q), z[q], blk.norm);
            }
            return;
        }
    }
    auto val = [&](int h, int i) -> float {
        const int col = blk.off + (h << blk.log_len) + i;
        const float v = act_to_f32<XT>(xr[min(col, in_features - 1)]) * (float)sv[col];
        return col < in_features ? v : 0.0f;
    };
    if (blk.nsub == 1 && blk.log_len >= 11) stage_signed_slices<RHT_THREADS, 8, 1>(s, blk.log_len, 1, 0, val);
    else stage_signed_slices<RHT_THREADS>(s, blk.log_len, blk.nsub, blk.r, val);
    fht_staged(s, blk.log_len, store);
}

template <typename XT, typename OT>
__global__ void __launch_bounds__(RHT_THREADS)
input_rht_kernel(const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv,
                 OT *__restrict__ out, int in_features, int n_pad,
                 const glqh_block_meta *__restrict__ meta, glqh_meta_args margs,
                 float single_norm, int spb, int log_slice) {
    extern __shared__ float s[];
    input_rht_body<XT, OT>(x, x_stride, sv, out, in_features, n_pad, meta, margs, single_norm, spb, log_slice, s);
}

// The same rows under several sign vectors in one launch (layers of a group that were quantized with their own
// input signs): blockIdx.z picks the sign vector and its output.
struct rht_in_multi {
    const f16 *sv[GLQH_MAX_GROUP];
    f16 *out[GLQH_MAX_GROUP];
};
template <typename XT>
__global__ void __launch_bounds__(RHT_THREADS)
input_rht_multi_kernel(const XT *__restrict__ x, int64_t x_stride, rht_in_multi g, int in_features, int n_pad,
                       const glqh_block_meta *__restrict__ meta, glqh_meta_args margs, float single_norm, int spb,
                       int log_slice) {
    extern __shared__ float s[];
    input_rht_body<XT, f16>(x, x_stride, g.sv[blockIdx.z], g.out[blockIdx.z], in_features, n_pad, meta, margs,
                            single_norm, spb, log_slice, s);
}

// ---- many tokens: whole blocks, 16-byte accesses ------------------------------------
// With many tokens the transforms are bound by HBM, and what matters is how many bytes each
// thread keeps in flight and how the stores coalesce.  A workgroup owns one whole block
// (at most 8192 points) of one token and every thread moves runs of eight consecutive elements
// (16 bytes of 16-bit data) in and out.
constexpr int WIDE_LOG_MAX = 13;

template <typename T> __device__ __forceinline__ void load8(const T *p, float *f);
template <> __device__ __forceinline__ void load8<float>(const float *p, float *f) {
    const f32x4 a = *(const f32x4 *)p, b = *(const f32x4 *)(p + 4);
#pragma unroll
    for (int e = 0; e < 4; ++e) { f[e] = a[e]; f[4 + e] = b[e]; }
}
template <> __device__ __forceinline__ void load8<f16>(const f16 *p, float *f) {
    const u32x4 w = *(const u32x4 *)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const uint32_t we = w[e];                    // (bit_cast straight from a vector element reads element 0)
        const f16x2 h = __builtin_bit_cast(f16x2, we);
        f[2 * e] = (float)h[0];
        f[2 * e + 1] = (float)h[1];
    }
}
template <> __device__ __forceinline__ void load8<uint16_t>(const uint16_t *p, float *f) {   // bf16
    const u32x4 w = *(const u32x4 *)p;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        f[2 * e] = __builtin_bit_cast(float, w[e] << 16);
        f[2 * e + 1] = __builtin_bit_cast(float, w[e] & 0xffff0000u);
    }
}
template <typename T> __device__ __forceinline__ void store8(T *p, const float *f);
template <> __device__ __forceinline__ void store8<float>(float *p, const float *f) {
    *(f32x4 *)p = f32x4{f[0], f[1], f[2], f[3]};
    *(f32x4 *)(p + 4) = f32x4{f[4], f[5], f[6], f[7]};
}
template <> __device__ __forceinline__ void store8<f16>(f16 *p, const float *f) {
    u32x4 w;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const f16x2 h = {(f16)f[2 * e], (f16)f[2 * e + 1]};
        w[e] = __builtin_bit_cast(uint32_t, h);
    }
    *(u32x4 *)p = w;
}
template <> __device__ __forceinline__ void store8<uint16_t>(uint16_t *p, const float *f) {  // bf16
    u32x4 w;
#pragma unroll
    for (int e = 0; e < 4; ++e)
        w[e] = (uint32_t)f32_to_bf16_bits(f[2 * e]) | ((uint32_t)f32_to_bf16_bits(f[2 * e + 1]) << 16);
    *(u32x4 *)p = w;
}

// blockIdx.x = block, blockIdx.y = token.  Requires canonical blocks of 8..8192 points, 16-byte
// aligned rows of x (x_stride % 8 == 0 elements for 16-bit types) and out.  The transform runs
// in registers (fht_wave<E>): thread t of 512 holds elements E*t .. E*t+E-1 of the block (E = 16
// for 8192 points, 8 below), log2(E) butterfly levels stay in the thread, six run across the
// lanes, up to log2(E) across the waves through one LDS exchange; the results, which the exchange
// leaves strided over the threads, pass through LDS once more so that every thread writes a run
// of E consecutive elements.  84 LDS-pipe instructions per thread for an 8192-point block where
// passes through LDS (fht_staged) take 320, and three barriers instead of ten: 4096 tokens x
// 14336 points 117 -> 71 us in, 139 -> 87 us out.
constexpr int REG_THREADS = 512;
__device__ __forceinline__ int reg_pad(int p) { return p + ((p >> 5) << 2); }   // 16-byte groups stay whole
size_t rht_reg_lds_bytes(int log_bs) {
    const size_t n = (size_t)1 << log_bs;
    return (n + n / 8 + 16) * sizeof(float);
}

// v (element tid + q * nthr when the transform went through the exchange, E * tid + q otherwise)
// -> E consecutive elements E * tid + q, through s.  Every thread of the workgroup calls.
template <int E>
__device__ __forceinline__ void reg_gather_runs(float (&v)[E], int log_len, float *s, int tid, bool active) {
    constexpr int LE = fht_wave_log<E>::v;
    if (log_len <= 6 + LE) return;                           // uniform: already consecutive
    const int nthr = 1 << (log_len - LE);
    __syncthreads();                                         // the exchange buffer has been read
    if (active) {
#pragma unroll
        for (int q = 0; q < E; ++q) s[reg_pad(tid + q * nthr)] = v[q];
    }
    __syncthreads();
    if (active) {
#pragma unroll
        for (int q = 0; q < E; q += 4) {
            const f32x4 w = *(const f32x4 *)(s + reg_pad(E * tid + q));
            v[q] = w[0]; v[q + 1] = w[1]; v[q + 2] = w[2]; v[q + 3] = w[3];
        }
    }
}

// What a thread of a whole-block workgroup does.  Blocks of 1024 points and more: one token (row) per
// workgroup, thread te = tid.  Blocks of at most 512 points are transformed inside one wave (eight elements
// per thread, no exchange through LDS), so a workgroup takes 4096 / bs tokens at once: thread tid works on
// token tid / (bs / 8) of them as thread te = tid % (bs / 8), with staging space of its own.
struct wide_role {
    int te, tok, nthr, lds_off;                              // tok: the token's number inside the workgroup
    bool active;                                             // false: past the workgroup's tokens
};

__device__ __forceinline__ wide_role wide_role_of(const rht_slice &blk, int ntok) {
    wide_role r;
    const int tid = threadIdx.x;
    if (blk.log_bs > 9) {
        r.te = tid; r.tok = 0; r.nthr = REG_THREADS; r.lds_off = 0; r.active = true;
    } else {
        const int lthr = blk.log_bs - 3;
        r.te = tid & ((1 << lthr) - 1);
        r.tok = tid >> lthr;
        r.nthr = 1 << lthr;
        r.lds_off = r.tok * (blk.bs + (blk.bs >> 3) + 8);
        r.active = r.tok < ntok;
    }
    return r;
}
constexpr int WIDE_SMALL_LOG = 9;                            // blocks up to 512 points: 4096 / bs tokens per workgroup
// LDS for the staging of a small block's tokens (layout 2: blocks of 32 points and more)
constexpr size_t WIDE_SMALL_LDS = (size_t)(4096 + 512 + 8 * 128) * sizeof(float);

// LAYOUT of the transformed row: 0 = row-major (out + token * n_pad); 1 and 2 = the tile kernels'
// operand layouts out[col / 32][token][4][8]: 32 columns of one token are 64 contiguous bytes, as
// four 8-column blocks in order (1, E8) or as the four slots q = 0..3 holding columns
// 2q + {0,1,8,9,16,17,24,25} of the k-pair (2, trellis).  Both save the tile kernels' repacking pass.
template <int E, typename XT, typename OT, int LAYOUT>
__device__ __forceinline__ void input_rht_wide_body(const XT *__restrict__ x, int64_t x_stride,
                                                   const f16 *__restrict__ sv, OT *__restrict__ out,
                                                   int in_features, int n_pad, int Mp, int token,
                                                   const rht_slice &blk, float *s, const wide_role role) {
    // te: the thread's number among those of its token; st: the token's staging space in LDS
    const int tid = threadIdx.x, te = role.te;
    const bool active = role.active && E * te < blk.bs;
    float *st = s + role.lds_off;
    const int i = E * te;
    float v[E];
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = 0.0f;
    if (active) {
        const XT *xr = x + (int64_t)token * x_stride + blk.off;
        const int lim = in_features - blk.off;               // elements of the block inside the row
        float sf[E];
#pragma unroll
        for (int e = 0; e < E; e += 8) load8<f16>(sv + blk.off + i + e, sf + e);
        if (i + E <= lim) {
#pragma unroll
            for (int e = 0; e < E; e += 8) load8<XT>(xr + i + e, v + e);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e) v[e] = i + e < lim ? act_to_f32<XT>(xr[i + e]) : 0.0f;
        }
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] *= sf[e];
    }
    fht_wave<E>(v, blk.log_len, s, tid);
    if constexpr (LAYOUT == 2) {
        // every element through LDS, then one 16-byte slot (k-pair, q) per thread and round
        constexpr int LE = fht_wave_log<E>::v;
        const bool strided = blk.log_len > 6 + LE;           // uniform
        const int nthr = 1 << (blk.log_len - LE);
        __syncthreads();                                      // the exchange buffer has been read
        if (active) {
#pragma unroll
            for (int q = 0; q < E; ++q) st[reg_pad(strided ? te + q * nthr : E * te + q)] = v[q] * blk.norm;
        }
        __syncthreads();
        for (int p = te; role.active && p < (blk.bs >> 3); p += role.nthr) {   // blocks are multiples of 32 columns
            const int kp = p >> 2, q = p & 3;
            float w[8];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                const f32x2 t = *(const f32x2 *)(st + reg_pad(32 * kp + 2 * q + 8 * j));
                w[2 * j] = t[0];
                w[2 * j + 1] = t[1];
            }
            store8<OT>(out + ((((int64_t)(blk.off >> 5) + kp) * Mp + token) * 4 + q) * 8, w);
        }
        return;
    }
    reg_gather_runs<E>(v, blk.log_len, s, tid, active);
    if (active) {
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] *= blk.norm;
        if constexpr (LAYOUT == 1) {
#pragma unroll
            for (int e = 0; e < E; e += 8) {
                const int kb = (blk.off + i + e) >> 3;
                store8<OT>(out + (((int64_t)(kb >> 2) * Mp + token) * 4 + (kb & 3)) * 8, v + e);
            }
        } else {
            OT *orow = out + (int64_t)token * n_pad + blk.off + i;
#pragma unroll
            for (int e = 0; e < E; e += 8) store8<OT>(orow + e, v + e);
        }
    }
}

// blocks of 8192 points take 16 elements per thread, smaller ones 8 (all 512 threads busy on 4096).
// One-dimensional grid: workgroup L runs on XCD L % 8, XCD r owns tokens r * ceil(B / 8) ..., and the
// workgroups of an XCD come in sets of eight that take the same block of eight consecutive tokens: in the
// token-fast layouts the 16-byte pieces of eight consecutive tokens share a 128-byte line, which is then
// completed inside one L2 instead of written back in eight parts; and the blocks of a row differ in size
// (11008 = 8192 + 2048 + 512 + 256), so dealing a token's four blocks to neighbouring workgroups, which go
// to the four shader engines of an XCD in turn, put every 8192-point block on the same engine
// (4096 x 11008: 112 -> 70 us; rows of one or three blocks: no change).
template <typename XT, typename OT, int LAYOUT>
__global__ void __launch_bounds__(REG_THREADS)
input_rht_wide_kernel(const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv,
                     OT *__restrict__ out, int in_features, int n_pad, int Mp, int B, int n_blocks,
                     glqh_meta_args margs, float single_norm) {
    extern __shared__ float s[];
    const int L = blockIdx.x, per_xcd = (B + 7) >> 3;
    const int j = L >> 3;
    const int member = j & 7, rest = j >> 3, g = rest / n_blocks;
    const rht_slice blk = rht_slice_of(margs, single_norm, rest % n_blocks);
    if (blk.log_bs <= WIDE_SMALL_LOG) {
        // one workgroup of 4096 / bs / 8 sets takes all their tokens (the eight members in turn, so that the
        // work reaches every shader engine), the others retire
        const int lsets = 12 - blk.log_bs - 3;
        if ((g & ((1 << lsets) - 1)) != 0 || member != ((g >> lsets) & 7)) return;
        const int t_in = g * 8, tok0 = (L & 7) * per_xcd + t_in;
        if (t_in >= per_xcd || tok0 >= B) return;
        const int ntok = min(8 << lsets, min(per_xcd - t_in, B - tok0));
        const wide_role role = wide_role_of(blk, ntok);
        input_rht_wide_body<8, XT, OT, LAYOUT>(x, x_stride, sv, out, in_features, n_pad, Mp,
                                               tok0 + min(role.tok, ntok - 1), blk, s, role);
        return;
    }
    const int t_in = g * 8 + member;                          // token, counted inside the XCD's share
    const int token = (L & 7) * per_xcd + t_in;
    if (token >= B || t_in >= per_xcd) return;                // uniform over the workgroup
    const wide_role role = wide_role_of(blk, 1);
    if (blk.log_bs > 12)
        input_rht_wide_body<16, XT, OT, LAYOUT>(x, x_stride, sv, out, in_features, n_pad, Mp, token, blk, s, role);
    else
        input_rht_wide_body<8, XT, OT, LAYOUT>(x, x_stride, sv, out, in_features, n_pad, Mp, token, blk, s, role);
}

// The same rows under several sign vectors in one launch, trellis operand layout out (layers of a group that were
// quantized with their own input signs, 17..64 tokens): blockIdx.y picks the sign vector and its output; the
// dealing of rows and blocks is input_rht_wide_kernel's.
struct rht_in_wide_multi {
    const f16 *sv[GLQH_MAX_GROUP];
    f16 *out[GLQH_MAX_GROUP];
};
template <typename XT>
__global__ void __launch_bounds__(REG_THREADS)
input_rht_wide_multi_kernel(const XT *__restrict__ x, int64_t x_stride, rht_in_wide_multi mg, int in_features, int n_pad,
                            int Mp, int B, int n_blocks, glqh_meta_args margs, float single_norm) {
    extern __shared__ float s[];
    const f16 *sv = mg.sv[blockIdx.y];
    f16 *out = mg.out[blockIdx.y];
    const int L = blockIdx.x, per_xcd = (B + 7) >> 3;
    const int j = L >> 3;
    const int member = j & 7, rest = j >> 3, g = rest / n_blocks;
    const rht_slice blk = rht_slice_of(margs, single_norm, rest % n_blocks);
    if (blk.log_bs <= WIDE_SMALL_LOG) {
        const int lsets = 12 - blk.log_bs - 3;
        if ((g & ((1 << lsets) - 1)) != 0 || member != ((g >> lsets) & 7)) return;
        const int t_in = g * 8, tok0 = (L & 7) * per_xcd + t_in;
        if (t_in >= per_xcd || tok0 >= B) return;
        const int ntok = min(8 << lsets, min(per_xcd - t_in, B - tok0));
        const wide_role role = wide_role_of(blk, ntok);
        input_rht_wide_body<8, XT, f16, 2>(x, x_stride, sv, out, in_features, n_pad, Mp, tok0 + min(role.tok, ntok - 1), blk, s,
                                           role);
        return;
    }
    const int t_in = g * 8 + member;
    const int token = (L & 7) * per_xcd + t_in;
    if (token >= B || t_in >= per_xcd) return;                // uniform over the workgroup
    const wide_role role = wide_role_of(blk, 1);
    if (blk.log_bs > 12) input_rht_wide_body<16, XT, f16, 2>(x, x_stride, sv, out, in_features, n_pad, Mp, token, blk, s, role);
    else input_rht_wide_body<8, XT, f16, 2>(x, x_stride, sv, out, in_features, n_pad, Mp, token, blk, s, role);
}

// v = the transformed sums of elements E * tid .. E * tid + E - 1 of block `blk`, row b (before the
// signs and the 1/sqrt(bs)): direct rows or split-K partial sums in, register transform, runs restored.
// Every thread of the workgroup calls.
// (the first half, what a thread reads: callers that transform several rows in turn request the next row's
// sums before they transform this one's)
template <int E>
__device__ __forceinline__ void output_wide_load(float (&v)[E], const glqh_ysrc &src, int64_t b, int m_pad,
                                                 const rht_slice &blk, bool active, int te) {
    const int i = E * te;
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = 0.0f;
    if (active) {
        if (src.nparts == 0) {
            const float *d = src.direct + b * src.stride + blk.off + i;
#pragma unroll
            for (int e = 0; e < E; e += 8) load8<float>(d + e, v + e);
        } else {
            // v = sum_stage scale * (sum_k partial), in this fixed order (as stage_partials)
            const int64_t ebase = b * (int64_t)m_pad + blk.off + i;
            for (int st = 0; st < src.nparts; ++st) {
                float acc[E];
#pragma unroll
                for (int e = 0; e < E; ++e) acc[e] = 0.0f;
                const int64_t eoff = ebase + st * src.part_sstride;
                for (int k = 0; k < src.ksplit; ++k) {
                    float t0[E];
                    if (src.part_f16) {                         // uniform over the launch
#pragma unroll
                        for (int e = 0; e < E; e += 8) load8<f16>((const f16 *)src.part + eoff + k * src.part_kstride + e, t0 + e);
                    } else {
#pragma unroll
                        for (int e = 0; e < E; e += 8) load8<float>(src.part + eoff + k * src.part_kstride + e, t0 + e);
                    }
#pragma unroll
                    for (int e = 0; e < E; ++e) acc[e] += t0[e];
                }
                const float sc = st == 0 ? src.scale[0] : st == 1 ? src.scale[1]
                               : st == 2 ? src.scale[2] : src.scale[3];
#pragma unroll
                for (int e = 0; e < E; ++e) v[e] += sc * acc[e];
            }
            if (src.copy_out) {
                float *c = src.copy_out + b * src.copy_stride + blk.off + i;
#pragma unroll
                for (int e = 0; e < E; e += 8) store8<float>(c + e, v + e);
            }
        }
    }
}

template <int E>
__device__ __forceinline__ void output_wide_transform(float (&v)[E], const rht_slice &blk, float *s, int tid, bool active) {
    fht_wave<E>(v, blk.log_len, s, tid);
    reg_gather_runs<E>(v, blk.log_len, s, tid, active);
}

template <int E>
__device__ __forceinline__ void output_wide_values(float (&v)[E], const glqh_ysrc &src, int64_t b, int m_pad,
                                                   const rht_slice &blk, float *s, int tid, bool active, int te) {
    output_wide_load<E>(v, src, b, m_pad, blk, active, te);
    output_wide_transform<E>(v, blk, s, tid, active);
}

template <int E, typename YT>
__device__ __forceinline__ void output_rht_wide_body(const glqh_ysrc &src, const f16 *__restrict__ su,
                                                    YT *__restrict__ y, int64_t y_stride, int out_features,
                                                    int m_pad, const rht_slice &blk, float *s, int64_t b,
                                                    const wide_role role) {
    const int tid = threadIdx.x;
    const bool active = role.active && E * role.te < blk.bs;
    float v[E];
    output_wide_values<E>(v, src, b, m_pad, blk, s, tid, active, role.te);
    const int row = blk.off + E * role.te;
    if (active && row < out_features) {
        float f[E];
#pragma unroll
        for (int e = 0; e < E; e += 8) load8<f16>(su + row + e, f + e);   // su has m_pad entries
#pragma unroll
        for (int e = 0; e < E; ++e) v[e] *= blk.norm * f[e];
        YT *yrow = y + b * y_stride;
        if (row + E <= out_features) {
#pragma unroll
            for (int e = 0; e < E; e += 8) store8<YT>(yrow + row + e, v + e);
        } else {
#pragma unroll
            for (int e = 0; e < E; ++e)
                if (row + e < out_features) yrow[row + e] = f32_to_act<YT>(v[e]);
        }
    }
}

template <typename YT>
__global__ void __launch_bounds__(REG_THREADS)
output_rht_wide_kernel(glqh_ysrc src, const f16 *__restrict__ su, YT *__restrict__ y, int64_t y_stride,
                      int out_features, int m_pad, int B, int n_blocks, glqh_meta_args margs, float single_norm) {
    extern __shared__ float s[];
    // Workgroup L runs on XCD L % 8 and, inside it, on shader engine (L / 8) % 4: the 64 workgroups that
    // follow each other take the same block of 64 consecutive rows, so that the large blocks of a row of
    // several (11008 = 8192 + 2048 + 512 + 256) reach every engine.  Dealt out block by block, a row of four
    // blocks put every 8192-point block on the same engine of each XCD: 4096 x 11008 127 -> 72 us.
    const int L = blockIdx.x, xcd = L & 7, member = (L >> 3) & 7, rest = L >> 6, g = rest / n_blocks;
    const rht_slice blk = rht_slice_of(margs, single_norm, rest % n_blocks);
    const int r0 = g * 64 + member * 8;                       // first row of the eight workgroups (member, 0..7)
    if (blk.log_bs <= WIDE_SMALL_LOG) {
        // one workgroup of every 4096 / bs rows takes them all (the XCDs in turn), the others retire
        const int lt = 12 - blk.log_bs, T = 1 << lt;
        if ((r0 & (T - 1)) != 0 || xcd != ((r0 >> lt) & 7) || r0 >= B) return;
        const int ntok = min(T, B - r0);
        const wide_role role = wide_role_of(blk, ntok);
        output_rht_wide_body<8, YT>(src, su, y, y_stride, out_features, m_pad, blk, s,
                                    (int64_t)r0 + min(role.tok, ntok - 1), role);
        return;
    }
    const int64_t b = (int64_t)r0 + xcd;
    if (b >= B) return;                                       // uniform over the workgroup
    const wide_role role = wide_role_of(blk, 1);
    if (blk.log_bs > 12) output_rht_wide_body<16, YT>(src, su, y, y_stride, out_features, m_pad, blk, s, b, role);
    else output_rht_wide_body<8, YT>(src, su, y, y_stride, out_features, m_pad, blk, s, b, role);
}

template <typename YT, bool PARTS>
__device__ __forceinline__ void
output_rht_body(const glqh_ysrc &src, const f16 *__restrict__ su, YT *__restrict__ y, int64_t y_stride,
                int out_features, int m_pad, const glqh_block_meta *__restrict__ meta,
                glqh_meta_args margs, float single_norm, int spb, int log_slice, float *s) {
    const rht_slice blk = rht_get_slice(meta, margs, single_norm, spb, log_slice);
    if (!blk.live) return;
    const int64_t b = blockIdx.y;
    const int base = blk.off + (blk.r << blk.log_len);
    struct {
        YT *yrow;
        const f16 *su;
        int base, out_features;
        float norm;
        // su has m_pad entries, so the load is always in bounds
        __device__ float aux(int i) const { return norm * (float)su[base + i]; }
        __device__ void put(int i, float v, float f) const {
            const int row = base + i;
            if (row < out_features) yrow[row] = f32_to_act<YT>(v * f);
        }
    } store = {y + b * y_stride, su, base, out_features, blk.norm};
    // slices of 4 .. 1024 points with 16-byte aligned rows are transformed in registers
    bool in_regs;                                              // uniform over the workgroup
    if constexpr (PARTS) in_regs = stage_partials_quad_ok(src, blk, b, m_pad);
    else
        in_regs = blk.log_len >= 2 && blk.log_len <= fht_wave_max_log<4>() &&
                  ((uintptr_t)(src.direct + b * src.stride + blk.off) & 15) == 0;
    if (in_regs) {
        const int tid = threadIdx.x;
        const bool active = 4 * tid < (1 << blk.log_len);
        int idx[4];
        float z[4];
        f16 su_raw[4];                                         // in flight beside the row, used after it
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            idx[q] = fht_wave_index<4>(blk.log_len, active ? tid : 0, q);
            su_raw[q] = su[base + idx[q]];
        }
        if constexpr (PARTS) stage_partials_quad_n(z, src, blk, b, m_pad, tid);
        else stage_signed_row_quad<8>(z, src.direct + b * src.stride + blk.off, blk.log_len, blk.nsub, blk.r, tid);
        fht_wave<4>(z, blk.log_len, s, tid);
        if (active) {
#pragma unroll
            for (int q = 0; q < 4; ++q) store.put(idx[q], z[q], blk.norm * (float)su_raw[q]);
        }
        return;
    }
    if constexpr (!PARTS) {
        const float *__restrict__ d = src.direct + b * src.stride + blk.off;
        auto val = [&](int h, int i) -> float { return d[(h << blk.log_len) + i]; };
        if (blk.nsub == 1 && blk.log_len >= 11) stage_signed_slices<RHT_THREADS, 8, 1>(s, blk.log_len, 1, 0, val);
        else stage_signed_slices<RHT_THREADS>(s, blk.log_len, blk.nsub, blk.r, val);
    } else {
        const int total = blk.nsub * src.nparts * src.ksplit;
        if (total == 1 && blk.log_len >= 11) stage_partials<RHT_THREADS, 8, 1>(s, src, blk, b, m_pad);
        else stage_partials<RHT_THREADS, 4, 8>(s, src, blk, b, m_pad);
    }
    fht_staged(s, blk.log_len, store);
}

template <typename YT, bool PARTS>
__global__ void __launch_bounds__(RHT_THREADS)
output_rht_kernel(glqh_ysrc src, const f16 *__restrict__ su, YT *__restrict__ y, int64_t y_stride,
                  int out_features, int m_pad, const glqh_block_meta *__restrict__ meta,
                  glqh_meta_args margs, float single_norm, int spb, int log_slice) {
    extern __shared__ float s[];
    output_rht_body<YT, PARTS>(src, su, y, y_stride, out_features, m_pad, meta, margs, single_norm, spb,
                               log_slice, s);
}

// The output transforms of several layers in one launch (blockIdx.z = shard), each from its
// own single-stage split-K partials; block sizes are the canonical decomposition of m_pad.
struct rht_out_group {
    const float *part[GLQH_MAX_GROUP];
    const f16 *su[GLQH_MAX_GROUP];
    void *y[GLQH_MAX_GROUP];
    float scale[GLQH_MAX_GROUP];
    int m_pad[GLQH_MAX_GROUP], out_features[GLQH_MAX_GROUP], nwg[GLQH_MAX_GROUP];
};

template <typename YT>
__global__ void __launch_bounds__(RHT_THREADS)
output_rht_group_kernel(rht_out_group g, int64_t y_stride, int B, int ksplit, int spb, int log_slice) {
    extern __shared__ float s[];
    const int z = blockIdx.z;
    const float *part = g.part[0];
    const f16 *su = g.su[0];
    void *y = g.y[0];
    float scale = g.scale[0];
    int m_pad = g.m_pad[0], out_features = g.out_features[0], nwg = g.nwg[0];
#pragma unroll
    for (int i = 1; i < GLQH_MAX_GROUP; ++i)
        if (i == z) {
            part = g.part[i]; su = g.su[i]; y = g.y[i]; scale = g.scale[i];
            m_pad = g.m_pad[i]; out_features = g.out_features[i]; nwg = g.nwg[i];
        }
    if ((int)blockIdx.x >= nwg) return;
    glqh_ysrc src = {};
    src.part = part;
    src.part_kstride = (int64_t)B * m_pad;
    src.ksplit = ksplit;
    src.scale[0] = scale;
    src.nparts = 1;
    glqh_meta_args margs;
    margs.canon = m_pad;
    output_rht_body<YT, true>(src, su, (YT *)y, y_stride, out_features, m_pad, nullptr, margs, 0.0f, spb,
                              log_slice, s);
}

// The same for layers whose Hadamard blocks have at most G slices: one workgroup per block,
// one group of 1024 / E threads per slice (E elements per thread).  Every group sums the split-K terms of its own rows only and the groups
// combine each other's sums through LDS, where the kernel above has every slice re-read the
// whole block: same terms, same order, same bits, 1/nsub of the loads.  Rows are multiples
// of E and the partial sums 16-byte aligned (checked by the launcher).
template <typename YT, int G, int E>
__global__ void __launch_bounds__((1024 / E) * G)
output_rht_block_kernel(rht_out_group g, int64_t y_stride, int B, int ksplit, int log_slice) {
    constexpr int GS = 1024 / E;                   // threads per slice
    extern __shared__ float s[];                   // G exchange buffers, then G sum buffers, one slice each
    const int z = blockIdx.z;
    const float *part = g.part[0];
    const f16 *su = g.su[0];
    void *y = g.y[0];
    float scale = g.scale[0];
    int m_pad = g.m_pad[0], out_features = g.out_features[0];
#pragma unroll
    for (int i = 1; i < GLQH_MAX_GROUP; ++i)
        if (i == z) {
            part = g.part[i]; su = g.su[i]; y = g.y[i]; scale = g.scale[i];
            m_pad = g.m_pad[i]; out_features = g.out_features[i];
        }
    if ((int)blockIdx.x >= __builtin_popcount((unsigned)m_pad)) return;
    glqh_meta_args margs;
    margs.canon = m_pad;
    const glqh_block_meta bm = glqh_meta_row(margs, nullptr, blockIdx.x);
    const int log_len = min(bm.log_bs, log_slice);
    const int nsub = bm.bs >> log_len;                         // <= G
    const int grp = threadIdx.x / GS, gt = threadIdx.x % GS;
    const bool mine = grp < nsub, live = mine && E * gt < (1 << log_len);
    const int base = bm.offset + (grp << log_len);             // this group's rows: slice grp of the block
    const float norm = rsqrt_pow2(bm.log_bs);
    const int64_t b = blockIdx.y;
    float *xchg = s + (grp << log_slice);
    float *sums = s + (G << log_slice);
    f16 su_raw[E];                                             // in flight beside the partial sums, used after them
#pragma unroll
    for (int q = 0; q < E; ++q) su_raw[q] = su[mine ? base + fht_wave_index<E>(log_len, live ? gt : 0, q) : 0];
    if (mine) {
        glqh_ysrc src = {};
        src.part = part;
        src.part_kstride = (int64_t)B * m_pad;
        src.ksplit = ksplit;
        src.scale[0] = scale;
        src.nparts = 1;
        rht_slice own = {};                                    // v_h for h = grp: rows base .. base + len - 1
        own.off = base; own.bs = 1 << log_len; own.log_bs = own.log_len = log_len;
        own.nsub = 1; own.r = 0; own.live = true;
        float v[E];
        // terms in flight: as many as there are (clamped repeats still cost their issue slots)
        if (ksplit <= 2) stage_partials_vec<E, 2>(v, src, own, b, m_pad, gt);
        else if (ksplit <= 4) stage_partials_vec<E, 4>(v, src, own, b, m_pad, gt);
        else if (ksplit <= 8) stage_partials_vec<E, 8>(v, src, own, b, m_pad, gt);
        else if (ksplit <= 12 || G > 2) stage_partials_vec<E, 12>(v, src, own, b, m_pad, gt);
        else stage_partials_vec<E, 24>(v, src, own, b, m_pad, gt);
        if (live) {
#pragma unroll
            for (int w = 0; w < E; w += 4)
                *(f32x4 *)(sums + (grp << log_slice) + E * gt + w) = f32x4{v[w], v[w + 1], v[w + 2], v[w + 3]};
        }
    }
    __syncthreads();
    float zv[E];                                               // slice r = grp: sum_h sign(r, h) v_h, h ascending
#pragma unroll
    for (int e = 0; e < E; ++e) zv[e] = 0.0f;
    if (live) {
        for (int h = 0; h < nsub; ++h) {
#pragma unroll
            for (int w = 0; w < E; w += 4) {
                const f32x4 vh = *(const f32x4 *)(sums + (h << log_slice) + E * gt + w);
#pragma unroll
                for (int e = 0; e < 4; ++e) zv[w + e] += had_sign(grp, h, vh[e]);
            }
        }
    }
    fht_wave<E, true>(zv, log_len, xchg, gt);
    if (live) {
        YT *yrow = (YT *)y + b * y_stride;
#pragma unroll
        for (int q = 0; q < E; ++q) {
            const int row = base + fht_wave_index<E>(log_len, gt, q);
            if (row < out_features) yrow[row] = f32_to_act<YT>(zv[q] * (norm * (float)su_raw[q]));
        }
    }
}

// Few tokens: 1024-point slices, one workgroup each, so that a single row still spreads
// over the chip (each slice re-reads its whole block).  Many tokens fill the chip by
// themselves: blocks up to 8192 points are then transformed whole, read once.
int rht_log_slice(int64_t B) { return B > 64 ? 13 : LOG_SLICE; }

int rht_slices_per_block(int64_t max_bs, int log_slice) {
    int64_t spb = max_bs >> log_slice;
    return spb < 1 ? 1 : (int)spb;
}

size_t rht_lds_bytes(int log_slice) {
    return (((size_t)1 << log_slice) + ((size_t)1 << log_slice) / 32 + 32) * sizeof(float);
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

namespace {
// whole-block 16-byte kernels: many tokens, canonical blocks of 8..8192 points
bool rht_wide_ok(int64_t B, const glqh_meta_args &margs, int64_t total, int64_t max_bs) {
    if (B <= 64 || margs.canon == 0 || max_bs > (1 << WIDE_LOG_MAX)) return false;
    return (total & 7) == 0;                                 // smallest block >= 8
}
bool aligned16(const void *p) { return ((uintptr_t)p & 15) == 0; }
}  // namespace

namespace {
// layout 0: rows of n_pad; 1 / 2: the tile kernels' token-fast blocks with Mp padded tokens (fp16 only)
int launch_input_rht_wide(const void *x, int x_dtype, int64_t x_stride, const void *sv, void *out, int out_dtype,
                          int layout, int64_t Mp, int64_t B, int64_t in_features, int64_t n_pad,
                          const glqh_meta_args &margs, int n_blocks, int64_t max_bs, float rsqrt_n,
                          hipStream_t stream) {
    const int64_t wgs = 64 * (((B + 7) / 8 + 7) / 8) * n_blocks;
    GLQH_REQUIRE(wgs <= 2147483647ll, "input_rht: too many blocks");
    const dim3 wgrid((unsigned)wgs);
    const size_t lds = std::max(rht_reg_lds_bytes(ilog2(max_bs)), layout == 2 ? WIDE_SMALL_LDS : (size_t)0);
#define GLQH_INW_LAUNCH(XT, OT, LAYOUT)                                                             \
    hipLaunchKernelGGL((input_rht_wide_kernel<XT, OT, LAYOUT>), wgrid, dim3(REG_THREADS), lds, stream, \
                       (const XT *)x, x_stride, (const f16 *)sv, (OT *)out, (int)in_features,       \
                       (int)n_pad, (int)Mp, (int)B, n_blocks, margs, rsqrt_n)
#define GLQH_INW_X(OT, LAYOUT)                                                                      \
    do {                                                                                            \
        if (x_dtype == GLQH_F16) GLQH_INW_LAUNCH(f16, OT, LAYOUT);                                  \
        else if (x_dtype == GLQH_BF16) GLQH_INW_LAUNCH(uint16_t, OT, LAYOUT);                       \
        else GLQH_INW_LAUNCH(float, OT, LAYOUT);                                                    \
    } while (0)
    if (layout == 1) GLQH_INW_X(f16, 1);
    else if (layout == 2) GLQH_INW_X(f16, 2);
    else if (out_dtype == GLQH_F32) GLQH_INW_X(float, 0);
    else GLQH_INW_X(f16, 0);
#undef GLQH_INW_X
#undef GLQH_INW_LAUNCH
    GLQH_LAUNCH_CHECK("input_rht launch");
    return 0;
}
}  // namespace

// The input transform written straight into a tile kernel's operand layout (layout 1: E8, 2:
// trellis; Mp padded tokens).  Returns -1 without launching when the call does not qualify
// (non-canonical blocks, blocks over 8192 points, unaligned rows): the caller then transforms into
// rows and lets the tile launcher repack.
int glqh_launch_input_rht_blocked(const void *x, int x_dtype, int64_t x_stride, const void *sv, void *xb,
                                  int layout, int64_t Mp, int64_t B, int64_t in_features, int64_t n_pad,
                                  const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream) {
    glqh_range range("input_rht");
    if (!x || !sv || !xb || B < 1 || in_features < 1 || in_features > n_pad) return -1;
    if (x_dtype != GLQH_F16 && x_dtype != GLQH_BF16 && x_dtype != GLQH_F32) return -1;
    glqh_meta_args margs;
    int64_t max_bs = n_pad;
    if (n_blocks > 1) {
        if (!blocks_host) return -1;
        max_bs = 0;
        for (int64_t i = 0; i < n_blocks; ++i) max_bs = blocks_host[i] > max_bs ? blocks_host[i] : max_bs;
    } else {
        n_blocks = 1;
    }
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, n_pad) || margs.canon != n_pad) return -1;
    const int x_size = x_dtype == GLQH_F32 ? 4 : 2;
    if (max_bs > (1 << WIDE_LOG_MAX) || (n_pad & 31) != 0) return -1;
    if (!aligned16(x) || !aligned16(xb) || !aligned16(sv) || (x_stride * x_size) % 16 != 0) return -1;
    return launch_input_rht_wide(x, x_dtype, x_stride, sv, xb, GLQH_F16, layout, Mp, B, in_features, n_pad, margs,
                                 (int)n_blocks, max_bs, 0.0f, stream);
}

int glqh_launch_input_rht(const void *x, int x_dtype, int64_t x_stride, const void *sv,
                          void *out, int out_dtype, int64_t B, int64_t in_features, int64_t n_pad,
                          const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                          int64_t n_blocks, float rsqrt_n, hipStream_t stream) {
    glqh_range range("input_rht");
    GLQH_REQUIRE(x && sv && out, "input_rht: null pointer");
    GLQH_REQUIRE(B >= 1 && B <= 65535, "input_rht: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(in_features >= 1 && in_features <= n_pad,
                 "input_rht: in_features %lld must be in 1..n_pad=%lld", (long long)in_features,
                 (long long)n_pad);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16 || x_dtype == GLQH_F32,
                 "input_rht: bad x dtype");
    GLQH_REQUIRE(out_dtype == GLQH_F32 || out_dtype == GLQH_F16, "input_rht: out must be f32 or f16");
    int64_t max_bs = n_pad;
    glqh_meta_args margs;
    if (n_blocks > 1) {
        GLQH_REQUIRE(meta_dev && blocks_host, "input_rht: block-diagonal call needs meta and sizes");
        if (check_blocks(blocks_host, n_blocks, n_pad, &max_bs, "input_rht")) return 1;
    } else {
        GLQH_REQUIRE((n_pad & (n_pad - 1)) == 0, "input_rht: single block n_pad=%lld is not a power of two",
                     (long long)n_pad);
        meta_dev = nullptr;
        n_blocks = 1;
    }
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, n_pad))
        margs.canon = 0;                               // not canonical: kernel reads meta_dev
    const int x_size = x_dtype == GLQH_F32 ? 4 : 2, o_size = out_dtype == GLQH_F32 ? 4 : 2;
    if (rht_wide_ok(B, margs, n_pad, max_bs) && aligned16(x) && aligned16(out) && aligned16(sv) &&
        (x_stride * x_size) % 16 == 0 && (n_pad * o_size) % 16 == 0)
        return launch_input_rht_wide(x, x_dtype, x_stride, sv, out, out_dtype, 0, 0, B, in_features, n_pad, margs,
                                     (int)n_blocks, max_bs, rsqrt_n, stream);
    const int log_slice = rht_log_slice(B);
    const int spb = rht_slices_per_block(max_bs, log_slice);
    GLQH_REQUIRE(n_blocks * spb <= 2147483647ll, "input_rht: too many slices");
    dim3 grid((unsigned)(n_blocks * spb), (unsigned)B);
#define GLQH_IN_LAUNCH(XT, OT)                                                                      \
    hipLaunchKernelGGL((input_rht_kernel<XT, OT>), grid, dim3(RHT_THREADS),                         \
                       rht_lds_bytes(log_slice), stream, (const XT *)x, x_stride, (const f16 *)sv,  \
                       (OT *)out, (int)in_features, (int)n_pad, meta_dev, margs, rsqrt_n, spb,      \
                       log_slice)
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

// n (up to GLQH_MAX_GROUP) sign vectors on the same rows, each into its own buffer in the trellis tile kernels' operand
// layout: one launch.  -1 (nothing launched) where glqh_launch_input_rht_blocked would not apply either.
int glqh_launch_input_rht_blocked_multi(const void *x, int x_dtype, int64_t x_stride, const void *const sv[],
                                        void *const xb[], int n, int64_t Mp, int64_t B, int64_t in_features, int64_t n_pad,
                                        const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream) {
    if (!x || n < 1 || n > GLQH_MAX_GROUP || B < 1 || in_features < 1 || in_features > n_pad) return -1;
    if (x_dtype != GLQH_F16 && x_dtype != GLQH_BF16) return -1;
    glqh_meta_args margs;
    int64_t max_bs = n_pad;
    if (n_blocks > 1) {
        if (!blocks_host) return -1;
        max_bs = 0;
        for (int64_t i = 0; i < n_blocks; ++i) max_bs = blocks_host[i] > max_bs ? blocks_host[i] : max_bs;
    } else {
        n_blocks = 1;
    }
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, n_pad) || margs.canon != n_pad) return -1;
    if (max_bs > (1 << WIDE_LOG_MAX) || (n_pad & 31) != 0) return -1;
    if (!aligned16(x) || (x_stride * 2) % 16 != 0) return -1;
    rht_in_wide_multi mg = {};
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        const int j = i < n ? i : 0;
        if (!sv[j] || !xb[j] || !aligned16(sv[j]) || !aligned16(xb[j])) return -1;
        mg.sv[i] = (const f16 *)sv[j];
        mg.out[i] = (f16 *)xb[j];
    }
    const int64_t wgs = 64 * (((B + 7) / 8 + 7) / 8) * n_blocks;
    if (wgs > 2147483647ll) return -1;
    glqh_range range("input_rht");
    const dim3 wgrid((unsigned)wgs, (unsigned)n);
    const size_t lds = std::max(rht_reg_lds_bytes(ilog2(max_bs)), WIDE_SMALL_LDS);
    if (x_dtype == GLQH_F16)
        hipLaunchKernelGGL((input_rht_wide_multi_kernel<f16>), wgrid, dim3(REG_THREADS), lds, stream, (const f16 *)x, x_stride,
                           mg, (int)in_features, (int)n_pad, (int)Mp, (int)B, (int)n_blocks, margs, 0.0f);
    else
        hipLaunchKernelGGL((input_rht_wide_multi_kernel<uint16_t>), wgrid, dim3(REG_THREADS), lds, stream,
                           (const uint16_t *)x, x_stride, mg, (int)in_features, (int)n_pad, (int)Mp, (int)B, (int)n_blocks,
                           margs, 0.0f);
    GLQH_LAUNCH_CHECK("input_rht group launch");
    return 0;
}

// n (up to GLQH_MAX_GROUP) sign vectors on the same rows, fp16 out, few rows (the small-batch kernel): one launch.
// -1 (nothing launched) when the call is one for the whole-block kernels or the dtypes are others.
int glqh_launch_input_rht_multi(const void *x, int x_dtype, int64_t x_stride, const void *const sv[], void *const out[],
                                int n, int64_t B, int64_t in_features, int64_t n_pad, const glqh_block_meta *meta_dev,
                                const int64_t *blocks_host, int64_t n_blocks, hipStream_t stream) {
    if (n < 1 || n > GLQH_MAX_GROUP || B < 1 || B > 65535 || in_features < 1 || in_features > n_pad) return -1;
    if (x_dtype != GLQH_F16 && x_dtype != GLQH_BF16) return -1;
    int64_t max_bs = n_pad;
    glqh_meta_args margs;
    if (n_blocks > 1) {
        if (!meta_dev || !blocks_host || check_blocks(blocks_host, n_blocks, n_pad, &max_bs, "input_rht")) return -1;
    } else {
        if ((n_pad & (n_pad - 1)) != 0) return -1;
        meta_dev = nullptr;
        n_blocks = 1;
    }
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, n_pad)) margs.canon = 0;
    if (rht_wide_ok(B, margs, n_pad, max_bs)) return -1;       // many rows: the whole-block kernels, one launch each
    glqh_range range("input_rht");
    const int log_slice = rht_log_slice(B);
    const int spb = rht_slices_per_block(max_bs, log_slice);
    if (n_blocks * spb > 2147483647ll) return -1;
    rht_in_multi g = {};
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        g.sv[i] = (const f16 *)sv[i < n ? i : 0];
        g.out[i] = (f16 *)out[i < n ? i : 0];
    }
    dim3 grid((unsigned)(n_blocks * spb), (unsigned)B, (unsigned)n);
    if (x_dtype == GLQH_F16)
        hipLaunchKernelGGL((input_rht_multi_kernel<f16>), grid, dim3(RHT_THREADS), rht_lds_bytes(log_slice), stream,
                           (const f16 *)x, x_stride, g, (int)in_features, (int)n_pad, meta_dev, margs, 0.0f, spb, log_slice);
    else
        hipLaunchKernelGGL((input_rht_multi_kernel<uint16_t>), grid, dim3(RHT_THREADS), rht_lds_bytes(log_slice), stream,
                           (const uint16_t *)x, x_stride, g, (int)in_features, (int)n_pad, meta_dev, margs, 0.0f, spb,
                           log_slice);
    GLQH_LAUNCH_CHECK("input_rht group launch");
    return 0;
}

namespace {
// The whole-block kernels for canonical blocks and many rows; -1 (nothing launched) when they do not apply.
int launch_output_rht_wide(const glqh_ysrc &src, const void *su, void *y, int y_dtype, int64_t y_stride, int64_t B,
                           int64_t out_features, int64_t m_pad, const glqh_meta_args &margs, int64_t n_blocks,
                           int64_t max_bs, float rsqrt_m, hipStream_t stream) {
    const int y_size = y_dtype == GLQH_F32 ? 4 : 2;
    const int pq = src.part_f16 ? 8 : 4;                     // elements per 16 bytes of partial sums
    const bool src_ok = src.nparts == 0
        ? (aligned16(src.direct) && src.stride % 4 == 0)
        : (aligned16(src.part) && m_pad % pq == 0 && src.part_kstride % pq == 0 && src.part_sstride % pq == 0 &&
           (!src.copy_out || (aligned16(src.copy_out) && src.copy_stride % 4 == 0)));
    // whole blocks per workgroup also from 32 tokens on when the rows are many (whole linear,
    // 64 tokens: 11008 x 2048 56.9 -> 45.3 us, 14336 x 4096 70.4 -> 61.6; 2048 x 11008 41.5 -> 43.7)
    const int64_t Bw = ((B >= 32 && m_pad >= 8192) || B > 32) ? 65 : B;
    if (!(rht_wide_ok(Bw, margs, m_pad, max_bs) && src_ok && aligned16(y) && aligned16(su) &&
          (y_stride * y_size) % 16 == 0))
        return -1;
    dim3 wgrid((unsigned)(64 * ((B + 63) / 64) * n_blocks));
    const size_t lds = rht_reg_lds_bytes(ilog2(max_bs));
#define GLQH_OUTW_LAUNCH(YT)                                                                        \
    hipLaunchKernelGGL((output_rht_wide_kernel<YT>), wgrid, dim3(REG_THREADS), lds, stream, src,    \
                       (const f16 *)su, (YT *)y, y_stride, (int)out_features, (int)m_pad, (int)B, (int)n_blocks, margs, \
                       rsqrt_m)
    if (y_dtype == GLQH_F16) GLQH_OUTW_LAUNCH(f16);
    else if (y_dtype == GLQH_BF16) GLQH_OUTW_LAUNCH(uint16_t);
    else GLQH_OUTW_LAUNCH(float);
#undef GLQH_OUTW_LAUNCH
    GLQH_LAUNCH_CHECK("output_rht launch");
    return 0;
}
}  // namespace

// Output transform of a layer whose blocks are the canonical ones of m_pad (descending powers of two), many rows:
// the whole-block kernels.  -1 (nothing launched) when they do not apply (a block above 8192 rows, alignment).
int glqh_launch_output_rht_canon_wide(const glqh_ysrc &src, const void *su, void *y, int y_dtype, int64_t y_stride,
                                      int64_t B, int64_t out_features, int64_t m_pad, hipStream_t stream) {
    int64_t blocks[64];
    int n = 0;
    for (int bit = 62; bit >= 0; --bit)
        if (m_pad & ((int64_t)1 << bit)) blocks[n++] = (int64_t)1 << bit;
    glqh_meta_args margs;
    if (n == 0 || !glqh_fill_meta_args(&margs, n > 1 ? blocks : nullptr, n > 1 ? n : 1, m_pad)) return -1;
    return launch_output_rht_wide(src, su, y, y_dtype, y_stride, B, out_features, m_pad, margs, n, blocks[0], 0.0f, stream);
}

int glqh_launch_output_rht(const glqh_ysrc &src, const void *su, void *y, int y_dtype,
                           int64_t y_stride, int64_t B, int64_t out_features, int64_t m_pad,
                           const glqh_block_meta *meta_dev, const int64_t *blocks_host,
                           int64_t n_blocks, int64_t max_bs_hint, float rsqrt_m,
                           hipStream_t stream) {
    glqh_range range("output_rht");
    GLQH_REQUIRE(B >= 1 && B <= 65535, "output_rht: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(y != nullptr && su != nullptr, "output_rht: null y or su");
    GLQH_REQUIRE(out_features >= 1 && out_features <= m_pad,
                 "output_rht: out_features %lld must be in 1..m_pad=%lld", (long long)out_features,
                 (long long)m_pad);
    GLQH_REQUIRE(y_dtype == GLQH_F16 || y_dtype == GLQH_BF16 || y_dtype == GLQH_F32,
                 "output_rht: bad y dtype");
    int64_t max_bs = m_pad;
    glqh_meta_args margs;
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
    if (meta_dev && !blocks_host) margs.canon = 0;         // shard-batched call: device meta only
    else if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, m_pad)) margs.canon = 0;
    {
        const int rc = launch_output_rht_wide(src, su, y, y_dtype, y_stride, B, out_features, m_pad, margs, n_blocks,
                                              max_bs, rsqrt_m, stream);
        if (rc >= 0) return rc;
    }
    GLQH_REQUIRE(!src.part_f16, "output_rht: fp16 partial sums need the whole-block kernels (more than 32 tokens, "
                                "canonical blocks of at most 8192 rows)");
    const int log_slice = rht_log_slice(B);
    const int spb = rht_slices_per_block(max_bs, log_slice);
    GLQH_REQUIRE(n_blocks * spb <= 2147483647ll, "output_rht: too many slices");
    dim3 grid((unsigned)(n_blocks * spb), (unsigned)B);
#define GLQH_OUT_LAUNCH(YT, PARTS)                                                                  \
    hipLaunchKernelGGL((output_rht_kernel<YT, PARTS>), grid, dim3(RHT_THREADS),                     \
                       rht_lds_bytes(log_slice), stream, src, (const f16 *)su, (YT *)y, y_stride,   \
                       (int)out_features, (int)m_pad, meta_dev, margs, rsqrt_m, spb, log_slice)
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

int glqh_output_rht_wide_eligible(int64_t B, const int64_t *blocks_host, int64_t n_blocks, int64_t m_pad) {
    glqh_meta_args margs;
    int64_t max_bs = m_pad;
    if (n_blocks > 1) {
        if (!blocks_host || check_blocks(blocks_host, n_blocks, m_pad, &max_bs, "output_rht")) return 0;
    } else if (m_pad & (m_pad - 1)) {
        return 0;
    }
    if (!glqh_fill_meta_args(&margs, n_blocks > 1 ? blocks_host : nullptr, n_blocks > 1 ? n_blocks : 1, m_pad)) return 0;
    const int64_t Bw = ((B >= 32 && m_pad >= 8192) || B > 32) ? 65 : B;
    return rht_wide_ok(Bw, margs, m_pad, max_bs) ? 1 : 0;
}

int glqh_rht_init(void) { return 0; }

// ---- routed experts (glq/csrc/glq_cuda.cu:5030-5250) ------------------------------------------
// The finishing launches of the two projections of a mixture-of-experts layer.  Rows are slots
// (token, choice); the slot's expert, read from topk_ids on the device, selects the output signs
// (su_base + expert * m_pad) and the scale.  Partial sums: [K slot][slot][row].
namespace {
struct moe_out_args {
    const float *part;
    int ks, part_f16, n_slots, n_experts;
    const int64_t *topk_ids;
    const f16 *su_base;
    const float *wscale_dev;
    int out_features, m_pad;
};

// (fp16 sums -- the tile form's -- carry the expert's scale already: an unscaled sum over a long row of large
// activations can pass the fp16 range where the scaled one, of the size of the layer's output, does not)
__device__ __forceinline__ glqh_ysrc moe_src(const moe_out_args &a, float scale) {
    if (a.part_f16 && scale != 0.0f) scale = 1.0f;
    glqh_ysrc src = {};
    src.part = a.part;
    src.part_kstride = (int64_t)a.n_slots * a.m_pad;
    src.ksplit = a.ks;
    src.part_f16 = a.part_f16;
    src.scale[0] = scale;
    src.nparts = 1;
    return src;
}

// first projection: h[slot][row] = su * H(sum) * Wscale, fp16 (slots of an invalid expert: zeros)
__global__ void __launch_bounds__(REG_THREADS)
moe_output_rht_kernel(moe_out_args a, f16 *__restrict__ h, int64_t h_stride, glqh_meta_args margs) {
    extern __shared__ float s[];
    const rht_slice blk = rht_slice_of(margs, 0.0f, blockIdx.x);
    const int slot = blockIdx.y;
    const int64_t e = a.topk_ids[slot];
    if (e < 0 || e >= a.n_experts) {                            // uniform over the workgroup
        for (int i = threadIdx.x; i < blk.bs; i += REG_THREADS)
            if (blk.off + i < a.out_features) h[slot * h_stride + blk.off + i] = (f16)0.0f;
        return;
    }
    const glqh_ysrc src = moe_src(a, a.wscale_dev[e]);
    const f16 *su = a.su_base + e * a.m_pad;
    const wide_role role = {(int)threadIdx.x, 0, REG_THREADS, 0, true};   // one row per workgroup
    if (blk.log_bs > 12) output_rht_wide_body<16, f16>(src, su, h, h_stride, a.out_features, a.m_pad, blk, s, slot, role);
    else output_rht_wide_body<8, f16>(src, su, h, h_stride, a.out_features, a.m_pad, blk, s, slot, role);
}

// The same for many slots, dealt out like output_rht_wide_kernel's rows: eight slots per workgroup group on the
// eight XCDs, blocks of up to 512 rows with 4096 / bs slots per workgroup.  A thread's slot decides its signs and
// scale; slots of an invalid expert read nothing (their sums were never written) and get zeros.
template <int E>
__device__ __forceinline__ void moe_output_wide_row(const moe_out_args &a, f16 *__restrict__ h, int64_t h_stride,
                                                    const rht_slice &blk, float *s, int64_t slot, const wide_role role) {
    const int64_t e = a.topk_ids[slot];
    const bool valid = e >= 0 && e < a.n_experts;
    const glqh_ysrc src = moe_src(a, valid ? a.wscale_dev[e] : 0.0f);
    const f16 *su = a.su_base + (valid ? e : 0) * a.m_pad;
    wide_role r = role;
    r.active = role.active && valid;
    output_rht_wide_body<E, f16>(src, su, h, h_stride, a.out_features, a.m_pad, blk, s, slot, r);
    if (role.active && !valid && E * role.te < blk.bs) {
        const int row = blk.off + E * role.te;
#pragma unroll
        for (int j = 0; j < E; ++j)
            if (row + j < a.out_features) h[slot * h_stride + row + j] = (f16)0.0f;
    }
}

__global__ void __launch_bounds__(REG_THREADS)
moe_output_rht_wide_kernel(moe_out_args a, f16 *__restrict__ h, int64_t h_stride, int n_blocks, glqh_meta_args margs) {
    extern __shared__ float s[];
    const int L = blockIdx.x, xcd = L & 7, member = (L >> 3) & 7, rest = L >> 6, g = rest / n_blocks;
    const rht_slice blk = rht_slice_of(margs, 0.0f, rest % n_blocks);
    const int r0 = g * 64 + member * 8, B = a.n_slots;
    if (blk.log_bs <= WIDE_SMALL_LOG) {
        const int lt = 12 - blk.log_bs, T = 1 << lt;
        if ((r0 & (T - 1)) != 0 || xcd != ((r0 >> lt) & 7) || r0 >= B) return;
        const int ntok = min(T, B - r0);
        const wide_role role = wide_role_of(blk, ntok);
        moe_output_wide_row<8>(a, h, h_stride, blk, s, (int64_t)r0 + min(role.tok, ntok - 1), role);
        return;
    }
    const int64_t b = (int64_t)r0 + xcd;
    if (b >= B) return;                                       // uniform over the workgroup
    const wide_role role = wide_role_of(blk, 1);
    if (blk.log_bs > 12) moe_output_wide_row<16>(a, h, h_stride, blk, s, b, role);
    else moe_output_wide_row<8>(a, h, h_stride, blk, s, b, role);
}

__device__ __forceinline__ float moe_gate(float g, int act) {
    if (act == 0) return g / (1.0f + expf(-g));
    if (act == 1) return 0.5f * g * (1.0f + tanhf(0.7978845608028654f * (g + 0.044715f * g * g * g)));
    const float q = fmaxf(g, 0.0f);
    return q * q;
}

// Everything between the two decode launches for a slot whose rows are grouped by expert, in one workgroup per
// slot: the first projection's output transform (sums -> h, rounded to fp16 as the separate launch stores
// it), act(gate) * up (fp16), and the second projection's input transform, written where its decode launch reads:
// LAYOUT 0 row `slot` of (n_slots, n_pad2), LAYOUT 2 position `pos` of the tile kernel's blocked operand.  h and
// the activated row live in LDS only.  The workgroups walk the sorted order (eight neighbouring positions on
// one XCD: in the blocked layout their 16-byte pieces share lines); slots of an invalid expert are not in it.
struct moe_mid_args {
    moe_out_args o;
    const f16 *sv2;
    const int *perm, *pexp, *n_valid;                            // slot and expert of every position of the sorted order
    int intermediate, act, n_pad2, Mp, nb13, nb2, s_floats;
};

template <int LAYOUT>
__global__ void __launch_bounds__(REG_THREADS)
moe_mid_kernel(moe_mid_args a, f16 *__restrict__ out, glqh_meta_args m13, glqh_meta_args m2) {
    extern __shared__ float s[];
    const int L = blockIdx.x, pos = (L >> 6) * 64 + (L & 7) * 8 + ((L >> 3) & 7);
    if (pos >= *a.n_valid) return;                               // uniform over the workgroup
    const int slot = a.perm[pos];
    const int64_t e = a.pexp[pos];
    f16 *hrow = (f16 *)(s + a.s_floats), *arow = hrow + a.o.m_pad;
    const int tid = threadIdx.x;
    const wide_role role = {tid, 0, (int)blockDim.x, 0, true};
    const glqh_ysrc src = moe_src(a.o, a.o.wscale_dev[e]);
    const f16 *su = a.o.su_base + e * a.o.m_pad;
    // the blocks of the first projection's row in turn, eight elements per thread; the next block's sums and
    // signs are requested before this one's are transformed (a block of 8192 points: sixteen per thread, by itself)
    struct req {
        float v[8], f[8];
    };
    auto request = [&](req &r, const rht_slice &blk) {
        const bool active = 8 * tid < blk.bs;
        output_wide_load<8>(r.v, src, slot, a.o.m_pad, blk, active, tid);
#pragma unroll
        for (int j = 0; j < 8; ++j) r.f[j] = 0.0f;
        if (active && blk.off + 8 * tid < a.o.out_features) load8<f16>(su + blk.off + 8 * tid, r.f);
    };
    const int big = rht_slice_of(m13, 0.0f, 0).bs > 8 * (int)blockDim.x ? 1 : 0;   // only the first block can be
    req cur, nxt;
    if (big < a.nb13) request(cur, rht_slice_of(m13, 0.0f, big));
    if (big) output_rht_wide_body<16, f16>(src, su, hrow, 0, a.o.out_features, a.o.m_pad, rht_slice_of(m13, 0.0f, 0), s, slot, role);
    for (int bi = big; bi < a.nb13; ++bi) {
        const rht_slice blk = rht_slice_of(m13, 0.0f, bi);
        if (bi + 1 < a.nb13) request(nxt, rht_slice_of(m13, 0.0f, bi + 1));
        if (bi) __syncthreads();                                 // the previous block is done with the exchange space
        const bool active = 8 * tid < blk.bs;
        output_wide_transform<8>(cur.v, blk, s, tid, active);
        const int row = blk.off + 8 * tid;
        if (active && row < a.o.out_features) {
            float w[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) w[j] = cur.v[j] * (blk.norm * cur.f[j]);
            if (row + 8 <= a.o.out_features) {
                store8<f16>(hrow + row, w);
            } else {
#pragma unroll
                for (int j = 0; j < 8; ++j)
                    if (row + j < a.o.out_features) hrow[row + j] = (f16)w[j];
            }
        }
        cur = nxt;
    }
    __syncthreads();
    for (int i = threadIdx.x; i < a.intermediate; i += blockDim.x)
        arow[i] = (f16)(moe_gate((float)hrow[i], a.act) * (float)hrow[a.intermediate + i]);
    for (int bi = 0; bi < a.nb2; ++bi) {
        const rht_slice blk = rht_slice_of(m2, 0.0f, bi);
        __syncthreads();                                         // arow written / the previous block done with s
        const int token = LAYOUT == 2 ? pos : slot;
        if (blk.bs > 8 * (int)blockDim.x)
            input_rht_wide_body<16, f16, f16, LAYOUT>(arow, 0, a.sv2, out, a.intermediate, a.n_pad2, a.Mp, token, blk, s, role);
        else
            input_rht_wide_body<8, f16, f16, LAYOUT>(arow, 0, a.sv2, out, a.intermediate, a.n_pad2, a.Mp, token, blk, s, role);
    }
}

// The second projection's output transform and the weighted sum over a token's choices in one launch, for many
// tokens: rows = tokens, dealt out like output_rht_wide_kernel's; a thread transforms its part of every choice in
// turn, rounds it to fp16 as the separate launch stores it, and adds it times the routing weight in fp32, choices
// in order (glq_moe_weighted_scatter_reduce_kernel, glq/csrc/glq_cuda.cu:4520-4537).
template <int E, typename YT>
__device__ __forceinline__ void moe_final_row(const moe_out_args &a, const float *__restrict__ topk_w, int top_k,
                                              YT *__restrict__ out, int64_t out_stride, const rht_slice &blk, float *s,
                                              int64_t token, const wide_role role) {
    const int tid = threadIdx.x;
    const bool active = role.active && E * role.te < blk.bs;
    const int row = blk.off + E * role.te;
    float acc[E];
#pragma unroll
    for (int j = 0; j < E; ++j) acc[j] = 0.0f;
    // the next choice's sums, signs and weight are requested before this one's are transformed
    struct choice {
        float v[E], f[E], w;
        bool valid;
    };
    auto request = [&](choice &ch, int c) {
        const int64_t slot = token * top_k + c;
        const int64_t e = a.topk_ids[slot];
        ch.valid = e >= 0 && e < a.n_experts;
        const glqh_ysrc src = moe_src(a, ch.valid ? a.wscale_dev[e] : 0.0f);
        output_wide_load<E>(ch.v, src, slot, a.m_pad, blk, active && ch.valid, role.te);
        ch.w = 0.0f;
#pragma unroll
        for (int j = 0; j < E; ++j) ch.f[j] = 0.0f;
        if (active && ch.valid && row < a.out_features) {
#pragma unroll
            for (int j = 0; j < E; j += 8) load8<f16>(a.su_base + e * a.m_pad + row + j, ch.f + j);
            ch.w = topk_w[slot];
        }
    };
    choice cur, nxt;
    request(cur, 0);
    for (int c = 0; c < top_k; ++c) {
        if (c + 1 < top_k) request(nxt, c + 1);
        if (c) __syncthreads();                                  // the previous choice is done with the exchange space
        output_wide_transform<E>(cur.v, blk, s, tid, active && cur.valid);
        if (active && cur.valid && row < a.out_features) {
#pragma unroll
            for (int j = 0; j < E; ++j) acc[j] += cur.w * (float)(f16)(cur.v[j] * (blk.norm * cur.f[j]));
        }
        cur = nxt;
    }
    if (active && row < a.out_features) {
        YT *orow = out + token * out_stride;
        if (row + E <= a.out_features) {
#pragma unroll
            for (int j = 0; j < E; j += 8) store8<YT>(orow + row + j, acc + j);
        } else {
#pragma unroll
            for (int j = 0; j < E; ++j)
                if (row + j < a.out_features) orow[row + j] = f32_to_act<YT>(acc[j]);
        }
    }
}

// BIG: the row has a block of 8192 points (sixteen elements per thread there, and their registers: a kernel of
// its own, so that the others keep their occupancy)
template <typename YT, bool BIG>
__global__ void __launch_bounds__(REG_THREADS)
moe_final_kernel(moe_out_args a, const float *__restrict__ topk_w, int top_k, int num_tokens, YT *__restrict__ out,
                 int64_t out_stride, int n_blocks, glqh_meta_args margs) {
    extern __shared__ float s[];
    const int L = blockIdx.x, xcd = L & 7, member = (L >> 3) & 7, rest = L >> 6, g = rest / n_blocks;
    const rht_slice blk = rht_slice_of(margs, 0.0f, rest % n_blocks);
    const int r0 = g * 64 + member * 8, B = num_tokens;
    if (blk.log_bs <= WIDE_SMALL_LOG) {
        const int lt = 12 - blk.log_bs, T = 1 << lt;
        if ((r0 & (T - 1)) != 0 || xcd != ((r0 >> lt) & 7) || r0 >= B) return;
        const int ntok = min(T, B - r0);
        const wide_role role = wide_role_of(blk, ntok);
        moe_final_row<8, YT>(a, topk_w, top_k, out, out_stride, blk, s, (int64_t)r0 + min(role.tok, ntok - 1), role);
        return;
    }
    const int64_t b = (int64_t)r0 + xcd;
    if (b >= B) return;                                       // uniform over the workgroup
    const wide_role role = wide_role_of(blk, 1);
    if constexpr (BIG) {
        if (blk.bs > 8 * (int)blockDim.x) {
            moe_final_row<16, YT>(a, topk_w, top_k, out, out_stride, blk, s, b, role);
            return;
        }
    }
    moe_final_row<8, YT>(a, topk_w, top_k, out, out_stride, blk, s, b, role);
}

// out[slot][i] = act(h[slot][i]) * h[slot][intermediate + i]: 0 SiLU, 1 GELU (tanh form), 2 squared ReLU
// (glq/csrc/glq_cuda.cu:4540-4559).  V elements per thread (8 when the rows allow 16-byte accesses).
template <int V>
__global__ void __launch_bounds__(256)
moe_gated_act_kernel(const f16 *__restrict__ h, int64_t h_stride, f16 *__restrict__ out, int n_slots,
                     int intermediate, int act) {
    const int per_row = intermediate / V;
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (idx >= (int64_t)n_slots * per_row) return;
    const int slot = (int)(idx / per_row), i = V * (int)(idx % per_row);
    float g[V], up[V], r[V];
    if constexpr (V == 8) {
        load8<f16>(h + slot * h_stride + i, g);
        load8<f16>(h + slot * h_stride + intermediate + i, up);
    } else {
        g[0] = (float)h[slot * h_stride + i];
        up[0] = (float)h[slot * h_stride + intermediate + i];
    }
#pragma unroll
    for (int j = 0; j < V; ++j) r[j] = (float)(f16)(moe_gate(g[j], act) * up[j]);
    if constexpr (V == 8) store8<f16>(out + (int64_t)slot * intermediate + i, r);
    else out[(int64_t)slot * intermediate + i] = (f16)r[0];
}

// out[token][row] = sum_j w[token][j] * y[token * top_k + j][row], j in order, fp32 accumulation of the fp16
// per-slot results (glq_moe_weighted_scatter_reduce_kernel, glq/csrc/glq_cuda.cu:4520-4537); slots of an
// invalid expert are skipped.  One thread per 8 rows.
template <typename YT>
__global__ void __launch_bounds__(256)
moe_weighted_sum_kernel(const f16 *__restrict__ y, int64_t y_stride, const int64_t *__restrict__ topk_ids,
                        const float *__restrict__ topk_w, int top_k, int n_experts, int out_features,
                        YT *__restrict__ out, int64_t out_stride) {
    const int token = blockIdx.y;
    const int row = 8 * (blockIdx.x * 256 + threadIdx.x);
    if (row >= out_features) return;
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int j = 0; j < top_k; ++j) {
        const int slot = token * top_k + j;
        const int64_t ex = topk_ids[slot];
        if (ex < 0 || ex >= n_experts) continue;
        float v[8];
        load8<f16>(y + slot * y_stride + row, v);
        const float w = topk_w[slot];
#pragma unroll
        for (int e = 0; e < 8; ++e) acc[e] += w * v[e];
    }
    store8<YT>(out + (int64_t)token * out_stride + row, acc);
}

// Slots grouped by expert, without a sort: wave e counts the valid slots of experts below e
// (offs[e]; wave n_experts: the total, offs[n_experts]) and then writes its own slots, in ascending
// slot order, from that position on.  Fixed by the routing alone: the same table on every call.
__global__ void __launch_bounds__(256)
moe_route_kernel(const int64_t *__restrict__ topk_ids, int n_slots, int n_experts, int *__restrict__ perm,
                 int *__restrict__ pexp, int *__restrict__ offs) {
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63;
    if (e > n_experts) return;                                   // uniform over the wave
    constexpr int U = 8;                                         // 512 slots requested before the first is looked at
    int below = 0;
    for (int base = 0; base < n_slots; base += 64 * U) {
        int64_t id[U];
#pragma unroll
        for (int u = 0; u < U; ++u) id[u] = base + 64 * u + lane < n_slots ? topk_ids[base + 64 * u + lane] : -1;
#pragma unroll
        for (int u = 0; u < U; ++u) below += __builtin_popcountll(__ballot(id[u] >= 0 && id[u] < e));
    }
    if (lane == 0) offs[e] = below;
    if (e == n_experts) return;
    int mine = 0;
    for (int base = 0; base < n_slots; base += 64 * U) {
        int64_t id[U];
#pragma unroll
        for (int u = 0; u < U; ++u) id[u] = base + 64 * u + lane < n_slots ? topk_ids[base + 64 * u + lane] : -1;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned long long hit = __ballot(id[u] == e);
            if (id[u] == e) {
                const int at = below + mine + __builtin_popcountll(hit & ((1ull << lane) - 1ull));
                perm[at] = base + 64 * u + lane;
                pexp[at] = e;
            }
            mine += __builtin_popcountll(hit);
        }
    }
}

// The same table for many slots, in two launches: the slots in SEG segments, wave (expert, segment) first counts
// its expert's slots in its segment (cnt[segment][expert], expert n_experts = every valid slot), then finds its
// first position from the counts of the experts below and of the segments before it.  The one launch above has
// every expert's wave walk all the slots twice: 80 us at 32768 slots, 21 us at 8192.
constexpr int MOE_ROUTE_SEG_SLOTS = 2048;
constexpr int MOE_ROUTE_MAX_SEG = 32;
constexpr int MOE_OUT_WIDE_MIN = 64;

__device__ __forceinline__ int moe_route_count(const int64_t *__restrict__ topk_ids, int s0, int s1, int e, int n_experts,
                                               int lane) {
    int n = 0;
    constexpr int U = 8;
    for (int base = s0; base < s1; base += 64 * U) {
        int64_t id[U];
#pragma unroll
        for (int u = 0; u < U; ++u) id[u] = base + 64 * u + lane < s1 ? topk_ids[base + 64 * u + lane] : -1;
#pragma unroll
        for (int u = 0; u < U; ++u)
            n += __builtin_popcountll(__ballot(e == n_experts ? (id[u] >= 0 && id[u] < n_experts) : id[u] == e));
    }
    return n;
}

__global__ void __launch_bounds__(256)
moe_route_count_kernel(const int64_t *__restrict__ topk_ids, int n_slots, int n_experts, int seg_slots,
                       int *__restrict__ cnt) {
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, seg = blockIdx.y;
    if (e > n_experts) return;                                   // uniform over the wave
    const int s0 = seg * seg_slots, s1 = min(s0 + seg_slots, n_slots);
    const int n = moe_route_count(topk_ids, s0, s1, e, n_experts, lane);
    if (lane == 0) cnt[seg * (n_experts + 1) + e] = n;
}

__global__ void __launch_bounds__(256)
moe_route_place_kernel(const int64_t *__restrict__ topk_ids, int n_slots, int n_experts, int seg_slots, int n_seg,
                       const int *__restrict__ cnt, int *__restrict__ perm, int *__restrict__ pexp,
                       int *__restrict__ offs) {
    const int e = blockIdx.x * 4 + (threadIdx.x >> 6), lane = threadIdx.x & 63, seg = blockIdx.y;
    if (e > n_experts) return;                                   // uniform over the wave
    // slots of the experts below e in every segment, and of e itself in the segments before this one
    int below = 0;
    const int stride = n_experts + 1;
    for (int idx = lane; idx < n_seg * stride; idx += 64) {
        const int sg = idx / stride, ex = idx - sg * stride;
        if (ex < n_experts && (ex < e || (ex == e && sg < seg))) below += cnt[idx];
    }
#pragma unroll
    for (int d = 32; d >= 1; d >>= 1) below += __shfl_xor(below, d, 64);
    if (seg == 0 && lane == 0) offs[e] = below;                  // e = n_experts: the total
    if (e == n_experts) return;
    const int s0 = seg * seg_slots, s1 = min(s0 + seg_slots, n_slots);
    int mine = 0;
    constexpr int U = 8;
    for (int base = s0; base < s1; base += 64 * U) {
        int64_t id[U];
#pragma unroll
        for (int u = 0; u < U; ++u) id[u] = base + 64 * u + lane < s1 ? topk_ids[base + 64 * u + lane] : -1;
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const unsigned long long hit = __ballot(id[u] == e);
            if (id[u] == e) {
                const int at = below + mine + __builtin_popcountll(hit & ((1ull << lane) - 1ull));
                perm[at] = base + 64 * u + lane;
                pexp[at] = e;
            }
            mine += __builtin_popcountll(hit);
        }
    }
}

int moe_check_blocks(const int64_t *blocks_m, int64_t n_blocks_m, int64_t m_pad, glqh_meta_args *margs,
                     int64_t *max_bs) {
    GLQH_REQUIRE(glqh_fill_meta_args(margs, n_blocks_m > 1 ? blocks_m : nullptr, n_blocks_m > 1 ? n_blocks_m : 1,
                                     m_pad) && margs->canon == m_pad,
                 "routed experts: output block sizes must be the descending power-of-two decomposition of m_pad");
    *max_bs = (int64_t)1 << (63 - __builtin_clzll((unsigned long long)m_pad));
    GLQH_REQUIRE(*max_bs <= (1 << WIDE_LOG_MAX) && (m_pad & 7) == 0,
                 "routed experts: output blocks of 8..8192 rows, got m_pad %lld", (long long)m_pad);
    return 0;
}
}  // namespace

int glqh_launch_moe_output_rht(const float *part, int ks, int part_f16, int n_slots, int n_experts, const int64_t *topk_ids,
                               const void *su_base, const float *wscale_dev, int64_t out_features, int64_t m_pad,
                               const int64_t *blocks_m, int64_t n_blocks_m, void *h_f16, int64_t h_stride,
                               hipStream_t stream) {
    glqh_range range("output_rht");
    glqh_meta_args margs;
    int64_t max_bs;
    if (moe_check_blocks(blocks_m, n_blocks_m, m_pad, &margs, &max_bs)) return 1;
    GLQH_REQUIRE(aligned16(part) && aligned16(su_base) && aligned16(h_f16) && (h_stride & 7) == 0,
                 "routed experts: unaligned rows");
    const moe_out_args a = {part, ks, part_f16, n_slots, n_experts, topk_ids, (const f16 *)su_base, wscale_dev,
                            (int)out_features, (int)m_pad};
    const int nb = __builtin_popcountll((unsigned long long)m_pad);
    if (n_slots >= MOE_OUT_WIDE_MIN)
        hipLaunchKernelGGL(moe_output_rht_wide_kernel, dim3((unsigned)(64 * ((n_slots + 63) / 64) * nb)), dim3(REG_THREADS),
                           rht_reg_lds_bytes(ilog2(max_bs)), stream, a, (f16 *)h_f16, h_stride, nb, margs);
    else
        hipLaunchKernelGGL(moe_output_rht_kernel, dim3((unsigned)nb, (unsigned)n_slots), dim3(REG_THREADS),
                           rht_reg_lds_bytes(ilog2(max_bs)), stream, a, (f16 *)h_f16, h_stride, margs);
    GLQH_LAUNCH_CHECK("routed-expert output_rht launch");
    return 0;
}

int glqh_launch_moe_gated_act(const void *h_f16, int64_t h_stride, void *out_f16, int n_slots, int64_t intermediate,
                              int act, hipStream_t stream) {
    GLQH_REQUIRE(act >= 0 && act <= 2, "routed experts: gated activations 0 (silu), 1 (gelu-tanh), 2 (relu2), got %d", act);
    const int64_t total = (int64_t)n_slots * intermediate;
    // (eight elements per thread only where there are many: a few slots finish sooner spread over more threads)
    if (n_slots >= 1024 && intermediate % 8 == 0 && h_stride % 8 == 0 && aligned16(h_f16) && aligned16(out_f16))
        hipLaunchKernelGGL(moe_gated_act_kernel<8>, dim3((unsigned)((total / 8 + 255) / 256)), dim3(256), 0, stream,
                           (const f16 *)h_f16, h_stride, (f16 *)out_f16, n_slots, (int)intermediate, act);
    else
        hipLaunchKernelGGL(moe_gated_act_kernel<1>, dim3((unsigned)((total + 255) / 256)), dim3(256), 0, stream,
                           (const f16 *)h_f16, h_stride, (f16 *)out_f16, n_slots, (int)intermediate, act);
    GLQH_LAUNCH_CHECK("routed-expert activation launch");
    return 0;
}

// 1 when the launch below serves these shapes: canonical blocks of at most 8192 points on both sides, the
// second projection's a multiple of 32 columns
int glqh_moe_mid_eligible(int64_t m_pad13, const int64_t *blocks_m13, int64_t n_blocks_m13, int64_t n_pad2,
                          const int64_t *blocks_n2, int64_t n_blocks_n2) {
    glqh_meta_args m13, m2;
    if (!glqh_fill_meta_args(&m13, n_blocks_m13 > 1 ? blocks_m13 : nullptr, n_blocks_m13 > 1 ? n_blocks_m13 : 1, m_pad13) ||
        m13.canon != m_pad13)
        return 0;
    if (!glqh_fill_meta_args(&m2, n_blocks_n2 > 1 ? blocks_n2 : nullptr, n_blocks_n2 > 1 ? n_blocks_n2 : 1, n_pad2) ||
        m2.canon != n_pad2)
        return 0;
    const int64_t b13 = (int64_t)1 << (63 - __builtin_clzll((unsigned long long)m_pad13));
    const int64_t b2 = (int64_t)1 << (63 - __builtin_clzll((unsigned long long)n_pad2));
    return b13 <= (1 << WIDE_LOG_MAX) && b2 <= (1 << WIDE_LOG_MAX) && (m_pad13 & 7) == 0 && (n_pad2 & 31) == 0;
}

// sums of the first projection -> transformed activations of the second (layout 0: rows by slot; 2: the tile
// kernel's blocked operand by sorted position, Mp positions), for the slots listed in perm[0 .. *n_valid)
int glqh_launch_moe_mid(const float *part, int ks, int part_f16, int n_slots, int n_experts, const int64_t *topk_ids,
                        const void *su_base, const float *wscale_dev, int64_t out_features13, int64_t m_pad13,
                        const int64_t *blocks_m13, int64_t n_blocks_m13, const int *perm, const int *pexp, const int *n_valid,
                        int64_t intermediate, int act, const void *sv2, int64_t n_pad2, const int64_t *blocks_n2,
                        int64_t n_blocks_n2, void *out_f16, int layout, int64_t Mp, hipStream_t stream) {
    glqh_range range("output_rht");
    GLQH_REQUIRE(glqh_moe_mid_eligible(m_pad13, blocks_m13, n_blocks_m13, n_pad2, blocks_n2, n_blocks_n2),
                 "routed experts: block sizes not served by the fused middle launch");
    GLQH_REQUIRE(act >= 0 && act <= 2, "routed experts: gated activations 0 (silu), 1 (gelu-tanh), 2 (relu2), got %d", act);
    GLQH_REQUIRE(aligned16(part) && aligned16(su_base) && aligned16(sv2) && aligned16(out_f16), "routed experts: unaligned rows");
    glqh_meta_args m13, m2;
    glqh_fill_meta_args(&m13, n_blocks_m13 > 1 ? blocks_m13 : nullptr, n_blocks_m13 > 1 ? n_blocks_m13 : 1, m_pad13);
    glqh_fill_meta_args(&m2, n_blocks_n2 > 1 ? blocks_n2 : nullptr, n_blocks_n2 > 1 ? n_blocks_n2 : 1, n_pad2);
    const int64_t b13 = (int64_t)1 << (63 - __builtin_clzll((unsigned long long)m_pad13));
    const int64_t b2 = (int64_t)1 << (63 - __builtin_clzll((unsigned long long)n_pad2));
    const int64_t max_bs = b13 > b2 ? b13 : b2;
    // sixteen elements per thread on the largest block, eight on the others (each at most half of it): a row of
    // 1024 + 512 points is one wave's work, with no exchange between waves
    int threads = 64;
    while (threads < REG_THREADS && 16 * threads < max_bs) threads <<= 1;
    const size_t s_bytes = (rht_reg_lds_bytes(ilog2(max_bs)) + 15) & ~(size_t)15;
    const size_t lds = s_bytes + (size_t)(m_pad13 + n_pad2) * sizeof(f16);
    moe_mid_args a = {};
    a.o = {part, ks, part_f16, n_slots, n_experts, topk_ids, (const f16 *)su_base, wscale_dev, (int)out_features13,
           (int)m_pad13};
    a.sv2 = (const f16 *)sv2;
    a.perm = perm;
    a.pexp = pexp;
    a.n_valid = n_valid;
    a.intermediate = (int)intermediate;
    a.act = act;
    a.n_pad2 = (int)n_pad2;
    a.Mp = (int)Mp;
    a.nb13 = __builtin_popcountll((unsigned long long)m_pad13);
    a.nb2 = __builtin_popcountll((unsigned long long)n_pad2);
    a.s_floats = (int)(s_bytes / sizeof(float));
    const dim3 grid((unsigned)(64 * ((n_slots + 63) / 64)));
    if (layout == 2)
        hipLaunchKernelGGL(moe_mid_kernel<2>, grid, dim3((unsigned)threads), lds, stream, a, (f16 *)out_f16, m13, m2);
    else
        hipLaunchKernelGGL(moe_mid_kernel<0>, grid, dim3((unsigned)threads), lds, stream, a, (f16 *)out_f16, m13, m2);
    GLQH_LAUNCH_CHECK("routed-expert middle launch");
    return 0;
}

// out[token] = sum over the token's choices of w * (second projection's output row of the slot), many tokens
int glqh_launch_moe_final(const float *part, int ks, int part_f16, int num_tokens, int top_k, int n_experts,
                          const int64_t *topk_ids, const float *topk_w, const void *su_base, const float *wscale_dev,
                          int64_t out_features, int64_t m_pad, const int64_t *blocks_m, int64_t n_blocks_m, void *out,
                          int out_dtype, int64_t out_stride, hipStream_t stream) {
    glqh_range range("output_rht");
    glqh_meta_args margs;
    int64_t max_bs;
    if (moe_check_blocks(blocks_m, n_blocks_m, m_pad, &margs, &max_bs)) return 1;
    GLQH_REQUIRE(out_dtype == GLQH_F16 || out_dtype == GLQH_BF16, "routed experts: output must be f16 or bf16");
    GLQH_REQUIRE(aligned16(part) && aligned16(su_base) && aligned16(out) && (out_stride & 7) == 0,
                 "routed experts: unaligned rows");
    const moe_out_args a = {part, ks, part_f16, num_tokens * top_k, n_experts, topk_ids, (const f16 *)su_base, wscale_dev,
                            (int)out_features, (int)m_pad};
    const int nb = __builtin_popcountll((unsigned long long)m_pad);
    const dim3 grid((unsigned)(64 * ((num_tokens + 63) / 64) * nb));
    const size_t lds = rht_reg_lds_bytes(ilog2(max_bs));
    // rows without small blocks (which take several tokens per workgroup of 512 threads): as many threads as the
    // largest block has groups of eight elements
    // (sixteen elements per thread on half as many threads: slower, the whole call of 32768 slots x 2048 rows 701 -> 714 us
    // -- the registers of two choices in flight cost occupancy)
    int threads = REG_THREADS;
    if ((m_pad & 1023) == 0 && max_bs <= 2048) threads = (int)(max_bs / 8);
#define GLQH_MOE_FINAL(YT, BIG)                                                                                  \
    hipLaunchKernelGGL((moe_final_kernel<YT, BIG>), grid, dim3((unsigned)threads), lds, stream, a, topk_w, top_k, num_tokens, \
                       (YT *)out, out_stride, nb, margs)
    const bool big = max_bs > 8 * threads;
    if (out_dtype == GLQH_F16) { if (big) GLQH_MOE_FINAL(f16, true); else GLQH_MOE_FINAL(f16, false); }
    else { if (big) GLQH_MOE_FINAL(uint16_t, true); else GLQH_MOE_FINAL(uint16_t, false); }
#undef GLQH_MOE_FINAL
    GLQH_LAUNCH_CHECK("routed-expert final launch");
    return 0;
}

// segments of the two-launch form (1: the single launch), and the ints of scratch it needs
int glqh_moe_route_segments(int n_slots, int n_experts) {
    if (n_slots < 2 * MOE_ROUTE_SEG_SLOTS || n_experts > 4096) return 1;
    const int n = (n_slots + MOE_ROUTE_SEG_SLOTS - 1) / MOE_ROUTE_SEG_SLOTS;
    return n < MOE_ROUTE_MAX_SEG ? n : MOE_ROUTE_MAX_SEG;
}

size_t glqh_moe_route_scratch_ints(int n_slots, int n_experts) {
    const int n = glqh_moe_route_segments(n_slots, n_experts);
    return n > 1 ? (size_t)n * (n_experts + 1) : 0;
}

// perm / pexp: slot and expert of every position of the expert-sorted order, offs: first position per expert
int glqh_launch_moe_route(const int64_t *topk_ids, int n_slots, int n_experts, int *perm, int *pexp, int *offs,
                          int *scratch, hipStream_t stream) {
    const int n_seg = glqh_moe_route_segments(n_slots, n_experts);
    const unsigned wgs = (unsigned)((n_experts + 1 + 3) / 4);
    if (n_seg == 1) {
        hipLaunchKernelGGL(moe_route_kernel, dim3(wgs), dim3(256), 0, stream, topk_ids, n_slots, n_experts, perm, pexp, offs);
    } else {
        const int seg_slots = ((n_slots + n_seg - 1) / n_seg + 63) & ~63;
        hipLaunchKernelGGL(moe_route_count_kernel, dim3(wgs, (unsigned)n_seg), dim3(256), 0, stream, topk_ids, n_slots,
                           n_experts, seg_slots, scratch);
        hipLaunchKernelGGL(moe_route_place_kernel, dim3(wgs, (unsigned)n_seg), dim3(256), 0, stream, topk_ids, n_slots,
                           n_experts, seg_slots, n_seg, scratch, perm, pexp, offs);
    }
    GLQH_LAUNCH_CHECK("routed-expert routing launch");
    return 0;
}

int glqh_launch_moe_weighted_sum(const void *y_f16, int64_t y_stride, int num_tokens, int top_k, int n_experts,
                                 const int64_t *topk_ids, const float *topk_w, int64_t out_features, void *out,
                                 int out_dtype, int64_t out_stride, hipStream_t stream) {
    GLQH_REQUIRE(out_dtype == GLQH_F16 || out_dtype == GLQH_BF16, "routed experts: output must be f16 or bf16");
    GLQH_REQUIRE(aligned16(y_f16) && aligned16(out) && (out_stride & 7) == 0 && (y_stride & 7) == 0 &&
                     (out_features & 7) == 0,
                 "routed experts: unaligned rows");
    const dim3 grid((unsigned)((out_features / 8 + 255) / 256), (unsigned)num_tokens);
    if (out_dtype == GLQH_F16)
        hipLaunchKernelGGL((moe_weighted_sum_kernel<f16>), grid, dim3(256), 0, stream, (const f16 *)y_f16, y_stride,
                           topk_ids, topk_w, top_k, n_experts, (int)out_features, (f16 *)out, out_stride);
    else
        hipLaunchKernelGGL((moe_weighted_sum_kernel<uint16_t>), grid, dim3(256), 0, stream, (const f16 *)y_f16,
                           y_stride, topk_ids, topk_w, top_k, n_experts, (int)out_features, (uint16_t *)out,
                           out_stride);
    GLQH_LAUNCH_CHECK("routed-expert weighted sum launch");
    return 0;
}

int glqh_launch_output_rht_group(const float *const part[], const void *const su[], void *const y[],
                                 const float scale[], const int64_t m_pad[], const int64_t out_features[],
                                 int n_shards, int y_dtype, int64_t y_stride, int64_t B, int ksplit,
                                 hipStream_t stream) {
    glqh_range range("output_rht");
    GLQH_REQUIRE(n_shards >= 1 && n_shards <= GLQH_MAX_GROUP, "output_rht group: 1..%d shards", GLQH_MAX_GROUP);
    GLQH_REQUIRE(B >= 1 && B <= 65535, "output_rht group: B=%lld out of range", (long long)B);
    GLQH_REQUIRE(y_dtype == GLQH_F16 || y_dtype == GLQH_BF16 || y_dtype == GLQH_F32, "output_rht group: bad y dtype");
    const int log_slice = rht_log_slice(B);
    rht_out_group g = {};
    int64_t max_bs = 1;
    int max_nwg = 0;
    for (int i = 0; i < n_shards; ++i) {                       // largest block = top bit of m_pad
        int64_t top = 1;
        while (top * 2 <= m_pad[i]) top *= 2;
        if (top > max_bs) max_bs = top;
    }
    const int spb = rht_slices_per_block(max_bs, log_slice);
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        const int j = i < n_shards ? i : 0;
        GLQH_REQUIRE(part[j] && su[j] && y[j] && m_pad[j] >= 1 && m_pad[j] <= 0x40000000ll &&
                         out_features[j] >= 1 && out_features[j] <= m_pad[j],
                     "output_rht group: bad shard %d", j);
        g.part[i] = part[j];
        g.su[i] = (const f16 *)su[j];
        g.y[i] = y[j];
        g.scale[i] = scale[j];
        g.m_pad[i] = (int)m_pad[j];
        g.out_features[i] = (int)out_features[j];
        g.nwg[i] = __builtin_popcountll((unsigned long long)m_pad[j]) * spb;
        if (g.nwg[i] > max_nwg) max_nwg = g.nwg[i];
    }
    // blocks of at most four slices: one workgroup per block (see output_rht_block_kernel); larger
    // blocks are faster as one workgroup per slice (measured with eight slices on 1024 threads)
    bool aligned = spb <= 4 && log_slice == LOG_SLICE;
    int max_blocks = 0;
    for (int i = 0; i < n_shards && aligned; ++i) {
        aligned = (m_pad[i] & 3) == 0 && ((uintptr_t)part[i] & 15) == 0;
        const int nb = __builtin_popcountll((unsigned long long)m_pad[i]);
        if (nb > max_blocks) max_blocks = nb;
    }
    if (aligned) {
        const int G = spb <= 1 ? 1 : spb <= 2 ? 2 : 4;
        dim3 bgrid((unsigned)max_blocks, (unsigned)B, (unsigned)n_shards);
        const size_t blds = ((size_t)2 * G << log_slice) * sizeof(float);
#define GLQH_BLK(YT)                                                                                          \
    do {                                                                                                      \
        if (G == 1) hipLaunchKernelGGL((output_rht_block_kernel<YT, 1, 4>), bgrid, dim3(256), blds, stream,   \
                                       g, y_stride, (int)B, ksplit, log_slice);                               \
        else if (G == 2) hipLaunchKernelGGL((output_rht_block_kernel<YT, 2, 4>), bgrid, dim3(512), blds,      \
                                            stream, g, y_stride, (int)B, ksplit, log_slice);                  \
        else hipLaunchKernelGGL((output_rht_block_kernel<YT, 4, 4>), bgrid, dim3(1024), blds, stream, g,      \
                                y_stride, (int)B, ksplit, log_slice);                                         \
    } while (0)
        if (y_dtype == GLQH_F16) GLQH_BLK(f16);
        else if (y_dtype == GLQH_BF16) GLQH_BLK(uint16_t);
        else GLQH_BLK(float);
#undef GLQH_BLK
        GLQH_LAUNCH_CHECK("output_rht block launch");
        return 0;
    }
    dim3 grid((unsigned)max_nwg, (unsigned)B, (unsigned)n_shards);
    const size_t lds = rht_lds_bytes(log_slice);
    if (y_dtype == GLQH_F16)
        hipLaunchKernelGGL(output_rht_group_kernel<f16>, grid, dim3(RHT_THREADS), lds, stream, g, y_stride, (int)B, ksplit, spb, log_slice);
    else if (y_dtype == GLQH_BF16)
        hipLaunchKernelGGL(output_rht_group_kernel<uint16_t>, grid, dim3(RHT_THREADS), lds, stream, g, y_stride, (int)B, ksplit, spb, log_slice);
    else
        hipLaunchKernelGGL(output_rht_group_kernel<float>, grid, dim3(RHT_THREADS), lds, stream, g, y_stride, (int)B, ksplit, spb, log_slice);
    GLQH_LAUNCH_CHECK("output_rht group launch");
    return 0;
}
