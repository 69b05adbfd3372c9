// Device-side Walsh-Hadamard transform of a block staged in LDS, shared by the RHT
// kernels and by the fused input transform of the trellis GEMV.
#pragma once

#include "common.h"

// ---------------------------------------------------------------------------------
// The log2(n) index bits are split into fields of at most RMAX bits, taken from the top
// bit down.  In one pass a thread owns groups of 2^r elements that differ only in the
// field's bits, runs the field's r butterfly stages (lo, hi) <- (a + b, a - b) in
// registers and puts the group back; the last pass hands the elements to `store`.  The
// block lives in LDS with one pad word per 32 so that the strided accesses of the low
// fields stay conflict-free.  The stages of different bits commute, so the result is the
// Walsh-Hadamard transform of the block (summation order differs from the
// ascending-distance order of glq/hadamard.py:10-28 by fp32 rounding only).
//
// Blocks larger than a slice (a launch parameter) are not transformed whole: H_bs factors as
// H_(bs/len) (x) H_len, so slice r of the output is
//     H_len( sum_h (-1)^popcount(r & h) * in[h*len + i] ),
// one pass over the block's inputs followed by a short transform -- which lets every slice
// go to its own workgroup.
//
// `store` is an object with aux(i) -> float (a per-element factor that may come from
// memory; all of a group's factors are requested before the butterflies) and
// put(i, value, factor).  RMAX is kept small on purpose: a pass is straight-line code that
// runs once per launch, and instruction fetch of a 32-point pass costs more than the extra
// barrier of two 8-point passes.
// ---------------------------------------------------------------------------------
#ifndef GLQH_RMAX
#define GLQH_RMAX 4
#endif
#ifndef GLQH_LOG_SLICE
#define GLQH_LOG_SLICE 10
#endif
constexpr int RMAX = GLQH_RMAX;
constexpr int LOG_SLICE = GLQH_LOG_SLICE;

__device__ __forceinline__ int lds_pad(int i) { return i + (i >> 5); }

// Workgroup barrier for exchanges through LDS: waits for this wave's LDS operations only.
// __syncthreads() also drains the wave's global loads, which stalls a transform that runs
// while a long-latency request of its caller is in flight.
template <bool LDS_ONLY>
__device__ __forceinline__ void fht_barrier() {
    if constexpr (LDS_ONLY) asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    else __syncthreads();
}

template <int R, bool LAST, class Store>
__device__ __forceinline__ void fht_pass(float *lds, int n, int s, Store &store, int tid, int nthr) {
    constexpr int N = 1 << R;
    const int ngroups = n >> R;
    for (int g = tid; g < ngroups; g += nthr) {
        const int lo = g & ((1 << s) - 1);
        const int base = ((g >> s) << (s + R)) | lo;
        float v[N], aux[N];
#pragma unroll
        for (int j = 0; j < N; ++j) {
            const int idx = base + (j << s);
            v[j] = lds[lds_pad(idx)];
            if constexpr (LAST) aux[j] = store.aux(idx);
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
            if constexpr (LAST) store.put(idx, v[j], aux[j]);
            else lds[lds_pad(idx)] = v[j];
        }
    }
}

template <bool LAST, class Store>
__device__ __forceinline__ void fht_pass_r(int r, float *lds, int n, int s, Store &store, int tid, int nthr) {
    switch (r) {
    case 1: fht_pass<1, LAST>(lds, n, s, store, tid, nthr); break;
    case 2: fht_pass<2, LAST>(lds, n, s, store, tid, nthr); break;
    case 3: fht_pass<3, LAST>(lds, n, s, store, tid, nthr); break;
#if GLQH_RMAX >= 5
    case 4: fht_pass<4, LAST>(lds, n, s, store, tid, nthr); break;
    default: fht_pass<5, LAST>(lds, n, s, store, tid, nthr); break;
#else
    default: fht_pass<4, LAST>(lds, n, s, store, tid, nthr); break;
#endif
    }
}

// Transform lds[0 .. 2^log_n) (padded layout, already staged and visible to the whole
// workgroup) and pass the result to `store`.  All threads of the workgroup must call it.
// A workgroup may run several transforms of the same size side by side: each group of nthr
// threads (numbered tid = 0..nthr-1) passes its own buffer; the barriers are shared.
template <bool LDS_ONLY = false, class Store>
__device__ __forceinline__ void fht_staged(float *lds, int log_n, Store store, int tid = threadIdx.x,
                                           int nthr = blockDim.x) {
    const int n = 1 << log_n;
    if (log_n == 0) {
        if (tid == 0) store.put(0, lds[0], store.aux(0));
        return;
    }
    const int npass = (log_n + RMAX - 1) / RMAX;
    int s = log_n;
    for (int p = 0; p < npass; ++p) {
        const int left = npass - p;
        const int r = (s + left - 1) / left;              // balanced field widths
        s -= r;
        if (p == npass - 1) fht_pass_r<true>(r, lds, n, s, store, tid, nthr);
        else {
            fht_pass_r<false>(r, lds, n, s, store, tid, nthr);
            fht_barrier<LDS_ONLY>();
        }
    }
}

struct lds_writeback {                                   // last pass: results stay in LDS
    float *lds;
    __device__ float aux(int) const { return 0.0f; }
    __device__ void put(int i, float v, float) const { lds[lds_pad(i)] = v; }
};

// ---------------------------------------------------------------------------------
// Register form of short transforms.  The LDS passes above cost a few hundred instructions
// per thread, and in the one-token kernels a wave has its SIMD to itself, so every one of
// them is paid in full (4+ cycles each, nothing to overlap with).  Here thread tid holds E
// consecutive elements, E*tid .. E*tid+E-1, of a 2^log_n-point vector in registers:
// log2(E) butterfly levels stay inside the thread, up to six run across the lanes of the
// wave (DPP quad permutes, ds_swizzle, ds_bpermute: no LDS storage, no barrier), and up to
// log2(E) more, across waves, take one exchange through LDS.  log2(E) <= log_n <=
// 6 + 2*log2(E); threads tid >= n/E carry don't-care values but must make the call.
//
// After the call the thread holds elements fht_wave_index<E>(log_n, tid, q), q = 0..E-1.
// The exchange contains the call's only __syncthreads(); with ALWAYS_SYNC the shorter
// transforms pass one too, so that thread groups of one workgroup may run transforms of
// different sizes side by side (each with its own tid numbering and exchange buffer).
// ---------------------------------------------------------------------------------
template <int E> struct fht_wave_log { };
template <> struct fht_wave_log<4> { static constexpr int v = 2; };
template <> struct fht_wave_log<8> { static constexpr int v = 3; };
template <> struct fht_wave_log<16> { static constexpr int v = 4; };

template <int E>
__device__ __forceinline__ constexpr int fht_wave_max_log() { return 6 + 2 * fht_wave_log<E>::v; }

template <int E>
__device__ __forceinline__ int fht_wave_index(int log_n, int tid, int q) {
    constexpr int LE = fht_wave_log<E>::v;
    return log_n > LE + 6 ? tid + (q << (log_n - LE)) : tid * E + q;
}

// value of the lane whose number differs in bit K
template <int K>
__device__ __forceinline__ float fht_lane_partner(float v, int swap32_addr) {
    const int b = __builtin_bit_cast(int, v);
    int o;
    if constexpr (K == 0) o = __builtin_amdgcn_mov_dpp(b, 0xB1, 0xF, 0xF, true);        // quad_perm [1,0,3,2]
    else if constexpr (K == 1) o = __builtin_amdgcn_mov_dpp(b, 0x4E, 0xF, 0xF, true);   // quad_perm [2,3,0,1]
    else if constexpr (K < 5) o = __builtin_amdgcn_ds_swizzle(b, ((1 << K) << 10) | 0x1F);  // xor mask, 32-lane groups
    else o = __builtin_amdgcn_ds_bpermute(swap32_addr, b);
    return __builtin_bit_cast(float, o);
}

template <int K, int E>
__device__ __forceinline__ void fht_lane_level(float (&v)[E], int lane, int swap32_addr) {
    const float sgn = ((lane >> K) & 1) ? -1.0f : 1.0f;      // upper element of the pair: partner - own
    float o[E];
#pragma unroll
    for (int j = 0; j < E; ++j) o[j] = fht_lane_partner<K>(v[j], swap32_addr);
#pragma unroll
    for (int j = 0; j < E; ++j) v[j] = __builtin_fmaf(v[j], sgn, o[j]);   // exact: one rounding, like the add
}

template <int E, bool ALWAYS_SYNC = false, bool LDS_ONLY = false>
__device__ __forceinline__ void fht_wave(float (&v)[E], int log_n, float *xchg, int tid) {
    constexpr int LE = fht_wave_log<E>::v;
#pragma unroll
    for (int h = 1; h < E; h <<= 1) {
#pragma unroll
        for (int j = 0; j < E; ++j) {
            if ((j & h) == 0) {
                const float a = v[j], b = v[j | h];
                v[j] = a + b;
                v[j | h] = a - b;
            }
        }
    }
    const int lane = tid & 63;
    const int lane_bits = min(log_n - LE, 6);                // uniform
    const int swap32_addr = (lane ^ 32) << 2;
    if (lane_bits > 0) fht_lane_level<0>(v, lane, swap32_addr);
    if (lane_bits > 1) fht_lane_level<1>(v, lane, swap32_addr);
    if (lane_bits > 2) fht_lane_level<2>(v, lane, swap32_addr);
    if (lane_bits > 3) fht_lane_level<3>(v, lane, swap32_addr);
    if (lane_bits > 4) fht_lane_level<4>(v, lane, swap32_addr);
    if (lane_bits > 5) fht_lane_level<5>(v, lane, swap32_addr);
    if (log_n <= LE + 6) {
        if constexpr (ALWAYS_SYNC) fht_barrier<LDS_ONLY>();   // the barrier the longer transforms take
        return;
    }
    // levels LE+6 .. log_n-1 pair elements held by different waves: through LDS once, after
    // which thread u holds elements u + q * (n / E) and the open levels are the top bits of q
    const int wave_bits = log_n - LE - 6;                     // 1 .. LE
    const int nthr = 1 << (log_n - LE);
    if (tid < nthr) {
#pragma unroll
        for (int j = 0; j < E; j += 4)
            *(f32x4 *)(xchg + E * tid + j) = f32x4{v[j], v[j + 1], v[j + 2], v[j + 3]};
    }
    fht_barrier<LDS_ONLY>();
    if (tid < nthr) {
#pragma unroll
        for (int q = 0; q < E; ++q) v[q] = xchg[tid + q * nthr];
    }
#pragma unroll
    for (int c = 0; c < LE; ++c) {
        if (c >= LE - wave_bits) {                            // uniform
            const int h = 1 << c;
#pragma unroll
            for (int j = 0; j < E; ++j) {
                if ((j & h) == 0) {
                    const float a = v[j], b = v[j | h];
                    v[j] = a + b;
                    v[j | h] = a - b;
                }
            }
        }
    }
}

// sign of element (r, h) of the Sylvester matrix
__device__ __forceinline__ float had_sign(int r, int h, float v) {
    return (__builtin_popcount(r & h) & 1) ? -v : v;
}

// lds[pad(i)] = sum_h sign(r, h) * val(h, i) for i < 2^log_len: slice r of the first
// factor of H_(nsub*len).  Loads of C terms x U elements are issued before any of them is
// used; indices are clamped instead of branched on so that the loads cluster (callers pick
// U <= len / T and C <= nsub where they can, clamped loads are wasted issue slots).  Ends
// with a barrier.
template <int T, int U = 4, int C = 8, class Val>
__device__ __forceinline__ void stage_signed_slices(float *lds, int log_len, int nsub, int r, Val val) {
    const int len = 1 << log_len;
    for (int i0 = threadIdx.x; i0 < len; i0 += U * T) {
        float z[U];
#pragma unroll
        for (int u = 0; u < U; ++u) z[u] = 0.0f;
        for (int h0 = 0; h0 < nsub; h0 += C) {
            float vals[C][U];
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int u = 0; u < U; ++u)
                    vals[c][u] = val(min(h0 + c, nsub - 1), min(i0 + u * T, len - 1));
#pragma unroll
            for (int c = 0; c < C; ++c)
#pragma unroll
                for (int u = 0; u < U; ++u)
                    z[u] += (h0 + c < nsub) ? had_sign(r, h0 + c, vals[c][u]) : 0.0f;
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (i0 + u * T < len) lds[lds_pad(i0 + u * T)] = z[u];
    }
    __syncthreads();
}

// The same staging for the input transform when the activations are 16-bit and the block lies
// wholly inside the row: lds[pad(i)] = sum_h sign(r, h) * x[h*len + i] * sv[h*len + i], in the
// same order and with the same roundings as the element-wise form above, but a thread owns
// four consecutive elements and reads them with one 8-byte load per operand (the prologue of
// the fused-input GEMV is bound by instruction issue, not by latency).  xb / svb point at the
// block's first element and must be 8-byte aligned; len >= 4.  Ends with a barrier.
template <typename XT> __device__ __forceinline__ void unpack_quad(uint2 w, float *f);
template <> __device__ __forceinline__ void unpack_quad<f16>(uint2 w, float *f) {
    const f16x2 a = __builtin_bit_cast(f16x2, w.x), b = __builtin_bit_cast(f16x2, w.y);
    f[0] = (float)a[0]; f[1] = (float)a[1]; f[2] = (float)b[0]; f[3] = (float)b[1];
}
template <> __device__ __forceinline__ void unpack_quad<uint16_t>(uint2 w, float *f) {   // bf16
    f[0] = __builtin_bit_cast(float, w.x << 16); f[1] = __builtin_bit_cast(float, w.x & 0xffff0000u);
    f[2] = __builtin_bit_cast(float, w.y << 16); f[3] = __builtin_bit_cast(float, w.y & 0xffff0000u);
}

// elements i0 .. i0+3 of that vector into registers (i0 a multiple of 4, i0 + 3 < len);
// `issued` runs once, right after the first round of loads has been issued and before any of
// them is waited for (a place for the caller's own, longer-latency requests)
struct fht_nothing {
    __device__ void operator()() const {}
};

template <typename XT, int C = 8, class Issued = fht_nothing>
__device__ __forceinline__ void signed_input_quad(float (&z)[4], unsigned i0, int log_len, int nsub, int r,
                                                  const XT *__restrict__ xb, const f16 *__restrict__ svb,
                                                  Issued issued = Issued()) {
#pragma unroll
    for (int e = 0; e < 4; ++e) z[e] = 0.0f;
    for (int h0 = 0; h0 < nsub; h0 += C) {
        uint2 xv[C], sg[C];
#pragma unroll
        for (int c = 0; c < C; ++c) {
            // uniform base + 32-bit lane offset: the load takes its base from scalar registers
            const size_t hb = (size_t)min(h0 + c, nsub - 1) << log_len;
            xv[c] = *(const uint2 *)(xb + hb + i0);
            sg[c] = *(const uint2 *)(svb + hb + i0);
        }
        if (h0 == 0) issued();
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (h0 + c < nsub) {                              // uniform
                float xf[4], sf[4];
                unpack_quad<XT>(xv[c], xf);
                unpack_quad<f16>(sg[c], sf);
                const float sgn = (__builtin_popcount(r & (h0 + c)) & 1) ? -1.0f : 1.0f;
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float v = xf[e] * sf[e];
                    z[e] = __builtin_fmaf(v, sgn, z[e]);      // z +- v, rounded once like the add
                }
            }
        }
    }
}

// signed_input_quad with as many terms in flight as the block has sub-slices, up to eight
// (a clamped repeat of the last term still costs its issue slots)
template <typename XT, class Issued = fht_nothing>
__device__ __forceinline__ void signed_input_quad_n(float (&z)[4], unsigned i0, int log_len, int nsub, int r,
                                                    const XT *__restrict__ xb, const f16 *__restrict__ svb,
                                                    Issued issued = Issued()) {
    if (nsub <= 1) signed_input_quad<XT, 1>(z, i0, log_len, nsub, r, xb, svb, issued);
    else if (nsub <= 2) signed_input_quad<XT, 2>(z, i0, log_len, nsub, r, xb, svb, issued);
    else if (nsub <= 4) signed_input_quad<XT, 4>(z, i0, log_len, nsub, r, xb, svb, issued);
    else signed_input_quad<XT, 8>(z, i0, log_len, nsub, r, xb, svb, issued);
}

template <int T, typename XT, int C = 8, bool LDS_ONLY = false, class Issued = fht_nothing>
__device__ __forceinline__ void stage_signed_input_quads(float *lds, int log_len, int nsub, int r,
                                                         const XT *__restrict__ xb,
                                                         const f16 *__restrict__ svb, Issued issued = Issued()) {
    const unsigned len = 1u << log_len;
    bool pending = true;                                       // waves without elements still run `issued`
    for (unsigned i0 = 4 * threadIdx.x; i0 < len; i0 += 4 * T) {
        float z[4];
        if (pending) signed_input_quad<XT, C>(z, i0, log_len, nsub, r, xb, svb, issued);
        else signed_input_quad<XT, C>(z, i0, log_len, nsub, r, xb, svb);
        pending = false;
#pragma unroll
        for (int e = 0; e < 4; ++e) lds[lds_pad(i0 + e)] = z[e];
    }
    if (pending) issued();
    fht_barrier<LDS_ONLY>();
}

// One workgroup's share of an output transform: the Hadamard block and the slice of it.
struct rht_slice {
    int off, bs, log_bs;     // the Hadamard block
    int log_len, r, nsub;    // this workgroup's slice: len = 2^log_len, index r of nsub
    float norm;
    bool live;
};

// Split-K partials -> LDS.  Element e of the block is v(e) = sum_stage scale * (sum_k
// partial), summed in this fixed order (the same order as the stand-alone reduction, so
// both give the same bits); slice r needs sum_h sign(r,h) v(h*len + i).  The (h, stage, k)
// terms are walked as one flat sequence so that C terms x U elements of loads are in flight.
template <int T, int U, int C>
__device__ __forceinline__ void stage_partials(float *s, const glqh_ysrc &src, const rht_slice &blk,
                                           int64_t b, int m_pad, int tid = threadIdx.x) {
    const int len = 1 << blk.log_len;
    const int ks = src.ksplit, nst = src.nparts;
    const int total = blk.nsub * nst * ks;
    const float *__restrict__ pbase = src.part + b * (int64_t)m_pad + blk.off;
    for (int i0 = tid; i0 < len; i0 += U * T) {
        float z[U], v[U], acc[U];
#pragma unroll
        for (int u = 0; u < U; ++u) z[u] = v[u] = acc[u] = 0.0f;
        int h = 0, st = 0, k = 0;                       // position of term t0 (uniform)
        for (int t0 = 0; t0 < total; t0 += C) {
            float vals[C][U];
            int hh = h, ss = st, kk = k;
#pragma unroll
            for (int c = 0; c < C; ++c) {
                const float *p = pbase + ss * src.part_sstride + kk * src.part_kstride + (hh << blk.log_len);
#pragma unroll
                for (int u = 0; u < U; ++u) vals[c][u] = p[min(i0 + u * T, len - 1)];
                if (t0 + c + 1 < total) {               // advance, clamped at the last term
                    if (++kk == ks) { kk = 0; if (++ss == nst) { ss = 0; ++hh; } }
                }
            }
#pragma unroll
            for (int c = 0; c < C; ++c) {
                if (t0 + c < total) {
#pragma unroll
                    for (int u = 0; u < U; ++u) acc[u] += vals[c][u];
                    if (++k == ks) {
                        const float sc = st == 0 ? src.scale[0] : st == 1 ? src.scale[1]
                                       : st == 2 ? src.scale[2] : src.scale[3];
#pragma unroll
                        for (int u = 0; u < U; ++u) { v[u] += sc * acc[u]; acc[u] = 0.0f; }
                        k = 0;
                        if (++st == nst) {
#pragma unroll
                            for (int u = 0; u < U; ++u) {
                                const int i = i0 + u * T;
                                if (src.copy_out && blk.r == 0 && i < len)
                                    src.copy_out[b * src.copy_stride + blk.off + (h << blk.log_len) + i] = v[u];
                                z[u] += had_sign(blk.r, h, v[u]);
                                v[u] = 0.0f;
                            }
                            st = 0;
                            ++h;
                        }
                    }
                }
            }
        }
#pragma unroll
        for (int u = 0; u < U; ++u)
            if (i0 + u * T < len) s[lds_pad(i0 + u * T)] = z[u];
    }
    __syncthreads();
}

// stage_partials for the register transform: the same sums in the same order, but thread tid
// takes elements E*tid .. E*tid+E-1 of the slice (E = 4 or 8) with E/4 16-byte loads per term
// and keeps them in registers.  The caller has checked log2(E) <= log_len and that every term's
// row is 16-byte aligned.
template <int E, int C>
__device__ __forceinline__ void stage_partials_vec(float (&z)[E], const glqh_ysrc &src, const rht_slice &blk,
                                                   int64_t b, int m_pad, int tid) {
    constexpr int NV = E / 4;
    const int len = 1 << blk.log_len;
    const int ks = src.ksplit, nst = src.nparts;
    const int total = blk.nsub * nst * ks;
    const float *__restrict__ pbase = src.part + b * (int64_t)m_pad + blk.off;
    const bool active = E * tid < len;
    const int i0 = E * tid;
    float v[E], acc[E];
#pragma unroll
    for (int e = 0; e < E; ++e) z[e] = v[e] = acc[e] = 0.0f;
    if (!active) return;                                    // threads without elements issue nothing
    int h = 0, st = 0, k = 0;                               // position of term t0 (uniform)
    for (int t0 = 0; t0 < total; t0 += C) {
        f32x4 vals[C][NV];
        int hh = h, ss = st, kk = k;
#pragma unroll
        for (int c = 0; c < C; ++c) {
            const float *p = pbase + ss * src.part_sstride + kk * src.part_kstride + (hh << blk.log_len);
#pragma unroll
            for (int w = 0; w < NV; ++w) vals[c][w] = *(const f32x4 *)(p + i0 + 4 * w);
            if (t0 + c + 1 < total) {                       // advance, clamped at the last term
                if (++kk == ks) { kk = 0; if (++ss == nst) { ss = 0; ++hh; } }
            }
        }
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (t0 + c < total) {
#pragma unroll
                for (int e = 0; e < E; ++e) acc[e] += vals[c][e >> 2][e & 3];
                if (++k == ks) {
                    const float sc = st == 0 ? src.scale[0] : st == 1 ? src.scale[1]
                                   : st == 2 ? src.scale[2] : src.scale[3];
#pragma unroll
                    for (int e = 0; e < E; ++e) { v[e] += sc * acc[e]; acc[e] = 0.0f; }
                    k = 0;
                    if (++st == nst) {
#pragma unroll
                        for (int e = 0; e < E; ++e) {
                            if (src.copy_out && blk.r == 0)
                                src.copy_out[b * src.copy_stride + blk.off + (h << blk.log_len) + i0 + e] = v[e];
                            z[e] += had_sign(blk.r, h, v[e]);
                            v[e] = 0.0f;
                        }
                        st = 0;
                        ++h;
                    }
                }
            }
        }
    }
}

template <int C>
__device__ __forceinline__ void stage_partials_quad(float (&z)[4], const glqh_ysrc &src, const rht_slice &blk,
                                                    int64_t b, int m_pad, int tid) {
    stage_partials_vec<4, C>(z, src, blk, b, m_pad, tid);
}

// with as many terms in flight as the slice has, up to sixteen (a clamped repeat of the last
// term still costs its issue slots)
__device__ __forceinline__ void stage_partials_quad_n(float (&z)[4], const glqh_ysrc &src, const rht_slice &blk,
                                                      int64_t b, int m_pad, int tid) {
    const int total = blk.nsub * src.nparts * src.ksplit;
    if (total <= 2) stage_partials_vec<4, 2>(z, src, blk, b, m_pad, tid);
    else if (total <= 4) stage_partials_vec<4, 4>(z, src, blk, b, m_pad, tid);
    else if (total <= 8) stage_partials_vec<4, 8>(z, src, blk, b, m_pad, tid);
    else stage_partials_vec<4, 16>(z, src, blk, b, m_pad, tid);
}

// The same for a plain fp32 row: z[e] = sum_h sign(r, h) * d[h * len + 4*tid + e], h ascending
// as in stage_signed_slices.  d must be 16-byte aligned, 2 <= log_len.
template <int C>
__device__ __forceinline__ void stage_signed_row_quad(float (&z)[4], const float *__restrict__ d, int log_len,
                                                      int nsub, int r, int tid) {
    const int len = 1 << log_len;
    const int i0 = 4 * tid;
#pragma unroll
    for (int e = 0; e < 4; ++e) z[e] = 0.0f;
    if (i0 >= len) return;                                   // threads without elements issue nothing
    for (int h0 = 0; h0 < nsub; h0 += C) {
        f32x4 vals[C];
#pragma unroll
        for (int c = 0; c < C; ++c) vals[c] = *(const f32x4 *)(d + ((size_t)min(h0 + c, nsub - 1) << log_len) + i0);
#pragma unroll
        for (int c = 0; c < C; ++c) {
            if (h0 + c < nsub) {
#pragma unroll
                for (int e = 0; e < 4; ++e) z[e] += had_sign(r, h0 + c, vals[c][e]);
            }
        }
    }
}

__device__ __forceinline__ bool stage_partials_quad_ok(const glqh_ysrc &src, const rht_slice &blk, int64_t b,
                                                       int m_pad) {
    const uintptr_t base = (uintptr_t)(src.part + b * (int64_t)m_pad + blk.off);
    return blk.log_len >= 2 && blk.log_len <= fht_wave_max_log<4>() &&
           ((base | (uintptr_t)(src.part_sstride * 4) | (uintptr_t)(src.part_kstride * 4)) & 15) == 0;
}

// One slice of an output transform, from split-K partial sums to transform values in
// registers: thread tid (active when it returns true) ends up with value z[q] of slice
// element idx[q].  Requires stage_partials_quad_ok().
template <bool ALWAYS_SYNC = false>
__device__ __forceinline__ bool partials_fht_quad(float (&z)[4], int (&idx)[4], const glqh_ysrc &src,
                                                  const rht_slice &blk, int64_t b, int m_pad, float *xchg,
                                                  int tid) {
    const bool active = 4 * tid < (1 << blk.log_len);
#pragma unroll
    for (int q = 0; q < 4; ++q) idx[q] = fht_wave_index<4>(blk.log_len, active ? tid : 0, q);
    stage_partials_quad_n(z, src, blk, b, m_pad, tid);
    fht_wave<4, ALWAYS_SYNC>(z, blk.log_len, xchg, tid);
    return active;
}

template <typename T> __device__ __forceinline__ float act_to_f32(T v);
template <> __device__ __forceinline__ float act_to_f32<f16>(f16 v) { return (float)v; }
template <> __device__ __forceinline__ float act_to_f32<uint16_t>(uint16_t v) { return bf16_bits_to_f32(v); }
template <> __device__ __forceinline__ float act_to_f32<float>(float v) { return v; }
template <typename T> __device__ __forceinline__ T f32_to_act(float v);
template <> __device__ __forceinline__ f16 f32_to_act<f16>(float v) { return (f16)v; }
template <> __device__ __forceinline__ uint16_t f32_to_act<uint16_t>(float v) { return f32_to_bf16_bits(v); }
template <> __device__ __forceinline__ float f32_to_act<float>(float v) { return v; }

// 1/sqrt(2^L) exactly rounded: a power of two, times 1/sqrt(2) when L is odd.
__device__ __forceinline__ float rsqrt_pow2(int log_bs) {
    return ldexpf((log_bs & 1) ? 0.70710678118654752f : 1.0f, -(log_bs >> 1));
}

// blockIdx.x = block * spb + slice; workgroups past a block's slice count retire.
// whole canonical block j as one slice
__device__ __forceinline__ rht_slice rht_slice_of(const glqh_meta_args margs, float single_norm, int j) {
    const glqh_block_meta mrow = glqh_meta_row(margs, nullptr, j);
    rht_slice b;
    b.off = mrow.offset;
    b.bs = mrow.bs;
    b.log_bs = b.log_len = mrow.log_bs;
    b.nsub = 1;
    b.r = 0;
    b.live = true;
    if ((margs.canon & (margs.canon - 1)) == 0 && margs.canon != 0 && single_norm != 0.0f) b.norm = single_norm;
    else b.norm = rsqrt_pow2(mrow.log_bs);
    return b;
}

__device__ __forceinline__ rht_slice rht_get_slice(const glqh_block_meta *meta, const glqh_meta_args margs,
                                                   float single_norm, int spb, int log_slice) {
    const int j = blockIdx.x / spb;
    glqh_block_meta mrow = glqh_meta_row(margs, meta, j);
    rht_slice b;
    b.off = mrow.offset;
    b.bs = mrow.bs;
    b.log_bs = mrow.log_bs;
    b.log_len = min(mrow.log_bs, log_slice);
    b.nsub = mrow.bs >> b.log_len;
    b.r = blockIdx.x % spb;
    b.live = b.r < b.nsub;
    if (mrow.w != 0) b.norm = __builtin_bit_cast(float, mrow.w);
    else if ((margs.canon & (margs.canon - 1)) == 0 && margs.canon != 0 && single_norm != 0.0f) b.norm = single_norm;
    else b.norm = rsqrt_pow2(mrow.log_bs);
    return b;
}

