// Trellis-3INST GEMV / small-batch GEMM on the matrix cores (gfx950, wave64).
//
// The decoded weights never leave registers: the lane that decodes a state already holds
// it where v_mfma_f32_16x16x32_f16 expects its A operand.
//
//   * A wave step covers 64 rows x 32 columns: the block (m-pair, k-pair) = (2*bx + hm, kp)
//     for hm = 0, 1.  Lane L = 16*q + i takes stream lane l = 4*(i & 7) + q of block
//     hm = i >> 3.  That stream lane owns, in each of the four row groups s = 0..3
//     (rows 32*hm + (i & 7) + 8*s) and each k-tile ks, the four weights of columns
//     16*ks + 2*q + {0, 1, 8, 9} (glq/trellis.py:99-101).
//   * 3INST yields a weight as the sum of two fp16 halves packed in one register
//     (glq/trellis.py:122-134).  The halves are fed to the MFMA unadded, as two k-elements
//     that meet the same activation, so the A operand of (row i, k-group q) is simply the
//     four hash registers {w, w', w'', w'''} = 8 fp16 values, with no repacking.
//   * The B operand of (k-group q, token t) is then the activation pairs
//     (x[c], x[c]), (x[c+1], x[c+1]), (x[c+8], x[c+8]), (x[c+9], x[c+9]), c = 16*ks + 2*q:
//     16 bytes, staged once per workgroup into LDS in exactly that form, one slot per
//     (k-pair, token tile, ks, q, token).
//   * D[i][t] accumulates in fp32 over k; lane L holds rows 4*(L >> 4) + {0..3} of token
//     L & 15.
//
// One MFMA multiplies 16 rows x 32 fp16 against 16 tokens, so 1..16 tokens cost the same
// vector-ALU work (the state decode), and the dot products are off the vector ALU.
// K is split into contiguous slots (shape-only, so that row b of a batched call sums in
// exactly the order of the GEMV on x[b]; glq/csrc/glq_trellis.cu:555-715); the four waves
// of a workgroup take the slot's k-pairs round-robin and are summed in wave order.
#include "common.h"
#include "fht_device.h"
#include "trellis_device.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));
typedef float f32x4 __attribute__((ext_vector_type(4)));

template <int NT>
struct mma_acc {
    f32x4 v[4][NT];          // [row group s][token tile]
};

// 16-byte slots per (k-pair, token tile, ks, q) group: 17 for full tiles so that the
// staging writes of one wave (q fastest) land in distinct banks.
template <int TP>
constexpr int mma_tps() { return TP == 16 ? 17 : TP; }

__host__ __device__ constexpr int mma_slot_bytes(int TP, int NT) {
    return NT * 8 * (TP == 16 ? 17 : TP) * 16;                  // LDS bytes per k-pair
}

// decode one record (32 weights per lane) and multiply it against NT token tiles
template <int R, int TP, int NT>
__device__ __forceinline__ mma_acc<NT> mma_record(const tr_record<R> r, int next1, int next2,
                                                  const u32x4 *xs, mma_acc<NT> acc) {
    constexpr int TPS = mma_tps<TP>();
    uint32_t cont[4];
    tr_continuation_from<R>(r, next1, next2, cont);
#pragma unroll
    for (int ks = 0; ks < 2; ++ks) {
        f16x8 bf[NT];
#pragma unroll
        for (int tt = 0; tt < NT; ++tt) {
            bf[tt] = __builtin_bit_cast(f16x8, xs[((tt * 2 + ks) * 4) * TPS]);
        }
#pragma unroll
        for (int ms = 0; ms < 2; ++ms) {
            const int ci = ks * 2 + ms;
            uint32_t h[8];
#pragma unroll
            for (int j = 0; j < 8; ++j) h[j] = tr_hash(tr_state<R>(r.c[ci], cont[ci], j));
            const f16x8 a0 = __builtin_bit_cast(f16x8, u32x4{h[0], h[1], h[4], h[5]});
            const f16x8 a1 = __builtin_bit_cast(f16x8, u32x4{h[2], h[3], h[6], h[7]});
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) {
                acc.v[2 * ms][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a0, bf[tt], acc.v[2 * ms][tt], 0, 0, 0);
                acc.v[2 * ms + 1][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(a1, bf[tt], acc.v[2 * ms + 1][tt], 0, 0, 0);
            }
        }
    }
    return acc;
}

// (lo, lo) / (hi, hi) of a packed fp16 pair
__device__ __forceinline__ uint32_t splat_lo(uint32_t v) { return __builtin_amdgcn_perm(v, v, 0x05040504u); }
__device__ __forceinline__ uint32_t splat_hi(uint32_t v) { return __builtin_amdgcn_perm(v, v, 0x07060706u); }

struct mma_lane {
    int i, q, hm, l, next1, next2, tokl;
    bool live;
};

template <int TP>
__device__ __forceinline__ mma_lane mma_lane_of(int lane) {
    mma_lane a;
    a.i = lane & 15;
    a.q = lane >> 4;
    a.hm = a.i >> 3;
    a.l = 4 * (a.i & 7) + a.q;
    const int l1 = (a.l + 1) & 31, l2 = (a.l + 2) & 31;
    a.next1 = 16 * (l1 & 3) + 8 * a.hm + (l1 >> 2);
    a.next2 = 16 * (l2 & 3) + 8 * a.hm + (l2 >> 2);
    a.tokl = lane & 15;
    a.live = a.tokl < TP;
    return a;
}

// Sum the four waves' accumulators through LDS in wave order and write them out, G row
// groups per pass (all four when the buffer allows).  red: [TR_WAVES][G][NT][4][4*TP] floats.
template <int NT>
constexpr int mma_red_groups() { return NT <= 2 ? 4 : 2; }

template <int TP, int NT>
constexpr int mma_red_bytes() { return TR_WAVES * mma_red_groups<NT>() * NT * 4 * 4 * TP * 4; }

template <int TP, int NT>
__device__ __forceinline__ void mma_reduce_store(const mma_acc<NT> acc, float *red, const mma_lane a,
                                                 int wave, int B, int m, int tok0, int row0, int slot,
                                                 float *__restrict__ part, int direct, float scale,
                                                 int accum, int64_t out_stride) {
    constexpr int CL = 4 * TP;
    constexpr int G = mma_red_groups<NT>();
    constexpr int PER_WAVE = G * NT * 4 * CL;
#pragma unroll
    for (int s0 = 0; s0 < 4; s0 += G) {
        __syncthreads();
        if (a.live) {
            const int cl = a.q * TP + a.tokl;
#pragma unroll
            for (int sg = 0; sg < G; ++sg)
#pragma unroll
                for (int tt = 0; tt < NT; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        red[wave * PER_WAVE + ((sg * NT + tt) * 4 + r) * CL + cl] = acc.v[s0 + sg][tt][r];
        }
        __syncthreads();
        for (int e = threadIdx.x; e < PER_WAVE; e += TR_THREADS) {
            const int cl = e % CL;
            int rest = e / CL;
            const int r = rest & 3;
            rest >>= 2;
            const int tt = rest % NT, sg = rest / NT;
            const int i = 4 * (cl / TP) + r;
            const int row = row0 + 32 * (i >> 3) + (i & 7) + 8 * (s0 + sg);
            const int tok = tok0 + 16 * tt + (cl % TP);
            if (tok >= B || row >= m) continue;
            float v = red[e];
#pragma unroll
            for (int w = 1; w < TR_WAVES; ++w) v += red[w * PER_WAVE + e];
            if (direct) {
                float *o = part + (int64_t)tok * out_stride + row;
                *o = accum ? (*o + scale * v) : scale * v;
            } else {
                part[((int64_t)slot * B + tok) * m + row] = scale * v;   // 1.0f unless a stage is pre-scaled
            }
        }
    }
}

// Stage the activations of k-pairs [c0, c0+n) and tokens [tok0, tok0 + 16*NT) into the LDS
// slots.  One item = 32 bytes of one token (columns 16ks..16ks+15 of a k-pair): its dword q
// and dword 4+q, each splat into a duplicated pair, are the whole 16-byte slot (ks, q, token)
// -- one LDS write per q.  U items (2U loads) are requested before any is written.
template <int TP, int NT>
__device__ __forceinline__ void mma_stage(uint32_t *xs, const f16 *__restrict__ x, int B, int k, int tok0,
                                          int c0, int n) {
    constexpr int TPS = mma_tps<TP>();
    constexpr int U = 2;
    const int total = NT * TP * n * 2;
    for (int base = 0; base < total; base += U * TR_THREADS) {
        u32x4 v[U][2];
        int dst[U];
#pragma unroll
        for (int uu = 0; uu < U; ++uu) {
            const int idx = min(base + uu * TR_THREADS + (int)threadIdx.x, total - 1);
            const int ks = idx & 1;
            const int u = (idx >> 1) % n, tk = (idx >> 1) / n;
            const int tt = tk / TP, tl = tk % TP;
            const int tok = tok0 + 16 * tt + tl;
            const f16 *p = x + (int64_t)min(tok, B - 1) * k + 32 * (c0 + u) + 16 * ks;
            const u32x4 l0 = *(const u32x4 *)p, l1 = *(const u32x4 *)(p + 8);
            v[uu][0] = tok < B ? l0 : u32x4{0u, 0u, 0u, 0u};
            v[uu][1] = tok < B ? l1 : u32x4{0u, 0u, 0u, 0u};
            // dword index of slot (u, tt, ks, q = 0, tl)
            dst[uu] = ((((u * NT + tt) * 2 + ks) * 4) * TPS + tl) * 4;
        }
#pragma unroll
        for (int uu = 0; uu < U; ++uu) {
            if (base + uu * TR_THREADS + (int)threadIdx.x < total) {
#pragma unroll
                for (int qq = 0; qq < 4; ++qq)
                    *(u32x4 *)(xs + dst[uu] + qq * TPS * 4) =
                        u32x4{splat_lo(v[uu][0][qq]), splat_hi(v[uu][0][qq]), splat_lo(v[uu][1][qq]), splat_hi(v[uu][1][qq])};
            }
        }
    }
}

// ---------------------------------------------------------------------------------
// x given as fp16 (B, k) in the transformed domain.
// grid = (ceil(m/64), ksplit, ceil(B / (16*NT))); slot s owns k-pairs [s*S, (s+1)*S); the
// slot's activations are staged through LDS in chunks of CH k-pairs (CH % 4 == 0).
// ---------------------------------------------------------------------------------
// R2 > 0: a residual stage of R2 bits/weight decoded in the same pass against the same staged activations, its
// sums added times rs2 before the waves' sums are combined (one launch and one set of partial sums for a stacked
// layer at 1..16 tokens).
template <int R, int TP, int NT, int R2 = 0>
__device__ __forceinline__ void
tr_mma_body(const uint8_t *__restrict__ packed, const f16 *__restrict__ x, int B, int m, int k, int S, int CH,
            float *__restrict__ part, int direct, float scale, int accum, int64_t out_stride, u32x4 *xs_lds,
            const uint8_t *__restrict__ packed2 = nullptr, float rs2 = 0.0f) {
    constexpr int TPS = mma_tps<TP>();
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const mma_lane a = mma_lane_of<TP>(lane);
    const int nkp = k >> 5;
    const int mpairs = m >> 5;
    const int slot = blockIdx.y;
    const int kp0 = slot * S;
    const int kp1 = min(kp0 + S, nkp);
    const int tok0 = blockIdx.z * (16 * NT);
    const int mp = min(2 * (int)blockIdx.x + a.hm, mpairs - 1);      // odd m/32: clamp, rows dropped later

    constexpr int REC = 4 * R;
    const uint8_t *lane_base = packed + ((int64_t)mp * nkp * 32 + a.l) * REC;   // + kp * 32 * REC
    constexpr int RB = R2 > 0 ? R2 : 1, REC2 = 4 * RB;
    const uint8_t *lane_base2 = R2 > 0 ? packed2 + ((int64_t)mp * nkp * 32 + a.l) * REC2 : nullptr;
    int kp = kp0 + wave;
    tr_record<R> cur = {};
    tr_record<RB> curb = {};
    if (kp < kp1) {
        cur = tr_load_record<R>(lane_base + (int64_t)kp * 32 * REC);
        if constexpr (R2 > 0) curb = tr_load_record<RB>(lane_base2 + (int64_t)kp * 32 * REC2);
    }

    mma_acc<NT> acc, accb;
#pragma unroll
    for (int s = 0; s < 4; ++s)
#pragma unroll
        for (int tt = 0; tt < NT; ++tt) acc.v[s][tt] = accb.v[s][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

    // lanes past the token count read a zeroed block (one k-pair's worth, after the chunk)
    u32x4 *zero_blk = xs_lds + CH * (NT * 8 * TPS);
    if constexpr (TP < 16) {
        for (int i = threadIdx.x; i < NT * 8 * TPS; i += TR_THREADS) zero_blk[i] = u32x4{0u, 0u, 0u, 0u};
    }
    for (int c0 = kp0; c0 < kp1; c0 += CH) {
        const int c1 = min(c0 + CH, kp1);
        // LDS-only barriers: the record requested ahead stays in flight across them
        fht_barrier<true>();                                   // previous chunk consumed
        mma_stage<TP, NT>((uint32_t *)xs_lds, x, B, k, tok0, c0, c1 - c0);
        fht_barrier<true>();
        for (; kp < c1; kp += TR_WAVES) {
            tr_record<R> nxt = cur;
            tr_record<RB> nxtb = curb;
            if (kp + TR_WAVES < kp1) {
                nxt = tr_load_record<R>(lane_base + (int64_t)(kp + TR_WAVES) * 32 * REC);
                if constexpr (R2 > 0) nxtb = tr_load_record<RB>(lane_base2 + (int64_t)(kp + TR_WAVES) * 32 * REC2);
            }
            const u32x4 *xs = a.live ? xs_lds + ((kp - c0) * NT * 8 + a.q) * TPS + a.tokl : zero_blk;
            acc = mma_record<R, TP, NT>(cur, a.next1, a.next2, xs, acc);
            if constexpr (R2 > 0) accb = mma_record<RB, TP, NT>(curb, a.next1, a.next2, xs, accb);
            cur = nxt;
            curb = nxtb;
        }
    }
    if constexpr (R2 > 0) {
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) acc.v[s][tt] += rs2 * accb.v[s][tt];
    }
    mma_reduce_store<TP, NT>(acc, (float *)xs_lds, a, wave, B, m, tok0, 64 * blockIdx.x, slot, part,
                             direct, scale, accum, out_stride);
}

template <int R, int TP, int NT>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_kernel(const uint8_t *__restrict__ packed, const f16 *__restrict__ x, int B, int m, int k,
              int S, int CH, float *__restrict__ part, int direct, float scale, int accum,
              int64_t out_stride) {
    extern __shared__ u32x4 xs_lds[];
    tr_mma_body<R, TP, NT>(packed, x, B, m, k, S, CH, part, direct, scale, accum, out_stride, xs_lds);
}

// both stages of a stacked layer (first stage 4 bits/weight), 1..16 tokens
template <int R2, int TP>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_rvq_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ packed2, float rs2,
                  const f16 *__restrict__ x, int B, int m, int k, int S, int CH, float *__restrict__ part) {
    extern __shared__ u32x4 xs_lds[];
    tr_mma_body<4, TP, 1, R2>(packed, x, B, m, k, S, CH, part, 0, 1.0f, 0, 0, xs_lds, packed2, rs2);
}

// ---------------------------------------------------------------------------------
// GEMV with the input transform folded in (1..4 tokens), MFMA form.
//
// grid = (ceil(m/64), ksplit[, layers]).  K slot s owns the S = 2^j k-pairs starting at s*S,
// i.e. the Ls = 32*S columns [s*Ls, (s+1)*Ls) of the transformed activations.  A Hadamard
// block of size bs >= Ls that contains the slice factors as H_bs = H_(bs/Ls) (x) H_Ls, so the
// slice r of its output is
//     H_Ls( sum_h (-1)^popcount(r & h) * xs[h*Ls + j] ) / sqrt(bs),   xs = sv * x,
// one pass over the block's inputs (they sit in L2) and a short transform in LDS; smaller
// blocks are transformed whole (glq/hadamard.py:166-178, glq/csrc/glq_trellis.cu:315-370).
// The last pass writes each value as the duplicated fp16 pair of its B-operand slot, and the
// decode loop is mma_record.
// ---------------------------------------------------------------------------------
template <int TP>
__host__ __device__ constexpr int fi_xs_slots(int S) {
    return S * 8 * mma_tps<TP>() + (TP < 16 ? 8 * mma_tps<TP>() : 0);          // slots + zero block
}

// R2 > 0: a residual stage of R2 bits/weight (glq/trellis.py stacked RVQ) decoded in the same launch against the
// same activations: its own stream, its own accumulators, added with its scale rs2 before the waves' sums are
// combined -- one launch, one transform of x and one set of partial sums where two launches wrote two.
template <int R, typename XT, int TP, int R2 = 0>
__device__ __forceinline__ void
tr_mma_fusein_body(const uint8_t *__restrict__ packed, const XT *__restrict__ x, int64_t x_stride,
                   const f16 *__restrict__ sv, int B, int m, int k, int in_features, int S,
                   const glqh_block_meta *__restrict__ bn_meta, int n_blocks, glqh_meta_args margs,
                   float *__restrict__ part, float pscale, u32x4 *lds, int part_B = 0,
                   const uint8_t *__restrict__ packed2 = nullptr, float rs2 = 0.0f) {
    constexpr int TPS = mma_tps<TP>();
    const int Ls = S << 5;
    uint32_t *xs32 = (uint32_t *)lds;
    u32x4 *zero_blk = lds + S * 8 * TPS;
    float *fbuf = (float *)(lds + fi_xs_slots<TP>(S));          // Ls + Ls/32 floats
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const mma_lane a = mma_lane_of<TP>(lane);
    const int nkp = k >> 5;
    const int mpairs = m >> 5;
    const int slot = blockIdx.y;
    const int kp0 = slot * S;
    const int kp1 = min(kp0 + S, nkp);
    const int c0 = kp0 << 5;
    const int mp = min(2 * (int)blockIdx.x + a.hm, mpairs - 1);

    constexpr int REC = 4 * R;
    const uint8_t *lane_base = packed + ((int64_t)mp * nkp * 32 + a.l) * REC;
    constexpr int RB = R2 > 0 ? R2 : 1, REC2 = 4 * RB;
    const uint8_t *lane_base2 = R2 > 0 ? packed2 + ((int64_t)mp * nkp * 32 + a.l) * REC2 : nullptr;
    int kp = kp0 + wave;
    tr_record<R> cur, nx1;
    tr_record<RB> curb = {}, nx1b = {};
    bool requested = false;

    if constexpr (TP < 16) {
        for (int i = threadIdx.x; i < 8 * TPS; i += TR_THREADS) zero_blk[i] = u32x4{0u, 0u, 0u, 0u};
    }
    // 8-byte loads of four activations / signs are possible (uniform over the launch)
    const bool quads = (((uintptr_t)x | (uintptr_t)sv) & 7) == 0 && (x_stride & 3) == 0;
    // ---- prologue: transformed activations of this slot's columns -> B-operand slots ----
    for (int jb = 0; jb < n_blocks; ++jb) {
        const glqh_block_meta bm = glqh_meta_row(margs, bn_meta, jb);
        const int lo = max(bm.offset, c0), hi = min(bm.offset + bm.bs, c0 + Ls);
        if (lo >= hi) continue;                                  // uniform over the workgroup
        const int len = hi - lo;                                 // min(bs, Ls), a power of two
        const int log_len = 31 - __builtin_clz(len);
        const int nsub = bm.bs >> log_len;
        const int r = (lo - bm.offset) >> log_len;
        const float norm = bm.w != 0 ? __builtin_bit_cast(float, bm.w) : rsqrt_pow2(bm.log_bs);
        for (int t = 0; t < TP; ++t) {
            if (t >= B) break;
            const XT *xr = x + (int64_t)t * x_stride;
            fht_barrier<true>();                                 // fbuf free again (record loads stay in flight)
            // The wave's first records are requested as soon as the activations have been: loads
            // complete in order, so the transform waits for the activations only and the packed
            // stream's first bytes are on their way while it runs.
            auto request = [&]() {
                if (!requested) {
                    requested = true;
                    cur = tr_load_record<R>(lane_base + (int64_t)min(kp, kp1 - 1) * 32 * REC);
                    nx1 = tr_load_record<R>(lane_base + (int64_t)min(kp + TR_WAVES, kp1 - 1) * 32 * REC);
                    if constexpr (R2 > 0) {
                        curb = tr_load_record<RB>(lane_base2 + (int64_t)min(kp, kp1 - 1) * 32 * REC2);
                        nx1b = tr_load_record<RB>(lane_base2 + (int64_t)min(kp + TR_WAVES, kp1 - 1) * 32 * REC2);
                    }
                }
            };
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
                    for (int q = 0; q < 4; ++q) {
                        const int i = fht_wave_index<4>(log_len, tid, q);
                        const int c = lo - c0 + i;               // column inside the slot
                        const int u = c >> 5, ks = (c >> 4) & 1, qq = (c >> 1) & 3;
                        const int p = 2 * ((c >> 3) & 1) + (c & 1);
                        const f16 hv = (f16)(z[q] * norm);
                        const f16x2 pair = {hv, hv};
                        xs32[((((u * 2 + ks) * 4) + qq) * mma_tps<TP>() + t) * 4 + p] = __builtin_bit_cast(uint32_t, pair);
                    }
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
                uint32_t *xs32;
                int c_rel, t;
                float norm;
                __device__ float aux(int) const { return norm; }
                __device__ void put(int i, float v, float f) const {
                    const int c = c_rel + i;                     // column inside the slot
                    const int u = c >> 5, ks = (c >> 4) & 1, q = (c >> 1) & 3;
                    const int p = 2 * ((c >> 3) & 1) + (c & 1);
                    const f16 hv = (f16)(v * f);
                    const f16x2 pair = {hv, hv};
                    xs32[((((u * 2 + ks) * 4) + q) * mma_tps<TP>() + t) * 4 + p] = __builtin_bit_cast(uint32_t, pair);
                }
            } store = {xs32, lo - c0, t, norm};
            fht_staged<true>(fbuf, log_len, store);             // barriers that leave the record loads in flight
        }
    }
    if (!requested) {
        cur = tr_load_record<R>(lane_base + (int64_t)min(kp, kp1 - 1) * 32 * REC);
        nx1 = tr_load_record<R>(lane_base + (int64_t)min(kp + TR_WAVES, kp1 - 1) * 32 * REC);
        if constexpr (R2 > 0) {
            curb = tr_load_record<RB>(lane_base2 + (int64_t)min(kp, kp1 - 1) * 32 * REC2);
            nx1b = tr_load_record<RB>(lane_base2 + (int64_t)min(kp + TR_WAVES, kp1 - 1) * 32 * REC2);
        }
    }
    if constexpr (TP > 1) {
        // tokens past B read zeros: clear their slots once (every k-pair of the slot)
        for (int idx = threadIdx.x; idx < S * 8 * (TP - 1); idx += TR_THREADS) {
            const int t = 1 + idx % (TP - 1), g = idx / (TP - 1);
            if (t >= B) lds[g * TPS + t] = u32x4{0u, 0u, 0u, 0u};
        }
    }
    __syncthreads();

    mma_acc<1> acc, accb;
#pragma unroll
    for (int s = 0; s < 4; ++s) acc.v[s][0] = accb.v[s][0] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (; kp < kp1; kp += TR_WAVES) {
        tr_record<R> nx2 = nx1;                                  // nothing is requested past the wave's last record
        tr_record<RB> nx2b = nx1b;
        if (kp + 2 * TR_WAVES < kp1) {
            nx2 = tr_load_record<R>(lane_base + (int64_t)(kp + 2 * TR_WAVES) * 32 * REC);
            if constexpr (R2 > 0) nx2b = tr_load_record<RB>(lane_base2 + (int64_t)(kp + 2 * TR_WAVES) * 32 * REC2);
        }
        const u32x4 *xsl = a.live ? lds + ((kp - kp0) * 8 + a.q) * TPS + a.tokl : zero_blk;
        acc = mma_record<R, TP, 1>(cur, a.next1, a.next2, xsl, acc);
        if constexpr (R2 > 0) accb = mma_record<RB, TP, 1>(curb, a.next1, a.next2, xsl, accb);
        cur = nx1;
        nx1 = nx2;
        curb = nx1b;
        nx1b = nx2b;
    }
    if constexpr (R2 > 0) {
#pragma unroll
        for (int s = 0; s < 4; ++s) acc.v[s][0] += rs2 * accb.v[s][0];
    }
    // part_B: rows per K slot of the partial-sum array when it holds more rows than this call's
    // tokens (the routed-expert launch: one row per (token, expert) slot, `part` offset to this one)
    mma_reduce_store<TP, 1>(acc, (float *)lds, a, wave, part_B > 0 ? part_B : B, m, 0, 64 * blockIdx.x, slot, part,
                            0, pscale, 0, 0);
}

template <int R, typename XT, int TP>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_kernel(const uint8_t *__restrict__ packed, const XT *__restrict__ x, int64_t x_stride,
                     const f16 *__restrict__ sv, int B, int m, int k, int in_features, int S,
                     const glqh_block_meta *__restrict__ bn_meta, int n_blocks, glqh_meta_args margs,
                     float *__restrict__ part, float pscale) {
    extern __shared__ u32x4 xs_lds[];
    tr_mma_fusein_body<R, XT, TP>(packed, x, x_stride, sv, B, m, k, in_features, S, bn_meta, n_blocks, margs,
                                  part, pscale, xs_lds);
}

// Both stages of a stacked layer (first stage 4 bits/weight, as every recipe of the reference has it:
// glq_vllm/linear_method.py trellis recipes 5..8 bpw = 4 + 1..4), one token.
template <int R2, typename XT>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_rvq_kernel(const uint8_t *__restrict__ packed, const uint8_t *__restrict__ packed2, float rs2,
                         const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv, int m, int k,
                         int in_features, int S, const glqh_block_meta *__restrict__ bn_meta, int n_blocks,
                         glqh_meta_args margs, float *__restrict__ part) {
    extern __shared__ u32x4 xs_lds[];
    tr_mma_fusein_body<4, XT, 1, R2>(packed, x, x_stride, sv, 1, m, k, in_features, S, bn_meta, n_blocks, margs,
                                     part, 1.0f, xs_lds, 0, packed2, rs2);
}

// Several layers that read the same activations (fused q/k/v, gate/up:
// glq_vllm/linear_method.py:664-710) in one launch: blockIdx.z picks the layer, each with
// its own packed stream, input signs and partial-sum buffer; workgroups past a layer's rows
// retire.
struct tr_fusein_group {
    const uint8_t *packed[GLQH_MAX_GROUP];
    const f16 *sv[GLQH_MAX_GROUP];
    float *part[GLQH_MAX_GROUP];
    int m[GLQH_MAX_GROUP];
};

template <int R, typename XT, int TP>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_group_kernel(tr_fusein_group g, const XT *__restrict__ x, int64_t x_stride, int B, int k,
                           int in_features, int S, const glqh_block_meta *__restrict__ bn_meta,
                           int n_blocks, glqh_meta_args margs) {
    extern __shared__ u32x4 xs_lds[];
    const int z = blockIdx.z;
    const uint8_t *packed = g.packed[0];
    const f16 *sv = g.sv[0];
    float *part = g.part[0];
    int m = g.m[0];
#pragma unroll
    for (int i = 1; i < GLQH_MAX_GROUP; ++i)
        if (i == z) { packed = g.packed[i]; sv = g.sv[i]; part = g.part[i]; m = g.m[i]; }
    if ((int)blockIdx.x * 64 >= m) return;
    tr_mma_fusein_body<R, XT, TP>(packed, x, x_stride, sv, B, m, k, in_features, S, bn_meta, n_blocks, margs,
                                  part, 1.0f, xs_lds);
}

// several stacked layers (4 + R2 bits/weight each) on the same token: blockIdx.z = layer
struct tr_fusein_group_rvq {
    const uint8_t *packed2[GLQH_MAX_GROUP];
    float rs2[GLQH_MAX_GROUP];
};

template <int R2, typename XT>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_group_rvq_kernel(tr_fusein_group g, tr_fusein_group_rvq g2, const XT *__restrict__ x, int64_t x_stride,
                               int k, int in_features, int S, const glqh_block_meta *__restrict__ bn_meta,
                               int n_blocks, glqh_meta_args margs) {
    extern __shared__ u32x4 xs_lds[];
    const int z = blockIdx.z;
    const uint8_t *packed = g.packed[0], *packed2 = g2.packed2[0];
    const f16 *sv = g.sv[0];
    float *part = g.part[0];
    float rs2 = g2.rs2[0];
    int m = g.m[0];
#pragma unroll
    for (int i = 1; i < GLQH_MAX_GROUP; ++i)
        if (i == z) { packed = g.packed[i]; packed2 = g2.packed2[i]; rs2 = g2.rs2[i]; sv = g.sv[i]; part = g.part[i]; m = g.m[i]; }
    if ((int)blockIdx.x * 64 >= m) return;
    tr_mma_fusein_body<4, XT, 1, R2>(packed, x, x_stride, sv, 1, m, k, in_features, S, bn_meta, n_blocks, margs, part, 1.0f,
                                     xs_lds, 0, packed2, rs2);
}

// Routed experts of a mixture-of-experts layer, one token each (glq/csrc/glq_cuda.cu:5030-5250,
// glq/csrc/glq_trellis.cu:539-588): blockIdx.z = slot = (token, choice); the slot's expert comes
// from topk_ids on the device, so nothing about the routing is known to the host and the launch
// can be captured.  Every expert has its own packed stream (stride_bytes apart) and scale; the
// input signs are shared.  x row of slot s is s / x_div (the token for the first projection, the
// slot itself for the second).  Partial sums: [K slot][slot][row].  Slots whose expert id is out
// of range write nothing and are skipped by the finishing kernels as well.
struct tr_moe_args {
    const uint8_t *packed;                       // expert 0
    int64_t stride_bytes;                        // from one expert's stream to the next
    const int64_t *topk_ids;                     // (n_slots,)
    const float *pscale_dev;                     // per-expert factor of the partial sums (a residual stage), or NULL
    float *part;
    int n_slots, n_experts, x_div;
};

template <int R, typename XT>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_moe_kernel(tr_moe_args g, const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv,
                         int m, int k, int in_features, int S, const glqh_block_meta *__restrict__ bn_meta,
                         int n_blocks, glqh_meta_args margs) {
    extern __shared__ u32x4 xs_lds[];
    const int slot = blockIdx.z;
    const int64_t e = g.topk_ids[slot];
    if (e < 0 || e >= g.n_experts) return;                      // uniform over the workgroup
    tr_mma_fusein_body<R, XT, 1>(g.packed + e * g.stride_bytes, x + (int64_t)(slot / g.x_div) * x_stride, x_stride,
                                 sv, 1, m, k, in_features, S, bn_meta, n_blocks, margs,
                                 g.part + (int64_t)slot * m, g.pscale_dev ? g.pscale_dev[e] : 1.0f, xs_lds,
                                 g.n_slots);
}

// Two-stage experts (first stage 4 bits/weight): both streams of the slot's expert in the same launch, the second
// one's sums times the expert's inv_resid_scale2 (read on the device) added in registers.
template <int R2, typename XT>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_fusein_moe_rvq_kernel(tr_moe_args g, const uint8_t *__restrict__ packed2, int64_t stride2_bytes,
                             const XT *__restrict__ x, int64_t x_stride, const f16 *__restrict__ sv, int m, int k,
                             int in_features, int S, const glqh_block_meta *__restrict__ bn_meta, int n_blocks,
                             glqh_meta_args margs) {
    extern __shared__ u32x4 xs_lds[];
    const int slot = blockIdx.z;
    const int64_t e = g.topk_ids[slot];
    if (e < 0 || e >= g.n_experts) return;                      // uniform over the workgroup
    tr_mma_fusein_body<4, XT, 1, R2>(g.packed + e * g.stride_bytes, x + (int64_t)(slot / g.x_div) * x_stride, x_stride,
                                     sv, 1, m, k, in_features, S, bn_meta, n_blocks, margs,
                                     g.part + (int64_t)slot * m, 1.0f, xs_lds, g.n_slots, packed2 + e * stride2_bytes,
                                     g.pscale_dev[e]);
}

// The same step for many slots: the slots are grouped by expert (perm: slot numbers sorted by
// expert, offs: first position of every expert, both made on the device by the routing launch), and
// workgroup (row block, K slot, expert) reads its expert's stream once per 16 of the expert's rows
// (glq/csrc/glq_trellis.cu:1475-1540 pads every expert to tiles of 16 rows in the same way).  x: fp16
// rows in the transformed domain, row of slot s = s / x_div.  Experts without rows retire.
struct tr_moe_group_args {
    const uint8_t *packed;
    int64_t stride_bytes;
    const uint8_t *packed2;                      // residual streams of stacked experts (kernels with R2 > 0): pscale_dev
    int64_t stride2_bytes;                       // is then their scale, applied to the second stream's sums
    const int *perm, *offs;
    const float *pscale_dev;
    float *part;                                 // [K slot][slot][row]
    int n_slots, x_div;
};

// One pass over the K slot for NT tiles of 16 of the expert's rows, positions [t0, t0 + 16 NT) of its run in perm.
template <int R, int NT, int R2 = 0>
__device__ __forceinline__ void moe_group_pass(const tr_moe_group_args &g, const f16 *__restrict__ x, int m, int k,
                                               int kp0, int kp1, int CH, const uint8_t *lane_base, const mma_lane a,
                                               int wave, int o0, int cnt, int t0, float pscale, int kslot,
                                               u32x4 *xs_lds, int *slotmap, const uint8_t *lane_base2 = nullptr) {
    constexpr int TPS = mma_tps<16>();
    constexpr int REC = 4 * R;
    constexpr int RB = R2 > 0 ? R2 : 1, REC2 = 4 * RB;
    constexpr int G = mma_red_groups<NT>();                      // row groups per round of the final sum
    constexpr int PER_WAVE = G * NT * 256;
    uint32_t *xs = (uint32_t *)xs_lds;
    float *red = (float *)xs_lds;                                // [TR_WAVES][G][NT][4][64]
    __syncthreads();                                             // the previous pass is done with slotmap and red
    if (threadIdx.x < 16 * NT)
        slotmap[threadIdx.x] = t0 + (int)threadIdx.x < cnt ? g.perm[o0 + t0 + threadIdx.x] : -1;
    int kp = kp0 + wave;
    tr_record<R> cur = {};
    tr_record<RB> curb = {};
    if (kp < kp1) {
        cur = tr_load_record<R>(lane_base + (int64_t)kp * 32 * REC);
        if constexpr (R2 > 0) curb = tr_load_record<RB>(lane_base2 + (int64_t)kp * 32 * REC2);
    }
    mma_acc<NT> acc, accb;
#pragma unroll
    for (int sg = 0; sg < 4; ++sg)
#pragma unroll
        for (int tt = 0; tt < NT; ++tt) acc.v[sg][tt] = accb.v[sg][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
    for (int c0 = kp0; c0 < kp1; c0 += CH) {
        const int c1 = min(c0 + CH, kp1), n = c1 - c0;
        fht_barrier<true>();                                     // slotmap written / previous chunk consumed
        // one item = 32 bytes of one row: columns 16 ks .. 16 ks + 15 of k-pair c0 + u
        for (int idx = threadIdx.x; idx < 32 * NT * n; idx += TR_THREADS) {
            const int ks = idx & 1, u = (idx >> 1) % n, tk = (idx >> 1) / n;
            const int tt = tk >> 4, tl = tk & 15;
            const int sl = slotmap[tk];
            const f16 *p = x + (int64_t)(sl < 0 ? 0 : sl / g.x_div) * k + 32 * (c0 + u) + 16 * ks;
            u32x4 l0 = *(const u32x4 *)p, l1 = *(const u32x4 *)(p + 8);
            if (sl < 0) l0 = l1 = u32x4{0u, 0u, 0u, 0u};
            uint32_t *dst = xs + (((((u * NT + tt) * 2 + ks) * 4) * TPS) + tl) * 4;
#pragma unroll
            for (int qq = 0; qq < 4; ++qq)
                *(u32x4 *)(dst + qq * TPS * 4) =
                    u32x4{splat_lo(l0[qq]), splat_hi(l0[qq]), splat_lo(l1[qq]), splat_hi(l1[qq])};
        }
        fht_barrier<true>();
        for (; kp < c1; kp += TR_WAVES) {
            tr_record<R> nxt = cur;
            tr_record<RB> nxtb = curb;
            if (kp + TR_WAVES < kp1) {
                nxt = tr_load_record<R>(lane_base + (int64_t)(kp + TR_WAVES) * 32 * REC);
                if constexpr (R2 > 0) nxtb = tr_load_record<RB>(lane_base2 + (int64_t)(kp + TR_WAVES) * 32 * REC2);
            }
            const u32x4 *xsl = xs_lds + ((kp - c0) * NT * 8 + a.q) * TPS + a.tokl;
            acc = mma_record<R, 16, NT>(cur, a.next1, a.next2, xsl, acc);
            if constexpr (R2 > 0) accb = mma_record<RB, 16, NT>(curb, a.next1, a.next2, xsl, accb);
            cur = nxt;
            curb = nxtb;
        }
    }
    if constexpr (R2 > 0) {                                      // pscale is the residual scale here, not a factor of the sum
#pragma unroll
        for (int sg = 0; sg < 4; ++sg)
#pragma unroll
            for (int tt = 0; tt < NT; ++tt) acc.v[sg][tt] += pscale * accb.v[sg][tt];
        pscale = 1.0f;
    }
    // the four waves' sums in wave order, G row groups per round, then one row of part per (K slot, slot)
#pragma unroll
    for (int s0 = 0; s0 < 4; s0 += G) {
        __syncthreads();
        {
            const int cl = a.q * 16 + a.tokl;
#pragma unroll
            for (int sg = 0; sg < G; ++sg)
#pragma unroll
                for (int tt = 0; tt < NT; ++tt)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        red[wave * PER_WAVE + ((sg * NT + tt) * 4 + r) * 64 + cl] = acc.v[s0 + sg][tt][r];
        }
        __syncthreads();
        for (int i2 = threadIdx.x; i2 < PER_WAVE; i2 += TR_THREADS) {
            const int cl = i2 & 63, r = (i2 >> 6) & 3, tt = (i2 >> 8) % NT, sg = (i2 >> 8) / NT;
            const int i = 4 * (cl >> 4) + r;
            const int row = 64 * blockIdx.x + 32 * (i >> 3) + (i & 7) + 8 * (s0 + sg);
            const int sl = slotmap[16 * tt + (cl & 15)];
            if (sl < 0 || row >= m) continue;
            float v = red[i2];
#pragma unroll
            for (int w = 1; w < TR_WAVES; ++w) v += red[w * PER_WAVE + i2];
            g.part[((int64_t)kslot * g.n_slots + sl) * m + row] = pscale * v;
        }
    }
}

// Chunk lengths (k-pairs staged per barrier pair) of the passes with one, two and four row tiles.
struct moe_chunks {
    int ch1, ch2, ch4;
};

// WIDE = false: passes of 16 rows only (few rows per expert: the registers of the wide passes would cost
// occupancy for nothing).
template <int R, bool WIDE, int R2 = 0>
__global__ void __launch_bounds__(TR_THREADS)
tr_mma_moe_grouped_kernel(tr_moe_group_args g, const f16 *__restrict__ x, int m, int k, int S, moe_chunks ch) {
    extern __shared__ u32x4 xs_lds[];
    __shared__ int slotmap[64];
    const int e = blockIdx.z;
    const int o0 = g.offs[e], cnt = g.offs[e + 1] - o0;
    if (cnt <= 0) return;                                        // uniform over the workgroup
    const uint8_t *packed = g.packed + (int64_t)e * g.stride_bytes;
    const float pscale = g.pscale_dev ? g.pscale_dev[e] : 1.0f;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const mma_lane a = mma_lane_of<16>(lane);
    const int nkp = k >> 5;
    const int mpairs = m >> 5;
    const int kslot = blockIdx.y;
    const int kp0 = kslot * S;
    const int kp1 = min(kp0 + S, nkp);
    const int mp = min(2 * (int)blockIdx.x + a.hm, mpairs - 1);
    constexpr int REC = 4 * R;
    const uint8_t *lane_base = packed + ((int64_t)mp * nkp * 32 + a.l) * REC;
    constexpr int REC2 = 4 * (R2 > 0 ? R2 : 1);
    const uint8_t *lane_base2 =
        R2 > 0 ? g.packed2 + (int64_t)e * g.stride2_bytes + ((int64_t)mp * nkp * 32 + a.l) * REC2 : nullptr;

    // The stream is read once per pass: as many of the expert's rows per pass as there are, up to 64.
    for (int t0 = 0; t0 < cnt;) {
        const int rem = WIDE ? cnt - t0 : 0;
        if (rem > 32) {
            moe_group_pass<R, 4, R2>(g, x, m, k, kp0, kp1, ch.ch4, lane_base, a, wave, o0, cnt, t0, pscale, kslot, xs_lds, slotmap, lane_base2);
            t0 += 64;
        } else if (rem > 16) {
            moe_group_pass<R, 2, R2>(g, x, m, k, kp0, kp1, ch.ch2, lane_base, a, wave, o0, cnt, t0, pscale, kslot, xs_lds, slotmap, lane_base2);
            t0 += 32;
        } else {
            moe_group_pass<R, 1, R2>(g, x, m, k, kp0, kp1, ch.ch1, lane_base, a, wave, o0, cnt, t0, pscale, kslot, xs_lds, slotmap, lane_base2);
            t0 += 16;
        }
    }
}

template <int TP>
size_t fi_lds_bytes(int S) {
    const size_t Ls = (size_t)S * 32;
    size_t b = (size_t)fi_xs_slots<TP>(S) * 16 + (Ls + Ls / 32 + 32) * sizeof(float);
    if (b < (size_t)mma_red_bytes<TP, 1>()) b = mma_red_bytes<TP, 1>();
    return b;
}

constexpr int FI_MAX_S = 256;                                    // 8192 columns per slot
constexpr int FI_MAX_S_TP4 = 128;

// LDS per workgroup: a chunk of CH k-pairs (CH % 4 == 0) plus, for partial token tiles, one
// zeroed block; small enough that the register-limited number of workgroups fits a CU.
constexpr int MMA_LDS_MAX = 64 * 1024;

template <int TP, int NT>
constexpr int mma_chunk_cap() {
    return TP == 1 ? 448 : TP == 4 ? 64 : NT == 1 ? 16 : 4;
}

template <int R, int TP, int NT>
int launch_mma(const void *x, int64_t B, const void *packed, int64_t m, int64_t k, int S, int ksplit,
               float *part, int direct, float scale, int accum, int64_t out_stride, hipStream_t stream) {
    const int per_kp = mma_slot_bytes(TP, NT);
    int CH = mma_chunk_cap<TP, NT>();
    if (CH > S) CH = (S + 3) & ~3;
    size_t lds = (size_t)(CH + (TP < 16 ? 1 : 0)) * per_kp;
    if (lds < (size_t)mma_red_bytes<TP, NT>()) lds = mma_red_bytes<TP, NT>();
    dim3 grid((unsigned)((m + 63) / 64), (unsigned)ksplit, (unsigned)((B + 16 * NT - 1) / (16 * NT)));
    hipLaunchKernelGGL((tr_mma_kernel<R, TP, NT>), grid, dim3(TR_THREADS), lds, stream,
                       (const uint8_t *)packed, (const f16 *)x, (int)B, (int)m, (int)k, S, CH, part, direct,
                       scale, accum, out_stride);
    GLQH_LAUNCH_CHECK("trellis mma launch");
    return 0;
}

template <int R2, int TP>
int launch_mma_rvq(const void *x, int64_t B, const void *packed, const void *packed2, float rs2, int64_t m, int64_t k,
                   int S, int ksplit, float *part, hipStream_t stream) {
    const int per_kp = mma_slot_bytes(TP, 1);
    int CH = mma_chunk_cap<TP, 1>();
    if (CH > S) CH = (S + 3) & ~3;
    size_t lds = (size_t)(CH + (TP < 16 ? 1 : 0)) * per_kp;
    if (lds < (size_t)mma_red_bytes<TP, 1>()) lds = mma_red_bytes<TP, 1>();
    dim3 grid((unsigned)((m + 63) / 64), (unsigned)ksplit, 1);
    hipLaunchKernelGGL((tr_mma_rvq_kernel<R2, TP>), grid, dim3(TR_THREADS), lds, stream, (const uint8_t *)packed,
                       (const uint8_t *)packed2, rs2, (const f16 *)x, (int)B, (int)m, (int)k, S, CH, part);
    GLQH_LAUNCH_CHECK("trellis mma two-stage launch");
    return 0;
}

template <int R2>
int launch_mma_rvq_R(const void *x, int64_t B, const void *packed, const void *packed2, float rs2, int64_t m, int64_t k,
                     int S, int ksplit, float *part, hipStream_t stream) {
    if (B == 1) return launch_mma_rvq<R2, 1>(x, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    if (B <= 4) return launch_mma_rvq<R2, 4>(x, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    return launch_mma_rvq<R2, 16>(x, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
}

template <int R>
int launch_mma_R(const void *x, int64_t B, const void *packed, int64_t m, int64_t k, int S, int ksplit,
                 float *part, int direct, float scale, int accum, int64_t out_stride, hipStream_t stream) {
#define GLQH_MMA(TP, NT) launch_mma<R, TP, NT>(x, B, packed, m, k, S, ksplit, part, direct, scale, accum, \
                                               out_stride, stream)
    if (B == 1) return GLQH_MMA(1, 1);
    if (B <= 4) return GLQH_MMA(4, 1);
    if (B <= 16) return GLQH_MMA(16, 1);
    if (B <= 32) return GLQH_MMA(16, 2);
    return GLQH_MMA(16, 4);
#undef GLQH_MMA
}

template <typename K>
int mma_set_lds(K kernel) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              MMA_LDS_MAX),
                          "trellis mma attribute");
}

template <int R>
int mma_init_R() {
    return mma_set_lds(tr_mma_kernel<R, 1, 1>) || mma_set_lds(tr_mma_kernel<R, 4, 1>) ||
           mma_set_lds(tr_mma_kernel<R, 16, 1>) || mma_set_lds(tr_mma_kernel<R, 16, 2>) ||
           mma_set_lds(tr_mma_kernel<R, 16, 4>) || mma_set_lds(tr_mma_moe_grouped_kernel<R, false>) ||
           mma_set_lds(tr_mma_moe_grouped_kernel<R, true>) || mma_set_lds(tr_mma_moe_grouped_kernel<4, false, R>) ||
           mma_set_lds(tr_mma_rvq_kernel<R, 1>) ||
           mma_set_lds(tr_mma_rvq_kernel<R, 4>) || mma_set_lds(tr_mma_rvq_kernel<R, 16>);
}

}  // namespace

// K slots: S k-pairs (32 columns) each, a multiple of the wave count, chosen from the
// layer shape only; about four workgroups per CU.
int glqh_trellis_mma_plan(int64_t m, int64_t k, int *S_out, int *ksplit_out) {
    const int64_t nkp = k / 32;
    const int64_t wgs = (m + 63) / 64;
    const int64_t target = (int64_t)glqh_device_cus() * 4;
    int64_t ks = (target + wgs - 1) / wgs;
    if (ks > 64) ks = 64;
    if (ks < 1) ks = 1;
    int64_t S = (nkp + ks - 1) / ks;
    S = (S + TR_WAVES - 1) / TR_WAVES * TR_WAVES;
    *S_out = (int)S;
    *ksplit_out = (int)((nkp + S - 1) / S);
    return 1;
}

int glqh_launch_trellis_mma(const void *x_f16, int64_t B, const void *packed, int R, int64_t m, int64_t k,
                            int S, int ksplit, float *part, int direct, float scale, int accum,
                            int64_t out_stride, hipStream_t stream) {
    switch (R) {
    case 1: return launch_mma_R<1>(x_f16, B, packed, m, k, S, ksplit, part, direct, scale, accum, out_stride, stream);
    case 2: return launch_mma_R<2>(x_f16, B, packed, m, k, S, ksplit, part, direct, scale, accum, out_stride, stream);
    case 3: return launch_mma_R<3>(x_f16, B, packed, m, k, S, ksplit, part, direct, scale, accum, out_stride, stream);
    case 4: return launch_mma_R<4>(x_f16, B, packed, m, k, S, ksplit, part, direct, scale, accum, out_stride, stream);
    }
    return glqh_fail("trellis kernel supports R (bits/weight) 1-4, got %d", R);
}

// Both stages of a stacked layer (4 + R2 bits/weight) against 1..16 transformed tokens in one launch:
// part[(slot * B + token) * m + row] = sum1 + rs2 * sum2, K plan as glqh_launch_trellis_mma's.
int glqh_launch_trellis_mma_rvq(const void *x_f16, int64_t B, const void *packed, const void *packed2, int R2, float rs2,
                                int64_t m, int64_t k, int S, int ksplit, float *part, hipStream_t stream) {
    if (B < 1 || B > 16) return glqh_fail("trellis two-stage kernel: 1..16 tokens, got %lld", (long long)B);
    switch (R2) {
    case 1: return launch_mma_rvq_R<1>(x_f16, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    case 2: return launch_mma_rvq_R<2>(x_f16, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    case 3: return launch_mma_rvq_R<3>(x_f16, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    case 4: return launch_mma_rvq_R<4>(x_f16, B, packed, packed2, rs2, m, k, S, ksplit, part, stream);
    }
    return glqh_fail("trellis two-stage kernel: second stage of 1-4 bits/weight, got %d", R2);
}

// ---- fused-input GEMV (MFMA form): plan and launch -----------------------------------
// S k-pairs per K slot: a power of two >= 8 chosen so that about four workgroups per CU are
// in flight; the slice 32*S is capped by LDS (8192 columns at one token, 4096 at 2..4).
int glqh_trellis_mma_fusein_plan(int64_t wgs_rows, int64_t k, int64_t B, int *S_out, int *ksplit_out) {
    if (B < 1 || B > 4 || wgs_rows < 1) return 0;
    const int64_t nkp = k / 32;
    const int64_t target = (int64_t)glqh_device_cus() * 4;
    int64_t ks_target = (target + wgs_rows - 1) / wgs_rows;
    if (ks_target < 1) ks_target = 1;
    const int64_t want = (nkp + ks_target - 1) / ks_target;
    int64_t S = 2 * TR_WAVES;                                   // at least 256 columns per slot
    // Every workgroup sums the (block / slice) sub-slices of its Hadamard block before it
    // decodes anything: 256-column slices of a block of 4096 points or more are 16+ terms in
    // front of two records per wave (4096 x 4096: 17.6 us per linear with them, 11.9 us with
    // 512-column slices).
    if (k >= 4096) S = 4 * TR_WAVES;
    while (S < want) S <<= 1;
    const int64_t cap = B == 1 ? FI_MAX_S : FI_MAX_S_TP4;
    if (S > cap) S = cap;
    *S_out = (int)S;
    *ksplit_out = (int)((nkp + S - 1) / S);
    return 1;
}

template <int R, typename XT, int TP>
static int launch_mma_fusein(const tr_fusein_group &g, int n_layers, int64_t max_m, const void *x,
                             int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int S, int ksplit,
                             const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                             float pscale, hipStream_t stream) {
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    const glqh_block_meta *meta = n_blocks > 1 ? bn_meta : nullptr;
    const int nb = n_blocks > 1 ? n_blocks : 1;
    const size_t lds = fi_lds_bytes<TP>(S);
    if (n_layers == 1) {
        dim3 grid((unsigned)((max_m + 63) / 64), (unsigned)ksplit, 1);
        hipLaunchKernelGGL((tr_mma_fusein_kernel<R, XT, TP>), grid, dim3(TR_THREADS), lds, stream, g.packed[0],
                           (const XT *)x, x_stride, g.sv[0], (int)B, g.m[0], (int)k, (int)in_features, S, meta, nb,
                           margs, g.part[0], pscale);
    } else {
        dim3 grid((unsigned)((max_m + 63) / 64), (unsigned)ksplit, (unsigned)n_layers);
        hipLaunchKernelGGL((tr_mma_fusein_group_kernel<R, XT, TP>), grid, dim3(TR_THREADS), lds, stream, g,
                           (const XT *)x, x_stride, (int)B, (int)k, (int)in_features, S, meta, nb, margs);
    }
    GLQH_LAUNCH_CHECK("trellis fused-input gemv launch");
    return 0;
}

// packed / sv / part / m: one entry per layer (1..GLQH_MAX_GROUP)
int glqh_launch_trellis_mma_fusein(const void *const packed[], const void *const sv[], float *const part[],
                                   const int64_t m[], int n_layers, int R, const void *x, int x_dtype,
                                   int64_t x_stride, int64_t B, int64_t k, int64_t in_features, int S,
                                   int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                   int n_blocks, float pscale, hipStream_t stream) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(n_layers >= 1 && n_layers <= GLQH_MAX_GROUP, "trellis group: 1..%d layers", GLQH_MAX_GROUP);
    GLQH_REQUIRE(n_layers == 1 || pscale == 1.0f, "trellis group: pre-scaled partial sums are a single-layer option");
    GLQH_REQUIRE(B >= 1 && B <= 4, "fused-input trellis kernel serves 1..4 tokens");
    tr_fusein_group g = {};
    int64_t max_m = 0;
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        const int j = i < n_layers ? i : 0;
        g.packed[i] = (const uint8_t *)packed[j];
        g.sv[i] = (const f16 *)sv[j];
        g.part[i] = part[j];
        g.m[i] = (int)m[j];
        if (m[j] > max_m) max_m = m[j];
    }
#define GLQH_FI(RR, XT, TP) launch_mma_fusein<RR, XT, TP>(g, n_layers, max_m, x, x_stride, B, k, in_features, S, \
                                                          ksplit, bn_meta, blocks_host, n_blocks, pscale, stream)
#define GLQH_FI_R(RR)                                                                   \
    (B == 1 ? (x_dtype == GLQH_F16 ? GLQH_FI(RR, f16, 1) : GLQH_FI(RR, uint16_t, 1))     \
            : (x_dtype == GLQH_F16 ? GLQH_FI(RR, f16, 4) : GLQH_FI(RR, uint16_t, 4)))
    switch (R) {
    case 1: return GLQH_FI_R(1);                               // second stage of the 5 bpw recipe
    case 2: return GLQH_FI_R(2);
    case 3: return GLQH_FI_R(3);
    case 4: return GLQH_FI_R(4);
    }
#undef GLQH_FI_R
#undef GLQH_FI
    return glqh_fail("fused-input trellis kernel supports R (bits/weight) 1-4, got %d", R);
}

// One token through both stages of stacked layers (4 + R2 bits/weight each, 1..GLQH_MAX_GROUP layers on the same
// token) in one launch: part[l][K slot][row].
int glqh_launch_trellis_mma_fusein_rvq(const void *const packed[], const void *const packed2[], int R2, const float rs2[],
                                       const void *const sv[], float *const part[], const int64_t m[], int n_layers,
                                       const void *x, int x_dtype, int64_t x_stride, int64_t k, int64_t in_features,
                                       int S, int ksplit, const glqh_block_meta *bn_meta, const int64_t *blocks_host,
                                       int n_blocks, hipStream_t stream) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(n_layers >= 1 && n_layers <= GLQH_MAX_GROUP, "trellis group: 1..%d layers", GLQH_MAX_GROUP);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "fused-input trellis kernel: x must be f16 or bf16");
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    const glqh_block_meta *meta = n_blocks > 1 ? bn_meta : nullptr;
    const int nb = n_blocks > 1 ? n_blocks : 1;
    const size_t lds = fi_lds_bytes<1>(S);
    tr_fusein_group g = {};
    tr_fusein_group_rvq g2 = {};
    int64_t max_m = 0;
    for (int i = 0; i < GLQH_MAX_GROUP; ++i) {
        const int j = i < n_layers ? i : 0;
        g.packed[i] = (const uint8_t *)packed[j];
        g.sv[i] = (const f16 *)sv[j];
        g.part[i] = part[j];
        g.m[i] = (int)m[j];
        g2.packed2[i] = (const uint8_t *)packed2[j];
        g2.rs2[i] = rs2[j];
        if (m[j] > max_m) max_m = m[j];
    }
    const dim3 grid((unsigned)((max_m + 63) / 64), (unsigned)ksplit, (unsigned)n_layers);
#define GLQH_FI2(RR, XT)                                                                                        \
    do {                                                                                                        \
        if (n_layers == 1)                                                                                      \
            hipLaunchKernelGGL((tr_mma_fusein_rvq_kernel<RR, XT>), grid, dim3(TR_THREADS), lds, stream,         \
                               g.packed[0], g2.packed2[0], g2.rs2[0], (const XT *)x, x_stride, g.sv[0], g.m[0], \
                               (int)k, (int)in_features, S, meta, nb, margs, g.part[0]);                        \
        else                                                                                                    \
            hipLaunchKernelGGL((tr_mma_fusein_group_rvq_kernel<RR, XT>), grid, dim3(TR_THREADS), lds, stream, g, g2, \
                               (const XT *)x, x_stride, (int)k, (int)in_features, S, meta, nb, margs);          \
    } while (0)
#define GLQH_FI2_R(RR)                                                \
    do {                                                              \
        if (x_dtype == GLQH_F16) GLQH_FI2(RR, f16);                   \
        else GLQH_FI2(RR, uint16_t);                                  \
    } while (0)
    switch (R2) {
    case 1: GLQH_FI2_R(1); break;
    case 2: GLQH_FI2_R(2); break;
    case 3: GLQH_FI2_R(3); break;
    case 4: GLQH_FI2_R(4); break;
    default: return glqh_fail("fused-input trellis kernel: second stage of 1-4 bits/weight, got %d", R2);
    }
#undef GLQH_FI2_R
#undef GLQH_FI2
    GLQH_LAUNCH_CHECK("trellis fused-input two-stage launch");
    return 0;
}

template <int R, typename XT>
static int launch_mma_fusein_moe(const tr_moe_args &g, const void *x, int64_t x_stride, const void *sv, int64_t m,
                                 int64_t k, int64_t in_features, int S, int ksplit, const glqh_block_meta *bn_meta,
                                 const int64_t *blocks_host, int n_blocks, hipStream_t stream) {
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    const glqh_block_meta *meta = n_blocks > 1 ? bn_meta : nullptr;
    const int nb = n_blocks > 1 ? n_blocks : 1;
    dim3 grid((unsigned)((m + 63) / 64), (unsigned)ksplit, (unsigned)g.n_slots);
    hipLaunchKernelGGL((tr_mma_fusein_moe_kernel<R, XT>), grid, dim3(TR_THREADS), fi_lds_bytes<1>(S), stream, g,
                       (const XT *)x, x_stride, (const f16 *)sv, (int)m, (int)k, (int)in_features, S, meta, nb, margs);
    GLQH_LAUNCH_CHECK("trellis routed-expert gemv launch");
    return 0;
}

// One projection of all routed experts: part[K slot][slot][row], one token per slot.
int glqh_launch_trellis_mma_fusein_moe(const void *packed, int64_t stride_bytes, int R, const int64_t *topk_ids,
                                       int n_slots, int n_experts, int x_div, const float *pscale_dev,
                                       const void *x, int x_dtype, int64_t x_stride, const void *sv, int64_t m,
                                       int64_t k, int64_t in_features, int S, int ksplit, float *part,
                                       const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                                       hipStream_t stream) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(n_slots >= 1 && n_slots <= 65535, "routed experts: %d slots (1..65535)", n_slots);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "routed experts: x must be f16 or bf16");
    tr_moe_args g;
    g.packed = (const uint8_t *)packed;
    g.stride_bytes = stride_bytes;
    g.topk_ids = topk_ids;
    g.pscale_dev = pscale_dev;
    g.part = part;
    g.n_slots = n_slots;
    g.n_experts = n_experts;
    g.x_div = x_div;
#define GLQH_MOE(RR)                                                                                      \
    (x_dtype == GLQH_F16                                                                                  \
         ? launch_mma_fusein_moe<RR, f16>(g, x, x_stride, sv, m, k, in_features, S, ksplit, bn_meta,      \
                                          blocks_host, n_blocks, stream)                                  \
         : launch_mma_fusein_moe<RR, uint16_t>(g, x, x_stride, sv, m, k, in_features, S, ksplit, bn_meta, \
                                               blocks_host, n_blocks, stream))
    switch (R) {
    case 1: return GLQH_MOE(1);
    case 2: return GLQH_MOE(2);
    case 3: return GLQH_MOE(3);
    case 4: return GLQH_MOE(4);
    }
#undef GLQH_MOE
    return glqh_fail("routed experts: R (bits/weight) 1-4, got %d", R);
}

// Both stages of two-stage experts (4 + R2 bits/weight) per slot in one launch: part[K slot][slot][row] =
// sum1 + inv_rs2_dev[expert] * sum2.
int glqh_launch_trellis_mma_fusein_moe_rvq(const void *packed, int64_t stride_bytes, const void *packed2,
                                           int64_t stride2_bytes, int R2, const float *inv_rs2_dev,
                                           const int64_t *topk_ids, int n_slots, int n_experts, int x_div, const void *x,
                                           int x_dtype, int64_t x_stride, const void *sv, int64_t m, int64_t k,
                                           int64_t in_features, int S, int ksplit, float *part,
                                           const glqh_block_meta *bn_meta, const int64_t *blocks_host, int n_blocks,
                                           hipStream_t stream) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(n_slots >= 1 && n_slots <= 65535, "routed experts: %d slots (1..65535)", n_slots);
    GLQH_REQUIRE(x_dtype == GLQH_F16 || x_dtype == GLQH_BF16, "routed experts: x must be f16 or bf16");
    GLQH_REQUIRE(inv_rs2_dev && packed2, "routed experts: second stage missing");
    tr_moe_args g;
    g.packed = (const uint8_t *)packed;
    g.stride_bytes = stride_bytes;
    g.topk_ids = topk_ids;
    g.pscale_dev = inv_rs2_dev;
    g.part = part;
    g.n_slots = n_slots;
    g.n_experts = n_experts;
    g.x_div = x_div;
    glqh_meta_args margs;
    if (!glqh_fill_meta_args(&margs, blocks_host, n_blocks, k)) margs.canon = 0;
    const glqh_block_meta *meta = n_blocks > 1 ? bn_meta : nullptr;
    const int nb = n_blocks > 1 ? n_blocks : 1;
    const dim3 grid((unsigned)((m + 63) / 64), (unsigned)ksplit, (unsigned)n_slots);
#define GLQH_MOE2(RR, XT)                                                                                          \
    hipLaunchKernelGGL((tr_mma_fusein_moe_rvq_kernel<RR, XT>), grid, dim3(TR_THREADS), fi_lds_bytes<1>(S), stream, g, \
                       (const uint8_t *)packed2, stride2_bytes, (const XT *)x, x_stride, (const f16 *)sv, (int)m,  \
                       (int)k, (int)in_features, S, meta, nb, margs)
#define GLQH_MOE2_R(RR)                                               \
    do {                                                              \
        if (x_dtype == GLQH_F16) GLQH_MOE2(RR, f16);                  \
        else GLQH_MOE2(RR, uint16_t);                                 \
    } while (0)
    switch (R2) {
    case 1: GLQH_MOE2_R(1); break;
    case 2: GLQH_MOE2_R(2); break;
    case 3: GLQH_MOE2_R(3); break;
    case 4: GLQH_MOE2_R(4); break;
    default: return glqh_fail("routed experts: second stage of 1-4 bits/weight, got %d", R2);
    }
#undef GLQH_MOE2_R
#undef GLQH_MOE2
    GLQH_LAUNCH_CHECK("trellis routed-expert two-stage gemv launch");
    return 0;
}

static int moe_wide_min_rows() {                                // GLQ_MOE_WIDE_MIN_ROWS: average rows per expert
    static const int v = [] {
        const char *e = getenv("GLQ_MOE_WIDE_MIN_ROWS");
        const int n = e ? atoi(e) : 12;
        return n < 1 ? 1 : n;
    }();
    return v;
}

// One projection of all routed experts, rows grouped by expert: part[K slot][slot][row].
// 1: the grouped launch of this many slots takes up to 64 rows per pass (an average of GLQ_MOE_WIDE_MIN_ROWS rows
// per expert, 12 unless set)
int glqh_moe_grouped_wide(int n_slots, int n_experts) {
    return (int64_t)n_slots >= (int64_t)moe_wide_min_rows() * n_experts;
}

// packed2 (with stride2_bytes, R2; R = 4; passes of 16 rows only): stacked experts, both streams in the same passes,
// the second one's sums times pscale_dev[expert] added in registers.  (With the passes of up to 64 rows the second
// set of accumulators costs the occupancy: 166 registers, 256 tokens of 6 bpw experts 421 -> 578 us; those keep a
// launch per stage.)
int glqh_launch_trellis_mma_moe_grouped(const void *packed, int64_t stride_bytes, int R, const int *perm,
                                        const int *offs, int n_slots, int n_experts, int x_div,
                                        const float *pscale_dev, const void *x_f16, int64_t m, int64_t k, int S,
                                        int ksplit, float *part, hipStream_t stream, const void *packed2,
                                        int64_t stride2_bytes, int R2) {
    glqh_range range("dequant_matmul");
    GLQH_REQUIRE(!packed2 || (R == 4 && pscale_dev), "routed experts: two streams per pass need a 4-bit first stage and the residual scales");
    GLQH_REQUIRE(n_experts >= 1 && n_experts <= 65535 && n_slots >= 1 && x_div >= 1,
                 "routed experts: %d experts (1..65535), %d slots", n_experts, n_slots);
    GLQH_REQUIRE(S >= 1 && ksplit >= 1 && (int64_t)S * ksplit >= k / 32, "routed experts: K plan does not cover the row");
    // Wide passes from an average of 12 rows per expert on (a third of the experts then has more than 16).
    const bool wide = glqh_moe_grouped_wide(n_slots, n_experts) != 0;
    GLQH_REQUIRE(!(packed2 && wide), "routed experts: two streams per pass are served with passes of 16 rows only");
    // chunk of the one-tile pass as in tr_mma_kernel; the wider passes take what the same LDS holds
    moe_chunks ch;
    ch.ch1 = mma_chunk_cap<16, 1>();
    ch.ch2 = std::max(4, (ch.ch1 / 2) & ~3);
    ch.ch4 = std::max(4, (ch.ch1 / 4) & ~3);
    const int s4 = (S + 3) & ~3;
    ch.ch1 = std::min(ch.ch1, s4);
    ch.ch2 = std::min(ch.ch2, s4);
    ch.ch4 = std::min(ch.ch4, s4);
    size_t lds = std::max({(size_t)ch.ch1 * mma_slot_bytes(16, 1), (size_t)ch.ch2 * mma_slot_bytes(16, 2),
                           (size_t)ch.ch4 * mma_slot_bytes(16, 4), (size_t)mma_red_bytes<16, 4>()});
    tr_moe_group_args g = {(const uint8_t *)packed, stride_bytes, (const uint8_t *)packed2, stride2_bytes, perm, offs,
                           pscale_dev, part, n_slots, x_div};
    const dim3 grid((unsigned)((m + 63) / 64), (unsigned)ksplit, (unsigned)n_experts);
    if (packed2) {
#define GLQH_MOEG2(RR)                                                                                          \
    hipLaunchKernelGGL((tr_mma_moe_grouped_kernel<4, false, RR>), grid, dim3(TR_THREADS), lds, stream, g,        \
                       (const f16 *)x_f16, (int)m, (int)k, S, ch)
        switch (R2) {
        case 1: GLQH_MOEG2(1); break;
        case 2: GLQH_MOEG2(2); break;
        case 3: GLQH_MOEG2(3); break;
        case 4: GLQH_MOEG2(4); break;
        default: return glqh_fail("routed experts: second stage of 1-4 bits/weight, got %d", R2);
        }
#undef GLQH_MOEG2
        GLQH_LAUNCH_CHECK("trellis grouped routed-expert two-stage launch");
        return 0;
    }
#define GLQH_MOEG(RR)                                                                                        \
    do {                                                                                                     \
        if (wide)                                                                                            \
            hipLaunchKernelGGL((tr_mma_moe_grouped_kernel<RR, true>), grid, dim3(TR_THREADS), lds, stream, g, \
                               (const f16 *)x_f16, (int)m, (int)k, S, ch);                                    \
        else                                                                                                 \
            hipLaunchKernelGGL((tr_mma_moe_grouped_kernel<RR, false>), grid, dim3(TR_THREADS), lds, stream, g, \
                               (const f16 *)x_f16, (int)m, (int)k, S, ch);                                    \
    } while (0)
    switch (R) {
    case 1: GLQH_MOEG(1); break;
    case 2: GLQH_MOEG(2); break;
    case 3: GLQH_MOEG(3); break;
    case 4: GLQH_MOEG(4); break;
    default: return glqh_fail("routed experts: R (bits/weight) 1-4, got %d", R);
    }
#undef GLQH_MOEG
    GLQH_LAUNCH_CHECK("trellis grouped routed-expert launch");
    return 0;
}

template <typename K>
static int fi_set_lds(K kernel, size_t bytes) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)bytes),
                          "trellis fused-input attribute");
}

template <int R>
static int fi_init_R() {
    const size_t b1 = fi_lds_bytes<1>(FI_MAX_S), b4 = fi_lds_bytes<4>(FI_MAX_S_TP4);
    if (fi_set_lds(tr_mma_fusein_moe_kernel<R, f16>, b1) || fi_set_lds(tr_mma_fusein_moe_kernel<R, uint16_t>, b1)) return 1;
    if (fi_set_lds(tr_mma_fusein_moe_rvq_kernel<R, f16>, b1) || fi_set_lds(tr_mma_fusein_moe_rvq_kernel<R, uint16_t>, b1))
        return 1;
    if (fi_set_lds(tr_mma_fusein_rvq_kernel<R, f16>, b1) || fi_set_lds(tr_mma_fusein_rvq_kernel<R, uint16_t>, b1)) return 1;
    if (fi_set_lds(tr_mma_fusein_group_rvq_kernel<R, f16>, b1) || fi_set_lds(tr_mma_fusein_group_rvq_kernel<R, uint16_t>, b1))
        return 1;
    return fi_set_lds(tr_mma_fusein_kernel<R, f16, 1>, b1) || fi_set_lds(tr_mma_fusein_kernel<R, uint16_t, 1>, b1) ||
           fi_set_lds(tr_mma_fusein_kernel<R, f16, 4>, b4) || fi_set_lds(tr_mma_fusein_kernel<R, uint16_t, 4>, b4) ||
           fi_set_lds(tr_mma_fusein_group_kernel<R, f16, 1>, b1) ||
           fi_set_lds(tr_mma_fusein_group_kernel<R, uint16_t, 1>, b1) ||
           fi_set_lds(tr_mma_fusein_group_kernel<R, f16, 4>, b4) ||
           fi_set_lds(tr_mma_fusein_group_kernel<R, uint16_t, 4>, b4);
}

int glqh_trellis_mma_init(void) {
    return mma_init_R<1>() || mma_init_R<2>() || mma_init_R<3>() || mma_init_R<4>() ||
           fi_init_R<1>() || fi_init_R<2>() || fi_init_R<3>() || fi_init_R<4>();
}
