// E8 shell codebook GEMV / small-batch GEMM on the matrix cores with the table in LDS
// (gfx950, wave64).
//
// One 16-bit index stands for 8 consecutive weights of one row (glq/codebook.py:280-282):
// exactly the A operand a lane supplies to v_mfma_f32_16x16x32_f16 (row L & 15, k-group
// L >> 4, eight consecutive k).  A lane reads a 16-byte run of 8 indices of its row, looks
// each one up, expands the eight 4-bit codes to fp16 and issues one MFMA per index against
// the 8 activations of the same columns (B operand, 16 bytes per token, from LDS).  Up to
// 16 tokens share the decode.
//
// The lookup is what bounds this codebook: a random 4-byte gather from L2 sustains well
// under one lane per clock and CU, an LDS gather about twenty times that.  The nibble-packed
// table is 256 KiB and LDS 160 KiB, but the table is sorted by norm and both the first-stage
// indices and, more so, the residual-stage indices concentrate on the low-norm shells, so
// each workgroup keeps the first P entries (a launch parameter, ~120-144 KiB) in LDS and
// sends only the tail to L2.  Lanes that hit LDS all point their L2 load at entry 0, so the
// loads stay unconditional (exact wait counts) and coalesce.  Workgroups are persistent
// (one per CU, 16 waves) so the table prefix is loaded once per CU and launch.
//
// Work split: tile = (16*WR rows) x (one K slot); the 16 waves of a workgroup form WR row
// groups x WK k-parts (WK = 4 for up to 4 tokens, 1 above); k-parts are summed through LDS
// in a fixed order; every stage keeps its own accumulator and partial sum, combined by the
// consumer in stage order (glq/quantized_linear.py:1177-1194).
#include "e8_device.h"

namespace {


constexpr int EM_WAVES = 16;
constexpr int EM_THREADS = EM_WAVES * GLQH_WAVE;
constexpr int EM_STEP_BLKS = 32;               // 8-column blocks a wave covers per step

// FOLD: the folded form of the streams (glqh_e8_fold_table / glqh_e8_fold_indices).  The 65536
// codewords of the shell table are built from only 1286 distinct half codewords (columns 0..3 or
// 4..7 with their signs), so a table of those as finished fp16 values (8 bytes each, 10 KB) fits
// LDS whole: a lookup is two 8-byte LDS reads that are the MFMA operand as they arrive, no lookup
// leaves the CU and nothing is expanded.  An index becomes two 11-bit half numbers, stored as a
// 16-bit word (first half | low 5 bits of the second << 11) and a byte (its high 6 bits): 3 bytes
// instead of 2.
template <int NS, bool FOLD>
struct em_idx {
    u32x4 v[NS];                               // 8 indices per stage, two per dword
    u32x2 sg[FOLD ? NS : 1];                   // FOLD: their 8 high bytes
};

struct em_signs {
    const uint8_t *p[4];                       // byte planes of the folded form, (m_pad, n_pad / 8) bytes per stage
};

template <int NS, bool FOLD>
__device__ __forceinline__ em_idx<NS, FOLD> em_load_idx(const uint16_t *const q[4], const em_signs &sp, int64_t off) {
    em_idx<NS, FOLD> r;
#pragma unroll
    for (int s = 0; s < NS; ++s) {
        r.v[s] = __builtin_nontemporal_load((const u32x4 *)(q[s] + off));
        if constexpr (FOLD) r.sg[s] = __builtin_nontemporal_load((const u32x2 *)(sp.p[s] + off));
    }
    return r;
}

template <int NS, int TP, int WK, bool FOLD>
__global__ void __launch_bounds__(EM_THREADS)
e8_mma_kernel(const uint16_t *__restrict__ q1, const uint16_t *__restrict__ q2,
              const uint16_t *__restrict__ q3, const uint16_t *__restrict__ q4, em_signs sp,
              const uint32_t *__restrict__ t1, const uint32_t *__restrict__ t2, uint32_t n1, uint32_t n2,
              int t2_is_t1, const f16 *__restrict__ x, int B, int m_pad, int n_pad, int P, int slot_blks,
              int xs_slots, int ksplit, int ns_total, int s_off, float *__restrict__ part,
              glqh_e8_pscale ps, int direct) {                  // ps.v[s]: factor of stage s_off + s
                                                                // direct (one K slot, WK > 1): part is the (B, m_pad)
                                                                // result, the scaled stage sums added in stage order
    constexpr int WR = EM_WAVES / WK;
    constexpr int ROWS = 16 * WR;
    extern __shared__ u32x4 lds[];
    uint32_t *tab = (uint32_t *)lds;                           // P words (FOLD: the stage-1 half codewords, two
                                                               // words each, then stage 2's if they differ)
    u32x4 *xs = lds + P / 4;                                   // xs_slots slots, then 8*TP zero slots
    const int nblk = n_pad >> 3;
    const int lane = threadIdx.x & 63;
    const int wave = threadIdx.x >> 6;
    const int wr = wave / WK, wk = wave % WK;
    const int i = lane & 15, g = lane >> 4;
    const bool live = i < TP;                                  // token column of this lane
    u32x4 *zero_slots = xs + xs_slots;

    const uint16_t *const qs[4] = {q1, q2, q3, q4};
    const int RB = (m_pad + ROWS - 1) / ROWS;
    const int ntiles = RB * ksplit;
    const uint32_t P2 = t2_is_t1 ? (uint32_t)P : 0u;           // a separate stage-2 table stays in L2

    // The wave's steps over all of its workgroup's tiles form one sequence; the index runs
    // of the next steps are requested while step n is looked up, across tile boundaries,
    // and the first ones before the table is copied in.
    const int spt = slot_blks / (WK * EM_STEP_BLKS);           // steps per tile
    const int my_tiles = (ntiles - (int)blockIdx.x + (int)gridDim.x - 1) / (int)gridDim.x;
    const int nsteps = my_tiles * spt;
    auto idx_offset = [&](int sidx) -> int64_t {
        sidx = min(sidx, nsteps - 1);
        const int tile = blockIdx.x + (sidx / spt) * gridDim.x;
        const int slot = tile / RB, rb = tile % RB;
        const int row = rb * ROWS + wr * 16 + i;
        const int b0 = slot * slot_blks + ((sidx % spt) * WK + wk) * EM_STEP_BLKS;
        if constexpr (FOLD) {                                  // tile (16 rows, 32 indices), 8 entries per lane
            const int col_tiles = (nblk + 31) >> 5, row_tiles = (m_pad + 15) >> 4;
            const int rt = min(rb * WR + wr, row_tiles - 1), ct = min(b0 >> 5, col_tiles - 1);
            return (((int64_t)rt * col_tiles + ct) * 64 + lane) * 8;
        }
        return (int64_t)min(row, m_pad - 1) * nblk + min(b0 + 8 * g, nblk - 8);
    };
    // a step whose 32 blocks all lie past the row (the last slot of a row that is not a multiple of the
    // step round) is skipped: no index run is requested for it, nothing is looked up (uniform over the wave)
    auto step_live = [&](int sidx) -> bool {
        if (sidx >= nsteps) return false;
        const int tile = blockIdx.x + (sidx / spt) * gridDim.x;
        return (tile / RB) * slot_blks + ((sidx % spt) * WK + wk) * EM_STEP_BLKS < nblk;
    };
    em_idx<NS, FOLD> cur = em_load_idx<NS, FOLD>(qs, sp, idx_offset(0));
    // On the indices the runs of steps n + 1 and n + 2 are in flight while step n is looked up.  The folded
    // form requests one step ahead only: with more in flight the waves' requests queue up behind each other
    // in the memory system (4096 x 14336, one token, whole call: three steps ahead 16.7 us, two 15.0, one 13.7).
    em_idx<NS, FOLD> nx1 = cur;
    if (!FOLD && step_live(1)) nx1 = em_load_idx<NS, FOLD>(qs, sp, idx_offset(1));
    // FOLD: byte offset of stage 2's half codewords inside tab
    const uint32_t n1r = (n1 + 1u) & ~1u;
    const uint32_t tab2_off = t2_is_t1 ? 0u : 8u * n1r;

    // activations of a slot: one 16-byte LDS slot per (block, token), zero past B and n_pad
    auto x_load = [&](int sb0, int j) -> u32x4 {
        j = min(j, slot_blks * TP - 1);
        const int tl = j / slot_blks, blk = j % slot_blks;
        const u32x4 ld = *(const u32x4 *)(x + (int64_t)min(tl, B - 1) * n_pad + 8 * min(sb0 + blk, nblk - 1));
        return (tl < B && sb0 + blk < nblk) ? ld : u32x4{0u, 0u, 0u, 0u};
    };
    auto x_store = [&](int j, u32x4 v) {
        if (j < slot_blks * TP) xs[(j % slot_blks) * TP + j / slot_blks] = v;
    };
    // The first round of the first tile's activations is requested first, then the table prefix,
    // as loads that write LDS directly (1 KB per wave and instruction, no registers in between).
    // (P is a multiple of 1024 entries, so a wave's 64 x 16 bytes lie inside the prefix or outside.
    // Running the first step on L2 lookups alone while the table arrives was tried: that step then
    // asks L2 for six times the lines of a normal one, 36.4 us per call against 28.2.)
    {
        constexpr int U = 10;                                  // 10 * 1024 * 16 bytes = 160 KiB >= P * 4
        u32x4 xv[4];
        const int sb0 = ((int)blockIdx.x / RB) * slot_blks;
#pragma unroll
        for (int u = 0; u < 4; ++u) xv[u] = x_load(sb0, u * EM_THREADS + (int)threadIdx.x);
        if constexpr (FOLD) {
            for (uint32_t j = threadIdx.x; j < 2u * n1; j += EM_THREADS) tab[j] = t1[j];
            if (!t2_is_t1)
                for (uint32_t j = threadIdx.x; j < 2u * n2; j += EM_THREADS) tab[2u * n1r + j] = t2[j];
        } else {
#pragma unroll
            for (int u = 0; u < U; ++u) {
                if ((u * EM_WAVES + wave) * GLQH_WAVE < P / 4)     // uniform over the wave
                    __builtin_amdgcn_global_load_lds((const u32x4 *)t1 + u * EM_THREADS + threadIdx.x,
                                                     lds + (u * EM_WAVES + wave) * GLQH_WAVE, 16, 0, 0);
            }
        }
#pragma unroll
        for (int u = 0; u < 4; ++u) x_store(u * EM_THREADS + (int)threadIdx.x, xv[u]);
    }
    for (int j = threadIdx.x; j < 8 * TP; j += EM_THREADS) zero_slots[j] = u32x4{0u, 0u, 0u, 0u};

    const int nblk_r = (nblk + EM_STEP_BLKS - 1) / EM_STEP_BLKS * EM_STEP_BLKS;
    int sidx = 0;
    for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        const int slot = tile / RB, rb = tile % RB;
        const int sb0 = slot * slot_blks;
        const bool first = tile == (int)blockIdx.x;
        if (!first) __syncthreads();                           // previous tile is done with xs
        for (int j0 = first ? 4 * EM_THREADS : 0; j0 < slot_blks * TP; j0 += 4 * EM_THREADS) {
            u32x4 v[4];
#pragma unroll
            for (int u = 0; u < 4; ++u) v[u] = x_load(sb0, j0 + u * EM_THREADS + (int)threadIdx.x);
#pragma unroll
            for (int u = 0; u < 4; ++u) x_store(j0 + u * EM_THREADS + (int)threadIdx.x, v[u]);
        }
        __syncthreads();                                       // (first tile: also drains the table loads)

        f32x4 acc[NS];
#pragma unroll
        for (int s = 0; s < NS; ++s) acc[s] = f32x4{0.f, 0.f, 0.f, 0.f};

        for (int st = 0; st < spt; ++st, ++sidx) {
            const int b0 = sb0 + (st * WK + wk) * EM_STEP_BLKS;  // blocks [b0, b0+32), lane's run b0 + 8g
            const u32x4 *xl = live ? xs + (b0 - sb0 + 8 * g) * TP + i : zero_slots;
            if constexpr (FOLD) {
                em_idx<NS, FOLD> nxt = cur;
                if (step_live(sidx + 1)) nxt = em_load_idx<NS, FOLD>(qs, sp, idx_offset(sidx + 1));   // uniform
                const char *tb = (const char *)tab;
                if (b0 < nblk) {                               // uniform
#pragma unroll
                for (int h = 0; h < 2; ++h) {                  // four lookups per stage at a time: 32 registers of operands
                    u32x4 af[NS][4];
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const int t = 4 * h + u;
#pragma unroll
                        for (int s = 0; s < NS; ++s) {
                            const uint32_t w = cur.v[s][t >> 1], sw = cur.sg[s][t >> 2];
                            // byte offsets 8 * half number: first half from bits 0..10 of the index's 16-bit
                            // word, second from its bits 11..15 and the index's byte
                            const uint32_t lo = t & 1 ? (w >> 13) & 0x3FF8u : (w << 3) & 0x3FF8u;
                            const uint32_t h5 = t & 1 ? (w >> 24) & 0xF8u : (w >> 8) & 0xF8u;
                            const uint32_t b6 = u == 0 ? (sw << 8) & 0x3F00u : u == 1 ? sw & 0x3F00u
                                              : u == 2 ? (sw >> 8) & 0x3F00u : (sw >> 16) & 0x3F00u;
                            const char *tbs = tb + (s == 1 ? tab2_off : 0u);
                            const u32x2 c03 = *(const u32x2 *)(tbs + lo), c47 = *(const u32x2 *)(tbs + (h5 | b6));
                            af[s][u] = u32x4{c03[0], c03[1], c47[0], c47[1]};
                        }
                    }
#pragma unroll
                    for (int u = 0; u < 4; ++u) {
                        const f16x8 bf = __builtin_bit_cast(f16x8, xl[(4 * h + u) * TP]);
#pragma unroll
                        for (int s = 0; s < NS; ++s)
                            acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(__builtin_bit_cast(f16x8, af[s][u]), bf, acc[s], 0, 0, 0);
                    }
                }
                }
                cur = nxt;
                continue;
            }
            // all lookups of the step first: LDS for the prefix, L2 for the tail
            uint32_t wl[NS][8], wg[NS][8];
            bool hit[NS][8];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    uint32_t idx = (cur.v[s][t >> 1] >> (16 * (t & 1))) & 0xFFFFu;
                    const uint32_t *tg = s == 1 ? t2 : t1;
                    const uint32_t pre = s == 1 ? P2 : (uint32_t)P;
                    if (s == 1) idx = min(idx, n2 - 1);
                    // hits read LDS and aim their L2 load at one shared entry; misses the reverse
                    hit[s][t] = idx < pre;
                    wg[s][t] = tg[max(idx, pre)];
                    wl[s][t] = tab[min(idx, (uint32_t)P - 1)];
                }
            }
            // requested after the lookups, so that waiting for those does not wait for this
            em_idx<NS, FOLD> nx2 = nx1;
            if (step_live(sidx + 2)) nx2 = em_load_idx<NS, FOLD>(qs, sp, idx_offset(sidx + 2));   // uniform
            if (b0 < nblk_r) {                                 // uniform; past the row the activations are zero
#pragma unroll
                for (int t = 0; t < 8; ++t) {
                    const f16x8 bf = __builtin_bit_cast(f16x8, xl[t * TP]);
#pragma unroll
                    for (int s = 0; s < NS; ++s) {
                        const f16x8 af = em_expand(hit[s][t] ? wl[s][t] : wg[s][t]);
                        acc[s] = __builtin_amdgcn_mfma_f32_16x16x32_f16(af, bf, acc[s], 0, 0, 0);
                    }
                }
            }
            cur = nx1;
            nx1 = nx2;
        }

        // lane holds rows 4g .. 4g+3 of token i (D layout of the 16x16 MFMA)
        if constexpr (WK == 1) {
            if (live && i < B) {
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int r = 0; r < 4; ++r) {
                        const int orow = rb * ROWS + wr * 16 + 4 * g + r;
                        if (orow < m_pad) part[(((int64_t)slot * ns_total + s_off + s) * B + i) * m_pad + orow] = ps.v[s] * acc[s][r];
                    }
            }
        } else {
            __syncthreads();                                   // xs is free: reuse it for the k-part sums
            float *red = (float *)xs;                          // [WK][NS][TP][ROWS]
            if (live) {
#pragma unroll
                for (int s = 0; s < NS; ++s)
#pragma unroll
                    for (int r = 0; r < 4; ++r)
                        red[((wk * NS + s) * TP + i) * ROWS + wr * 16 + 4 * g + r] = acc[s][r];
            }
            __syncthreads();
            for (int e = threadIdx.x; e < NS * TP * ROWS; e += EM_THREADS) {
                const int rl = e % ROWS, tl = (e / ROWS) % TP, s = e / (ROWS * TP);
                const int orow = rb * ROWS + rl;
                if (tl >= B || orow >= m_pad) continue;
                float v = red[e];
#pragma unroll
                for (int w = 1; w < WK; ++w) v += red[w * NS * TP * ROWS + e];
                if (!direct) part[(((int64_t)slot * ns_total + s_off + s) * B + tl) * m_pad + orow] = ps.v[s] * v;
                else red[e] = ps.v[s] * v;                     // own element: nobody else reads or writes it
            }
            if (direct) {                                      // uniform
                __syncthreads();
                for (int e = threadIdx.x; e < TP * ROWS; e += EM_THREADS) {
                    const int rl = e % ROWS, tl = e / ROWS;
                    const int orow = rb * ROWS + rl;
                    if (tl >= B || orow >= m_pad) continue;
                    float v = red[e];
#pragma unroll
                    for (int s = 1; s < NS; ++s) v += red[s * TP * ROWS + e];
                    part[(int64_t)tl * m_pad + orow] = v;
                }
            }
        }
    }
}

struct em_plan {
    int TP, WK, P, slot_blks, xs_slots, ksplit, grid;
    size_t lds;
};

constexpr size_t EM_LDS_TOTAL = 160 * 1024;

// 0 when the shape is better served by the plain gather kernel
int em_make_plan(int64_t m_pad, int64_t n_pad, int64_t B, int64_t n1, bool fold, em_plan *p) {
    const int64_t nblk = n_pad / 8;
    if (B < 1 || B > 16 || nblk < 8 || (nblk & 7) || n1 < 4096) return 0;
    // the table load would dominate (2048 x 2048, two stages, whole linear: 15.7 us here against
    // 13.3 us with L2 gathers at one token, 16.5 against 16.6 at four; 3072 x 3072: 18.6 against 21.3;
    // on folded streams, whose table is small, the two kernels tie below these sizes: 960 x 960 11.9
    // against 10.1 us, 2048 x 2048 12.8 against 12.4, 1024 x 4096 13.2 against 13.4)
    if (m_pad * n_pad < (B == 1 ? (int64_t)6 << 20 : (int64_t)1 << 22)) return 0;
    p->TP = B == 1 ? 1 : B <= 4 ? 4 : 16;
    // 5..16 tokens on folded streams: LDS has room for 512-block slots of sixteen tokens (128 KB), so four
    // K parts x 64-row tiles instead of 256-row tiles with up to sixteen K slots for the finishing kernel
    // (whole two-stage linear at 16 tokens: 2048 x 2048 17.8 -> 15.0 us, 3072 x 3072 19.8 -> 15.6,
    // 2048 x 11008 25.6 -> 21.7; unfused 14336 x 4096 20.2 -> 19.0; not for rows of more than 1536 blocks:
    // 4096 x 14336 21.1 -> 24.3, every workgroup then stages 128 KB of activations for four steps)
    p->WK = p->TP == 16 ? (fold && nblk <= 1536 ? 4 : 1) : 4;
    // On folded streams (no table to speak of in LDS, room for whole rows of activations) all sixteen waves
    // of a workgroup split K among themselves when 16-row tiles fill the chip at most once and the row fits:
    // no K slot leaves the workgroup and the sums can be written finished (4096 x 14336, whole unfused call
    // at one token: 19.1 -> 17.7 us with the reduction launch kept, 15.8 without; at four tokens 20.1 -> 18.8;
    // whole linear 4096 x 4096 at sixteen tokens 25.8 -> 19.6.  Not taken: 14336 x 4096, 896 such tiles,
    // 17.6 -> 21.7 us; 4096 x 14336 at sixteen tokens, a row of 448 KB in four slots, 21.1 -> 39.3)
    if (fold && (m_pad + 15) / 16 <= glqh_device_cus() && nblk >= 16 * EM_STEP_BLKS && nblk <= (p->TP == 16 ? 512 : 2048))
        p->WK = 16;                                              // the whole row of activations in 128 KB / 32 KB of LDS
    const int rows = 16 * (EM_WAVES / p->WK);
    const int64_t RB = (m_pad + rows - 1) / rows;
    const int unit = p->WK * EM_STEP_BLKS;                      // blocks per workgroup step
    const int64_t nunits = (nblk + unit - 1) / unit;
    // activations: at most 32 KB of LDS; slots as long as that allows, so that a workgroup has one
    // tile (and one table fill per tile) where the shape permits
    const int slot_cap_blks = p->WK == 16 ? (p->TP == 16 ? 512 : 2048) : p->TP == 16 ? (p->WK == 4 ? 512 : 128) : 512;   // 128 KB / 32 KB of activations
    const int cus = glqh_device_cus();
    int64_t ks = RB >= cus ? 1 : cus / RB;                      // one tile per workgroup where possible
    if (ks > nunits) ks = nunits;
    if (ks < 1) ks = 1;
    int64_t slot_units = (nunits + ks - 1) / ks;
    if (slot_units * unit > slot_cap_blks) slot_units = slot_cap_blks / unit;
    if (slot_units < 1) slot_units = 1;
    p->slot_blks = (int)(slot_units * unit);
    p->ksplit = (int)((nunits + slot_units - 1) / slot_units);
    // LDS: activations (or the k-part sums that reuse their space) + 8*TP zero slots + table
    size_t xbytes = (size_t)p->slot_blks * p->TP * 16;
    const size_t red = (size_t)p->WK * 4 * p->TP * rows * sizeof(float);
    if (p->WK > 1 && xbytes < red) xbytes = red;
    p->xs_slots = (int)(xbytes / 16);
    const size_t rest = xbytes + (size_t)8 * p->TP * 16;
    int64_t P = (int64_t)((EM_LDS_TOTAL - rest) / 4) & ~(int64_t)1023;
    if (P > n1) P = n1 & ~(int64_t)3;
    p->P = (int)P;
    p->lds = (size_t)P * 4 + rest;
    const int64_t ntiles = RB * p->ksplit;
    p->grid = (int)(ntiles < cus ? ntiles : cus);
    return 1;
}

template <int NS, int TP, int WK, bool FOLD>
int em_launch(const em_plan &p, const void *x, int64_t B, const void *const q[4], const em_signs &sp,
              const uint32_t *t1, const uint32_t *t2, int64_t n1, int64_t n2, int64_t m_pad, int64_t n_pad,
              int ns_total, int s_off, float *part, hipStream_t stream, glqh_e8_pscale ps, int direct = 0) {
    hipLaunchKernelGGL((e8_mma_kernel<NS, TP, WK, FOLD>), dim3((unsigned)p.grid), dim3(EM_THREADS), p.lds, stream,
                       (const uint16_t *)q[0], (const uint16_t *)q[1], (const uint16_t *)q[2],
                       (const uint16_t *)q[3], sp, t1, t2, (uint32_t)n1, (uint32_t)n2, (int)(t1 == t2 && n1 == n2),
                       (const f16 *)x, (int)B, (int)m_pad, (int)n_pad, p.P, p.slot_blks, p.xs_slots, p.ksplit,
                       ns_total, s_off, part, ps, direct);
    GLQH_LAUNCH_CHECK("e8 mma launch");
    return 0;
}

template <int NS, bool FOLD>
int em_launch_NS(const em_plan &p, const void *x, int64_t B, const void *const q[4], const em_signs &sp,
                 const uint32_t *t1, const uint32_t *t2, int64_t n1, int64_t n2, int64_t m_pad, int64_t n_pad,
                 int ns_total, int s_off, float *part, hipStream_t stream, const float *pscale, int direct = 0) {
    glqh_e8_pscale ps = {{1.0f, 1.0f, 1.0f, 1.0f}};
    if (pscale)
        for (int i = 0; i + s_off < 4; ++i) ps.v[i] = pscale[s_off + i];
#define GLQH_EM(TP, WK) em_launch<NS, TP, WK, FOLD>(p, x, B, q, sp, t1, t2, n1, n2, m_pad, n_pad, ns_total, s_off, \
                                                    part, stream, ps, direct)
    if (p.TP == 1 && p.WK == 16) return GLQH_EM(1, 16);
    if (p.TP == 4 && p.WK == 16) return GLQH_EM(4, 16);
    if (p.TP == 16 && p.WK == 16) return GLQH_EM(16, 16);
    if (p.TP == 1) return GLQH_EM(1, 4);
    if (p.TP == 4) return GLQH_EM(4, 4);
    if (p.TP == 16 && p.WK == 4) return GLQH_EM(16, 4);
    return GLQH_EM(16, 1);
#undef GLQH_EM
}

template <typename K>
int em_set_lds(K kernel) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)EM_LDS_TOTAL),
                          "e8 mma attribute");
}

template <int NS>
int em_init_NS() {
    return em_set_lds(e8_mma_kernel<NS, 1, 4, false>) || em_set_lds(e8_mma_kernel<NS, 4, 4, false>) ||
           em_set_lds(e8_mma_kernel<NS, 16, 1, false>) || em_set_lds(e8_mma_kernel<NS, 1, 4, true>) ||
           em_set_lds(e8_mma_kernel<NS, 4, 4, true>) || em_set_lds(e8_mma_kernel<NS, 16, 1, true>) ||
           em_set_lds(e8_mma_kernel<NS, 1, 16, true>) || em_set_lds(e8_mma_kernel<NS, 1, 16, false>) ||
           em_set_lds(e8_mma_kernel<NS, 4, 16, true>) || em_set_lds(e8_mma_kernel<NS, 4, 16, false>) ||
           em_set_lds(e8_mma_kernel<NS, 16, 16, true>) || em_set_lds(e8_mma_kernel<NS, 16, 16, false>) ||
           em_set_lds(e8_mma_kernel<NS, 16, 4, true>) || em_set_lds(e8_mma_kernel<NS, 16, 4, false>);
}

}  // namespace

int glqh_e8_mma_init(void) { return em_init_NS<1>() || em_init_NS<2>(); }

// ksplit of the LDS-table kernel for this call, or 0 when the shape is not eligible
int glqh_e8_mma_ksplit(int64_t m_pad, int64_t n_pad, int64_t B, int64_t n1, int fold) {
    em_plan p;
    return em_make_plan(m_pad, n_pad, B, n1, fold != 0, &p) ? p.ksplit : 0;
}

// One launch covers two stages (the register budget of the three-deep pipeline); layers of
// three and four stages take a second launch for stages 3-4, which index the primary table.
// fold: the folded streams of the same layer (then q and the tables are not read).
int glqh_launch_e8_mma(const void *x, int64_t B, const void *const q[4], int nstages, const uint32_t *t1,
                       int64_t n1, const uint32_t *t2, int64_t n2, int64_t m_pad, int64_t n_pad, float *part,
                       hipStream_t stream, const float *pscale, const glqh_e8_folded *fold, int direct) {
    em_plan p;
    if (!em_make_plan(m_pad, n_pad, B, n1, fold != nullptr, &p)) return glqh_fail("e8 mma: shape not eligible");
    if (nstages < 1 || nstages > 4) return glqh_fail("e8 matmul: %d stages unsupported (1-4)", nstages);
    if (fold) {
        const bool own2 = nstages >= 2 && fold->halves2 && fold->halves2 != fold->halves1;
        const uint32_t *a1 = (const uint32_t *)fold->halves1, *a2 = own2 ? (const uint32_t *)fold->halves2 : a1;
        const int64_t na1 = fold->n_halves1, na2 = own2 ? fold->n_halves2 : fold->n_halves1;
        GLQH_REQUIRE(a1 && na1 >= 1 && na1 <= 2048 && na2 >= 1 && na2 <= 2048, "e8 folded: 1..2048 half codewords per table");
        for (int s = 0; s < nstages; ++s)
            GLQH_REQUIRE(fold->lo16[s] && fold->hi8[s], "e8 folded: stage %d has no folded stream", s + 1);
        // LDS: stage-1 half codewords (two words each), stage 2's if they are a table of their own
        const size_t rest = p.lds - (size_t)p.P * 4;
        em_plan p12 = p, p34 = p;
        p12.P = (int)(2 * ((na1 + 1) & ~(int64_t)1) + (own2 ? 2 * ((na2 + 1) & ~(int64_t)1) : 0));
        p12.lds = (size_t)p12.P * 4 + rest;
        p34.P = (int)(2 * ((na1 + 1) & ~(int64_t)1));
        p34.lds = (size_t)p34.P * 4 + rest;
        const void *const i12[4] = {fold->lo16[0], fold->lo16[nstages >= 2 ? 1 : 0], fold->lo16[0], fold->lo16[0]};
        const em_signs s12 = {{fold->hi8[0], fold->hi8[nstages >= 2 ? 1 : 0], fold->hi8[0], fold->hi8[0]}};
        GLQH_REQUIRE(!direct || (p.WK > 1 && p.ksplit == 1 && nstages <= 2), "e8 folded: finished sums need one K slot");
        if (nstages == 1)
            return em_launch_NS<1, true>(p12, x, B, i12, s12, a1, a1, na1, na1, m_pad, n_pad, 1, 0, part, stream, pscale, direct);
        if (em_launch_NS<2, true>(p12, x, B, i12, s12, a1, a2, na1, na2, m_pad, n_pad, nstages, 0, part, stream, pscale, direct))
            return 1;
        if (nstages == 2) return 0;
        const void *const i34[4] = {fold->lo16[2], fold->lo16[nstages == 4 ? 3 : 2], fold->lo16[2], fold->lo16[2]};
        const em_signs s34 = {{fold->hi8[2], fold->hi8[nstages == 4 ? 3 : 2], fold->hi8[2], fold->hi8[2]}};
        if (nstages == 3) return em_launch_NS<1, true>(p34, x, B, i34, s34, a1, a1, na1, na1, m_pad, n_pad, 3, 2, part, stream, pscale);
        return em_launch_NS<2, true>(p34, x, B, i34, s34, a1, a1, na1, na1, m_pad, n_pad, 4, 2, part, stream, pscale);
    }
    GLQH_REQUIRE(!direct, "e8 mma: finished sums are an option of the folded form");
    const em_signs none = {{nullptr, nullptr, nullptr, nullptr}};
    if (nstages == 1) return em_launch_NS<1, false>(p, x, B, q, none, t1, t2, n1, n2, m_pad, n_pad, 1, 0, part, stream, pscale);
    if (em_launch_NS<2, false>(p, x, B, q, none, t1, t2, n1, n2, m_pad, n_pad, nstages, 0, part, stream, pscale)) return 1;
    if (nstages == 2) return 0;
    const void *const q34[4] = {q[2], q[3], q[2], q[3]};
    if (nstages == 3) return em_launch_NS<1, false>(p, x, B, q34, none, t1, t1, n1, n1, m_pad, n_pad, 3, 2, part, stream, pscale);
    return em_launch_NS<2, false>(p, x, B, q34, none, t1, t1, n1, n1, m_pad, n_pad, 4, 2, part, stream, pscale);
}

// 1 when a call of this shape on folded streams keeps K inside the workgroups (one K slot, K parts summed
// in LDS), so that up to two stages can be written as finished sums without a reduction launch
int glqh_e8_mma_direct_ok(int64_t m_pad, int64_t n_pad, int64_t B, int nstages) {
    em_plan p;
    return em_make_plan(m_pad, n_pad, B, 65536, true, &p) && p.WK > 1 && p.ksplit == 1 && nstages <= 2;
}
