// E8 shell codebook GEMM for many tokens on the compressed indices (gfx950, wave64).
//
// Y_rht[token, row] = sum_k X_rht[token, k] * W[row, k] with W[row, 8j..8j+7] = cb[q1[row, j]]
// + r2 * cb2[q2[row, j]] + ... (glq/codebook.py:280-282, glq/quantized_linear.py:1177-1194;
// the reference's tensor-core kernel for B >= 2 is glq/csrc/glq_cuda.cu:791-955).  Looking an
// index up and expanding its eight 4-bit codes costs far more than the eight multiply-adds of
// one token, so a decoded weight has to meet as many tokens as possible:
//
//   workgroup tile = 128 rows x (128 * NTW) tokens, 8 waves (two per SIMD);
//   wave w DECODES row fragment w (16 rows) of every 64-column step into LDS, in the operand
//   layout of v_mfma_f32_16x16x32_f16 (lane L's 16 bytes at slot L: conflict-free both ways),
//   and MULTIPLIES all 8 row fragments, read back from LDS, with ITS OWN 16 * NTW tokens, whose
//   activations it holds in registers, straight from global memory.
//
// The B operand of the MFMA puts consecutive tokens in consecutive lanes, so row-major activations
// would be read as 64 scattered 16-byte pieces per instruction (one lane per clock in the memory
// pipeline: measured 2.7 us per 64-column step and CU, three times the multiplications).  They are
// repacked once per call (or written that way by the input transform) into groups of four
// 8-column blocks with the token as the next index, xb[k / 32][token][(k / 8) % 4][k % 8], which
// turns every operand load of a wave into two runs of 512 contiguous bytes and keeps the 32
// columns of one token together (64 bytes) for whoever writes them.
//
// Every weight is therefore looked up once per 128 * NTW tokens (once per 512 at NTW = 4), the
// B operands never pass through LDS, and LDS carries 16 KB of A operands per step and CU.  The
// table's low-norm prefix (32768 entries, 128 KB) lives in LDS as in the small-batch kernel
// (e8_mma.hip); the tail is read from L2.  Stages are combined into one fp16 operand per stage
// in sequence, a = fma(c_s, r_s, a) in fp16 (the reference rounds to fp16 after every stage as
// well, glq/csrc/glq_cuda.cu:868-899).  Workgroups are persistent (one per CU) and walk tiles in
// an order that gives the CUs of one XCD the same tokens at the same time, so the activations
// are served by that XCD's L2.  K is split into slots only while the tiles alone would leave CUs
// idle; partial sums [slot][token][row] are combined in slot order by the consumer.
//
// FOLD: the same kernel on the folded streams (glqh_e8_fold_table / glqh_e8_fold_indices, e8_mma.hip):
// an index is two 11-bit half-codeword numbers, the table of half codewords as finished fp16 values
// (at most 16 KB per table) sits in LDS whole, and a lookup is two 8-byte LDS reads whose result is
// the operand: no table word comes from L2, nothing is expanded, 128 KB of table fill per workgroup
// fall away.  The fp16 values and the stage arithmetic are the same, so the results are bit-identical.
#include "e8_device.h"

namespace {

constexpr int ET_WAVES = 8;
constexpr int ET_THREADS = ET_WAVES * GLQH_WAVE;
constexpr int ET_FRAGS = 8;                        // 16-row fragments per tile, one per wave
constexpr int ET_ROWS = 16 * ET_FRAGS;
constexpr int ET_P = 32767;                        // table entries kept in LDS; word ET_P is a sentinel
constexpr int ET_SMALL_TOKENS = 256;               // up to here the folded form runs e8_tile_small_kernel
constexpr uint32_t ET_MISS = 0xFFFFFFFFu;          // no table word has a code above 12
constexpr int ET_BUF = 2 * ET_FRAGS * GLQH_WAVE;   // 16-byte slots per A buffer: 2 sub-steps x 8 fragments
constexpr size_t ET_LDS = (size_t)(ET_P + 1) * 4 + (size_t)2 * ET_BUF * 16;   // 128 KB + 32 KB
constexpr int ET_EP_STRIDE = ET_ROWS + 4;          // floats per token of a wave's output staging space (FOLD)
constexpr size_t ET_EP_BYTES = (size_t)ET_WAVES * 16 * ET_EP_STRIDE * sizeof(float);   // 66 KB

struct et_args {
    const uint16_t *q[4];                          // FOLD: the 16-bit words of the folded streams
    const uint8_t *hi8[4];                         // FOLD: their byte planes
    const uint32_t *t1, *t2;                       // FOLD: half-codeword tables, two words per entry
    uint32_t n2;
    uint32_t nh1, nh2;                             // FOLD: entries of the half-codeword tables
    int t2_is_t1;
    float r[3];                                    // factors of stages 2..4 relative to stage 1
    const f16 *xb;                                 // transformed activations, (n_pad / 32, Mp, 4, 8) fp16
    int Mp;                                        // M rounded up to whole token tiles
    int M, m_pad, n_pad;
    int RT, TT, KS, slot_ds;                       // row tiles, token tiles, K slots, 64-column steps per slot
    float *part;                                   // [slot][token][row]
    int staged;                                    // FOLD: sums leave through LDS (m_pad % 4 == 0; % 8 with out_f16)
    int out_f16;                                   // FOLD, staged: sums as fp16, times scale
    float scale;
};

__device__ __forceinline__ void et_barrier() {     // waits for LDS only: global prefetches stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

template <int NS, int NTW, bool FOLD>
__global__ void __launch_bounds__(ET_THREADS)
e8_tile_kernel(const et_args a) {
    extern __shared__ u32x4 lds[];
    const uint32_t *tab = (const uint32_t *)lds;
    // FOLD: stage 1's half codewords (an even number of 8-byte entries), then stage 2's if they differ
    const uint32_t nh1r = (a.nh1 + 1u) & ~1u, nh2r = (a.nh2 + 1u) & ~1u;
    const uint32_t tab2_off = a.t2_is_t1 ? 0u : 8u * nh1r;     // bytes
    u32x4 *abuf = lds + (FOLD ? (nh1r + (a.t2_is_t1 ? 0u : nh2r)) / 2 : (uint32_t)(ET_P + 1) / 4);
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int nblk = a.n_pad >> 3, nds = a.n_pad >> 6;
    constexpr int NFB = FOLD ? NS : 1;                         // stages with a byte run

    if constexpr (FOLD) {
        uint32_t *tw = (uint32_t *)lds;
        for (uint32_t j = threadIdx.x; j < 2u * a.nh1; j += ET_THREADS) tw[j] = a.t1[j];
        if (!a.t2_is_t1)
            for (uint32_t j = threadIdx.x; j < 2u * a.nh2; j += ET_THREADS) tw[2u * nh1r + j] = a.t2[j];
    } else {
        // table prefix -> LDS, all loads of a round in flight before its first write
        constexpr int PER = (ET_P + 1) / 4 / ET_THREADS;       // 16 x 16 bytes per thread
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            u32x4 v[PER / 2];
#pragma unroll
            for (int u = 0; u < PER / 2; ++u) v[u] = ((const u32x4 *)a.t1)[(h * (PER / 2) + u) * ET_THREADS + threadIdx.x];
#pragma unroll
            for (int u = 0; u < PER / 2; ++u) lds[(h * (PER / 2) + u) * ET_THREADS + threadIdx.x] = v[u];
        }
    }
    __syncthreads();
    if (!FOLD && threadIdx.x == 0) ((uint32_t *)lds)[ET_P] = ET_MISS;   // what a lookup past the prefix reads
    __syncthreads();

    // a separate stage-2 table stays in L2: its LDS lookups are all sent to the sentinel
    const uint32_t P2 = a.t2_is_t1 ? (uint32_t)ET_P : 0u, force2 = a.t2_is_t1 ? 0u : 0xFFFFu;
    f16x2 rs[3];
#pragma unroll
    for (int s = 0; s < 3; ++s) rs[s] = f16x2{(f16)a.r[s], (f16)a.r[s]};

    // Workgroups with equal blockIdx % 8 run on one XCD and share its L2: each XCD takes a
    // contiguous range of the item list, whose fastest index is the row tile, so its CUs read
    // the same activations at the same time.
    const int nitems = a.TT * a.KS * a.RT;
    const int per_xcd = (nitems + 7) >> 3;
    const int xcd = blockIdx.x & 7, bx = blockIdx.x >> 3;
    const int nbx = ((int)gridDim.x - xcd + 7) >> 3;
    for (int w = bx; w < per_xcd; w += nbx) {
        const int item = xcd * per_xcd + w;
        if (item >= nitems) break;                              // uniform
        const int rt = item % a.RT, slot = (item / a.RT) % a.KS, tt0 = item / (a.RT * a.KS);
        const int r0 = rt * ET_ROWS, tok0 = tt0 * (ET_WAVES * 16 * NTW) + wave * 16 * NTW;
        const int ds0 = slot * a.slot_ds, ds1 = min(ds0 + a.slot_ds, nds);

        // decode role: row fragment `wave`; lane (i, g) owns blocks 8d + 2g, 8d + 2g + 1 of step d
        const int drow = min(r0 + 16 * wave + i, a.m_pad - 1);
        const u32x4 *qrow[NS];                                  // 8 indices = the 64 columns of step 4q + g
#pragma unroll
        for (int s = 0; s < NS; ++s) qrow[s] = (const u32x4 *)(a.q[s] + (int64_t)drow * nblk) + (ds0 >> 2) * 4 + g;
        // FOLD: a stream tile is 16 rows x 32 indices = this wave's rows x one group of four steps; lane
        // (i, g) holds indices 8g .. 8g+7 of row i at entry 8 * lane
        const int64_t fbase = (((int64_t)min((r0 >> 4) + wave, ((a.m_pad + 15) >> 4) - 1) * (nblk >> 5) + (ds0 >> 2)) * 64 + lane) * 8;
        // multiply role: token 16 * tt + i of the wave's tokens, blocks 8d + 2g and 8d + 2g + 1
        // (the token dimension of xb is padded to whole tiles: no clamping, constant offsets)
        // block 8 d + 2 g + u of step d: group of four blocks 2 d + (g >> 1), position 2 (g & 1) + u
        const int64_t kstep = (int64_t)a.Mp * 64;               // elements from one 64-column step to the next
        const f16 *xrow = a.xb + (int64_t)(g >> 1) * a.Mp * 32 + (int64_t)(tok0 + i) * 32 + (g & 1) * 16;

        // Every load below is unconditional with a clamped step index, so the wait counts the
        // compiler derives are exact and nothing waits for a request younger than the one it needs.
        // The L2 words of a step are requested LA steps before its operands are expanded (hits aim
        // their load at one shared entry); the LDS words are read at expansion time from the index
        // pairs, which travel with the L2 words (misses read the sentinel).
        struct looked {
            uint32_t wg[NS][2], pair[NS];
        };
        auto index_of = [&](uint32_t pair, int s, int u) {
            uint32_t idx = (pair >> (16 * u)) & 0xFFFFu;
            if (s == 1) idx = min(idx, a.n2 - 1);
            return idx;
        };
        auto lookups = [&](const uint32_t (&T)[NS][4], int dd) {
            looked r;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                r.pair[s] = T[s][dd];
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint32_t *tg = s == 1 ? a.t2 : a.t1;
                    const uint32_t pre = s == 1 ? P2 : (uint32_t)ET_P;
                    r.wg[s][u] = tg[max(index_of(r.pair[s], s, u), pre)];
                }
            }
            return r;
        };
        struct lds_words {
            uint32_t w[NS][2];
        };
        auto lds_lookups = [&](const looked &r) {
            lds_words wl;
#pragma unroll
            for (int s = 0; s < NS; ++s)
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint32_t idx = index_of(r.pair[s], s, u);
                    wl.w[s][u] = tab[min(s == 1 ? idx | force2 : idx, (uint32_t)ET_P)];
                }
            return wl;
        };
        auto expand_half = [&](const looked &r, const lds_words &wlw, int u, u32x4 *dst) {   // one A fragment
            const auto &wl = wlw.w;
            {
                f16x8 af = em_expand(wl[0][u] != ET_MISS ? wl[0][u] : r.wg[0][u]);
#pragma unroll
                for (int s = 1; s < NS; ++s) {
                    const f16x8 e = em_expand(wl[s][u] != ET_MISS ? wl[s][u] : r.wg[s][u]);
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const f16x2 ev = {e[2 * p], e[2 * p + 1]}, av = {af[2 * p], af[2 * p + 1]};
                        const f16x2 rv = __builtin_elementwise_fma(ev, rs[s - 1], av);
                        af[2 * p] = rv[0];
                        af[2 * p + 1] = rv[1];
                    }
                }
                dst[(u * ET_FRAGS + wave) * GLQH_WAVE + lane] = __builtin_bit_cast(u32x4, af);
            }
        };
        auto emit = [&](const looked &r, u32x4 *dst) {          // two A fragments of this wave's rows
            const lds_words wl = lds_lookups(r);
            expand_half(r, wl, 0, dst);
            expand_half(r, wl, 1, dst);
        };
        // Index runs are requested 16 bytes per lane, a whole group of four steps ahead of their
        // use.  Lane (i, g) receives the 8 indices of step 4q + g of its row, but in step 4q + dd
        // it decodes index pair g of that step: a 4 x 4 transpose of dwords over the four lanes
        // that share row i (lane distance 16), done with two pairs of lane-swap instructions.
        const int nquads = (ds1 - ds0) >> 2;
        auto load_quad = [&](u32x4 (&run)[NS], u32x2 (&runb)[NFB], int q) {
            q = min(q, nquads - 1);
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                if constexpr (FOLD) {
                    run[s] = __builtin_nontemporal_load((const u32x4 *)(a.q[s] + fbase + (int64_t)q * 512));
                    runb[FOLD ? s : 0] = __builtin_nontemporal_load((const u32x2 *)(a.hi8[s] + fbase + (int64_t)q * 512));
                } else {
                    run[s] = __builtin_nontemporal_load(qrow[s] + 4 * q);
                }
            }
        };
        auto transpose4 = [&](uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint32_t (&T)[4]) {
            const auto p02 = __builtin_amdgcn_permlane32_swap(d0, d2, false, false);
            const auto p13 = __builtin_amdgcn_permlane32_swap(d1, d3, false, false);
            const auto lo = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
            const auto hi = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
            T[0] = lo[0];
            T[1] = lo[1];
            T[2] = hi[0];
            T[3] = hi[1];
        };
        // T[s][dd] = the index pair this lane decodes in step dd; FOLD: TB[s][dd] = the pair's two bytes
        // in bits 0..15 (the 16-bit pieces of the byte run take the same way as the dwords of the word run)
        auto transpose = [&](const u32x4 (&run)[NS], const u32x2 (&runb)[NFB], uint32_t (&T)[NS][4], uint32_t (&TB)[NFB][4]) {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                transpose4(run[s][0], run[s][1], run[s][2], run[s][3], T[s]);
                if constexpr (FOLD) transpose4(runb[s][0], runb[s][0] >> 16, runb[s][1], runb[s][1] >> 16, TB[s]);   // s < NFB
            }
        };
        // FOLD: the half codewords of a step's two index pairs, as they come out of LDS
        struct halves {
            u32x2 c[NS][2][2];                                  // [stage][pair member][half]
        };
        auto fold_lookups = [&](const uint32_t (&T)[NS][4], const uint32_t (&TB)[NFB][4], int dd) {
            halves h;
            const char *tb = (const char *)tab;
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const uint32_t w = T[s][dd], by = TB[FOLD ? s : 0][dd];
                const char *tbs = tb + (s == 1 ? tab2_off : 0u);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    // byte offsets 8 * half number: first half from bits 0..10 of the index's 16-bit word,
                    // second from its bits 11..15 and the index's byte
                    const uint32_t lo = u ? (w >> 13) & 0x3FF8u : (w << 3) & 0x3FF8u;
                    const uint32_t h5 = u ? (w >> 24) & 0xF8u : (w >> 8) & 0xF8u;
                    const uint32_t b6 = u ? by & 0x3F00u : (by << 8) & 0x3F00u;
                    h.c[s][u][0] = *(const u32x2 *)(tbs + lo);
                    h.c[s][u][1] = *(const u32x2 *)(tbs + (h5 | b6));
                }
            }
            return h;
        };
        auto fold_emit_half = [&](const halves &h, int u, u32x4 *dst) {   // one A fragment
            f16x8 af = __builtin_bit_cast(f16x8, u32x4{h.c[0][u][0][0], h.c[0][u][0][1], h.c[0][u][1][0], h.c[0][u][1][1]});
#pragma unroll
            for (int s = 1; s < NS; ++s) {
                const f16x8 e = __builtin_bit_cast(f16x8, u32x4{h.c[s][u][0][0], h.c[s][u][0][1], h.c[s][u][1][0], h.c[s][u][1][1]});
#pragma unroll
                for (int p = 0; p < 4; ++p) {
                    const f16x2 ev = {e[2 * p], e[2 * p + 1]}, av = {af[2 * p], af[2 * p + 1]};
                    const f16x2 rv = __builtin_elementwise_fma(ev, rs[s - 1], av);
                    af[2 * p] = rv[0];
                    af[2 * p + 1] = rv[1];
                }
            }
            dst[(u * ET_FRAGS + wave) * GLQH_WAVE + lane] = __builtin_bit_cast(u32x4, af);
        };
        auto load_b = [&](u32x4 (&b)[NTW][2], int d) {
            d = min(d, ds1 - 1);
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) {
                b[tt][0] = *(const u32x4 *)(xrow + d * kstep + tt * 512);
                b[tt][1] = *(const u32x4 *)(xrow + d * kstep + 8 + tt * 512);
            }
        };

        f32x4 acc[ET_FRAGS][NTW];
#pragma unroll
        for (int f = 0; f < ET_FRAGS; ++f)
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) acc[f][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

        // Software pipeline over the 64-column steps.  At step d: the operands of d + 1 are expanded
        // into the other LDS buffer from table entries requested LA steps earlier, the entries of
        // d + 1 + LA are requested, and the activations of d + 1 are requested -- a whole step ahead
        // into a second register set where registers allow (NTW <= 2), otherwise half a step ahead
        // into the registers the half-step just multiplied has freed.  Index runs arrive a group of
        // four steps ahead.
        constexpr int LA = NTW <= 2 ? 2 : 1;
        // operand fragments read ahead of their multiplications: with one or two token tiles per wave a
        // fragment is multiplied in 16-32 matrix-pipe cycles, less than an LDS read takes; with four token
        // tiles two ahead changes nothing (527 against 525 us at 4096 tokens, one run) and costs registers
        constexpr int PF = NTW <= 2 ? 2 : 1;
        constexpr bool BDB = NTW <= 2;
        u32x4 run[NS];
        u32x2 runb[NFB];
        uint32_t T[NS][4], TB[NFB][4];
        u32x4 b[BDB ? 2 : 1][NTW][2];
        looked lk[LA];
        load_quad(run, runb, 0);
        load_b(b[0], ds0);
        transpose(run, runb, T, TB);
        load_quad(run, runb, 1);
        if constexpr (FOLD) {
            const halves first = fold_lookups(T, TB, 0);
            fold_emit_half(first, 0, abuf);
            fold_emit_half(first, 1, abuf);
        } else {
            const looked first = lookups(T, 0);
            emit(first, abuf);
            static_assert(LA <= 3, "the prologue requests entries from the first index group only");
#pragma unroll
            for (int j = 1; j <= LA; ++j) lk[j % LA] = lookups(T, j & 3);
        }
        et_barrier();

        for (int q = 0; q < nquads; ++q) {
#pragma unroll
            for (int dd = 0; dd < 4; ++dd) {
                const int d = ds0 + 4 * q + dd;
                const int cur = BDB ? (dd & 1) : 0, nxt = BDB ? (cur ^ 1) : 0;
                const u32x4 *rd = abuf + (dd & 1) * ET_BUF;
                u32x4 *wr = abuf + ((dd & 1) ^ 1) * ET_BUF;
                const int dn = min(d + 1, ds1 - 1);
                if constexpr (BDB) load_b(b[nxt], d + 1);
                looked lke, lkn;
                lds_words wle;
                halves hv;
                if constexpr (FOLD) {                           // the half codewords of d + 1
                    if (dd == 3) {                              // the next group's indices take over
                        transpose(run, runb, T, TB);
                        load_quad(run, runb, q + 2);
                    }
                    hv = fold_lookups(T, TB, (dd + 1) & 3);
                } else {
                    lke = lk[(dd + 1) % LA];                    // entries of d + 1: expanded during this step
                    wle = lds_lookups(lke);
                    const int sl = dd + 1 + LA;                 // step looked up now, relative to 4q
                    if ((sl & 3) == 0) {                        // its group's indices take over
                        transpose(run, runb, T, TB);
                        load_quad(run, runb, q + (sl >> 2) + 1);
                    }
                    lkn = lookups(T, sl & 3);
                }
                // 16 operand fragments (2 half-steps x 8 row fragments), each read from LDS one
                // fragment ahead of the multiplications that use it; the expansion of the next
                // step's operands is spread between them
                f16x8 ring[PF];
#pragma unroll
                for (int j = 0; j < PF; ++j) ring[j] = __builtin_bit_cast(f16x8, rd[j * GLQH_WAVE + lane]);
                __builtin_amdgcn_sched_barrier(0);              // requests stay ahead of the multiplications
#pragma unroll
                for (int k = 0; k < 2 * ET_FRAGS; ++k) {
                    const int u = k / ET_FRAGS, f = k % ET_FRAGS;
                    const f16x8 af = ring[k % PF];
                    if (k + PF < 2 * ET_FRAGS) ring[k % PF] = __builtin_bit_cast(f16x8, rd[(k + PF) * GLQH_WAVE + lane]);
#pragma unroll
                    for (int tt = 0; tt < NTW; ++tt)
                        acc[f][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                            af, __builtin_bit_cast(f16x8, b[cur][tt][u]), acc[f][tt], 0, 0, 0);
                    if constexpr (FOLD) {
                        if (k == 1) fold_emit_half(hv, 0, wr);  // operands of d + 1 (unused after the last step)
                        if (k == 9) fold_emit_half(hv, 1, wr);
                    } else {
                        if (k == 1) expand_half(lke, wle, 0, wr);
                        if (k == 9) expand_half(lke, wle, 1, wr);
                    }
                    if constexpr (!BDB) {
                        if (f == ET_FRAGS - 1) {                // this half's activations are free: request the next
                            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
                            for (int tt = 0; tt < NTW; ++tt) b[0][tt][u] = *(const u32x4 *)(xrow + dn * kstep + u * 8 + tt * 512);
                            __builtin_amdgcn_sched_barrier(0);
                        }
                    }
                }
                if constexpr (!FOLD) lk[(dd + 1) % LA] = lkn;
                et_barrier();                                   // rd has been read, wr is written
            }
        }

        // lane holds rows 4g .. 4g+3 of token i of every (fragment, token tile): sixteen bytes here, sixteen
        // bytes a whole row of sums further on for the next token -- stored like that a wave's instruction
        // touches 64 lines.  On the folded streams (whose tables leave the room) every wave passes its sums
        // through LDS once, its own 16 tokens x 128 rows in a space of its own (no barrier: a wave's LDS
        // operations complete in order), and stores whole runs of a token's rows: two tokens x 512 bytes per
        // instruction in fp32, four tokens x 256 bytes in fp16.
        if constexpr (FOLD) {
            if (a.staged) {                                     // uniform
                float *ep = (float *)(abuf + 2 * ET_BUF) + wave * (16 * ET_EP_STRIDE);
#pragma unroll
                for (int tt = 0; tt < NTW; ++tt) {
#pragma unroll
                    for (int f = 0; f < ET_FRAGS; ++f) *(f32x4 *)(ep + i * ET_EP_STRIDE + 16 * f + 4 * g) = acc[f][tt];
                    asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
                    if (a.out_f16) {
                        const int rl = 8 * (lane & 15), row = r0 + rl;
#pragma unroll 2
                        for (int j = 0; j < 4; ++j) {
                            const int tl = 4 * j + (lane >> 4), tok = tok0 + 16 * tt + tl;
                            const f32x4 v0 = *(const f32x4 *)(ep + tl * ET_EP_STRIDE + rl) * a.scale;
                            const f32x4 v1 = *(const f32x4 *)(ep + tl * ET_EP_STRIDE + rl + 4) * a.scale;
                            if (tok >= a.M || row >= a.m_pad) continue;   // m_pad is a multiple of 8: whole runs of eight
                            typedef _Float16 f16x8o __attribute__((ext_vector_type(8)));
                            *(f16x8o *)((f16 *)a.part + ((int64_t)slot * a.M + tok) * a.m_pad + row) =
                                f16x8o{(f16)v0[0], (f16)v0[1], (f16)v0[2], (f16)v0[3], (f16)v1[0], (f16)v1[1], (f16)v1[2], (f16)v1[3]};
                        }
                    } else {
                        const int rl = 4 * (lane & 31), row = r0 + rl;
#pragma unroll 2
                        for (int j = 0; j < 8; ++j) {
                            const int tl = 2 * j + (lane >> 5), tok = tok0 + 16 * tt + tl;
                            const f32x4 v = *(const f32x4 *)(ep + tl * ET_EP_STRIDE + rl);
                            if (tok >= a.M || row >= a.m_pad) continue;   // m_pad is a multiple of 4
                            *(f32x4 *)(a.part + ((int64_t)slot * a.M + tok) * a.m_pad + row) = v;
                        }
                    }
                }
                continue;
            }
        }
        const bool vec = (a.m_pad & 3) == 0;
#pragma unroll
        for (int tt = 0; tt < NTW; ++tt) {
            const int tok = tok0 + 16 * tt + i;
            if (tok >= a.M) continue;
            float *orow = a.part + ((int64_t)slot * a.M + tok) * a.m_pad;
#pragma unroll
            for (int f = 0; f < ET_FRAGS; ++f) {
                const int row = r0 + 16 * f + 4 * g;
                if (vec && row + 3 < a.m_pad) {
                    *(f32x4 *)(orow + row) = acc[f][tt];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (row + e < a.m_pad) orow[row + e] = acc[f][tt][e];
                }
            }
        }
    }
}

// 17..256 tokens on the folded streams: one token tile, one barrier per group of four steps.  With one token
// tile per wave every wave of the kernel above reads the whole 16 KB operand buffer of a step from LDS (128 KB
// per step and workgroup: 1024 LDS cycles for 256-512 cycles of multiplications), and at 17..64 tokens most
// waves multiply padding.  Here the 8 waves split the multiplications of a step by token group AND row
// fragment: TG = 2, 4 or 8 token groups of 16 NTW tokens, wave w takes token group w % TG and the row
// fragments w / TG + (8 / TG) j, j < TG -- 2 TG operand reads and 2 TG NTW MFMAs per wave and step, every
// product computed once.  Decoding is as above (wave w decodes row fragment w).
template <int NS, int TG, int NTW>
__global__ void __launch_bounds__(ET_THREADS)
e8_tile_small_kernel(const et_args a) {
    constexpr int RG = ET_FRAGS / TG;                          // row-fragment groups
    extern __shared__ u32x4 lds[];
    const uint32_t nh1r = (a.nh1 + 1u) & ~1u, nh2r = (a.nh2 + 1u) & ~1u;
    const uint32_t tab2_off = a.t2_is_t1 ? 0u : 8u * nh1r;     // bytes
    u32x4 *abuf = lds + (nh1r + (a.t2_is_t1 ? 0u : nh2r)) / 2;
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, g = lane >> 4;
    const int nblk = a.n_pad >> 3, nds = a.n_pad >> 6;
    const int tg = wave % TG, rg = wave / TG;
    {
        uint32_t *tw = (uint32_t *)lds;
        for (uint32_t j = threadIdx.x; j < 2u * a.nh1; j += ET_THREADS) tw[j] = a.t1[j];
        if (!a.t2_is_t1)
            for (uint32_t j = threadIdx.x; j < 2u * a.nh2; j += ET_THREADS) tw[2u * nh1r + j] = a.t2[j];
    }
    __syncthreads();
    f16x2 rs[3];
#pragma unroll
    for (int s = 0; s < 3; ++s) rs[s] = f16x2{(f16)a.r[s], (f16)a.r[s]};
    const char *tb = (const char *)lds;

    const int nitems = a.KS * a.RT;                            // one token tile
    for (int item = blockIdx.x; item < nitems; item += gridDim.x) {
        const int rt = item % a.RT, slot = item / a.RT;
        const int r0 = rt * ET_ROWS;
        const int ds0 = slot * a.slot_ds, ds1 = min(ds0 + a.slot_ds, nds);
        const int nquads = (ds1 - ds0) >> 2;
        const int64_t fbase = (((int64_t)min((r0 >> 4) + wave, ((a.m_pad + 15) >> 4) - 1) * (nblk >> 5) + (ds0 >> 2)) * 64 + lane) * 8;
        const int64_t kstep = (int64_t)a.Mp * 64;
        const f16 *xrow = a.xb + (int64_t)(g >> 1) * a.Mp * 32 + (int64_t)(16 * NTW * tg + i) * 32 + (g & 1) * 16;

        u32x4 run[NS];
        u32x2 runb[NS];
        uint32_t T[NS][4], TB[NS][4];
        auto load_quad = [&](int q) {
            q = min(q, nquads - 1);
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                run[s] = __builtin_nontemporal_load((const u32x4 *)(a.q[s] + fbase + (int64_t)q * 512));
                runb[s] = __builtin_nontemporal_load((const u32x2 *)(a.hi8[s] + fbase + (int64_t)q * 512));
            }
        };
        auto transpose4 = [&](uint32_t d0, uint32_t d1, uint32_t d2, uint32_t d3, uint32_t (&O)[4]) {
            const auto p02 = __builtin_amdgcn_permlane32_swap(d0, d2, false, false);
            const auto p13 = __builtin_amdgcn_permlane32_swap(d1, d3, false, false);
            const auto lo = __builtin_amdgcn_permlane16_swap(p02[0], p13[0], false, false);
            const auto hi = __builtin_amdgcn_permlane16_swap(p02[1], p13[1], false, false);
            O[0] = lo[0];
            O[1] = lo[1];
            O[2] = hi[0];
            O[3] = hi[1];
        };
        auto transpose = [&]() {
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                transpose4(run[s][0], run[s][1], run[s][2], run[s][3], T[s]);
                transpose4(runb[s][0], runb[s][0] >> 16, runb[s][1], runb[s][1] >> 16, TB[s]);
            }
        };
        // the two operand fragments (sub-steps u = 0, 1) of this wave's rows for the step whose index pair is
        // (T, TB)[.][dd]: looked up, stages combined, written in operand layout
        auto decode = [&](int dd, u32x4 *dst) {
            u32x2 c[NS][2][2];
#pragma unroll
            for (int s = 0; s < NS; ++s) {
                const uint32_t w = T[s][dd], by = TB[s][dd];
                const char *tbs = tb + (s == 1 ? tab2_off : 0u);
#pragma unroll
                for (int u = 0; u < 2; ++u) {
                    const uint32_t lo = u ? (w >> 13) & 0x3FF8u : (w << 3) & 0x3FF8u;
                    const uint32_t h5 = u ? (w >> 24) & 0xF8u : (w >> 8) & 0xF8u;
                    const uint32_t b6 = u ? by & 0x3F00u : (by << 8) & 0x3F00u;
                    c[s][u][0] = *(const u32x2 *)(tbs + lo);
                    c[s][u][1] = *(const u32x2 *)(tbs + (h5 | b6));
                }
            }
#pragma unroll
            for (int u = 0; u < 2; ++u) {
                f16x8 af = __builtin_bit_cast(f16x8, u32x4{c[0][u][0][0], c[0][u][0][1], c[0][u][1][0], c[0][u][1][1]});
#pragma unroll
                for (int s = 1; s < NS; ++s) {
                    const f16x8 e = __builtin_bit_cast(f16x8, u32x4{c[s][u][0][0], c[s][u][0][1], c[s][u][1][0], c[s][u][1][1]});
#pragma unroll
                    for (int p = 0; p < 4; ++p) {
                        const f16x2 ev = {e[2 * p], e[2 * p + 1]}, av = {af[2 * p], af[2 * p + 1]};
                        const f16x2 rv = __builtin_elementwise_fma(ev, rs[s - 1], av);
                        af[2 * p] = rv[0];
                        af[2 * p + 1] = rv[1];
                    }
                }
                dst[(u * ET_FRAGS + wave) * GLQH_WAVE + lane] = __builtin_bit_cast(u32x4, af);
            }
        };
        auto load_b = [&](u32x4 (&b)[NTW][2], int d) {
            d = min(d, ds1 - 1);
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) {
                b[tt][0] = *(const u32x4 *)(xrow + d * kstep + tt * 512);
                b[tt][1] = *(const u32x4 *)(xrow + d * kstep + 8 + tt * 512);
            }
        };

        f32x4 acc[TG][NTW];
#pragma unroll
        for (int j = 0; j < TG; ++j)
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) acc[j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};
        // One barrier per group of four steps (256 columns): the operands of a whole group are decoded into one
        // of two 64 KB buffers while the previous group is multiplied out of the other.  Activations are
        // requested three steps ahead (a step is a few hundred cycles, less than an L2 round trip), index runs
        // two groups ahead.
        u32x4 b[4][NTW][2];
        load_quad(0);
#pragma unroll
        for (int j = 0; j < 3; ++j) load_b(b[j], ds0 + j);
        transpose();
        load_quad(1);
        if (item != (int)blockIdx.x) et_barrier();              // the previous item's last buffer has been read
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) decode(dd, abuf + dd * ET_BUF);
        et_barrier();
        for (int q = 0; q < nquads; q += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {                       // group q + h: buffers and registers h
                if (q + h < nquads) {                           // uniform
                    const u32x4 *rd = abuf + h * 4 * ET_BUF + rg * GLQH_WAVE + lane;
                    u32x4 *wr = abuf + (h ^ 1) * 4 * ET_BUF;
                    transpose();                                // the next group's indices take over
                    load_quad(q + h + 2);
#pragma unroll
                    for (int dd = 0; dd < 4; ++dd) {
                        // operand k of the step: sub-step k / TG, fragment rg + RG (k % TG); read PF ahead
                        constexpr int NK = 2 * TG, PF = NK < 4 ? NK : 4;
                        auto frag = [&](int k) {
                            return __builtin_bit_cast(f16x8, rd[dd * ET_BUF + ((k / TG) * ET_FRAGS + RG * (k % TG)) * GLQH_WAVE]);
                        };
                        f16x8 ring[PF];
#pragma unroll
                        for (int k = 0; k < PF; ++k) ring[k] = frag(k);
                        load_b(b[(dd + 3) & 3], ds0 + 4 * (q + h) + dd + 3);
                        decode(dd, wr + dd * ET_BUF);           // operands of the next group (unused after the last)
#pragma unroll
                        for (int k = 0; k < NK; ++k) {
                            const f16x8 af = ring[k % PF];
                            if (k + PF < NK) ring[k % PF] = frag(k + PF);
#pragma unroll
                            for (int tt = 0; tt < NTW; ++tt)
                                acc[k % TG][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                    af, __builtin_bit_cast(f16x8, b[dd][tt][k / TG]), acc[k % TG][tt], 0, 0, 0);
                        }
                    }
                    et_barrier();                               // rd has been read, wr is written
                }
            }
        }
        // lane holds rows 4g .. 4g+3 of token i of every (fragment, token tile)
        const bool vec = (a.m_pad & 3) == 0;
#pragma unroll
        for (int tt = 0; tt < NTW; ++tt) {
            const int tok = 16 * NTW * tg + 16 * tt + i;
            if (tok >= a.M) continue;
            float *orow = a.part + ((int64_t)slot * a.M + tok) * a.m_pad;
#pragma unroll
            for (int j = 0; j < TG; ++j) {
                const int row = r0 + 16 * (rg + RG * j) + 4 * g;
                if (vec && row + 3 < a.m_pad) {
                    *(f32x4 *)(orow + row) = acc[j][tt];
                } else {
#pragma unroll
                    for (int e = 0; e < 4; ++e)
                        if (row + e < a.m_pad) orow[row + e] = acc[j][tt][e];
                }
            }
        }
    }
}

// (M, n_pad) row-major fp16 -> (n_pad / 32, Mp, 4, 8): 64 tokens x 16 blocks per workgroup through
// LDS, reads in runs of 256 bytes, writes in runs of 4 KB.
__global__ void __launch_bounds__(256)
e8_pack_blocked_kernel(const f16 *__restrict__ x, f16 *__restrict__ xb, int M, int Mp, int n_pad) {
    __shared__ u32x4 tile[16][65];
    const int tok0 = blockIdx.x * 64, kb0 = blockIdx.y * 16, nblk = n_pad >> 3;
    const int t = threadIdx.x;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int tl = r * 16 + (t >> 4), kb = t & 15;
        const int tok = min(tok0 + tl, M - 1), b = min(kb0 + kb, nblk - 1);
        tile[kb][tl] = *(const u32x4 *)(x + (int64_t)tok * n_pad + 8 * b);
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {                               // group of four blocks r: 64 tokens x 64 bytes contiguous
        const int tl = t >> 2, pos = t & 3, kb = 4 * r + pos;
        if (tok0 + tl < M && kb0 + kb < nblk)
            *(u32x4 *)(xb + ((((int64_t)(kb0 + kb) >> 2) * Mp + tok0 + tl) * 4 + pos) * 8) = tile[kb][tl];
    }
}

// token tiles per wave: 512-token workgroup tiles from 257 tokens on; layers of three and four stages
// stay at 256 (the registers of their longer lookup pipeline)
static int et_ntw(int64_t M, int nstages) {
    static const int forced = [] { const char *e = getenv("GLQ_ET_NTW"); return e ? atoi(e) : 0; }();
    if (forced && M > 256 && nstages <= 2) return forced;
    return M <= 128 ? 1 : (M <= 256 || nstages > 2) ? 2 : 4;
}

static int64_t et_padded_tokens(int64_t M, int nstages) {
    const int64_t tile = ET_WAVES * 16 * et_ntw(M, nstages);
    return (M + tile - 1) / tile * tile;
}

struct et_plan {
    int NTW, RT, TT, KS, slot_ds, grid;
};

// Widths the kernels walk: whole groups of four 64-column steps.  On folded streams a row of any multiple
// of 32 columns is served: the folded tiles are padded to 32 indices with the zero codeword and the blocked
// activations to the same width with zeros (the kernel's n_pad is then the padded width).
static int64_t et_width(int64_t n_pad) { return (n_pad + 255) / 256 * 256; }

static int et_plan_for(int NTW, int64_t m_pad, int64_t n_pad, int64_t M, et_plan *p) {
    p->NTW = NTW;
    const int tile_tok = ET_WAVES * 16 * p->NTW;
    p->RT = (int)((m_pad + ET_ROWS - 1) / ET_ROWS);
    p->TT = (int)((M + tile_tok - 1) / tile_tok);
    const int nds = (int)(n_pad / 64);
    const int cus = glqh_device_cus();
    const int64_t base = (int64_t)p->RT * p->TT;
    int64_t ks = 1;
    if (base < cus) {
        ks = cus / base;
        const int64_t cap_len = nds / 8 > 0 ? nds / 8 : 1;      // slots of at least 512 columns
        if (ks > cap_len) ks = cap_len;
        // partial sums stay under 128 MB
        const int64_t cap_bytes = ((int64_t)128 << 20) / (M * m_pad * 4);
        if (ks > cap_bytes) ks = cap_bytes;
        if (ks < 1) ks = 1;
    }
    p->slot_ds = (int)((nds / 4 + ks - 1) / ks) * 4;            // whole groups of four steps
    p->KS = (nds + p->slot_ds - 1) / p->slot_ds;
    const int64_t items = base * p->KS;
    p->grid = (int)(items < cus ? items : cus);
    return 1;
}

// Expected microseconds of a plan, as for the trellis tile kernel: rounds x steps x the time of a step (2.75 us
// with 512-token tiles, 1.65 with 256: two-stage layers on folded streams, full chip), a last round of at least
// half, +0.6 x the idle share when a single round leaves CUs idle, and the K slots' fp32 sums written and read
// at about 4 TB/s.
static double et_plan_cost(const et_plan &p, int64_t m_pad, int64_t M) {
    const int cus = glqh_device_cus();
    const int64_t items = (int64_t)p.RT * p.TT * p.KS;
    const int64_t full = items / cus, rem = items % cus;
    double rounds = (double)full, slow = 1.0;
    if (full == 0) {
        rounds = 1.0;
        slow = 1.0 + 0.6 * (1.0 - (double)items / cus);
    } else if (rem > 0) {
        rounds += std::max(0.5, (double)rem / cus);
    }
    double t = rounds * p.slot_ds * (p.NTW == 4 ? 2.75 : 1.65) * slow;
    if (p.KS > 1) t += 2.0 * p.KS * (double)M * (double)m_pad * 4.0 / 4.0e6;
    return t;
}

// Above 256 tokens: 512-token tiles (one- and two-stage layers) unless 256-token tiles are expected to be at
// least 5 % faster, which they are where row tiles are few (11008 x 11008 at 1024 tokens: 548 -> 384 us,
// 11008 x 2048: 151 -> 115).  GLQ_ET_NTW forces a tile.
int et_make_plan(int64_t m_pad, int64_t n_pad, int64_t M, int nstages, et_plan *p) {
    if (M < 1 || m_pad < 1 || n_pad < 256 || (n_pad & 255) || M > ((int64_t)1 << 22) || m_pad > ((int64_t)1 << 24))
        return 0;
    const int top = et_ntw(M, nstages);
    et_plan_for(top, m_pad, n_pad, M, p);
    static const bool forced = getenv("GLQ_ET_NTW") != nullptr;
    if (top < 4 || forced) return 1;
    et_plan p2;
    et_plan_for(2, m_pad, n_pad, M, &p2);
    if (et_plan_cost(p2, m_pad, M) < 0.95 * et_plan_cost(*p, m_pad, M)) *p = p2;
    return 1;
}

// FOLD: two tables of at most 2048 half codewords of 8 bytes, and the A buffers
constexpr size_t ET_LDS_FOLD = (size_t)2 * 2048 * 8 + (size_t)2 * ET_BUF * 16 + ET_EP_BYTES;

template <int NS, int NTW, bool FOLD>
int et_launch(const et_plan &p, const et_args &a, hipStream_t stream) {
    size_t lds = ET_LDS;
    if (FOLD) lds = (size_t)(((a.nh1 + 1u) & ~1u) + (a.t2_is_t1 ? 0u : (a.nh2 + 1u) & ~1u)) * 8 + (size_t)2 * ET_BUF * 16 + ET_EP_BYTES;
    hipLaunchKernelGGL((e8_tile_kernel<NS, NTW, FOLD>), dim3((unsigned)p.grid), dim3(ET_THREADS), lds, stream, a);
    GLQH_LAUNCH_CHECK("e8 tile launch");
    return 0;
}

template <int NS, bool FOLD>
int et_launch_NS(const et_plan &p, const et_args &a, hipStream_t stream) {
    if (p.NTW == 1) return et_launch<NS, 1, FOLD>(p, a, stream);
    if (p.NTW == 2) return et_launch<NS, 2, FOLD>(p, a, stream);
    if constexpr (NS <= 2) return et_launch<NS, 4, FOLD>(p, a, stream);
    return glqh_fail("e8 tile kernel: no 512-token tiles for %d stages", NS);
}

template <typename K>
int et_set_lds(K kernel, size_t bytes) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)bytes),
                          "e8 tile attribute");
}

template <int NS, int TG, int NTW>
int et_launch_small(const et_plan &p, const et_args &a, hipStream_t stream) {
    const size_t lds = (size_t)(((a.nh1 + 1u) & ~1u) + (a.t2_is_t1 ? 0u : (a.nh2 + 1u) & ~1u)) * 8 + (size_t)8 * ET_BUF * 16;
    hipLaunchKernelGGL((e8_tile_small_kernel<NS, TG, NTW>), dim3((unsigned)p.grid), dim3(ET_THREADS), lds, stream, a);
    GLQH_LAUNCH_CHECK("e8 small tile launch");
    return 0;
}

template <int NS>
int et_launch_small_NS(const et_plan &p, const et_args &a, hipStream_t stream) {
    if (a.M <= 32) return et_launch_small<NS, 2, 1>(p, a, stream);
    if (a.M <= 64) return et_launch_small<NS, 4, 1>(p, a, stream);
    if (a.M <= 128) return et_launch_small<NS, 8, 1>(p, a, stream);
    return et_launch_small<NS, 8, 2>(p, a, stream);
}

template <int NS>
int et_init_NS() {
    constexpr size_t small_lds = (size_t)2 * 2048 * 8 + (size_t)8 * ET_BUF * 16;    // 32 KB + 128 KB
    if (et_set_lds(e8_tile_small_kernel<NS, 2, 1>, small_lds) || et_set_lds(e8_tile_small_kernel<NS, 4, 1>, small_lds) ||
        et_set_lds(e8_tile_small_kernel<NS, 8, 1>, small_lds) || et_set_lds(e8_tile_small_kernel<NS, 8, 2>, small_lds))
        return 1;
    if (et_set_lds(e8_tile_kernel<NS, 1, false>, ET_LDS) || et_set_lds(e8_tile_kernel<NS, 2, false>, ET_LDS) ||
        et_set_lds(e8_tile_kernel<NS, 1, true>, ET_LDS_FOLD) || et_set_lds(e8_tile_kernel<NS, 2, true>, ET_LDS_FOLD))
        return 1;
    if constexpr (NS <= 2)
        return et_set_lds(e8_tile_kernel<NS, 4, false>, ET_LDS) || et_set_lds(e8_tile_kernel<NS, 4, true>, ET_LDS_FOLD);
    return 0;
}

}  // namespace

int glqh_e8_tile_init(void) { return et_init_NS<1>() || et_init_NS<2>() || et_init_NS<3>() || et_init_NS<4>(); }

// bytes of the repacked activations (the larger tile size bounds the padding; width padded as on folded streams)
size_t glqh_e8_tile_xb_bytes(int64_t n_pad, int64_t M) { return (size_t)et_padded_tokens(M, 1) * et_width(n_pad) * sizeof(f16); }

// K slots of the many-token kernel for this call, or 0 when the shape is not eligible: n_pad must be a
// multiple of 256 on the indices themselves, of 32 on folded streams
int glqh_e8_tile_ksplit(int64_t m_pad, int64_t n_pad, int64_t M, int nstages, int fold) {
    et_plan p;
    if (fold && n_pad >= 32 && (n_pad & 31) == 0) n_pad = et_width(n_pad);
    return et_make_plan(m_pad, n_pad, M, nstages, &p) ? p.KS : 0;
}

namespace {
__global__ void __launch_bounds__(256) et_zero_kernel(u32x4 *__restrict__ p, int64_t n16) {
    for (int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x; i < n16; i += (int64_t)gridDim.x * 256)
        p[i] = u32x4{0u, 0u, 0u, 0u};
}
}  // namespace

// fp16 sums are written by the large tiles of the folded form only
int glqh_e8_tile_f16_sums_ok(int64_t M, int fold, int64_t m_pad) { return fold && M > ET_SMALL_TOKENS && m_pad % 8 == 0; }

// part[(slot * M + token) * m_pad + row] = sum over the slot's columns of x[token, k] * W[row, k],
// W = cb[q0] + rel[0] * cb2[q1] + rel[1] * cb[q2] + rel[2] * cb[q3] (nstages terms), unscaled (fp32), or
// times f16_scale and rounded to fp16 with out_f16 (glqh_e8_tile_f16_sums_ok).
// x_f16 is (M, n_pad) row-major; xb_scratch takes its repacked copy (glqh_e8_tile_xb_bytes).
// tokens of the blocked activation layout: M padded to whole workgroup tiles
int64_t glqh_e8_tile_padded_tokens(int64_t M, int nstages) { return et_padded_tokens(M, nstages); }

int glqh_launch_e8_tile(const void *x_f16, void *xb_scratch, int64_t M, const void *const q[4], int nstages,
                        const uint32_t *t1, const uint32_t *t2, int64_t n2, const float rel[3], int64_t m_pad,
                        int64_t n_pad, float *part, hipStream_t stream, const glqh_e8_folded *fold, int out_f16,
                        float f16_scale) {
    glqh_range range("dequant_matmul");
    et_plan p;
    if (out_f16 && !glqh_e8_tile_f16_sums_ok(M, fold != nullptr, m_pad))
        return glqh_fail("e8 tile kernel: fp16 sums are partial sums of the large tiles on folded streams");
    const int64_t n_cols = n_pad;                              // columns the caller's rows and activations have
    if (fold && n_pad >= 32 && (n_pad & 31) == 0) n_pad = et_width(n_pad);
    if (!et_make_plan(m_pad, n_pad, M, nstages, &p))
        return glqh_fail("e8 tile kernel: shape not eligible (n_pad %% 256, or %% 32 on folded streams)");
    if (n_pad != n_cols) {                                     // zero activations for the padding columns
        const int64_t Mp = et_padded_tokens(M, nstages);
        const int64_t n16 = (n_pad - n_cols) / 32 * Mp * 4;    // 16-byte slots of the k-pairs past the row
        hipLaunchKernelGGL(et_zero_kernel, dim3((unsigned)((n16 + 255) / 256 < 1024 ? (n16 + 255) / 256 : 1024)), dim3(256), 0,
                           stream, (u32x4 *)((f16 *)xb_scratch + n_cols / 32 * Mp * 32), n16);
        GLQH_LAUNCH_CHECK("e8 tile padding launch");
    }
    if (x_f16) {                                               // NULL: xb_scratch already holds the blocked layout
        hipLaunchKernelGGL(e8_pack_blocked_kernel, dim3((unsigned)((M + 63) / 64), (unsigned)((n_cols / 8 + 15) / 16)),
                           dim3(256), 0, stream, (const f16 *)x_f16, (f16 *)xb_scratch, (int)M,
                           (int)et_padded_tokens(M, nstages), (int)n_cols);
        GLQH_LAUNCH_CHECK("e8 pack launch");
    }
    et_args a;
    for (int s = 0; s < 4; ++s) a.q[s] = (const uint16_t *)q[s];
    for (int s = 0; s < 4; ++s) a.hi8[s] = nullptr;
    a.t1 = t1;
    a.t2 = t2;
    a.n2 = (uint32_t)n2;
    a.nh1 = a.nh2 = 0;
    a.t2_is_t1 = (t1 == t2 && n2 == 65536);
    if (fold) {                                                // the folded streams take the indices' place
        const bool own2 = nstages >= 2 && !a.t2_is_t1;
        GLQH_REQUIRE(!own2 || fold->halves2, "e8 folded: stage 2 has a table of its own but no folded table");
        a.t1 = (const uint32_t *)fold->halves1;
        a.t2 = own2 ? (const uint32_t *)fold->halves2 : a.t1;
        a.nh1 = (uint32_t)fold->n_halves1;
        a.nh2 = (uint32_t)(own2 ? fold->n_halves2 : fold->n_halves1);
        a.t2_is_t1 = !own2;
        GLQH_REQUIRE(a.t1 && fold->n_halves1 >= 1 && fold->n_halves1 <= 2048 && a.nh2 >= 1 && a.nh2 <= 2048,
                     "e8 folded: 1..2048 half codewords per table");
        for (int s = 0; s < nstages; ++s) {
            GLQH_REQUIRE(fold->lo16[s] && fold->hi8[s], "e8 folded: stage %d has no folded stream", s + 1);
            a.q[s] = fold->lo16[s];
            a.hi8[s] = fold->hi8[s];
        }
    }
    for (int s = 0; s < 3; ++s) a.r[s] = rel[s];
    a.xb = (const f16 *)xb_scratch;
    a.M = (int)M;
    a.Mp = (int)et_padded_tokens(M, nstages);
    a.m_pad = (int)m_pad;
    a.n_pad = (int)n_pad;
    a.RT = p.RT;
    a.TT = p.TT;
    a.KS = p.KS;
    a.slot_ds = p.slot_ds;
    a.part = part;
    a.staged = fold && m_pad % 4 == 0;
    a.out_f16 = out_f16;
    a.scale = out_f16 ? f16_scale : 1.0f;
    if (fold && M <= ET_SMALL_TOKENS) {                        // one token tile: TT = 1
        switch (nstages) {
        case 1: return et_launch_small_NS<1>(p, a, stream);
        case 2: return et_launch_small_NS<2>(p, a, stream);
        case 3: return et_launch_small_NS<3>(p, a, stream);
        case 4: return et_launch_small_NS<4>(p, a, stream);
        }
    }
    // (A second launch of 256-token tiles for a half-empty last round, as the trellis tile launcher has, was
    // measured here and not kept: 14336 x 4096 at 4096 tokens 593 -> 617 us, at 2048 tokens 289 -> 297;
    // 11008 x 2048 at 2048 tokens 170 -> 162.)
    switch (nstages * 2 + (fold ? 1 : 0)) {
    case 2: return et_launch_NS<1, false>(p, a, stream);
    case 3: return et_launch_NS<1, true>(p, a, stream);
    case 4: return et_launch_NS<2, false>(p, a, stream);
    case 5: return et_launch_NS<2, true>(p, a, stream);
    case 6: return et_launch_NS<3, false>(p, a, stream);
    case 7: return et_launch_NS<3, true>(p, a, stream);
    case 8: return et_launch_NS<4, false>(p, a, stream);
    case 9: return et_launch_NS<4, true>(p, a, stream);
    }
    return glqh_fail("e8 matmul: %d stages unsupported (1-4)", nstages);
}
