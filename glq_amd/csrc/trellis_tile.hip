// Trellis-3INST GEMM for many tokens on the packed stream (gfx950, wave64).
//
// Y_rht[token, row] = sum_k X_rht[token, k] * W[row, k], W the exact fp16 dequantizer values
// (glq/trellis.py:122-134, 629-643; the reference's batched kernel is
// glq/csrc/glq_trellis.cu:555-715 and above 64 tokens it dequantizes to a dense weight for a
// library GEMM, :1322-1334).  Decoding a state costs about four vector instructions, as much as
// the multiply-adds of a dozen tokens on the matrix cores, so a decoded weight has to meet as many
// tokens as possible:
//
//   workgroup tile = 128 rows x (128 * NTW) tokens, 8 waves (two per SIMD);
//   a step is 64 columns = two k-pairs of the four 32-row blocks of the tile.  Wave w DECODES half
//   a record per lane -- block pair w >> 2, k-pair (w >> 1) & 1, m-tile w & 1: 16 states, two A
//   operands of v_mfma_f32_16x16x32_f16 with the two fp16 halves of every weight added first (the
//   dequantizer's rounding) -- and writes them to LDS in operand layout (lane L's 16 bytes at slot
//   L: conflict-free both ways).  Every wave then MULTIPLIES all 16 operands of the step, read
//   back from LDS one ahead of their use, with ITS OWN 16 * NTW tokens, whose activations it
//   holds in registers, straight from global memory.
//
// A lane's eight weights of an operand are columns 2q + {0,1,8,9,16,17,24,25} of the k-pair
// (glq/trellis.py:99-101), and the B operand puts consecutive tokens in consecutive lanes, so the
// activations are repacked once per call (or written that way by the input transform) into
// xb[k-pair][token][q][those 8 columns]: every operand load of a wave is then one run of 1 KB, and
// the 32 columns of one token are 64 contiguous bytes for whoever writes them.  Workgroups are persistent and walk tiles in an
// order that gives the CUs of one XCD the same tokens at the same time.  K is split into slots only
// while the tiles alone would leave CUs idle; partial sums [slot][token][row] are combined in slot
// order by the consumer, or, with one slot, the scaled result is written (or added) in place.
#include <algorithm>
#include "common.h"
#include "trellis_device.h"

namespace {

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

constexpr int TT_WAVES = 8;
constexpr int TT_THREADS = TT_WAVES * GLQH_WAVE;
constexpr int TT_FRAGS = 8;                        // 16-row operands per 64-column half-step: 128 rows
constexpr int TT_ROWS = 128;
constexpr int TT_BUF = 2 * TT_FRAGS * GLQH_WAVE;   // 16-byte slots per A buffer
constexpr int TT_EP_STRIDE = TT_ROWS + 4;          // floats per token of a wave's output staging space
// two operand buffers (32 KB); after the last step every wave stages 16 tokens x 128 sums there (66 KB)
constexpr size_t TT_LDS = (size_t)TT_WAVES * 16 * TT_EP_STRIDE * sizeof(float);
static_assert(TT_LDS >= (size_t)2 * TT_BUF * 16, "the operand buffers fit the staging space");

struct tt_args {
    const uint8_t *packed;
    const f16 *xb;                                 // (k / 32, 4, Mp, 8) fp16
    int M, Mp, m, k;
    int RT, TT, KS, slot_ds;                       // row tiles, token tiles, K slots, 64-column steps per slot
    float *out;                                    // partial sums [slot][token][row], or the result rows
    int direct, accum;
    float scale;
    int64_t out_stride;
    int out_f16;                                   // partial sums as fp16 (not with direct)
    int rt0;                                       // first row tile of this launch (RT counts from there)
    const uint8_t *packed2;                        // the residual stage's stream of a stacked layer (kernels with R2 > 0)
    float rs2;                                     // and its scale
};

// Several layers that share the activations' shape (fused q/k/v, gate/up: glq_vllm/linear_method.py:664-710) in
// one launch of the tile kernel: their row tiles are numbered through, layer l owns tiles rt0[l] .. rt0[l + 1) - 1
// and has its own stream, rows, repacked activations (layers quantized with different input signs see different
// transformed activations) and output.  The K plan is common.
constexpr int TT_MAX_GROUP = 4;
struct tt_group {
    const uint8_t *packed[TT_MAX_GROUP];
    const f16 *xb[TT_MAX_GROUP];
    float *out[TT_MAX_GROUP];
    int m[TT_MAX_GROUP], rt0[TT_MAX_GROUP];
    float scale[TT_MAX_GROUP];                     // factor of the layer's fp16 sums (its Wscale)
    int n;
};

// Routed experts of a mixture-of-experts layer with many rows per expert (glq/csrc/glq_trellis.cu:1475-1540 is the
// reference's grouped kernel; its caller loops over whole per-expert linears beyond 256 tokens,
// glq_vllm/fused_moe_method.py:702): the (token, choice) slots sorted by expert are the "tokens" of the tile
// kernel, the activations are packed in that order, and a token tile is a run of up to 128 NTW positions of ONE
// expert, listed by a small launch from the routing's offsets -- an expert with 300 rows gets two tiles of 160 and
// 140 positions, not one full and one almost empty.  Waves whose 16 NTW positions lie past the end of the run
// only decode.  Sums leave for row perm[position] of the output, times the expert's factor (a second stage's
// scale) if there is one.
struct tt_moe {
    int64_t stride_bytes;                          // expert e's stream at packed + e * stride_bytes
    int64_t stride2_bytes;                         // and its residual stream at packed2 + e * stride2_bytes (R2 > 0)
    const int *perm;                               // position in the expert-sorted order -> slot
    const int4 *tiles;                             // (expert, first position, positions, -)
    const int *n_tiles;
    const float *pscale_dev;
    const float *wscale_dev;                       // the expert's scale, applied before the sums are rounded to fp16
};

enum { TT_PLAIN = 0, TT_GROUP = 1, TT_MOE = 2 };

__device__ __forceinline__ void tt_barrier() {     // waits for LDS only: global prefetches stay in flight
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
}

// Decode role of a wave in both tile kernels: from half a record (block pair `unit` of the tile, k-pair `kpi` of the
// step, m-tile `ms`) the two A operands of row groups 2 ms and 2 ms + 1, the two fp16 halves of every weight added
// first (the dequantizer's rounding), written in operand layout (lane L's 16 bytes at slot L of operand
// kpi * 8 + unit * 4 + 2 ms + rh).  half = -1: both operands; 0 / 1: operand rh = half only.
template <int R>
__device__ __forceinline__ void tt_decode(const tr_record<R> &r, int ms, int next1, int next2, u32x4 (&af)[2], int half) {
    uint32_t c0 = ms ? r.c[1] : r.c[0], c1 = ms ? r.c[3] : r.c[2];
    uint32_t n0, n1;
    if constexpr (R >= 2) {
        constexpr int sh = 8 * R - 16;
        const uint32_t t = ((c0 >> sh) & 0xFFFFu) | (((c1 >> sh) & 0xFFFFu) << 16);
        const uint32_t n = (uint32_t)__shfl((int)t, next1, GLQH_WAVE);
        n0 = n & 0xFFFFu;
        n1 = n >> 16;
    } else {
        const uint32_t t = c0 | (c1 << 8);
        const uint32_t x1 = (uint32_t)__shfl((int)t, next1, GLQH_WAVE);
        const uint32_t x2 = (uint32_t)__shfl((int)t, next2, GLQH_WAVE);
        n0 = ((x1 & 0xFFu) << 8) | (x2 & 0xFFu);
        n1 = (x1 & 0xFF00u) | ((x2 >> 8) & 0xFFu);
    }
    uint32_t h0[8], h1[8];                                      // k-tiles 0 and 1 of m-tile ms
#pragma unroll
    for (int j = 0; j < 8; ++j) {
        if (half >= 0 && ((j >> 1) & 1) != half) continue;      // operand rh takes states 2rh, 2rh+1, 2rh+4, 2rh+5
        h0[j] = tr_hash(tr_state<R>(c0, n0, j));
        h1[j] = tr_hash(tr_state<R>(c1, n1, j));
    }
#pragma unroll
    for (int rh = 0; rh < 2; ++rh) {
        if (half >= 0 && rh != half) continue;
        const int j0 = 2 * rh;
        af[rh] = pair_sum4(h0[j0], h0[j0 + 1], h0[j0 + 4], h0[j0 + 5], h1[j0], h1[j0 + 1], h1[j0 + 4], h1[j0 + 5]);
    }
}

template <int R>
__device__ __forceinline__ void tt_emit(const tr_record<R> &r, int unit, int kpi, int ms, int next1, int next2, int lane,
                                        u32x4 *dst, int half = -1) {
    u32x4 af[2];
    tt_decode<R>(r, ms, next1, next2, af, half);
#pragma unroll
    for (int rh = 0; rh < 2; ++rh)
        if (half < 0 || rh == half) dst[(kpi * TT_FRAGS + unit * 4 + 2 * ms + rh) * GLQH_WAVE + lane] = af[rh];
}

// A stacked layer (glq/trellis.py:923-933: W = W1 + inv_resid_scale2 * W2): both stages' weights of the operand,
// combined in fp32 and rounded to fp16 once -- the weight of the reference's many-token route, which adds the
// decompressed stages into one fp16 matrix before its GEMM (glq/csrc/glq_trellis.cu:1322-1334,
// glq/quantized_linear.py:986-1010) -- so the products of a stacked layer are those of a single one.
template <int R, int R2>
__device__ __forceinline__ void tt_emit2(const tr_record<R> &r, const tr_record<R2> &rb, float rs2, int unit, int kpi,
                                         int ms, int next1, int next2, int lane, u32x4 *dst, int half = -1) {
    u32x4 af[2], bf[2];
    tt_decode<R>(r, ms, next1, next2, af, half);
    tt_decode<R2>(rb, ms, next1, next2, bf, half);
#pragma unroll
    for (int rh = 0; rh < 2; ++rh) {
        if (half >= 0 && rh != half) continue;
        const f16x8 x = __builtin_bit_cast(f16x8, af[rh]), y = __builtin_bit_cast(f16x8, bf[rh]);
        f16x8 o;
#pragma unroll
        for (int e = 0; e < 8; ++e) o[e] = (f16)((float)x[e] + rs2 * (float)y[e]);
        dst[(kpi * TT_FRAGS + unit * 4 + 2 * ms + rh) * GLQH_WAVE + lane] = __builtin_bit_cast(u32x4, o);
    }
}

// PC: the waves of a SIMD take one role each instead of both in turn.  Waves 0..3 (one per SIMD) only MULTIPLY,
// 16 NTW tokens each against all 16 operands of a step; waves 4..7 only DECODE, a whole record per lane and step
// (both m-tiles: block pair (w >> 1) & 1, k-pair w & 1).  The tile is 128 rows x 64 NTW tokens: half as many waves
// read the operands back from LDS (64 KB per step and workgroup instead of 128, which at 16 or 32 tokens per
// wave costs more cycles than their products), and a SIMD's decode runs beside its products instead of between
// them.  Same tiles, K slots and order of summation as the plain form with NTW / 2: the same bits.
template <int R, int NTW, int MODE, int R2 = 0, bool PC = false>
__device__ __forceinline__ void tr_tile_body(const tt_args &a, const tt_group &g, const tt_moe &mo) {
    constexpr bool GROUP = MODE == TT_GROUP, MOE = MODE == TT_MOE;
    constexpr int MW = PC ? 4 : TT_WAVES;                       // multiplying waves
    constexpr int RB = R2 > 0 ? R2 : 1, REC2 = 4 * RB;
    extern __shared__ u32x4 abuf[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int nkp = a.k >> 5, nds = a.k >> 6;
    constexpr int REC = 4 * R;

    // decode role (PC: of waves 4..7, both m-tiles)
    const bool producer = PC && wave >= 4;                      // uniform over the wave
    const int dw = PC ? 2 * (wave & 3) : wave;
    const int unit = dw >> 2, kpi = (dw >> 1) & 1, ms = dw & 1;
    const int hm = i >> 3, l = 4 * (i & 7) + q;
    const int l1 = (l + 1) & 31, l2 = (l + 2) & 31;
    const int next1 = 16 * (l1 & 3) + 8 * hm + (l1 >> 2), next2 = 16 * (l2 & 3) + 8 * hm + (l2 >> 2);

    int nitems = a.TT * a.KS * a.RT;
    if constexpr (MOE) nitems = *mo.n_tiles * a.RT * a.TT;      // one K slot; TT = workgroup tiles per run
    const int per_xcd = (nitems + 7) >> 3;
    const int xcd = blockIdx.x & 7, bx = blockIdx.x >> 3;
    const int nbx = ((int)gridDim.x - xcd + 7) >> 3;
    for (int w = bx; w < per_xcd; w += nbx) {
        const int item = xcd * per_xcd + w;
        if (item >= nitems) break;                              // uniform
        const int slot = (item / a.RT) % a.KS, tt0 = item / (a.RT * a.KS);
        int rt = a.rt0 + item % a.RT;                           // row tile of its layer
        int lm = a.m;
        const uint8_t *lpacked = a.packed;
        const f16 *lxb = a.xb;
        float *lout = a.out;
        // fp16 sums leave times the layer's scale: an unscaled sum over a long row of large activations can pass
        // the fp16 range where the scaled one, of the size of the layer's output, does not
        float f16sc = a.scale;
        if constexpr (GROUP) {
            int first = 0;
            lm = g.m[0]; lpacked = g.packed[0]; lxb = g.xb[0]; lout = g.out[0]; f16sc = g.scale[0];
#pragma unroll
            for (int j = 1; j < TT_MAX_GROUP; ++j)
                if (j < g.n && rt >= g.rt0[j]) { first = g.rt0[j]; lm = g.m[j]; lpacked = g.packed[j]; lxb = g.xb[j]; lout = g.out[j]; f16sc = g.scale[j]; }
            rt -= first;
        }
        const int mpairs = lm >> 5;
        int tok0 = tt0 * (MW * 16 * NTW) + (PC ? wave & 3 : wave) * 16 * NTW, limit = a.M;
        float osc = 1.0f;
        bool active = true;                                     // uniform over the wave
        const uint8_t *lpacked2 = a.packed2;
        float lrs2 = a.rs2;
        if constexpr (MOE) {
            // a run of the table may be longer than this kernel's tile (a stacked expert's streams are decoded
            // into one operand in tiles of at most 256 positions): TT workgroup tiles per run, in order
            constexpr int WG_TOK = MW * 16 * NTW;
            const int4 tile = mo.tiles[item / (a.RT * a.TT)];
            const int sub = (item / a.RT) % a.TT;
            const int first = tile.y + sub * WG_TOK, cnt = min(WG_TOK, tile.z - sub * WG_TOK);
            if (cnt <= 0) continue;                             // uniform over the workgroup
            lpacked = a.packed + tile.x * mo.stride_bytes;
            tok0 = first + __builtin_amdgcn_readfirstlane(PC ? wave & 3 : wave) * 16 * NTW;   // uniform: scalar registers
            limit = first + cnt;
            osc = mo.wscale_dev[tile.x];
            if constexpr (R2 > 0) {
                lpacked2 = a.packed2 + tile.x * mo.stride2_bytes;
                lrs2 = mo.pscale_dev[tile.x];
            } else if (mo.pscale_dev) {
                osc *= mo.pscale_dev[tile.x];
            }
            active = __builtin_amdgcn_readfirstlane((int)(tok0 < limit)) != 0;
        }
        const int r0 = rt * TT_ROWS;
        const int ds0 = slot * a.slot_ds, ds1 = min(ds0 + a.slot_ds, nds);

        const int mp = min(2 * (2 * rt + unit) + hm, mpairs - 1);
        const uint8_t *rec_base = lpacked + ((int64_t)mp * nkp * 32 + l) * REC + (int64_t)kpi * 32 * REC;
        auto load_rec = [&](int d) {                            // the record of k-pair 2d + kpi
            return tr_load_record<R>(rec_base + (int64_t)min(d, ds1 - 1) * 64 * REC);
        };
        const uint8_t *rec_base2 = R2 > 0 ? lpacked2 + ((int64_t)mp * nkp * 32 + l) * REC2 + (int64_t)kpi * 32 * REC2 : nullptr;
        auto load_rec2 = [&](int d) {
            tr_record<RB> r = {};
            if constexpr (R2 > 0) r = tr_load_record<RB>(rec_base2 + (int64_t)min(d, ds1 - 1) * 64 * REC2);
            return r;
        };
        auto emit = [&](const tr_record<R> &r, const tr_record<RB> &rb, u32x4 *dst, int half = -1) {
            if constexpr (R2 > 0) tt_emit2<R, RB>(r, rb, lrs2, unit, kpi, ms, next1, next2, lane, dst, half);
            else tt_emit<R>(r, unit, kpi, ms, next1, next2, lane, dst, half);
        };
        // multiply role: token 16 * tt + i of the wave's tokens; k-pair kp, slot q at xb[(kp * Mp + token) * 4 + q]
        // (the token dimension of xb is padded to whole tiles: no clamping, constant offsets)
        const int64_t bstep = (int64_t)a.Mp * 32;               // elements from one k-pair to the next
        const f16 *xrow = lxb + (int64_t)(tok0 + i) * 32 + q * 8;

        f32x4 acc[TT_FRAGS][NTW];
#pragma unroll
        for (int f = 0; f < TT_FRAGS; ++f)
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) acc[f][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

        // Software pipeline over the 64-column steps: records arrive two steps ahead and the operands
        // of step d + 1 are written to the other LDS buffer during step d.
        // Activations in three register sets of one k-half each, rotating: the set a half has just
        // finished with takes the half two ahead, so every request has a whole step to arrive.
        u32x4 bs[3][NTW];
        auto load_half = [&](u32x4 (&dst)[NTW], int hidx) {     // half hidx of the slot: step ds0 + hidx / 2, k-half hidx & 1
            const int d = min(ds0 + (hidx >> 1), ds1 - 1);
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) dst[tt] = *(const u32x4 *)(xrow + (2 * d + (hidx & 1)) * bstep + tt * 512);
        };
        if constexpr (PC) {
            if (producer) {                                     // as many barriers as the multiplying waves meet
                auto emit_both = [&](const tr_record<R> &r, const tr_record<RB> &rb, u32x4 *dst) {
#pragma unroll
                    for (int mt = 0; mt < 2; ++mt) {
                        if constexpr (R2 > 0) tt_emit2<R, RB>(r, rb, lrs2, unit, kpi, mt, next1, next2, lane, dst);
                        else tt_emit<R>(r, unit, kpi, mt, next1, next2, lane, dst);
                    }
                };
                tr_record<R> p1 = load_rec(ds0 + 1), p2 = load_rec(ds0 + 2);
                tr_record<RB> p1b = load_rec2(ds0 + 1), p2b = load_rec2(ds0 + 2);
                emit_both(load_rec(ds0), load_rec2(ds0), abuf);
                tt_barrier();
                for (int d = ds0; d < ds1; ++d) {
                    const tr_record<R> p3 = load_rec(d + 3);
                    const tr_record<RB> p3b = load_rec2(d + 3);
                    emit_both(p1, p1b, abuf + (((d - ds0) & 1) ^ 1) * TT_BUF);
                    tt_barrier();
                    p1 = p2;
                    p2 = p3;
                    p1b = p2b;
                    p2b = p3b;
                }
            }
        }
        auto load_rec_m = [&](int d) {                          // PC: the multiplying waves hold no records
            tr_record<R> r = {};
            if constexpr (!PC) r = load_rec(d);
            return r;
        };
        auto load_rec2_m = [&](int d) {
            tr_record<RB> r = {};
            if constexpr (!PC) r = load_rec2(d);
            return r;
        };
        if (!producer) {
        tr_record<R> rc = load_rec_m(ds0);
        tr_record<RB> rcb = load_rec2_m(ds0);
        load_half(bs[0], 0);
        load_half(bs[1], 1);
        tr_record<R> r1 = load_rec_m(ds0 + 1), r2 = load_rec_m(ds0 + 2);
        tr_record<RB> r1b = load_rec2_m(ds0 + 1), r2b = load_rec2_m(ds0 + 2);
        if constexpr (!PC) emit(rc, rcb, abuf);
        tt_barrier();
        for (int d0 = ds0; d0 < ds1; d0 += 3) {
#pragma unroll
          for (int j = 0; j < 3; ++j) {                         // static register sets: six halves = 0 mod 3
            const int d = d0 + j;
            if (d >= ds1) break;                                // uniform
            const int par = (d - ds0) & 1;
            const u32x4 *rd = abuf + par * TT_BUF;
            u32x4 *wr = abuf + (par ^ 1) * TT_BUF;
            const tr_record<R> r3 = load_rec_m(d + 3);
            const tr_record<RB> r3b = load_rec2_m(d + 3);
            if (MOE && !active) {                               // no positions of the run left for this wave
                if constexpr (!PC) {
                    emit(r1, r1b, wr, 0);
                    emit(r1, r1b, wr, 1);
                }
            } else {
            f16x8 ring[2];
            ring[0] = __builtin_bit_cast(f16x8, rd[lane]);
            ring[1] = __builtin_bit_cast(f16x8, rd[GLQH_WAVE + lane]);
            __builtin_amdgcn_sched_barrier(0);
#pragma unroll
            for (int kk = 0; kk < 2 * TT_FRAGS; ++kk) {
                const int u = kk / TT_FRAGS, f = kk % TT_FRAGS;
                if (f == 0) {
                    load_half(bs[(2 * j + u + 2) % 3], 2 * (d - ds0) + u + 2);
                    __builtin_amdgcn_sched_barrier(0);
                }
                const f16x8 af = ring[kk & 1];
                if (kk + 2 < 2 * TT_FRAGS) ring[kk & 1] = __builtin_bit_cast(f16x8, rd[(kk + 2) * GLQH_WAVE + lane]);
#pragma unroll
                for (int tt = 0; tt < NTW; ++tt)
                    acc[f][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                        af, __builtin_bit_cast(f16x8, bs[(2 * j + u) % 3][tt]), acc[f][tt], 0, 0, 0);
                if constexpr (!PC) {
                    if (kk == 1) emit(r1, r1b, wr, 0);
                    if (kk == TT_FRAGS + 1) emit(r1, r1b, wr, 1);
                }
            }
            }
            tt_barrier();                                       // rd has been read, wr is written
            r1 = r2;
            r2 = r3;
            r1b = r2b;
            r2b = r3b;
          }
        }
        }
        // Lane (i, q) holds four consecutive rows of token i for every (operand, token tile): operand
        // f = 4 unit' + s covers rows 64 unit' + 32 h + 8 s + (0..7), h = 0, 1 -- sixteen bytes here, sixteen
        // bytes 44 KB further on for the next token: stored like that, a wave's instruction touches 64 lines and
        // the sums of a tile leave as 16384 separate requests (a tenth of a 4096-token linear, a fifth of a
        // 512-token one).  So every wave passes its sums through LDS once (its own 16 tokens x 128 rows, no
        // barrier: a wave's LDS operations complete in order) and stores whole runs of a token's rows: two
        // tokens x 512 bytes per instruction in fp32, four tokens x 256 bytes in fp16.
        const int rlane = 32 * (q >> 1) + 4 * (q & 1);
        float *ep = (float *)abuf + wave * (16 * TT_EP_STRIDE);
#pragma unroll
        for (int tt = 0; tt < NTW; ++tt) {
            if ((MOE && !active) || producer) break;
#pragma unroll
            for (int f = 0; f < TT_FRAGS; ++f)
                *(f32x4 *)(ep + i * TT_EP_STRIDE + 64 * (f >> 2) + 8 * (f & 3) + rlane) = acc[f][tt];
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
            if (!a.direct && a.out_f16) {                       // uniform
                const int rl = 8 * (lane & 15), row = r0 + rl;
#pragma unroll
                for (int j = 0; j < 4; ++j) {
                    const int tl = 4 * j + (lane >> 4);
                    int tok = tok0 + 16 * tt + tl;
                    f32x4 v0 = *(const f32x4 *)(ep + tl * TT_EP_STRIDE + rl);
                    f32x4 v1 = *(const f32x4 *)(ep + tl * TT_EP_STRIDE + rl + 4);
                    if constexpr (MOE) { v0 *= osc; v1 *= osc; }
                    else { v0 *= f16sc; v1 *= f16sc; }
                    if (tok >= limit || row >= lm) continue;    // m is a multiple of 32: whole runs of eight
                    if constexpr (MOE) tok = mo.perm[tok];
                    typedef _Float16 f16x8o __attribute__((ext_vector_type(8)));
                    const int64_t e = ((int64_t)slot * a.M + tok) * lm + row;
                    *(f16x8o *)((f16 *)lout + e) = f16x8o{(f16)v0[0], (f16)v0[1], (f16)v0[2], (f16)v0[3],
                                                           (f16)v1[0], (f16)v1[1], (f16)v1[2], (f16)v1[3]};
                }
            } else {
                const int rl = 4 * (lane & 31), row = r0 + rl;
#pragma unroll
                for (int j = 0; j < 8; ++j) {
                    const int tl = 2 * j + (lane >> 5);
                    int tok = tok0 + 16 * tt + tl;
                    f32x4 v = *(const f32x4 *)(ep + tl * TT_EP_STRIDE + rl);
                    if constexpr (MOE) v *= osc;
                    if (tok >= limit || row >= lm) continue;
                    if constexpr (MOE) tok = mo.perm[tok];
                    if (!a.direct) {
                        *(f32x4 *)(lout + ((int64_t)slot * a.M + tok) * lm + row) = v;
                    } else {
                        float *o = lout + (int64_t)tok * a.out_stride + row;
                        if ((a.out_stride & 3) == 0) {
                            f32x4 w = v * a.scale;
                            if (a.accum) w += *(f32x4 *)o;
                            *(f32x4 *)o = w;
                        } else {
#pragma unroll
                            for (int e = 0; e < 4; ++e) o[e] = a.accum ? o[e] + v[e] * a.scale : v[e] * a.scale;
                        }
                    }
                }
            }
        }
        tt_barrier();                                           // the next item's first operands overwrite this space
    }
}

template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_kernel(const tt_args a) {
    tr_tile_body<R, NTW, TT_PLAIN>(a, tt_group{}, tt_moe{});
}

// up to 256 tokens per tile: decoding and multiplying waves (NTW = 2, 4: tiles of 128, 256 tokens)
template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_pc_kernel(const tt_args a) {
    tr_tile_body<R, NTW, TT_PLAIN, 0, true>(a, tt_group{}, tt_moe{});
}

template <int R2, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_rvq_pc_kernel(const tt_args a) {
    tr_tile_body<4, NTW, TT_PLAIN, R2, true>(a, tt_group{}, tt_moe{});
}

template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_group_pc_kernel(const tt_args a, const tt_group g) {
    tr_tile_body<R, NTW, TT_GROUP, 0, true>(a, g, tt_moe{});
}

// a stacked layer (first stage 4 bits/weight): both streams decoded into one operand
template <int R2, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_rvq_kernel(const tt_args a) {
    tr_tile_body<4, NTW, TT_PLAIN, R2>(a, tt_group{}, tt_moe{});
}

template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_group_kernel(const tt_args a, const tt_group g) {
    tr_tile_body<R, NTW, TT_GROUP>(a, g, tt_moe{});
}

template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_moe_kernel(const tt_args a, const tt_moe mo) {
    tr_tile_body<R, NTW, TT_MOE>(a, tt_group{}, mo);
}

template <int R, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_moe_pc_kernel(const tt_args a, const tt_moe mo) {
    tr_tile_body<R, NTW, TT_MOE, 0, true>(a, tt_group{}, mo);
}

template <int R2, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_moe_rvq_pc_kernel(const tt_args a, const tt_moe mo) {
    tr_tile_body<4, NTW, TT_MOE, R2, true>(a, tt_group{}, mo);
}

// stacked experts (first stage 4 bits/weight): both streams of the run's expert into one operand
template <int R2, int NTW>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_moe_rvq_kernel(const tt_args a, const tt_moe mo) {
    tr_tile_body<4, NTW, TT_MOE, R2>(a, tt_group{}, mo);
}

// Token tiles of the routed experts: expert e's positions [offs[e], offs[e + 1]) of the sorted order in
// ceil(count / tile_tok) runs of equal length (a multiple of 32, the last one shorter).  One workgroup; thread t
// takes experts t * per .. (t + 1) * per - 1.
__global__ void __launch_bounds__(256)
tr_moe_tiles_kernel(const int *__restrict__ offs, int n_experts, int tile_tok, int4 *__restrict__ tiles,
                    int *__restrict__ n_tiles) {
    __shared__ int sums[256];
    const int t = threadIdx.x, per = (n_experts + 255) / 256;
    const int e0 = min(t * per, n_experts), e1 = min(e0 + per, n_experts);
    int mine = 0;
    for (int e = e0; e < e1; ++e) mine += (offs[e + 1] - offs[e] + tile_tok - 1) / tile_tok;
    sums[t] = mine;
    __syncthreads();
    int at = 0;
    for (int j = 0; j < t; ++j) at += sums[j];
    if (t == 255) *n_tiles = at + mine;
    for (int e = e0; e < e1; ++e) {
        const int o0 = offs[e], cnt = offs[e + 1] - o0, nt = (cnt + tile_tok - 1) / tile_tok;
        if (nt == 0) continue;
        const int len = ((cnt + nt - 1) / nt + 31) & ~31;
        for (int j = 0; j < nt; ++j) tiles[at++] = int4{e, o0 + j * len, max(0, min(len, cnt - j * len)), 0};
    }
}

// Up to 64 tokens: one barrier per group of four steps instead of one per step, and the eight waves split a
// step's products by token group AND row fragment.  With one token tile per wave
// every wave of the kernel above reads the whole 16 KB operand buffer of a step (128 KB per step and workgroup:
// 1024 LDS cycles for 256-512 cycles of multiplications) and below 128 tokens most waves multiply padding.
// Here: TG = 2 or 4 token groups of 16 NTW tokens; wave w takes token group w % TG and the operands
// w / TG + (8 / TG) j, j < TG, of each half-step -- 2 TG operand reads and 2 TG NTW MFMAs per wave and step,
// every product computed once.  The operands of a whole group of four steps (256 columns) are decoded into one
// of two 64 KB buffers while the previous group is multiplied out of the other; decoding is as above (wave w:
// block pair w >> 2, k-pair (w >> 1) & 1, m-tile w & 1).  Same K slots and order of summation as above.
constexpr size_t TT_SMALL_LDS = (size_t)8 * TT_BUF * 16;       // 128 KB

template <int R, int TG, int NTW, int R2 = 0>
__global__ void __launch_bounds__(TT_THREADS)
tr_tile_small_kernel(const tt_args a) {
    constexpr int RG = TT_FRAGS / TG;                          // operand groups
    constexpr int RB = R2 > 0 ? R2 : 1, REC2 = 4 * RB;         // R2 > 0: a stacked layer, both streams into one operand
    extern __shared__ u32x4 abuf[];
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int i = lane & 15, q = lane >> 4;
    const int nkp = a.k >> 5, nds = a.k >> 6, mpairs = a.m >> 5;
    constexpr int REC = 4 * R;
    const int tg = wave % TG, rg = wave / TG;

    // decode role
    const int unit = wave >> 2, kpi = (wave >> 1) & 1, ms = wave & 1;
    const int hm = i >> 3, l = 4 * (i & 7) + q;
    const int l1 = (l + 1) & 31, l2 = (l + 2) & 31;
    const int next1 = 16 * (l1 & 3) + 8 * hm + (l1 >> 2), next2 = 16 * (l2 & 3) + 8 * hm + (l2 >> 2);

    const int nitems = a.KS * a.RT;                            // one token tile
    for (int item = blockIdx.x; item < nitems; item += gridDim.x) {
        const int rt = item % a.RT, slot = item / a.RT;
        const int r0 = rt * TT_ROWS;
        const int ds0 = slot * a.slot_ds, ds1 = min(ds0 + a.slot_ds, nds);
        const int nquads = (ds1 - ds0 + 3) >> 2;

        const int mp = min(2 * (2 * rt + unit) + hm, mpairs - 1);
        const uint8_t *rec_base = a.packed + ((int64_t)mp * nkp * 32 + l) * REC + (int64_t)kpi * 32 * REC;
        auto load_rec = [&](int d) {                            // the record of k-pair 2d + kpi
            return tr_load_record<R>(rec_base + (int64_t)min(d, ds1 - 1) * 64 * REC);
        };
        const uint8_t *rec_base2 = R2 > 0 ? a.packed2 + ((int64_t)mp * nkp * 32 + l) * REC2 + (int64_t)kpi * 32 * REC2 : nullptr;
        auto load_rec2 = [&](int d) {
            tr_record<RB> r = {};
            if constexpr (R2 > 0) r = tr_load_record<RB>(rec_base2 + (int64_t)min(d, ds1 - 1) * 64 * REC2);
            return r;
        };
        auto emit = [&](const tr_record<R> r, const tr_record<RB> rb, u32x4 *dst) {
            if constexpr (R2 > 0) tt_emit2<R, RB>(r, rb, a.rs2, unit, kpi, ms, next1, next2, lane, dst);
            else tt_emit<R>(r, unit, kpi, ms, next1, next2, lane, dst);
        };
        // multiply role: token 16 * tt + i of the wave's token group
        const int64_t bstep = (int64_t)a.Mp * 32;               // elements from one k-pair to the next
        const f16 *xrow = a.xb + (int64_t)(16 * NTW * tg + i) * 32 + q * 8;
        auto load_b = [&](u32x4 (&bb)[NTW][2], int d) {
            d = min(d, ds1 - 1);
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) {
                bb[tt][0] = *(const u32x4 *)(xrow + 2 * d * bstep + tt * 512);
                bb[tt][1] = *(const u32x4 *)(xrow + (2 * d + 1) * bstep + tt * 512);
            }
        };

        f32x4 acc[TG][NTW];
#pragma unroll
        for (int j = 0; j < TG; ++j)
#pragma unroll
            for (int tt = 0; tt < NTW; ++tt) acc[j][tt] = f32x4{0.f, 0.f, 0.f, 0.f};

        // records of a group arrive a group ahead, activations three steps ahead (a step is a few hundred
        // cycles, less than an L2 round trip)
        tr_record<R> rc[4], rn[4];
        tr_record<RB> rcb[4], rnb[4];
        u32x4 b[4][NTW][2];
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) { rc[dd] = load_rec(ds0 + dd); rcb[dd] = load_rec2(ds0 + dd); }
#pragma unroll
        for (int j = 0; j < 3; ++j) load_b(b[j], ds0 + j);
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) { rn[dd] = load_rec(ds0 + 4 + dd); rnb[dd] = load_rec2(ds0 + 4 + dd); }
        if (item != (int)blockIdx.x) tt_barrier();              // the previous item's last buffer has been read
#pragma unroll
        for (int dd = 0; dd < 4; ++dd) emit(rc[dd], rcb[dd], abuf + dd * TT_BUF);
        tt_barrier();
        for (int qd = 0; qd < nquads; qd += 2) {
#pragma unroll
            for (int h = 0; h < 2; ++h) {                       // group qd + h: buffer h
                if (qd + h < nquads) {                          // uniform
                    const int d0 = ds0 + 4 * (qd + h);
                    const u32x4 *rd = abuf + h * 4 * TT_BUF + rg * GLQH_WAVE + lane;
                    u32x4 *wr = abuf + (h ^ 1) * 4 * TT_BUF;
#pragma unroll
                    for (int dd = 0; dd < 4; ++dd) {
                        rc[dd] = rn[dd];
                        rn[dd] = load_rec(d0 + 8 + dd);
                        rcb[dd] = rnb[dd];
                        rnb[dd] = load_rec2(d0 + 8 + dd);
                    }
#pragma unroll
                    for (int dd = 0; dd < 4; ++dd) {
                        // operand kk of the step: half-step kk / TG, operand rg + RG (kk % TG); read PF ahead
                        constexpr int NK = 2 * TG, PF = NK < 4 ? NK : 4;
                        auto frag = [&](int kk) {
                            return __builtin_bit_cast(f16x8, rd[dd * TT_BUF + ((kk / TG) * TT_FRAGS + RG * (kk % TG)) * GLQH_WAVE]);
                        };
                        f16x8 ring[PF];
#pragma unroll
                        for (int kk = 0; kk < PF; ++kk) ring[kk] = frag(kk);
                        load_b(b[(dd + 3) & 3], d0 + dd + 3);
                        emit(rc[dd], rcb[dd], wr + dd * TT_BUF);   // operands of the next group (unused after the last)
                        if (d0 + dd < ds1) {                    // uniform: a slot need not be whole groups
#pragma unroll
                            for (int kk = 0; kk < NK; ++kk) {
                                const f16x8 af = ring[kk % PF];
                                if (kk + PF < NK) ring[kk % PF] = frag(kk + PF);
#pragma unroll
                                for (int tt = 0; tt < NTW; ++tt)
                                    acc[kk % TG][tt] = __builtin_amdgcn_mfma_f32_16x16x32_f16(
                                        af, __builtin_bit_cast(f16x8, b[dd][tt][kk / TG]), acc[kk % TG][tt], 0, 0, 0);
                            }
                        }
                    }
                    tt_barrier();                               // rd has been read, wr is written
                }
            }
        }

        // lane holds four consecutive rows of token i for every (operand, token tile): operand
        // f = 4 unit' + s covers rows 64 unit' + 32 h + 8 s + (0..7), h = 0, 1
        const int rlane = 32 * (q >> 1) + 4 * (q & 1);
#pragma unroll
        for (int tt = 0; tt < NTW; ++tt) {
            const int tok = 16 * NTW * tg + 16 * tt + i;
            if (tok >= a.M) continue;
#pragma unroll
            for (int j = 0; j < TG; ++j) {
                const int f = rg + RG * j;
                const int row = r0 + 64 * (f >> 2) + 8 * (f & 3) + rlane;
                if (row >= a.m) continue;                       // m is a multiple of 32: whole groups of four
                if (!a.direct) {
                    *(f32x4 *)(a.out + ((int64_t)slot * a.M + tok) * a.m + row) = acc[j][tt];
                } else {
                    float *o = a.out + (int64_t)tok * a.out_stride + row;
                    if ((a.out_stride & 3) == 0) {
                        f32x4 v = acc[j][tt] * a.scale;
                        if (a.accum) v += *(f32x4 *)o;
                        *(f32x4 *)o = v;
                    } else {
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = a.accum ? o[e] + acc[j][tt][e] * a.scale : acc[j][tt][e] * a.scale;
                    }
                }
            }
        }
    }
}

// (M, k) row-major fp16 -> xb[k-pair][token][q][8]: slot q of a k-pair takes columns
// 2q + {0,1,8,9,16,17,24,25}, i.e. dword q of each of its four 16-byte items.  64 tokens x 4
// k-pairs per workgroup through LDS; reads in runs of 256 bytes, writes in runs of 4 KB.
// GATHER: token t of xb is row perm[t] / x_div of x, for the *n_valid first t (the expert-sorted order of the
// routed experts' slots).
template <bool GATHER>
__global__ void __launch_bounds__(256)
tr_pack_blocked_kernel(const f16 *__restrict__ x, f16 *__restrict__ xb, int M, int Mp, int k,
                       const int *__restrict__ perm, const int *__restrict__ n_valid, int x_div) {
    __shared__ u32x4 tile[16][65];                              // [k-pair * 4 + q][token]
    const int tok0 = blockIdx.x * 64, kp0 = blockIdx.y * 4, nkp = k >> 5;
    const int t = threadIdx.x;
    if constexpr (GATHER) {
        M = *n_valid;
        if (tok0 >= M) return;                                  // uniform
    }
    {
        const int kpi = t & 3, tl = t >> 2;
        int tok = min(tok0 + tl, M - 1);
        if constexpr (GATHER) tok = perm[tok] / x_div;
        const int kp = min(kp0 + kpi, nkp - 1);
        const u32x4 *src = (const u32x4 *)(x + (int64_t)tok * k + 32 * kp);
        const u32x4 v0 = src[0], v1 = src[1], v2 = src[2], v3 = src[3];
#pragma unroll
        for (int qq = 0; qq < 4; ++qq) tile[kpi * 4 + qq][tl] = u32x4{v0[qq], v1[qq], v2[qq], v3[qq]};
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {                               // k-pair r: 64 tokens x 4 slots = 4 KB contiguous
        const int tl = t >> 2, qq = t & 3;
        const int kp = kp0 + r;
        if (tok0 + tl < M && kp < nkp)
            *(u32x4 *)(xb + (((int64_t)kp * Mp + tok0 + tl) * 4 + qq) * 8) = tile[r * 4 + qq][tl];
    }
}

int tt_ntw(int64_t M) {
    static const int forced = [] { const char *e = getenv("GLQ_TT_NTW"); return e ? atoi(e) : 0; }();
    if (forced && M > 256) return forced;
    return M <= 128 ? 1 : M <= 256 ? 2 : 4;
}

int64_t tt_padded_tokens(int64_t M) {
    const int64_t tile = TT_WAVES * 16 * tt_ntw(M);
    return (M + tile - 1) / tile * tile;
}

struct tt_plan {
    int NTW, RT, TT, KS, slot_ds, grid;
};

// K slots and grid for token tiles of 128 NTW tokens
void tt_plan_for(int NTW, int64_t m, int64_t k, int64_t M, tt_plan *p) {
    p->NTW = NTW;
    const int tile_tok = TT_WAVES * 16 * p->NTW;
    p->RT = (int)((m + TT_ROWS - 1) / TT_ROWS);
    p->TT = (int)((M + tile_tok - 1) / tile_tok);
    const int nds = (int)(k / 64);
    const int cus = glqh_device_cus();
    const int64_t base = (int64_t)p->RT * p->TT;
    int64_t ks = 1;
    if (base < cus) {
        ks = cus / base;
        const int64_t cap_len = nds / 8 > 0 ? nds / 8 : 1;      // slots of at least 512 columns
        if (ks > cap_len) ks = cap_len;
        const int64_t cap_bytes = ((int64_t)128 << 20) / (M * m * 4);   // partial sums stay under 128 MB
        if (ks > cap_bytes) ks = cap_bytes;
        if (ks < 1) ks = 1;
    }
    p->slot_ds = (int)((nds + ks - 1) / ks);
    p->KS = (nds + p->slot_ds - 1) / p->slot_ds;
    const int64_t items = base * p->KS;
    p->grid = (int)(items < cus ? items : cus);
}

// Microseconds a plan is expected to take: rounds of workgroups x steps x the time of a step (2.26 us with
// 512-token tiles, 1.7 with 256), a last round that counts at least half, a step that is slower when a single
// round leaves CUs idle (+ 0.6 x the idle share: 172 workgroups on 256 CUs take 2.75 / 2.0 us per step, measured),
// and what K slots cost on top (their sums, esz bytes each, written and read again at about 4 TB/s).
double tt_plan_cost(const tt_plan &p, int64_t m, int64_t M, int esz) {
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
    const double step = p.NTW == 4 ? 2.26 : p.NTW == 2 ? 1.7 : 1.3;
    double t = rounds * p.slot_ds * step * slow;
    if (p.KS > 1) t += 2.0 * p.KS * (double)M * (double)m * esz / 4.0e6;
    return t;
}

// Up to 256 tokens the tile follows the token count; above, 512-token tiles unless 256-token tiles are expected
// to be at least 5 % faster: few row tiles (small layers, a few hundred tokens) fill the chip with neither, and
// the smaller tile then needs fewer K slots or leaves a shorter last round (2048 x 2048 at 2048 tokens: 4 x 4
// tiles x 2 slots -> 8 x 4 tiles x 1 slot, 73 -> 58 us; 11008 x 11008 at 1024 tokens: 172 tiles in one round ->
// 344 in two short ones, 474 -> 366 us).  The model is rough: on a sweep of 15 shapes (512..14336 rows x
// 2048..11008 columns) x 512..4096 tokens through the matmul entry it ends within 3 % of the faster tile in 48 of
// 60 cases, 25 % off at worst (14336 x 2048 at 512 tokens, a gain it misses), 3 % below 512-token tiles everywhere
// in total; the seven linears of a 3B-shape layer: 505 -> 444 us at 1024 tokens.  GLQ_TT_NTW forces a tile
// above 256 tokens.
// max_ntw = 2: a stacked layer decoded into one operand (two streams' records and temporaries do not fit beside the
// accumulators of a 512-token tile).
void tt_make_plan(int64_t m, int64_t k, int64_t M, tt_plan *p, int max_ntw = 4) {
    const int top = std::min(tt_ntw(M), max_ntw);
    tt_plan_for(top, m, k, M, p);
    static const bool forced = getenv("GLQ_TT_NTW") != nullptr;
    if (top < 4 || forced) return;
    tt_plan p2;
    tt_plan_for(2, m, k, M, &p2);
    // (3 bytes per sum, between fp16 and fp32: the K-slot query and the launch must arrive at the same plan,
    // whatever the width the sums leave with)
    if (tt_plan_cost(p2, m, M, 3) < 0.95 * tt_plan_cost(*p, m, M, 3)) *p = p2;
}

// Tiles of up to 256 tokens run with decoding and multiplying waves (the tr_tile_*_pc_kernel forms) when a K
// slot has min_steps steps or more; GLQ_TT_PC=0: never, GLQ_TT_PC_STEPS: another shortest slot.  Whole linears,
// both forms in one run, us: 14336 x 4096 at 96 / 128 / 192 / 256 tokens 50.9 / 52.7 / 64.1 / 66.0 -> 47.1 / 48.4 /
// 59.8 / 61.4, 4096 x 14336 48.5 / 50.3 / 61.5 / 63.5 -> 43.8 / 45.7 / 57.0 / 59.1; with slots of 8 steps a
// single-stage layer loses (4096 x 4096 at 96 / 128 tokens 30.5 / 33.6 -> 35.2 / 35.1: the first operands of a
// slot are decoded by half as many waves), so it asks for 16.  Stacked layers, whose decode is twice as long, and
// grouped layers gain from 8 steps on: 4 + 2 bits 14336 x 4096 75.5 / 76.3 / 89.9 -> 60.0 / 62.3 / 72.4 at 96 /
// 128 / 256 tokens and 154 -> 120 at 512, 4096 x 4096 35.4 / 45.1 / 61.3 -> 33.2 / 42.1 / 53.2 at 128 / 256 / 512;
// grouped gate/up of a 4096-wide model 84.2 / 84.6 / 110.8 -> 72.1 / 74.3 / 98.5, q/k/v 43.3 / 51.7 -> 41.6 / 50.2.
bool tt_split_roles(const tt_plan &p, int min_steps) {
    static const int pc = [] { const char *e = getenv("GLQ_TT_PC"); return e ? atoi(e) : 1; }();
    static const int pc_steps = [] { const char *e = getenv("GLQ_TT_PC_STEPS"); return e ? atoi(e) : 0; }();
    return pc && p.NTW <= 2 && p.slot_ds >= (pc_steps > 0 ? pc_steps : min_steps);
}

template <int R, int NTW>
int tt_launch(const tt_plan &p, const tt_args &a, hipStream_t stream) {
    hipLaunchKernelGGL((tr_tile_kernel<R, NTW>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_LDS, stream, a);
    GLQH_LAUNCH_CHECK("trellis tile launch");
    return 0;
}

template <int R2>
int tt_launch_rvq(const tt_plan &p, const tt_args &a, hipStream_t stream) {
    const dim3 grid((unsigned)p.grid), block(TT_THREADS);
    if (a.M <= 32) hipLaunchKernelGGL((tr_tile_small_kernel<4, 2, 1, R2>), grid, block, TT_SMALL_LDS, stream, a);
    else if (a.M <= 64) hipLaunchKernelGGL((tr_tile_small_kernel<4, 4, 1, R2>), grid, block, TT_SMALL_LDS, stream, a);
    else if (tt_split_roles(p, 8) && p.NTW == 1) hipLaunchKernelGGL((tr_tile_rvq_pc_kernel<R2, 2>), grid, block, TT_LDS, stream, a);
    else if (tt_split_roles(p, 8)) hipLaunchKernelGGL((tr_tile_rvq_pc_kernel<R2, 4>), grid, block, TT_LDS, stream, a);
    else if (p.NTW == 1) hipLaunchKernelGGL((tr_tile_rvq_kernel<R2, 1>), grid, block, TT_LDS, stream, a);
    else hipLaunchKernelGGL((tr_tile_rvq_kernel<R2, 2>), grid, block, TT_LDS, stream, a);
    GLQH_LAUNCH_CHECK("trellis two-stage tile launch");
    return 0;
}

template <int R, int TG, int NTW>
int tt_launch_small(const tt_plan &p, const tt_args &a, hipStream_t stream) {
    hipLaunchKernelGGL((tr_tile_small_kernel<R, TG, NTW>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_SMALL_LDS, stream, a);
    GLQH_LAUNCH_CHECK("trellis small tile launch");
    return 0;
}

template <int R>
int tt_launch_R(const tt_plan &p, const tt_args &a, hipStream_t stream) {
    // (with eight token groups, 65..256 tokens, the kernel above is as fast or faster: whole linear 4096 x 4096
    // 31.4 against 33.3 us at 128 tokens, 4096 x 14336 59.7 against 64.4 at 256, both in one run)
    if (a.M <= 32) return tt_launch_small<R, 2, 1>(p, a, stream);
    if (a.M <= 64) return tt_launch_small<R, 4, 1>(p, a, stream);
    if (tt_split_roles(p, 16)) {
        if (p.NTW == 1) hipLaunchKernelGGL((tr_tile_pc_kernel<R, 2>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_LDS, stream, a);
        else hipLaunchKernelGGL((tr_tile_pc_kernel<R, 4>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_LDS, stream, a);
        GLQH_LAUNCH_CHECK("trellis tile launch");
        return 0;
    }
    if (p.NTW == 1) return tt_launch<R, 1>(p, a, stream);
    if (p.NTW == 2) return tt_launch<R, 2>(p, a, stream);
    return tt_launch<R, 4>(p, a, stream);
}

template <typename K>
int tt_set_lds(K kernel) {
    return glqh_check_hip(hipFuncSetAttribute((const void *)kernel, hipFuncAttributeMaxDynamicSharedMemorySize,
                                              (int)TT_SMALL_LDS),
                          "trellis tile attribute");
}

template <int R>
int tt_init_R() {
    return tt_set_lds(tr_tile_small_kernel<R, 2, 1>) || tt_set_lds(tr_tile_small_kernel<R, 4, 1>) ||
           tt_set_lds(tr_tile_kernel<R, 1>) || tt_set_lds(tr_tile_kernel<R, 2>) || tt_set_lds(tr_tile_kernel<R, 4>) ||
           tt_set_lds(tr_tile_pc_kernel<R, 2>) || tt_set_lds(tr_tile_pc_kernel<R, 4>) ||
           tt_set_lds(tr_tile_rvq_pc_kernel<R, 2>) || tt_set_lds(tr_tile_rvq_pc_kernel<R, 4>) ||
           tt_set_lds(tr_tile_group_pc_kernel<R, 2>) || tt_set_lds(tr_tile_group_pc_kernel<R, 4>) ||
           tt_set_lds(tr_tile_moe_pc_kernel<R, 2>) || tt_set_lds(tr_tile_moe_pc_kernel<R, 4>) ||
           tt_set_lds(tr_tile_moe_rvq_pc_kernel<R, 2>) || tt_set_lds(tr_tile_moe_rvq_pc_kernel<R, 4>) ||
           tt_set_lds(tr_tile_group_kernel<R, 1>) || tt_set_lds(tr_tile_group_kernel<R, 2>) ||
           tt_set_lds(tr_tile_small_kernel<4, 2, 1, R>) || tt_set_lds(tr_tile_small_kernel<4, 4, 1, R>) ||
           tt_set_lds(tr_tile_rvq_kernel<R, 1>) || tt_set_lds(tr_tile_rvq_kernel<R, 2>) ||
           tt_set_lds(tr_tile_moe_rvq_kernel<R, 1>) || tt_set_lds(tr_tile_moe_rvq_kernel<R, 2>) ||
           tt_set_lds(tr_tile_group_kernel<R, 4>) || tt_set_lds(tr_tile_moe_kernel<R, 1>) ||
           tt_set_lds(tr_tile_moe_kernel<R, 2>) || tt_set_lds(tr_tile_moe_kernel<R, 4>);
}

}  // namespace

int glqh_trellis_tile_init(void) { return tt_init_R<1>() || tt_init_R<2>() || tt_init_R<3>() || tt_init_R<4>(); }

// bytes of the repacked activations of a many-token call
size_t glqh_trellis_tile_xb_bytes(int64_t k, int64_t M) { return (size_t)tt_padded_tokens(M) * k * sizeof(f16); }

// K slots the many-token kernel uses for this call (1: it can write the result in place)
int glqh_trellis_tile_ksplit(int64_t m, int64_t k, int64_t M, int two_stage) {
    tt_plan p;
    tt_make_plan(m, k, M, &p, two_stage ? 2 : 4);
    return p.KS;
}

// direct == 0: out[(slot * M + token) * m + row] = the slot's partial sum, unscaled (fp32) or times scale (out_f16);
// direct == 1 (one slot only): out[token * out_stride + row] = (accum ? out : 0) + scale * sum.
// x_f16 is (M, k) row-major; xb_scratch takes its repacked copy (glqh_trellis_tile_xb_bytes).
// tokens of the blocked activation layout: M padded to whole workgroup tiles
int64_t glqh_trellis_tile_padded_tokens(int64_t M) { return tt_padded_tokens(M); }

// packed2 (with R2, rs2): the residual stage of a stacked layer whose first stage has 4 bits/weight; both streams are
// decoded into one operand, W = fp16(W1 + rs2 * W2), in tiles of at most 256 tokens
// (glqh_trellis_tile_ksplit(.., two_stage = 1) gives the K slots).
int glqh_launch_trellis_tile(const void *x_f16, void *xb_scratch, int64_t M, const void *packed, int R, int64_t m,
                             int64_t k, float *out, int direct, float scale, int accum, int64_t out_stride,
                             hipStream_t stream, int out_f16, const void *packed2, int R2, float rs2) {
    if (packed2 && R != 4) return glqh_fail("trellis tile kernel: two streams in one operand need a first stage of 4 bits/weight");
    tt_plan p;
    tt_make_plan(m, k, M, &p, packed2 ? 2 : 4);
    if (direct && p.KS != 1) return glqh_fail("trellis tile kernel: in-place output needs a single K slot");
    if (out_f16 && (direct || M <= 64)) return glqh_fail("trellis tile kernel: fp16 sums are partial sums of the large tiles");
    const int Mp = (int)tt_padded_tokens(M);
    if (x_f16) {                                               // NULL: xb_scratch already holds the blocked layout
        hipLaunchKernelGGL(tr_pack_blocked_kernel<false>, dim3((unsigned)((M + 63) / 64), (unsigned)((k / 32 + 3) / 4)),
                           dim3(256), 0, stream, (const f16 *)x_f16, (f16 *)xb_scratch, (int)M, Mp, (int)k,
                           (const int *)nullptr, (const int *)nullptr, 1);
        GLQH_LAUNCH_CHECK("trellis pack launch");
    }
    tt_args a;
    a.packed = (const uint8_t *)packed;
    a.xb = (const f16 *)xb_scratch;
    a.M = (int)M;
    a.Mp = Mp;
    a.m = (int)m;
    a.k = (int)k;
    a.RT = p.RT;
    a.TT = p.TT;
    a.KS = p.KS;
    a.slot_ds = p.slot_ds;
    a.out = out;
    a.direct = direct;
    a.accum = accum;
    a.scale = scale;
    a.out_stride = out_stride;
    a.out_f16 = out_f16;
    a.rt0 = 0;
    a.packed2 = (const uint8_t *)packed2;
    a.rs2 = rs2;
    if (packed2) {
        switch (R2) {
        case 1: return tt_launch_rvq<1>(p, a, stream);
        case 2: return tt_launch_rvq<2>(p, a, stream);
        case 3: return tt_launch_rvq<3>(p, a, stream);
        case 4: return tt_launch_rvq<4>(p, a, stream);
        }
        return glqh_fail("trellis tile kernel: second stage of 1-4 bits/weight, got %d", R2);
    }
    // The last round of tiles: when the 512-token tiles fill at most half of the CUs in their last round,
    // the row tiles of that remainder go to a second launch as 256-token tiles, twice as many, each a good
    // half of the time (14336 rows at 4096 tokens: 896 tiles on 256 CUs = 3.5 rounds -> 3 rounds of 96 row
    // tiles + one of 16 row tiles x 16 half token tiles; both forms replayed from a graph in one run:
    // 577-586 -> 548 us).
    tt_plan tail = p;
    tail.RT = 0;
    const int cus = glqh_device_cus();
    if (p.NTW == 4 && p.KS == 1) {
        const int64_t T = (int64_t)p.RT * p.TT, rounds = T / cus, rem = T - rounds * cus;
        if (rounds >= 1 && rem > 0 && 2 * rem <= cus) {
            const int rt_tail = (int)((rem + p.TT - 1) / p.TT);
            const int tt2 = (int)((M + 255) / 256);
            if (rt_tail < p.RT && (int64_t)rt_tail * tt2 <= cus) {
                tail.RT = rt_tail;
                tail.TT = tt2;
                tail.NTW = 2;
                tail.grid = rt_tail * tt2;
                p.RT -= rt_tail;
                const int64_t items = (int64_t)p.RT * p.TT;
                p.grid = (int)(items < cus ? items : cus);
                a.RT = p.RT;
            }
        }
    }
    int rc = 1;
    switch (R) {
    case 1: rc = tt_launch_R<1>(p, a, stream); break;
    case 2: rc = tt_launch_R<2>(p, a, stream); break;
    case 3: rc = tt_launch_R<3>(p, a, stream); break;
    case 4: rc = tt_launch_R<4>(p, a, stream); break;
    default: return glqh_fail("trellis kernel supports R (bits/weight) 1-4, got %d", R);
    }
    if (rc || tail.RT == 0) return rc;
    a.rt0 = p.RT;
    a.RT = tail.RT;
    a.TT = tail.TT;
    tail.slot_ds = p.slot_ds;
    if (tt_split_roles(tail, 16)) {                            // 256-token tiles: decoding and multiplying waves
        const dim3 tgrid((unsigned)tail.grid), tblock(TT_THREADS);
        switch (R) {
        case 1: hipLaunchKernelGGL((tr_tile_pc_kernel<1, 4>), tgrid, tblock, TT_LDS, stream, a); break;
        case 2: hipLaunchKernelGGL((tr_tile_pc_kernel<2, 4>), tgrid, tblock, TT_LDS, stream, a); break;
        case 3: hipLaunchKernelGGL((tr_tile_pc_kernel<3, 4>), tgrid, tblock, TT_LDS, stream, a); break;
        default: hipLaunchKernelGGL((tr_tile_pc_kernel<4, 4>), tgrid, tblock, TT_LDS, stream, a); break;
        }
        GLQH_LAUNCH_CHECK("trellis tile launch");
        return 0;
    }
    switch (R) {
    case 1: return tt_launch<1, 2>(tail, a, stream);
    case 2: return tt_launch<2, 2>(tail, a, stream);
    case 3: return tt_launch<3, 2>(tail, a, stream);
    default: return tt_launch<4, 2>(tail, a, stream);
    }
}

// ---- several layers in one launch (many tokens) ---------------------------------------------------
namespace {
void tt_make_group_plan(const int64_t *m, int n_layers, int64_t k, int64_t M, tt_plan *p) {
    int64_t rt = 0, mtot = 0;
    for (int l = 0; l < n_layers; ++l) {
        rt += (m[l] + TT_ROWS - 1) / TT_ROWS;
        mtot += m[l];
    }
    tt_make_plan(TT_ROWS * rt, k, M, p);                        // same rule, on the row tiles of all layers
    (void)mtot;
}

template <int R>
int tt_launch_group_R(const tt_plan &p, const tt_args &a, const tt_group &g, hipStream_t stream) {
#define GLQH_TTG(NTW)                                                                                      \
    hipLaunchKernelGGL((tr_tile_group_kernel<R, NTW>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_LDS, stream, a, g)
#define GLQH_TTGP(NTW)                                                                                     \
    hipLaunchKernelGGL((tr_tile_group_pc_kernel<R, NTW>), dim3((unsigned)p.grid), dim3(TT_THREADS), TT_LDS, stream, a, g)
    if (tt_split_roles(p, 8) && p.NTW == 1) GLQH_TTGP(2);
    else if (tt_split_roles(p, 8)) GLQH_TTGP(4);
    else if (p.NTW == 1) GLQH_TTG(1);
    else if (p.NTW == 2) GLQH_TTG(2);
    else GLQH_TTG(4);
#undef GLQH_TTG
#undef GLQH_TTGP
    GLQH_LAUNCH_CHECK("trellis tile group launch");
    return 0;
}
}  // namespace

int glqh_trellis_tile_group_ksplit(const int64_t *m, int n_layers, int64_t k, int64_t M) {
    tt_plan p;
    tt_make_group_plan(m, n_layers, k, M, &p);
    return p.KS;
}

// Layers l < n_layers (at most 4) of the same width k and bits/weight against the same M > 64 tokens: partial
// sums out[l][(slot * M + token) * m[l] + row] (fp16 with out_f16, then times f16_scale[l] if given), K slots from
// glqh_trellis_tile_group_ksplit.
// xb[l]: the layer's activations in the blocked layout (glqh_trellis_tile_padded_tokens(M) tokens).
int glqh_launch_trellis_tile_group(const void *const xb[], int64_t M, const void *const packed[], int R,
                                   const int64_t m[], int n_layers, int64_t k, float *const out[], int out_f16,
                                   hipStream_t stream, const float f16_scale[]) {
    GLQH_REQUIRE(n_layers >= 1 && n_layers <= TT_MAX_GROUP, "trellis tile group: %d layers (1..%d)", n_layers, TT_MAX_GROUP);
    GLQH_REQUIRE(M > 64, "trellis tile group: more than 64 tokens");
    tt_plan p;
    tt_make_group_plan(m, n_layers, k, M, &p);
    tt_args a = {};
    tt_group g = {};
    g.n = n_layers;
    int rt = 0;
    for (int l = 0; l < n_layers; ++l) {
        g.packed[l] = (const uint8_t *)packed[l];
        g.xb[l] = (const f16 *)xb[l];
        g.out[l] = out[l];
        g.scale[l] = out_f16 && f16_scale ? f16_scale[l] : 1.0f;
        g.m[l] = (int)m[l];
        g.rt0[l] = rt;
        rt += (int)((m[l] + TT_ROWS - 1) / TT_ROWS);
    }
    a.M = (int)M;
    a.Mp = (int)tt_padded_tokens(M);
    a.m = 0;
    a.k = (int)k;
    a.RT = p.RT;
    a.TT = p.TT;
    a.KS = p.KS;
    a.slot_ds = p.slot_ds;
    a.out_f16 = out_f16;
    switch (R) {
    case 1: return tt_launch_group_R<1>(p, a, g, stream);
    case 2: return tt_launch_group_R<2>(p, a, g, stream);
    case 3: return tt_launch_group_R<3>(p, a, g, stream);
    case 4: return tt_launch_group_R<4>(p, a, g, stream);
    }
    return glqh_fail("trellis kernel supports R (bits/weight) 1-4, got %d", R);
}

// x (M, k) fp16 row-major -> the blocked layout of the tile kernels (glqh_trellis_tile_xb_bytes)
int glqh_launch_trellis_pack(const void *x_f16, void *xb, int64_t M, int64_t k, hipStream_t stream) {
    const int Mp = (int)tt_padded_tokens(M);
    hipLaunchKernelGGL(tr_pack_blocked_kernel<false>, dim3((unsigned)((M + 63) / 64), (unsigned)((k / 32 + 3) / 4)), dim3(256), 0,
                       stream, (const f16 *)x_f16, (f16 *)xb, (int)M, Mp, (int)k, (const int *)nullptr,
                       (const int *)nullptr, 1);
    GLQH_LAUNCH_CHECK("trellis pack launch");
    return 0;
}


// ---- routed experts with many rows per expert -----------------------------------------------------
// Positions per token tile of the routed-expert form for n_slots slots over n_experts experts, by the average
// number of rows per expert: 128 below 112, 256 below 224, 512 above (whole call, 128 experts of 2048 -> 2 x 768 ->
// 2048 with 8 choices, us with 128 / 256 / 512, the first two with decoding and multiplying waves: 48 rows 287 /
// 338 / 383, 96 rows 340 / 386 / 431, 128 rows 471 / 416 / 462, 160 rows 597 / 450 / 493, 192 rows 630 / 496 / 533,
// 256 rows 802 / 684 / 670).  GLQ_MOE_TILE_NTW (1, 2, 4; read once) forces 128 / 256 / 512.
int glqh_trellis_tile_moe_tokens(int64_t n_slots, int64_t n_experts) {
    static const int forced = [] { const char *e = getenv("GLQ_MOE_TILE_NTW"); return e ? atoi(e) : 0; }();
    if (forced == 1 || forced == 2 || forced == 4) return 128 * forced;
    const int64_t live = n_experts < n_slots ? n_experts : n_slots;
    const int64_t avg = n_slots / (live > 0 ? live : 1);
    return avg >= 224 ? 512 : avg >= 112 ? 256 : 128;
}

// positions of the packed activations: the slots plus one tile that a run's last tile may read into
int64_t glqh_trellis_tile_moe_padded(int64_t n_slots, int64_t n_experts) {
    return (n_slots + glqh_trellis_tile_moe_tokens(n_slots, n_experts) + 63) / 64 * 64;
}

// upper bound on the token tiles: every expert with rows ends in at most one partial tile
int64_t glqh_trellis_tile_moe_max_tiles(int64_t n_slots, int64_t n_experts) {
    const int64_t live = n_experts < n_slots ? n_experts : n_slots;
    return n_slots / glqh_trellis_tile_moe_tokens(n_slots, n_experts) + live + 1;
}

// tiles (glqh_trellis_tile_moe_max_tiles int4) and *n_tiles from the routing's offsets
int glqh_launch_trellis_tile_moe_table(const int *offs, int n_slots, int n_experts, void *tiles, int *n_tiles,
                                       hipStream_t stream) {
    hipLaunchKernelGGL(tr_moe_tiles_kernel, dim3(1), dim3(256), 0, stream, offs, n_experts,
                       glqh_trellis_tile_moe_tokens(n_slots, n_experts), (int4 *)tiles, n_tiles);
    GLQH_LAUNCH_CHECK("routed-expert tile table launch");
    return 0;
}

// xb[k-pair][position][q][8] from the transformed rows x (row of slot s = s / x_div), positions in the sorted order
int glqh_launch_trellis_pack_moe(const void *x_f16, void *xb, const int *perm, const int *offs, int n_slots,
                                 int n_experts, int x_div, int64_t k, hipStream_t stream) {
    const int Mp = (int)glqh_trellis_tile_moe_padded(n_slots, n_experts);
    hipLaunchKernelGGL(tr_pack_blocked_kernel<true>, dim3((unsigned)((n_slots + 63) / 64), (unsigned)((k / 32 + 3) / 4)),
                       dim3(256), 0, stream, (const f16 *)x_f16, (f16 *)xb, n_slots, Mp, (int)k, perm, offs + n_experts,
                       x_div);
    GLQH_LAUNCH_CHECK("routed-expert pack launch");
    return 0;
}

// out[slot][row] (fp16 with out_f16) = wscale[expert] * pscale[expert] * sum over k, for every slot with a valid expert
// packed2 (with stride2_bytes, R2; R = 4): stacked experts, both streams decoded into one operand with the expert's
// pscale_dev as the residual scale, W = fp16(W1 + pscale[e] * W2), in workgroup tiles of at most 256 positions.
int glqh_launch_trellis_tile_moe(const void *xb, const void *packed, int64_t stride_bytes, int R, const int *perm,
                                 const void *tiles, const int *n_tiles, const float *pscale_dev, const float *wscale_dev,
                                 int n_slots, int n_experts, int64_t m, int64_t k, void *out, int out_f16,
                                 hipStream_t stream, const void *packed2, int64_t stride2_bytes, int R2) {
    if (!wscale_dev) return glqh_fail("routed experts: the tile form needs the experts' scales");
    const int tile_tok = glqh_trellis_tile_moe_tokens(n_slots, n_experts);
    if (packed2 && (R != 4 || !pscale_dev)) return glqh_fail("routed experts: two streams in one operand need a 4-bit first stage and the residual scales");
    tt_args a = {};
    a.packed = (const uint8_t *)packed;
    a.xb = (const f16 *)xb;
    a.M = n_slots;
    a.Mp = (int)glqh_trellis_tile_moe_padded(n_slots, n_experts);
    a.m = (int)m;
    a.k = (int)k;
    a.RT = (int)((m + TT_ROWS - 1) / TT_ROWS);
    a.TT = packed2 && tile_tok == 512 ? 2 : 1;                  // workgroup tiles per run of the table
    a.KS = 1;
    a.slot_ds = (int)(k / 64);
    a.out = (float *)out;
    a.out_f16 = out_f16;
    a.packed2 = (const uint8_t *)packed2;
    const tt_moe mo = {stride_bytes, stride2_bytes, perm, (const int4 *)tiles, n_tiles, pscale_dev, wscale_dev};
    const int64_t max_items = glqh_trellis_tile_moe_max_tiles(n_slots, n_experts) * a.RT * a.TT;
    const int cus = glqh_device_cus();
    const dim3 grid((unsigned)(max_items < cus ? max_items : cus));
    tt_plan pl = {};
    pl.NTW = tile_tok == 128 ? 1 : 2;
    pl.slot_ds = a.slot_ds;
    const bool split = (packed2 || tile_tok <= 256) && tt_split_roles(pl, 8);
    if (packed2) {
#define GLQH_TTM2(RR)                                                                                              \
    do {                                                                                                           \
        if (split && tile_tok == 128)                                                                              \
            hipLaunchKernelGGL((tr_tile_moe_rvq_pc_kernel<RR, 2>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);  \
        else if (split)                                                                                            \
            hipLaunchKernelGGL((tr_tile_moe_rvq_pc_kernel<RR, 4>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);  \
        else if (tile_tok == 128)                                                                                  \
            hipLaunchKernelGGL((tr_tile_moe_rvq_kernel<RR, 1>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);     \
        else                                                                                                       \
            hipLaunchKernelGGL((tr_tile_moe_rvq_kernel<RR, 2>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);     \
    } while (0)
        switch (R2) {
        case 1: GLQH_TTM2(1); break;
        case 2: GLQH_TTM2(2); break;
        case 3: GLQH_TTM2(3); break;
        case 4: GLQH_TTM2(4); break;
        default: return glqh_fail("routed experts: second stage of 1-4 bits/weight, got %d", R2);
        }
#undef GLQH_TTM2
        GLQH_LAUNCH_CHECK("routed-expert two-stage tile launch");
        return 0;
    }
#define GLQH_TTM(RR)                                                                                          \
    do {                                                                                                      \
        if (split && tile_tok == 128)                                                                         \
            hipLaunchKernelGGL((tr_tile_moe_pc_kernel<RR, 2>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo); \
        else if (split)                                                                                       \
            hipLaunchKernelGGL((tr_tile_moe_pc_kernel<RR, 4>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo); \
        else if (tile_tok == 128)                                                                             \
            hipLaunchKernelGGL((tr_tile_moe_kernel<RR, 1>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);    \
        else if (tile_tok == 256)                                                                             \
            hipLaunchKernelGGL((tr_tile_moe_kernel<RR, 2>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);    \
        else                                                                                                  \
            hipLaunchKernelGGL((tr_tile_moe_kernel<RR, 4>), grid, dim3(TT_THREADS), TT_LDS, stream, a, mo);    \
    } while (0)
    switch (R) {
    case 1: GLQH_TTM(1); break;
    case 2: GLQH_TTM(2); break;
    case 3: GLQH_TTM(3); break;
    case 4: GLQH_TTM(4); break;
    default: return glqh_fail("trellis kernel supports R (bits/weight) 1-4, got %d", R);
    }
#undef GLQH_TTM
    GLQH_LAUNCH_CHECK("routed-expert tile launch");
    return 0;
}
