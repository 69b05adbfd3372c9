// Device helpers shared by the trellis-3INST kernels: record loads, continuation bits,
// state extraction and the 3INST hash (glq/trellis.py:122-134, 486-523, 580-602;
// glq/csrc/glq_trellis.cu:138-143, 264-271).
#pragma once
#include "common.h"

namespace {

constexpr int TR_WAVES = 4;
constexpr int TR_THREADS = TR_WAVES * GLQH_WAVE;
constexpr int TR_PRE = 4;      // records a wave keeps in flight in the fused-input GEMV

// (s * 89226354 + 64248484) mod 2^32, masked and xored: the two fp16 halves of 3INST.
// The multiply-add is issued as one v_mad_u64_u32 (its low half is the 32-bit result): measured
// 1.3 issue slots on gfx950 against 2 for v_mul_lo_u32 + v_add_u32, and the decode is bound by
// vector-ALU issue.
__device__ __forceinline__ uint32_t tr_hash(uint32_t s) {
#ifdef GLQH_HASH_MUL_ADD
    uint32_t h = s * 89226354u + 64248484u;
#else
    uint64_t wide, carry;
    asm("v_mad_u64_u32 %0, %1, %2, %3, %4"
        : "=v"(wide), "=s"(carry)
        : "v"(s), "v"(89226354u), "s"((uint64_t)64248484ull));
    uint32_t h = (uint32_t)wide;
#endif
    return (h & 0x8FFF8FFFu) ^ 0x3B603B60u;
}

// Exact reference weight: the two halves added in fp16 with one rounding.
__device__ __forceinline__ f16 tr_weight(uint32_t s) {
    f16x2 r = __builtin_bit_cast(f16x2, tr_hash(s));
    return r.y + r.x;
}

template <int R>
struct tr_record {
    uint32_t c[4];      // 8R-bit chunks of tiles (k0,m0),(k0,m1),(k1,m0),(k1,m1)
    uint32_t raw;       // R == 1 only: the four 8-bit chunks as loaded
};

template <int R>
__device__ __forceinline__ tr_record<R> tr_load_record(const uint8_t *__restrict__ p) {
    tr_record<R> r;
    r.raw = 0;
    if constexpr (R == 4) {
        u32x4 v = __builtin_nontemporal_load((const u32x4 *)p);
        r.c[0] = v.x; r.c[1] = v.y; r.c[2] = v.z; r.c[3] = v.w;
    } else if constexpr (R == 3) {
        const uint32_t *q = (const uint32_t *)p;
        uint32_t r0 = __builtin_nontemporal_load(q);
        uint32_t r1 = __builtin_nontemporal_load(q + 1);
        uint32_t r2 = __builtin_nontemporal_load(q + 2);
        r.c[0] = r0 & 0xFFFFFFu;
        r.c[1] = ((r0 >> 24) | (r1 << 8)) & 0xFFFFFFu;
        r.c[2] = ((r1 >> 16) | (r2 << 16)) & 0xFFFFFFu;
        r.c[3] = r2 >> 8;
    } else if constexpr (R == 2) {
        u32x2 v = __builtin_nontemporal_load((const u32x2 *)p);
        r.c[0] = v.x & 0xFFFFu; r.c[1] = v.x >> 16;
        r.c[2] = v.y & 0xFFFFu; r.c[3] = v.y >> 16;
    } else {
        uint32_t v = __builtin_nontemporal_load((const uint32_t *)p);
        r.raw = v;
        r.c[0] = v & 0xFFu; r.c[1] = (v >> 8) & 0xFFu;
        r.c[2] = (v >> 16) & 0xFFu; r.c[3] = v >> 24;
    }
    return r;
}

// 16 continuation bits per chunk, fetched from the lanes that hold stream lanes l+1 (and
// l+2 for R = 1) of the same block.
template <int R>
__device__ __forceinline__ void tr_continuation_from(const tr_record<R> &r, int next1, int next2,
                                                     uint32_t cont[4]) {
    if constexpr (R >= 2) {
        constexpr int sh = 8 * R - 16;
        uint32_t t01 = ((r.c[0] >> sh) & 0xFFFFu) | (((r.c[1] >> sh) & 0xFFFFu) << 16);
        uint32_t t23 = ((r.c[2] >> sh) & 0xFFFFu) | (((r.c[3] >> sh) & 0xFFFFu) << 16);
        uint32_t n01 = (uint32_t)__shfl((int)t01, next1, GLQH_WAVE);
        uint32_t n23 = (uint32_t)__shfl((int)t23, next1, GLQH_WAVE);
        cont[0] = n01 & 0xFFFFu; cont[1] = n01 >> 16;
        cont[2] = n23 & 0xFFFFu; cont[3] = n23 >> 16;
    } else {
        uint32_t a = (uint32_t)__shfl((int)r.raw, next1, GLQH_WAVE);
        uint32_t b = (uint32_t)__shfl((int)r.raw, next2, GLQH_WAVE);
#pragma unroll
        for (int i = 0; i < 4; ++i)
            cont[i] = (((a >> (8 * i)) & 0xFFu) << 8) | ((b >> (8 * i)) & 0xFFu);
    }
}

// lanes 0..31 / 32..63 each hold the 32 stream lanes of one block in order
template <int R>
__device__ __forceinline__ void tr_continuation(const tr_record<R> &r, int lane, uint32_t cont[4]) {
    const int half = lane & 32;
    tr_continuation_from<R>(r, half | ((lane + 1) & 31), half | ((lane + 2) & 31), cont);
}

template <int R>
__device__ __forceinline__ uint32_t tr_state(uint32_t chunk, uint32_t cont, int j) {
    uint64_t ext = ((uint64_t)chunk << 16) | cont;
    return (uint32_t)(ext >> (8 * R - R * j)) & 0xFFFFu;
}

// One A operand: four words (a.lo + a.hi, b.lo + b.hi) in fp16 from eight hash results, as
// eight SDWA adds.  gfx950 needs one wait state between an instruction that writes part of a
// register (dst_sel) and the next one that reads that register, and the compiler cannot see
// into an asm block: the four low-half writes come first and the four high-half writes (which
// read their destination to preserve it) after them, and a trailing s_nop covers whoever reads
// the last word next.  (Adjacent pairs, as this was first written, gave wrong rows once the
// scheduler moved an MFMA right behind them.)
__device__ __forceinline__ u32x4 pair_sum4(uint32_t a0, uint32_t b0, uint32_t a1, uint32_t b1, uint32_t a2,
                                           uint32_t b2, uint32_t a3, uint32_t b3) {
    uint32_t d0, d1, d2, d3;
    asm("v_add_f16_sdwa %0, %4, %4 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %1, %6, %6 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %2, %8, %8 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %3, %10, %10 dst_sel:WORD_0 dst_unused:UNUSED_PAD src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %0, %5, %5 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %1, %7, %7 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %2, %9, %9 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "v_add_f16_sdwa %3, %11, %11 dst_sel:WORD_1 dst_unused:UNUSED_PRESERVE src0_sel:WORD_0 src1_sel:WORD_1\n\t"
        "s_nop 0"
        : "=&v"(d0), "=&v"(d1), "=&v"(d2), "=&v"(d3)
        : "v"(a0), "v"(b0), "v"(a1), "v"(b1), "v"(a2), "v"(b2), "v"(a3), "v"(b3));
    return u32x4{d0, d1, d2, d3};
}

}  // namespace
