// Device helpers shared by the E8 shell codebook kernels that feed the matrix cores (gfx950).
#pragma once

#include "common.h"

typedef _Float16 f16x8 __attribute__((ext_vector_type(8)));

// eight 4-bit codes (interleaved: nibble p = column 2p, nibble p+4 = column 2p+1) -> 8 fp16.
// A code c in mantissa bits 0..3 of an fp16 with exponent 2^9 reads 512 + c/2, in bits 4..7
// it reads 512 + 8c; one fused multiply-add each gives c/2 - 3 exactly.  The upper byte of
// each half needs one shift first.
__device__ __forceinline__ uint32_t em_and_or(uint32_t a, uint32_t mask, uint32_t magic) {
    uint32_t d;                                    // (a & mask) | magic in one VOP3 (magic in a VGPR:
    asm("v_and_or_b32 %0, %1, %2, %3" : "=v"(d) : "v"(a), "s"(mask), "v"(magic));   // one scalar operand only)
    return d;
}

__device__ __forceinline__ f16x8 em_expand(uint32_t word) {
    const f16x2 one = {(f16)1.0f, (f16)1.0f}, sixteenth = {(f16)0.0625f, (f16)0.0625f};
    const f16x2 off0 = {(f16)-515.0f, (f16)-515.0f}, off1 = {(f16)-35.0f, (f16)-35.0f};
    const uint32_t magic = 0x60006000u;
    const uint32_t hi = word >> 8;
    const f16x2 p0 = __builtin_bit_cast(f16x2, em_and_or(word, 0x000F000Fu, magic));
    const f16x2 p1 = __builtin_bit_cast(f16x2, em_and_or(word, 0x00F000F0u, magic));
    const f16x2 p2 = __builtin_bit_cast(f16x2, em_and_or(hi, 0x000F000Fu, magic));
    const f16x2 p3 = __builtin_bit_cast(f16x2, em_and_or(hi, 0x00F000F0u, magic));
    u32x4 r;
    r[0] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(p0, one, off0));
    r[1] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(p1, sixteenth, off1));
    r[2] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(p2, one, off0));
    r[3] = __builtin_bit_cast(uint32_t, __builtin_elementwise_fma(p3, sixteenth, off1));
    return __builtin_bit_cast(f16x8, r);
}
