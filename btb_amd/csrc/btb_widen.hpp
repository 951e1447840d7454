// The stored weight forms and their in-register widening. Each form is a policy the streaming matvec kernel is
// instantiated over: what one lane loads in one step (a "unit" of UW consecutive weights of a row) and how those
// bytes become f32 weights. The scalar decode functions are __host__ __device__, so the same source is compiled
// for the CPU in the tests and checked there against the oracle, bit for bit, where no GPU is present.
//
//   bf16    bits << 16                                                   (reference: native/src/gemv.rs:40-43)
//   pack12  (table[code] << 24) | (lo << 16), escapes patched by index   (native/src/gemv.rs:769-793, 736-767)
//   fp8     bf16_rne(e4m3fn(byte) * block_scale) as f32                  (native/src/gemv.rs:2996-3085)
//   mxfp4   fp4_e2m1(nibble) * 2^(scale - 127), low nibble first         (native/src/gemv.rs:1032-1119)
#pragma once

#include "btb_common.hpp"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// scalar decodes (host + device): the definitions the vector forms below must equal
// ------------------------------------------------------------------------------------------------------------

// pack12: weight `i` of a packed tensor before its escape is applied
__host__ __device__ __forceinline__ uint16_t p12_plain_bits(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table,
                                                            size_t i) {
    const uint8_t byte = hi4[i >> 1];
    const unsigned code = (i & 1) ? (byte >> 4) : (byte & 0x0F);
    return (uint16_t)(((unsigned)table[code] << 8) | lo[i]);
}

// e4m3fn byte to f32 by integer arithmetic: exponent 0 is m * 2^-9, 0x7F / 0xFF are NaN, there is no infinity
__host__ __device__ __forceinline__ float f8_e4m3_f32(uint8_t b) {
    const uint32_t a = b & 0x7Fu;
    uint32_t mag;
    if (a == 0x7Fu)
        mag = 0x7FC00000u;
    else if (a < 8u)
        mag = f32_bits((float)a * (1.0f / 512.0f));
    else
        mag = (a << 20) + (120u << 23);
    return bits_f32(mag | ((uint32_t)(b & 0x80u) << 24));
}

// the weight an FP8 byte stands for under its block's scale: the nearest bf16 to e4m3 * scale, as f32
__host__ __device__ __forceinline__ float f8_held(uint8_t b, float scale) {
    return round_bf16_f32(f8_e4m3_f32(b) * scale);
}

// fp4 e2m1 code to f32: 0, .5, 1, 1.5, 2, 3, 4, 6 and their negatives
__host__ __device__ __forceinline__ float fp4_e2m1_f32(unsigned code) {
    // bf16 patterns of the eight magnitudes, two to a dword
    const uint32_t pats[4] = {0x3F000000u, 0x3FC03F80u, 0x40404000u, 0x40C04080u};
    const unsigned m = code & 7u;
    const uint32_t p = (pats[m >> 1] >> ((m & 1u) * 16u)) & 0xFFFFu;
    return bits_f32((p << 16) | ((uint32_t)(code & 8u) << 28));
}

// 2^(s - 127) exactly for an e8m0 byte: s == 0 is 2^-127 (built as 2^-126 * 0.5), s == 255 is +inf
__host__ __device__ __forceinline__ float e8m0_f32(uint8_t s) {
    const float f = bits_f32((uint32_t)(s == 0 ? 1 : s) << 23);
    return s == 0 ? f * 0.5f : f;
}

__host__ __device__ __forceinline__ float mx4_weight(uint8_t byte, int high, uint8_t scale) {
    return fp4_e2m1_f32(high ? (byte >> 4) : (byte & 0x0F)) * e8m0_f32(scale);
}

}  // namespace btb
