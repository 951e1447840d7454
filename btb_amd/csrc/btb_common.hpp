// Shared device helpers for the gfx950 (CDNA4) decode kernels: bf16 bit handling, streaming loads, and
// cross-lane sums over a 64-wide wavefront in a fixed order.
#pragma once

#include <hip/hip_runtime.h>
#include <stddef.h>
#include <stdint.h>

namespace btb {

// return codes of the C ABI: the reference crate's (native/src/lib.rs:17-33)
constexpr int32_t OK = 0;
constexpr int32_t ERR_NULL = -1;
constexpr int32_t ERR_OVERFLOW = -5;
constexpr int32_t ERR_DOMAIN = -6;
constexpr int32_t ERR_PANIC = -7;  // a HIP runtime error at the boundary (the crate's "panic caught")
// between the library's own files only, never across the C ABI: "this form of the kernel does not take the shape"
constexpr int32_t ERR_UNSUPPORTED = -100;

constexpr int WAVE = 64;

typedef __attribute__((ext_vector_type(2))) float f32x2;
typedef __attribute__((ext_vector_type(4))) float f32x4;
typedef __attribute__((ext_vector_type(2))) __bf16 bf16x2;
typedef __attribute__((ext_vector_type(8))) __bf16 bf16x8;

__host__ __device__ __forceinline__ float bits_f32(uint32_t b) {
    union {
        uint32_t u;
        float f;
    } v;
    v.u = b;
    return v.f;
}
__host__ __device__ __forceinline__ uint32_t f32_bits(float f) {
    union {
        uint32_t u;
        float f;
    } v;
    v.f = f;
    return v.u;
}

// a bf16 bit pattern as f32: exact
__host__ __device__ __forceinline__ float bf16_f32(uint16_t b) { return bits_f32((uint32_t)b << 16); }
// the two bf16 halves of a dword as f32
__host__ __device__ __forceinline__ float bf16lo_f32(uint32_t p) { return bits_f32(p << 16); }
__host__ __device__ __forceinline__ float bf16hi_f32(uint32_t p) { return bits_f32(p & 0xFFFF0000u); }

// nearest bf16, ties to even, by integer arithmetic (the reference's round_bf16, native/src/gemv.rs:3003-3007),
// kept as f32
__host__ __device__ __forceinline__ float round_bf16_f32(float f) {
    const uint32_t b = f32_bits(f);
    return bits_f32((b + 0x7FFFu + ((b >> 16) & 1u)) & 0xFFFF0000u);
}

// f32 to a stored bf16: nearest even; a NaN becomes the quiet NaN torch's cast writes (sign kept). On the device this
// is one v_cvt_pk_bf16_f32, which gives the integer rule's bits on every input - finite values, ties, denormals,
// infinities, and NaNs of any payload (btb_hip_round_bf16 exposes it; tests/test_widen_gpu.py holds it to the
// integer rule over bit patterns of every kind) - where the rule itself is nine instructions and sat in every
// staging loop.
__host__ __device__ __forceinline__ uint16_t f32_bf16(float f) {
#if defined(__HIP_DEVICE_COMPILE__)
    return __builtin_bit_cast(uint16_t, (__bf16)f);
#else
    const uint32_t b = f32_bits(f);
    if ((b & 0x7FFFFFFFu) > 0x7F800000u) return (uint16_t)((b >> 16) | 0x0040u);
    return (uint16_t)((b + 0x7FFFu + ((b >> 16) & 1u)) >> 16);
#endif
}
__host__ __device__ __forceinline__ float bfround(float f) { return bf16_f32(f32_bf16(f)); }
// two values as a packed pair of stored bf16 (lo in the low half): one conversion instruction on the device
__host__ __device__ __forceinline__ uint32_t f32x2_bf16(float lo, float hi) {
#if defined(__HIP_DEVICE_COMPILE__)
    typedef __attribute__((ext_vector_type(2))) __bf16 pair_t;
    const pair_t p = {(__bf16)lo, (__bf16)hi};
    return __builtin_bit_cast(uint32_t, p);
#else
    return (uint32_t)f32_bf16(lo) | ((uint32_t)f32_bf16(hi) << 16);
#endif
}

// a 16-byte streaming load of weights: read once per token, so it is marked non-temporal
typedef __attribute__((ext_vector_type(4))) uint32_t u32x4;
typedef __attribute__((ext_vector_type(2))) uint32_t u32x2;
__device__ __forceinline__ uint4 load_stream16(const uint4* p) {
    const u32x4 v = __builtin_nontemporal_load(reinterpret_cast<const u32x4*>(p));
    return make_uint4(v.x, v.y, v.z, v.w);
}
__device__ __forceinline__ uint2 load_stream8(const uint2* p) {
    const u32x2 v = __builtin_nontemporal_load(reinterpret_cast<const u32x2*>(p));
    return make_uint2(v.x, v.y);
}
__device__ __forceinline__ uint32_t load_stream4(const uint32_t* p) { return __builtin_nontemporal_load(p); }

template <int CTRL, int ROW_MASK = 0xF, int BANK_MASK = 0xF, bool BOUND = true>
__device__ __forceinline__ float dpp_f32(float v) {
    return __builtin_bit_cast(
        float, __builtin_amdgcn_update_dpp(0, __builtin_bit_cast(int, v), CTRL, ROW_MASK, BANK_MASK, BOUND));
}

// sum over each aligned group of LANES lanes (16, 32 or 64), the same fixed tree whatever the data; every
// lane of the group's first row of 16 ends up holding it (lane 0 of the group is the one that is read)
template <int LANES>
__device__ __forceinline__ float group_sum(float v) {
    v += dpp_f32<0xB1>(v);   // quad_perm [1,0,3,2]: lane ^ 1
    v += dpp_f32<0x4E>(v);   // quad_perm [2,3,0,1]: lane ^ 2
    v += dpp_f32<0x141>(v);  // row_half_mirror: the other quad of each 8
    v += dpp_f32<0x140>(v);  // row_mirror: the other half of each 16
    if (LANES >= 32) v += __shfl_xor(v, 16, WAVE);
    if (LANES >= 64) v += __shfl_xor(v, 32, WAVE);
    return v;
}

// The same sum, the same bits (the same pairs are added, some the other way round), for a caller that needs it in one
// lane only: the group's LAST lane. The steps across rows of 16 are row broadcasts on the vector ALU (lane 15 of a row
// into the next row, lane 31 into the upper half) in place of two exchanges through the LDS unit, which a wave's
// last tile has nothing to hide behind. Other lanes end up with partial sums.
template <int LANES>
__device__ __forceinline__ float group_sum_last(float v) {
    v += dpp_f32<0xB1>(v);
    v += dpp_f32<0x4E>(v);
    v += dpp_f32<0x141>(v);
    v += dpp_f32<0x140>(v);
    if (LANES >= 32) v += dpp_f32<0x142, 0xA>(v);  // row_bcast:15 into rows 1 and 3 (the others add 0)
    if (LANES >= 64) v += dpp_f32<0x143, 0xC>(v);  // row_bcast:31 into rows 2 and 3
    return v;
}
// the whole wave's sum in every lane: the last lane's, handed round as a scalar. The same bits as group_sum<64>
// (there every lane ends with the same pairs added, some the other way round).
__device__ __forceinline__ float wave_sum(float v) {
    v = group_sum_last<64>(v);
    return __builtin_bit_cast(float, __builtin_amdgcn_readlane(__builtin_bit_cast(int, v), 63));
}
// lane l ^ 32's value, on the vector ALU: v_permlane32_swap of a register with itself leaves the lower half's values
// in both halves of one result and the upper half's in both halves of the other. (__shfl_xor goes through the LDS unit.)
__device__ __forceinline__ float xor32(float v) {
    const int i = __builtin_bit_cast(int, v);
    const auto r = __builtin_amdgcn_permlane32_swap(i, i, false, false);
    return __builtin_bit_cast(float, (threadIdx.x & 32) ? r[0] : r[1]);
}
// a value of the last lane of the lower neighbouring group of LANES lanes (16 or 32), in the lanes of the upper one
template <int LANES>
__device__ __forceinline__ float from_lower_group(float v) {
    static_assert(LANES == 16 || LANES == 32, "groups of 16 or 32 lanes");
    return LANES == 16 ? dpp_f32<0x142, 0xA>(v) : dpp_f32<0x143, 0xC>(v);
}

}  // namespace btb
