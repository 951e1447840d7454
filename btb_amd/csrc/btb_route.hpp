// The routing of one row of router logits by one wave (the routing kernels of moe.hip).
#pragma once

#include <type_traits>

#include "btb_common.hpp"

namespace btb {

template <bool F32>
__device__ __forceinline__ float logit_at(const void* base, size_t i) {
    return F32 ? static_cast<const float*>(base)[i] : bf16_f32(static_cast<const uint16_t*>(base)[i]);
}

__device__ __forceinline__ float wave_max(float v) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) v = fmaxf(v, __shfl_xor(v, s, WAVE));
    return v;
}

// Up to 256 experts: the row's probabilities stay in registers, P a lane, and a pick is the maximum of 64-bit keys
// (the probability's bits above the complement of the index: p >= 0, so the bits order as p does, and of equal p the
// lower index has the greater key). A taken key is 0, below every live one. The same arithmetic in the same order as
// moe_route_kernel (moe.hip), so the same picks and weights; a row of NaN probabilities takes the experts 0..k-1.
__device__ __forceinline__ unsigned long long wave_max_u64(unsigned long long v) {
    auto step = [&](auto ctrl) {
        constexpr int C = decltype(ctrl)::value;
        const uint32_t lo = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)v, C, 0xF, 0xF, true);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_update_dpp(0, (int)(uint32_t)(v >> 32), C, 0xF, 0xF, true);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        v = o > v ? o : v;
    };
    step(std::integral_constant<int, 0xB1>{});
    step(std::integral_constant<int, 0x4E>{});
    step(std::integral_constant<int, 0x141>{});
    step(std::integral_constant<int, 0x140>{});
    unsigned long long best = 0;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t lo = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)v, 16 * r);
        const uint32_t hi = (uint32_t)__builtin_amdgcn_readlane((int)(uint32_t)(v >> 32), 16 * r);
        const unsigned long long o = ((unsigned long long)hi << 32) | lo;
        best = o > best ? o : best;
    }
    return best;
}

// one wave routes row t, whose logits start at logits[base]
// this launch and are read past the first-level cache
template <bool F32, int P>
__device__ __forceinline__ void route_row_reg(const void* __restrict__ logits, size_t base, int t, int lane, int E, int k,
                                              int32_t* __restrict__ idx, uint16_t* __restrict__ w,
                                              float* __restrict__ w32, uint16_t* __restrict__ logits16) {
    float lv[P];
#pragma unroll
    for (int s = 0; s < P; ++s) {
        const int e = lane + WAVE * s;
        lv[s] = e < E ? logit_at<F32>(logits, base + e) : bits_f32(0xff800000u);
    }
    if (logits16 != nullptr) {
#pragma unroll
        for (int s = 0; s < P; ++s) {
            const int e = lane + WAVE * s;
            if (e < E) logits16[(size_t)t * E + e] = f32_bf16(lv[s]);
        }
    }
    float m = bits_f32(0xff800000u);
#pragma unroll
    for (int s = 0; s < P; ++s) m = fmaxf(m, lv[s]);
    m = wave_max(m);
    float pr[P], sum_p = 0.f;
#pragma unroll
    for (int s = 0; s < P; ++s) {
        const int e = lane + WAVE * s;
        pr[s] = e < E ? expf(lv[s] - m) : 0.f;
        if (e < E) sum_p += pr[s];
    }
    sum_p = wave_sum(sum_p);
    unsigned long long key[P];
#pragma unroll
    for (int s = 0; s < P; ++s) {
        const int e = lane + WAVE * s;
        const float p = pr[s] / sum_p;
        const uint32_t bits = p != p ? 0x7fc00000u : f32_bits(p);
        key[s] = e < E ? (((unsigned long long)bits << 32) | (0xFFFFFFFFu - (uint32_t)e)) : 0ull;
    }
    float topv = 0.f;  // lane j keeps pick j
    int topi = 0;
    for (int j = 0; j < k; ++j) {
        unsigned long long best = key[0];
#pragma unroll
        for (int s = 1; s < P; ++s) best = key[s] > best ? key[s] : best;
        best = wave_max_u64(best);
        const int e = (int)(0xFFFFFFFFu - (uint32_t)best);
        if (lane == j) {
            topv = bits_f32((uint32_t)(best >> 32));
            topi = e;
        }
#pragma unroll
        for (int s = 0; s < P; ++s)
            if (lane + WAVE * s == e) key[s] = 0ull;
    }
    float sum = 0.f;
    for (int j = 0; j < k; ++j) sum += __shfl(topv, j, WAVE);
    if (lane < k) {
        const float wv = topv / sum;
        const size_t o = (size_t)t * k + lane;
        idx[o] = topi;
        w[o] = f32_bf16(wv);
        if (w32 != nullptr) w32[o] = wv;
    }
}


}  // namespace btb
