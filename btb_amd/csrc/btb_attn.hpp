// Decode attention's shared pieces (head_dim 128): the q / k RMSNorm + rope of one head by one wave, and a key
// stream's batch loads and online-softmax update - used by the stand-alone attention kernel that reads the fused qkv
// row (glue.hip) and by the persistent step (step.hip).
#pragma once

#include "btb_common.hpp"

namespace btb {

// device-scope relaxed access: a store written through to memory, a load that bypasses the caches - what two
// workgroups of one running kernel use to hand data to each other (the dies' L2s are not coherent with each other)
template <class T>
__device__ __forceinline__ T ld_dev(const T* p) {
    return __hip_atomic_load(p, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}
template <class T>
__device__ __forceinline__ void st_dev(T* p, T v) {
    __hip_atomic_store(p, v, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
}


constexpr int AD = 128;

// one head's 128 values: RMSNorm (weight wn or none), rope at `pos`; lane holds dims 2 * lane, 2 * lane + 1. In two
// steps, so that a caller can request the head's inputs, then other data, and only then wait for the inputs.
struct HeadIn {
    uint32_t raw, wn, cs, sn;  // the lane's pair of values, of norm weights, of cosines and of sines
};
template <bool DEV>
__device__ __forceinline__ HeadIn head_request(const uint16_t* src, const uint16_t* wn, const uint16_t* cos_t,
                                               const uint16_t* sin_t, int pos, int lane) {
    HeadIn in;
    const uint32_t* src2 = reinterpret_cast<const uint32_t*>(src) + lane;
    in.raw = DEV ? ld_dev(src2) : *src2;
    in.wn = reinterpret_cast<const uint32_t*>(wn != nullptr ? wn : cos_t)[lane];  // no weight: any word, unused
    in.cs = reinterpret_cast<const uint32_t*>(cos_t + (size_t)pos * AD)[lane];
    in.sn = reinterpret_cast<const uint32_t*>(sin_t + (size_t)pos * AD)[lane];
    return in;
}
__device__ __forceinline__ void head_finish(const HeadIn& in, bool has_wn, float eps, int centered, int lane,
                                            uint16_t (&out)[2]) {
    float v[2] = {bf16lo_f32(in.raw), bf16hi_f32(in.raw)};
    if (has_wn) {
        float ss = fmaf(v[1], v[1], fmaf(v[0], v[0], 0.f));
        ss = group_sum<64>(ss);
        const float rstd = rsqrtf(ss / (float)AD + eps);
        const float w2[2] = {bf16lo_f32(in.wn), bf16hi_f32(in.wn)};
#pragma unroll
        for (int e = 0; e < 2; ++e) v[e] = bfround(v[e] * rstd * (centered ? 1.f + w2[e] : w2[e]));
    }
    const float sgn = lane < 32 ? -1.f : 1.f;
    const float c2[2] = {bf16lo_f32(in.cs), bf16hi_f32(in.cs)}, s2[2] = {bf16lo_f32(in.sn), bf16hi_f32(in.sn)};
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float rot = __shfl_xor(v[e], 32, WAVE);
        const float qc = bfround(v[e] * c2[e]);
        out[e] = f32_bf16(fmaf(sgn * rot, s2[e], qc));
    }
}
template <bool DEV>
__device__ __forceinline__ void head_norm_rope(const uint16_t* src, const uint16_t* wn, float eps, int centered,
                                               const uint16_t* cos_t, const uint16_t* sin_t, int pos, int lane,
                                               uint16_t (&out)[2]) {
    const HeadIn in = head_request<DEV>(src, wn, cos_t, sin_t, pos, lane);
    head_finish(in, wn != nullptr, eps, centered, lane, out);
}

// one batch of a key stream: eight keys sixteen apart, their K and V rows (this lane's 8 dims) requested together
constexpr int KB = 8;
struct KeyBatch {
    uint4 k[KB], v[KB];
};
__device__ __forceinline__ void load_keys(KeyBatch& kb, const uint16_t* Kh, const uint16_t* Vh, long long rs, int key0,
                                          int k_end, int n0) {
#pragma unroll
    for (int b = 0; b < KB; ++b) {
        const int key = min(key0 + 16 * b, k_end - 1);  // a key past the span's end is loaded again, not used
        // slot n0 is this step's own row: it is taken from LDS, the cache's copy may not have landed yet
        const int safe = key == n0 ? max(n0 - 1, 0) : key;
        kb.k[b] = *reinterpret_cast<const uint4*>(Kh + (size_t)safe * rs);
        kb.v[b] = *reinterpret_cast<const uint4*>(Vh + (size_t)safe * rs);
    }
}

// the batch's keys, in ascending order, folded into the G query heads' online-softmax states (attn_decode_kernel's
// arithmetic). A key's rows are widened once and meet all G heads before the next key is touched.
template <int G>
__device__ __forceinline__ void use_keys(const KeyBatch& kb, int key0, int k_end, int n0, const uint16_t* s_k,
                                         const uint16_t* s_v, int dl, const float (&qv)[G][8], float (&m)[G],
                                         float (&l)[G], float (&acc)[G][8]) {
#pragma unroll
    for (int b = 0; b < KB; ++b) {
        if (key0 + 16 * b < k_end) {
            uint4 kr = kb.k[b], vr = kb.v[b];
            if (key0 + 16 * b == n0) {  // the step's own row, from LDS
                kr = *reinterpret_cast<const uint4*>(s_k + dl * 8);
                vr = *reinterpret_cast<const uint4*>(s_v + dl * 8);
            }
            const float kf[8] = {bf16lo_f32(kr.x), bf16hi_f32(kr.x), bf16lo_f32(kr.y), bf16hi_f32(kr.y),
                                 bf16lo_f32(kr.z), bf16hi_f32(kr.z), bf16lo_f32(kr.w), bf16hi_f32(kr.w)};
            const float vf[8] = {bf16lo_f32(vr.x), bf16hi_f32(vr.x), bf16lo_f32(vr.y), bf16hi_f32(vr.y),
                                 bf16lo_f32(vr.z), bf16hi_f32(vr.z), bf16lo_f32(vr.w), bf16hi_f32(vr.w)};
#pragma unroll
            for (int j = 0; j < G; ++j) {
                float sc = 0.f;
#pragma unroll
                for (int e = 0; e < 8; ++e) sc = fmaf(qv[j][e], kf[e], sc);
                sc = group_sum<16>(sc);
                const float mn = fmaxf(m[j], sc);
                const float corr = exp2f(m[j] - mn);  // 0 on the stream's first key (m = -inf)
                const float pp = exp2f(sc - mn);
                l[j] = fmaf(l[j], corr, pp);
#pragma unroll
                for (int e = 0; e < 8; ++e) acc[j][e] = fmaf(pp, vf[e], acc[j][e] * corr);
                m[j] = mn;
            }
        }
        __builtin_amdgcn_sched_barrier(0);  // a key at a time: widening every key's rows ahead costs the registers
    }
}

}  // namespace btb
