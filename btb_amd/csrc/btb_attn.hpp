// Decode attention's shared pieces (head_dim 128): the q / k RMSNorm + rope of one head by one wave, and a key
// stream's batch loads and online-softmax update - used by the stand-alone attention kernel that reads the fused qkv
// row (glue.hip).
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
        ss = wave_sum(ss);
        const float rstd = rsqrtf(ss / (float)AD + eps);
        const float w2[2] = {bf16lo_f32(in.wn), bf16hi_f32(in.wn)};
#pragma unroll
        for (int e = 0; e < 2; ++e) v[e] = bfround(v[e] * rstd * (centered ? 1.f + w2[e] : w2[e]));
    }
    const float sgn = lane < 32 ? -1.f : 1.f;
    const float c2[2] = {bf16lo_f32(in.cs), bf16hi_f32(in.cs)}, s2[2] = {bf16lo_f32(in.sn), bf16hi_f32(in.sn)};
#pragma unroll
    for (int e = 0; e < 2; ++e) {
        const float rot = xor32(v[e]);
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

// A pass whose T rows are T sequences of their own, a token each (a fork's rows, which share one prefix, or a batch's,
// which lie end to end) - the reference's rows layout (native/cuda/btb_kernels.cu:232-249): one int32 array on the
// device, [base, steps, W, then (col, off, len) a row]. Row t's keys in logical order are its prefix - len cache
// slots from off - and then its own steps, step i at slot base + i * W + col; it stands at position len + steps.
// len < 0: a padding row, for which nothing is computed.
struct SeqPlace {
    int base, step, W, col, off, len;
    __device__ __forceinline__ void read(const int32_t* rw, int t) {
        base = rw[0], step = rw[1], W = rw[2];
        col = rw[3 + 3 * t], off = rw[4 + 3 * t], len = rw[5 + 3 * t];
    }
    __device__ __forceinline__ int slot(int j) const { return j < len ? off + j : base + (j - len) * W + col; }
};

// one batch of a key stream: eight keys sixteen apart, their K and V rows (this lane's 8 dims) requested together
constexpr int KB = 8;
struct KeyBatch {
    uint4 k[KB], v[KB];
};
__device__ __forceinline__ void load_keys(KeyBatch& kb, const uint16_t* Kh, const uint16_t* Vh, long long rs, int key0,
                                          int k_end, int n0, const int32_t* tbl = nullptr,
                                          const SeqPlace* seq = nullptr) {
#pragma unroll
    for (int b = 0; b < KB; ++b) {
        const int key = min(key0 + 16 * b, k_end - 1);  // a key past the span's end is loaded again, not used
        // slot n0 is this step's own row: it is taken from LDS, the cache's copy may not have landed yet
        int safe = key == n0 ? max(n0 - 1, 0) : key;
        // the cache's row map (the reference's `tbl`, native/cuda/btb_attn_flash.cuh:34): logical slot -> cache row;
        // or the row's own sequence: logical key -> cache slot
        if (tbl != nullptr) safe = tbl[safe];
        if (seq != nullptr) safe = seq->slot(safe);
        kb.k[b] = *reinterpret_cast<const uint4*>(Kh + (size_t)safe * rs);
        kb.v[b] = *reinterpret_cast<const uint4*>(Vh + (size_t)safe * rs);
    }
}

// the same batch with addresses that do not depend on how many keys the cache holds: a key at or past `lim` (the end of
// the span or of the cache's capacity) reads slot lim - 1 again. Which of the batch's keys count is decided when they
// are used; the step's own slot may be read here before its row has landed - use_keys takes that key from LDS.
__device__ __forceinline__ void load_keys_upto(KeyBatch& kb, const uint16_t* Kh, const uint16_t* Vh, long long rs,
                                               int key0, int lim) {
#pragma unroll
    for (int b = 0; b < KB; ++b) {
        const int key = min(key0 + 16 * b, lim - 1);
        kb.k[b] = *reinterpret_cast<const uint4*>(Kh + (size_t)key * rs);
        kb.v[b] = *reinterpret_cast<const uint4*>(Vh + (size_t)key * rs);
    }
}

// ------------------------------------------------------------------------------------------------------------
// A key stream's state and the fold of one batch of keys into it.
//
// A stream is a group of 16 lanes; a lane holds 8 dims of every key row it loads. A batch is 8 keys; with G query heads
// that is 8 G scores, each a sum over the 16 lanes. They are summed "transposed": the 16 lanes start with 8 G partial
// sums each and end with 8 G / 16 finished scores each (lane dl: key dl % 8, head 2 r + dl / 8 in slot r; one head: both
// halves of the group hold the same 8), so a score is scaled, masked and exponentiated once, by one lane, and a
// batch's maximum is a three-step exchange among the 8 lanes of a head. The weights then go back to all 16 lanes through
// a few words of LDS (the stream's exchange area; a wave's own LDS traffic is served in order, so no barrier), two
// neighbouring keys' weights rounded to bf16 and packed in a word: the value rows of the two keys are zipped into bf16
// pairs as well and meet the weights in v_dot2_f32_bf16 (products exact, f32 sums). The running sum is made of the
// same rounded weights, so the weights of a head still add up to one - the reference's card kernel rounds its
// weights to bf16 for its tensor cores in the same way (native/cuda/btb_attn_flash.cuh:90-125).
// ------------------------------------------------------------------------------------------------------------
constexpr int attn_slots(int G) { return G <= 2 ? 1 : G / 2; }
constexpr int XCH = 48;  // floats of LDS a stream exchanges through: weight pairs at 0.., corrections at 32.., heads' state

template <int G>
struct AttnState {
    static constexpr int R = attn_slots(G);
    float ms[R];      // running maximum of the slot's head, log2 units (the same in the 8 lanes of a head)
    float ls[R];      // this lane's share of the running sum: its own key slot's weights
    float acc[G][8];  // the heads' outputs, this lane's 8 dims
    __device__ __forceinline__ void init() {
#pragma unroll
        for (int r = 0; r < R; ++r) {
            ms[r] = bits_f32(0xff800000u);
            ls[r] = 0.f;
        }
#pragma unroll
        for (int j = 0; j < G; ++j)
#pragma unroll
            for (int e = 0; e < 8; ++e) acc[j][e] = 0.f;
    }
};
template <int G>
__device__ __forceinline__ int slot_head(int r, int dl) {
    return G == 1 ? 0 : 2 * r + (dl >> 3);
}

// 16 values a lane, summed over the 16 lanes of the group: lane dl ends up with the sum of value dl. Each step pairs
// the lanes off (15 - i, then 7 - i within 8, i ^ 2, i ^ 1), a lane keeping the half of its values its side of the
// pairing owns, plus the partner's same half.
__device__ __forceinline__ float tsum16(const float* v, int dl) {
    float a[8], b[4], c[2];
    const bool u1 = dl >= 8, u2 = (dl & 7) >= 4, u3 = (dl & 3) >= 2, u4 = (dl & 1) != 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) {
        const float lo = v[k] + dpp_f32<0x140>(v[k]), hi = v[k + 8] + dpp_f32<0x140>(v[k + 8]);
        a[k] = u1 ? hi : lo;
    }
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float lo = a[k] + dpp_f32<0x141>(a[k]), hi = a[k + 4] + dpp_f32<0x141>(a[k + 4]);
        b[k] = u2 ? hi : lo;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float lo = b[k] + dpp_f32<0x4E>(b[k]), hi = b[k + 2] + dpp_f32<0x4E>(b[k + 2]);
        c[k] = u3 ? hi : lo;
    }
    const float lo = c[0] + dpp_f32<0xB1>(c[0]), hi = c[1] + dpp_f32<0xB1>(c[1]);
    return u4 ? hi : lo;
}
// 8 values a lane: lane dl ends up with the sum of value dl % 8
__device__ __forceinline__ float tsum8(const float* v, int dl) {
    float a[8], b[4], c[2];
    const bool u2 = (dl & 7) >= 4, u3 = (dl & 3) >= 2, u4 = (dl & 1) != 0;
#pragma unroll
    for (int k = 0; k < 8; ++k) a[k] = v[k] + dpp_f32<0x140>(v[k]);
#pragma unroll
    for (int k = 0; k < 4; ++k) {
        const float lo = a[k] + dpp_f32<0x141>(a[k]), hi = a[k + 4] + dpp_f32<0x141>(a[k + 4]);
        b[k] = u2 ? hi : lo;
    }
#pragma unroll
    for (int k = 0; k < 2; ++k) {
        const float lo = b[k] + dpp_f32<0x4E>(b[k]), hi = b[k + 2] + dpp_f32<0x4E>(b[k + 2]);
        c[k] = u3 ? hi : lo;
    }
    const float lo = c[0] + dpp_f32<0xB1>(c[0]), hi = c[1] + dpp_f32<0xB1>(c[1]);
    return u4 ? hi : lo;
}

// The batch's keys folded into the stream's state. A key past the span's end scores -inf and weighs 0. qp: the heads'
// q, this lane's 8 dims as 4 bf16 pairs. own >= 0: the step's own row is key `own` and is taken from LDS (s_k, s_v) -
// the cache's copy may not have landed yet. tree_base >= 0: the keys from slot tree_base on are the pass's own rows,
// and of those the row sees the ones whose bit is set in tree_mask (its ancestors and itself: a verify pass's tree).
// ZERO_DEAD: a key that does not count may have been loaded from a slot the cache has never written
// (load_keys_upto), so its value row is taken as zeros - weight 0 times whatever bits lie there must not make a NaN.
// xch: the stream's XCH floats of LDS.
template <int G, bool ZERO_DEAD = false>
__device__ __forceinline__ void use_keys(KeyBatch& kb, int key0, int k_end, int own, const uint16_t* s_k,
                                         const uint16_t* s_v, int dl, const uint32_t (&qp)[G][4], float scale_log2,
                                         AttnState<G>& st, float* xch, int tree_base = -1, uint32_t tree_mask = 0u,
                                         int k_first = 0) {
    constexpr int R = attn_slots(G);
    static_assert(G == 1 || G == 2 || G == 4 || G == 8, "1, 2, 4 or 8 query heads a stream");
    const float ninf = bits_f32(0xff800000u);
    if (own >= 0) {  // uniform: only a workgroup whose span holds the slot gets here with own set
#pragma unroll
        for (int b = 0; b < KB; ++b)
            if (key0 + 16 * b == own) {
                kb.k[b] = *reinterpret_cast<const uint4*>(s_k + dl * 8);
                kb.v[b] = *reinterpret_cast<const uint4*>(s_v + dl * 8);
            }
    }
    // this lane's 8 dims of every (head, key) score
    float part[(G == 1 ? 1 : G) * KB];
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
        for (int b = 0; b < KB; ++b) {
            const uint4 kr = kb.k[b];
            float sc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr.x), __builtin_bit_cast(bf16x2, qp[j][0]), 0.f, false);
            sc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr.y), __builtin_bit_cast(bf16x2, qp[j][1]), sc, false);
            sc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr.z), __builtin_bit_cast(bf16x2, qp[j][2]), sc, false);
            sc = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, kr.w), __builtin_bit_cast(bf16x2, qp[j][3]), sc, false);
            part[j * KB + b] = sc;
        }
    // the lane's own key slot
    const int bk = dl & 7;
    const int key = key0 + 16 * bk;
    // a cache key counts from the window's first key on (k_first; 0: no window); one of the pass's own rows counts when
    // the mask names it (the window is already in the mask: those rows stand at their depth, not at their slot)
    bool live = key < k_end;
    if (tree_base >= 0 && key >= tree_base)
        live = live && ((tree_mask >> min(key - tree_base, 31)) & 1u) != 0u;
    else
        live = live && key >= k_first;
    uint32_t* xw = reinterpret_cast<uint32_t*>(xch);
#pragma unroll
    for (int r = 0; r < R; ++r) {
        const float raw = G == 1 ? tsum8(part, dl) : tsum16(part + 16 * r, dl);
        const float s = live ? raw * scale_log2 : ninf;
        float bm = s;  // the batch's maximum for this slot's head: over the 8 lanes that hold its keys
        bm = fmaxf(bm, dpp_f32<0xB1>(bm));
        bm = fmaxf(bm, dpp_f32<0x4E>(bm));
        bm = fmaxf(bm, dpp_f32<0x141>(bm));
        const float mn = fmaxf(st.ms[r], bm);
        // nothing seen yet and nothing live in the batch: mn is still -inf, the weight 0 and the state as it was
        const float p = s == ninf ? 0.f : __builtin_amdgcn_exp2f(s - mn);
        const float corr = st.ms[r] == ninf ? 0.f : __builtin_amdgcn_exp2f(st.ms[r] - mn);
        const float pn = dpp_f32<0xB1>(p);  // the neighbouring key's weight
        const bool odd = (dl & 1) != 0;
        const bf16x2 pr = {(__bf16)(odd ? pn : p), (__bf16)(odd ? p : pn)};  // keys 2 i and 2 i + 1, rounded to bf16
        const uint32_t pw = __builtin_bit_cast(uint32_t, pr);
        st.ls[r] = fmaf(st.ls[r], corr, odd ? bf16hi_f32(pw) : bf16lo_f32(pw));
        st.ms[r] = mn;
        const int j = slot_head<G>(r, dl);
        xw[j * 4 + (bk >> 1)] = pw;       // both lanes of a pair write the same word
        if (bk == 0) xch[32 + j] = corr;
    }
    __builtin_amdgcn_wave_barrier();  // the writes above before the reads below, as written (one wave: served in order)
    uint4 pw4[G];
    float corr_all[G];
#pragma unroll
    for (int j = 0; j < G; ++j) {
        pw4[j] = reinterpret_cast<const uint4*>(xch)[j];
        corr_all[j] = xch[32 + j];
    }
    __builtin_amdgcn_wave_barrier();  // and these reads before the next batch's writes
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
        for (int e = 0; e < 8; ++e) st.acc[j][e] *= corr_all[j];
    if (ZERO_DEAD) {
        if (key0 + 16 * (KB - 1) >= k_end) {
#pragma unroll
            for (int b = 0; b < KB; ++b)
                if (key0 + 16 * b >= k_end) kb.v[b] = make_uint4(0u, 0u, 0u, 0u);
        }
    }
#pragma unroll
    for (int pi = 0; pi < KB / 2; ++pi) {
        const uint4 va = kb.v[2 * pi], vb = kb.v[2 * pi + 1];
        const uint32_t wa[4] = {va.x, va.y, va.z, va.w}, wb[4] = {vb.x, vb.y, vb.z, vb.w};
        uint32_t zl[4], zh[4];  // (dim 2 q of key a, of key b), (dim 2 q + 1 of key a, of key b)
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            zl[q] = __builtin_amdgcn_perm(wb[q], wa[q], 0x05040100u);
            zh[q] = __builtin_amdgcn_perm(wb[q], wa[q], 0x07060302u);
        }
#pragma unroll
        for (int j = 0; j < G; ++j) {
            const uint32_t pj = pi == 0 ? pw4[j].x : pi == 1 ? pw4[j].y : pi == 2 ? pw4[j].z : pw4[j].w;
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                st.acc[j][2 * q] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, zl[q]),
                                                                  __builtin_bit_cast(bf16x2, pj), st.acc[j][2 * q], false);
                st.acc[j][2 * q + 1] = __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, zh[q]),
                                                                      __builtin_bit_cast(bf16x2, pj), st.acc[j][2 * q + 1], false);
            }
        }
    }
}

// the stream's state per head, in every lane: the maximum, and the sum over the head's 8 key slots
template <int G>
__device__ __forceinline__ void heads_state(const AttnState<G>& st, int dl, float* xch, float (&m)[G], float (&l)[G]) {
    constexpr int R = attn_slots(G);
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int r = 0; r < R; ++r) {
        float ls = st.ls[r];
        ls += dpp_f32<0xB1>(ls);
        ls += dpp_f32<0x4E>(ls);
        ls += dpp_f32<0x141>(ls);
        if ((dl & 7) == 0) {
            const int j = slot_head<G>(r, dl);
            xch[j] = st.ms[r];
            xch[8 + j] = ls;
        }
    }
    __builtin_amdgcn_wave_barrier();
#pragma unroll
    for (int j = 0; j < G; ++j) {
        m[j] = xch[j];
        l[j] = xch[8 + j];
    }
    __builtin_amdgcn_wave_barrier();
}

// A workgroup's 16 key streams folded into one state per query head, in stream order. Each stream first brings its own
// state to the workgroup's maximum (the 16 maxima meet in LDS; one exp2 per head and lane), then the scaled sums and
// outputs are added up in stream order: thread (j, d) of 256 makes output d of head j, G * 128 / 256 of them a
// thread, and hands it to `store(j, d, M, L, A)` (M and L are the head's; use them where d == 0). s_m and s_l hold
// 16 * G floats, s_acc 16 * G * 128; xch is the stream's exchange area. 256 threads, all of them call.
template <int G, class Store>
__device__ __forceinline__ void fold_streams(const AttnState<G>& st, int grp, int dl, float* xch, float* s_m, float* s_l,
                                             float* s_acc, int tid, Store store) {
    const float ninf = bits_f32(0xff800000u);
    float m[G], l[G];
    heads_state<G>(st, dl, xch, m, l);
    if (dl == 0) {
#pragma unroll
        for (int j = 0; j < G; ++j) s_m[grp * G + j] = m[j];
    }
    __syncthreads();
#pragma unroll
    for (int j = 0; j < G; ++j) {
        float M = ninf;
#pragma unroll
        for (int s2 = 0; s2 < 16; ++s2) M = fmaxf(M, s_m[s2 * G + j]);
        const float f = m[j] == ninf ? 0.f : __builtin_amdgcn_exp2f(m[j] - M);
        if (dl == 0) s_l[grp * G + j] = l[j] * f;
        // the lane's eight values as two 16-byte stores (s_acc is 16-byte aligned): one value a store would put
        // lanes four apart on one bank
        float4* dst = reinterpret_cast<float4*>(s_acc + (grp * G + j) * AD + dl * 8);
        dst[0] = make_float4(st.acc[j][0] * f, st.acc[j][1] * f, st.acc[j][2] * f, st.acc[j][3] * f);
        dst[1] = make_float4(st.acc[j][4] * f, st.acc[j][5] * f, st.acc[j][6] * f, st.acc[j][7] * f);
    }
    __syncthreads();
    for (int o = tid; o < G * AD; o += 256) {
        const int j = o / AD, d = o - j * AD;
        float A = 0.f;
#pragma unroll
        for (int s2 = 0; s2 < 16; ++s2) A += s_acc[(s2 * G + j) * AD + d];
        float M = ninf, L = 0.f;
        if (d == 0) {
#pragma unroll
            for (int s2 = 0; s2 < 16; ++s2) {
                M = fmaxf(M, s_m[s2 * G + j]);
                L += s_l[s2 * G + j];
            }
        }
        store(j, d, M, L, A);
    }
}

// The S spans' states of one (row, kv head) folded in span order by a workgroup of 256 into G * 128 outputs
// bf16(O / L). Every state a thread needs in the first pass - the spans' maxima and sums, and 32 spans' partial
// outputs of its G / 2 outputs (one, for a single query head) - is requested before anything waits: one round trip.
// Then every span's factor exp2(m_s - M) and scaled sum are made once, in parallel, and each output adds up its spans
// in order. DEV: the states were written by other workgroups of the same launch (st_dev) and are read with ld_dev.
// lds: 2 * S * G floats. `out` is the row's attention output, [Hq * 128]; `base` the state index of the head's span 0.
template <int G, bool DEV>
__device__ __forceinline__ void merge_spans(uint16_t* out, int g, int S, size_t base, const float* part_m,
                                            const float* part_l, const float* part_acc, float* lds, int tid) {
    constexpr int NOUT = G >= 2 ? G / 2 : 1;  // outputs a thread makes: (j, d) = ((tid + 256 q) / 128, tid % 128)
    constexpr int MS = NOUT <= 2 ? 40 : 20;  // spans a pass (a 4096-key cache is 33 to 36 spans: one pass)
    const float ninf = bits_f32(0xff800000u);
    auto ld = [](const float* p) { return DEV ? ld_dev(p) : *p; };
    float* f_m = lds;          // [S][G] maxima, then the factors
    float* f_l = lds + S * G;  // [S][G] sums, then the scaled sums
    const int d = tid & (AD - 1);
    int jq[NOUT];
#pragma unroll
    for (int q = 0; q < NOUT; ++q) jq[q] = min((tid + 256 * q) / AD, G - 1);
    const bool mine = tid < G * AD;  // a single query head: half the workgroup has no output
    float v[NOUT][MS];
    const int s_first = min(S, MS);
#pragma unroll
    for (int s2 = 0; s2 < MS; ++s2)
#pragma unroll
        for (int q = 0; q < NOUT; ++q)
            v[q][s2] = ld(&part_acc[((base + min(s2, s_first - 1)) * G + jq[q]) * AD + d]);  // past the last: it again
    for (int o = tid; o < S * G; o += 256) {
        f_m[o] = ld(&part_m[base * G + o]);
        f_l[o] = ld(&part_l[base * G + o]);
    }
    __syncthreads();
    // each state's factor and scaled sum, by the thread that brought it in
    float fac[4], lsc[4];  // S * G <= 1024 states over 256 threads
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int o = tid + 256 * r;
        fac[r] = lsc[r] = 0.f;
        if (o < S * G) {
            const int j = o % G;
            float M = ninf;
            for (int s2 = 0; s2 < S; ++s2) M = fmaxf(M, f_m[s2 * G + j]);
            const float pm = f_m[o];
            fac[r] = pm == ninf ? 0.f : __builtin_amdgcn_exp2f(pm - M);
            lsc[r] = f_l[o] * fac[r];
        }
    }
    __syncthreads();
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const int o = tid + 256 * r;
        if (o < S * G) {
            f_m[o] = fac[r];
            f_l[o] = lsc[r];
        }
    }
    __syncthreads();
    float A[NOUT], L[NOUT];
#pragma unroll
    for (int q = 0; q < NOUT; ++q) {
        A[q] = 0.f;
        L[q] = 0.f;
        for (int s2 = 0; s2 < S; ++s2) L[q] += f_l[s2 * G + jq[q]];
    }
#pragma unroll
    for (int s2 = 0; s2 < MS; ++s2)
        if (s2 < s_first) {
#pragma unroll
            for (int q = 0; q < NOUT; ++q) A[q] = fmaf(v[q][s2], f_m[s2 * G + jq[q]], A[q]);
        }
    for (int s0 = MS; s0 < S; s0 += MS) {
        const int left = min(S - s0, MS);
#pragma unroll
        for (int s2 = 0; s2 < MS; ++s2)
#pragma unroll
            for (int q = 0; q < NOUT; ++q)
                v[q][s2] = ld(&part_acc[((base + s0 + min(s2, left - 1)) * G + jq[q]) * AD + d]);
#pragma unroll
        for (int s2 = 0; s2 < MS; ++s2)
            if (s2 < left) {
#pragma unroll
                for (int q = 0; q < NOUT; ++q) A[q] = fmaf(v[q][s2], f_m[(s0 + s2) * G + jq[q]], A[q]);
            }
    }
    if (mine) {
#pragma unroll
        for (int q = 0; q < NOUT; ++q) {
            const uint16_t o = f32_bf16(A[q] * (1.f / L[q]));
            uint16_t* dst = &out[((size_t)g * G + jq[q]) * AD + d];
            if (DEV)
                st_dev(dst, o);
            else
                *dst = o;
        }
    }
}

// The same fold for a few spans (S <= MS <= 64), with nothing shared between waves: a workgroup of 128 threads takes
// one query head. A thread asks for its output's partial values of every span at once, and lane s of its wave for span
// s's maximum and sum - one trip to memory, no LDS, no barrier. Lane s makes span s's factor; every lane reads it back
// by lane number. The operations and their order are merge_spans': the same bits.
template <int GS, int MS>
__device__ __forceinline__ void merge_spans_few(uint16_t* out, int g, int j, int S, size_t base, const float* part_m,
                                                const float* part_l, const float* part_acc, int d) {
    const float ninf = bits_f32(0xff800000u);
    const int lane = d & 63, last = S - 1;
    const size_t sl = (base + min(lane, last)) * GS + j;
    const float m = part_m[sl], l = part_l[sl];
    float v[MS];
#pragma unroll
    for (int s2 = 0; s2 < MS; ++s2)  // past the last span: it again, unused
        v[s2] = part_acc[((base + min(s2, last)) * GS + j) * AD + d];
    float M = lane < S ? m : ninf;  // the spans' maximum, in every lane that holds a span
    M = fmaxf(M, dpp_f32<0xB1>(M));
    M = fmaxf(M, dpp_f32<0x4E>(M));
    M = fmaxf(M, dpp_f32<0x141>(M));
    M = fmaxf(M, dpp_f32<0x140>(M));
    {   // across the rows of 16 lanes: their last lanes' values as scalars (no trip through the LDS unit)
        auto row = [&](int l) { return bits_f32((uint32_t)__builtin_amdgcn_readlane((int)f32_bits(M), l)); };
        const float lo = fmaxf(row(15), row(31));
        M = MS > 32 ? fmaxf(lo, fmaxf(row(47), row(63))) : lo;
    }
    // No branch on S below: with one, the compiler moves each load into its span's branch, a trip to memory a span.
    // A span past the last adds a zero to the sum and leaves the output's value as it is (its factor and its partial
    // value are made zero).
    const float fac = (lane >= S || m == ninf) ? 0.f : __builtin_amdgcn_exp2f(m - M);
    const float lsc = l * fac;
    float A = 0.f, L = 0.f;
#pragma unroll
    for (int s2 = 0; s2 < MS; ++s2) {
        L += bits_f32((uint32_t)__builtin_amdgcn_readlane((int)f32_bits(lsc), s2));
        A = fmaf(s2 < S ? v[s2] : 0.f, bits_f32((uint32_t)__builtin_amdgcn_readlane((int)f32_bits(fac), s2)), A);
    }
    out[((size_t)g * GS + j) * AD + d] = f32_bf16(A * (1.f / L));
}

// What row t of a pass sees. A chain of rows (par null): the cache's keys and the pass's rows up to itself. A tree
// (par[t] the row's parent among the pass's rows, -1 at a root; the reference's TREE form,
// native/cuda/btb_attn_flash.cuh:284-286, 407-419): the cache's keys, and of the pass's rows - slots n0 .. n0 + T - 1 -
// its ancestors and itself.
struct RowView {
    int n;               // one past the last slot the row may see
    int tree_base;       // -1 for a chain; else the first of the pass's own slots
    uint32_t tree_mask;  // the pass's rows the row sees (a tree)
    int k_first;         // the window's first key (0: no window)
};
__device__ __forceinline__ RowView row_view(const int32_t* __restrict__ par, int t, int T, int n0, int win) {
    RowView v;
    v.tree_base = -1;
    v.tree_mask = 0u;
    v.n = n0 + t + 1;
    int last = n0 + t;  // the row's own logical position: a chain's row t stands at n0 + t, a tree's at n0 + its depth
    if (par != nullptr) {
        v.tree_base = n0;
        v.n = n0 + T;
        int depth = -1;
        for (int p = t, hops = 0; p >= 0 && p < T && hops < 32; p = par[p], ++hops) ++depth;
        last = n0 + depth;
        // the row's keys among the pass's rows: itself and its ancestors, the one at depth d standing at n0 + d - under
        // a window (the reference's `first = last + 1 - win`, native/cuda/btb_attn_flash.cuh:437) those at or past it
        const int first_depth = win > 0 ? last + 1 - win - n0 : 0;
        int d = depth;
        for (int p = t, hops = 0; p >= 0 && p < T && hops < 32; p = par[p], ++hops, --d)
            if (d >= first_depth) v.tree_mask |= 1u << p;
    }
    v.k_first = win > 0 ? max(last + 1 - win, 0) : 0;
    return v;
}

}  // namespace btb
