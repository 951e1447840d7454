// Decode attention for a pass of several rows on the matrix cores.
//
// The rows of a verify pass that share a kv head - T rows x G query heads - all meet the same keys. Here a workgroup
// takes one kv head, one span of 128 keys and up to 64 of those (row, head) pairs at once: the span's K and V leave
// memory once a workgroup and are asked for in one go, the scores of all the pairs against all the keys are two
// handfuls of v_mfma_f32_16x16x32_bf16, and so is weights x values. On the vector ALUs (attn_decode_rows_kernel: a
// workgroup a row) the same pass spends 8 x the L2 reads and a 16-stream fold per row.
//
// Four waves. Scores, transposed: S^T [keys x pairs] = K [keys x 128] Q^T. Wave w owns keys 32 w .. 32 w + 31 (two
// 16-key tiles): operand A of a step is 16 keys x 32 dims - lane l: key l % 16, dims 8 (l / 16) .., sixteen bytes of a
// K row, read from memory as they lie; operand B is 32 dims x 16 pairs - lane l: pair l % 16, the same dims of its q
// row. A result tile holds, in lane l, pair l % 16 against keys 4 (l / 16) .. + 3. A pair's maximum over the span:
// over the lane's 8 scores, the 4 lanes of the pair, then the 4 waves through LDS. The weights 2^(s - m), rounded to
// bf16 (the reference's card kernel rounds its weights for its tensor cores the same way,
// native/cuda/btb_attn_flash.cuh:90-125; the sum l is made of the rounded weights), go to LDS as P^T [keys x pairs] in
// the order operand B of the next product wants them.
// Outputs, transposed: O^T [128 dims x pairs] = V^T [dims x keys] P^T. Wave w owns dims 32 w .. 32 w + 31 over all 128
// keys, so no sums cross waves: operand A is 16 dims x 32 keys - lane l: dim l % 16, keys 8 (l / 16) .. + 7, eight
// 2-byte reads down a column of the V tile in LDS (V goes memory -> registers -> LDS in whole rows); operand B is 32
// keys x 16 pairs, sixteen bytes of P^T. A result tile holds, in lane l, pair l % 16 and dims 4 (l / 16) .. + 3: one
// 16-byte store into the pair's partial state.
//
// What comes out is the (m, l, acc[128]) state per (row, head, span) that attn_decode_kernel leaves, for the same
// merge kernel; the arithmetic is the same up to the order of the f32 sums (the matrix cores' instead of the
// 16-stream fold's). Which keys a row sees - chain or tree, window - is row_view's, as there.

#include "btb_attn.hpp"
#include "btb_common.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

constexpr int AM_D = 128;     // head_dim
constexpr int AM_SPAN = 128;  // keys a workgroup
constexpr int AM_VROW = 272;  // bytes a V row takes in LDS: 256 + 16, so the eight rows a fragment read touches differ in bank
constexpr int AM_PROW = 80;   // bytes a pair's 32 weights of a step take: 64 + 16, sixteen pairs in sixteen bank groups

__device__ __forceinline__ float xor_lanes16(float v) {  // the value of lane l ^ 16
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(((int)(threadIdx.x & 63) ^ 16) << 2, __builtin_bit_cast(int, v)));
}
__device__ __forceinline__ float xor_lanes32(float v) {
    return __builtin_bit_cast(float, __builtin_amdgcn_ds_bpermute(((int)(threadIdx.x & 63) ^ 32) << 2, __builtin_bit_cast(int, v)));
}

// A tile of 16 heads (q heads of a pass's rows, or the rows' k heads) prepared - RMSNorm, rope - in the layout the
// matrix cores take an operand in: lane (c, a) holds head c's dims 32 ds + 8 a .. + 7 for ds = 0 .. 3. Under rope the
// partner of a dim, 64 dims away, is chunk ds ^ 2 of the same lane. The sum of squares folds in the order of
// head_finish's (a lane l there holds dims 2 l, 2 l + 1 and the lanes fold by group_sum<64>: l ^ 1, ^ 2, ^ 4 .. ^ 32;
// here l = 16 ds + 4 a + e / 2), so the bits that come out are head_finish's.
struct HeadTile {
    uint4 raw[4], wn[4], cs[4], sn[4];
    uint4 vrow[4];  // with a k tile: the rows' v, as they come
};
__device__ __forceinline__ void tile_request(HeadTile& h, const uint16_t* src, const uint16_t* wn, int a) {
    const uint16_t* wsrc = wn != nullptr ? wn : src;  // no weight: any words, unused
#pragma unroll
    for (int ds = 0; ds < 4; ++ds) {
        h.raw[ds] = *reinterpret_cast<const uint4*>(src + ds * 32 + a * 8);
        h.wn[ds] = *reinterpret_cast<const uint4*>(wsrc + ds * 32 + a * 8);
    }
}
__device__ __forceinline__ void cs_sn_request(HeadTile& h, const uint16_t* cos_t, const uint16_t* sin_t, int pos, int a) {
#pragma unroll
    for (int ds = 0; ds < 4; ++ds) {
        h.cs[ds] = *reinterpret_cast<const uint4*>(cos_t + (size_t)pos * AM_D + ds * 32 + a * 8);
        h.sn[ds] = *reinterpret_cast<const uint4*>(sin_t + (size_t)pos * AM_D + ds * 32 + a * 8);
    }
}
__device__ __forceinline__ float bf16_of(const uint4& q, int e) {  // element e of eight
    const uint32_t w = e < 2 ? q.x : e < 4 ? q.y : e < 6 ? q.z : q.w;
    return (e & 1) ? bf16hi_f32(w) : bf16lo_f32(w);
}
__device__ __forceinline__ void tile_norm(const HeadTile& h, bool has_wn, float eps, int centered, float (&v)[4][8]) {
#pragma unroll
    for (int ds = 0; ds < 4; ++ds)
#pragma unroll
        for (int e = 0; e < 8; ++e) v[ds][e] = bf16_of(h.raw[ds], e);
    if (has_wn) {
        float t[4];
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) {
            float sq[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2)
                sq[e2] = fmaf(v[ds][2 * e2 + 1], v[ds][2 * e2 + 1], fmaf(v[ds][2 * e2], v[ds][2 * e2], 0.f));
            t[ds] = (sq[0] + sq[1]) + (sq[2] + sq[3]);  // l ^ 1, then l ^ 2
        }
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) t[ds] += xor_lanes16(t[ds]);  // l ^ 4
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) t[ds] += xor_lanes32(t[ds]);  // l ^ 8
        const float ss = (t[0] + t[1]) + (t[2] + t[3]);              // l ^ 16, then l ^ 32
        const float rstd = rsqrtf(ss / (float)AM_D + eps);
#pragma unroll
        for (int ds = 0; ds < 4; ++ds)
#pragma unroll
            for (int e = 0; e < 8; ++e) {
                const float w = bf16_of(h.wn[ds], e);
                v[ds][e] = bfround(v[ds][e] * rstd * (centered ? 1.f + w : w));
            }
    }
}
__device__ __forceinline__ void tile_rope(const float (&v)[4][8], const HeadTile& h, uint4 (&out)[4]) {
#pragma unroll
    for (int ds = 0; ds < 4; ++ds) {
        const float sgn = ds < 2 ? -1.f : 1.f;
        uint32_t w[4];
#pragma unroll
        for (int e2 = 0; e2 < 4; ++e2) {
            float o[2];
#pragma unroll
            for (int i = 0; i < 2; ++i) {
                const int e = 2 * e2 + i;
                const float qc = bfround(v[ds][e] * bf16_of(h.cs[ds], e));
                o[i] = fmaf(sgn * v[ds ^ 2][e], bf16_of(h.sn[ds], e), qc);
            }
            w[e2] = f32x2_bf16(o[0], o[1]);
        }
        out[ds] = make_uint4(w[0], w[1], w[2], w[3]);
    }
}

// What the variant that starts from the pass's fused qkv rows [T, (Hq + 2 Hk) 128] needs on top: the q / k norm
// weights (or none), the rope tables, the rows' depths (a tree) or none (a chain: row t stands at *n0 + t), the cache
// to write the new rows into.
struct AmQkv {
    const uint16_t* qkv;
    const uint16_t* wq;
    const uint16_t* wk;
    const uint16_t* cos_t;
    const uint16_t* sin_t;
    const int32_t* depth;
    uint16_t* Kw;
    uint16_t* Vw;
    float eps;
    int centered;
};
constexpr int AM_QROW = 272;  // bytes a prepared q or k row takes in LDS: 256 + 16, as for V

__host__ __device__ constexpr size_t am_lds_bytes(int G, int NQT, bool QKV, int ZG = 1) {
    const size_t NQ = 16 * (size_t)NQT, TPW = NQ / (size_t)G;
    const size_t weights = 4 * NQ * AM_PROW, heads = QKV ? (NQ + (size_t)ZG * TPW) * AM_QROW : 0;
    return (size_t)AM_SPAN * AM_VROW + 2 * 4 * NQ * sizeof(float) + (weights > heads ? weights : heads);
}

// NQT tiles of 16 (row, head) pairs a workgroup: pair r of the workgroup is row t_base + r / G, head r % G
// TBL: the cache has a row map (a template argument, not a test of the pointer: a branch between two loads makes the
// compiler wait for the first before it issues the second, and the span's rows then arrive one trip at a time)
// QKV: the rows come as the fused qkv rows, before the q / k norm and rope (DEPTH: with the rows' depths). The whole
// pass is one workgroup's pairs then (T G <= 16 NQT <= 32; ZG below: two workgroups'). The q heads are prepared by the workgroup itself, a tile of
// 16 a wave, and passed through LDS - q never reaches memory - and so are the k heads of the pass's rows: the
// workgroups whose span holds some of the pass's own slots *n0 .. *n0 + T - 1 write those and the raw v rows into the
// cache, and take them from LDS in place of what they read from the cache, which is not written yet. The arithmetic is
// norm_rope_kv_kernel's, then this kernel's. ZG = 2: the pass's pairs are two workgroups' (gridDim.z = 2, up to 64 pairs
// a kv head): each prepares the q heads of its own rows and the k heads of all the rows, the first of the two writes
// the cache.
template <int G, int NQT, bool TBL, bool QKV, bool DEPTH, int ZG = 1>
__global__ void __launch_bounds__(256) attn_decode_mfma_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ K, const uint16_t* __restrict__ V,
    const int32_t* __restrict__ n0p, const int32_t* __restrict__ par, int T, int Hq, int Hk, long long hs, long long rs,
    float scale_log2, float* __restrict__ part_m, float* __restrict__ part_l, float* __restrict__ part_acc, int cap,
    int win, const int32_t* __restrict__ tbl, AmQkv x) {
    constexpr int D = AM_D, NQ = 16 * NQT, TPW = NQ / G;
    static_assert(NQ % G == 0, "whole rows a workgroup");
    static_assert(!(QKV && TBL), "the fused rows go with a cache without a row map");
    extern __shared__ __align__(16) uint8_t lds[];
    uint8_t* v_lds = lds;                                                 // [128 keys][AM_VROW]
    float* red_m = reinterpret_cast<float*>(lds + AM_SPAN * AM_VROW);     // [4 waves][NQ]
    float* red_l = red_m + 4 * NQ;                                        // [4 waves][NQ]
    // [4 steps of 32 keys][NQ pairs][AM_PROW]; before the scores are done the prepared heads lie here:
    // q [NQ][AM_QROW], then the pass's own k rows [ZG TPW][AM_QROW]
    uint8_t* p_lds = reinterpret_cast<uint8_t*>(red_l + 4 * NQ);
    const int g = blockIdx.x, sp = blockIdx.y, S = gridDim.y;
    const int t_base = blockIdx.z * TPW;
    const int tid = threadIdx.x, lane = tid & 63;
    // QKV: the wave's number as a scalar, so that which tile a wave prepares, and with which weights, is decided on the
    // scalar unit (a per-lane choice between two kernel arguments becomes a vector load of the argument)
    const int wv = QKV ? __builtin_amdgcn_readfirstlane(tid >> 6) : tid >> 6;
    const int c = lane & 15, a = lane >> 4;
    const int k_begin = sp * AM_SPAN;
    const float ninf = bits_f32(0xff800000u);

    // Everything the workgroup reads from memory is asked for before anything is waited for. Without a row map the
    // addresses do not depend on *n0: a slot at or past the cache's capacity reads the last slot again, and which keys
    // count is decided afterwards (what a dead slot held is replaced by zeros: it may never have been written).
    int n_lim = 1;  // with a row map: one past the last slot any of the workgroup's rows may see (the map ends there)
    if (TBL) {
        const int n0_early = *n0p;
        n_lim = max(par != nullptr ? n0_early + T : n0_early + min(T, t_base + TPW), 1);
    }
    auto slot_of = [&](int key) {
        const int s = min(key, cap - 1);
        return TBL ? tbl[min(s, n_lim - 1)] : s;
    };
    // QKV: the heads to prepare come as tiles of 16 - NQT tiles of q heads (tile qt: the workgroup's pairs 16 qt ..),
    // then the pass's rows' k heads 16 at a time; wave wv takes tile wv. What does not depend on *n0 (the
    // heads' values, the norm weights, the rows' v) is asked for first, ahead of the span's K and V, so the norms are
    // done while those travel; the rope tables' rows come last.
    constexpr int NKT = (ZG * TPW + 15) / 16, NTASK = QKV ? NQT + NKT : 0;
    static_assert(NTASK <= 4, "a tile a wave");
    auto task_row = [&](int id) {  // the lane's row of the pass in tile id (a q tile: of its pair); unclamped
        return id < NQT ? t_base + (id * 16 + c) / G : (id - NQT) * 16 + c;
    };
    HeadTile task0;
    auto request = [&](int id, HeadTile& h) {
        const size_t width = (size_t)(Hq + 2 * Hk) * D;
        const bool is_k = id >= NQT;
        const uint16_t* row = x.qkv + (size_t)min(task_row(id), T - 1) * width;
        const uint16_t* src = row + (size_t)(is_k ? Hq + g : g * G + (id * 16 + c) % G) * D;
        tile_request(h, src, is_k ? x.wk : x.wq, a);
        const uint16_t* vsrc = is_k ? row + (size_t)(Hq + Hk + g) * D : src;
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) h.vrow[ds] = *reinterpret_cast<const uint4*>(vsrc + ds * 32 + a * 8);
    };
    if constexpr (QKV) {
        if (wv < NTASK) request(wv, task0);
    }
    // QKV: V is asked for after the rope tables' rows, which wait for *n0 - V is not needed before the weights are
    // made, and the span's K keeps the memory busy meanwhile; so q and the new k rows are ready before K is there.
    uint4 vreg[8];
    auto request_v = [&]() {
#pragma unroll
        for (int i = 0; i < 8; ++i) {
            const int key = k_begin + (tid >> 4) + 16 * i;
            vreg[i] = *reinterpret_cast<const uint4*>(V + (size_t)g * hs + (size_t)slot_of(key) * rs + (tid & 15) * 8);
        }
    };
    if constexpr (!QKV) request_v();
    uint4 kreg[2][4];
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int key = k_begin + 32 * wv + 16 * h + c;
        const uint16_t* kr = K + (size_t)g * hs + (size_t)slot_of(key) * rs + a * 8;
#pragma unroll
        for (int ds = 0; ds < 4; ++ds) kreg[h][ds] = *reinterpret_cast<const uint4*>(kr + ds * 32);
    }
    uint4 qreg[NQT][4];
    if constexpr (!QKV) {
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
            const int r = qt * 16 + c, t = min(t_base + r / G, T - 1), j = r % G;
            const uint16_t* qr = q + ((size_t)t * Hq + (size_t)g * G + j) * D + a * 8;
#pragma unroll
            for (int ds = 0; ds < 4; ++ds) qreg[qt][ds] = *reinterpret_cast<const uint4*>(qr + ds * 32);
        }
    }
    const int n0 = *n0p;
    const int t_end = min(T, t_base + TPW);
    // the keys any of the workgroup's rows may see end at n_max (a chain's last row, or the whole pass for a tree)
    const int n_max = par != nullptr ? n0 + T : n0 + t_end;
    const int k_lim = min(n_max, k_begin + AM_SPAN);
    if constexpr (QKV) {
        auto tables = [&](int id, HeadTile& h) {
            const int t = min(task_row(id), T - 1);
            cs_sn_request(h, x.cos_t, x.sin_t, n0 + (DEPTH ? x.depth[t] : t), a);
        };
        if (wv < NTASK) tables(wv, task0);
        request_v();
        uint8_t* q_lds = p_lds;
        uint8_t* kn_lds = p_lds + NQ * AM_QROW;
        auto finish = [&](int id, const HeadTile& h) {
            const bool is_k = id >= NQT;
            float v[4][8];
            tile_norm(h, (is_k ? x.wk : x.wq) != nullptr, x.eps, x.centered, v);
            uint4 out[4];
            tile_rope(v, h, out);
            if (!is_k) {
#pragma unroll
                for (int ds = 0; ds < 4; ++ds)
                    *reinterpret_cast<uint4*>(q_lds + (id * 16 + c) * AM_QROW + ds * 64 + a * 16) = out[ds];
            } else {
                const int tr = task_row(id), slot = n0 + tr;
                // (a slot at or past the cache's capacity is not written: the caller has let the cache overflow)
                if (tr < T && slot >= k_begin && slot < min(k_begin + AM_SPAN, cap)) {
                    uint16_t* kc = x.Kw + (size_t)g * hs + (size_t)slot * rs + a * 8;
                    uint16_t* vc = x.Vw + (size_t)g * hs + (size_t)slot * rs + a * 8;
                    const bool seen = slot < k_lim;          // by one of this workgroup's rows (else: zeros, as below)
                    const bool writes = ZG == 1 || blockIdx.z == 0;  // the cache's rows are written once
#pragma unroll
                    for (int ds = 0; ds < 4; ++ds) {
                        *reinterpret_cast<uint4*>(kn_lds + tr * AM_QROW + ds * 64 + a * 16) = out[ds];
                        *reinterpret_cast<uint4*>(v_lds + (slot - k_begin) * AM_VROW + ds * 64 + a * 16) =
                            seen ? h.vrow[ds] : make_uint4(0u, 0u, 0u, 0u);
                        if (writes) {
                            *reinterpret_cast<uint4*>(kc + ds * 32) = out[ds];
                            *reinterpret_cast<uint4*>(vc + ds * 32) = h.vrow[ds];
                        }
                    }
                }
            }
        };
        if (wv < NTASK) finish(wv, task0);
        __syncthreads();
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt)
#pragma unroll
            for (int ds = 0; ds < 4; ++ds)
                qreg[qt][ds] = *reinterpret_cast<const uint4*>(q_lds + (qt * 16 + c) * AM_QROW + ds * 64 + a * 16);
        if (k_begin < n0 + T && n0 < k_begin + AM_SPAN) {  // some of the pass's own slots lie in this span
#pragma unroll
            for (int h = 0; h < 2; ++h) {
                const int own = k_begin + 32 * wv + 16 * h + c - n0;  // which of the pass's rows this key is, if any
                const bool is_new = own >= 0 && own < T;
                const uint8_t* kn = kn_lds + min(max(own, 0), T - 1) * AM_QROW + a * 16;
#pragma unroll
                for (int ds = 0; ds < 4; ++ds) {
                    const uint4 v = *reinterpret_cast<const uint4*>(kn + ds * 64);
                    if (is_new) kreg[h][ds] = v;
                }
            }
        }
    }

    // V into LDS, dead slots as zeros (weight 0 times whatever bits lie there must not make a NaN)
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int kl = (tid >> 4) + 16 * i;
        const uint4 v = k_begin + kl < k_lim ? vreg[i] : make_uint4(0u, 0u, 0u, 0u);
        // the pass's own rows are in place already (they were prepared above; the cache does not hold them yet)
        if (!QKV || k_begin + kl < n0 || k_begin + kl >= n0 + T)
            *reinterpret_cast<uint4*>(v_lds + kl * AM_VROW + (tid & 15) * 16) = v;
    }

    // scores: S^T tile [h][qt], lane: pair c of tile qt against keys 32 wv + 16 h + 4 a .. + 3
    f32x4 st[2][NQT];
#pragma unroll
    for (int h = 0; h < 2; ++h)
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
            f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int ds = 0; ds < 4; ++ds)
                acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, kreg[h][ds]),
                                                              __builtin_bit_cast(bf16x8, qreg[qt][ds]), acc, 0, 0, 0);
            st[h][qt] = acc;
        }

    // masked, scaled; the pair's maximum over the span
    float mrow[NQT];
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        const int r = qt * 16 + c, t = t_base + r / G;
        const bool row_ok = t < T;
        const RowView rv = row_view(par, min(t, T - 1), T, n0, win);
        // branch-free: this runs once a workgroup, and a path that short is bound by how fast its code arrives
        const int k_end = row_ok ? min(rv.n, k_lim) : 0;
        const int tb = rv.tree_base >= 0 ? rv.tree_base : 0x7FFFFFFF;  // the first of the pass's own slots, if a tree
        float m = ninf;
#pragma unroll
        for (int h = 0; h < 2; ++h)
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int key = k_begin + 32 * wv + 16 * h + 4 * a + i;
                const uint32_t named = (rv.tree_mask >> min(max(key - tb, 0), 31)) & 1u;
                const bool inside = key >= tb ? named != 0u : key >= rv.k_first;
                const bool live = (key < k_end) & inside;
                const float s = live ? st[h][qt][i] * scale_log2 : ninf;
                st[h][qt][i] = s;
                m = fmaxf(m, s);
            }
        m = fmaxf(m, xor_lanes16(m));
        m = fmaxf(m, xor_lanes32(m));
        if (a == 0) red_m[wv * NQ + r] = m;
        mrow[qt] = m;
    }
    __syncthreads();
    // weights, rounded to bf16; P^T into LDS; the wave's share of the sums
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        const int r = qt * 16 + c;
        const float m = fmaxf(fmaxf(red_m[r], red_m[NQ + r]), fmaxf(red_m[2 * NQ + r], red_m[3 * NQ + r]));
        mrow[qt] = m;
        float l = 0.f;
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            uint32_t pw[2];
#pragma unroll
            for (int i2 = 0; i2 < 2; ++i2) {
                const float s0 = st[h][qt][2 * i2], s1 = st[h][qt][2 * i2 + 1];
                const float p0 = s0 == ninf ? 0.f : __builtin_amdgcn_exp2f(s0 - m);
                const float p1 = s1 == ninf ? 0.f : __builtin_amdgcn_exp2f(s1 - m);
                const bf16x2 pr = {(__bf16)p0, (__bf16)p1};
                pw[i2] = __builtin_bit_cast(uint32_t, pr);
                l += bf16lo_f32(pw[i2]);
                l += bf16hi_f32(pw[i2]);
            }
            // step wv (the wave's 32 keys), pair r, slots 16 h + 4 a .. + 3
            *reinterpret_cast<uint2*>(p_lds + (wv * NQ + r) * AM_PROW + (16 * h + 4 * a) * 2) = make_uint2(pw[0], pw[1]);
        }
        l += xor_lanes16(l);
        l += xor_lanes32(l);
        if (a == 0) red_l[wv * NQ + r] = l;
    }
    __syncthreads();
    // the pairs' maximum and sum out (wave 0, one lane a pair)
    if (wv == 0 && a == 0) {
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) {
            const int r = qt * 16 + c, t = t_base + r / G, j = r % G;
            if (t < T) {
                const size_t prow = ((size_t)t * Hk + g) * S + sp;
                part_m[prow * G + j] = mrow[qt];
                part_l[prow * G + j] = ((red_l[r] + red_l[NQ + r]) + red_l[2 * NQ + r]) + red_l[3 * NQ + r];
            }
        }
    }
    // outputs: O^T tile [dt][qt], lane: pair c of tile qt, dims 32 wv + 16 dt + 4 a .. + 3
    f32x4 ot[2][NQT];
#pragma unroll
    for (int dt = 0; dt < 2; ++dt)
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt) ot[dt][qt] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
    for (int ks = 0; ks < 4; ++ks) {
        uint4 pfrag[NQT];
#pragma unroll
        for (int qt = 0; qt < NQT; ++qt)
            pfrag[qt] = *reinterpret_cast<const uint4*>(p_lds + (ks * NQ + qt * 16 + c) * AM_PROW + a * 16);
#pragma unroll
        for (int dt = 0; dt < 2; ++dt) {
            // V^T fragment: dim 32 wv + 16 dt + c, keys 32 ks + 8 a .. + 7
            const uint8_t* col = v_lds + (32 * ks + 8 * a) * AM_VROW + (32 * wv + 16 * dt + c) * 2;
            uint32_t vw[4];
#pragma unroll
            for (int e2 = 0; e2 < 4; ++e2) {
                const uint32_t lo = *reinterpret_cast<const uint16_t*>(col + (2 * e2) * AM_VROW);
                const uint32_t hi = *reinterpret_cast<const uint16_t*>(col + (2 * e2 + 1) * AM_VROW);
                vw[e2] = lo | (hi << 16);
            }
            const bf16x8 vfrag = __builtin_bit_cast(bf16x8, make_uint4(vw[0], vw[1], vw[2], vw[3]));
#pragma unroll
            for (int qt = 0; qt < NQT; ++qt)
                ot[dt][qt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(vfrag, __builtin_bit_cast(bf16x8, pfrag[qt]),
                                                                     ot[dt][qt], 0, 0, 0);
        }
    }
#pragma unroll
    for (int qt = 0; qt < NQT; ++qt) {
        const int r = qt * 16 + c, t = t_base + r / G, j = r % G;
        if (t < T) {
            const size_t prow = ((size_t)t * Hk + g) * S + sp;
            float* dst = part_acc + (prow * G + j) * D + 32 * wv + 4 * a;
#pragma unroll
            for (int dt = 0; dt < 2; ++dt)
                *reinterpret_cast<float4*>(dst + 16 * dt) =
                    make_float4(ot[dt][qt][0], ot[dt][qt][1], ot[dt][qt][2], ot[dt][qt][3]);
        }
    }
}

template <int G, int NQT>
static void launch_am(const uint16_t* q, const uint16_t* K, const uint16_t* V, const int32_t* n0, const int32_t* par, int T,
               int Hq, int Hk, long long hs, long long rs, float scale_log2, float* part_m, float* part_l,
               float* part_acc, int S, int cap, int win, const int32_t* tbl, hipStream_t st) {
    constexpr int NQ = 16 * NQT, TPW = NQ / G;
    const size_t lds = am_lds_bytes(G, NQT, false);
    const dim3 grid((unsigned)Hk, (unsigned)S, (unsigned)((T + TPW - 1) / TPW));
    const AmQkv none{};
    if (tbl != nullptr)
        hipLaunchKernelGGL((attn_decode_mfma_kernel<G, NQT, true, false, false>), grid, dim3(256), lds, st, q, K, V, n0,
                           par, T, Hq, Hk, hs, rs, scale_log2, part_m, part_l, part_acc, cap, win, tbl, none);
    else
        hipLaunchKernelGGL((attn_decode_mfma_kernel<G, NQT, false, false, false>), grid, dim3(256), lds, st, q, K, V, n0,
                           par, T, Hq, Hk, hs, rs, scale_log2, part_m, part_l, part_acc, cap, win, tbl, none);
}

// the variant that starts from the fused qkv rows: one workgroup per (kv head, span), the whole pass in it
template <int G, int NQT, int ZG>
static void launch_am_qkv(const AmQkv& x, const int32_t* n0, const int32_t* par, int T, int Hq, int Hk, long long hs,
                          long long rs, float scale_log2, float* part_m, float* part_l, float* part_acc, int S, int cap,
                          hipStream_t st) {
    const size_t lds = am_lds_bytes(G, NQT, true, ZG);
    static_assert(am_lds_bytes(G, NQT, true, ZG) <= 64 * 1024, "within what a workgroup gets without asking for more");
    const dim3 grid((unsigned)Hk, (unsigned)S, (unsigned)ZG);
    const uint16_t* none = nullptr;
    if (x.depth != nullptr)
        hipLaunchKernelGGL((attn_decode_mfma_kernel<G, NQT, false, true, true, ZG>), grid, dim3(256), lds, st, none, x.Kw,
                           x.Vw, n0, par, T, Hq, Hk, hs, rs, scale_log2, part_m, part_l, part_acc, cap, 0, nullptr, x);
    else
        hipLaunchKernelGGL((attn_decode_mfma_kernel<G, NQT, false, true, false, ZG>), grid, dim3(256), lds, st, none, x.Kw,
                           x.Vw, n0, par, T, Hq, Hk, hs, rs, scale_log2, part_m, part_l, part_acc, cap, 0, nullptr, x);
}

// whether the pass takes this kernel: spans of 128 keys, 2 or 4 query heads a kv head
bool attn_mfma_fits(size_t T, size_t G, int span) {
    return T >= 2 && span == AM_SPAN && (G == 2 || G == 4) && tuning("attn_mfma") != 0;
}
// ... and starting from the fused qkv rows: a tile to prepare for each wave at most, so 32 pairs a workgroup, and up to
// 64 as two workgroups per (kv head, span). (64 pairs in one workgroup, a wave preparing two tiles one after the other,
// loses: the second tile's code no longer overlaps the keys' flight - 27.2 us a layer at 16 rows x 4 heads against
// 23.4 for norm_rope_kv + the kernel above + the merge.)
bool attn_mfma_qkv_fits(size_t T, size_t G, int span) {
    const int knob = tuning("attn_rows_fused");  // 0: never; 1: one workgroup's 32 pairs only; else up to 64 in two
    return attn_mfma_fits(T, G, span) && T * G <= (knob == 1 ? 32 : 64) && knob != 0;
}

// the partial states of every (row, head, span), for attn_merge_kernel
int32_t attn_decode_mfma(const void* q, const void* K, const void* V, const int32_t* n0, const int32_t* par, size_t T,
                         size_t Hq, size_t Hk, long long hs, long long rs, float scale_log2, float* part_m,
                         float* part_l, float* part_acc, size_t S, size_t cap, int win, const int32_t* tbl,
                         hipStream_t st) {
    const size_t G = Hq / Hk;
    const size_t pairs = T * G;  // of one kv head
    const int nqt = pairs <= 16 ? 1 : pairs <= 32 ? 2 : 4;
    const int capi = (int)(cap < 0x7FFFFFFFu ? cap : 0x7FFFFFFFu);
#define AM(GG, NN)                                                                                                    \
    launch_am<GG, NN>(static_cast<const uint16_t*>(q), static_cast<const uint16_t*>(K), static_cast<const uint16_t*>(V), \
                      n0, par, (int)T, (int)Hq, (int)Hk, hs, rs, scale_log2, part_m, part_l, part_acc, (int)S, capi, win, \
                      tbl, st)
    if (G == 4) {
        if (nqt == 1) AM(4, 1); else if (nqt == 2) AM(4, 2); else AM(4, 4);
    } else {
        if (nqt == 1) AM(2, 1); else if (nqt == 2) AM(2, 2); else AM(2, 4);
    }
#undef AM
    return hip_status(hipGetLastError(), "attn_decode_mfma launch");
}

// the same states from the fused qkv rows; the new K / V rows land in the cache on the way
int32_t attn_decode_mfma_qkv(const void* qkv, const void* wq, const void* wk, float eps, int centered, const void* cos_t,
                             const void* sin_t, const int32_t* n0, const int32_t* depth, const int32_t* par, void* K,
                             void* V, size_t T, size_t Hq, size_t Hk, long long hs, long long rs, float scale_log2,
                             float* part_m, float* part_l, float* part_acc, size_t S, size_t cap, hipStream_t st) {
    const size_t G = Hq / Hk;
    const size_t pairs = T * G;
    const int nqt = pairs <= 16 ? 1 : 2;
    const int capi = (int)(cap < 0x7FFFFFFFu ? cap : 0x7FFFFFFFu);
    AmQkv x;
    x.qkv = static_cast<const uint16_t*>(qkv);
    x.wq = static_cast<const uint16_t*>(wq);
    x.wk = static_cast<const uint16_t*>(wk);
    x.cos_t = static_cast<const uint16_t*>(cos_t);
    x.sin_t = static_cast<const uint16_t*>(sin_t);
    x.depth = depth;
    x.Kw = static_cast<uint16_t*>(K);
    x.Vw = static_cast<uint16_t*>(V);
    x.eps = eps;
    x.centered = centered;
#define AMQ(GG, NN, ZZ)                                                                                               \
    launch_am_qkv<GG, NN, ZZ>(x, n0, par, (int)T, (int)Hq, (int)Hk, hs, rs, scale_log2, part_m, part_l, part_acc,     \
                              (int)S, capi, st)
    if (G == 4) {
        if (nqt == 1) AMQ(4, 1, 1); else if (pairs <= 32) AMQ(4, 2, 1); else AMQ(4, 2, 2);
    } else {
        if (nqt == 1) AMQ(2, 1, 1); else if (pairs <= 32) AMQ(2, 2, 1); else AMQ(2, 2, 2);
    }
#undef AMQ
    return hip_status(hipGetLastError(), "attn_decode_mfma_qkv launch");
}

}  // namespace btb
