// The whole decode step as ONE persistent kernel.
//
// Why: on MI355X every kernel launch costs 3-4 us of ramp and drain during which HBM idles, and a Qwen3-4B-shaped step
// is ~220 launches of 5-30 us each even after fusion. Here the grid (two workgroups a CU, all resident) walks the
// step's phases itself and meets at a grid-wide barrier between them; before a wave waits at the barrier in front of a
// matvec it has already requested the first items of its share of that matvec, so weights keep streaming while
// the barrier resolves. The arithmetic of every phase is the arithmetic of the stand-alone kernels (gemv.hip,
// glue.hip): same lane order, same reduction trees, same bf16 rounding points, so the step's logits are those of the
// launch-per-operator sequence bit for bit.
//
// Phases of a layer:  qkv matvec (residual add + RMSNorm in its x load)  |  q/k norm + rope + cache write + attention
// over key spans, each head's spans folded by the workgroup that finishes the head's last span  |  o matvec  |
// gate/up/SiLU matvec (add + norm in its x load)  |  down matvec.
// Then the head matvec with the final norm, the greedy pick and the publish.
//
// Visibility between workgroups (the eight dies' L2s are not coherent with each other): everything one phase hands to
// the next - activations, attention states, barrier words - is written with device-scope relaxed stores (write-through)
// and read with device-scope relaxed loads (cache-bypassing); weights and the cache's old rows are read-only during the
// step and take ordinary loads. No cache-flushing fence is issued anywhere: on this GPU such a fence costs ~0.8 us per
// workgroup and the workgroups of a die queue behind one another. The barrier is a two-level counter tree (16
// workgroups a leaf), ~2.5-3 us per crossing. Every wait is bounded: a barrier that does not complete within its spin
// limit raises the step's error word and every later barrier falls through, so the kernel always ends.
//
// Measured on MI355X the step comes out slower this way than as a replayed graph of the stand-alone kernels (about
// 4 ms against 2.3 ms): a barrier and the skew of its arrivals cost what a kernel boundary costs, and the phases lose
// the stand-alone kernels' per-shape tile choices. It is kept as an option, not as the default.

#include <cstring>

#include "btb_attn.hpp"
#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_stream.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// device-scope access, the barrier
// ------------------------------------------------------------------------------------------------------------

// The thread's index as a value the compiler cannot see through: address arithmetic built on it inside a phase stays in
// that phase instead of being hoisted out of the layer loop, where a dozen phases' worth of it would sit in registers
// (or in scratch) for the whole step.
__device__ __forceinline__ int phase_tid() {
    int t = threadIdx.x;
    asm volatile("" : "+v"(t));
    return t;
}

constexpr unsigned SYNC_LEAF = 16;          // workgroups per leaf counter
constexpr unsigned SYNC_SPIN = 1u << 18;    // polls before a barrier gives up
// the barrier's words (u32 indices into StepArgs.sync): leaf counters one per 128 bytes from SYNC_LEAVES
constexpr unsigned SYNC_TOP = 0, SYNC_GEN = 32, SYNC_ERR = 64, SYNC_LEAVES = 128;
constexpr unsigned SYNC_MAX_WGS = 4096, SYNC_MAX_HEADS = 64;
// the attention's arrival counters, one per kv head, behind the leaves
constexpr unsigned SYNC_HEADS = SYNC_LEAVES + 32 * (SYNC_MAX_WGS / SYNC_LEAF);

// The counters only ever count up: generation g is over when a leaf has seen lsize * (g + 1) arrivals and the top
// nleaves * (g + 1) leaves (in 32-bit wrap-around arithmetic), so no counter is reset while another workgroup may
// already be arriving for the next generation. The words carry over from launch to launch (same grid size).
__device__ __forceinline__ void grid_barrier(unsigned* sync, unsigned nblocks) {
    // the workgroup's own stores are complete (and the whole workgroup is here) before it is counted in
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (threadIdx.x == 0 && ld_dev(&sync[SYNC_ERR]) == 0u) {
        const unsigned g = ld_dev(&sync[SYNC_GEN]);  // cannot move on before this workgroup has arrived
        const unsigned leaf = blockIdx.x / SYNC_LEAF;
        const unsigned nleaves = (nblocks + SYNC_LEAF - 1) / SYNC_LEAF;
        const unsigned lsize = leaf == nleaves - 1 ? nblocks - leaf * SYNC_LEAF : SYNC_LEAF;
        unsigned* lc = &sync[SYNC_LEAVES + leaf * 32];
        bool released = false;
        if (__hip_atomic_fetch_add(lc, 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 == lsize * (g + 1)) {
            if (__hip_atomic_fetch_add(&sync[SYNC_TOP], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT) + 1 ==
                nleaves * (g + 1)) {
                __hip_atomic_fetch_add(&sync[SYNC_GEN], 1u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                released = true;
            }
        }
        if (!released) {
            unsigned spins = 0;
            while (ld_dev(&sync[SYNC_GEN]) == g) {
                __builtin_amdgcn_s_sleep(1);
                if (++spins > SYNC_SPIN) {
                    st_dev(&sync[SYNC_ERR], 1u);  // every later barrier falls through; the host reads this word
                    break;
                }
            }
        }
    }
    __syncthreads();
}

// ------------------------------------------------------------------------------------------------------------
// the step's arguments
// ------------------------------------------------------------------------------------------------------------

struct StepMat {  // one matrix in its stored form (bf16: w only)
    const void* w;
    const void* hi4;
    const void* table;
    const void* esc_idx;
    const void* esc_val;
    const void* row_ptr;
};

struct StepLayer {
    StepMat qkv, o, gu, down;
    const uint16_t* ln1;
    const uint16_t* ln2;
    const uint16_t* wq;
    const uint16_t* wk;
    uint16_t* K;
    uint16_t* V;
};

struct StepArgs {
    const StepLayer* layers;
    int nlayers, H, Hq, Hk, I, vocab, S, span;
    long long hs, rs;
    float eps, scale_log2;
    int centered;
    const uint16_t* embed;
    const uint16_t* norm_w;
    StepMat head;
    const uint16_t* cos_t;
    const uint16_t* sin_t;
    int32_t* ids;
    int32_t* picked;
    int32_t* n0;
    uint16_t* h_a;
    uint16_t* h_b;
    uint16_t* qkv;
    uint16_t* att;
    uint16_t* y;
    uint16_t* m;
    uint16_t* logits;
    float* part;      // attention states: m [Hq * S], l [Hq * S], acc [Hq * S * D]
    float* cand_v;    // the head phase's per-wave best logit ...
    int32_t* cand_i;  // ... and its row
    unsigned* sync;
    int32_t* host_tok;
    int32_t* host_n0;
    long long* host_ts;
    long long* trace;  // or null: workgroup 0's clock before and after every barrier
};

template <class F>
__device__ __forceinline__ typename F::Params mat_params(const StepMat& m);
template <>
__device__ __forceinline__ FmtBf16::Params mat_params<FmtBf16>(const StepMat& m) {
    return FmtBf16::Params{static_cast<const uint4*>(m.w)};
}
template <>
__device__ __forceinline__ FmtP12::Params mat_params<FmtP12>(const StepMat& m) {
    return FmtP12::Params{static_cast<const uint8_t*>(m.w),       static_cast<const uint8_t*>(m.hi4),
                          static_cast<const uint8_t*>(m.table),   static_cast<const int32_t*>(m.esc_idx),
                          static_cast<const uint8_t*>(m.esc_val), static_cast<const int32_t*>(m.row_ptr),
                          make_uint4(0, 0, 0, 0)};
}

// ------------------------------------------------------------------------------------------------------------
// x staging with device-scope loads (the rows were written by other workgroups in the phase before)
// ------------------------------------------------------------------------------------------------------------

// n8 eight-byte words from memory other workgroups have just written into LDS; four loads a thread in flight
__device__ __forceinline__ void copy_dev8(unsigned long long* dst, const unsigned long long* src, int n8) {
    const int tid = phase_tid();
    for (int base = 0; base < n8; base += 4 * 256) {
        unsigned long long v[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = base + q * 256 + tid;
            if (i < n8) v[q] = ld_dev(&src[i]);
        }
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            const int i = base + q * 256 + tid;
            if (i < n8) dst[i] = v[q];
        }
    }
}

__device__ __forceinline__ void stage_rows(uint32_t* xs, const uint16_t* x, int C) {
    copy_dev8(reinterpret_cast<unsigned long long*>(xs), reinterpret_cast<const unsigned long long*>(x), C / 4);
    __syncthreads();
}

// h' = bf16(h + y), x = bf16(h' * rsqrt(mean(h'^2) + eps) * w): stage_x<X_ADDNORM>'s arithmetic and order (thread i
// takes the 4-element words i, i + 256, ...). The two rows come into LDS first, in wide loads all in flight at once (one round
// trip to memory), behind the x row: LDS holds 3 * C values here. `fresh` is false where h is read-only data (the
// embedding row).
__device__ __forceinline__ void stage_addnorm(uint32_t* xs, const uint16_t* h, bool fresh, const uint16_t* y,
                                              const uint16_t* w, uint16_t* h_out, float eps, int centered, int C,
                                              float* red) {
    const int tid = phase_tid();
    uint16_t* row = reinterpret_cast<uint16_t*>(xs);
    uint16_t* hraw = row + C;
    uint16_t* yraw = row + 2 * C;
    if (fresh) {
        copy_dev8(reinterpret_cast<unsigned long long*>(hraw), reinterpret_cast<const unsigned long long*>(h), C / 4);
    } else {
        const uint2* src = reinterpret_cast<const uint2*>(h);
        uint2* dst = reinterpret_cast<uint2*>(hraw);
        for (int i = tid; i < C / 4; i += 256) dst[i] = src[i];
    }
    if (y != nullptr)
        copy_dev8(reinterpret_cast<unsigned long long*>(yraw), reinterpret_cast<const unsigned long long*>(y), C / 4);
    __syncthreads();
    float ss = 0.f;
    for (int wd = tid; wd < C / 4; wd += 256) {  // 4-element words, a word's elements in order
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int i = 4 * wd + e;
            float hv = bf16_f32(hraw[i]);
            if (y != nullptr) hv = bfround(hv + bf16_f32(yraw[i]));
            row[i] = f32_bf16(hv);
            ss = fmaf(hv, hv, ss);
        }
    }
    const float rstd = rsqrtf(block_sum256(ss, red) / (float)C + eps);
    for (int i = tid; i < C; i += 256) {
        const uint16_t hb = row[i];
        if (blockIdx.x == 0 && h_out != nullptr) st_dev(&h_out[i], hb);
        const float wv = bf16_f32(w[i]);
        row[i] = f32_bf16(bf16_f32(hb) * rstd * (centered ? 1.f + wv : wv));
    }
    __syncthreads();
}

// ------------------------------------------------------------------------------------------------------------
// a matvec phase: gemv_stream's tile loop (a tile: RPW sets of 64 / LPR rows, LPR lanes a row, U units of each row in
// flight per span; GLU: the gate row and the up row of an output together), with the first span of the wave's first
// tile requested before the barrier in front of the phase. A lane meets its row's units in ascending order, as in
// gemv_stream: the sums are its sums bit for bit. The loads of a span are issued together and then used in order, in
// straight-line code: the form whose waits the compiler counts exactly.
// ------------------------------------------------------------------------------------------------------------

template <class F, int LPR, int EPI, int RPW_, int U_>
struct Pre {
    static constexpr int RPW = EPI == E_GLU ? 2 : RPW_;
    static constexpr int U = U_;
    typename F::Raw raw[U][RPW];
};

// how a phase's tiles are dealt to the grid's waves: every active wave the same count (the last may get fewer)
struct Deal {
    int first, last;  // this wave's tiles: [first, last)
};
template <int LPR, int EPI, int RPW>
__device__ __forceinline__ Deal deal_tiles(int R, int wave, int nwaves) {
    constexpr int ROWS = EPI == E_GLU ? WAVE / LPR : (WAVE / LPR) * RPW;
    const int Rout = EPI == E_GLU ? R / 2 : R;
    const int ntiles = (Rout + ROWS - 1) / ROWS;
    const int per_wave = (ntiles + nwaves - 1) / nwaves;
    Deal d;
    d.first = min(wave * per_wave, ntiles);
    d.last = min(d.first + per_wave, ntiles);
    return d;
}

// the tile's weight rows (a row past the end reads the last row again - no divergence in the stream - and is not
// written) and the rows its sums are written to
template <class F, int LPR, int EPI, int RPW>
__device__ __forceinline__ void tile_rows(const typename F::Params& p, int tile, int R, int units, int lane,
                                          typename F::RowCtx (&ctx)[RPW], int (&rows)[RPW], int (&outs)[RPW]) {
    constexpr int G = WAVE / LPR;
    const int Rout = EPI == E_GLU ? R / 2 : R;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
        if (EPI == E_GLU) {
            outs[j] = tile * G + lane / LPR;
            rows[j] = min(outs[j], Rout - 1) + j * Rout;
        } else {
            outs[j] = tile * G * RPW + j * G + lane / LPR;
            rows[j] = min(outs[j], R - 1);
        }
        ctx[j] = F::row_ctx(p, (size_t)rows[j], units);
    }
}

#define PRE_ARGS class F, int LPR, int EPI, int RPW_, int U_
#define PRE_T Pre<F, LPR, EPI, RPW_, U_>

template <PRE_ARGS>
__device__ __forceinline__ void prefetch_span(PRE_T& pre, const StepMat& mat, int R, int C, int wave, int nwaves) {
    constexpr int RPW = PRE_T::RPW, U = PRE_T::U;
    const Deal d = deal_tiles<LPR, EPI, RPW>(R, wave, nwaves);
    if (d.first >= d.last) return;
    typename F::Params p = mat_params<F>(mat);
    F::prepare(p);
    const int units = C / F::UW;
    const int lane = phase_tid() & 63;
    typename F::RowCtx ctx[RPW];
    int rows[RPW], outs[RPW];
    tile_rows<F, LPR, EPI, RPW>(p, d.first, R, units, lane, ctx, rows, outs);
    load_span<F, LPR, RPW, U, true>(pre.raw, ctx, 0, lane % LPR, units);
}

// the finished sums of a tile: y (or the GLU fold m); HEAD: also track the wave's best logit for the pick
template <class F, int LPR, int EPI, int RPW, bool HEAD>
__device__ __forceinline__ void tile_out(float (&acc)[RPW][1], const int (&outs)[RPW], int sl, int R, uint16_t* y,
                                         float& best_v, int& best_i) {
    if (EPI == E_GLU) {
        const float g = bfround(group_sum<LPR>(acc[0][0]));
        const float up = bfround(group_sum<LPR>(acc[RPW - 1][0]));
        const float sg = bfround(g / (1.f + expf(-g)));
        if (sl == 0 && outs[0] < R / 2) st_dev(&y[outs[0]], f32_bf16(sg * up));
    } else {
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            const float sum = group_sum<LPR>(acc[j][0]);
            if (sl == 0 && outs[j] < R) {
                const uint16_t b = f32_bf16(sum);
                st_dev(&y[outs[j]], b);
                if (HEAD) {
                    const float v = bf16_f32(b);
                    if (v > best_v) {  // rows ascend within the lane: a tie keeps the earlier; a NaN never wins
                        best_v = v;
                        best_i = outs[j];
                    }
                }
            }
        }
    }
}

// one tile. PRIMED: its first span is the one requested before the barrier.
template <bool HEAD, bool PRIMED, PRE_ARGS>
__device__ __forceinline__ void tile_body(PRE_T& pre, const typename F::Params& p, int tile, const uint32_t* xs,
                                          uint16_t* y, int R, int C, int lane, float& best_v, int& best_i) {
    constexpr int RPW = PRE_T::RPW, U = PRE_T::U;
    const int units = C / F::UW, sl = lane % LPR, span = U * LPR;
    const uint4* xs4 = reinterpret_cast<const uint4*>(xs);
    typename F::RowCtx ctx[RPW];
    int rows[RPW], outs[RPW];
    tile_rows<F, LPR, EPI, RPW>(p, tile, R, units, lane, ctx, rows, outs);
    float acc[RPW][1];
#pragma unroll
    for (int j = 0; j < RPW; ++j) acc[j][0] = 0.f;
    int k0 = 0;
    if (PRIMED) {
        fma_span<F, 1, LPR, RPW, U, true>(pre.raw, ctx, 0, sl, units, xs4, C / 8, acc);
        k0 = span;
    }
    for (; k0 < units; k0 += span) {
        typename F::Raw raw[U][RPW];
        load_span<F, LPR, RPW, U, true>(raw, ctx, k0, sl, units);
        fma_span<F, 1, LPR, RPW, U, true>(raw, ctx, k0, sl, units, xs4, C / 8, acc);
    }
#pragma unroll
    for (int j = 0; j < RPW; ++j) F::template tail<1>(p, ctx[j], (size_t)rows[j], sl, LPR, C, xs, acc[j]);
    tile_out<F, LPR, EPI, RPW, HEAD>(acc, outs, sl, R, y, best_v, best_i);
}

template <bool HEAD, PRE_ARGS>
__device__ __forceinline__ void matvec_phase(PRE_T& pre, const StepMat& mat, const uint32_t* xs, uint16_t* y, int R,
                                             int C, int wave, int nwaves, float& best_v, int& best_i) {
    const Deal d = deal_tiles<LPR, EPI, PRE_T::RPW>(R, wave, nwaves);
    typename F::Params p = mat_params<F>(mat);
    F::prepare(p);
    const int lane = phase_tid() & 63;
    if (d.first >= d.last) return;
    tile_body<HEAD, true>(pre, p, d.first, xs, y, R, C, lane, best_v, best_i);
    for (int tile = d.first + 1; tile < d.last; ++tile)
        tile_body<HEAD, false>(pre, p, tile, xs, y, R, C, lane, best_v, best_i);
}

// ------------------------------------------------------------------------------------------------------------
// attention: q/k norm + rope + cache write + the spans' states (glue.hip's norm_rope_kv and attn_decode), then the
// fold (attn_merge). head_dim 128, G = Hq / Hk = 4.
// ------------------------------------------------------------------------------------------------------------

// the spans of kv head g folded in span order (the merge kernel's routine) by the workgroup that finished the head's
// last span
template <int G>
__device__ __forceinline__ void merge_head(const StepArgs& a, int g, float* lds) {
    const int S = a.S, Hq = a.Hq;
    merge_spans<G, true>(a.att, g, S, (size_t)g * S, a.part, a.part + (size_t)Hq * S, a.part + 2 * (size_t)Hq * S, lds,
                         phase_tid());
    __syncthreads();
}

// one (kv head, span) item: q/k norm + rope, the cache write, the span's keys, the state out; the workgroup that
// completes a head's last span folds the head
template <int G>
__device__ __forceinline__ void attention_item(const StepArgs& a, const StepLayer& L, int g, int sp, int n0,
                                               float* lds) {
    const int tid = phase_tid();
    static_assert(G == 4, "four waves: one query head each, the fourth also the new key and value rows");
    // LDS: q [G][128] f32 (scaled), the new key and value rows [128] bf16 each, then the 16 streams' states
    float* s_q = lds;
    uint16_t* s_k = reinterpret_cast<uint16_t*>(lds + G * AD);
    uint16_t* s_v = s_k + AD;
    float* s_m = lds + G * AD + AD;  // [16][G]
    float* s_l = s_m + 16 * G;       // [16][G]
    float* s_acc = s_l + 16 * G;     // [16][G][128]
    __shared__ __align__(16) float s_xs[16 * XCH];  // the streams' exchange areas
    float* s_x = s_xs;
    __shared__ int s_last;
    const int lane = tid & 63, wv = tid >> 6;
    const int Hq = a.Hq, Hk = a.Hk;
    const int sub = lane >> 4, dl = lane & 15, grp = wv * 4 + sub;
    const int k_begin = sp * a.span, k_end = min(n0 + 1, k_begin + a.span);
    const uint16_t* Kh = L.K + (size_t)g * a.hs + dl * 8;
    const uint16_t* Vh = L.V + (size_t)g * a.hs + dl * 8;
    // the stream's first keys are requested before anything else: they do not wait for q
    KeyBatch kb = {};  // defined on every path: nothing of it is carried from item to item
    const int key_first = k_begin + grp;
    if (key_first < k_end) load_keys(kb, Kh, Vh, a.rs, key_first, k_end, n0);

    const uint16_t* qkv = a.qkv;
    {
        uint16_t o[2];
        head_norm_rope<true>(qkv + (size_t)(g * G + wv) * AD, L.wq, a.eps, a.centered, a.cos_t, a.sin_t, n0, lane, o);
        reinterpret_cast<uint32_t*>(s_q)[wv * (AD / 2) + lane] = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
    }
    // the step's own key and value of this kv head: every span's workgroup makes them, the one whose span holds
    // slot n0 uses them (from LDS) and writes them into the cache
    if (wv == 3 && n0 >= k_begin && n0 < k_begin + a.span) {
        uint16_t o[2];
        head_norm_rope<true>(qkv + (size_t)(Hq + g) * AD, L.wk, a.eps, a.centered, a.cos_t, a.sin_t, n0, lane, o);
        const uint32_t vraw = ld_dev(reinterpret_cast<const uint32_t*>(qkv + (size_t)(Hq + Hk + g) * AD) + lane);
        s_k[lane * 2] = o[0];
        s_k[lane * 2 + 1] = o[1];
        s_v[lane * 2] = (uint16_t)(vraw & 0xFFFFu);
        s_v[lane * 2 + 1] = (uint16_t)(vraw >> 16);
        uint32_t* kd = reinterpret_cast<uint32_t*>(L.K + (size_t)g * a.hs + (size_t)n0 * a.rs) + lane;
        uint32_t* vd = reinterpret_cast<uint32_t*>(L.V + (size_t)g * a.hs + (size_t)n0 * a.rs) + lane;
        *kd = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
        *vd = vraw;
    }
    __syncthreads();

    uint32_t qp[G][4];
#pragma unroll
    for (int j = 0; j < G; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) qp[j][e] = reinterpret_cast<const uint32_t*>(s_q)[j * (AD / 2) + dl * 4 + e];
    AttnState<G> st;
    st.init();
    for (int key0 = key_first; key0 < k_end;) {
        use_keys<G>(kb, key0, k_end, (n0 >= k_begin && n0 < k_begin + a.span) ? n0 : -1, s_k, s_v, dl, qp, a.scale_log2, st, s_x + grp * XCH);
        key0 += 16 * KB;
        if (key0 < k_end) load_keys(kb, Kh, Vh, a.rs, key0, k_end, n0);
    }
    float* part_m = a.part;
    float* part_l = a.part + (size_t)Hq * a.S;
    float* part_acc = a.part + 2 * (size_t)Hq * a.S;
    const size_t prow = (size_t)g * a.S + sp;
    fold_streams<G>(st, grp, dl, s_x + grp * XCH, s_m, s_l, s_acc, tid, [&](int j, int d, float M, float Lsum, float A) {
        st_dev(&part_acc[(prow * G + j) * AD + d], A);
        if (d == 0) {
            st_dev(&part_m[prow * G + j], M);
            st_dev(&part_l[prow * G + j], Lsum);
        }
    });
    // the head's arrival count only ever counts up (S arrivals a layer): the workgroup that brings it to a multiple of
    // S came last, every other span's state was complete before its own arrival, and it folds the head
    __builtin_amdgcn_fence(__ATOMIC_RELEASE, "workgroup");
    __syncthreads();
    if (tid == 0) {
        const unsigned old = __hip_atomic_fetch_add(&a.sync[SYNC_HEADS + 32 * g], 1u, __ATOMIC_RELAXED,
                                                    __HIP_MEMORY_SCOPE_AGENT);
        s_last = (old + 1) % (unsigned)a.S == 0 ? 1 : 0;
    }
    __syncthreads();
    if (s_last) merge_head<G>(a, g, lds);
    __syncthreads();  // the LDS is reused by the workgroup's next item
}

// a barrier between two phases, with workgroup 0's clock before and after it when the caller asked for a timeline
__device__ __forceinline__ void phase_end(const StepArgs& a, unsigned nb, int& stamp) {
    if (a.trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0) a.trace[stamp] = (long long)wall_clock64();
    grid_barrier(a.sync, nb);
    if (a.trace != nullptr && blockIdx.x == 0 && threadIdx.x == 0) a.trace[stamp + 1] = (long long)wall_clock64();
    stamp += 2;
}

template <class F, int LQ, int LO, int LD>
__global__ void __launch_bounds__(256, 2) decode_step_kernel(StepArgs a) {
    extern __shared__ __align__(16) uint32_t lds[];
    __shared__ float red[4];
    constexpr int G = 4;
    // spans: two rows by eight units where rows are short (the whole of a wave's share of qkv in one request), one
    // row by eight where a row fills the span
    constexpr bool WIDE = sizeof(typename F::Raw) <= 16;  // a packed unit takes more registers: half the rows in flight
    using PQ = Pre<F, LQ, E_PLAIN, WIDE ? 2 : 1, 8>;
    using PO = Pre<F, LO, E_PLAIN, 1, 8>;
    using PG = Pre<F, LQ, E_GLU, 2, WIDE ? 8 : 4>;
    using PD = Pre<F, LD, E_PLAIN, 1, 8>;
    const int wave = blockIdx.x * 4 + __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = gridDim.x * 4;
    const unsigned nb = gridDim.x;
    const int n0 = *a.n0;      // written only by the step's last phase, after its last barrier
    const int token = min(max(a.ids[0], 0), a.vocab - 1);
    const int H = a.H, QR = (a.Hq + 2 * a.Hk) * AD, OC = a.Hq * AD, I = a.I;
    float best_v = bits_f32(0xff800000u);
    int best_i = 0x7fffffff;
    int stamp = 0;

    PQ pq = {};
    prefetch_span(pq, a.layers[0].qkv, QR, H, wave, nwaves);
    const uint16_t* y_prev = nullptr;
    for (int li = 0; li < a.nlayers; ++li) {
        const StepLayer& L = a.layers[li];
        // zeroed, not left indeterminate: a span's guarded loads define only part of it, and what they leave would
        // otherwise count as carried around the layer loop (and hold registers through every phase)
        PO po = {};
        PG pg = {};
        PD pd = {};
        // qkv = W (rmsnorm(h + y) * ln1); the first layer's h is the token's embedding row
        stage_addnorm(lds, li == 0 ? a.embed + (size_t)token * H : a.h_a, li != 0, y_prev, L.ln1, a.h_b, a.eps, a.centered, H, red);
        matvec_phase<false>(pq, L.qkv, lds, a.qkv, QR, H, wave, nwaves, best_v, best_i);
        phase_end(a, nb, stamp);
        // attention over (kv head, span) items; a head's last workgroup folds its spans into att
        for (int item = blockIdx.x; item < a.Hk * a.S; item += nb)
            attention_item<G>(a, L, item / a.S, item % a.S, n0, reinterpret_cast<float*>(lds));
        prefetch_span(po, L.o, H, OC, wave, nwaves);
        phase_end(a, nb, stamp);
        // y = Wo att
        stage_rows(lds, a.att, OC);
        matvec_phase<false>(po, L.o, lds, a.y, H, OC, wave, nwaves, best_v, best_i);
        prefetch_span(pg, L.gu, 2 * I, H, wave, nwaves);
        phase_end(a, nb, stamp);
        // m = silu(gate) * up over rmsnorm(h + y) * ln2
        stage_addnorm(lds, a.h_b, true, a.y, L.ln2, a.h_a, a.eps, a.centered, H, red);
        matvec_phase<false>(pg, L.gu, lds, a.m, 2 * I, H, wave, nwaves, best_v, best_i);
        prefetch_span(pd, L.down, H, I, wave, nwaves);
        phase_end(a, nb, stamp);
        // y = Wdown m
        stage_rows(lds, a.m, I);
        matvec_phase<false>(pd, L.down, lds, a.y, H, I, wave, nwaves, best_v, best_i);
        pq = {};
        if (li + 1 < a.nlayers)
            prefetch_span(pq, a.layers[li + 1].qkv, QR, H, wave, nwaves);
        else
            prefetch_span(pq, a.head, a.vocab, H, wave, nwaves);
        phase_end(a, nb, stamp);
        y_prev = a.y;
    }
    // logits = Whead (rmsnorm(h + y) * norm); each wave keeps its best row
    stage_addnorm(lds, a.h_a, true, y_prev, a.norm_w, nullptr, a.eps, a.centered, H, red);
    matvec_phase<true>(pq, a.head, lds, a.logits, a.vocab, H, wave, nwaves, best_v, best_i);
    // lane 0 of each row group holds a candidate; fold the wave's (rows ascend with the group index)
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float ov = __shfl_xor(best_v, s, WAVE);
        const int oi = __shfl_xor(best_i, s, WAVE);
        if (ov > best_v || (ov == best_v && oi < best_i)) {
            best_v = ov;
            best_i = oi;
        }
    }
    if ((threadIdx.x & 63) == 0) {
        st_dev(&a.cand_v[wave], best_v);
        st_dev(&a.cand_i[wave], best_i);
    }
    phase_end(a, nb, stamp);
    if (blockIdx.x != 0) return;
    // the pick: the largest logit, the lowest row on ties; then the step's bookkeeping and the host's copy
    float bv = bits_f32(0xff800000u);
    int bi = 0x7fffffff;
    for (int w = threadIdx.x; w < nwaves; w += 256) {
        const float v = ld_dev(&a.cand_v[w]);
        const int i = ld_dev(&a.cand_i[w]);
        if (v > bv || (v == bv && i < bi)) {
            bv = v;
            bi = i;
        }
    }
    __shared__ float s_bv[256];
    __shared__ int s_bi[256];
    s_bv[threadIdx.x] = bv;
    s_bi[threadIdx.x] = bi;
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int k = 1; k < 256; ++k)
            if (s_bv[k] > bv || (s_bv[k] == bv && s_bi[k] < bi)) {
                bv = s_bv[k];
                bi = s_bi[k];
            }
        if (bi == 0x7fffffff) bi = 0;  // nothing above -inf: index 0, as the reference's scan
        a.picked[0] = bi;
        a.ids[0] = bi;
        a.n0[0] = n0 + 1;
        if (a.host_tok != nullptr) {
            *a.host_tok = bi;
            if (a.host_ts != nullptr) *a.host_ts = (long long)wall_clock64();
            __threadfence_system();
            if (a.host_n0 != nullptr) *a.host_n0 = n0 + 1;
        }
    }
}

static int lanes_for_units(int units) {
    if (units % 64 == 0 || units >= 256) return 64;
    if (units % 32 == 0 || units >= 96) return 32;
    return 16;
}

}  // namespace btb

using namespace btb;

extern "C" {

static_assert(sizeof(StepMat) == sizeof(btb_hip_step_mat) && sizeof(StepLayer) == sizeof(btb_hip_step_layer) &&
                  sizeof(StepArgs) == sizeof(btb_hip_step_args),
              "the kernel's typed view of the step's arguments is the header's struct");

size_t btb_hip_step_sync_bytes(void) { return sizeof(unsigned) * (SYNC_HEADS + 32 * SYNC_MAX_HEADS); }

int32_t btb_hip_decode_step(const btb_hip_step_args* args, int32_t packed, int32_t workgroups, void* stream) {
    if (args == nullptr) return ERR_NULL;
    StepArgs a;
    std::memcpy(&a, args, sizeof(a));
    if (a.layers == nullptr || a.embed == nullptr || a.norm_w == nullptr || a.head.w == nullptr || a.cos_t == nullptr ||
        a.sin_t == nullptr || a.ids == nullptr || a.picked == nullptr || a.n0 == nullptr || a.h_a == nullptr ||
        a.h_b == nullptr || a.qkv == nullptr || a.att == nullptr || a.y == nullptr || a.m == nullptr ||
        a.logits == nullptr || a.part == nullptr || a.cand_v == nullptr || a.cand_i == nullptr || a.sync == nullptr)
        return ERR_NULL;
    if (a.nlayers <= 0 || a.H <= 0 || a.Hq <= 0 || a.Hk <= 0 || a.I <= 0 || a.vocab <= 0 || a.S <= 0 || a.span <= 0 ||
        a.hs <= 0 || a.rs <= 0 || !(a.eps >= 0.f) || workgroups <= 0 || workgroups > (int32_t)SYNC_MAX_WGS || a.Hk > (int32_t)SYNC_MAX_HEADS)
        return ERR_DOMAIN;
    if (a.Hq != 4 * a.Hk || a.S > 128) {
        set_error("decode_step: 4 query heads per kv head, head_dim 128, at most 128 key spans");
        return ERR_DOMAIN;
    }
    const int uw = packed ? FmtP12::UW : FmtBf16::UW;
    if (a.H % uw != 0 || a.H % 4 != 0 || a.I % uw != 0 || a.I % 4 != 0 || (a.Hq * AD) % uw != 0) return ERR_DOMAIN;
    if (packed && (a.head.hi4 == nullptr || a.head.table == nullptr || a.head.row_ptr == nullptr)) return ERR_NULL;
    const int lq = lanes_for_units(a.H / uw), lo = lanes_for_units(a.Hq * AD / uw), ld = lanes_for_units(a.I / uw);
    // LDS: the widest x row, or the attention item's q + new rows + 16 streams' states, or the fold's factors
    size_t lds = (size_t)2 * (a.I > a.Hq * AD ? a.I : a.Hq * AD);
    if ((size_t)6 * a.H > lds) lds = (size_t)6 * a.H;  // the staged x row and the two raw rows of the add + norm
    const size_t att = sizeof(float) * (4 * AD + AD + 2 * 16 * 4 + 16 * 4 * AD);
    const size_t mrg = sizeof(float) * (2 * (size_t)a.S * 4 + 4);
    if (att > lds) lds = att;
    if (mrg > lds) lds = mrg;
    hipStream_t st = static_cast<hipStream_t>(stream);
    void (*kern)(StepArgs) = nullptr;
    if (!packed) {
        if (lq == 64 && lo == 64 && ld == 64) kern = decode_step_kernel<FmtBf16, 64, 64, 64>;
    } else {
        if (lq == 64 && lo == 64 && ld == 64) kern = decode_step_kernel<FmtP12, 64, 64, 64>;
        else if (lq == 32 && lo == 64 && ld == 64) kern = decode_step_kernel<FmtP12, 32, 64, 64>;
    }
    if (kern == nullptr) {
        set_error("decode_step: no instance for this shape's lanes-per-row combination");
        return ERR_DOMAIN;
    }
    int per_cu = 0;
    hipError_t e = hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, reinterpret_cast<const void*>(kern), 256, lds);
    if (e != hipSuccess) return hip_status(e, "hipOccupancyMaxActiveBlocksPerMultiprocessor");
    if ((long long)per_cu * device_info().cus < workgroups) {
        set_error("decode_step: the grid would not be resident at once (the barrier needs every workgroup running)");
        return ERR_DOMAIN;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)workgroups), dim3(256), lds, st, a);
    return hip_status(hipGetLastError(), "decode_step launch");
}

}  // extern "C"
