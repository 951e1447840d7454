// The routed top-k MoE decode layer on the GPU, all experts resident in VRAM:
//
//   route      per token: f32 softmax over the E logits, the top k in the total order (p descending, index ascending),
//              weights p / sum(top k) summed in rank order, rounded to bf16 - the reference's btb_moe_route
//              (native/cuda/btb_kernels.cu:845-948) and Qwen4Router.forward (btb/engine/families/qwen4/router.py:43-51)
//   gate_up    for every (token, pick): g, u = bf16(W_gu[expert] . x[token]) (f32 accumulate), a wave holding gate row
//              r and up row I + r together and writing h[r] = bf16(bf16(silu(g)) * u); the experts' matrices are
//              streamed once per pick with the dense matvec's loop (btb_stream.hpp)
//   down       for every token and output row: the k experts in ASCENDING expert id, each d = bf16(W_dn[e] . h_e), then
//              y = bf16(y + bf16(d * w_e)) - the dtype chain and the summation order of _Experts._one_row / _loop
//              (btb/engine/host.py:508-569, 906-967)
//
// Nothing goes back to the host between the steps, so the layer records into a hipGraph.

#include <type_traits>

#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_route.hpp"
#include "btb_stream.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

int32_t lane16_bf16_rows16(const uint16_t* w, size_t rows, size_t cols, const uint16_t* x, size_t b, float* y,
                           hipStream_t st);  // lane16.hip

constexpr int ROUTE_MAX_K = 32;  // the reference's ROUTE_MAX_K (native/cuda/btb_kernels.cu:859)

// ------------------------------------------------------------------------------------------------------------
// route: one wave per token
// ------------------------------------------------------------------------------------------------------------

// the (value, index) maximum over the wave in the total order: value descending, then index ascending; an index of
// NONE is "nothing"
constexpr int NONE = 0x7fffffff;
__device__ __forceinline__ void wave_argmax(float& v, int& i) {
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float ov = __shfl_xor(v, s, WAVE);
        const int oi = __shfl_xor(i, s, WAVE);
        if (oi != NONE && (i == NONE || ov > v || (ov == v && oi < i))) {
            v = ov;
            i = oi;
        }
    }
}

template <bool F32>
__global__ void __launch_bounds__(64) moe_route_kernel(const void* __restrict__ logits, size_t ls, int E, int k,
                                                       int32_t* __restrict__ idx, uint16_t* __restrict__ w,
                                                       float* __restrict__ w32) {
    extern __shared__ float pr[];  // [E] the row's probabilities; a picked one is set below every live one
    const int t = blockIdx.x, lane = threadIdx.x;
    const size_t base = (size_t)t * ls;
    float m = bits_f32(0xff800000u);
    for (int e = lane; e < E; e += WAVE) m = fmaxf(m, logit_at<F32>(logits, base + e));
    m = wave_max(m);
    float s = 0.f;
    for (int e = lane; e < E; e += WAVE) {
        const float p = expf(logit_at<F32>(logits, base + e) - m);
        pr[e] = p;
        s += p;
    }
    s = wave_sum(s);
    for (int e = lane; e < E; e += WAVE) pr[e] = pr[e] / s;
    __syncthreads();
    // k rounds of the maximum; probabilities are >= 0, so -1 is below every live one and a pick is marked -2. A row of
    // NaN probabilities compares below nothing: it still takes live experts, the first it meets, as the reference's
    // kernel does (native/cuda/btb_kernels.cu:891-900)
    float topv = 0.f;  // lane j keeps pick j
    int topi = 0;
    for (int j = 0; j < k; ++j) {
        float bv = -1.f;
        int bi = NONE;
        for (int e = lane; e < E; e += WAVE) {
            const float v = pr[e];
            if (v > bv || (bi == NONE && v != -2.f)) {  // e ascends within the lane, so a tie keeps the lower index
                bv = v;
                bi = e;
            }
        }
        wave_argmax(bv, bi);
        if (lane == j) {
            topv = bv;
            topi = bi;
        }
        if (lane == 0 && bi != NONE) pr[bi] = -2.f;
        __syncthreads();
    }
    // the weights: sum of the top k in rank order, each p / sum
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

template <bool F32, int P>
__global__ void __launch_bounds__(64) moe_route_reg_kernel(const void* __restrict__ logits, size_t ls, int E, int k,
                                                           int32_t* __restrict__ idx, uint16_t* __restrict__ w,
                                                           float* __restrict__ w32, uint16_t* __restrict__ logits16) {
    route_row_reg<F32, P>(logits, (size_t)blockIdx.x * ls, (int)blockIdx.x, (int)threadIdx.x, E, k, idx, w, w32,
                                 logits16);
}

// a row's logits rounded to bf16, for the wide rows the kernel above does not take
__global__ void __launch_bounds__(256) round_rows_kernel(const float* __restrict__ src, size_t ls, int E,
                                                         uint16_t* __restrict__ dst) {
    const int t = blockIdx.y, e = blockIdx.x * 256 + threadIdx.x;
    if (e < E) dst[(size_t)t * E + e] = f32_bf16(src[(size_t)t * ls + e]);
}

template <bool F32>
static int32_t launch_route(const void* logits, size_t ls, int E, int k, int T, int32_t* idx, uint16_t* w, float* w32,
                            uint16_t* logits16, hipStream_t st) {
    const int P = (E + WAVE - 1) / WAVE;
#define BTB_ROUTE_REG(P_)                                                                                            \
    hipLaunchKernelGGL((moe_route_reg_kernel<F32, P_>), dim3((unsigned)T), dim3(64), 0, st, logits, ls, E, k, idx, w, \
                       w32, logits16)
    if (P == 1)
        BTB_ROUTE_REG(1);
    else if (P == 2)
        BTB_ROUTE_REG(2);
    else if (P <= 4)
        BTB_ROUTE_REG(4);
    else {
        hipLaunchKernelGGL(moe_route_kernel<F32>, dim3((unsigned)T), dim3(64), E * 4, st, logits, ls, E, k, idx, w, w32);
        if (logits16 != nullptr && F32)
            hipLaunchKernelGGL(round_rows_kernel, dim3((E + 255) / 256, T), dim3(256), 0, st,
                               static_cast<const float*>(logits), ls, E, logits16);
    }
#undef BTB_ROUTE_REG
    return hip_status(hipGetLastError(), "moe_route launch");
}

// ------------------------------------------------------------------------------------------------------------
// group_picks: a call's (pick, row) pairs sorted by expert, stable (btb/engine/host.py:283-296)
// ------------------------------------------------------------------------------------------------------------

// The pairs in the order of picks.T.reshape(-1) - pick position j outermost, row t within it - are f = j T + t, with
// expert idx[t k + j]. A thread owns an expert: it counts its pairs, the counts are summed over the experts before it
// (within the workgroup by a scan; over the workgroups before this one by counting the pairs whose expert lies below
// the workgroup's first), and a second walk in the same order writes the expert's pairs from its offset on - so an
// expert's pairs keep the order of f, which is what a stable sort leaves. Every id must lie in [0, E).
__global__ void __launch_bounds__(256) moe_group_picks_kernel(const int32_t* __restrict__ idx, int T, int k, int E,
                                                              int32_t* __restrict__ slot, int32_t* __restrict__ token,
                                                              int32_t* __restrict__ offs, int32_t* __restrict__ counts) {
    __shared__ int s_wave[4];
    __shared__ int s_cnt[256];
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), wv = tid / WAVE;
    const int base = blockIdx.x * 256, e = base + tid;
    const int n = T * k;
    int below = 0;
    for (int p = tid; p < n; p += 256) below += idx[p] < base;  // any order: a count
    below = (int)group_sum<64>((float)below);                     // exact: n <= 65535
    below = __shfl(below, 0, WAVE);
    if (lane == 0) s_wave[wv] = below;
    int cnt = 0;
    if (e < E)
        for (int p = 0; p < n; ++p) cnt += idx[p] == e;
    s_cnt[tid] = cnt;
    __syncthreads();
    int off = s_wave[0] + s_wave[1] + s_wave[2] + s_wave[3];
    for (int i = 0; i < tid; ++i) off += s_cnt[i];
    if (e >= E) return;
    counts[e] = cnt;
    offs[e] = off;
    if (cnt == 0) return;
    for (int j = 0; j < k; ++j)
        for (int t = 0; t < T; ++t)
            if (idx[(size_t)t * k + j] == e) {
                slot[off] = j;
                token[off] = t;
                ++off;
            }
}

// ------------------------------------------------------------------------------------------------------------
// the experts' stacks in their stored form, and the layer's middle
// ------------------------------------------------------------------------------------------------------------

// bf16: a = the weights [E, R, C]. MXFP4 (the checkpoint's layout, btb/mxfp4.py:4-29): a = blocks u8 [E, R, C / 32, 16],
// b = scales u8 [E, R, C / 32]. An expert's matrix is a slice of the stack; nothing is widened ahead of the matvec.
struct Stack {
    const void* a;
    const void* b;
};
template <class F>
__device__ __forceinline__ typename F::Params expert_of(const Stack& s, int expert, int R, int units);
template <>
__device__ __forceinline__ FmtBf16::Params expert_of<FmtBf16>(const Stack& s, int expert, int R, int units) {
    return FmtBf16::Params{static_cast<const uint4*>(s.a) + (size_t)expert * R * units};
}
template <>
__device__ __forceinline__ FmtMx4::Params expert_of<FmtMx4>(const Stack& s, int expert, int R, int units) {
    return FmtMx4::Params{static_cast<const uint8_t*>(s.a) + (size_t)expert * R * units * 16,
                          static_cast<const uint8_t*>(s.b) + (size_t)expert * R * units};
}

// What becomes of an expert's gate and up sums (each already the rows' dtype: bf16(sum)).
// OSS = false: the families that concatenate the halves - gate row r, up row I + r - and h = bf16(bf16(silu(g)) * u)
// (`_silu_gate`, btb/engine/host.py:439-441). OSS = true: gpt-oss - the halves interleaved (gate row 2 r, up row
// 2 r + 1), the expert's bias added to both, the gate clamped above and the up half on both sides, and
// h = (up + 1) * (gate * sigmoid(alpha * gate)) with every operation rounded to the rows' dtype as torch rounds it
// (`gpt_oss_gate`, host.py:443-451; `_act` adds the bias first, :414-419).
struct Glu {
    const uint16_t* bias;  // [E, 2I] bf16, or null
    float alpha, limit;
};
template <bool OSS>
__device__ __forceinline__ int glu_row(int r, int j, int I) {
    return OSS ? 2 * r + j : r + j * I;
}
template <bool OSS>
__device__ __forceinline__ uint16_t glu_out(float g, float u, const Glu& a, int expert, int r, int I) {
    if (!OSS) return f32_bf16(bfround(g / (1.f + expf(-g))) * u);
    if (a.bias != nullptr) {
        const uint16_t* b = a.bias + (size_t)expert * 2 * I + 2 * r;
        g = bfround(g + bf16_f32(b[0]));
        u = bfround(u + bf16_f32(b[1]));
    }
    g = g > a.limit ? a.limit : g;  // a NaN stays a NaN, as in torch's clamp
    u = u > a.limit ? a.limit : (u < -a.limit ? -a.limit : u);
    const float t = bfround(g * a.alpha);
    const float sg = bfround(1.f / (1.f + expf(-t)));
    const float glu = bfround(g * sg);
    const float up1 = bfround(u + 1.f);
    return f32_bf16(up1 * glu);
}

// ------------------------------------------------------------------------------------------------------------
// gate_up: the dense loop over (token, pick) pairs; blockIdx.y is the pair
// ------------------------------------------------------------------------------------------------------------

// A wave takes gate row r and up row I + r together (RPW = 2) and writes h[r] = bf16(bf16(silu(bf16(g))) * bf16(u)): the
// pair's gu row is never stored, the down kernel finds its x ready.
template <class F, bool OSS, int LPR, int RPW, int U>
__global__ void __launch_bounds__(256) moe_gate_up_kernel(Stack stack, const uint16_t* __restrict__ x,
                                                          const int32_t* __restrict__ idx, uint16_t* __restrict__ h,
                                                          int R, int C, int k, int E, Glu glu) {
    static_assert(RPW == 2, "gate and up");
    extern __shared__ __align__(16) uint32_t xs[];
    constexpr int G = WAVE / LPR, ROWS = G;
    const int pair = blockIdx.y;
    const int token = pair / k;
    int expert = idx[pair];
    expert = expert < 0 ? 0 : (expert >= E ? E - 1 : expert);  // a bad id reads a real expert and is the caller's
    const int units = C / F::UW;
    const int lane = threadIdx.x & (WAVE - 1), sl = lane % LPR;
    const int wave = blockIdx.x * (blockDim.x / WAVE) + (threadIdx.x / WAVE);
    const int nwaves = gridDim.x * (blockDim.x / WAVE);
    const int I = R / 2;
    const int ntiles = (I + ROWS - 1) / ROWS;
    const int span = U * LPR;
    const typename F::Params p = expert_of<F>(stack, expert, R, units);
    uint16_t* y = h + (size_t)pair * I;

    // the wave's first span of weights is requested right behind x's own loads, before anything waits for x: the
    // weights do not depend on x, and nothing about these loads is conditional (a wave past the last tile requests the
    // last tile's and drops them)
    typename F::Raw first[U][RPW] = {};
    stage_x<X_PLAIN, 0, false, 256>(xs, XArgs{x + (size_t)token * C, nullptr, nullptr, nullptr, 0.f, 0}, 1, C, [&] {
        typename F::RowCtx c0[RPW];
#pragma unroll
        for (int j = 0; j < RPW; ++j)
            c0[j] = F::row_ctx(p, (size_t)glu_row<OSS>(min(min(wave, ntiles - 1) * ROWS + lane / LPR, I - 1), j, I), units);
        load_span_always<F, LPR, RPW, U>(first, c0, 0, sl, units);
    });
    const uint4* xs4 = reinterpret_cast<const uint4*>(xs);
    for (int tile = wave; tile < ntiles; tile += nwaves) {
        typename F::RowCtx ctx[RPW];
        int rows[RPW];
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            rows[j] = tile * ROWS + lane / LPR;
            ctx[j] = F::row_ctx(p, (size_t)glu_row<OSS>(min(rows[j], I - 1), j, I), units);
        }
        float acc[RPW][1];
#pragma unroll
        for (int j = 0; j < RPW; ++j) acc[j][0] = 0.f;
        int k0 = 0;
        if (tile == wave) {
            fma_span<F, 1, LPR, RPW, U, true>(first, ctx, 0, sl, units, xs4, C / 8, acc);
            k0 = span;
        }
        for (; k0 < units; k0 += span) {
            typename F::Raw raw[U][RPW];
            if (k0 + span <= units) {
                load_span<F, LPR, RPW, U, false>(raw, ctx, k0, sl, units);
                fma_span<F, 1, LPR, RPW, U, false>(raw, ctx, k0, sl, units, xs4, C / 8, acc);
            } else {
                load_span<F, LPR, RPW, U, true>(raw, ctx, k0, sl, units);
                fma_span<F, 1, LPR, RPW, U, true>(raw, ctx, k0, sl, units, xs4, C / 8, acc);
            }
        }
        const float g = bfround(group_sum_last<LPR>(acc[0][0]));  // in the group's last lane: the one that stores
        const float u = bfround(group_sum_last<LPR>(acc[1][0]));
        if (sl == LPR - 1 && rows[0] < I) y[rows[0]] = glu_out<OSS>(g, u, glu, expert, rows[0], I);
    }
}

// The same with the rows that picked an expert taken together: blockIdx.y is still a pair, but only an expert's FIRST
// pair (in pair order) has work - it gathers every pair of its expert and streams the expert's rows once, MC of the
// gathered rows of x a pass, where the kernel above streams them once a pair. The workgroups of the later pairs leave
// before asking memory for anything. A product is a row of x against a row of weights in the lane order above, so
// each h row has the bits the kernel above gives it. n = T k <= GROUP_MAX_PAIRS.
constexpr int GROUP_MAX_PAIRS = 256;
template <class F, bool OSS, int LPR, int RPW, int U, int MC>
__global__ void __launch_bounds__(256) moe_gate_up_grouped_kernel(Stack stack, const uint16_t* __restrict__ x,
                                                                  const int32_t* __restrict__ idx, uint16_t* __restrict__ h,
                                                                  int R, int C, int k, int E, int n, Glu glu) {
    static_assert(RPW == 2, "gate and up");
    extern __shared__ __align__(16) uint32_t xs[];  // [MC][C / 2]
    constexpr int G = WAVE / LPR, ROWS = G;
    constexpr int NM = GROUP_MAX_PAIRS / WAVE;  // ballots that cover the pairs
    const int pair = blockIdx.y;
    auto clamp = [E](int v) { return v < 0 ? 0 : (v >= E ? E - 1 : v); };
    const int tid = threadIdx.x, lane = tid & (WAVE - 1), sl = lane % LPR, wv = tid / WAVE;
    // Which pairs picked this pair's expert: every wave finds out for itself - a lane a pair, 64 pairs a ballot, the
    // picks asked for together with the pair's own - so there is nothing to exchange and no barrier, and the scan
    // costs the one trip to the picks that the kernel above makes for its expert anyway.
    const int own = idx[pair];
    int picks[NM];
#pragma unroll
    for (int i = 0; i < NM; ++i) picks[i] = idx[min(i * WAVE + lane, n - 1)];
    const int expert = clamp(own);
    unsigned long long mask[NM];
#pragma unroll
    for (int i = 0; i < NM; ++i)
        mask[i] = i * WAVE < n ? __ballot(i * WAVE + lane < n && clamp(picks[i]) == expert) : 0ull;
    // an earlier pair of the same expert does the work
    {
        unsigned long long earlier = 0ull;
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            unsigned long long m = mask[i];
            if (i == pair / WAVE) m &= (1ull << (pair % WAVE)) - 1ull;
            if (i > pair / WAVE) m = 0ull;
            earlier |= m;
        }
        if (earlier != 0ull) return;  // uniform
    }
    int rows_n = 0;
#pragma unroll
    for (int i = 0; i < NM; ++i) rows_n += __builtin_popcountll(mask[i]);
    // the r-th of the expert's pairs, ascending (uniform arithmetic on the ballots)
    auto pair_of = [&](int r) {
        int found = 0;
#pragma unroll
        for (int i = 0; i < NM; ++i) {
            unsigned long long m = mask[i];
            const int c = __builtin_popcountll(m);
            if (r >= 0 && r < c) {
                for (int q = 0; q < r; ++q) m &= m - 1ull;
                found = i * WAVE + __builtin_ctzll(m);
            }
            r -= c;
        }
        return found;
    };

    const int units = C / F::UW;
    const int wave = blockIdx.x * (blockDim.x / WAVE) + wv;
    const int nwaves = gridDim.x * (blockDim.x / WAVE);
    const int I = R / 2;
    const int ntiles = (I + ROWS - 1) / ROWS;
    const int span = U * LPR;
    const typename F::Params p = expert_of<F>(stack, expert, R, units);
    const int per = C / 8;  // 16-byte pieces a row of x
    uint4* xd = reinterpret_cast<uint4*>(xs);
    const uint4* xs4 = reinterpret_cast<const uint4*>(xs);
    // one pass: M of the gathered rows against every row of the expert. The wave's first span of weights is asked
    // for before the rows of x are staged (it needs the expert only), as in the kernel above.
    auto pass = [&](auto mtag, int r0, int mc) {
        constexpr int M = decltype(mtag)::value;
        typename F::Raw first[U][RPW] = {};
        {
            typename F::RowCtx c0[RPW];
#pragma unroll
            for (int j = 0; j < RPW; ++j)
                c0[j] = F::row_ctx(p, (size_t)glu_row<OSS>(min(min(wave, ntiles - 1) * ROWS + lane / LPR, I - 1), j, I),
                                   units);
            load_span_always<F, LPR, RPW, U>(first, c0, 0, sl, units);
        }
        if (r0 != 0) __syncthreads();  // the previous pass has read its rows
        // the pass's rows of x, a row past the last being the last again (its sums are dropped)
        int prs[M];
#pragma unroll
        for (int m = 0; m < M; ++m) prs[m] = pair_of(r0 + min(m, mc - 1));
        for (int i = tid; i < M * per; i += 256) {
            const int m = i / per, c = i - m * per;
            int tok = prs[0] / k;
#pragma unroll
            for (int m2 = 1; m2 < M; ++m2) tok = m == m2 ? prs[m2] / k : tok;
            xd[i] = reinterpret_cast<const uint4*>(x + (size_t)tok * C)[c];
        }
        __syncthreads();
        for (int tile = wave; tile < ntiles; tile += nwaves) {
            typename F::RowCtx ctx[RPW];
            int rows[RPW];
#pragma unroll
            for (int j = 0; j < RPW; ++j) {
                rows[j] = tile * ROWS + lane / LPR;
                ctx[j] = F::row_ctx(p, (size_t)glu_row<OSS>(min(rows[j], I - 1), j, I), units);
            }
            float acc[RPW][M];
#pragma unroll
            for (int j = 0; j < RPW; ++j)
#pragma unroll
                for (int m = 0; m < M; ++m) acc[j][m] = 0.f;
            int k0 = 0;
            if (tile == wave) {
                fma_span<F, M, LPR, RPW, U, true>(first, ctx, 0, sl, units, xs4, C / 8, acc);
                k0 = span;
            }
            for (; k0 < units; k0 += span) {
                typename F::Raw raw[U][RPW];
                if (k0 + span <= units) {
                    load_span<F, LPR, RPW, U, false>(raw, ctx, k0, sl, units);
                    fma_span<F, M, LPR, RPW, U, false>(raw, ctx, k0, sl, units, xs4, C / 8, acc);
                } else {
                    load_span<F, LPR, RPW, U, true>(raw, ctx, k0, sl, units);
                    fma_span<F, M, LPR, RPW, U, true>(raw, ctx, k0, sl, units, xs4, C / 8, acc);
                }
            }
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float g = bfround(group_sum_last<LPR>(acc[0][m]));
                const float u = bfround(group_sum_last<LPR>(acc[1][m]));
                if (sl == LPR - 1 && rows[0] < I && m < mc)
                    h[(size_t)prs[m] * I + rows[0]] = glu_out<OSS>(g, u, glu, expert, rows[0], I);
            }
        }
    };
    for (int r0 = 0; r0 < rows_n; r0 += MC) {
        const int mc = min(MC, rows_n - r0);
        if (mc == 1)
            pass(std::integral_constant<int, 1>{}, r0, mc);
        else if (mc == 2)
            pass(std::integral_constant<int, 2>{}, r0, mc);
        else
            pass(std::integral_constant<int, MC>{}, r0, mc);
    }
}

// ------------------------------------------------------------------------------------------------------------
// down + weighted sum: blockIdx.y is the token; the k experts of a row are walked in ascending expert id
// ------------------------------------------------------------------------------------------------------------

// `bias` ([E, R] bf16 or null; gpt-oss): added to the expert's product after its rounding to the rows' dtype and before
// the pick's weight, as `_down` adds it (btb/engine/host.py:427-432).
template <class F, int LPR, int RPW, int U, int KB>
__global__ void __launch_bounds__(256) moe_down_kernel(Stack stack, const uint16_t* __restrict__ h,
                                                       const int32_t* __restrict__ idx, const uint16_t* __restrict__ wts,
                                                       uint16_t* __restrict__ y, int R, int C, int k, int E,
                                                       const uint16_t* __restrict__ bias) {
    extern __shared__ __align__(16) uint32_t hs[];  // [k][C / 2] the k experts' h rows, in ascending expert order
    __shared__ int s_expert[ROUTE_MAX_K];
    __shared__ float s_weight[ROUTE_MAX_K];
    constexpr int G = WAVE / LPR, ROWS = G * RPW;
    const int token = blockIdx.y;
    const int units = C / F::UW;
    const int lane = threadIdx.x & (WAVE - 1), sl = lane % LPR;
    const int wave = blockIdx.x * (blockDim.x / WAVE) + (threadIdx.x / WAVE);
    const int nwaves = gridDim.x * (blockDim.x / WAVE);
    const int ntiles = (R + ROWS - 1) / ROWS;
    const int span = U * LPR;

    // the token's picks by ascending expert id: pick j goes to place #{i : id_i < id_j} (ids of a row are distinct; a
    // repeated id keeps its rank order)
    if ((int)threadIdx.x < k) {
        const int j = threadIdx.x;
        const int mine = idx[(size_t)token * k + j];
        int place = 0;
        for (int i = 0; i < k; ++i) {
            const int other = idx[(size_t)token * k + i];
            place += (other < mine) || (other == mine && i < j);
        }
        s_expert[place] = mine < 0 ? 0 : (mine >= E ? E - 1 : mine);
        s_weight[place] = bf16_f32(wts[(size_t)token * k + j]);
        // the h row of this pick, staged at its place below
        s_expert[place] |= j << 20;
    }
    __syncthreads();
    // Requests in the order their answers are needed (loads come back in order), none of them conditional (a wait
    // is counted exactly only over loads that are certain to have been issued): the first pieces of the k picks' h
    // rows - out of L2, staged first - then the first KB experts' rows of the wave's first tile, which need the picks
    // only and whose trip to memory (long: a layer's experts lie megabytes apart) runs while the h rows are staged.
    const int per = C / 8;  // 16-byte pieces a row
    const uint4* hsrc = reinterpret_cast<const uint4*>(h);
    uint4* hdst = reinterpret_cast<uint4*>(hs);
    const int n = k * per;
    auto piece = [&](int i) {  // the i-th piece of the rows in ascending expert order
        const int q = i / per, c = i - q * per;
        return hsrc[((size_t)token * k + (s_expert[q] >> 20)) * per + c];
    };
    constexpr int PER = 4;
    uint4 hv[PER];
#pragma unroll
    for (int t = 0; t < PER; ++t) hv[t] = piece(min((int)threadIdx.x + t * 256, n - 1));

    typename F::RowCtx ctx[KB][RPW];
    typename F::Raw first[KB][U][RPW] = {};
    auto request = [&](int tile, int q0, auto always) {
#pragma unroll
        for (int b = 0; b < KB; ++b) {
            const int expert = s_expert[min(q0 + b, k - 1)] & 0xFFFFF;
            const typename F::Params p = expert_of<F>(stack, expert, R, units);
#pragma unroll
            for (int j = 0; j < RPW; ++j)
                ctx[b][j] = F::row_ctx(p, (size_t)min(tile * ROWS + j * G + lane / LPR, R - 1), units);
            if constexpr (decltype(always)::value)
                load_span_always<F, LPR, RPW, U>(first[b], ctx[b], 0, sl, units);  // past the k-th: the k-th again
            else if (q0 + b < k)
                load_span<F, LPR, RPW, U, true>(first[b], ctx[b], 0, sl, units);
        }
    };
    request(min(wave, ntiles - 1), 0, std::true_type{});

    // a piece past the end is the last piece again and is written to the last piece's place again
#pragma unroll
    for (int t = 0; t < PER; ++t) hdst[min((int)threadIdx.x + t * 256, n - 1)] = hv[t];
    for (int i = threadIdx.x + PER * 256; i < n; i += 256) hdst[i] = piece(i);
    __syncthreads();
    const uint4* hs4 = reinterpret_cast<const uint4*>(hs);

    for (int tile = wave; tile < ntiles; tile += nwaves) {
        int rows[RPW];
#pragma unroll
        for (int j = 0; j < RPW; ++j) rows[j] = tile * ROWS + j * G + lane / LPR;
        float out[RPW];
#pragma unroll
        for (int j = 0; j < RPW; ++j) out[j] = 0.f;
        for (int q0 = 0; q0 < k; q0 += KB) {
            if (tile != wave || q0 != 0) request(tile, q0, std::false_type{});
#pragma unroll
            for (int b = 0; b < KB; ++b) {
                const int q = q0 + b;
                if (q < k) {
                    float acc[RPW][1];
#pragma unroll
                    for (int j = 0; j < RPW; ++j) acc[j][0] = 0.f;
                    const uint4* xq = hs4 + (size_t)q * (C / 8);
                    fma_span<F, 1, LPR, RPW, U, true>(first[b], ctx[b], 0, sl, units, xq, C / 8, acc);
                    for (int k0 = span; k0 < units; k0 += span) {
                        typename F::Raw raw[U][RPW];
                        load_span<F, LPR, RPW, U, true>(raw, ctx[b], k0, sl, units);
                        fma_span<F, 1, LPR, RPW, U, true>(raw, ctx[b], k0, sl, units, xq, C / 8, acc);
                    }
                    const float wq = s_weight[q];
#pragma unroll
                    for (int j = 0; j < RPW; ++j) {
                        // the expert's down product, as the row's dtype (in the group's last lane, which stores)
                        float d = bfround(group_sum_last<LPR>(acc[j][0]));
                        if (bias != nullptr)
                            d = bfround(d + bf16_f32(bias[(size_t)(s_expert[q] & 0xFFFFF) * R + min(rows[j], R - 1)]));
                        out[j] = bfround(out[j] + bfround(d * wq));    // times its weight, added in bf16
                    }
                }
            }
        }
#pragma unroll
        for (int j = 0; j < RPW; ++j)
            if (sl == LPR - 1 && rows[j] < R) y[(size_t)token * R + rows[j]] = f32_bf16(out[j]);
    }
}

static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// lanes a row: enough that a lane's share of a row is a few units (one 16-byte load each)
static int lanes_for(int units) {
    if (units % 64 == 0 || units >= 256) return 64;
    if (units % 32 == 0 || units >= 96) return 32;
    return 16;
}
// an MXFP4 unit is 32 weights, so rows hold few of them (64 in a 2048-wide row): fewer lanes a row, more rows a wave
static int lanes_for_mx4(int units) {
    if (units >= 256) return 64;
    if (units >= 128) return 32;
    return 16;
}

template <class F, bool OSS, int LPR>
static int32_t launch_gate_up(Stack stack, const void* x, const int32_t* idx, void* gu, int R, int C, int k, int E,
                              int pairs, Glu glu, hipStream_t st) {
    constexpr int RPW = 2, U = 4, G = WAVE / LPR;
    const int ntiles = (R / 2 + G - 1) / G;
    const int grid = (ntiles + 3) / 4;
    // From eight rows on, the rows that share an expert go through it together. Fewer rows share few experts (4 rows of
    // top-8 over 128 experts: 30 distinct of 32 picks) and the wider pass costs more than the sharing saves: measured on
    // the Qwen3-30B-A3B shape, a layer takes 64 against 62 us at 4 rows, 88 against 86 at 6, 106 against 109 at 8, 180
    // against 198 at 16, 295 against 374 at 32. The knob moe_grouped forces either (1 / 0). Asking for the expert's
    // first rows before the pairs are sorted out - as the pair kernel does - was tried and loses (8 rows: 122 us): a
    // wave's first span is its whole share of the expert, so the later pairs of a shared expert ask for everything
    // they then drop.
    constexpr int MC = 4;
    const int grouped = tuning("moe_grouped");
    const bool wanted = grouped >= 0 ? grouped != 0 && pairs > k : pairs >= 8 * k;
    if (wanted && pairs <= GROUP_MAX_PAIRS && (size_t)MC * C * 2 <= (size_t)device_info().lds_bytes - 16 * 1024) {
        auto kern = moe_gate_up_grouped_kernel<F, OSS, LPR, RPW, U, MC>;
        const size_t lds = (size_t)MC * C * 2;
        if (lds > 48 * 1024) {
            hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
            if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
        }
        hipLaunchKernelGGL(kern, dim3(grid, pairs), dim3(256), lds, st, stack, static_cast<const uint16_t*>(x), idx,
                           static_cast<uint16_t*>(gu), R, C, k, E, pairs, glu);
        return hip_status(hipGetLastError(), "moe gate_up launch");
    }
    hipLaunchKernelGGL((moe_gate_up_kernel<F, OSS, LPR, RPW, U>), dim3(grid, pairs), dim3(256), (size_t)C * 2, st, stack,
                       static_cast<const uint16_t*>(x), idx, static_cast<uint16_t*>(gu), R, C, k, E, glu);
    return hip_status(hipGetLastError(), "moe gate_up launch");
}

template <class F, int LPR>
static int32_t launch_down(Stack stack, const void* gu, const int32_t* idx, const void* w, void* y, int R, int C, int k,
                           int E, int T, const void* bias, hipStream_t st) {
    constexpr int RPW = 1, G = WAVE / LPR;
    const int ntiles = (R + G * RPW - 1) / (G * RPW);
    const int grid = (ntiles + 3) / 4;
    const size_t lds = (size_t)k * C * 2;
    // a row of at most three units a lane (the 768-wide experts of the C4 shape: 96 bf16 units over 64 lanes, 24 MXFP4
    // units over 16): all eight picks' rows in one request
    const int upl = (C / F::UW + LPR - 1) / LPR;
    auto kern = upl <= 2   ? moe_down_kernel<F, LPR, RPW, 2, 8>
                : upl <= 3 ? moe_down_kernel<F, LPR, RPW, 3, 8>
                           : moe_down_kernel<F, LPR, RPW, 4, 4>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(kern, dim3(grid, T), dim3(256), lds, st, stack, static_cast<const uint16_t*>(gu), idx,
                       static_cast<const uint16_t*>(w), static_cast<uint16_t*>(y), R, C, k, E,
                       static_cast<const uint16_t*>(bias));
    return hip_status(hipGetLastError(), "moe down launch");
}

// the two launches of the experts over either stored form
template <class F, bool OSS>
static int32_t launch_experts(Stack gate_up, Stack down, const void* x, const int32_t* idx, const void* w, void* gu,
                              void* y, size_t T, size_t k, size_t E, size_t H, size_t I, Glu glu, const void* dn_bias,
                              hipStream_t st) {
    const int R1 = (int)(2 * I), C1 = (int)H, R2 = (int)H, C2 = (int)I;
    constexpr bool MX = std::is_same<F, FmtMx4>::value;
    const int l1 = MX ? lanes_for_mx4(C1 / F::UW) : lanes_for(C1 / F::UW);
    const int l2 = MX ? lanes_for_mx4(C2 / F::UW) : lanes_for(C2 / F::UW);
    int32_t rc;
    switch (l1) {
        case 64: rc = launch_gate_up<F, OSS, 64>(gate_up, x, idx, gu, R1, C1, (int)k, (int)E, (int)(T * k), glu, st); break;
        case 32: rc = launch_gate_up<F, OSS, 32>(gate_up, x, idx, gu, R1, C1, (int)k, (int)E, (int)(T * k), glu, st); break;
        default: rc = launch_gate_up<F, OSS, 16>(gate_up, x, idx, gu, R1, C1, (int)k, (int)E, (int)(T * k), glu, st); break;
    }
    if (rc != OK) return rc;
    switch (l2) {
        case 64: return launch_down<F, 64>(down, gu, idx, w, y, R2, C2, (int)k, (int)E, (int)T, dn_bias, st);
        case 32: return launch_down<F, 32>(down, gu, idx, w, y, R2, C2, (int)k, (int)E, (int)T, dn_bias, st);
        default: return launch_down<F, 16>(down, gu, idx, w, y, R2, C2, (int)k, (int)E, (int)T, dn_bias, st);
    }
}

}  // namespace btb

using namespace btb;

extern "C" {

int32_t btb_hip_moe_route(const void* logits, int32_t logits_f32, size_t ls, size_t E, size_t k, size_t T, int32_t* idx,
                          void* w, float* w32, void* stream) {
    if (logits == nullptr || idx == nullptr || w == nullptr) return ERR_NULL;
    if (E == 0 || k == 0 || T == 0 || k > E || k > (size_t)ROUTE_MAX_K || ls < E || E > 8192 || T > 0x7FFFFFFFull)
        return ERR_DOMAIN;
    if (!al(logits, logits_f32 ? 4 : 2) || !al(idx, 4) || !al(w, 2) || !al(w32, 4)) return ERR_DOMAIN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (logits_f32)
        return launch_route<true>(logits, ls, (int)E, (int)k, (int)T, idx, static_cast<uint16_t*>(w), w32, nullptr, st);
    return launch_route<false>(logits, ls, (int)E, (int)k, (int)T, idx, static_cast<uint16_t*>(w), w32, nullptr, st);
}

int32_t btb_hip_moe_group_picks(const int32_t* idx, size_t T, size_t k, size_t E, int32_t* slot, int32_t* token,
                                int32_t* offs, int32_t* counts, void* stream) {
    if (idx == nullptr || slot == nullptr || token == nullptr || offs == nullptr || counts == nullptr) return ERR_NULL;
    if (T == 0 || k == 0 || E == 0 || T * k > 65535 || E > (1u << 20)) return ERR_DOMAIN;
    if (!al(idx, 4) || !al(slot, 4) || !al(token, 4) || !al(offs, 4) || !al(counts, 4)) return ERR_DOMAIN;
    hipLaunchKernelGGL(moe_group_picks_kernel, dim3((unsigned)((E + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), idx, (int)T, (int)k, (int)E, slot, token, offs, counts);
    return hip_status(hipGetLastError(), "moe_group_picks launch");
}

int32_t btb_hip_moe_router_bf16(const void* router, const void* x, size_t T, size_t E, size_t H, size_t k, float* logits,
                                void* logits16, int32_t* idx, void* w, float* w32, void* stream) {
    if (router == nullptr || x == nullptr || logits == nullptr || idx == nullptr || w == nullptr) return ERR_NULL;
    if (E == 0 || k == 0 || T == 0 || H == 0 || k > E || k > (size_t)ROUTE_MAX_K || E > 8192 || T > 65535)
        return ERR_DOMAIN;
    if (!al(router, 2) || !al(x, 2) || !al(logits, 4) || !al(logits16, 2) || !al(idx, 4) || !al(w, 2) || !al(w32, 4))
        return ERR_DOMAIN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t rc =
        lane16_bf16_rows16(static_cast<const uint16_t*>(router), E, H, static_cast<const uint16_t*>(x), T, logits, st);
    if (rc != OK) return rc;
    return launch_route<true>(logits, E, (int)E, (int)k, (int)T, idx, static_cast<uint16_t*>(w), w32,
                              static_cast<uint16_t*>(logits16), st);
}

int32_t btb_hip_moe_experts_bf16(const void* gate_up, const void* down, const void* x, const int32_t* idx, const void* w,
                                 void* gu, void* y, size_t T, size_t k, size_t E, size_t H, size_t I, void* stream) {
    if (gate_up == nullptr || down == nullptr || x == nullptr || idx == nullptr || w == nullptr || gu == nullptr ||
        y == nullptr)
        return ERR_NULL;
    if (T == 0 || k == 0 || E == 0 || H == 0 || I == 0 || k > (size_t)ROUTE_MAX_K || T * k > 65535 || H % 8 != 0 ||
        I % 8 != 0 || H > (1u << 20) || I > (1u << 20) || E > (1u << 20))
        return ERR_DOMAIN;
    if (!al(gate_up, 16) || !al(down, 16) || !al(x, 16) || !al(gu, 16) || !al(idx, 4) || !al(w, 2) || !al(y, 2))
        return ERR_DOMAIN;
    const DeviceInfo& dev = device_info();
    if (k * I * 2 > (size_t)dev.lds_bytes || H * 2 > (size_t)dev.lds_bytes) {
        set_error("moe: the staged rows do not fit LDS");
        return ERR_DOMAIN;
    }
    return launch_experts<FmtBf16, false>(Stack{gate_up, nullptr}, Stack{down, nullptr}, x, idx, w, gu, y, T, k, E, H, I,
                                          Glu{nullptr, 0.f, 0.f}, nullptr, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_moe_experts_mxfp4(const void* gu_blocks, const void* gu_scales, const void* dn_blocks,
                                  const void* dn_scales, const void* gu_bias, const void* dn_bias, const void* x,
                                  const int32_t* idx, const void* w, void* h, void* y, size_t T, size_t k, size_t E,
                                  size_t H, size_t I, int32_t oss, float alpha, float limit, void* stream) {
    if (gu_blocks == nullptr || gu_scales == nullptr || dn_blocks == nullptr || dn_scales == nullptr || x == nullptr ||
        idx == nullptr || w == nullptr || h == nullptr || y == nullptr)
        return ERR_NULL;
    if (T == 0 || k == 0 || E == 0 || H == 0 || I == 0 || k > (size_t)ROUTE_MAX_K || T * k > 65535 || H % 32 != 0 ||
        I % 32 != 0 || H > (1u << 20) || I > (1u << 20) || E > (1u << 20))
        return ERR_DOMAIN;
    if (!al(gu_blocks, 16) || !al(dn_blocks, 16) || !al(x, 16) || !al(h, 16) || !al(idx, 4) || !al(w, 2) || !al(y, 2) ||
        !al(gu_bias, 2) || !al(dn_bias, 2))
        return ERR_DOMAIN;
    if (!oss && (gu_bias != nullptr || dn_bias != nullptr)) {
        set_error("moe_experts_mxfp4: biases belong to the gpt-oss form (oss != 0)");
        return ERR_DOMAIN;
    }
    if (oss && !(limit > 0.f && alpha == alpha)) return ERR_DOMAIN;
    const DeviceInfo& dev = device_info();
    if (k * I * 2 > (size_t)dev.lds_bytes || H * 2 > (size_t)dev.lds_bytes) {
        set_error("moe: the staged rows do not fit LDS");
        return ERR_DOMAIN;
    }
    hipStream_t st = static_cast<hipStream_t>(stream);
    const Stack gs{gu_blocks, gu_scales}, ds{dn_blocks, dn_scales};
    if (oss)
        return launch_experts<FmtMx4, true>(gs, ds, x, idx, w, h, y, T, k, E, H, I,
                                            Glu{static_cast<const uint16_t*>(gu_bias), alpha, limit}, dn_bias, st);
    return launch_experts<FmtMx4, false>(gs, ds, x, idx, w, h, y, T, k, E, H, I, Glu{nullptr, 0.f, 0.f}, nullptr, st);
}

}  // extern "C"
