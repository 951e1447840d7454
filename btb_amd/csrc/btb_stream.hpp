// The streaming matvec's building blocks, shared by the dense kernels (gemv.hip) and the routed-expert kernels
// (moe.hip): staging x in LDS, the span loads, and the pair-wise products of one unit against the rows of x.
#pragma once

#include "btb_common.hpp"
#include "btb_formats.hpp"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// x staging: the M rows of x into LDS as packed bf16 pairs - copied as they are, made by the SwiGLU fold from a
// [M, 2C] gate/up block, or made by the residual add + RMSNorm from the residual stream
// ------------------------------------------------------------------------------------------------------------

enum XMode { X_PLAIN = 0, X_SILU = 1, X_ADDNORM = 2 };

// where x comes from. X_PLAIN: x [M, C]. X_SILU: x is gu [M, 2C]. X_ADDNORM: x is the residual h [M, C]; y the block
// output added to it (or null), norm_w the norm's weight, h_out where the new residual is written (not h itself:
// other workgroups are still reading it). With `ids` (X_ADDNORM only) x is an embedding table [vocab, C] and row m of
// the residual is table[ids[m]] (an id outside the table is clamped into it): the step's first layer, whose residual
// is the token's embedding.
struct XArgs {
    const uint16_t* x;
    const uint16_t* y;
    const uint16_t* norm_w;
    uint16_t* h_out;
    float eps;
    int centered;
    const int32_t* ids = nullptr;
    int vocab = 0;
};

// the fold the reference's btb_gemv_silu_bf16 makes in its x load (native/cuda/btb_kernels.cu:168-209):
// x = bf16(bf16(silu(g)) * u), g and u the two halves of a [M, 2C] row
__device__ __forceinline__ uint32_t silu_pair(uint32_t g2, uint32_t u2) {
    const float s0 = bfround(bf16lo_f32(g2) / (1.f + expf(-bf16lo_f32(g2))));
    const float s1 = bfround(bf16hi_f32(g2) / (1.f + expf(-bf16hi_f32(g2))));
    return f32x2_bf16(s0 * bf16lo_f32(u2), s1 * bf16hi_f32(u2));
}

// sum over a 256-thread block in a fixed order: each wave's DPP tree, then waves 0..3 in order
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = group_sum_last<64>(v);
    const int wv = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 63) red[wv] = v;
    __syncthreads();
    const float s = ((red[0] + red[1]) + red[2]) + red[3];
    __syncthreads();
    return s;
}

// LDS the staging needs for M rows of C values: the rows themselves, and for X_ADDNORM three raw rows (h, y and the
// norm's weight) behind them
__host__ __device__ constexpr size_t stage_lds_bytes(int xmode, int M, int C) {
    return (size_t)(M + (xmode == X_ADDNORM ? 1 : 0)) * (size_t)C * 2;
}

// Leaves the rows in xs (a barrier included). 256 threads. `after_issue` is called once, right after the first loads
// of the staging have been issued and before anything waits for them: the caller requests its first weights there,
// so they travel while the staging's own (short) round trip and arithmetic run.
// MR: the number of rows where the caller knows it at compile time (M is then MR), 0 otherwise. KEEP: the one-row
// add + norm keeps its words in registers across the sum (see there).
// a scheduling barrier that only loads and stores of global memory may not cross (ALU and LDS instructions may)
constexpr int VMEM_STAYS = 0x38F;

// NT: the workgroup's threads (256; 320 for the plain copy, where five waves a workgroup fill the CUs evenly).
template <int XMODE, int MR = 0, bool KEEP = false, int NT = 256, class AfterIssue>
__device__ __forceinline__ void stage_x(uint32_t* xs, const XArgs& a, int M, int C, AfterIssue after_issue) {
    static_assert(NT == 256 || XMODE == X_PLAIN, "only the plain copy is written for other workgroup sizes");
    const int tid = threadIdx.x, nt = blockDim.x;
    if (XMODE == X_PLAIN) {
        // the first five 16-byte pieces a thread copies (rows up to 10240 values) are requested together and
        // unconditionally - a piece past the end reads the last piece again - so that the wait for them is counted
        // exactly and does not take in the weights requested behind them. The stores are unconditional as well (a
        // load whose only use sits in a branch is moved into it, behind the weights): the repeated piece is written
        // to its own place again
        // (the pieces wait in an array of compiler vectors: an array of HIP's uint4 structs goes to scratch memory once
        // the scheduling barrier below stands between its writes and its reads)
        const u32x4* src = reinterpret_cast<const u32x4*>(a.x);
        u32x4* dst = reinterpret_cast<u32x4*>(xs);
        const int n = M * C / 8;
        constexpr int PER = 1280 / NT;  // rows up to 10240 values in the one request
        u32x4 v[PER];
#pragma unroll
        for (int q = 0; q < PER; ++q) v[q] = src[min(tid + q * NT, n - 1)];
        // the caller's weights stay behind these loads: moved ahead of them by the scheduler, the staging below waited
        // for weights out of HBM where it needs x out of L2 (loads come back in order)
        __builtin_amdgcn_sched_barrier(VMEM_STAYS);
        after_issue();
#pragma unroll
        for (int q = 0; q < PER; ++q) dst[min(tid + q * NT, n - 1)] = v[q];
        for (int i = tid + PER * NT; i < n; i += NT) dst[i] = src[i];
    } else if (XMODE == X_SILU) {
        after_issue();
        const int half = C / 2;  // pairs per row
        const uint32_t* src = reinterpret_cast<const uint32_t*>(a.x);
        for (int i = tid; i < M * half; i += nt) {
            const int m = i / half, c = i - m * half;
            xs[i] = silu_pair(src[(size_t)m * 2 * half + c], src[(size_t)m * 2 * half + half + c]);
        }
    } else {
        // h' = bf16(h + y); x = bf16(h' * rsqrt(mean(h'^2) + eps) * w): the arithmetic and the summation order of the
        // stand-alone add_rmsnorm kernel (thread i takes the 4-element words i, i + 256, ..., a word's elements in
        // order), so the bits are its bits. Every workgroup makes the whole row for itself; the first also writes the
        // new residual out. A thread's words come in with 8-byte loads, all issued together, and it works on them in
        // registers: h' and the norm weight wait in the thread's own LDS slots while the block sums the squares, so
        // no barrier is needed besides the sum's own.
        __shared__ float red[4];
        uint2* rows4 = reinterpret_cast<uint2*>(xs);
        const int n4 = C / 4;  // 8-byte words per row (C is a multiple of the format's unit, at least 8)
        uint2* wkeep = rows4 + (size_t)M * n4;
        constexpr int PER = 3;  // words a thread holds at once: rows up to 3072 wide take one pass
        const bool writer = blockIdx.x == 0 && blockIdx.y == 0 && a.h_out != nullptr;
        if (KEEP && MR == 1 && n4 <= PER * 256) {
            // One row, one pass (the decode step's own launches): the thread's words stay in registers between the
            // sum of squares and the scaling - nothing of them goes to LDS and comes back - and the one sum needs
            // one barrier, not two (its four partial sums are not written again). The arithmetic, its order and the
            // stores are the loop's below. Taken by the forms that widen in registers (the packed step 2.063 ->
            // 2.054 ms); the bf16 kernels lose by it (qkv 7.40 -> 7.50 us, the step 2.026 -> 2.035 ms) and keep the
            // loop.
            uint2 hv[PER], yv[PER], wv[PER];
            size_t hrow = 0;
            if (a.ids != nullptr) hrow = (size_t)min(max(a.ids[0], 0), a.vocab - 1);
            const uint2* hs = reinterpret_cast<const uint2*>(a.x + hrow * C);
            const uint2* ys = a.y == nullptr ? hs : reinterpret_cast<const uint2*>(a.y);
            const uint2* ws = reinterpret_cast<const uint2*>(a.norm_w);
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const int i = min(q * 256 + tid, n4 - 1);
                hv[q] = hs[i];
                yv[q] = ys[i];
                wv[q] = ws[i];
            }
            after_issue();
            const bool has_y = a.y != nullptr;
            float f[PER][4];
            float ss = 0.f;
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const bool live = q * 256 + tid < n4;
                const float h4[4] = {bf16lo_f32(hv[q].x), bf16hi_f32(hv[q].x), bf16lo_f32(hv[q].y), bf16hi_f32(hv[q].y)};
                const float g[4] = {bf16lo_f32(yv[q].x), bf16hi_f32(yv[q].x), bf16lo_f32(yv[q].y), bf16hi_f32(yv[q].y)};
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float sum = bfround(h4[e] + g[e]);
                    f[q][e] = has_y ? sum : h4[e];
                    const float sq = fmaf(f[q][e], f[q][e], ss);
                    ss = live ? sq : ss;
                }
                if (writer)
                    reinterpret_cast<uint2*>(a.h_out)[min(q * 256 + tid, n4 - 1)] =
                        make_uint2(f32x2_bf16(f[q][0], f[q][1]), f32x2_bf16(f[q][2], f[q][3]));
            }
            ss = group_sum_last<64>(ss);
            if ((tid & 63) == 63) red[tid >> 6] = ss;
            __syncthreads();
            const float rstd = rsqrtf((((red[0] + red[1]) + red[2]) + red[3]) / (float)C + a.eps);
#pragma unroll
            for (int q = 0; q < PER; ++q) {
                const float g[4] = {bf16lo_f32(wv[q].x), bf16hi_f32(wv[q].x), bf16lo_f32(wv[q].y), bf16hi_f32(wv[q].y)};
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f[q][e] * rstd * (a.centered ? 1.f + g[e] : g[e]);
                rows4[min(q * 256 + tid, n4 - 1)] = make_uint2(f32x2_bf16(o[0], o[1]), f32x2_bf16(o[2], o[3]));
            }
            __syncthreads();
            return;
        }
        if (MR > 1 && n4 <= PER * 256) {
            // Several rows, each one pass: every row's words are requested before anything waits - and before the
            // caller's first weights, which travel behind them. Row by row (the loop below) a row's loads queue
            // behind those weights, and since loads return in order every further row waited for a span of weights:
            // [19456 x 2560] with add + norm, 2 / 4 rows: 25.4 / 36.5 us against 18.9 / 21.8 for the plain matvec.
            // The arithmetic, its order and the stores are the loop's.
            constexpr int MRC = MR > 1 ? MR : 1;
            uint2 hv[MRC][PER], yv[MRC][PER], wv[PER];
            const uint2* ws = reinterpret_cast<const uint2*>(a.norm_w);
#pragma unroll
            for (int m = 0; m < MRC; ++m) {
                size_t hrow = (size_t)m;
                if (a.ids != nullptr) hrow = (size_t)min(max(a.ids[m], 0), a.vocab - 1);
                const uint2* hs = reinterpret_cast<const uint2*>(a.x + hrow * C);
                const uint2* ys = a.y == nullptr ? hs : reinterpret_cast<const uint2*>(a.y + (size_t)m * C);
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = min(q * 256 + tid, n4 - 1);
                    hv[m][q] = hs[i];
                    yv[m][q] = ys[i];
                    if (m == 0) wv[q] = ws[i];
                }
            }
            after_issue();
            const bool has_y = a.y != nullptr;
#pragma unroll
            for (int m = 0; m < MRC; ++m) {
                uint2* row = rows4 + (size_t)m * n4;
                float ss = 0.f;
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = q * 256 + tid;
                    const bool live = i < n4;
                    float f[4] = {bf16lo_f32(hv[m][q].x), bf16hi_f32(hv[m][q].x), bf16lo_f32(hv[m][q].y), bf16hi_f32(hv[m][q].y)};
                    const float g[4] = {bf16lo_f32(yv[m][q].x), bf16hi_f32(yv[m][q].x), bf16lo_f32(yv[m][q].y), bf16hi_f32(yv[m][q].y)};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float sum = bfround(f[e] + g[e]);
                        f[e] = has_y ? sum : f[e];
                        const float sq = fmaf(f[e], f[e], ss);
                        ss = live ? sq : ss;
                    }
                    const uint2 hb = make_uint2(f32x2_bf16(f[0], f[1]), f32x2_bf16(f[2], f[3]));
                    const int ic = min(i, n4 - 1);
                    row[ic] = hb;
                    if (m == 0) wkeep[ic] = wv[q];
                    if (writer) reinterpret_cast<uint2*>(a.h_out + (size_t)m * C)[ic] = hb;
                }
                const float rstd = rsqrtf(block_sum256(ss, red) / (float)C + a.eps);
                for (int i = tid; i < n4; i += 256) {
                    const uint2 hb = row[i], wb = wkeep[i];
                    const float f[4] = {bf16lo_f32(hb.x), bf16hi_f32(hb.x), bf16lo_f32(hb.y), bf16hi_f32(hb.y)};
                    const float g[4] = {bf16lo_f32(wb.x), bf16hi_f32(wb.x), bf16lo_f32(wb.y), bf16hi_f32(wb.y)};
                    float o[4];
#pragma unroll
                    for (int e = 0; e < 4; ++e) o[e] = f[e] * rstd * (a.centered ? 1.f + g[e] : g[e]);
                    row[i] = make_uint2(f32x2_bf16(o[0], o[1]), f32x2_bf16(o[2], o[3]));
                }
            }
            __syncthreads();
            return;
        }
        for (int m = 0; m < M; ++m) {
            size_t hrow = (size_t)m;
            if (a.ids != nullptr) hrow = (size_t)min(max(a.ids[m], 0), a.vocab - 1);  // uniform: one scalar load
            const uint2* hs = reinterpret_cast<const uint2*>(a.x + hrow * C);
            const uint2* ys = a.y == nullptr ? hs : reinterpret_cast<const uint2*>(a.y + (size_t)m * C);
            const uint2* ws = reinterpret_cast<const uint2*>(a.norm_w);
            uint2* row = rows4 + (size_t)m * n4;
            float ss = 0.f;
            for (int base = 0; base < n4; base += PER * 256) {
                uint2 hv[PER], yv[PER], wv[PER];
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    // a word past the row's end reads the last word again: the loads stay unconditional, and the
                    // wait for them is then counted exactly (they are not held up behind the weights requested next)
                    const int i = min(base + q * 256 + tid, n4 - 1);
                    hv[q] = hs[i];
                    yv[q] = ys[i];  // no y: h again, unused
                    wv[q] = ws[i];
                }
                if (m == 0 && base == 0) after_issue();
                // the arithmetic and the stores are unconditional too (selects, not branches: a load whose only use
                // sits in a branch is moved into it, behind the weights); a word past the end is the last word
                // again, and is written to the last word's place again
                const bool has_y = a.y != nullptr;
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = base + q * 256 + tid;
                    const bool live = i < n4;
                    float f[4] = {bf16lo_f32(hv[q].x), bf16hi_f32(hv[q].x), bf16lo_f32(hv[q].y), bf16hi_f32(hv[q].y)};
                    const float g[4] = {bf16lo_f32(yv[q].x), bf16hi_f32(yv[q].x), bf16lo_f32(yv[q].y), bf16hi_f32(yv[q].y)};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float sum = bfround(f[e] + g[e]);
                        f[e] = has_y ? sum : f[e];
                        const float sq = fmaf(f[e], f[e], ss);
                        ss = live ? sq : ss;
                    }
                    const uint2 hb = make_uint2(f32x2_bf16(f[0], f[1]), f32x2_bf16(f[2], f[3]));
                    const int ic = min(i, n4 - 1);
                    row[ic] = hb;
                    wkeep[ic] = wv[q];
                    if (writer) reinterpret_cast<uint2*>(a.h_out + (size_t)m * C)[ic] = hb;
                }
            }
            const float rstd = rsqrtf(block_sum256(ss, red) / (float)C + a.eps);
            for (int i = tid; i < n4; i += 256) {
                const uint2 hb = row[i], wb = wkeep[i];
                const float f[4] = {bf16lo_f32(hb.x), bf16hi_f32(hb.x), bf16lo_f32(hb.y), bf16hi_f32(hb.y)};
                const float g[4] = {bf16lo_f32(wb.x), bf16hi_f32(wb.x), bf16lo_f32(wb.y), bf16hi_f32(wb.y)};
                float o[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = f[e] * rstd * (a.centered ? 1.f + g[e] : g[e]);
                row[i] = make_uint2(f32x2_bf16(o[0], o[1]), f32x2_bf16(o[2], o[3]));
            }
        }
    }
    __syncthreads();
}

template <int XMODE>
__device__ __forceinline__ void stage_x(uint32_t* xs, const XArgs& a, int M, int C) {
    stage_x<XMODE, 0, false, 256>(xs, a, M, C, [] {});
}

// ------------------------------------------------------------------------------------------------------------
// the kernel
// ------------------------------------------------------------------------------------------------------------

// one unit of every one of the RPW rows against the M rows of x. x is read once from LDS, eight values (four bf16
// pairs) at a time; a weight pair meets its x pair in one v_dot2_f32_bf16: acc += w0 * x0 + w1 * x1 with the products
// exact and the sum kept in f32, pairs in ascending column order.
__device__ __forceinline__ float dot2(uint32_t w, uint32_t x, float acc) {
    return __builtin_amdgcn_fdot2_f32_bf16(__builtin_bit_cast(bf16x2, w), __builtin_bit_cast(bf16x2, x), acc, false);
}

template <class F, int M, int RPW>
__device__ __forceinline__ void fma_unit_x(const typename F::RowCtx (&ctx)[RPW], const typename F::Raw (&raw)[RPW],
                                           int unit, const uint4 (&xv)[F::UW / 8][M], float (&acc)[RPW][M]) {
    constexpr int UW = F::UW;
    constexpr int H = UW / 8;
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
        uint32_t w[UW / 2];
        F::widen(ctx[j], raw[j], unit, w);
#pragma unroll
        for (int h = 0; h < H; ++h)
#pragma unroll
            for (int m = 0; m < M; ++m) {
                float a = acc[j][m];
                a = dot2(w[h * 4 + 0], xv[h][m].x, a);
                a = dot2(w[h * 4 + 1], xv[h][m].y, a);
                a = dot2(w[h * 4 + 2], xv[h][m].z, a);
                a = dot2(w[h * 4 + 3], xv[h][m].w, a);
                acc[j][m] = a;
            }
    }
}
template <class F, int M, int RPW>
__device__ __forceinline__ void fma_unit(const typename F::RowCtx (&ctx)[RPW], const typename F::Raw (&raw)[RPW],
                                         int unit, const uint4* xs4, int xrow4, float (&acc)[RPW][M]) {
    constexpr int H = F::UW / 8;
    uint4 xv[H][M];
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
        for (int m = 0; m < M; ++m) xv[h][m] = xs4[m * xrow4 + unit * H + h];
    fma_unit_x<F, M, RPW>(ctx, raw, unit, xv, acc);
}

// what a finished pair of row sums becomes. E_PLAIN: y[m][r] = bf16(sum). E_GLU: the matrix is [2I, C], gate rows then
// up rows; a wave works on gate row r and up row I + r together and writes m[m][r] = bf16(bf16(silu(g)) * u) with
// g, u the two sums rounded to bf16 first - the values the gate_up matvec followed by btb_silu_mul would have
// written (the reference's btb_gemv_mma_glu_silu does the same fold: native/cuda/btb_gemv_mma.cuh:216-315).
// E_GLU_SPLIT: the same fold with the gate row and the up row side by side in one wave - even row groups of the
// wave take gate rows, the odd group next to each its up row (rows of at most 32 lanes) - and the two sums meeting by
// one cross-lane exchange: the tile shape of a one-row-per-lane pass, which the register-hungry packed forms prefer.
enum Epilogue { E_PLAIN = 0, E_GLU = 1, E_GLU_SPLIT = 2 };

// output rows a wave's tile covers, and the weight row of the lane's row group (set j) with the row its sum goes to
template <int LPR, int RPW, int EPI>
__host__ __device__ constexpr int tile_outputs() {
    return EPI == E_GLU ? WAVE / LPR : EPI == E_GLU_SPLIT ? WAVE / LPR / 2 : (WAVE / LPR) * RPW;
}
template <int LPR, int RPW, int EPI>
__device__ __forceinline__ int tile_row(int tile, int j, int lane, int R, int& out_row) {
    constexpr int G = WAVE / LPR;
    const int grp = lane / LPR;
    if (EPI == E_GLU) {
        out_row = tile * G + grp;
        return min(out_row, R / 2 - 1) + j * (R / 2);
    }
    if (EPI == E_GLU_SPLIT) {
        out_row = tile * (G / 2) + grp / 2;
        return min(out_row, R / 2 - 1) + (grp & 1) * (R / 2);
    }
    out_row = tile * G * RPW + j * G + grp;
    return min(out_row, R - 1);  // a row past the end reads the last row again (no divergence) and is not written
}

// the loads of one span: U units of each of the RPW rows; a unit past the row's end is not loaded
template <class F, int LPR, int RPW, int U, bool GUARD>
__device__ __forceinline__ void load_span(typename F::Raw (&raw)[U][RPW], const typename F::RowCtx (&ctx)[RPW], int k0,
                                          int sl, int units) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int unit = k0 + u * LPR + sl;
        if (!GUARD || unit < units) {
#pragma unroll
            for (int j = 0; j < RPW; ++j) raw[u][j] = F::load(ctx[j], unit);
        }
    }
}

// the same loads with nothing conditional about them: a unit past the row's end reads the row's last unit again (and
// is not used). Requested ahead of a wait for earlier loads, every one of these is certain to have been issued, so that
// wait is counted exactly and does not hold out for these as well.
template <class F, int LPR, int RPW, int U>
__device__ __forceinline__ void load_span_always(typename F::Raw (&raw)[U][RPW], const typename F::RowCtx (&ctx)[RPW],
                                                 int k0, int sl, int units) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int unit = min(k0 + u * LPR + sl, units - 1);
#pragma unroll
        for (int j = 0; j < RPW; ++j) raw[u][j] = F::load(ctx[j], unit);
    }
}

template <class F, int M, int LPR, int RPW, int U, bool GUARD>
__device__ __forceinline__ void fma_span(const typename F::Raw (&raw)[U][RPW], const typename F::RowCtx (&ctx)[RPW],
                                         int k0, int sl, int units, const uint4* xs4, int xrow4,
                                         float (&acc)[RPW][M]) {
    constexpr int H = F::UW / 8;
    constexpr bool WIDENS = sizeof(typename F::Raw) != 16;  // everything but plain bf16
    if constexpr (!WIDENS && (M == 1 || (M <= 3 && U * H * M <= 8))) {
        // bf16, one row of x (or two or three, where that is at most 32 registers): the span's x values are all asked
        // of LDS before the first product, so their trips overlap one another (and, for a span still on its way from
        // memory, the weights' flight) instead of standing one behind the other between the products. A unit past the
        // row's end reads the row's last unit (and is not used). Measured: the one-row bf16 step 2.150 -> 2.115 ms,
        // a pass of two rows 0.6 % faster. At four rows the registers cost more than the overlap returns (bf16
        // [9728 x 2560] 11.8 -> 12.6 us, the grouped MoE gate/up 109 -> 124 us a layer at 8 tokens), and so they do
        // for the forms that widen in registers at any width (one row: pack12 9.75 -> 11.2 us, FP8 26.7 -> 28.2, the
        // packed step 2.14 -> 2.27 ms).
        uint4 xv[U][H][M];
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int unit = GUARD ? min(k0 + u * LPR + sl, units - 1) : k0 + u * LPR + sl;
#pragma unroll
            for (int h = 0; h < H; ++h)
#pragma unroll
                for (int m = 0; m < M; ++m) xv[u][h][m] = xs4[m * xrow4 + unit * H + h];
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int unit = k0 + u * LPR + sl;
            if (!GUARD || unit < units) fma_unit_x<F, M, RPW>(ctx, raw[u], unit, xv[u], acc);
            __builtin_amdgcn_sched_barrier(0);
        }
    } else {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int unit = k0 + u * LPR + sl;
            if (!GUARD || unit < units) fma_unit<F, M, RPW>(ctx, raw[u], unit, xs4, xrow4, acc);
            // one unit's widening and products at a time: without the fence the scheduler hoists every unit's
            // widening ahead of the first product and the live registers cost the kernel its occupancy
            __builtin_amdgcn_sched_barrier(0);
        }
    }
}

}  // namespace btb
