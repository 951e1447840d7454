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
// other workgroups are still reading it).
struct XArgs {
    const uint16_t* x;
    const uint16_t* y;
    const uint16_t* norm_w;
    uint16_t* h_out;
    float eps;
    int centered;
};

// the fold the reference's btb_gemv_silu_bf16 makes in its x load (native/cuda/btb_kernels.cu:168-209):
// x = bf16(bf16(silu(g)) * u), g and u the two halves of a [M, 2C] row
__device__ __forceinline__ uint32_t silu_pair(uint32_t g2, uint32_t u2) {
    const float s0 = bfround(bf16lo_f32(g2) / (1.f + expf(-bf16lo_f32(g2))));
    const float s1 = bfround(bf16hi_f32(g2) / (1.f + expf(-bf16hi_f32(g2))));
    const uint32_t lo = f32_bf16(s0 * bf16lo_f32(u2));
    const uint32_t hi = f32_bf16(s1 * bf16hi_f32(u2));
    return lo | (hi << 16);
}

// sum over a 256-thread block in a fixed order: each wave's DPP tree, then waves 0..3 in order
__device__ __forceinline__ float block_sum256(float v, float* red) {
    v = group_sum<64>(v);
    const int wv = threadIdx.x >> 6;
    if ((threadIdx.x & 63) == 0) red[wv] = v;
    __syncthreads();
    const float s = ((red[0] + red[1]) + red[2]) + red[3];
    __syncthreads();
    return s;
}

// LDS the staging needs for M rows of C values: the rows themselves, and for X_ADDNORM three raw rows (h, y and the
// norm's weight) behind them
__host__ __device__ constexpr size_t stage_lds_bytes(int xmode, int M, int C) {
    return (size_t)(M + (xmode == X_ADDNORM ? 3 : 0)) * (size_t)C * 2;
}

// Leaves the rows in xs (a barrier included). 256 threads. `after_issue` is called once, right after the first loads
// of the staging have been issued and before anything waits for them: the caller requests its first weights there,
// so they travel while the staging's own (short) round trip and arithmetic run.
template <int XMODE, class AfterIssue>
__device__ __forceinline__ void stage_x(uint32_t* xs, const XArgs& a, int M, int C, AfterIssue after_issue) {
    const int tid = threadIdx.x, nt = blockDim.x;
    if (XMODE == X_PLAIN) {
        const uint4* src = reinterpret_cast<const uint4*>(a.x);
        uint4* dst = reinterpret_cast<uint4*>(xs);
        const int n = M * C / 8;
        const uint4 v0 = src[min(tid, n - 1)];
        after_issue();
        if (tid < n) dst[tid] = v0;
        for (int i = tid + nt; i < n; i += nt) dst[i] = src[i];
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
        // stand-alone add_rmsnorm kernel (thread i takes elements i, i + 256, ...), so the bits are its bits. Every
        // workgroup makes the whole row for itself; the first also writes the new residual out. The row's inputs
        // come in with 8-byte loads, all issued together, into raw rows in LDS; the arithmetic then reads LDS in its
        // own element order.
        __shared__ float red[4];
        uint16_t* xs16 = reinterpret_cast<uint16_t*>(xs);
        uint16_t* hraw = xs16 + (size_t)M * C;
        uint16_t* yraw = hraw + C;
        uint16_t* wraw = yraw + C;
        const int n4 = C / 4;  // 8-byte words per row (C is a multiple of the format's unit, at least 8)
        constexpr int PER = 3;  // words a thread holds at once: rows up to 3072 wide take one pass
        for (int m = 0; m < M; ++m) {
            const uint2* hs = reinterpret_cast<const uint2*>(a.x + (size_t)m * C);
            const uint2* ys = a.y == nullptr ? nullptr : reinterpret_cast<const uint2*>(a.y + (size_t)m * C);
            const uint2* ws = reinterpret_cast<const uint2*>(a.norm_w);
            for (int base = 0; base < n4; base += PER * 256) {
                uint2 hv[PER], yv[PER], wv[PER];
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    // a word past the row's end reads the last word again: the loads stay unconditional, and the
                    // wait for them is then counted exactly (they are not held up behind the weights requested next)
                    const int i = min(base + q * 256 + tid, n4 - 1);
                    hv[q] = hs[i];
                    yv[q] = ys != nullptr ? ys[i] : make_uint2(0, 0);
                    wv[q] = ws[i];
                }
                if (m == 0 && base == 0) after_issue();
#pragma unroll
                for (int q = 0; q < PER; ++q) {
                    const int i = base + q * 256 + tid;
                    if (i < n4) {
                        reinterpret_cast<uint2*>(hraw)[i] = hv[q];
                        reinterpret_cast<uint2*>(yraw)[i] = yv[q];
                        if (m == 0) reinterpret_cast<uint2*>(wraw)[i] = wv[q];
                    }
                }
            }
            __syncthreads();
            uint16_t* row = xs16 + (size_t)m * C;
            float ss = 0.f;
            for (int i = tid; i < C; i += 256) {
                float hv = bf16_f32(hraw[i]);
                if (ys != nullptr) hv = bfround(hv + bf16_f32(yraw[i]));
                row[i] = f32_bf16(hv);
                ss = fmaf(hv, hv, ss);
            }
            const float rstd = rsqrtf(block_sum256(ss, red) / (float)C + a.eps);
            for (int i = tid; i < C; i += 256) {
                const uint16_t hb = row[i];
                if (blockIdx.x == 0 && blockIdx.y == 0 && a.h_out != nullptr) a.h_out[(size_t)m * C + i] = hb;
                const float wv = bf16_f32(wraw[i]);
                row[i] = f32_bf16(bf16_f32(hb) * rstd * (a.centered ? 1.f + wv : wv));
            }
            __syncthreads();  // the raw rows are free for the next row
        }
    }
    __syncthreads();
}

template <int XMODE>
__device__ __forceinline__ void stage_x(uint32_t* xs, const XArgs& a, int M, int C) {
    stage_x<XMODE>(xs, a, M, C, [] {});
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
__device__ __forceinline__ void fma_unit(const typename F::RowCtx (&ctx)[RPW], const typename F::Raw (&raw)[RPW],
                                         int unit, const uint4* xs4, int xrow4, float (&acc)[RPW][M]) {
    constexpr int UW = F::UW;
    constexpr int H = UW / 8;
    uint4 xv[H][M];
#pragma unroll
    for (int h = 0; h < H; ++h)
#pragma unroll
        for (int m = 0; m < M; ++m) xv[h][m] = xs4[m * xrow4 + unit * H + h];
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

// where the kernel reads x from: LDS (staged once per workgroup) or straight from global memory through the caches
enum XSrc { XS_LDS = 0, XS_GLOBAL = 1 };

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

template <class F, int M, int LPR, int RPW, int U, bool GUARD>
__device__ __forceinline__ void fma_span(const typename F::Raw (&raw)[U][RPW], const typename F::RowCtx (&ctx)[RPW],
                                         int k0, int sl, int units, const uint4* xs4, int xrow4,
                                         float (&acc)[RPW][M]) {
#pragma unroll
    for (int u = 0; u < U; ++u) {
        const int unit = k0 + u * LPR + sl;
        if (!GUARD || unit < units) fma_unit<F, M, RPW>(ctx, raw[u], unit, xs4, xrow4, acc);
        // one unit's widening and products at a time: without the fence the scheduler hoists every unit's widening
        // ahead of the first product and the live registers cost the kernel its occupancy
        __builtin_amdgcn_sched_barrier(0);
    }
}

}  // namespace btb
