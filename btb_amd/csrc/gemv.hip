// The decode weight matvec for gfx950: y[m][r] = sum_c W[r][c] * x[m][c], M = 1..4 rows of x on the vector ALUs
// (M = 5..32 take the MFMA kernels in gemv_mfma_lds.hip / gemv_mfma.hip). Memory-bound: every weight byte is read once, with 16-byte
// per-lane non-temporal loads, a wave covering 1 KiB of a row per load instruction and keeping RPW * U of them in
// flight; x is staged once per workgroup in LDS (optionally through the SwiGLU fold) and read from there with
// ds_read_b128, shared by the RPW rows a lane works on. A row is summed by LPR lanes (64, 32 or 16, chosen from the
// row length alone), each lane running its units in ascending column order, a pair of weights per v_dot2_f32_bf16
// (f32 accumulate), then a fixed DPP tree over the lanes: the sequence for (m, r) depends on neither M nor the launch, so row m of a wide pass
// equals the one-row pass bit for bit - the law the reference's card kernels keep (native/cuda/btb_kernels.cu:84-88).
//
// The same loop serves every stored form through a policy (btb_widen.hpp semantics, vector forms here): the bytes a
// lane loads are widened in its registers, never through a dequantised copy in memory.

#include <type_traits>

#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_stream.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// the kernel
// ------------------------------------------------------------------------------------------------------------


// one tile of gemv_stream: its RPW rows' sums over the M rows of x, written out. PRIMED: the tile's first span is
// already in `first` (requested before x was staged) and its rows' contexts in `first_ctx`.
template <class F, int M, int LPR, int RPW, int U, int EPI, bool PRIMED>
__device__ __forceinline__ void gemv_tile(const typename F::Params& p, const typename F::Raw (&first)[U][RPW],
                                          const typename F::RowCtx (&first_ctx)[RPW], int tile, const uint4* xs4,
                                          uint16_t* __restrict__ y, int R, int C, int lane) {
    const int Rout = EPI == E_PLAIN ? R : R / 2;
    const int units = C / F::UW;         // units per row
    const int sl = lane % LPR;           // the lane's place among its row's lanes
    const int span = U * LPR;
    const int xrow4 = C / 8;             // uint4 per row of x
    typename F::RowCtx ctx[RPW];
    int rows[RPW];   // weight rows
    int outs[RPW];   // the rows their sums are written to (the GLU forms: the output row of the pair)
#pragma unroll
    for (int j = 0; j < RPW; ++j) {
        rows[j] = tile_row<LPR, RPW, EPI>(tile, j, lane, R, outs[j]);
        // PRIMED: the rows' contexts were made where the span was requested - what a context asks of memory (pack12: the
        // row's slice of the escape list) was asked for ahead of the weights, not after the staging's barrier
        ctx[j] = PRIMED ? first_ctx[j] : F::row_ctx(p, (size_t)rows[j], units, sl);
    }
    float acc[RPW][M];
#pragma unroll
    for (int j = 0; j < RPW; ++j)
#pragma unroll
        for (int m = 0; m < M; ++m) acc[j][m] = 0.f;

    int k0 = 0;
    if (PRIMED) {
        if (span <= units)  // uniform: the first span is a full one, nothing in it to guard
            fma_span<F, M, LPR, RPW, U, false>(first, ctx, 0, sl, units, xs4, xrow4, acc);
        else
            fma_span<F, M, LPR, RPW, U, true>(first, ctx, 0, sl, units, xs4, xrow4, acc);
        k0 = span;
    }
    for (; k0 < units; k0 += span) {
        typename F::Raw raw[U][RPW];
        if (k0 + span <= units) {
            load_span<F, LPR, RPW, U, false>(raw, ctx, k0, sl, units);
            fma_span<F, M, LPR, RPW, U, false>(raw, ctx, k0, sl, units, xs4, xrow4, acc);
        } else {
            load_span<F, LPR, RPW, U, true>(raw, ctx, k0, sl, units);
            fma_span<F, M, LPR, RPW, U, true>(raw, ctx, k0, sl, units, xs4, xrow4, acc);
        }
    }
#pragma unroll
    for (int j = 0; j < RPW; ++j)
        F::template tail<M>(p, ctx[j], (size_t)rows[j], sl, LPR, C, reinterpret_cast<const uint32_t*>(xs4), acc[j]);
    // the row's sum is needed by the one lane that stores it: the group's last (group_sum_last)
    constexpr int LAST = LPR - 1;
    if constexpr (EPI == E_GLU) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float g = bfround(group_sum_last<LPR>(acc[0][m]));
            const float u = bfround(group_sum_last<LPR>(acc[RPW - 1][m]));
            const float sg = bfround(g / (1.f + expf(-g)));
            if (sl == LAST && outs[0] < Rout) y[(size_t)m * Rout + outs[0]] = f32_bf16(sg * u);
        }
    } else if constexpr (EPI == E_GLU_SPLIT) {
#pragma unroll
        for (int m = 0; m < M; ++m) {
            // the gate row's group is the lower neighbour of the up row's: the up group's last lane takes the gate's sum
            const float mine = group_sum_last<LPR>(acc[0][m]);
            const float g = bfround(from_lower_group<LPR>(mine)), u = bfround(mine);
            const float sg = bfround(g / (1.f + expf(-g)));
            if (sl == LAST && ((lane / LPR) & 1) == 1 && outs[0] < Rout) y[(size_t)m * Rout + outs[0]] = f32_bf16(sg * u);
        }
    } else {
#pragma unroll
        for (int j = 0; j < RPW; ++j)
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float s = group_sum_last<LPR>(acc[j][m]);
                if (sl == LAST && outs[j] < R) y[(size_t)m * R + outs[j]] = f32_bf16(s);
            }
    }
}

// The wave's first span of weights is requested while x is being staged - right after the staging's own loads have
// been issued, so those (served by L2) are not queued behind the weights: the weights do not depend on x, and their
// round trip to HBM overlaps the staging (for the add + norm form a block-wide sum and a second pass) instead of
// following it.
template <class F, int M, int LPR, int RPW, int U, int XMODE, int EPI, int NT = 256>
__global__ void __launch_bounds__(NT) gemv_stream(typename F::Params p, XArgs xa, uint16_t* __restrict__ y, int R, int C) {
    extern __shared__ __align__(16) uint32_t xs[];  // [M][C / 2] packed bf16 pairs
    static_assert(EPI != E_GLU || RPW == 2, "the GLU form pairs a gate row with an up row");
    static_assert(EPI != E_GLU_SPLIT || (RPW == 1 && LPR <= 32), "the split GLU form: gate and up in neighbouring row groups");
    constexpr int ROWS = tile_outputs<LPR, RPW, EPI>();
    const int Rout = EPI == E_PLAIN ? R : R / 2;
    const int units = C / F::UW;
    const int lane = threadIdx.x & (WAVE - 1);
    const int wave = blockIdx.x * (blockDim.x / WAVE) + (threadIdx.x / WAVE);
    const int nwaves = gridDim.x * (blockDim.x / WAVE);
    const int ntiles = (Rout + ROWS - 1) / ROWS;
    F::prepare(p);

    typename F::Raw first[U][RPW] = {};
    typename F::RowCtx first_ctx[RPW];
    stage_x<XMODE, M, sizeof(typename F::Raw) != 16, NT>(xs, xa, M, C, [&] {
        // a wave with no tile requests the last tile's span and drops it: nothing here is conditional (see
        // load_span_always)
#pragma unroll
        for (int j = 0; j < RPW; ++j) {
            int out_row;
            first_ctx[j] =
                F::row_ctx(p, (size_t)tile_row<LPR, RPW, EPI>(min(wave, ntiles - 1), j, lane, R, out_row), units,
                           lane % LPR);
        }
        load_span_always<F, LPR, RPW, U>(first, first_ctx, 0, lane % LPR, units);
        F::prepare_finish(p);
    });
    const uint4* xs4 = reinterpret_cast<const uint4*>(xs);
    if (wave >= ntiles) return;
    gemv_tile<F, M, LPR, RPW, U, EPI, true>(p, first, first_ctx, wave, xs4, y, R, C, lane);
    for (int tile = wave + nwaves; tile < ntiles; tile += nwaves)
        gemv_tile<F, M, LPR, RPW, U, EPI, false>(p, first, first_ctx, tile, xs4, y, R, C, lane);
}

// A bf16 row too long for one span of a wave (5121 .. 10240 values: more than ten 16-byte units a lane), by two waves:
// each takes a half of the row's units in one span, the second half's sum reaches the first half's wave through LDS.
// Twice the waves, each with one trip to memory where the whole row's wave made two - and 2560 such rows, 2.5 a SIMD,
// lie on the SIMDs as five halves each where whole rows lay three on some and two on others (a launch ends with its
// fullest SIMD): down [2560 x 9728] 10.15 -> 9.4 us, the step 1.993 -> 1.973 ms; the pass of 3 / 4 rows 2.575 / 2.780
// -> 2.403 / 2.667 ms. A workgroup's waves come in pairs, a row a pair and turn. The split comes from the row length
// alone and is the same at every M up to four, in every x mode and under the gate / up fold: a row's bits depend on
// none of them. Written over the format policy (what a form does past the stream is the first half's wave's), taken
// by bf16 only: pack12 rows of that length gain 0.4 % of the packed step at one row of x and 3 - 4 % of the pass at
// three and four, and lose 3.3 % at two (2.158 -> 2.230 ms), and every width has to take the same split.
// E_GLU: a pair of waves on gate row r, the next pair on up row I + r; the four sums meet in LDS and the up pair's
// first wave writes bf16(bf16(silu(g)) * u), g and u added up as the plain form adds them - the bits of the plain
// matvec followed by silu_mul.
template <class F, int M, int U, int XMODE, int EPI, int NT>
__global__ void __launch_bounds__(NT) gemv_halves(typename F::Params p, XArgs xa, uint16_t* __restrict__ y, int R, int C) {
    static_assert(EPI == E_PLAIN || EPI == E_GLU, "plain rows, or gate and up rows folded");
    static_assert(EPI == E_PLAIN || NT % (4 * WAVE) == 0, "the folded form: four waves an output");
    extern __shared__ __align__(16) uint32_t xs[];
    constexpr int NW = NT / WAVE;
    constexpr int OW = EPI == E_GLU ? NW / 4 : NW / 2;  // outputs a workgroup's turn
    __shared__ float part[2][NW][M];                    // [turn's parity][wave][row of x]: the waves' sums
    const int Rout = EPI == E_GLU ? R / 2 : R;
    const int units = C / F::UW;
    const int lane = threadIdx.x & (WAVE - 1), wib = threadIdx.x / WAVE;
    const int half = wib & 1;
    const int mine = EPI == E_GLU ? wib >> 2 : wib >> 1;  // the wave's output of the turn
    const bool up = EPI == E_GLU && (wib & 2) != 0;
    const int ua = (units + 1) / 2;  // the first half's units
    const int u0 = half ? ua : 0, u1 = half ? units : ua;
    const int xrow4 = C / 8;
    auto row_of = [&](int out) { return min(out, Rout - 1) + (up ? Rout : 0); };  // the weight row
    F::prepare(p);

    typename F::Raw first[U][1] = {};
    typename F::RowCtx ctx[1];
    stage_x<XMODE, M, sizeof(typename F::Raw) != 16, NT>(xs, xa, M, C, [&] {
        ctx[0] = F::row_ctx(p, (size_t)row_of((int)blockIdx.x * OW + mine), units, lane);
        load_span_always<F, WAVE, 1, U>(first, ctx, u0, lane, u1);
        F::prepare_finish(p);
    });
    const uint4* xs4 = reinterpret_cast<const uint4*>(xs);

    // a half is one span (U * 64 units hold it: launch_halves): the first turn's was requested above, a later turn
    // requests its own. The x values are read a unit at a time: asked for a span ahead, as the whole-row kernel does
    // at one row, they cost the registers that decide how many waves a SIMD holds.
    auto products = [&](const typename F::Raw (&raw)[U][1], float (&acc)[1][M]) {
#pragma unroll
        for (int u = 0; u < U; ++u) {
            const int unit = u0 + u * WAVE + lane;
            if (unit < u1) fma_unit<F, M, 1>(ctx, raw[u], unit, xs4, xrow4, acc);
        }
    };
    auto finish = [&](float (&acc)[1][M], int out, int parity) {
        if (half == 0) F::template tail<M>(p, ctx[0], (size_t)row_of(out), lane, WAVE, C, xs, acc[0]);
        float s[M];
#pragma unroll
        for (int m = 0; m < M; ++m) {
            s[m] = group_sum_last<WAVE>(acc[0][m]);
            if ((EPI == E_GLU || half == 1) && lane == WAVE - 1) part[parity][wib][m] = s[m];
        }
        __syncthreads();  // one a turn: the next turn writes the other parity's slots
        if (half == 0 && lane == WAVE - 1 && out < Rout && (EPI == E_PLAIN || up)) {
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float mine_sum = s[m] + part[parity][wib + 1][m];
                if constexpr (EPI == E_GLU) {
                    const float g = bfround(part[parity][wib - 2][m] + part[parity][wib - 1][m]), u = bfround(mine_sum);
                    const float sg = bfround(g / (1.f + expf(-g)));
                    y[(size_t)m * Rout + out] = f32_bf16(sg * u);
                } else {
                    y[(size_t)m * Rout + out] = f32_bf16(mine_sum);
                }
            }
        }
    };
    {
        float acc[1][M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[0][m] = 0.f;
        products(first, acc);
        finish(acc, blockIdx.x * OW + mine, 0);
    }
    int parity = 1;
    for (int base = (blockIdx.x + gridDim.x) * OW; base < Rout; base += gridDim.x * OW, parity ^= 1) {  // every wave alike
        ctx[0] = F::row_ctx(p, (size_t)row_of(base + mine), units, lane);
        typename F::Raw raw[U][1];
        load_span<F, WAVE, 1, U, true>(raw, ctx, u0, lane, u1);
        float acc[1][M];
#pragma unroll
        for (int m = 0; m < M; ++m) acc[0][m] = 0.f;
        products(raw, acc);
        finish(acc, base + mine, parity);
    }
}

// the row lengths gemv_halves takes
static bool halves_fit(int C) { return C > 5120 && C <= 10240 && tuning("gemv_halves") != 0; }

template <class F, int M, int XMODE, int EPI>
static int32_t launch_halves(const typename F::Params& p, const XArgs& xa, void* y, int R, int C, hipStream_t st) {
    const DeviceInfo& dev = device_info();
    const size_t lds = stage_lds_bytes(XMODE, M, C);
    if (lds > (size_t)dev.lds_bytes) {
        set_error("gemv: the x rows do not fit LDS");
        return ERR_DOMAIN;
    }
    // a half's units a lane: 6 to 10 of bf16 (spans of 8 or 10); the 16-weight forms' 3 to 5 would be a span of 5
    constexpr bool BF = std::is_same<F, FmtBf16>::value;
    const int half_lane = ((C / F::UW + 1) / 2 + WAVE - 1) / WAVE;
    // Ten waves a workgroup (five rows a turn) where x is copied as it is: 2560 rows are then two workgroups a CU, and
    // x is staged twice a CU, not five times (the bf16 pass of 2 / 3 / 4 rows with workgroups of four waves 2.28 /
    // 2.63 / 2.89 ms, of eight 2.20 / 2.46 / 2.66, of ten 2.17 / 2.40 / 2.67; one row level); eight for the folded
    // form, four waves an output. The other x modes are written for workgroups of 256 threads.
    constexpr int NT = XMODE != X_PLAIN ? 256 : EPI == E_GLU ? 512 : 640;
    constexpr int OW = EPI == E_GLU ? NT / (4 * WAVE) : NT / (2 * WAVE);
    const int Rout = EPI == E_GLU ? R / 2 : R;
    constexpr int LONGEST = BF ? 10 : 5;
    auto kern = BF && half_lane <= 8 ? gemv_halves<F, M, 8, XMODE, EPI, NT> : gemv_halves<F, M, LONGEST, XMODE, EPI, NT>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    int grid = (Rout + OW - 1) / OW;
    const int cap = dev.cus * 20 * WAVE / NT;  // twenty waves a CU and turn
    if (grid > cap) grid = cap;
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NT), lds, st, p, xa, static_cast<uint16_t*>(y), R, C);
    return hip_status(hipGetLastError(), "gemv_halves launch");
}

// ------------------------------------------------------------------------------------------------------------
// launch
// ------------------------------------------------------------------------------------------------------------

// lanes a row is summed by: from the row length alone, so a row's bits do not depend on M or on R
static int lanes_per_row(int units) {
    if (units % 64 == 0 || units >= 256) return 64;
    if (units % 32 == 0 || units >= 96) return 32;
    return 16;
}

template <class F, int M, int LPR, int RPW, int U, int XMODE, int EPI>
static int32_t launch_variant(const typename F::Params& p, const XArgs& xa, void* y, int R, int C, hipStream_t st) {
    constexpr int ROWS = tile_outputs<LPR, RPW, EPI>();
    const DeviceInfo& dev = device_info();
    const size_t lds = stage_lds_bytes(XMODE, M, C);
    if (lds > (size_t)dev.lds_bytes) {
        set_error("gemv: the x rows do not fit LDS");
        return ERR_DOMAIN;
    }
    // Every workgroup stages x once, so the grid is kept to a few workgroups a CU and each wave walks a whole number
    // of tiles (the last wave of the grid may walk fewer): tiles_per_wave is the smallest count that fits the cap.
    const int Rout = EPI == E_PLAIN ? R : R / 2;
    const int ntiles = (Rout + ROWS - 1) / ROWS;
    auto kern = gemv_stream<F, M, LPR, RPW, U, XMODE, EPI>;
    int per_cu = tuning("gemv_wgs_per_cu");
    // Six workgroups' worth of waves a CU, measured best for the plain forms (more, smaller workgroups than are resident
    // even out the grid's tail), five for the pack12 form with the pair table (the head matvec [151936 x 2560] 97 us
    // instead of 113), and four for the gate / up forms at one or two rows of x, whose waves then walk three tiles
    // instead of two: bf16 gate/up 17.55 -> 17.0 us and the step 2.022 -> 2.004 ms, packed 16.3 -> 15.5 us and
    // 1.928 -> 1.914 ms; at three rows the pass loses by it (2.58 -> 2.67 ms), and so does the plain one-row packed
    // [9728 x 2560] (8.25 -> 9.15 us).
    // One row of bf16 x with the add + norm in the x load, plain output (qkv, the head): two, which the even cut
    // below turns into one workgroup a CU whose waves walk three tiles each for qkv's 3072 - the add + norm is then
    // made once a CU, not three times side by side: qkv 7.36 -> 6.97 us, the step 1.967 -> 1.961 ms (the head level;
    // from two rows of x on and for the packed form it loses: 2.16 -> 2.21 ms at two rows, packed qkv 6.63 -> 7.42 us).
    constexpr bool BF16_NORM_ROW =
        std::is_same<F, FmtBf16>::value && M == 1 && XMODE == X_ADDNORM && EPI == E_PLAIN;
    if (per_cu <= 0)
        per_cu = BF16_NORM_ROW ? 2 : (EPI != E_PLAIN && M <= 2) ? 4 : std::is_same<F, FmtP12G>::value ? 5 : 6;
    const int cap_waves = dev.cus * per_cu * 4;
    // ... and of the counts from there to two more, the one whose workgroups fill the CUs' turns most evenly (when it
    // gains a twentieth or more): a launch ends with its fullest CU, and the forms that widen are bound by what a CU
    // computes (MXFP4 [18432 x 7168]: 1152 workgroups of 2 tiles a wave, 4.5 a CU, 15.7 us; 768 of 3, 3 a CU, 14.4).
    auto grid_of = [&](int tpw) { return ((ntiles + tpw - 1) / tpw + 3) / 4; };
    auto evenness = [&](int g) { return (double)g / (double)(((g + dev.cus - 1) / dev.cus) * dev.cus); };
    int tiles_per_wave = (ntiles + cap_waves - 1) / cap_waves;
    if (tuning("gemv_even_grid") != 0) {
        const int base = tiles_per_wave;
        for (int t = base + 1; t <= base + 2; ++t)
            if (evenness(grid_of(t)) >= evenness(grid_of(tiles_per_wave)) + 0.04) tiles_per_wave = t;
    }
    int grid = grid_of(tiles_per_wave);
    if (grid < 1) grid = 1;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    // One row of x, one tile a wave, plain: a launch is then a single turn over the CUs and ends with the CU that
    // holds the most waves. Workgroups of four waves put 2560 one-row tiles on the CUs as 640 workgroups, 12 waves on
    // half the CUs and 8 on the others; workgroups of five put 10 on each (a bf16 matrix of 2048 rows of 9728, which divides evenly, ran
    // at 8.1 us where 2304 rows took 10.1).
    if constexpr (M == 1 && XMODE == X_PLAIN && EPI == E_PLAIN) {
        const int waves = (ntiles + tiles_per_wave - 1) / tiles_per_wave;
        const int g5 = (waves + 4) / 5;
        // (measured: pack12 down 9.45 -> 8.45 us and o level, the packed step 1.910 -> 1.893 ms; bf16 o 5.28 -> 5.13 us
        // but down, whose rows are two spans, 10.1 -> 10.6: bf16 takes five waves only where a row is one span)
        constexpr bool WIDENS = sizeof(typename F::Raw) != 16;
        const bool suits = WIDENS || U * LPR >= C / F::UW;
        if (suits && tiles_per_wave == 1 && tuning("gemv_five_waves") != 0 && evenness(g5) >= evenness(grid) + 0.1) {
            auto kern5 = gemv_stream<F, M, LPR, RPW, U, XMODE, EPI, 320>;
            if (lds > 64 * 1024) {
                hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern5),
                                                   hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
                if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
            }
            hipLaunchKernelGGL(kern5, dim3(g5), dim3(320), lds, st, p, xa, static_cast<uint16_t*>(y), R, C);
            return hip_status(hipGetLastError(), "gemv launch");
        }
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(256), lds, st, p, xa, static_cast<uint16_t*>(y), R, C);
    return hip_status(hipGetLastError(), "gemv launch");
}

template <class F, int M, int LPR, int XMODE, int EPI>
static int32_t launch_stream(const typename F::Params& p, const XArgs& xa, void* y, int R, int C, hipStream_t st) {
    // Rows per wave tile (RPW) and units in flight per row (U), measured on MI355X. bf16 at M <= 2: two rows by four
    // units where the matrix has rows enough to give every SIMD several waves that way, else one row by eight. The
    // forms that widen in registers spend those registers on the widening, and run best with half the span and more
    // waves resident: one row by four (pack12, MXFP4), two rows by two (FP8, whose two rows share a scale fetch
    // pattern). Neither choice changes a result bit (a lane's units stay in ascending order).
    constexpr bool WIDENS = sizeof(typename F::Raw) != 16;  // everything but plain bf16
    // One bf16 row of x (the decode step proper): where a slightly longer span saves a whole round trip to memory - a
    // row of 5 units a lane read as 5, not 4 + 1; 19 as 10 + 9, not 8 + 8 + 3 - the span is stretched to 5 (10 for one
    // row a wave). The span of 5 at two rows of x as well (the bf16 pass of two rows 2.309 -> 2.2 ms, nearly all of it
    // the gate / up form's); at three rows it loses (2.59 -> 2.61).
    const int per_lane = (C / F::UW + LPR - 1) / LPR;
    auto fewer = [per_lane](int u_new, int u_base) { return (per_lane + u_new - 1) / u_new < (per_lane + u_base - 1) / u_base; };
    if constexpr (EPI == E_GLU) {
        // long bf16 rows (LPR is 64 there): the folded form of the split the plain form makes
        if constexpr (LPR == 64 && !WIDENS) {
            if (halves_fit(C)) return launch_halves<F, M, XMODE, E_GLU>(p, xa, y, R, C, st);
        }
        if constexpr (WIDENS && LPR <= 32) {
            // a widening form whose rows take at most 32 lanes: gate and up side by side, one row a lane
            if constexpr (M <= 4 && std::is_base_of<FmtP12, F>::value) {
                if (per_lane == 5) return launch_variant<F, M, LPR, 1, 5, XMODE, E_GLU_SPLIT>(p, xa, y, R, C, st);
            }
            return launch_variant<F, M, LPR, 1, 4, XMODE, E_GLU_SPLIT>(p, xa, y, R, C, st);
        } else if constexpr (WIDENS) {
            return launch_variant<F, M, LPR, 2, 2, XMODE, E_GLU>(p, xa, y, R, C, st);
        } else {
            if constexpr (M <= 2) {
                if (fewer(5, 4)) return launch_variant<F, M, LPR, 2, 5, XMODE, E_GLU>(p, xa, y, R, C, st);
            }
            return launch_variant<F, M, LPR, 2, (M <= 2 ? 4 : 2), XMODE, E_GLU>(p, xa, y, R, C, st);
        }
    } else if constexpr (WIDENS) {
        if constexpr (F::TWO_ROWS) {
            if constexpr (M == 1 && XMODE == X_PLAIN) {
                // One row of x over FP8: a lane's 5 to 8 units of a row asked for at once, one row a wave - one trip to
                // memory for the row instead of three or four spans of two units ([18432 x 7168], 7 units a lane:
                // 26.3 -> 24.4 us; two rows by four units 25.1, by three 25.4, one row by four 27.2).
                switch (per_lane) {
                    case 5: return launch_variant<F, M, LPR, 1, 5, XMODE, E_PLAIN>(p, xa, y, R, C, st);
                    case 6: return launch_variant<F, M, LPR, 1, 6, XMODE, E_PLAIN>(p, xa, y, R, C, st);
                    case 7: return launch_variant<F, M, LPR, 1, 7, XMODE, E_PLAIN>(p, xa, y, R, C, st);
                    case 8: return launch_variant<F, M, LPR, 1, 8, XMODE, E_PLAIN>(p, xa, y, R, C, st);
                    default: break;
                }
            }
            return launch_variant<F, M, LPR, 2, 2, XMODE, E_PLAIN>(p, xa, y, R, C, st);
        } else {
            // up to four rows of x over pack12 rows of five units a lane (2560 columns): the five at once, one trip for
            // the row where four and one were two (the one-row [9728 x 2560] 8.8 -> 8.3 us, qkv + norm 7.3 -> 6.9, the
            // packed pass of two / three rows 2.31 / 2.76 -> 2.18 / 2.65 ms; rows of four or ten units a lane lose by it:
            // o 5.06 -> 5.22, down 9.3 -> 9.4)
            if constexpr (M <= 4 && std::is_base_of<FmtP12, F>::value) {
                if (per_lane == 5) return launch_variant<F, M, LPR, 1, 5, XMODE, E_PLAIN>(p, xa, y, R, C, st);
            }
            return launch_variant<F, M, LPR, 1, 4, XMODE, E_PLAIN>(p, xa, y, R, C, st);
        }
    } else {
        if constexpr (LPR == 64) {
            if (halves_fit(C)) return launch_halves<F, M, XMODE, E_PLAIN>(p, xa, y, R, C, st);
        }
        const bool tall = R >= 4096 * (WAVE / LPR);
        if constexpr (M <= 2) {
            if (tall && fewer(5, 4)) return launch_variant<F, M, LPR, 2, 5, XMODE, E_PLAIN>(p, xa, y, R, C, st);
            if constexpr (M == 1) {
                if (!tall && fewer(10, 8)) return launch_variant<F, M, LPR, 1, 10, XMODE, E_PLAIN>(p, xa, y, R, C, st);
            }
            if (tall) return launch_variant<F, M, LPR, 2, 4, XMODE, E_PLAIN>(p, xa, y, R, C, st);
            return launch_variant<F, M, LPR, 1, 8, XMODE, E_PLAIN>(p, xa, y, R, C, st);
        } else {
            if (tall) return launch_variant<F, M, LPR, 2, 2, XMODE, E_PLAIN>(p, xa, y, R, C, st);
            return launch_variant<F, M, LPR, 1, 4, XMODE, E_PLAIN>(p, xa, y, R, C, st);
        }
    }
}

template <class F, int M, int XMODE, int EPI>
static int32_t launch_by_lanes(const typename F::Params& p, const XArgs& xa, void* y, int R, int C, hipStream_t st) {
    switch (lanes_per_row(C / F::UW)) {
        case 64:
            return launch_stream<F, M, 64, XMODE, EPI>(p, xa, y, R, C, st);
        case 32:
            return launch_stream<F, M, 32, XMODE, EPI>(p, xa, y, R, C, st);
        default:
            return launch_stream<F, M, 16, XMODE, EPI>(p, xa, y, R, C, st);
    }
}

template <class F, int XMODE, int EPI>
static int32_t launch_by_m(const typename F::Params& p, const XArgs& xa, void* y, int R, int C, int M, hipStream_t st) {
    switch (M) {
        case 1:
            return launch_by_lanes<F, 1, XMODE, EPI>(p, xa, y, R, C, st);
        case 2:
            return launch_by_lanes<F, 2, XMODE, EPI>(p, xa, y, R, C, st);
        case 3:
            return launch_by_lanes<F, 3, XMODE, EPI>(p, xa, y, R, C, st);
        case 4:
            return launch_by_lanes<F, 4, XMODE, EPI>(p, xa, y, R, C, st);
        default:
            return ERR_DOMAIN;
    }
}

// wider passes run as passes of at most four rows: each row's bits are those of its own one-row pass
template <class F, int XMODE, int EPI>
static int32_t run_rows(const typename F::Params& p, XArgs xa, void* y, size_t R, size_t C, size_t M, hipStream_t st) {
    const size_t x_row = XMODE == X_SILU ? 2 * C : C;
    const size_t y_row = EPI == E_GLU ? R / 2 : R;
    uint16_t* yp = static_cast<uint16_t*>(y);
    for (size_t m0 = 0; m0 < M; m0 += 4) {
        const int mm = (int)(M - m0 < 4 ? M - m0 : 4);
        int32_t rc = launch_by_m<F, XMODE, EPI>(p, xa, yp + m0 * y_row, (int)R, (int)C, mm, st);
        if (rc != OK) return rc;
        if (xa.ids != nullptr)
            xa.ids += 4;
        else
            xa.x += 4 * x_row;
        if (xa.y != nullptr) xa.y += 4 * C;
        if (xa.h_out != nullptr) xa.h_out += 4 * C;
    }
    return OK;
}

static XArgs plain_x(const void* x) { return XArgs{static_cast<const uint16_t*>(x), nullptr, nullptr, nullptr, 0.f, 0}; }

// the matrix-core forms of the matvec for the verify widths (gemv_mfma.hip, gemv_mfma_lds.hip)
int32_t gemv_mfma_bf16(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st);
bool mfma_lds_fits_bf16(int R, int C);
bool mfma_lds_fits_packed(int R, int C);
int32_t gemv_mfma_lds_bf16(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st);
int32_t gemv_mfma_lds_glu_bf16(const void* w, const void* x, void* y, int I, int C, int M, hipStream_t st);
bool mfma_lds_norm_fits(int R, int C, int M);
int32_t gemv_mfma_lds_norm_bf16(const void* w, const XArgs& xa, void* y, int R, int C, int M, int I, hipStream_t st);
int32_t gemv_mfma_lds_fp8(const void* w, const float* scales, int sc, int bm, int bn, const void* x, void* y, int R,
                          int C, int M, hipStream_t st);
int32_t gemv_mfma_lds_mxfp4(const void* blocks, const void* scales, const void* x, void* y, int R, int C, int M,
                            hipStream_t st);
int32_t gemv_mfma_lds_p12(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const int32_t* esc_idx,
                          const uint8_t* esc_val, const int32_t* row_ptr, const void* x, void* y, int R, int C, int M,
                          hipStream_t st);

// the direct-to-LDS form of the matrix-core matvec for the long rows of the block-scaled forms (gemv_mfma_dl.hip)
bool mfma_dl_fits(int R, int C, int M);
bool mfma_dl_fits_fp8(int R, int C, int M, int bm, int bn);
int32_t gemv_mfma_dl_fp8(const void* w, const float* scales, int sc, int bm, int bn, const void* x, void* y, int R,
                         int C, int M, hipStream_t st);
int32_t gemv_mfma_dl_mxfp4(const void* blocks, const void* scales, const void* x, void* y, int R, int C, int M,
                           hipStream_t st);
// and for pack12 rows of the lengths it has shapes for
bool mfma_dl_fits_p12(int R, int C, int M);
int32_t gemv_mfma_dl_p12(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const uint16_t* pairs,
                         const int32_t* esc_idx,
                         const uint8_t* esc_val, const int32_t* row_ptr, const void* x, void* y, int R, int C, int M,
                         hipStream_t st);

// whether a pass of M rows goes to the matrix cores through the LDS-staged kernel: from `from` rows on (the knob
// gemv_mfma_from, when set, replaces every form's own figure)
static bool wide_pass(size_t M, size_t R, size_t C, bool packed, size_t from = 5) {
    if (tuning("gemv_mfma_from") > 0) from = (size_t)tuning("gemv_mfma_from");
    return M >= from && (packed ? mfma_lds_fits_packed((int)R, (int)C) : mfma_lds_fits_bf16((int)R, (int)C)) &&
           tuning("gemv_no_mfma") <= 0 && tuning("mfma_lds") != 0;
}

// the block-scaled forms' vector kernels pay for every further row of x in LDS reads and in widening, the matrix-core
// kernels' time does not move up to 16 rows: on large matrices these take the pass earlier than at five rows
// (measured: MXFP4 [18432 x 7168] at 2 / 3 / 4 rows 23.6 / 30.0 / 37.8 us on the vector kernel, 19 us on the matrix
// cores; FP8 33.3 / 45.1 us at 3 / 4 rows against 30.7; under 4 M weights the vector kernel wins to four rows)
static size_t mx4_matrix_from(size_t R, size_t C) {
    const size_t n = R * C;
    return n >= (1u << 25) ? 2 : n >= (1u << 23) ? 3 : n >= (1u << 22) ? 4 : 5;
}
static size_t fp8_matrix_from(size_t R, size_t C) { return R * C >= (1u << 25) ? 3 : 5; }

static bool aligned16(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 15u) == 0; }
static bool aligned2(const void* p) { return (reinterpret_cast<uintptr_t>(p) & 1u) == 0; }

static int32_t check_dims(size_t R, size_t C, size_t M, size_t uw) {
    if (R == 0 || C == 0 || M == 0) return ERR_DOMAIN;
    if (R > 0x7FFFFFFFu / 4 || C > (1u << 24) || M > 1024 || C % uw != 0) return ERR_DOMAIN;
    return OK;
}

// the residual-and-norm arguments of the fused entry points, checked
static int32_t norm_args(const void* h_in, const void* y, const void* norm_w, float eps, int32_t centered, void* h_out,
                         XArgs* xa) {
    if (h_in == nullptr || norm_w == nullptr) return ERR_NULL;
    if (!(eps >= 0.f) || h_out == h_in) return ERR_DOMAIN;
    if (!aligned2(h_in) || !aligned2(y) || !aligned2(norm_w) || !aligned2(h_out)) return ERR_DOMAIN;
    *xa = XArgs{static_cast<const uint16_t*>(h_in), static_cast<const uint16_t*>(y),
                static_cast<const uint16_t*>(norm_w), static_cast<uint16_t*>(h_out), eps, centered ? 1 : 0};
    return OK;
}

// the arguments of the entry points whose residual is an embedding row per id
static int32_t embed_args(const void* table, const int32_t* ids, size_t vocab, const void* norm_w, float eps,
                          int32_t centered, void* h_out, XArgs* xa) {
    if (table == nullptr || ids == nullptr || norm_w == nullptr) return ERR_NULL;
    if (!(eps >= 0.f) || vocab == 0 || vocab > 0x7FFFFFFFull) return ERR_DOMAIN;
    if (!aligned16(table) || (reinterpret_cast<uintptr_t>(ids) & 3u) || !aligned2(norm_w) || !aligned2(h_out)) return ERR_DOMAIN;
    *xa = XArgs{static_cast<const uint16_t*>(table), nullptr, static_cast<const uint16_t*>(norm_w),
                static_cast<uint16_t*>(h_out), eps, centered ? 1 : 0, ids, (int)vocab};
    return OK;
}

// whether a matvec with the add + norm folded in goes to the matrix cores: a shape that kernel makes the rows for,
// every row of the residual stream a whole number of 8-byte words at an 8-byte boundary
static bool norm_on_mfma(const XArgs& xa, size_t R, size_t C, size_t M, bool glu) {
    auto al8 = [](const void* p) { return (reinterpret_cast<uintptr_t>(p) & 7u) == 0; };
    return tuning("gemv_no_mfma") <= 0 && tuning("mfma_lds") != 0 && C % 32 == 0 && (!glu || (R / 2) % 16 == 0) &&
           mfma_lds_norm_fits((int)R, (int)C, (int)M) && al8(xa.x) && al8(xa.y) && al8(xa.norm_w) && al8(xa.h_out);
}

static int32_t p12_params(const void* lo, const void* hi4, const void* table, const void* pairs, const void* esc_idx,
                          const void* esc_val, size_t n_esc, const void* row_ptr, const void* row_esc, size_t R,
                          size_t C, FmtP12::Params* p) {
    if (lo == nullptr || hi4 == nullptr || table == nullptr || row_ptr == nullptr) return ERR_NULL;
    if (reinterpret_cast<uintptr_t>(pairs) & 1u) return ERR_DOMAIN;
    if (n_esc > 0 && (esc_idx == nullptr || esc_val == nullptr)) return ERR_NULL;
    if (R * C > 0x7FFFFFFFull) return ERR_DOMAIN;  // the escape indices are int32
    if (!aligned16(lo) || (reinterpret_cast<uintptr_t>(hi4) & 7u) || (reinterpret_cast<uintptr_t>(row_ptr) & 3u) ||
        (reinterpret_cast<uintptr_t>(esc_idx) & 3u) || (reinterpret_cast<uintptr_t>(row_esc) & 3u))
        return ERR_DOMAIN;
    if (row_esc != nullptr && C > FmtP12::ROW_ESC_NONE) return ERR_DOMAIN;  // a word's column field
    *p = FmtP12::Params{static_cast<const uint8_t*>(lo),      static_cast<const uint8_t*>(hi4),
                        static_cast<const uint8_t*>(table),   static_cast<const int32_t*>(esc_idx),
                        static_cast<const uint8_t*>(esc_val), static_cast<const int32_t*>(row_ptr),
                        make_uint4(0, 0, 0, 0), static_cast<const uint16_t*>(pairs), 0u,
                        static_cast<const uint32_t*>(row_esc)};
    return OK;
}

}  // namespace btb

using namespace btb;

extern "C" {

int32_t btb_hip_gemv_bf16(const void* w, const void* x, void* y, size_t R, size_t C, size_t M, void* stream) {
    if (w == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    int32_t rc = check_dims(R, C, M, FmtBf16::UW);
    if (rc != OK) return rc;
    if (!aligned16(w) || !aligned16(x) || !aligned2(y)) return ERR_DOMAIN;
    // the verify widths go to the matrix cores, 32 rows of x a pass (from five rows on where the LDS-staged kernel takes
    // the shape: one pass there against two of the vector ALUs'); narrower passes stay on the vector ALUs
    if ((M >= 8 || wide_pass(M, R, C, false)) && C % 32 == 0 && tuning("gemv_no_mfma") <= 0) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 32) {
            const int mm = (int)(M - m0 < 32 ? M - m0 : 32);
            rc = wide_pass(M, R, C, false) ? gemv_mfma_lds_bf16(w, xp + m0 * C, yp + m0 * R, (int)R, (int)C, mm,
                                                      static_cast<hipStream_t>(stream))
                                 : gemv_mfma_bf16(w, xp + m0 * C, yp + m0 * R, (int)R, (int)C, mm,
                                                  static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    FmtBf16::Params p{static_cast<const uint4*>(w)};
    return run_rows<FmtBf16, X_PLAIN, E_PLAIN>(p, plain_x(x), y, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_silu_bf16(const void* w, const void* gu, void* y, size_t R, size_t C, size_t M, void* stream) {
    if (w == nullptr || gu == nullptr || y == nullptr) return ERR_NULL;
    int32_t rc = check_dims(R, C, M, FmtBf16::UW);
    if (rc != OK) return rc;
    if (!aligned16(w) || !aligned16(gu) || !aligned2(y)) return ERR_DOMAIN;
    FmtBf16::Params p{static_cast<const uint4*>(w)};
    return run_rows<FmtBf16, X_SILU, E_PLAIN>(p, plain_x(gu), y, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_glu_silu_bf16(const void* w, const void* x, void* m, size_t I, size_t C, size_t M, void* stream) {
    if (w == nullptr || x == nullptr || m == nullptr) return ERR_NULL;
    int32_t rc = check_dims(2 * I, C, M, FmtBf16::UW);
    if (rc != OK) return rc;
    if (!aligned16(w) || !aligned16(x) || !aligned2(m)) return ERR_DOMAIN;
    if (I % 16 == 0 && wide_pass(M, 2 * I, C, false)) {  // the verify widths: the matrix cores, 32 rows of x a pass
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* mp = static_cast<uint16_t*>(m);
        for (size_t m0 = 0; m0 < M; m0 += 32) {
            const int mm = (int)(M - m0 < 32 ? M - m0 : 32);
            rc = gemv_mfma_lds_glu_bf16(w, xp + m0 * C, mp + m0 * I, (int)I, (int)C, mm, static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    FmtBf16::Params p{static_cast<const uint4*>(w)};
    return run_rows<FmtBf16, X_PLAIN, E_GLU>(p, plain_x(x), m, 2 * I, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_bf16_norm(const void* w, const void* h_in, const void* y, const void* norm_w, float eps,
                               int32_t centered, void* h_out, void* out, size_t R, size_t C, size_t M, int32_t glu,
                               void* stream) {
    if (w == nullptr || out == nullptr) return ERR_NULL;
    XArgs xa;
    int32_t rc = norm_args(h_in, y, norm_w, eps, centered, h_out, &xa);
    if (rc != OK) return rc;
    rc = check_dims(R, C, M, FmtBf16::UW);
    if (rc != OK) return rc;
    if (!aligned16(w) || !aligned2(out) || (glu && R % 2 != 0)) return ERR_DOMAIN;
    FmtBf16::Params p{static_cast<const uint4*>(w)};
    hipStream_t st = static_cast<hipStream_t>(stream);
    // the verify widths: the matrix cores, the rows made by each workgroup ahead of its first tile
    if (norm_on_mfma(xa, R, C, M, glu != 0))
        return gemv_mfma_lds_norm_bf16(w, xa, out, (int)R, (int)C, (int)M, glu ? (int)(R / 2) : 0, st);
    return glu ? run_rows<FmtBf16, X_ADDNORM, E_GLU>(p, xa, out, R, C, M, st)
               : run_rows<FmtBf16, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, st);
}

int32_t btb_hip_gemv_bf16_embed_norm(const void* w, const void* table, const int32_t* ids, size_t vocab,
                                     const void* norm_w, float eps, int32_t centered, void* h_out, void* out, size_t R,
                                     size_t C, size_t M, void* stream) {
    if (w == nullptr || out == nullptr) return ERR_NULL;
    XArgs xa;
    int32_t rc = embed_args(table, ids, vocab, norm_w, eps, centered, h_out, &xa);
    if (rc != OK) return rc;
    rc = check_dims(R, C, M, FmtBf16::UW);
    if (rc != OK) return rc;
    if (!aligned16(w) || !aligned2(out)) return ERR_DOMAIN;
    FmtBf16::Params p{static_cast<const uint4*>(w)};
    if (norm_on_mfma(xa, R, C, M, false))
        return gemv_mfma_lds_norm_bf16(w, xa, out, (int)R, (int)C, (int)M, 0, static_cast<hipStream_t>(stream));
    return run_rows<FmtBf16, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_p12(const void* lo, const void* hi4, const void* table, const void* pairs, const void* esc_idx,
                         const void* esc_val, size_t n_esc, const void* row_ptr, const void* row_esc, const void* x,
                         void* y, size_t R, size_t C, size_t M, void* stream) {
    if (x == nullptr || y == nullptr || lo == nullptr || hi4 == nullptr || table == nullptr || row_ptr == nullptr)
        return ERR_NULL;
    if (n_esc > 0 && (esc_idx == nullptr || esc_val == nullptr)) return ERR_NULL;
    int32_t rc = check_dims(R, C, M, FmtP12::UW);
    if (rc != OK) return rc;
    FmtP12::Params p;
    rc = p12_params(lo, hi4, table, pairs, esc_idx, esc_val, n_esc, row_ptr, row_esc, R, C, &p);
    if (rc != OK) return rc;
    if (!aligned16(x) || !aligned2(y)) return ERR_DOMAIN;
    // the verify widths: the matrix cores. Weights straight into LDS, 16 rows of x a pass, where that kernel has a
    // shape for the row length
    if (wide_pass(M, R, C, true) && aligned16(hi4) && aligned16(lo) && (reinterpret_cast<uintptr_t>(table) & 3u) == 0 &&
        mfma_dl_fits_p12((int)R, (int)C, 16)) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 16) {
            const int mm = (int)(M - m0 < 16 ? M - m0 : 16);
            rc = gemv_mfma_dl_p12(p.lo, p.hi4, p.table, p.pairs, p.esc_idx, p.esc_val, p.row_ptr, xp + m0 * C, yp + m0 * R, (int)R,
                                  (int)C, mm, static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    if (wide_pass(M, R, C, true) && aligned16(hi4)) {  // through registers and LDS, 32 rows of x a pass
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 32) {
            const int mm = (int)(M - m0 < 32 ? M - m0 : 32);
            rc = gemv_mfma_lds_p12(p.lo, p.hi4, p.table, p.esc_idx, p.esc_val, p.row_ptr, xp + m0 * C, yp + m0 * R,
                                   (int)R, (int)C, mm, static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    // The lookups go through the pair table in LDS where the caller has one (made at upload; 1.5 vector instructions
    // a weight against the in-register lookup's 3.4). While an escape still cost a launch three trips to memory at
    // its end, a launch of one tile a wave did better with the lookup in registers (o [2560 x 4096] 5.62 against
    // 6.35 us); with the rows' words the table wins or draws at every shape of the step (down [2560 x 9728] 9.3
    // against 9.6 us, o level). The knob p12_pair_table forces either (1 / 0).
    const int knob = tuning("p12_pair_table");
    if (pairs != nullptr && knob != 0)
        return run_rows<FmtP12G, X_PLAIN, E_PLAIN>(p, plain_x(x), y, R, C, M, static_cast<hipStream_t>(stream));
    return run_rows<FmtP12, X_PLAIN, E_PLAIN>(p, plain_x(x), y, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_p12_norm(const void* lo, const void* hi4, const void* table, const void* pairs,
                              const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                              const void* row_esc, const void* h_in, const void* y,
                              const void* norm_w, float eps, int32_t centered, void* h_out, void* out, size_t R,
                              size_t C, size_t M, int32_t glu, void* stream) {
    if (out == nullptr) return ERR_NULL;
    FmtP12::Params p;
    XArgs xa;
    int32_t rc = norm_args(h_in, y, norm_w, eps, centered, h_out, &xa);
    if (rc == ERR_NULL) return rc;
    const int32_t rp = p12_params(lo, hi4, table, pairs, esc_idx, esc_val, n_esc, row_ptr, row_esc, R, C, &p);
    if (rp == ERR_NULL) return rp;
    if (rc != OK) return rc;
    if (rp != OK) return rp;
    rc = check_dims(R, C, M, FmtP12::UW);
    if (rc != OK) return rc;
    if (!aligned2(out) || (glu && R % 2 != 0)) return ERR_DOMAIN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (pairs != nullptr && tuning("p12_pair_table") != 0)
        return glu ? run_rows<FmtP12G, X_ADDNORM, E_GLU>(p, xa, out, R, C, M, st)
                   : run_rows<FmtP12G, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, st);
    return glu ? run_rows<FmtP12, X_ADDNORM, E_GLU>(p, xa, out, R, C, M, st)
               : run_rows<FmtP12, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, st);
}

int32_t btb_hip_gemv_p12_embed_norm(const void* lo, const void* hi4, const void* table, const void* pairs,
                                    const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                                    const void* row_esc, const void* embed,
                                    const int32_t* ids, size_t vocab, const void* norm_w, float eps, int32_t centered,
                                    void* h_out, void* out, size_t R, size_t C, size_t M, void* stream) {
    if (out == nullptr) return ERR_NULL;
    FmtP12::Params p;
    XArgs xa;
    int32_t rc = embed_args(embed, ids, vocab, norm_w, eps, centered, h_out, &xa);
    if (rc == ERR_NULL) return rc;
    const int32_t rp = p12_params(lo, hi4, table, pairs, esc_idx, esc_val, n_esc, row_ptr, row_esc, R, C, &p);
    if (rp == ERR_NULL) return rp;
    if (rc != OK) return rc;
    if (rp != OK) return rp;
    rc = check_dims(R, C, M, FmtP12::UW);
    if (rc != OK) return rc;
    if (!aligned2(out)) return ERR_DOMAIN;
    if (pairs != nullptr && tuning("p12_pair_table") != 0)
        return run_rows<FmtP12G, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, static_cast<hipStream_t>(stream));
    return run_rows<FmtP12, X_ADDNORM, E_PLAIN>(p, xa, out, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_fp8(const void* w, const void* scales, size_t sr, size_t sc, const void* x, void* y, size_t R,
                         size_t C, size_t M, void* stream) {
    if (w == nullptr || scales == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (sr == 0 || sc == 0) return ERR_DOMAIN;
    int32_t rc = check_dims(R, C, M, FmtF8::UW);
    if (rc != OK) return rc;
    if (R % sr != 0 || C % sc != 0 || (C / sc) % FmtF8::UW != 0) return ERR_DOMAIN;
    if (!aligned16(w) || !aligned16(x) || (reinterpret_cast<uintptr_t>(scales) & 3u) || !aligned2(y)) return ERR_DOMAIN;
    const size_t from = fp8_matrix_from(R, C);
    if (wide_pass(M, R, C, true, from) && mfma_dl_fits_fp8((int)R, (int)C, 16, (int)(R / sr), (int)(C / sc))) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);  // the long rows: weights straight into LDS, 16 rows a pass
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 16) {
            const int mm = (int)(M - m0 < 16 ? M - m0 : 16);
            rc = gemv_mfma_dl_fp8(w, static_cast<const float*>(scales), (int)sc, (int)(R / sr), (int)(C / sc), xp + m0 * C,
                                  yp + m0 * R, (int)R, (int)C, mm, static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    if (wide_pass(M, R, C, true, from)) {  // the verify widths: the matrix cores, 32 rows of x a pass
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 32) {
            const int mm = (int)(M - m0 < 32 ? M - m0 : 32);
            rc = gemv_mfma_lds_fp8(w, static_cast<const float*>(scales), (int)sc, (int)(R / sr), (int)(C / sc),
                                   xp + m0 * C, yp + m0 * R, (int)R, (int)C, mm, static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    const uint32_t upb = (uint32_t)(C / sc / FmtF8::UW);
    FmtF8::Params p{static_cast<const uint8_t*>(w), static_cast<const float*>(scales), (int)sc, (int)(R / sr),
                    (int)upb, upb > 1 ? (uint32_t)(0x100000000ull / upb + 1) : 0u};
    return run_rows<FmtF8, X_PLAIN, E_PLAIN>(p, plain_x(x), y, R, C, M, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_mxfp4(const void* blocks, const void* scales, const void* x, void* y, size_t R, size_t C, size_t M,
                           void* stream) {
    if (blocks == nullptr || scales == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    int32_t rc = check_dims(R, C, M, FmtMx4::UW);
    if (rc != OK) return rc;
    if (!aligned16(blocks) || !aligned16(x) || !aligned2(y)) return ERR_DOMAIN;
    const size_t from = mx4_matrix_from(R, C);
    if (wide_pass(M, R, C, true, from) && mfma_dl_fits((int)R, (int)C, 16) &&
        (reinterpret_cast<uintptr_t>(scales) & 3u) == 0) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);  // the long rows: weights straight into LDS, 16 rows a pass
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 16) {
            const int mm = (int)(M - m0 < 16 ? M - m0 : 16);
            rc = gemv_mfma_dl_mxfp4(blocks, scales, xp + m0 * C, yp + m0 * R, (int)R, (int)C, mm,
                                    static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    if (wide_pass(M, R, C, true, from)) {
        const uint16_t* xp = static_cast<const uint16_t*>(x);
        uint16_t* yp = static_cast<uint16_t*>(y);
        for (size_t m0 = 0; m0 < M; m0 += 32) {
            const int mm = (int)(M - m0 < 32 ? M - m0 : 32);
            rc = gemv_mfma_lds_mxfp4(blocks, scales, xp + m0 * C, yp + m0 * R, (int)R, (int)C, mm,
                                     static_cast<hipStream_t>(stream));
            if (rc != OK) return rc;
        }
        return OK;
    }
    FmtMx4::Params p{static_cast<const uint8_t*>(blocks), static_cast<const uint8_t*>(scales)};
    return run_rows<FmtMx4, X_PLAIN, E_PLAIN>(p, plain_x(x), y, R, C, M, static_cast<hipStream_t>(stream));
}

}  // extern "C"
