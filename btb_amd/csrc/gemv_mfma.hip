// The skinny matmul of the speculative-verify widths (M = 8..32 rows of x) on the matrix cores:
// y[m][r] = sum_c W[r][c] * x[m][c], bf16 in, f32 accumulate, bf16 out. Still memory-bound (every weight byte is read
// once); the MFMA only keeps the vector ALUs free, which at M >= 8 could no longer keep up with the stream.
//
// One v_mfma_f32_16x16x32_bf16 multiplies a 16-row x 32-column tile of W (operand A: lane l holds row l % 16, columns
// 8 * (l / 16) .. + 7, one 16-byte load) by the same 32 columns of 16 rows of x (operand B, the same lane layout over
// x's rows) into a 16 x 16 f32 tile (lane l: x row l % 16, W rows 4 * (l / 16) .. + 3). A workgroup owns RT * 16 rows
// of W; its four waves split the columns in interleaved 128-column chunks and fold their partial tiles through LDS in
// wave order 0, 1, 2, 3, so a row's bits depend on neither M nor the launch. The reference's counterpart is
// btb_gemv_mma_bf16 (native/cuda/btb_gemv_mma.cuh:1-214).

#include "btb_common.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

constexpr int KC = 128;  // columns a wave covers per step: four MFMAs deep

// MT: 16-row tiles of x (1: M <= 16, 2: M <= 32); RT: 16-row tiles of W per workgroup
template <int MT, int RT>
__global__ void __launch_bounds__(256) gemv_mfma_kernel(const uint4* __restrict__ w, const uint4* __restrict__ x,
                                                        uint16_t* __restrict__ y, int R, int C, int M) {
    __shared__ f32x4 part[3][RT][MT][WAVE];  // the partial tiles of waves 1..3
    const int lane = threadIdx.x & (WAVE - 1);
    const int wv = threadIdx.x / WAVE;
    const int li = lane & 15, lg = lane >> 4;
    const int chunk4 = C / 8;  // uint4 per row
    const int r0 = blockIdx.x * (RT * 16);

    const uint4* arow[RT];
#pragma unroll
    for (int t = 0; t < RT; ++t) {
        const int r = min(r0 + t * 16 + li, R - 1);  // a row past the end reads the last row and is not written
        arow[t] = w + (size_t)r * chunk4 + lg;
    }
    const uint4* brow[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) brow[t] = x + (size_t)min(t * 16 + li, M - 1) * chunk4 + lg;

    f32x4 acc[RT][MT];
#pragma unroll
    for (int a = 0; a < RT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b) acc[a][b] = f32x4{0.f, 0.f, 0.f, 0.f};

    // wave wv takes the 128-column chunks wv, wv + 4, ...; a chunk is four 32-column MFMA steps
    for (int c0 = wv * KC; c0 < C; c0 += 4 * KC) {
        uint4 av[RT][4], bv[MT][4];
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const int col = c0 + s * 32;  // C is a multiple of 32: a step is whole or absent
            const bool on = col < C;
#pragma unroll
            for (int t = 0; t < RT; ++t) av[t][s] = on ? load_stream16(arow[t] + col / 8) : make_uint4(0, 0, 0, 0);
#pragma unroll
            for (int t = 0; t < MT; ++t) bv[t][s] = on ? brow[t][col / 8] : make_uint4(0, 0, 0, 0);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s)
#pragma unroll
            for (int a = 0; a < RT; ++a)
#pragma unroll
                for (int b = 0; b < MT; ++b)
                    acc[a][b] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, av[a][s]),
                                                                        __builtin_bit_cast(bf16x8, bv[b][s]),
                                                                        acc[a][b], 0, 0, 0);
    }
    if (wv > 0) {
#pragma unroll
        for (int a = 0; a < RT; ++a)
#pragma unroll
            for (int b = 0; b < MT; ++b) part[wv - 1][a][b][lane] = acc[a][b];
    }
    __syncthreads();
    if (wv != 0) return;
#pragma unroll
    for (int a = 0; a < RT; ++a)
#pragma unroll
        for (int b = 0; b < MT; ++b) {
            f32x4 s = acc[a][b];
#pragma unroll
            for (int q = 0; q < 3; ++q) {
                const f32x4 o = part[q][a][b][lane];
                s.x += o.x;
                s.y += o.y;
                s.z += o.z;
                s.w += o.w;
            }
            const int m = b * 16 + li;
            const int row = r0 + a * 16 + lg * 4;
            if (m < M) {
                uint16_t* o = y + (size_t)m * R + row;
                if (row + 0 < R) o[0] = f32_bf16(s.x);
                if (row + 1 < R) o[1] = f32_bf16(s.y);
                if (row + 2 < R) o[2] = f32_bf16(s.z);
                if (row + 3 < R) o[3] = f32_bf16(s.w);
            }
        }
}

// ------------------------------------------------------------------------------------------------------------
// The same product with x held still. A workgroup of KS waves owns 16 rows of W at a time; wave k owns a fixed slice
// of the columns - `spw` consecutive 32-column MFMA steps - and keeps the x fragments of that slice (operand B of every
// step) in its registers for the whole kernel, so x is read once per wave instead of once per row tile. The
// workgroup then walks row tiles (blockIdx.x, + gridDim.x, ...): each wave streams its slice of the tile's 16 rows
// (a contiguous run of up to 1280 bytes a row), multiplies, and the KS partial tiles fold through LDS in wave order.
// KS and the slices come from C alone, so a row's bits depend on neither M nor R nor the launch. A second tile of x
// rows (M > 16) takes its fragments from memory (L2) step by step, with the same column slices and fold order: rows
// 0..15 keep the bits they have at M <= 16.
// ------------------------------------------------------------------------------------------------------------
constexpr int XS_SPW = 20;  // steps a wave can hold x for: KS * 20 * 32 >= C

template <int KS, int MT, int AB>
__global__ void __launch_bounds__(KS * 64) gemv_mfma_xs(const uint4* __restrict__ w, const uint4* __restrict__ x,
                                                        uint16_t* __restrict__ y, int R, int C, int M) {
    __shared__ f32x4 part[KS][MT][WAVE];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wv = threadIdx.x / WAVE;
    const int li = lane & 15, lg = lane >> 4;
    const int chunk4 = C / 8;  // uint4 per row
    const int nsteps = C / 32;
    const int spw = (nsteps + KS - 1) / KS;
    const int s0 = wv * spw;
    const int n = max(min(s0 + spw, nsteps) - s0, 0);  // this wave's steps: s0 .. s0 + n - 1

    const uint4* xr0 = x + (size_t)min(li, M - 1) * chunk4 + lg + (size_t)s0 * 4;
    const uint4* xr1 = x + (size_t)min(16 + li, M - 1) * chunk4 + lg + (size_t)s0 * 4;
    uint4 xb[XS_SPW];
#pragma unroll
    for (int i = 0; i < XS_SPW; ++i) xb[i] = i < n ? xr0[i * 4] : make_uint4(0, 0, 0, 0);

    const int from = 4 * (4 * li + lg);  // the lane (as a byte address) whose loaded piece this lane multiplies
    const int ntiles = (R + 15) / 16;
    for (int tile = blockIdx.x; tile < ntiles; tile += gridDim.x) {
        // The 64 bytes a row contributes to a step are loaded by four neighbouring lanes (lane 4 r + p: row r, piece
        // p), so the memory pipeline sees sixteen 64-byte runs per load instead of sixty-four scattered 16-byte pieces;
        // a cross-lane permute then hands every piece to the lane the MFMA wants it in (lane r + 16 p).
        const int r = min(tile * 16 + (lane >> 2), R - 1);  // a row past the end reads the last row and is not written
        const uint4* ar = w + (size_t)r * chunk4 + (lane & 3) + (size_t)s0 * 4;
        f32x4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
        for (int i0 = 0; i0 < XS_SPW; i0 += AB) {
            if (i0 < n) {
                uint4 a[AB], b1[AB];
#pragma unroll
                for (int j = 0; j < AB; ++j) {
                    const bool on = i0 + j < n;
                    a[j] = on ? load_stream16(ar + (i0 + j) * 4) : make_uint4(0, 0, 0, 0);
                    if (MT == 2) b1[j] = on ? xr1[(i0 + j) * 4] : make_uint4(0, 0, 0, 0);
                }
#pragma unroll
                for (int j = 0; j < AB; ++j) {
                    if (i0 + j < XS_SPW) {
                        a[j].x = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)a[j].x);
                        a[j].y = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)a[j].y);
                        a[j].z = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)a[j].z);
                        a[j].w = (uint32_t)__builtin_amdgcn_ds_bpermute(from, (int)a[j].w);
                        acc[0] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[j]),
                                                                         __builtin_bit_cast(bf16x8, xb[i0 + j < XS_SPW ? i0 + j : 0]),
                                                                         acc[0], 0, 0, 0);
                        if (MT == 2)
                            acc[MT - 1] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(bf16x8, a[j]),
                                                                                  __builtin_bit_cast(bf16x8, b1[j]),
                                                                                  acc[MT - 1], 0, 0, 0);
                    }
                }
            }
        }
#pragma unroll
        for (int t = 0; t < MT; ++t) part[wv][t][lane] = acc[t];
        __syncthreads();
        if (wv < MT) {
            f32x4 s = part[0][wv][lane];
            for (int q = 1; q < KS; ++q) {
                const f32x4 o = part[q][wv][lane];
                s.x += o.x;
                s.y += o.y;
                s.z += o.z;
                s.w += o.w;
            }
            const int m = wv * 16 + li;
            const int row = tile * 16 + lg * 4;
            if (m < M) {
                uint16_t* o = y + (size_t)m * R + row;
                if (row + 0 < R) o[0] = f32_bf16(s.x);
                if (row + 1 < R) o[1] = f32_bf16(s.y);
                if (row + 2 < R) o[2] = f32_bf16(s.z);
                if (row + 3 < R) o[3] = f32_bf16(s.w);
            }
        }
        __syncthreads();
    }
}

template <int KS, int MT, int AB>
static int32_t launch_xs(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    const int ntiles = (R + 15) / 16;
    int per_cu = tuning("mfma_wgs_per_cu");
    if (per_cu <= 0) per_cu = KS >= 8 ? 1 : 3;  // what the registers leave resident
    const int cap = device_info().cus * per_cu;
    // whole turns of the grid over the tiles: the grid is the smallest that walks them in ceil(ntiles / cap) turns
    const int turns = (ntiles + cap - 1) / cap;
    const int grid = (ntiles + turns - 1) / turns;
    hipLaunchKernelGGL((gemv_mfma_xs<KS, MT, AB>), dim3(grid), dim3(KS * 64), 0, st, static_cast<const uint4*>(w),
                       static_cast<const uint4*>(x), static_cast<uint16_t*>(y), R, C, M);
    return hip_status(hipGetLastError(), "gemv_mfma launch");
}

template <int MT>
static int32_t launch_mfma(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    // 32 rows a workgroup where that still leaves every CU a few workgroups, else 16
    const bool tall = R >= 32 * 4 * device_info().cus;
    if (tall) {
        hipLaunchKernelGGL((gemv_mfma_kernel<MT, 2>), dim3((R + 31) / 32), dim3(256), 0, st,
                           static_cast<const uint4*>(w), static_cast<const uint4*>(x), static_cast<uint16_t*>(y), R, C,
                           M);
    } else {
        hipLaunchKernelGGL((gemv_mfma_kernel<MT, 1>), dim3((R + 15) / 16), dim3(256), 0, st,
                           static_cast<const uint4*>(w), static_cast<const uint4*>(x), static_cast<uint16_t*>(y), R, C,
                           M);
    }
    return hip_status(hipGetLastError(), "gemv_mfma launch");
}

// M = 5..32 and C a multiple of 32: the caller (gemv.hip) checks both before it comes here. Rows up to 5120 wide
// take the x-stationary kernel, with as few waves per row tile as can hold x for the row's length (measured 3-15 %
// ahead of the column-interleaved kernel at the Qwen3-4B shapes); wider rows would need sixteen waves a tile, which
// the register file does not hold with x resident, and stay with the column-interleaved kernel.
int32_t gemv_mfma_bf16(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    const int nsteps = C / 32;
    if (nsteps <= 8 * XS_SPW && tuning("mfma_classic") <= 0) {
        if (M <= 16) {
            if (nsteps <= 4 * XS_SPW) return launch_xs<4, 1, 10>(w, x, y, R, C, M, st);
            return launch_xs<8, 1, 10>(w, x, y, R, C, M, st);
        }
        if (nsteps <= 4 * XS_SPW) return launch_xs<4, 2, 5>(w, x, y, R, C, M, st);
        return launch_xs<8, 2, 5>(w, x, y, R, C, M, st);
    }
    return M <= 16 ? launch_mfma<1>(w, x, y, R, C, M, st) : launch_mfma<2>(w, x, y, R, C, M, st);
}

}  // namespace btb
