// The host matvec's bits on the GPU: the device twins of the reference crate's CPU entry points, f32 x and y, every
// output computed in exactly the CPU's order so the result is bit-identical to btb_gemv_*_rows on the host
// (native/src/gemv.rs:84-123, 45-58). Sixteen lanes work on a row: lane j runs the columns = j (mod 16) in ascending
// order, one fused multiply-add each, and the sixteen lane sums fold pairwise ((l0+l1)+(l2+l3))+... - the same
// tree as the host's reduce16, since every step adds the two halves of an aligned group. The reference's card has the
// same pair of kernels for bf16 and MXFP4 (btb_gemv_lane16_f32_m*, btb_gemv_lane16_mx4_f32_m*:
// native/cuda/btb_kernels.cu:1635-1766); here all four stored forms have one, each weight made by the scalar
// definition of btb_widen.hpp. These are the parity and routing kernels (the router's logits must be the CPU's, bit
// for bit, for the top-k picks to be); the bandwidth path is gemv.hip.

#include <algorithm>
#include <type_traits>

#include "btb_common.hpp"
#include "btb_route.hpp"
#include "btb_tuning.hpp"
#include "btb_widen.hpp"

#include "../../include/btb_hip.h"

namespace btb {

struct W16Bf16 {
    const uint16_t* w;
    __device__ __forceinline__ float at(size_t r, size_t c, size_t cols) const { return bf16_f32(w[r * cols + c]); }
};

struct W16P12 {
    const uint8_t* lo;
    const uint8_t* hi4;
    const uint8_t* table;
    const int32_t* esc_idx;
    const uint8_t* esc_val;
    size_t n_esc;
    __device__ __forceinline__ float at(size_t r, size_t c, size_t cols) const {
        const size_t i = r * cols + c;
        const uint8_t byte = hi4[i >> 1];
        const unsigned code = (i & 1) ? (byte >> 4) : (byte & 0x0F);
        uint32_t hi = table[code];
        if (code == 15u && n_esc != 0) {
            // an escaped weight: its high byte is in the list, found by its index
            size_t a = 0, b = n_esc;
            while (a < b) {
                const size_t m = a + (b - a) / 2;
                if ((size_t)esc_idx[m] < i)
                    a = m + 1;
                else
                    b = m;
            }
            if (a < n_esc && (size_t)esc_idx[a] == i) hi = esc_val[a];
        }
        return bits_f32((hi << 24) | ((uint32_t)lo[i] << 16));
    }
};

struct W16Mx4 {
    const uint8_t* blocks;
    const uint8_t* scales;
    __device__ __forceinline__ float at(size_t r, size_t c, size_t cols) const {
        const size_t i = r * cols + c;
        const size_t g = i >> 5;
        const unsigned k = (unsigned)(i & 31);
        return mx4_weight(blocks[g * 16 + (k >> 1)], (int)(k & 1), scales[g]);
    }
};

// the same weights in ggml's layout (a GGUF's): 17-byte blocks, the e8m0 scale first, then 16 bytes whose low nibbles are
// weights 0..15 and high nibbles 16..31 (native/src/gemv.rs:1034-1078)
struct W16Mx4Ggml {
    const uint8_t* raw;
    __device__ __forceinline__ float at(size_t r, size_t c, size_t cols) const {
        const size_t i = r * cols + c;
        const uint8_t* blk = raw + (i >> 5) * 17;
        const unsigned k = (unsigned)(i & 31);
        return mx4_weight(blk[1 + (k & 15)], (int)(k >> 4), blk[0]);
    }
};

struct W16F8 {
    const uint8_t* w;
    const float* scales;
    size_t sc, bm, bn;
    __device__ __forceinline__ float at(size_t r, size_t c, size_t cols) const {
        return f8_held(w[r * cols + c], scales[(r / bm) * sc + c / bn]);
    }
};

// x is f32, or bf16 widened on the way in (exact, so the sums are those of the widened copy)
__device__ __forceinline__ float x_at(const float* x, size_t i) { return x[i]; }
__device__ __forceinline__ float x_at(const uint16_t* x, size_t i) { return bf16_f32(x[i]); }

// B rows of x per pass (the host walks up to 8 at a time; the order within one (row, vector) pair is the same)
template <class W, int B, class XT>
__global__ void __launch_bounds__(256) lane16_kernel(W w, const XT* __restrict__ x, float* __restrict__ y, size_t rows,
                                                     size_t cols, size_t b0, size_t btotal) {
    const int j = threadIdx.x & 15;
    const size_t r = (size_t)blockIdx.x * (blockDim.x >> 4) + (threadIdx.x >> 4);
    const bool live = r < rows;
    const size_t rr = live ? r : rows - 1;
    float acc[B];
#pragma unroll
    for (int i = 0; i < B; ++i) acc[i] = 0.f;
    // a batch of the lane's columns: their loads are issued together, the products then taken in column order
    constexpr int UB = B == 1 ? 32 : 8;
    size_t c = (size_t)j;
    for (; c + 16 * (UB - 1) < cols; c += 16 * UB) {
        float wv[UB], xv[UB][B];
#pragma unroll
        for (int u = 0; u < UB; ++u) {
            wv[u] = w.at(rr, c + 16 * u, cols);
#pragma unroll
            for (int i = 0; i < B; ++i) xv[u][i] = b0 + i < btotal ? x_at(x, (b0 + i) * cols + c + 16 * u) : 0.f;
        }
#pragma unroll
        for (int u = 0; u < UB; ++u)
#pragma unroll
            for (int i = 0; i < B; ++i)
                if (b0 + i < btotal) acc[i] = fmaf(wv[u], xv[u][i], acc[i]);
    }
    for (; c < cols; c += 16) {
        const float wv = w.at(rr, c, cols);
#pragma unroll
        for (int i = 0; i < B; ++i) {
            if (b0 + i < btotal) acc[i] = fmaf(wv, x_at(x, (b0 + i) * cols + c), acc[i]);
        }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
        const float s = group_sum<16>(acc[i]);
        if (j == 0 && live && b0 + i < btotal) y[(b0 + i) * rows + r] = s;
    }
}

// bf16 rows 128 columns wide a step: the group's sixteen lanes bring 256 contiguous bytes in with one 16-byte load each
// and hand them round through a slab of LDS the group owns, where lane j then finds its columns j, j + 16, ... - one
// request a lane for eight of its columns instead of eight. x is staged once a workgroup, as f32. The sums are the same
// chain of fused multiply-adds in the same column order. Writes and reads of a slab are one wave's, which LDS serves in
// program order: no barrier between them.
template <int B, int NB, class XT>
__global__ void __launch_bounds__(256) lane16_bf16_wide_kernel(const uint16_t* __restrict__ w, const XT* __restrict__ x,
                                                               float* __restrict__ y, size_t rows, size_t cols, size_t b0,
                                                               size_t btotal) {
    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int BP = B == 3 ? 4 : B;  // a column's B values of x side by side, one LDS read
    float* xs = reinterpret_cast<float*>(smem);           // [cols][BP]
    unsigned char* slabs = smem + (size_t)BP * cols * 4;  // [16 groups][NB][256]
    b0 += (size_t)blockIdx.y * B;
    const int tid = threadIdx.x, j = tid & 15, grp = tid >> 4;
    const size_t r = (size_t)blockIdx.x * 16 + grp;
    const bool live = r < rows;
    const uint4* wrow = reinterpret_cast<const uint4*>(w + (live ? r : rows - 1) * cols);
    const int nchunks = (int)(cols / 128);
    // a compiler vector, not HIP's uint4: an array of the struct type that lives across the loop below is kept in scratch
    // memory - written there as soon as it is loaded, which waits for the loads at once - and a vector's is not
    u32x4 raw[NB];
    auto request = [&](int n0) {
#pragma unroll
        for (int n = 0; n < NB; ++n)
            raw[n] = *reinterpret_cast<const u32x4*>(wrow + (size_t)min(n0 + n, nchunks - 1) * 16 + j);
    };
    request(0);
    // x in 16-byte pieces (rows are 16-byte aligned: cols is a multiple of 128), every piece of every row requested
    // before the first is spread out
    constexpr int PER = 16 / (int)sizeof(XT);  // values a piece
    const size_t pieces = cols / PER;
#pragma unroll
    for (int b = 0; b < B; ++b) {
        const bool have = b0 + b < btotal;
        const uint4* src = reinterpret_cast<const uint4*>(x + (have ? b0 + b : b0) * cols);
        for (size_t i = tid; i < pieces; i += 256) {
            const uint4 v = src[i];
            const uint32_t d[4] = {v.x, v.y, v.z, v.w};
            float* dst = xs + i * PER * BP + b;
#pragma unroll
            for (int e = 0; e < PER; ++e) {
                float f;
                if (sizeof(XT) == 4)
                    f = bits_f32(d[e]);
                else
                    f = (e & 1) ? bf16hi_f32(d[e >> 1]) : bf16lo_f32(d[e >> 1]);
                dst[e * BP] = have ? f : 0.f;
            }
        }
    }
    __syncthreads();
    unsigned char* mine = slabs + (size_t)grp * (NB * 256);
    float acc[B];
#pragma unroll
    for (int i = 0; i < B; ++i) acc[i] = 0.f;
    for (int n0 = 0; n0 < nchunks; n0 += NB) {
#pragma unroll
        for (int n = 0; n < NB; ++n) *reinterpret_cast<u32x4*>(mine + n * 256 + 16 * j) = raw[n];
        if (n0 + NB < nchunks) request(n0 + NB);
#pragma unroll
        for (int n = 0; n < NB; ++n) {
            if (n0 + n < nchunks) {
#pragma unroll
                for (int u = 0; u < 8; ++u) {
                    const float wv = bf16_f32(*reinterpret_cast<const uint16_t*>(mine + n * 256 + 2 * (j + 16 * u)));
                    const size_t c = (size_t)(n0 + n) * 128 + j + 16 * u;
#pragma unroll
                    for (int i = 0; i < B; ++i) acc[i] = fmaf(wv, xs[c * BP + i], acc[i]);
                }
            }
        }
    }
#pragma unroll
    for (int i = 0; i < B; ++i) {
        const float s = group_sum<16>(acc[i]);
        if (j == 0 && live && b0 + i < btotal) y[(b0 + i) * rows + r] = s;
    }
}

template <int B, int NB, class XT>
static bool launch_wide(const uint16_t* w, const XT* x, float* y, size_t rows, size_t cols, size_t b0, size_t b,
                        unsigned passes, hipStream_t st) {
    const size_t lds = (size_t)(B == 3 ? 4 : B) * cols * 4 + 16 * NB * 256;  // x, the slabs
    if (lds > (size_t)device_info().lds_bytes) return false;
    auto kern = lane16_bf16_wide_kernel<B, NB, XT>;
    static bool raised = false;  // per instance; the attribute is the function's, set before its first large launch
    if (lds > 64 * 1024 && !raised) {
        if (hipFuncSetAttribute(reinterpret_cast<const void*>(kern), hipFuncAttributeMaxDynamicSharedMemorySize,
                                device_info().lds_bytes) != hipSuccess)
            return false;
        raised = true;
    }
    hipLaunchKernelGGL(kern, dim3((unsigned)((rows + 15) / 16), passes), dim3(256), lds, st, w, x, y, rows, cols, b0, b);
    return true;
}

template <class W, class XT>
static int32_t launch_lane16(const W& w, const XT* x, float* y, size_t rows, size_t cols, size_t b, hipStream_t st) {
    const unsigned grid = (unsigned)((rows + 15) / 16);
    size_t b0 = 0;
    if constexpr (std::is_same<W, W16Bf16>::value) {
        if (cols % 128 == 0 && ((reinterpret_cast<uintptr_t>(w.w) | reinterpret_cast<uintptr_t>(x)) & 15) == 0) {
            // every pass of four rows of x in one launch (the pass is the grid's second dimension), then the rest
            bool done = true;
            // A few rows of x against a small matrix (a router at the verify widths): a pass a row, all in one launch.
            // The matrix is re-read once a row out of L2, but every row's sums start at once, where passes of four
            // rows take four times the arithmetic each behind a fourfold staging (8 rows against the 128 x 2048
            // router: 13.2 -> 8.9 us). A (row, vector) sum is the same chain of operations in every form.
            if (b > 1 && b <= 16 && rows * cols <= (1u << 20)) {
                done = launch_wide<1, 16>(w.w, x, y, rows, cols, 0, b, (unsigned)b, st);
                if (done) b0 = b;
            }
            const size_t fours = b0 < b ? std::min<size_t>(b / 4, 65535) : 0;
            if (fours > 0) {
                // few rows of weights (a router): every step of a row asked for at once, as the one-row pass does
                done = rows <= 1024 && launch_wide<4, 16>(w.w, x, y, rows, cols, 0, b, (unsigned)fours, st);
                if (!done) done = launch_wide<4, 4>(w.w, x, y, rows, cols, 0, b, (unsigned)fours, st);
                if (done) b0 = 4 * fours;
            }
            while (done && b0 < b) {
                const size_t left = b - b0;
                if (left >= 4) {
                    done = launch_wide<4, 4>(w.w, x, y, rows, cols, b0, b, 1, st);
                    if (done) b0 += 4;
                } else {
                    done = left >= 2 ? launch_wide<3, 4>(w.w, x, y, rows, cols, b0, b, 1, st)
                                     : launch_wide<1, 16>(w.w, x, y, rows, cols, b0, b, 1, st);
                    if (done) b0 = b;
                }
            }
            int32_t rc = hip_status(hipGetLastError(), "lane16 launch");
            if (rc != OK) return rc;
        }
    }
    for (; b0 < b; b0 += 4) {
        const size_t left = b - b0;
        if (left >= 4)
            hipLaunchKernelGGL((lane16_kernel<W, 4, XT>), dim3(grid), dim3(256), 0, st, w, x, y, rows, cols, b0, b);
        else if (left >= 2)
            hipLaunchKernelGGL((lane16_kernel<W, 3, XT>), dim3(grid), dim3(256), 0, st, w, x, y, rows, cols, b0, b);
        else
            hipLaunchKernelGGL((lane16_kernel<W, 1, XT>), dim3(grid), dim3(256), 0, st, w, x, y, rows, cols, b0, b);
        int32_t rc = hip_status(hipGetLastError(), "lane16 launch");
        if (rc != OK) return rc;
    }
    return OK;
}

static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

// the crate's shape rule (native/src/gemv.rs:4216-4222), with the grid's 2^31 limit on rows / 16
static bool shape_ok(size_t rows, size_t cols, size_t b) {
    const size_t cap = (size_t)INTPTR_MAX / 4;
    size_t n;
    if (__builtin_mul_overflow(rows, cols, &n) || n > cap) return false;
    if (__builtin_mul_overflow(b, cols, &n) || n > cap) return false;
    if (__builtin_mul_overflow(b, rows, &n) || n > cap) return false;
    return rows / 16 < 0x7FFFFFFFull;
}

// the router's logits from the rows as they are held (bf16): the f32 copy the host path makes first is the widening
// done in the load
int32_t lane16_bf16_rows16(const uint16_t* w, size_t rows, size_t cols, const uint16_t* x, size_t b, float* y,
                           hipStream_t st) {
    if (!shape_ok(rows, cols, b)) return ERR_DOMAIN;
    return launch_lane16(W16Bf16{w}, x, y, rows, cols, b, st);
}

}  // namespace btb

using namespace btb;

extern "C" {

int32_t btb_hip_gemv_bf16_rows(const uint16_t* w, size_t rows, size_t cols, const float* x, size_t b, float* y,
                               void* stream) {
    if (w == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0) return ERR_DOMAIN;
    if (!shape_ok(rows, cols, b) || !al(w, 2) || !al(x, 4) || !al(y, 4)) return ERR_DOMAIN;
    return launch_lane16(W16Bf16{w}, x, y, rows, cols, b, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_bf16_group(size_t n, const uint16_t* const* w, const size_t* rows, const size_t* cols,
                                const float* const* x, const size_t* b, float* const* y, void* stream) {
    if (w == nullptr || rows == nullptr || cols == nullptr || x == nullptr || b == nullptr || y == nullptr)
        return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    // every task is checked before the first is launched: a refused call launches nothing
    for (size_t t = 0; t < n; ++t) {
        if (w[t] == nullptr || x[t] == nullptr || y[t] == nullptr) return ERR_NULL;
        if (rows[t] == 0 || cols[t] == 0 || b[t] == 0) return ERR_DOMAIN;
        if (!shape_ok(rows[t], cols[t], b[t]) || !al(w[t], 2) || !al(x[t], 4) || !al(y[t], 4)) return ERR_DOMAIN;
    }
    for (size_t t = 0; t < n; ++t) {
        int32_t rc = launch_lane16(W16Bf16{w[t]}, x[t], y[t], rows[t], cols[t], b[t], static_cast<hipStream_t>(stream));
        if (rc != OK) return rc;
    }
    return OK;
}

int32_t btb_hip_gemv_p12_rows(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const int32_t* esc_idx,
                              const uint8_t* esc_val, size_t n_esc, size_t rows, size_t cols, const float* x, size_t b,
                              float* y, void* stream) {
    if (lo == nullptr || hi4 == nullptr || table == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (n_esc > 0 && (esc_idx == nullptr || esc_val == nullptr)) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0) return ERR_DOMAIN;
    if (!shape_ok(rows, cols, b) || !al(x, 4) || !al(y, 4)) return ERR_DOMAIN;
    if (n_esc > 0 && (n_esc > rows * cols || !al(esc_idx, 4))) return ERR_DOMAIN;
    // the list's order is the caller's to keep on the device (the host entry point walks it; here that would be a
    // copy back): an index absent from the list leaves the table's byte in place
    return launch_lane16(W16P12{lo, hi4, table, esc_idx, esc_val, n_esc}, x, y, rows, cols, b,
                         static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_mxfp4_rows(const uint8_t* blocks, const uint8_t* scales, size_t rows, size_t cols, const float* x,
                                size_t b, float* y, void* stream) {
    if (blocks == nullptr || scales == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0 || cols % 32 != 0 || !shape_ok(rows, cols, b) || !al(x, 4) || !al(y, 4))
        return ERR_DOMAIN;
    return launch_lane16(W16Mx4{blocks, scales}, x, y, rows, cols, b, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_mxfp4_ggml_rows(const uint8_t* raw, size_t rows, size_t cols, const float* x, size_t b, float* y,
                                     void* stream) {
    if (raw == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0 || cols % 32 != 0 || !shape_ok(rows, cols, b) || !al(x, 4) || !al(y, 4))
        return ERR_DOMAIN;
    return launch_lane16(W16Mx4Ggml{raw}, x, y, rows, cols, b, static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_mxfp4_group(size_t n, const uint8_t* const* blocks, const uint8_t* const* scales,
                                 const size_t* rows, const size_t* cols, const float* const* x, const size_t* b,
                                 float* const* y, void* stream) {
    if (blocks == nullptr || scales == nullptr || rows == nullptr || cols == nullptr || x == nullptr || b == nullptr ||
        y == nullptr)
        return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    for (size_t t = 0; t < n; ++t) {
        if (blocks[t] == nullptr || scales[t] == nullptr || x[t] == nullptr || y[t] == nullptr) return ERR_NULL;
        if (rows[t] == 0 || cols[t] == 0 || b[t] == 0 || cols[t] % 32 != 0 || !shape_ok(rows[t], cols[t], b[t]) ||
            !al(x[t], 4) || !al(y[t], 4))
            return ERR_DOMAIN;
    }
    for (size_t t = 0; t < n; ++t) {
        int32_t rc = launch_lane16(W16Mx4{blocks[t], scales[t]}, x[t], y[t], rows[t], cols[t], b[t],
                                   static_cast<hipStream_t>(stream));
        if (rc != OK) return rc;
    }
    return OK;
}

int32_t btb_hip_gemv_fp8_rows(const uint8_t* w, const float* scales, size_t rows, size_t cols, size_t sr, size_t sc,
                              const float* x, size_t b, float* y, void* stream) {
    if (w == nullptr || scales == nullptr || x == nullptr || y == nullptr) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0 || sr == 0 || sc == 0) return ERR_DOMAIN;
    if (rows % sr != 0 || cols % sc != 0 || !shape_ok(rows, cols, b) || !al(scales, 4) || !al(x, 4) || !al(y, 4))
        return ERR_DOMAIN;
    return launch_lane16(W16F8{w, scales, sc, rows / sr, cols / sc}, x, y, rows, cols, b,
                         static_cast<hipStream_t>(stream));
}

int32_t btb_hip_gemv_fp8_group(size_t n, const uint8_t* const* w, const float* const* scales, const size_t* rows,
                               const size_t* cols, const size_t* sr, const size_t* sc, const float* const* x,
                               const size_t* b, float* const* y, void* stream) {
    if (w == nullptr || scales == nullptr || rows == nullptr || cols == nullptr || sr == nullptr || sc == nullptr ||
        x == nullptr || b == nullptr || y == nullptr)
        return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    for (size_t t = 0; t < n; ++t) {
        if (w[t] == nullptr || scales[t] == nullptr || x[t] == nullptr || y[t] == nullptr) return ERR_NULL;
        if (rows[t] == 0 || cols[t] == 0 || b[t] == 0 || sr[t] == 0 || sc[t] == 0) return ERR_DOMAIN;
        if (rows[t] % sr[t] != 0 || cols[t] % sc[t] != 0 || !shape_ok(rows[t], cols[t], b[t]) || !al(scales[t], 4) ||
            !al(x[t], 4) || !al(y[t], 4))
            return ERR_DOMAIN;
    }
    for (size_t t = 0; t < n; ++t) {
        int32_t rc = launch_lane16(W16F8{w[t], scales[t], sc[t], rows[t] / sr[t], cols[t] / sc[t]}, x[t], y[t], rows[t],
                                   cols[t], b[t], static_cast<hipStream_t>(stream));
        if (rc != OK) return rc;
    }
    return OK;
}

}  // extern "C"
