// The widenings on their own: packed bytes to bf16 (or f32) in memory. The decode path never runs these - the
// matvec widens in registers - they exist (a) so the in-register widen of every stored form can be checked bit for
// bit against the CPU definitions, through the very policy code the matvec uses (btb_formats.hpp), and (b) as the
// reference's btb_mx4_widen operator (native/cuda/btb_kernels.cu:710-738), which a caller may still launch by name.
// Also here: the per-row escape offsets of a pack12 matrix, built once when it is uploaded.

#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

// one thread a unit of 16 weights; the tail (n % 16 weights) takes the scalar definition
__global__ void __launch_bounds__(256) p12_widen_kernel(FmtP12::Params p, size_t n, uint16_t* __restrict__ out) {
    const size_t unit = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    const size_t units = n / FmtP12::UW;
    if (unit < units) {
        FmtP12::RowCtx c;
        c.lo = reinterpret_cast<const uint4*>(p.lo);
        c.hi4 = reinterpret_cast<const uint2*>(p.hi4);
        c.table = FmtP12::load_table(p.table);
        c.e0 = c.e1 = 0;
        // plain (cached) loads: the matvec's own stream is non-temporal, the bytes are the same
        FmtP12::Raw raw{c.lo[unit], c.hi4[unit]};
        uint32_t packed[FmtP12::UW / 2];
        FmtP12::widen(c, raw, 0, packed);
        uint4* o = reinterpret_cast<uint4*>(out) + unit * 2;
        o[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        o[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    } else if (unit == units) {
        for (size_t i = units * FmtP12::UW; i < n; ++i) out[i] = p12_plain_bits(p.lo, p.hi4, p.table, i);
    }
}

// the escapes written over the widened tensor: out[esc_idx[k]] = esc_val[k] << 8 | lo
__global__ void __launch_bounds__(256) p12_patch_kernel(const uint8_t* __restrict__ lo, const int32_t* __restrict__ esc_idx,
                                                        const uint8_t* __restrict__ esc_val, size_t n_esc, size_t n,
                                                        uint16_t* __restrict__ out) {
    const size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_esc) return;
    const int32_t at = esc_idx[k];
    if (at < 0 || (size_t)at >= n) return;  // a list btb_hip_p12_check would refuse: never a write outside the tensor
    const size_t i = (size_t)at;
    out[i] = (uint16_t)(((uint32_t)esc_val[k] << 8) | lo[i]);
}

// *bad |= 1 unless the list is strictly ascending inside [0, n): entry k against its left neighbour
__global__ void __launch_bounds__(256) p12_check_kernel(const int32_t* __restrict__ esc_idx, size_t n_esc, size_t n,
                                                        int32_t* __restrict__ bad) {
    const size_t k = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_esc) return;
    const int32_t v = esc_idx[k];
    const bool ok = v >= 0 && (size_t)v < n && (k == 0 || esc_idx[k - 1] < v);
    if (!ok) atomicOr(bad, 1);
}

// row_ptr[r] = the number of escapes below r * cols: a binary search per row over the ascending list
__global__ void __launch_bounds__(256) p12_row_ptr_kernel(const int32_t* __restrict__ esc_idx, size_t n_esc, size_t rows,
                                                          size_t cols, int32_t* __restrict__ row_ptr) {
    const size_t r = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (r > rows) return;
    const size_t start = r * cols;
    size_t a = 0, b = n_esc;
    while (a < b) {
        const size_t m = a + (b - a) / 2;
        if ((size_t)esc_idx[m] < start)
            a = m + 1;
        else
            b = m;
    }
    row_ptr[r] = (int32_t)a;
}

// one thread a unit of 16 weights of an FP8 matrix; OUT_F32 keeps the f32 that holds the bf16 value
template <bool OUT_F32>
__global__ void __launch_bounds__(256) fp8_widen_kernel(FmtF8::Params p, int R, int C, void* __restrict__ out) {
    const int units = C / FmtF8::UW;
    const size_t t = (size_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (t >= (size_t)R * units) return;
    const size_t r = t / units;
    const int unit = (int)(t - r * units);
    const FmtF8::RowCtx c = FmtF8::row_ctx(p, r, units);
    const int blk = c.upb == 1 ? unit : (int)__umulhi((uint32_t)unit, c.magic);
    FmtF8::Raw raw{c.row[unit], c.srow[blk]};
    uint32_t packed[FmtF8::UW / 2];
    FmtF8::widen(c, raw, unit, packed);
    if (OUT_F32) {
        float4* o = reinterpret_cast<float4*>(out) + t * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k)
            o[k] = make_float4(bf16lo_f32(packed[2 * k]), bf16hi_f32(packed[2 * k]), bf16lo_f32(packed[2 * k + 1]),
                               bf16hi_f32(packed[2 * k + 1]));
    } else {
        uint4* o = reinterpret_cast<uint4*>(out) + t * 2;
        o[0] = make_uint4(packed[0], packed[1], packed[2], packed[3]);
        o[1] = make_uint4(packed[4], packed[5], packed[6], packed[7]);
    }
}

// one thread a block of 32 weights: fp4 * 2^(s - 127) as bf16 (the reference card's btb_mx4_widen; exact for every
// scale below 255), or with OUT_F32 the same values as f32 (the CPU matvec's weight). `seats` picks
// the stacks (experts) to widen, or is null for the identity.
template <bool OUT_F32>
__global__ void __launch_bounds__(256) mx4_widen_kernel(FmtMx4::Params p, const int32_t* __restrict__ seats,
                                                        long long groups, void* __restrict__ out) {
    const long long g = (long long)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= groups) return;
    const long long seat = seats != nullptr ? (long long)seats[blockIdx.y] : (long long)blockIdx.y;
    const long long at = seat * groups + g;
    FmtMx4::RowCtx c{reinterpret_cast<const uint4*>(p.blocks), p.scales};
    FmtMx4::Raw raw{c.row[at], (uint32_t)c.srow[at]};
    uint32_t packed[FmtMx4::UW / 2];
    FmtMx4::widen(c, raw, 0, packed);
    FmtMx4::patch255(raw, packed);
    const long long o0 = (long long)blockIdx.y * groups + g;
    if (OUT_F32) {
        float4* o = reinterpret_cast<float4*>(out) + o0 * 8;
#pragma unroll
        for (int k = 0; k < 8; ++k)
            o[k] = make_float4(bf16lo_f32(packed[2 * k]), bf16hi_f32(packed[2 * k]), bf16lo_f32(packed[2 * k + 1]),
                               bf16hi_f32(packed[2 * k + 1]));
    } else {
        uint4* o = reinterpret_cast<uint4*>(out) + o0 * 4;
#pragma unroll
        for (int k = 0; k < 4; ++k) o[k] = make_uint4(packed[4 * k], packed[4 * k + 1], packed[4 * k + 2], packed[4 * k + 3]);
    }
}

static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace btb

using namespace btb;

namespace btb {
// f32 values rounded to stored bf16 by the library's own f32_bf16, a thread a value
__global__ void __launch_bounds__(256) round_bf16_kernel(const float* __restrict__ x, uint16_t* __restrict__ out, size_t n) {
    const size_t i = (size_t)blockIdx.x * 256 + threadIdx.x;
    if (i < n) out[i] = f32_bf16(x[i]);
}
}  // namespace btb

// entry b of the pair table: the high bytes of the two weights whose codes are byte b's nibbles (the earlier weight
// the low nibble, its high byte the entry's low byte); slot 15 - the escape code - counts as 0 whatever the table says
__global__ void __launch_bounds__(256) p12_pairs_kernel(const uint8_t* __restrict__ table, uint16_t* __restrict__ pairs) {
    const uint32_t b = threadIdx.x;
    const uint32_t c0 = b & 15u, c1 = b >> 4;
    const uint32_t h0 = c0 == 15u ? 0u : table[c0], h1 = c1 == 15u ? 0u : table[c1];
    pairs[b] = (uint16_t)(h0 | (h1 << 8));
}

extern "C" {

// a row's first 8 or 16 escapes as words of the row's own (FmtP12::row_escapes reads them, FmtP12::tail uses them)
__global__ void __launch_bounds__(256) p12_row_esc_kernel(const uint8_t* __restrict__ lo, const int32_t* __restrict__ esc_idx,
                                                          const uint8_t* __restrict__ esc_val,
                                                          const int32_t* __restrict__ row_ptr, int rows, int cols,
                                                          uint32_t* __restrict__ out) {
    const int r = blockIdx.x * 256 + threadIdx.x;
    if (r >= rows) return;
    const int e0 = row_ptr[r], e1 = row_ptr[r + 1];
    const int slots = FmtP12::row_esc_slots(cols);
    const uint32_t more = e1 - e0 > slots ? 0x80000000u : 0u;
    for (int k = 0; k < slots; ++k) {
        uint32_t w = FmtP12::ROW_ESC_NONE << 16;
        if (e0 + k < e1) {
            const size_t i = (size_t)esc_idx[e0 + k];
            w = (uint32_t)lo[i] | ((uint32_t)esc_val[e0 + k] << 8) | ((uint32_t)(i - (size_t)r * cols) << 16);
        }
        out[(size_t)r * slots + k] = w | more;
    }
}

int32_t btb_hip_p12_row_esc(const void* lo, const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                            size_t rows, size_t cols, void* row_esc, void* stream) {
    if (lo == nullptr || row_ptr == nullptr || row_esc == nullptr) return ERR_NULL;
    if (n_esc > 0 && (esc_idx == nullptr || esc_val == nullptr)) return ERR_NULL;
    if (rows == 0 || cols == 0 || cols > FmtP12::ROW_ESC_NONE || rows * cols > 0x7FFFFFFFull) return ERR_DOMAIN;
    if (!al(esc_idx, 4) || !al(row_ptr, 4) || !al(row_esc, 4)) return ERR_DOMAIN;
    hipLaunchKernelGGL(p12_row_esc_kernel, dim3((unsigned)((rows + 255) / 256)), dim3(256), 0,
                       static_cast<hipStream_t>(stream), static_cast<const uint8_t*>(lo),
                       static_cast<const int32_t*>(esc_idx), static_cast<const uint8_t*>(esc_val),
                       static_cast<const int32_t*>(row_ptr), (int)rows, (int)cols, static_cast<uint32_t*>(row_esc));
    return hip_status(hipGetLastError(), "p12_row_esc launch");
}

int32_t btb_hip_p12_pairs(const void* table, void* pairs, void* stream) {
    if (table == nullptr || pairs == nullptr) return ERR_NULL;
    if (!al(pairs, 2)) return ERR_DOMAIN;
    hipLaunchKernelGGL(p12_pairs_kernel, dim3(1), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint8_t*>(table), static_cast<uint16_t*>(pairs));
    return hip_status(hipGetLastError(), "p12_pairs launch");
}

int32_t btb_hip_p12_row_ptr(const void* esc_idx, size_t n_esc, size_t rows, size_t cols, void* row_ptr, void* stream) {
    if (row_ptr == nullptr || (n_esc > 0 && esc_idx == nullptr)) return ERR_NULL;
    if (rows == 0 || cols == 0 || rows > 0x7FFFFFFEull || cols > 0x7FFFFFFFull || rows * cols > 0x7FFFFFFFull ||
        n_esc > rows * cols)
        return ERR_DOMAIN;
    if (!al(esc_idx, 4) || !al(row_ptr, 4)) return ERR_DOMAIN;
    const unsigned grid = (unsigned)((rows + 1 + 255) / 256);
    hipLaunchKernelGGL(p12_row_ptr_kernel, dim3(grid), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const int32_t*>(esc_idx), n_esc, rows, cols, static_cast<int32_t*>(row_ptr));
    return hip_status(hipGetLastError(), "p12_row_ptr launch");
}

int32_t btb_hip_p12_check(const void* esc_idx, size_t n_esc, size_t n, int32_t* flag, void* stream) {
    if (n_esc == 0) return n == 0 || n > 0x7FFFFFFFull ? ERR_DOMAIN : OK;
    if (esc_idx == nullptr || flag == nullptr) return ERR_NULL;
    if (n == 0 || n > 0x7FFFFFFFull || n_esc > n || !al(esc_idx, 4) || !al(flag, 4)) return ERR_DOMAIN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    hipError_t e = hipMemsetAsync(flag, 0, sizeof(int32_t), st);
    if (e != hipSuccess) return hip_status(e, "p12_check clear");
    hipLaunchKernelGGL(p12_check_kernel, dim3((unsigned)((n_esc + 255) / 256)), dim3(256), 0, st,
                       static_cast<const int32_t*>(esc_idx), n_esc, n, flag);
    int32_t rc = hip_status(hipGetLastError(), "p12_check launch");
    if (rc != OK) return rc;
    int32_t bad = 0;
    e = hipMemcpyAsync(&bad, flag, sizeof(int32_t), hipMemcpyDeviceToHost, st);
    if (e == hipSuccess) e = hipStreamSynchronize(st);
    if (e != hipSuccess) return hip_status(e, "p12_check read-back");
    if (bad != 0) {
        set_error("p12_check: the escape list is not strictly ascending inside [0, n)");
        return ERR_DOMAIN;
    }
    return OK;
}

int32_t btb_hip_p12_widen(const void* lo, const void* hi4, const void* table, const void* esc_idx, const void* esc_val,
                          size_t n_esc, size_t n, void* out, void* stream) {
    if (lo == nullptr || hi4 == nullptr || table == nullptr || out == nullptr) return ERR_NULL;
    if (n_esc > 0 && (esc_idx == nullptr || esc_val == nullptr)) return ERR_NULL;
    if (n == 0 || n > 0x7FFFFFFFull || n_esc > n) return ERR_DOMAIN;
    if (!al(lo, 16) || !al(hi4, 8) || !al(out, 16) || !al(esc_idx, 4)) return ERR_DOMAIN;
    hipStream_t st = static_cast<hipStream_t>(stream);
    FmtP12::Params p{static_cast<const uint8_t*>(lo),      static_cast<const uint8_t*>(hi4),
                     static_cast<const uint8_t*>(table),   static_cast<const int32_t*>(esc_idx),
                     static_cast<const uint8_t*>(esc_val), nullptr, make_uint4(0, 0, 0, 0), nullptr, 0u, nullptr};
    const size_t threads = n / FmtP12::UW + 1;
    hipLaunchKernelGGL(p12_widen_kernel, dim3((unsigned)((threads + 255) / 256)), dim3(256), 0, st, p, n,
                       static_cast<uint16_t*>(out));
    int32_t rc = hip_status(hipGetLastError(), "p12_widen launch");
    if (rc != OK || n_esc == 0) return rc;
    hipLaunchKernelGGL(p12_patch_kernel, dim3((unsigned)((n_esc + 255) / 256)), dim3(256), 0, st,
                       static_cast<const uint8_t*>(lo), static_cast<const int32_t*>(esc_idx),
                       static_cast<const uint8_t*>(esc_val), n_esc, n, static_cast<uint16_t*>(out));
    return hip_status(hipGetLastError(), "p12_patch launch");
}

int32_t btb_hip_fp8_widen(const void* w, const void* scales, size_t rows, size_t cols, size_t sr, size_t sc, void* out,
                          int32_t out_f32, void* stream) {
    if (w == nullptr || scales == nullptr || out == nullptr) return ERR_NULL;
    if (rows == 0 || cols == 0 || sr == 0 || sc == 0) return ERR_DOMAIN;
    if (rows % sr != 0 || cols % sc != 0 || (cols / sc) % FmtF8::UW != 0 || rows > 0x7FFFFFFFull || cols > (1u << 24))
        return ERR_DOMAIN;
    if (!al(w, 16) || !al(scales, 4) || !al(out, 16)) return ERR_DOMAIN;
    const uint32_t upb = (uint32_t)(cols / sc / FmtF8::UW);
    FmtF8::Params p{static_cast<const uint8_t*>(w), static_cast<const float*>(scales), (int)sc, (int)(rows / sr),
                    (int)upb, upb > 1 ? (uint32_t)(0x100000000ull / upb + 1) : 0u};
    const size_t threads = rows * (cols / FmtF8::UW);
    const dim3 grid((unsigned)((threads + 255) / 256));
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (out_f32)
        hipLaunchKernelGGL(fp8_widen_kernel<true>, grid, dim3(256), 0, st, p, (int)rows, (int)cols, out);
    else
        hipLaunchKernelGGL(fp8_widen_kernel<false>, grid, dim3(256), 0, st, p, (int)rows, (int)cols, out);
    return hip_status(hipGetLastError(), "fp8_widen launch");
}

int32_t btb_hip_mx4_widen(const void* blocks, const void* scales, const void* seats, size_t n_seats, int64_t groups,
                          void* out, int32_t out_f32, void* stream) {
    if (blocks == nullptr || scales == nullptr || out == nullptr) return ERR_NULL;
    if (n_seats == 0 || n_seats > 65535 || groups <= 0 || groups > (1ll << 40)) return ERR_DOMAIN;
    if (!al(blocks, 16) || !al(out, 16) || !al(seats, 4)) return ERR_DOMAIN;
    FmtMx4::Params p{static_cast<const uint8_t*>(blocks), static_cast<const uint8_t*>(scales)};
    const dim3 grid((unsigned)((groups + 255) / 256), (unsigned)n_seats);
    hipStream_t st = static_cast<hipStream_t>(stream);
    if (out_f32)
        hipLaunchKernelGGL(mx4_widen_kernel<true>, grid, dim3(256), 0, st, p, static_cast<const int32_t*>(seats),
                           (long long)groups, out);
    else
        hipLaunchKernelGGL(mx4_widen_kernel<false>, grid, dim3(256), 0, st, p, static_cast<const int32_t*>(seats),
                           (long long)groups, out);
    return hip_status(hipGetLastError(), "mx4_widen launch");
}

int32_t btb_hip_round_bf16(const void* x, void* out, size_t n, void* stream) {
    if (x == nullptr || out == nullptr) return ERR_NULL;
    if (n == 0 || n > (1ull << 40)) return ERR_DOMAIN;
    if (!al(x, 4) || !al(out, 2)) return ERR_DOMAIN;
    hipLaunchKernelGGL(round_bf16_kernel, dim3((unsigned)((n + 255) / 256)), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const float*>(x), static_cast<uint16_t*>(out), n);
    return hip_status(hipGetLastError(), "round_bf16 launch");
}

}  // extern "C"
