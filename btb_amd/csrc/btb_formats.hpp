// The stored weight forms as policies of the streaming matvec (gemv.hip) and of the widen kernels (widen.hip): what
// one lane loads in one step - a "unit" of UW consecutive weights of a row - and how those bytes become f32 weights
// in its registers. The vector forms here must equal the scalar definitions of btb_widen.hpp bit for bit; the widen
// kernels expose them so the tests can check exactly that, over every byte value.
#pragma once

#include "btb_common.hpp"
#include "btb_widen.hpp"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// bf16 rows: a unit is 8 weights, one 16-byte load
// ------------------------------------------------------------------------------------------------------------
struct FmtBf16 {
    static constexpr int UW = 8;
    struct Params {
        const uint4* w;
    };
    struct Raw {
        uint4 v;
    };
    struct RowCtx {
        const uint4* row;
    };
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units) {
        return RowCtx{p.w + r * (size_t)units};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) { return Raw{load_stream16(c.row + unit)}; }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, float (&w)[UW]) {
        w[0] = bf16lo_f32(r.v.x);
        w[1] = bf16hi_f32(r.v.x);
        w[2] = bf16lo_f32(r.v.y);
        w[3] = bf16hi_f32(r.v.y);
        w[4] = bf16lo_f32(r.v.z);
        w[5] = bf16hi_f32(r.v.z);
        w[6] = bf16lo_f32(r.v.w);
        w[7] = bf16hi_f32(r.v.w);
    }
    // nothing past the stream
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

// ------------------------------------------------------------------------------------------------------------
// pack12: a unit is 16 weights - 16 low bytes (one 16-byte load) and 16 four-bit codes (one 8-byte load). A code
// becomes its high byte through the 16-entry table held in four registers: two byte-permutes pick from entries 0..7
// and 8..15, a bit-select on the code's top bit chooses between them; a third permute per weight zips the high byte
// over its low byte into the top half of an f32. An escaped weight (code 15) comes out of the stream with
// table[15]'s high byte; `tail` then replaces its term from the escape list: acc += (true - streamed) * x, two
// fused multiply-adds per escape, found through the row's slice of the list (row_ptr).
// ------------------------------------------------------------------------------------------------------------
struct FmtP12 {
    static constexpr int UW = 16;
    struct Params {
        const uint8_t* lo;
        const uint8_t* hi4;
        const uint8_t* table;  // the 16 high bytes (any alignment)
        const int32_t* esc_idx;
        const uint8_t* esc_val;
        const int32_t* row_ptr;  // [rows + 1] first escape at or past each row's start
    };
    struct Raw {
        uint4 lo;
        uint2 codes;
    };
    struct RowCtx {
        const uint4* lo;
        const uint2* hi4;
        uint4 table;
        int e0, e1;  // the row's escapes: [e0, e1) of the list
    };
    // the table's 16 bytes as four registers, entry k in byte k
    __device__ static __forceinline__ uint4 load_table(const uint8_t* t) {
        uint32_t d[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            d[k] = (uint32_t)t[4 * k] | ((uint32_t)t[4 * k + 1] << 8) | ((uint32_t)t[4 * k + 2] << 16) |
                   ((uint32_t)t[4 * k + 3] << 24);
        return make_uint4(d[0], d[1], d[2], d[3]);
    }
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units) {
        RowCtx c;
        c.lo = reinterpret_cast<const uint4*>(p.lo) + r * (size_t)units;
        c.hi4 = reinterpret_cast<const uint2*>(p.hi4) + r * (size_t)units;
        c.table = load_table(p.table);
        c.e0 = p.row_ptr[r];
        c.e1 = p.row_ptr[r + 1];
        return c;
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        return Raw{load_stream16(c.lo + unit), load_stream8(c.hi4 + unit)};
    }
    // four codes (one per byte of v) to their four table bytes
    __device__ static __forceinline__ uint32_t lut16(const uint4& t, uint32_t v) {
        const uint32_t sel = v & 0x07070707u;
        const uint32_t a = __builtin_amdgcn_perm(t.y, t.x, sel);  // entries 0..7
        const uint32_t b = __builtin_amdgcn_perm(t.w, t.z, sel);  // entries 8..15
        const uint32_t m = ((v >> 3) & 0x01010101u) * 0xFFu;      // 0xFF in the bytes whose code is 8..15
        return (b & m) | (a & ~m);
    }
    // eight weights: codes c (weight k in nibble k), their low bytes l0 (weights 0..3) and l1 (4..7)
    __device__ static __forceinline__ void widen8(const uint4& t, uint32_t c, uint32_t l0, uint32_t l1, float* w) {
        const uint32_t he = lut16(t, c & 0x0F0F0F0Fu);         // high bytes of weights 0, 2, 4, 6
        const uint32_t ho = lut16(t, (c >> 4) & 0x0F0F0F0Fu);  // of weights 1, 3, 5, 7
        // f32 bits = high byte << 24 | low byte << 16: selector 4..7 takes a byte of the first operand, 0..3 of the
        // second, 0x0c is zero
        w[0] = bits_f32(__builtin_amdgcn_perm(he, l0, 0x04000c0cu));
        w[1] = bits_f32(__builtin_amdgcn_perm(ho, l0, 0x04010c0cu));
        w[2] = bits_f32(__builtin_amdgcn_perm(he, l0, 0x05020c0cu));
        w[3] = bits_f32(__builtin_amdgcn_perm(ho, l0, 0x05030c0cu));
        w[4] = bits_f32(__builtin_amdgcn_perm(he, l1, 0x06000c0cu));
        w[5] = bits_f32(__builtin_amdgcn_perm(ho, l1, 0x06010c0cu));
        w[6] = bits_f32(__builtin_amdgcn_perm(he, l1, 0x07020c0cu));
        w[7] = bits_f32(__builtin_amdgcn_perm(ho, l1, 0x07030c0cu));
    }
    __device__ static __forceinline__ void widen(const RowCtx& c, const Raw& r, int /*unit*/, float (&w)[UW]) {
        widen8(c.table, r.codes.x, r.lo.x, r.lo.y, w);
        widen8(c.table, r.codes.y, r.lo.z, r.lo.w, w + 8);
    }
    // the row's escapes, spread over the row's lanes: the streamed term out, the true term in
    template <int M>
    __device__ static __forceinline__ void tail(const Params& p, const RowCtx& c, size_t r, int sl, int lpr, int C,
                                                const uint32_t* xs, float (&acc)[M]) {
        const uint32_t t15 = c.table.w >> 24;
        const uint16_t* x16 = reinterpret_cast<const uint16_t*>(xs);
        for (int e = c.e0 + sl; e < c.e1; e += lpr) {
            const size_t i = (size_t)p.esc_idx[e];
            const uint32_t lo = p.lo[i];
            const float streamed = bits_f32((t15 << 24) | (lo << 16));
            const float truth = bits_f32(((uint32_t)p.esc_val[e] << 24) | (lo << 16));
            const int col = (int)(i - r * (size_t)C);
#pragma unroll
            for (int m = 0; m < M; ++m) {
                const float xv = bf16_f32(x16[(size_t)m * C + col]);
                acc[m] = fmaf(truth, xv, fmaf(-streamed, xv, acc[m]));
            }
        }
    }
};

// ------------------------------------------------------------------------------------------------------------
// FP8 e4m3fn with an f32 scale per block of a [sr, sc] grid: a unit is 16 weights, one 16-byte load, under one
// scale (the block's width is a multiple of 16). weight = bf16_rne(e4m3 * scale): the byte pair is converted by
// v_cvt_pk_f32_fp8 (exact: every e4m3 value is an f32), multiplied by the scale once in f32, and rounded to bf16 by
// the integer rule of btb_common.hpp.
// ------------------------------------------------------------------------------------------------------------
struct FmtF8 {
    static constexpr int UW = 16;
    struct Params {
        const uint8_t* w;
        const float* scales;
        int sc;        // scales per grid row
        int bm;        // rows per block
        int upb;       // units (of 16 columns) per block
        uint32_t magic;  // unit / upb == umulhi(unit, magic) for every unit of a row (upb > 1)
    };
    struct Raw {
        uint4 v;
        float scale;
    };
    struct RowCtx {
        const uint4* row;
        const float* srow;
        int upb;
        uint32_t magic;
    };
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units) {
        return RowCtx{reinterpret_cast<const uint4*>(p.w) + r * (size_t)units, p.scales + (r / p.bm) * (size_t)p.sc,
                      p.upb, p.magic};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        const int blk = c.upb == 1 ? unit : (int)__umulhi((uint32_t)unit, c.magic);
        return Raw{load_stream16(c.row + unit), c.srow[blk]};
    }
    __device__ static __forceinline__ void widen4(uint32_t q, float s, float* w) {
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(q, false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(q, true);
        w[0] = round_bf16_f32(a.x * s);
        w[1] = round_bf16_f32(a.y * s);
        w[2] = round_bf16_f32(b.x * s);
        w[3] = round_bf16_f32(b.y * s);
    }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, float (&w)[UW]) {
        widen4(r.v.x, r.scale, w);
        widen4(r.v.y, r.scale, w + 4);
        widen4(r.v.z, r.scale, w + 8);
        widen4(r.v.w, r.scale, w + 12);
    }
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

// ------------------------------------------------------------------------------------------------------------
// MXFP4: a unit is one block of 32 weights - 16 bytes of packed e2m1 codes (the earlier weight of a pair in the low
// nibble) and one e8m0 scale byte. weight = fp4 * 2^(scale - 127) in f32 (exact wherever it is a normal f32):
// v_cvt_scalef32_pk_f32_fp4 converts a byte's two codes and applies the scale in one instruction.
// ------------------------------------------------------------------------------------------------------------
struct FmtMx4 {
    static constexpr int UW = 32;
    struct Params {
        const uint8_t* blocks;
        const uint8_t* scales;
    };
    struct Raw {
        uint4 v;
        uint32_t s;
    };
    struct RowCtx {
        const uint4* row;
        const uint8_t* srow;
    };
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units) {
        return RowCtx{reinterpret_cast<const uint4*>(p.blocks) + r * (size_t)units, p.scales + r * (size_t)units};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        return Raw{load_stream16(c.row + unit), (uint32_t)__builtin_nontemporal_load(c.srow + unit)};
    }
    __device__ static __forceinline__ void widen8(uint32_t q, float s, float* w) {
        const f32x2 a = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q, s, 0);
        const f32x2 b = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q, s, 1);
        const f32x2 c = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q, s, 2);
        const f32x2 d = __builtin_amdgcn_cvt_scalef32_pk_f32_fp4(q, s, 3);
        w[0] = a.x;
        w[1] = a.y;
        w[2] = b.x;
        w[3] = b.y;
        w[4] = c.x;
        w[5] = c.y;
        w[6] = d.x;
        w[7] = d.y;
    }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, float (&w)[UW]) {
        // the scale as an f32 power of two; 0 (2^-127) and 255 (inf) are not normal f32 exponents and take the
        // scalar definition
        const uint32_t s = r.s;
        if (__builtin_expect(s == 0u || s == 255u, 0)) {
            const uint32_t q[4] = {r.v.x, r.v.y, r.v.z, r.v.w};
#pragma unroll
            for (int j = 0; j < 16; ++j) {
                const uint8_t byte = (uint8_t)(q[j >> 2] >> ((j & 3) * 8));
                w[2 * j] = mx4_weight(byte, 0, (uint8_t)s);
                w[2 * j + 1] = mx4_weight(byte, 1, (uint8_t)s);
            }
            return;
        }
        const float sf = bits_f32(s << 23);
        widen8(r.v.x, sf, w);
        widen8(r.v.y, sf, w + 8);
        widen8(r.v.z, sf, w + 16);
        widen8(r.v.w, sf, w + 24);
    }
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

}  // namespace btb
