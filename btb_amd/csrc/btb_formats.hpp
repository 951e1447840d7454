// The stored weight forms as policies of the streaming matvec (gemv.hip) and of the widen kernels (widen.hip): what
// one lane loads in one step - a "unit" of UW consecutive weights of a row - and how those bytes become f32 weights
// in its registers, as bf16 pairs (every form's weight is exactly a bf16: a stored one, a table byte over a low
// byte, the nearest bf16 to e4m3 * scale, or an fp4 value times a power of two). The vector forms here must equal the
// scalar definitions of btb_widen.hpp bit for bit; the widen kernels expose them so the tests can check exactly
// that, over every byte value.
#pragma once

#include "btb_common.hpp"
#include "btb_widen.hpp"

namespace btb {

// ------------------------------------------------------------------------------------------------------------
// bf16 rows: a unit is 8 weights, one 16-byte load
// ------------------------------------------------------------------------------------------------------------
struct FmtBf16 {
    static constexpr int UW = 8;
    static constexpr bool TWO_ROWS = false;  // the tile shape the streaming matvec prefers for this form (gemv.hip)
    struct Params {
        const uint4* w;
    };
    struct Raw {
        uint4 v;
    };
    struct RowCtx {
        const uint4* row;
    };
    __device__ static __forceinline__ void prepare(Params&) {}
    __device__ static __forceinline__ void prepare_finish(Params&) {}
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units, int sl = 0) {
        return RowCtx{p.w + r * (size_t)units};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) { return Raw{load_stream16(c.row + unit)}; }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, uint32_t (&w)[UW / 2]) {
        w[0] = r.v.x;
        w[1] = r.v.y;
        w[2] = r.v.z;
        w[3] = r.v.w;
    }
    // nothing past the stream
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

// ------------------------------------------------------------------------------------------------------------
// pack12: a unit is 16 weights - 16 low bytes (one 16-byte load) and 16 four-bit codes (one 8-byte load). A code
// becomes its high byte through the 16-entry table held in four registers: two byte-permutes pick from entries 0..7
// and 8..15, a bit-select on the code's top bit chooses between them; one more permute per pair of weights zips the
// high bytes over their low bytes into a bf16 pair. An escaped weight (code 15) comes out of the stream with
// table[15]'s high byte; `tail` then replaces its term from the escape list: acc += (true - streamed) * x, two
// fused multiply-adds per escape, found through the row's slice of the list (row_ptr).
// ------------------------------------------------------------------------------------------------------------
struct FmtP12 {
    static constexpr int UW = 16;
    static constexpr bool TWO_ROWS = false;
    struct Params {
        const uint8_t* lo;
        const uint8_t* hi4;
        const uint8_t* table;  // the 16 high bytes (any alignment)
        const int32_t* esc_idx;
        const uint8_t* esc_val;
        const int32_t* row_ptr;  // [rows + 1] first escape at or past each row's start
        uint4 tbl;               // the table in registers: filled by prepare() on the device, not by the host
        const uint16_t* pairs;   // [256] the pair table made at upload (FmtP12G), or null
        uint32_t pair_reg;       // this thread's entry of it on its way to LDS (prepare -> prepare_finish)
        const uint32_t* row_esc; // [rows][4] every row's first four escapes, a word each, made at upload, or null
    };
    struct Raw {
        uint4 lo;
        uint2 codes;
    };
    struct RowCtx {
        const uint4* lo;
        const uint2* hi4;
        uint4 table;
        int e0, e1;  // the row's escapes: [e0, e1) of the list; where the matrix has the rows' words: the lane's word
    };
    // A row's words (row_esc, made at upload: btb_hip_p12_row_esc): its first row_esc_slots(C) escapes, one a word -
    // low byte in bits 0..7, true high byte in 8..15, column in 16..30 (ROW_ESC_NONE: no such escape) - and in bit 31 of
    // every word of the row: the row has more escapes than words. Eight words a row up to 4096 columns, sixteen beyond:
    // a launch ends with its slowest wave, so what counts is that next to no row of a launch has more (at 0.02 % of
    // the weights escaped a row of 2560 holds more than four once in six thousand rows - three rows of every gate/up
    // launch - and more than eight once in 10^8; a row of 9728 more than eight once in five thousand, more than
    // sixteen never).
    static constexpr uint32_t ROW_ESC_NONE = 0x7FFFu;
    __host__ __device__ static constexpr int row_esc_slots(int C) { return C <= 4096 ? 8 : 16; }
    // The part of a row's context that comes out of memory: the lane's word of the row's words where the matrix has
    // them (lane sl of the row's lanes: word min(sl, slots - 1)), else the row's slice of the list. Two 4-byte loads
    // from addresses chosen without a branch: a branch here makes the compiler wait for what was loaded before it,
    // ahead of the row's weights.
    __device__ static __forceinline__ void row_escapes(const Params& p, size_t r, int units, int sl, RowCtx& c) {
        const bool words = p.row_esc != nullptr;
        const int slots = row_esc_slots(units * UW);
        const int32_t* base = words ? reinterpret_cast<const int32_t*>(p.row_esc) : p.row_ptr;
        const size_t at = words ? r * (size_t)slots + (size_t)min(sl, slots - 1) : r;
        c.e0 = base[at];
        c.e1 = base[words ? at : at + 1];
    }
    // the table's 16 bytes as four registers, entry k in byte k
    __device__ static __forceinline__ uint4 load_table(const uint8_t* t) {
        uint32_t d[4];
#pragma unroll
        for (int k = 0; k < 4; ++k)
            d[k] = (uint32_t)t[4 * k] | ((uint32_t)t[4 * k + 1] << 8) | ((uint32_t)t[4 * k + 2] << 16) |
                   ((uint32_t)t[4 * k + 3] << 24);
        return make_uint4(d[0], d[1], d[2], d[3]);
    }
    // once per kernel (or phase), before any row_ctx: the table's 16 bytes are read here and only here
    __device__ static __forceinline__ void prepare(Params& p) { p.tbl = load_table(p.table); }
    __device__ static __forceinline__ void prepare_finish(Params&) {}
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units, int sl = 0) {
        RowCtx c;
        c.lo = reinterpret_cast<const uint4*>(p.lo) + r * (size_t)units;
        c.hi4 = reinterpret_cast<const uint2*>(p.hi4) + r * (size_t)units;
        c.table = p.tbl;
        row_escapes(p, r, units, sl, c);
        return c;
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        return Raw{load_stream16(c.lo + unit), load_stream8(c.hi4 + unit)};
    }
    // four codes (one per byte of v) to their four table bytes: two byte-permutes look the code's low three bits up
    // in entries 0..7 and in entries 8..15, a third picks per byte between the two by the code's top bit (selector
    // i takes byte i of the first lookup, 4 + i of the second)
    __device__ static __forceinline__ uint32_t lut16(const uint4& t, uint32_t v) {
        const uint32_t sel = v & 0x07070707u;
        const uint32_t a = __builtin_amdgcn_perm(t.y, t.x, sel);  // entries 0..7
        const uint32_t b = __builtin_amdgcn_perm(t.w, t.z, sel);  // entries 8..15
        const uint32_t pick = 0x03020100u | ((v & 0x08080808u) >> 1);
        return __builtin_amdgcn_perm(b, a, pick);
    }
    // eight weights as four bf16 pairs: codes c (weight k in nibble k), their low bytes l0 (weights 0..3), l1 (4..7).
    // A byte-permute's selector 0..3 takes a byte of its second operand, 4..7 of its first.
    __device__ static __forceinline__ void widen8(const uint4& t, uint32_t c, uint32_t l0, uint32_t l1, uint32_t* w) {
        const uint32_t even = c & 0x0F0F0F0Fu;         // codes of weights 0, 2, 4, 6
        const uint32_t odd = (c >> 4) & 0x0F0F0F0Fu;   // of weights 1, 3, 5, 7
        const uint32_t c03 = __builtin_amdgcn_perm(odd, even, 0x05010400u);  // codes 0, 1, 2, 3 a byte each
        const uint32_t c47 = __builtin_amdgcn_perm(odd, even, 0x07030602u);  // codes 4, 5, 6, 7
        const uint32_t h03 = lut16(t, c03), h47 = lut16(t, c47);             // their high bytes
        w[0] = __builtin_amdgcn_perm(h03, l0, 0x05010400u);  // lo0 hi0 lo1 hi1
        w[1] = __builtin_amdgcn_perm(h03, l0, 0x07030602u);  // lo2 hi2 lo3 hi3
        w[2] = __builtin_amdgcn_perm(h47, l1, 0x05010400u);
        w[3] = __builtin_amdgcn_perm(h47, l1, 0x07030602u);
    }
    __device__ static __forceinline__ void widen(const RowCtx& c, const Raw& r, int /*unit*/, uint32_t (&w)[UW / 2]) {
        widen8(c.table, r.codes.x, r.lo.x, r.lo.y, w);
        widen8(c.table, r.codes.y, r.lo.z, r.lo.w, w + 4);
    }
    // The row's escapes, spread over the row's lanes (escape k of the row: lane k % lpr, in list order): the streamed
    // term out, the true term in. Out of the list that is three round trips one behind the other - the row's slice,
    // its entries, the low bytes they name - at the end of a tile, where a wave has nothing left to hide them behind:
    // a tenth of the packed decode step, and a launch ends with its slowest wave, so it is not enough to spare most
    // rows the walk. Hence the rows' words: a row's first eight (or sixteen) escapes stand in words of the row's own,
    // whose address the row number gives, and lane k asks for word k ahead of the row's weights - it has all it needs
    // when the products are done. Only a row with more escapes than words walks the list, from the first entry that
    // has no word on.
    template <int M>
    __device__ static __forceinline__ void esc_term(const RowCtx& c, int C, const uint32_t* xs, float (&acc)[M], int col,
                                                    uint32_t val, uint32_t lo) {
        const uint32_t t15 = c.table.w >> 24;
        const uint16_t* x16 = reinterpret_cast<const uint16_t*>(xs);
        const float streamed = bits_f32((t15 << 24) | (lo << 16));
        const float truth = bits_f32((val << 24) | (lo << 16));
#pragma unroll
        for (int m = 0; m < M; ++m) {
            const float xv = bf16_f32(x16[(size_t)m * C + col]);
            acc[m] = fmaf(truth, xv, fmaf(-streamed, xv, acc[m]));
        }
    }
    template <int M>
    __device__ static __forceinline__ void tail(const Params& p, const RowCtx& c, size_t r, int sl, int lpr, int C,
                                                const uint32_t* xs, float (&acc)[M]) {
        int e0 = c.e0, e1 = c.e1, from = sl;
        if (p.row_esc != nullptr) {  // uniform
            const uint32_t rec = (uint32_t)c.e0, col = (rec >> 16) & 0x7FFFu;
            const int slots = row_esc_slots(C);
            if (sl < slots && col != ROW_ESC_NONE)
                esc_term<M>(c, C, xs, acc, (int)col, (rec >> 8) & 0xFFu, rec & 0xFFu);
            if ((rec >> 31) == 0u) return;
            e0 = p.row_ptr[r];
            e1 = p.row_ptr[r + 1];
            from = sl < slots ? sl + lpr : sl;  // those with a word are done
        }
        for (int e = e0 + from; e < e1; e += lpr) {
            const size_t i = (size_t)p.esc_idx[e];
            esc_term<M>(c, C, xs, acc, (int)(i - r * (size_t)C), (uint32_t)p.esc_val[e], (uint32_t)p.lo[i]);
        }
    }
};

// The same form with the table lookups done in LDS: a 256-entry table of PAIRS - entry b holds the high bytes of the
// two weights whose codes are byte b's nibbles - and a byte of codes becomes its two high bytes with one 16-bit LDS
// read where the in-register lookup takes two byte-permutes, a select and the nibble split per four codes. Eight
// weights: 4 byte extractions, 4 LDS reads, 4 byte-permutes that zip high and low bytes (23 vector instructions
// before). The table is made once, at upload (btb_hip_p12_pairs: 512 bytes beside row_ptr, slot 15 of the 16-byte
// table taken as 0), and a workgroup of 256 threads brings it in with one 2-byte load a thread: prepare() asks for
// it before anything else, prepare_finish() - called once the kernel's first weights have been requested - puts it
// into LDS, and the workgroup barrier that ends the x staging makes it visible. Nothing of it sits on the way of the
// weights: building the table in the kernel did (the plain forms lost 0.3 us a launch to it).
struct FmtP12G : FmtP12 {
    __device__ static __forceinline__ uint16_t* pair_table() {
        __shared__ uint16_t pairs[256];
        return pairs;
    }
    __device__ static __forceinline__ void prepare(Params& p) { p.pair_reg = p.pairs[threadIdx.x & 255]; }
    __device__ static __forceinline__ void prepare_finish(Params& p) {
        if (threadIdx.x < 256) pair_table()[threadIdx.x] = (uint16_t)p.pair_reg;
    }
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units, int sl = 0) {
        RowCtx c;
        c.lo = reinterpret_cast<const uint4*>(p.lo) + r * (size_t)units;
        c.hi4 = reinterpret_cast<const uint2*>(p.hi4) + r * (size_t)units;
        c.table = make_uint4(0u, 0u, 0u, 0u);  // not read: the lookups go through LDS, an escape streams as slot 15 = 0
        row_escapes(p, r, units, sl, c);
        return c;
    }
    // eight weights: codes c (weight k in nibble k), low bytes l0 (weights 0..3), l1 (4..7)
    __device__ static __forceinline__ void widen8(uint32_t c, uint32_t l0, uint32_t l1, uint32_t* w) {
        const uint16_t* t = pair_table();
        const uint32_t h01 = t[c & 0xFFu], h23 = t[(c >> 8) & 0xFFu], h45 = t[(c >> 16) & 0xFFu], h67 = t[c >> 24];
        // a byte-permute's selector 0..3 takes a byte of its second operand, 4..7 of its first
        w[0] = __builtin_amdgcn_perm(h01, l0, 0x05010400u);  // lo0 hi0 lo1 hi1
        w[1] = __builtin_amdgcn_perm(h23, l0, 0x05030402u);  // lo2 hi2 lo3 hi3
        w[2] = __builtin_amdgcn_perm(h45, l1, 0x05010400u);
        w[3] = __builtin_amdgcn_perm(h67, l1, 0x05030402u);
    }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, uint32_t (&w)[UW / 2]) {
        widen8(r.codes.x, r.lo.x, r.lo.y, w);
        widen8(r.codes.y, r.lo.z, r.lo.w, w + 4);
    }
};

// ------------------------------------------------------------------------------------------------------------
// FP8 e4m3fn with an f32 scale per block of a [sr, sc] grid: a unit is 16 weights, one 16-byte load, under one
// scale (the block's width is a multiple of 16). weight = bf16_rne(e4m3 * scale): the byte pair is converted by
// v_cvt_pk_f32_fp8 (exact: every e4m3 value is an f32), multiplied by the scale once in f32, and rounded to bf16,
// nearest even, by v_cvt_pk_bf16_f32 - the same bits as the integer rule of btb_common.hpp on every byte and scale
// (the widen kernel's test sweeps them all).
// ------------------------------------------------------------------------------------------------------------
struct FmtF8 {
    static constexpr int UW = 16;
    static constexpr bool TWO_ROWS = true;
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
    __device__ static __forceinline__ void prepare(Params&) {}
    __device__ static __forceinline__ void prepare_finish(Params&) {}
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units, int sl = 0) {
        return RowCtx{reinterpret_cast<const uint4*>(p.w) + r * (size_t)units, p.scales + (r / p.bm) * (size_t)p.sc,
                      p.upb, p.magic};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        const int blk = c.upb == 1 ? unit : (int)__umulhi((uint32_t)unit, c.magic);
        return Raw{load_stream16(c.row + unit), c.srow[blk]};
    }
    // four bytes to two bf16 pairs: exact conversion to f32, one f32 multiply by the scale, nearest-even to bf16
    __device__ static __forceinline__ void widen4(uint32_t q, float s, uint32_t* w) {
        const f32x2 a = __builtin_amdgcn_cvt_pk_f32_fp8(q, false);
        const f32x2 b = __builtin_amdgcn_cvt_pk_f32_fp8(q, true);
        const bf16x2 p0 = {(__bf16)(a.x * s), (__bf16)(a.y * s)};
        const bf16x2 p1 = {(__bf16)(b.x * s), (__bf16)(b.y * s)};
        w[0] = __builtin_bit_cast(uint32_t, p0);
        w[1] = __builtin_bit_cast(uint32_t, p1);
    }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, uint32_t (&w)[UW / 2]) {
        widen4(r.v.x, r.scale, w);
        widen4(r.v.y, r.scale, w + 2);
        widen4(r.v.z, r.scale, w + 4);
        widen4(r.v.w, r.scale, w + 6);
    }
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

// ------------------------------------------------------------------------------------------------------------
// MXFP4: a unit is one block of 32 weights - 16 bytes of packed e2m1 codes (the earlier weight of a pair in the low
// nibble) and one e8m0 scale byte. weight = fp4 * 2^(scale - 127): an fp4 value has two significant bits, so the
// product is exact in bf16 for every scale below 255 (bf16 has f32's exponent range), and
// v_cvt_scalef32_pk_bf16_fp4 converts a byte's two codes and applies the scale in one instruction.
// ------------------------------------------------------------------------------------------------------------
struct FmtMx4 {
    static constexpr int UW = 32;
    static constexpr bool TWO_ROWS = false;
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
    __device__ static __forceinline__ void prepare(Params&) {}
    __device__ static __forceinline__ void prepare_finish(Params&) {}
    __device__ static __forceinline__ RowCtx row_ctx(const Params& p, size_t r, int units, int sl = 0) {
        return RowCtx{reinterpret_cast<const uint4*>(p.blocks) + r * (size_t)units, p.scales + r * (size_t)units};
    }
    __device__ static __forceinline__ Raw load(const RowCtx& c, int unit) {
        return Raw{load_stream16(c.row + unit), (uint32_t)__builtin_nontemporal_load(c.srow + unit)};
    }
    // eight codes to four bf16 pairs
    __device__ static __forceinline__ void widen8(uint32_t q, float s, uint32_t* w) {
        w[0] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, s, 0));
        w[1] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, s, 1));
        w[2] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, s, 2));
        w[3] = __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(q, s, 3));
    }
    // a pair under scale 255 (2^128, past f32: +inf): the CPU's product is +-inf, or NaN for a zero code
    __device__ static __forceinline__ uint32_t inf_pair(uint32_t byte) {
        const uint32_t lo = ((byte & 7u) ? 0x7F80u : 0x7FC0u) | ((byte & 8u) << 12);
        const uint32_t hi = ((byte & 0x70u) ? 0x7F80u : 0x7FC0u) | ((byte & 0x80u) << 8);
        return lo | (hi << 16);
    }
    __device__ static __forceinline__ void widen(const RowCtx&, const Raw& r, int /*unit*/, uint32_t (&w)[UW / 2]) {
        // the instruction reads the scale's exponent field, so the e8m0 byte goes in as f32 bits s << 23 - for
        // s == 0 too, which it takes as 2^-127 (the widen kernel's test covers every scale)
        const float sf = bits_f32(r.s << 23);
        widen8(r.v.x, sf, w);
        widen8(r.v.y, sf, w + 4);
        widen8(r.v.z, sf, w + 8);
        widen8(r.v.w, sf, w + 12);
    }
    // Scale 255 is 2^128, not a finite f32; no quantizer writes it. The CPU's product there is +-inf (NaN for a
    // zero code); the widen kernel patches its output to exactly that, the matvec leaves what the conversion
    // instruction gives (non-finite either way).
    __device__ static __forceinline__ void patch255(const Raw& r, uint32_t (&w)[UW / 2]) {
        if (r.s != 255u) return;
        const uint32_t q[4] = {r.v.x, r.v.y, r.v.z, r.v.w};
#pragma unroll
        for (int j = 0; j < 16; ++j) w[j] = inf_pair((q[j >> 2] >> ((j & 3) * 8)) & 0xFFu);
    }
    template <int M>
    __device__ static __forceinline__ void tail(const Params&, const RowCtx&, size_t, int, int, int, const uint32_t*,
                                                float (&)[M]) {}
};

}  // namespace btb
