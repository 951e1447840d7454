// The verify widths (M = 5..16 rows of x a pass) on the matrix cores with the weights going from memory straight into
// LDS: the long rows of the block-scaled forms (FP8 e4m3 + block scales, MXFP4: 7168 columns) and pack12 rows of the
// lengths it has shapes for (2560, up to 4096, around 9728 columns).
//
// gemv_mfma_lds.hip brings a sub-block of weights into registers, parks it in LDS and reads it back in the MFMA's
// layout. On rows as long as 7168 columns the x fragments a wave keeps (x-stationary: 28 steps x 4 registers) leave
// room for one such sub-block of registers, so a wave has 4 KB on its way at a time, a CU 32 KB - a third of what the
// memory's latency needs at these rates (measured: 33 % of HBM peak for FP8, 25 % for MXFP4). Here the bytes never
// touch a register on their way in: global_load_lds_dwordx4 writes lane l's 16 bytes at the LDS base held in M0 plus
// 16 l, so what is in flight is bounded by LDS, not by registers, and a wave keeps a ring of NBUF sub-blocks: one
// being multiplied, NBUF - 1 on their way.
//
// A load instruction costs the same with fourteen lanes as with sixty-four, so every one is a full one: 8 rows x 128
// bytes (lane l: row l % 8, 16-byte granule l / 8 of the 128). The LDS side of it is then fixed - granule-major, row
// within granule: [8 granules][8 rows][16 B] = 1 KB - and that is also what the fragment reads want: a step's read
// touches one or two granules of all sixteen rows, 8 rows x 16 B = 128 contiguous bytes a half, the upper eight rows'
// block placed 128 bytes off a multiple of 256 so the two halves fall in different banks. A sub-block is GB such
// 128-byte column blocks of the tile's sixteen rows: 2 GB load instructions, plus one or two more direct loads for
// what goes with them (the MXFP4 scale bytes of its rows and steps; the FP8 block scales of its steps - a tile's
// sixteen rows share them: blocks are a multiple of 16 rows tall; the pack12 code nibbles).
//
// Waiting is by count: loads complete in order, a sub-block is LOADS load instructions, so "sub-block q has landed" is
// "at most (sub-blocks issued behind it) x LOADS loads outstanding" - an immediate, picked by how many were issued
// behind it. The output stores of a tile's end count as outstanding too and may complete in any order: they are left
// out of the immediate, which can only make a wait longer. A slot is asked for again only after the reads of its last
// use have returned (the MFMAs that take them have been issued). The waves that stream never load into a register
// the compiler knows to be outstanding (x comes through load_untracked, a form's constants through scalar loads):
// behind a direct-to-LDS load the compiler's own wait for such a register is a wait for every load there is.
//
// The fold of the KS partial tiles in wave order and every rounding are gemv_mfma_lds's; which steps a wave sums
// differs (see the kernel), so the two kernels agree to f32 summation order, not to the bit. Every M of a pass takes
// the same path here, so a row of x gets the same bits whatever the other rows of the pass are.

#include <type_traits>

#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {

typedef __attribute__((address_space(3))) void lds_void;

// s_waitcnt vmcnt(N) alone, with the two LDS offsets the reads behind it use passed through it. A direct-to-LDS load
// is, to the compiler, a store that happened where it was issued: left alone it may (and did) move a slot's reads
// ahead of the wait that says the slot has landed. The reads' addresses are made of values this statement "writes",
// so they come after it; the statement itself keeps its place among the loads' issue (both have side effects).
template <int N>
__device__ __forceinline__ void wait_loads(uint32_t& a, uint32_t& b) {
    static_assert(N >= 0 && N < 64, "vmcnt is six bits");
    asm volatile("s_waitcnt vmcnt(%2)" : "+v"(a), "+v"(b) : "n"(N) : "memory");
}
// the wait for "at most `behind` sub-blocks of LOADS loads each behind the one read next", behind in 0..MAXB
template <int LOADS, int MAXB>
__device__ __forceinline__ void wait_behind(int behind, uint32_t& a, uint32_t& b) {
    static_assert(MAXB * LOADS < 64 && MAXB >= 1 && MAXB <= 6, "the waits count up to 63 loads");
    if (MAXB >= 6 && behind == 6)
        wait_loads<(MAXB >= 6 ? 6 : 0) * LOADS>(a, b);
    else if (MAXB >= 5 && behind == 5)
        wait_loads<(MAXB >= 5 ? 5 : 0) * LOADS>(a, b);
    else if (MAXB >= 4 && behind == 4)
        wait_loads<(MAXB >= 4 ? 4 : 0) * LOADS>(a, b);
    else if (MAXB >= 3 && behind == 3)
        wait_loads<(MAXB >= 3 ? 3 : 0) * LOADS>(a, b);
    else if (MAXB >= 2 && behind == 2)
        wait_loads<(MAXB >= 2 ? 2 : 0) * LOADS>(a, b);
    else if (behind == 1)
        wait_loads<LOADS>(a, b);
    else
        wait_loads<0>(a, b);
}
// the same in the kernel's first tile, where behind the sub-block read next there are also XP parts of x of XL loads
// each (XP is known where this is called; it arrives as a number that folds)
template <int LOADS, int MAXB, int XL, int XP>
__device__ __forceinline__ void wait_first_x(int behind, uint32_t& a, uint32_t& b) {
    auto imm = [](int n) constexpr { return n * LOADS + XP * XL < 64 ? n * LOADS + XP * XL : 0; };
    if (MAXB >= 6 && behind == 6)
        wait_loads<imm(MAXB >= 6 ? 6 : 0)>(a, b);
    else if (MAXB >= 5 && behind == 5)
        wait_loads<imm(MAXB >= 5 ? 5 : 0)>(a, b);
    else if (MAXB >= 4 && behind == 4)
        wait_loads<imm(MAXB >= 4 ? 4 : 0)>(a, b);
    else if (MAXB >= 3 && behind == 3)
        wait_loads<imm(MAXB >= 3 ? 3 : 0)>(a, b);
    else if (MAXB >= 2 && behind == 2)
        wait_loads<imm(MAXB >= 2 ? 2 : 0)>(a, b);
    else if (behind == 1)
        wait_loads<imm(1)>(a, b);
    else
        wait_loads<imm(0)>(a, b);
}
template <int LOADS, int MAXB, int XL>
__device__ __forceinline__ void wait_first(int behind, int xparts, uint32_t& a, uint32_t& b) {
    if (xparts == 6)
        wait_first_x<LOADS, MAXB, XL, 6>(behind, a, b);
    else if (xparts == 5)
        wait_first_x<LOADS, MAXB, XL, 5>(behind, a, b);
    else if (xparts == 4)
        wait_first_x<LOADS, MAXB, XL, 4>(behind, a, b);
    else if (xparts == 3)
        wait_first_x<LOADS, MAXB, XL, 3>(behind, a, b);
    else if (xparts == 2)
        wait_first_x<LOADS, MAXB, XL, 2>(behind, a, b);
    else if (xparts == 1)
        wait_first_x<LOADS, MAXB, XL, 1>(behind, a, b);
    else
        wait_first_x<LOADS, MAXB, XL, 0>(behind, a, b);
}

// A 16-byte load whose being outstanding the compiler does not know of, and the statement that says "these four have
// landed" (it follows the counted wait that makes it true). The compiler's own wait for a loaded register is exact
// only while no direct-to-LDS load is outstanding: those are FLAT-encoded instructions that name LDS, after which it
// takes the order of returns to be unknown and waits for every load there is, the ring's included. The kernel's first
// tile wants its part of x and nothing younger, so x comes through these two. Between the two statements the registers
// are named by nothing else.
__device__ __forceinline__ u32x4 load_untracked(const u32x4* p) {
    u32x4 v;
    asm volatile("global_load_dwordx4 %0, %1, off" : "=v"(v) : "v"(p) : "memory");
    return v;
}
__device__ __forceinline__ void landed(u32x4& a, u32x4& b, u32x4& c, u32x4& d) {
    asm volatile("" : "+v"(a), "+v"(b), "+v"(c), "+v"(d));
}

// the slot's data: column block gb of 128 bytes at gb * BLK, rows 8..15 of it HALF further on
constexpr int HALF = 1024 + 128;
constexpr int BLK = 2 * HALF;

// ---- the two forms ------------------------------------------------------------------------------------------------
// A form says how many bytes of a row a 32-column step takes, how a sub-block's scales get into the slot's scale area
// (a direct-to-LDS load too: nothing a sub-block needs comes through a register, so no load's destination is carried
// round the loop and every wait in it is one of the counted ones), and how a step's A fragment is made from LDS.

struct DlNoTail {
    static constexpr bool TAIL = false;  // no list of exceptions to the streamed weights
    struct Ctx {};                       // what a form keeps in registers for the whole kernel
};

struct DlF8 : DlNoTail {
    static constexpr int STEPB = 32;
    struct Mat {
        const uint8_t* w;
        const float* scales;
        int sc;  // scales per grid row
        int bm;  // rows per block (a multiple of 16: a tile's sixteen rows share their scales)
        int bn;  // columns per block (a multiple of 32: a step lies in one block)
    };
    __device__ static __forceinline__ Ctx make_ctx(const Mat&) { return Ctx{}; }
    __host__ __device__ static constexpr int scale_bytes(int /*sbs*/) { return 4 * WAVE; }
    __host__ __device__ static constexpr int aux_loads(int /*sbs*/) { return 1; }  // load instructions beside the data's
    __host__ __device__ static constexpr int scale_words(int sbs) { return sbs; }
    // lane t brings the scale of the sub-block's step min(t, SBS - 1): f32 [64] in the scale area, the first SBS of
    // them read. Every lane loads: no branch round the instruction.
    template <int SBS>
    __device__ static __forceinline__ void issue_scales(const Mat& m, int tile, int /*nsteps*/, int step0, uint8_t* dst,
                                                        int lane) {
        static_assert(SBS <= 64, "a lane a step");
        const float* srow = m.scales + (size_t)(tile * 16 / m.bm) * m.sc;
        __builtin_amdgcn_global_load_lds(srow + (step0 + min(lane, SBS - 1)) * 32 / m.bn, (lds_void*)dst, 4, 0, 0);
    }
    // where in a slot's data the lane's reads start (row li, 8-column group lg), and what step t adds to that
    __device__ static __forceinline__ uint32_t lane_off(int li, int lg) {
        return (uint32_t)((li >> 3) * HALF + (li & 7) * 16 + (lg >> 1) * 128 + (lg & 1) * 8);
    }
    __host__ __device__ static constexpr int step_off(int t) { return (t / 4) * BLK + (t % 4) * 256; }
    __device__ static __forceinline__ uint32_t scale_off(int /*li*/, int /*lg*/, int /*sbs*/) { return 0; }
    // the words a lane needs of the scale area for the whole sub-block, from the area + scale_off on
    template <int SBS>
    __device__ static __forceinline__ void read_scales(const uint8_t* mine, uint32_t (&ew)[SBS]) {
#pragma unroll
        for (int t = 0; t < SBS; ++t) ew[t] = reinterpret_cast<const uint32_t*>(mine)[t];
    }
    // p: the slot's data + lane_off + step_off(t)
    template <int N>
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, const uint32_t (&ew)[N], int t, const Ctx&) {
        const uint2 q = *reinterpret_cast<const uint2*>(p);
        const float scale = bits_f32(ew[t]);
        uint32_t w[4];
        FmtF8::widen4(q.x, scale, w);
        FmtF8::widen4(q.y, scale, w + 2);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

struct DlMx4 : DlNoTail {
    static constexpr int STEPB = 16;
    struct Mat {
        const uint8_t* w;
        const uint8_t* scales;
    };
    __device__ static __forceinline__ Ctx make_ctx(const Mat&) { return Ctx{}; }
    __host__ __device__ static constexpr int scale_bytes(int sbs) { return 16 * sbs; }
    __host__ __device__ static constexpr int aux_loads(int /*sbs*/) { return 1; }
    __host__ __device__ static constexpr int scale_words(int sbs) { return sbs / 4; }
    // the e8m0 bytes of the sub-block, row r's SBS bytes as SBS / 4 words: lane l brings word l % (SBS / 4) of row
    // l / (SBS / 4), and they land in lane order, i.e. as [16][SBS] bytes
    template <int SBS>
    __device__ static __forceinline__ void issue_scales(const Mat& m, int tile, int nsteps, int step0, uint8_t* dst,
                                                        int lane) {
        static_assert(SBS % 4 == 0 && 4 * SBS <= 64, "whole words of scale bytes, a lane a word");
        constexpr int per = SBS / 4;
        if (16 * per == WAVE || lane < 16 * per) {  // no branch where every lane has a word
            const int r = lane / per, j = lane - r * per;
            __builtin_amdgcn_global_load_lds(m.scales + (size_t)(tile * 16 + r) * nsteps + step0 + 4 * j, (lds_void*)dst,
                                             4, 0, 0);
        }
    }
    __device__ static __forceinline__ uint32_t lane_off(int li, int lg) {
        return (uint32_t)((li >> 3) * HALF + (li & 7) * 16 + lg * 4);
    }
    __host__ __device__ static constexpr int step_off(int t) { return (t / 8) * BLK + (t % 8) * 128; }
    __device__ static __forceinline__ uint32_t scale_off(int li, int /*lg*/, int sbs) { return (uint32_t)(li * sbs); }
    template <int SBS>
    __device__ static __forceinline__ void read_scales(const uint8_t* mine, uint32_t (&ew)[SBS / 4]) {
#pragma unroll
        for (int j = 0; j < SBS / 4; ++j) ew[j] = *reinterpret_cast<const uint32_t*>(mine + 4 * j);
    }
    template <int N>
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, const uint32_t (&ew)[N], int t, const Ctx&) {
        const uint32_t q = *reinterpret_cast<const uint32_t*>(p);
        const uint32_t ebyte = (ew[t / 4] >> (8 * (t & 3))) & 0xFFu;
        const float s = bits_f32(ebyte << 23);
        uint32_t w[4];
        FmtMx4::widen8(q, s, w);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

// 12 bits a weight in two arrays: the low bytes take the place of the FP8 bytes above (32 a step, the same blocks in
// LDS), the code nibbles (16 bytes a row and step) the place of the scales. SBS 4: the codes of a sub-block are
// 16 rows x 64 bytes, one load instruction (lane l: row l % 16, granule l / 16), in LDS [4 granules = steps][16 rows]
// [16 B]. SBS 8: 16 rows x 128 bytes, two instructions of 8 rows like the data's, [8 granules = steps][8 rows][16 B] a
// half. A fragment is eight low bytes and eight codes zipped through the 16-entry table of high bytes, which the
// lanes keep in four registers. The escapes - weights whose high byte is not in the table; the matrix cores multiply
// the table's last entry in their place - are not this wave's business: see escape_wave below.
// PAIRS: the high bytes come out of the 256-entry pair table (btb_hip_p12_pairs: entry b = the high bytes of the two
// weights whose codes are byte b's nibbles, slot 15 taken as 0), which the escape wave - the one wave here whose loads
// are ordinary ones - brings into LDS before the first tile: eight weights are then four 2-byte LDS reads and four
// byte-permutes in place of the in-register lookup's two dozen instructions.
template <int SBS_, bool PAIRS_>
struct DlP12 {
    static_assert(SBS_ == 4 || SBS_ == 8, "a sub-block's codes are one or two load instructions");
    static constexpr int STEPB = 32;
    static constexpr bool TAIL = true;
    static constexpr bool PAIRS = PAIRS_;
    struct Mat {
        const uint8_t* w;  // lo
        const uint8_t* codes;
        const uint8_t* table;
        const int32_t* esc_idx;
        const uint8_t* esc_val;
        const int32_t* row_ptr;
        const uint16_t* pairs;
    };
    struct Ctx {
        uint4 tbl;
    };
    // the table's sixteen bytes (4-byte aligned: the host checks), read before the kernel stores anything
    __device__ static __forceinline__ Ctx make_ctx(const Mat& m) {
        const u32x4 t = *reinterpret_cast<const u32x4*>(m.table);
        // with the pair table an escape streams as slot 15 = 0, whatever the 16-byte table holds there
        return Ctx{make_uint4(t.x, t.y, t.z, PAIRS ? (t.w & 0x00FFFFFFu) : t.w)};
    }
    // one wave brings the pair table in: four entries a lane
    __device__ static __forceinline__ void stage_pairs(const Mat& m, int lane) {
        const u32x2 v = reinterpret_cast<const u32x2*>(m.pairs)[lane];
        reinterpret_cast<u32x2*>(FmtP12G::pair_table())[lane] = v;
    }
    __host__ __device__ static constexpr int scale_bytes(int sbs) { return sbs == 4 ? 1024 : 2 * (1024 + 128); }
    __host__ __device__ static constexpr int aux_loads(int sbs) { return sbs == 4 ? 1 : 2; }
    __host__ __device__ static constexpr int scale_words(int sbs) { return sbs; }
    template <int SBS>
    __device__ static __forceinline__ void issue_scales(const Mat& m, int tile, int nsteps, int step0, uint8_t* dst,
                                                        int lane) {
        static_assert(SBS == SBS_, "the form's own sub-block");
        const size_t rowbytes2 = (size_t)nsteps * 16;
        if (SBS == 4) {
            const uint8_t* src = m.codes + ((size_t)tile * 16 + (lane & 15)) * rowbytes2 + (size_t)step0 * 16 + (lane >> 4) * 16;
            __builtin_amdgcn_global_load_lds(src, (lds_void*)dst, 16, 0, 0);
        } else {
            const uint8_t* src = m.codes + ((size_t)tile * 16 + (lane & 7)) * rowbytes2 + (size_t)step0 * 16 + (lane >> 3) * 16;
            __builtin_amdgcn_global_load_lds(src, (lds_void*)dst, 16, 0, 0);
            __builtin_amdgcn_global_load_lds(src + 8 * rowbytes2, (lds_void*)(dst + 1024 + 128), 16, 0, 0);
        }
    }
    __device__ static __forceinline__ uint32_t lane_off(int li, int lg) {
        return (uint32_t)((li >> 3) * (1024 + 128) + (li & 7) * 16 + (lg >> 1) * 128 + (lg & 1) * 8);
    }
    __host__ __device__ static constexpr int step_off(int t) { return (t / 4) * (2 * (1024 + 128)) + (t % 4) * 256; }
    __device__ static __forceinline__ uint32_t scale_off(int li, int lg, int sbs) {
        return (uint32_t)(sbs == 4 ? li * 16 + lg * 4 : (li >> 3) * (1024 + 128) + (li & 7) * 16 + lg * 4);
    }
    template <int SBS>
    __device__ static __forceinline__ void read_scales(const uint8_t* mine, uint32_t (&ew)[SBS]) {
#pragma unroll
        for (int t = 0; t < SBS; ++t) ew[t] = *reinterpret_cast<const uint32_t*>(mine + t * (SBS == 4 ? 256 : 128));
    }
    template <int N>
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, const uint32_t (&ew)[N], int t, const Ctx& ctx) {
        const uint2 l = *reinterpret_cast<const uint2*>(p);
        uint32_t w[4];
        if constexpr (PAIRS)
            FmtP12G::widen8(ew[t], l.x, l.y, w);
        else
            FmtP12::widen8(ctx.tbl, ew[t], l.x, l.y, w);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

// ---- the pack12 escapes: a wave of their own ------------------------------------------------------------------------
// The waves that stream a tile never load into a register (every wait of theirs is a count of direct-to-LDS loads),
// so the escapes of a tile - list entries, the low byte and the x values each one names: ordinary dependent loads -
// go to one more wave of the workgroup, whose waits are its own. Per tile it builds a partial tile like the others'
// out of "the streamed term out, the true term in" for every escape of the tile's sixteen rows, thirty-two escapes at
// a time (lane j: escape j % 32, eight of the sixteen x rows j / 32), added in list order whatever M is, and meets
// the other waves at the tile's barrier. The list positions of a tile's escapes are asked for two tiles ahead, the
// first thirty-two entries one tile ahead, so a tile waits for one trip to memory (low bytes and x), not three.

constexpr int ESC_SCRATCH = 32 * 16 * 4 + 32 * 4 + 16;  // [32 escapes][16 x rows] f32, [32] rows, two flags

struct EscEntry {
    uint32_t idx, val;
};
template <class Mat>
__device__ __forceinline__ EscEntry esc_request(const Mat& mat, int first, int e1, int lane) {
    // every load unconditional: a lane with no escape reads a harmless place (the row index, the table)
    const int e = first + (lane & 31);
    const bool ok = e < e1;
    const int32_t* pi = ok ? mat.esc_idx + e : mat.row_ptr;
    const uint8_t* pv = ok ? mat.esc_val + e : mat.table;
    const uint32_t i = (uint32_t)*pi;
    EscEntry c;
    c.val = *pv;
    c.idx = ok ? i : 0u;
    return c;
}
struct EscOperands {
    uint32_t lo;
    int row;         // of the whole matrix
    uint32_t xv[4];  // eight x values, two a register
};
template <class Mat>
__device__ __forceinline__ EscOperands esc_operands(const Mat& mat, const EscEntry& c, const uint16_t* xrows, int C,
                                                    int have, int lane) {
    EscOperands o;
    o.lo = mat.w[c.idx];
    o.row = (int)(c.idx / (uint32_t)C);
    const uint32_t col = c.idx - (uint32_t)o.row * (uint32_t)C;
    const int m0 = (lane >> 5) * 8;
#pragma unroll
    for (int q = 0; q < 4; ++q) {  // sixteen rows of at most 2^24 columns: the offsets fit 32 bits
        const uint32_t o0 = (uint32_t)min(m0 + 2 * q, have - 1) * (uint32_t)C + col;
        const uint32_t o1 = (uint32_t)min(m0 + 2 * q + 1, have - 1) * (uint32_t)C + col;
        o.xv[q] = (uint32_t)xrows[o0] | ((uint32_t)xrows[o1] << 16);
    }
    return o;
}
// cnt escapes: their terms into LDS, then added to the lane's rows (x row li, the tile's rows 4 lg ..) in list order
__device__ __forceinline__ void esc_apply(const uint4& tbl, const EscEntry& c, const EscOperands& op, int tile, int cnt,
                                          int lane, uint8_t* scratch, f32x4& s) {
    float* dl = reinterpret_cast<float*>(scratch);            // [32 escapes][16 x rows]
    int* rw = reinterpret_cast<int*>(scratch + 32 * 16 * 4);  // [32] the escape's row within the tile
    const uint32_t t15 = tbl.w >> 24;
    const int li = lane & 15, row0 = (lane >> 4) * 4;
    const float streamed = bits_f32((t15 << 24) | (op.lo << 16));
    const float truth = bits_f32((c.val << 24) | (op.lo << 16));
    float d[8];
#pragma unroll
    for (int q = 0; q < 8; ++q) {
        const float xv = (q & 1) ? bf16hi_f32(op.xv[q / 2]) : bf16lo_f32(op.xv[q / 2]);
        d[q] = fmaf(truth, xv, -(streamed * xv));
    }
    float4* o = reinterpret_cast<float4*>(dl + (lane & 31) * 16 + (lane >> 5) * 8);
    o[0] = make_float4(d[0], d[1], d[2], d[3]);
    o[1] = make_float4(d[4], d[5], d[6], d[7]);
    rw[lane & 31] = op.row - tile * 16;  // both halves write the same value
#pragma unroll 2
    for (int j = 0; j < cnt; ++j) {
        const int k = rw[j] - row0;
        const float v = dl[j * 16 + li];
        s.x = k == 0 ? s.x + v : s.x;
        s.y = k == 1 ? s.y + v : s.y;
        s.z = k == 2 ? s.z + v : s.z;
        s.w = k == 3 ? s.w + v : s.w;
    }
}
// part: the two sets of KS + 1 partial tiles; this wave's is number KS. flags[k & 1]: whether tile k has escapes at all
// (a tile without gets nothing added, not a tile of zeros: a sum of -0 stays -0).
template <class DF, int KS>
__device__ __forceinline__ void escape_wave(const typename DF::Mat& mat, const typename DF::Ctx& ctx,
                                            const uint16_t* xrows, int C, int M, int first, int grid, int nt, int lane,
                                            uint8_t* scratch, f32x4* part) {
    int* flags = reinterpret_cast<int*>(scratch + 32 * 16 * 4 + 32 * 4);
    auto span_of = [&](int k) {
        const int t = first + min(k, nt - 1) * grid;
        return make_int2(mat.row_ptr[t * 16], mat.row_ptr[t * 16 + 16]);
    };
    int2 span = span_of(0), span_next = span_of(1);
    EscEntry nxt = esc_request(mat, span.x, span.y, lane);
    for (int k = 0; k < nt; ++k) {
        const int tile = first + k * grid;
        const int e0 = __builtin_amdgcn_readfirstlane(span.x), e1 = __builtin_amdgcn_readfirstlane(span.y);
        EscEntry cur = nxt;
        EscOperands op = esc_operands(mat, cur, xrows, C, M, lane);
        span = span_next;
        nxt = esc_request(mat, span.x, span.y, lane);
        span_next = span_of(k + 2);
        f32x4 s = f32x4{0.f, 0.f, 0.f, 0.f};
        if (e0 < e1) {
            esc_apply(ctx.tbl, cur, op, tile, min(32, e1 - e0), lane, scratch, s);
            for (int f = e0 + 32; f < e1; f += 32) {  // a crowd: fetched here
                cur = esc_request(mat, f, e1, lane);
                op = esc_operands(mat, cur, xrows, C, M, lane);
                esc_apply(ctx.tbl, cur, op, tile, min(32, e1 - f), lane, scratch, s);
            }
        }
        part[(size_t)(k & 1) * (KS + 1) * WAVE + KS * WAVE + lane] = s;
        if (lane == 0) flags[k & 1] = e0 < e1 ? 1 : 0;
        asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    }
}

// ---- the kernel ---------------------------------------------------------------------------------------------------

// whether a form brings a table into LDS before the first tile (pack12 with its pair table)
template <class DF, class = void>
struct dl_pairs : std::false_type {};
template <class DF>
struct dl_pairs<DF, std::enable_if_t<DF::PAIRS>> : std::true_type {};

// The loads of one sub-block into `slot` (tile `tile`, the wave's steps step0 .. step0 + SBS - 1: GB column blocks).
// `slot` is a __restrict__ parameter on purpose, here and in sub_block below: the compiler orders an LDS read behind
// every direct-to-LDS load that may alias it - behind all of them when it cannot tell them apart, which would drain
// the ring at every sub-block. The ring slot being filled and the slot being read are told apart by these
// no-alias promises (they never coincide: a slot is refilled only after its last read), and the real dependence - the
// slot read now was filled NBUF - 1 sub-blocks ago - is kept by the counted waits.
template <class DF, int GB, int SBS>
__device__ __forceinline__ void issue_loads(const typename DF::Mat& mat, uint8_t* __restrict__ slot, int tile, int step0,
                                            int nsteps, size_t rowbytes, int lane) {
    const uint8_t* src =
        mat.w + ((size_t)tile * 16 + (lane & 7)) * rowbytes + (size_t)step0 * DF::STEPB + (lane >> 3) * 16;
#pragma unroll
    for (int gb = 0; gb < GB; ++gb) {
        __builtin_amdgcn_global_load_lds(src + gb * 128, (lds_void*)(slot + gb * BLK), 16, 0, 0);
        __builtin_amdgcn_global_load_lds(src + gb * 128 + 8 * rowbytes, (lds_void*)(slot + gb * BLK + HALF), 16, 0, 0);
    }
    DF::template issue_scales<SBS>(mat, tile, nsteps, step0, slot + GB * BLK, lane);
}

// one sub-block multiplied out of `cur` while `fill` (another slot) receives the loads of the sub-block NBUF - 1 ahead
template <class DF, int SPW, int GB, int SBS, int NBUF>
__device__ __forceinline__ f32x4 sub_block(const typename DF::Mat& mat, const typename DF::Ctx& ctx,
                                           const uint8_t* __restrict__ cur, uint8_t* __restrict__ fill, bool do_fill,
                                           int fill_tile, int fill_step0, int nsteps, size_t rowbytes, int lane, int li,
                                           int lg, int behind, int sb, u32x4 (&xb)[SPW], f32x4 acc, int xparts = -1,
                                           bool x_none = false) {
    constexpr int LOADS = 2 * GB + DF::aux_loads(SBS);  // load instructions a sub-block
    if (do_fill) issue_loads<DF, GB, SBS>(mat, fill, fill_tile, fill_step0, nsteps, rowbytes, lane);
    // `cur` has landed once at most the loads issued behind it are outstanding
    uint32_t roff = DF::lane_off(li, lg), soff = DF::scale_off(li, lg, SBS);
    // xparts >= 0: the kernel's first tile - behind this sub-block are also that many of the parts of x (SBS loads each)
    if (xparts >= 0) {
        static_assert(SBS % 4 == 0, "parts of x in fours");
        wait_first<LOADS, NBUF - 1, SBS>(behind, xparts, roff, soff);
#pragma unroll
        for (int t = 0; t < SBS; t += 4)
            landed(xb[sb * SBS + t], xb[sb * SBS + t + 1], xb[sb * SBS + t + 2], xb[sb * SBS + t + 3]);
        if (x_none) {  // uniform: a sub-block past the row's end (its weights are some other sub-block's, its x zeros)
#pragma unroll
            for (int t = 0; t < SBS; ++t) xb[sb * SBS + t] = u32x4{0u, 0u, 0u, 0u};
        }
    } else
        wait_behind<LOADS, NBUF - 1>(behind, roff, soff);
    __builtin_amdgcn_sched_barrier(0);
    const uint8_t* rowp = cur + roff;
    uint32_t ew[DF::scale_words(SBS)];  // what the lane needs of the sub-block's scales
    DF::template read_scales<SBS>(cur + GB * BLK + soff, ew);
#pragma unroll
    for (int t = 0; t < SBS; ++t) {
        const int i = sb * SBS + t;  // the wave's step: a compile-time index once the callers' loops are unrolled
        const bf16x8 a = DF::frag(rowp + DF::step_off(t), ew, t, ctx);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, xb[i]), acc, 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    return acc;
}

// the KS partial tiles folded in wave order (then the escape wave's, where the form has one and the tile any escape)
// and the tile's outputs written; `mine` is this tile's set of partials
template <int KS, bool TAIL>
__device__ __forceinline__ void fold_tile(f32x4* __restrict__ mine, const int* flag, f32x4 acc, int wv, int lane, int li,
                                          int lg, int M, int R, int tile, uint16_t* __restrict__ y) {
    mine[wv * WAVE + lane] = acc;
    // A barrier for LDS traffic only: the partial tile above has been written (LDS operations of a wave complete in
    // order) before the wave arrives. __syncthreads() would also wait for every load in flight - the ring's - and
    // drain it at each tile's end; nothing the other waves read here comes from those loads.
    asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
    if (wv == 0) {
        f32x4 s = mine[lane];
        for (int w2 = 1; w2 < KS; ++w2) {
            const f32x4 o = mine[w2 * WAVE + lane];
            s.x += o.x;
            s.y += o.y;
            s.z += o.z;
            s.w += o.w;
        }
        if (TAIL && *flag != 0) {  // uniform
            const f32x4 o = mine[KS * WAVE + lane];
            s.x += o.x;
            s.y += o.y;
            s.z += o.z;
            s.w += o.w;
        }
        if (li < M) {
            uint16_t* o = y + (size_t)li * R + tile * 16 + lg * 4;
            o[0] = f32_bf16(s.x);
            o[1] = f32_bf16(s.y);
            o[2] = f32_bf16(s.z);
            o[3] = f32_bf16(s.w);
        }
    }
}

// KS waves a workgroup, each the owner of up to SPW steps of every row; GB 128-byte column blocks a sub-block; NBUF ring
// slots a wave. A tile is MAXSB sub-blocks a wave; the tile loop's body covers a multiple of NBUF of them, so every
// sub-block's slot is a compile-time number. One tile of up to sixteen x rows. A row is a whole number of sub-blocks,
// more than KS (MAXSB - 1) and at most KS MAXSB of them: where that is fewer than KS MAXSB, the waves left without a
// last sub-block stream their first one again against zeros of x, so that every wave issues the same loads.
//
// LEAD is set by the host when every workgroup has tiles enough that each sub-block of its first tile has its full
// NBUF - 1 sub-blocks asked for behind it: every count in that tile is then a constant, and the tile half the code of
// the general form, which matters for a path that runs once, from a cold instruction cache, ahead of everything else
// (FP8 [18432, 7168], 8 rows: 31.4 us with it, 32.7 with the general form).
template <class DF, int KS, int SPW, int GB, int NBUF, bool LEAD>
__global__ void __launch_bounds__((KS + (DF::TAIL ? 1 : 0)) * 64)
    gemv_mfma_dl(typename DF::Mat mat, const uint4* __restrict__ x, uint16_t* __restrict__ y, int R, int C, int M) {
    constexpr int SBS = GB * 128 / DF::STEPB;  // steps a sub-block
    constexpr int SLOT = GB * BLK + DF::scale_bytes(SBS);
    constexpr int MAXSB = SPW / SBS;
    constexpr int TPB = MAXSB >= NBUF ? 1 : NBUF / MAXSB;  // tiles a loop body covers
    constexpr int NW = KS + (DF::TAIL ? 1 : 0);            // waves, and partial tiles a set
    constexpr int LOADS = 2 * GB + DF::aux_loads(SBS);
    static_assert(SPW % SBS == 0 && SLOT % 16 == 0 && (SPW * DF::STEPB) % 128 == 0, "shape");
    static_assert(NBUF >= 2 && NBUF <= 7 && MAXSB <= 7, "ring depth; at most six parts of x behind a sub-block");
    static_assert((NBUF - 1) * LOADS + (MAXSB - 1) * SBS < 64, "the first tile's waits count up to 63 loads");
    static_assert((MAXSB >= NBUF && MAXSB % NBUF == 0) || (MAXSB < NBUF && NBUF % MAXSB == 0), "slots by position");
    // KS rings of NBUF slots, two sets of NW partial tiles, the escape wave's exchange buffer
    extern __shared__ __align__(16) uint8_t lds[];
    const int lane = threadIdx.x & (WAVE - 1);
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int li = lane & 15, lg = lane >> 4;
    f32x4* part = reinterpret_cast<f32x4*>(lds + (size_t)KS * NBUF * SLOT);
    [[maybe_unused]] uint8_t* esc = lds + (size_t)KS * NBUF * SLOT + 2 * (size_t)NW * WAVE * sizeof(f32x4);
    [[maybe_unused]] const int* flags = reinterpret_cast<const int*>(esc + 32 * 16 * 4 + 32 * 4);
    const typename DF::Ctx ctx = DF::make_ctx(mat);

    const int nsteps = C / 32;
    const int ntiles = R / 16;
    const int grid = (int)gridDim.x, first = (int)blockIdx.x;
    const int nt = first < ntiles ? (ntiles - first + grid - 1) / grid : 0;  // this workgroup's tiles
    if constexpr (DF::TAIL) {
        if (wv == KS) {
            if constexpr (dl_pairs<DF>::value) {  // the pair table into LDS; the streaming waves wait below
                DF::stage_pairs(mat, lane);
                asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory");
            }
            escape_wave<DF, KS>(mat, ctx, reinterpret_cast<const uint16_t*>(x), C, M, first, grid, nt, lane, esc, part);
            return;
        }
    }
    uint8_t* ring = lds + (size_t)wv * NBUF * SLOT;
    // the wave's steps: its sub-blocks are dealt round the waves, so that the workgroup's waves, which run more or less
    // abreast, ask for neighbouring blocks of a row at about the same time (a little faster than a slice of SPW
    // consecutive steps a wave: 30.5 against 31.8 us on FP8 [18432, 7168])
    const int s0 = wv * SBS;
    constexpr int SB_STEP = KS * SBS;  // from one sub-block of the wave to its next, in steps
    const size_t rowbytes = (size_t)nsteps * DF::STEPB;
    const int chunk4 = C / 8;  // uint4 per row of x
    // whether the wave's last sub-block exists (uniform), and the steps sub-block j of a tile starts at
    const bool last_ok = s0 + (MAXSB - 1) * SB_STEP < nsteps;
    auto step0_of = [&](int j) { return (j == MAXSB - 1 && !last_ok) ? s0 : s0 + j * SB_STEP; };

    const int total = nt * MAXSB;  // the wave's sub-blocks
    // sub-block q of the wave: tile first + (q / MAXSB) grid, steps (q % MAXSB) SBS .. of the wave's slice, slot q % NBUF.
    //
    // The x fragments of the wave's steps stay in registers for the whole kernel (row li of x, the lane's 8 columns of
    // each step); part j of them - SBS loads - is what sub-block j of any tile multiplies by. They and the ring's first
    // loads are asked for in the order the first tile uses them: x part 0, sub-block 0, x part 1, sub-block 1, ...
    // Loads come back in that order, so the first tile's sub-block j can start as soon as its own weights and its own
    // part of x are there, the later parts still on their way out of L2 (every CU reads all of x, 115 KB at 8 rows,
    // and all at once: asked for and waited for in one piece it held the first product back by 2.7 us per 8 rows).
    u32x4 xb[SPW];
    const u32x4* xr = reinterpret_cast<const u32x4*>(x) + (size_t)min(li, M - 1) * chunk4 + lg;
#pragma unroll
    for (int q = 0; q < (NBUF - 1 > MAXSB ? NBUF - 1 : MAXSB); ++q) {
        if (q < MAXSB) {
            const u32x4* xq = xr + (size_t)step0_of(q) * 4;
#pragma unroll
            for (int t = 0; t < SBS; ++t) {
                xb[q * SBS + t] = load_untracked(xq + t * 4);
            }
            __builtin_amdgcn_sched_barrier(0);  // issued here, not where the scheduler would like them
        }
        if (q < NBUF - 1) {
            if (LEAD || q < total)
                issue_loads<DF, GB, SBS>(mat, ring + (q % NBUF) * SLOT, first + (q / MAXSB) * grid,
                                         step0_of(q % MAXSB), nsteps, rowbytes, lane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // the pair table is in LDS once the escape wave has arrived (a barrier for LDS traffic only: the loads above stay out)
    if constexpr (dl_pairs<DF>::value) asm volatile("s_barrier" ::: "memory");
    // One body of the tile loop: TPB tiles. FIRST: the kernel's first body, whose first tile's waits let the parts of x
    // asked for behind a sub-block's own stay outstanding.
    auto body = [&](int k0, auto first_tag) {
        constexpr bool FIRST = decltype(first_tag)::value;
#pragma unroll
        for (int kk = 0; kk < TPB; ++kk) {
            const int k = k0 + kk;
            if (k < nt) {  // uniform
                const int tile = first + k * grid;
                f32x4 acc = f32x4{0.f, 0.f, 0.f, 0.f};
#pragma unroll
                for (int sb = 0; sb < MAXSB; ++sb) {
                    const int q = k * MAXSB + sb;
                    // compile-time slots: q % NBUF = (kk * MAXSB + sb) % NBUF, because the body covers a multiple of NBUF
                    const int cur_slot = (kk * MAXSB + sb) % NBUF, fill_slot = (kk * MAXSB + sb + NBUF - 1) % NBUF;
                    const int qf = q + NBUF - 1;  // the sub-block asked for now, into the slot the previous one left
                    const bool sure = LEAD && FIRST && kk == 0;  // the first tile of a workgroup with tiles enough
                    const int behind = sure ? NBUF - 1 : min(NBUF - 1, total - 1 - q);
                    // First tile: the weights of its sub-blocks 0 .. NBUF - 2 were asked for between the parts of x, each
                    // behind its own part, so x parts sb + 1 .. MAXSB - 1 are behind such a sub-block's weights; the later
                    // sub-blocks' weights were asked for by this tile, behind all of x.
                    const int xbehind = sb < NBUF - 1 ? MAXSB - 1 - sb : 0;
                    acc = sub_block<DF, SPW, GB, SBS, NBUF>(
                        mat, ctx, ring + cur_slot * SLOT, ring + fill_slot * SLOT, sure || qf < total,
                        first + (qf / MAXSB) * grid, step0_of(qf % MAXSB), nsteps, rowbytes, lane, li, lg, behind, sb, xb,
                        acc, FIRST && kk == 0 ? xbehind : -1, sb == MAXSB - 1 && !last_ok);
                }
                fold_tile<KS, DF::TAIL>(part + (size_t)(k & 1) * NW * WAVE, flags + (k & 1), acc, wv, lane, li, lg, M, R,
                                        tile, y);
            }
        }
    };
    body(0, std::true_type{});
    for (int k0 = TPB; k0 < nt; k0 += TPB) body(k0, std::false_type{});
}

template <class DF, int KS, int SPW, int GB, int NBUF>
static int32_t launch_dl(const typename DF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    constexpr int SBS = GB * 128 / DF::STEPB;
    constexpr int SLOT = GB * BLK + DF::scale_bytes(SBS);
    constexpr int MAXSB = SPW / SBS;
    constexpr int NW = KS + (DF::TAIL ? 1 : 0);
    const size_t lds = (size_t)KS * NBUF * SLOT + 2 * (size_t)NW * WAVE * sizeof(f32x4) + (DF::TAIL ? ESC_SCRATCH : 0);
    const int nsteps = C / 32;
    // a row: whole sub-blocks, every wave a first one, only the waves' last ones missing
    const bool row_ok = C % 32 == 0 && nsteps % SBS == 0 && nsteps > KS * (MAXSB - 1) * SBS && nsteps <= KS * SPW;
    constexpr size_t fixed = dl_pairs<DF>::value ? 512 : 0;  // the pair table, a static array beside the dynamic ones
    if (lds + fixed > (size_t)device_info().lds_bytes || !row_ok || R % 16 != 0 || M < 1 || M > 16) {
        set_error("gemv_mfma_dl: a shape this kernel does not take");
        return ERR_DOMAIN;
    }
    const int ntiles = R / 16;
    // The rings take most of a CU's LDS: one workgroup a CU, and every CU one. What bounds a workgroup is how fast its
    // own waves turn bytes into products (each CU takes in 21-23 GB/s here, whatever the others do), so the workgroup
    // with the most tiles sets the time and spreading the tiles evenly over fewer workgroups buys nothing: FP8
    // [18432, 7168] 231 workgroups of 5 tiles and 256 of 4 or 5 take the same 31 us, pack12 [9728, 2560] 203 of 3 take
    // 15.2 and 256 of 2 or 3 14.6.
    const int cap = device_info().cus;
    int grid = std::min(ntiles, cap);
    if (tuning("mfma_direct_grid") > 0) grid = std::min(std::min(tuning("mfma_direct_grid"), cap), ntiles);
    const bool lead = (ntiles / grid) * MAXSB >= MAXSB + NBUF - 1;  // the workgroup with the fewest tiles has enough
    auto kern = lead ? gemv_mfma_dl<DF, KS, SPW, GB, NBUF, true> : gemv_mfma_dl<DF, KS, SPW, GB, NBUF, false>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(NW * 64), lds, st, mat, static_cast<const uint4*>(x),
                       static_cast<uint16_t*>(y), R, C, M);
    return hip_status(hipGetLastError(), "gemv_mfma_dl launch");
}

// The shapes this kernel takes: 16-row tiles, at most sixteen rows of x, and the row lengths it has shapes for, by steps
// of 32 columns: 224 (7168 columns, the block-scaled forms' long rows), 80 (2560), 97..128 (to 4096) and 281..336
// (around 9728) - classes 0..3, -1: none. A row is a whole number of the class's sub-blocks (`unit` steps).
static int row_class(int C, int unit_narrow, int unit_wide) {
    if (C % 32 != 0) return -1;
    const int nsteps = C / 32;
    if (nsteps == 224) return 0;
    if (nsteps == 80) return 1;
    if (nsteps > 96 && nsteps <= 128 && nsteps % unit_narrow == 0) return 2;
    if (nsteps > 280 && nsteps <= 336 && nsteps % unit_wide == 0) return 3;
    return -1;
}
static bool pass_ok(int R, int M) { return R % 16 == 0 && M >= 1 && M <= 16 && tuning("mfma_direct") != 0; }

// MXFP4: sub-blocks of 8 steps on the shorter rows, of 16 on the long ones (19 of them over seven waves at 9728 columns)
bool mfma_dl_fits(int R, int C, int M) { return pass_ok(R, M) && row_class(C, 8, 16) >= 0; }
int32_t gemv_mfma_dl_mxfp4(const void* blocks, const void* scales, const void* x, void* y, int R, int C, int M,
                           hipStream_t st) {
    const DlMx4::Mat mat{static_cast<const uint8_t*>(blocks), static_cast<const uint8_t*>(scales)};
    switch (row_class(C, 8, 16)) {
        case 0: return launch_dl<DlMx4, 7, 32, 2, 4>(mat, x, y, R, C, M, st);
        case 1: return launch_dl<DlMx4, 5, 16, 1, 4>(mat, x, y, R, C, M, st);
        case 2: return launch_dl<DlMx4, 8, 16, 1, 4>(mat, x, y, R, C, M, st);
        case 3: return launch_dl<DlMx4, 7, 48, 2, 3>(mat, x, y, R, C, M, st);
        default: set_error("gemv_mfma_dl: a row length this kernel has no shape for"); return ERR_DOMAIN;
    }
}

// FP8: sub-blocks of 4 steps, of 8 at 9728 columns; blocks a whole number of tiles tall and of steps wide
bool mfma_dl_fits_fp8(int R, int C, int M, int bm, int bn) {
    return pass_ok(R, M) && row_class(C, 4, 8) >= 0 && bm % 16 == 0 && bn % 32 == 0;
}
int32_t gemv_mfma_dl_fp8(const void* w, const float* scales, int sc, int bm, int bn, const void* x, void* y, int R,
                         int C, int M, hipStream_t st) {
    const DlF8::Mat mat{static_cast<const uint8_t*>(w), scales, sc, bm, bn};
    switch (row_class(C, 4, 8)) {
        case 0: return launch_dl<DlF8, 8, 28, 1, 7>(mat, x, y, R, C, M, st);
        case 1: return launch_dl<DlF8, 10, 8, 1, 4>(mat, x, y, R, C, M, st);
        case 2: return launch_dl<DlF8, 8, 16, 1, 4>(mat, x, y, R, C, M, st);
        case 3: return launch_dl<DlF8, 7, 48, 2, 3>(mat, x, y, R, C, M, st);
        default: set_error("gemv_mfma_dl: a row length this kernel has no shape for"); return ERR_DOMAIN;
    }
}

// pack12: rows of 2560 columns (20 sub-blocks of 4 steps: ten waves, two each), 3073..4096 (eight waves, four each),
// 9217..10752 in whole 256-column sub-blocks (seven waves, six sub-blocks of 8 steps each)
bool mfma_dl_fits_p12(int R, int C, int M) {
    const int cls = row_class(C, 4, 8);
    return pass_ok(R, M) && cls >= 1;
}
int32_t gemv_mfma_dl_p12(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const uint16_t* pairs,
                         const int32_t* esc_idx, const uint8_t* esc_val, const int32_t* row_ptr, const void* x, void* y,
                         int R, int C, int M, hipStream_t st) {
    // the pair table (made at upload) where the caller has one and it can be read eight bytes a lane
    const bool tab = pairs != nullptr && (reinterpret_cast<uintptr_t>(pairs) & 7u) == 0 && tuning("p12_pair_table") != 0;
#define P12DL(SB, KS, SPW, GB, NB)                                                                                    \
    return tab ? launch_dl<DlP12<SB, true>, KS, SPW, GB, NB>(                                                         \
                     DlP12<SB, true>::Mat{lo, hi4, table, esc_idx, esc_val, row_ptr, pairs}, x, y, R, C, M, st)       \
               : launch_dl<DlP12<SB, false>, KS, SPW, GB, NB>(                                                        \
                     DlP12<SB, false>::Mat{lo, hi4, table, esc_idx, esc_val, row_ptr, pairs}, x, y, R, C, M, st)
    switch (row_class(C, 4, 8)) {
        case 1: P12DL(4, 10, 8, 1, 4);
        case 2: P12DL(4, 8, 16, 1, 4);
        case 3:  // its rings and partial tiles leave 112 bytes of the CU's LDS: no room for the table
            return launch_dl<DlP12<8, false>, 7, 48, 2, 3>(
                DlP12<8, false>::Mat{lo, hi4, table, esc_idx, esc_val, row_ptr, pairs}, x, y, R, C, M, st);
        default: set_error("gemv_mfma_dl: a row length this kernel has no shape for"); return ERR_DOMAIN;
    }
#undef P12DL
}

}  // namespace btb
