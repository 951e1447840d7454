// The verify widths (M = 5..32 rows of x) on the matrix cores, with the weights brought in the way memory likes them.
//
// A v_mfma_f32_16x16x32_bf16 wants its A operand as "lane l: row l % 16, eight columns"; loading it that way straight
// from memory makes every load instruction touch sixteen rows, 64 bytes of each, and HBM then runs at half speed
// (measured: 3.1 TB/s against 4.5 for the same bytes read in long runs). So here a wave reads its share of the 16-row
// tile in long contiguous runs per row (one 16-byte load per lane, a load instruction covering one or a few whole row
// segments), parks the bytes in a private slab of LDS - still in their stored form - and reads them back in the MFMA's
// layout, widening the packed forms to bf16 in registers on the way (FP8: v_cvt_pk_f32_fp8, one multiply by the block
// scale, v_cvt_pk_bf16_f32; MXFP4: v_cvt_scalef32_pk_bf16_fp4). Nothing is synchronised between waves inside a tile:
// a wave's LDS traffic is its own and executes in order.
//
// Decomposition. A workgroup of KS waves owns 16 rows of W at a time; wave k owns a fixed slice of the columns -
// `spw` consecutive 32-column MFMA steps - and keeps the x fragments of that slice (operand B of every step, for one or
// two 16-row tiles of x) in registers for the whole kernel, so x is read once per wave instead of once per row tile. The workgroup walks row
// tiles (blockIdx.x, + gridDim.x, ...); the next sub-block's loads - also across a tile's end - are in flight while the
// current one is multiplied. The KS partial tiles fold through LDS in wave order. KS and the slices come from C alone,
// so a row's bits depend on neither M nor R nor the launch.
// The reference's counterpart is btb_gemv_mma_bf16 (native/cuda/btb_gemv_mma.cuh:1-214); it has no packed forms.

#include <type_traits>

#include "btb_common.hpp"
#include "btb_formats.hpp"
#include "btb_stream.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

namespace btb {


// ---- the stored forms: bytes a row contributes to a 32-column step, and the step's A fragment out of LDS ----------

// STEPB2 > 0: a second byte stream per row (its own slab), for the form that keeps a weight in two arrays
struct MfNoTail {
    static constexpr int TWO_TILES_STEPS = 128;  // the longest row (in steps) whose kernel holds two tiles of x rows
    static constexpr int STEPB2 = 0;
    static constexpr bool TAIL = false;
    static constexpr int TAIL_BYTES = 0;
    struct Tail {};
    __device__ static __forceinline__ int2 tail_span(...) { return make_int2(0, 0); }
    __device__ static __forceinline__ bool tail_any(const Tail&) { return false; }
};

struct MfBf16 : MfNoTail {
    static constexpr int STEPB = 64;
    static constexpr int SB_NARROW = 8, SB_WIDE = 8;  // steps per sub-block: rows up to 4096 columns, wider rows
    struct Mat {
        const uint8_t* w;
    };
    struct RowInfo {};
    __device__ static __forceinline__ RowInfo row_info(const Mat&, int, int) { return RowInfo{}; }
    // p: the lane's row in the slab, at the step's first byte; g: the lane's 8-column group of the step
    // the step's scale for this lane (none here), requested a sub-block ahead of its use
    template <int SB>
    __device__ static __forceinline__ void scales(const Mat&, const RowInfo&, int /*g*/, int /*step0*/, int /*nsteps*/,
                                                  uint32_t (&)[SB]) {}
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, int g, uint32_t /*scale*/) {
        return __builtin_bit_cast(bf16x8, *reinterpret_cast<const uint4*>(p + g * 16));
    }
};

struct MfF8 : MfNoTail {
    static constexpr int STEPB = 32;
    static constexpr int SB_NARROW = 16, SB_WIDE = 8;  // the wide rows' x fragments leave room for four loads in flight
    struct Mat {
        const uint8_t* w;
        const float* scales;
        int sc;  // scales per grid row
        int bm;  // rows per block
        int bn;  // columns per block (a multiple of 16)
    };
    struct RowInfo {
        const float* srow;
    };
    __device__ static __forceinline__ RowInfo row_info(const Mat& m, int row, int) {
        return RowInfo{m.scales + (size_t)(row / m.bm) * m.sc};
    }
    // The scales of SB steps from step0 on, for the lane's row and its 8-column group g - every load unconditional (a
    // step past the row's end takes the row's last scale, unused). Blocks a multiple of 128 columns wide, reached at
    // a multiple of four steps: one scale serves four steps, a quarter of the loads. Otherwise one division finds
    // the first block and the rest follow by stepping (a block is at least 16 columns, a step is 32).
    template <int SB>
    __device__ static __forceinline__ void scales(const Mat& m, const RowInfo& ri, int g, int step0, int nsteps,
                                                  uint32_t (&scl)[SB]) {
        const int last = (nsteps * 32 - 1) / m.bn;
        if (m.bn % 128 == 0 && step0 % 4 == 0 && SB % 4 == 0) {
            const int b0 = step0 * 32 / m.bn, per = m.bn / 128;  // `per` groups of four steps share a block
            int left = per - (step0 / 4) % per, b = b0;
#pragma unroll
            for (int q = 0; q < SB / 4; ++q) {
                const uint32_t v = f32_bits(ri.srow[min(b, last)]);
#pragma unroll
                for (int t = 0; t < 4; ++t) scl[4 * q + t] = v;
                if (--left == 0) {
                    ++b;
                    left = per;
                }
            }
            return;
        }
        const int col0 = step0 * 32 + g * 8;
        int b = col0 / m.bn, rem = col0 - b * m.bn;
#pragma unroll
        for (int t = 0; t < SB; ++t) {
            scl[t] = f32_bits(ri.srow[min(b, last)]);
            rem += 32;
#pragma unroll
            for (int k = 0; k < 2; ++k) {
                const bool over = rem >= m.bn;
                b += over ? 1 : 0;
                rem -= over ? m.bn : 0;
            }
        }
    }
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, int g, uint32_t scale) {
        const uint2 q = *reinterpret_cast<const uint2*>(p + g * 8);
        const float s = bits_f32(scale);
        uint32_t w[4];
        FmtF8::widen4(q.x, s, w);
        FmtF8::widen4(q.y, s, w + 2);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

struct MfMx4 : MfNoTail {
    static constexpr int STEPB = 16;
    static constexpr int SB_NARROW = 16, SB_WIDE = 16;
    struct Mat {
        const uint8_t* w;
        const uint8_t* scales;
    };
    struct RowInfo {
        const uint8_t* srow;
    };
    __device__ static __forceinline__ RowInfo row_info(const Mat& m, int row, int nsteps) {
        return RowInfo{m.scales + (size_t)row * nsteps};
    }
    // The e8m0 bytes of SB steps from step0 on (a step is one 32-weight block of the lane's row), unconditional: four
    // bytes a load where the row's bytes are reached at a multiple of four (rows are a multiple of four blocks long
    // then too, so the last word ends with the row), else a byte a load, a step past the end taking the last byte.
    template <int SB>
    __device__ static __forceinline__ void scales(const Mat& m, const RowInfo& ri, int /*g*/, int step0, int nsteps,
                                                  uint32_t (&scl)[SB]) {
        if (step0 % 4 == 0 && nsteps % 4 == 0 && SB % 4 == 0 && (reinterpret_cast<uintptr_t>(m.scales) & 3) == 0) {
#pragma unroll
            for (int q = 0; q < SB / 4; ++q) {
                const uint32_t v = *reinterpret_cast<const uint32_t*>(ri.srow + min(step0 + 4 * q, nsteps - 4));
#pragma unroll
                for (int t = 0; t < 4; ++t) scl[4 * q + t] = (v >> (8 * t)) & 0xFFu;
            }
            return;
        }
#pragma unroll
        for (int t = 0; t < SB; ++t) scl[t] = (uint32_t)ri.srow[min(step0 + t, nsteps - 1)];
    }
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, int g, uint32_t scale) {
        const uint32_t q = *reinterpret_cast<const uint32_t*>(p + g * 4);
        const float s = bits_f32(scale << 23);
        uint32_t w[4];
        FmtMx4::widen8(q, s, w);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

// 12 bits a weight: the low bytes (32 a step) and the code nibbles (16 a step) are two arrays, each streamed into a
// slab of its own; a fragment is eight low bytes and eight codes zipped through the 16-entry table of high bytes
// (FmtP12::widen8). The escapes - weights whose high byte is not in the table - are rare: the matrix cores multiply the
// table's last entry in their place, and after the fold each escape of the tile's sixteen rows takes that term out and
// puts the true one in, in list order, whatever M is.
struct MfP12 {
    static constexpr int STEPB = 32;
    static constexpr int STEPB2 = 16;
    static constexpr bool TAIL = true;
    static constexpr int TAIL_BYTES = 32 * 16 * 4 + 32 * 4;
    static constexpr int TWO_TILES_STEPS = 80;
    static constexpr int SB_NARROW = 8, SB_WIDE = 8;
    struct Mat {
        const uint8_t* w;   // lo
        const uint8_t* w2;  // hi4
        const uint8_t* table;
        const int32_t* esc_idx;
        const uint8_t* esc_val;
        const int32_t* row_ptr;
    };
    struct RowInfo {};
    __device__ static __forceinline__ RowInfo row_info(const Mat&, int, int) { return RowInfo{}; }
    template <int SB>
    __device__ static __forceinline__ void scales(const Mat&, const RowInfo&, int, int, int, uint32_t (&)[SB]) {}
    __device__ static __forceinline__ uint4 table(const Mat& m) { return FmtP12::load_table(m.table); }
    __device__ static __forceinline__ bf16x8 frag2(const uint8_t* p, const uint8_t* p2, int g, const uint4& tbl) {
        const uint2 l = *reinterpret_cast<const uint2*>(p + g * 8);
        const uint32_t c = *reinterpret_cast<const uint32_t*>(p2 + g * 4);
        uint32_t w[4];
        FmtP12::widen8(tbl, c, l.x, l.y, w);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
    // The escapes of a tile: each of the KS waves takes those of 16 / KS of the tile's rows into its own partial tile
    // (lane: x row li, the tile's rows 4 lg .. 4 lg + 3), thirty-two at a time. Lane j takes escape j % 32 and eight
    // of the sixteen x rows (j / 32): its index and value are requested when the tile starts, its low byte and x
    // values while the tile's first sub-block is multiplied, so the products wait for neither. The terms go through
    // LDS (a small buffer of the wave's own) and are added in list order, whatever M is.
    struct Tail {
        int e0, e1;
        uint32_t idx, val, lo;
        int row;         // of the whole matrix
        uint32_t xv[4];  // eight x values, two a register
    };
    // Every load below is unconditional - a lane with no escape reads a harmless place (the row index, the table,
    // weight 0) - and so is every use of what the tile-ahead requests bring: a load whose only use sits in a branch
    // would be moved into that branch, behind the loads issued after it.
    __device__ static __forceinline__ void tail_request(const Mat& mat, Tail& t, int first, int lane) {
        const int e = first + (lane & 31);
        const bool ok = e < t.e1;
        const int32_t* pi = ok ? mat.esc_idx + e : mat.row_ptr;
        const uint8_t* pv = ok ? mat.esc_val + e : mat.table;
        const uint32_t i = (uint32_t)*pi;
        t.val = *pv;
        t.idx = ok ? i : 0u;
    }
    // the list positions of the escapes of rows row .. row + nrows - 1: asked for well ahead of tail_begin, which
    // cannot form an address without them
    __device__ static __forceinline__ int2 tail_span(const Mat& mat, int row, int nrows) {
        return make_int2(mat.row_ptr[row], mat.row_ptr[row + nrows]);
    }
    __device__ static __forceinline__ bool tail_any(const Tail& t) {
        return __builtin_amdgcn_readfirstlane(t.e0) < __builtin_amdgcn_readfirstlane(t.e1);
    }
    __device__ static __forceinline__ Tail tail_begin(const Mat& mat, int2 span, int lane) {
        Tail t;
        t.e0 = span.x;
        t.e1 = span.y;
        tail_request(mat, t, t.e0, lane);
        return t;
    }
    // xrows: the first of the sixteen x rows, of which `have` exist
    __device__ static __forceinline__ void tail_loads(const Mat& mat, Tail& t, const uint16_t* xrows, int C, int have,
                                                      int lane) {
        t.lo = mat.w[t.idx];
        t.row = (int)(t.idx / (uint32_t)C);
        const uint32_t col = t.idx - (uint32_t)t.row * (uint32_t)C;
        const int m0 = (lane >> 5) * 8;
#pragma unroll
        for (int q = 0; q < 4; ++q) {  // sixteen rows of at most 2^24 columns: the offsets fit 32 bits
            const uint32_t o0 = (uint32_t)min(m0 + 2 * q, have - 1) * (uint32_t)C + col;
            const uint32_t o1 = (uint32_t)min(m0 + 2 * q + 1, have - 1) * (uint32_t)C + col;
            t.xv[q] = (uint32_t)xrows[o0] | ((uint32_t)xrows[o1] << 16);
        }
    }
    // the thirty-two escapes in t: their terms into LDS, then added to the lane's rows in list order
    __device__ static __forceinline__ void tail_chunk(const uint4& tbl, const Tail& t, int tile, int first, int lane,
                                                      uint8_t* scratch, f32x4& s) {
        float* dl = reinterpret_cast<float*>(scratch);            // [32 escapes][16 x rows]
        int* rw = reinterpret_cast<int*>(scratch + 32 * 16 * 4);  // [32] the escape's row within the tile
        const uint32_t t15 = tbl.w >> 24;
        const int li = lane & 15, row0 = (lane >> 4) * 4;
        const float streamed = bits_f32((t15 << 24) | (t.lo << 16));
        const float truth = bits_f32((t.val << 24) | (t.lo << 16));
        float d[8];
#pragma unroll
        for (int q = 0; q < 8; ++q) {
            const float xv = (q & 1) ? bf16hi_f32(t.xv[q / 2]) : bf16lo_f32(t.xv[q / 2]);
            d[q] = fmaf(truth, xv, -(streamed * xv));
        }
        float4* o = reinterpret_cast<float4*>(dl + (lane & 31) * 16 + (lane >> 5) * 8);
        o[0] = make_float4(d[0], d[1], d[2], d[3]);
        o[1] = make_float4(d[4], d[5], d[6], d[7]);
        rw[lane & 31] = t.row - tile * 16;  // both halves write the same value
        const int cnt = max(min(32, t.e1 - first), 0);
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
    // fetched: the first thirty-two are already in t (tail_begin, tail_loads with these x rows)
    __device__ static __forceinline__ void tail_apply(const Mat& mat, const uint4& tbl, Tail& t, int tile,
                                                      const uint16_t* xrows, int C, int have, int lane, uint8_t* scratch,
                                                      bool fetched, f32x4& s) {
        if (!fetched) {  // other x rows than the ones asked for ahead
            tail_request(mat, t, t.e0, lane);
            tail_loads(mat, t, xrows, C, have, lane);
        }
        tail_chunk(tbl, t, tile, t.e0, lane, scratch, s);
        for (int first = t.e0 + 32; first < t.e1; first += 32) {  // a crowd: fetched here
            tail_request(mat, t, first, lane);
            tail_loads(mat, t, xrows, C, have, lane);
            tail_chunk(tbl, t, tile, first, lane, scratch, s);
        }
    }
};

// ---- the kernel -----------------------------------------------------------------------------------------------------

// KS waves a workgroup; MT 16-row tiles of x; SPW the steps a wave holds x fragments for (MT * SPW fragments in
// registers); SB steps per sub-block (a slab holds 16 rows x SB steps). XS: the x fragments are not held - each
// sub-block's come in with its weights (x is small and stays in L2), so a row may be as long as SPW allows without
// the registers x-stationary rows of that length would take
// XN: x is not given but made - the residual add and RMSNorm of a.x (+ a.y) with a.norm_w, as add_rmsnorm_kernel
// computes them (or the embedding rows a.ids name) - by every workgroup for itself before its first tile, the first
// workgroup also writing the new residual to a.h_out. 256 threads take a row, word i + 256 k of it thread i (the order
// that kernel sums in, so the bits are its bits); the rows lie in LDS where the slabs will be, a wave takes its
// fragments from there and holds them as it holds a given x. Making the rows costs a workgroup 5 us (5 rows) to 8.6 us
// (16) on MI355X ([6144 x 2560]: 14.3 / 15.6 / 19.3 us at 5 / 8 / 16 rows against 9.2 / 9.7 / 10.7 for the matvec
// alone), about twice what a launch of add_rmsnorm ahead of the plain matvec adds (2.5 us back to back): this is the
// entry point's kernel for passes of five rows and more - passes of four rows of the vector kernel took twice as
// long - not the fastest way to run such a pass, which is the two launches.
// TR: the rows of a tile that are rows of the matrix (a divisor of R, a multiple of a load's rows): the tile is rows
// TR tile .. + TR - 1, its other rows are not read and what the matrix cores make of them is not written. A template
// argument: a load that a run-time test decides on is a load the compiler cannot count, and it then waits for all.
template <class MF, int KS, int MT, int SPW, int SB, bool XS = false, bool XN = false, int TR = 16>
__global__ void __launch_bounds__(KS * 64) gemv_mfma_lds(typename MF::Mat mat, const uint4* __restrict__ x,
                                                         uint16_t* __restrict__ y, int R, int C, int M, int half,
                                                         XArgs xa) {
    constexpr int tr = TR;
    constexpr int ROWB = SB * MF::STEPB;      // bytes a row contributes to a sub-block
    constexpr int STRIDE = ROWB + 16;         // the slab's row stride: 4 banks past a multiple of 64, so the sixteen
                                              // rows a fragment read touches fall in sixteen different bank groups
    constexpr int SLAB = 16 * STRIDE;
    constexpr int NLD = 16 * ROWB / 1024;     // 16-byte-per-lane loads a sub-block takes
    constexpr int MAXSB = (SPW + SB - 1) / SB;
    static_assert((16 * ROWB) % 1024 == 0 && NLD >= 1, "a sub-block is a whole number of wave loads");
    // the second stream of a two-array form, the same way
    constexpr int STEPB2 = MF::STEPB2;
    constexpr bool TWO = STEPB2 > 0;
    constexpr int ROWB2 = TWO ? SB * STEPB2 : 1024;
    constexpr int STRIDE2 = ROWB2 + 16;
    constexpr int SLAB2 = TWO ? 16 * STRIDE2 : 0;
    constexpr int NLD2 = TWO ? 16 * ROWB2 / 1024 : 0;
    static_assert(!TWO || ((16 * ROWB2) % 1024 == 0 && NLD2 >= 1 && 1024 % ROWB2 == 0), "the second stream's sub-block");
    extern __shared__ __align__(16) uint8_t lds[];  // KS slabs (and second slabs), then two sets of KS * MT partial tiles
    const int lane = threadIdx.x & (WAVE - 1);
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int li = lane & 15, lg = lane >> 4;
    uint8_t* slab = lds + wv * SLAB;
    uint8_t* slab2 = lds + KS * SLAB + wv * SLAB2;
    constexpr int TAILB = MF::TAIL ? MF::TAIL_BYTES : 0;  // a wave's exchange buffer for the escapes' terms
    [[maybe_unused]] uint8_t* tailbuf = lds + KS * (SLAB + SLAB2) + wv * TAILB;
    f32x4* part = reinterpret_cast<f32x4*>(lds + KS * (SLAB + SLAB2 + TAILB));

    const int chunk4 = C / 8;  // uint4 per row of x
    const int nsteps = C / 32;
    const int spw = (nsteps + KS - 1) / KS;
    const int s0 = wv * spw;
    const int n = max(min(s0 + spw, nsteps) - s0, 0);  // this wave's steps: s0 .. s0 + n - 1
    const size_t rowbytes = (size_t)nsteps * MF::STEPB;

    uint4 xb[MT][XS ? 1 : SPW];
    const uint4* xr[MT];
#pragma unroll
    for (int t = 0; t < MT; ++t) {
        xr[t] = x + (size_t)min(t * 16 + li, M - 1) * chunk4 + lg + (size_t)s0 * 4;
        if constexpr (!XS && !XN) {
#pragma unroll
            for (int i = 0; i < SPW; ++i) xb[t][i] = i < n ? xr[t][i * 4] : make_uint4(0, 0, 0, 0);
        }
    }
    // XN: the rows' words, asked for ahead of the first weights (which would otherwise return first, in order)
    static_assert(!XN || (KS % 4 == 0 && MT == 1 && !XS), "256 threads a row, one tile of rows, fragments held");
    constexpr int XN_GROUPS = XN ? KS / 4 : 1;       // rows in the making at once
    constexpr int XN_RPG = XN ? 16 / XN_GROUPS : 1;  // rows a group of 256 threads makes, one after the other
    constexpr int XN_PER = 3;                        // 8-byte words of a row a thread takes: rows up to 3072 values
    const int xn_gid = threadIdx.x >> 8, xn_t = threadIdx.x & 255, xn_n4 = C / 4;
    const int xn_stride = C * 2 + 16;  // a row's bytes in LDS: 4 banks past a multiple of 64, as a slab's rows
    [[maybe_unused]] uint2 xn_h[XN_RPG][XN_PER], xn_y[XN_RPG][XN_PER], xn_w[XN_PER];
    if constexpr (XN) {
        const uint2* ws = reinterpret_cast<const uint2*>(xa.norm_w);
#pragma unroll
        for (int q = 0; q < XN_PER; ++q) xn_w[q] = ws[min(q * 256 + xn_t, xn_n4 - 1)];
#pragma unroll
        for (int r = 0; r < XN_RPG; ++r) {
            const int m = r * XN_GROUPS + xn_gid;
            if (m < M) {
                size_t hrow = (size_t)m;
                if (xa.ids != nullptr) hrow = (size_t)min(max(xa.ids[m], 0), xa.vocab - 1);
                const uint2* hs = reinterpret_cast<const uint2*>(xa.x + hrow * C);
                const uint2* ys = xa.y == nullptr ? hs : reinterpret_cast<const uint2*>(xa.y + (size_t)m * C);
#pragma unroll
                for (int q = 0; q < XN_PER; ++q) {
                    const int i = min(q * 256 + xn_t, xn_n4 - 1);
                    xn_h[r][q] = hs[i];
                    xn_y[r][q] = ys[i];  // no y: h again, unused
                }
            }
        }
    }
    [[maybe_unused]] uint4 xs[MT][XS ? SB : 1];  // XS: the x fragments of the sub-block in flight

    // A load instruction covers RPI whole rows of the sub-block (ROWB bytes each); the lane's place in it - row and
    // byte within the row - is the same for every load of the kernel, so every address is a uniform base (tile, load,
    // sub-block) plus one per-lane offset
    constexpr int RPI = 1024 / ROWB;
    static_assert(ROWB <= 1024 && 1024 % ROWB == 0, "a load instruction covers whole rows of a sub-block");
    const uint32_t lane_row = (uint32_t)(lane * 16) / ROWB, lane_byte = (uint32_t)(lane * 16) % ROWB;
    const uint32_t goff = lane_row * (uint32_t)rowbytes + lane_byte;
    const uint32_t loff = lane_row * STRIDE + lane_byte;
    constexpr int RPI2 = 1024 / ROWB2;
    const uint32_t lane_row2 = (uint32_t)(lane * 16) / ROWB2, lane_byte2 = (uint32_t)(lane * 16) % ROWB2;
    const size_t rowbytes2 = (size_t)nsteps * STEPB2;
    const uint32_t goff2 = lane_row2 * (uint32_t)rowbytes2 + lane_byte2;
    const uint32_t loff2 = lane_row2 * STRIDE2 + lane_byte2;
    uint4 tbl = make_uint4(0, 0, 0, 0);  // the table of a form that looks its weights up
    if constexpr (TWO) tbl = MF::table(mat);
    uint4 raw[NLD] = {};
    uint4 raw2[TWO ? NLD2 : 1] = {};
    uint32_t scl[SB] = {};  // the scales of the sub-block in flight, one per step, for this lane's row and column group
    auto request = [&](int tile, int sb) {  // the loads of sub-block sb of the tile (R is a multiple of 16)
        if constexpr (XS) {  // out of L2, ahead of the weights they will meet: a step past the wave's last takes the last
            // the same addresses every tile: a zero the compiler cannot see through keeps it from loading them all
            // once, ahead of the loop, into the registers this form is there to save
            int zero = 0;
            asm volatile("" : "+s"(zero));
#pragma unroll
            for (int t = 0; t < SB; ++t) {
                const int i = min(sb * SB + t, n - 1) + zero;
#pragma unroll
                for (int m = 0; m < MT; ++m) xs[m][t] = xr[m][i * 4];
            }
        }
        const uint32_t valid = (uint32_t)(min(SB, n - sb * SB) * MF::STEPB);
        const typename MF::RowInfo rn = MF::row_info(mat, tile * 16 + li, nsteps);
        MF::template scales<SB>(mat, rn, lg, s0 + sb * SB, nsteps, scl);
#pragma unroll
        for (int q = 0; q < NLD; ++q) {
            // half > 0: the tile's rows 0..7 are gate rows 8 tile .., its rows 8..15 the up rows of the same outputs
            const int row0 = half ? tile * 8 + q * RPI + (q * RPI >= 8 ? half * 16 - 8 : 0) : tile * tr + q * RPI;
            const uint8_t* base = mat.w + (size_t)row0 * rowbytes + (size_t)(s0 + sb * SB) * MF::STEPB;
            if (q * RPI < tr) {
                if (lane_byte < valid) raw[q] = load_stream16(reinterpret_cast<const uint4*>(base + goff));
            }
        }
        if constexpr (TWO) {
            const uint32_t valid2 = (uint32_t)(min(SB, n - sb * SB) * STEPB2);
#pragma unroll
            for (int q = 0; q < NLD2; ++q) {
                const uint8_t* base =
                    mat.w2 + (size_t)(tile * 16 + q * RPI2) * rowbytes2 + (size_t)(s0 + sb * SB) * STEPB2;
                if (lane_byte2 < valid2) raw2[q] = load_stream16(reinterpret_cast<const uint4*>(base + goff2));
            }
        }
    };

    const int ntiles = R / tr;
    const int nsb = (n + SB - 1) / SB;
    // The tiles a workgroup visits: blockIdx.x, + gridDim.x, ... With half > 0 (W is a gate matrix over an up matrix,
    // half tiles of 16 rows each, and y their fold bf16(bf16(silu(g)) * u), [M, R / 2]) a tile is eight gate rows over
    // the eight up rows of the same outputs: as many tiles as without the fold, so the grid walks them the same way
    // (taking a gate tile and then its up tile, a pair a workgroup, made the last turn two tiles long: [19456 x 2560]
    // on 256 CUs took six tiles' time where the plain matvec takes five).
    static_assert(RPI <= 8 || !std::is_same<MF, MfBf16>::value, "a load's rows lie in one half of a folded tile");
    const int grid = (int)gridDim.x, first = (int)blockIdx.x;
    auto tile_of = [&](int k) { return first + k * grid; };
    auto live = [&](int k) { return first + k * grid < ntiles; };
    int tile = tile_of(0);
    // the escapes of the wave's rows of a tile: their indices are asked for a tile ahead, the rest of what they need
    // while the tile's first sub-block is multiplied
    [[maybe_unused]] typename MF::Tail tl, tnext;
    [[maybe_unused]] int2 span_next = make_int2(0, 0);
    constexpr int TROWS = 16 / KS;  // the rows of a tile whose escapes this wave takes
    if constexpr (MF::TAIL) {
        if (tile < ntiles) tnext = MF::tail_begin(mat, MF::tail_span(mat, tile * 16 + wv * TROWS, TROWS), lane);
    }
    if (tile < ntiles && nsb > 0) request(tile, 0);
    if constexpr (XN) {
        float* red = reinterpret_cast<float*>(lds + 16 * xn_stride);  // [16 rows][4 waves of the row's group]
        const bool has_y = xa.y != nullptr;
        const bool writer = blockIdx.x == 0 && xa.h_out != nullptr;
#pragma unroll
        for (int r = 0; r < XN_RPG; ++r) {
            const int m = r * XN_GROUPS + xn_gid;
            if (m < M) {
                float ss = 0.f;
#pragma unroll
                for (int q = 0; q < XN_PER; ++q) {
                    const int i = q * 256 + xn_t;
                    const bool in_row = i < xn_n4;
                    float f[4] = {bf16lo_f32(xn_h[r][q].x), bf16hi_f32(xn_h[r][q].x), bf16lo_f32(xn_h[r][q].y),
                                  bf16hi_f32(xn_h[r][q].y)};
                    const float g[4] = {bf16lo_f32(xn_y[r][q].x), bf16hi_f32(xn_y[r][q].x), bf16lo_f32(xn_y[r][q].y),
                                        bf16hi_f32(xn_y[r][q].y)};
#pragma unroll
                    for (int e = 0; e < 4; ++e) {
                        const float sum = bfround(f[e] + g[e]);
                        f[e] = has_y ? sum : f[e];
                        const float sq = fmaf(f[e], f[e], ss);
                        ss = in_row ? sq : ss;
                    }
                    const uint2 hb = make_uint2(f32x2_bf16(f[0], f[1]), f32x2_bf16(f[2], f[3]));
                    if (in_row) {
                        *reinterpret_cast<uint2*>(lds + (size_t)m * xn_stride + (size_t)i * 8) = hb;
                        if (writer) reinterpret_cast<uint2*>(xa.h_out + (size_t)m * C)[i] = hb;
                    }
                }
                ss = group_sum_last<64>(ss);
                if (lane == 63) red[m * 4 + (wv & 3)] = ss;
            }
        }
        __syncthreads();
#pragma unroll
        for (int r = 0; r < XN_RPG; ++r) {
            const int m = r * XN_GROUPS + xn_gid;
            if (m < M) {
                const float sum = ((red[m * 4] + red[m * 4 + 1]) + red[m * 4 + 2]) + red[m * 4 + 3];
                const float rstd = rsqrtf(sum / (float)C + xa.eps);
#pragma unroll
                for (int q = 0; q < XN_PER; ++q) {
                    const int i = q * 256 + xn_t;
                    if (i < xn_n4) {
                        uint2* slot = reinterpret_cast<uint2*>(lds + (size_t)m * xn_stride + (size_t)i * 8);
                        const uint2 hb = *slot;
                        const float f[4] = {bf16lo_f32(hb.x), bf16hi_f32(hb.x), bf16lo_f32(hb.y), bf16hi_f32(hb.y)};
                        const float g[4] = {bf16lo_f32(xn_w[q].x), bf16hi_f32(xn_w[q].x), bf16lo_f32(xn_w[q].y),
                                            bf16hi_f32(xn_w[q].y)};
                        float o[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = f[e] * rstd * (xa.centered ? 1.f + g[e] : g[e]);
                        *slot = make_uint2(f32x2_bf16(o[0], o[1]), f32x2_bf16(o[2], o[3]));
                    }
                }
            }
        }
        __syncthreads();
        const uint8_t* xrow = lds + (size_t)min(li, M - 1) * xn_stride + (size_t)(s0 * 32 + lg * 8) * 2;
#pragma unroll
        for (int i = 0; i < SPW; ++i)
            xb[0][i] = i < n ? *reinterpret_cast<const uint4*>(xrow + i * 64) : make_uint4(0, 0, 0, 0);
        __syncthreads();  // the rows have been read: the slabs may take their place
    }
    for (int turn = 0; live(turn); ++turn) {
        tile = tile_of(turn);
        f32x4 acc[MT];
#pragma unroll
        for (int t = 0; t < MT; ++t) acc[t] = f32x4{0.f, 0.f, 0.f, 0.f};
        const bool more = live(turn + 1);
        const int next = tile_of(turn + 1);
        [[maybe_unused]] const uint16_t* xrows = reinterpret_cast<const uint16_t*>(x);
        if constexpr (MF::TAIL) tl = tnext;
#pragma unroll
        for (int sb = 0; sb < MAXSB; ++sb) {
            if (sb < nsb) {
                // the sub-block's bytes into the slab, as stored
#pragma unroll
                for (int q = 0; q < NLD; ++q) *reinterpret_cast<uint4*>(slab + q * RPI * STRIDE + loff) = raw[q];
                if constexpr (TWO) {
#pragma unroll
                    for (int q = 0; q < NLD2; ++q)
                        *reinterpret_cast<uint4*>(slab2 + q * RPI2 * STRIDE2 + loff2) = raw2[q];
                }
                uint32_t sc[SB];
#pragma unroll
                for (int t = 0; t < SB; ++t) sc[t] = scl[t];
                [[maybe_unused]] uint4 xc[MT][XS ? SB : 1];
                if constexpr (XS) {
#pragma unroll
                    for (int m = 0; m < MT; ++m)
#pragma unroll
                        for (int t = 0; t < SB; ++t) xc[m][t] = xs[m][t];
                }
                if constexpr (MF::TAIL) {
                    if (sb == 0) {
                        MF::tail_loads(mat, tl, xrows, C, min(M, 16), lane);
                        span_next = MF::tail_span(mat, min(next, ntiles - 1) * 16 + wv * TROWS, TROWS);
                    }
                }
                // the next sub-block - of this tile, or the first of the workgroup's next tile - on its way
                if (sb + 1 < nsb) {
                    request(tile, sb + 1);
                } else if (more) {
                    if constexpr (MF::TAIL) tnext = MF::tail_begin(mat, span_next, lane);
                    request(next, 0);
                }
#pragma unroll
                for (int t = 0; t < SB; ++t) {
                    const int i = sb * SB + t;  // the wave's step (a compile-time index into xb)
                    if (i < SPW && i < n) {
                        bf16x8 a;
                        if constexpr (TWO)
                            a = MF::frag2(slab + li * STRIDE + t * MF::STEPB, slab2 + li * STRIDE2 + t * STEPB2, lg,
                                          tbl);
                        else
                            a = MF::frag(slab + li * STRIDE + t * MF::STEPB, lg, sc[t]);
#pragma unroll
                        for (int m = 0; m < MT; ++m)
                            acc[m] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                                a, __builtin_bit_cast(bf16x8, XS ? xc[m][t] : xb[m][XS ? 0 : (i < SPW ? i : 0)]), acc[m],
                                0, 0, 0);
                    }
                }
            }
        }
        if constexpr (MF::TAIL) {
            // a wave with no step of its own (a short row) has not been through the loop above
            if (nsb == 0) {
                MF::tail_loads(mat, tl, xrows, C, min(M, 16), lane);
                if (more)
                    tnext = MF::tail_begin(mat, MF::tail_span(mat, next * 16 + wv * TROWS, TROWS), lane);
            }
            if (MF::tail_any(tl)) {  // the same for the whole wave
#pragma unroll
                for (int t = 0; t < MT; ++t)
                    if (t == 0 || t * 16 < M)
                        MF::tail_apply(mat, tbl, tl, tile, xrows + (size_t)t * 16 * C, C, min(M - t * 16, 16), lane,
                                       tailbuf, t == 0, acc[t]);
            }
        }
        // the KS partial tiles, folded in wave order; two sets of partials alternate so one barrier a tile suffices
        f32x4* mine = part + (size_t)(turn & 1) * KS * MT * WAVE;
#pragma unroll
        for (int t = 0; t < MT; ++t) mine[(wv * MT + t) * WAVE + lane] = acc[t];
        __syncthreads();
        if (wv < MT) {
            f32x4 s = mine[(0 * MT + wv) * WAVE + lane];
            for (int q = 1; q < KS; ++q) {
                const f32x4 o = mine[(q * MT + wv) * WAVE + lane];
                s.x += o.x;
                s.y += o.y;
                s.z += o.z;
                s.w += o.w;
            }
            const int m = wv * 16 + li;
            if (half) {
                // lanes of row groups 0, 1 hold gate sums, the lanes 32 further on the up sums of the same outputs
                const f32x4 up = f32x4{xor32(s.x), xor32(s.y), xor32(s.z), xor32(s.w)};
                if (m < M && lg < 2) {
                    // the arithmetic of the stand-alone fold over the two rounded outputs (silu_pair)
                    auto fold = [](float g, float u) {
                        const float gb = bfround(g), ub = bfround(u);
                        return f32_bf16(bfround(gb / (1.f + expf(-gb))) * ub);
                    };
                    uint16_t* o = y + (size_t)m * (R / 2) + tile * 8 + lg * 4;
                    o[0] = fold(s.x, up.x);
                    o[1] = fold(s.y, up.y);
                    o[2] = fold(s.z, up.z);
                    o[3] = fold(s.w, up.w);
                }
            } else {
                const int in_tile = lg * 4, row = tile * tr + in_tile;
                if (m < M) {
                    uint16_t* o = y + (size_t)m * R + row;
                    if (in_tile + 0 < tr && row + 0 < R) o[0] = f32_bf16(s.x);
                    if (in_tile + 1 < tr && row + 1 < R) o[1] = f32_bf16(s.y);
                    if (in_tile + 2 < tr && row + 2 < R) o[2] = f32_bf16(s.z);
                    if (in_tile + 3 < tr && row + 3 < R) o[3] = f32_bf16(s.w);
                }
            }
        }
    }
}

template <class MF, int KS, int MT, int SPW, int SB, bool XS, bool XN, int TR>
static int32_t launch_lds_tr(const typename MF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st,
                             int half, const XArgs& xa, int cap) {
    constexpr int SLAB = 16 * (SB * MF::STEPB + 16) + (MF::STEPB2 > 0 ? 16 * (SB * MF::STEPB2 + 16) : 0) + MF::TAIL_BYTES;
    size_t lds = (size_t)KS * SLAB + 2 * (size_t)KS * MT * WAVE * sizeof(f32x4);
    if (XN) {  // the made rows (and the sums' exchange) lie where the slabs will be
        const size_t rows = 16 * ((size_t)C * 2 + 16) + 16 * 4 * sizeof(float);
        if (rows > lds) lds = rows;
    }
    const int ntiles = R / TR;
    // whole turns of the grid over the tiles: the smallest grid that walks them in ceil(ntiles / cap) turns
    const int turns = (ntiles + cap - 1) / cap;
    const int grid = (ntiles + turns - 1) / turns;
    auto kern = gemv_mfma_lds<MF, KS, MT, SPW, SB, XS, XN, TR>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(KS * 64), lds, st, mat, static_cast<const uint4*>(x),
                       static_cast<uint16_t*>(y), R, C, M, half, xa);
    return hip_status(hipGetLastError(), "gemv_mfma launch");
}

template <class MF, int KS, int MT, int SPW, int SB, bool XS = false, bool XN = false>
static int32_t launch_lds(const typename MF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st,
                          int half = 0, const XArgs& xa = XArgs{}) {
    int per_cu = tuning("mfma_wgs_per_cu");
    if (per_cu <= 0) per_cu = 12 / KS;  // twelve waves a CU: what the kernel's registers leave resident
    const int cap = device_info().cus * per_cu;
    // Rows a tile: sixteen, or twelve or ten where that fills the CUs better - what a launch takes is the busiest
    // workgroup's rows, turns x rows a tile, and 2560 rows are 160 tiles of sixteen (one turn of 160 workgroups on 256
    // CUs, sixteen rows each) but 256 tiles of ten; 6144 rows two turns of sixteen or of twelve. bf16 rows as they are
    // and eight waves: a tile's loads are whole rows two at a time, and a row's bits do not depend on the tile it
    // came in. Measured at 8 rows of x, MI355X: [2560 x 9728] 17.9 -> 15.0 us, [6144 x 2560] 11.2 -> 10.5,
    // [2560 x 4096] 7.8 -> 7.6.
    if constexpr (std::is_same<MF, MfBf16>::value && KS == 8 && !XN) {
        if (half == 0 && tuning("mfma_tile_rows") != 0) {
            auto rows_of = [&](int t) { return (long)((R / t + cap - 1) / cap) * t; };
            int tr = 16;
            // (a lower tile has fewer bytes in flight a workgroup, which costs where the tiles are many: eight rows a
            // tile took [9728 x 2560] from 12.7 to 14.2 us and the head [151936 x 2560] from 130 to 173 although both
            // count fewer rows for the busiest workgroup that way - so only twelve and ten, and only for an eighth
            // fewer rows or better)
            if (R % 12 == 0 && rows_of(12) * 8 <= rows_of(16) * 7) tr = 12;
            if (R % 10 == 0 && rows_of(10) * 8 <= rows_of(16) * 7 && rows_of(10) < rows_of(tr)) tr = 10;
            if (tr == 12) return launch_lds_tr<MF, KS, MT, SPW, SB, XS, XN, 12>(mat, x, y, R, C, M, st, half, xa, cap);
            if (tr == 10) return launch_lds_tr<MF, KS, MT, SPW, SB, XS, XN, 10>(mat, x, y, R, C, M, st, half, xa, cap);
        }
    }
    return launch_lds_tr<MF, KS, MT, SPW, SB, XS, XN, 16>(mat, x, y, R, C, M, st, half, xa, cap);
}

// The split of the columns over a workgroup's waves comes from the row length alone: at most eight waves (a workgroup
// of sixteen would leave each wave 128 registers, less than the x fragments and a sub-block in flight need), each
// holding x for 10, 16 or 28 steps. Up to 16 steps a wave there is room for two tiles of x rows; at 28 for one, and a
// pass of more than 16 rows runs as two. Rows up to 7168 wide fit that way; up to 10240 the x fragments are streamed
// (XS); wider ones stay with the column-interleaved kernel (bf16) or the vector-ALU passes (packed forms).
template <class MF>
static bool lds_fits(int R, int C) {
    return R % 16 == 0 && C % 32 == 0 && C / 32 <= 8 * 40;
}
bool mfma_lds_fits_bf16(int R, int C) { return lds_fits<MfBf16>(R, C); }
bool mfma_lds_fits_packed(int R, int C) { return lds_fits<MfF8>(R, C); }

template <class MF, int MT>
static int32_t run_narrow(const typename MF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st,
                          int half = 0) {
    constexpr int SB = MF::SB_NARROW;
    const int nsteps = C / 32;
    if (nsteps <= 20) return launch_lds<MF, 2, MT, 10, 8>(mat, x, y, R, C, M, st, half);
    if (nsteps <= 40) return launch_lds<MF, 4, MT, 10, 8>(mat, x, y, R, C, M, st, half);
    if (nsteps <= 80) return launch_lds<MF, 8, MT, 10, 8>(mat, x, y, R, C, M, st, half);
    return launch_lds<MF, 8, MT, 16, SB>(mat, x, y, R, C, M, st, half);
}

template <class MF>
static int32_t run_lds(const typename MF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st,
                          int half = 0) {
    const int nsteps = C / 32;
    if (nsteps <= MF::TWO_TILES_STEPS)
        return M <= 16 ? run_narrow<MF, 1>(mat, x, y, R, C, M, st, half) : run_narrow<MF, 2>(mat, x, y, R, C, M, st, half);
    const uint16_t* xp = static_cast<const uint16_t*>(x);
    uint16_t* yp = static_cast<uint16_t*>(y);
    const int yrow = half ? R / 2 : R;  // values a row of y holds
    if (nsteps <= 128) {  // sixteen steps a wave, registers for one tile of x rows
        for (int m0 = 0; m0 < M; m0 += 16) {
            int32_t rc = run_narrow<MF, 1>(mat, xp + (size_t)m0 * C, yp + (size_t)m0 * yrow, R, C, M - m0 < 16 ? M - m0 : 16, st, half);
            if (rc != OK) return rc;
        }
        return OK;
    }
    constexpr int SBW = MF::SB_WIDE;
    // (sixteen steps a sub-block for the streamed rows - twice the bytes in flight - spills: [2560 x 9728] 13.7 -> 22.5 us)
    // up to 28 steps a wave the x fragments stay in registers; longer rows (to 40 steps: 10240 columns) stream them
    const bool stream_x = nsteps > 8 * 28 || tuning("mfma_stream_x") > 0;
    for (int m0 = 0; m0 < M; m0 += 16) {
        const int mm = M - m0 < 16 ? M - m0 : 16;
        int32_t rc = stream_x ? (nsteps > 8 * 28
                                     ? launch_lds<MF, 8, 1, 40, 8, true>(mat, xp + (size_t)m0 * C, yp + (size_t)m0 * yrow, R, C, mm, st, half)
                                     : launch_lds<MF, 8, 1, 28, 8, true>(mat, xp + (size_t)m0 * C, yp + (size_t)m0 * yrow, R, C, mm, st, half))
                              : launch_lds<MF, 8, 1, 28, SBW>(mat, xp + (size_t)m0 * C, yp + (size_t)m0 * yrow, R, C, mm, st, half);
        if (rc != OK) return rc;
    }
    return OK;
}

// M = 5..32 and a shape the fits() above take (whole 16-row tiles among them): the callers (gemv.hip) check before
// they come here
int32_t gemv_mfma_lds_bf16(const void* w, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    return run_lds<MfBf16>(MfBf16::Mat{static_cast<const uint8_t*>(w)}, x, y, R, C, M, st);
}
// W = [gate; up], 2I rows: y [M, I] = bf16(bf16(silu(g)) * u)
int32_t gemv_mfma_lds_glu_bf16(const void* w, const void* x, void* y, int I, int C, int M, hipStream_t st) {
    return run_lds<MfBf16>(MfBf16::Mat{static_cast<const uint8_t*>(w)}, x, y, 2 * I, C, M, st, I / 16);
}
// ... with x made by the residual add and RMSNorm (XArgs); I > 0: W = [gate; up] and y the fold, as above. Rows of
// 1312 .. 2560 columns (the widths whose workgroups are 512 threads: two rows in the making at once), 16 rows of the
// residual stream a pass.
bool mfma_lds_norm_fits(int R, int C, int M) {
    return lds_fits<MfBf16>(R, C) && C / 32 > 40 && C / 32 <= 80 && M >= 5 && tuning("mfma_lds_norm") != 0;
}
int32_t gemv_mfma_lds_norm_bf16(const void* w, const XArgs& xa, void* y, int R, int C, int M, int I, hipStream_t st) {
    const MfBf16::Mat mat{static_cast<const uint8_t*>(w)};
    const int half = I > 0 ? I / 16 : 0;
    XArgs a = xa;
    uint16_t* yp = static_cast<uint16_t*>(y);
    const size_t yrow = I > 0 ? (size_t)I : (size_t)R;
    for (int m0 = 0; m0 < M; m0 += 16) {
        const int32_t rc = launch_lds<MfBf16, 8, 1, 10, 8, false, true>(mat, nullptr, yp + (size_t)m0 * yrow, R, C,
                                                                        M - m0 < 16 ? M - m0 : 16, st, half, a);
        if (rc != OK) return rc;
        if (a.ids != nullptr)
            a.ids += 16;
        else
            a.x += (size_t)16 * C;
        if (a.y != nullptr) a.y += (size_t)16 * C;
        if (a.h_out != nullptr) a.h_out += (size_t)16 * C;
    }
    return OK;
}
int32_t gemv_mfma_lds_fp8(const void* w, const float* scales, int sc, int bm, int bn, const void* x, void* y, int R,
                          int C, int M, hipStream_t st) {
    return run_lds<MfF8>(MfF8::Mat{static_cast<const uint8_t*>(w), scales, sc, bm, bn}, x, y, R, C, M, st);
}
int32_t gemv_mfma_lds_p12(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const int32_t* esc_idx,
                          const uint8_t* esc_val, const int32_t* row_ptr, const void* x, void* y, int R, int C, int M,
                          hipStream_t st) {
    return run_lds<MfP12>(MfP12::Mat{lo, hi4, table, esc_idx, esc_val, row_ptr}, x, y, R, C, M, st);
}
int32_t gemv_mfma_lds_mxfp4(const void* blocks, const void* scales, const void* x, void* y, int R, int C, int M,
                            hipStream_t st) {
    return run_lds<MfMx4>(MfMx4::Mat{static_cast<const uint8_t*>(blocks), static_cast<const uint8_t*>(scales)}, x, y, R,
                          C, M, st);
}

}  // namespace btb
