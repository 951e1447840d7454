// The verify widths (M = 5..16 rows of x a pass) on the matrix cores for the long rows of the block-scaled forms
// (FP8 e4m3 + block scales, MXFP4), with the weights going from memory straight into LDS.
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
// 128-byte column blocks of the tile's sixteen rows: 2 GB load instructions, plus one dword-sized direct load for its
// scales (the MXFP4 bytes of its rows and steps, or the FP8 block scales of its steps - a tile's sixteen rows share
// them: blocks are a multiple of 16 rows tall).
//
// Waiting is by count: loads complete in order, a sub-block is LOADS load instructions, so "sub-block q has landed" is
// "at most (sub-blocks issued behind it) x LOADS loads outstanding" - an immediate, picked by how many were issued
// behind it. The output stores of a tile's end count as outstanding too and may complete in any order: they are left
// out of the immediate, which can only make a wait longer. A slot is asked for again only after the reads of its last
// use have returned (the MFMAs that take them have been issued).
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
// the same with the full MAXB sub-blocks behind and, behind them too, `xparts` (0..6) parts of x of XL loads each
template <int LOADS, int MAXB, int XL>
__device__ __forceinline__ void wait_lead(int xparts, uint32_t& a, uint32_t& b) {
    constexpr int BASE = MAXB * LOADS;
    auto imm = [](int n) constexpr { return BASE + n * XL < 64 ? BASE + n * XL : 0; };
    if (xparts == 6)
        wait_loads<imm(6)>(a, b);
    else if (xparts == 5)
        wait_loads<imm(5)>(a, b);
    else if (xparts == 4)
        wait_loads<imm(4)>(a, b);
    else if (xparts == 3)
        wait_loads<imm(3)>(a, b);
    else if (xparts == 2)
        wait_loads<imm(2)>(a, b);
    else if (xparts == 1)
        wait_loads<imm(1)>(a, b);
    else
        wait_loads<BASE>(a, b);
}

// A 16-byte load whose being outstanding the compiler does not know of, and the statement that says "these four have
// landed" (it follows the counted wait that makes it true). The compiler's own wait for a loaded register is exact
// only while no direct-to-LDS load is outstanding: those are FLAT-encoded instructions that name LDS, after which it
// takes the order of returns to be unknown and waits for every load there is, the ring's included. The kernel's first
// tile wants its part of x and nothing younger, so x comes through these two where that tile is on its own straight
// path. Between the two statements the registers are named by nothing else.
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

struct DlF8 {
    static constexpr int STEPB = 32;
    struct Mat {
        const uint8_t* w;
        const float* scales;
        int sc;  // scales per grid row
        int bm;  // rows per block (a multiple of 16: a tile's sixteen rows share their scales)
        int bn;  // columns per block (a multiple of 32: a step lies in one block)
    };
    __host__ __device__ static constexpr int scale_bytes(int /*sbs*/) { return 4 * WAVE; }
    __host__ __device__ static constexpr int scale_words(int sbs) { return sbs; }
    // lane t brings the scale of the sub-block's step min(t, SBS - 1): f32 [64] in the scale area, the first SBS of
    // them read. Every lane loads, so that there is no branch round the instruction: the compiler counts the loads
    // outstanding exactly only through straight-line code, and the kernel's first tile depends on that.
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
    __device__ static __forceinline__ uint32_t scale_off(int /*li*/, int /*sbs*/) { return 0; }
    // the words a lane needs of the scale area for the whole sub-block, from the area + scale_off on
    template <int SBS>
    __device__ static __forceinline__ void read_scales(const uint8_t* mine, uint32_t (&ew)[SBS]) {
#pragma unroll
        for (int t = 0; t < SBS; ++t) ew[t] = reinterpret_cast<const uint32_t*>(mine)[t];
    }
    // p: the slot's data + lane_off + step_off(t)
    template <int N>
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, const uint32_t (&ew)[N], int t) {
        const uint2 q = *reinterpret_cast<const uint2*>(p);
        const float scale = bits_f32(ew[t]);
        uint32_t w[4];
        FmtF8::widen4(q.x, scale, w);
        FmtF8::widen4(q.y, scale, w + 2);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

struct DlMx4 {
    static constexpr int STEPB = 16;
    struct Mat {
        const uint8_t* w;
        const uint8_t* scales;
    };
    __host__ __device__ static constexpr int scale_bytes(int sbs) { return 16 * sbs; }
    __host__ __device__ static constexpr int scale_words(int sbs) { return sbs / 4; }
    // the e8m0 bytes of the sub-block, row r's SBS bytes as SBS / 4 words: lane l brings word l % (SBS / 4) of row
    // l / (SBS / 4), and they land in lane order, i.e. as [16][SBS] bytes
    template <int SBS>
    __device__ static __forceinline__ void issue_scales(const Mat& m, int tile, int nsteps, int step0, uint8_t* dst,
                                                        int lane) {
        static_assert(SBS % 4 == 0 && 4 * SBS <= 64, "whole words of scale bytes, a lane a word");
        constexpr int per = SBS / 4;
        if (16 * per == WAVE || lane < 16 * per) {  // no branch where every lane has a word (the first tile relies on it)
            const int r = lane / per, j = lane - r * per;
            __builtin_amdgcn_global_load_lds(m.scales + (size_t)(tile * 16 + r) * nsteps + step0 + 4 * j, (lds_void*)dst,
                                             4, 0, 0);
        }
    }
    __device__ static __forceinline__ uint32_t lane_off(int li, int lg) {
        return (uint32_t)((li >> 3) * HALF + (li & 7) * 16 + lg * 4);
    }
    __host__ __device__ static constexpr int step_off(int t) { return (t / 8) * BLK + (t % 8) * 128; }
    __device__ static __forceinline__ uint32_t scale_off(int li, int sbs) { return (uint32_t)(li * sbs); }
    template <int SBS>
    __device__ static __forceinline__ void read_scales(const uint8_t* mine, uint32_t (&ew)[SBS / 4]) {
#pragma unroll
        for (int j = 0; j < SBS / 4; ++j) ew[j] = *reinterpret_cast<const uint32_t*>(mine + 4 * j);
    }
    template <int N>
    __device__ static __forceinline__ bf16x8 frag(const uint8_t* p, const uint32_t (&ew)[N], int t) {
        const uint32_t q = *reinterpret_cast<const uint32_t*>(p);
        const uint32_t ebyte = (ew[t / 4] >> (8 * (t & 3))) & 0xFFu;
        const float s = bits_f32(ebyte << 23);
        uint32_t w[4];
        FmtMx4::widen8(q, s, w);
        return __builtin_bit_cast(bf16x8, make_uint4(w[0], w[1], w[2], w[3]));
    }
};

// ---- the kernel ---------------------------------------------------------------------------------------------------

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
__device__ __forceinline__ f32x4 sub_block(const typename DF::Mat& mat, const uint8_t* __restrict__ cur,
                                           uint8_t* __restrict__ fill, bool do_fill, int fill_tile, int fill_step0,
                                           int nsteps, size_t rowbytes, int lane, int li, int lg, int behind, int sb,
                                           u32x4 (&xb)[SPW], f32x4 acc, int xparts = -1) {
    if (do_fill) issue_loads<DF, GB, SBS>(mat, fill, fill_tile, fill_step0, nsteps, rowbytes, lane);
    // `cur` has landed once at most the loads issued behind it are outstanding
    uint32_t roff = DF::lane_off(li, lg), soff = DF::scale_off(li, SBS);
    // xparts >= 0: the kernel's first tile - the full NBUF - 1 sub-blocks are behind this one, and so are that many of
    // the parts of x (SBS loads each)
    if (xparts >= 0) {
        static_assert(SBS % 4 == 0, "parts of x in fours");
        wait_lead<2 * GB + 1, NBUF - 1, SBS>(xparts, roff, soff);
#pragma unroll
        for (int t = 0; t < SBS; t += 4)
            landed(xb[sb * SBS + t], xb[sb * SBS + t + 1], xb[sb * SBS + t + 2], xb[sb * SBS + t + 3]);
    } else
        wait_behind<2 * GB + 1, NBUF - 1>(behind, roff, soff);
    __builtin_amdgcn_sched_barrier(0);
    const uint8_t* rowp = cur + roff;
    uint32_t ew[DF::scale_words(SBS)];  // what the lane needs of the sub-block's scales
    DF::template read_scales<SBS>(cur + GB * BLK + soff, ew);
#pragma unroll
    for (int t = 0; t < SBS; ++t) {
        const int i = sb * SBS + t;  // the wave's step: a compile-time index once the callers' loops are unrolled
        const bf16x8 a = DF::frag(rowp + DF::step_off(t), ew, t);
        acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(a, __builtin_bit_cast(bf16x8, xb[i]), acc, 0, 0, 0);
    }
    __builtin_amdgcn_sched_barrier(0);
    return acc;
}

// the KS partial tiles folded in wave order and the tile's outputs written; `mine` is this tile's set of partials
template <int KS>
__device__ __forceinline__ void fold_tile(f32x4* __restrict__ mine, f32x4 acc, int wv, int lane, int li, int lg, int M,
                                          int R, int tile, uint16_t* __restrict__ y) {
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
        if (li < M) {
            uint16_t* o = y + (size_t)li * R + tile * 16 + lg * 4;
            o[0] = f32_bf16(s.x);
            o[1] = f32_bf16(s.y);
            o[2] = f32_bf16(s.z);
            o[3] = f32_bf16(s.w);
        }
    }
}

// KS waves a workgroup, each the owner of SPW steps of every row (C = 32 KS SPW); GB 128-byte column blocks a
// sub-block; NBUF ring slots a wave. A tile is MAXSB sub-blocks; the tile loop's body covers a multiple of
// NBUF of them, so every sub-block's slot is a compile-time number. One tile of up to sixteen x rows.
//
// LEAD is set by the host when every workgroup has tiles enough that each sub-block of its first tile still has its full
// NBUF - 1 sub-blocks asked for behind it: the first tile is then straight-line code with nothing conditional in it (the
// compiler counts the loads outstanding exactly only through such code; with a branch round any of them, or this choice
// made inside the kernel, it falls back to waiting for all of them), and its waits let the parts of x asked for behind a
// sub-block's own stay outstanding as well.
template <class DF, int KS, int SPW, int GB, int NBUF, bool LEAD>
__global__ void __launch_bounds__(KS * 64) gemv_mfma_dl(typename DF::Mat mat, const uint4* __restrict__ x,
                                                        uint16_t* __restrict__ y, int R, int C, int M) {
    constexpr int SBS = GB * 128 / DF::STEPB;  // steps a sub-block
    constexpr int SLOT = GB * BLK + DF::scale_bytes(SBS);
    constexpr int MAXSB = SPW / SBS;
    constexpr int TPB = MAXSB >= NBUF ? 1 : NBUF / MAXSB;  // tiles a loop body covers
    static_assert(SPW % SBS == 0 && SLOT % 16 == 0 && (SPW * DF::STEPB) % 128 == 0, "shape");
    static_assert(NBUF >= 2 && NBUF <= 7 && MAXSB <= 7, "ring depth; at most six parts of x behind a sub-block");
    static_assert((NBUF - 1) * (2 * GB + 1) + (MAXSB - 1) * SBS < 64, "the first tile's waits count up to 63 loads");
    static_assert((MAXSB >= NBUF && MAXSB % NBUF == 0) || (MAXSB < NBUF && NBUF % MAXSB == 0), "slots by position");
    extern __shared__ __align__(16) uint8_t lds[];  // KS rings of NBUF slots, then two sets of KS partial tiles
    const int lane = threadIdx.x & (WAVE - 1);
    const int wv = __builtin_amdgcn_readfirstlane(threadIdx.x / WAVE);
    const int li = lane & 15, lg = lane >> 4;
    uint8_t* ring = lds + (size_t)wv * NBUF * SLOT;
    f32x4* part = reinterpret_cast<f32x4*>(lds + (size_t)KS * NBUF * SLOT);

    const int nsteps = C / 32;
    // the wave's steps: its sub-blocks are dealt round the waves, so that the workgroup's waves, which run more or less
    // abreast, ask for neighbouring blocks of a row at about the same time (a little faster than a slice of SPW
    // consecutive steps a wave: 30.5 against 31.8 us on FP8 [18432, 7168])
    const int s0 = wv * SBS;
    constexpr int SB_STEP = KS * SBS;  // from one sub-block of the wave to its next, in steps
    const size_t rowbytes = (size_t)nsteps * DF::STEPB;
    const int chunk4 = C / 8;  // uint4 per row of x

    const int ntiles = R / 16;
    const int grid = (int)gridDim.x, first = (int)blockIdx.x;
    const int nt = first < ntiles ? (ntiles - first + grid - 1) / grid : 0;  // this workgroup's tiles
    const int total = nt * MAXSB;                                            // and the wave's sub-blocks
    // sub-block q of the wave: tile first + (q / MAXSB) grid, steps (q % MAXSB) SBS .. of the wave's slice, slot q % NBUF.
    //
    // The x fragments of the wave's steps stay in registers for the whole kernel (row li of x, the lane's 8 columns of
    // each step); part j of them - SBS loads - is what sub-block j of any tile multiplies by. They and the ring's first
    // loads are asked for in the order the first tile uses them: x part 0, sub-block 0, x part 1, sub-block 1, ...
    // Loads come back in that order, so the first tile's sub-block j can start as soon as its own weights and its own
    // part of x are there, the later parts still on their way out of L2 (every CU reads all of x, 115 KB at 8 rows,
    // and all at once: asked for and waited for in one piece it held the first product back by 2.7 us per 8 rows).
    u32x4 xb[SPW];
    const u32x4* xr = reinterpret_cast<const u32x4*>(x) + (size_t)min(li, M - 1) * chunk4 + lg + (size_t)s0 * 4;
#pragma unroll
    for (int q = 0; q < (NBUF - 1 > MAXSB ? NBUF - 1 : MAXSB); ++q) {
        if (q < MAXSB) {
#pragma unroll
            for (int t = 0; t < SBS; ++t)
                xb[q * SBS + t] = LEAD ? load_untracked(xr + (q * SB_STEP + t) * 4) : xr[(q * SB_STEP + t) * 4];
            __builtin_amdgcn_sched_barrier(0);  // issued here, not where the scheduler would like them
        }
        if (q < NBUF - 1) {
            if (LEAD || q < total)
                issue_loads<DF, GB, SBS>(mat, ring + (q % NBUF) * SLOT, first + (q / MAXSB) * grid,
                                         s0 + (q % MAXSB) * SB_STEP, nsteps, rowbytes, lane);
            __builtin_amdgcn_sched_barrier(0);
        }
    }
    // one body of the tile loop: TPB tiles; FIRST: the kernel's first body under LEAD
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
                    if (FIRST && kk == 0) {
                        // x parts sb + 1 .. MAXSB - 1 were asked for behind this sub-block's weights and its part of x
                        acc = sub_block<DF, SPW, GB, SBS, NBUF>(
                            mat, ring + cur_slot * SLOT, ring + fill_slot * SLOT, true, first + (qf / MAXSB) * grid,
                            s0 + (qf % MAXSB) * SB_STEP, nsteps, rowbytes, lane, li, lg, NBUF - 1, sb, xb, acc,
                            MAXSB - 1 - sb);
                    } else {
                        const int behind = min(NBUF - 1, total - 1 - q);
                        acc = sub_block<DF, SPW, GB, SBS, NBUF>(
                            mat, ring + cur_slot * SLOT, ring + fill_slot * SLOT, qf < total, first + (qf / MAXSB) * grid,
                            s0 + (qf % MAXSB) * SB_STEP, nsteps, rowbytes, lane, li, lg, behind, sb, xb, acc);
                    }
                }
                fold_tile<KS>(part + (size_t)(k & 1) * KS * WAVE, acc, wv, lane, li, lg, M, R, tile, y);
            }
        }
    };
    int k0 = 0;
    if (LEAD) {
        body(0, std::true_type{});
        k0 = TPB;
    }
    for (; k0 < nt; k0 += TPB) body(k0, std::false_type{});
}

template <class DF, int KS, int SPW, int GB, int NBUF>
static int32_t launch_dl(const typename DF::Mat& mat, const void* x, void* y, int R, int C, int M, hipStream_t st) {
    constexpr int SLOT = GB * BLK + DF::scale_bytes(GB * 128 / DF::STEPB);
    const size_t lds = (size_t)KS * NBUF * SLOT + 2 * (size_t)KS * WAVE * sizeof(f32x4);
    if (lds > (size_t)device_info().lds_bytes || C != KS * SPW * 32 || R % 16 != 0 || M < 1 || M > 16) {
        set_error("gemv_mfma_dl: a shape this kernel does not take");
        return ERR_DOMAIN;
    }
    const int ntiles = R / 16;
    const int cap = device_info().cus;  // the rings take most of a CU's LDS: one workgroup a CU
    const int turns = (ntiles + cap - 1) / cap;
    const int grid = (ntiles + turns - 1) / turns;
    constexpr int MAXSB = SPW / (GB * 128 / DF::STEPB);
    const bool lead = (ntiles / grid) * MAXSB >= MAXSB + NBUF - 1;  // the workgroup with the fewest tiles has enough
    auto kern = lead ? gemv_mfma_dl<DF, KS, SPW, GB, NBUF, true> : gemv_mfma_dl<DF, KS, SPW, GB, NBUF, false>;
    if (lds > 64 * 1024) {
        hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void*>(kern),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds);
        if (e != hipSuccess) return hip_status(e, "hipFuncSetAttribute");
    }
    hipLaunchKernelGGL(kern, dim3(grid), dim3(KS * 64), lds, st, mat, static_cast<const uint4*>(x),
                       static_cast<uint16_t*>(y), R, C, M);
    return hip_status(hipGetLastError(), "gemv_mfma_dl launch");
}

// the shapes this kernel takes: 16-row tiles, rows of exactly 7168 columns (8 waves x 28 steps for FP8, 7 x 32 for
// MXFP4), at most sixteen rows of x; FP8 blocks a whole number of tiles tall and of steps wide
bool mfma_dl_fits(int R, int C, int M) {
    return R % 16 == 0 && C == 7168 && M >= 1 && M <= 16 && tuning("mfma_direct") != 0;
}

int32_t gemv_mfma_dl_fp8(const void* w, const float* scales, int sc, int bm, int bn, const void* x, void* y, int R,
                         int C, int M, hipStream_t st) {
    return launch_dl<DlF8, 8, 28, 1, 7>(DlF8::Mat{static_cast<const uint8_t*>(w), scales, sc, bm, bn}, x, y, R, C, M, st);
}
bool mfma_dl_fits_fp8(int R, int C, int M, int bm, int bn) {
    return mfma_dl_fits(R, C, M) && bm % 16 == 0 && bn % 32 == 0;
}

int32_t gemv_mfma_dl_mxfp4(const void* blocks, const void* scales, const void* x, void* y, int R, int C, int M,
                           hipStream_t st) {
    return launch_dl<DlMx4, 7, 32, 2, 4>(DlMx4::Mat{static_cast<const uint8_t*>(blocks), static_cast<const uint8_t*>(scales)},
                                         x, y, R, C, M, st);
}

}  // namespace btb
