// The decode step's kernels between the matvecs, each rounding to bf16 exactly where the reference's card kernels
// do (native/cuda/btb_kernels.cu:250-423, 448-488; the attention's contract: native/cuda/btb_attn_flash.cuh):
//
//   embed           h[t] = table[ids[t]]
//   add_rmsnorm     h = bf16(h + y); x = bf16(h * rsqrt(mean(h^2) + eps) * w)            (or * (1 + w))
//   norm_rope_kv    q/k RMSNorm per head, rope, the row written into the K/V cache at its slot, q out
//   attn_decode     softmax(q K^T * scale) V over the cached keys, split over the keys, last arriver folds
//   silu_mul        m = bf16(bf16(silu(g)) * u) over a [T, 2I] block
//   argmax          the largest logit's index, the lowest on ties (native/src/sample.rs:53-67)
//   publish         token, clock and cache length into pinned host memory at the graph's end; the step's own
//                   bookkeeping (the next token id, the cache length + 1) stays on the device
//
// Every reduction runs in an order fixed by the element's index alone, so a replayed graph repeats its bits.

#include <mutex>

#include "btb_attn.hpp"
#include "btb_common.hpp"
#include "btb_stream.hpp"
#include "btb_tuning.hpp"

#include "../../include/btb_hip.h"

// The partial attention states of btb_hip_attn_decode_noalloc: 4 MiB that every GPU the library runs on holds until
// the process ends. In host code this name is only a stand-in for the symbol; the array's address on a device comes
// from hipGetSymbolAddress (scratch_on_device below) and is what the kernels are handed.
constexpr size_t ATTN_STATIC_FLOATS = BTB_HIP_ATTN_NOALLOC_FLOATS;
static __device__ __align__(256) float scratch[ATTN_STATIC_FLOATS];

namespace btb {

constexpr int MAX_DEVICES = 64;
static float* g_scratch_ptr[MAX_DEVICES];  // per device: where that device's copy of `scratch` lies
static std::mutex g_scratch_lock;

// the current device's copy of `scratch`, looked up once per device (not an allocation: the array is part of the
// code object the device loaded)
static int32_t scratch_on_device(float** out) {
    int dev = 0;
    hipError_t e = hipGetDevice(&dev);
    if (e != hipSuccess) return hip_status(e, "hipGetDevice");
    if (dev < 0 || dev >= MAX_DEVICES) {
        set_error("attn_decode_noalloc: device ordinal beyond the table of per-device scratch addresses");
        return ERR_DOMAIN;
    }
    std::lock_guard<std::mutex> hold(g_scratch_lock);
    if (g_scratch_ptr[dev] == nullptr) {
        float* p = nullptr;
        e = hipGetSymbolAddress(reinterpret_cast<void**>(&p), HIP_SYMBOL(scratch));
        if (e != hipSuccess) return hip_status(e, "hipGetSymbolAddress(scratch)");
        if (p == nullptr) {
            set_error("attn_decode_noalloc: the scratch symbol has no address on this device");
            return ERR_PANIC;
        }
        g_scratch_ptr[dev] = p;
    }
    *out = g_scratch_ptr[dev];
    return OK;
}

// called by btb_hip_init with the device current, so that the first attention call finds the address there already
int32_t attn_static_bind() {
    float* p = nullptr;
    return scratch_on_device(&p);
}

__global__ void __launch_bounds__(256) embed_kernel(const uint4* __restrict__ table, const int32_t* __restrict__ ids,
                                                    uint4* __restrict__ h, int H8, int vocab) {
    const int t = blockIdx.x;
    int id = ids[t];
    id = id < 0 ? 0 : (id >= vocab ? vocab - 1 : id);
    for (int i = threadIdx.x; i < H8; i += 256) h[(size_t)t * H8 + i] = table[(size_t)id * H8 + i];
}

// FAST: rows of a whole number of 8-byte words, at most 4096 values, every pointer 8-byte aligned - a thread's words
// come in with 8-byte loads, all issued together, and stay in registers between the sum and the scaling
template <bool FAST>
__global__ void __launch_bounds__(256) add_rmsnorm_kernel(uint16_t* __restrict__ h, const uint16_t* __restrict__ y,
                                                          const uint16_t* __restrict__ w, float eps,
                                                          uint16_t* __restrict__ x, int H, int centered) {
    __shared__ float red[4];
    const int t = blockIdx.x, tid = threadIdx.x;
    uint16_t* hr = h + (size_t)t * H;
    const uint16_t* yr = y == nullptr ? nullptr : y + (size_t)t * H;
    uint16_t* xr = x + (size_t)t * H;
    // thread i takes the 4-element words i, i + 256, ... of the row, a word's elements in order (the order the matvec's
    // fused staging sums in, where a word is one 8-byte load)
    if constexpr (FAST) {
        constexpr int PER = 4;
        const int n4 = H / 4;
        const uint2* h2 = reinterpret_cast<const uint2*>(hr);
        const uint2* y2 = reinterpret_cast<const uint2*>(yr == nullptr ? hr : yr);
        const uint2* w2 = reinterpret_cast<const uint2*>(w);
        uint2 hv[PER], yv[PER], wv[PER];
#pragma unroll
        for (int k = 0; k < PER; ++k) {  // unconditional, past the row's end the last word again
            const int wd = min(tid + 256 * k, n4 - 1);
            hv[k] = h2[wd];
            yv[k] = y2[wd];
            wv[k] = w2[wd];
        }
        float f[PER][4];
        float ss = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const bool live = tid + 256 * k < n4;
            const uint32_t hw[2] = {hv[k].x, hv[k].y}, yw[2] = {yv[k].x, yv[k].y};
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                float v = (e & 1) ? bf16hi_f32(hw[e / 2]) : bf16lo_f32(hw[e / 2]);
                if (yr != nullptr) v = bfround(v + ((e & 1) ? bf16hi_f32(yw[e / 2]) : bf16lo_f32(yw[e / 2])));
                f[k][e] = v;
                ss = live ? fmaf(v, v, ss) : ss;
            }
            if (yr != nullptr && live)
                reinterpret_cast<uint2*>(hr)[tid + 256 * k] =
                    make_uint2(f32x2_bf16(f[k][0], f[k][1]), f32x2_bf16(f[k][2], f[k][3]));
        }
        const float rstd = rsqrtf(block_sum256(ss, red) / (float)H + eps);
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const uint32_t ww[2] = {wv[k].x, wv[k].y};
            float o[4];
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float wf = (e & 1) ? bf16hi_f32(ww[e / 2]) : bf16lo_f32(ww[e / 2]);
                o[e] = f[k][e] * rstd * (centered ? 1.f + wf : wf);
            }
            if (tid + 256 * k < n4)
                reinterpret_cast<uint2*>(xr)[tid + 256 * k] = make_uint2(f32x2_bf16(o[0], o[1]), f32x2_bf16(o[2], o[3]));
        }
        return;
    }
    float ss = 0.f;
    for (int wd = tid; 4 * wd < H; wd += 256) {
        for (int i = 4 * wd; i < min(4 * wd + 4, H); ++i) {
            float hv = bf16_f32(hr[i]);
            if (yr != nullptr) {
                hv = bfround(hv + bf16_f32(yr[i]));
                hr[i] = f32_bf16(hv);
            }
            ss = fmaf(hv, hv, ss);
        }
    }
    const float rstd = rsqrtf(block_sum256(ss, red) / (float)H + eps);
    for (int i = tid; i < H; i += 256) {
        const float wv = bf16_f32(w[i]);
        xr[i] = f32_bf16(bf16_f32(hr[i]) * rstd * (centered ? 1.f + wv : wv));
    }
}

// one wave per (head, row): a lane holds D / 64 consecutive dims; the rotated half is D / 2 dims away, lane ^ 32
template <int D>
__global__ void __launch_bounds__(64) norm_rope_kv_kernel(const uint16_t* __restrict__ qkv, const uint16_t* __restrict__ wq,
                                                          const uint16_t* __restrict__ wk, float eps,
                                                          const uint16_t* __restrict__ cos_t,
                                                          const uint16_t* __restrict__ sin_t, const int32_t* __restrict__ n0p,
                                                          const int32_t* __restrict__ depth, uint16_t* __restrict__ K,
                                                          uint16_t* __restrict__ V, uint16_t* __restrict__ qo, int Hq,
                                                          int Hk, long long hs, long long rs, int centered,
                                                          const int32_t* __restrict__ tbl,
                                                          const int32_t* __restrict__ rw) {
    constexpr int E = D / 64;
    const int head = blockIdx.x, t = blockIdx.y, lane = threadIdx.x;
    int slot, pos;
    if (rw != nullptr) {  // row t is a sequence of its own: it stands past its prefix and steps, at its step's slot
        SeqPlace sq;
        sq.read(rw, t);
        if (sq.len < 0) return;
        pos = sq.len + sq.step;
        slot = sq.slot(pos);
    } else {
        const int n0 = *n0p;
        slot = n0 + t;
        pos = n0 + (depth != nullptr ? depth[t] : t);
    }
    if (tbl != nullptr) slot = tbl[slot];  // the cache's row map: the row lands where the attention's walk reads it
    const int width = (Hq + 2 * Hk) * D;
    const uint16_t* src = qkv + (size_t)t * width + (size_t)head * D + lane * E;
    if (head >= Hq + Hk) {
        uint16_t* dst = V + (size_t)(head - Hq - Hk) * hs + (size_t)slot * rs + lane * E;
#pragma unroll
        for (int e = 0; e < E; ++e) dst[e] = src[e];
        return;
    }
    const bool is_q = head < Hq;
    const uint16_t* wn = is_q ? wq : wk;
    float v[E];
#pragma unroll
    for (int e = 0; e < E; ++e) v[e] = bf16_f32(src[e]);
    if (wn != nullptr) {
        float ss = 0.f;
#pragma unroll
        for (int e = 0; e < E; ++e) ss = fmaf(v[e], v[e], ss);
        ss = wave_sum(ss);
        const float rstd = rsqrtf(ss / (float)D + eps);
#pragma unroll
        for (int e = 0; e < E; ++e) {
            const float wv = bf16_f32(wn[lane * E + e]);
            v[e] = bfround(v[e] * rstd * (centered ? 1.f + wv : wv));
        }
    }
    // rope: out = bf16(fma(rot, sin, bf16(v * cos))), rot = -v[i + D/2] in the first half, v[i - D/2] in the second
    const uint16_t* cp = cos_t + (size_t)pos * D + lane * E;
    const uint16_t* sp = sin_t + (size_t)pos * D + lane * E;
    const float sgn = lane < 32 ? -1.f : 1.f;
    uint16_t* dst = is_q ? (qo + ((size_t)t * Hq + head) * D + lane * E)
                         : (K + (size_t)(head - Hq) * hs + (size_t)slot * rs + lane * E);
#pragma unroll
    for (int e = 0; e < E; ++e) {
        const float rot = xor32(v[e]);
        const float qc = bfround(v[e] * bf16_f32(cp[e]));
        dst[e] = f32_bf16(fmaf(sgn * rot, bf16_f32(sp[e]), qc));
    }
}

// ------------------------------------------------------------------------------------------------------------
// decode attention, D = 128. A workgroup takes one kv head and one span of the keys; its four waves take the span's
// keys four at a time (16 lanes a key, 8 dims a lane: a wave's load covers four whole 256-byte rows). Each 16-lane
// group keeps an online-softmax state (max, sum, 8 output dims) for each of the G query heads over its own keys, in
// log2 units (the scale carries log2 e, exp is exp2). The groups' states fold through LDS in a fixed order, the
// spans' through memory: every workgroup writes its state, and a second small kernel folds the spans in span order and
// writes bf16(O / L). (A last-arriver fold inside one kernel needs a device-scope fence per workgroup; on this GPU the
// fences of a die's workgroups queue behind one another and cost more than the second launch.) G <= 8.
// ------------------------------------------------------------------------------------------------------------
constexpr int ATT_D = 128;
constexpr int ATT_MAXG = 8;
constexpr int ATT_MAX_STATES = 1024;  // (span, head) states of one kv head that merge_spans turns into factors
// the pass of several rows on the matrix cores (attn_mfma.hip): the partial states of every (row, head, span)
bool attn_mfma_fits(size_t T, size_t G, int span);
int32_t attn_decode_mfma(const void* q, const void* K, const void* V, const int32_t* n0, const int32_t* par, size_t T,
                         size_t Hq, size_t Hk, long long hs, long long rs, float scale_log2, float* part_m,
                         float* part_l, float* part_acc, size_t S, size_t cap, int win, const int32_t* tbl,
                         hipStream_t st);
bool attn_mfma_qkv_fits(size_t T, size_t G, int span);
int32_t attn_decode_mfma_qkv(const void* qkv, const void* wq, const void* wk, float eps, int centered, const void* cos_t,
                             const void* sin_t, const int32_t* n0, const int32_t* depth, const int32_t* par, void* K,
                             void* V, size_t T, size_t Hq, size_t Hk, long long hs, long long rs, float scale_log2,
                             float* part_m, float* part_l, float* part_acc, size_t S, size_t cap, hipStream_t st);

template <int G>
__global__ void __launch_bounds__(256) attn_decode_kernel(const uint16_t* __restrict__ q, const uint16_t* __restrict__ K,
                                                          const uint16_t* __restrict__ V,
                                                          const int32_t* __restrict__ n0p,
                                                          const int32_t* __restrict__ par, int T, int Hq, int Hk, long long hs,
                                                          long long rs, float scale_log2, float* __restrict__ part_m,
                                                          float* __restrict__ part_l, float* __restrict__ part_acc,
                                                          int span, int win, const int32_t* __restrict__ tbl,
                                                          const int32_t* __restrict__ rw) {
    constexpr int D = ATT_D;
    __shared__ float s_m[16][G], s_l[16][G];
    __shared__ __align__(16) float s_acc[16][G][D];
    __shared__ __align__(16) float s_x[16][XCH];  // the streams' exchange areas
    const int g = blockIdx.x, sp = blockIdx.y, t = blockIdx.z, S = gridDim.y;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int sub = lane >> 4, dl = lane & 15;   // the lane's key within a quad of keys, its 8 dims
    const int grp = wv * 4 + sub;                // one of the workgroup's 16 key streams
    SeqPlace sq;
    const SeqPlace* seq = nullptr;
    RowView rv;
    if (rw != nullptr) {
        // row t is a sequence of its own: its keys, in logical order, are its prefix and its own steps up to this one
        sq.read(rw, t);
        if (sq.len < 0) return;  // a padding row: no state is left, and the merge leaves its output alone
        seq = &sq;
        const int last = sq.len + sq.step;
        rv.n = last + 1;
        rv.tree_base = -1;
        rv.tree_mask = 0u;
        rv.k_first = win > 0 ? max(last + 1 - win, 0) : 0;
    } else {
        rv = row_view(par, t, T, *n0p, win);
    }
    const int tree_base = rv.tree_base, n = rv.n, k_first = rv.k_first;
    const uint32_t tree_mask = rv.tree_mask;
    const int k_begin = sp * span, k_end = min(n, k_begin + span);

    // the row's G query heads, the lane's 8 dims of each as bf16 pairs (the scale meets the folded score)
    uint32_t qp[G][4];
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const uint4 raw = *reinterpret_cast<const uint4*>(q + ((size_t)t * Hq + (size_t)g * G + j) * D + dl * 8);
        qp[j][0] = raw.x;
        qp[j][1] = raw.y;
        qp[j][2] = raw.z;
        qp[j][3] = raw.w;
    }
    AttnState<G> st;
    st.init();
    const uint16_t* Kh = K + (size_t)g * hs + dl * 8;
    const uint16_t* Vh = V + (size_t)g * hs + dl * 8;
    // eight keys of the stream a batch: their sixteen loads are issued together, and the next batch's before this one
    // is folded in (past the span's end they fall on its last key again, unused), so a span of several batches - a
    // pass of many rows takes long spans - pays the trip to memory once
    KeyBatch kb;
    load_keys(kb, Kh, Vh, rs, k_begin + grp, max(k_end, 1), -1, tbl, seq);
    for (int key0 = k_begin + grp; key0 < k_end; key0 += 16 * KB) {
        KeyBatch nx;
        load_keys(nx, Kh, Vh, rs, key0 + 16 * KB, k_end, -1, tbl, seq);
        use_keys<G>(kb, key0, k_end, -1, nullptr, nullptr, dl, qp, scale_log2, st, &s_x[grp][0], tree_base, tree_mask,
                    k_first);
        kb = nx;
    }
    // the 16 streams folded in stream order, the workgroup's state out
    const size_t prow = ((size_t)t * Hk + g) * S + sp;  // this workgroup's slot among the partial states
    fold_streams<G>(st, grp, dl, &s_x[grp][0], &s_m[0][0], &s_l[0][0], &s_acc[0][0][0], threadIdx.x,
                    [&](int j, int d, float M, float L, float A) {
                        part_acc[(prow * G + j) * D + d] = A;
                        if (d == 0) {
                            part_m[prow * G + j] = M;
                            part_l[prow * G + j] = L;
                        }
                    });
}

// The same for a pass of several rows and short spans: a workgroup takes one kv head, one span of NBT batches of keys
// (128 NBT keys) and one of the pass's rows. The span's K and V rows are all asked for at once and stay in registers; the
// row brings its G query heads, folds the span's batches into a fresh state and leaves its partial state. A row's
// arithmetic is attn_decode_kernel's at the same span length: a key the row does not see scores -inf there and here,
// and weighs 0. (Several rows of a pass sharing a workgroup's keys was built and measured: it loses - the rows run one
// after another, each with its own fold of the 16 streams, which costs more than the other rows' workgroups reading
// the same keys out of L2; 8 rows over 4096 keys: 3.67 ms a pass with one row a workgroup, 3.71 with two, 4.23 with
// eight.)
template <int G, int NBT>
__global__ void __launch_bounds__(256) attn_decode_rows_kernel(
    const uint16_t* __restrict__ q, const uint16_t* __restrict__ K, const uint16_t* __restrict__ V,
    const int32_t* __restrict__ n0p, const int32_t* __restrict__ par, int T, int Hq, int Hk, long long hs, long long rs,
    float scale_log2, float* __restrict__ part_m, float* __restrict__ part_l, float* __restrict__ part_acc, int win,
    const int32_t* __restrict__ tbl) {
    constexpr int D = ATT_D, SPAN = 16 * KB * NBT;
    __shared__ float s_m[16][G], s_l[16][G];
    __shared__ __align__(16) float s_acc[16][G][D];
    __shared__ __align__(16) float s_x[16][XCH];  // the streams' exchange areas
    const int g = blockIdx.x, sp = blockIdx.y, S = gridDim.y, t = blockIdx.z;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int sub = lane >> 4, dl = lane & 15;
    const int grp = wv * 4 + sub;
    const int n0 = *n0p;
    // the keys the row may see end at n_max (a chain's row t, or the whole pass for a tree)
    const int n_max = par != nullptr ? n0 + T : n0 + t + 1;
    const int k_begin = sp * SPAN, k_lim = min(n_max, k_begin + SPAN);
    const uint16_t* Kh = K + (size_t)g * hs + dl * 8;
    const uint16_t* Vh = V + (size_t)g * hs + dl * 8;
    KeyBatch kb[NBT];
#pragma unroll
    for (int nb = 0; nb < NBT; ++nb) load_keys(kb[nb], Kh, Vh, rs, k_begin + grp + nb * 16 * KB, max(k_lim, 1), -1, tbl);
    const RowView rv = row_view(par, t, T, n0, win);
    const int k_end = min(rv.n, k_begin + SPAN);
    uint32_t qp[G][4];
#pragma unroll
    for (int j = 0; j < G; ++j) {
        const uint4 raw = *reinterpret_cast<const uint4*>(q + ((size_t)t * Hq + (size_t)g * G + j) * D + dl * 8);
        qp[j][0] = raw.x;
        qp[j][1] = raw.y;
        qp[j][2] = raw.z;
        qp[j][3] = raw.w;
    }
    AttnState<G> st;
    st.init();
#pragma unroll
    for (int nb = 0; nb < NBT; ++nb) {
        const int key0 = k_begin + grp + nb * 16 * KB;
        if (key0 < k_end)
            use_keys<G>(kb[nb], key0, k_end, -1, nullptr, nullptr, dl, qp, scale_log2, st, &s_x[grp][0], rv.tree_base,
                        rv.tree_mask, rv.k_first);
    }
    const size_t prow = ((size_t)t * Hk + g) * S + sp;
    fold_streams<G>(st, grp, dl, &s_x[grp][0], &s_m[0][0], &s_l[0][0], &s_acc[0][0][0], threadIdx.x,
                    [&](int j, int d, float M, float L, float A) {
                        part_acc[(prow * G + j) * D + d] = A;
                        if (d == 0) {
                            part_m[prow * G + j] = M;
                            part_l[prow * G + j] = L;
                        }
                    });
}

// The step's own form (one row): the kernel reads the fused qkv row itself. A workgroup takes GW of a kv head's query
// heads (all of them, or fewer: the heads of one kv head then sit in workgroups that share a die's L2, so the keys still
// leave memory once) and one span of the keys. It norms and ropes its query heads (a wave a head; the result never
// leaves LDS), and a workgroup whose span holds slot *n0 also norms and ropes the new key and copies the new value
// into LDS, where its stream takes them from; the first of those workgroups writes both into the cache. One launch
// (norm_rope_kv) less. The key stream's first batch is requested before anything else and its addresses do not depend
// on *n0 (they are clamped to the span and the cache's capacity; which keys count is decided afterwards), so the
// batch travels while *n0, the rope tables and the heads' inputs come in and the heads are prepared. The arithmetic
// is norm_rope_kv_kernel's followed by attn_decode_kernel's: the states it leaves are theirs.
template <int GW>
__global__ void __launch_bounds__(256) attn_decode_qkv_kernel(const uint16_t* __restrict__ qkv, const uint16_t* __restrict__ wq,
                                                              const uint16_t* __restrict__ wk, float eps, int centered,
                                                              const uint16_t* __restrict__ cos_t,
                                                              const uint16_t* __restrict__ sin_t,
                                                              const int32_t* __restrict__ n0p, uint16_t* __restrict__ K,
                                                              uint16_t* __restrict__ V, int Hq, int Hk, long long hs,
                                                              long long rs, float scale_log2, float* __restrict__ part_m,
                                                              float* __restrict__ part_l, float* __restrict__ part_acc,
                                                              int span, int cap) {
    constexpr int D = ATT_D;
    __shared__ uint32_t s_q[GW][D / 2];  // the heads' q after norm and rope, bf16 pairs
    __shared__ __align__(16) uint16_t s_k[D], s_v[D];
    __shared__ float s_m[16][GW], s_l[16][GW];
    __shared__ __align__(16) float s_acc[16][GW][D];
    __shared__ __align__(16) float s_x[16][XCH];  // the streams' exchange areas
    const int Gt = Hq / Hk;                                  // query heads a kv head
    const int g = blockIdx.x % Hk, part = blockIdx.x / Hk;   // consecutive workgroups: consecutive kv heads
    const int j0 = part * GW;                                // the first of this workgroup's heads among the Gt
    const int sp = blockIdx.y, S = gridDim.y;
    const int lane = threadIdx.x & 63, wv = threadIdx.x >> 6;
    const int sub = lane >> 4, dl = lane & 15, grp = wv * 4 + sub;
    const int k_begin = sp * span;
    const int k_lim = max(min(k_begin + span, cap), 1);      // the last slot of the cache this span may touch, + 1
    const uint16_t* Kh = K + (size_t)g * hs + dl * 8;
    const uint16_t* Vh = V + (size_t)g * hs + dl * 8;
    const int key_first = k_begin + grp;
    KeyBatch kb;
    load_keys_upto(kb, Kh, Vh, rs, key_first, k_lim);

    const int n0 = *n0p;
    const int k_end = min(n0 + 1, k_begin + span);
    if (k_begin > n0) {
        // A span past the row's keys (spans are cut from the cache's capacity, not from its length): the state the fold
        // below would leave - no maximum, no sum, zeros - written at once; the workgroup prepares no head, waits for no
        // key and leaves its CU to the workgroups that have work.
        const size_t prow = (size_t)g * gridDim.y + sp;
        for (int o = threadIdx.x; o < GW * D; o += 256) {
            const int j = o / D, d = o - j * D;
            part_acc[((prow * Gt) + j0 + j) * D + d] = 0.f;
            if (d == 0) {
                part_m[prow * Gt + j0 + j] = bits_f32(0xff800000u);
                part_l[prow * Gt + j0 + j] = 0.f;
            }
        }
        return;
    }
    constexpr int NQ = (GW + 3) / 4;  // query heads a wave prepares
    HeadIn qin[NQ];
#pragma unroll
    for (int i = 0; i < NQ; ++i)
        qin[i] = head_request<false>(qkv + (size_t)(g * Gt + j0 + min(wv + 4 * i, GW - 1)) * D, wq, cos_t, sin_t, n0, lane);
    const bool holds_own = n0 >= k_begin && n0 < k_begin + span;  // this workgroup's span holds the new slot
    const bool preps_k = wv == 3 && holds_own;
    const HeadIn kin = head_request<false>(qkv + (size_t)(Hq + g) * D, wk, cos_t, sin_t, n0, lane);
    const uint32_t vraw = reinterpret_cast<const uint32_t*>(qkv + (size_t)(Hq + Hk + g) * D)[lane];

#pragma unroll
    for (int i = 0; i < NQ; ++i) {
        const int j = wv + 4 * i;
        uint16_t o[2];
        head_finish(qin[i], wq != nullptr, eps, centered, lane, o);
        if (j < GW) s_q[j][lane] = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
    }
    if (preps_k) {
        uint16_t o[2];
        head_finish(kin, wk != nullptr, eps, centered, lane, o);
        s_k[lane * 2] = o[0];
        s_k[lane * 2 + 1] = o[1];
        s_v[lane * 2] = (uint16_t)(vraw & 0xFFFFu);
        s_v[lane * 2 + 1] = (uint16_t)(vraw >> 16);
        if (part == 0 && n0 < cap) {  // a slot past the cache's end is never written (spans are rounded up past it)
            reinterpret_cast<uint32_t*>(K + (size_t)g * hs + (size_t)n0 * rs)[lane] = (uint32_t)o[0] | ((uint32_t)o[1] << 16);
            reinterpret_cast<uint32_t*>(V + (size_t)g * hs + (size_t)n0 * rs)[lane] = vraw;
        }
    }
    __syncthreads();

    uint32_t qp[GW][4];
#pragma unroll
    for (int j = 0; j < GW; ++j)
#pragma unroll
        for (int e = 0; e < 4; ++e) qp[j][e] = s_q[j][dl * 4 + e];
    AttnState<GW> st;
    st.init();
    // a span of several batches asks for the next one before it folds the current one in (past the span's end the
    // request falls on its last key again and is dropped)
    const bool batches = k_begin + 16 * KB < k_end;  // uniform: the span holds more than one batch of live keys
    for (int key0 = key_first; key0 < k_end; key0 += 16 * KB) {
        KeyBatch nx;
        if (batches) load_keys_upto(nx, Kh, Vh, rs, key0 + 16 * KB, k_lim);
        use_keys<GW, true>(kb, key0, k_end, holds_own ? n0 : -1, s_k, s_v, dl, qp, scale_log2, st, &s_x[grp][0]);
        if (batches) kb = nx;
    }
    const size_t prow = (size_t)g * S + sp;
    fold_streams<GW>(st, grp, dl, &s_x[grp][0], &s_m[0][0], &s_l[0][0], &s_acc[0][0][0], threadIdx.x,
                     [&](int j, int d, float M, float L, float A) {
                         part_acc[((prow * Gt) + j0 + j) * D + d] = A;
                         if (d == 0) {
                             part_m[prow * Gt + j0 + j] = M;
                             part_l[prow * Gt + j0 + j] = L;
                         }
                     });
}

// the spans' states folded in span order: one workgroup per (row, kv head). Launched right after attn_decode_kernel,
// it reads what that kernel wrote across a kernel boundary, so no fence or arrival count is needed.
template <int G>
__global__ void __launch_bounds__(256) attn_merge_kernel(uint16_t* __restrict__ att, int Hq, int Hk, int S,
                                                         const float* __restrict__ part_m,
                                                         const float* __restrict__ part_l,
                                                         const float* __restrict__ part_acc,
                                                         const int32_t* __restrict__ rw) {
    extern __shared__ float f_m[];  // [S][G] maxima / factors, then [S][G] sums
    const int g = blockIdx.x, t = blockIdx.y;
    if (rw != nullptr && rw[5 + 3 * t] < 0) return;  // a padding row of a pass of sequences: its output is left alone
    merge_spans<G, false>(att + (size_t)t * Hq * ATT_D, g, S, ((size_t)t * Hk + g) * S, part_m, part_l, part_acc, f_m,
                          threadIdx.x);
}

// the fold of a few spans (up to MERGE_FEW: the step's 18 are such): one workgroup of 128 per (row, query head)
constexpr int MERGE_FEW = 20;
template <int G, bool SEQS, int MS>
__global__ void __launch_bounds__(128) attn_merge_few_kernel(uint16_t* __restrict__ att, int Hq, int Hk, int S,
                                                             const float* __restrict__ part_m,
                                                             const float* __restrict__ part_l,
                                                             const float* __restrict__ part_acc,
                                                             const int32_t* __restrict__ rw) {
    const int g = blockIdx.x / G, j = blockIdx.x % G, t = blockIdx.y;
    // SEQS: a pass of sequences, whose padding rows are skipped. A kernel of its own, so that the others do not read
    // rw's pointer ahead of everything else (a trip for the kernel's arguments of its own: the step's pair of launches
    // 12.1 -> 15.6 us a layer with it).
    if constexpr (SEQS) {
        if (rw[5 + 3 * t] < 0) return;
    }
    merge_spans_few<G, MS>(att + (size_t)t * Hq * ATT_D, g, j, S, ((size_t)t * Hk + g) * S, part_m, part_l,
                                  part_acc, threadIdx.x);
}

// The fold behind every attention kernel here. Up to 64 spans: the fold that shares nothing, built for 20, 40 and 64
// spans (the step's pair of launches 13.6 -> 11.75 us a layer against the general fold at 18 spans; a pass
// of 4 / 8 rows over 36 spans 2.95 / 2.96 -> 2.86 / 2.91 ms); more: the general one. The same bits either way.
template <int G>
void launch_merge(hipStream_t st, void* att, size_t T, size_t Hq, size_t Hk, size_t S, const float* part_m,
                  const float* part_l, const float* part_acc, const int32_t* rw) {
    size_t S_few = MERGE_FEW;
#define FEW(SEQS, MS)                                                                                               \
    hipLaunchKernelGGL((attn_merge_few_kernel<G, SEQS, MS>), dim3((unsigned)(Hk * G), (unsigned)T), dim3(128), 0, st, \
                       static_cast<uint16_t*>(att), (int)Hq, (int)Hk, (int)S, part_m, part_l, part_acc, rw)
    if (tuning("attn_merge_few") == 0) S_few = 0;  // 0: the general fold whatever the count (the tests compare the two)
    if (S <= S_few && rw == nullptr) FEW(false, MERGE_FEW);
    else if (S <= S_few) FEW(true, MERGE_FEW);
    else if (S <= 2 * S_few && rw == nullptr) FEW(false, 2 * MERGE_FEW);
    else if (S <= 2 * S_few) FEW(true, 2 * MERGE_FEW);
    else if (S_few != 0 && S <= 64 && rw == nullptr) FEW(false, 64);  // a lane a span: as many as a wave has lanes
    else if (S_few != 0 && S <= 64) FEW(true, 64);
    else
        hipLaunchKernelGGL(attn_merge_kernel<G>, dim3((unsigned)Hk, (unsigned)T), dim3(256), 2 * S * G * sizeof(float),
                           st, static_cast<uint16_t*>(att), (int)Hq, (int)Hk, (int)S, part_m, part_l, part_acc, rw);
#undef FEW
}

__global__ void __launch_bounds__(256) silu_mul_kernel(const uint16_t* __restrict__ gu, uint16_t* __restrict__ m,
                                                       size_t T, size_t I) {
    const size_t n = T * I;
    for (size_t k = (size_t)blockIdx.x * 256 + threadIdx.x; k < n; k += (size_t)gridDim.x * 256) {
        const size_t t = k / I, i = k - t * I;
        const float g = bf16_f32(gu[t * 2 * I + i]);
        const float u = bf16_f32(gu[t * 2 * I + I + i]);
        const float s = bfround(g / (1.f + expf(-g)));
        m[k] = f32_bf16(s * u);
    }
}

// one workgroup of 1024 per row: each thread its own strided elements in ascending order, taking an element only when
// it is strictly larger than its best so far (a tie keeps the earlier; a NaN never wins; the scan starts from -inf as
// native/src/sample.rs:53-67 does), then the (value, index) maximum over the block in the total order value descending,
// index ascending
// PUBLISH: one row, and the thread that holds the pick goes on with the step's end (publish_kernel's duties) - one
// launch less at the end of a step.
template <bool PUBLISH>
__global__ void __launch_bounds__(1024) argmax_kernel(const uint16_t* __restrict__ logits, int32_t* __restrict__ out,
                                                      int V, int32_t* __restrict__ n0, int32_t* __restrict__ next_ids,
                                                      int32_t* out_tok, int32_t* out_n0, long long* out_ts) {
    __shared__ float s_v[16];
    __shared__ int s_i[16];
    const int t = blockIdx.x, tid = threadIdx.x;
    const uint16_t* row = logits + (size_t)t * V;
    float bv = bits_f32(0xff800000u);
    int bi = 0x7fffffff;
    if ((V & 7) == 0 && (reinterpret_cast<uintptr_t>(row) & 15u) == 0) {
        // eight logits a load, four loads in flight: a thread meets its elements in ascending index order
        const uint4* row8 = reinterpret_cast<const uint4*>(row);
        const int n8 = V / 8;
        for (int base = tid; base < n8; base += 4 * 1024) {
            uint4 v[4];
#pragma unroll
            for (int q = 0; q < 4; ++q) v[q] = row8[min(base + q * 1024, n8 - 1)];
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const int i8 = base + q * 1024;
                if (i8 < n8) {
                    const uint32_t w[4] = {v[q].x, v[q].y, v[q].z, v[q].w};
#pragma unroll
                    for (int e = 0; e < 8; ++e) {
                        const float x = (e & 1) ? bf16hi_f32(w[e >> 1]) : bf16lo_f32(w[e >> 1]);
                        if (x > bv) {
                            bv = x;
                            bi = i8 * 8 + e;
                        }
                    }
                }
            }
        }
    } else {
        for (int i = tid; i < V; i += 1024) {
            const float v = bf16_f32(row[i]);
            if (v > bv) {
                bv = v;
                bi = i;
            }
        }
    }
#pragma unroll
    for (int s = 32; s > 0; s >>= 1) {
        const float ov = __shfl_xor(bv, s, WAVE);
        const int oi = __shfl_xor(bi, s, WAVE);
        if (ov > bv || (ov == bv && oi < bi)) {
            bv = ov;
            bi = oi;
        }
    }
    if ((tid & 63) == 0) {
        s_v[tid >> 6] = bv;
        s_i[tid >> 6] = bi;
    }
    __syncthreads();
    if (tid == 0) {
        for (int k = 1; k < 16; ++k)
            if (s_v[k] > bv || (s_v[k] == bv && s_i[k] < bi)) {
                bv = s_v[k];
                bi = s_i[k];
            }
        const int tok = bi == 0x7fffffff ? 0 : bi;  // nothing above -inf (or only NaNs): index 0, as the reference's scan
        out[t] = tok;
        if constexpr (PUBLISH) {
            const int len = *n0 + 1;
            if (next_ids != nullptr) *next_ids = tok;
            *n0 = len;
            if (out_tok != nullptr) {
                *out_tok = tok;
                if (out_ts != nullptr) *out_ts = (long long)wall_clock64();
                __threadfence_system();
                if (out_n0 != nullptr) *out_n0 = len;
            }
        }
    }
}

// the step's end: the picked token becomes the next step's input and the cache grows by one on the device; with
// pinned host buffers, the token, the GPU clock and then (after a system fence) the new length go to the host
__global__ void publish_kernel(int32_t* __restrict__ n0, const int32_t* __restrict__ picked, int32_t* __restrict__ next_ids,
                               int32_t* out_tok, int32_t* out_n0, long long* out_ts, int advance) {
    if (threadIdx.x != 0 || blockIdx.x != 0) return;
    const int tok = *picked;
    const int len = *n0 + (advance ? 1 : 0);
    if (next_ids != nullptr) *next_ids = tok;
    if (advance) *n0 = len;
    if (out_tok != nullptr) {
        *out_tok = tok;
        if (out_ts != nullptr) *out_ts = (long long)wall_clock64();
        __threadfence_system();
        if (out_n0 != nullptr) *out_n0 = len;
    }
}

static bool al(const void* p, uintptr_t a) { return (reinterpret_cast<uintptr_t>(p) & (a - 1)) == 0; }

}  // namespace btb

using namespace btb;

extern "C" {

int32_t btb_hip_embed(const void* table, const int32_t* ids, void* h, size_t T, size_t H, size_t vocab, void* stream) {
    if (table == nullptr || ids == nullptr || h == nullptr) return ERR_NULL;
    if (T == 0 || H == 0 || vocab == 0 || H % 8 != 0 || T > 65535 || vocab > 0x7FFFFFFFull) return ERR_DOMAIN;
    if (!al(table, 16) || !al(h, 16) || !al(ids, 4)) return ERR_DOMAIN;
    hipLaunchKernelGGL(embed_kernel, dim3((unsigned)T), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint4*>(table), ids, static_cast<uint4*>(h), (int)(H / 8), (int)vocab);
    return hip_status(hipGetLastError(), "embed launch");
}

int32_t btb_hip_add_rmsnorm(void* h, const void* y, const void* w, float eps, void* x, size_t T, size_t H,
                            int32_t centered, void* stream) {
    if (h == nullptr || w == nullptr || x == nullptr) return ERR_NULL;
    if (T == 0 || H == 0 || T > 0x7FFFFFFFull || H > 0x7FFFFFFFull || !(eps >= 0.f)) return ERR_DOMAIN;
    if (!al(h, 2) || !al(y, 2) || !al(w, 2) || !al(x, 2)) return ERR_DOMAIN;
    const bool fast = H % 4 == 0 && H <= 4096 && al(h, 8) && al(y, 8) && al(w, 8) && al(x, 8);
    auto kern = fast ? add_rmsnorm_kernel<true> : add_rmsnorm_kernel<false>;
    hipLaunchKernelGGL(kern, dim3((unsigned)T), dim3(256), 0, static_cast<hipStream_t>(stream), static_cast<uint16_t*>(h), static_cast<const uint16_t*>(y),
                       static_cast<const uint16_t*>(w), eps, static_cast<uint16_t*>(x), (int)H, centered);
    return hip_status(hipGetLastError(), "add_rmsnorm launch");
}

static int32_t norm_rope_kv_any(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                                const void* sin_t, const int32_t* n0, const int32_t* depth, void* K, void* V, void* q,
                                size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered,
                                const int32_t* tbl, void* stream, const int32_t* rw = nullptr) {
    if (qkv == nullptr || cos_t == nullptr || sin_t == nullptr || (n0 == nullptr && rw == nullptr) || K == nullptr ||
        V == nullptr || q == nullptr)
        return ERR_NULL;
    if (T == 0 || Hq == 0 || Hk == 0 || T > 65535 || Hq + 2 * Hk > 0x7FFFFFFFull || hs <= 0 || rs <= 0 ||
        !(eps >= 0.f) || !al(tbl, 4) || !al(rw, 4))
        return ERR_DOMAIN;
    if (D != 64 && D != 128 && D != 256) return ERR_DOMAIN;
    const dim3 grid((unsigned)(Hq + 2 * Hk), (unsigned)T);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define NRK(DD)                                                                                                      \
    hipLaunchKernelGGL(norm_rope_kv_kernel<DD>, grid, dim3(64), 0, st, static_cast<const uint16_t*>(qkv),             \
                       static_cast<const uint16_t*>(wq), static_cast<const uint16_t*>(wk), eps,                      \
                       static_cast<const uint16_t*>(cos_t), static_cast<const uint16_t*>(sin_t), n0, depth,          \
                       static_cast<uint16_t*>(K), static_cast<uint16_t*>(V), static_cast<uint16_t*>(q), (int)Hq,      \
                       (int)Hk, (long long)hs, (long long)rs, centered, tbl, rw)
    if (D == 64)
        NRK(64);
    else if (D == 128)
        NRK(128);
    else
        NRK(256);
#undef NRK
    return hip_status(hipGetLastError(), "norm_rope_kv launch");
}

int32_t btb_hip_norm_rope_kv(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                             const void* sin_t, const int32_t* n0, const int32_t* depth, void* K, void* V, void* q,
                             size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered,
                             void* stream) {
    return norm_rope_kv_any(qkv, wq, wk, eps, cos_t, sin_t, n0, depth, K, V, q, T, Hq, Hk, D, hs, rs, centered, nullptr,
                            stream);
}

int32_t btb_hip_norm_rope_kv_tbl(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                                 const void* sin_t, const int32_t* n0, const int32_t* depth, void* K, void* V, void* q,
                                 size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered,
                                 const int32_t* tbl, void* stream) {
    if (tbl == nullptr) return ERR_NULL;
    return norm_rope_kv_any(qkv, wq, wk, eps, cos_t, sin_t, n0, depth, K, V, q, T, Hq, Hk, D, hs, rs, centered, tbl,
                            stream);
}

int32_t btb_hip_norm_rope_kv_seqs(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                                  const void* sin_t, const int32_t* rw, void* K, void* V, void* q, size_t T, size_t Hq,
                                  size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered, void* stream) {
    if (rw == nullptr) return ERR_NULL;
    return norm_rope_kv_any(qkv, wq, wk, eps, cos_t, sin_t, nullptr, nullptr, K, V, q, T, Hq, Hk, D, hs, rs, centered,
                            nullptr, stream, rw);
}

size_t btb_hip_attn_scratch_floats(size_t T, size_t Hq, size_t Hk, size_t D, size_t S) {
    // part_m and part_l [T, Hk, S, G], part_acc [T, Hk, S, G, D]: Hk * G = Hq
    (void)Hk;
    return T * Hq * S * (2 + D);
}

// `work` is the caller's workspace, or nullptr for the library's own static array on the current device
// `parts`: the caller's own three state arrays (part_m, part_l [T Hq S], part_acc [T Hq S D]) in place of one workspace;
// the call then takes spans of `cap / S` keys exactly and only the kernel whose loads stay on live keys, so `cap` need
// not be the cache's true capacity
static int32_t attn_decode_any(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                               const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                               float scale, size_t cap, size_t S, float* work, bool own_scratch, void* stream,
                               int64_t win = 0, const int32_t* tbl = nullptr, float* const* parts = nullptr,
                               const int32_t* rw = nullptr) {
    if (q == nullptr || K == nullptr || V == nullptr || att == nullptr || (n0 == nullptr && rw == nullptr) ||
        (!own_scratch && work == nullptr && parts == nullptr))
        return ERR_NULL;
    if (rw != nullptr && (parts == nullptr || par != nullptr || tbl != nullptr || !al(rw, 4))) return ERR_DOMAIN;
    if (parts != nullptr && (parts[0] == nullptr || parts[1] == nullptr || parts[2] == nullptr)) return ERR_NULL;
    if (T == 0 || Hq == 0 || Hk == 0 || S == 0 || cap == 0 || T > 65535 || S > 1024 || Hq % Hk != 0 || hs <= 0 ||
        rs <= 0 || !(scale == scale))
        return ERR_DOMAIN;
    const size_t G = Hq / Hk;
    if (D != (size_t)ATT_D || G > (size_t)ATT_MAXG) {
        set_error("attn_decode: head_dim 128 and at most 8 query heads per kv head");
        return ERR_DOMAIN;
    }
    if (!al(q, 16) || !al(K, 16) || !al(V, 16) || !al(par, 4) || !al(tbl, 4) || (rs % 8) != 0 || (hs % 8) != 0 ||
        win < 0 || win > 0x7FFFFFFF)
        return ERR_DOMAIN;
    if (par != nullptr && T > 32) {
        set_error("attn_decode: a tree pass holds at most 32 rows");
        return ERR_DOMAIN;
    }
    if (S * G > (size_t)ATT_MAX_STATES) {
        set_error("attn_decode: spans * (query heads per kv head) is at most 1024");
        return ERR_DOMAIN;
    }
    if (own_scratch) {
        if (T * Hq * S > ATTN_STATIC_FLOATS / (2 + D)) {
            set_error("attn_decode_noalloc: T * Hq * S * (2 + D) floats of partial states exceed the 4 MiB the library "
                      "holds; use fewer spans or btb_hip_attn_decode with a workspace");
            return ERR_DOMAIN;
        }
        const int32_t rc = scratch_on_device(&work);
        if (rc != OK) return rc;
    }
    // a span is a whole number of the workgroup's batches of keys (16 streams by 8 keys): a batch is the unit of its
    // work, and a span that ends inside one pays for all of it
    const int span = (int)(((cap + S - 1) / S + 127) / 128 * 128);
    float* part_m = parts != nullptr ? parts[0] : work;
    float* part_l = parts != nullptr ? parts[1] : work + T * Hq * S;
    float* part_acc = parts != nullptr ? parts[2] : work + 2 * T * Hq * S;
    if (parts != nullptr && (!al(part_m, 4) || !al(part_l, 4) || !al(part_acc, 16))) return ERR_DOMAIN;
    const float scale_log2 = scale * 1.4426950408889634f;
    const dim3 grid((unsigned)Hk, (unsigned)S, (unsigned)T);
    hipStream_t st = static_cast<hipStream_t>(stream);
#define ATT(GG)                                                                                                      \
    hipLaunchKernelGGL(attn_decode_kernel<GG>, grid, dim3(256), 0, st, static_cast<const uint16_t*>(q),              \
                       static_cast<const uint16_t*>(K), static_cast<const uint16_t*>(V), n0, par, (int)T, (int)Hq,   \
                       (int)Hk, (long long)hs, (long long)rs, scale_log2, part_m, part_l, part_acc, span, (int)win,   \
                       tbl, rw);                                                                                    \
    launch_merge<GG>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, rw)
    // Several rows and spans of 128 keys: the matrix cores, every row of the pass that shares a kv head in one workgroup
    // (attn_mfma.hip). A pass of 8 rows over 4096 keys: 22.7 us a layer on the vector kernel below (spans of one or two
    // batches of keys, asked for at once and kept in registers, a workgroup a row), which stays for spans of 256 keys
    // and behind the knob attn_mfma = 0.
    if (parts == nullptr && attn_mfma_fits(T, G, span)) {
        const int32_t rc = attn_decode_mfma(q, K, V, n0, par, T, Hq, Hk, (long long)hs, (long long)rs, scale_log2, part_m,
                                            part_l, part_acc, S, cap, (int)win, tbl, st);
        if (rc != OK) return rc;
        if (G == 4) launch_merge<4>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, nullptr);
        else launch_merge<2>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, nullptr);
        return hip_status(hipGetLastError(), "attn_decode launch");
    }
    if (parts == nullptr && T >= 2 && (span == 128 || span == 256) && (G == 2 || G == 4)) {
        const dim3 rgrid((unsigned)Hk, (unsigned)S, (unsigned)T);
#define ATTR(GG, NB)                                                                                                  \
    hipLaunchKernelGGL((attn_decode_rows_kernel<GG, NB>), rgrid, dim3(256), 0, st, static_cast<const uint16_t*>(q),   \
                       static_cast<const uint16_t*>(K), static_cast<const uint16_t*>(V), n0, par, (int)T, (int)Hq,    \
                       (int)Hk, (long long)hs, (long long)rs, scale_log2, part_m, part_l, part_acc, (int)win, tbl);      \
    launch_merge<GG>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, nullptr)
        if (G == 4 && span == 128) { ATTR(4, 1); }
        else if (G == 4) { ATTR(4, 2); }
        else if (span == 128) { ATTR(2, 1); }
        else { ATTR(2, 2); }
#undef ATTR
        return hip_status(hipGetLastError(), "attn_decode launch");
    }
    switch (G) {
        case 1: ATT(1); break;
        case 2: ATT(2); break;
        case 4: ATT(4); break;
        case 8: ATT(8); break;
        default:
            set_error("attn_decode: 1, 2, 4 or 8 query heads per kv head");
            return ERR_DOMAIN;
    }
#undef ATT
    return hip_status(hipGetLastError(), "attn_decode launch");
}

int32_t btb_hip_attn_decode(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                            const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                            float scale, size_t cap, size_t S, float* workspace, void* stream) {
    return attn_decode_any(q, K, V, att, n0, par, T, Hq, Hk, D, hs, rs, scale, cap, S, workspace, false, stream);
}

int32_t btb_hip_attn_decode_win(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                                float scale, size_t cap, size_t S, int64_t win, const int32_t* tbl, float* workspace,
                                void* stream) {
    return attn_decode_any(q, K, V, att, n0, par, T, Hq, Hk, D, hs, rs, scale, cap, S, workspace, false, stream, win,
                           tbl);
}

int32_t btb_hip_attn_decode_parts(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                  const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                                  float scale, size_t span, size_t S, int64_t win, const int32_t* tbl, float* part_m,
                                  float* part_l, float* part_acc, void* stream) {
    if (span == 0 || span % 128 != 0 || S == 0 || span > 0x7FFFFFFFull / (S ? S : 1)) {
        set_error("attn_decode_parts: spans are a whole number of 128-key batches");
        return ERR_DOMAIN;
    }
    float* const parts[3] = {part_m, part_l, part_acc};
    return attn_decode_any(q, K, V, att, n0, par, T, Hq, Hk, D, hs, rs, scale, span * S, S, nullptr, false, stream, win,
                           tbl, parts);
}

int32_t btb_hip_attn_decode_seqs(const void* q, const void* K, const void* V, void* att, const int32_t* rw, size_t T,
                                 size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, float scale, size_t span,
                                 size_t S, int64_t win, float* part_m, float* part_l, float* part_acc, void* stream) {
    if (rw == nullptr) return ERR_NULL;
    if (span == 0 || span % 128 != 0 || S == 0 || span > 0x7FFFFFFFull / (S ? S : 1)) {
        set_error("attn_decode_seqs: spans are a whole number of 128-key batches");
        return ERR_DOMAIN;
    }
    float* const parts[3] = {part_m, part_l, part_acc};
    return attn_decode_any(q, K, V, att, nullptr, nullptr, T, Hq, Hk, D, hs, rs, scale, span * S, S, nullptr, false,
                           stream, win, nullptr, parts, rw);
}

int32_t btb_hip_attn_decode_noalloc(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                    const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs,
                                    int64_t rs, float scale, size_t cap, size_t S, void* stream) {
    return attn_decode_any(q, K, V, att, n0, par, T, Hq, Hk, D, hs, rs, scale, cap, S, nullptr, true, stream);
}

int32_t btb_hip_attn_decode_qkv(const void* qkv, const void* wq, const void* wk, float eps, int32_t centered,
                                const void* cos_t, const void* sin_t, const int32_t* n0, void* K, void* V, void* att,
                                size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, float scale, size_t cap,
                                size_t S, float* workspace, void* stream) {
    if (qkv == nullptr || cos_t == nullptr || sin_t == nullptr || n0 == nullptr || K == nullptr || V == nullptr ||
        att == nullptr || workspace == nullptr)
        return ERR_NULL;
    if (Hq == 0 || Hk == 0 || S == 0 || cap == 0 || S > 1024 || Hq % Hk != 0 || hs <= 0 || rs <= 0 ||
        !(scale == scale) || !(eps >= 0.f))
        return ERR_DOMAIN;
    const size_t G = Hq / Hk;
    if (D != (size_t)ATT_D || G > (size_t)ATT_MAXG) {
        set_error("attn_decode_qkv: head_dim 128 and at most 8 query heads per kv head");
        return ERR_DOMAIN;
    }
    if (!al(qkv, 4) || !al(K, 16) || !al(V, 16) || (rs % 8) != 0 || (hs % 8) != 0) return ERR_DOMAIN;
    if (S * G > (size_t)ATT_MAX_STATES) {
        set_error("attn_decode_qkv: spans * (query heads per kv head) is at most 1024");
        return ERR_DOMAIN;
    }
    // a span is a whole number of the workgroup's batches of keys (16 streams by 8 keys): a batch is the unit of its
    // work, and a span that ends inside one pays for all of it
    const int span = (int)(((cap + S - 1) / S + 127) / 128 * 128);
    float* part_m = workspace;
    float* part_l = workspace + Hq * S;
    float* part_acc = workspace + 2 * Hq * S;
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    // query heads a workgroup takes: all G of its kv head, or fewer (the workgroups of one kv head are Hk apart in
    // the grid, which on this GPU - workgroups dealt to its eight dies in turn - keeps them on one die when Hk is 8)
    // Measured on MI355X (Qwen3-4B shape, 4096 keys of 4608 slots, whole step): two heads a workgroup and 18 spans (of
    // 256 keys) 2.215 ms, four heads 2.249, one head 2.333; two heads with 16 spans (288 keys: 2.25 batches) 2.274.
    int gw = tuning("attn_heads_per_wg");
    if (gw <= 0 || gw > (int)G || G % gw != 0 || (gw & (gw - 1)) != 0) gw = G >= 4 ? 2 : (int)G;
    const dim3 grid((unsigned)(Hk * (G / gw)), (unsigned)S);
#define ATT(GW)                                                                                                      \
    hipLaunchKernelGGL(attn_decode_qkv_kernel<GW>, grid, dim3(256), 0, st, static_cast<const uint16_t*>(qkv),        \
                       static_cast<const uint16_t*>(wq), static_cast<const uint16_t*>(wk), eps, centered ? 1 : 0,    \
                       static_cast<const uint16_t*>(cos_t), static_cast<const uint16_t*>(sin_t), n0,                 \
                       static_cast<uint16_t*>(K), static_cast<uint16_t*>(V), (int)Hq, (int)Hk, (long long)hs,        \
                       (long long)rs, scale_log2, part_m, part_l, part_acc, span, (int)cap)
#define MERGE(GG) launch_merge<GG>(st, att, 1, Hq, Hk, S, part_m, part_l, part_acc, nullptr)
    if (G != 1 && G != 2 && G != 4 && G != 8) {
        set_error("attn_decode_qkv: 1, 2, 4 or 8 query heads per kv head");
        return ERR_DOMAIN;
    }
    switch (gw) {
        case 1: ATT(1); break;
        case 2: ATT(2); break;
        case 4: ATT(4); break;
        default: ATT(8); break;
    }
    switch (G) {
        case 1: MERGE(1); break;
        case 2: MERGE(2); break;
        case 4: MERGE(4); break;
        default: MERGE(8); break;
    }
#undef ATT
#undef MERGE
    return hip_status(hipGetLastError(), "attn_decode_qkv launch");
}

int32_t btb_hip_attn_rows_fused(size_t T, size_t Hq, size_t Hk, size_t D, size_t cap, size_t S) {
    if (T == 0 || Hq == 0 || Hk == 0 || S == 0 || cap == 0 || Hq % Hk != 0 || D != (size_t)ATT_D) return 0;
    const int span = (int)(((cap + S - 1) / S + 127) / 128 * 128);
    return attn_mfma_qkv_fits(T, Hq / Hk, span) ? 1 : 0;
}

int32_t btb_hip_attn_decode_qkv_rows(const void* qkv, const void* wq, const void* wk, float eps, int32_t centered,
                                     const void* cos_t, const void* sin_t, const int32_t* n0, const int32_t* depth,
                                     const int32_t* par, void* K, void* V, void* att, size_t T, size_t Hq, size_t Hk,
                                     size_t D, int64_t hs, int64_t rs, float scale, size_t cap, size_t S,
                                     float* workspace, void* stream) {
    if (qkv == nullptr || cos_t == nullptr || sin_t == nullptr || n0 == nullptr || K == nullptr || V == nullptr ||
        att == nullptr || workspace == nullptr)
        return ERR_NULL;
    if (T == 0 || Hq == 0 || Hk == 0 || S == 0 || cap == 0 || S > 1024 || Hq % Hk != 0 || hs <= 0 || rs <= 0 ||
        !(scale == scale) || !(eps >= 0.f))
        return ERR_DOMAIN;
    const size_t G = Hq / Hk;
    if (!al(qkv, 4) || !al(K, 16) || !al(V, 16) || !al(par, 4) || !al(depth, 4) || (rs % 8) != 0 || (hs % 8) != 0)
        return ERR_DOMAIN;
    if (par != nullptr && T > 32) {
        set_error("attn_decode_qkv_rows: a tree pass holds at most 32 rows");
        return ERR_DOMAIN;
    }
    if (S * G > (size_t)ATT_MAX_STATES) {
        set_error("attn_decode_qkv_rows: spans * (query heads per kv head) is at most 1024");
        return ERR_DOMAIN;
    }
    if (btb_hip_attn_rows_fused(T, Hq, Hk, D, cap, S) == 0) {
        set_error("attn_decode_qkv_rows: head_dim 128, spans of 128 keys, 2 or 4 query heads per kv head and 2 or more "
                  "rows with rows * (query heads per kv head) <= 64 (btb_hip_attn_rows_fused tells); otherwise "
                  "btb_hip_norm_rope_kv + btb_hip_attn_decode");
        return ERR_DOMAIN;
    }
    float* part_m = workspace;
    float* part_l = workspace + T * Hq * S;
    float* part_acc = workspace + 2 * T * Hq * S;
    const float scale_log2 = scale * 1.4426950408889634f;
    hipStream_t st = static_cast<hipStream_t>(stream);
    const int32_t rc = attn_decode_mfma_qkv(qkv, wq, wk, eps, centered ? 1 : 0, cos_t, sin_t, n0, depth, par, K, V, T, Hq,
                                            Hk, (long long)hs, (long long)rs, scale_log2, part_m, part_l, part_acc, S, cap,
                                            st);
    if (rc != OK) return rc;
    if (G == 4) launch_merge<4>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, nullptr);
    else launch_merge<2>(st, att, T, Hq, Hk, S, part_m, part_l, part_acc, nullptr);
    return hip_status(hipGetLastError(), "attn_decode_qkv_rows launch");
}

int32_t btb_hip_silu_mul(const void* gu, void* m, size_t T, size_t I, void* stream) {
    if (gu == nullptr || m == nullptr) return ERR_NULL;
    if (T == 0 || I == 0) return ERR_DOMAIN;
    size_t blocks = (T * I + 255) / 256;
    if (blocks > 4096) blocks = 4096;
    hipLaunchKernelGGL(silu_mul_kernel, dim3((unsigned)blocks), dim3(256), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(gu), static_cast<uint16_t*>(m), T, I);
    return hip_status(hipGetLastError(), "silu_mul launch");
}

int32_t btb_hip_argmax(const void* logits, int32_t* out, size_t T, size_t V, void* stream) {
    if (logits == nullptr || out == nullptr) return ERR_NULL;
    if (T == 0 || V == 0 || T > 0x7FFFFFFFull || V > 0x7FFFFFFEull) return ERR_DOMAIN;
    hipLaunchKernelGGL(argmax_kernel<false>, dim3((unsigned)T), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(logits), out, (int)V, nullptr, nullptr, nullptr, nullptr, nullptr);
    return hip_status(hipGetLastError(), "argmax launch");
}

int32_t btb_hip_argmax_publish(const void* logits, size_t V, int32_t* picked, int32_t* n0, int32_t* next_ids,
                               int32_t* out_tok, int32_t* out_n0, int64_t* out_ts, void* stream) {
    if (logits == nullptr || picked == nullptr || n0 == nullptr) return ERR_NULL;
    if (V == 0 || V > 0x7FFFFFFEull) return ERR_DOMAIN;
    hipLaunchKernelGGL(argmax_kernel<true>, dim3(1), dim3(1024), 0, static_cast<hipStream_t>(stream),
                       static_cast<const uint16_t*>(logits), picked, (int)V, n0, next_ids, out_tok, out_n0,
                       reinterpret_cast<long long*>(out_ts));
    return hip_status(hipGetLastError(), "argmax_publish launch");
}

int32_t btb_hip_publish(int32_t* n0, const int32_t* picked, int32_t* next_ids, int32_t* out_tok, int32_t* out_n0,
                        int64_t* out_ts, void* stream) {
    if (n0 == nullptr || picked == nullptr) return ERR_NULL;
    hipLaunchKernelGGL(publish_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), n0, picked, next_ids,
                       out_tok, out_n0, reinterpret_cast<long long*>(out_ts), 1);
    return hip_status(hipGetLastError(), "publish launch");
}

int32_t btb_hip_publish_only(const int32_t* n0, const int32_t* ids, int32_t* out_tok, int32_t* out_n0, int64_t* out_ts,
                             void* stream) {
    if (n0 == nullptr || ids == nullptr || out_tok == nullptr) return ERR_NULL;
    hipLaunchKernelGGL(publish_kernel, dim3(1), dim3(64), 0, static_cast<hipStream_t>(stream), const_cast<int32_t*>(n0),
                       ids, static_cast<int32_t*>(nullptr), out_tok, out_n0, reinterpret_cast<long long*>(out_ts), 0);
    return hip_status(hipGetLastError(), "publish launch");
}

}  // extern "C"
