/*
 * TEST INFRASTRUCTURE - the CPU oracle. Not part of the product: only the tests, the smoke check and the
 * benchmark's cpu_baseline leg may load this library; the HIP library never links or calls it.
 *
 * A restatement in plain C of the arithmetic of the reference's native CPU crate for the decode weight
 * matvec, behind the same C symbol names, argument orders and return codes. The reference is Rust (cargo and
 * rustc are absent from this image), so it is restated from its text rather than built:
 *
 *   return codes, null-before-domain order      native/src/lib.rs:17-33, gemv.rs:4007-4016
 *   bf16 widen (bits << 16)                     native/src/gemv.rs:40-43
 *   16 lane sums, lane j <- columns = j mod 16  native/src/gemv.rs:84-123
 *   pairwise fold of the 16 lanes               native/src/gemv.rs:45-58
 *   row chunks per thread                       native/src/gemv.rs:10-34
 *   pack12 widen and escape patch               native/src/gemv.rs:736-793, 4150-4214
 *   MXFP4 code table, scale, widen              native/src/gemv.rs:1032-1119, 4224-4263
 *   FP8 e4m3 value, bf16 rounding, block scale  native/src/gemv.rs:2996-3085, 4865-4924
 *   grouped calls                               native/src/gemv.rs:4096-4147, 4798-4860, 4927-4979
 *
 * The value of output (i, r) is fixed by this order alone (it depends on neither the thread count, the batch
 * width, the ISA tier nor the alignment):
 *
 *   acc[0..15] = 0
 *   for c = 0 .. cols-1:  acc[c mod 16] = fma(widen(W[r][c]), x[i][c], acc[c mod 16])
 *   y[i][r] = ((a0+a1)+(a2+a3) + (a4+a5)+(a6+a7)) + ((a8+a9)+(a10+a11) + (a12+a13)+(a14+a15))
 *
 * Three tiers compute it: scalar (the bit-defining one), AVX2+FMA and AVX-512, the vector tiers holding the
 * sixteen lane sums in vector registers. They agree bit for bit; tests/test_oracle.py checks that.
 *
 * Parity status of each function (what pins it is listed in tests/test_oracle.py and tests/test_codecs.py):
 *   bf16 widen, lane order, fold: pinned (hand cases of the reference's tests, f64 bound, brute force).
 *   pack12 widen + matvec:        pinned (the reference's committed pack12 fixtures; packed == bf16 bits).
 *   MXFP4 table/scale/widen:      pinned (the reference's constants; all 256 bytes x 256 scales vs ldexp).
 *   FP8 value/round/widen:        pinned (all 256 bytes vs torch.float8_e4m3fn; tie cases; fixtures).
 */
#define _GNU_SOURCE
#include <immintrin.h>
#include <math.h>
#include <stddef.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#ifdef _OPENMP
#include <omp.h>
#endif

#define OK 0
#define ERR_NULL (-1)
#define ERR_OVERFLOW (-5)
#define ERR_DOMAIN (-6)
#define ERR_PANIC (-7)

#define LANES 16
#define ROW_GROUP 4
#define COL_TILE 512
#define VEC_TILE 8
#define MAX_THREADS 1024
#define MX_BLOCK 32

#define EXPORT __attribute__((visibility("default")))

/* ------------------------------------------------------------------------------------------------ */
/* scalar pieces                                                                                      */

static inline float f32_from_bits(uint32_t b) {
    float f;
    memcpy(&f, &b, 4);
    return f;
}
static inline uint32_t f32_bits(float f) {
    uint32_t b;
    memcpy(&b, &f, 4);
    return b;
}

static inline float bf16_widen(uint16_t w) { return f32_from_bits((uint32_t)w << 16); }

/* nearest bf16, ties to even, kept as an f32 (gemv.rs:3003-3007) */
static inline float round_bf16(float f) {
    uint32_t b = f32_bits(f);
    return f32_from_bits((b + 0x7FFFu + ((b >> 16) & 1u)) & 0xFFFF0000u);
}

/* e4m3fn byte to f32 (gemv.rs:3009-3020): exponent 0 is m * 2^-9, 0x7F / 0xFF are NaN, no infinity */
static inline float f8_value(uint8_t b) {
    uint32_t a = b & 0x7Fu;
    float mag;
    if (a == 0x7Fu)
        mag = f32_from_bits(0x7FC00000u);
    else if (a < 8u)
        mag = (float)a * (1.0f / 512.0f);
    else
        mag = f32_from_bits((a << 20) + (120u << 23));
    return f32_from_bits(f32_bits(mag) | ((uint32_t)(b & 0x80u) << 24));
}

/* fp4 e2m1 code to f32 through the two byte halves of its bf16 pattern (gemv.rs:1038-1050) */
static const uint8_t FP4_HI[16] = {0x00, 0x3F, 0x3F, 0x3F, 0x40, 0x40, 0x40, 0x40,
                                   0x80, 0xBF, 0xBF, 0xBF, 0xC0, 0xC0, 0xC0, 0xC0};
static const uint8_t FP4_LO[16] = {0x00, 0x00, 0x80, 0xC0, 0x00, 0x40, 0x80, 0xC0,
                                   0x00, 0x00, 0x80, 0xC0, 0x00, 0x40, 0x80, 0xC0};
static inline float fp4_value(uint8_t code) {
    unsigned i = code & 0x0Fu;
    return f32_from_bits(((uint32_t)FP4_HI[i] << 24) | ((uint32_t)FP4_LO[i] << 16));
}

/* 2^(s-127) exactly; s == 0 is 2^-126 * 0.5 (gemv.rs:1054-1062) */
static inline float mx_scale(uint8_t s) {
    float f = f32_from_bits((uint32_t)(s == 0 ? 1 : s) << 23);
    return s == 0 ? f * 0.5f : f;
}

static inline float fold16(const float* a) {
    float t[8];
    for (int j = 0; j < 8; ++j) t[j] = a[2 * j] + a[2 * j + 1];
    float u0 = t[0] + t[1], u1 = t[2] + t[3], u2 = t[4] + t[5], u3 = t[6] + t[7];
    float v0 = u0 + u1, v1 = u2 + u3;
    return v0 + v1;
}

/* ------------------------------------------------------------------------------------------------ */
/* the stored forms: each widens `n` weights of one row, from column c0, to f32                      */

enum { FORM_BF16 = 0, FORM_P12 = 1, FORM_MX4 = 2, FORM_F8 = 3 };
enum { TIER_SCALAR = 0, TIER_AVX2 = 1, TIER_AVX512 = 2 };

typedef struct {
    int form;
    /* bf16 */
    const uint16_t* w;
    /* pack12 */
    const uint8_t* lo;
    const uint8_t* hi4;
    const uint8_t* table;
    const int32_t* esc_idx;
    const uint8_t* esc_val;
    size_t n_esc;
    /* mxfp4 */
    const uint8_t* blocks;
    const uint8_t* scales8;
    int ggml; /* 17-byte blocks, the scale first, low nibbles weights 0..15, high nibbles 16..31 (gemv.rs:1034-1078) */
    /* fp8 */
    const uint8_t* q;
    const float* scales;
    size_t sc, bm, bn;
} Stored;

typedef struct {
    Stored w;
    const float* x;
    float* y;
    size_t rows, cols, b;
} Job;

static void widen_bf16_scalar(const uint16_t* src, size_t n, float* dst) {
    for (size_t j = 0; j < n; ++j) dst[j] = bf16_widen(src[j]);
}

__attribute__((target("avx2"))) static void widen_bf16_avx2(const uint16_t* src, size_t n, float* dst) {
    size_t j = 0;
    for (; j + 8 <= n; j += 8) {
        __m128i v = _mm_loadu_si128((const __m128i*)(src + j));
        _mm256_storeu_ps(dst + j, _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(v), 16)));
    }
    for (; j < n; ++j) dst[j] = bf16_widen(src[j]);
}

__attribute__((target("avx512f,avx512bw"))) static void widen_bf16_avx512(const uint16_t* src, size_t n,
                                                                           float* dst) {
    size_t j = 0;
    for (; j + 16 <= n; j += 16) {
        __m256i v = _mm256_loadu_si256((const __m256i*)(src + j));
        _mm512_storeu_ps(dst + j, _mm512_castsi512_ps(_mm512_slli_epi32(_mm512_cvtepu16_epi32(v), 16)));
    }
    for (; j < n; ++j) dst[j] = bf16_widen(src[j]);
}

/* weight i of a packed tensor without its escape: table[code_i] high byte over lo[i] */
static inline float p12_plain(const Stored* s, size_t i) {
    uint8_t byte = s->hi4[i >> 1];
    unsigned code = (i & 1) ? (byte >> 4) : (byte & 0x0F);
    return f32_from_bits(((uint32_t)s->table[code] << 24) | ((uint32_t)s->lo[i] << 16));
}

static void widen_p12_scalar(const Stored* s, size_t start, size_t n, float* dst) {
    for (size_t j = 0; j < n; ++j) dst[j] = p12_plain(s, start + j);
}

/* 16 weights a step: the nibbles split, looked up in the table with a byte shuffle, zipped over the low
 * bytes and shifted into the top half of each f32. An odd start takes the scalar form. */
__attribute__((target("avx2"))) static void widen_p12_avx2(const Stored* s, size_t start, size_t n,
                                                            float* dst) {
    if (start & 1) {
        widen_p12_scalar(s, start, n, dst);
        return;
    }
    const __m128i tbl = _mm_loadu_si128((const __m128i*)s->table);
    const __m128i nib = _mm_set1_epi8(0x0F);
    size_t j = 0;
    for (; j + 16 <= n; j += 16) {
        size_t i = start + j;
        __m128i h = _mm_loadl_epi64((const __m128i*)(s->hi4 + (i >> 1)));           /* 8 bytes = 16 codes */
        __m128i even = _mm_and_si128(h, nib), odd = _mm_and_si128(_mm_srli_epi16(h, 4), nib);
        __m128i codes = _mm_unpacklo_epi8(even, odd);                                /* code order */
        __m128i hi = _mm_shuffle_epi8(tbl, codes);
        __m128i lo = _mm_loadu_si128((const __m128i*)(s->lo + i));
        __m128i w0 = _mm_unpacklo_epi8(lo, hi), w1 = _mm_unpackhi_epi8(lo, hi);     /* 16 x u16 */
        _mm256_storeu_ps(dst + j, _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(w0), 16)));
        _mm256_storeu_ps(dst + j + 8,
                         _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(w1), 16)));
    }
    if (j < n) widen_p12_scalar(s, start + j, n - j, dst + j);
}

/* escapes of [start, start + n) written over the widened tile; *cur is the row's cursor into the list */
static void p12_patch(const Stored* s, size_t start, size_t n, float* dst, size_t* cur) {
    size_t k = *cur, end = start + n;
    while (k < s->n_esc && (size_t)s->esc_idx[k] < start) ++k;
    for (; k < s->n_esc; ++k) {
        size_t i = (size_t)s->esc_idx[k];
        if (i >= end) break;
        dst[i - start] = f32_from_bits(((uint32_t)s->esc_val[k] << 24) | ((uint32_t)s->lo[i] << 16));
    }
    *cur = k;
}

/* first escape at or past `start` */
static size_t p12_cursor(const Stored* s, size_t start) {
    size_t a = 0, b = s->n_esc;
    while (a < b) {
        size_t m = a + (b - a) / 2;
        if ((size_t)s->esc_idx[m] < start)
            a = m + 1;
        else
            b = m;
    }
    return a;
}

static void widen_mx4(const Stored* s, size_t start, size_t n, float* dst) {
    for (size_t blk = 0; blk < n / MX_BLOCK; ++blk) {
        size_t g = start / MX_BLOCK + blk;
        if (s->ggml) { /* gemv.rs:1147-1151: the same values in the same places, read from the other layout */
            const uint8_t* raw = s->blocks + g * 17;
            float sc = mx_scale(raw[0]);
            float* o = dst + blk * MX_BLOCK;
            for (int j = 0; j < 16; ++j) {
                o[j] = fp4_value(raw[1 + j] & 0x0F) * sc;
                o[16 + j] = fp4_value(raw[1 + j] >> 4) * sc;
            }
            continue;
        }
        const uint8_t* bytes = s->blocks + g * 16;
        float sc = mx_scale(s->scales8[g]);
        float* o = dst + blk * MX_BLOCK;
        for (int j = 0; j < 16; ++j) {
            o[2 * j] = fp4_value(bytes[j] & 0x0F) * sc;
            o[2 * j + 1] = fp4_value(bytes[j] >> 4) * sc;
        }
    }
}

static void widen_f8(const Stored* s, size_t row, size_t row_len, size_t c0, size_t n, float* dst) {
    const float* srow = s->scales + (row / s->bm) * s->sc;
    const uint8_t* src = s->q + row * row_len;
    size_t c = c0;
    while (c < c0 + n) {
        size_t end = (c / s->bn + 1) * s->bn;
        if (end > c0 + n) end = c0 + n;
        float sc = srow[c / s->bn];
        for (size_t j = c; j < end; ++j) dst[j - c0] = round_bf16(f8_value(src[j]) * sc);
        c = end;
    }
}

/* ------------------------------------------------------------------------------------------------ */
/* accumulation: `n` columns of a widened tile times x into a row's 16 lane sums                     */

static void accum_scalar(float* acc, const float* w, const float* x, size_t n) {
    for (size_t c = 0; c < n; ++c) acc[c % LANES] = fmaf(w[c], x[c], acc[c % LANES]);
}

__attribute__((target("avx2,fma"))) static void accum_avx2(float* acc, const float* w, const float* x,
                                                            size_t n) {
    __m256 a0 = _mm256_loadu_ps(acc), a1 = _mm256_loadu_ps(acc + 8);
    size_t c = 0;
    for (; c + LANES <= n; c += LANES) {
        a0 = _mm256_fmadd_ps(_mm256_loadu_ps(w + c), _mm256_loadu_ps(x + c), a0);
        a1 = _mm256_fmadd_ps(_mm256_loadu_ps(w + c + 8), _mm256_loadu_ps(x + c + 8), a1);
    }
    _mm256_storeu_ps(acc, a0);
    _mm256_storeu_ps(acc + 8, a1);
    for (size_t j = 0; c + j < n; ++j) acc[j] = fmaf(w[c + j], x[c + j], acc[j]);
}

__attribute__((target("avx512f,fma"))) static void accum_avx512(float* acc, const float* w,
                                                                 const float* x, size_t n) {
    __m512 a = _mm512_loadu_ps(acc);
    size_t c = 0;
    for (; c + LANES <= n; c += LANES) a = _mm512_fmadd_ps(_mm512_loadu_ps(w + c), _mm512_loadu_ps(x + c), a);
    _mm512_storeu_ps(acc, a);
    for (size_t j = 0; c + j < n; ++j) acc[j] = fmaf(w[c + j], x[c + j], acc[j]);
}

/* one vector straight from bf16 rows, four rows a pass, no widened tile between (the b == 1 decode case) */
__attribute__((target("avx512f,avx512bw,fma"))) static void rows4_bf16_avx512(const uint16_t* w, size_t cols,
                                                                               const float* x, float* y4) {
    __m512 a0 = _mm512_setzero_ps(), a1 = a0, a2 = a0, a3 = a0;
    size_t c = 0;
    for (; c + LANES <= cols; c += LANES) {
        __m512 xv = _mm512_loadu_ps(x + c);
#define W16(r) \
    _mm512_castsi512_ps(_mm512_slli_epi32(_mm512_cvtepu16_epi32(_mm256_loadu_si256((const __m256i*)(w + (r) * cols + c))), 16))
        a0 = _mm512_fmadd_ps(W16(0), xv, a0);
        a1 = _mm512_fmadd_ps(W16(1), xv, a1);
        a2 = _mm512_fmadd_ps(W16(2), xv, a2);
        a3 = _mm512_fmadd_ps(W16(3), xv, a3);
#undef W16
    }
    float acc[4][LANES];
    _mm512_storeu_ps(acc[0], a0);
    _mm512_storeu_ps(acc[1], a1);
    _mm512_storeu_ps(acc[2], a2);
    _mm512_storeu_ps(acc[3], a3);
    for (int r = 0; r < 4; ++r) {
        for (size_t j = 0; c + j < cols; ++j)
            acc[r][j] = fmaf(bf16_widen(w[r * cols + c + j]), x[c + j], acc[r][j]);
        y4[r] = fold16(acc[r]);
    }
}

__attribute__((target("avx2,fma"))) static void rows4_bf16_avx2(const uint16_t* w, size_t cols, const float* x,
                                                                 float* y4) {
    __m256 a[4][2];
    for (int r = 0; r < 4; ++r) a[r][0] = a[r][1] = _mm256_setzero_ps();
    size_t c = 0;
    for (; c + LANES <= cols; c += LANES) {
        __m256 x0 = _mm256_loadu_ps(x + c), x1 = _mm256_loadu_ps(x + c + 8);
        for (int r = 0; r < 4; ++r) {
            __m256i v = _mm256_loadu_si256((const __m256i*)(w + r * cols + c));
            __m256 w0 = _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(_mm256_castsi256_si128(v)), 16));
            __m256 w1 = _mm256_castsi256_ps(_mm256_slli_epi32(_mm256_cvtepu16_epi32(_mm256_extracti128_si256(v, 1)), 16));
            a[r][0] = _mm256_fmadd_ps(w0, x0, a[r][0]);
            a[r][1] = _mm256_fmadd_ps(w1, x1, a[r][1]);
        }
    }
    for (int r = 0; r < 4; ++r) {
        float acc[LANES];
        _mm256_storeu_ps(acc, a[r][0]);
        _mm256_storeu_ps(acc + 8, a[r][1]);
        for (size_t j = 0; c + j < cols; ++j) acc[j] = fmaf(bf16_widen(w[r * cols + c + j]), x[c + j], acc[j]);
        y4[r] = fold16(acc);
    }
}

/* ------------------------------------------------------------------------------------------------ */
/* tier selection                                                                                     */

static int g_tier = -1;

static int detect_tier(void) {
    const char* env = getenv("BTB_NATIVE_ISA");
    int best = TIER_SCALAR;
    __builtin_cpu_init();
    if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) best = TIER_AVX2;
    if (best == TIER_AVX2 && __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw"))
        best = TIER_AVX512;
    if (env != NULL) {
        int want = best;
        if (!strcasecmp(env, "scalar")) want = TIER_SCALAR;
        else if (!strcasecmp(env, "avx2")) want = TIER_AVX2;
        else if (!strcasecmp(env, "avx512")) want = TIER_AVX512;
        if (want <= best) best = want; /* a tier the machine lacks is never picked */
    }
    return best;
}

static int tier(void) {
    if (g_tier < 0) g_tier = detect_tier();
    return g_tier;
}

EXPORT const char* btb_isa(void) {
    static const char* names[] = {"scalar", "avx2", "avx512"};
    return names[tier()];
}

/* test hook: force a tier (clamped to what the machine has); returns the tier now in force */
EXPORT int btb_oracle_set_tier(int t) {
    int best = detect_tier();
    if (getenv("BTB_NATIVE_ISA") != NULL) { /* detect_tier honoured the env; find the machine's own best */
        best = TIER_SCALAR;
        if (__builtin_cpu_supports("avx2") && __builtin_cpu_supports("fma")) best = TIER_AVX2;
        if (best == TIER_AVX2 && __builtin_cpu_supports("avx512f") && __builtin_cpu_supports("avx512bw"))
            best = TIER_AVX512;
    }
    if (t < 0) t = best;
    g_tier = t > best ? best : t;
    return g_tier;
}

/* ------------------------------------------------------------------------------------------------ */
/* a job's rows r0..r1                                                                                */

static void widen_tile(const Stored* s, int t, size_t row, size_t cols, size_t c0, size_t n, float* dst,
                       size_t* cur) {
    switch (s->form) {
        case FORM_BF16: {
            const uint16_t* src = s->w + row * cols + c0;
            if (t == TIER_AVX512) widen_bf16_avx512(src, n, dst);
            else if (t == TIER_AVX2) widen_bf16_avx2(src, n, dst);
            else widen_bf16_scalar(src, n, dst);
            break;
        }
        case FORM_P12: {
            size_t start = row * cols + c0;
            if (t != TIER_SCALAR) widen_p12_avx2(s, start, n, dst);
            else widen_p12_scalar(s, start, n, dst);
            if (s->n_esc) p12_patch(s, start, n, dst, cur);
            break;
        }
        case FORM_MX4:
            widen_mx4(s, row * cols + c0, n, dst);
            break;
        default:
            widen_f8(s, row, cols, c0, n, dst);
            break;
    }
}

static void run_rows(const Job* job, size_t r0, size_t r1) {
    const int t = tier();
    const size_t cols = job->cols, rows = job->rows, b = job->b;
    const Stored* s = &job->w;
    size_t r = r0;
    /* the decode case: one vector over bf16 rows, accumulated straight from the rows */
    if (s->form == FORM_BF16 && b == 1 && t != TIER_SCALAR) {
        for (; r + 4 <= r1; r += 4) {
            if (t == TIER_AVX512) rows4_bf16_avx512(s->w + r * cols, cols, job->x, job->y + r);
            else rows4_bf16_avx2(s->w + r * cols, cols, job->x, job->y + r);
        }
    }
    float tile[COL_TILE];
    float acc[VEC_TILE][LANES];
    for (; r < r1; ++r) {
        for (size_t i0 = 0; i0 < b; i0 += VEC_TILE) {
            size_t bt = b - i0 < VEC_TILE ? b - i0 : VEC_TILE;
            memset(acc, 0, sizeof(acc));
            size_t cur = (s->form == FORM_P12 && s->n_esc) ? p12_cursor(s, r * cols) : 0;
            for (size_t c0 = 0; c0 < cols; c0 += COL_TILE) {
                size_t n = cols - c0 < COL_TILE ? cols - c0 : COL_TILE;
                widen_tile(s, t, r, cols, c0, n, tile, &cur);
                for (size_t i = 0; i < bt; ++i) {
                    const float* xv = job->x + (i0 + i) * cols + c0;
                    if (t == TIER_AVX512) accum_avx512(acc[i], tile, xv, n);
                    else if (t == TIER_AVX2) accum_avx2(acc[i], tile, xv, n);
                    else accum_scalar(acc[i], tile, xv, n);
                }
            }
            for (size_t i = 0; i < bt; ++i) job->y[(i0 + i) * rows + r] = fold16(acc[i]);
        }
    }
}

/* rows a chunk: ceil(rows / (threads * 4)), at least four (gemv.rs:29-34) */
static size_t chunk_rows(size_t rows, size_t nt) {
    size_t c = (rows + nt * 4 - 1) / (nt * 4);
    return c < ROW_GROUP ? ROW_GROUP : c;
}

static int resolve_threads(size_t threads, size_t* out) {
    if (threads > MAX_THREADS) return 0;
    if (threads == 0) {
#ifdef _OPENMP
        threads = (size_t)omp_get_num_procs();
#else
        threads = 1;
#endif
    }
    *out = threads ? threads : 1;
    return 1;
}

static int run_jobs(const Job* jobs, size_t n, size_t total_rows, size_t threads) {
    size_t nt;
    if (!resolve_threads(threads, &nt)) return ERR_DOMAIN;
    size_t chunk = chunk_rows(total_rows, nt);
    /* every job's rows cut into chunks, all chunks spread over the threads together */
    size_t nchunks = 0;
    for (size_t t = 0; t < n; ++t) nchunks += (jobs[t].rows + chunk - 1) / chunk;
    typedef struct {
        size_t job, r0, r1;
    } Piece;
    Piece* pieces = (Piece*)malloc(nchunks * sizeof(Piece));
    if (pieces == NULL) return ERR_PANIC;
    size_t k = 0;
    for (size_t t = 0; t < n; ++t)
        for (size_t r0 = 0; r0 < jobs[t].rows; r0 += chunk) {
            pieces[k].job = t;
            pieces[k].r0 = r0;
            pieces[k].r1 = r0 + chunk < jobs[t].rows ? r0 + chunk : jobs[t].rows;
            ++k;
        }
    tier(); /* resolved before the threads start */
#ifdef _OPENMP
#pragma omp parallel for schedule(dynamic, 1) num_threads((int)nt) if (nt > 1 && nchunks > 1)
#endif
    for (size_t p = 0; p < nchunks; ++p) run_rows(&jobs[pieces[p].job], pieces[p].r0, pieces[p].r1);
    free(pieces);
    return OK;
}

/* ------------------------------------------------------------------------------------------------ */
/* boundary checks                                                                                    */

#define MAX_ELEMS ((size_t)(INTPTR_MAX) / 4)

static int mul_fits(size_t a, size_t b) {
    size_t n;
    return !__builtin_mul_overflow(a, b, &n) && n <= MAX_ELEMS;
}
static int shape_ok(size_t rows, size_t cols, size_t b) {
    return mul_fits(rows, cols) && mul_fits(b, cols) && mul_fits(b, rows);
}
static int aligned_to(const void* p, size_t a) { return ((uintptr_t)p % a) == 0; }

static int check_bf16(const uint16_t* w, size_t rows, size_t cols, const float* x, size_t b, float* y, Job* job) {
    if (w == NULL || x == NULL || y == NULL) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0) return ERR_DOMAIN;
    if (!shape_ok(rows, cols, b) || !aligned_to(w, 2) || !aligned_to(x, 4) || !aligned_to(y, 4)) return ERR_DOMAIN;
    memset(job, 0, sizeof(*job));
    job->w.form = FORM_BF16;
    job->w.w = w;
    job->x = x;
    job->y = y;
    job->rows = rows;
    job->cols = cols;
    job->b = b;
    return OK;
}

static int check_mx4(const uint8_t* blocks, const uint8_t* scales, size_t rows, size_t cols, const float* x,
                     size_t b, float* y, Job* job) {
    if (blocks == NULL || scales == NULL || x == NULL || y == NULL) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0 || cols % MX_BLOCK != 0 || !shape_ok(rows, cols, b) ||
        !aligned_to(x, 4) || !aligned_to(y, 4))
        return ERR_DOMAIN;
    memset(job, 0, sizeof(*job));
    job->w.form = FORM_MX4;
    job->w.blocks = blocks;
    job->w.scales8 = scales;
    job->x = x;
    job->y = y;
    job->rows = rows;
    job->cols = cols;
    job->b = b;
    return OK;
}

static int check_f8(const uint8_t* w, const float* scales, size_t rows, size_t cols, size_t sr, size_t sc,
                    const float* x, size_t b, float* y, Job* job) {
    if (w == NULL || scales == NULL || x == NULL || y == NULL) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0 || sr == 0 || sc == 0) return ERR_DOMAIN;
    if (rows % sr != 0 || cols % sc != 0 || !shape_ok(rows, cols, b) || !aligned_to(scales, 4) ||
        !aligned_to(x, 4) || !aligned_to(y, 4))
        return ERR_DOMAIN;
    memset(job, 0, sizeof(*job));
    job->w.form = FORM_F8;
    job->w.q = w;
    job->w.scales = scales;
    job->w.sc = sc;
    job->w.bm = rows / sr;
    job->w.bn = cols / sc;
    job->x = x;
    job->y = y;
    job->rows = rows;
    job->cols = cols;
    job->b = b;
    return OK;
}

/* ------------------------------------------------------------------------------------------------ */
/* the C ABI of the reference's native crate (native/src/lib.rs), same names and argument orders      */

EXPORT int32_t btb_gemv_bf16_rows(const uint16_t* w, size_t rows, size_t cols, const float* x, size_t b, float* y,
                                  size_t threads) {
    Job job;
    int rc = check_bf16(w, rows, cols, x, b, y, &job);
    if (rc != OK) return rc;
    return run_jobs(&job, 1, rows, threads);
}

EXPORT int32_t btb_gemv_bf16_group(size_t n, const uint16_t* const* w, const size_t* rows, const size_t* cols,
                                   const float* const* x, const size_t* b, float* const* y, size_t threads) {
    if (w == NULL || rows == NULL || cols == NULL || x == NULL || b == NULL || y == NULL) return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    Job* jobs = (Job*)malloc(n * sizeof(Job));
    if (jobs == NULL) return ERR_PANIC;
    size_t total = 0;
    int rc = OK;
    for (size_t t = 0; t < n && rc == OK; ++t) {
        rc = check_bf16(w[t], rows[t], cols[t], x[t], b[t], y[t], &jobs[t]);
        if (rc == OK && __builtin_add_overflow(total, rows[t], &total)) rc = ERR_DOMAIN;
    }
    if (rc == OK) rc = run_jobs(jobs, n, total, threads);
    free(jobs);
    return rc;
}

EXPORT int32_t btb_gemv_p12_rows(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const int32_t* esc_idx,
                                 const uint8_t* esc_val, size_t n_esc, size_t rows, size_t cols, const float* x,
                                 size_t b, float* y, size_t threads) {
    if (lo == NULL || hi4 == NULL || table == NULL || x == NULL || y == NULL) return ERR_NULL;
    if (n_esc > 0 && (esc_idx == NULL || esc_val == NULL)) return ERR_NULL;
    if (rows == 0 || cols == 0 || b == 0) return ERR_DOMAIN;
    if (!shape_ok(rows, cols, b) || !aligned_to(x, 4) || !aligned_to(y, 4)) return ERR_DOMAIN;
    size_t n = rows * cols;
    if (n_esc > 0) {
        if (n_esc > n || !aligned_to(esc_idx, 4)) return ERR_DOMAIN;
        int64_t prev = -1;
        for (size_t k = 0; k < n_esc; ++k) {
            int64_t v = esc_idx[k];
            if (v <= prev || v >= (int64_t)n) return ERR_DOMAIN;
            prev = v;
        }
    }
    Job job;
    memset(&job, 0, sizeof(job));
    job.w.form = FORM_P12;
    job.w.lo = lo;
    job.w.hi4 = hi4;
    job.w.table = table;
    job.w.esc_idx = esc_idx;
    job.w.esc_val = esc_val;
    job.w.n_esc = n_esc;
    job.x = x;
    job.y = y;
    job.rows = rows;
    job.cols = cols;
    job.b = b;
    return run_jobs(&job, 1, rows, threads);
}

EXPORT int32_t btb_gemv_mxfp4_rows(const uint8_t* blocks, const uint8_t* scales, size_t rows, size_t cols,
                                   const float* x, size_t b, float* y, size_t threads) {
    Job job;
    int rc = check_mx4(blocks, scales, rows, cols, x, b, y, &job);
    if (rc != OK) return rc;
    return run_jobs(&job, 1, rows, threads);
}

/* btb_gemv_mxfp4_ggml_rows (native/src/lib.rs:162-183): the same matvec over ggml's 17-byte blocks */
EXPORT int32_t btb_gemv_mxfp4_ggml_rows(const uint8_t* raw, size_t rows, size_t cols, const float* x, size_t b, float* y,
                                        size_t threads) {
    Job job;
    int rc = check_mx4(raw, raw, rows, cols, x, b, y, &job);
    if (rc != OK) return rc;
    job.w.scales8 = NULL;
    job.w.ggml = 1;
    return run_jobs(&job, 1, rows, threads);
}

EXPORT int32_t btb_gemv_mxfp4_group(size_t n, const uint8_t* const* blocks, const uint8_t* const* scales,
                                    const size_t* rows, const size_t* cols, const float* const* x, const size_t* b,
                                    float* const* y, size_t threads) {
    if (blocks == NULL || scales == NULL || rows == NULL || cols == NULL || x == NULL || b == NULL || y == NULL)
        return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    Job* jobs = (Job*)malloc(n * sizeof(Job));
    if (jobs == NULL) return ERR_PANIC;
    size_t total = 0;
    int rc = OK;
    for (size_t t = 0; t < n && rc == OK; ++t) {
        rc = check_mx4(blocks[t], scales[t], rows[t], cols[t], x[t], b[t], y[t], &jobs[t]);
        if (rc == OK && __builtin_add_overflow(total, rows[t], &total)) rc = ERR_DOMAIN;
    }
    if (rc == OK) rc = run_jobs(jobs, n, total, threads);
    free(jobs);
    return rc;
}

EXPORT int32_t btb_gemv_fp8_rows(const uint8_t* w, const float* scales, size_t rows, size_t cols, size_t sr, size_t sc,
                                 const float* x, size_t b, float* y, size_t threads) {
    Job job;
    int rc = check_f8(w, scales, rows, cols, sr, sc, x, b, y, &job);
    if (rc != OK) return rc;
    return run_jobs(&job, 1, rows, threads);
}

EXPORT int32_t btb_gemv_fp8_group(size_t n, const uint8_t* const* w, const float* const* scales, const size_t* rows,
                                  const size_t* cols, const size_t* sr, const size_t* sc, const float* const* x,
                                  const size_t* b, float* const* y, size_t threads) {
    if (w == NULL || scales == NULL || rows == NULL || cols == NULL || sr == NULL || sc == NULL || x == NULL ||
        b == NULL || y == NULL)
        return ERR_NULL;
    if (n == 0) return ERR_DOMAIN;
    Job* jobs = (Job*)malloc(n * sizeof(Job));
    if (jobs == NULL) return ERR_PANIC;
    size_t total = 0;
    int rc = OK;
    for (size_t t = 0; t < n && rc == OK; ++t) {
        rc = check_f8(w[t], scales[t], rows[t], cols[t], sr[t], sc[t], x[t], b[t], y[t], &jobs[t]);
        if (rc == OK && __builtin_add_overflow(total, rows[t], &total)) rc = ERR_DOMAIN;
    }
    if (rc == OK) rc = run_jobs(jobs, n, total, threads);
    free(jobs);
    return rc;
}

/* ------------------------------------------------------------------------------------------------ */
/* the widenings on their own, for the bit-exact checks of the device widen kernels                   */

/* a packed tensor of n weights back to its bf16 bit patterns */
EXPORT int32_t btb_oracle_unpack_p12(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table,
                                     const int32_t* esc_idx, const uint8_t* esc_val, size_t n_esc, size_t n,
                                     uint16_t* out) {
    if (lo == NULL || hi4 == NULL || table == NULL || out == NULL) return ERR_NULL;
    if (n_esc > 0 && (esc_idx == NULL || esc_val == NULL)) return ERR_NULL;
    Stored s;
    memset(&s, 0, sizeof(s));
    s.form = FORM_P12;
    s.lo = lo;
    s.hi4 = hi4;
    s.table = table;
    s.esc_idx = esc_idx;
    s.esc_val = esc_val;
    s.n_esc = n_esc;
    float tile[COL_TILE];
    size_t cur = 0;
    for (size_t c0 = 0; c0 < n; c0 += COL_TILE) {
        size_t m = n - c0 < COL_TILE ? n - c0 : COL_TILE;
        widen_p12_scalar(&s, c0, m, tile);
        if (n_esc) p12_patch(&s, c0, m, tile, &cur);
        for (size_t j = 0; j < m; ++j) out[c0 + j] = (uint16_t)(f32_bits(tile[j]) >> 16);
    }
    return OK;
}

/* nblocks MXFP4 blocks (16 bytes + 1 scale each) to 32 f32 each: fp4 * 2^(s-127), one f32 multiply */
EXPORT int32_t btb_oracle_widen_mxfp4(const uint8_t* blocks, const uint8_t* scales, size_t nblocks, float* out) {
    if (blocks == NULL || scales == NULL || out == NULL) return ERR_NULL;
    Stored s;
    memset(&s, 0, sizeof(s));
    s.blocks = blocks;
    s.scales8 = scales;
    widen_mx4(&s, 0, nblocks * MX_BLOCK, out);
    return OK;
}

/* an FP8 matrix to the f32 holding bf16(e4m3 * scale) for every weight */
EXPORT int32_t btb_oracle_widen_fp8(const uint8_t* w, const float* scales, size_t rows, size_t cols, size_t sr,
                                    size_t sc, float* out) {
    if (w == NULL || scales == NULL || out == NULL) return ERR_NULL;
    if (rows == 0 || cols == 0 || sr == 0 || sc == 0 || rows % sr != 0 || cols % sc != 0) return ERR_DOMAIN;
    Stored s;
    memset(&s, 0, sizeof(s));
    s.q = w;
    s.scales = scales;
    s.sc = sc;
    s.bm = rows / sr;
    s.bn = cols / sc;
    for (size_t r = 0; r < rows; ++r) widen_f8(&s, r, cols, 0, cols, out + r * cols);
    return OK;
}

EXPORT float btb_oracle_round_bf16(float f) { return round_bf16(f); }
EXPORT float btb_oracle_f8_value(uint8_t b) { return f8_value(b); }
EXPORT float btb_oracle_fp4_value(uint8_t c) { return fp4_value(c); }
EXPORT float btb_oracle_mx_scale(uint8_t s) { return mx_scale(s); }
EXPORT float btb_oracle_fold16(const float* a) { return fold16(a); }
