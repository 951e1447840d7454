/*
 * libbtb_hip: the decode weight-matvec path of btb for one AMD MI355X (gfx950), as a C ABI.
 *
 * Conventions, kept from the reference's native crate (native/src/lib.rs:1-9, 17-33):
 *   - every function returns 0 on success or a negative code; buffers are caller-owned and written in place; a
 *     refused call writes nothing and launches nothing;
 *   - BTB_ERR_NULL is checked before BTB_ERR_DOMAIN;
 *   - all sizes are size_t, all pointers are plain device pointers (hipMalloc'd or torch-owned), `stream` is a
 *     hipStream_t passed as void* (NULL is the default stream). Work is queued on that stream and the call
 *     returns without waiting, so every entry point may be recorded into a hipGraph capture;
 *   - re-entrant; the result for an output row depends on neither the number of x rows in the call nor on the
 *     launch geometry.
 *
 * Two faces are exported, as in the reference: the device twins of the crate's CPU entry points (f32 x and y, the
 * host's summation order, bit for bit: btb_hip_gemv_*_rows) and the card operators the CUDA backend launches by
 * kernel name (bf16 x and y: btb_hip_gemv_bf16 and friends).
 */
#ifndef BTB_HIP_H
#define BTB_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define BTB_OK 0
#define BTB_ERR_NULL (-1)
#define BTB_ERR_OVERFLOW (-5)
#define BTB_ERR_DOMAIN (-6)
#define BTB_ERR_PANIC (-7) /* a HIP runtime failure at the boundary; btb_hip_last_error() names it */

/* ---- process ------------------------------------------------------------------------------------------- */

/* Binds the calling process to `device` (hipSetDevice) and reads its compute-unit count and LDS size. Optional:
 * the first operator call does the same for the current device. Replaces the module load of the reference's
 * `_Cuda.__init__` (btb/engine/native.py:1263-1300). */
int32_t btb_hip_init(int32_t device);

/* The GPU architecture the kernels were compiled for ("gfx950"): the tier a benchmark's numbers belong to.
 * Replaces btb_isa (native/src/lib.rs:43-50). Static NUL-terminated string. */
const char* btb_hip_arch(void);

/* Compute units of the bound device: `_Cuda.sms` (btb/engine/native.py:1297). */
int32_t btb_hip_sms(void);

/* The message of the last BTB_ERR_PANIC / refused call on this thread (static storage, never NULL). */
const char* btb_hip_last_error(void);

/* Overrides a launch-tuning knob (e.g. "gemv_wgs_per_cu"); value < 0 restores the default. Unknown keys are
 * BTB_ERR_DOMAIN. For measurement only: no knob changes a result bit within a kernel family ("gemv_no_mfma" and
 * "gemv_mfma_from" choose between the vector and the matrix-core family, whose sums round in another order).
 * No counterpart in the reference. */
int32_t btb_hip_set_tuning(const char* key, int32_t value);

/* A measurement aid: the streaming matvec's loads without the matvec. Reads a [rows, 2560] bf16-shaped matrix (rows
 * even, 5120 bytes a row, 16-byte aligned) the way btb_hip_gemv_bf16_norm's gate/up form does - a wave a pair of rows
 * half the matrix apart, ten 16-byte non-temporal loads a lane in flight, the streaming kernel's grid - folds what
 * arrives with a few integer instructions and writes nothing (`sink`, a device word or NULL, is never written in
 * practice). bytes / time of this launch is what the memory system gives a kernel of the matvec's load structure at
 * this size: the practical ceiling beside the data sheet's 8 TB/s (`bench.py --workload ceiling`). No counterpart in
 * the reference. */
int32_t btb_hip_stream_probe(const void* a, size_t rows, uint32_t* sink, void* stream);

/* ---- card operators: bf16 activations in, f32 accumulate, bf16 out ------------------------------------- */

/* y[m][r] = bf16(sum_c w[r][c] * x[m][c]).  w [R, C] bf16 row-major, x [M, C] bf16, y [M, R] bf16; C a multiple
 * of 8, w and x 16-byte aligned. Replaces the kernels btb_gemv_bf16_m{1,2,4,8,16,32}
 * (native/cuda/btb_kernels.cu:84-155) and btb_gemv_mma_bf16 (native/cuda/btb_gemv_mma.cuh:196-200); M is an
 * argument, any value from 1 to 1024. */
int32_t btb_hip_gemv_bf16(const void* w, const void* x, void* y, size_t R, size_t C, size_t M, void* stream);

/* The down projection with the SwiGLU fold in its x load: gu [M, 2C] bf16 (gate then up),
 * x[m][c] = bf16(bf16(silu(g)) * u). Replaces btb_gemv_silu_bf16_m{M} (native/cuda/btb_kernels.cu:168-227). */
int32_t btb_hip_gemv_silu_bf16(const void* w, const void* gu, void* y, size_t R, size_t C, size_t M, void* stream);

/* Gate, up and the activation in one kernel: w [2I, C] bf16 (gate rows, then up rows), x [M, C], m [M, I] =
 * bf16(bf16(silu(g)) * u) with g = bf16(w[i] . x), u = bf16(w[I + i] . x): the bits of btb_hip_gemv_bf16 followed by
 * btb_hip_silu_mul. Replaces btb_gemv_mma_glu_silu (native/cuda/btb_gemv_mma.cuh:216-315). */
int32_t btb_hip_gemv_glu_silu_bf16(const void* w, const void* x, void* m, size_t I, size_t C, size_t M, void* stream);

/* The matvec with the residual add and the RMSNorm folded into its x load: h' = bf16(h_in + y) (y NULL: h' = h_in),
 * x = bf16(h' * rsqrt(mean(h'^2) + eps) * norm_w) (or * (1 + norm_w) when centered), out = W x; h' is written to
 * h_out (NULL: not kept; never h_in itself). With glu != 0, W is [R = 2I, C] and out is the gate/up fold m [M, I] of
 * btb_hip_gemv_glu_silu_bf16. The bits are those of btb_hip_add_rmsnorm followed by the matvec; it replaces that
 * pair of launches of the reference's step (btb/engine/cuda.py:1730-1733, 1770-1793). */
int32_t btb_hip_gemv_bf16_norm(const void* w, const void* h_in, const void* y, const void* norm_w, float eps,
                               int32_t centered, void* h_out, void* out, size_t R, size_t C, size_t M, int32_t glu,
                               void* stream);

/* btb_hip_gemv_bf16_norm for the step's first layer, whose residual is the tokens' embedding rows: h' [m] =
 * table[ids[m]] (table [vocab, C] bf16, ids i32 [M] on the device, an id outside the table clamped into it), no y;
 * h' goes to h_out, out = W rmsnorm(h'). The bits of btb_hip_embed followed by btb_hip_gemv_bf16_norm, in one launch
 * (the reference gathers the row with torch before its graph: btb/engine/cuda.py:1722-1729). */
int32_t btb_hip_gemv_bf16_embed_norm(const void* w, const void* table, const int32_t* ids, size_t vocab,
                                     const void* norm_w, float eps, int32_t centered, void* h_out, void* out, size_t R,
                                     size_t C, size_t M, void* stream);

/* ---- the stored weight forms, widened in registers inside the matvec ------------------------------------ */

/* The matvec over a pack12 matrix (n = R * C weights): lo u8[n], hi4 u8[(n + 1) / 2] (weight 2k in the low nibble
 * of byte k), table u8[16], esc_idx i32[n_esc] strictly ascending, esc_val u8[n_esc] - the arrays of
 * btb_gemv_p12_rows (native/src/lib.rs:114-135), on the device, the list validated at upload by btb_hip_p12_check -
 * plus three arrays made once at upload: row_ptr i32[R + 1] from btb_hip_p12_row_ptr, pairs u16[256] from
 * btb_hip_p12_pairs (NULL: the table is looked up in registers instead, a slower kernel with the same bits) and
 * row_esc u32[S R] from btb_hip_p12_row_esc (S = 8 words a row up to 4096 columns, 16 beyond; NULL: every escape is
 * fetched through the list at the end of its row's tile, slower with the same bits; with it C <= 32767).
 * x [M, C] bf16, y [M, R] bf16; C a multiple of 16, lo 16-byte and hi4 8-byte aligned. The reference has no card
 * kernel for this form (it widens a packed layer to bf16 before the card holds it: btb/engine/tiers.py:1200-1216). */
int32_t btb_hip_gemv_p12(const void* lo, const void* hi4, const void* table, const void* pairs, const void* esc_idx,
                         const void* esc_val, size_t n_esc, const void* row_ptr, const void* row_esc, const void* x,
                         void* y, size_t R, size_t C, size_t M, void* stream);

/* btb_hip_gemv_bf16_norm over a pack12 matrix (the arrays of btb_hip_gemv_p12). */
int32_t btb_hip_gemv_p12_norm(const void* lo, const void* hi4, const void* table, const void* pairs,
                              const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                              const void* row_esc, const void* h_in, const void* y, const void* norm_w, float eps,
                              int32_t centered, void* h_out, void* out, size_t R, size_t C, size_t M, int32_t glu,
                              void* stream);

/* btb_hip_gemv_bf16_embed_norm over a pack12 matrix (`table` is the matrix's 16 high bytes, `embed` the embedding). */
int32_t btb_hip_gemv_p12_embed_norm(const void* lo, const void* hi4, const void* table, const void* pairs,
                                    const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                                    const void* row_esc, const void* embed, const int32_t* ids, size_t vocab,
                                    const void* norm_w, float eps, int32_t centered, void* h_out, void* out, size_t R,
                                    size_t C, size_t M, void* stream);

/* pairs[b] = table[b & 15] | table[b >> 4] << 8 for every byte b of codes, the escape code's slot 15 taken as 0: the
 * high bytes of the two weights a byte of codes stands for, so that the matvec turns a byte of codes into two high
 * bytes with one 2-byte read of its copy of these 512 bytes in LDS. Made once at upload, beside row_ptr; an escaped
 * weight then streams as (0, low byte) and the escape list puts its true value in (the matrix should carry 0 in
 * table[15], as the packer writes it: the kernels that look the table up in registers stream table[15] there). */
int32_t btb_hip_p12_pairs(const void* table, void* pairs, void* stream);

/* row_esc[S r + k] = row r's escape k (k < S; S = 8 where cols <= 4096, else 16) as one word: the weight's low byte
 * in bits 0..7, its true high byte in 8..15, its column in 16..30 (0x7FFF: the row has no such escape); bit 31 of all
 * the row's words: the row has more than S. The matvec asks for a row's words ahead of the row's weights, so an escape costs it no trip to memory of
 * its own at the end of the row (the list does: its slice, its entries, the low bytes they name). Made once at upload
 * from the list, the low bytes and row_ptr; cols <= 32767 (BTB_ERR_DOMAIN beyond). No counterpart in the reference. */
int32_t btb_hip_p12_row_esc(const void* lo, const void* esc_idx, const void* esc_val, size_t n_esc, const void* row_ptr,
                            size_t rows, size_t cols, void* row_esc, void* stream);

/* row_ptr[r] = how many escapes lie below weight r * cols, r = 0..rows: the per-row slices of the escape list the
 * matvec reads. Run once when a packed matrix is uploaded; replaces the per-call search of p12_cursors
 * (native/src/gemv.rs:719-734). */
int32_t btb_hip_p12_row_ptr(const void* esc_idx, size_t n_esc, size_t rows, size_t cols, void* row_ptr, void* stream);

/* Validates a packed tensor's escape list on the device, once, when it is uploaded: BTB_ERR_DOMAIN unless esc_idx
 * i32[n_esc] is strictly ascending with every entry in [0, n) - the lists btb_gemv_p12_rows refuses per call
 * (native/src/gemv.rs:4171-4189; native/src/lib.rs:114-135 "strictly ascending"). The matvec and widen entry points
 * index the low bytes and x with these entries and do not re-check them, so a list from an untrusted store goes
 * through here first. `flag` is one device int32 the check may write. Synchronous (it reads the verdict back and
 * waits for `stream`), so it is not for graph capture. n_esc == 0 launches nothing. */
int32_t btb_hip_p12_check(const void* esc_idx, size_t n_esc, size_t n, int32_t* flag, void* stream);

/* A packed tensor of n weights back to bf16 [n], escapes applied: unpack_bf16 (btb/pack12.py:70-97) on the device,
 * through the same in-register widen the matvec uses. out 16-byte aligned. */
int32_t btb_hip_p12_widen(const void* lo, const void* hi4, const void* table, const void* esc_idx, const void* esc_val,
                          size_t n_esc, size_t n, void* out, void* stream);

/* The matvec over an FP8 matrix: w u8[R * C] e4m3fn, scales f32[sr * sc] row-major (one per block of R / sr rows by
 * C / sc columns), weight = bf16(e4m3 * scale) - btb_gemv_fp8_rows (native/src/lib.rs:511-526) with bf16 x and y.
 * sr divides R, sc divides C, and a block is a multiple of 16 columns wide. */
int32_t btb_hip_gemv_fp8(const void* w, const void* scales, size_t sr, size_t sc, const void* x, void* y, size_t R,
                         size_t C, size_t M, void* stream);

/* out u16[n] = the stored bf16 nearest to x f32[n], ties to even, a NaN the quiet NaN with its sign and upper payload -
 * the crate's round_bf16 (native/src/gemv.rs:3003-3007) over an array, with the NaN rule of a torch cast; the rounding
 * every bf16 output of this library goes through. */
int32_t btb_hip_round_bf16(const void* x, void* out, size_t n, void* stream);

/* An FP8 matrix widened to the held weights bf16(e4m3 * scale): bf16 [rows, cols] (out_f32 == 0) or the same values
 * as f32 (out_f32 != 0). fp8.held (btb/fp8.py:97-100) on the device. */
int32_t btb_hip_fp8_widen(const void* w, const void* scales, size_t rows, size_t cols, size_t sr, size_t sc, void* out,
                          int32_t out_f32, void* stream);

/* The matvec over an MXFP4 matrix in the checkpoint's layout: blocks u8[R * C / 32 * 16], scales u8[R * C / 32],
 * weight = fp4(code) * 2^(scale - 127) - btb_gemv_mxfp4_rows (native/src/lib.rs:147-160) with bf16 x and y. C a
 * multiple of 32. */
int32_t btb_hip_gemv_mxfp4(const void* blocks, const void* scales, const void* x, void* y, size_t R, size_t C, size_t M,
                           void* stream);

/* MXFP4 stacks widened block by block: for seat i (seats[i], or i when seats is NULL) the `groups` blocks at
 * blocks[seat * groups ..] become out[i * groups * 32 ..], bf16 (out_f32 == 0: the kernel btb_mx4_widen,
 * native/cuda/btb_kernels.cu:718-738) or the unrounded f32 product (out_f32 != 0: the CPU matvec's weight,
 * native/src/gemv.rs:1090-1119). n_seats <= 65535. */
int32_t btb_hip_mx4_widen(const void* blocks, const void* scales, const void* seats, size_t n_seats, int64_t groups,
                          void* out, int32_t out_f32, void* stream);

/* ---- the crate's CPU entry points on the device: f32 x and y, the host's bits ------------------------------ */

/* y[i][r] = sum_c bf16(w[r][c]) * x[i][c] in f32, in the host's order (16 lane sums, lane j the columns = j mod 16,
 * the pairwise fold): bit-identical to btb_gemv_bf16_rows on the CPU (native/src/lib.rs:69-80) for every b. w
 * [rows, cols] bf16 bit patterns, x [b, cols] f32, y [b, rows] f32, all on the device; `threads` is replaced by the
 * stream. Also the reference card's btb_gemv_lane16_f32_m* (native/cuda/btb_kernels.cu:1635-1699). */
int32_t btb_hip_gemv_bf16_rows(const uint16_t* w, size_t rows, size_t cols, const float* x, size_t b, float* y,
                               void* stream);

/* n independent tasks (native/src/lib.rs:91-104): the arrays of pointers and sizes are host arrays, what they point
 * to is on the device. Every task is checked before the first is launched. */
int32_t btb_hip_gemv_bf16_group(size_t n, const uint16_t* const* w, const size_t* rows, const size_t* cols,
                                const float* const* x, const size_t* b, float* const* y, void* stream);

/* btb_gemv_p12_rows (native/src/lib.rs:114-135) on the device, bit-identical to it and so to the bf16 form. The
 * escape list is not re-checked per call (that would copy a verdict back to the host every time): validate it once
 * at upload with btb_hip_p12_check. */
int32_t btb_hip_gemv_p12_rows(const uint8_t* lo, const uint8_t* hi4, const uint8_t* table, const int32_t* esc_idx,
                              const uint8_t* esc_val, size_t n_esc, size_t rows, size_t cols, const float* x, size_t b,
                              float* y, void* stream);

/* btb_gemv_mxfp4_rows / _group (native/src/lib.rs:147-160, 193-209) on the device, bit-identical to them; the
 * reference card's btb_gemv_lane16_mx4_f32_m* (native/cuda/btb_kernels.cu:1701-1766). */
int32_t btb_hip_gemv_mxfp4_rows(const uint8_t* blocks, const uint8_t* scales, size_t rows, size_t cols, const float* x,
                                size_t b, float* y, void* stream);
/* btb_gemv_mxfp4_ggml_rows (native/src/lib.rs:162-183) on the device: the same matvec over ggml's MXFP4 layout (a
 * GGUF's) - raw holds 17-byte blocks, the e8m0 scale first, then 16 bytes whose low nibbles are weights 0..15 and high
 * nibbles 16..31. The same arithmetic in the same order: the bits of btb_hip_gemv_mxfp4_rows for the same weights. */
int32_t btb_hip_gemv_mxfp4_ggml_rows(const uint8_t* raw, size_t rows, size_t cols, const float* x, size_t b, float* y,
                                     void* stream);
int32_t btb_hip_gemv_mxfp4_group(size_t n, const uint8_t* const* blocks, const uint8_t* const* scales,
                                 const size_t* rows, const size_t* cols, const float* const* x, const size_t* b,
                                 float* const* y, void* stream);

/* btb_gemv_fp8_rows / _group (native/src/lib.rs:511-552) on the device, bit-identical to them. */
int32_t btb_hip_gemv_fp8_rows(const uint8_t* w, const float* scales, size_t rows, size_t cols, size_t sr, size_t sc,
                              const float* x, size_t b, float* y, void* stream);
int32_t btb_hip_gemv_fp8_group(size_t n, const uint8_t* const* w, const float* const* scales, const size_t* rows,
                               const size_t* cols, const size_t* sr, const size_t* sc, const float* const* x,
                               const size_t* b, float* const* y, void* stream);

/* ---- routed experts ---------------------------------------------------------------------------------------- */

/* Per row t of logits [T, ls] (bf16, or f32 when logits_f32 != 0): f32 softmax over the first E, the top k in the
 * total order (p descending, index ascending), weights p / sum(top k) summed in rank order. idx i32 [T, k], w bf16
 * [T, k], and the unrounded weights into w32 f32 [T, k] when it is not NULL. k <= 32. Replaces the kernel
 * btb_moe_route (native/cuda/btb_kernels.cu:861-948; its host-publish arguments have no use with experts resident
 * in VRAM) and the softmax / topk / renormalise of Qwen4Router.forward (btb/engine/families/qwen4/router.py:43-51). */
int32_t btb_hip_moe_route(const void* logits, int32_t logits_f32, size_t ls, size_t E, size_t k, size_t T, int32_t* idx,
                          void* w, float* w32, void* stream);

/* group_picks (btb/engine/host.py:283-296) on the device: the (pick position, row) pairs of idx i32 [T, k] sorted by
 * expert with a stable sort of idx.T.reshape(-1) - so an expert's pairs come pick-major, then row - into slot i32
 * [T k] and token i32 [T k], and each expert's first place and count among them into offs i32 [E] and counts i32 [E].
 * Every id must lie in [0, E) (btb_hip_moe_route's do). T k <= 65535. The experts kernel below does this grouping in
 * place (an expert's first pair gathers the others); this entry point is the reference's function as data. */
int32_t btb_hip_moe_group_picks(const int32_t* idx, size_t T, size_t k, size_t E, int32_t* slot, int32_t* token,
                                int32_t* offs, int32_t* counts, void* stream);

/* Qwen4Router.forward for bf16 rows in two launches (btb/engine/families/qwen4/router.py:43-51): the f32 logits of
 * x [T, H] bf16 against router [E, H] bf16 in the host matvec's order (btb_hip_gemv_bf16_rows of the rows widened to
 * f32, to the bit) into logits f32 [T, E], then btb_hip_moe_route over them. logits16, when not NULL, receives the
 * logits rounded to bf16 [T, E] (the reference hands them back in the rows' dtype). k <= 32, E <= 8192, T <= 65535. */
int32_t btb_hip_moe_router_bf16(const void* router, const void* x, size_t T, size_t E, size_t H, size_t k, float* logits,
                                void* logits16, int32_t* idx, void* w, float* w32, void* stream);

/* The routed experts of T rows: gate_up [E, 2I, H] and down [E, H, I] bf16 stacks (gate rows then up rows), x [T, H]
 * bf16, the picks idx [T, k] and weights w bf16 [T, k] of btb_hip_moe_route, gu [T, k, 2I] bf16 scratch the caller
 * owns (the kernels keep the picks' h rows in it), y [T, H] bf16. Per pick: gu = bf16(W_gu x), h = bf16(bf16(silu(g)) * u), d = bf16(W_dn h); per row
 * y = sum over the picks in ASCENDING expert id of bf16(d * w), each addition rounded to bf16: the arithmetic of
 * _Experts._one_row / _loop (btb/engine/host.py:508-569, 906-967). T * k <= 65535. */
int32_t btb_hip_moe_experts_bf16(const void* gate_up, const void* down, const void* x, const int32_t* idx, const void* w,
                                 void* gu, void* y, size_t T, size_t k, size_t E, size_t H, size_t I, void* stream);

/* btb_hip_moe_experts_bf16 over MXFP4 expert stacks as the checkpoint stores them (btb/mxfp4.py:4-29): gu_blocks u8
 * [E, 2I, H / 32, 16] and gu_scales u8 [E, 2I, H / 32], dn_blocks u8 [E, H, I / 32, 16] and dn_scales u8 [E, H, I / 32];
 * every weight fp4 * 2^(scale - 127), made in registers inside the matvec, no widened copy. The grouped device form of
 * _Experts over `btb_gemv_mxfp4_group` (native/src/lib.rs:193-209; btb/engine/host.py:508-569, 906-967).
 * oss == 0: the gate and up rows concatenated, h = bf16(bf16(silu(g)) * u), no biases (gu_bias, dn_bias NULL).
 * oss != 0: gpt-oss's experts (host.py:414-451): gate row 2 r and up row 2 r + 1 interleaved; gu_bias bf16 [E, 2I]
 * (or NULL) added to the rounded products; the gate clamped to <= limit and the up half to +-limit;
 * h = (up + 1) * (gate * sigmoid(alpha * gate)), every operation rounded to bf16 as torch rounds it; dn_bias bf16
 * [E, H] (or NULL) added to the expert's rounded down product before its weight. h [T, k, I] bf16 is scratch the
 * caller owns. H and I multiples of 32; the other limits are btb_hip_moe_experts_bf16's. */
int32_t btb_hip_moe_experts_mxfp4(const void* gu_blocks, const void* gu_scales, const void* dn_blocks,
                                  const void* dn_scales, const void* gu_bias, const void* dn_bias, const void* x,
                                  const int32_t* idx, const void* w, void* h, void* y, size_t T, size_t k, size_t E,
                                  size_t H, size_t I, int32_t oss, float alpha, float limit, void* stream);

/* ---- the decode step's kernels between the matvecs ---------------------------------------------------------- */

/* h[t] = table[ids[t]]: the step's input row (the reference gathers it with torch before its graph). table
 * [vocab, H] bf16, ids i32 [T] on the device, h [T, H] bf16; H a multiple of 8. */
int32_t btb_hip_embed(const void* table, const int32_t* ids, void* h, size_t T, size_t H, size_t vocab, void* stream);

/* h [T, H] bf16 in place: h = bf16(h + y) when y is not NULL; x = bf16(h * rsqrt(mean(h^2) + eps) * w), or
 * * (1 + w) when centered. Replaces btb_add_rmsnorm (native/cuda/btb_kernels.cu:360-393). */
int32_t btb_hip_add_rmsnorm(void* h, const void* y, const void* w, float eps, void* x, size_t T, size_t H,
                            int32_t centered, void* stream);

/* q/k RMSNorm per head (wq / wk [D], NULL: none), rope from the bf16 tables cos / sin [positions, D], row t of the
 * pass written into the caches at slot *n0 + t and q [T, Hq, D] out. qkv [T, (Hq + 2 Hk) D] bf16; head g's slot j
 * of K / V at g * hs + j * rs elements; row t's position is *n0 + depth[t] (depth NULL: *n0 + t). D 64, 128 or
 * 256. Replaces btb_norm_rope_kv_d{D} (native/cuda/btb_kernels.cu:250-358). */
int32_t btb_hip_norm_rope_kv(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                             const void* sin_t, const int32_t* n0, const int32_t* depth, void* K, void* V, void* q,
                             size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered,
                             void* stream);

/* btb_hip_norm_rope_kv with the cache's row map: row t of the pass lands in cache row tbl[*n0 + t] (tbl i32 on the
 * device, one entry per logical slot), where btb_hip_attn_decode_win's walk reads it. Replaces
 * btb_norm_rope_kv_tbl_d{D} (native/cuda/btb_kernels.cu:268-283, 347-354). */
int32_t btb_hip_norm_rope_kv_tbl(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                                 const void* sin_t, const int32_t* n0, const int32_t* depth, void* K, void* V, void* q,
                                 size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered,
                                 const int32_t* tbl, void* stream);

/* The same for a pass whose T rows are T sequences of their own, a token each - a fork's rows, which share one
 * prefix, or a batch's, whose prefixes lie end to end in the cache. rw is the reference's rows layout, int32 on the
 * device: [base, steps, W, then (col, off, len) a row]. Row t's keys in logical order are its prefix (len cache slots
 * from off) and then its own steps, step i at slot base + i * W + col; the row stands at position len + steps and is
 * written to that step's slot. A row with len < 0 is padding: nothing is read or written for it. The layout is
 * trusted as the reference's kernel trusts it: every slot it names must lie inside the cache. Replaces
 * btb_norm_rope_kv_rows_d{D} (native/cuda/btb_kernels.cu:232-249, 339-346). */
int32_t btb_hip_norm_rope_kv_seqs(const void* qkv, const void* wq, const void* wk, float eps, const void* cos_t,
                                  const void* sin_t, const int32_t* rw, void* K, void* V, void* q, size_t T, size_t Hq,
                                  size_t Hk, size_t D, int64_t hs, int64_t rs, int32_t centered, void* stream);

/* floats of scratch btb_hip_attn_decode needs for T rows and S key spans */
size_t btb_hip_attn_scratch_floats(size_t T, size_t Hq, size_t Hk, size_t D, size_t S);

/* Decode attention: att [T, Hq * D] = softmax(q K^T * scale) V, f32 throughout, bf16 out. par NULL: a chain of rows,
 * row t over the keys 0 .. *n0 + t. par given (a verify pass's tree, T <= 32: par[t] the row's parent among the
 * pass's rows, -1 at a root): row t over the cache's keys 0 .. *n0 - 1 and, of the pass's own rows at slots
 * *n0 .. *n0 + T - 1, its ancestors and itself - the reference's TREE form (native/cuda/btb_attn_flash.cuh:284-286,
 * 407-419). The keys (capacity `cap`: K and V hold at least that many slots) are cut into S spans, a workgroup per
 * (kv head, span, row) - per (kv head, span) with every row of the pass, on the matrix cores, where the pass has several
 * rows, spans of 128 keys and 2 or 4 query heads a kv head - leaving its online-softmax state in `workspace`
 * (btb_hip_attn_scratch_floats floats); a second small launch folds the spans in span order. head_dim 128, Hq / Hk in {1, 2, 4, 8}, S * (Hq / Hk) <= 1024. Replaces btb_attn_flash_d128's decode form
 * (native/cuda/btb_attn_flash.cuh:277-675); its window and row map arguments are btb_hip_attn_decode_win's. */
int32_t btb_hip_attn_decode(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                            const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                            float scale, size_t cap, size_t S, float* workspace, void* stream);

/* btb_hip_attn_decode under a sliding window and through the cache's row map, the two remaining arguments of the
 * reference's decode form (native/cuda/btb_attn_flash.cuh:372-379, 437, 517, 537). win > 0: a row standing at logical
 * position `last` (*n0 + t in a chain, *n0 + its depth in a tree) sees the positions last + 1 - win .. last only; 0: no
 * window. tbl (NULL: none): logical slot j of the cache is its row tbl[j] (i32 on the device, `cap` entries) - an
 * address, never a bit: the result is the unmapped cache's. */
int32_t btb_hip_attn_decode_win(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                                float scale, size_t cap, size_t S, int64_t win, const int32_t* tbl, float* workspace,
                                void* stream);

/* btb_attn_flash_d128 with the reference kernel's own scratch arguments (native/cuda/btb_attn_flash.cuh:372-379): the
 * spans' states go into the caller's three arrays - part_m and part_l of S * T * Hq floats, part_acc of S * T * Hq * 128,
 * the sizes the reference's card graph allocates (btb/engine/cuda.py:1563-1583), in this library's own order - so a
 * launch by the reference's kernel name allocates nothing and a captured graph keeps reading the arrays it was recorded
 * with. `span` keys a span (a multiple of 128; the reference's key group is 512), S spans: S * span need not be the
 * cache's capacity, only reach it - every load stays on a key the row sees. The bits are btb_hip_attn_decode_win's at
 * cap = S * span on its general kernel; the reference's arrival counter is not needed (a second launch folds). */
int32_t btb_hip_attn_decode_parts(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                  const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs,
                                  float scale, size_t span, size_t S, int64_t win, const int32_t* tbl, float* part_m,
                                  float* part_l, float* part_acc, void* stream);

/* btb_hip_attn_decode for callers that cannot allocate device memory or pass a workspace: code under hipGraph
 * capture, tight serving loops, harnesses that forbid hipMalloc. No counterpart in the reference. The spans' partial
 * states go into an array the library itself holds on every GPU it runs on (BTB_HIP_ATTN_NOALLOC_FLOATS floats =
 * 4 MiB per GPU, until the process ends), so the call allocates nothing and takes no workspace; otherwise the
 * arguments, limits, kernels and result bits are btb_hip_attn_decode's. BTB_ERR_DOMAIN (and a message) when
 * btb_hip_attn_scratch_floats(T, Hq, Hk, D, S) exceeds BTB_HIP_ATTN_NOALLOC_FLOATS. The array's address on a device is
 * looked up once, by btb_hip_init or by the first call there. Every call on a GPU shares that GPU's array: calls that
 * overlap on one GPU (two streams, two threads) race on it - serialise them or use btb_hip_attn_decode. Nothing in
 * the array needs clearing between calls: every state a call reads, it has written first. */
/* Decode attention for a pass of T sequences a token each (rw: the rows layout of btb_hip_norm_rope_kv_seqs). Row t
 * attends to its own sequence's len + steps + 1 keys, walked in logical order in S spans of `span` keys (a multiple
 * of 128), under a window of `win` keys when win > 0: the partition, the arithmetic and so the bits are those of
 * btb_hip_attn_decode_parts at T = 1 over a cache that holds that sequence alone, whatever rows step beside it. The
 * spans' states go into the caller's part_m, part_l (T Hq S floats each) and part_acc (T Hq S D floats); a padding
 * row's output is left as it was. head_dim 128. Replaces btb_attn_flash_rows_d128
 * (native/cuda/btb_attn_flash.cuh:395-404, 663-672; btb/engine/cuda.py:1752-1756). */
int32_t btb_hip_attn_decode_seqs(const void* q, const void* K, const void* V, void* att, const int32_t* rw, size_t T,
                                 size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, float scale, size_t span,
                                 size_t S, int64_t win, float* part_m, float* part_l, float* part_acc, void* stream);

#define BTB_HIP_ATTN_NOALLOC_FLOATS ((size_t)1 << 20)
int32_t btb_hip_attn_decode_noalloc(const void* q, const void* K, const void* V, void* att, const int32_t* n0,
                                    const int32_t* par, size_t T, size_t Hq, size_t Hk, size_t D, int64_t hs,
                                    int64_t rs, float scale, size_t cap, size_t S, void* stream);

/* The decode step's own attention (one row), straight from the fused qkv row [(Hq + 2 Hk) D] bf16: what
 * btb_hip_norm_rope_kv followed by btb_hip_attn_decode compute at T = 1, bit for bit, in one launch less - the
 * q / k norm and rope happen inside the attention workgroups (q never reaches memory), the workgroup whose key span
 * holds slot *n0 writes the new K / V row - unless *n0 >= cap: a cache that is already full is not written past
 * (the keys the row then attends to are the cache's `cap` and its own, taken from the chip). Same scratch, spans and
 * limits as btb_hip_attn_decode. Replaces the pair
 * btb_norm_rope_kv_d128 + btb_attn_flash_d128 of the reference's card step (btb/engine/cuda.py:1756-1790). */
int32_t btb_hip_attn_decode_qkv(const void* qkv, const void* wq, const void* wk, float eps, int32_t centered,
                                const void* cos_t, const void* sin_t, const int32_t* n0, void* K, void* V, void* att,
                                size_t Hq, size_t Hk, size_t D, int64_t hs, int64_t rs, float scale, size_t cap,
                                size_t S, float* workspace, void* stream);

/* The same for a pass of T >= 2 rows on the matrix cores: qkv [T, (Hq + 2 Hk) D] bf16, depth (i32 [T], device) the
 * rows' depths for a tree pass or NULL for a chain (row t stands at *n0 + t), par as for btb_hip_attn_decode. What
 * btb_hip_norm_rope_kv followed by btb_hip_attn_decode compute, bit for bit, in one launch less: each workgroup
 * prepares the pass's q heads itself, the workgroups whose key span holds some of slots *n0 .. *n0 + T - 1 prepare
 * and write those K / V rows. For head_dim 128, spans of 128 keys, 2 or 4 query heads a kv head and
 * T * (Hq / Hk) <= 64: btb_hip_attn_rows_fused returns 1 for such a pass and 0 otherwise, where this call fails with
 * BTB_HIP_ERR_DOMAIN and the two calls it replaces remain. Workspace: btb_hip_attn_scratch_floats(T, ...). Replaces
 * btb_norm_rope_kv_d128 + btb_attn_flash_d128 of the reference's verify pass (btb/engine/cuda.py:1756-1790,
 * native/cuda/btb_attn_flash.cuh:400-470). */
int32_t btb_hip_attn_rows_fused(size_t T, size_t Hq, size_t Hk, size_t D, size_t cap, size_t S);
int32_t btb_hip_attn_decode_qkv_rows(const void* qkv, const void* wq, const void* wk, float eps, int32_t centered,
                                     const void* cos_t, const void* sin_t, const int32_t* n0, const int32_t* depth,
                                     const int32_t* par, void* K, void* V, void* att, size_t T, size_t Hq, size_t Hk,
                                     size_t D, int64_t hs, int64_t rs, float scale, size_t cap, size_t S,
                                     float* workspace, void* stream);

/* m [T, I] = bf16(bf16(silu(g)) * u) over gu [T, 2I] (gate then up). Replaces btb_silu_mul
 * (native/cuda/btb_kernels.cu:467-484); the matvec btb_hip_gemv_silu_bf16 folds the same values into its x load. */
int32_t btb_hip_silu_mul(const void* gu, void* m, size_t T, size_t I, void* stream);

/* out[t] = the index of row t's largest logit, the lowest index on ties (native/src/sample.rs:53-67). logits
 * [T, V] bf16. */
int32_t btb_hip_argmax(const void* logits, int32_t* out, size_t T, size_t V, void* stream);

/* btb_hip_argmax over one row followed by btb_hip_publish, in one launch: the thread that ends up with the pick
 * writes it to *picked and goes on with the step's end. Replaces the greedy pick (native/src/sample.rs:53-67) and
 * btb_publish (native/cuda/btb_kernels.cu:448-465) at the end of the reference's step graph. */
int32_t btb_hip_argmax_publish(const void* logits, size_t V, int32_t* picked, int32_t* n0, int32_t* next_ids,
                               int32_t* out_tok, int32_t* out_n0, int64_t* out_ts, void* stream);

/* The step's end, one thread: *next_ids = *picked (the next step's input, when not NULL), *n0 += 1, and with
 * out_tok not NULL (pinned host memory) the token and the GPU's clock, then - after a system fence - the new
 * length, so a host that sees the length sees the token. Replaces btb_publish (native/cuda/btb_kernels.cu:448-465). */
int32_t btb_hip_publish(int32_t* n0, const int32_t* picked, int32_t* next_ids, int32_t* out_tok, int32_t* out_n0,
                        int64_t* out_ts, void* stream);

/* The reference's btb_publish as it is (native/cuda/btb_kernels.cu:455-465): the step's token *ids and the card's
 * clock into pinned host memory, then - after a system fence - the cache's length *n0; nothing on the device changes. */
int32_t btb_hip_publish_only(const int32_t* n0, const int32_t* ids, int32_t* out_tok, int32_t* out_n0, int64_t* out_ts,
                             void* stream);

#ifdef __cplusplus
}
#endif

#endif /* BTB_HIP_H */
