/*
 * rwkv_hip.h -- C ABI of librwkv_hip.so: the MI355X (gfx950) backend for the
 * FASTQUANT (fp32i8) RWKV-4 forward path.
 *
 * Conventions for every entry point
 *   - returns 0 (RWKV_OK) or a negative rwkv_status; never throws, never
 *     synchronises the device, never retains caller pointers past the call
 *     (the model handle retains the pointers in its descriptor by design);
 *   - all data pointers are DEVICE pointers unless a comment says "host";
 *   - work is enqueued on `stream` (a hipStream_t passed as void*; NULL is the
 *     null stream) and is ordered with other work on that stream;
 *   - arguments are validated on the host (null pointers, sizes, alignment)
 *     before anything is launched; rwkv_last_error() describes the last
 *     failure on the calling thread.
 *
 * File:line citations name the reference interface each entry point replaces,
 * relative to the reference repository's src/rwkvstic/.
 */
#ifndef RWKV_HIP_H
#define RWKV_HIP_H

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef void *rwkv_stream_t; /* hipStream_t */

typedef enum rwkv_status {
    RWKV_OK = 0,
    RWKV_ERR_ARG = -1,       /* null pointer / non-positive size / bad enum   */
    RWKV_ERR_ALIGN = -2,     /* pointer or stride not aligned as documented   */
    RWKV_ERR_SIZE = -3,      /* shape outside what the kernels support        */
    RWKV_ERR_WORKSPACE = -4, /* workspace too small                           */
    RWKV_ERR_HIP = -5,       /* a HIP runtime call failed                     */
    RWKV_ERR_DEVICE = -6     /* no gfx950 device                              */
} rwkv_status;

int rwkv_version(void);
const char *rwkv_last_error(void);

/* ------------------------------------------------------------------------
 * 1. The three operators of the reference's native library "rwkv"
 *    (agnostic/backends/cuda/wrapper.cpp:131-141), same argument meaning,
 *    same in-place semantics, reference memory layouts.
 * ---------------------------------------------------------------------- */

/* Bytes of scratch rwkv_mm8_one / rwkv_mm8_three need for a given shape
 * (n_mat = 1 or 3).  The scratch holds per-row-split partial sums that are
 * then added in a fixed order, which makes the result deterministic (the
 * reference races 16 atomicAdds per output, operators32.cu:38). */
size_t rwkv_mm8_workspace_bytes(int64_t n_in, int64_t n_out, int n_mat);

/* mm8_one (wrapper.cpp:52-79, operators32.cu:18-40,105-115):
 *   y[k] += sum_j x[j] * (w[j*w_stride + k] * r[j]),  j < n_in, k < n_out.
 * x[n_in], r[n_in], y[n_out] float32 (y is accumulated into, as in the
 * reference where the caller zero-fills it, matmul.py:44); w uint8 rows of
 * n_out bytes, row stride w_stride >= n_out bytes.  The zero-point term is
 * NOT added here (the reference adds it in Python, matmul.py:59-62). */
int rwkv_mm8_one(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                 const float *x, const uint8_t *w, int64_t w_stride,
                 float *y, const float *r,
                 void *workspace, size_t workspace_bytes);

/* rwkv_mm8_one without a workspace argument and without any allocation, for
 * callers that cannot allocate device memory: code under HIP graph capture,
 * tight serving loops, harnesses that forbid hipMalloc.  It has no counterpart
 * in the reference.  The partial sums go to a fixed array inside the library's
 * device image (rwkv_mm8_one_static_max_bytes() = 12 MiB per GPU, held until
 * the process ends); shapes that need more
 * (rwkv_mm8_workspace_bytes(n_in, n_out, 1) > the maximum) are rejected with
 * RWKV_ERR_SIZE.  Same arithmetic, same kernels and bit-identical results as
 * rwkv_mm8_one.  All calls on one GPU share the array: calls that overlap on
 * one GPU (two streams, two threads) race; calls on one stream do not.
 * The first use on a device looks up the array's device address (a symbol
 * look-up, not a stream operation): it must happen outside a stream capture.
 * rwkv_mm8_one_static_max_bytes() performs that look-up for the current device,
 * so a caller about to capture calls it (or the entry point itself) once
 * before; later calls enqueue two kernels and nothing else. */
size_t rwkv_mm8_one_static_max_bytes(void);
int rwkv_mm8_one_static(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                        const float *x, const uint8_t *w, int64_t w_stride,
                        float *y, const float *r);

/* mm8_three (wrapper.cpp:82-127, operators32.cu:44-104): three independent
 * (x, w, r, y) problems sharing n_in and n_out in one launch. */
int rwkv_mm8_three(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                   const float *x0, const float *x1, const float *x2,
                   const uint8_t *w0, int64_t w0_stride,
                   const uint8_t *w1, int64_t w1_stride,
                   const uint8_t *w2, int64_t w2_stride,
                   float *y0, float *y1, float *y2,
                   const float *r0, const float *r1, const float *r2,
                   void *workspace, size_t workspace_bytes);

/* The float64 instances of the two operators (the `double` branch of
 * wrapper.cpp:60-77,95-127; kernels operators.cu:58-80,84-118): x, r, y and
 * the sums are float64, everything else as above.  FASTQUANT itself only ever
 * calls the float32 instances (matmul.py:58,72-74). */
size_t rwkv_mm8_f64_workspace_bytes(int64_t n_in, int64_t n_out, int n_mat);
int rwkv_mm8_one_f64(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                     const double *x, const uint8_t *w, int64_t w_stride,
                     double *y, const double *r,
                     void *workspace, size_t workspace_bytes);
int rwkv_mm8_three_f64(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                       const double *x0, const double *x1, const double *x2,
                       const uint8_t *w0, int64_t w0_stride,
                       const uint8_t *w1, int64_t w1_stride,
                       const uint8_t *w2, int64_t w2_stride,
                       double *y0, double *y1, double *y2,
                       const double *r0, const double *r1, const double *r2,
                       void *workspace, size_t workspace_bytes);

/* wkv_forward (wrapper.cpp:45-50, operators.cu:6-44), float64, reference
 * state convention: k, v, y are [B, T, C]; w (= -exp(time_decay)), u are [C];
 * aa, bb, pp are [B, C] and are updated in place; on return aa, bb hold the
 * reference's e^w-premultiplied sums and pp is left untouched.  Internally
 * the recurrence runs in the max-shifted form, so it does not overflow where
 * the reference's naive form would not either. */
int rwkv_wkv_forward_f64(rwkv_stream_t stream, int64_t B, int64_t T, int64_t C,
                         const double *w, const double *u,
                         const double *k, const double *v, double *y,
                         double *aa, double *bb, double *pp);

/* ------------------------------------------------------------------------
 * 2. Quantiser and weight layouts (agnostic/backends/modules/matmul.py:18-40)
 * ---------------------------------------------------------------------- */

/* MM8.QuantizeMatrix: weight[n_out, n_in] float32 row-major (the checkpoint
 * orientation) -> codes[n_in, n_out] uint8 row-major (the reference/.rwkv
 * layout), range[n_in] float32, offset[n_in] float64; one scale and one
 * minimum per INPUT channel, float64 arithmetic, truncating codes, mean
 * truncated fraction folded into the offset.  A constant input channel
 * (max == min) gets range 0, codes 0, offset = the constant (the reference
 * divides by zero there). */
int rwkv_quantize_u8(rwkv_stream_t stream, const float *weight,
                     int64_t n_out, int64_t n_in,
                     uint8_t *codes, float *range, double *offset);

/* Device layout the matvec/GEMM kernels stream: 1 KiB blocks of 8 output
 * columns x 128 input rows, blocks ordered [ceil(n_out/8)][ceil(n_in/128)],
 * zero padded.  Within a block, byte 16*(8*s + c) + 4*m + e holds
 * codes[128*kb + 32*m + 4*s + e][8*ct + c]  (c, s < 8; m, e < 4), so that a
 * 64-lane wavefront reads the block with one 16-byte load per lane and lane
 * (s, c) multiplies against four 16-byte LDS reads that are conflict free. */
size_t rwkv_packed_bytes(int64_t n_in, int64_t n_out);
int rwkv_pack_u8(rwkv_stream_t stream, const uint8_t *codes, int64_t codes_stride,
                 int64_t n_in, int64_t n_out, uint8_t *packed);
/* Inverse of rwkv_pack_u8 (used by .rwkv export and by the parity tests). */
int rwkv_unpack_u8(rwkv_stream_t stream, const uint8_t *packed,
                   int64_t n_in, int64_t n_out, uint8_t *codes, int64_t codes_stride);

/* Second device layout, for the single-token matrix-core kernel: 1 KiB blocks
 * of 16 output columns x 64 input rows, blocks ordered
 * [ceil(n_out/16)][ceil(n_in/64)], zero padded; byte 16*(16*g + n) + i of a
 * block holds codes[64*kb + 16*g + i][16*ct + n] - 128 as a signed byte
 * (g < 4, n < 16, i < 16): one wavefront-wide 16-byte load is the B operand
 * of v_mfma_i32_16x16x64_i8. */
size_t rwkv_packed_m16_bytes(int64_t n_in, int64_t n_out);
int rwkv_pack_m16(rwkv_stream_t stream, const uint8_t *codes, int64_t codes_stride,
                  int64_t n_in, int64_t n_out, uint8_t *packed);
int rwkv_unpack_m16(rwkv_stream_t stream, const uint8_t *packed,
                    int64_t n_in, int64_t n_out, uint8_t *codes, int64_t codes_stride);

/* Canonical dequantisation fp32(fp64(code)*fp64(range[j]) + offset[j]) of a
 * packed matrix into dq[n_in, n_out] float32 row-major (parity/debug). */
int rwkv_dequant_packed(rwkv_stream_t stream, const uint8_t *packed,
                        const float *range, const double *offset,
                        int64_t n_in, int64_t n_out, float *dq);

/* ------------------------------------------------------------------------
 * 3. Stand-alone kernels on the packed layout
 * ---------------------------------------------------------------------- */

/* Quantised matrix-vector product with the general four-vector dequantisation
 *   dq[j,k] = code[j,k]*r_row[j]*r_col[k] + m_row[j] + m_col[k]
 *   y[b,k]  = r_col[k]*sum_j fp32(x[b,j]*r_row[j])*code[j,k]
 *             + sum_j x[b,j]*m_row[j] + m_col[k]*sum_j x[b,j]
 * for b < B, B in {1, 2, 4, 8}.  x[B, n_in] float32, y[B, n_out] float64 (float32
 * accumulation of the matrix term, float64 zero-point terms, as in
 * MM8.forward matmul.py:51-62).  r_col / m_col may be NULL (= 1 / 0): that
 * is the reference layout.  Replaces MM8.forward for T == 1. */
int rwkv_mm8_packed(rwkv_stream_t stream, int64_t B, int64_t n_in, int64_t n_out,
                    const float *x, const uint8_t *packed,
                    const float *r_row, const double *m_row,
                    const float *r_col, const float *m_col,
                    double *y);

/* The same product on the matrix cores, for any B in 1..8, on the M16 layout
 * (rwkv_pack_m16).  Two launches: the vectors are rewritten once as exact
 * fixed-point digits (fp32(x*r_row) to 30 bits, one power-of-two scale per
 * vector and chunk of 256 input rows), then every 16-column tile is
 * multiplied with v_mfma_i32_16x16x64_i8; the integer sums are exact and the
 * result is the real-number sum over the float32 values fp32(x*r_row) to
 * float64 rounding: where rwkv_mm8_packed accumulates in float32 (as
 * operators32.cu:18-40 does), this one does not round at all.  With B >= 2 the
 * vector pipeline of rwkv_mm8_packed is the limit, not memory; this routine
 * stays memory-bound.  workspace: rwkv_mm8_m16_workspace_bytes(B, n_in) bytes,
 * 256-byte aligned, overwritten. */
size_t rwkv_mm8_m16_workspace_bytes(int64_t B, int64_t n_in);
int rwkv_mm8_m16(rwkv_stream_t stream, int64_t B, int64_t n_in, int64_t n_out,
                 const float *x, const uint8_t *packed16,
                 const float *r_row, const double *m_row,
                 const float *r_col, const float *m_col,
                 double *y, void *workspace, size_t workspace_bytes);

/* Max-shifted float32 WKV recurrence, state in registers: one thread per
 * (b, c) for short sequences; from 256 steps on (and C a multiple of 32) a
 * scan over chunks of the sequence inside a workgroup.  With at least 512
 * groups of 32 channels (B * C / 32) every chunk stays in registers between
 * the pass that sums it up and the pass that writes y, so k and v are read
 * once; smaller problems use 8 or 16 chunks per sequence and read them twice.
 * Either way the results differ from the serial order by float32 rounding
 * only.  k, v, y [B, T, C]; w, u [C]; state (aa, bb, pp) [B, C] updated
 * in place and related to the reference's naive state by
 * aa_ref = aa*exp(pp), bb_ref = bb*exp(pp) (operators.cu:21-36; closed form
 * of the shifted recurrence: agnostic/agnosticRwkv.py:68-103). */
int rwkv_wkv_f32(rwkv_stream_t stream, int64_t B, int64_t T, int64_t C,
                 const float *w, const float *u,
                 const float *k, const float *v, float *y,
                 float *aa, float *bb, float *pp);

/* ------------------------------------------------------------------------
 * 4. Whole-model forward (replaces myRWKV.forward, agnostic/backends/opt.py:61-76,
 *    and everything it calls: modules/block.py:56-102, modules/layernorm.py:11-20,
 *    modules/emb.py:9, modules/matmul.py:51-102, modules/wkv.py:8-19)
 * ---------------------------------------------------------------------- */

typedef struct rwkv_qmat {
    const uint8_t *packed;   /* rwkv_pack_u8 layout, 16-byte aligned          */
    const uint8_t *packed16; /* rwkv_pack_m16 layout, 16-byte aligned, or NULL:
                                without it the single-token step runs as one
                                launch per phase instead of one per token     */
    const float *range;      /* [n_in]                                        */
    const double *offset;    /* [n_in]                                        */
    int64_t n_in, n_out;
} rwkv_qmat;

typedef struct rwkv_layer_desc {
    const double *ln1_w, *ln1_b, *ln2_w, *ln2_b; /* [C]                       */
    const double *att_mix;    /* [3, C]  rows k, v, r   (block.py:35-37)     */
    const double *ffn_mix;    /* [2, C]  rows k, r      (block.py:46-47)     */
    const double *time_decay; /* [C]  = -exp(raw)       (block.py:41)        */
    const double *time_first; /* [C]                    (block.py:39)        */
    rwkv_qmat att_k, att_v, att_r, att_o, ffn_k, ffn_r, ffn_v;
} rwkv_layer_desc;

typedef struct rwkv_model_desc {
    int64_t n_layer, n_embd, n_ffn, n_vocab;
    const float *emb;            /* [V, C] float32, device                    */
    const double *ln0_w, *ln0_b; /* blocks.0.ln0 (opt.py:40-43)               */
    const double *ln_out_w, *ln_out_b;
    rwkv_qmat head;
    const rwkv_layer_desc *layers; /* HOST array of n_layer descriptors       */
} rwkv_model_desc;

typedef struct rwkv_model rwkv_model;

/* Copies the descriptor; the device buffers it names must outlive the handle.
 * This is the one entry point that allocates device memory: one block with the
 * tables of the single-token kernel (packed per-layer constants, column sums,
 * 4 KiB of owner record and 128 bytes of job pointers per layer and
 * 16-channel tile), which rwkv_model_destroy frees, and the kernel's exchange
 * vectors, taken from a process-wide pool of uncached device memory that
 * later handles reuse and that is never returned to the driver.
 * One forward call may be in flight per handle at a time, on one stream; while
 * a single-token step runs, that stream must have the device to itself: the
 * workgroups of the persistent kernel (n_embd / 16, or n_embd / 32 at
 * n_embd = 5120) wait for each other and must all be resident.  A step that
 * cannot make progress gives up after a bounded wait and is reported by
 * rwkv_model_check; it never hangs. */
int rwkv_model_create(const rwkv_model_desc *desc, rwkv_model **out);
void rwkv_model_destroy(rwkv_model *m);

/* 1 if single-token steps of this handle run as one persistent launch (all
 * matrices have packed16 and the shape is supported), else 0. */
int rwkv_model_has_fused_step(const rwkv_model *m);

/* Diagnostics: when device_buffer is non-NULL, every workgroup g of every
 * following single-token launch writes 100 MHz wall-clock stamps of its phase
 * boundaries into device_buffer[g][layer][24]; NULL switches it off.  The
 * buffer must hold rwkv_model_trace_workgroups(m) * n_layer * 24 int64 values:
 * the owner workgroups (n_embd / 16, or n_embd / 32 at n_embd = 5120) followed
 * by the helper workgroups of the ffn key matrix where the kernel has them
 * (80 at n_embd = 2560), whose six stamps are: records seen, statistics,
 * digits written, tiles multiplied, results published, next weights fetched. */
int rwkv_model_trace_workgroups(const rwkv_model *m);
int rwkv_model_set_trace(rwkv_model *m, int64_t *device_buffer);

/* Synchronises the device and returns RWKV_ERR_HIP if a single-token launch
 * since the previous check gave up waiting for another workgroup (logits and
 * state written since then are invalid), else RWKV_OK.  The condition is
 * reported once: the flag is cleared, later steps run normally. */
int rwkv_model_check(rwkv_model *m);

/* Measurement aid (no counterpart in the reference): feeds the token at *token
 * n times (the state advances n steps) with HIP events recorded on the stream
 * immediately before and after each launch of the persistent single-token
 * kernel - the per-token preparation launch stays outside the pair - then
 * synchronises the stream and returns the kernel's average duration in
 * microseconds.  Creates and destroys 2 n events.  Only models with
 * rwkv_model_has_fused_step. */
int rwkv_model_time_token_kernel(rwkv_model *m, rwkv_stream_t stream, const int64_t *token, double *state,
                                 double *logits, int n, float *avg_us);

/* Self-test of the single-token kernel's failure path (no counterpart in the
 * reference): launches one token step whose input is never published and whose
 * waits give up after a few hundred polls instead of the usual million, so
 * that every workgroup runs into its bounded wait, raises the abort flag and
 * leaves - the launch ends normally within a millisecond.  state and logits
 * are left untouched.  The next rwkv_model_check reports the aborted step
 * (and clears the flag); token steps after that run as usual.  Only models
 * with rwkv_model_has_fused_step. */
int rwkv_model_selftest_timeout(rwkv_model *m, rwkv_stream_t stream, double *state, double *logits);

/* Scratch needed by rwkv_model_forward for chunks of up to max_tokens tokens. */
size_t rwkv_model_workspace_bytes(const rwkv_model *m, int64_t max_tokens);

/* logits[V], state = forward(tokens[T], state):  emb -> ln0 -> L x Block ->
 * ln_out -> head(last token).  tokens: int64 [T] on the device; state:
 * float64 [L, 5, C] on the device, rows (att shift, ffn shift, aa, bb, pp),
 * updated in place.  WKV rows hold the max-shifted triple (see rwkv_wkv_f32);
 * the reference's empty state (0, 0, 0, 0, -1e30) is valid as is.
 * logits: float64 [V].  Path: T >= 4 with the M16 layout of every matrix and
 * n_embd, n_ffn multiples of 64 takes the many-row (GEMM) kernels; fewer tokens
 * go one at a time through the persistent single-token kernel where
 * rwkv_model_has_fused_step, else as one-row prompts through the many-row
 * kernels, and only without the M16 layout as one launch per phase. */
int rwkv_model_forward(rwkv_model *m, rwkv_stream_t stream,
                       const int64_t *tokens, int64_t T,
                       double *state, double *logits,
                       void *workspace, size_t workspace_bytes);

/* Prompt / batch GEMM on the matrix cores: y[T, n_out] = x[T, n_in] x quantised
 * matrix, the T > 1 branch of MM8.forward (matmul.py:56-57; the reference
 * rounds to bfloat16 there, this routine keeps the single-token arithmetic:
 * fp32(x * range) as exact 32-bit fixed point per row, integer dot products,
 * zero-point term in float64).  x, y float64 row-major; packed16 from
 * rwkv_pack_m16; n_in a multiple of 64. */
size_t rwkv_gemm8_workspace_bytes(int64_t T, int64_t n_in, int64_t n_out);
int rwkv_gemm8(rwkv_stream_t stream, int64_t T, int64_t n_in, int64_t n_out,
               const double *x, const uint8_t *packed16, const float *range,
               const double *offset, double *y,
               void *workspace, size_t workspace_bytes);

/* Diagnostics: the launch plan rwkv_gemm8 / the model's many-row path follows for
 * n_products (1..3) products x[T, n_in] x matrix[n_in, n_out] sharing a launch
 * (k, v, r do; matmul.py:86-94): plan = {kernel variant (0: at most 8 rows, 1: 9-32
 * rows, 2: 64 x 128 tiles, 3: 64 x 160 tiles), grid x, grid y, splits of the
 * contraction}, and in *tot_bytes_per_product the bytes of integer totals the
 * workspace reserves per product.  Host-only: launches nothing. */
int rwkv_gemm8_plan(int64_t T, int64_t n_in, int64_t n_out, int n_products,
                    int plan[4], size_t *tot_bytes_per_product);

/* One token for each of `batch` independent sequences (the reference has no
 * batched entry point on this path: it would call myRWKV.forward, opt.py:61-76,
 * once per sequence).  tokens[batch]; states[batch][n_layer][5][n_embd] updated
 * in place; logits[batch][n_vocab].  Needs the M16 layout of every matrix. */
size_t rwkv_model_batch_workspace_bytes(const rwkv_model *m, int64_t batch);
int rwkv_model_forward_batch(rwkv_model *m, rwkv_stream_t stream,
                             const int64_t *tokens, int64_t batch,
                             double *states, double *logits,
                             void *workspace, size_t workspace_bytes);

/* Greedy decode entirely on the device: for i < n:
 *   logits, state = forward(tokens[i], state); tokens[i+1] = argmax(logits).
 * tokens: int64 [n + 1] on the device, tokens[0] is the input token.  This is
 * RWKVMaster.forward(number=n) (rwkvMaster.py:28-56) with the sampler
 * replaced by argmax and no host round trip per token. */
int rwkv_model_decode_greedy(rwkv_model *m, rwkv_stream_t stream,
                             int64_t *tokens, int64_t n,
                             double *state, double *logits,
                             void *workspace, size_t workspace_bytes);

/* The choice of the next token on the device (agnostic/samplers/typical.py:1-17 and the
 * logit adjustment of rwkvMaster.py:37): logits[0] += end_adj (in place), then either
 * the first maximum (greedy != 0) or locally typical sampling: softmax in float32,
 * tokens ordered by |surprise - entropy|, the shortest prefix of that order whose mass
 * reaches tau kept, kept p^(1/temp) sampled with the uniform number hash(seed, counter).
 * V <= 53248.  out_token: device int64 [1]. */
int rwkv_sample_token(rwkv_stream_t stream, double *logits, int64_t V, int greedy,
                      float temp, float tau, double end_adj,
                      uint64_t seed, uint64_t counter, int64_t *out_token);

/* RWKVMaster.forward(number=n) (rwkvMaster.py:28-56) entirely on the device:
 *   for i < n: logits, state = forward(tokens[i], state);
 *              tokens[i+1] = rwkv_sample_token(logits, ..., counter = i);
 *              stop if tokens[i+1] is one of stop_tokens[n_stop].
 * stop_flag (device int32, zero on entry) is set when a stop token was chosen; the
 * launches queued after that return without touching state or logits, so both are
 * those of the stopping step.  n_done (device int64, zero on entry) counts the tokens
 * chosen: tokens[1 .. n_done] are valid.  Only for handles with
 * rwkv_model_has_fused_step; other shapes return RWKV_ERR_SIZE (sample from the logits
 * of rwkv_model_forward instead). */
int rwkv_model_decode_sample(rwkv_model *m, rwkv_stream_t stream,
                             int64_t *tokens, int64_t n,
                             double *state, double *logits,
                             void *workspace, size_t workspace_bytes,
                             int greedy, float temp, float tau, double end_adj,
                             uint64_t seed, const int64_t *stop_tokens, int n_stop,
                             int32_t *stop_flag, int64_t *n_done);

/* out_token[0] = index of the first maximum of logits[V]. */
int rwkv_argmax_f64(rwkv_stream_t stream, const double *logits, int64_t V,
                    int64_t *out_token);

#ifdef __cplusplus
}
#endif
#endif /* RWKV_HIP_H */
