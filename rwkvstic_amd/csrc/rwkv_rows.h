// Interface of the many-row (prompt / batch) kernels to the model host code.
#pragma once

#include "rwkv_common.h"

namespace rwkv {

// ROW_STORE_F32: the product's `out` points at a float32 [R, N] array (k, v, r and the ffn receptance: their consumers
// round them to float32 anyway, as the single-token kernel does, and the arrays are read several times)
// ROW_RELU2 also stores float32 (its only consumer, the row quantiser, scales the values to float32 next).
enum RowTail { ROW_STORE = 0, ROW_RELU2 = 1, ROW_ADD = 2, ROW_GATE_ADD = 3, ROW_STORE_F32 = 4 };

// One quantised left operand of a product: R rows rewritten as fixed-point digit fragments plus the
// per-row constants of the tail (scale, sum of the fixed-point values, zero-point sum).
struct RowsOperand {
    signed char *dig;       // rows_dig_bytes(R, K)
    double *S, *qs, *zp;    // [R] each
};
struct RowsProduct {        // out[R, N] (tail op) a x quantised matrix in M16 blocks
    RowsOperand a;
    const uint8_t *w16;
    double *out;
};
constexpr int kRowsMaxProducts = 3;     // products of equal shape and tail that share one launch
// A product whose contraction was split, handed on unfinished: its consumer (the LayerNorm kernel for the two
// residual updates, the WKV kernel for k, v, r) adds the slices of integer totals up itself and applies the tail,
// which saves the launch that would otherwise do only that.  tot == nullptr: nothing is pending (the product was not
// split and its epilogue applied the tail).  Only for batches of fewer than kRowsDeferMax independent rows.
struct RowsDeferred {
    const long long *tot;   // [slices][slice] totals of this product; element (t, j) at t * ldd + j
    size_t slice;
    int slices, ldd, op;    // op: the RowTail still to be applied
    const double *S, *qs, *zp;
    const float *gate;      // ROW_GATE_ADD
};
constexpr int64_t kRowsDeferMax = 128;
constexpr int kRowsDeferSlices = 4;     // a contraction split further than this is finished by a launch of its own
size_t rows_dig_bytes(int64_t R, int64_t K);
size_t rows_tot_bytes(int64_t R, int64_t N);        // integer totals of ONE product (times the products in a launch)
size_t rows_wkv_scratch_bytes(int64_t R, int64_t C);
size_t rows_quant_scratch_bytes(int64_t R, int64_t K);   // what rows_quant writes into its scratch area (0: unused)
// The plan rows_products follows for n products [R, K] x [K, N]: out = {kernel kind, grid x, grid y, splits}.
void rows_plan_describe(int64_t R, int64_t K, int64_t N, int n, int out[4]);
bool rows_ln_width_supported(int64_t C);            // widths the fused LayerNorm + mix + quantise kernel holds in registers

int rows_embed(hipStream_t st, const int64_t *tokens, int64_t R, int V, int C, const float *emb, const double *w,
               const double *b, double *x);
// LayerNorm + token shift + time mix of R rows, each mixed row quantised for its matrix (range / offset per
// input channel): n_mix in {0, 2, 3}; 0 = LayerNorm only, one output.  See LnQuantArgs in rwkv_rows.hip for
// the meaning of prev0 / shift_dst / prev_stride.
int rows_ln_mix_quant(hipStream_t st, int n_mix, int64_t R, int C, bool sequence, const double *x, const double *ln_w,
                      const double *ln_b, const double *mu, const double *prev0, double *shift_dst,
                      int64_t prev_stride, const float *const *range, const double *const *offset,
                      const RowsOperand *out, const RowsDeferred *add = nullptr /* pending residual update of x: applied
                      and stored first (x is then written too); batch rows only */);
// Rows of float64 values quantised for a matrix with the given per-input-channel range / offset.
// scratch: rows_quant_scratch_bytes(R, K) bytes (any buffer free until the product starts, e.g. its totals), or null.
int rows_quant(hipStream_t st, int64_t R, int64_t K, const void *in, bool in_f32, const float *range, const double *offset,
               const RowsOperand &out, double *scratch);
// n (<= kRowsMaxProducts) products of the same shape [R, K] x [K, N] and tail in one launch;
// tot: n * rows_tot_bytes(R, N) bytes of scratch.
// defer (null, or n entries): where the contraction is split (in at most kRowsDeferSlices) and R < kRowsDeferMax the tail is left to the consumer
// and described here (tot and the operand's row constants must stay untouched until that kernel has run); entries of
// products that were finished here get tot = nullptr.
int rows_products(hipStream_t st, int n, const RowsProduct *p, long long *tot, int64_t R, int64_t K, int64_t N, int op,
                  const float *gate, RowsDeferred *defer = nullptr);
// kvr (null, or 3 entries, batch rows only): k, v, r still pending as split products (ROW_STORE_F32) where tot is set.
int rows_wkv(hipStream_t st, int64_t R, int C, bool sequence, const float *k, const float *v, const float *r,
             const double *w, const double *u, double *state, int64_t state_stride, float *out,
             double *scratch /* rows_wkv_scratch_bytes(R, C), or null: serial over the rows */,
             const RowsDeferred *kvr = nullptr);

// Stand-alone product of 1..8 float32 vectors with one matrix in M16 blocks, four-vector dequantisation (row and
// column ranges / offsets; r_col, m_col may be null); ws: rows_mv16_workspace_bytes(B, n_in) bytes, 256-byte aligned.
size_t rows_mv16_workspace_bytes(int64_t B, int64_t n_in);
int rows_mv16(hipStream_t st, int64_t B, int64_t n_in, int64_t n_out, const float *x, const uint8_t *w16,
              const float *r_row, const double *m_row, const float *r_col, const float *m_col, double *y, void *ws);

}  // namespace rwkv
