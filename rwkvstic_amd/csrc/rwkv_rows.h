// Interface of the many-row (prompt / batch) kernels to the model host code.
#pragma once

#include "rwkv_common.h"

namespace rwkv {

enum RowTail { ROW_STORE = 0, ROW_RELU2 = 1, ROW_ADD = 2, ROW_GATE_ADD = 3 };

// Device scratch one rows_matmul call needs for R rows (sizes from the helpers below,
// taken at the largest contraction length K and output width N that will be used).
struct RowsScratch {
    signed char *dig;       // rows_dig_bytes(R, K)
    long long *tot;         // rows_tot_bytes(R, N)
    double *S, *qs, *zp;    // [R] each
};
size_t rows_dig_bytes(int64_t R, int64_t K);
size_t rows_tot_bytes(int64_t R, int64_t N);
size_t rows_wkv_scratch_bytes(int64_t R, int64_t C);

int rows_embed(hipStream_t st, const int64_t *tokens, int64_t R, int V, int C, const float *emb, const double *w,
               const double *b, double *x);
// n_mix in {0, 2, 3}; see LnMixArgs in rwkv_rows.hip for the meaning of prev0 / shift_dst / prev_stride.
int rows_ln_mix(hipStream_t st, int n_mix, int64_t R, int C, bool sequence, const double *x, const double *ln_w,
                const double *ln_b, const double *mu, const double *prev0, double *shift_dst, int64_t prev_stride,
                double *mix);
// out[R, N] (tail op) in[R, K] x quantised matrix (M16 blocks, per-input-channel range / offset).
int rows_matmul(hipStream_t st, const RowsScratch &s, int64_t R, int64_t K, int64_t N, const double *in,
                const uint8_t *w16, const float *range, const double *offset, int op, double *out,
                const double *gate);
int rows_wkv(hipStream_t st, int64_t R, int C, bool sequence, const double *k, const double *v, const double *r,
             const double *w, const double *u, double *state, int64_t state_stride, double *out,
             double *scratch /* rows_wkv_scratch_bytes(R, C), or null: serial over the rows */);

}  // namespace rwkv
