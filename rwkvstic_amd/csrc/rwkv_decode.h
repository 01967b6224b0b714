// Interface between the model host code and the persistent single-token kernel.
#pragma once

#include "rwkv_common.h"

namespace rwkv {

typedef unsigned long long u64;

struct DQ {                 // one quantised matrix as the decode kernel sees it
    const uint8_t *w16;     // M16 layout (code - 128), 1 KiB blocks [n_out/16][n_in/64]
    const float *range;     // [n_in]
    const double *offset;   // [n_in]
};

struct DLayer {
    DQ att_k, att_v, att_r, att_o, ffn_k, ffn_r, ffn_v;
    const double *ln1_w, *ln1_b, *ln2_w, *ln2_b;
    const double *att_mix, *ffn_mix, *time_decay, *time_first;
};

struct DModel {
    int L, C, F, V;
    const float *emb;
    const double *ln0_w, *ln0_b, *lnout_w, *lnout_b;
    DQ head;
    const DLayer *layers;   // device array [L]
};

// Exchange buffers of tagged 8-byte words {epoch:32 | float32 payload}; they
// must be zero-filled once before the first launch and belong to one model
// handle (one decode step in flight at a time).
struct DecodeBuffers {
    u64 *X;                 // [C]  residual stream, float32 view
    u64 *A;                 // [C]  wkv * sigmoid(r)
    u64 *H;                 // [F]  relu(k)^2
    unsigned *abort_flag;   // set to 1 by any workgroup whose wait ran out
};

bool decode_supported(int64_t L, int64_t C, int64_t F, int64_t V);
unsigned decode_epochs_per_token(int64_t L);
int decode_launch(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                  const int64_t *token, double *state, double *logits);

}  // namespace rwkv
