// Device-side choice of the next token (typical sampling or argmax) with logit adjustment and stop tokens.
#pragma once

#include "rwkv_common.h"

namespace rwkv {

struct SampleArgs {
    double *logits;               // [V]; logits[0] += end_adj in place (rwkvMaster.py:37)
    int V;
    int greedy;                   // 1: first maximum instead of sampling
    float temp, tau;
    double end_adj;
    unsigned long long seed, counter;    // draw = hash(seed, counter): reproducible, one counter value per token
    int64_t *out_token;           // [1]
    const int64_t *stop_tokens;   // [n_stop] device, may be null when n_stop == 0
    int n_stop;
    int *stop_flag;               // device word or null: set to 1 when the chosen token is a stop token; while it is 1
                                  // the kernel (and the token kernels of the loop) return at once
    int64_t *n_done;              // device counter of tokens chosen, or null
};

int sample_launch(hipStream_t st, const SampleArgs &a);

}  // namespace rwkv
