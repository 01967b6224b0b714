// Persistent single-token kernel: interface between the model host code and rwkv_decode.hip.
#pragma once

#include "rwkv_common.h"
#include "rwkv_sample.h"

namespace rwkv {

typedef unsigned long long u64;

struct DQ {                 // one quantised matrix as the host describes it
    const uint8_t *w16;     // M16 layout (code - 128), 1 KiB blocks [n_out/16][n_in/64]
    const float *range;     // [n_in]
    const double *offset;   // [n_in]
};

// Matrix order used by every per-layer table below.
enum { MAT_ATT_K = 0, MAT_ATT_V, MAT_ATT_R, MAT_ATT_O, MAT_FFN_R, MAT_FFN_K, MAT_FFN_V, MAT_COUNT };
// LayerNorm-fed products of a layer, in the order of the constant tables: att k, v, r, ffn k, r.
constexpr int kLnMats = 5;

// Device table entry, one per layer: the M16 blocks of the seven matrices.
struct DLayer {
    const uint8_t *w[MAT_COUNT];
    const uint8_t *pad;
};

// Device table entry, one per layer: what the preparation and model-creation kernels read.
struct DPrep {
    const double *ln1_w, *ln1_b, *ln2_w, *ln2_b, *att_mix, *ffn_mix, *time_decay, *time_first;
    const float *range_o, *range_v;
    const double *offset_o, *offset_v;
    const float *range[kLnMats];
    const double *offset[kLnMats];
};

// Per-layer scalars of the LayerNorm-fed products (row L of the tables is the head, matrix 0).
struct DScal {
    double sumPO[kLnMats];   // sum_c PO[c]
    double sumQO[kLnMats];   // sum_c (ln_b mu + shift (1 - mu)) (offset + 128 range)   (per token)
    float maxP[kLnMats];     // max_c |P32[c]|
    float pad1;
    float maxQ[kLnMats];     // max_c |Q32[c]|                                             (per token)
    float pad2;
};
static_assert(sizeof(DScal) == 128, "DScal is read as a 128-byte record");

struct DModel {
    int L, C, F, V, G;           // G = C / 16 groups of 16 channels
    int NWG;                     // workgroups of the single-token kernel: G, or G / 2 where a workgroup owns two groups (C = 5120)
    const float *emb;
    const double *ln0_w, *ln0_b;
    const uint8_t *w_head;
    const DLayer *layers;        // device [L]
    const DPrep *prep;           // device [L]
    // Per output column: sum over input rows of (code - 128).  Per layer one slab of 6C+F ints in
    // the order att k, v, r, o, ffn r [C each], ffn k [F], ffn v [C]; cs_head [round_up(V, 16)].
    const int *cs;
    const int *cs_head;
    const u64 *jt;               // [NWG][L+1][16] job base addresses per workgroup, of its first group (row L: first head tiles)
    const u64 *ownrec;           // [L][G][512] per-layer constants of each workgroup's own channels
    // With xy = ln(x), mixed = xy mu + shift (1 - mu) and t = (x - mean) rsd:
    //   fp32(mixed range)          = fp32(t P + Q),  P = ln_w mu range,  Q = (ln_b mu + shift (1 - mu)) range
    //   sum_c mixed (offset + 128 range) = rsd (sum_c x PO - mean sum_c PO) + sumQO,  PO = ln_w mu (offset + 128 range)
    float *P32;                  // [L+1][5][C]
    float *Q32;                  // [L+1][5][C]   rows < L rewritten for every token
    double *PO;                  // [L+1][5][C]
    DScal *sc;                   // [L+1]
    DScal *scp;                  // [L][C/512] per-token scalars (sumQO, maxQ) of each 512-channel part of a layer
    double *amax_val;            // [NWG] device-side argmax: first maximum of the logits each workgroup wrote, and its index
    int *amax_idx;
    double *X0;                  // [C] ln0(emb[token]) of the launch in flight
};

// Exchange buffers of tagged 8-byte words {epoch:32 | float32 payload}; zero-filled once before
// the first launch; they belong to one model handle (one token step in flight at a time).
struct DecodeBuffers {
    u64 *X;                 // [C]       residual stream
    u64 *XR;                // [11][G]   per group of 16 channels: sum x, squared deviations from the group's mean, then per matrix max |x P|, sum x PO (hi, lo)
    u64 *A;                 // [C]       fp32(wkv * sigmoid(r) * range_o)
    u64 *AR;                // [3][G]    per workgroup: max |A|, zero-point share (hi, lo)
    u64 *H;                 // [F]       fp32(relu(k)^2 * range_v)
    u64 *HR;                // [3][G]
    unsigned *abort_flag;   // set to 1 by any workgroup whose wait ran out
    long long *trace;       // optional: [NWG][L][24] 100 MHz timestamps of every workgroup's phase boundaries (null = off)
};

// Host-side description from which the tables are built.
struct DLayerSrc {
    DQ att_k, att_v, att_r, att_o, ffn_k, ffn_r, ffn_v;
    const double *ln1_w, *ln1_b, *ln2_w, *ln2_b, *att_mix, *ffn_mix, *time_decay, *time_first;
};
struct DSetup {
    int64_t L, C, F, V;
    const float *emb;
    const double *ln0_w, *ln0_b, *lnout_w, *lnout_b;
    DQ head;
    const DLayerSrc *layers;   // host [L]
};

bool decode_supported(int64_t L, int64_t C, int64_t F, int64_t V);
int64_t decode_helper_workgroups(int64_t C);   // workgroups that only stream the ffn key matrix (launched after the owners)
int64_t decode_workgroups(int64_t C);          // grid of the single-token kernel (C / 16, or C / 32 where a workgroup owns two groups)
unsigned decode_epochs_per_token(int64_t L);
constexpr int kTraceStampsPerLayer = 24;

// Bytes of the single device allocation that holds tables and constants, and of the exchange buffers.
size_t decode_block_bytes(int64_t L, int64_t C, int64_t F, int64_t V);
size_t decode_exchange_bytes(int64_t C, int64_t F);
// Fills `block` (device, decode_block_bytes, zero-filled by the caller) and the two descriptors; `exchange`
// (device, decode_exchange_bytes, zero-filled by the caller) becomes the exchange buffers.
// Synchronises the device (model creation only).
int decode_setup(void *block, void *exchange, const DSetup &s, DModel *dm, DecodeBuffers *db);

// Zero-fills the exchange buffers on the stream (a kernel, so the call may be captured); the next launch must
// use epoch 1.
int decode_clear_exchange(hipStream_t st, const DModel &m, const DecodeBuffers &b);

// One token: token[0] -> logits[V], state [L,5,C] updated in place.  epoch0 must grow by
// decode_epochs_per_token() between launches on the same buffers and never be 0.
int decode_launch(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                  const int64_t *token, double *state, double *logits);
// decode_launch with events recorded on the stream around the token kernel alone (after the preparation launch).
int decode_launch_bracketed(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, const int64_t *token,
                            double *state, double *logits, hipEvent_t before, hipEvent_t after);

// One token step whose input never arrives, with waits that give up after spin_limit polls (self-test of the
// failure path: the launch ends normally with the abort flag set; logits and state are left as they were).
int decode_launch_unfed(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, double *state, double *logits,
                        unsigned spin_limit);

// n greedy steps: tokens[i + 1] = argmax(forward(tokens[i])); uses n * decode_epochs_per_token() epochs.
int decode_launch_greedy(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                         int64_t *tokens, int64_t n, double *state, double *logits);

// n sampled steps: tokens[i + 1] = choice(forward(tokens[i])) by the sampler described in `sa` (its logits, V and
// out_token are filled in here; sa.counter counts up per token).  A chosen stop token sets *sa.stop_flag, after
// which the remaining launches return at once and leave state and logits as they are.
int decode_launch_sampled(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, int64_t *tokens, int64_t n,
                          double *state, double *logits, SampleArgs sa);

}  // namespace rwkv
