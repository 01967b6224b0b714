// Next-token choice on the device: the reference's `typical` sampler (agnostic/samplers/typical.py:1-17) and
// argmax, with the logit adjustment and the stop-token test of RWKVMaster.forward (rwkvMaster.py:34-54), so
// that a generation loop needs no host round trip per token.
//
// typical(logits, temp, tau):  p = softmax(float32(logits));  s = -log p;  H = sum p s (entropy);
// d = |s - H|;  in ascending order of d, the tokens before the first one whose running mass reaches tau, and
// that one, are kept (everything with d greater than its d is zeroed);  kept p^(1/temp) is sampled.
// The order itself is never needed: the cut is the smallest d* among the tokens with mass{d <= d*} >= tau,
// found by a radix search over the bit pattern of d (non-negative floats order like their bits), two bits
// per round.  One workgroup of 1024 threads; thread t owns the contiguous tokens [t * CH, (t + 1) * CH).
#include "rwkv_common.h"
#include "rwkv_sample.h"

namespace rwkv {

namespace {

constexpr int kST = 1024;            // threads
constexpr int kSMaxPer = 52;         // tokens per thread kept in registers (probability and key): vocabularies up to 53248

__device__ __forceinline__ float block_sum_f(float v, float *scr) {
    v = wave_sum(v);
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scr[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = 0.f;
#pragma unroll
    for (int w = 0; w < kST / 64; ++w) s += scr[w];
    return s;
}
__device__ __forceinline__ float block_max_f(float v, float *scr) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    __syncthreads();
    if ((threadIdx.x & 63) == 0) scr[threadIdx.x >> 6] = v;
    __syncthreads();
    float s = -INFINITY;
#pragma unroll
    for (int w = 0; w < kST / 64; ++w) s = fmaxf(s, scr[w]);
    return s;
}

// splitmix64 of (seed, counter) -> uniform in [0, 1) with 24 bits
__device__ __forceinline__ float uniform01(unsigned long long seed, unsigned long long counter) {
    unsigned long long z = seed + 0x9E3779B97F4A7C15ull * (counter + 1ull);
    z = (z ^ (z >> 30)) * 0xBF58476D1CE4E5B9ull;
    z = (z ^ (z >> 27)) * 0x94D049BB133111EBull;
    z ^= z >> 31;
    return (float)(z >> 40) * (1.0f / 16777216.0f);
}

template <int PER>
__global__ void __launch_bounds__(kST)
sample_kernel(SampleArgs a) {
    __shared__ float scr[3 * (kST / 64)];
    __shared__ float wsum[kST / 64];
    __shared__ int s_tok;
    if (a.stop_flag && *a.stop_flag) return;         // a stop token ended the sequence: the rest of the loop is skipped
    const int V = a.V, tid = threadIdx.x;
    const int CH = (V + kST - 1) / kST, i0 = tid * CH;
    if (a.end_adj != 0.0 && tid == 0) a.logits[0] += a.end_adj;       // rwkvMaster.py:37, kept in the returned logits
    __syncthreads();
    float p[PER];                                    // first the float32 logits, then the probabilities
    float mx = -INFINITY;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const int i = i0 + k;
        p[k] = (k < CH && i < V) ? (float)a.logits[i] : -INFINITY;
        mx = fmaxf(mx, p[k]);
    }
    mx = block_max_f(mx, scr);
    int token = 0;
    if (a.greedy) {
        // first maximum (float64 comparison on the stored logits, as the greedy loop does)
        double best = -INFINITY; int bi = 0x7fffffff;
        for (int k = 0; k < CH; ++k) { const int i = i0 + k; if (i < V) { const double x = a.logits[i]; if (x > best) { best = x; bi = i; } } }
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const double ob = __shfl_xor(best, off, 64); const int oi = __shfl_xor(bi, off, 64);
            if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
        }
        __shared__ double sv[kST / 64]; __shared__ int si[kST / 64];
        if ((tid & 63) == 0) { sv[tid >> 6] = best; si[tid >> 6] = bi; }
        __syncthreads();
        if (tid == 0) {
            for (int w = 1; w < kST / 64; ++w) if (sv[w] > best || (sv[w] == best && si[w] < bi)) { best = sv[w]; bi = si[w]; }
            s_tok = bi == 0x7fffffff ? 0 : bi;
        }
        __syncthreads();
        token = s_tok;
    } else {
        // softmax in float32 (typical.py:5)
        float z = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) { p[k] = expf(p[k] - mx); z += p[k]; }       // exp(-inf) = 0 past the end
        z = block_sum_f(z, scr);
        const float rz = 1.0f / z;
        // surprise, entropy (nansum: terms with p == 0 are skipped), distance from the entropy
        float h = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            p[k] *= rz;
            if (p[k] > 0.f) h -= logf(p[k]) * p[k];
        }
        h = block_sum_f(h, scr);
        unsigned key[PER];
#pragma unroll
        for (int k = 0; k < PER; ++k) key[k] = p[k] > 0.f ? __float_as_uint(fabsf(-logf(p[k]) - h)) : 0x7f800000u;   // p == 0: d = inf
        // radix search, most significant bits first: the largest prefix P with mass{key < P} < tau
        unsigned prefix = 0;
        for (int shift = 30; shift >= 0; shift -= 2) {
            float m1 = 0.f, m2 = 0.f, m3 = 0.f;
            const unsigned c1 = prefix | (1u << shift), c2 = prefix | (2u << shift), c3 = prefix | (3u << shift);
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                m1 += key[k] < c1 ? p[k] : 0.f;
                m2 += key[k] < c2 ? p[k] : 0.f;
                m3 += key[k] < c3 ? p[k] : 0.f;
            }
            // three sums with one pair of barriers
            m1 = wave_sum(m1); m2 = wave_sum(m2); m3 = wave_sum(m3);
            __syncthreads();
            if ((tid & 63) == 0) { scr[tid >> 6] = m1; scr[kST / 64 + (tid >> 6)] = m2; scr[2 * (kST / 64) + (tid >> 6)] = m3; }
            __syncthreads();
            float t1 = 0.f, t2 = 0.f, t3 = 0.f;
#pragma unroll
            for (int w = 0; w < kST / 64; ++w) { t1 += scr[w]; t2 += scr[kST / 64 + w]; t3 += scr[2 * (kST / 64) + w]; }
            if (t3 < a.tau) prefix = c3; else if (t2 < a.tau) prefix = c2; else if (t1 < a.tau) prefix = c1;
        }
        // prefix = d* as bits (mass{key < d*} < tau <= mass{key <= d*}); if the whole mass stays below tau every
        // finite key passes.  Kept tokens, temperature, total.
        const float inv_t = a.temp != 1.0f ? 1.0f / a.temp : 1.0f;
        float q = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            float w = (key[k] <= prefix && p[k] > 0.f) ? p[k] : 0.f;
            if (a.temp != 1.0f && w > 0.f) w = powf(w, inv_t);
            p[k] = w;
            q += w;
        }
        // inverse CDF in token order: scan of the per-thread sums, then a walk inside one thread's tokens
        float own = q;
        float incl = own;
#pragma unroll
        for (int off = 1; off < 64; off <<= 1) { const float o = __shfl_up(incl, off, 64); if ((tid & 63) >= off) incl += o; }
        __syncthreads();
        if ((tid & 63) == 63) wsum[tid >> 6] = incl;
        __syncthreads();
        float before = 0.f, total = 0.f;
#pragma unroll
        for (int w = 0; w < kST / 64; ++w) { if (w < (tid >> 6)) before += wsum[w]; total += wsum[w]; }
        const float lo = before + incl - own, hi = before + incl;
        const float target = uniform01(a.seed, a.counter) * total;
        if (tid == 0) s_tok = -1;
        __syncthreads();
        if (own > 0.f && target >= lo && target < hi) {
            float acc = lo;
            int pick = -1;
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                if (pick < 0 && p[k] > 0.f) { acc += p[k]; if (target < acc) pick = i0 + k; }
            }
            if (pick < 0) {                            // rounding at the upper edge: the thread's last kept token
#pragma unroll
                for (int k = 0; k < PER; ++k) if (p[k] > 0.f) pick = i0 + k;
            }
            atomicMax(&s_tok, pick);
        }
        __syncthreads();
        if (s_tok < 0) {                               // target fell on a boundary nobody claimed (or the total is 0): most probable token
            // argmax over float32 logits kept in key order is gone; fall back on the first maximum of p
            float bp = -1.f; int bi = 0;
#pragma unroll
            for (int k = 0; k < PER; ++k) if (p[k] > bp) { bp = p[k]; bi = i0 + k; }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                const float ob = __shfl_xor(bp, off, 64); const int oi = __shfl_xor(bi, off, 64);
                if (ob > bp || (ob == bp && oi < bi)) { bp = ob; bi = oi; }
            }
            __shared__ float fv[kST / 64]; __shared__ int fi[kST / 64];
            if ((tid & 63) == 0) { fv[tid >> 6] = bp; fi[tid >> 6] = bi; }
            __syncthreads();
            if (tid == 0) {
                for (int w = 1; w < kST / 64; ++w) if (fv[w] > bp || (fv[w] == bp && fi[w] < bi)) { bp = fv[w]; bi = fi[w]; }
                s_tok = bi < V ? bi : 0;
            }
            __syncthreads();
        }
        token = s_tok;
    }
    if (tid == 0) {
        a.out_token[0] = token;
        if (a.n_done) a.n_done[0] += 1;
        bool stop = false;
        for (int i = 0; i < a.n_stop; ++i) stop = stop || a.stop_tokens[i] == (int64_t)token;
        if (stop && a.stop_flag) *a.stop_flag = 1;     // rwkvMaster.py:49-50: the stop token itself is still part of the output
    }
}

}  // namespace

int sample_launch(hipStream_t st, const SampleArgs &a) {
    if (a.V <= 0 || a.V > kST * kSMaxPer) return set_error(RWKV_ERR_SIZE, "sampler: vocabulary %d exceeds %d", a.V, kST * kSMaxPer);
    if (a.V <= kST * 8) hipLaunchKernelGGL(sample_kernel<8>, dim3(1), dim3(kST), 0, st, a);
    else hipLaunchKernelGGL(sample_kernel<kSMaxPer>, dim3(1), dim3(kST), 0, st, a);
    RWKV_CHECK_LAUNCH("sample_kernel");
    return RWKV_OK;
}

}  // namespace rwkv
