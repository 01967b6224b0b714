// Next-token choice on the device: the reference's `typical` sampler (agnostic/samplers/typical.py:1-17) and
// argmax, with the logit adjustment and the stop-token test of RWKVMaster.forward (rwkvMaster.py:34-54), so
// that a generation loop needs no host round trip per token.
//
// typical(logits, temp, tau):  p = softmax(float32(logits));  s = -log p;  H = sum p s (entropy);
// d = |s - H|;  in ascending order of d, the tokens before the first one whose running mass reaches tau, and
// that one, are kept (everything with d greater than its d is zeroed);  kept p^(1/temp) is sampled.
// The order itself is never needed: the cut is the smallest d* among the tokens with mass{d <= d*} >= tau,
// found by a radix search over the bit pattern of d (non-negative floats order like their bits), two bits
// per round.  One workgroup of 1024 threads; thread t owns the tokens t, t + 1024, ... (coalesced reads of the
// logits).  The probabilities stay in registers; of the keys the first kSKeysLds per thread live in LDS and the
// rest in registers: both arrays in registers would not fit the 128 registers a wave of a 1024-thread workgroup has.
#include "rwkv_common.h"
#include "rwkv_sample.h"

#include <mutex>

namespace rwkv {

namespace {

constexpr int kST = 1024;            // threads
constexpr int kSMaxPer = 52;         // tokens per thread: vocabularies up to 53248
constexpr int kSFirstBit = 16;       // full passes settle the key's bits down to this one before the first attempt to list the undecided tokens
constexpr int kSList = 2048;         // tokens that share the upper half of the cut's key: finished by one wave
constexpr int kSKeysLds = 32;        // keys per thread kept in LDS ([k][thread]: conflict-free), 128 KiB

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
    constexpr int KL = PER < kSKeysLds ? PER : kSKeysLds, KR = PER - KL > 0 ? PER - KL : 1;
    extern __shared__ unsigned key_lds[];            // [KL][kST]
    __shared__ float scr[3 * (kST / 64)];
    __shared__ float wsum[kST / 64];
    __shared__ int s_tok, s_cnt;
    __shared__ unsigned s_prefix;
    __shared__ unsigned list_key[kSList];
    __shared__ float list_p[kSList];
    if (a.stop_flag && *a.stop_flag) return;         // a stop token ended the sequence: the rest of the loop is skipped
    const int V = a.V, tid = threadIdx.x;
    if (a.end_adj != 0.0 && tid == 0) a.logits[0] += a.end_adj;       // rwkvMaster.py:37, kept in the returned logits
    __syncthreads();
    float p[PER];                                    // first the float32 logits, then the probabilities
    float mx = -INFINITY;
    int token = 0;
    if (a.greedy) {
        // first maximum (float64 comparison on the stored logits, as the greedy loop does)
        double best = -INFINITY; int bi = 0x7fffffff;
#pragma unroll 13
        for (int k = 0; k < PER; ++k) {
            const int i = tid + kST * k;
            if (i < V) { const double x = a.logits[i]; if (x > best) { best = x; bi = i; } }      // i grows with k: the first of equals stays
        }
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
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const int i = tid + kST * k;
            p[k] = i < V ? (float)a.logits[i] : -INFINITY;
            mx = fmaxf(mx, p[k]);
            if (k % 13 == 12) __builtin_amdgcn_sched_barrier(0);      // at most 13 float64 loads in flight: all 52 at once would not fit the registers
        }
        mx = block_max_f(mx, scr);
        // softmax in float32 (typical.py:5); the hardware exponential (about one ulp) is enough here: only a tie at
        // the edge of the kept set could fall the other way.  p[k] holds t = logit - max until the last pass.
        float z = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) { p[k] -= mx; z += __expf(p[k]); }          // exp(-inf) = 0 past the end
        z = block_sum_f(z, scr);
        const float rz = 1.0f / z, logz = logf(z);
        // surprise s = -log p = log z - t (no logarithm per token), entropy (nansum: terms with p == 0 are skipped)
        float h = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const float pk = __expf(p[k]) * rz;
            if (pk > 0.f) h += (logz - p[k]) * pk;
        }
        h = block_sum_f(h, scr);
        // distance from the entropy as the search key
        unsigned kreg[KR];
#define RWKV_KEY(k) ((k) < KL ? key_lds[(k) * kST + tid] : kreg[(k) - KL < KR ? (k) - KL : 0])
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            const float pk = __expf(p[k]) * rz;
            const unsigned key = pk > 0.f ? __float_as_uint(fabsf(logz - p[k] - h)) : 0x7f800000u;   // p == 0: d = inf
            if (k < KL) key_lds[k * kST + tid] = key; else kreg[k - KL < KR ? k - KL : 0] = key;      // (each thread reads back only its own)
            p[k] = pk;
        }
        // Radix search, most significant bits first, two bits per round: the largest prefix P with mass{key < P} < tau.
        // `below` = mass{key < prefix}.
        // A prefix with no mass at all below it is always taken: typical.py:13-14 keeps the token at position
        // #(cumulative < tau) of the sorted distances, so the token nearest the entropy stays even with tau = 0.
        unsigned prefix = 0;
        float below = 0.f;
#define RWKV_BELOW(t) ((t) < a.tau || (t) <= 0.f)
#define RWKV_FULL_ROUND(shift)                                                                                           \
        {                                                                                                                \
            float m1 = 0.f, m2 = 0.f, m3 = 0.f;                                                                          \
            const unsigned c1 = prefix | (1u << (shift)), c2 = prefix | (2u << (shift)), c3 = prefix | (3u << (shift));  \
            _Pragma("unroll") for (int k = 0; k < PER; ++k) {                                                            \
                const unsigned key = RWKV_KEY(k);                                                                        \
                m1 += key < c1 ? p[k] : 0.f;                                                                             \
                m2 += key < c2 ? p[k] : 0.f;                                                                             \
                m3 += key < c3 ? p[k] : 0.f;                                                                             \
            }                                                                                                            \
            m1 = wave_sum(m1); m2 = wave_sum(m2); m3 = wave_sum(m3);       /* three sums with one pair of barriers */     \
            __syncthreads();                                                                                             \
            if ((tid & 63) == 0) { scr[tid >> 6] = m1; scr[kST / 64 + (tid >> 6)] = m2; scr[2 * (kST / 64) + (tid >> 6)] = m3; } \
            __syncthreads();                                                                                             \
            float t1 = 0.f, t2 = 0.f, t3 = 0.f;                                                                          \
            _Pragma("unroll") for (int w = 0; w < kST / 64; ++w) { t1 += scr[w]; t2 += scr[kST / 64 + w]; t3 += scr[2 * (kST / 64) + w]; } \
            if (RWKV_BELOW(t3)) { prefix = c3; below = t3; } else if (RWKV_BELOW(t2)) { prefix = c2; below = t2; }       \
            else if (RWKV_BELOW(t1)) { prefix = c1; below = t1; }                                                        \
        }
        // After 16 (or 20, 24, 28) bits only the tokens that share those bits with the cut can still decide the rest.
        // As soon as they fit a list of kSList entries, one wave finishes alone: no pass over all tokens, no barriers.
        int shift = 30;
        for (; shift >= kSFirstBit; shift -= 2) RWKV_FULL_ROUND(shift)
        bool listed = false;
        while (shift >= 0) {                           // (uniform) shift = next undecided bit pair
            if (tid == 0) s_cnt = 0;
            __syncthreads();
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                const unsigned key = RWKV_KEY(k);
                if (((key ^ prefix) >> (shift + 2)) == 0u) {
                    const int at = atomicAdd(&s_cnt, 1);
                    if (at < kSList) { list_key[at] = key; list_p[at] = p[k]; }
                }
            }
            __syncthreads();
            if (s_cnt <= kSList) { listed = true; break; }
            __syncthreads();                           // everybody has read the count before it is cleared again
            RWKV_FULL_ROUND(shift)
            shift -= 2;
            if (shift >= 0) { RWKV_FULL_ROUND(shift) shift -= 2; }
        }
        if (listed) {
            const int n_list = s_cnt;
            if (tid < 64) {
                for (; shift >= 0; shift -= 2) {
                    float m1 = 0.f, m2 = 0.f, m3 = 0.f;
                    const unsigned c1 = prefix | (1u << shift), c2 = prefix | (2u << shift), c3 = prefix | (3u << shift);
                    for (int i = tid; i < n_list; i += 64) {
                        const unsigned key = list_key[i];
                        const float pi = list_p[i];
                        m1 += key < c1 ? pi : 0.f;
                        m2 += key < c2 ? pi : 0.f;
                        m3 += key < c3 ? pi : 0.f;
                    }
                    const float t1 = below + wave_sum(m1), t2 = below + wave_sum(m2), t3 = below + wave_sum(m3);
                    if (RWKV_BELOW(t3)) prefix = c3; else if (RWKV_BELOW(t2)) prefix = c2; else if (RWKV_BELOW(t1)) prefix = c1;
                }
                if (tid == 0) s_prefix = prefix;
            }
            __syncthreads();
            prefix = s_prefix;
        }
#undef RWKV_FULL_ROUND
#undef RWKV_BELOW
        // prefix = d* as bits (mass{key < d*} < tau <= mass{key <= d*}); if the whole mass stays below tau every
        // finite key passes.  Kept tokens, temperature, total.
        const float inv_t = a.temp != 1.0f ? 1.0f / a.temp : 1.0f;
        float q = 0.f;
#pragma unroll
        for (int k = 0; k < PER; ++k) {
            float w = (RWKV_KEY(k) <= prefix && p[k] > 0.f) ? p[k] : 0.f;
            if (a.temp != 1.0f && w > 0.f) w = __powf(w, inv_t);      // hardware log2 / exp2: a few ulp, immaterial for a sampling weight
            p[k] = w;
            q += w;
        }
        // inverse CDF in the order (thread, k): scan of the per-thread sums, then a walk inside one thread's tokens
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
                if (pick < 0 && p[k] > 0.f) { acc += p[k]; if (target < acc) pick = tid + kST * k; }
            }
            if (pick < 0) {                            // rounding at the upper edge: the thread's last kept token
#pragma unroll
                for (int k = 0; k < PER; ++k) if (p[k] > 0.f) pick = tid + kST * k;
            }
            atomicMax(&s_tok, pick);
        }
        __syncthreads();
        if (s_tok < 0) {
            // The target fell on a boundary nobody claimed, or every kept weight underflowed under the temperature
            // (total 0): the kept token with the largest logit, the first of equals.  p[] holds the weights by now, so
            // the logits are read again; the kept set is never empty (the token nearest the entropy is always in it).
            double bp = -INFINITY; int bi = 0x7fffffff;
#pragma unroll
            for (int k = 0; k < PER; ++k) {
                const int i = tid + kST * k;
                if (i < V && RWKV_KEY(k) <= prefix) { const double x = a.logits[i]; if (x > bp) { bp = x; bi = i; } }
            }
#pragma unroll
            for (int off = 32; off >= 1; off >>= 1) {
                const double ob = __shfl_xor(bp, off, 64); const int oi = __shfl_xor(bi, off, 64);
                if (ob > bp || (ob == bp && oi < bi)) { bp = ob; bi = oi; }
            }
            __shared__ double fv[kST / 64]; __shared__ int fi[kST / 64];
            if ((tid & 63) == 0) { fv[tid >> 6] = bp; fi[tid >> 6] = bi; }
            __syncthreads();
            if (tid == 0) {
                for (int w = 1; w < kST / 64; ++w) if (fv[w] > bp || (fv[w] == bp && fi[w] < bi)) { bp = fv[w]; bi = fi[w]; }
                s_tok = bi < V ? bi : 0;
            }
            __syncthreads();
        }
#undef RWKV_KEY
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
    constexpr size_t kSmall = (size_t)8 * kST * 4, kLarge = (size_t)kSKeysLds * kST * 4;
    {   // the large variant's dynamic LDS exceeds the default limit: raised once per device
        static std::mutex mu;
        static bool configured[64] = {};
        int dev = 0;
        if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return set_error(RWKV_ERR_DEVICE, "sampler: no current device");
        std::lock_guard<std::mutex> lock(mu);
        if (!configured[dev]) {
            const hipError_t e = hipFuncSetAttribute(reinterpret_cast<const void *>(&sample_kernel<kSMaxPer>),
                                                     hipFuncAttributeMaxDynamicSharedMemorySize, (int)kLarge);
            if (e != hipSuccess) return set_error(RWKV_ERR_HIP, "sampler: %s", hipGetErrorString(e));
            configured[dev] = true;
        }
    }
    if (a.V <= kST * 8) hipLaunchKernelGGL(sample_kernel<8>, dim3(1), dim3(kST), kSmall, st, a);
    else hipLaunchKernelGGL(sample_kernel<kSMaxPer>, dim3(1), dim3(kST), kLarge, st, a);
    RWKV_CHECK_LAUNCH("sample_kernel");
    return RWKV_OK;
}

}  // namespace rwkv
