// Persistent single-token kernel for the FASTQUANT RWKV-4 forward path
// (reference agnostic/backends/opt.py:61-76, modules/block.py:56-102 at T == 1).
//
// One launch = one token through every layer and the head.  The grid is
// C/16 workgroups of 512 threads, all resident at once; workgroup g owns the
// 16 channels [16g, 16g+16) for the whole token (their residual value, WKV
// state and receptance gate live in its registers) and the matching 16-column
// tiles of every matrix.
//
// Dot products.  A matrix-vector product needs every input for every output,
// so each of the 4 products per layer is a chip-wide dependency.  Weights are
// streamed as 1 KiB blocks of 16 columns x 64 rows (layout "M16", stored as
// code - 128) straight into v_mfma_i32_16x16x64_i8 as the B operand.  The
// activation vector fp32(x * range) is rewritten once per phase as 32-bit
// fixed point q = round(xs / S), S a power of two with |q| <= 2^30, split into
// four signed base-256 digits; the digits are the A operand (rows 0..3), so a
// single instruction yields the four digit sums of 16 columns over 64 rows.
// Everything is integer: the result S * (sum_d 256^(3-d) D_d + 128 sum q) is
// independent of summation order (deterministic) and differs from the
// float32 sum over the same fp32(x * range) only by the |xs - S q| <= S/2
// representation error, which is below one float32 ulp of the largest input.
//
// Exchange.  Cross-workgroup vectors (residual, wkv*r, relu^2) travel as
// 8-byte words {epoch : 32, float32 payload : 32} written and polled with
// agent-scope atomics; a consumer spins until every word it needs carries the
// epoch of the producing phase.  There is no grid barrier and no cache
// flush.  A buffer is rewritten only after every workgroup has consumed the
// previous contents (each rewrite is downstream of a phase that needed all
// workgroups' outputs of the phase that read it).
//
// Weight stream.  The order in which a workgroup needs its weight blocks is
// fixed, so each wave keeps a ring of R jobs (one job = its share of a
// 16-column x C-row tile) in registers and refills a slot right after using
// it: the loads for the next ~R jobs are in flight while the workgroup waits
// for its inputs, which is what hides the exchange latency behind HBM time.
#include "rwkv_decode.h"

namespace rwkv {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kDT = 512;   // threads per workgroup
constexpr int kDW = 8;     // waves per workgroup
constexpr int kJobsPerLayer = 15;   // 13 real jobs padded to a multiple of the ring depth (3 or 5)
constexpr int kMaxJobsPerPhase = 5;
constexpr unsigned kSpinLimit = 1u << 21;

#define ALOAD(p) __hip_atomic_load((p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define ASTORE(p, v) __hip_atomic_store((p), (v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

struct DArgs {
    DModel m;
    DecodeBuffers b;
    unsigned epoch0;
    const int64_t *token;
    double *state;
    double *logits;
};

// ---- workgroup reductions (512 threads, fixed order) -----------------------
template <int N>
__device__ __forceinline__ void wg_sum(double (&v)[N], double *scr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const double s = wave_sum(v[i]);
        if (lane == 0) scr[i * kDW + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kDW; ++w) s += scr[i * kDW + w];
        v[i] = s;
    }
    __syncthreads();
}

template <int N>
__device__ __forceinline__ void wg_max(float (&v)[N], float *scr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float s = v[i];
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) s = fmaxf(s, __shfl_xor(s, off, 64));
        if (lane == 0) scr[i * kDW + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float s = scr[i * kDW];
#pragma unroll
        for (int w = 1; w < kDW; ++w) s = fmaxf(s, scr[i * kDW + w]);
        v[i] = s;
    }
    __syncthreads();
}

// Per-wave partial sums parked in LDS; the epilogue adds the 8 partials in order.
template <int N>
__device__ __forceinline__ void park_partials(const double (&v)[N], double *part /*[kDW][8]*/, int base) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const double s = wave_sum(v[i]);
        if (lane == 0) part[wave * 8 + base + i] = s;
    }
}
__device__ __forceinline__ double sum_partials(const double *part, int idx) {
    double s = 0.0;
#pragma unroll
    for (int w = 0; w < kDW; ++w) s += part[w * 8 + idx];
    return s;
}

// ---- fixed-point digits ------------------------------------------------------
__device__ __forceinline__ void scale_from_amax(float amax, double &S, double &invS) {
    if (!(amax > 0.f) || !(amax < INFINITY)) { S = 0.0; invS = 0.0; return; }
    int e;
    frexpf(amax, &e);                 // amax = f * 2^e, f in [0.5, 1)  =>  |xs| < 2^e
    S = ldexp(1.0, e - 30);
    invS = ldexp(1.0, 30 - e);
}

// q = round(xs / S) as four signed base-256 digits, most significant in plane 0.
__device__ __forceinline__ double put_digits(signed char *dig, int plane_stride, int idx, float xs, double invS) {
    int q = __double2int_rn((double)xs * invS);
    const double qd = (double)q;
    const int d3 = (int)(signed char)(q & 0xff); q = (q - d3) >> 8;
    const int d2 = (int)(signed char)(q & 0xff); q = (q - d2) >> 8;
    const int d1 = (int)(signed char)(q & 0xff); q = (q - d1) >> 8;
    dig[idx] = (signed char)q;
    dig[plane_stride + idx] = (signed char)d1;
    dig[2 * plane_stride + idx] = (signed char)d2;
    dig[3 * plane_stride + idx] = (signed char)d3;
    return qd;
}

// ---- tagged exchange ---------------------------------------------------------
__device__ __forceinline__ void put_word(u64 *dst, unsigned epoch, float v) {
    ASTORE(dst, ((u64)epoch << 32) | (u64)__float_as_uint(v));
}

// Every thread fetches words tid, tid+512, ... ; returns false if the wait ran out
// or another workgroup raised the abort flag.
template <int N>
__device__ __forceinline__ bool poll_words(const u64 *src, unsigned epoch, float (&out)[N], unsigned *abort_flag) {
    u64 w[N];
    unsigned pending = (N >= 32) ? 0xffffffffu : ((1u << N) - 1u);
    unsigned spins = 0;
    bool ok = true;
    while (true) {
#pragma unroll
        for (int u = 0; u < N; ++u)
            if (pending & (1u << u)) w[u] = ALOAD(src + threadIdx.x + kDT * u);
#pragma unroll
        for (int u = 0; u < N; ++u)
            if ((pending & (1u << u)) && (unsigned)(w[u] >> 32) == epoch) pending &= ~(1u << u);
        if (!pending) break;
        ++spins;
        if ((spins & 255u) == 0u && (spins > kSpinLimit || ALOAD(abort_flag) != 0u)) { ok = false; break; }
    }
#pragma unroll
    for (int u = 0; u < N; ++u) out[u] = __uint_as_float((unsigned)w[u]);
    return ok;
}

// ---- weight ring ----------------------------------------------------------------
template <int KBW>
__device__ __forceinline__ void load_slot(uint4 (&slot)[KBW], const uint8_t *p) {
    if (p) {
        const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
        const uint8_t *q = p + (size_t)wave * 1024 + lane * 16;
#pragma unroll
        for (int b = 0; b < KBW; ++b) slot[b] = *reinterpret_cast<const uint4 *>(q + (size_t)b * (kDW * 1024));
    }
}

// D += digits(rows koff ..) x job tile.  Wave w handles blocks w, w+8, ...
template <int KBW>
__device__ __forceinline__ void mfma_job(const uint4 (&slot)[KBW], const signed char *dig, int plane_stride,
                                         int koff, v4i &D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int n = lane & 15, g4 = lane >> 4;
    const signed char *ap = dig + n * plane_stride + koff + 64 * wave + 16 * g4;
#pragma unroll
    for (int b = 0; b < KBW; ++b) {
        v4i A = {0, 0, 0, 0};
        if (n < 4) A = *reinterpret_cast<const v4i *>(ap + b * (64 * kDW));
        const v4i B = {(int)slot[b].x, (int)slot[b].y, (int)slot[b].z, (int)slot[b].w};
        D = __builtin_amdgcn_mfma_i32_16x16x64_i8(A, B, D, 0, 0, 0);
    }
}

// Lanes 0..15 of every wave hold the digit sums of column `lane`; park them.
__device__ __forceinline__ void park_tile(int *red, int j, const v4i &D) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane < 16) *reinterpret_cast<v4i *>(red + ((wave * kMaxJobsPerPhase + j) * 16 + lane) * 4) = D;
}

__device__ __forceinline__ double finish_col(const int *red, int j, int n, double S, double qsumS, double zp) {
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#pragma unroll
    for (int w = 0; w < kDW; ++w) {
        const v4i v = *reinterpret_cast<const v4i *>(red + ((w * kMaxJobsPerPhase + j) * 16 + n) * 4);
        d0 += v.x; d1 += v.y; d2 += v.z; d3 += v.w;
    }
    const long long tot = ((((long long)d0 * 256 + d1) * 256 + d2) * 256) + d3;
    // codes = (code - 128) + 128:  S * (sum (code-128) q + 128 sum q)  + zero-point term
    return S * (double)tot + 128.0 * qsumS + zp;
}

// ---- LayerNorm on KBW values per thread (layernorm.py:15-20) ------------------
template <int KBW>
__device__ __forceinline__ void layernorm_wg(double (&v)[KBW], int C, const double *__restrict__ w,
                                             const double *__restrict__ b, double *scr) {
    double s[2] = {0.0, 0.0};
#pragma unroll
    for (int i = 0; i < KBW; ++i) { s[0] += v[i]; s[1] += v[i] * v[i]; }
    wg_sum<2>(s, scr);
    const double mean = s[0] / (double)C;
    double var = s[1] / (double)C - mean * mean;
    if (var < 0.0) var = 0.0;
    const double rsd = 1.0 / sqrt(var + 1e-5);
#pragma unroll
    for (int i = 0; i < KBW; ++i) {
        const int c = threadIdx.x + kDT * i;
        v[i] = w[c] * ((v[i] - mean) * rsd) + b[c];
    }
}

// =============================================================================
template <int KBW>
__global__ void __launch_bounds__(kDT) decode_kernel(const DArgs a) {
    constexpr int C = KBW * kDT, F = 4 * C, NKB = C / 64;
    constexpr int R = 3;                           // ring depth in jobs
    constexpr int JPL = kJobsPerLayer;
    constexpr int PS = C + 64, PSF = F + 64;        // digit plane strides (+64: conflict-free A reads)
    constexpr size_t kTileBytes = (size_t)NKB * 1024;
    static_assert(JPL % R == 0, "ring depth must divide the padded job count");

    extern __shared__ __align__(16) unsigned char smem[];
    constexpr int DIG_BYTES = (3 * 4 * PS > 4 * PSF) ? 3 * 4 * PS : 4 * PSF;
    signed char *dig = reinterpret_cast<signed char *>(smem);
    int *red = reinterpret_cast<int *>(smem + DIG_BYTES);                           // [2][8][5][16][4]
    constexpr int RED_INTS = kDW * kMaxJobsPerPhase * 16 * 4;
    double *part = reinterpret_cast<double *>(red + 2 * RED_INTS);                  // [2][8][8]
    double *scr = part + 2 * kDW * 8;                                               // [4*8]
    double *own_x = scr + 4 * kDW;                                                  // [16]
    double *own_ln1 = own_x + 16;                                                   // [16]
    double *own_ln2 = own_ln1 + 16;                                                 // [16]

    const int g = blockIdx.x, G = gridDim.x;
    const int tid = threadIdx.x;
    const int L = a.m.L, V = a.m.V;
    const int v_tiles = (V + 15) / 16;
    const int head_jobs = (((v_tiles + G - 1) / G + R - 1) / R) * R;
    unsigned *abort_flag = a.b.abort_flag;

    auto layer_job = [&](int l, int j) -> const uint8_t * {
        const DLayer &Ly = a.m.layers[l];
        if (j == 0) return Ly.att_k.w16 + (size_t)g * kTileBytes;
        if (j == 1) return Ly.att_v.w16 + (size_t)g * kTileBytes;
        if (j == 2) return Ly.att_r.w16 + (size_t)g * kTileBytes;
        if (j == 3) return Ly.att_o.w16 + (size_t)g * kTileBytes;
        if (j == 4) return Ly.ffn_r.w16 + (size_t)g * kTileBytes;
        if (j <= 8) return Ly.ffn_k.w16 + (size_t)(g + G * (j - 5)) * kTileBytes;
        if (j <= 12) return Ly.ffn_v.w16 + ((size_t)g * 4 + (j - 9)) * kTileBytes;
        return nullptr;
    };
    auto head_job = [&](int hj) -> const uint8_t * {
        const int tile = g + G * hj;
        return (hj < head_jobs && tile < v_tiles) ? a.m.head.w16 + (size_t)tile * kTileBytes : nullptr;
    };
    auto flat_job = [&](int l, int j) -> const uint8_t * {   // j may run past the layer
        if (j == 13 || j == 14) j += R;     // padding jobs own no data: their slot goes to its next user
        if (j < JPL) return layer_job(l, j);
        if (l + 1 < L) return layer_job(l + 1, j - JPL);
        return head_job(j - JPL);
    };

    uint4 ring[R][KBW];
#pragma unroll
    for (int s = 0; s < R; ++s) load_slot<KBW>(ring[s], layer_job(0, s));

    int64_t tok = a.token[0];
    if (tok < 0) tok = 0;
    if (tok >= V) tok = V - 1;

    double x_own = 0.0;       // residual value of channel 16g + tid (threads 0..15)
    unsigned parity = 0;      // LDS double buffering of red/part

    for (int l = 0; l < L; ++l) {
        const DLayer &Ly = a.m.layers[l];
        double *sl = a.state + (size_t)l * 5 * C;
        const unsigned e_base = a.epoch0 + 4u * (unsigned)l;
        const int c_own = 16 * g + tid;     // meaningful for tid < 16

        // per-channel scalars the epilogues need; fetched early, off the critical path
        double td = 0, tf = 0, st_aa = 0, st_bb = 0, st_pp = 0;
        if (tid < 16) {
            td = Ly.time_decay[c_own]; tf = Ly.time_first[c_own];
            st_aa = sl[2 * (size_t)C + c_own]; st_bb = sl[3 * (size_t)C + c_own]; st_pp = sl[4 * (size_t)C + c_own];
        }

        // ===================== phase 1: att k, v, r ============================
        {
            double xv[KBW];
            if (l == 0) {
#pragma unroll
                for (int i = 0; i < KBW; ++i) xv[i] = (double)a.m.emb[(size_t)tok * C + tid + kDT * i];
                layernorm_wg<KBW>(xv, C, a.m.ln0_w, a.m.ln0_b, scr);     // opt.py:64
#pragma unroll
                for (int i = 0; i < KBW; ++i) {
                    const int c = tid + kDT * i;
                    if ((c >> 4) == g) own_x[c & 15] = xv[i];
                }
            } else {
                float xf[KBW];
                const bool ok = poll_words<KBW>(a.b.X, e_base, xf, abort_flag);
                if (__syncthreads_or(!ok)) { if (tid == 0) ASTORE(abort_flag, 1u); return; }
#pragma unroll
                for (int i = 0; i < KBW; ++i) xv[i] = (double)xf[i];
            }
            layernorm_wg<KBW>(xv, C, Ly.ln1_w, Ly.ln1_b, scr);           // block.py:58
            float xs[3][KBW];
            double zq[6] = {0, 0, 0, 0, 0, 0};                            // zp[3], qsum[3]
            float amax[3] = {0.f, 0.f, 0.f};
            const DQ *mats[3] = {&Ly.att_k, &Ly.att_v, &Ly.att_r};
#pragma unroll
            for (int i = 0; i < KBW; ++i) {
                const int c = tid + kDT * i;
                const double xy = xv[i];
                if ((c >> 4) == g) own_ln1[c & 15] = xy;
                const double sh = sl[c];                                   // block.py:61-64
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    const double mu = Ly.att_mix[(size_t)m * C + c];
                    const double mixed = xy * mu + sh * (1.0 - mu);       // block.py:67
                    xs[m][i] = (float)(mixed * (double)mats[m]->range[c]); // matmul.py:131
                    zq[m] += mixed * mats[m]->offset[c];
                    amax[m] = fmaxf(amax[m], fabsf(xs[m][i]));
                }
            }
            wg_max<3>(amax, reinterpret_cast<float *>(scr));
            double S[3], invS[3];
#pragma unroll
            for (int m = 0; m < 3; ++m) scale_from_amax(amax[m], S[m], invS[m]);
#pragma unroll
            for (int i = 0; i < KBW; ++i)
#pragma unroll
                for (int m = 0; m < 3; ++m)
                    zq[3 + m] += put_digits(dig + m * 4 * PS, PS, tid + kDT * i, xs[m][i], invS[m]);
            double *pp_ = part + parity * (kDW * 8);
            park_partials<6>(zq, pp_, 0);
            __syncthreads();

            v4i D[3];
#pragma unroll
            for (int j = 0; j < 3; ++j) {
                D[j] = v4i{0, 0, 0, 0};
                mfma_job<KBW>(ring[j % R], dig + j * 4 * PS, PS, 0, D[j]);
                load_slot<KBW>(ring[j % R], flat_job(l, j + R));
            }
            int *rd = red + parity * RED_INTS;
#pragma unroll
            for (int j = 0; j < 3; ++j) park_tile(rd, j, D[j]);
            __syncthreads();
            if (tid < 16) {
                double y[3];
#pragma unroll
                for (int j = 0; j < 3; ++j)
                    y[j] = finish_col(rd, j, tid, S[j], S[j] * sum_partials(pp_, 3 + j), sum_partials(pp_, j));
                const float r = sigmoid_f32((float)y[2]);                 // block.py:72
                float aa = (float)st_aa, bb = (float)st_bb;
                double pp = st_pp;
                const float wkv = wkv_step_f32(td, tf, (float)y[0], (float)y[1], aa, bb, pp);
                put_word(a.b.A + c_own, e_base + 1u, wkv * r);            // block.py:78
                sl[2 * (size_t)C + c_own] = (double)aa;
                sl[3 * (size_t)C + c_own] = (double)bb;
                sl[4 * (size_t)C + c_own] = pp;
                if (l == 0) x_own = own_x[tid];
            }
            parity ^= 1u;
        }

        // ===================== phase 2: att output =============================
        {
            float af[KBW];
            const bool ok = poll_words<KBW>(a.b.A, e_base + 1u, af, abort_flag);
            if (__syncthreads_or(!ok)) { if (tid == 0) ASTORE(abort_flag, 1u); return; }
            float xs[KBW];
            double zq[2] = {0, 0};
            float amax[1] = {0.f};
#pragma unroll
            for (int i = 0; i < KBW; ++i) {
                const int c = tid + kDT * i;
                const double v = (double)af[i];
                xs[i] = (float)(v * (double)Ly.att_o.range[c]);
                zq[0] += v * Ly.att_o.offset[c];
                amax[0] = fmaxf(amax[0], fabsf(xs[i]));
            }
            wg_max<1>(amax, reinterpret_cast<float *>(scr));
            double S, invS;
            scale_from_amax(amax[0], S, invS);
#pragma unroll
            for (int i = 0; i < KBW; ++i) zq[1] += put_digits(dig, PS, tid + kDT * i, xs[i], invS);
            double *pp_ = part + parity * (kDW * 8);
            park_partials<2>(zq, pp_, 0);
            __syncthreads();
            v4i D = {0, 0, 0, 0};
            mfma_job<KBW>(ring[3 % R], dig, PS, 0, D);
            load_slot<KBW>(ring[3 % R], flat_job(l, 3 + R));
            int *rd = red + parity * RED_INTS;
            park_tile(rd, 0, D);
            __syncthreads();
            if (tid < 16) {
                const double y = finish_col(rd, 0, tid, S, S * sum_partials(pp_, 1), sum_partials(pp_, 0));
                x_own = x_own + y;                                        // block.py:80
                put_word(a.b.X + c_own, e_base + 2u, (float)x_own);
                sl[c_own] = own_ln1[tid];                                 // block.py:63-64
            }
            parity ^= 1u;
        }

        // ===================== phase 3: ffn receptance + key ===================
        double rf_own = 0.0;
        {
            float xf[KBW];
            const bool ok = poll_words<KBW>(a.b.X, e_base + 2u, xf, abort_flag);
            if (__syncthreads_or(!ok)) { if (tid == 0) ASTORE(abort_flag, 1u); return; }
            double xv[KBW];
#pragma unroll
            for (int i = 0; i < KBW; ++i) xv[i] = (double)xf[i];
            layernorm_wg<KBW>(xv, C, Ly.ln2_w, Ly.ln2_b, scr);           // block.py:82
            float xs[2][KBW];
            double zq[4] = {0, 0, 0, 0};                                  // zp k, zp r, qsum k, qsum r
            float amax[2] = {0.f, 0.f};
            const DQ *mats[2] = {&Ly.ffn_k, &Ly.ffn_r};
#pragma unroll
            for (int i = 0; i < KBW; ++i) {
                const int c = tid + kDT * i;
                const double dd = xv[i];
                if ((c >> 4) == g) own_ln2[c & 15] = dd;
                const double sh = sl[(size_t)C + c];                      // block.py:84-88
#pragma unroll
                for (int m = 0; m < 2; ++m) {
                    const double mu = Ly.ffn_mix[(size_t)m * C + c];
                    const double mixed = dd * mu + sh * (1.0 - mu);      // block.py:91
                    xs[m][i] = (float)(mixed * (double)mats[m]->range[c]);
                    zq[m] += mixed * mats[m]->offset[c];
                    amax[m] = fmaxf(amax[m], fabsf(xs[m][i]));
                }
            }
            wg_max<2>(amax, reinterpret_cast<float *>(scr));
            double S[2], invS[2];
#pragma unroll
            for (int m = 0; m < 2; ++m) scale_from_amax(amax[m], S[m], invS[m]);
#pragma unroll
            for (int i = 0; i < KBW; ++i)
#pragma unroll
                for (int m = 0; m < 2; ++m)
                    zq[2 + m] += put_digits(dig + m * 4 * PS, PS, tid + kDT * i, xs[m][i], invS[m]);
            double *pp_ = part + parity * (kDW * 8);
            park_partials<4>(zq, pp_, 0);
            __syncthreads();
            v4i D[5];
#pragma unroll
            for (int jj = 0; jj < 5; ++jj) {
                const int j = 4 + jj;                                     // job 4: ffn_r ; 5..8: ffn_k tiles
                D[jj] = v4i{0, 0, 0, 0};
                mfma_job<KBW>(ring[j % R], dig + (jj == 0 ? 1 : 0) * 4 * PS, PS, 0, D[jj]);
                load_slot<KBW>(ring[j % R], flat_job(l, j + R));
            }
            int *rd = red + parity * RED_INTS;
#pragma unroll
            for (int jj = 0; jj < 5; ++jj) park_tile(rd, jj, D[jj]);
            __syncthreads();
            if (tid < 80) {
                const int jj = tid >> 4, n = tid & 15;
                const int m = jj == 0 ? 1 : 0;
                const double y = finish_col(rd, jj, n, S[m], S[m] * sum_partials(pp_, 2 + m), sum_partials(pp_, m));
                if (jj == 0) {
                    rf_own = (double)sigmoid_f32((float)y);              // block.py:95
                } else {
                    const double h = y > 0.0 ? y : 0.0;                  // block.py:97-98
                    put_word(a.b.H + 16 * (g + G * (jj - 1)) + n, e_base + 3u, (float)(h * h));
                }
            }
            parity ^= 1u;
        }

        // ===================== phase 4: ffn value ==============================
        {
            float hf[4 * KBW];
            double zq[2] = {0, 0};
            float amax[1] = {0.f};
            bool ok = true;
#pragma unroll
            for (int q = 0; q < 4; ++q) {          // a quarter (C words) at a time keeps the live set small
                float part_h[KBW];
                ok = poll_words<KBW>(a.b.H + (size_t)q * C, e_base + 3u, part_h, abort_flag) && ok;
#pragma unroll
                for (int i = 0; i < KBW; ++i) {
                    const int f = q * C + tid + kDT * i;
                    const double h = (double)part_h[i];
                    const float x = (float)(h * (double)Ly.ffn_v.range[f]);
                    zq[0] += h * Ly.ffn_v.offset[f];
                    amax[0] = fmaxf(amax[0], fabsf(x));
                    hf[q * KBW + i] = x;
                }
            }
            if (__syncthreads_or(!ok)) { if (tid == 0) ASTORE(abort_flag, 1u); return; }
            wg_max<1>(amax, reinterpret_cast<float *>(scr));
            double S, invS;
            scale_from_amax(amax[0], S, invS);
#pragma unroll
            for (int i = 0; i < 4 * KBW; ++i) zq[1] += put_digits(dig, PSF, tid + kDT * i, hf[i], invS);
            double *pp_ = part + parity * (kDW * 8);
            park_partials<2>(zq, pp_, 0);
            __syncthreads();
            v4i D = {0, 0, 0, 0};
#pragma unroll
            for (int kq = 0; kq < 4; ++kq) {
                const int j = 9 + kq;                                     // the four C-row quarters of the tile
                mfma_job<KBW>(ring[j % R], dig, PSF, kq * C, D);
                load_slot<KBW>(ring[j % R], flat_job(l, j + R));
            }
            int *rd = red + parity * RED_INTS;
            park_tile(rd, 0, D);
            __syncthreads();
            if (tid < 16) {
                const double y = finish_col(rd, 0, tid, S, S * sum_partials(pp_, 1), sum_partials(pp_, 0));
                x_own = y * rf_own + x_own;                               // block.py:100
                put_word(a.b.X + c_own, e_base + 4u, (float)x_own);
                sl[(size_t)C + c_own] = own_ln2[tid];                     // block.py:87-88
            }
            parity ^= 1u;
        }
    }

    // ========================= head (opt.py:71-73) ==============================
    {
        float xf[KBW];
        const bool ok = poll_words<KBW>(a.b.X, a.epoch0 + 4u * (unsigned)L, xf, abort_flag);
        if (__syncthreads_or(!ok)) { if (tid == 0) ASTORE(abort_flag, 1u); return; }
        double xv[KBW];
#pragma unroll
        for (int i = 0; i < KBW; ++i) xv[i] = (double)xf[i];
        layernorm_wg<KBW>(xv, C, a.m.lnout_w, a.m.lnout_b, scr);
        float xs[KBW];
        double zq[2] = {0, 0};
        float amax[1] = {0.f};
#pragma unroll
        for (int i = 0; i < KBW; ++i) {
            const int c = tid + kDT * i;
            xs[i] = (float)(xv[i] * (double)a.m.head.range[c]);
            zq[0] += xv[i] * a.m.head.offset[c];
            amax[0] = fmaxf(amax[0], fabsf(xs[i]));
        }
        wg_max<1>(amax, reinterpret_cast<float *>(scr));
        double S, invS;
        scale_from_amax(amax[0], S, invS);
#pragma unroll
        for (int i = 0; i < KBW; ++i) zq[1] += put_digits(dig, PS, tid + kDT * i, xs[i], invS);
        double *pp_ = part + parity * (kDW * 8);
        park_partials<2>(zq, pp_, 0);
        __syncthreads();
        const double zp = sum_partials(pp_, 0), qsumS = S * sum_partials(pp_, 1);
        unsigned rpar = parity;
        for (int h0 = 0; h0 < head_jobs; h0 += R) {
            v4i D[R];
#pragma unroll
            for (int s = 0; s < R; ++s) {
                D[s] = v4i{0, 0, 0, 0};
                if (head_job(h0 + s)) mfma_job<KBW>(ring[s], dig, PS, 0, D[s]);
                load_slot<KBW>(ring[s], head_job(h0 + s + R));
            }
            int *rd = red + rpar * RED_INTS;
#pragma unroll
            for (int s = 0; s < R; ++s) park_tile(rd, s, D[s]);
            __syncthreads();
            if (tid < 16 * R) {
                const int s = tid >> 4, n = tid & 15;
                const int v = 16 * (g + G * (h0 + s)) + n;
                if (h0 + s < head_jobs && v < V) a.logits[v] = finish_col(rd, s, n, S, qsumS, zp);
            }
            rpar ^= 1u;
        }
    }
}

// ---------------------------------------------------------------------------
template <int KBW>
static size_t decode_lds_bytes() {
    constexpr int C = KBW * kDT, F = 4 * C;
    constexpr int PS = C + 64, PSF = F + 64;
    constexpr int DIG_BYTES = (3 * 4 * PS > 4 * PSF) ? 3 * 4 * PS : 4 * PSF;
    return (size_t)DIG_BYTES + 2 * (kDW * kMaxJobsPerPhase * 16 * 4) * sizeof(int) +
           (2 * kDW * 8 + 4 * kDW + 48) * sizeof(double);
}

bool decode_supported(int64_t L, int64_t C, int64_t F, int64_t V) {
    if (L <= 0 || V <= 0 || F != 4 * C) return false;
    // one 16-column tile per workgroup, all workgroups resident: C/16 <= 256 CUs
    return C == 1024 || C == 2048 || C == 2560 || C == 4096;
}

unsigned decode_epochs_per_token(int64_t L) { return (unsigned)(4 * L + 1); }

template <int KBW>
static int launch_one(hipStream_t st, const DArgs &args) {
    const size_t lds = decode_lds_bytes<KBW>();
    static bool configured = false;
    if (!configured) {
        RWKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_kernel<KBW>),
                                           hipFuncAttributeMaxDynamicSharedMemorySize, (int)lds));
        configured = true;
    }
    hipLaunchKernelGGL(decode_kernel<KBW>, dim3(args.m.C / 16), dim3(kDT), lds, st, args);
    RWKV_CHECK_LAUNCH("decode_kernel");
    return RWKV_OK;
}

int decode_launch(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                  const int64_t *token, double *state, double *logits) {
    DArgs args;
    args.m = m; args.b = b; args.epoch0 = epoch0; args.token = token; args.state = state; args.logits = logits;
    switch (m.C) {
        case 1024: return launch_one<2>(st, args);
        case 2048: return launch_one<4>(st, args);
        case 2560: return launch_one<5>(st, args);
        case 4096: return launch_one<8>(st, args);
        default: return set_error(RWKV_ERR_SIZE, "decode kernel: n_embd %d not supported", m.C);
    }
}

}  // namespace rwkv
