// Many-row path of the FASTQUANT RWKV-4 forward pass: a prompt (T tokens of one
// sequence; reference agnostic/backends/opt.py:61-76 with T > 1,
// modules/matmul.py:56-57,86-94) or a batch (B independent sequences, one token
// each).  Rows are tokens; every matrix product is a GEMM on the matrix cores.
//
// Arithmetic.  Exactly the single-token kernel's: each row of
// xs = fp32(x * range) is rewritten as 32-bit fixed point q = round(xs / S),
// S a power of two chosen per row so that |q| <= 2^30, and split into four
// signed base-256 digits.  The digit rows (4 per token) are the A operand and
// the weights, stored as code - 128 in 1 KiB blocks of 16 columns x 64 rows
// ("M16"), the B operand of v_mfma_i32_16x16x64_i8.  Integer sums are exact and
// independent of tiling and of any split of the contraction, so a prompt
// processed here gives the same products as the same tokens fed one at a time.
// (The reference rounds this product to bfloat16, matmul.py:57; nothing here
// is rounded below float32 class.)
//
// Digit rows are stored in fragment order: for M-tile mt (tokens 4mt..4mt+3) and
// contraction block kb (rows 64kb..64kb+63) one 1 KiB fragment whose lane
// 16g + m holds bytes k = 64kb + 16g + i (i < 16) of digit row m = 4*(t % 4) + d;
// a wavefront loads a fragment with one coalesced 16-byte-per-lane request and
// hands it to the matrix instruction unchanged.
#include "rwkv_rows.h"

namespace rwkv {

namespace {

constexpr int kRT = 256;           // threads of the row kernels
constexpr int kRW = kRT / 64;

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ double wsum(double v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wmaxf(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v = fmaxf(v, __shfl_xor(v, off, 64));
    return v;
}

// Sum of N values per thread over the workgroup (fixed order), broadcast.
template <int N>
__device__ __forceinline__ void rsum(double (&v)[N], double *red /*[N*kRW]*/) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const double s = wsum(v[i]);
        if (lane == 0) red[i * kRW + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kRW; ++w) s += red[i * kRW + w];
        v[i] = s;
    }
    __syncthreads();
}

// ---------------------------------------------------------------------------
// x[t] = ln0(emb[token[t]])          (emb.py:9, opt.py:63-64)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kRT)
rows_embed_kernel(const int64_t *__restrict__ tokens, int V, int C, const float *__restrict__ emb,
                  const double *__restrict__ w, const double *__restrict__ b, double *__restrict__ x) {
    __shared__ double red[2 * kRW];
    const int t = blockIdx.x;
    int64_t tok = tokens[t];
    if (tok < 0) tok = 0;
    if (tok >= V) tok = V - 1;
    const float *e = emb + (size_t)tok * C;
    double s[1] = {0.0};
    for (int c = threadIdx.x; c < C; c += kRT) s[0] += (double)e[c];
    rsum<1>(s, red);
    const double mean = s[0] / (double)C;
    double q[1] = {0.0};
    for (int c = threadIdx.x; c < C; c += kRT) { const double d = (double)e[c] - mean; q[0] += d * d; }
    rsum<1>(q, red);
    const double sd = sqrt(q[0] / (double)C + 1e-5);
    for (int c = threadIdx.x; c < C; c += kRT) x[(size_t)t * C + c] = w[c] * (((double)e[c] - mean) / sd) + b[c];
}

// ---------------------------------------------------------------------------
// Fixed-point digits of four consecutive values of a row (columns c0..c0+3 of token t), written into
// the row's fragments; returns the sum of the four fixed-point values.
// ---------------------------------------------------------------------------
__device__ __forceinline__ double emit_quad(const float (&x4)[4], double invS, int c0, int t, int KB,
                                            signed char *dig) {
    // q = sum_k d_k 256^k with signed digits d_k in [-128, 127]  <=>  q + 0x80808080 has the unsigned bytes
    // d_k + 128, and b - 128 is b ^ 0x80 as a signed byte: two instructions give all four digits of a value.
    unsigned u[4];
    double qsum = 0.0;
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int q = __double2int_rn((double)x4[i] * invS);
        qsum += (double)q;
        u[i] = ((unsigned)q + 0x80808080u) ^ 0x80808080u;
    }
    // 4 x 4 byte transpose: one dword per digit plane, most significant first
    const unsigned x0 = __builtin_amdgcn_perm(u[1], u[0], 0x05010400u), x1 = __builtin_amdgcn_perm(u[1], u[0], 0x07030602u);
    const unsigned y0 = __builtin_amdgcn_perm(u[3], u[2], 0x05010400u), y1 = __builtin_amdgcn_perm(u[3], u[2], 0x07030602u);
    const unsigned pl[4] = {__builtin_amdgcn_perm(y1, x1, 0x07060302u), __builtin_amdgcn_perm(y1, x1, 0x05040100u),
                            __builtin_amdgcn_perm(y0, x0, 0x07060302u), __builtin_amdgcn_perm(y0, x0, 0x05040100u)};
    const int mt = t >> 2, m0 = (t & 3) * 4;
    const int kb = c0 >> 6, g = (c0 & 63) >> 4, j = (c0 & 15) >> 2;
    // The four lanes j = 0..3 that hold the 16 channels of one fragment slot transpose their 4 x 4 dwords
    // (two exchanges, with the neighbour and with the lane two further): lane j ends up with digit plane j of all 16
    // channels and writes it with ONE 16-byte store; the four lanes together fill a whole 64-byte line.  (Four
    // 4-byte stores per lane into four different lines cost the quantisers a third of their time.)  Callers
    // guarantee whole groups of four lanes: c0 = 4 * (a multiple-of-4-aligned lane index), widths multiples of 16.
    unsigned a4[4] = {pl[0], pl[1], pl[2], pl[3]};
    {
        const bool odd = j & 1;
        const unsigned s0 = odd ? a4[0] : a4[1], s1 = odd ? a4[2] : a4[3];
        const unsigned r0 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)s0, 0xB1, 0xf, 0xf, false);
        const unsigned r1 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)s1, 0xB1, 0xf, 0xf, false);
        if (odd) { a4[0] = r0; a4[2] = r1; } else { a4[1] = r0; a4[3] = r1; }
        const bool hi = j & 2;
        const unsigned t0 = hi ? a4[0] : a4[2], t1 = hi ? a4[1] : a4[3];
        const unsigned q0 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)t0, 0x4E, 0xf, 0xf, false);
        const unsigned q1 = (unsigned)__builtin_amdgcn_update_dpp(0, (int)t1, 0x4E, 0xf, 0xf, false);
        if (hi) { a4[0] = q0; a4[1] = q1; } else { a4[2] = q0; a4[3] = q1; }
    }
    signed char *slot = dig + ((size_t)mt * KB + kb) * 1024 + (16 * g + m0 + j) * 16;
    *reinterpret_cast<uint4 *>(slot) = make_uint4(a4[0], a4[1], a4[2], a4[3]);
    return qsum;
}

// Power-of-two scale of a row whose largest |xs| is amax: |xs / S| <= 2^30.
__device__ __forceinline__ void row_scale(float amax, double &S, double &invS) {
    S = 0.0; invS = 0.0;
    if (amax > 0.f && amax < INFINITY) {
        int e;
        frexpf(amax, &e);                  // amax = f * 2^e, f in [0.5, 1)  =>  |xs| < 2^e
        S = ldexp(1.0, e - 30);
        invS = ldexp(1.0, 30 - e);
    }
}

// ---------------------------------------------------------------------------
// LayerNorm + token shift + time mix + row quantiser      (layernorm.py:15-20, block.py:58-67,82-91,
// matmul.py:59-62,131-133)
//   xy = ln(x[t]);  prev = sequence ? (t == 0 ? prev0 : ln(x[t-1])) : prev0[t];
//   mix_m[t] = xy * mu_m + prev * (1 - mu_m), quantised for matrix m; the newest xy becomes the shift state.
// NM == 0: LayerNorm only, one output (the head's ln_out).
// One workgroup per row; a thread keeps its NSEG groups of four channels in registers from the one
// read of x to the digits, so the mixed rows never travel through memory.
// ---------------------------------------------------------------------------
// Element (t, j) of a product handed on unfinished: the slices added up (integers: exact in any order), then
// y = S_t * tot + 128 * S_t * sum q_t + zp_t as in rows_finish_kernel.
__device__ __forceinline__ double deferred_y(const RowsDeferred &d, int t, long long tot) {
    const double S = d.S[t];
    return S * (double)tot + 128.0 * (S * d.qs[t]) + d.zp[t];
}
// The slices are requested together, without a branch (always kRowsDeferSlices of them: one past the last reads
// slice 0 again and is not counted): a loop over a run-time count would wait for every slice before asking for the
// next, and a branch would keep the loads of a thread's channel groups apart.
__device__ __forceinline__ long long slices_sum1(const long long *tp, size_t slice, int slices) {
    long long u[kRowsDeferSlices], tot = 0;
#pragma unroll
    for (int z = 0; z < kRowsDeferSlices; ++z) u[z] = tp[(size_t)(z < slices ? z : 0) * slice];
#pragma unroll
    for (int z = 0; z < kRowsDeferSlices; ++z) tot += z < slices ? u[z] : 0;
    return tot;
}
__device__ __forceinline__ void slices_sum4(const long long *tp, size_t slice, int slices, long long (&tot)[4]) {
    longlong2 u[kRowsDeferSlices][2];
#pragma unroll
    for (int z = 0; z < kRowsDeferSlices; ++z) {
        const long long *q = tp + (size_t)(z < slices ? z : 0) * slice;
        u[z][0] = *reinterpret_cast<const longlong2 *>(q); u[z][1] = *reinterpret_cast<const longlong2 *>(q + 2);
    }
#pragma unroll
    for (int z = 0; z < kRowsDeferSlices; ++z) {
        const bool on = z < slices;
        tot[0] += on ? u[z][0].x : 0; tot[1] += on ? u[z][0].y : 0; tot[2] += on ? u[z][1].x : 0; tot[3] += on ? u[z][1].y : 0;
    }
}
__device__ __forceinline__ double deferred_value(const RowsDeferred &d, int t, int j) {
    return deferred_y(d, t, slices_sum1(d.tot + (size_t)t * d.ldd + j, d.slice, d.slices));
}

struct LnQuantArgs {
    int C, R, sequence;
    const double *x;            // [R, C]
    RowsDeferred add;           // batch rows, 512 threads per row: x += this product first, stored to x_rw (tot null: none)
    double *x_rw;
    const double *ln_w, *ln_b;  // [C]
    const double *mu;           // [NM, C]
    const double *prev0;        // sequence: [C]; batch: row t at prev0 + t * prev_stride
    double *shift_dst;          // sequence: [C] (written by row R-1); batch: row t at shift_dst + t * prev_stride
    int64_t prev_stride;
    const float *range[3];      // per output: the matrix's per-input-channel range / offset
    const double *offset[3];
    signed char *dig[3];        // per output: fragments [ceil(R/4)][C/64][1024] and the row constants
    double *S[3], *qs[3], *zp[3];
};

constexpr int kLnMaxThreads = 512;      // the LayerNorm kernel runs 512 threads per row for few rows, 256 for many

// Sum of N values per thread over the kLW wavefronts of the workgroup (fixed order), broadcast.
template <int N, int kLW>
__device__ __forceinline__ void lsum(double (&v)[N], double *red /*[N*kLW]*/) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const double s = wsum(v[i]);
        if (lane == 0) red[i * kLW + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kLW; ++w) s += red[i * kLW + w];
        v[i] = s;
    }
    __syncthreads();
}

template <int NM, int NSEG, int kLT>
__global__ void __launch_bounds__(kLT) rows_ln_mix_quant_kernel(const LnQuantArgs a) {
#include "rwkv_rows_ln_body.inc"
}
// The same for so few rows that at most two workgroups share a compute unit: twice the registers, so that the
// parameter vectors of all of a thread's channels can be on their way at once instead of one group after the other.
template <int NM, int NSEG, int kLT>
__global__ void __launch_bounds__(kLT) __attribute__((amdgpu_waves_per_eu(1, 2))) rows_ln_mix_quant_few_kernel(const LnQuantArgs a) {
#include "rwkv_rows_ln_body.inc"
}

// ---------------------------------------------------------------------------
// Row quantiser: xs = fp32(v * range), S from the row's max |xs|, digits in
// fragment order, zero-point term sum v * offset and sum q   (matmul.py:59-62,131-133).
// ---------------------------------------------------------------------------
struct QuantArgs {
    int K;                      // contraction length, multiple of 64
    const void *in;             // [R, K] float64, or float32 (the kernels' TIn): what the WKV kernels and the relu^2 tail write
    const float *range;         // [K]
    const double *offset;       // [K]
    signed char *dig;           // fragments [ceil(R/4)][K/64][1024]
    double *S, *qs, *zp;        // [R]
};

// Two / four consecutive values of a float64 or float32 row as float64.
__device__ __forceinline__ double2 row_ld2(const double *p) { return *reinterpret_cast<const double2 *>(p); }
__device__ __forceinline__ double2 row_ld2(const float *p) { const float2 f = *reinterpret_cast<const float2 *>(p); return make_double2((double)f.x, (double)f.y); }
__device__ __forceinline__ void row_ld4(const double *p, double2 &a, double2 &b) { a = row_ld2(p); b = row_ld2(p + 2); }
__device__ __forceinline__ void row_ld4(const float *p, double2 &a, double2 &b) {
    const float4 f = *reinterpret_cast<const float4 *>(p);
    a = make_double2((double)f.x, (double)f.y); b = make_double2((double)f.z, (double)f.w);
}

// kQuantSeg: 16-element segments a thread keeps in registers (rows up to 16 * kRT * kQuantSeg long in one
// read): 3 covers 12288 with registers to spare for four workgroups per compute unit, 5 covers 20480.
template <int kQuantSeg, typename TIn>
__global__ void __launch_bounds__(kRT) rows_quant_kernel(const QuantArgs a) {
    __shared__ double red[2 * kRW];
    __shared__ float redf[kRW];
    const int t = blockIdx.x, K = a.K;
    const TIn *row = static_cast<const TIn *>(a.in) + (size_t)t * K;
    // The thread that will write a 16-element group of digits reads it once: xs stays in registers
    // between the pass that finds the row's scale and the pass that forms the digits (longer rows
    // fall back to a second read).
    float xs[kQuantSeg][16];
    const bool fits = K <= kQuantSeg * 16 * kRT;
    float amax = 0.f;
    double z[1] = {0.0};
    if (fits) {
#pragma unroll
        for (int s = 0; s < kQuantSeg; ++s) {
            const int c0 = (threadIdx.x + s * kRT) * 16;
            if (c0 < K) {
#pragma unroll
                for (int i = 0; i < 16; i += 2) {
                    const double2 v = row_ld2(row + c0 + i);
                    const float2 r = *reinterpret_cast<const float2 *>(a.range + c0 + i);
                    const double2 o = *reinterpret_cast<const double2 *>(a.offset + c0 + i);
                    xs[s][i] = (float)(v.x * (double)r.x);
                    xs[s][i + 1] = (float)(v.y * (double)r.y);
                    amax = fmaxf(amax, fmaxf(fabsf(xs[s][i]), fabsf(xs[s][i + 1])));
                    z[0] += v.x * o.x;
                    z[0] += v.y * o.y;
                }
            }
        }
    } else {
        for (int c = threadIdx.x; c < K; c += kRT) {
            const double v = (double)row[c];
            amax = fmaxf(amax, fabsf((float)(v * (double)a.range[c])));
            z[0] += v * a.offset[c];
        }
    }
    amax = wmaxf(amax);
    if ((threadIdx.x & 63) == 0) redf[threadIdx.x >> 6] = amax;
    rsum<1>(z, red);                       // (its barriers also publish redf)
    amax = redf[0];
#pragma unroll
    for (int w = 1; w < kRW; ++w) amax = fmaxf(amax, redf[w]);
    double S, invS;
    row_scale(amax, S, invS);
    const int KB = K >> 6;
    const int mt = t >> 2, m0 = (t & 3) * 4;
    double qsum[1] = {0.0};
    auto emit = [&](int c0, const float (&x16)[16]) {
        unsigned pl[4][4];
#pragma unroll
        for (int d = 0; d < 4; ++d)
#pragma unroll
            for (int j = 0; j < 4; ++j) pl[d][j] = 0u;
#pragma unroll
        for (int i = 0; i < 16; ++i) {
            int q = __double2int_rn((double)x16[i] * invS);
            qsum[0] += (double)q;
            const int d3 = (int)(signed char)(q & 0xff); q = (q - d3) >> 8;
            const int d2 = (int)(signed char)(q & 0xff); q = (q - d2) >> 8;
            const int d1 = (int)(signed char)(q & 0xff); q = (q - d1) >> 8;
            const int sh = 8 * (i & 3);
            pl[0][i >> 2] |= (unsigned)(q & 0xff) << sh;
            pl[1][i >> 2] |= (unsigned)(d1 & 0xff) << sh;
            pl[2][i >> 2] |= (unsigned)(d2 & 0xff) << sh;
            pl[3][i >> 2] |= (unsigned)(d3 & 0xff) << sh;
        }
        const int kb = c0 >> 6, g = (c0 & 63) >> 4;
        signed char *frag = a.dig + ((size_t)mt * KB + kb) * 1024;
#pragma unroll
        for (int d = 0; d < 4; ++d)
            *reinterpret_cast<uint4 *>(frag + (16 * g + m0 + d) * 16) = make_uint4(pl[d][0], pl[d][1], pl[d][2], pl[d][3]);
    };
    if (fits) {
#pragma unroll
        for (int s = 0; s < kQuantSeg; ++s) {
            const int c0 = (threadIdx.x + s * kRT) * 16;
            if (c0 < K) emit(c0, xs[s]);
        }
    } else {
        for (int c0 = threadIdx.x * 16; c0 < K; c0 += kRT * 16) {
            float x16[16];
#pragma unroll
            for (int i = 0; i < 16; ++i) x16[i] = (float)((double)row[c0 + i] * (double)a.range[c0 + i]);
            emit(c0, x16);
        }
    }
    rsum<1>(qsum, red);
    if (threadIdx.x == 0) { a.S[t] = S; a.qs[t] = qsum[0]; a.zp[t] = z[0]; }
}

// The same quantiser with a thread owning groups of four values (NSEG of them, 4 * kRT * NSEG values per row in
// one read): every thread of the workgroup has work whatever the row length, and few registers are held.
template <int NSEG, typename TIn>
__global__ void __launch_bounds__(kRT) rows_quant4_kernel(const QuantArgs a) {
    __shared__ double red[2 * kRW];
    __shared__ float redf[kRW];
    const int t = blockIdx.x, K = a.K, tid = threadIdx.x;
    const TIn *row = static_cast<const TIn *>(a.in) + (size_t)t * K;
    float xs[NSEG][4];
    float amax = 0.f;
    double z[1] = {0.0};
#pragma unroll
    for (int g = 0; g < NSEG; ++g) {
        const int c0 = 4 * (tid + g * kRT);
        if (c0 < K) {
            double2 v0, v1;
            row_ld4(row + c0, v0, v1);
            const float4 r = *reinterpret_cast<const float4 *>(a.range + c0);
            const double2 o0 = *reinterpret_cast<const double2 *>(a.offset + c0), o1 = *reinterpret_cast<const double2 *>(a.offset + c0 + 2);
            xs[g][0] = (float)(v0.x * (double)r.x); xs[g][1] = (float)(v0.y * (double)r.y);
            xs[g][2] = (float)(v1.x * (double)r.z); xs[g][3] = (float)(v1.y * (double)r.w);
            amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xs[g][0]), fabsf(xs[g][1]))), fmaxf(fabsf(xs[g][2]), fabsf(xs[g][3])));
            z[0] += v0.x * o0.x; z[0] += v0.y * o0.y; z[0] += v1.x * o1.x; z[0] += v1.y * o1.y;
        }
    }
    amax = wmaxf(amax);
    if ((tid & 63) == 0) redf[tid >> 6] = amax;
    rsum<1>(z, red);                       // (its barriers also publish redf)
    amax = redf[0];
#pragma unroll
    for (int w = 1; w < kRW; ++w) amax = fmaxf(amax, redf[w]);
    double S, invS;
    row_scale(amax, S, invS);
    const int KB = K >> 6;
    double qsum[1] = {0.0};
#pragma unroll
    for (int g = 0; g < NSEG; ++g) {
        const int c0 = 4 * (tid + g * kRT);
        if (c0 < K) qsum[0] += emit_quad(xs[g], invS, c0, t, KB, a.dig);
    }
    rsum<1>(qsum, red);
    if (tid == 0) { a.S[t] = S; a.qs[t] = qsum[0]; a.zp[t] = z[0]; }
}

// A handful of long rows (one token of a wide ffn): one workgroup per row would pull the whole row and its
// range / offset vectors through a single compute unit.  Two launches instead, G workgroups per row: the first
// leaves each part's max |xs| and zero-point share in `part`, the second turns them into the row's scale and
// writes the digits of its part.  The sum of the fixed-point values is added up with atomics: integers below
// 2^53, exact in any order.
constexpr int kQuantPartSeg = 3;        // groups of four values per thread: parts of up to 3072 values

struct QuantPartArgs {
    QuantArgs q;
    int G, quads_per_part;
    double *part;               // [R][G][2]: max |xs|, zero-point share
};

template <bool EMIT, typename TIn>
__global__ void __launch_bounds__(kRT) rows_quant_part_kernel(const QuantPartArgs a) {
    __shared__ double red[2 * kRW];
    __shared__ float redf[kRW];
    const int g = blockIdx.x, t = blockIdx.y, K = a.q.K, tid = threadIdx.x;
    const TIn *row = static_cast<const TIn *>(a.q.in) + (size_t)t * K;
    const int q0 = g * a.quads_per_part, q1 = min(q0 + a.quads_per_part, K >> 2);
    float xs[kQuantPartSeg][4];
    float amax = 0.f;
    double z[1] = {0.0};
#pragma unroll
    for (int s = 0; s < kQuantPartSeg; ++s) {
        const int qi = q0 + tid + s * kRT;
        if (qi < q1) {
            const int c0 = 4 * qi;
            double2 v0, v1;
            row_ld4(row + c0, v0, v1);
            const float4 r = *reinterpret_cast<const float4 *>(a.q.range + c0);
            xs[s][0] = (float)(v0.x * (double)r.x); xs[s][1] = (float)(v0.y * (double)r.y);
            xs[s][2] = (float)(v1.x * (double)r.z); xs[s][3] = (float)(v1.y * (double)r.w);
            if (!EMIT) {
                const double2 o0 = *reinterpret_cast<const double2 *>(a.q.offset + c0), o1 = *reinterpret_cast<const double2 *>(a.q.offset + c0 + 2);
                amax = fmaxf(fmaxf(amax, fmaxf(fabsf(xs[s][0]), fabsf(xs[s][1]))), fmaxf(fabsf(xs[s][2]), fabsf(xs[s][3])));
                z[0] += v0.x * o0.x; z[0] += v0.y * o0.y; z[0] += v1.x * o1.x; z[0] += v1.y * o1.y;
            }
        }
    }
    double *part = a.part + (size_t)t * a.G * 2;
    if (!EMIT) {
        amax = wmaxf(amax);
        if ((tid & 63) == 0) redf[tid >> 6] = amax;
        rsum<1>(z, red);                   // (its barriers also publish redf)
        if (tid == 0) {
            amax = redf[0];
#pragma unroll
            for (int w = 1; w < kRW; ++w) amax = fmaxf(amax, redf[w]);
            part[2 * g] = (double)amax; part[2 * g + 1] = z[0];
            if (g == 0) a.q.qs[t] = 0.0;
        }
        return;
    }
    float am = 0.f;
    double zp = 0.0;
    for (int i = 0; i < a.G; ++i) { am = fmaxf(am, (float)part[2 * i]); zp += part[2 * i + 1]; }     // fixed order
    double S, invS;
    row_scale(am, S, invS);
    const int KB = K >> 6;
    double qsum[1] = {0.0};
#pragma unroll
    for (int s = 0; s < kQuantPartSeg; ++s) {
        const int qi = q0 + tid + s * kRT;
        if (qi < q1) qsum[0] += emit_quad(xs[s], invS, 4 * qi, t, KB, a.q.dig);
    }
    rsum<1>(qsum, red);
    if (tid == 0) {
        atomicAdd(a.q.qs + t, qsum[0]);
        if (g == 0) { a.q.S[t] = S; a.q.zp[t] = zp; }
    }
}

// ---------------------------------------------------------------------------
// GEMM: tot[t, j] = sum_k q[t, k] * (code[k, j] - 128), exact in int64.
// Workgroup = 8 wavefronts = 64 tokens x 128 (or 160) columns; wavefront (wm, wn) holds
// 4 M-tiles x 4 (or 5) N-tiles of accumulators; variants for at most 32 and at most 8 rows
// follow.  With few rows the contraction is split over several workgroups; each split writes
// its own slice of integer totals and the tail kernel adds the slices (integer sums: exact in
// any order).
//
// Launch order.  Workgroups are handed to the 8 XCDs round robin, and each XCD has its own L2.  The
// grid is 1-D and workgroup i works for XCD i % 8 on that XCD's own row blocks (row block r belongs
// to XCD r % 8), walking through the column blocks with the row blocks innermost: the digit
// fragments of an XCD's rows (a few hundred KB) stay in its L2 for the whole product, and a weight
// block fetched for one row block is reused by the next.  Without this every XCD pulls every digit
// fragment through the fabric once per column block.  With fewer row blocks than XCDs (a batch of
// single tokens) the column blocks are dealt out to the XCDs instead.
// ---------------------------------------------------------------------------
constexpr int kXcds = 8;
struct GemmArgs {
    // up to kRowsMaxProducts products of one shape share a launch (the grid's split index also counts products)
    const signed char *dig[kRowsMaxProducts];   // fragments [MT][KB][1024]
    const uint8_t *w16[kRowsMaxProducts];       // blocks [NT][KB][1024]
    const double *S[kRowsMaxProducts], *qs[kRowsMaxProducts], *zp[kRowsMaxProducts];
    double *out[kRowsMaxProducts];
    long long *tot;             // [products][splits][4*MT][ldd]
    int MT, NT, KB, ldd, kb_per_split, split;     // split > 1: the contraction is split, each part writes its slice of tot
    size_t slice;                   // elements between the slices of tot
    int gx, gy, gz, per_xcd, by_rows;   // logical grid (column blocks, row blocks, splits x products) behind the 1-D launch
    // when the contraction is not split the tail of the product is applied here (see rows_finish_kernel)
    int tail, R, N;                 // tail < 0: totals only
    const float *gate;
};

constexpr int kGemmNT = 8, kGemmWideNT = 10;     // N-tiles per workgroup (two wavefronts side by side)
constexpr int kWideRing = 4;                     // LDS buffers of the 64 x 160 variant

// Workgroup barrier that orders LDS traffic only.  __syncthreads() also waits for every global load
// the wavefront has in flight, which would drain the prefetched contraction blocks at every step.
__device__ __forceinline__ void lds_barrier() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); }

// 16 bytes per lane from global memory straight into LDS at lds_byte_offset + 16 * lane (the offset is uniform
// for the wavefront and travels in M0; one wait state between writing M0 and the load that reads it).
__device__ __forceinline__ void dma16(const v4i *g, unsigned lds_byte_offset) {
    asm volatile("s_mov_b32 m0, %1\n\ts_nop 0\n\tglobal_load_lds_dwordx4 %0, off" :: "v"(g), "s"(lds_byte_offset) : "memory");
}

// Accumulators of one wavefront (GM M-tiles x GN N-tiles from (mt0, nt0)) to totals or, when the
// contraction is not split, straight through the product's tail.
template <int GM, int GN>
__device__ __forceinline__ void gemm_epilogue(const GemmArgs &a, const v4i (&acc)[GM][GN], int mt0, int nt0, int mat,
                                              int bz, int lane) {
    // lane 16g + n, register i  <->  digit i of token 4*mt + g, column 16*nt + n
    const int g = lane >> 4, n = lane & 15;
    const double *Sv = mat == 0 ? a.S[0] : mat == 1 ? a.S[1] : a.S[2];
    const double *qsv = mat == 0 ? a.qs[0] : mat == 1 ? a.qs[1] : a.qs[2];
    const double *zpv = mat == 0 ? a.zp[0] : mat == 1 ? a.zp[1] : a.zp[2];
    double *outv = mat == 0 ? a.out[0] : mat == 1 ? a.out[1] : a.out[2];
    long long *totv = a.tot + (size_t)(mat * a.split + bz) * a.slice;      // this part's slice
#pragma unroll
    for (int i = 0; i < GM; ++i) {
        if (mt0 + i >= a.MT) continue;
        const int t = 4 * (mt0 + i) + g;
        double S = 0.0, add = 0.0;
        if (a.tail >= 0 && t < a.R) { S = Sv[t]; add = 128.0 * (S * qsv[t]) + zpv[t]; }
#pragma unroll
        for (int j = 0; j < GN; ++j) {
            if (nt0 + j >= a.NT) continue;
            const v4i d = acc[i][j];
            const long long tot = ((((long long)d.x * 256 + d.y) * 256 + d.z) * 256) + d.w;
            const int col = 16 * (nt0 + j) + n;
            if (a.tail >= 0) {
                if (t < a.R && col < a.N) {
                    const double y = S * (double)tot + add;
                    double *o = outv + (size_t)t * a.N + col;
                    if (a.tail == ROW_STORE) *o = y;
                    else if (a.tail == ROW_STORE_F32) reinterpret_cast<float *>(outv)[(size_t)t * a.N + col] = (float)y;
                    else if (a.tail == ROW_RELU2) {                                                                 // block.py:97, kept as float32 (see RowTail)
                        const double r = y > 0.0 ? y : 0.0;
                        reinterpret_cast<float *>(outv)[(size_t)t * a.N + col] = (float)(r * r);
                    }
                    else if (a.tail == ROW_ADD) *o += y;                                                            // block.py:80
                    else *o += y * (double)sigmoid_f32(a.gate[(size_t)t * a.N + col]);       // block.py:95-100; the gate in float32 as in the single-token kernel
                }
                continue;
            }
            totv[(size_t)t * a.ldd + col] = tot;
        }
    }
}

// One workgroup of the product: 64 tokens x 32*GN columns, 2*WM wavefronts as WM x 2, each 16/WM M-tiles x GN
// N-tiles, RING LDS buffers.  <4, 4, 3> is the general shape (8 wavefronts of 4 x 4 tiles, two workgroups per
// compute unit); <5, 4, 4> (4 x 5 tiles, one workgroup per compute unit) is used where it turns a grid of 1.25
// workgroups per compute unit into exactly one (2560 columns: 16 column blocks instead of 20).
template <int GN, int WM, int RING>
__device__ __forceinline__ void gemm8_body(const GemmArgs a) {
    // Both operands of a contraction block are fetched once per workgroup into LDS and read from there by
    // the wavefronts that need each fragment (one barrier per block).
    constexpr int kGN = GN, kNT = 2 * GN, kGM = 16 / WM, kNW = 2 * WM;
    constexpr int kGemmFrags = 16 + kNT;                // fragments of one contraction block: 16 M-tiles of digits, kNT N-tiles of weights
    constexpr int kGemmLoads = (kGemmFrags + kNW - 1) / kNW;    // per thread and contraction block (wave w fetches fragments w, w + kNW, ...)
    constexpr int kSlots = kNW * kGemmLoads, kGemmRing = RING;
    __shared__ v4i frag[kGemmRing][kSlots][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int wm = wave % WM, wn = wave / WM;
    const int xcd = blockIdx.x % kXcds;
    int item = blockIdx.x / kXcds, bx, by, bz;
    if (a.by_rows) {                                    // (split, column block, row slot) of this XCD, row slot fastest
        const int rslot = item % a.per_xcd; item /= a.per_xcd;
        bx = item % a.gx; bz = item / a.gx;
        by = xcd + kXcds * rslot;
    } else {                                            // few row blocks: the XCDs share out the column blocks instead
        const int cslot = item % a.per_xcd; item /= a.per_xcd;
        by = item % a.gy; bz = item / a.gy;
        bx = xcd + kXcds * cslot;
    }
    if (by >= a.gy || bx >= a.gx || bz >= a.gz) return;
    const int mat = bz / a.split;                       // which product; then which part of its contraction
    bz -= mat * a.split;
    const signed char *dig = mat == 0 ? a.dig[0] : mat == 1 ? a.dig[1] : a.dig[2];
    const uint8_t *w16 = mat == 0 ? a.w16[0] : mat == 1 ? a.w16[1] : a.w16[2];
    const int mt0 = by * 16 + wm * kGM, nt0 = bx * kNT + wn * kGN;
    const int kb0 = bz * a.kb_per_split;
    int kb1 = kb0 + a.kb_per_split;
    if (kb1 > a.KB) kb1 = a.KB;
    if (kb0 >= kb1) return;                             // (uniform for the workgroup)
    const int nk = kb1 - kb0;

    const v4i *src[kGemmLoads];
#pragma unroll
    for (int i = 0; i < kGemmLoads; ++i) {
        const int f = wave + kNW * i;                   // fragment this thread helps to fetch
        if (f < 16) {
            int mt = by * 16 + f;
            if (mt >= a.MT) mt = a.MT - 1;              // clamped: loads stay unconditional, results are dropped
            src[i] = reinterpret_cast<const v4i *>(dig + ((size_t)mt * a.KB + kb0) * 1024) + lane;
        } else {
            int nt = bx * kNT + (f - 16 < kNT ? f - 16 : 0);   // (slots past the last fragment: a copy nobody reads)
            if (nt >= a.NT) nt = a.NT - 1;
            src[i] = reinterpret_cast<const v4i *>(w16 + ((size_t)nt * a.KB + kb0) * 1024) + lane;
        }
    }
    v4i acc[kGM][kGN];
#pragma unroll
    for (int i = 0; i < kGM; ++i)
#pragma unroll
        for (int j = 0; j < kGN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    // Contraction blocks travel from memory straight into a ring of kGemmRing LDS buffers (direct-to-LDS
    // loads: no registers, no LDS write instructions); block K + kGemmRing - 1 is requested in step K, into the
    // buffer block K - 1 has just left.  The compiler does not see these loads, so the waits are written here:
    // before the barrier of step K a wavefront waits until only the requests of the blocks after K are still out.
    const unsigned lds0 = (unsigned)(size_t)&frag[0][0][0] + (unsigned)wave * 1024u;
#define RWKV_GEMM_DMA(SLOT, K)                                                                       \
    do {                                                                                             \
        const size_t o_ = (size_t)((K) < nk ? (K) : nk - 1) * 64; /* past the end: the last block again (unused) */ \
        _Pragma("unroll") for (int i = 0; i < kGemmLoads; ++i)                                       \
            dma16(src[i] + o_, lds0 + (unsigned)(((SLOT) * kSlots + kNW * i) * 1024));               \
    } while (0)
#define RWKV_GEMM_STEP(SLOT, K)                                                                      \
    {                                                                                                \
        asm volatile("s_waitcnt vmcnt(%0)\n\ts_waitcnt lgkmcnt(0)\n\ts_barrier" :: "n"((kGemmRing - 2) * kGemmLoads) : "memory"); \
        v4i Bv_[kGN];                                                                                \
        _Pragma("unroll") for (int j = 0; j < kGN; ++j) {                                            \
            Bv_[j] = frag[SLOT][16 + wn * kGN + j][lane];                                            \
        }                                                                                            \
        v4i Av_ = frag[SLOT][wm * kGM][lane], Aw_ = frag[SLOT][wm * kGM + 1][lane];                  \
        /* the next block is requested after this step's first LDS reads are on their way, and the wavefront */ \
        /* holds the higher issue priority while it has matrix instructions to issue (measured: -3 %)        */ \
        RWKV_GEMM_DMA(((SLOT) + kGemmRing - 1) % kGemmRing, (K) + kGemmRing - 1);                    \
        __builtin_amdgcn_s_setprio(1);                                                               \
        _Pragma("unroll") for (int i = 0; i < kGM; ++i) {                                            \
            const v4i An_ = frag[SLOT][wm * kGM + (i + 2 < kGM ? i + 2 : i)][lane];   /* two groups ahead */ \
            _Pragma("unroll") for (int j = 0; j < kGN; ++j)                                          \
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Av_, Bv_[j], acc[i][j], 0, 0, 0);  \
            Av_ = Aw_; Aw_ = An_;                                                                    \
        }                                                                                            \
        __builtin_amdgcn_s_setprio(0);                                                               \
        __builtin_amdgcn_sched_group_barrier(0x100, kGN + 3, 0);                                     \
        _Pragma("unroll") for (int i = 0; i < kGM; ++i) {                                            \
            __builtin_amdgcn_sched_group_barrier(0x008, kGN, 0);                                     \
            if (i + 3 < kGM) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                      \
        }                                                                                            \
    }
#pragma unroll
    for (int s = 0; s + 1 < kGemmRing; ++s) RWKV_GEMM_DMA(s, s);
    int k0 = 0;
    for (; k0 + kGemmRing <= nk; k0 += kGemmRing) {     // whole turns of the ring: the buffer of a step is a constant
#pragma unroll
        for (int s = 0; s < kGemmRing; ++s) RWKV_GEMM_STEP(s, k0 + s)
    }
#pragma unroll
    for (int s = 0; s + 1 < kGemmRing; ++s)
        if (k0 + s < nk) RWKV_GEMM_STEP(s, k0 + s)
#undef RWKV_GEMM_STEP
#undef RWKV_GEMM_DMA
    asm volatile("s_waitcnt vmcnt(0)" ::: "memory");    // nothing of this wavefront may still be writing LDS when it leaves
    gemm_epilogue<kGM, kGN>(a, acc, mt0, nt0, mat, bz, lane);
}

__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(4, 4))) gemm8_kernel(const GemmArgs a) {
    gemm8_body<4, 4, 3>(a);
}
__global__ void __launch_bounds__(512) __attribute__((amdgpu_waves_per_eu(2, 2))) gemm8_wide_kernel(const GemmArgs a) {
    gemm8_body<5, 4, kWideRing>(a);
}

// ---------------------------------------------------------------------------
// The same product for at most 32 rows (a batch of single tokens): the weights are read once and
// hardly reused, so what counts is how many weight bytes a compute unit has in flight.  Workgroup =
// 4 wavefronts side by side = 8 M-tiles x 8 N-tiles (wavefront: 8 x 2); a contraction block is 8 digit
// fragments + 8 weight fragments, fetched kSkinnyAhead blocks ahead (48 KiB of weights per workgroup).
// ---------------------------------------------------------------------------
constexpr int kSkinnyMT = 8, kSkinnyGN = 2, kSkinnyNT = 4 * kSkinnyGN;
constexpr int kSkinnyFrags = kSkinnyMT + kSkinnyNT;     // 16: wave w fetches fragments w, w + 4, w + 8, w + 12
constexpr int kSkinnyAhead = 6;

__global__ void __launch_bounds__(256) __attribute__((amdgpu_waves_per_eu(2, 2))) gemm8_skinny_kernel(const GemmArgs a) {
    __shared__ v4i frag[2][kSkinnyFrags][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int xcd = blockIdx.x % kXcds;
    int item = blockIdx.x / kXcds;
    const int cslot = item % a.per_xcd; item /= a.per_xcd;      // the XCDs share out the column blocks
    const int bx = xcd + kXcds * cslot;
    int bz = item;
    if (bx >= a.gx || bz >= a.gz) return;
    const int mat = bz / a.split;
    bz -= mat * a.split;
    const signed char *dig = mat == 0 ? a.dig[0] : mat == 1 ? a.dig[1] : a.dig[2];
    const uint8_t *w16 = mat == 0 ? a.w16[0] : mat == 1 ? a.w16[1] : a.w16[2];
    const int nt0 = bx * kSkinnyNT + wave * kSkinnyGN;
    const int kb0 = bz * a.kb_per_split;
    int kb1 = kb0 + a.kb_per_split;
    if (kb1 > a.KB) kb1 = a.KB;
    if (kb0 >= kb1) return;                             // (uniform for the workgroup)
    const int nk = kb1 - kb0;

    const v4i *src[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        const int f = wave + 4 * i;
        if (f < kSkinnyMT) {
            const int mt = f < a.MT ? f : a.MT - 1;     // clamped: loads stay unconditional, results are dropped
            src[i] = reinterpret_cast<const v4i *>(dig + ((size_t)mt * a.KB + kb0) * 1024) + lane;
        } else {
            int nt = bx * kSkinnyNT + (f - kSkinnyMT);
            if (nt >= a.NT) nt = a.NT - 1;
            src[i] = reinterpret_cast<const v4i *>(w16 + ((size_t)nt * a.KB + kb0) * 1024) + lane;
        }
    }
    v4i acc[kSkinnyMT][kSkinnyGN];
#pragma unroll
    for (int i = 0; i < kSkinnyMT; ++i)
#pragma unroll
        for (int j = 0; j < kSkinnyGN; ++j) acc[i][j] = v4i{0, 0, 0, 0};

    static_assert(kSkinnyAhead == 6, "six named stages below");
    struct Fly { v4i v0, v1, v2, v3; };                 // named members, not an array: they must stay registers
    Fly fly0, fly1, fly2, fly3, fly4, fly5;
#define RWKV_SKINNY_FETCH(F, K)                                                                      \
    do {                                                                                             \
        const size_t o_ = (size_t)((K) < nk ? (K) : nk - 1) * 64; /* past the end: the last block again (unused) */ \
        F.v0 = src[0][o_]; F.v1 = src[1][o_]; F.v2 = src[2][o_]; F.v3 = src[3][o_];                  \
    } while (0)
#define RWKV_SKINNY_PARK(F, B)                                                                       \
    do {                                                                                             \
        frag[B][wave][lane] = F.v0; frag[B][wave + 4][lane] = F.v1;                                  \
        frag[B][wave + 8][lane] = F.v2; frag[B][wave + 12][lane] = F.v3;                             \
    } while (0)
    // (same step as gemm8_body: the next block is parked, and its registers refilled, piece by piece between
    // this block's groups of matrix instructions)
#define RWKV_SKINNY_MOVE(FN, I, V, B, O)                                                             \
    { frag[B][wave + 4 * (I)][lane] = FN.V; FN.V = src[I][O]; }
#define RWKV_SKINNY_STEP(FN, K)                                                                      \
    {                                                                                                \
        const int buf_ = (K) & 1;                                                                    \
        const size_t on_ = (size_t)((K) + 1 + kSkinnyAhead < nk ? (K) + 1 + kSkinnyAhead : nk - 1) * 64; \
        lds_barrier();                                                                               \
        v4i Bv_[kSkinnyGN];                                                                          \
        _Pragma("unroll") for (int j = 0; j < kSkinnyGN; ++j)                                        \
            Bv_[j] = frag[buf_][kSkinnyMT + wave * kSkinnyGN + j][lane];                             \
        v4i Av_ = frag[buf_][0][lane];                                                               \
        _Pragma("unroll") for (int i = 0; i < kSkinnyMT; ++i) {                                      \
            const v4i An_ = frag[buf_][i + 1 < kSkinnyMT ? i + 1 : i][lane];                         \
            if (i == 0) RWKV_SKINNY_MOVE(FN, 0, v0, buf_ ^ 1, on_)                                   \
            if (i == 2) RWKV_SKINNY_MOVE(FN, 1, v1, buf_ ^ 1, on_)                                   \
            if (i == 4) RWKV_SKINNY_MOVE(FN, 2, v2, buf_ ^ 1, on_)                                   \
            if (i == 6) RWKV_SKINNY_MOVE(FN, 3, v3, buf_ ^ 1, on_)                                   \
            _Pragma("unroll") for (int j = 0; j < kSkinnyGN; ++j)                                    \
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Av_, Bv_[j], acc[i][j], 0, 0, 0);  \
            Av_ = An_;                                                                               \
        }                                                                                            \
        __builtin_amdgcn_sched_group_barrier(0x100, kSkinnyGN + 2, 0);                               \
        _Pragma("unroll") for (int i = 0; i < kSkinnyMT; ++i) {                                      \
            if (i % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x200, 1, 0);                       \
            __builtin_amdgcn_sched_group_barrier(0x008, kSkinnyGN, 0);                               \
            if (i + 2 < kSkinnyMT) __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                \
            if (i % 2 == 0) __builtin_amdgcn_sched_group_barrier(0x020, 1, 0);                       \
        }                                                                                            \
    }
    RWKV_SKINNY_FETCH(fly0, 0); RWKV_SKINNY_FETCH(fly1, 1); RWKV_SKINNY_FETCH(fly2, 2);
    RWKV_SKINNY_FETCH(fly3, 3); RWKV_SKINNY_FETCH(fly4, 4); RWKV_SKINNY_FETCH(fly5, 5);
    RWKV_SKINNY_PARK(fly0, 0);
    RWKV_SKINNY_FETCH(fly0, kSkinnyAhead);
    int k0 = 0;
    for (; k0 + kSkinnyAhead <= nk; k0 += kSkinnyAhead) {      // whole rounds: no branch between the steps
        RWKV_SKINNY_STEP(fly1, k0)
        RWKV_SKINNY_STEP(fly2, k0 + 1)
        RWKV_SKINNY_STEP(fly3, k0 + 2)
        RWKV_SKINNY_STEP(fly4, k0 + 3)
        RWKV_SKINNY_STEP(fly5, k0 + 4)
        RWKV_SKINNY_STEP(fly0, k0 + 5)
    }
    if (k0 < nk) RWKV_SKINNY_STEP(fly1, k0)
    if (k0 + 1 < nk) RWKV_SKINNY_STEP(fly2, k0 + 1)
    if (k0 + 2 < nk) RWKV_SKINNY_STEP(fly3, k0 + 2)
    if (k0 + 3 < nk) RWKV_SKINNY_STEP(fly4, k0 + 3)
    if (k0 + 4 < nk) RWKV_SKINNY_STEP(fly5, k0 + 4)
#undef RWKV_SKINNY_STEP
#undef RWKV_SKINNY_MOVE
#undef RWKV_SKINNY_PARK
#undef RWKV_SKINNY_FETCH
    gemm_epilogue<kSkinnyMT, kSkinnyGN>(a, acc, 0, nt0, mat, bz, lane);
}

// ---------------------------------------------------------------------------
// The same product for at most 8 rows (MT <= 2 M-tiles: a single token of a shape the persistent kernel does
// not serve, a small batch): pure weight streaming.  No LDS staging and no barrier in the loop: workgroup =
// one 16-column tile and one part of the contraction, its 4 wavefronts take every fourth block (together
// they read the tile's blocks in order) and each keeps 8 blocks of weights in flight on its own, so that a
// slow load holds up one wavefront, not the workgroup.  The digit fragments (L2-resident) are read by every
// wavefront itself.  One cross-wavefront sum in LDS at the end, then the common epilogue.
// ---------------------------------------------------------------------------
constexpr int kVecMT = 2;

// kVecBlocks: weight blocks a wavefront has in flight
template <int MT, int kVecBlocks>
__global__ void __launch_bounds__(256) gemv16_kernel(const GemmArgs a) {
    __shared__ v4i red[4][MT][64];
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    int item = blockIdx.x;
    const int nt = item % a.NT; item /= a.NT;
    const int bz = item % a.split, mat = item / a.split;
    const signed char *dig = mat == 0 ? a.dig[0] : mat == 1 ? a.dig[1] : a.dig[2];
    const uint8_t *w16 = mat == 0 ? a.w16[0] : mat == 1 ? a.w16[1] : a.w16[2];
    const int kb0 = bz * a.kb_per_split;
    int kb1 = kb0 + a.kb_per_split;
    if (kb1 > a.KB) kb1 = a.KB;
    const v4i *bsrc = reinterpret_cast<const v4i *>(w16 + (size_t)nt * a.KB * 1024) + lane;
    const v4i *asrc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m)
        asrc[m] = reinterpret_cast<const v4i *>(dig + (size_t)(m < a.MT ? m : a.MT - 1) * a.KB * 1024) + lane;
    v4i acc[MT][1];
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m][0] = v4i{0, 0, 0, 0};
    for (int k = kb0 + wave; k < kb1; k += 4 * kVecBlocks) {
        v4i B[kVecBlocks], A[MT][kVecBlocks];
#pragma unroll
        for (int i = 0; i < kVecBlocks; ++i) {
            const size_t o = (size_t)min(k + 4 * i, a.KB - 1) * 64;       // past the end: a block nobody multiplies
            B[i] = bsrc[o];
#pragma unroll
            for (int m = 0; m < MT; ++m) A[m][i] = asrc[m][o];
        }
#pragma unroll
        for (int i = 0; i < kVecBlocks; ++i) {
            if (k + 4 * i < kb1) {          // uniform for the wavefront
#pragma unroll
                for (int m = 0; m < MT; ++m)
                    acc[m][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[m][i], B[i], acc[m][0], 0, 0, 0);
            }
        }
    }
    // digit sums of at most a few hundred blocks: far inside int32
#pragma unroll
    for (int m = 0; m < MT; ++m) red[wave][m][lane] = acc[m][0];
    __syncthreads();
    if (wave != 0) return;
#pragma unroll
    for (int m = 0; m < MT; ++m) acc[m][0] = red[0][m][lane] + red[1][m][lane] + red[2][m][lane] + red[3][m][lane];
    gemm_epilogue<MT, 1>(a, acc, 0, nt, mat, bz, lane);
}

// ---------------------------------------------------------------------------
// y[t, j] = S_t * tot + 128 * S_t * sum q_t + zp_t, then the phase's element-wise tail.
// ---------------------------------------------------------------------------
struct FinishArgs {
    int R, N, ldd, slices;
    size_t slice;
    const long long *tot;       // [products][slices][...]
    const double *S[kRowsMaxProducts], *qs[kRowsMaxProducts], *zp[kRowsMaxProducts];
    double *out[kRowsMaxProducts];      // [R, N] each
    const float *gate;          // ROW_GATE_ADD: raw receptance [R, N]
};

template <int OP>
__global__ void __launch_bounds__(256) rows_finish_kernel(const FinishArgs a) {
    const int t = blockIdx.y, mat = blockIdx.z;
    const int j = blockIdx.x * 256 + threadIdx.x;
    if (j >= a.N) return;
    const double *Sv = mat == 0 ? a.S[0] : mat == 1 ? a.S[1] : a.S[2];
    const double *qsv = mat == 0 ? a.qs[0] : mat == 1 ? a.qs[1] : a.qs[2];
    const double *zpv = mat == 0 ? a.zp[0] : mat == 1 ? a.zp[1] : a.zp[2];
    double *outv = mat == 0 ? a.out[0] : mat == 1 ? a.out[1] : a.out[2];
    const double S = Sv[t];
    long long tot = 0;                                   // integer partial sums of the contraction splits: exact in any order
    const long long *tp = a.tot + (size_t)mat * a.slices * a.slice + (size_t)t * a.ldd + j;
    for (int z = 0; z < a.slices; ++z) tot += tp[(size_t)z * a.slice];
    const double y = S * (double)tot + 128.0 * (S * qsv[t]) + zpv[t];
    double *o = outv + (size_t)t * a.N + j;
    if (OP == ROW_STORE) *o = y;
    else if (OP == ROW_STORE_F32) reinterpret_cast<float *>(outv)[(size_t)t * a.N + j] = (float)y;
    else if (OP == ROW_RELU2) { const double r = y > 0.0 ? y : 0.0; reinterpret_cast<float *>(outv)[(size_t)t * a.N + j] = (float)(r * r); }   // block.py:97
    else if (OP == ROW_ADD) *o += y;                                                          // block.py:80
    else if (OP == ROW_GATE_ADD) *o += y * (double)sigmoid_f32(a.gate[(size_t)t * a.N + j]);          // block.py:95-100
}

// ---------------------------------------------------------------------------
// WKV + receptance gate           (block.py:69-78, wkv.py:23-39, operators.cu:6-37)
// Arithmetic of the single-token kernel: sums, exponentials and the gate in float32, the exponent pp in float64
// (wkv_step_f32).  A float64 exponential is some fifty dependent instructions, and with one wavefront per 64
// channels and chunk there is nothing to hide them behind: the float64 form took three times as long.
// sequence: thread = channel, serial over the T rows; batch: thread = (row, channel).
// ---------------------------------------------------------------------------
struct WkvRowsArgs {
    int C, R, sequence;
    const float *k, *v, *r;     // [R, C]  float32: what the single-token kernel rounds them to as well
    const double *w, *u;        // [C]  (w = -exp(time_decay))
    double *state;              // rows aa, bb, pp of the layer: state + 2C; batch: + row * state_stride
    int64_t state_stride;
    float *out;                 // [R, C]  wkv * sigmoid(r): a float32 product
    RowsDeferred pend[3];       // batch rows: k, v, r still in slices (tot null: read from the arrays above)
};

__global__ void __launch_bounds__(64) wkv_rows_kernel(const WkvRowsArgs a) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= a.C) return;
    const int C = a.C;
    const double w = a.w[c], u = a.u[c];
    const int t0 = a.sequence ? 0 : blockIdx.y, t1 = a.sequence ? a.R : blockIdx.y + 1;
    double *st = a.state + (a.sequence ? 0 : (size_t)blockIdx.y * a.state_stride);
    float aa = (float)st[c], bb = (float)st[C + c];
    double pp = st[2 * C + c];
    for (int t = t0; t < t1; ++t) {
        const size_t i = (size_t)t * C + c;
        // (uniform branches; a pending product is rounded to float32 exactly as ROW_STORE_F32 would have stored it)
        const float kk = a.pend[0].tot ? (float)deferred_value(a.pend[0], t, c) : a.k[i];
        const float vv = a.pend[1].tot ? (float)deferred_value(a.pend[1], t, c) : a.v[i];
        const float rr = a.pend[2].tot ? (float)deferred_value(a.pend[2], t, c) : a.r[i];
        const float y = wkv_step_f32(w, u, kk, vv, aa, bb, pp);
        a.out[i] = y * sigmoid_f32(rr);
    }
    st[c] = (double)aa; st[C + c] = (double)bb; st[2 * C + c] = pp;
}


// Long sequences: the recurrence is linear in (aa, bb), so T steps split into chunks of kWkvChunk:
// (1) every chunk's own contribution from an empty state, in parallel; (2) a short serial pass that
// turns them into each chunk's incoming state (a chunk decays its input by e^{n w}); (3) every chunk
// replays its steps from that state, in parallel.  Same sums as the serial order up to float64 rounding.
constexpr int kWkvChunk = 32;

// The kernels read their inputs kWkvGroup steps ahead of the serial recurrence (registers, two groups): a
// thread that fetched each step's k and v when it needed them would wait out a memory round trip per step.
constexpr int kWkvGroup = 8;
static_assert(kWkvChunk % kWkvGroup == 0, "whole groups");

__global__ void __launch_bounds__(64) wkv_chunk_local_kernel(const WkvRowsArgs a, double *scr) {
    const int c = blockIdx.x * 64 + threadIdx.x, j = blockIdx.y;
    if (c >= a.C) return;
    const int C = a.C;
    const double w = a.w[c], u = a.u[c];
    const int t0 = j * kWkvChunk, t1 = min(t0 + kWkvChunk, a.R);
    float aa = 0.f, bb = 0.f;
    double pp = -1e30;
    float kc[kWkvGroup], vc[kWkvGroup], kn[kWkvGroup], vn[kWkvGroup];
#pragma unroll
    for (int i = 0; i < kWkvGroup; ++i) {
        const size_t o = (size_t)min(t0 + i, t1 - 1) * C + c;
        kc[i] = a.k[o]; vc[i] = a.v[o];
    }
    for (int g = t0; g < t1; g += kWkvGroup) {
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) {
            const size_t o = (size_t)min(g + kWkvGroup + i, t1 - 1) * C + c;      // past the end: the last row again (unused)
            kn[i] = a.k[o]; vn[i] = a.v[o];
        }
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i)
            if (g + i < t1) (void)wkv_step_f32(w, u, kc[i], vc[i], aa, bb, pp);
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) { kc[i] = kn[i]; vc[i] = vn[i]; }
    }
    double *o = scr + (size_t)j * 3 * C;
    o[c] = (double)aa; o[C + c] = (double)bb; o[2 * C + c] = pp;
}

__global__ void __launch_bounds__(64) wkv_chunk_prefix_kernel(const WkvRowsArgs a, double *scr, int n_chunks) {
    const int c = blockIdx.x * 64 + threadIdx.x;
    if (c >= a.C) return;
    const int C = a.C;
    const double w = a.w[c];
    double aa = a.state[c], bb = a.state[C + c], pp = a.state[2 * C + c];
    double la[kWkvGroup], lb[kWkvGroup], lp[kWkvGroup], na[kWkvGroup], nb[kWkvGroup], np[kWkvGroup];
#pragma unroll
    for (int i = 0; i < kWkvGroup; ++i) {
        const double *o = scr + (size_t)min(i, n_chunks - 1) * 3 * C;
        la[i] = o[c]; lb[i] = o[C + c]; lp[i] = o[2 * C + c];
    }
    for (int g = 0; g < n_chunks; g += kWkvGroup) {
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) {
            const double *o = scr + (size_t)min(g + kWkvGroup + i, n_chunks - 1) * 3 * C;
            na[i] = o[c]; nb[i] = o[C + c]; np[i] = o[2 * C + c];
        }
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) {
            const int j = g + i;
            if (j < n_chunks) {
                double *o = scr + (size_t)j * 3 * C;
                o[c] = aa; o[C + c] = bb; o[2 * C + c] = pp;              // incoming state of chunk j
                const int n = min(kWkvChunk, a.R - j * kWkvChunk);
                const double s = pp + (double)n * w;
                const double p = fmax(s, lp[i]);
                const double f1 = (double)expf((float)(s - p)), f2 = (double)expf((float)(lp[i] - p));   // (one of them is e^0)
                aa = f1 * aa + f2 * la[i];
                bb = f1 * bb + f2 * lb[i];
                pp = p;
            }
        }
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) { la[i] = na[i]; lb[i] = nb[i]; lp[i] = np[i]; }
    }
    a.state[c] = aa; a.state[C + c] = bb; a.state[2 * C + c] = pp;
}

__global__ void __launch_bounds__(64) wkv_chunk_replay_kernel(const WkvRowsArgs a, const double *scr) {
    const int c = blockIdx.x * 64 + threadIdx.x, j = blockIdx.y;
    if (c >= a.C) return;
    const int C = a.C;
    const double w = a.w[c], u = a.u[c];
    const int t0 = j * kWkvChunk, t1 = min(t0 + kWkvChunk, a.R);
    const double *in = scr + (size_t)j * 3 * C;
    float aa = (float)in[c], bb = (float)in[C + c];
    double pp = in[2 * C + c];
    float kc[kWkvGroup], vc[kWkvGroup], rc[kWkvGroup], kn[kWkvGroup], vn[kWkvGroup], rn[kWkvGroup];
#pragma unroll
    for (int i = 0; i < kWkvGroup; ++i) {
        const size_t o = (size_t)min(t0 + i, t1 - 1) * C + c;
        kc[i] = a.k[o]; vc[i] = a.v[o]; rc[i] = a.r[o];
    }
    for (int g = t0; g < t1; g += kWkvGroup) {
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) {
            const size_t o = (size_t)min(g + kWkvGroup + i, t1 - 1) * C + c;
            kn[i] = a.k[o]; vn[i] = a.v[o]; rn[i] = a.r[o];
        }
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) {
            if (g + i < t1) {
                const float y = wkv_step_f32(w, u, kc[i], vc[i], aa, bb, pp);
                a.out[(size_t)(g + i) * C + c] = y * sigmoid_f32(rc[i]);
            }
        }
#pragma unroll
        for (int i = 0; i < kWkvGroup; ++i) { kc[i] = kn[i]; vc[i] = vn[i]; rc[i] = rn[i]; }
    }
}

// ---------------------------------------------------------------------------
// Stand-alone matrix-vector product for 1..8 vectors on the M16 layout, four-vector dequantisation
//   y[b,k] = r_col[k] * sum_j fp32(x[b,j] r_row[j]) code[j,k] + sum_j x[b,j] m_row[j] + m_col[k] sum_j x[b,j]
// (the T == 1 branch of MM8.forward, matmul.py:51-62, with per-column factors on top).
//
// Two launches.  mv16_quant_kernel rewrites the vectors once, for every workgroup of the product, as fixed-point
// digit fragments; the contraction is cut into chunks of CB = 4 blocks (256 rows) and every (vector, chunk) has its
// own power-of-two scale, so no workgroup of the quantiser waits for another and the fixed point is as fine as
// the chunk allows.  mv16_kernel gives one 16-column tile to a workgroup whose wavefronts take the chunks in
// turn: all loads of a chunk (CB weight blocks from HBM, CB fragments per group of four vectors from L2) are
// requested before the first matrix instruction, the integer digit sums of a chunk are exact and enter a float64
// sum scaled by the chunk's scale; the wavefronts' sums are added in a fixed order.
// ---------------------------------------------------------------------------
struct Mv16Args {
    int B, n_in, n_out, KB, n_chunks;
    const float *x;             // [B, n_in]
    const float *r_row;         // [n_in]
    const double *m_row;        // [n_in]
    const float *r_col, *m_col; // [n_out] or null
    const uint8_t *w16;         // M16 blocks [ceil(n_out/16)][KB][1024]
    signed char *dig;           // fragments [ceil(B/4)][KB][1024]
    double *rec;                // [B][n_chunks][4]: scale, 128 * scale * sum q, zero-point share, sum x
    double *y;                  // [B, n_out]
};

template <int CB>
__global__ void __launch_bounds__(256) mv16_quant_kernel(const Mv16Args a) {
    // workgroup = (chunk, group of four vectors); wavefront = one vector; a lane holds CB / 4 groups of four values
    constexpr int QPT = CB / 4;
    const int c = blockIdx.x, mt = blockIdx.y;
    const int lane = threadIdx.x & 63, t = 4 * mt + (threadIdx.x >> 6);
    if (t >= a.B) return;                          // (whole wavefronts; the kernel has no barrier)
    float xs[QPT][4];
    float amax = 0.f;
    double zp = 0.0, xsum = 0.0;
    const bool vec = (a.n_in & 3) == 0 && ((reinterpret_cast<uintptr_t>(a.x) | reinterpret_cast<uintptr_t>(a.r_row)) & 15) == 0 &&
                     (reinterpret_cast<uintptr_t>(a.m_row) & 15) == 0;
#pragma unroll
    for (int s = 0; s < QPT; ++s) {
        const int c0 = c * CB * 64 + 4 * (lane + 64 * s);
        float xv[4] = {0.f, 0.f, 0.f, 0.f}, rv[4] = {0.f, 0.f, 0.f, 0.f};
        double mv[4] = {0.0, 0.0, 0.0, 0.0};
        if (vec && c0 + 3 < a.n_in) {
            const float4 x4 = *reinterpret_cast<const float4 *>(a.x + (size_t)t * a.n_in + c0);
            const float4 r4 = *reinterpret_cast<const float4 *>(a.r_row + c0);
            const double2 m0 = *reinterpret_cast<const double2 *>(a.m_row + c0), m1 = *reinterpret_cast<const double2 *>(a.m_row + c0 + 2);
            xv[0] = x4.x; xv[1] = x4.y; xv[2] = x4.z; xv[3] = x4.w;
            rv[0] = r4.x; rv[1] = r4.y; rv[2] = r4.z; rv[3] = r4.w;
            mv[0] = m0.x; mv[1] = m0.y; mv[2] = m1.x; mv[3] = m1.y;
        } else {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                const int j = c0 + i;
                if (j < a.n_in) { xv[i] = a.x[(size_t)t * a.n_in + j]; rv[i] = a.r_row[j]; mv[i] = a.m_row[j]; }
            }
        }
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            const double xd = (double)xv[i];
            xs[s][i] = (float)(xd * (double)rv[i]);                                   // matmul.py:131
            zp += xd * mv[i];
            xsum += xd;
            amax = fmaxf(amax, fabsf(xs[s][i]));
        }
    }
    amax = wmaxf(amax);
    double S, invS;
    row_scale(amax, S, invS);
    double qsum = 0.0;
#pragma unroll
    for (int s = 0; s < QPT; ++s) {
        const int c0 = c * CB * 64 + 4 * (lane + 64 * s);
        if (c0 < a.KB * 64) qsum += emit_quad(xs[s], invS, c0, t, a.KB, a.dig);      // (whole groups of 16 lanes)
    }
    qsum = wsum(qsum); zp = wsum(zp); xsum = wsum(xsum);
    if (lane == 0) {
        double *r = a.rec + ((size_t)t * a.n_chunks + c) * 4;
        r[0] = S; r[1] = 128.0 * (S * qsum); r[2] = zp; r[3] = xsum;
    }
}

template <int MT, int CB, int NTW>
__global__ void __launch_bounds__(1024) mv16_kernel(const Mv16Args a) {
    extern __shared__ double mv_red[];            // [NW][MT][NTW][64] tile sums, then [4 MT][3] row constants
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6), NW = blockDim.x >> 6;
    const int g = lane >> 4, n = lane & 15, NT = (a.n_out + 15) >> 4;
    // NTW neighbouring tiles per workgroup share every digit fragment a wavefront fetches
    const v4i *bsrc[NTW];
#pragma unroll
    for (int j = 0; j < NTW; ++j)
        bsrc[j] = reinterpret_cast<const v4i *>(a.w16 + (size_t)min((int)blockIdx.x * NTW + j, NT - 1) * a.KB * 1024) + lane;
    const v4i *asrc[MT];
#pragma unroll
    for (int m = 0; m < MT; ++m) asrc[m] = reinterpret_cast<const v4i *>(a.dig + (size_t)m * a.KB * 1024) + lane;
    double sum[MT][NTW];
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int j = 0; j < NTW; ++j) sum[m][j] = 0.0;
    double *red = mv_red, *rc3 = mv_red + (size_t)NW * MT * NTW * 64;
    for (int c = wave; c < a.n_chunks; c += NW) {
        v4i Bf[NTW][CB], Af[MT][CB];
        const int kb0 = c * CB;
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            const size_t o = (size_t)min(kb0 + i, a.KB - 1) * 64;                   // past the end: a block nobody multiplies
#pragma unroll
            for (int j = 0; j < NTW; ++j) Bf[j][i] = __builtin_nontemporal_load(bsrc[j] + o);
#pragma unroll
            for (int m = 0; m < MT; ++m) Af[m][i] = asrc[m][o];
        }
        double rS[MT];
#pragma unroll
        for (int m = 0; m < MT; ++m) rS[m] = a.rec[((size_t)min(4 * m + g, a.B - 1) * a.n_chunks + c) * 4];
        if (c == wave && wave == NW - 1) {
            // The last wavefront, while its first blocks travel: the per-vector constants.  Lane 8 t + p adds the
            // chunks p, p + 8, ... of vector t (its loads are independent of each other), then the eight partial
            // sums are added in a fixed order.
            const int t = lane >> 3, p8 = lane & 7;
            double ad = 0.0, z = 0.0, xsm = 0.0;
            const double *r = a.rec + (size_t)min(t, a.B - 1) * a.n_chunks * 4;
#pragma unroll 4
            for (int cc = p8; cc < a.n_chunks; cc += 8) { ad += r[4 * cc + 1]; z += r[4 * cc + 2]; xsm += r[4 * cc + 3]; }
#pragma unroll
            for (int off = 1; off < 8; off <<= 1) {
                ad += __shfl_xor(ad, off, 64); z += __shfl_xor(z, off, 64); xsm += __shfl_xor(xsm, off, 64);
            }
            if (p8 == 0 && t < 4 * MT) { rc3[3 * t] = ad; rc3[3 * t + 1] = z; rc3[3 * t + 2] = xsm; }
        }
        v4i acc[MT][NTW];
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < NTW; ++j) acc[m][j] = v4i{0, 0, 0, 0};
#pragma unroll
        for (int i = 0; i < CB; ++i) {
            if (kb0 + i < a.KB) {                                                     // uniform for the wavefront
#pragma unroll
                for (int m = 0; m < MT; ++m)
#pragma unroll
                    for (int j = 0; j < NTW; ++j)
                        acc[m][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(Af[m][i], Bf[j][i], acc[m][j], 0, 0, 0);
            }
        }
#pragma unroll
        for (int m = 0; m < MT; ++m)
#pragma unroll
            for (int j = 0; j < NTW; ++j) {
                // digit sums of at most 64 CB terms of magnitude <= 2^14 each; the weighted total is below 2^53: exact
                const v4i d = acc[m][j];
                const long long tot = ((((long long)d.x * 256 + d.y) * 256 + d.z) * 256) + d.w;
                sum[m][j] += rS[m] * (double)tot;
            }
    }
#pragma unroll
    for (int m = 0; m < MT; ++m)
#pragma unroll
        for (int j = 0; j < NTW; ++j) red[(((size_t)wave * MT + m) * NTW + j) * 64 + lane] = sum[m][j];
    __syncthreads();
    // wavefront j adds up tile j (fixed order) and writes its 16 columns
    if (wave >= NTW) return;
#pragma unroll
    for (int j = 0; j < NTW; ++j) {
        if (j != wave) continue;
        const int nt = blockIdx.x * NTW + j, col = 16 * nt + n;
#pragma unroll
        for (int m = 0; m < MT; ++m) {
            double s = 0.0;
            for (int w = 0; w < NW; ++w) s += red[(((size_t)w * MT + m) * NTW + j) * 64 + lane];
            const int t = 4 * m + g;
            if (nt < NT && t < a.B && col < a.n_out) {
                const double rc = a.r_col ? (double)a.r_col[col] : 1.0;
                const double mc = a.m_col ? (double)a.m_col[col] : 0.0;
                a.y[(size_t)t * a.n_out + col] = rc * (s + rc3[3 * t]) + rc3[3 * t + 1] + mc * rc3[3 * t + 2];
            }
        }
    }
}

}  // namespace

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
size_t rows_dig_bytes(int64_t R, int64_t K) { return (size_t)(ceil_div(R, 4) * (K / 64) * 1024); }
size_t rows_wkv_scratch_bytes(int64_t R, int64_t C) { return (size_t)(ceil_div(R, kWkvChunk) * 3 * C * 8); }
constexpr int kVecFillWgs = 128;        // products of at most 8 rows: the contraction is split until there are this many workgroups (batch step of 8 / 4 sequences, 3B shape: 3.06 / 2.64 ms at 128, 3.19 / 2.81 at 256, 3.30 / 2.94 at 512)
constexpr int kMaxSplit = 8;
constexpr int kGemmWideNum = 10, kGemmWideDen = 9;     // the 64 x 160 variant is taken when its cost is below 9/10 of the 64 x 128 variant's
// ... except a contraction of 200 blocks and more, which splits in two while the grid is below the device (14B shape,
// 256-token chunks: the [256 x 20480] x [20480 x 5120] product; 14,080 against 13,190 tokens/s)
constexpr int kGemmLongFillWgs = 256, kGemmLongBlocks = 200;
constexpr int kSkinnyFillWgs = 128;     // 9..32 rows (weight streaming): the contraction is split until the grid has this many workgroups (batch-32 step: 8.07 ms at 128, 8.73 at 256, 9.17 at 64 for the 14B shape; 4.06 / 4.13 / 4.11 ms for the 3B shape)
constexpr int kGemmFillWgs = 96;         // larger products: split until the grid has this many workgroups.  A split costs a second launch and a round trip of the integer totals through memory, so it only pays for grids far below the device (3B shape, tokens/s in chunks of 64 / 128 / 256 / 512 tokens: 13,180 / 23,640 / 37,610 / 52,070 at 96; 12,480 / 21,280 / 34,650 / 49,380 at 256; 12,540 / 21,470 / 31,520 / 51,160 at 64)

// Which kernel serves n products of MT row tiles x NT column tiles over KB contraction blocks, its grid and
// the number of contraction splits.  The ONE place these are decided: the launches and the sizing of the
// totals buffer both call it, so the buffer always holds every slice the kernel writes.
enum { PLAN_VEC = 0, PLAN_SKINNY, PLAN_GENERAL, PLAN_WIDE };
struct ProductPlan { int kind, gx, gy, split; };
static ProductPlan plan_products(int64_t MT, int64_t NT, int64_t KB, int n) {
    ProductPlan p;
    p.split = 1;
    if (MT <= kVecMT) {
        // a handful of rows: one 16-column tile per workgroup; only products with fewer tiles than compute
        // units split the contraction (their integer slices are added by the tail kernel)
        p.kind = PLAN_VEC; p.gx = (int)NT; p.gy = 1;
        while (NT * n * p.split < kVecFillWgs && KB / (p.split * 2) >= 8 && p.split < kMaxSplit) p.split *= 2;
        // a very long contraction: one split (the 14B shape's ffn value product, 8 sequences: 6.97 against 7.26 ms per step)
        if (p.split == 1 && NT * n < 512 && KB >= kGemmLongBlocks) p.split = 2;
        return p;
    }
    p.gy = (int)ceil_div(MT, 16);
    p.kind = MT <= kSkinnyMT ? PLAN_SKINNY : PLAN_GENERAL;      // few rows: the weight-streaming variant
    if (p.kind == PLAN_GENERAL) {
        // Rounds of workgroups on 256 compute units, in matrix instructions per step: two general workgroups
        // share a compute unit (2 x 32), a wide one has it alone (40).
        const int64_t w4 = ceil_div(NT, kGemmNT) * p.gy * n, w5 = ceil_div(NT, kGemmWideNT) * p.gy * n;
        const int64_t rem = w4 % 512;
        const int64_t cost4 = (w4 / 512) * 64 + (rem == 0 ? 0 : rem <= 256 ? 32 : 64), cost5 = ceil_div(w5, 256) * 40;
        if (w4 >= 256 && kGemmWideNum * cost5 < kGemmWideDen * cost4) p.kind = PLAN_WIDE;
    }
    p.gx = (int)ceil_div(NT, p.kind == PLAN_SKINNY ? kSkinnyNT : p.kind == PLAN_WIDE ? kGemmWideNT : kGemmNT);
    // Split the contraction until the grid has a few workgroups per compute unit.
    const int fill = p.kind == PLAN_SKINNY ? kSkinnyFillWgs : kGemmFillWgs;
    while ((int64_t)p.gx * p.gy * n * p.split < fill && KB / (p.split * 2) >= 8 && p.split < kMaxSplit) p.split *= 2;
    // a long contraction on a grid still below the device: one split more (two slices at most)
    if (p.kind != PLAN_SKINNY && p.split == 1 && (int64_t)p.gx * p.gy * n < kGemmLongFillWgs && KB >= kGemmLongBlocks) p.split = 2;
    return p;
}
// Upper bound of the splits plan_products chooses for R rows and N columns, whatever the contraction length and
// the number of products in the launch: a longer contraction only lifts the limit on the split, so the
// plan for an unbounded one bounds every real one.
static int gemm_split_bound(int64_t R, int64_t N) {
    const int64_t MT = ceil_div(R, 4), NT = ceil_div(N, 16);
    int s = 1;
    for (int n = 1; n <= kRowsMaxProducts; ++n) {
        const int sp = plan_products(MT, NT, (int64_t)1 << 40, n).split;
        if (sp > s) s = sp;
    }
    return s;
}
size_t rows_tot_bytes(int64_t R, int64_t N) {
    return (size_t)(ceil_div(R, 4) * 4 * round_up(N, 16) * 8) * (size_t)gemm_split_bound(R, N);
}
// What rows_quant keeps in its scratch area for R rows of K values (0: that shape does not use it).
// (a few long rows are quantised by several workgroups each, in two launches: one workgroup per row leaves most of the
// device idle - 14B shape, batch step of 32 sequences: 7.78 against 8.10 ms)
static bool quant_uses_parts(int64_t R, int64_t K) { return R <= 64 && K >= 8192; }
size_t rows_quant_scratch_bytes(int64_t R, int64_t K) {
    if (!quant_uses_parts(R, K)) return 0;
    return (size_t)(R * ceil_div(K, 4 * kRT * kQuantPartSeg) * 2 * 8);
}
void rows_plan_describe(int64_t R, int64_t K, int64_t N, int n, int out[4]) {
    const ProductPlan p = plan_products(ceil_div(R, 4), ceil_div(N, 16), K / 64, n);
    out[0] = p.kind; out[1] = p.gx; out[2] = p.gy; out[3] = p.split;
}

int rows_embed(hipStream_t st, const int64_t *tokens, int64_t R, int V, int C, const float *emb, const double *w,
               const double *b, double *x) {
    hipLaunchKernelGGL(rows_embed_kernel, dim3((unsigned)R), dim3(kRT), 0, st, tokens, V, C, emb, w, b, x);
    RWKV_CHECK_LAUNCH("rows_embed_kernel");
    return RWKV_OK;
}

bool rows_ln_width_supported(int64_t C) { return C % 4 == 0 && C <= 3 * 4 * kLnMaxThreads; }

int rows_ln_mix_quant(hipStream_t st, int n_mix, int64_t R, int C, bool sequence, const double *x, const double *ln_w,
                      const double *ln_b, const double *mu, const double *prev0, double *shift_dst,
                      int64_t prev_stride, const float *const *range, const double *const *offset,
                      const RowsOperand *out, const RowsDeferred *add) {
    if (C % 64 != 0 || !rows_ln_width_supported(C))
        return set_error(RWKV_ERR_SIZE, "rows_ln_mix_quant: width %d is not a multiple of 64 up to %d", C, 3 * 4 * kLnMaxThreads);
    LnQuantArgs a;
    a.C = C; a.R = (int)R; a.sequence = sequence ? 1 : 0; a.x = x; a.ln_w = ln_w; a.ln_b = ln_b; a.mu = mu;
    a.add.tot = nullptr; a.x_rw = nullptr;
    if (add && add->tot) {
        // every row is read and rewritten by its own workgroup only: rows of a sequence read their neighbour's x too
        if (sequence || R >= kRowsDeferMax || (add->op != ROW_ADD && add->op != ROW_GATE_ADD))
            return set_error(RWKV_ERR_ARG, "rows_ln_mix_quant: a pending product needs fewer than %d batch rows and a residual tail",
                             (int)kRowsDeferMax);
        a.add = *add; a.x_rw = const_cast<double *>(x);
    }
    a.prev0 = prev0; a.shift_dst = shift_dst; a.prev_stride = prev_stride;
    const int n_out = n_mix > 0 ? n_mix : 1;
    for (int m = 0; m < 3; ++m) {
        const int k = m < n_out ? m : 0;
        a.range[m] = range[k]; a.offset[m] = offset[k];
        a.dig[m] = out[k].dig; a.S[m] = out[k].S; a.qs[m] = out[k].qs; a.zp[m] = out[k].zp;
    }
    // few rows: 512 threads per row shorten the chain of dependent steps; many rows: 256 threads with twice
    // the channels each keep more rows resident per compute unit
    const bool many = R >= kRowsDeferMax;           // (a pending product is only ever handed to the 512-thread form)
    const dim3 grid((unsigned)R), block(many ? 256 : 512);
    const bool small = many ? C <= 3 * 4 * 256 : C <= 2 * 4 * 512;
#define RWKV_LNQ(NM)                                                                                  \
    do {                                                                                              \
        if (many && small && R <= 512) hipLaunchKernelGGL((rows_ln_mix_quant_few_kernel<NM, 3, 256>), grid, block, 0, st, a);   \
        else if (many && small) hipLaunchKernelGGL((rows_ln_mix_quant_kernel<NM, 3, 256>), grid, block, 0, st, a);   \
        else if (many) hipLaunchKernelGGL((rows_ln_mix_quant_kernel<NM, 6, 256>), grid, block, 0, st, a);       \
        else if (small) hipLaunchKernelGGL((rows_ln_mix_quant_kernel<NM, 2, 512>), grid, block, 0, st, a);      \
        else hipLaunchKernelGGL((rows_ln_mix_quant_kernel<NM, 3, 512>), grid, block, 0, st, a);                 \
    } while (0)
    switch (n_mix) {
        case 0: RWKV_LNQ(0); break;
        case 2: RWKV_LNQ(2); break;
        case 3: RWKV_LNQ(3); break;
        default: return set_error(RWKV_ERR_ARG, "rows_ln_mix_quant: unsupported mix count %d", n_mix);
    }
#undef RWKV_LNQ
    RWKV_CHECK_LAUNCH("rows_ln_mix_quant_kernel");
    return RWKV_OK;
}

int rows_quant(hipStream_t st, int64_t R, int64_t K, const void *in, bool in_f32, const float *range, const double *offset,
               const RowsOperand &out, double *scratch) {
    if (K % 64 != 0) return set_error(RWKV_ERR_SIZE, "rows_quant: contraction length %lld is not a multiple of 64",
                                      (long long)K);
    QuantArgs q;
    q.K = (int)K; q.in = in; q.range = range; q.offset = offset; q.dig = out.dig; q.S = out.S; q.qs = out.qs; q.zp = out.zp;
    const dim3 grid((unsigned)R), block(kRT);
    if (scratch && quant_uses_parts(R, K)) {
        QuantPartArgs pa;
        pa.q = q; pa.G = (int)ceil_div(K, 4 * kRT * kQuantPartSeg); pa.quads_per_part = (int)round_up(ceil_div(K / 4, pa.G), 4);    // whole groups of 16 values: four lanes share a fragment slot
        pa.part = scratch;
        const dim3 pg((unsigned)pa.G, (unsigned)R);
        if (in_f32) {
            hipLaunchKernelGGL((rows_quant_part_kernel<false, float>), pg, block, 0, st, pa);
            hipLaunchKernelGGL((rows_quant_part_kernel<true, float>), pg, block, 0, st, pa);
        } else {
            hipLaunchKernelGGL((rows_quant_part_kernel<false, double>), pg, block, 0, st, pa);
            hipLaunchKernelGGL((rows_quant_part_kernel<true, double>), pg, block, 0, st, pa);
        }
        RWKV_CHECK_LAUNCH("rows_quant_part_kernel");
        return RWKV_OK;
    }
#define RWKV_QUANT_LAUNCH(T)                                                                          \
    do {                                                                                              \
        if (K <= 3 * 4 * kRT) hipLaunchKernelGGL((rows_quant4_kernel<3, T>), grid, block, 0, st, q);          \
        else if (K <= 6 * 4 * kRT) hipLaunchKernelGGL((rows_quant4_kernel<6, T>), grid, block, 0, st, q);     \
        else if (K <= 10 * 4 * kRT) hipLaunchKernelGGL((rows_quant4_kernel<10, T>), grid, block, 0, st, q);   \
        else if (K <= 20 * 4 * kRT) hipLaunchKernelGGL((rows_quant4_kernel<20, T>), grid, block, 0, st, q);   \
        else hipLaunchKernelGGL((rows_quant_kernel<3, T>), grid, block, 0, st, q);      /* any length: a second read past 12288 */ \
    } while (0)
    if (in_f32) RWKV_QUANT_LAUNCH(float);
    else RWKV_QUANT_LAUNCH(double);
#undef RWKV_QUANT_LAUNCH
    RWKV_CHECK_LAUNCH("rows_quant_kernel");
    return RWKV_OK;
}

int rows_products(hipStream_t st, int n, const RowsProduct *p, long long *tot, int64_t R, int64_t K, int64_t N, int op,
                  const float *gate, RowsDeferred *defer) {
    if (K % 64 != 0) return set_error(RWKV_ERR_SIZE, "rows_products: contraction length %lld is not a multiple of 64",
                                      (long long)K);
    if (n < 1 || n > kRowsMaxProducts) return set_error(RWKV_ERR_ARG, "rows_products: %d products in one launch", n);
    if (op < ROW_STORE || op > ROW_STORE_F32) return set_error(RWKV_ERR_ARG, "rows_products: unknown tail %d", op);
    GemmArgs g;
    FinishArgs f;
    for (int m = 0; m < kRowsMaxProducts; ++m) {
        const RowsProduct &q = p[m < n ? m : 0];
        g.dig[m] = q.a.dig; g.w16[m] = q.w16; g.S[m] = q.a.S; g.qs[m] = q.a.qs; g.zp[m] = q.a.zp; g.out[m] = q.out;
        f.S[m] = q.a.S; f.qs[m] = q.a.qs; f.zp[m] = q.a.zp; f.out[m] = q.out;
    }
    g.tot = tot;
    g.MT = (int)ceil_div(R, 4); g.NT = (int)ceil_div(N, 16); g.KB = (int)(K / 64); g.ldd = g.NT * 16;
    const int gy = (int)ceil_div(g.MT, 16);
    g.R = (int)R; g.N = (int)N; g.gate = gate;
    const ProductPlan pl = plan_products(g.MT, g.NT, g.KB, n);
    const int split = pl.split;
    g.kb_per_split = (int)ceil_div(g.KB, split);
    g.split = split;
    g.slice = (size_t)g.MT * 4 * g.ldd;
    g.gz = split * n;
    g.tail = split > 1 ? -1 : op;
    if (pl.kind == PLAN_VEC) {
        g.gx = g.NT; g.gy = 1; g.by_rows = 0; g.per_xcd = 0;
        const dim3 grid((unsigned)(g.NT * g.gz));
        if (g.MT == 1) hipLaunchKernelGGL((gemv16_kernel<1, 8>), grid, dim3(256), 0, st, g);
        else hipLaunchKernelGGL((gemv16_kernel<2, 8>), grid, dim3(256), 0, st, g);
        RWKV_CHECK_LAUNCH("gemv16_kernel");
    } else {
        g.gx = pl.gx; g.gy = gy; g.by_rows = gy >= kXcds;
        g.per_xcd = ((g.by_rows ? gy : pl.gx) + kXcds - 1) / kXcds;
        const dim3 grid((unsigned)(kXcds * g.per_xcd * (g.by_rows ? pl.gx : gy) * g.gz));
        if (pl.kind == PLAN_SKINNY) hipLaunchKernelGGL(gemm8_skinny_kernel, grid, dim3(256), 0, st, g);
        else if (pl.kind == PLAN_WIDE) hipLaunchKernelGGL(gemm8_wide_kernel, grid, dim3(512), 0, st, g);
        else hipLaunchKernelGGL(gemm8_kernel, grid, dim3(512), 0, st, g);
        RWKV_CHECK_LAUNCH("gemm8_kernel");
    }
    for (int m = 0; defer && m < n; ++m) defer[m].tot = nullptr;
    if (split == 1) return RWKV_OK;     // the tail was applied in the product's epilogue
    if (defer && R < kRowsDeferMax && split <= kRowsDeferSlices) {   // the consumer adds the slices up
        for (int m = 0; m < n; ++m)
            defer[m] = RowsDeferred{tot + (size_t)m * split * g.slice, g.slice, split, g.ldd, op, p[m].a.S, p[m].a.qs, p[m].a.zp, gate};
        return RWKV_OK;
    }

    f.R = (int)R; f.N = (int)N; f.ldd = g.ldd; f.slices = split; f.slice = g.slice; f.tot = tot; f.gate = gate;
    const dim3 fg((unsigned)ceil_div(N, 256), (unsigned)R, (unsigned)n), fb(256);
    switch (op) {
        case ROW_STORE: hipLaunchKernelGGL(rows_finish_kernel<ROW_STORE>, fg, fb, 0, st, f); break;
        case ROW_RELU2: hipLaunchKernelGGL(rows_finish_kernel<ROW_RELU2>, fg, fb, 0, st, f); break;
        case ROW_ADD: hipLaunchKernelGGL(rows_finish_kernel<ROW_ADD>, fg, fb, 0, st, f); break;
        case ROW_STORE_F32: hipLaunchKernelGGL(rows_finish_kernel<ROW_STORE_F32>, fg, fb, 0, st, f); break;
        default: hipLaunchKernelGGL(rows_finish_kernel<ROW_GATE_ADD>, fg, fb, 0, st, f); break;
    }
    RWKV_CHECK_LAUNCH("rows_finish_kernel");
    return RWKV_OK;
}

int rows_wkv(hipStream_t st, int64_t R, int C, bool sequence, const float *k, const float *v, const float *r,
             const double *w, const double *u, double *state, int64_t state_stride, float *out, double *scratch,
             const RowsDeferred *kvr) {
    WkvRowsArgs a;
    a.C = C; a.R = (int)R; a.sequence = sequence ? 1 : 0; a.k = k; a.v = v; a.r = r; a.w = w; a.u = u;
    a.state = state; a.state_stride = state_stride; a.out = out;
    for (int i = 0; i < 3; ++i) {
        if (kvr) a.pend[i] = kvr[i];
        else a.pend[i].tot = nullptr;
        if (a.pend[i].tot && (sequence || a.pend[i].op != ROW_STORE_F32))
            return set_error(RWKV_ERR_ARG, "rows_wkv: a pending product needs batch rows and the float32 store tail");
    }
    if (sequence && scratch && R >= 2 * kWkvChunk) {
        const int n_chunks = (int)ceil_div(R, kWkvChunk);
        const dim3 grid((unsigned)ceil_div(C, 64), (unsigned)n_chunks);
        hipLaunchKernelGGL(wkv_chunk_local_kernel, grid, dim3(64), 0, st, a, scratch);
        hipLaunchKernelGGL(wkv_chunk_prefix_kernel, dim3(grid.x), dim3(64), 0, st, a, scratch, n_chunks);
        hipLaunchKernelGGL(wkv_chunk_replay_kernel, grid, dim3(64), 0, st, a, (const double *)scratch);
        RWKV_CHECK_LAUNCH("wkv_chunk kernels");
        return RWKV_OK;
    }
    hipLaunchKernelGGL(wkv_rows_kernel, dim3((unsigned)ceil_div(C, 64), sequence ? 1u : (unsigned)R), dim3(64), 0, st, a);
    RWKV_CHECK_LAUNCH("wkv_rows_kernel");
    return RWKV_OK;
}

// Plan of the stand-alone product: tiles per workgroup ntw and wavefronts per workgroup nw (chunks of kMvCB blocks).
// Every workgroup must be resident at once - a second round of workgroups would start its loads only when the
// first has drained - so the wavefronts take several chunks in turn where one chunk each would not fit.  Two
// tiles per workgroup (half the fragment traffic) only where that leaves a workgroup for every compute unit.
constexpr int kMvCB = 4;
struct Mv16Plan { int ntw, nw, n_chunks; };

static Mv16Plan mv16_plan(int64_t KB, int64_t NT, int MT) {
    const int n_chunks = (int)ceil_div(KB, kMvCB);
    const int ntw = NT >= 512 ? 2 : 1;
    const int vgprs = ntw == 2 ? (MT == 2 ? 112 : 88) : (MT == 2 ? 96 : 64);      // mv16_kernel<MT, ntw> as compiled
    const int waves_per_cu = 4 * (512 / vgprs > 8 ? 8 : 512 / vgprs);
    const int64_t grid = ceil_div(NT, ntw);
    for (int rounds = 1; rounds <= n_chunks; ++rounds) {
        const int nw = (int)ceil_div(n_chunks, rounds);
        if (nw > 16) continue;
        if (nw <= ntw || grid <= 256 * (int64_t)(waves_per_cu / nw)) return Mv16Plan{ntw, nw < ntw ? ntw : nw, n_chunks};
    }
    return Mv16Plan{ntw, ntw, n_chunks};
}

size_t rows_mv16_workspace_bytes(int64_t B, int64_t n_in) {
    if (B <= 0 || n_in <= 0) return 0;
    const int64_t KB = ceil_div(n_in, 64), MT = ceil_div(B, 4);
    return (size_t)(MT * KB * 1024) + (size_t)round_up(B * ceil_div(KB, 4) * 4 * 8, 256);
}

int rows_mv16(hipStream_t st, int64_t B, int64_t n_in, int64_t n_out, const float *x, const uint8_t *w16,
              const float *r_row, const double *m_row, const float *r_col, const float *m_col, double *y, void *ws) {
    Mv16Args a;
    a.B = (int)B; a.n_in = (int)n_in; a.n_out = (int)n_out; a.KB = (int)ceil_div(n_in, 64);
    const int MT = (int)ceil_div(B, 4);
    const int64_t NT = ceil_div(n_out, 16);
    const Mv16Plan pl = mv16_plan(a.KB, NT, MT);
    const int nw = pl.nw, ntw = pl.ntw;
    a.n_chunks = pl.n_chunks;
    a.x = x; a.r_row = r_row; a.m_row = m_row; a.r_col = r_col; a.m_col = m_col; a.w16 = w16; a.y = y;
    a.dig = static_cast<signed char *>(ws);
    a.rec = reinterpret_cast<double *>(static_cast<char *>(ws) + (size_t)MT * a.KB * 1024);
    const dim3 qg((unsigned)a.n_chunks, (unsigned)MT);
    hipLaunchKernelGGL(mv16_quant_kernel<kMvCB>, qg, dim3(256), 0, st, a);
    RWKV_CHECK_LAUNCH("mv16_quant_kernel");
    const dim3 grid((unsigned)ceil_div(NT, ntw)), block((unsigned)(64 * nw));
    const size_t lds = ((size_t)nw * MT * ntw * 64 + 4 * MT * 3) * sizeof(double);
    if (ntw == 2) {
        if (MT == 1) hipLaunchKernelGGL((mv16_kernel<1, kMvCB, 2>), grid, block, lds, st, a);
        else hipLaunchKernelGGL((mv16_kernel<2, kMvCB, 2>), grid, block, lds, st, a);
    } else {
        if (MT == 1) hipLaunchKernelGGL((mv16_kernel<1, kMvCB, 1>), grid, block, lds, st, a);
        else hipLaunchKernelGGL((mv16_kernel<2, kMvCB, 1>), grid, block, lds, st, a);
    }
    RWKV_CHECK_LAUNCH("mv16_kernel");
    return RWKV_OK;
}

}  // namespace rwkv
