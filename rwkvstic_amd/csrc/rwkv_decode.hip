// Persistent single-token kernel for the FASTQUANT RWKV-4 forward path
// (reference agnostic/backends/opt.py:61-76, modules/block.py:56-102 at T == 1).
//
// One launch of decode_kernel = one token through every layer and the head; a
// small launch of prep_kernel before it turns the token and the shift state
// into the per-token constants.  The grid is C/16 workgroups, all resident at
// once; workgroup g owns the 16 channels [16g, 16g+16) for the whole token
// (their residual value, WKV state and receptance gate stay in its LDS) and
// the matching 16-column tiles of every matrix.
//
// Dot products.  Weights are streamed as 1 KiB blocks of 16 columns x 64 rows
// (layout "M16", stored as code - 128) straight into v_mfma_i32_16x16x64_i8 as
// the B operand.  The activation vector xs = fp32(x * range) is rewritten once
// per product as 32-bit fixed point q = round(xs / S), S a power of two with
// |q| <= 2^30, split into four base-256 digits; the digits are the A operand
// (rows 0..3), so one instruction yields the four digit sums of 16 columns
// over 64 rows.  The sums are integers: the matrix term
// S * sum_c q_c (code_c - 128) is independent of summation order.  The rest of
// the product, sum_c v_c (offset_c + 128 range_c) with v the unrounded input,
// is a float64 dot product that does not depend on the output column; it is
// computed once by the workgroups that own the channels and travels with the
// activations.
//
// Exchange.  Each of the 4 products per layer needs every channel, so each is
// a chip-wide dependency.  Vectors travel as 8-byte words
// {epoch : 32, float32 payload : 32} written and polled with relaxed
// agent-scope atomics; a consumer spins until every word it needs carries the
// epoch of the producing phase.  There is no grid barrier and no cache flush.
// A buffer is rewritten only after every workgroup has consumed the previous
// contents (each rewrite is downstream of a phase that needed all workgroups'
// outputs of the phase that read it).  Every wait is bounded and raises an
// abort flag that all workgroups observe, so the grid always drains.
//
// Roles.  Vector loads of one wave return in order, so a wave that polls would
// first drain whatever it had prefetched.  The workgroup is therefore split:
// "front" waves talk to the other workgroups (one of them polls, the others
// wait on LDS flags), do the per-channel arithmetic, write the digit planes to
// LDS and finish the 16 owned columns of each product; 8 "back" waves own the
// weight stream.  A back wave's program is one generated assembly statement
// (gen_decode_back.py -> rwkv_decode_back.inc): the 1 KiB blocks of its share
// of the workgroup's 13 tiles per layer form one sequence of positions,
// position p lives in register slot p % R of a fixed ring that is reloaded in
// place, and every wait count is known when the program is generated.  A
// slot's reload (the block R positions ahead, possibly of a later phase or
// layer) is issued after the barrier that hands the phase's partial sums to
// the front waves, a few loads at a time, so the reloads do not delay the
// products and the weight stream keeps running while the front waves wait for
// the other workgroups.  Back waves wait on nothing but LDS barriers and
// their own loads.
#include "rwkv_decode.h"

#include <mutex>
#include <type_traits>
#include <vector>

namespace rwkv {

typedef int v4i __attribute__((ext_vector_type(4)));

constexpr int kBW = 8;                 // back (streaming) waves per workgroup
constexpr int kRealJobs = 13;          // tile jobs per layer: k v r | o | ffn_r, 4 x ffn_k | 4 quarters of ffn_v
constexpr unsigned kSpinLimit = 1u << 20;        // polls before a wait gives up (DArgs::spin_limit; a self-test passes a small one)
constexpr int kStatRows = 2;           // XR rows 0-1: sum x of a workgroup's 16 channels, and their squared deviations from the workgroup's own mean
constexpr int kLnRows = kStatRows + 3 * 3;     // rows of the XR record table
constexpr int kEarlyDiv = 4;           // gathers start when all but G / kEarlyDiv workgroups have published (measured flat from G/20 to G)
constexpr int kSlotsPerGroup = 5;      // parked-tile slots a group of 16 channels needs at once (ffn receptance + 4 ffn key tiles)
constexpr int kHeadCsPerThread = 4;    // head column sums a front thread fetches: 16 per head tile of the workgroup

// LDS flag words
enum { FLAG_ARRIVED = 0, FLAG_SCALE = 1, FLAG_ABORT = 2, FLAG_GO = 3, FLAG_COUNT = 4 };   // FLAG_GO: see the reload gate of the generated back-wave program

// Pointers that were themselves loaded from memory are "flat" to the compiler, and a flat load
// counts against the LDS counter as well as the vector-memory counter: every wait for an LDS read
// would then also wait for every weight load in flight.  All global accesses therefore go through
// explicit global-address-space pointers, and the LDS flag words through LDS-address-space ones.
#define RWKV_GLOBAL __attribute__((address_space(1)))
#define RWKV_LDS __attribute__((address_space(3)))
typedef RWKV_LDS volatile int lds_flag_t;

template <typename T>
__device__ __forceinline__ T gld(const T *p) { return *(const RWKV_GLOBAL T *)p; }
template <typename T>
__device__ __forceinline__ void gst(T *p, T v) { *(RWKV_GLOBAL T *)p = v; }

#define ALOAD(p) __hip_atomic_load((RWKV_GLOBAL u64 *)(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define ASTORE(p, v) __hip_atomic_store((RWKV_GLOBAL u64 *)(p), (u64)(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define ALOAD32(p) __hip_atomic_load((RWKV_GLOBAL unsigned *)(p), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)
#define ASTORE32(p, v) __hip_atomic_store((RWKV_GLOBAL unsigned *)(p), (unsigned)(v), __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT)

// A workgroup owns NT groups of 16 channels (and their tiles): one up to C = 4096, two at C = 5120, whose 320
// groups would not all be resident on 256 compute units.  Wave gi < NT of the front waves finishes group NT w + gi.
template <int KW>
struct GroupShape {
    static constexpr int NT = KW > 8 ? 2 : 1, G = 32 * KW, NWG = G / NT;
};

// Helper workgroups.  At C = 2560 the grid of C / 16 = 160 owner workgroups leaves 96 compute units without
// work; 80 more workgroups there own the ffn key matrix (31 % of a layer's bytes): helper h keeps its 8 tiles of
// the NEXT layer in registers (fetched right after it has multiplied the current ones, a whole layer ahead of
// their use), waits like everybody else for the input of the ffn phase, and publishes relu(k)^2 with its records.
// The owner workgroups then stream 9 tiles per layer instead of 13 and have the ffn receptance tile only to
// multiply in that phase.
constexpr int kHelperPace = 20;        // s_sleep units (64 cycles) between groups of three weight loads of a helper (10 and 30: within 0.5 %; 0: +2 %, 60: +3 %)
template <int KW>
struct DecodeLdsDigBytes {          // bytes of the digit planes at the start of LDS (three C-row sets, or one F-row set)
    static constexpr int value = (3 * 4 * (512 * KW + 64) > 4 * (2048 * KW + 64)) ? 3 * 4 * (512 * KW + 64) : 4 * (2048 * KW + 64);
};

template <int KW>
struct HelperShape {
    static constexpr int NH = KW == 5 ? 80 : 0;                    // helper workgroups
    static constexpr int TILES = NH ? (4 * 32 * KW) / NH : 1;      // ffn key tiles of 16 columns per helper
    static constexpr int LDS_BLOCKS = 4;                           // weight blocks per wavefront that wait in LDS instead of registers
};

struct DArgs {
    DModel m;
    DecodeBuffers b;
    unsigned epoch0;
    const int64_t *token;
    double *state;
    double *logits;
    unsigned spin_limit;    // polls before a wait gives up
    const int *stop;        // device word or null: when it reads non-zero the launch does nothing (a sampled stop token
                            // ended the sequence; the remaining launches of a generation loop then leave the state alone)
};

// ---- the back (weight-streaming) waves ------------------------------------------
// Their program is generated (gen_decode_back.py -> rwkv_decode_back.inc): one asm statement with
// its own register map, so that the ring of in-flight weight blocks sits in fixed registers that
// are reloaded in place.  It meets the compiled front waves only at LDS and workgroup barriers.
#include "rwkv_decode_back.inc"

// ---- cross-lane reductions (DPP, fixed order) --------------------------------
template <int CTRL>
__device__ __forceinline__ int dpp_i(int v) { return __builtin_amdgcn_update_dpp(0, v, CTRL, 0xf, 0xf, false); }
template <int CTRL>
__device__ __forceinline__ float dpp_f(float v) { return __int_as_float(dpp_i<CTRL>(__float_as_int(v))); }
template <int CTRL>
__device__ __forceinline__ double dpp_d(double v) {
    return __hiloint2double(dpp_i<CTRL>(__double2hiint(v)), dpp_i<CTRL>(__double2loint(v)));
}
__device__ __forceinline__ double readlane_d(double v, int lane) {
    return __hiloint2double(__builtin_amdgcn_readlane(__double2hiint(v), lane),
                            __builtin_amdgcn_readlane(__double2loint(v), lane));
}
// Sum / maximum over the 16 lanes of a DPP row (all 16 must be active); every lane gets the result.
__device__ __forceinline__ double row16_sum(double v) {
    v += dpp_d<0xB1>(v); v += dpp_d<0x4E>(v); v += dpp_d<0x141>(v); v += dpp_d<0x140>(v);
    return v;
}
__device__ __forceinline__ float row16_max(float v) {
    v = fmaxf(v, dpp_f<0xB1>(v)); v = fmaxf(v, dpp_f<0x4E>(v));
    v = fmaxf(v, dpp_f<0x141>(v)); v = fmaxf(v, dpp_f<0x140>(v));
    return v;
}
// Over all 64 lanes (all active); the result is wave-uniform.
__device__ __forceinline__ double wave_sum_dpp(double v) {
    v = row16_sum(v);
    return (readlane_d(v, 0) + readlane_d(v, 16)) + (readlane_d(v, 32) + readlane_d(v, 48));
}
__device__ __forceinline__ float wave_max_dpp(float v) {
    v = row16_max(v);
    const int i = __float_as_int(v);
    return fmaxf(fmaxf(__int_as_float(__builtin_amdgcn_readlane(i, 0)), __int_as_float(__builtin_amdgcn_readlane(i, 16))),
                 fmaxf(__int_as_float(__builtin_amdgcn_readlane(i, 32)), __int_as_float(__builtin_amdgcn_readlane(i, 48))));
}

// ---- fixed-point digits ------------------------------------------------------
// Scale for a vector with |xs| <= amax: S = 2^(e-30) with 2^e > amax.  Below 2^-90 the whole vector
// is treated as zero (its products are far under any float32 ulp that matters here and 2^(30-e)
// would leave the float range).
__device__ __forceinline__ void scale_from_amax(float amax, double &S, float &invS) {
    if (!(amax > 0x1p-90f) || !(amax < INFINITY)) { S = 0.0; invS = 0.f; return; }
    int e;
    frexpf(amax, &e);                 // amax = f * 2^e, f in [0.5, 1)  =>  |xs| < 2^e
    S = ldexp(1.0, e - 30);
    invS = ldexpf(1.f, 30 - e);
}

// Four consecutive channels' q -> one dword per digit plane (4x4 byte transpose).  The three low
// bytes are stored XOR 0x80, i.e. as the signed bytes b - 128; the top byte is signed as it is:
//   q = sum_k s_k 256^k + 0x808080.
__device__ __forceinline__ void write_digits4(signed char *dig, int plane_stride, int idx4, int q0, int q1, int q2, int q3) {
    const unsigned u0 = (unsigned)q0 ^ 0x00808080u, u1 = (unsigned)q1 ^ 0x00808080u;
    const unsigned u2 = (unsigned)q2 ^ 0x00808080u, u3 = (unsigned)q3 ^ 0x00808080u;
    const unsigned x0 = __builtin_amdgcn_perm(u1, u0, 0x05010400u), x1 = __builtin_amdgcn_perm(u1, u0, 0x07030602u);
    const unsigned y0 = __builtin_amdgcn_perm(u3, u2, 0x05010400u), y1 = __builtin_amdgcn_perm(u3, u2, 0x07030602u);
    unsigned *d = reinterpret_cast<unsigned *>(dig + idx4);
    d[0] = __builtin_amdgcn_perm(y1, x1, 0x07060302u);                          // most significant byte
    d[plane_stride / 4] = __builtin_amdgcn_perm(y1, x1, 0x05040100u);
    d[2 * (plane_stride / 4)] = __builtin_amdgcn_perm(y0, x0, 0x07060302u);
    d[3 * (plane_stride / 4)] = __builtin_amdgcn_perm(y0, x0, 0x05040100u);      // least significant byte
}

// Value of `v` in lane `src` of the wave (no lane-id arithmetic, unlike __shfl).
__device__ __forceinline__ double lane_read_f64(double v, int src) {
    const long long b = __double_as_longlong(v);
    const int lo = __builtin_amdgcn_ds_bpermute(src << 2, (int)b), hi = __builtin_amdgcn_ds_bpermute(src << 2, (int)(b >> 32));
    return __longlong_as_double(((long long)hi << 32) | (unsigned)lo);
}

// ---- tagged exchange ---------------------------------------------------------
__device__ __forceinline__ void put_word(u64 *dst, unsigned epoch, float v) {
    ASTORE(dst, ((u64)epoch << 32) | (u64)__float_as_uint(v));
}

// Values derived from the thread index are loop invariants; the compiler would compute every
// address and predicate that depends on them once, ahead of the layer loop, and keep hundreds of
// registers alive (or spilled).  An empty asm makes the index opaque where a phase begins, so such
// values are recomputed next to their use.
__device__ __forceinline__ int opaque(int v) {
    asm volatile("" : "+v"(v));
    return v;
}

struct Front {
    int tid, wave, lane;
    unsigned *abort_flag;
    lds_flag_t *flags;
    unsigned spin_limit;
    bool ok;
    __device__ __forceinline__ void refresh() {
        tid = opaque((int)threadIdx.x);
        lane = tid & 63;
        wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    }
    __device__ __forceinline__ void fail() {
        ok = false;
        flags[FLAG_ABORT] = 1;
        ASTORE32(abort_flag, 1u);
    }
};

// Gathers read 16 bytes per lane through a raw buffer descriptor with the agent-coherent cache
// policy: half as many memory instructions as 8-byte atomic loads of the same words.  A 16-byte
// aligned read returns each of its two 8-byte words as some store left it (words are only ever
// written whole).
typedef unsigned v4u __attribute__((ext_vector_type(4)));
typedef __amdgpu_buffer_rsrc_t xtab_t;
__device__ __forceinline__ xtab_t make_xtab(const u64 *p, int words) {
    return __builtin_amdgcn_make_buffer_rsrc(const_cast<u64 *>(p), 0, words * 8, 0x00020000);
}
constexpr int kAuxAgent = 16;      // cache policy bit sc1: coherent at agent scope

// A whole wave fetches NR consecutive rows of a [rows][G] record table as one range of NR * G words,
// 16 bytes (two words) per lane and read, spinning until every word carries `epoch`.  Lane l holds
// words 2 (l + 64 k) + j (k < K, j < 2) of the range; word i belongs to row i / G.  Wave-uniform
// control flow.
template <int NR, int G>
struct RowPoll {
    static constexpr int PAIRS = NR * G / 2, K = (PAIRS + 63) / 64;
    static_assert(G % 2 == 0, "two words per lane");
    float v[K][2];
    // early_seq != 0: FLAG_ARRIVED is raised to early_seq as soon as at most `early_missing` words are
    // still outstanding (at the latest when none is) and on_early() runs, so that the gathers overlap
    // the wait for the last few workgroups; the words that had not arrived are re-read later.
    struct Nothing { __device__ __forceinline__ void operator()() const {} };
    template <typename F = Nothing>
    __device__ __forceinline__ void poll(Front &fx, const u64 *rows, unsigned epoch, int early_seq = 0, int early_missing = 0, F on_early = F()) {
        const xtab_t t = make_xtab(rows, NR * G);
        v4u w[K];
        unsigned spins = 0;
        bool raised = early_seq == 0;
        while (fx.ok) {
            int missing = 0;
#pragma unroll
            for (int k = 0; k < K; ++k)
                if (fx.lane + 64 * k < PAIRS) w[k] = __builtin_amdgcn_raw_buffer_load_b128(t, (fx.lane + 64 * k) * 16, 0, kAuxAgent);
#pragma unroll
            for (int k = 0; k < K; ++k) {
                const bool in = fx.lane + 64 * k < PAIRS;
                missing += __popcll(__ballot(in && w[k].y != epoch)) + __popcll(__ballot(in && w[k].w != epoch));
            }
            if (!raised && missing <= early_missing) {
                if (fx.lane == 0) fx.flags[FLAG_ARRIVED] = early_seq;
                raised = true;
                on_early();                    // this wave's own gather
            }
            if (missing == 0) break;
            __builtin_amdgcn_s_sleep(2);
            if ((++spins & 63u) == 0u && (spins > fx.spin_limit || ALOAD32(fx.abort_flag) != 0u || fx.flags[FLAG_ABORT])) fx.fail();
        }
#pragma unroll
        for (int k = 0; k < K; ++k) {
            const bool in = fx.lane + 64 * k < PAIRS;
            v[k][0] = in ? __uint_as_float(w[k].x) : 0.f;
            v[k][1] = in ? __uint_as_float(w[k].z) : 0.f;
        }
    }
    // this lane's share of row r: sum (float64) and maximum of its words (0 where it holds none)
    __device__ __forceinline__ double lane_sum(const Front &fx, int r) const {
        double acc = 0.0;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if ((2 * (fx.lane + 64 * k) + j) / G == r) acc += (double)v[k][j];
        return acc;
    }
    // this lane's share of sum over the words w of row r of 16 (w / 16 - mean)^2
    __device__ __forceinline__ double lane_group_dev2(const Front &fx, int r, double mean) const {
        double acc = 0.0;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if ((2 * (fx.lane + 64 * k) + j) / G == r && 2 * (fx.lane + 64 * k) + j < NR * G) {
                    const double d = (double)v[k][j] * (1.0 / 16.0) - mean;
                    acc += 16.0 * d * d;
                }
        return acc;
    }
    __device__ __forceinline__ float lane_max(const Front &fx, int r) const {
        float acc = 0.f;
#pragma unroll
        for (int k = 0; k < K; ++k)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                if ((2 * (fx.lane + 64 * k) + j) / G == r) acc = fmaxf(acc, v[k][j]);
        return acc;
    }
};

// Spin on an LDS sequence word written by wave 0.
__device__ __forceinline__ void wait_flag(Front &fx, int which, int seq) {
    unsigned spins = 0;
    while (fx.ok && fx.flags[which] < seq) {
        __builtin_amdgcn_s_sleep(1);
        if ((++spins & 255u) == 0u && (spins > (fx.spin_limit << 4) || fx.flags[FLAG_ABORT])) fx.fail();
    }
}

// Thread ft of FT front threads owns quads (groups of 4 consecutive words) ft, ft + FT, ...
template <int FT, int N>
__device__ __forceinline__ void issue_quads(xtab_t src, int ft, int first, int nq, u64 (&w)[N][4]) {
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const int qi = ft + FT * (first + i);
        if (qi < nq) {
            const v4u lo = __builtin_amdgcn_raw_buffer_load_b128(src, qi * 32, 0, kAuxAgent);
            const v4u hi = __builtin_amdgcn_raw_buffer_load_b128(src, qi * 32 + 16, 0, kAuxAgent);
            w[i][0] = ((u64)lo.y << 32) | lo.x; w[i][1] = ((u64)lo.w << 32) | lo.z;
            w[i][2] = ((u64)hi.y << 32) | hi.x; w[i][3] = ((u64)hi.w << 32) | hi.z;
        }
    }
}
// Re-reads the quads that hold a word without the epoch until none is left (normally the first
// read is complete; with an early start of the gathers the last workgroups' words come later).
template <int FT, int N>
__device__ __forceinline__ void settle_quads(Front &fx, xtab_t src, int first, int nq, unsigned epoch, u64 (&w)[N][4]) {
    unsigned spins = 0;
    while (fx.ok) {
        bool all = true;
#pragma unroll
        for (int i = 0; i < N; ++i) {
            const int qi = fx.tid + FT * (first + i);
            bool good = true;
#pragma unroll
            for (int e = 0; e < 4; ++e) good = good && ((unsigned)(w[i][e] >> 32) == epoch);
            if (qi < nq && !good) {
                all = false;
                const v4u lo = __builtin_amdgcn_raw_buffer_load_b128(src, qi * 32, 0, kAuxAgent);
                const v4u hi = __builtin_amdgcn_raw_buffer_load_b128(src, qi * 32 + 16, 0, kAuxAgent);
                w[i][0] = ((u64)lo.y << 32) | lo.x; w[i][1] = ((u64)lo.w << 32) | lo.z;
                w[i][2] = ((u64)hi.y << 32) | hi.x; w[i][3] = ((u64)hi.w << 32) | hi.z;
            }
        }
        if (all) break;
        __builtin_amdgcn_s_sleep(4);
        if ((++spins & 63u) == 0u && (spins > fx.spin_limit || ALOAD32(fx.abort_flag) != 0u)) { fx.fail(); break; }
    }
}

// Sum of the 8 back waves' digit sums of column n of parked tile `slot`, digits recombined:
// sum_k 256^k sum_c s_k,c w_c.  Every digit sum is below 2^28 in magnitude and the total below 2^52,
// so each step of the float64 Horner form is exact.
__device__ __forceinline__ double tile_total(const v4i *red, int slot, int n) {
    int d0 = 0, d1 = 0, d2 = 0, d3 = 0;
#pragma unroll
    for (int h = 0; h < kBW; h += 4) {
        v4i v[4];
#pragma unroll
        for (int w = 0; w < 4; ++w) v[w] = red[(slot * kBW + h + w) * 16 + n];
#pragma unroll
        for (int w = 0; w < 4; ++w) { d0 += v[w].x; d1 += v[w].y; d2 += v[w].z; d3 += v[w].w; }
    }
    return fma(fma(fma((double)d0, 256.0, (double)d1), 256.0, (double)d2), 256.0, (double)d3);
}
// y = S (sum_c q_c (code_c - 128)) + zp  with  sum_c q_c w_c = total + 0x808080 sum_c w_c.  S is a power
// of two and the sum an integer below 2^53: one rounding, in the addition of zp.
__device__ __forceinline__ double finish_col(const v4i *red, int slot, int n, double S, int colsum, double zp) {
    return fma(S, tile_total(red, slot, n) + (double)(0x808080LL * (long long)colsum), zp);
}

// LayerNorm statistics of the 16 channels a DPP row owns, and everything a consumer of x needs that
// is linear in x: published with x itself.  P, PO: this channel's constants for the NM products the
// normalised vector feeds.  Called by the 16 lanes of row 0 of wave 0.
template <int NM>
__device__ __forceinline__ void publish_ln_input(u64 *X, u64 *XR, int G, int g, int n, unsigned epoch, double x,
                                                 const float (&P)[NM], const double (&PO)[NM]) {
    put_word(X + 16 * g + n, epoch, (float)x);
    // The statistics travel as float32: the sum of the 16 channels and the sum of their squared deviations
    // from the workgroup's OWN mean.  The consumer combines the groups (the parallel form of the variance),
    // so no term is a difference of two numbers that are large against the spread, whatever the mean.
    const double sx = row16_sum(x);
    const float sxf = (float)sx;
    const double dev = x - (double)sxf * (1.0 / 16.0);
    const double m2 = row16_sum(dev * dev);
    float val = n == 0 ? sxf : (float)m2;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        const float mx = row16_max(fabsf((float)(x * (double)P[m])));
        const double so = row16_sum(x * PO[m]);
        const float hi = (float)so, lo = (float)(so - (double)hi);
        if (n == kStatRows + 3 * m) val = mx;
        if (n == kStatRows + 1 + 3 * m) val = hi;
        if (n == kStatRows + 2 + 3 * m) val = lo;
    }
    if (n < kStatRows + 3 * NM) put_word(XR + (size_t)n * G + g, epoch, val);
}

// The same for an epilogue wave whose four DPP rows all hold the same 16 channels (lane n of every
// row: channel n, value x): row 0 publishes x, row 1 + m reduces and publishes the two quantities of
// product m (Pm, POm: that product's constants of channel n) and row 1 also sum x and sum x^2, so the
// reductions of all products run side by side and everything leaves in ONE store instruction (a
// store has to queue behind the weight loads the back waves have just issued).  Values and
// reduction order are those of publish_ln_input.
template <int NM>
__device__ __forceinline__ void publish_ln_input_rows(u64 *X, u64 *XR, int G, int g, int n, int row, unsigned epoch, double x,
                                                      float Pm, double POm) {
    static_assert(NM >= 1 && NM <= 3, "one row per product");
    const double sx = row16_sum(x);
    const float sxf = (float)sx;
    const double dev = x - (double)sxf * (1.0 / 16.0);
    const double m2 = row16_sum(dev * dev);
    const double so = row16_sum(x * POm);
    const float mc = row16_max(fabsf((float)(x * (double)Pm)));
    const float hi = (float)so, lo = (float)(so - (double)hi);
    u64 *dst = X + 16 * g + n;
    float val = (float)x;
    bool on = row == 0;
    if (row >= 1 && row <= NM && n < 3) {
        dst = XR + (size_t)(kStatRows + 3 * (row - 1) + n) * G + g;
        val = n == 0 ? mc : (n == 1 ? hi : lo);
        on = true;
    }
    if (row == 1 && (n == 3 || n == 4)) {                      // the statistics, see publish_ln_input
        dst = XR + (size_t)(n - 3) * G + g;
        val = n == 3 ? sxf : (float)m2;
        on = true;
    }
    if (on) put_word(dst, epoch, val);
}

// ---- owner records --------------------------------------------------------------
// Everything the owner of 16 channels needs of one layer besides its inputs sits in one 4 KiB
// record of 8-byte slots, built at model creation (build_ownrec_kernel) in the order below.  The
// front threads copy the next layer's record, the three WKV state rows of the channels and the
// layer's scalars into LDS while they wait for the matrix cores, so the epilogues read LDS instead
// of keeping dozens of prefetched values in registers across the phases.
enum {
    OR_DECAY = 0, OR_FIRST, OR_LN1W, OR_LN1B, OR_LN2W, OR_LN2B, OR_OFFO,      // float64 per channel
    OR_RNGO_CSO,     // {float32 range_o, int colsum att_o}
    OR_CSK_CSV,      // {colsum att_k, colsum att_v}
    OR_CSR_CSFR,     // {colsum att_r, colsum ffn_r}
    OR_CSFV,         // {colsum ffn_v, 0}
    OR_POFK, OR_POFR,            // PO of this layer's ffn k, r
    OR_PF,                       // {P32 ffn k, P32 ffn r}
    OR_PON0, OR_PON1, OR_PON2,   // PO of the next LayerNorm-fed products (next layer's att k, v, r; or the head)
    OR_PN01, OR_PN2,             // {P32 next 0, P32 next 1}, {P32 next 2, 0}
    OR_FIELDS
};
constexpr int kOrOffV = OR_FIELDS * 16;          // 64 slots: float64 offset_v of the workgroup's ffn_k columns
constexpr int kOrRngVCs = kOrOffV + 64;          // 64 slots: {float32 range_v, int colsum ffn_k}
constexpr int kOrStatic = kOrRngVCs + 64;        // slots that come from the static record
constexpr int kOrState = kOrStatic;              // 48 slots: aa, bb, pp of the 16 channels (per token)
constexpr int kOrScal = kOrState + 48;           // 16 slots: the layer's DScal, byte for byte
constexpr int kOrSlots = 512;
static_assert(kOrScal + 16 <= kOrSlots && sizeof(DScal) == 16 * 8, "owner record");

__device__ __forceinline__ double or_d(const u64 *rec, int slot) { return __longlong_as_double((long long)rec[slot]); }
__device__ __forceinline__ unsigned or_lo(const u64 *rec, int slot) { return (unsigned)rec[slot]; }
__device__ __forceinline__ unsigned or_hi(const u64 *rec, int slot) { return (unsigned)(rec[slot] >> 32); }
__device__ __forceinline__ double or_sumPO(const u64 *rec, int m) { return or_d(rec, kOrScal + m); }
__device__ __forceinline__ double or_sumQO(const u64 *rec, int m) { return or_d(rec, kOrScal + 5 + m); }
__device__ __forceinline__ float or_maxP(const u64 *rec, int m) { return reinterpret_cast<const float *>(rec + kOrScal)[20 + m]; }
__device__ __forceinline__ float or_maxQ(const u64 *rec, int m) { return reinterpret_cast<const float *>(rec + kOrScal)[26 + m]; }

// l == L stages the head's scalars only.
template <int FT, int PARTS>
__device__ __forceinline__ void stage_owner_record(const DArgs &a, int l, int g, int G, int C, u64 *dst, int tid) {
    const bool layer = l < a.m.L;
#pragma unroll
    for (int i = 0; i < kOrSlots / FT; ++i) {
        const int t = tid + FT * i;
        u64 v = 0;
        if (t < kOrStatic) {
            if (layer) v = a.m.ownrec[((size_t)l * G + g) * kOrSlots + t];
        } else if (t < kOrScal) {
            const int k = (t - kOrState) >> 4, n = (t - kOrState) & 15;
            if (layer) v = (u64)__double_as_longlong(a.state[((size_t)l * 5 + 2 + k) * C + 16 * g + n]);
        } else if (t < kOrScal + 16) {
            // slots 0-4 sum PO, 5-9 sum QO, 10-12 max P, 13-15 max Q (float pairs); the per-token
            // ones of a layer are the combination, in a fixed order, of its parts
            const int sidx = t - kOrScal;
            v = reinterpret_cast<const u64 *>(a.m.sc + l)[sidx];
            const bool per_token = (sidx >= 5 && sidx < 10) || sidx >= 13;
            if (layer && per_token) {
                const DScal *sp = a.m.scp + (size_t)l * PARTS;
                if (sidx < 10) {
                    double part[PARTS];
#pragma unroll
                    for (int q = 0; q < PARTS; ++q) part[q] = sp[q].sumQO[sidx - 5];     // independent loads
                    double acc = 0.0;
#pragma unroll
                    for (int q = 0; q < PARTS; ++q) acc += part[q];
                    v = (u64)__double_as_longlong(acc);
                } else {
                    const int i0 = 2 * (sidx - 13), i1 = i0 + 1 < kLnMats ? i0 + 1 : i0;
                    float plo[PARTS], phi[PARTS];
#pragma unroll
                    for (int q = 0; q < PARTS; ++q) { plo[q] = sp[q].maxQ[i0]; phi[q] = sp[q].maxQ[i1]; }
                    float lo = 0.f, hi = 0.f;
#pragma unroll
                    for (int q = 0; q < PARTS; ++q) { lo = fmaxf(lo, plo[q]); hi = fmaxf(hi, phi[q]); }
                    if (i0 + 1 >= kLnMats) hi = 0.f;
                    v = ((u64)__float_as_uint(hi) << 32) | (u64)__float_as_uint(lo);
                }
            }
        }
        dst[t] = v;
    }
}

// Scale of the fixed-point digits of LayerNorm-fed product m (index in the layer's tables: m0 + m)
// from the statistics in `stat`:  |fp32(t P + Q)| <= rsd (max |x P| + |mean| max |P|) + max |Q|.
__device__ __forceinline__ void ln_scale(const double *stat, const u64 *rec, int m0, int m, double &S, float &invS) {
    const double bound = stat[1] * (stat[2 + 2 * m] + fabs(stat[0]) * (double)or_maxP(rec, m0 + m)) + (double)or_maxQ(rec, m0 + m);
    scale_from_amax((float)(bound * 1.000001) + 1e-37f, S, invS);
}
// sum_c mixed_c (offset_c + 128 range_c) of that product.
__device__ __forceinline__ double ln_zp(const double *stat, const u64 *rec, int m0, int m) {
    return stat[1] * (stat[3 + 2 * m] - stat[0] * or_sumPO(rec, m0 + m)) + or_sumQO(rec, m0 + m);
}

// Front side of a LayerNorm-fed product group (NM matrices sharing the normalised input):
// waits for x and its records, leaves mean, rsd and the per-product sums in stat[0..7] and each
// product's scale and zero-point sum in stat[8 + 2m], stat[9 + 2m], writes NM sets of digit planes.  Contains one workgroup barrier (statistics) and ends with the "digits
// ready" barrier.  rec: the LDS owner record of the layer (scalars).
template <int KW, int FW, int NM>
__device__ __forceinline__ void ln_front(Front &fx, int &seq, const DArgs &a, const float *P32, const float *Q32,
                                         const u64 *rec, int m0, unsigned epoch, signed char *dig, double *stat,
                                         long long *tr, long long *tp, int xr_m0 = 0) {
    // xr_m0: the first of the NM products among those the publisher wrote records for
    constexpr int C = 512 * KW, G = 32 * KW, FT = 64 * FW, NQ = C / 4, NQT = (NQ + FT - 1) / FT;
    constexpr int PS = C + 64;
    static_assert(FW >= 4, "one front wave per product plus wave 0");
    fx.refresh();
    // this thread's constants, requested before any waiting
    float4 P[NQT][NM], Q[NQT][NM];
#pragma unroll
    for (int i = 0; i < NQT; ++i) {
        const int qi = fx.tid + FT * i;
        if (qi < NQ) {
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                P[i][m] = *reinterpret_cast<const float4 *>(P32 + (size_t)(m0 + m) * C + 4 * qi);
                Q[i][m] = *reinterpret_cast<const float4 *>(Q32 + (size_t)(m0 + m) * C + 4 * qi);
            }
        }
    }
    ++seq;
    u64 w[NQT][4];
    const xtab_t xt = make_xtab(a.b.X, C);
    if (fx.wave == 0) {
        RowPoll<kStatRows, G> r;
        r.poll(fx, a.b.XR, epoch, seq, kStatRows * (G / kEarlyDiv), [&] { issue_quads<FT, NQT>(xt, fx.tid, 0, NQ, w); });
        if (fx.lane == 0) fx.flags[FLAG_GO] = seq;                // every workgroup's publish has been seen: opens the reload gate
        if (tp && fx.tid == 0) tp[0] = wall_clock64();
        // groups of 16 channels combined: mean of the group sums, variance from the groups' own squared
        // deviations plus the spread of the group means
        const double mean = wave_sum_dpp(r.lane_sum(fx, 0)) * (1.0 / (double)C);
        const double var = wave_sum_dpp(r.lane_sum(fx, 1) + r.lane_group_dev2(fx, 0, mean)) * (1.0 / (double)C);
        const double rsd = 1.0 / sqrt(var + 1e-5);                 // layernorm.py:15-20
        if (fx.lane == 0) { stat[0] = mean; stat[1] = rsd; }
    } else {
        wait_flag(fx, FLAG_ARRIVED, seq);
        issue_quads<FT, NQT>(xt, fx.tid, 0, NQ, w);
        const int m = fx.wave - 1;
        if (m < NM) {
            RowPoll<3, G> r;
            r.poll(fx, a.b.XR + (size_t)(kStatRows + 3 * (xr_m0 + m)) * G, epoch);
            const float mx = wave_max_dpp(r.lane_max(fx, 0));
            const double so = wave_sum_dpp(r.lane_sum(fx, 1) + r.lane_sum(fx, 2));
            if (fx.lane == 0) { stat[2 + 2 * m] = (double)mx; stat[3 + 2 * m] = so; }
        }
    }
    __syncthreads();                                               // statistics
    if (tr && fx.tid == 0) tr[0] = wall_clock64();
    if (fx.flags[FLAG_ABORT]) { fx.ok = false; return; }
    const double mean = stat[0], rsd = stat[1];
    float invS[NM];
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        double S;
        ln_scale(stat, rec, m0, m, S, invS[m]);
        if (fx.tid == 64 * (1 + m)) { stat[8 + 2 * m] = S; stat[9 + 2 * m] = ln_zp(stat, rec, m0, m); }   // for the epilogue
    }
    settle_quads<FT, NQT>(fx, xt, 0, NQ, epoch, w);
#pragma unroll
    for (int i = 0; i < NQT; ++i) {
        const int qi = fx.tid + FT * i;
        if (qi < NQ) {
            float t[4];
#pragma unroll
            for (int e = 0; e < 4; ++e)
                t[e] = (float)(((double)__uint_as_float((unsigned)w[i][e]) - mean) * rsd);
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const float p[4] = {P[i][m].x, P[i][m].y, P[i][m].z, P[i][m].w};
                const float qq[4] = {Q[i][m].x, Q[i][m].y, Q[i][m].z, Q[i][m].w};
                int q[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) q[e] = __float2int_rn(fmaf(t[e], p[e], qq[e]) * invS[m]);   // matmul.py:131
                write_digits4(dig + m * 4 * PS, PS, 4 * qi, q[0], q[1], q[2], q[3]);
            }
        }
    }
    __syncthreads();                                               // digits ready
    if (tr && fx.tid == 0) tr[1] = wall_clock64();
    if (fx.flags[FLAG_ABORT]) fx.ok = false;
}

// Front side of a product whose input was scaled by its producers (att output, ffn value):
// the records carry max |xs| and the shares of the zero-point sum.  Leaves the scale in stat[16],
// the zero-point sum in stat[17].  Ends with the "digits ready" barrier.
template <int KW, int FW, int NQT, int G = 32 * KW>     // G: workgroups that publish a record each
__device__ __forceinline__ void vec_front(Front &fx, int &seq, const u64 *src, const u64 *rec, int nq, unsigned epoch,
                                          signed char *dig, int plane_stride, double *stat, long long *tr, long long *tp) {
    constexpr int FT = 64 * FW;
    constexpr int CH = NQT <= 5 ? NQT : ((NQT + 1) / 2 <= 5 ? (NQT + 1) / 2 : 3), NCH = (NQT + CH - 1) / CH;
    fx.refresh();
    ++seq;
    const xtab_t st = make_xtab(src, 4 * nq);
    u64 w[NCH > 1 ? 2 : 1][CH][4];
    float invS;
    if (fx.wave == 0) {
        RowPoll<3, G> r;
        r.poll(fx, rec, epoch, seq, 3 * (G / kEarlyDiv), [&] { issue_quads<FT, CH>(st, fx.tid, 0, nq, w[0]); });
        if (fx.lane == 0) fx.flags[FLAG_GO] = seq;
        if (tp && fx.tid == 0) tp[0] = wall_clock64();
        const float mx = wave_max_dpp(r.lane_max(fx, 0));
        const double so = wave_sum_dpp(r.lane_sum(fx, 1) + r.lane_sum(fx, 2));
        double S;
        scale_from_amax(mx, S, invS);
        if (fx.lane == 0) { stat[16] = S; stat[17] = so; stat[18] = (double)invS; fx.flags[FLAG_SCALE] = seq; }
    } else {
        wait_flag(fx, FLAG_ARRIVED, seq);
        issue_quads<FT, CH>(st, fx.tid, 0, nq, w[0]);
        wait_flag(fx, FLAG_SCALE, seq);
        invS = (float)stat[18];
    }
    if (tr && fx.tid == 0) tr[0] = wall_clock64();
#pragma unroll
    for (int ch = 0; ch < NCH; ++ch) {
        if (ch + 1 < NCH) issue_quads<FT, CH>(st, fx.tid, (ch + 1) * CH, nq, w[(ch + 1) & 1]);
        settle_quads<FT, CH>(fx, st, ch * CH, nq, epoch, w[ch & 1]);
#pragma unroll
        for (int i = 0; i < CH; ++i) {
            const int qi = fx.tid + FT * (ch * CH + i);
            if (ch * CH + i < NQT && qi < nq) {
                int q[4];
#pragma unroll
                for (int e = 0; e < 4; ++e) q[e] = __float2int_rn(__uint_as_float((unsigned)w[ch & 1][i][e]) * invS);
                write_digits4(dig, plane_stride, 4 * qi, q[0], q[1], q[2], q[3]);
            }
        }
    }
    __syncthreads();                                               // digits ready
    if (tr && fx.tid == 0) tr[1] = wall_clock64();
    if (fx.flags[FLAG_ABORT]) fx.ok = false;
}

// =============================================================================
template <int KW, int FW, bool HELP> using BackOf = std::conditional_t<HELP, BackCfgH<KW, FW>, BackCfg<KW, FW>>;

template <int KW, int FW, bool TRACE, bool HELP>
__device__ __forceinline__ void front_path(const DArgs &a, signed char *dig, const v4i *red, double *stat, double *rf_lds,
                                           lds_flag_t *flags, u64 *own_lds, double *st_lds, long long *trace_lds) {
    constexpr int C = 512 * KW, F = 4 * C, G = GroupShape<KW>::G, NT = GroupShape<KW>::NT, NWG = GroupShape<KW>::NWG, FT = 64 * FW;
    constexpr int PS = C + 64, PSF = F + 64;
    constexpr int NQH = F / 4, NQTH = (NQH + FT - 1) / FT, NQC = C / 4, NQTC = (NQC + FT - 1) / FT;
    static_assert(FW >= NT, "one finishing wave per group");
    Front fx;
    fx.abort_flag = a.b.abort_flag; fx.flags = flags; fx.spin_limit = a.spin_limit; fx.ok = true;
    fx.refresh();
    const int wg = blockIdx.x, L = a.m.L, V = a.m.V;
    const bool fin = fx.wave < NT;                       // wave gi finishes the workgroup's group gi of 16 channels
    const int gi = fin ? fx.wave : 0;
    const int g = NT * wg + gi;
    red += gi * kSlotsPerGroup * kBW * 16;               // the group's parked tiles
    rf_lds += gi * 32;
    // stamps are collected in LDS and copied out after the head: a store to memory here would queue behind the weight stream
    long long *trace = TRACE ? trace_lds : nullptr;     // uniform; thread 0 stamps
    int seq = 0;
    int lane, n, row, c_own;                             // recomputed at the start of every phase
#define RWKV_IDS() do { fx.refresh(); lane = fx.lane; n = lane & 15; row = lane >> 4; c_own = 16 * g + n; } while (0)
    RWKV_IDS();

#pragma unroll
    for (int t = 0; t < NT; ++t) stage_owner_record<FT, KW>(a, 0, NT * wg + t, G, C, own_lds + (2 * t) * kOrSlots, fx.tid);   // read after the first barriers below
    // the residual value of the own channels lives in LDS between the epilogues (rf_lds[16 + n])
    double *x_lds = rf_lds + 16;
    if (fin && row == 0) x_lds[n] = a.m.X0[c_own];

    for (int l = 0; l < L && fx.ok; ++l) {
        const u64 *rec = own_lds + (2 * gi + (l & 1)) * kOrSlots;     // (waves that finish nothing read the layer's scalars from group 0's)
        // New state rows of the own channels are collected in LDS and written out once, after the
        // head: nobody else reads them during this token, and a store issued here would queue in
        // the compute unit's memory pipeline behind the weight stream, in front of the exchange.
        // With two groups per workgroup LDS has no room for that: the rows go straight to memory.
        auto put_state = [&](int r, int nn, double v) {
            if constexpr (NT == 1) st_lds[((size_t)l * 5 + r) * 16 + nn] = v;
            else gst(a.state + ((size_t)l * 5 + r) * C + 16 * g + nn, v);
        };
        const unsigned e = a.epoch0 + 4u * (unsigned)l;
        long long *tr = trace ? trace + (size_t)l * kTraceStampsPerLayer : nullptr;
        const float *P32 = a.m.P32 + (size_t)l * kLnMats * C, *Q32 = a.m.Q32 + (size_t)l * kLnMats * C;
        if (tr && fx.tid == 0) { tr[0] = wall_clock64(); tr[23] = clock64(); }     // [23]: shader clock, for its ratio to the wall clock

        // ===================== phase 1: att k, v, r ============================
        ln_front<KW, FW, 3>(fx, seq, a, P32, Q32, rec, 0, e, dig, stat, tr ? tr + 1 : nullptr, tr ? tr + 16 : nullptr);
        if (!fx.ok) break;
        RWKV_IDS();
        // while the matrix cores run: the LayerNorm output of the own channel is the new att shift state (block.py:58,63-64)
        if (fin && row == 0) put_state(0, n, or_d(rec, OR_LN1W * 16 + n) * ((x_lds[n] - stat[0]) * stat[1]) + or_d(rec, OR_LN1B * 16 + n));
        __syncthreads();                                                         // tile sums parked
        if (tr && fx.tid == 0) tr[3] = wall_clock64();
        if (fin) {
            const int j = row < 3 ? row : 0;             // rows 0..2: columns of k, v, r
            const int cs1 = (int)(j == 0 ? or_lo(rec, OR_CSK_CSV * 16 + n) : (j == 1 ? or_hi(rec, OR_CSK_CSV * 16 + n) : or_lo(rec, OR_CSR_CSFR * 16 + n)));
            const double y = finish_col(red, j, n, stat[8 + 2 * j], cs1, stat[9 + 2 * j]);
            const double yk = lane_read_f64(y, n), yv = lane_read_f64(y, n + 16), yr = lane_read_f64(y, n + 32);
            if (tr && fx.tid == 0) tr[20] = wall_clock64();
            {                                              // all four rows: the same 16 channels; one store instruction
                const double td = or_d(rec, OR_DECAY * 16 + n), tf = or_d(rec, OR_FIRST * 16 + n);
                const float r = sigmoid_f32((float)yr);                          // block.py:72
                float aa = (float)or_d(rec, kOrState + n), bb = (float)or_d(rec, kOrState + 16 + n);
                double pp = or_d(rec, kOrState + 32 + n);
                const float wkv = wkv_step_f32(td, tf, (float)yk, (float)yv, aa, bb, pp);
                const double av = (double)(wkv * r);                             // block.py:78
                const float xs = (float)(av * (double)__uint_as_float(or_lo(rec, OR_RNGO_CSO * 16 + n)));   // matmul.py:131
                const float mx = row16_max(fabsf(xs));
                const double so = row16_sum(av * or_d(rec, OR_OFFO * 16 + n) + 128.0 * (double)xs);
                const float hi = (float)so, lo = (float)(so - (double)hi);
                u64 *dst = a.b.A + c_own;
                float val = xs;
                if (row == 1) { dst = a.b.AR + (size_t)n * G + g; val = n == 0 ? mx : (n == 1 ? hi : lo); }
                if (row == 0 || (row == 1 && n < 3)) put_word(dst, e + 1u, val);
                if (row == 0) {
                    put_state(2, n, (double)aa);
                    put_state(3, n, (double)bb);
                    put_state(4, n, pp);
                }
            }
        }
        if (tr && fx.tid == 0) tr[4] = wall_clock64();

        // ===================== phase 2: att output =============================
        // The next layer's owner record (l + 1 == L: the head's scalars) is fetched here, where every wave
        // is about to wait for the other workgroups anyway: the copy to LDS has to wait for the loads.
        RWKV_IDS();
#pragma unroll
        for (int t = 0; t < NT; ++t)
            stage_owner_record<FT, KW>(a, l + 1, NT * wg + t, G, C, own_lds + (2 * t + ((l + 1) & 1)) * kOrSlots, fx.tid);
        vec_front<KW, FW, NQTC>(fx, seq, a.b.A, a.b.AR, NQC, e + 1u, dig, PS, stat, tr ? tr + 5 : nullptr, tr ? tr + 17 : nullptr);
        if (!fx.ok) break;
        __syncthreads();
        if (tr && fx.tid == 0) tr[7] = wall_clock64();
        RWKV_IDS();
        if (fin) {                                         // all four rows: the same 16 channels; row 1 + m reduces for product m
            const double x_own = x_lds[n] + finish_col(red, 0, n, stat[16], (int)or_hi(rec, OR_RNGO_CSO * 16 + n), stat[17]);   // block.py:80
            const int m = row == 2 ? 1 : 0;                // [0] ffn_k, [1] ffn_r
            const u64 pf = rec[OR_PF * 16 + n];
            const float Pm = __uint_as_float(m ? (unsigned)(pf >> 32) : (unsigned)pf);
            const double POm = or_d(rec, (OR_POFK + m) * 16 + n);
            if (tr && fx.tid == 0) tr[21] = wall_clock64();
            publish_ln_input_rows<2>(a.b.X, a.b.XR, G, g, n, row, e + 2u, x_own, Pm, POm);
            if (row == 0) x_lds[n] = x_own;                // after every row has read the old value
        }
        if (tr && fx.tid == 0) tr[8] = wall_clock64();

        // ===================== phase 3: ffn receptance + key ===================
        if constexpr (HELP)      // the ffn key tiles are the helper workgroups': the receptance alone, second of the two products published
            ln_front<KW, FW, 1>(fx, seq, a, P32, Q32, rec, 4, e + 2u, dig, stat, tr ? tr + 9 : nullptr, tr ? tr + 18 : nullptr, 1);
        else
            ln_front<KW, FW, 2>(fx, seq, a, P32, Q32, rec, 3, e + 2u, dig, stat, tr ? tr + 9 : nullptr, tr ? tr + 18 : nullptr);   // [0] ffn_k, [1] ffn_r
        if (!fx.ok) break;
        RWKV_IDS();
        // the LayerNorm output of the own channel is the new ffn shift state (block.py:82,87-88)
        if (fin && row == 0) put_state(1, n, or_d(rec, OR_LN2W * 16 + n) * ((x_lds[n] - stat[0]) * stat[1]) + or_d(rec, OR_LN2B * 16 + n));
        __syncthreads();
        if (tr && fx.tid == 0) tr[11] = wall_clock64();
        if constexpr (HELP) {
            if (fin && row == 0) {                         // the receptance gate of the own channels (block.py:95)
                const double yr = finish_col(red, 0, n, stat[8], (int)or_hi(rec, OR_CSR_CSFR * 16 + n), stat[9]);
                rf_lds[n] = (double)sigmoid_f32((float)yr);
            }
        } else if (fin) {
            // parked tiles: 0 = ffn_r, 1..4 = ffn_k tiles g, g+G, g+2G, g+3G
            const int f_own = 16 * (g + G * row) + n;      // column of ffn_k tile `row`
            const double y = finish_col(red, 1 + row, n, stat[8], (int)or_hi(rec, kOrRngVCs + lane), stat[9]);
            const double h = y > 0.0 ? y : 0.0;                                  // block.py:97-98
            const double hh = h * h;
            const float xs = (float)(hh * (double)__uint_as_float(or_lo(rec, kOrRngVCs + lane)));
            put_word(a.b.H + f_own, e + 3u, xs);
            const float mx = wave_max_dpp(fabsf(xs));
            const double so = wave_sum_dpp(hh * or_d(rec, kOrOffV + lane) + 128.0 * (double)xs);
            const float hi = (float)so, lo = (float)(so - (double)hi);
            if (lane < 3) put_word(a.b.HR + (size_t)lane * G + g, e + 3u, lane == 0 ? mx : (lane == 1 ? hi : lo));
            if (row == 0) {                                // after H is out: the receptance gate of the own channels (block.py:95)
                const double yr = finish_col(red, 0, n, stat[10], (int)or_hi(rec, OR_CSR_CSFR * 16 + n), stat[11]);
                rf_lds[n] = (double)sigmoid_f32((float)yr);
            }
        }
        if (tr && fx.tid == 0) tr[12] = wall_clock64();

        // ===================== phase 4: ffn value ==============================
        vec_front<KW, FW, NQTH, HELP ? 2 * HelperShape<KW>::NH : G>(fx, seq, a.b.H, a.b.HR, NQH, e + 3u, dig, PSF, stat, tr ? tr + 13 : nullptr,
                                                                tr ? tr + 19 : nullptr);
        if (!fx.ok) break;
        __syncthreads();
        if (tr && fx.tid == 0) tr[15] = wall_clock64();
        RWKV_IDS();
        if (fin) {                                         // all four rows: the same 16 channels; row 1 + m reduces for product m
            const double y = finish_col(red, 0, n, stat[16], (int)or_lo(rec, OR_CSFV * 16 + n), stat[17]);
            const double x_own = y * rf_lds[n] + x_lds[n];                       // block.py:100
            const int m = row >= 1 ? row - 1 : 0;          // next layer's att k, v, r (or the head: one product)
            const u64 pn = rec[(OR_PN01 + (m >> 1)) * 16 + n];
            const float Pm = __uint_as_float((m & 1) ? (unsigned)(pn >> 32) : (unsigned)pn);
            const double POm = or_d(rec, (OR_PON0 + m) * 16 + n);
            if (tr && fx.tid == 0) tr[22] = wall_clock64();
            if (l + 1 == L) publish_ln_input_rows<1>(a.b.X, a.b.XR, G, g, n, row, e + 4u, x_own, Pm, POm);
            else publish_ln_input_rows<3>(a.b.X, a.b.XR, G, g, n, row, e + 4u, x_own, Pm, POm);
            if (row == 0) x_lds[n] = x_own;                // after every row has read the old value
        }
    }

    // ========================= head (opt.py:71-73) ==============================
    const int v_tiles = (V + 15) / 16, head_rounds = (v_tiles + NWG - 1) / NWG;
    red -= gi * kSlotsPerGroup * kBW * 16;                 // the head's parked tiles belong to the workgroup
    const u64 *rec_h = own_lds + (L & 1) * kOrSlots;
    // column sums of the workgroup's head tiles: requested now, parked in the LDS half that held the
    // last layer's record once the wait for x is over (a load inside the loop below would cost a
    // round trip through the busy memory pipeline in every round)
    int *csh = reinterpret_cast<int *>(own_lds + ((L + 1) & 1) * kOrSlots);
    int csv[kHeadCsPerThread];
#pragma unroll
    for (int k = 0; k < kHeadCsPerThread; ++k) {
        const int i = fx.tid + FT * k, v = 16 * (wg + NWG * (i >> 4)) + (i & 15);
        csv[k] = (i < head_rounds * 16 && v < V) ? a.m.cs_head[v] : 0;
    }
    if (fx.ok)
        ln_front<KW, FW, 1>(fx, seq, a, a.m.P32 + (size_t)L * kLnMats * C, a.m.Q32 + (size_t)L * kLnMats * C, rec_h, 0,
                            a.epoch0 + 4u * (unsigned)L, dig, stat, nullptr, nullptr);
    if (!fx.ok) return;     // every wave leaves after the same barrier: the flag is tested after each one that follows a wait
#pragma unroll
    for (int k = 0; k < kHeadCsPerThread; ++k)
        if (fx.tid + FT * k < head_rounds * 16) csh[fx.tid + FT * k] = csv[k];
    RWKV_IDS();
#undef RWKV_IDS
    unsigned par = 0;
    constexpr int NS = BackOf<KW, FW, HELP>::NS;          // head tiles per barrier round
    double Sh;
    float invSh;
    ln_scale(stat, rec_h, 0, 0, Sh, invSh);
    const double zph = ln_zp(stat, rec_h, 0, 0);
    double best = -INFINITY;                               // first maximum of the logits this thread writes
    int best_i = 0x7fffffff;
    for (int h0 = 0; h0 < head_rounds; h0 += NS, par ^= 1u) {
        __syncthreads();                                   // (the first one also orders the csh writes above)
        const int s = fx.tid >> 4;                         // parked tile of this round
        if (s < NS && h0 + s < head_rounds) {
            const int v = 16 * (wg + NWG * (h0 + s)) + n;
            if (v < V) {
                const double y = finish_col(red + par * (NS * kBW * 16), s, n, Sh, csh[16 * (h0 + s) + n], zph);
                a.logits[v] = y;
                if (y > best) { best = y; best_i = v; }    // v grows with the round: an equal later value does not replace
            }
        }
    }
    // the workgroup's candidate for the greedy token: threads 0 .. 16 NS - 1 of wave 0 hold the values
    if (fx.wave == 0) {
#pragma unroll
        for (int off = 32; off >= 1; off >>= 1) {
            const double ob = __shfl_xor(best, off, 64);
            const int oi = __shfl_xor(best_i, off, 64);
            if (ob > best || (ob == best && oi < best_i)) { best = ob; best_i = oi; }
        }
        if (fx.lane == 0) { a.m.amax_val[wg] = best; a.m.amax_idx[wg] = best_i; }
    }
    // the state rows of the own channels: st_lds[l][row][n] -> state[l][row][16 g + n]
    if constexpr (NT == 1)
        for (int i = fx.tid; i < L * 5 * 16; i += FT) a.state[(size_t)(i >> 4) * C + 16 * wg + (i & 15)] = st_lds[i];
    if (TRACE)
        for (int i = fx.tid; i < L * kTraceStampsPerLayer; i += FT) a.b.trace[(size_t)wg * L * kTraceStampsPerLayer + i] = trace_lds[i];
}


// =============================================================================
// A helper workgroup (see HelperShape): all of its wavefronts gather and quantise the ffn phase's input, wavefront
// w multiplies NTW neighbouring tiles over one part of the contraction (every digit fragment it reads from LDS serves
// NTW matrix instructions: with one tile per wavefront the LDS reads of the fragments took longer than the matrix
// cores), wavefront 0 finishes the columns.
// Three workgroup barriers per layer, each followed by a test of the abort word, so that every wavefront leaves
// after the same barrier.
template <int KW, int FW>
__device__ __forceinline__ void helper_path(const DArgs &a, signed char *dig, v4i *red, double *stat, lds_flag_t *flags,
                                            v4i *stash) {
    constexpr int C = 512 * KW, G = GroupShape<KW>::G, NWG = GroupShape<KW>::NWG;
    constexpr int NH = HelperShape<KW>::NH, TPH = HelperShape<KW>::TILES, NWV = FW + kBW, FT = 64 * NWV;
    // NTW tiles per wavefront, WPT wavefronts (parts of the contraction) per tile, KB blocks per tile, KPW blocks of
    // the contraction per wavefront, BPW weight blocks per wavefront
    constexpr int NTW = 4, WPT = NWV * NTW / TPH, KB = 8 * KW, KPW = KB / WPT, BPW = NTW * KPW;
    static_assert(TPH % NTW == 0 && (TPH / NTW) * WPT == NWV && WPT * KPW == KB && TPH * 16 == 128 && NWV >= 3, "helper shape");
    // Of a wavefront's BPW blocks the last of every tile waits in LDS (64 lanes x 16 bytes each, `stash`), the others
    // in registers: all of them in registers would leave too few for the gather and the digits, and the compiler
    // would park blocks in scratch memory - a reload from memory in the middle of the phase.
    constexpr int BLDS = HelperShape<KW>::LDS_BLOCKS, BREG = BPW - BLDS, KREG = BREG / NTW;      // per tile: blocks 0 .. KREG - 1 in registers
    static_assert(BLDS == NTW && KREG == KPW - 1, "one block of every tile waits in LDS");
    constexpr int PS = C + 64, NQ = C / 4, NQT = (NQ + FT - 1) / FT, MFK = 3;      // MFK: the ffn key product in the layer's tables
    static_assert(NQT == 1, "one group of four channels per thread");
    // LDS behind the digit planes: this layer's constants, written by the thread that reads them back (they are
    // fetched a whole phase early, and holding them in registers through the wait would push weight blocks out)
    float4 *cP = reinterpret_cast<float4 *>(dig + 4 * PS), *cQ = cP + NQ;
    int *c_cs = reinterpret_cast<int *>(cQ + NQ);
    float *c_rg = reinterpret_cast<float *>(c_cs + 128);
    double *c_of = reinterpret_cast<double *>(c_rg + 128);
    static_assert(4 * PS + 2 * NQ * 16 + 128 * 16 <= DecodeLdsDigBytes<KW>::value, "constants fit between the digit planes and the parked sums");
    int *redi = reinterpret_cast<int *>(red);              // [TPH][16 columns][4 digit sums], added to by the WPT parts of a tile
    Front fx;
    fx.abort_flag = a.b.abort_flag; fx.flags = flags; fx.spin_limit = a.spin_limit; fx.ok = true;
    fx.refresh();
    const int h = (int)blockIdx.x - NWG, L = a.m.L;
    const int tile0 = h * TPH;
    int seq = 0;
    v4i W[BREG];
    auto load_weights = [&](int l, bool paced) {
        const int tid = opaque((int)threadIdx.x), wv = __builtin_amdgcn_readfirstlane(tid >> 6);
        // block b (of KPW) of tile t (of NTW) of this wavefront: tile tile0 + NTW (wv / WPT) + t, contraction block KPW (wv % WPT) + b
#ifdef RWKV_DIAG
        const uint8_t *base = a.m.w_head + (tid & 63) * 16;       // (see build_jobtab_kernel)
#else
        const uint8_t *base = gld(&a.m.layers[l].w[MAT_FFN_K]) + ((size_t)(tile0 + NTW * (wv / WPT)) * KB + (size_t)(wv % WPT) * KPW) * 1024 + (tid & 63) * 16;
#endif
        auto blk = [&](int t, int b) { return (const RWKV_GLOBAL v4i *)(base + ((size_t)t * KB + b) * 1024); };
        // The helpers' 26 MB per layer are not wanted anywhere for a whole layer: they are requested a few blocks at a
        // time with pauses in between, so that they never stand as one burst in front of the owners' polls, gathers
        // and weight stream.  (`paced` is off for the first layer, before anything runs.)
        v4i T[BLDS];
#pragma unroll
        for (int i = 0; i < BLDS; ++i) {
            if (paced && i % 3 == 0) asm volatile("s_sleep %0" :: "n"(kHelperPace) : "memory");
            T[i] = *blk(i, KREG);
        }
#pragma unroll
        for (int i = 0; i < BREG; ++i) {
            if (paced && i % 3 == 0) asm volatile("s_sleep %0" :: "n"(kHelperPace) : "memory");
            W[i] = *blk(i / KREG, i % KREG);
        }
#pragma unroll
        for (int i = 0; i < BLDS; ++i) stash[(wv * BLDS + i) * 64 + (tid & 63)] = T[i];
        // The blocks are needed a whole layer later; left alone, the compiler moves the loads down to their use,
        // into the critical path of the ffn phase.  Naming the values here pins the loads (and their wait) to this
        // point, where the helper has nothing else to do.
#pragma unroll
        for (int i = 0; i < BREG; ++i) asm volatile("" : "+v"(W[i]));
    };
    load_weights(0, false);
    for (int l = 0; l < L; ++l) {
        fx.refresh();
        const unsigned e = a.epoch0 + 4u * (unsigned)l + 2u;      // the input of the ffn phase
        // stamps of a helper: [0] records seen, [1] statistics, [2] digits, [3] tiles multiplied, [4] published, [5] next weights here
        long long *tr = (a.b.trace && fx.tid == 0) ? a.b.trace + ((size_t)blockIdx.x * L + l) * kTraceStampsPerLayer : nullptr;
        // this layer's constants -> LDS, long before they are needed
        if (fx.tid < NQ) {
            const float *P32 = a.m.P32 + ((size_t)l * kLnMats + MFK) * C, *Q32 = a.m.Q32 + ((size_t)l * kLnMats + MFK) * C;
            const float4 p4 = *reinterpret_cast<const float4 *>(P32 + 4 * fx.tid), q4 = *reinterpret_cast<const float4 *>(Q32 + 4 * fx.tid);
            cP[fx.tid] = p4; cQ[fx.tid] = q4;
        }
        if (fx.wave < 2) {                                 // the columns the two finishing wavefronts own: 64 wave + lane of the helper's 128
            const DPrep &pr = a.m.prep[l];
            const float *rv = gld(&pr.range_v);
            const double *ov = gld(&pr.offset_v);
            const int *csl = a.m.cs + (size_t)l * (6 * C + 4 * C) + 5 * C;
            const int col = 64 * fx.wave + fx.lane, f = 16 * tile0 + col;
            c_cs[col] = gld(csl + f); c_rg[col] = gld(rv + f); c_of[col] = gld(ov + f);
        }
        if (fx.wave == 2 && fx.lane == 0) {                // the product's scalars (the per-token ones: parts in a fixed order)
            const DScal *sc = a.m.sc + l, *sp = a.m.scp + (size_t)l * KW;
            double sq = 0.0;
            float mq = 0.f;
#pragma unroll
            for (int q = 0; q < KW; ++q) { sq += gld(&sp[q].sumQO[MFK]); mq = fmaxf(mq, gld(&sp[q].maxQ[MFK])); }
            stat[20] = gld(&sc->sumPO[MFK]); stat[21] = sq; stat[22] = (double)gld(&sc->maxP[MFK]); stat[23] = (double)mq;
        }
        ++seq;
        u64 w[NQT][4];
        const xtab_t xt = make_xtab(a.b.X, C);
        if (fx.wave == 0) {
            RowPoll<kStatRows, G> r;
            r.poll(fx, a.b.XR, e, seq, kStatRows * (G / kEarlyDiv), [&] { issue_quads<FT, NQT>(xt, fx.tid, 0, NQ, w); });
            const double mean = wave_sum_dpp(r.lane_sum(fx, 0)) * (1.0 / (double)C);
            const double var = wave_sum_dpp(r.lane_sum(fx, 1) + r.lane_group_dev2(fx, 0, mean)) * (1.0 / (double)C);
            const double rsd = 1.0 / sqrt(var + 1e-5);                 // layernorm.py:15-20
            if (fx.lane == 0) { stat[0] = mean; stat[1] = rsd; }
            if (tr) gst(tr + 0, (long long)wall_clock64());
        } else {
            wait_flag(fx, FLAG_ARRIVED, seq);
            issue_quads<FT, NQT>(xt, fx.tid, 0, NQ, w);
            if (fx.wave == 1) {
                RowPoll<3, G> r;
                r.poll(fx, a.b.XR + (size_t)kStatRows * G, e);          // the records of the first product published: ffn key
                const float mx = wave_max_dpp(r.lane_max(fx, 0));
                const double so = wave_sum_dpp(r.lane_sum(fx, 1) + r.lane_sum(fx, 2));
                if (fx.lane == 0) { stat[2] = (double)mx; stat[3] = so; }
            }
        }
        __syncthreads();                                               // statistics
        if (flags[FLAG_ABORT]) break;
        if (tr) gst(tr + 1, (long long)wall_clock64());
        const double mean = stat[0], rsd = stat[1];
        double S;
        float invS;
        {
            const double bound = rsd * (stat[2] + fabs(mean) * stat[22]) + stat[23];
            scale_from_amax((float)(bound * 1.000001) + 1e-37f, S, invS);
        }
        const double zp = rsd * (stat[3] - mean * stat[20]) + stat[21];
        settle_quads<FT, NQT>(fx, xt, 0, NQ, e, w);
        if (fx.tid < NQ) {
            const float4 p4 = cP[fx.tid], q4 = cQ[fx.tid];
            const float p[4] = {p4.x, p4.y, p4.z, p4.w}, qq[4] = {q4.x, q4.y, q4.z, q4.w};
            int q[4];
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                const float t = (float)(((double)__uint_as_float((unsigned)w[0][k]) - mean) * rsd);
                q[k] = __float2int_rn(fmaf(t, p[k], qq[k]) * invS);                             // matmul.py:131
            }
            write_digits4(dig, PS, 4 * fx.tid, q[0], q[1], q[2], q[3]);
        }
        if (fx.tid >= FT - 128) red[fx.tid - (FT - 128)] = v4i{0, 0, 0, 0};      // the sums the parts will add to
        __syncthreads();                                               // digits ready
        if (flags[FLAG_ABORT]) break;
        fx.refresh();
        tr = (a.b.trace && fx.tid == 0) ? a.b.trace + ((size_t)blockIdx.x * L + l) * kTraceStampsPerLayer : nullptr;
        if (tr) gst(tr + 2, (long long)wall_clock64());
        {
            // A operand: lane 16 g4 + m holds bytes 16 g4 .. 16 g4 + 15 of digit plane m & 3 of a 64-row block
            const int part = fx.wave % WPT, tq = fx.wave / WPT;
            const signed char *ap = dig + (fx.lane & 3) * PS + 16 * (fx.lane >> 4) + 64 * (part * KPW);
            const v4i *sp = stash + (fx.wave * BLDS) * 64 + fx.lane;
            // every digit fragment read from LDS serves NTW matrix instructions; the reads run two blocks ahead
            v4i A[3], acc[NTW], Bl[NTW];
#pragma unroll
            for (int t = 0; t < NTW; ++t) acc[t] = v4i{0, 0, 0, 0};
            A[0] = *reinterpret_cast<const v4i *>(ap); A[1] = *reinterpret_cast<const v4i *>(ap + 64);
#pragma unroll
            for (int b = 0; b < KPW; ++b) {
                if (b + 2 < KPW) A[(b + 2) % 3] = *reinterpret_cast<const v4i *>(ap + 64 * (b + 2));
                if (b + 2 == KPW) {
#pragma unroll
                    for (int t = 0; t < NTW; ++t) Bl[t] = sp[t * 64];
                }
#pragma unroll
                for (int t = 0; t < NTW; ++t)
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(A[b % 3], b < KREG ? W[t * KREG + (b < KREG ? b : 0)] : Bl[t], acc[t], 0, 0, 0);
            }
            // rows 0..3 of a result are the four digit sums of column `lane`: integers, added in any order
            if (fx.lane < 16) {
#pragma unroll
                for (int t = 0; t < NTW; ++t) {
                    int *dst = redi + ((NTW * tq + t) * 16 + fx.lane) * 4;
                    atomicAdd(dst + 0, acc[t].x); atomicAdd(dst + 1, acc[t].y); atomicAdd(dst + 2, acc[t].z); atomicAdd(dst + 3, acc[t].w);
                }
            }
        }
        __syncthreads();                                               // tiles multiplied
        if (tr) gst(tr + 3, (long long)wall_clock64());
        if (fx.wave < 2) {                                 // each of the two finishing wavefronts publishes its 64 columns and a record of its own
            const int col = 64 * fx.wave + fx.lane;
            const v4i d = red[col];
            const double tot = fma(fma(fma((double)d.x, 256.0, (double)d.y), 256.0, (double)d.z), 256.0, (double)d.w);
            const double y = fma(S, tot + (double)(0x808080LL * (long long)c_cs[col]), zp);
            const double hv = y > 0.0 ? y : 0.0;                                                 // block.py:97-98
            const double hh = hv * hv;
            const float xs = (float)(hh * (double)c_rg[col]);
            put_word(a.b.H + 16 * tile0 + col, e + 1u, xs);
            const float mx = wave_max_dpp(fabsf(xs));
            const double so = wave_sum_dpp(hh * c_of[col] + 128.0 * (double)xs);
            const float hi = (float)so, lo = (float)(so - (double)hi);
            if (fx.lane < 3) put_word(a.b.HR + (size_t)fx.lane * (2 * NH) + 2 * h + fx.wave, e + 1u, fx.lane == 0 ? mx : (fx.lane == 1 ? hi : lo));
        }
        if (tr) gst(tr + 4, (long long)wall_clock64());
        if (l + 1 < L) load_weights(l + 1, true);           // a whole layer ahead of their use, after the results are out
        if (tr) gst(tr + 5, (long long)wall_clock64());
    }
}

template <int KW, int FW, bool HELP = false>
struct DecodeLds {
    using Back = BackOf<KW, FW, HELP>;
    static constexpr int C = 512 * KW, F = 4 * C, NT = GroupShape<KW>::NT;
    static constexpr int PS = C + 64, PSF = F + 64;
    static constexpr int DIG_BYTES = (3 * 4 * PS > 4 * PSF) ? 3 * 4 * PS : 4 * PSF;
    static constexpr int RED_SLOTS = Back::RED_SLOTS;
    static constexpr int RED_BYTES = RED_SLOTS * kBW * 16 * 16;
    static constexpr int STAT_BYTES = 32 * 8, RF_BYTES = NT * 32 * 8, FLAG_BYTES = FLAG_COUNT * 4;   // RF: gate and residual of the own channels
    static constexpr int OWN_OFFSET = DIG_BYTES + RED_BYTES + STAT_BYTES + RF_BYTES + FLAG_BYTES;
    static constexpr int STATE_OFFSET = OWN_OFFSET + NT * 2 * kOrSlots * 8;
    static __host__ __device__ int state_bytes(int L) { return NT == 1 ? L * 5 * 16 * 8 : 0; }  // the new state rows of the own channels
    // a helper workgroup's stash of weight blocks lies over the owner records and state rows, which it does not have
    static constexpr int STASH_OFFSET = OWN_OFFSET;
    static constexpr int STASH_BYTES = HELP ? (FW + kBW) * HelperShape<KW>::LDS_BLOCKS * 1024 : 0;
    static __host__ __device__ int total(int L, bool trace = false) {                           // (+ the stamps)
        const int own = STATE_OFFSET + state_bytes(L);
        return (own > STASH_OFFSET + STASH_BYTES ? own : STASH_OFFSET + STASH_BYTES) + (trace ? L * kTraceStampsPerLayer * 8 : 0);
    }
    // the generated back-wave program addresses LDS by these offsets
    static_assert(Back::RED == DIG_BYTES, "parked tiles follow the digit planes");
    static_assert(Back::FLAG == DIG_BYTES + RED_BYTES + STAT_BYTES + RF_BYTES + FLAG_ABORT * 4, "abort flag offset");
    static_assert(RED_SLOTS >= kSlotsPerGroup * NT && RED_SLOTS >= 2 * Back::NS, "park slots");
    static_assert(DIG_BYTES == DecodeLdsDigBytes<KW>::value, "digit planes");
    static_assert(!HELP || RED_BYTES >= HelperShape<KW>::TILES * 256, "a helper's tile sums");
};

template <int KW, int FW, bool TRACE, bool HELP>
__global__ void __launch_bounds__((FW + kBW) * 64) decode_kernel(const DArgs a) {
    using Lds = DecodeLds<KW, FW, HELP>;
    extern __shared__ __align__(16) unsigned char smem[];
    signed char *dig = reinterpret_cast<signed char *>(smem);
    v4i *red = reinterpret_cast<v4i *>(smem + Lds::DIG_BYTES);
    double *stat = reinterpret_cast<double *>(smem + Lds::DIG_BYTES + Lds::RED_BYTES);
    double *rf_lds = stat + 32;
    lds_flag_t *flags = (lds_flag_t *)(rf_lds + 32 * Lds::NT);
    if (a.stop && gld(a.stop) != 0) return;          // written before this launch started: every workgroup reads the same value
    if (threadIdx.x < FLAG_COUNT) flags[threadIdx.x] = 0;
    __syncthreads();
    const int wave = __builtin_amdgcn_readfirstlane((int)(threadIdx.x >> 6));
    if constexpr (HELP) {
        if ((int)blockIdx.x >= GroupShape<KW>::NWG) {          // (uniform for the workgroup)
            helper_path<KW, FW>(a, dig, red, stat, flags, reinterpret_cast<v4i *>(smem + Lds::STASH_OFFSET));
            return;
        }
    }
    if (wave < FW) {
        front_path<KW, FW, TRACE, HELP>(a, dig, red, stat, rf_lds, flags, reinterpret_cast<u64 *>(smem + Lds::OWN_OFFSET),
                                  reinterpret_cast<double *>(smem + Lds::STATE_OFFSET),
                                  reinterpret_cast<long long *>(smem + Lds::total(a.m.L)));       // (total without the stamps = where they start)
    } else {
        constexpr int NWG = GroupShape<KW>::NWG;
        const int v_tiles = (a.m.V + 15) / 16, head_rounds = (v_tiles + NWG - 1) / NWG;
        const unsigned lds = (unsigned)(uintptr_t)(RWKV_LDS unsigned char *)smem;
        BackOf<KW, FW, HELP>::run(a.m.jt + (size_t)blockIdx.x * (a.m.L + 1) * 16, a.m.w_head, a.m.L, head_rounds, v_tiles,
                         (int)blockIdx.x, wave - FW, lds);
    }
}

// ---------------------------------------------------------------------------
// Per-token preparation: blocks 0..L-1 turn the shift rows of the state into Q32 and its scalars
// (they change with every token); block L computes x0 = ln0(emb[token]) (emb.py:9, opt.py:63-64)
// and publishes it, with its LayerNorm records, as the input of layer 0.
// ---------------------------------------------------------------------------
constexpr int kPrepThreads = 512;

template <int N>
__device__ __forceinline__ void prep_block_sum(double (&v)[N], double *scr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const double s = wave_sum_dpp(v[i]);
        if (lane == 0) scr[i * (kPrepThreads / 64) + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kPrepThreads / 64; ++w) s += scr[i * (kPrepThreads / 64) + w];
        v[i] = s;
    }
}
template <int N>
__device__ __forceinline__ void prep_block_max(float (&v)[N], float *scr) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        const float s = wave_max_dpp(v[i]);
        if (lane == 0) scr[i * (kPrepThreads / 64) + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        float s = 0.f;
#pragma unroll
        for (int w = 0; w < kPrepThreads / 64; ++w) s = fmaxf(s, scr[i * (kPrepThreads / 64) + w]);
        v[i] = s;
    }
}

// Channels [512 part, 512 part + 512) of layer l: Q32 and this part's share of the scalars.
__device__ __forceinline__ void prep_layer_part(const DArgs &a, int l, int part, double *scr) {
    const int C = a.m.C, KWr = C / kPrepThreads;
    const DPrep &p = a.m.prep[l];
    const double *sl = a.state + (size_t)l * 5 * C;
    const int c = part * kPrepThreads + threadIdx.x;
    double sq[kLnMats];
    float mq[kLnMats];
    const double sh0 = sl[c], sh1 = sl[(size_t)C + c], b1 = p.ln1_b[c], b2 = p.ln2_b[c];
#pragma unroll
    for (int m = 0; m < kLnMats; ++m) {
        const bool att = m < 3;
        const double mu = att ? p.att_mix[(size_t)m * C + c] : p.ffn_mix[(size_t)(m - 3) * C + c];
        const double base = (att ? b1 : b2) * mu + (att ? sh0 : sh1) * (1.0 - mu);   // block.py:67,91 without the x term
        const double rg = (double)p.range[m][c];
        const float q = (float)(base * rg);
        a.m.Q32[((size_t)l * kLnMats + m) * C + c] = q;
        sq[m] = base * (p.offset[m][c] + 128.0 * rg);
        mq[m] = fabsf(q);
    }
    prep_block_sum<kLnMats>(sq, scr);
    prep_block_max<kLnMats>(mq, reinterpret_cast<float *>(scr));
    if (threadIdx.x < kLnMats) {
        DScal &d = a.m.scp[(size_t)l * KWr + part];
        d.sumQO[threadIdx.x] = sq[threadIdx.x];
        d.maxQ[threadIdx.x] = mq[threadIdx.x];
    }
}

// x0 = ln0(emb[tok]) (emb.py:9, opt.py:63-64), published with its LayerNorm records as the input
// of layer 0 under `epoch`.  C is a multiple of 512 and thread t takes channels t, t + 512, ...
__device__ __forceinline__ void prep_token(const DArgs &a, int64_t tok, unsigned epoch, double *scr) {
    constexpr int kMaxParts = 10;                               // C <= 5120
    const int C = a.m.C, G = a.m.G, parts = C / kPrepThreads;
    if (tok < 0) tok = 0;
    if (tok >= a.m.V) tok = a.m.V - 1;
    // everything this thread needs is requested before the first use: the block is one chain of memory latencies otherwise
    double v[kMaxParts], lw[kMaxParts], lb[kMaxParts], PO[kMaxParts][3];
    float P[kMaxParts][3];
#pragma unroll
    for (int k = 0; k < kMaxParts; ++k) {
        const int c = threadIdx.x + k * kPrepThreads;
        if (k < parts) {
            v[k] = (double)a.m.emb[(size_t)tok * C + c];
            lw[k] = a.m.ln0_w[c]; lb[k] = a.m.ln0_b[c];
#pragma unroll
            for (int m = 0; m < 3; ++m) { P[k][m] = a.m.P32[(size_t)m * C + c]; PO[k][m] = a.m.PO[(size_t)m * C + c]; }
        }
    }
    double s[2] = {0.0, 0.0};
#pragma unroll
    for (int k = 0; k < kMaxParts; ++k)
        if (k < parts) { s[0] += v[k]; s[1] += v[k] * v[k]; }
    prep_block_sum<2>(s, scr);
    const double mean = s[0] / (double)C;
    double var = s[1] / (double)C - mean * mean;
    if (var < 0.0) var = 0.0;
    const double rsd = 1.0 / sqrt(var + 1e-5);
#pragma unroll
    for (int k = 0; k < kMaxParts; ++k) {                       // whole waves are in or out: C % 512 == 0
        if (k < parts) {
            const int c = threadIdx.x + k * kPrepThreads;
            const double x0 = lw[k] * ((v[k] - mean) * rsd) + lb[k];
            a.m.X0[c] = x0;
            publish_ln_input<3>(a.b.X, a.b.XR, G, c >> 4, c & 15, epoch, x0, P[k], PO[k]);
        }
    }
}

// grid: L * (C / 512) layer parts, then one block for the token.
__global__ void __launch_bounds__(kPrepThreads) prep_kernel(const DArgs a) {
    __shared__ double scr[8 * (kPrepThreads / 64)];
    if (a.stop && gld(a.stop) != 0) return;
    const int parts = a.m.C / kPrepThreads;
    const int b = blockIdx.x;
    if (b < a.m.L * parts) prep_layer_part(a, b / parts, b % parts, scr);
    else prep_token(a, a.token[0], a.epoch0, scr);
}

// Between two greedy tokens: the greedy token (the single-token kernel left one candidate per
// workgroup: the first maximum of the logits it wrote) -> out_token[0], and the preparation of the
// next step (which reads the state the step before has just updated) in the same launch.
// grid: L * (C / 512) layer parts, then one block for the token.  a.epoch0: the epoch of the NEXT
// token step.
__global__ void __launch_bounds__(kPrepThreads) next_token_kernel(const DArgs a, int64_t *__restrict__ out_token) {
    __shared__ double scr[8 * (kPrepThreads / 64)];
    __shared__ int sidx[kPrepThreads / 64];
    const int parts = a.m.C / kPrepThreads;
    const int b = blockIdx.x;
    if (b < a.m.L * parts) { prep_layer_part(a, b / parts, b % parts, scr); return; }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    auto better = [](double v, int i, double bv, int bi) { return v > bv || (v == bv && i < bi); };
    double best = -INFINITY;
    int bi = 0x7fffffff;
    if ((int)threadIdx.x < a.m.NWG) { best = a.m.amax_val[threadIdx.x]; bi = a.m.amax_idx[threadIdx.x]; }   // NWG <= 256
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const double ob = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (better(ob, oi, best, bi)) { best = ob; bi = oi; }
    }
    if (lane == 0) { scr[wave] = best; sidx[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < kPrepThreads / 64; ++wv)
            if (better(scr[wv], sidx[wv], best, bi)) { best = scr[wv]; bi = sidx[wv]; }
        sidx[0] = bi == 0x7fffffff ? 0 : bi;
        out_token[0] = sidx[0];
    }
    __syncthreads();
    prep_token(a, (int64_t)sidx[0], a.epoch0, scr);
}

// ---------------------------------------------------------------------------
// Model-creation kernels
// ---------------------------------------------------------------------------
// cs[16 t + n] = sum over rows of (code - 128) of column 16 t + n of an M16 matrix; one wave per tile.
__global__ void __launch_bounds__(64) colsum_m16_kernel(const uint8_t *__restrict__ w16, int n_kb, int *__restrict__ cs) {
    const int lane = threadIdx.x;
    const uint8_t *p = w16 + (size_t)blockIdx.x * n_kb * 1024 + lane * 16;
    int acc = 0;
    for (int kb = 0; kb < n_kb; ++kb) {
        const uint4 v = *reinterpret_cast<const uint4 *>(p + (size_t)kb * 1024);
        const unsigned d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int i = 0; i < 4; ++i)
            acc += (int)(signed char)(d[i] & 0xff) + (int)(signed char)((d[i] >> 8) & 0xff) +
                   (int)(signed char)((d[i] >> 16) & 0xff) + (int)(signed char)(d[i] >> 24);
    }
    acc += __shfl_xor(acc, 16, 64);
    acc += __shfl_xor(acc, 32, 64);
    if (lane < 16) cs[16 * blockIdx.x + lane] = acc;
}

// Owner records (see the OR_ slots above); grid (G, L), kOrSlots threads.
__global__ void __launch_bounds__(kOrSlots) build_ownrec_kernel(const DPrep *__restrict__ prep, const int *__restrict__ cs,
                                                               const float *__restrict__ P32, const double *__restrict__ PO,
                                                               int L, int C, int F, int G, u64 *__restrict__ ownrec) {
    const int g = blockIdx.x, l = blockIdx.y, t = threadIdx.x;
    const DPrep &p = prep[l];
    const int *csl = cs + (size_t)l * (6 * C + F);     // k v r o ffn_r [C each], ffn_k [F], ffn_v [C]
    const float *Pl = P32 + (size_t)l * kLnMats * C, *Pn = P32 + (size_t)(l + 1) * kLnMats * C;
    const double *POl = PO + (size_t)l * kLnMats * C, *POn = PO + (size_t)(l + 1) * kLnMats * C;
    const bool last = l + 1 == L;                      // the next row of the tables is the head: one product
    auto dbl = [](double v) { return (u64)__double_as_longlong(v); };
    auto pair = [](unsigned lo, unsigned hi) { return ((u64)hi << 32) | (u64)lo; };
    u64 v = 0;
    if (t < OR_FIELDS * 16) {
        const int field = t >> 4, c = 16 * g + (t & 15);
        switch (field) {
            case OR_DECAY: v = dbl(p.time_decay[c]); break;
            case OR_FIRST: v = dbl(p.time_first[c]); break;
            case OR_LN1W: v = dbl(p.ln1_w[c]); break;
            case OR_LN1B: v = dbl(p.ln1_b[c]); break;
            case OR_LN2W: v = dbl(p.ln2_w[c]); break;
            case OR_LN2B: v = dbl(p.ln2_b[c]); break;
            case OR_OFFO: v = dbl(p.offset_o[c]); break;
            case OR_RNGO_CSO: v = pair(__float_as_uint(p.range_o[c]), (unsigned)csl[3 * C + c]); break;
            case OR_CSK_CSV: v = pair((unsigned)csl[c], (unsigned)csl[C + c]); break;
            case OR_CSR_CSFR: v = pair((unsigned)csl[2 * C + c], (unsigned)csl[4 * C + c]); break;
            case OR_CSFV: v = pair((unsigned)csl[5 * C + F + c], 0u); break;
            case OR_POFK: v = dbl(POl[3 * C + c]); break;
            case OR_POFR: v = dbl(POl[4 * C + c]); break;
            case OR_PF: v = pair(__float_as_uint(Pl[3 * C + c]), __float_as_uint(Pl[4 * C + c])); break;
            case OR_PON0: v = dbl(POn[c]); break;
            case OR_PON1: v = last ? 0 : dbl(POn[C + c]); break;
            case OR_PON2: v = last ? 0 : dbl(POn[2 * C + c]); break;
            case OR_PN01: v = pair(__float_as_uint(Pn[c]), last ? 0u : __float_as_uint(Pn[C + c])); break;
            case OR_PN2: v = pair(last ? 0u : __float_as_uint(Pn[2 * C + c]), 0u); break;
            default: break;
        }
    } else if (t < kOrStatic) {
        const int i = (t - kOrOffV) & 63;              // lane of the ffn_k epilogue: tile i / 16, column i % 16
        const int f = 16 * (g + G * (i >> 4)) + (i & 15);
        if (t < kOrRngVCs) v = dbl(p.offset_v[f]);
        else v = pair(__float_as_uint(p.range_v[f]), (unsigned)csl[5 * C + f]);
    }
    ownrec[((size_t)l * G + g) * kOrSlots + t] = v;
}

// jt[g][l][16]: base address of job j of layer l for workgroup g (13 used); row L: the first head
// tiles of the workgroup (tiles past the end of the vocabulary point at tile 0, whose blocks stay
// hot in L2 and whose products are never used).  grid (G), any block size.
__global__ void build_jobtab_kernel(const DLayer *__restrict__ layers, const uint8_t *w_head, int L, int G, int NWG, int n_kb,
                                    int v_tiles, u64 *__restrict__ jt) {
    const int wg = blockIdx.x, g = (G / NWG) * wg;     // the workgroup's first group; the tiles of its next group follow at fixed strides
    const size_t TB = (size_t)n_kb * 1024;
    for (int i = threadIdx.x; i < (L + 1) * 16; i += blockDim.x) {
        const int l = i >> 4, j = i & 15;
        const uint8_t *p = w_head;
        if (l < L && j < kRealJobs) {
            const DLayer &Ly = layers[l];
            if (j <= 2) p = Ly.w[j] + (size_t)g * TB;
            else if (j == 3) p = Ly.w[MAT_ATT_O] + (size_t)g * TB;
            else if (j == 4) p = Ly.w[MAT_FFN_R] + (size_t)g * TB;
            else if (j <= 8) p = Ly.w[MAT_FFN_K] + (size_t)(g + G * (j - 5)) * TB;
            else p = Ly.w[MAT_FFN_V] + ((size_t)g * 4 + (j - 9)) * TB;
        } else if (l == L) {
            const int tile = wg + NWG * j;
            p = w_head + (size_t)(tile < v_tiles ? tile : 0) * TB;
        }
#ifdef RWKV_DIAG
        // Diagnostic build only (-DRWKV_DIAG, the one such switch of the library; results are wrong): every job
        // streams the same cache-resident tile, which takes HBM out of the picture and leaves the time of the
        // dependency chain between the workgroups.
        p = w_head;
#endif
        jt[(size_t)wg * (L + 1) * 16 + i] = (u64) reinterpret_cast<uintptr_t>(p);
    }
}

struct ConstArgs {
    int L, C;
    const DPrep *prep;
    const double *lnout_w, *lnout_b;
    const float *range_h;
    const double *offset_h;
    float *P32, *Q32;
    double *PO;
    DScal *sc;
};

// Token-independent constants of the LayerNorm-fed products; block l < L: layer l, block L: head.
__global__ void __launch_bounds__(kPrepThreads) build_consts_kernel(const ConstArgs a) {
    __shared__ double scr[8 * (kPrepThreads / 64)];
    const int C = a.C, l = blockIdx.x;
    const bool head = l == a.L;
    double sp[kLnMats] = {0, 0, 0, 0, 0}, sq[kLnMats] = {0, 0, 0, 0, 0};
    float mp[kLnMats] = {0, 0, 0, 0, 0}, mq[kLnMats] = {0, 0, 0, 0, 0};
    for (int c = threadIdx.x; c < C; c += kPrepThreads) {
#pragma unroll
        for (int m = 0; m < kLnMats; ++m) {
            if (head && m > 0) continue;
            double lw, mu, rg, of;
            if (head) {
                lw = a.lnout_w[c]; mu = 1.0; rg = (double)a.range_h[c]; of = a.offset_h[c];
            } else {
                const DPrep &p = a.prep[l];
                const bool att = m < 3;
                lw = att ? p.ln1_w[c] : p.ln2_w[c];
                mu = att ? p.att_mix[(size_t)m * C + c] : p.ffn_mix[(size_t)(m - 3) * C + c];
                rg = (double)p.range[m][c]; of = p.offset[m][c];
            }
            const float P = (float)(lw * mu * rg);
            const double PO = lw * mu * (of + 128.0 * rg);
            a.P32[((size_t)l * kLnMats + m) * C + c] = P;
            a.PO[((size_t)l * kLnMats + m) * C + c] = PO;
            sp[m] += PO;
            mp[m] = fmaxf(mp[m], fabsf(P));
            if (head) {
                const double base = a.lnout_b[c];
                const float Q = (float)(base * rg);
                a.Q32[((size_t)l * kLnMats + m) * C + c] = Q;
                sq[m] += base * (of + 128.0 * rg);
                mq[m] = fmaxf(mq[m], fabsf(Q));
            }
        }
    }
    prep_block_sum<kLnMats>(sp, scr);
    prep_block_sum<kLnMats>(sq, scr);
    prep_block_max<kLnMats>(mp, reinterpret_cast<float *>(scr));
    prep_block_max<kLnMats>(mq, reinterpret_cast<float *>(scr));
    if (threadIdx.x < kLnMats) {
        a.sc[l].sumPO[threadIdx.x] = sp[threadIdx.x];
        a.sc[l].maxP[threadIdx.x] = mp[threadIdx.x];
        if (head) { a.sc[l].sumQO[threadIdx.x] = sq[threadIdx.x]; a.sc[l].maxQ[threadIdx.x] = mq[threadIdx.x]; }
    }
}

// ---------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------
bool decode_supported(int64_t L, int64_t C, int64_t F, int64_t V) {
    if (L <= 0 || V <= 0 || F != 4 * C) return false;
    // one 16-column tile per workgroup, all workgroups resident: C/16 <= 256 CUs
    if (!(C == 1024 || C == 2048 || C == 2560 || C == 4096 || C == 5120)) return false;
    // the column sums of a workgroup's head tiles are staged by its front threads into half an owner record
    const int64_t NWG = decode_workgroups(C), head_rounds = ((V + 15) / 16 + NWG - 1) / NWG, front_threads = (C == 2560 || C == 5120) ? 512 : 256;
    return head_rounds * 16 <= kHeadCsPerThread * front_threads && head_rounds * 16 * (int64_t)sizeof(int) <= kOrSlots * 8;
}

int64_t decode_workgroups(int64_t C) { return C > 4096 ? C / 32 : C / 16; }
int64_t decode_helper_workgroups(int64_t C) { return C == 2560 ? HelperShape<5>::NH : 0; }

unsigned decode_epochs_per_token(int64_t L) { return (unsigned)(4 * L + 1); }

// 8-byte words of the exchange buffers (X, XR, A, AR, H, HR), one contiguous range starting at X
static size_t exchange_words(int64_t C, int64_t F) { return (size_t)(2 * C + F + (kLnRows + 6) * (C / 16)); }

namespace {
struct BlockPlan {
    size_t layers, prep, P32, Q32, PO, sc, X0, cs, ownrec, jt, scp, amax, abort, total;
    size_t cs_layer_ints;
};
BlockPlan plan_block(int64_t L, int64_t C, int64_t F, int64_t V) {
    BlockPlan p;
    size_t off = 0;
    auto take = [&](size_t bytes) { const size_t o = off; off += (size_t)round_up((int64_t)bytes, 256); return o; };
    const size_t G = (size_t)C / 16;
    p.layers = take((size_t)L * sizeof(DLayer));
    p.prep = take((size_t)L * sizeof(DPrep));
    p.P32 = take((size_t)(L + 1) * kLnMats * C * sizeof(float));
    p.Q32 = take((size_t)(L + 1) * kLnMats * C * sizeof(float));
    p.PO = take((size_t)(L + 1) * kLnMats * C * sizeof(double));
    p.sc = take((size_t)(L + 1) * sizeof(DScal));
    p.X0 = take((size_t)C * sizeof(double));
    p.cs_layer_ints = (size_t)(6 * C + F);
    p.cs = take(((size_t)L * p.cs_layer_ints + (size_t)round_up(V, 16)) * sizeof(int));
    p.ownrec = take((size_t)L * G * kOrSlots * sizeof(u64));
    p.jt = take(G * (size_t)(L + 1) * 16 * sizeof(u64));
    p.scp = take((size_t)L * (C / 512) * sizeof(DScal));
    p.amax = take((size_t)G * (sizeof(double) + sizeof(int)));
    p.abort = take(256);
    p.total = off;
    return p;
}
}  // namespace

size_t decode_block_bytes(int64_t L, int64_t C, int64_t F, int64_t V) { return plan_block(L, C, F, V).total; }
size_t decode_exchange_bytes(int64_t C, int64_t F) { return (size_t)round_up((int64_t)(exchange_words(C, F) * sizeof(u64)), 256); }

int decode_setup(void *block, void *exchange, const DSetup &s, DModel *dm, DecodeBuffers *db) {
    const int64_t L = s.L, C = s.C, F = s.F, V = s.V;
    if (!decode_supported(L, C, F, V)) return set_error(RWKV_ERR_SIZE, "decode_setup: unsupported shape");
    const BlockPlan p = plan_block(L, C, F, V);
    unsigned char *base = static_cast<unsigned char *>(block);
    const size_t G = (size_t)C / 16;
    int *cs = reinterpret_cast<int *>(base + p.cs);
    std::vector<DLayer> tab((size_t)L);
    std::vector<DPrep> prep((size_t)L);
    const int c_kb = (int)(C / 64), f_kb = (int)(F / 64);
    for (int64_t l = 0; l < L; ++l) {
        const DLayerSrc &src = s.layers[l];
        DLayer &t = tab[(size_t)l];
        const DQ *q[MAT_COUNT];
        q[MAT_ATT_K] = &src.att_k; q[MAT_ATT_V] = &src.att_v; q[MAT_ATT_R] = &src.att_r; q[MAT_ATT_O] = &src.att_o;
        q[MAT_FFN_R] = &src.ffn_r; q[MAT_FFN_K] = &src.ffn_k; q[MAT_FFN_V] = &src.ffn_v;
        int *csl = cs + (size_t)l * p.cs_layer_ints;
        t.pad = nullptr;
        for (int i = 0; i < MAT_COUNT; ++i) {
            t.w[i] = q[i]->w16;
            const int n_out = i == MAT_FFN_K ? (int)F : (int)C;
            const int n_kb = i == MAT_FFN_V ? f_kb : c_kb;
            // order inside the layer's column-sum slab: k v r o ffn_r [C each], ffn_k [F], ffn_v [C]
            int *dst = csl + (i <= MAT_FFN_R ? (size_t)i * C : (i == MAT_FFN_K ? (size_t)5 * C : (size_t)5 * C + F));
            hipLaunchKernelGGL(colsum_m16_kernel, dim3((unsigned)(n_out / 16)), dim3(64), 0, nullptr, q[i]->w16, n_kb, dst);
        }
        DPrep &pr = prep[(size_t)l];
        pr.ln1_w = src.ln1_w; pr.ln1_b = src.ln1_b; pr.ln2_w = src.ln2_w; pr.ln2_b = src.ln2_b;
        pr.att_mix = src.att_mix; pr.ffn_mix = src.ffn_mix;
        pr.time_decay = src.time_decay; pr.time_first = src.time_first;
        pr.range_o = src.att_o.range; pr.offset_o = src.att_o.offset;
        pr.range_v = src.ffn_v.range; pr.offset_v = src.ffn_v.offset;
        const DQ *lm[kLnMats] = {&src.att_k, &src.att_v, &src.att_r, &src.ffn_k, &src.ffn_r};
        for (int m = 0; m < kLnMats; ++m) { pr.range[m] = lm[m]->range; pr.offset[m] = lm[m]->offset; }
    }
    RWKV_CHECK_LAUNCH("colsum_m16_kernel");
    int *cs_head = cs + (size_t)L * p.cs_layer_ints;
    hipLaunchKernelGGL(colsum_m16_kernel, dim3((unsigned)ceil_div(V, 16)), dim3(64), 0, nullptr, s.head.w16, c_kb, cs_head);
    RWKV_CHECK_LAUNCH("colsum_m16_kernel");
    RWKV_CHECK_HIP(hipMemcpy(base + p.layers, tab.data(), (size_t)L * sizeof(DLayer), hipMemcpyHostToDevice));
    RWKV_CHECK_HIP(hipMemcpy(base + p.prep, prep.data(), (size_t)L * sizeof(DPrep), hipMemcpyHostToDevice));

    dm->L = (int)L; dm->C = (int)C; dm->F = (int)F; dm->V = (int)V; dm->G = (int)G; dm->NWG = (int)decode_workgroups(C);
    dm->emb = s.emb; dm->ln0_w = s.ln0_w; dm->ln0_b = s.ln0_b;
    dm->w_head = s.head.w16; dm->cs = cs; dm->cs_head = cs_head;
    dm->ownrec = reinterpret_cast<const u64 *>(base + p.ownrec);
    dm->scp = reinterpret_cast<DScal *>(base + p.scp);
    dm->amax_val = reinterpret_cast<double *>(base + p.amax);
    dm->amax_idx = reinterpret_cast<int *>(base + p.amax + (size_t)G * sizeof(double));
    dm->layers = reinterpret_cast<const DLayer *>(base + p.layers);
    dm->prep = reinterpret_cast<const DPrep *>(base + p.prep);
    dm->P32 = reinterpret_cast<float *>(base + p.P32);
    dm->Q32 = reinterpret_cast<float *>(base + p.Q32);
    dm->PO = reinterpret_cast<double *>(base + p.PO);
    dm->sc = reinterpret_cast<DScal *>(base + p.sc);
    dm->X0 = reinterpret_cast<double *>(base + p.X0);

    ConstArgs ca;
    dm->jt = reinterpret_cast<const u64 *>(base + p.jt);
    hipLaunchKernelGGL(build_jobtab_kernel, dim3((unsigned)dm->NWG), dim3(256), 0, nullptr, dm->layers, s.head.w16, (int)L,
                       (int)G, dm->NWG, c_kb, (int)ceil_div(V, 16), reinterpret_cast<u64 *>(base + p.jt));
    RWKV_CHECK_LAUNCH("build_jobtab_kernel");
    ca.L = (int)L; ca.C = (int)C; ca.prep = dm->prep;
    ca.lnout_w = s.lnout_w; ca.lnout_b = s.lnout_b; ca.range_h = s.head.range; ca.offset_h = s.head.offset;
    ca.P32 = dm->P32; ca.Q32 = dm->Q32; ca.PO = dm->PO; ca.sc = dm->sc;
    hipLaunchKernelGGL(build_consts_kernel, dim3((unsigned)(L + 1)), dim3(kPrepThreads), 0, nullptr, ca);
    RWKV_CHECK_LAUNCH("build_consts_kernel");
    hipLaunchKernelGGL(build_ownrec_kernel, dim3((unsigned)G, (unsigned)L), dim3(kOrSlots), 0, nullptr, dm->prep, dm->cs,
                       dm->P32, dm->PO, (int)L, (int)C, (int)F, (int)G, reinterpret_cast<u64 *>(base + p.ownrec));
    RWKV_CHECK_LAUNCH("build_ownrec_kernel");

    u64 *x = static_cast<u64 *>(exchange);
    db->X = x; x += C;
    db->XR = x; x += (size_t)kLnRows * G;
    db->A = x; x += C;
    db->AR = x; x += 3 * G;
    db->H = x; x += F;
    db->HR = x;
    db->abort_flag = reinterpret_cast<unsigned *>(base + p.abort);
    db->trace = nullptr;
    RWKV_CHECK_HIP(hipDeviceSynchronize());
    return RWKV_OK;
}

__global__ void __launch_bounds__(256) fill_zero_kernel(u64 *p, size_t n) {
    for (size_t i = (size_t)blockIdx.x * blockDim.x + threadIdx.x; i < n; i += (size_t)gridDim.x * blockDim.x) p[i] = 0;
}

int decode_clear_exchange(hipStream_t st, const DModel &m, const DecodeBuffers &b) {
    hipLaunchKernelGGL(fill_zero_kernel, dim3(64), dim3(256), 0, st, b.X, exchange_words(m.C, m.F));
    RWKV_CHECK_LAUNCH("fill_zero_kernel");
    return RWKV_OK;
}

constexpr int kMaxDevices = 64;

template <int KW, int FW>
static int launch_one(hipStream_t st, const DArgs &args, bool with_prep) {
    constexpr bool HELP = HelperShape<KW>::NH > 0;
    const bool trace = args.b.trace != nullptr;
    const int lds = DecodeLds<KW, FW, HELP>::total(args.m.L, trace);
    if (lds > 160 * 1024) return set_error(RWKV_ERR_SIZE, "decode kernel: %d layers need %d bytes of LDS", args.m.L, lds);
    // the dynamic LDS limit is a per-device attribute of the function; it only ever grows
    static std::mutex mu;
    static int configured[kMaxDevices] = {};
    int dev = 0;
    RWKV_CHECK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kMaxDevices) return set_error(RWKV_ERR_DEVICE, "decode kernel: device index %d", dev);
    {
        std::lock_guard<std::mutex> lock(mu);
        if (configured[dev] < lds) {
            RWKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_kernel<KW, FW, false, HELP>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            RWKV_CHECK_HIP(hipFuncSetAttribute(reinterpret_cast<const void *>(&decode_kernel<KW, FW, true, HELP>),
                                               hipFuncAttributeMaxDynamicSharedMemorySize, lds));
            configured[dev] = lds;
        }
    }
    if (with_prep) {
        hipLaunchKernelGGL(prep_kernel, dim3((unsigned)(args.m.L * (args.m.C / kPrepThreads) + 1)), dim3(kPrepThreads), 0, st, args);
        RWKV_CHECK_LAUNCH("prep_kernel");
    }
    // owner workgroups first, then the helpers: every one of them is resident at once (one per compute unit)
    const dim3 grid((unsigned)(args.m.NWG + HelperShape<KW>::NH));
    if (trace)
        hipLaunchKernelGGL((decode_kernel<KW, FW, true, HELP>), grid, dim3((FW + kBW) * 64), lds, st, args);
    else
        hipLaunchKernelGGL((decode_kernel<KW, FW, false, HELP>), grid, dim3((FW + kBW) * 64), lds, st, args);
    RWKV_CHECK_LAUNCH("decode_kernel");
    return RWKV_OK;
}

static int launch_step(hipStream_t st, const DArgs &args, bool with_prep) {
    switch (args.m.C) {
        case 1024: return launch_one<2, 4>(st, args, with_prep);
        case 2048: return launch_one<4, 4>(st, args, with_prep);
        case 2560: return launch_one<5, 8>(st, args, with_prep);
        case 4096: return launch_one<8, 4>(st, args, with_prep);
        case 5120: return launch_one<10, 8>(st, args, with_prep);
        default: return set_error(RWKV_ERR_SIZE, "decode kernel: n_embd %d not supported", args.m.C);
    }
}

int decode_launch(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                  const int64_t *token, double *state, double *logits) {
    DArgs args;
    args.m = m; args.b = b; args.epoch0 = epoch0; args.token = token; args.state = state; args.logits = logits;
    args.stop = nullptr; args.spin_limit = kSpinLimit;
    return launch_step(st, args, true);
}

// One token step with events recorded on the stream right before and right after the token kernel itself (the
// preparation launch stays outside the pair): the kernel's own duration, for measurements.
int decode_launch_bracketed(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, const int64_t *token,
                            double *state, double *logits, hipEvent_t before, hipEvent_t after) {
    DArgs args;
    args.m = m; args.b = b; args.epoch0 = epoch0; args.token = token; args.state = state; args.logits = logits;
    args.stop = nullptr; args.spin_limit = kSpinLimit;
    hipLaunchKernelGGL(prep_kernel, dim3((unsigned)(m.L * (m.C / kPrepThreads) + 1)), dim3(kPrepThreads), 0, st, args);
    RWKV_CHECK_LAUNCH("prep_kernel");
    RWKV_CHECK_HIP(hipEventRecord(before, st));
    const int rc = launch_step(st, args, false);
    if (rc) return rc;
    RWKV_CHECK_HIP(hipEventRecord(after, st));
    return RWKV_OK;
}

// A token step whose input is never published (no preparation launch under this epoch) and whose waits give up
// after spin_limit polls: every workgroup runs into its bounded wait, raises the abort flag and leaves.  Exercises
// the failure path without anything that could hang: the limit is a few hundred polls.
int decode_launch_unfed(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, double *state, double *logits,
                        unsigned spin_limit) {
    DArgs args;
    args.m = m; args.b = b; args.epoch0 = epoch0; args.token = nullptr; args.state = state; args.logits = logits;
    args.stop = nullptr; args.spin_limit = spin_limit;
    return launch_step(st, args, false);
}

int decode_launch_sampled(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0, int64_t *tokens, int64_t n,
                          double *state, double *logits, SampleArgs sa) {
    DArgs args;
    args.m = m; args.b = b; args.state = state; args.logits = logits;
    args.stop = sa.stop_flag; args.spin_limit = kSpinLimit;
    sa.logits = logits; sa.V = m.V;
    const unsigned ept = decode_epochs_per_token(m.L);
    for (int64_t i = 0; i < n; ++i) {
        args.epoch0 = epoch0 + (unsigned)i * ept;
        args.token = tokens + i;
        const int rc = launch_step(st, args, true);      // preparation (reads tokens[i]) + the token kernel
        if (rc) return rc;
        sa.out_token = tokens + i + 1;
        const int rs = sample_launch(st, sa);
        if (rs) return rs;
        sa.counter += 1;
    }
    return RWKV_OK;
}

int decode_launch_greedy(hipStream_t st, const DModel &m, const DecodeBuffers &b, unsigned epoch0,
                         int64_t *tokens, int64_t n, double *state, double *logits) {
    DArgs args;
    args.m = m; args.b = b; args.state = state; args.logits = logits;
    args.stop = nullptr; args.spin_limit = kSpinLimit;
    const unsigned ept = decode_epochs_per_token(m.L);
    for (int64_t i = 0; i < n; ++i) {
        args.epoch0 = epoch0 + (unsigned)i * ept;
        args.token = tokens + i;
        const int rc = launch_step(st, args, i == 0);
        if (rc) return rc;
        // argmax -> tokens[i + 1], and the preparation of step i + 1 (harmless after the last step:
        // the next forward call prepares again under the same epoch)
        args.epoch0 += ept;
        hipLaunchKernelGGL(next_token_kernel, dim3((unsigned)(m.L * (m.C / kPrepThreads) + 1)),
                           dim3(kPrepThreads), 0, st, args, tokens + i + 1);
        RWKV_CHECK_LAUNCH("next_token_kernel");
    }
    return RWKV_OK;
}

}  // namespace rwkv
