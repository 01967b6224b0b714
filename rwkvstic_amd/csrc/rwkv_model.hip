// Whole-model forward for the FASTQUANT RWKV-4 path (reference
// agnostic/backends/opt.py:61-76, modules/block.py:56-102).
//
// One token step is a chain of dependent "phases"; each phase is one launch
// whose workgroups own 8-column tiles of the phase's matrices:
//
//   embed    x = ln0(emb[token])
//   per layer
//     att_kvr  prologue: xy = ln1(x); mix_{k,v,r} = lerp(shift, xy); xs = fp32(mix*range)
//              product : k, v, r columns of the tile
//              epilogue: r = sigmoid(r); one WKV step on the tile's channels;
//                        att_in = wkv * r
//     att_out  prologue: xs = fp32(att_in*range)
//              epilogue: x += W_o(att_in)              ; commit att shift state
//     ffn_rk   prologue: ddd = ln2(x); mix_{k,r}
//              epilogue: rf = sigmoid(.) | h = relu(.)^2
//     ffn_v    prologue: xs = fp32(h*range)
//              epilogue: x = W_v(h)*rf + x             ; commit ffn shift state
//   head     prologue: ln_out(x)                       ; logits
//
// Numeric types follow the reference: residual stream, LayerNorm, token shift,
// lerp, zero-point dot products and state are float64 (block.py:37-47,
// layernorm.py:7-10); the matrix term is fp32(x*range) times uint8 codes with
// float32 accumulation (matmul.py:58,131); WKV runs in float32 in the
// max-shifted form.
#include "rwkv_common.h"
#include "rwkv_decode.h"
#include "rwkv_rows.h"

#include <mutex>
#include <new>
#include <string>
#include <vector>

namespace rwkv {

constexpr int kMaxCPT = 24;   // channels per thread in the LayerNorm prologue: C <= 6144
constexpr int kXsBudgetBlocks = 96;   // 96 blocks * 128 rows * 4 B = 48 KiB of staged activations

struct QMatDev {
    const uint8_t *packed;
    const float *range;
    const double *offset;
    int n_in, n_out, n_kb;
};

static QMatDev to_dev(const rwkv_qmat &q) {
    QMatDev d;
    d.packed = q.packed; d.range = q.range; d.offset = q.offset;
    d.n_in = (int)q.n_in; d.n_out = (int)q.n_out; d.n_kb = (int)ceil_div(q.n_in, kBlockRows);
    return d;
}

// ---------------------------------------------------------------------------
// LayerNorm over C channels held in registers: thread t owns channels
// t, t+256, ...  (layernorm.py:15-20: biased variance, eps inside the sqrt,
// division by the standard deviation).  val[] is replaced by the normalised
// values.  red: LDS scratch of kWaves doubles.
// ---------------------------------------------------------------------------
__device__ __forceinline__ void layernorm_regs(int C, double (&val)[kMaxCPT],
                                               const double *__restrict__ w,
                                               const double *__restrict__ b, double *red) {
    double s[1] = {0.0};
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < C) s[0] += val[i];
    }
    block_sum<1>(s, red);
    const double mean = s[0] / (double)C;
    double q[1] = {0.0};
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < C) { val[i] -= mean; q[0] += val[i] * val[i]; }
    }
    block_sum<1>(q, red);
    const double sd = sqrt(q[0] / (double)C + 1e-5);
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < C) val[i] = w[c] * (val[i] / sd) + b[c];
    }
}

// ---------------------------------------------------------------------------
// embed: x = ln0(emb[token])      (emb.py:9, opt.py:63-64)
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(kThreads)
embed_ln0_kernel(const int64_t *__restrict__ token, int V, int C, const float *__restrict__ emb,
                 const double *__restrict__ w, const double *__restrict__ b, double *__restrict__ x) {
    __shared__ double red[kWaves];
    int64_t tok = token[0];
    if (tok < 0) tok = 0;
    if (tok >= V) tok = V - 1;
    double val[kMaxCPT];
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        val[i] = c < C ? (double)emb[(size_t)tok * C + c] : 0.0;
    }
    layernorm_regs(C, val, w, b, red);
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < C) x[c] = val[i];
    }
}

// ---------------------------------------------------------------------------
// att_kvr
// ---------------------------------------------------------------------------
struct AttKvrArgs {
    int C;
    const double *x;
    const double *ln_w, *ln_b;
    const double *mix;          // [3, C] k, v, r
    double *state;              // this layer's [5, C]
    QMatDev k, v, r;
    const double *time_decay, *time_first;
    double *att_in;             // out: wkv * sigmoid(r)
    double *xy_tmp;             // out: ln1(x), committed to state[0] by att_out
};

__global__ void __launch_bounds__(kThreads)
att_kvr_kernel(const AttKvrArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int C = a.C;
    const int n_kb = a.k.n_kb;
    const int in_pad = n_kb * kBlockRows;
    float *xs = reinterpret_cast<float *>(smem);                         // [3][in_pad]
    double *dred = reinterpret_cast<double *>(xs + 3 * (size_t)in_pad);  // [3*kWaves]
    float *fred = reinterpret_cast<float *>(dred + 3 * kWaves);          // [3*kWaves*8]
    const int ct = blockIdx.x;

    double val[kMaxCPT];
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        val[i] = c < C ? a.x[c] : 0.0;
    }
    layernorm_regs(C, val, a.ln_w, a.ln_b, dred);

    double zp[3] = {0.0, 0.0, 0.0};
    const QMatDev *mats[3] = {&a.k, &a.v, &a.r};
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < in_pad) {
            if (c < C) {
                const double xy = val[i];
                const double sh = a.state[c];                 // state[0]: previous token's ln1 output
#pragma unroll
                for (int m = 0; m < 3; ++m) {
                    const double mu = a.mix[(size_t)m * C + c];
                    const double mixed = xy * mu + sh * (1.0 - mu);          // block.py:67
                    xs[(size_t)m * in_pad + c] = (float)(mixed * (double)mats[m]->range[c]);  // matmul.py:131
                    zp[m] += mixed * mats[m]->offset[c];
                }
                if (c / kTileCols == ct) a.xy_tmp[c] = xy;
            } else {
#pragma unroll
                for (int m = 0; m < 3; ++m) xs[(size_t)m * in_pad + c] = 0.f;
            }
        }
    }
    block_sum<3>(zp, dred);   // also orders the xs writes before the reads below

    const uint8_t *const wtile[3] = {a.k.packed + (size_t)ct * n_kb * kBlockBytes,
                                     a.v.packed + (size_t)ct * n_kb * kBlockBytes,
                                     a.r.packed + (size_t)ct * n_kb * kBlockBytes};
    const float *const xsp[3] = {xs, xs + in_pad, xs + 2 * (size_t)in_pad};
    float acc[3][1] = {{0.f}, {0.f}, {0.f}};
    tile_accumulate<3, 1>(wtile, xsp, in_pad, 0, n_kb, acc);
    float out[3][1];
    tile_reduce<3, 1>(acc, fred, out);

    if (threadIdx.x < kTileCols) {
        const int c = ct * kTileCols + threadIdx.x;
        if (c < C) {
            const double kd = (double)out[0][0] + zp[0];      // matmul.py:59-62
            const double vd = (double)out[1][0] + zp[1];
            const double rd = (double)out[2][0] + zp[2];
            const float r = sigmoid_f32((float)rd);           // block.py:72
            float aa = (float)a.state[2 * (size_t)C + c];
            float bb = (float)a.state[3 * (size_t)C + c];
            double pp = a.state[4 * (size_t)C + c];
            const float y = wkv_step_f32(a.time_decay[c], a.time_first[c], (float)kd, (float)vd, aa, bb, pp);
            a.state[2 * (size_t)C + c] = (double)aa;
            a.state[3 * (size_t)C + c] = (double)bb;
            a.state[4 * (size_t)C + c] = pp;
            a.att_in[c] = (double)(y * r);                    // block.py:78
        }
    }
}

// ---------------------------------------------------------------------------
// att_out / ffn_v: input vector already formed by the previous phase.
// ---------------------------------------------------------------------------
struct VecMatArgs {
    QMatDev w;
    const double *vin;        // [n_in]
    double *x;                // residual stream [n_out], updated in place
    const double *gate;       // ffn_v: rf [n_out]; att_out: null
    const double *shift_src;  // ln output of this token for the tile's channels
    double *shift_dst;        // state row to commit it to
    int kc_blocks;
};

__global__ void __launch_bounds__(kThreads)
vec_matvec_kernel(const VecMatArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int n_kb = a.w.n_kb, n_in = a.w.n_in;
    const int kc_rows = a.kc_blocks * kBlockRows;
    float *xs = reinterpret_cast<float *>(smem);                  // [kc_rows]
    double *dred = reinterpret_cast<double *>(xs + kc_rows);      // [kWaves]
    float *fred = reinterpret_cast<float *>(dred + kWaves);       // [kWaves*8]
    const int ct = blockIdx.x;
    const uint8_t *const wtile[1] = {a.w.packed + (size_t)ct * n_kb * kBlockBytes};
    const float *const xsp[1] = {xs};
    float acc[1][1] = {{0.f}};
    double zp[1] = {0.0};
    for (int kb0 = 0; kb0 < n_kb; kb0 += a.kc_blocks) {
        const int kb1 = min(kb0 + a.kc_blocks, n_kb);
        const int j0 = kb0 * kBlockRows;
        for (int i = threadIdx.x; i < (kb1 - kb0) * kBlockRows; i += kThreads) {
            const int j = j0 + i;
            float v = 0.f;
            if (j < n_in) {
                const double h = a.vin[j];
                v = (float)(h * (double)a.w.range[j]);
                zp[0] += h * a.w.offset[j];
            }
            xs[i] = v;
        }
        __syncthreads();
        tile_accumulate<1, 1>(wtile, xsp, kc_rows, kb0, kb1, acc);
        __syncthreads();
    }
    block_sum<1>(zp, dred);
    float out[1][1];
    tile_reduce<1, 1>(acc, fred, out);
    if (threadIdx.x < kTileCols) {
        const int c = ct * kTileCols + threadIdx.x;
        if (c < a.w.n_out) {
            const double y = (double)out[0][0] + zp[0];
            if (a.gate) a.x[c] = y * a.gate[c] + a.x[c];     // block.py:100
            else        a.x[c] = a.x[c] + y;                 // block.py:80
            a.shift_dst[c] = a.shift_src[c];                 // block.py:63-64 / 87-88
        }
    }
}

// ---------------------------------------------------------------------------
// ffn_rk / head: LayerNorm prologue, one matrix per tile.
// ---------------------------------------------------------------------------
enum { EPI_LOGITS = 0, EPI_FFN = 1 };

struct LnMatArgs {
    int C, mode;
    const double *x;
    const double *ln_w, *ln_b;
    // EPI_FFN: tiles [0, C/8) belong to `r` (mix row 1), the rest to `k` (mix row 0)
    const double *mix;          // [2, C] k, r   (null for the head)
    const double *shift;        // state[1]
    QMatDev k, r;               // head: only k is used
    double *out_k;              // EPI_FFN: h = relu(.)^2 [F]; EPI_LOGITS: logits [V]
    double *out_r;              // EPI_FFN: rf = sigmoid(.) [C]
    double *ln_tmp;             // EPI_FFN: ln2(x) for the tile's channels
};

__global__ void __launch_bounds__(kThreads)
ln_matvec_kernel(const LnMatArgs a) {
    extern __shared__ __align__(16) unsigned char smem[];
    const int C = a.C;
    const int n_kb = a.k.n_kb;
    const int in_pad = n_kb * kBlockRows;
    float *xs = reinterpret_cast<float *>(smem);                 // [in_pad]
    double *dred = reinterpret_cast<double *>(xs + in_pad);      // [kWaves]
    float *fred = reinterpret_cast<float *>(dred + kWaves);      // [kWaves*8]

    int ct = blockIdx.x;
    bool is_r = false;
    if (a.mode == EPI_FFN) {
        const int r_tiles = (a.r.n_out + kTileCols - 1) / kTileCols;
        if (ct < r_tiles) is_r = true; else ct -= r_tiles;
    }
    const QMatDev &W = is_r ? a.r : a.k;

    double val[kMaxCPT];
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        val[i] = c < C ? a.x[c] : 0.0;
    }
    layernorm_regs(C, val, a.ln_w, a.ln_b, dred);

    double zp[1] = {0.0};
#pragma unroll
    for (int i = 0; i < kMaxCPT; ++i) {
        const int c = threadIdx.x + i * kThreads;
        if (c < in_pad) {
            float v = 0.f;
            if (c < C) {
                double mixed = val[i];
                if (a.mix) {
                    const double mu = a.mix[(size_t)(is_r ? 1 : 0) * C + c];
                    mixed = val[i] * mu + a.shift[c] * (1.0 - mu);      // block.py:91
                    if (is_r && c / kTileCols == ct) a.ln_tmp[c] = val[i];
                }
                v = (float)(mixed * (double)W.range[c]);
                zp[0] += mixed * W.offset[c];
            }
            xs[c] = v;
        }
    }
    block_sum<1>(zp, dred);

    const uint8_t *const wtile[1] = {W.packed + (size_t)ct * n_kb * kBlockBytes};
    const float *const xsp[1] = {xs};
    float acc[1][1] = {{0.f}};
    tile_accumulate<1, 1>(wtile, xsp, in_pad, 0, n_kb, acc);
    float out[1][1];
    tile_reduce<1, 1>(acc, fred, out);
    if (threadIdx.x < kTileCols) {
        const int k = ct * kTileCols + threadIdx.x;
        if (k < W.n_out) {
            const double y = (double)out[0][0] + zp[0];
            if (a.mode == EPI_LOGITS) a.out_k[k] = y;
            else if (is_r) a.out_r[k] = (double)sigmoid_f32((float)y);   // block.py:95
            else { const double h = y > 0.0 ? y : 0.0; a.out_k[k] = h * h; }  // block.py:97-98
        }
    }
}

}  // namespace rwkv

using namespace rwkv;

// ---------------------------------------------------------------------------
// host side
// ---------------------------------------------------------------------------
struct rwkv_model {
    rwkv_model_desc d;
    std::vector<rwkv_layer_desc> layers;
    // single-token persistent kernel (absent when the shape or layouts do not allow it)
    bool fused = false;
    int device = 0;
    rwkv::DModel dm{};
    rwkv::DecodeBuffers db{};
    void *dev_block = nullptr;     // one allocation: layer table, constants, abort flag
    void *xchg_block = nullptr;    // exchange vectors (uncached device memory from the pool below)
    size_t xchg_bytes = 0;
    unsigned epoch = 0;
};

namespace {

struct Workspace {
    double *x, *xy_tmp, *ddd_tmp, *att_in, *rf, *h;
};

size_t ws_doubles(int64_t C, int64_t F) { return (size_t)(5 * C + F); }

Workspace carve(void *ws, int64_t C, int64_t F) {
    Workspace w;
    double *p = static_cast<double *>(ws);
    w.x = p; p += C;
    w.xy_tmp = p; p += C;
    w.ddd_tmp = p; p += C;
    w.att_in = p; p += C;
    w.rf = p; p += C;
    w.h = p; p += F;
    return w;
}

int check_qmat(const rwkv_qmat &q, int64_t n_in, int64_t n_out, const char *name) {
    if (!q.packed || !q.range || !q.offset)
        return set_error(RWKV_ERR_ARG, "rwkv_model_create: %s has a null pointer", name);
    if (q.n_in != n_in || q.n_out != n_out)
        return set_error(RWKV_ERR_SIZE, "rwkv_model_create: %s is %lldx%lld, expected %lldx%lld", name,
                         (long long)q.n_in, (long long)q.n_out, (long long)n_in, (long long)n_out);
    if (reinterpret_cast<uintptr_t>(q.packed) % 16)
        return set_error(RWKV_ERR_ALIGN, "rwkv_model_create: %s.packed must be 16-byte aligned", name);
    if (reinterpret_cast<uintptr_t>(q.range) % 4 || reinterpret_cast<uintptr_t>(q.offset) % 8)
        return set_error(RWKV_ERR_ALIGN, "rwkv_model_create: %s.range/offset misaligned", name);
    return RWKV_OK;
}

// One token through every layer; logits only when `with_head`.
int step_token(rwkv_model *m, hipStream_t st, const int64_t *token, double *state, double *logits,
               const Workspace &w, bool with_head) {
    const rwkv_model_desc &d = m->d;
    const int C = (int)d.n_embd, F = (int)d.n_ffn, V = (int)d.n_vocab;
    const int c_tiles = (int)ceil_div(C, kTileCols), f_tiles = (int)ceil_div(F, kTileCols);
    const int c_kb = (int)ceil_div(C, kBlockRows), f_kb = (int)ceil_div(F, kBlockRows);
    const size_t red_bytes = 3 * kWaves * 8 + 3 * kWaves * 8 * 4;

    hipLaunchKernelGGL(embed_ln0_kernel, dim3(1), dim3(kThreads), 0, st, token, V, C, d.emb, d.ln0_w, d.ln0_b, w.x);
    for (int64_t l = 0; l < d.n_layer; ++l) {
        const rwkv_layer_desc &L = m->layers[l];
        double *sl = state + (size_t)l * 5 * C;
        AttKvrArgs a;
        a.C = C; a.x = w.x; a.ln_w = L.ln1_w; a.ln_b = L.ln1_b; a.mix = L.att_mix; a.state = sl;
        a.k = to_dev(L.att_k); a.v = to_dev(L.att_v); a.r = to_dev(L.att_r);
        a.time_decay = L.time_decay; a.time_first = L.time_first; a.att_in = w.att_in; a.xy_tmp = w.xy_tmp;
        hipLaunchKernelGGL(att_kvr_kernel, dim3(c_tiles), dim3(kThreads),
                           3 * (size_t)c_kb * kBlockRows * 4 + red_bytes, st, a);

        VecMatArgs o;
        o.w = to_dev(L.att_o); o.vin = w.att_in; o.x = w.x; o.gate = nullptr;
        o.shift_src = w.xy_tmp; o.shift_dst = sl; o.kc_blocks = c_kb < kXsBudgetBlocks ? c_kb : kXsBudgetBlocks;
        hipLaunchKernelGGL(vec_matvec_kernel, dim3(c_tiles), dim3(kThreads),
                           (size_t)o.kc_blocks * kBlockRows * 4 + red_bytes, st, o);

        LnMatArgs f;
        f.C = C; f.mode = EPI_FFN; f.x = w.x; f.ln_w = L.ln2_w; f.ln_b = L.ln2_b; f.mix = L.ffn_mix;
        f.shift = sl + C; f.k = to_dev(L.ffn_k); f.r = to_dev(L.ffn_r);
        f.out_k = w.h; f.out_r = w.rf; f.ln_tmp = w.ddd_tmp;
        hipLaunchKernelGGL(ln_matvec_kernel, dim3(c_tiles + f_tiles), dim3(kThreads),
                           (size_t)c_kb * kBlockRows * 4 + red_bytes, st, f);

        VecMatArgs v;
        v.w = to_dev(L.ffn_v); v.vin = w.h; v.x = w.x; v.gate = w.rf;
        v.shift_src = w.ddd_tmp; v.shift_dst = sl + C; v.kc_blocks = f_kb < kXsBudgetBlocks ? f_kb : kXsBudgetBlocks;
        hipLaunchKernelGGL(vec_matvec_kernel, dim3(c_tiles), dim3(kThreads),
                           (size_t)v.kc_blocks * kBlockRows * 4 + red_bytes, st, v);
    }
    if (with_head) {
        LnMatArgs h;
        h.C = C; h.mode = EPI_LOGITS; h.x = w.x; h.ln_w = d.ln_out_w; h.ln_b = d.ln_out_b; h.mix = nullptr;
        h.shift = nullptr; h.k = to_dev(d.head); h.r = h.k; h.out_k = logits; h.out_r = nullptr; h.ln_tmp = nullptr;
        hipLaunchKernelGGL(ln_matvec_kernel, dim3((unsigned)ceil_div(V, kTileCols)), dim3(kThreads),
                           (size_t)c_kb * kBlockRows * 4 + red_bytes, st, h);
    }
    RWKV_CHECK_LAUNCH("token step");
    return RWKV_OK;
}

int check_forward_args(const rwkv_model *m, const void *tokens, const double *state, const double *logits,
                       const void *ws, size_t ws_bytes, int64_t T, const char *fn) {
    if (!m || !tokens || !state || !logits || !ws) return set_error(RWKV_ERR_ARG, "%s: null pointer", fn);
    if (T <= 0) return set_error(RWKV_ERR_ARG, "%s: token count must be positive", fn);
    if (reinterpret_cast<uintptr_t>(tokens) % 8 || reinterpret_cast<uintptr_t>(state) % 8 ||
        reinterpret_cast<uintptr_t>(logits) % 8 || reinterpret_cast<uintptr_t>(ws) % 16)
        return set_error(RWKV_ERR_ALIGN, "%s: tokens/state/logits need 8-byte, workspace 16-byte alignment", fn);
    const size_t need = rwkv_model_workspace_bytes(m, T);
    if (ws_bytes < need)
        return set_error(RWKV_ERR_WORKSPACE, "%s: workspace of %zu bytes needed, %zu given", fn, need, ws_bytes);
    return RWKV_OK;
}

rwkv::DQ to_dq(const rwkv_qmat &q) { return rwkv::DQ{q.packed16, q.range, q.offset}; }

// The exchange vectors of the persistent kernel live in uncached device memory: every access to them is
// an agent-coherent one that must not be served from an XCD's own L2, and on uncached pages such accesses
// go straight to the memory side, which shortens the polls (measured: a chip-wide flag barrier under a
// running weight stream takes 4.4 us on uncached pages against 6.0 us on ordinary ones).  Uncached
// allocations are never freed while the process lives (freeing one that a kernel has read has left later
// allocations with wrong contents on this platform): blocks go back to a per-device pool and are reused.
#define RWKV_TRY(expr) do { const int rc_ = (expr); if (rc_) return rc_; } while (0)

struct XchgBlock { int device; size_t bytes; void *ptr; bool busy; };
std::mutex xchg_mu;
std::vector<XchgBlock> xchg_pool;

int xchg_acquire(int device, size_t bytes, void **out) {
    std::lock_guard<std::mutex> lock(xchg_mu);
    for (XchgBlock &b : xchg_pool)
        if (!b.busy && b.device == device && b.bytes >= bytes) { b.busy = true; *out = b.ptr; return RWKV_OK; }
    void *p = nullptr;
    RWKV_CHECK_HIP(hipExtMallocWithFlags(&p, bytes, hipDeviceMallocUncached));
    xchg_pool.push_back(XchgBlock{device, bytes, p, true});
    *out = p;
    return RWKV_OK;
}
void xchg_release(void *p) {
    std::lock_guard<std::mutex> lock(xchg_mu);
    for (XchgBlock &b : xchg_pool)
        if (b.ptr == p) b.busy = false;
}

// Device-side copy of the layer table plus the exchange vectors of the
// persistent single-token kernel.  Leaves m->fused false when the shape or the
// supplied layouts do not allow that kernel.
int setup_fused(rwkv_model *m) {
    const rwkv_model_desc &d = m->d;
    if (!decode_supported(d.n_layer, d.n_embd, d.n_ffn, d.n_vocab)) return RWKV_OK;
    bool all16 = d.head.packed16 != nullptr;
    for (const rwkv_layer_desc &ld : m->layers)
        all16 = all16 && ld.att_k.packed16 && ld.att_v.packed16 && ld.att_r.packed16 && ld.att_o.packed16 &&
                ld.ffn_k.packed16 && ld.ffn_r.packed16 && ld.ffn_v.packed16;
    if (!all16) return RWKV_OK;
    const size_t total = decode_block_bytes(d.n_layer, d.n_embd, d.n_ffn, d.n_vocab);
    RWKV_CHECK_HIP(hipMalloc(&m->dev_block, total));
    RWKV_CHECK_HIP(hipMemset(m->dev_block, 0, total));
    m->xchg_bytes = decode_exchange_bytes(d.n_embd, d.n_ffn);
    RWKV_TRY(xchg_acquire(m->device, m->xchg_bytes, &m->xchg_block));
    RWKV_CHECK_HIP(hipMemset(m->xchg_block, 0, m->xchg_bytes));
    std::vector<DLayerSrc> src((size_t)d.n_layer);
    for (size_t l = 0; l < src.size(); ++l) {
        const rwkv_layer_desc &ld = m->layers[l];
        DLayerSrc &t = src[l];
        t.att_k = to_dq(ld.att_k); t.att_v = to_dq(ld.att_v); t.att_r = to_dq(ld.att_r); t.att_o = to_dq(ld.att_o);
        t.ffn_k = to_dq(ld.ffn_k); t.ffn_r = to_dq(ld.ffn_r); t.ffn_v = to_dq(ld.ffn_v);
        t.ln1_w = ld.ln1_w; t.ln1_b = ld.ln1_b; t.ln2_w = ld.ln2_w; t.ln2_b = ld.ln2_b;
        t.att_mix = ld.att_mix; t.ffn_mix = ld.ffn_mix; t.time_decay = ld.time_decay; t.time_first = ld.time_first;
    }
    DSetup s;
    s.L = d.n_layer; s.C = d.n_embd; s.F = d.n_ffn; s.V = d.n_vocab;
    s.emb = d.emb; s.ln0_w = d.ln0_w; s.ln0_b = d.ln0_b; s.lnout_w = d.ln_out_w; s.lnout_b = d.ln_out_b;
    s.head = to_dq(d.head);
    s.layers = src.data();
    const int rc = decode_setup(m->dev_block, m->xchg_block, s, &m->dm, &m->db);
    if (rc) return rc;
    m->epoch = 1;      // tag 0 is what the zero-filled exchange buffers hold
    m->fused = true;
    return RWKV_OK;
}

// ---- many-row path (prompts and batches) -----------------------------------
constexpr int64_t kRowsChunk = 1024;   // rows per pass: bounds the workspace of long prompts
constexpr int64_t kRowsMin = 4;        // shorter prompts go token by token

struct RowsWs {
    double *x, *kvr, *att, *h, *prev0, *wkv_scr;
    RowsOperand q[3];       // quantised left operands: q[0] up to n_ffn wide, q[1], q[2] n_embd wide
    long long *tot;
};

// n_head > 0: one more product, of a single row with n_head columns (the head after a prompt)
size_t rows_tot_ws_bytes(int64_t R, int64_t C, int64_t n_wide, int64_t n_head) {
    const size_t a = rows_tot_bytes(R, n_wide), b = 3 * rows_tot_bytes(R, C);     // k, v, r share a launch
    const size_t c = n_head > 0 ? rows_tot_bytes(1, n_head) : 0;
    // the quantisers of the att output and of h park their partial records here before the product starts
    const size_t q = rows_quant_scratch_bytes(R, n_wide > C ? n_wide : C);
    const size_t m = a > b ? (a > c ? a : c) : (b > c ? b : c);
    return m > q ? m : q;
}

// n_wide = widest product output (n_ffn, or the vocabulary when every row needs logits)
size_t rows_ws_bytes(int64_t R, int64_t C, int64_t F, int64_t n_wide, int64_t n_head) {
    size_t n = 0;
    n += round_up((size_t)R * C * 8, 256) * 5;          // x, kvr[3], att
    n += round_up((size_t)R * F * 8, 256);              // h
    n += round_up((size_t)C * 8, 256);                  // prev0
    n += round_up(rows_wkv_scratch_bytes(R, C), 256);
    n += round_up((size_t)R * 8, 256) * 9;              // S, qs, zp of three operands
    n += round_up(rows_dig_bytes(R, F), 256) + 2 * round_up(rows_dig_bytes(R, C), 256);
    n += round_up(rows_tot_ws_bytes(R, C, n_wide, n_head), 256);
    return n;
}

RowsWs rows_carve(void *ws, int64_t R, int64_t C, int64_t F, int64_t n_wide, int64_t n_head) {
    unsigned char *p = static_cast<unsigned char *>(ws);
    auto take = [&](size_t bytes) { void *q = p; p += round_up(bytes, 256); return q; };
    RowsWs w;
    w.x = (double *)take((size_t)R * C * 8);
    w.kvr = (double *)take((size_t)R * C * 8 * 3);
    w.att = (double *)take((size_t)R * C * 8);
    w.h = (double *)take((size_t)R * F * 8);
    w.prev0 = (double *)take((size_t)C * 8);
    w.wkv_scr = (double *)take(rows_wkv_scratch_bytes(R, C));
    for (int i = 0; i < 3; ++i) {
        w.q[i].S = (double *)take((size_t)R * 8);
        w.q[i].qs = (double *)take((size_t)R * 8);
        w.q[i].zp = (double *)take((size_t)R * 8);
        w.q[i].dig = (signed char *)take(rows_dig_bytes(R, i == 0 ? F : C));
    }
    w.tot = (long long *)take(rows_tot_ws_bytes(R, C, n_wide, n_head));
    return w;
}

bool rows_supported(const rwkv_model *m) {
    const rwkv_model_desc &d = m->d;
    if (d.n_embd % 64 || d.n_ffn % 64 || !d.head.packed16 || !rows_ln_width_supported(d.n_embd)) return false;
    for (const rwkv_layer_desc &ld : m->layers)
        if (!(ld.att_k.packed16 && ld.att_v.packed16 && ld.att_r.packed16 && ld.att_o.packed16 &&
              ld.ffn_k.packed16 && ld.ffn_r.packed16 && ld.ffn_v.packed16))
            return false;
    return true;
}

// R rows through every layer.  sequence: rows are consecutive tokens of one sequence whose state is
// `state` [L,5,C]; otherwise row b is one token of sequence b with state at state + b * state_stride.
// pending (batch rows only, or null): the last layer's ffn value product may come back unfinished, for the
// LayerNorm kernel in front of the head to finish.
int rows_layers(rwkv_model *m, hipStream_t st, const int64_t *tokens, int64_t R, bool sequence, double *state,
                int64_t state_stride, const RowsWs &w, RowsDeferred *pending = nullptr) {
    const rwkv_model_desc &d = m->d;
    const int C = (int)d.n_embd, F = (int)d.n_ffn, V = (int)d.n_vocab;
    const size_t RC = (size_t)R * C;
    RWKV_TRY(rows_embed(st, tokens, R, V, C, d.emb, d.ln0_w, d.ln0_b, w.x));
    // Few batch rows: the products split their contraction, and the three whose result goes straight into one
    // row-wise kernel (k, v, r -> WKV; the two residual updates -> the next LayerNorm) leave the sum of their slices
    // to that kernel instead of a launch of their own.
    const bool defer = !sequence && R < kRowsDeferMax;
    RowsDeferred dk[3], dx;
    dx.tot = nullptr;
    for (int64_t l = 0; l < d.n_layer; ++l) {
        const rwkv_layer_desc &L = m->layers[l];
        double *sl = state + (size_t)l * 5 * C;
        // TimeMix (block.py:58-80).  Row 0 of a sequence reads the shift state while the last row replaces it,
        // hence the copy; a single row is read and written by the same threads, in that order, and needs none.
        const bool copy_prev = sequence && R > 1;
        if (copy_prev) RWKV_CHECK_HIP(hipMemcpyAsync(w.prev0, sl, (size_t)C * 8, hipMemcpyDeviceToDevice, st));
        const rwkv_qmat *kvr[3] = {&L.att_k, &L.att_v, &L.att_r};
        const float *rg[3] = {kvr[0]->range, kvr[1]->range, kvr[2]->range};
        const double *of[3] = {kvr[0]->offset, kvr[1]->offset, kvr[2]->offset};
        RWKV_TRY(rows_ln_mix_quant(st, 3, R, C, sequence, w.x, L.ln1_w, L.ln1_b, L.att_mix, copy_prev ? w.prev0 : sl, sl,
                                   state_stride, rg, of, w.q, &dx));
        // k, v, r (and the ffn receptance below) are kept as float32 arrays in the kvr slab
        float *kvr32 = reinterpret_cast<float *>(w.kvr);
        RowsProduct pk[3];
        for (int i = 0; i < 3; ++i) { pk[i].a = w.q[i]; pk[i].w16 = kvr[i]->packed16; pk[i].out = reinterpret_cast<double *>(kvr32 + i * RC); }
        RWKV_TRY(rows_products(st, 3, pk, w.tot, R, C, C, ROW_STORE_F32, nullptr, defer ? dk : nullptr));
        RWKV_TRY(rows_wkv(st, R, C, sequence, kvr32, kvr32 + RC, kvr32 + 2 * RC, L.time_decay, L.time_first,
                          sl + 2 * (size_t)C, state_stride, reinterpret_cast<float *>(w.att), w.wkv_scr, defer ? dk : nullptr));
        RWKV_TRY(rows_quant(st, R, C, w.att, true, L.att_o.range, L.att_o.offset, w.q[0], (double *)w.tot));    // att and h: float32 arrays
        const RowsProduct po = {w.q[0], L.att_o.packed16, w.x};
        RWKV_TRY(rows_products(st, 1, &po, w.tot, R, C, C, ROW_ADD, nullptr, defer ? &dx : nullptr));
        // ChannelMix (block.py:82-100)
        if (copy_prev) RWKV_CHECK_HIP(hipMemcpyAsync(w.prev0, sl + C, (size_t)C * 8, hipMemcpyDeviceToDevice, st));
        const float *rg2[2] = {L.ffn_k.range, L.ffn_r.range};
        const double *of2[2] = {L.ffn_k.offset, L.ffn_r.offset};
        RWKV_TRY(rows_ln_mix_quant(st, 2, R, C, sequence, w.x, L.ln2_w, L.ln2_b, L.ffn_mix, copy_prev ? w.prev0 : sl + C,
                                   sl + C, state_stride, rg2, of2, w.q + 1, &dx));
        dx.tot = nullptr;
        const RowsProduct pfk = {w.q[1], L.ffn_k.packed16, w.h}, pfr = {w.q[2], L.ffn_r.packed16, w.kvr};
        RWKV_TRY(rows_products(st, 1, &pfk, w.tot, R, C, F, ROW_RELU2, nullptr));
        RWKV_TRY(rows_products(st, 1, &pfr, w.tot, R, C, C, ROW_STORE_F32, nullptr));
        RWKV_TRY(rows_quant(st, R, F, w.h, true, L.ffn_v.range, L.ffn_v.offset, w.q[0], (double *)w.tot));
        const RowsProduct pfv = {w.q[0], L.ffn_v.packed16, w.x};
        // (the ffn receptance stays in the kvr slab and the totals untouched until the next LayerNorm kernel has run)
        const bool hand_on = defer && (l + 1 < d.n_layer || pending);
        RWKV_TRY(rows_products(st, 1, &pfv, w.tot, R, F, C, ROW_GATE_ADD, kvr32, hand_on ? &dx : nullptr));
    }
    if (pending) *pending = dx;
    return RWKV_OK;
}

// Which path a sequence of T tokens takes: the many-row kernels for prompts, and for single tokens too when
// the persistent single-token kernel does not serve the shape (their integer products beat one launch per
// phase with float32 sums both in time and in accuracy).
bool use_rows(const rwkv_model *m, int64_t T) { return rows_supported(m) && (T >= kRowsMin || !m->fused); }

// T consecutive tokens of one sequence through the many-row kernels, in chunks of kRowsChunk rows; logits
// from the last row only.  workspace: as rwkv_model_workspace_bytes(m, T) sizes it.
int rows_sequence(rwkv_model *m, hipStream_t st, const int64_t *tokens, int64_t T, double *state, double *logits,
                  void *workspace) {
    const int64_t C = m->d.n_embd, F = m->d.n_ffn;
    unsigned char *rows_base = static_cast<unsigned char *>(workspace) + round_up(ws_doubles(C, F) * sizeof(double), 256);
    const int64_t Rmax = T < kRowsChunk ? T : kRowsChunk;
    const RowsWs rw = rows_carve(rows_base, Rmax, C, F, F, m->d.n_vocab);
    for (int64_t t0 = 0; t0 < T; t0 += kRowsChunk) {
        const int64_t R = T - t0 < kRowsChunk ? T - t0 : kRowsChunk;
        int rc = rows_layers(m, st, tokens + t0, R, true, state, 0, rw);
        if (rc) return rc;
        if (t0 + R == T) {
            // ln_out and the head on the last row (opt.py:72-74), as a one-row product with integer sums
            const rwkv_model_desc &d = m->d;
            const float *rg[1] = {d.head.range};
            const double *of[1] = {d.head.offset};
            rc = rows_ln_mix_quant(st, 0, 1, (int)C, false, rw.x + (size_t)(R - 1) * C, d.ln_out_w, d.ln_out_b, nullptr,
                                   nullptr, nullptr, 0, rg, of, rw.q);
            if (rc) return rc;
            const RowsProduct ph = {rw.q[0], d.head.packed16, logits};
            rc = rows_products(st, 1, &ph, rw.tot, 1, C, d.n_vocab, ROW_STORE, nullptr);
        }
        if (rc) return rc;
    }
    return RWKV_OK;
}

// The exchange words carry a 32-bit epoch that grows with every token step.  Before the counter would wrap
// (after some 2^32 / (4 L + 1) steps) the exchange buffers are cleared and the count starts again at 1, so no
// step ever runs under a tag an older word could still carry, and never under tag 0 (cleared memory).
int fused_epochs(rwkv_model *m, hipStream_t st, int64_t steps) {
    const uint64_t need = (uint64_t)steps * decode_epochs_per_token(m->d.n_layer);
    if (need >= 0xffffffffull) return set_error(RWKV_ERR_SIZE, "too many token steps in one call");
    if ((uint64_t)m->epoch + need < 0xffffffffull) return RWKV_OK;
    RWKV_TRY(decode_clear_exchange(st, m->dm, m->db));
    m->epoch = 1;
    return RWKV_OK;
}

// One token through the persistent kernel (argument checks done by the caller).
int fused_token(rwkv_model *m, hipStream_t st, const int64_t *token, double *state, double *logits) {
    RWKV_TRY(fused_epochs(m, st, 1));
    const int rc = decode_launch(st, m->dm, m->db, m->epoch, token, state, logits);
    m->epoch += decode_epochs_per_token(m->d.n_layer);
    return rc;
}

}  // namespace

extern "C" {

int rwkv_model_create(const rwkv_model_desc *desc, rwkv_model **out) {
    RWKV_CHECK_ARG(desc && out, "rwkv_model_create: null pointer");
    RWKV_CHECK_ARG(desc->layers, "rwkv_model_create: null layer table");
    const int64_t L = desc->n_layer, C = desc->n_embd, F = desc->n_ffn, V = desc->n_vocab;
    RWKV_CHECK_ARG(L > 0 && C > 0 && F > 0 && V > 0, "rwkv_model_create: sizes must be positive");
    if (C > (int64_t)kMaxCPT * kThreads)
        return set_error(RWKV_ERR_SIZE, "rwkv_model_create: n_embd %lld exceeds the supported %d", (long long)C,
                         kMaxCPT * kThreads);
    if (F >= (1 << 24) || V >= (1 << 28))
        return set_error(RWKV_ERR_SIZE, "rwkv_model_create: n_ffn/n_vocab too large");
    RWKV_CHECK_ARG(desc->emb && desc->ln0_w && desc->ln0_b && desc->ln_out_w && desc->ln_out_b,
                   "rwkv_model_create: null model-level pointer");
    int rc = check_qmat(desc->head, C, V, "head");
    if (rc) return rc;
    for (int64_t l = 0; l < L; ++l) {
        const rwkv_layer_desc &ld = desc->layers[l];
        RWKV_CHECK_ARG(ld.ln1_w && ld.ln1_b && ld.ln2_w && ld.ln2_b && ld.att_mix && ld.ffn_mix &&
                       ld.time_decay && ld.time_first, "rwkv_model_create: layer %lld has a null pointer", (long long)l);
        if ((rc = check_qmat(ld.att_k, C, C, "att_k")) || (rc = check_qmat(ld.att_v, C, C, "att_v")) ||
            (rc = check_qmat(ld.att_r, C, C, "att_r")) || (rc = check_qmat(ld.att_o, C, C, "att_o")) ||
            (rc = check_qmat(ld.ffn_k, C, F, "ffn_k")) || (rc = check_qmat(ld.ffn_r, C, C, "ffn_r")) ||
            (rc = check_qmat(ld.ffn_v, F, C, "ffn_v")))
            return rc;
    }
    int dev = 0;
    RWKV_CHECK_HIP(hipGetDevice(&dev));
    hipDeviceProp_t prop;
    RWKV_CHECK_HIP(hipGetDeviceProperties(&prop, dev));
    if (std::string(prop.gcnArchName).rfind("gfx950", 0) != 0)
        return set_error(RWKV_ERR_DEVICE, "rwkv_model_create: device is %s, this library is built for gfx950",
                         prop.gcnArchName);
    rwkv_model *m = new (std::nothrow) rwkv_model();
    if (!m) return set_error(RWKV_ERR_ARG, "rwkv_model_create: out of host memory");
    m->d = *desc;
    m->layers.assign(desc->layers, desc->layers + L);
    m->d.layers = m->layers.data();
    m->device = dev;
    rc = setup_fused(m);
    if (rc) { rwkv_model_destroy(m); return rc; }
    *out = m;
    return RWKV_OK;
}

void rwkv_model_destroy(rwkv_model *m) {
    if (!m) return;
    if (m->dev_block) (void)hipFree(m->dev_block);
    if (m->xchg_block) xchg_release(m->xchg_block);
    delete m;
}

int rwkv_model_has_fused_step(const rwkv_model *m) { return (m && m->fused) ? 1 : 0; }

int rwkv_model_trace_workgroups(const rwkv_model *m) {
    if (!m || !m->fused) return 0;
    return (int)(decode_workgroups(m->dm.C) + decode_helper_workgroups(m->dm.C));
}

int rwkv_model_set_trace(rwkv_model *m, int64_t *device_buffer) {
    RWKV_CHECK_ARG(m, "rwkv_model_set_trace: null handle");
    m->db.trace = reinterpret_cast<long long *>(device_buffer);
    return RWKV_OK;
}

int rwkv_model_check(rwkv_model *m) {
    RWKV_CHECK_ARG(m, "rwkv_model_check: null handle");
    RWKV_CHECK_HIP(hipDeviceSynchronize());
    if (!m->fused) return RWKV_OK;
    unsigned flag = 0;
    RWKV_CHECK_HIP(hipMemcpy(&flag, m->db.abort_flag, sizeof(flag), hipMemcpyDeviceToHost));
    if (flag) {
        // reported once: the flag is cleared so that later token steps run again (every wait of the kernel also
        // leaves when it sees the flag, so a set flag would cut every following step short)
        RWKV_CHECK_HIP(hipMemset(m->db.abort_flag, 0, sizeof(flag)));
        return set_error(RWKV_ERR_HIP, "a single-token launch gave up waiting for another workgroup; logits and "
                                       "state written since the last check are invalid");
    }
    return RWKV_OK;
}

int rwkv_model_time_token_kernel(rwkv_model *m, rwkv_stream_t stream, const int64_t *token, double *state, double *logits,
                                 int n, float *avg_us) {
    RWKV_CHECK_ARG(m && token && state && logits && avg_us, "rwkv_model_time_token_kernel: null pointer");
    RWKV_CHECK_ARG(n > 0 && n <= 4096, "rwkv_model_time_token_kernel: n must be in 1..4096");
    if (reinterpret_cast<uintptr_t>(token) % 8 || reinterpret_cast<uintptr_t>(state) % 8 || reinterpret_cast<uintptr_t>(logits) % 8)
        return set_error(RWKV_ERR_ALIGN, "rwkv_model_time_token_kernel: token, state and logits need 8-byte alignment");
    if (!m->fused) return set_error(RWKV_ERR_SIZE, "rwkv_model_time_token_kernel: this model does not run the persistent kernel");
    const hipStream_t st = (hipStream_t)stream;
    std::vector<hipEvent_t> ev((size_t)2 * n, nullptr);
    int rc = RWKV_OK;
    for (auto &e : ev)
        if (rc == RWKV_OK && hipEventCreate(&e) != hipSuccess) rc = set_error(RWKV_ERR_HIP, "rwkv_model_time_token_kernel: hipEventCreate failed");
    for (int i = 0; i < n && rc == RWKV_OK; ++i) {
        rc = fused_epochs(m, st, 1);
        if (rc == RWKV_OK) rc = decode_launch_bracketed(st, m->dm, m->db, m->epoch, token, state, logits, ev[2 * i], ev[2 * i + 1]);
        m->epoch += decode_epochs_per_token(m->d.n_layer);
    }
    if (rc == RWKV_OK && hipStreamSynchronize(st) != hipSuccess) rc = set_error(RWKV_ERR_HIP, "rwkv_model_time_token_kernel: synchronize failed");
    double total_ms = 0.0;
    for (int i = 0; i < n && rc == RWKV_OK; ++i) {
        float ms = 0.f;
        if (hipEventElapsedTime(&ms, ev[2 * i], ev[2 * i + 1]) != hipSuccess) rc = set_error(RWKV_ERR_HIP, "rwkv_model_time_token_kernel: hipEventElapsedTime failed");
        total_ms += (double)ms;
    }
    for (auto &e : ev)
        if (e) (void)hipEventDestroy(e);
    if (rc == RWKV_OK) *avg_us = (float)(total_ms * 1e3 / n);
    return rc;
}

int rwkv_model_selftest_timeout(rwkv_model *m, rwkv_stream_t stream, double *state, double *logits) {
    RWKV_CHECK_ARG(m && state && logits, "rwkv_model_selftest_timeout: null pointer");
    if (reinterpret_cast<uintptr_t>(state) % 8 || reinterpret_cast<uintptr_t>(logits) % 8)
        return set_error(RWKV_ERR_ALIGN, "rwkv_model_selftest_timeout: state and logits need 8-byte alignment");
    if (!m->fused) return set_error(RWKV_ERR_SIZE, "rwkv_model_selftest_timeout: this model does not run the persistent kernel");
    RWKV_TRY(fused_epochs(m, (hipStream_t)stream, 1));
    const int rc = decode_launch_unfed((hipStream_t)stream, m->dm, m->db, m->epoch, state, logits, 256u);
    m->epoch += decode_epochs_per_token(m->d.n_layer);
    return rc;
}

size_t rwkv_model_workspace_bytes(const rwkv_model *m, int64_t max_tokens) {
    if (!m || max_tokens <= 0) return 0;
    size_t n = round_up(ws_doubles(m->d.n_embd, m->d.n_ffn) * sizeof(double), 256);
    if (use_rows(m, max_tokens)) {
        const int64_t R = max_tokens < kRowsChunk ? max_tokens : kRowsChunk;
        n += rows_ws_bytes(R, m->d.n_embd, m->d.n_ffn, m->d.n_ffn, m->d.n_vocab);
    }
    return n;
}

size_t rwkv_model_batch_workspace_bytes(const rwkv_model *m, int64_t batch) {
    if (!m || batch <= 0 || !rows_supported(m)) return 0;
    const int64_t wide = m->d.n_ffn > m->d.n_vocab ? m->d.n_ffn : m->d.n_vocab;
    return rows_ws_bytes(batch, m->d.n_embd, m->d.n_ffn, wide, 0);
}

int rwkv_model_forward(rwkv_model *m, rwkv_stream_t stream, const int64_t *tokens, int64_t T, double *state,
                       double *logits, void *workspace, size_t workspace_bytes) {
    int rc = check_forward_args(m, tokens, state, logits, workspace, workspace_bytes, T, "rwkv_model_forward");
    if (rc) return rc;
    const Workspace w = carve(workspace, m->d.n_embd, m->d.n_ffn);
    if (use_rows(m, T)) return rows_sequence(m, (hipStream_t)stream, tokens, T, state, logits, workspace);
    for (int64_t t = 0; t < T; ++t) {
        if (m->fused) rc = fused_token(m, (hipStream_t)stream, tokens + t, state, logits);
        else rc = step_token(m, (hipStream_t)stream, tokens + t, state, logits, w, t == T - 1);
        if (rc) return rc;
    }
    return RWKV_OK;
}

int rwkv_model_forward_batch(rwkv_model *m, rwkv_stream_t stream, const int64_t *tokens, int64_t batch,
                             double *states, double *logits, void *workspace, size_t workspace_bytes) {
    if (!m || !tokens || !states || !logits || !workspace)
        return set_error(RWKV_ERR_ARG, "rwkv_model_forward_batch: null pointer");
    if (batch <= 0) return set_error(RWKV_ERR_ARG, "rwkv_model_forward_batch: batch must be positive");
    if (!rows_supported(m))
        return set_error(RWKV_ERR_SIZE, "rwkv_model_forward_batch: needs the M16 layout of every matrix and "
                                        "n_embd, n_ffn multiples of 64");
    if (reinterpret_cast<uintptr_t>(tokens) % 8 || reinterpret_cast<uintptr_t>(states) % 8 ||
        reinterpret_cast<uintptr_t>(logits) % 8 || reinterpret_cast<uintptr_t>(workspace) % 16)
        return set_error(RWKV_ERR_ALIGN, "rwkv_model_forward_batch: tokens/states/logits need 8-byte, workspace "
                                         "16-byte alignment");
    const size_t need = rwkv_model_batch_workspace_bytes(m, batch);
    if (workspace_bytes < need)
        return set_error(RWKV_ERR_WORKSPACE, "rwkv_model_forward_batch: workspace of %zu bytes needed, %zu given",
                         need, workspace_bytes);
    const hipStream_t st = (hipStream_t)stream;
    const rwkv_model_desc &d = m->d;
    const int64_t C = d.n_embd, F = d.n_ffn, V = d.n_vocab;
    const RowsWs rw = rows_carve(workspace, batch, C, F, F > V ? F : V, 0);
    RowsDeferred pending;
    int rc = rows_layers(m, st, tokens, batch, false, states, d.n_layer * 5 * C, rw, &pending);
    if (rc) return rc;
    const float *rg[1] = {d.head.range};
    const double *of[1] = {d.head.offset};
    rc = rows_ln_mix_quant(st, 0, batch, (int)C, false, rw.x, d.ln_out_w, d.ln_out_b, nullptr, nullptr, nullptr, 0, rg, of,
                           rw.q, &pending);
    if (rc) return rc;
    const RowsProduct ph = {rw.q[0], d.head.packed16, logits};
    return rows_products(st, 1, &ph, rw.tot, batch, C, V, ROW_STORE, nullptr);
}

int rwkv_gemm8(rwkv_stream_t stream, int64_t T, int64_t n_in, int64_t n_out, const double *x,
               const uint8_t *packed16, const float *range, const double *offset, double *y,
               void *workspace, size_t workspace_bytes) {
    RWKV_CHECK_ARG(x && packed16 && range && offset && y && workspace, "rwkv_gemm8: null pointer");
    RWKV_CHECK_ARG(T > 0 && n_in > 0 && n_out > 0, "rwkv_gemm8: sizes must be positive");
    if (n_in % 64) return set_error(RWKV_ERR_SIZE, "rwkv_gemm8: n_in must be a multiple of 64");
    RWKV_CHECK_ALIGN(packed16, 16);
    RWKV_CHECK_ALIGN(workspace, 16);
    RWKV_CHECK_ALIGN(x, 8);
    RWKV_CHECK_ALIGN(y, 8);
    const size_t need = rwkv_gemm8_workspace_bytes(T, n_in, n_out);
    if (workspace_bytes < need)
        return set_error(RWKV_ERR_WORKSPACE, "rwkv_gemm8: workspace of %zu bytes needed, %zu given", need,
                         workspace_bytes);
    unsigned char *p = static_cast<unsigned char *>(workspace);
    RowsOperand q;
    q.S = (double *)p; p += round_up((size_t)T * 8, 256);
    q.qs = (double *)p; p += round_up((size_t)T * 8, 256);
    q.zp = (double *)p; p += round_up((size_t)T * 8, 256);
    q.dig = (signed char *)p; p += round_up(rows_dig_bytes(T, n_in), 256);
    const hipStream_t st = (hipStream_t)stream;
    const int rc = rows_quant(st, T, n_in, x, false, range, offset, q, (double *)p);
    if (rc) return rc;
    const RowsProduct pr = {q, packed16, y};
    return rows_products(st, 1, &pr, (long long *)p, T, n_in, n_out, ROW_STORE, nullptr);
}

size_t rwkv_gemm8_workspace_bytes(int64_t T, int64_t n_in, int64_t n_out) {
    if (T <= 0 || n_in <= 0 || n_out <= 0) return 0;
    const size_t tot = rows_tot_bytes(T, n_out), qs = rows_quant_scratch_bytes(T, n_in);   // share one area
    return round_up((size_t)T * 8, 256) * 3 + round_up(rows_dig_bytes(T, n_in), 256) + round_up(tot > qs ? tot : qs, 256);
}

int rwkv_sample_token(rwkv_stream_t stream, double *logits, int64_t V, int greedy, float temp, float tau, double end_adj,
                      uint64_t seed, uint64_t counter, int64_t *out_token) {
    RWKV_CHECK_ARG(logits && out_token, "rwkv_sample_token: null pointer");
    RWKV_CHECK_ARG(V > 0 && V < (1ll << 31), "rwkv_sample_token: bad size");
    RWKV_CHECK_ARG(greedy || (temp > 0.f && tau >= 0.f), "rwkv_sample_token: temp must be positive, tau non-negative");
    SampleArgs sa{};
    sa.logits = logits; sa.V = (int)V; sa.greedy = greedy ? 1 : 0; sa.temp = temp; sa.tau = tau; sa.end_adj = end_adj;
    sa.seed = seed; sa.counter = counter; sa.out_token = out_token;
    return sample_launch((hipStream_t)stream, sa);
}

int rwkv_model_decode_sample(rwkv_model *m, rwkv_stream_t stream, int64_t *tokens, int64_t n, double *state, double *logits,
                             void *workspace, size_t workspace_bytes, int greedy, float temp, float tau, double end_adj,
                             uint64_t seed, const int64_t *stop_tokens, int n_stop, int32_t *stop_flag, int64_t *n_done) {
    int rc = check_forward_args(m, tokens, state, logits, workspace, workspace_bytes, 1, "rwkv_model_decode_sample");
    if (rc) return rc;
    RWKV_CHECK_ARG(n > 0, "rwkv_model_decode_sample: n must be positive");
    RWKV_CHECK_ARG(stop_flag && n_done, "rwkv_model_decode_sample: stop_flag and n_done must point to device words");
    RWKV_CHECK_ARG(n_stop >= 0 && (n_stop == 0 || stop_tokens), "rwkv_model_decode_sample: stop list");
    RWKV_CHECK_ARG(greedy || (temp > 0.f && tau >= 0.f), "rwkv_model_decode_sample: temp must be positive, tau non-negative");
    if (!m->fused)
        return set_error(RWKV_ERR_SIZE, "rwkv_model_decode_sample: this shape does not run the persistent single-token "
                                        "kernel; sample on the host from rwkv_model_forward's logits");
    if ((rc = fused_epochs(m, (hipStream_t)stream, n))) return rc;
    SampleArgs sa{};
    sa.greedy = greedy ? 1 : 0; sa.temp = temp; sa.tau = tau; sa.end_adj = end_adj; sa.seed = seed; sa.counter = 0;
    sa.stop_tokens = stop_tokens; sa.n_stop = n_stop; sa.stop_flag = stop_flag; sa.n_done = n_done;
    rc = decode_launch_sampled((hipStream_t)stream, m->dm, m->db, m->epoch, tokens, n, state, logits, sa);
    m->epoch += (unsigned)n * decode_epochs_per_token(m->d.n_layer);
    return rc;
}

int rwkv_gemm8_plan(int64_t T, int64_t n_in, int64_t n_out, int n_products, int plan[4], size_t *tot_bytes_per_product) {
    RWKV_CHECK_ARG(plan && tot_bytes_per_product, "rwkv_gemm8_plan: null pointer");
    RWKV_CHECK_ARG(T > 0 && n_in > 0 && n_out > 0 && n_products >= 1 && n_products <= kRowsMaxProducts,
                   "rwkv_gemm8_plan: bad sizes");
    if (n_in % 64) return set_error(RWKV_ERR_SIZE, "rwkv_gemm8_plan: n_in must be a multiple of 64");
    rows_plan_describe(T, n_in, n_out, n_products, plan);
    *tot_bytes_per_product = rows_tot_bytes(T, n_out);
    return RWKV_OK;
}

int rwkv_model_decode_greedy(rwkv_model *m, rwkv_stream_t stream, int64_t *tokens, int64_t n, double *state,
                             double *logits, void *workspace, size_t workspace_bytes) {
    int rc = check_forward_args(m, tokens, state, logits, workspace, workspace_bytes, 1, "rwkv_model_decode_greedy");
    if (rc) return rc;
    RWKV_CHECK_ARG(n > 0, "rwkv_model_decode_greedy: n must be positive");
    const Workspace w = carve(workspace, m->d.n_embd, m->d.n_ffn);
    if (m->fused) {
        if ((rc = fused_epochs(m, (hipStream_t)stream, n))) return rc;
        rc = decode_launch_greedy((hipStream_t)stream, m->dm, m->db, m->epoch, tokens, n, state, logits);
        m->epoch += (unsigned)n * decode_epochs_per_token(m->d.n_layer);
        return rc;
    }
    for (int64_t i = 0; i < n; ++i) {
        if (use_rows(m, 1)) rc = rows_sequence(m, (hipStream_t)stream, tokens + i, 1, state, logits, workspace);
        else rc = step_token(m, (hipStream_t)stream, tokens + i, state, logits, w, true);
        if (rc) return rc;
        rc = rwkv_argmax_f64(stream, logits, m->d.n_vocab, tokens + i + 1);
        if (rc) return rc;
    }
    return RWKV_OK;
}

}  // extern "C"
