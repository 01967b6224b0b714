// Stand-alone operators: the packed uint8 matvec, the WKV recurrences, argmax,
// and the reference-layout mm8_one / mm8_three drop-ins.
#include "rwkv_common.h"
#include "rwkv_rows.h"

#include <mutex>

namespace rwkv {

// ---------------------------------------------------------------------------
// y[b,k] = r_col[k] * sum_j fp32(x[b,j] r_row[j]) code[j,k]
//          + sum_j x[b,j] m_row[j] + m_col[k] sum_j x[b,j]
// One workgroup per 8-column tile.  The scaled activations are staged in LDS
// in chunks of kc_rows rows (NB * kc_rows * 4 bytes <= 64 KiB); the matrix is
// read exactly once, with one 16-byte load per lane per 1 KiB block.
// ---------------------------------------------------------------------------
template <int NB, int NT, int NW>
__global__ void __launch_bounds__(NW * 64)
mm8_packed_kernel(int n_in, int n_out, int n_kb, int kc_blocks,
                  const float *__restrict__ x, const uint8_t *__restrict__ packed,
                  const float *__restrict__ r_row, const double *__restrict__ m_row,
                  const float *__restrict__ r_col, const float *__restrict__ m_col,
                  double *__restrict__ y) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *xs = reinterpret_cast<float *>(smem);                    // [NB][kc_rows]
    const int kc_rows = kc_blocks * kBlockRows;
    constexpr int kPT = NW * 64;                                           // threads
    double *dred = reinterpret_cast<double *>(xs + (size_t)NB * kc_rows);   // [2*NB*NW]
    float *fred = reinterpret_cast<float *>(dred + 2 * NB * NW);            // [NT*NB*NW*8]

    // NT neighbouring column tiles per workgroup share one staging of the activations and every LDS read of
    // them: with NB = 8 a tile's weights (n_in x 8 bytes) are a quarter of the activations staged for it
    // (n_in x NB x 4 bytes), and each 16-byte LDS read feeds only four multiply-adds per tile.
    const int n_tiles = (n_out + kTileCols - 1) / kTileCols;
    const int ct0 = blockIdx.x * NT;
    const uint8_t *wtile[NT];
#pragma unroll
    for (int m = 0; m < NT; ++m)
        wtile[m] = packed + (size_t)min(ct0 + m, n_tiles - 1) * n_kb * kBlockBytes;       // past the end: the last tile again, its sums dropped

    float acc[NT][NB];
    double zsum[2 * NB];   // [b]: sum x*m_row ; [NB+b]: sum x
#pragma unroll
    for (int b = 0; b < NB; ++b) {
        zsum[b] = 0.0; zsum[NB + b] = 0.0;
#pragma unroll
        for (int m = 0; m < NT; ++m) acc[m][b] = 0.f;
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, s8 = lane >> 3;
    constexpr int kAhead = NT >= 4 ? 2 : NT == 2 ? 3 : kUnroll;     // blocks per tile a wavefront has in flight

    for (int kb0 = 0; kb0 < n_kb; kb0 += kc_blocks) {
        const int kb1 = min(kb0 + kc_blocks, n_kb);
        const int j0 = kb0 * kBlockRows;
        // kStageAhead rows per thread at a time, every load of the group issued before the first use: the loop is
        // otherwise a chain of dependent memory latencies (NB loads of x per row, one row after the other)
        constexpr int kStageAhead = NB >= 4 ? 4 : 8;
        const int rows_here = (kb1 - kb0) * kBlockRows;
        for (int i0 = threadIdx.x; i0 < rows_here; i0 += kStageAhead * kPT) {
            float xv[kStageAhead][NB], rr[kStageAhead];
            double mr[kStageAhead];
#pragma unroll
            for (int u = 0; u < kStageAhead; ++u) {
                const int i = i0 + u * kPT, j = j0 + i;
                const bool in = i < rows_here && j < n_in;
                rr[u] = in ? r_row[j] : 0.f;
                mr[u] = in ? m_row[j] : 0.0;
#pragma unroll
                for (int b = 0; b < NB; ++b) xv[u][b] = in ? x[(size_t)b * n_in + j] : 0.f;
            }
#pragma unroll
            for (int u = 0; u < kStageAhead; ++u) {
                const int i = i0 + u * kPT;
                if (i < rows_here) {
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        const double xd = (double)xv[u][b];
                        xs[(size_t)b * kc_rows + i] = (float)(xd * (double)rr[u]);      // matmul.py:131
                        zsum[b] += xd * mr[u];
                        zsum[NB + b] += xd;
                    }
                }
            }
        }
        __syncthreads();
        // wave w takes blocks kb0 + w, + kWaves, ...; lane (s8, column) accumulates its column over rows 32 q + 4 s8 + e
        // of each block (the order of tile_accumulate, so one tile per workgroup gives the same bits as before)
        for (int kbw = kb0 + wave; kbw < kb1; kbw += NW * kAhead) {
            uint4 wv[NT][kAhead];
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int kb = kbw + u * NW;
                if (kb < kb1) {
#pragma unroll
                    for (int m = 0; m < NT; ++m)
                        wv[m][u] = *reinterpret_cast<const uint4 *>(wtile[m] + (size_t)kb * kBlockBytes + lane * 16);
                }
            }
#pragma unroll
            for (int u = 0; u < kAhead; ++u) {
                const int kb = kbw + u * NW;
                if (kb < kb1) {
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        const float4 *xp = reinterpret_cast<const float4 *>(xs + (size_t)b * kc_rows + (kb - kb0) * kBlockRows + 4 * s8);
                        const float4 x0 = xp[0], x1 = xp[8], x2 = xp[16], x3 = xp[24];
#pragma unroll
                        for (int m = 0; m < NT; ++m) {
                            acc[m][b] = dot4_u8(wv[m][u].x, x0, acc[m][b]);
                            acc[m][b] = dot4_u8(wv[m][u].y, x1, acc[m][b]);
                            acc[m][b] = dot4_u8(wv[m][u].z, x2, acc[m][b]);
                            acc[m][b] = dot4_u8(wv[m][u].w, x3, acc[m][b]);
                        }
                    }
                }
            }
        }
        __syncthreads();
    }
    // sums over the workgroup's NW wavefronts in a fixed order (block_sum and tile_reduce for any NW)
#pragma unroll
    for (int i = 0; i < 2 * NB; ++i) {
        const double t = wave_sum(zsum[i]);
        if (lane == 0) dred[i * NW + wave] = t;
    }
    float out[NT][NB];
#pragma unroll
    for (int m = 0; m < NT; ++m)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float t = acc[m][b];
            t += __shfl_xor(t, 8, 64);
            t += __shfl_xor(t, 16, 64);
            t += __shfl_xor(t, 32, 64);
            if (lane < 8) fred[((m * NB + b) * NW + wave) * 8 + lane] = t;
        }
    __syncthreads();
    if (threadIdx.x < kTileCols) {
#pragma unroll
        for (int i = 0; i < 2 * NB; ++i) {
            double t = 0.0;
#pragma unroll
            for (int w = 0; w < NW; ++w) t += dred[i * NW + w];
            zsum[i] = t;
        }
#pragma unroll
        for (int m = 0; m < NT; ++m)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float t = 0.f;
#pragma unroll
                for (int w = 0; w < NW; ++w) t += fred[((m * NB + b) * NW + w) * 8 + threadIdx.x];
                out[m][b] = t;
            }
#pragma unroll
        for (int m = 0; m < NT; ++m) {
            const int k = (ct0 + m) * kTileCols + threadIdx.x;
            if (ct0 + m < n_tiles && k < n_out) {
                const double rc = r_col ? (double)r_col[k] : 1.0;
                const double mc = m_col ? (double)m_col[k] : 0.0;
#pragma unroll
                for (int b = 0; b < NB; ++b)
                    y[(size_t)b * n_out + k] = rc * (double)out[m][b] + zsum[b] + mc * zsum[NB + b];
            }
        }
    }
}

// ---------------------------------------------------------------------------
// The same product for ONE vector, laid out so that a compute unit moves little besides its share of the matrix:
// a workgroup of NW wavefronts owns NT neighbouring column tiles over the whole contraction (about one workgroup
// per compute unit), stages the scaled vector once for all of them, and every wavefront requests ALL its weight
// blocks (block kb = wave + NW v of each tile, v < VB) right after the loads of the staging - loads return in the
// order they were issued, so the staging data arrives first and is converted while the matrix is on its way.
// With one 8-column tile per workgroup the vector, its ranges and its float64 offsets (16 bytes per input row,
// re-read by every workgroup) are more bytes through a compute unit's vector-memory path than the tile itself.
// Arithmetic as in mm8_packed_kernel: float32 multiply-adds, fixed order (per lane by block, then lanes, then
// wavefronts).
// ---------------------------------------------------------------------------
typedef unsigned v4u __attribute__((ext_vector_type(4)));
constexpr int kOneStage = 10;           // input rows per thread: up to 10240 rows with 1024 threads

template <int NT, int VB>
__global__ void __launch_bounds__(1024)
mm8_packed_one_kernel(int n_in, int n_out, int n_kb,
                      const float *__restrict__ x, const uint8_t *__restrict__ packed,
                      const float *__restrict__ r_row, const double *__restrict__ m_row,
                      const float *__restrict__ r_col, const float *__restrict__ m_col,
                      double *__restrict__ y) {
    extern __shared__ __align__(16) unsigned char smem[];
    float *xs = reinterpret_cast<float *>(smem);                            // [n_kb * 128]
    const int NW = blockDim.x >> 6, kPT = blockDim.x;
    const int n_rows = n_kb * kBlockRows;
    double *dred = reinterpret_cast<double *>(xs + n_rows);                 // [2 * NW]
    float *fred = reinterpret_cast<float *>(dred + 2 * NW);                 // [NT][NW][8]
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6, s8 = lane >> 3;
    const int n_tiles = (n_out + kTileCols - 1) / kTileCols;
    // 1. the loads of the staging ...
    float xv[kOneStage], rr[kOneStage];
    double mr[kOneStage];
#pragma unroll
    for (int u = 0; u < kOneStage; ++u) {
        const int j = threadIdx.x + u * kPT;
        const bool in = j < n_in;
        xv[u] = in ? x[j] : 0.f;
        rr[u] = in ? r_row[j] : 0.f;
        mr[u] = in ? m_row[j] : 0.0;
    }
    // 2. ... then every weight block of this wavefront
    v4u wv[NT][VB];
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        const uint8_t *wtile = packed + (size_t)min(blockIdx.x * NT + t, n_tiles - 1) * n_kb * kBlockBytes;   // past the end: the last tile again, its sums dropped
#pragma unroll
        for (int v = 0; v < VB; ++v) {
            const int kb = min(wave + v * NW, n_kb - 1);                    // past the end: a block nobody multiplies
            wv[t][v] = __builtin_nontemporal_load(reinterpret_cast<const v4u *>(wtile + (size_t)kb * kBlockBytes) + lane);
        }
    }
    // 3. the staging data is here first
    double zs = 0.0, xsum = 0.0;
#pragma unroll
    for (int u = 0; u < kOneStage; ++u) {
        const int j = threadIdx.x + u * kPT;
        if (j < n_rows) {
            const double xd = (double)xv[u];
            xs[j] = (float)(xd * (double)rr[u]);                            // matmul.py:131
            zs += xd * mr[u];
            xsum += xd;
        }
    }
    zs = wave_sum(zs); xsum = wave_sum(xsum);
    if (lane == 0) { dred[wave] = zs; dred[NW + wave] = xsum; }
    __syncthreads();
    float acc[NT];
#pragma unroll
    for (int t = 0; t < NT; ++t) acc[t] = 0.f;
#pragma unroll
    for (int v = 0; v < VB; ++v) {
        const int kb = wave + v * NW;
        if (kb < n_kb) {
            const float4 *xp = reinterpret_cast<const float4 *>(xs + kb * kBlockRows + 4 * s8);
            const float4 x0 = xp[0], x1 = xp[8], x2 = xp[16], x3 = xp[24];
#pragma unroll
            for (int t = 0; t < NT; ++t) {
                acc[t] = dot4_u8(wv[t][v].x, x0, acc[t]);
                acc[t] = dot4_u8(wv[t][v].y, x1, acc[t]);
                acc[t] = dot4_u8(wv[t][v].z, x2, acc[t]);
                acc[t] = dot4_u8(wv[t][v].w, x3, acc[t]);
            }
        }
    }
#pragma unroll
    for (int t = 0; t < NT; ++t) {
        float a = acc[t];
        a += __shfl_xor(a, 8, 64);
        a += __shfl_xor(a, 16, 64);
        a += __shfl_xor(a, 32, 64);
        if (lane < 8) fred[(t * NW + wave) * 8 + lane] = a;
    }
    __syncthreads();
    if (threadIdx.x < NT * kTileCols) {
        const int t = threadIdx.x >> 3, c = threadIdx.x & 7;
        double z = 0.0, xm = 0.0;
        float sum = 0.f;
        for (int w = 0; w < NW; ++w) { z += dred[w]; xm += dred[NW + w]; sum += fred[(t * NW + w) * 8 + c]; }
        const int k = (blockIdx.x * NT + t) * kTileCols + c;
        if (blockIdx.x * NT + t < n_tiles && k < n_out) {
            const double rc = r_col ? (double)r_col[k] : 1.0;
            const double mc = m_col ? (double)m_col[k] : 0.0;
            y[k] = rc * (double)sum + z + mc * xm;
        }
    }
}

// ---------------------------------------------------------------------------
// WKV: one thread per (b, c), state in registers.  The recurrence is a serial chain of T steps per thread, and
// with B * C threads there is about one wavefront per compute unit, so nothing else hides a load: k and v are
// therefore fetched a whole group of steps ahead of the step that uses them (kWkvAhead independent loads in
// flight per thread), and the chain itself, not the memory latency, sets the pace.
// ---------------------------------------------------------------------------
constexpr int kWkvAhead = 16;

__global__ void __launch_bounds__(64)
wkv_f32_kernel(int B, int T, int C, const float *__restrict__ w, const float *__restrict__ u,
               const float *__restrict__ k, const float *__restrict__ v, float *__restrict__ y,
               float *__restrict__ aa, float *__restrict__ bb, float *__restrict__ pp) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * C) return;
    const int b = idx / C, c = idx % C;
    const size_t base = (size_t)b * T * C + c;
    const double wc = (double)w[c], uc = (double)u[c];
    float a = aa[idx], bsum = bb[idx];
    double p = (double)pp[idx];
    float kc[kWkvAhead], vc[kWkvAhead], kn[kWkvAhead], vn[kWkvAhead];
#pragma unroll
    for (int i = 0; i < kWkvAhead; ++i) {
        const size_t o = base + (size_t)min(i, T - 1) * C;
        kc[i] = k[o]; vc[i] = v[o];
    }
    for (int t0 = 0; t0 < T; t0 += kWkvAhead) {
#pragma unroll
        for (int i = 0; i < kWkvAhead; ++i) {           // the next group (clamped at the end: re-reads the last row)
            const size_t o = base + (size_t)min(t0 + kWkvAhead + i, T - 1) * C;
            kn[i] = k[o]; vn[i] = v[o];
        }
#pragma unroll
        for (int i = 0; i < kWkvAhead; ++i) {
            if (t0 + i < T) y[base + (size_t)(t0 + i) * C] = wkv_step_f32(wc, uc, kc[i], vc[i], a, bsum, p);
        }
#pragma unroll
        for (int i = 0; i < kWkvAhead; ++i) { kc[i] = kn[i]; vc[i] = vn[i]; }
    }
    aa[idx] = a; bb[idx] = bsum; pp[idx] = (float)p;
}

// Long sequences: the same recurrence as a two-pass scan inside one workgroup.  The recurrence is linear in
// (aa, bb), so the T steps split into 2 NW chunks: (1) every chunk scans its steps from an empty
// state, (2) its incoming state is the call's state joined with the contributions of the chunks before it
// (a chunk of n steps decays what came in by e^{n w}), (3) it replays its steps from there and writes y.  A
// thread's serial chain is T / NW steps instead of T, there are several wavefronts per SIMD instead
// of a third of one, and k and v are read twice.
// Workgroup = 32 channels of one sequence and NW wavefronts; lane = (chunk parity, channel), wavefront w holds
// chunks 2w and 2w + 1.  Both passes are bound by their vector instructions and the memory traffic once there are
// a few wavefronts per SIMD, so the host picks 8 chunks where that already fills the device and 16 otherwise
// (8 sequences of 2560 channels and 1024 steps: 94-97 us with 8 chunks, 98 with 16, 109 with 32).
constexpr int kWkvScanGroup = 8;
constexpr int kWkvScanMinT = 256;       // shorter sequences stay with the serial kernel

__device__ __forceinline__ void wkv_scan_join(double w, int n, double la, double lb, double lp, double &aa, double &bb, double &pp) {
    const double s = pp + (double)n * w;
    const double p = fmax(s, lp);
    const double f1 = (double)expf((float)(s - p)), f2 = (double)expf((float)(lp - p));   // (one of them is e^0)
    aa = f1 * aa + f2 * la;
    bb = f1 * bb + f2 * lb;
    pp = p;
}

template <int NW>
__global__ void __launch_bounds__(NW * 64)
wkv_f32_scan_kernel(int T, int C, int chunk, const float *__restrict__ w, const float *__restrict__ u,
                    const float *__restrict__ k, const float *__restrict__ v, float *__restrict__ y,
                    float *__restrict__ aa, float *__restrict__ bb, float *__restrict__ pp) {
    constexpr int kChunks = 2 * NW;
    __shared__ double sa[kChunks][32], sb[kChunks][32], sp[kChunks][32];
    const int per_b = C / 32;
    const int b = blockIdx.x / per_b, c = (blockIdx.x % per_b) * 32 + (threadIdx.x & 31);
    const int ch = threadIdx.x & 31, j = (int)(threadIdx.x >> 5);      // chunk of this thread
    const int idx = b * C + c;
    const size_t base = (size_t)b * T * C + c;
    const double wc = (double)w[c], uc = (double)u[c];
    const int t0 = min(j * chunk, T), t1 = min(t0 + chunk, T);
    float kc[kWkvScanGroup], vc[kWkvScanGroup], kn[kWkvScanGroup], vn[kWkvScanGroup];
    // (1) this chunk from an empty state
    float a = 0.f, bs = 0.f;
    double p = -1e30;
    if (t0 < t1) {
#pragma unroll
        for (int i = 0; i < kWkvScanGroup; ++i) {
            const size_t o = base + (size_t)min(t0 + i, t1 - 1) * C;
            kc[i] = k[o]; vc[i] = v[o];
        }
        for (int g = t0; g < t1; g += kWkvScanGroup) {
#pragma unroll
            for (int i = 0; i < kWkvScanGroup; ++i) {       // the next group (past the end: the last row again, unused)
                const size_t o = base + (size_t)min(g + kWkvScanGroup + i, t1 - 1) * C;
                kn[i] = k[o]; vn[i] = v[o];
            }
#pragma unroll
            for (int i = 0; i < kWkvScanGroup; ++i)
                if (g + i < t1) (void)wkv_step_f32(wc, uc, kc[i], vc[i], a, bs, p);
#pragma unroll
            for (int i = 0; i < kWkvScanGroup; ++i) { kc[i] = kn[i]; vc[i] = vn[i]; }
        }
    }
    sa[j][ch] = (double)a; sb[j][ch] = (double)bs; sp[j][ch] = p;
    // the first rows of the replay are on their way while the joins run
    if (t0 < t1) {
#pragma unroll
        for (int i = 0; i < kWkvScanGroup; ++i) {
            const size_t o = base + (size_t)min(t0 + i, t1 - 1) * C;
            kc[i] = k[o]; vc[i] = v[o];
        }
    }
    // the call's state is read ahead of the barrier: the thread with the last chunk overwrites it when it is done
    double ja = (double)aa[idx], jb = (double)bb[idx], jp = (double)pp[idx];
    __syncthreads();
    // (2) the state before this chunk
    for (int jj = 0; jj < j; ++jj) {
        const int n = min(chunk, T - min(jj * chunk, T));
        if (n > 0) wkv_scan_join(wc, n, sa[jj][ch], sb[jj][ch], sp[jj][ch], ja, jb, jp);
    }
    if (t0 >= t1) return;
    // (3) replay
    a = (float)ja; bs = (float)jb; p = jp;
    for (int g = t0; g < t1; g += kWkvScanGroup) {
#pragma unroll
        for (int i = 0; i < kWkvScanGroup; ++i) {
            const size_t o = base + (size_t)min(g + kWkvScanGroup + i, t1 - 1) * C;
            kn[i] = k[o]; vn[i] = v[o];
        }
#pragma unroll
        for (int i = 0; i < kWkvScanGroup; ++i)
            if (g + i < t1) y[base + (size_t)(g + i) * C] = wkv_step_f32(wc, uc, kc[i], vc[i], a, bs, p);
#pragma unroll
        for (int i = 0; i < kWkvScanGroup; ++i) { kc[i] = kn[i]; vc[i] = vn[i]; }
    }
    if (t1 == T) { aa[idx] = a; bb[idx] = bs; pp[idx] = (float)p; }     // the chunk with the last step: the state after it
}

// The same scan with one read of k and v: the sequence is cut into blocks of kWbNC * kWbSB steps that a workgroup
// (32 channels x kWbNC chunk positions) takes one after the other; a thread keeps the kWbSB steps of its chunk in
// registers from the pass that sums them up to the pass that writes y, and the block after next is requested
// while this one is computed.  One barrier per block (summaries and carried state are double-buffered in LDS).
//
// Written for the instruction count - with two and a half wavefronts per SIMD the scan is bound by its vector
// instructions as much as by memory:
//  * e^x for x <= 0 is one scaled v_exp_f32, the division a reciprocal and a multiply (a few ulp each, far inside
//    the 1e-4 the recurrence is held to);
//  * a chunk's summary is a direct sum: step i of n contributes e^{k_i + (n - i) w}, so with m = max_i of those
//    exponents the summary is (sum e^{x_i - m} v_i, sum e^{x_i - m}, m): float32 throughout, no chain;
//  * the state a chunk starts from, and the state a block hands on, are direct sums too: the carried state and
//    the summaries before the chunk, each decayed over the steps in between, with float64 exponents (one
//    exponential per term).  The exponent pp therefore never accumulates float32 roundings along the sequence;
//  * inside a chunk's second pass the exponent is float32, starting from the float32 rounding of the float64
//    exponent the chunk starts with: kWbSB roundings of 2^-24 |pp| at most, that end with the chunk.
template <int kWbNC, int kWbSB>
struct WkvBlockState {
    float kc[kWbSB], vc[kWbSB], kn[kWbSB], vn[kWbSB];
};

__device__ __forceinline__ float wkv_exp_neg(float x) { return __builtin_amdgcn_exp2f(x * 1.44269504088896341f); }   // x <= 0

// One block of kWbNC * kWbSB steps from step tb; buf = parity of the block.  FULL: the block and the block after
// it lie inside the sequence, so no load is clamped and no step is guarded.
template <int kWbNC, int kWbSB, bool FULL>
__device__ __forceinline__ void wkv_block(WkvBlockState<kWbNC, kWbSB> &st, int tb, int T, int C, int j, int ch, unsigned col,
                                          int buf, float wf, float uwf, const float *__restrict__ kb,
                                          const float *__restrict__ vb, float *__restrict__ yb,
                                          float (*sa)[kWbNC][32], float (*sb)[kWbNC][32], double (*sp)[kWbNC][32],
                                          float (*ca)[32], float (*cb)[32], double (*cp)[32]) {
    constexpr int kBlk = kWbNC * kWbSB;
    const double wc = (double)wf;
    const int t0 = FULL ? tb + j * kWbSB : min(tb + j * kWbSB, T), t1 = FULL ? t0 + kWbSB : min(t0 + kWbSB, T);
    const int tbn = FULL ? tb + kBlk : min(tb + kBlk, T), n = t1 - t0;
    // the next block's rows are requested one by one between the steps below, so that the requests of a compute
    // unit form a stream instead of a burst per block (past the end: the last row again, unused)
    const int tn = tb + kBlk + j * kWbSB;
    auto fetch_next = [&](int i) {
        const unsigned o = (unsigned)(FULL ? tn + i : min(tn + i, T - 1)) * (unsigned)C + col;
        st.kn[i] = __builtin_nontemporal_load(kb + o); st.vn[i] = __builtin_nontemporal_load(vb + o);
    };
    // (1) the chunk's summary
    float x[kWbSB], m = -1e30f;
#pragma unroll
    for (int i = 0; i < kWbSB; ++i) {
        x[i] = (FULL || i < n) ? st.kc[i] + (float)(n - i) * wf : -1e30f;
        m = fmaxf(m, x[i]);
    }
    float a = 0.f, bs = 0.f;
#pragma unroll
    for (int i = 0; i < kWbSB; ++i) {
        const float f = (FULL || i < n) ? wkv_exp_neg(x[i] - m) : 0.f;
        a = fmaf(f, st.vc[i], a);
        bs += f;
        if (i < kWbSB / 2) fetch_next(i);
    }
    sa[buf][j][ch] = a; sb[buf][j][ch] = bs; sp[buf][j][ch] = (double)m;
    __syncthreads();
    // (2) the state before this chunk: the carried state decayed over t0 - tb steps plus the summaries of the
    // chunks before it, each decayed over the steps between its end and t0; all on the common exponent pm
    const float car_a = ca[buf][ch], car_b = cb[buf][ch];
    const double car_p = cp[buf][ch];
    double e[kWbNC];
    const double e_car = car_p + (double)(t0 - tb) * wc;
    double pm = e_car;
#pragma unroll
    for (int i = 0; i < kWbNC - 1; ++i) {
        const int end_i = FULL ? tb + (i + 1) * kWbSB : min(tb + (i + 1) * kWbSB, T);
        e[i] = i < j ? sp[buf][i][ch] + (double)(t0 - end_i) * wc : -1e300;
        pm = fmax(pm, e[i]);
    }
    {
        const float f = wkv_exp_neg((float)(e_car - pm));
        a = f * car_a; bs = f * car_b;
    }
#pragma unroll
    for (int i = 0; i < kWbNC - 1; ++i) {
        if (i < j) {
            const float f = wkv_exp_neg((float)(e[i] - pm));
            a = fmaf(f, sa[buf][i][ch], a); bs = fmaf(f, sb[buf][i][ch], bs);
        }
    }
    // the thread of the last chunk position hands the block's end state on: the same sum taken at tbn, its own
    // summary included
    if (j == kWbNC - 1) {
        const double own = sp[buf][j][ch] + (double)(tbn - t1) * wc;
        const double shift = (double)(tbn - t0) * wc;               // everything above, decayed on to tbn
        const double pn = fmax(pm + shift, own);
        const float f0 = wkv_exp_neg((float)(pm + shift - pn)), f1 = wkv_exp_neg((float)(own - pn));
        ca[buf ^ 1][ch] = f0 * a + f1 * sa[buf][j][ch];
        cb[buf ^ 1][ch] = f0 * bs + f1 * sb[buf][j][ch];
        cp[buf ^ 1][ch] = pn;
    }
    // (3) second pass: the outputs (wkv_step_f32 with a float32 exponent)
    float pf = (float)pm;
#pragma unroll
    for (int i = 0; i < kWbSB; ++i) {
        if (FULL || i < n) {
            const float kk = st.kc[i], vv = st.vc[i];
            const float d2 = pf - kk, d = d2 - uwf;
            const float ee = wkv_exp_neg(-fabsf(d)), ff = wkv_exp_neg(-fabsf(d2));
            const float e1 = d >= 0.f ? 1.f : ee, e2 = d >= 0.f ? ee : 1.f;
            const float yv = (e1 * a + e2 * vv) * __builtin_amdgcn_rcpf(fmaf(e1, bs, e2));
            const float f1 = d2 >= 0.f ? 1.f : ff, f2 = d2 >= 0.f ? ff : 1.f;
            a = fmaf(f1, a, f2 * vv);
            bs = fmaf(f1, bs, f2);
            pf = fmaxf(pf, kk) + wf;
            __builtin_nontemporal_store(yv, yb + ((unsigned)(t0 + i) * (unsigned)C + col));
        }
        if (i < kWbSB - kWbSB / 2) fetch_next(kWbSB / 2 + i);
    }
#pragma unroll
    for (int i = 0; i < kWbSB; ++i) { st.kc[i] = st.kn[i]; st.vc[i] = st.vn[i]; }
}

template <int kWbNC, int kWbSB>
__global__ void __launch_bounds__(kWbNC * 32)
wkv_f32_block_kernel(int T, int C, const float *__restrict__ w, const float *__restrict__ u,
                     const float *__restrict__ k, const float *__restrict__ v, float *__restrict__ y,
                     float *__restrict__ aa, float *__restrict__ bb, float *__restrict__ pp) {
    __shared__ float sa[2][kWbNC][32], sb[2][kWbNC][32], ca[2][32], cb[2][32];
    __shared__ double sp[2][kWbNC][32], cp[2][32];
    const int per_b = C / 32;
    const int b = blockIdx.x / per_b, ch = threadIdx.x & 31, j = (int)(threadIdx.x >> 5);
    const unsigned col = (unsigned)((blockIdx.x % per_b) * 32 + ch);
    const int idx = b * C + (int)col;
    // element offsets inside one sequence fit 32 bits (the host checks T * C < 2^30): one uniform base per array
    const float *kb = k + (size_t)b * T * C, *vb = v + (size_t)b * T * C;
    float *yb = y + (size_t)b * T * C;
    const float wf = w[col], uwf = (float)((double)u[col] + (double)wf);
    constexpr int kBlk = kWbNC * kWbSB;
    WkvBlockState<kWbNC, kWbSB> st;
#pragma unroll
    for (int i = 0; i < kWbSB; ++i) {
        const unsigned o = (unsigned)min(j * kWbSB + i, T - 1) * (unsigned)C + col;
        st.kc[i] = __builtin_nontemporal_load(kb + o); st.vc[i] = __builtin_nontemporal_load(vb + o);
    }
    if (j == 0) { ca[0][ch] = aa[idx]; cb[0][ch] = bb[idx]; cp[0][ch] = (double)pp[idx]; }      // (read after the first block's barrier)
    int tb = 0, buf = 0;
    for (; tb + 2 * kBlk <= T; tb += kBlk, buf ^= 1)
        wkv_block<kWbNC, kWbSB, true>(st, tb, T, C, j, ch, col, buf, wf, uwf, kb, vb, yb, sa, sb, sp, ca, cb, cp);
    for (; tb < T; tb += kBlk, buf ^= 1)
        wkv_block<kWbNC, kWbSB, false>(st, tb, T, C, j, ch, col, buf, wf, uwf, kb, vb, yb, sa, sb, sp, ca, cb, cp);
    __syncthreads();
    if (j == 0) { aa[idx] = ca[buf][ch]; bb[idx] = cb[buf][ch]; pp[idx] = (float)cp[buf][ch]; }
}

// Reference convention (cuda/operators.cu:6-37): naive pre-multiplied state in
// and out, pp untouched; the max-shifted form runs in between.
__global__ void __launch_bounds__(64)
wkv_f64_ref_kernel(int B, int T, int C, const double *__restrict__ w, const double *__restrict__ u,
                   const double *__restrict__ k, const double *__restrict__ v, double *__restrict__ y,
                   double *__restrict__ aa, double *__restrict__ bb) {
    const int idx = blockIdx.x * blockDim.x + threadIdx.x;
    if (idx >= B * C) return;
    const int b = idx / C, c = idx % C;
    const size_t base = (size_t)b * T * C + c;
    const double wc = w[c], uc = u[c];
    // naive (aa, bb) == shifted (aa, bb, pp = 0)
    double a = aa[idx], bsum = bb[idx], p = 0.0;
    if (!(bsum > 0.0)) p = -1e300;   // empty state: let the first token dominate exactly
    for (int t = 0; t < T; ++t) {
        const size_t o = base + (size_t)t * C;
        y[o] = wkv_step<double>(wc, uc, k[o], v[o], a, bsum, p);
    }
    const double e = exp(p);
    aa[idx] = a * e;
    bb[idx] = bsum * e;
}

// First index of the maximum (torch.argmax tie rule is unspecified; greedy
// decoding here takes the lowest index).
__global__ void __launch_bounds__(1024)
argmax_f64_kernel(const double *__restrict__ logits, int V, int64_t *__restrict__ out) {
    __shared__ double sval[16];
    __shared__ int sidx[16];
    double best = -INFINITY;
    int bi = 0x7fffffff;
    for (int i = threadIdx.x; i < V; i += blockDim.x) {
        const double x = logits[i];
        if (x > best) { best = x; bi = i; }
    }
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) {
        const double ob = __shfl_xor(best, off, 64);
        const int oi = __shfl_xor(bi, off, 64);
        if (ob > best || (ob == best && oi < bi)) { best = ob; bi = oi; }
    }
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    if (lane == 0) { sval[wave] = best; sidx[wave] = bi; }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (int wv = 1; wv < (int)(blockDim.x >> 6); ++wv)
            if (sval[wv] > best || (sval[wv] == best && sidx[wv] < bi)) { best = sval[wv]; bi = sidx[wv]; }
        out[0] = (bi == 0x7fffffff) ? 0 : bi;
    }
}

// ---------------------------------------------------------------------------
// Reference layout w[n_in][n_out] (row stride w_stride), operators32.cu:18-83.
// Workgroup (ct, sp): columns 256*ct .. +255, rows of split sp.  Lane cx of
// wave ky handles VEC consecutive columns of rows ky, ky+4, ...; x[j]*r[j] is
// wave-uniform.  Partials go to scratch[sp][m][k]; mm8_ref_reduce_kernel adds
// them in split order and accumulates into y (deterministic).
// ---------------------------------------------------------------------------
constexpr int kRefSplitRows = 128;

// T: float (operators32.cu) or double (operators.cu:58-80, the dispatch of wrapper.cpp:60-77): the type of x, r, y and
// of the sums.
template <typename T, int NM, int VEC>
__global__ void __launch_bounds__(kThreads)
mm8_ref_partial_kernel(int n_in, int n_out,
                       const T *x0, const T *x1, const T *x2,
                       const uint8_t *w0, const uint8_t *w1, const uint8_t *w2,
                       int64_t s0, int64_t s1, int64_t s2,
                       const T *r0, const T *r1, const T *r2,
                       T *__restrict__ scratch) {
    __shared__ T xs[NM][kRefSplitRows];
    __shared__ T red[kWaves][NM][64 * VEC];
    const T *xp[3] = {x0, x1, x2};
    const T *rp[3] = {r0, r1, r2};
    const uint8_t *wp[3] = {w0, w1, w2};
    const int64_t sp_[3] = {s0, s1, s2};
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int j0 = blockIdx.y * kRefSplitRows;
    const int rows = min(kRefSplitRows, n_in - j0);
    for (int i = threadIdx.x; i < NM * kRefSplitRows; i += kThreads) {
        const int m = i / kRefSplitRows, jj = i % kRefSplitRows;
        // operators32.cu:33-36 multiplies x[j] * (w * r[j]); here x[j]*r[j] is
        // formed once per row (same rounding as the reference CPU path,
        // matmul.py:131).
        xs[m][jj] = jj < rows ? xp[m][j0 + jj] * rp[m][j0 + jj] : (T)0;
    }
    __syncthreads();
    const int k0 = (blockIdx.x * 64 + lane) * VEC;
    T acc[NM][VEC];
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int e = 0; e < VEC; ++e) acc[m][e] = (T)0;
    if (k0 < n_out) {
        for (int jj = wave; jj < rows; jj += kWaves) {
#pragma unroll
            for (int m = 0; m < NM; ++m) {
                const uint8_t *row = wp[m] + (size_t)(j0 + jj) * sp_[m] + k0;
                const T xv = xs[m][jj];
                if (VEC == 4) {
                    uint32_t d;
                    if (k0 + 4 <= n_out) {
                        d = *reinterpret_cast<const uint32_t *>(row);
                    } else {   // ragged last group: never read past the row
                        d = 0;
                        for (int e = 0; k0 + e < n_out; ++e) d |= (uint32_t)row[e] << (8 * e);
                    }
                    acc[m][0] = fma((T)ubyte0(d), xv, acc[m][0]);
                    acc[m][1] = fma((T)ubyte1(d), xv, acc[m][1]);
                    acc[m][2] = fma((T)ubyte2(d), xv, acc[m][2]);
                    acc[m][3] = fma((T)ubyte3(d), xv, acc[m][3]);
                } else {
                    acc[m][0] = fma((T)row[0], xv, acc[m][0]);
                }
            }
        }
    }
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int e = 0; e < VEC; ++e) red[wave][m][lane * VEC + e] = acc[m][e];
    __syncthreads();
    for (int i = threadIdx.x; i < NM * 64 * VEC; i += kThreads) {
        const int m = i / (64 * VEC), kk = i % (64 * VEC);
        const int k = blockIdx.x * 64 * VEC + kk;
        if (k < n_out)
            scratch[((size_t)blockIdx.y * NM + m) * n_out + k] =
                (red[0][m][kk] + red[1][m][kk]) + (red[2][m][kk] + red[3][m][kk]);
    }
}

template <typename T, int NM>
__global__ void __launch_bounds__(256)
mm8_ref_reduce_kernel(int n_out, int n_split, const T *__restrict__ scratch,
                      T *y0, T *y1, T *y2) {
    T *yp[3] = {y0, y1, y2};
    const int k = blockIdx.x * blockDim.x + threadIdx.x;
    if (k >= n_out) return;
#pragma unroll
    for (int m = 0; m < NM; ++m) {
        T s = (T)0;
        for (int sp = 0; sp < n_split; ++sp) s += scratch[((size_t)sp * NM + m) * n_out + k];
        yp[m][k] += s;   // the reference accumulates into y (operators32.cu:38)
    }
}

template <typename T>
static int mm8_ref_launch(hipStream_t st, int nm, int64_t n_in, int64_t n_out,
                          const T *const x[3], const uint8_t *const w[3], const int64_t stride[3],
                          T *const y[3], const T *const r[3], void *ws, size_t ws_bytes) {
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && n_in < (1 << 30) && n_out < (1 << 30), "mm8: bad sizes");
    bool vec4 = true;
    for (int m = 0; m < nm; ++m) {
        RWKV_CHECK_ARG(x[m] && w[m] && y[m] && r[m], "mm8: null pointer");
        RWKV_CHECK_ARG(stride[m] >= n_out, "mm8: w_stride < n_out");
        RWKV_CHECK_ALIGN(x[m], sizeof(T)); RWKV_CHECK_ALIGN(y[m], sizeof(T)); RWKV_CHECK_ALIGN(r[m], sizeof(T));
        if (reinterpret_cast<uintptr_t>(w[m]) % 4 || stride[m] % 4) vec4 = false;
    }
    const size_t need = (size_t)(ceil_div(n_in, kRefSplitRows) * nm * n_out) * sizeof(T);
    if (!ws || ws_bytes < need)
        return set_error(RWKV_ERR_WORKSPACE, "mm8: workspace of %zu bytes needed, %zu given", need, ws_bytes);
    RWKV_CHECK_ALIGN(ws, sizeof(T));
    const int n_split = (int)ceil_div(n_in, kRefSplitRows);
    T *scratch = static_cast<T *>(ws);
    const int vec = vec4 ? 4 : 1;
    dim3 grid((unsigned)ceil_div(n_out, 64 * vec), (unsigned)n_split);
#define LAUNCH_P(NM, VEC) \
    hipLaunchKernelGGL((mm8_ref_partial_kernel<T, NM, VEC>), grid, dim3(kThreads), 0, st, (int)n_in, (int)n_out, \
                       x[0], x[1], x[2], w[0], w[1], w[2], stride[0], stride[1], stride[2], r[0], r[1], r[2], scratch)
    if (nm == 1) { if (vec4) LAUNCH_P(1, 4); else LAUNCH_P(1, 1); }
    else         { if (vec4) LAUNCH_P(3, 4); else LAUNCH_P(3, 1); }
#undef LAUNCH_P
    RWKV_CHECK_LAUNCH("mm8_ref_partial_kernel");
    dim3 rgrid((unsigned)ceil_div(n_out, 256));
    if (nm == 1)
        hipLaunchKernelGGL((mm8_ref_reduce_kernel<T, 1>), rgrid, dim3(256), 0, st, (int)n_out, n_split, scratch, y[0], y[1], y[2]);
    else
        hipLaunchKernelGGL((mm8_ref_reduce_kernel<T, 3>), rgrid, dim3(256), 0, st, (int)n_out, n_split, scratch, y[0], y[1], y[2]);
    RWKV_CHECK_LAUNCH("mm8_ref_reduce_kernel");
    return RWKV_OK;
}

// ---------------------------------------------------------------------------
// Scratch for callers that cannot hand over (or allocate) a workspace: a fixed array in the library's own
// device image.  Every GPU the library runs on holds its own copy, at its own address, until the process
// ends; the array's name below is only the host-side handle of the symbol, the device address comes from
// hipGetSymbolAddress, once per device, with that device current.
// ---------------------------------------------------------------------------
constexpr size_t kStaticScratchBytes = (size_t)12 << 20;     // the [5120 x 50277] head of the 14B shape needs 8.05 MB
static __device__ __align__(256) unsigned char scratch[kStaticScratchBytes];

constexpr int kScratchMaxDevices = 64;
static std::mutex scratch_mu;
static void *scratch_ptr[kScratchMaxDevices] = {};

static int static_scratch(void **out) {
    int dev = 0;
    RWKV_CHECK_HIP(hipGetDevice(&dev));
    if (dev < 0 || dev >= kScratchMaxDevices) return set_error(RWKV_ERR_DEVICE, "device index %d out of range", dev);
    std::lock_guard<std::mutex> lock(scratch_mu);
    if (!scratch_ptr[dev]) {
        void *p = nullptr;
        RWKV_CHECK_HIP(hipGetSymbolAddress(&p, HIP_SYMBOL(scratch)));
        if (!p) return set_error(RWKV_ERR_HIP, "hipGetSymbolAddress returned a null address for the scratch array");
        scratch_ptr[dev] = p;
    }
    *out = scratch_ptr[dev];
    return RWKV_OK;
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

size_t rwkv_mm8_workspace_bytes(int64_t n_in, int64_t n_out, int n_mat) {
    if (n_in <= 0 || n_out <= 0 || n_mat <= 0) return 0;
    return (size_t)(ceil_div(n_in, kRefSplitRows) * n_mat * n_out) * sizeof(float);
}

int rwkv_mm8_one(rwkv_stream_t stream, int64_t n_in, int64_t n_out, const float *x, const uint8_t *w,
                 int64_t w_stride, float *y, const float *r, void *workspace, size_t workspace_bytes) {
    const float *xs[3] = {x, x, x};
    const uint8_t *ws_[3] = {w, w, w};
    const int64_t st[3] = {w_stride, w_stride, w_stride};
    float *ys[3] = {y, y, y};
    const float *rs[3] = {r, r, r};
    return mm8_ref_launch<float>((hipStream_t)stream, 1, n_in, n_out, xs, ws_, st, ys, rs, workspace, workspace_bytes);
}

size_t rwkv_mm8_one_static_max_bytes(void) {
    // Also the warm-up of rwkv_mm8_one_static on the current device: the symbol look-up of the first call is not
    // something a stream capture should contain, so a caller about to capture asks for the limit first.  Best
    // effort: without a usable device the limit is still returned and the entry point itself reports the error.
    void *p = nullptr;
    (void)static_scratch(&p);
    return kStaticScratchBytes;
}

int rwkv_mm8_one_static(rwkv_stream_t stream, int64_t n_in, int64_t n_out, const float *x, const uint8_t *w,
                        int64_t w_stride, float *y, const float *r) {
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && n_in < (1 << 30) && n_out < (1 << 30), "mm8: bad sizes");
    const size_t need = rwkv_mm8_workspace_bytes(n_in, n_out, 1);
    if (need > kStaticScratchBytes)
        return set_error(RWKV_ERR_SIZE, "rwkv_mm8_one_static: [%lld x %lld] needs %zu bytes of scratch, the built-in "
                                        "array holds %zu; use rwkv_mm8_one with a workspace",
                         (long long)n_in, (long long)n_out, need, kStaticScratchBytes);
    void *ws = nullptr;
    const int rc = static_scratch(&ws);
    if (rc) return rc;
    // every partial sum the reduce kernel reads is written by the partial kernel of the same call: nothing of
    // an earlier call's contents is read, so the array needs no clearing
    return rwkv_mm8_one(stream, n_in, n_out, x, w, w_stride, y, r, ws, kStaticScratchBytes);
}

int rwkv_mm8_three(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                   const float *x0, const float *x1, const float *x2,
                   const uint8_t *w0, int64_t w0_stride, const uint8_t *w1, int64_t w1_stride,
                   const uint8_t *w2, int64_t w2_stride, float *y0, float *y1, float *y2,
                   const float *r0, const float *r1, const float *r2,
                   void *workspace, size_t workspace_bytes) {
    const float *xs[3] = {x0, x1, x2};
    const uint8_t *ws_[3] = {w0, w1, w2};
    const int64_t st[3] = {w0_stride, w1_stride, w2_stride};
    float *ys[3] = {y0, y1, y2};
    const float *rs[3] = {r0, r1, r2};
    return mm8_ref_launch<float>((hipStream_t)stream, 3, n_in, n_out, xs, ws_, st, ys, rs, workspace, workspace_bytes);
}

size_t rwkv_mm8_f64_workspace_bytes(int64_t n_in, int64_t n_out, int n_mat) {
    if (n_in <= 0 || n_out <= 0 || n_mat <= 0) return 0;
    return (size_t)(ceil_div(n_in, kRefSplitRows) * n_mat * n_out) * sizeof(double);
}

int rwkv_mm8_one_f64(rwkv_stream_t stream, int64_t n_in, int64_t n_out, const double *x, const uint8_t *w,
                     int64_t w_stride, double *y, const double *r, void *workspace, size_t workspace_bytes) {
    const double *xs[3] = {x, x, x};
    const uint8_t *ws_[3] = {w, w, w};
    const int64_t st[3] = {w_stride, w_stride, w_stride};
    double *ys[3] = {y, y, y};
    const double *rs[3] = {r, r, r};
    return mm8_ref_launch<double>((hipStream_t)stream, 1, n_in, n_out, xs, ws_, st, ys, rs, workspace, workspace_bytes);
}

int rwkv_mm8_three_f64(rwkv_stream_t stream, int64_t n_in, int64_t n_out,
                       const double *x0, const double *x1, const double *x2,
                       const uint8_t *w0, int64_t w0_stride, const uint8_t *w1, int64_t w1_stride,
                       const uint8_t *w2, int64_t w2_stride, double *y0, double *y1, double *y2,
                       const double *r0, const double *r1, const double *r2,
                       void *workspace, size_t workspace_bytes) {
    const double *xs[3] = {x0, x1, x2};
    const uint8_t *ws_[3] = {w0, w1, w2};
    const int64_t st[3] = {w0_stride, w1_stride, w2_stride};
    double *ys[3] = {y0, y1, y2};
    const double *rs[3] = {r0, r1, r2};
    return mm8_ref_launch<double>((hipStream_t)stream, 3, n_in, n_out, xs, ws_, st, ys, rs, workspace, workspace_bytes);
}

int rwkv_wkv_forward_f64(rwkv_stream_t stream, int64_t B, int64_t T, int64_t C,
                         const double *w, const double *u, const double *k, const double *v,
                         double *y, double *aa, double *bb, double *pp) {
    RWKV_CHECK_ARG(w && u && k && v && y && aa && bb && pp, "rwkv_wkv_forward_f64: null pointer");
    RWKV_CHECK_ARG(B > 0 && T > 0 && C > 0 && B * C < (1ll << 31) && T < (1ll << 31), "rwkv_wkv_forward_f64: bad sizes");
    RWKV_CHECK_ALIGN(k, 8); RWKV_CHECK_ALIGN(v, 8); RWKV_CHECK_ALIGN(y, 8);
    hipLaunchKernelGGL(wkv_f64_ref_kernel, dim3((unsigned)ceil_div(B * C, 64)), dim3(64), 0, (hipStream_t)stream,
                       (int)B, (int)T, (int)C, w, u, k, v, y, aa, bb);
    RWKV_CHECK_LAUNCH("wkv_f64_ref_kernel");
    (void)pp;  // passed through untouched, as in the reference kernel
    return RWKV_OK;
}

int rwkv_wkv_f32(rwkv_stream_t stream, int64_t B, int64_t T, int64_t C, const float *w, const float *u,
                 const float *k, const float *v, float *y, float *aa, float *bb, float *pp) {
    RWKV_CHECK_ARG(w && u && k && v && y && aa && bb && pp, "rwkv_wkv_f32: null pointer");
    RWKV_CHECK_ARG(B > 0 && T > 0 && C > 0 && B * C < (1ll << 31) && T < (1ll << 31), "rwkv_wkv_f32: bad sizes");
    RWKV_CHECK_ALIGN(k, 4); RWKV_CHECK_ALIGN(v, 4); RWKV_CHECK_ALIGN(y, 4);
    if (T >= kWkvScanMinT && C % 32 == 0 && B * (C / 32) < (1ll << 31)) {
        const dim3 grid((unsigned)(B * (C / 32)));
        if (B * (C / 32) >= 512 && T * C < (1ll << 30)) {     // enough workgroups for the one-read form
            // 4 chunk positions of 16 steps: 128 threads, five workgroups per compute unit at 8 x 2560 channels
            hipLaunchKernelGGL((wkv_f32_block_kernel<4, 16>), grid, dim3(4 * 32), 0, (hipStream_t)stream, (int)T, (int)C,
                               w, u, k, v, y, aa, bb, pp);
            RWKV_CHECK_LAUNCH("wkv_f32_block_kernel");
            return RWKV_OK;
        }
        if (B * (C / 32) * 4 >= 2048) {         // 8 chunks already give every SIMD two wavefronts
            const int chunk = (int)round_up((size_t)ceil_div(T, 8), kWkvScanGroup);
            hipLaunchKernelGGL(wkv_f32_scan_kernel<4>, grid, dim3(4 * 64), 0, (hipStream_t)stream, (int)T, (int)C, chunk,
                               w, u, k, v, y, aa, bb, pp);
        } else {
            const int chunk = (int)round_up((size_t)ceil_div(T, 16), kWkvScanGroup);
            hipLaunchKernelGGL(wkv_f32_scan_kernel<8>, grid, dim3(8 * 64), 0, (hipStream_t)stream, (int)T, (int)C, chunk,
                               w, u, k, v, y, aa, bb, pp);
        }
        RWKV_CHECK_LAUNCH("wkv_f32_scan_kernel");
        return RWKV_OK;
    }
    hipLaunchKernelGGL(wkv_f32_kernel, dim3((unsigned)ceil_div(B * C, 64)), dim3(64), 0, (hipStream_t)stream,
                       (int)B, (int)T, (int)C, w, u, k, v, y, aa, bb, pp);
    RWKV_CHECK_LAUNCH("wkv_f32_kernel");
    return RWKV_OK;
}

int rwkv_argmax_f64(rwkv_stream_t stream, const double *logits, int64_t V, int64_t *out_token) {
    RWKV_CHECK_ARG(logits && out_token, "rwkv_argmax_f64: null pointer");
    RWKV_CHECK_ARG(V > 0 && V < (1ll << 31), "rwkv_argmax_f64: bad size");
    hipLaunchKernelGGL(argmax_f64_kernel, dim3(1), dim3(1024), 0, (hipStream_t)stream, logits, (int)V, out_token);
    RWKV_CHECK_LAUNCH("argmax_f64_kernel");
    return RWKV_OK;
}

int rwkv_mm8_packed(rwkv_stream_t stream, int64_t B, int64_t n_in, int64_t n_out, const float *x,
                    const uint8_t *packed, const float *r_row, const double *m_row,
                    const float *r_col, const float *m_col, double *y) {
    RWKV_CHECK_ARG(x && packed && r_row && m_row && y, "rwkv_mm8_packed: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && n_in < (1 << 30) && n_out < (1 << 30), "rwkv_mm8_packed: bad sizes");
    if (!(B == 1 || B == 2 || B == 4 || B == 8))
        return set_error(RWKV_ERR_SIZE, "rwkv_mm8_packed: B must be 1, 2, 4 or 8 (got %lld)", (long long)B);
    RWKV_CHECK_ALIGN(packed, 16);
    RWKV_CHECK_ALIGN(x, 4); RWKV_CHECK_ALIGN(r_row, 4); RWKV_CHECK_ALIGN(m_row, 8); RWKV_CHECK_ALIGN(y, 8);
    const int n_kb = (int)ceil_div(n_in, kBlockRows);
    hipStream_t st = (hipStream_t)stream;
    if (B == 1 && n_in <= kOneStage * 1024) {
        // One vector: the variant that stages once per workgroup and requests the whole matrix up front.
        // Workgroups of nw wavefronts (each takes every nw-th block of a tile, at most vb of them), nt tiles each,
        // so that there is about one workgroup per compute unit.
        const int64_t n_tiles1 = ceil_div(n_out, kTileCols);
        int nw = 4;
        while (nw < 16 && (ceil_div(n_kb, nw) > 5 || nw * 64 * kOneStage < n_in)) nw += (nw == 8 ? 2 : nw == 10 ? 6 : 4);   // 4, 8, 10, 16
        if (n_kb % 10 == 0 && n_kb / 10 <= 2 && nw < 10 && n_in <= 640 * kOneStage) nw = 10;     // 1280 or 2560 rows: an exact split over 10 wavefronts
        const int vb = (int)ceil_div(n_kb, nw);
        // as many tiles per workgroup as leave at least 160 workgroups: fewer re-reads of the vector, and every
        // workgroup resident at once (one workgroup of 10 or 16 wavefronts fills a compute unit's registers)
        const int nt = (vb <= 2 && n_tiles1 >= 5 * 160) ? 5 : n_tiles1 >= 2 * 160 ? 2 : 1;
        if (vb <= 5 && nw * 64 * kOneStage >= n_in) {
            const size_t lds1 = (size_t)n_kb * kBlockRows * 4 + 2 * nw * 8 + (size_t)nt * nw * 8 * 4;
            const dim3 grid1((unsigned)ceil_div(n_tiles1, nt)), block1((unsigned)(nw * 64));
#define LAUNCH_ONE(NT, VB) \
            hipLaunchKernelGGL((mm8_packed_one_kernel<NT, VB>), grid1, block1, lds1, st, (int)n_in, (int)n_out, n_kb, \
                               x, packed, r_row, m_row, r_col, m_col, y)
            if (nt == 5) LAUNCH_ONE(5, 2);
            else if (nt == 2) { if (vb <= 2) LAUNCH_ONE(2, 2); else LAUNCH_ONE(2, 5); }
            else if (vb <= 2) LAUNCH_ONE(1, 2);
            else LAUNCH_ONE(1, 5);
#undef LAUNCH_ONE
            RWKV_CHECK_LAUNCH("mm8_packed_one_kernel");
            return RWKV_OK;
        }
    }
    // LDS budget for the staged activations: 48 KiB per chunk
    int kc_blocks = (int)(49152 / (B * kBlockRows * 4));
    if (kc_blocks > n_kb) kc_blocks = n_kb;
    // Four column tiles per workgroup where four or eight activation vectors meet a wide matrix: the staging and
    // the LDS reads of the activations, shared by the four tiles, are then the larger part of a workgroup's
    // work, and the grid still has more workgroups than compute units.  (Measured at 8 vectors: [2560 x 10240]
    // 36 -> 29 us; with 320 tiles, two tiles per workgroup lose 1 to 5 us, and workgroups of 16 wavefronts lose more.)
    const int64_t n_tiles = ceil_div(n_out, kTileCols);
    const int nt = (B >= 4 && n_tiles >= 1024) ? 4 : 1;
    const size_t lds = (size_t)B * kc_blocks * kBlockRows * 4 + 2 * B * kWaves * 8 + (size_t)nt * B * kWaves * 8 * 4;
    dim3 grid((unsigned)ceil_div(n_tiles, nt));
#define LAUNCH_B(NB, NT) \
    hipLaunchKernelGGL((mm8_packed_kernel<NB, NT, kWaves>), grid, dim3(kThreads), lds, st, (int)n_in, (int)n_out, n_kb, kc_blocks, \
                       x, packed, r_row, m_row, r_col, m_col, y)
    switch (B) {
        case 1: LAUNCH_B(1, 1); break;
        case 2: LAUNCH_B(2, 1); break;
        case 4: if (nt == 4) LAUNCH_B(4, 4); else LAUNCH_B(4, 1); break;
        default: if (nt == 4) LAUNCH_B(8, 4); else LAUNCH_B(8, 1); break;
    }
#undef LAUNCH_B
    RWKV_CHECK_LAUNCH("mm8_packed_kernel");
    return RWKV_OK;
}

size_t rwkv_mm8_m16_workspace_bytes(int64_t B, int64_t n_in) {
    if (B <= 0 || B > 8 || n_in <= 0) return 0;
    return rows_mv16_workspace_bytes(B, n_in);
}

int rwkv_mm8_m16(rwkv_stream_t stream, int64_t B, int64_t n_in, int64_t n_out, const float *x,
                 const uint8_t *packed16, const float *r_row, const double *m_row,
                 const float *r_col, const float *m_col, double *y, void *workspace, size_t workspace_bytes) {
    RWKV_CHECK_ARG(x && packed16 && r_row && m_row && y, "rwkv_mm8_m16: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && n_in < (1 << 30) && n_out < (1 << 30), "rwkv_mm8_m16: bad sizes");
    if (B < 1 || B > 8) return set_error(RWKV_ERR_SIZE, "rwkv_mm8_m16: B must be 1..8 (got %lld)", (long long)B);
    RWKV_CHECK_ALIGN(packed16, 16);
    RWKV_CHECK_ALIGN(x, 4); RWKV_CHECK_ALIGN(r_row, 4); RWKV_CHECK_ALIGN(m_row, 8); RWKV_CHECK_ALIGN(y, 8);
    const size_t need = rows_mv16_workspace_bytes(B, n_in);
    if (!workspace || workspace_bytes < need)
        return set_error(RWKV_ERR_WORKSPACE, "rwkv_mm8_m16: workspace of %zu bytes needed, %zu given", need, workspace_bytes);
    RWKV_CHECK_ALIGN(workspace, 256);
    return rows_mv16((hipStream_t)stream, B, n_in, n_out, x, packed16, r_row, m_row, r_col, m_col, y, workspace);
}

}  // extern "C"
