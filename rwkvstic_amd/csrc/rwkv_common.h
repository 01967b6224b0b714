// Shared host/device helpers for librwkv_hip.so (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <stdio.h>
#include <stdarg.h>

#include "../../include/rwkv_hip.h"

namespace rwkv {

// ---- packed weight layout -------------------------------------------------
constexpr int kTileCols = 8;     // output columns per block
constexpr int kBlockRows = 128;  // input rows per block
constexpr int kBlockBytes = kTileCols * kBlockRows;  // 1024

constexpr int kWaves = 4;              // wavefronts per workgroup in the matvec kernels
constexpr int kThreads = kWaves * 64;  // 256

__host__ __device__ inline int64_t ceil_div(int64_t a, int64_t b) { return (a + b - 1) / b; }
__host__ __device__ inline int64_t round_up(int64_t a, int64_t b) { return ceil_div(a, b) * b; }

// ---- host-side error reporting --------------------------------------------
int set_error(int code, const char *fmt, ...);

#define RWKV_CHECK_ARG(cond, ...) \
    do { if (!(cond)) return ::rwkv::set_error(RWKV_ERR_ARG, __VA_ARGS__); } while (0)
#define RWKV_CHECK_ALIGN(ptr, a) \
    do { if ((reinterpret_cast<uintptr_t>(ptr) % (a)) != 0) \
        return ::rwkv::set_error(RWKV_ERR_ALIGN, #ptr " must be %d-byte aligned", int(a)); } while (0)
#define RWKV_CHECK_HIP(expr) \
    do { hipError_t e_ = (expr); if (e_ != hipSuccess) \
        return ::rwkv::set_error(RWKV_ERR_HIP, "%s: %s", #expr, hipGetErrorString(e_)); } while (0)
#define RWKV_CHECK_LAUNCH(name) \
    do { hipError_t e_ = hipGetLastError(); if (e_ != hipSuccess) \
        return ::rwkv::set_error(RWKV_ERR_HIP, "launch of %s: %s", name, hipGetErrorString(e_)); } while (0)

// ---- device helpers ---------------------------------------------------------
#if defined(__HIPCC__)

__device__ __forceinline__ float ubyte0(uint32_t d) { return (float)(d & 0xffu); }
__device__ __forceinline__ float ubyte1(uint32_t d) { return (float)((d >> 8) & 0xffu); }
__device__ __forceinline__ float ubyte2(uint32_t d) { return (float)((d >> 16) & 0xffu); }
__device__ __forceinline__ float ubyte3(uint32_t d) { return (float)(d >> 24); }

// acc += dot(4 codes packed in d, xv)
__device__ __forceinline__ float dot4_u8(uint32_t d, const float4 &xv, float acc) {
    acc = fmaf(ubyte0(d), xv.x, acc);
    acc = fmaf(ubyte1(d), xv.y, acc);
    acc = fmaf(ubyte2(d), xv.z, acc);
    acc = fmaf(ubyte3(d), xv.w, acc);
    return acc;
}

// Butterfly sums: every lane ends with the same value (x + y is commutative,
// so both partners of each exchange compute identical bits).
__device__ __forceinline__ double wave_sum(double v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}
__device__ __forceinline__ float wave_sum(float v) {
#pragma unroll
    for (int off = 32; off >= 1; off >>= 1) v += __shfl_xor(v, off, 64);
    return v;
}

// Sum of N values per thread across a workgroup of kWaves wavefronts; fixed
// order, result broadcast to all threads.  red: LDS scratch of N*kWaves doubles.
template <int N>
__device__ __forceinline__ void block_sum(double (&v)[N], double *red) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = wave_sum(v[i]);
        if (lane == 0) red[i * kWaves + wave] = s;
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < N; ++i) {
        double s = 0.0;
#pragma unroll
        for (int w = 0; w < kWaves; ++w) s += red[i * kWaves + w];
        v[i] = s;
    }
    __syncthreads();
}

__device__ __forceinline__ float sigmoid_f32(float x) { return 1.0f / (1.0f + expf(-x)); }

// One step of the max-shifted WKV recurrence on the e^w-premultiplied state:
//   y = (aa e^pp + e^{u+w+k} v) / (bb e^pp + e^{u+w+k});
//   aa e^pp <- e^w (aa e^pp) + e^{w+k} v   (same for bb).
template <typename F>
__device__ __forceinline__ F wkv_step(F w, F u, F k, F v, F &aa, F &bb, F &pp) {
    // Of each pair of exponentials one is e^0: with d = a - b, (e^{a - max}, e^{b - max}) is (1, e^{-d}) or
    // (e^{d}, 1), so one call per pair gives the same bits as two.
    const F q = u + w + k;
    const F d = pp - q;
    const F e = exp(-fabs(d));
    const F e1 = d >= F(0) ? F(1) : e, e2 = d >= F(0) ? e : F(1);
    const F y = (e1 * aa + e2 * v) / (e1 * bb + e2);
    const F s = pp + w, r = k + w;
    const F d2 = s - r;
    const F f = exp(-fabs(d2));
    const F p2 = fmax(s, r);
    const F f1 = d2 >= F(0) ? F(1) : f, f2 = d2 >= F(0) ? f : F(1);
    aa = f1 * aa + f2 * v;
    bb = f1 * bb + f2;
    pp = p2;
    return y;
}
// float32 sums with a float64 exponent.  Adding w to pp at every step in
// float32 would commit the same rounding error T times (a systematic drift of
// up to T * 2^-24 in the scale e^pp); the exponent bookkeeping is therefore
// carried in float64 while aa, bb, the exponentials and the output stay float32.
__device__ __forceinline__ float wkv_step_f32(double w, double u, float k, float v,
                                              float &aa, float &bb, double &pp) {
    // as in wkv_step: of each pair of exponentials one is e^0, so one call per pair gives the same bits as two
    // (the float32 rounding of a difference and of its negative are each other's negatives)
    const double d = pp - (u + w + (double)k);
    const float e = expf(-fabsf((float)d));
    const float e1 = d >= 0.0 ? 1.f : e, e2 = d >= 0.0 ? e : 1.f;
    const float y = (e1 * aa + e2 * v) / (e1 * bb + e2);
    const double s = pp + w, r = (double)k + w;
    const double d2 = s - r;
    const float f = expf(-fabsf((float)d2));
    const float f1 = d2 >= 0.0 ? 1.f : f, f2 = d2 >= 0.0 ? f : 1.f;
    aa = f1 * aa + f2 * v;
    bb = f1 * bb + f2;
    pp = fmax(s, r);
    return y;
}

// ---- the streaming tile product ---------------------------------------------
// One workgroup computes, for NM matrices that share n_in, the dot products of
// one 8-column tile with NB activation vectors held in LDS.
//   wtile[m] : first block of the tile in matrix m (blocks of the tile are
//              contiguous: kb-th block at wtile + kb*1024)
//   xs[m]    : LDS, NB vectors of `xs_stride` floats each (zero padded to a
//              multiple of 128), already multiplied by the per-row range
// Wave w takes blocks kb = kb_begin + w, + kWaves, ...; lane (s = lane/8,
// c = lane%8) accumulates column c over rows 32m+4s+e of each block.
// After the call acc[m][b] holds this lane's partial sums; reduce_tile() turns
// them into column sums.
constexpr int kUnroll = 5;

template <int NM, int NB>
__device__ __forceinline__ void tile_accumulate(const uint8_t *const (&wtile)[NM],
                                                const float *const (&xs)[NM], int xs_stride,
                                                int kb_begin, int kb_end,
                                                float (&acc)[NM][NB]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const int s = lane >> 3;
    for (int kb0 = kb_begin + wave; kb0 < kb_end; kb0 += kWaves * kUnroll) {
        uint4 wv[NM][kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int kb = kb0 + u * kWaves;
            if (kb < kb_end) {
#pragma unroll
                for (int m = 0; m < NM; ++m)
                    wv[m][u] = *reinterpret_cast<const uint4 *>(wtile[m] + (size_t)kb * kBlockBytes + lane * 16);
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int kb = kb0 + u * kWaves;
            if (kb < kb_end) {
#pragma unroll
                for (int m = 0; m < NM; ++m) {
                    const uint32_t d[4] = {wv[m][u].x, wv[m][u].y, wv[m][u].z, wv[m][u].w};
#pragma unroll
                    for (int b = 0; b < NB; ++b) {
                        const float4 *xp = reinterpret_cast<const float4 *>(
                            xs[m] + (size_t)b * xs_stride + (kb - kb_begin) * kBlockRows + 4 * s);
#pragma unroll
                        for (int q = 0; q < 4; ++q) acc[m][b] = dot4_u8(d[q], xp[8 * q], acc[m][b]);
                    }
                }
            }
        }
    }
}

// Reduce lane partials to column sums.  red: LDS scratch of NM*NB*kWaves*8
// floats.  On return, thread t < 8 holds in out[m][b] the sum for column t.
template <int NM, int NB>
__device__ __forceinline__ void tile_reduce(float (&acc)[NM][NB], float *red, float (&out)[NM][NB]) {
    const int lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
#pragma unroll
    for (int m = 0; m < NM; ++m)
#pragma unroll
        for (int b = 0; b < NB; ++b) {
            float a = acc[m][b];
            a += __shfl_xor(a, 8, 64);
            a += __shfl_xor(a, 16, 64);
            a += __shfl_xor(a, 32, 64);
            if (lane < 8) red[((m * NB + b) * kWaves + wave) * 8 + lane] = a;
        }
    __syncthreads();
    if (threadIdx.x < 8) {
#pragma unroll
        for (int m = 0; m < NM; ++m)
#pragma unroll
            for (int b = 0; b < NB; ++b) {
                float a = 0.f;
#pragma unroll
                for (int w = 0; w < kWaves; ++w) a += red[((m * NB + b) * kWaves + w) * 8 + threadIdx.x];
                out[m][b] = a;
            }
    }
    __syncthreads();
}

#endif  // __HIPCC__

}  // namespace rwkv
