// Quantiser (reference agnostic/backends/modules/matmul.py:18-40) and the
// packed weight layout: pack / unpack / canonical dequantisation.
#include "rwkv_common.h"

#include <string>

namespace rwkv {

static thread_local char g_err[512] = "";

int set_error(int code, const char *fmt, ...) {
    va_list ap;
    va_start(ap, fmt);
    vsnprintf(g_err, sizeof(g_err), fmt, ap);
    va_end(ap);
    return code;
}

// ---------------------------------------------------------------------------
// One workgroup owns 64 input channels of weight[n_out, n_in] and walks every
// row twice: thread (jx, ky) handles channel j0+jx, rows ky, ky+4, ... so each
// load is a coalesced 256-byte row segment.  Pass 1 finds min/max; pass 2
// forms the float64 quotient, writes the truncated codes (64x64 tiles
// transposed through LDS so the [n_in, n_out] store is coalesced too) and
// accumulates the truncated fractions for the offset.
// ---------------------------------------------------------------------------
__global__ void __launch_bounds__(256)
quantize_kernel(const float *__restrict__ W, int64_t n_out, int64_t n_in,
                uint8_t *__restrict__ codes, float *__restrict__ range,
                double *__restrict__ offset) {
    __shared__ float smin[4][64], smax[4][64];
    __shared__ double sfr[4][64];
    __shared__ uint8_t tile[64][68];
    const int jx = threadIdx.x & 63, ky = threadIdx.x >> 6;
    const int64_t j0 = (int64_t)blockIdx.x * 64;
    const int64_t j = j0 + jx;
    const bool live = j < n_in;

    float lo_f = INFINITY, hi_f = -INFINITY;
    if (live)
        for (int64_t k = ky; k < n_out; k += 4) {
            const float x = W[k * n_in + j];
            lo_f = fminf(lo_f, x);
            hi_f = fmaxf(hi_f, x);
        }
    smin[ky][jx] = lo_f;
    smax[ky][jx] = hi_f;
    __syncthreads();
    lo_f = fminf(fminf(smin[0][jx], smin[1][jx]), fminf(smin[2][jx], smin[3][jx]));
    hi_f = fmaxf(fmaxf(smax[0][jx], smax[1][jx]), fmaxf(smax[2][jx], smax[3][jx]));
    // matmul.py:31-33: min in float64; range = max(x - min) / 255 in float64
    const double lo = (double)lo_f;
    const double ran = ((double)hi_f - lo) / 255.0;

    double fr = 0.0;
    for (int64_t k0 = 0; k0 < n_out; k0 += 64) {
        for (int r = ky; r < 64; r += 4) {
            const int64_t k = k0 + r;
            uint8_t c = 0;
            if (live && k < n_out && ran > 0.0) {
                const double q = ((double)W[k * n_in + j] - lo) / ran;  // matmul.py:32-34
                const double t = trunc(q);
                c = (uint8_t)(int)t;     // .to(uint8) truncates, matmul.py:21
                fr += q - t;             // out.frac(), matmul.py:35
            }
            tile[jx][r] = c;
        }
        __syncthreads();
        for (int r = ky; r < 64; r += 4) {
            const int64_t jj = j0 + r, k = k0 + jx;
            if (jj < n_in && k < n_out) codes[jj * n_out + k] = tile[r][jx];
        }
        __syncthreads();
    }
    sfr[ky][jx] = fr;
    __syncthreads();
    if (ky == 0 && live) {
        const double fsum = (sfr[0][jx] + sfr[1][jx]) + (sfr[2][jx] + sfr[3][jx]);
        offset[j] = lo + (fsum / (double)n_out) * ran;   // matmul.py:36-37
        range[j] = (float)ran;                            // matmul.py:39
    }
}

// ---------------------------------------------------------------------------
// pack / unpack: one thread per 16-byte lane chunk of a block.
// ---------------------------------------------------------------------------
template <bool PACK>
__global__ void __launch_bounds__(256)
pack_kernel(uint8_t *__restrict__ codes, int64_t stride, int64_t n_in, int64_t n_out,
            uint8_t *__restrict__ packed, int64_t n_kb, int64_t n_chunks) {
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_chunks) return;
    const int lane = (int)(g & 63);
    const int64_t blk = g >> 6;
    const int64_t kb = blk % n_kb, ct = blk / n_kb;
    const int s = lane >> 3, c = lane & 7;
    const int64_t col = ct * kTileCols + c;
    uint8_t *p = packed + g * 16;
    if (PACK) {
        uint32_t d[4];
#pragma unroll
        for (int m = 0; m < 4; ++m) {
            uint32_t v = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = kb * kBlockRows + 32 * m + 4 * s + e;
                const uint32_t b = (row < n_in && col < n_out) ? codes[row * stride + col] : 0u;
                v |= b << (8 * e);
            }
            d[m] = v;
        }
        *reinterpret_cast<uint4 *>(p) = make_uint4(d[0], d[1], d[2], d[3]);
    } else {
        const uint4 v = *reinterpret_cast<const uint4 *>(p);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int m = 0; m < 4; ++m)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = kb * kBlockRows + 32 * m + 4 * s + e;
                if (row < n_in && col < n_out) codes[row * stride + col] = (uint8_t)(d[m] >> (8 * e));
            }
    }
}

__global__ void __launch_bounds__(256)
dequant_packed_kernel(const uint8_t *__restrict__ packed, const float *__restrict__ range,
                      const double *__restrict__ offset, int64_t n_in, int64_t n_out,
                      int64_t n_kb, float *__restrict__ dq) {
    // one thread per output element, consecutive threads along k
    const int64_t g = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (g >= n_in * n_out) return;
    const int64_t j = g / n_out, k = g % n_out;
    const int64_t ct = k / kTileCols, kb = j / kBlockRows;
    const int c = (int)(k % kTileCols), r = (int)(j % kBlockRows);
    const int m = r / 32, s = (r % 32) / 4, e = r % 4;
    const uint8_t code = packed[(ct * n_kb + kb) * kBlockBytes + 16 * (8 * s + c) + 4 * m + e];
    dq[g] = (float)((double)code * (double)range[j] + offset[j]);
}

// ---------------------------------------------------------------------------
// "M16" layout for the int8 matrix-core decode kernel: 1 KiB blocks of 16
// output columns x 64 input rows, ordered [ceil(n_out/16)][ceil(n_in/64)].
// Lane l = 16*g + n of a wavefront owns bytes 16*l .. 16*l+15 of the block:
// rows 64*kb + 16*g + (0..15) of column 16*ct + n, stored as code - 128
// (two's complement), i.e. exactly the B operand of v_mfma_i32_16x16x64_i8.
// Padding is stored as 0 (it only ever meets zero activation digits).
// ---------------------------------------------------------------------------
template <bool PACK>
__global__ void __launch_bounds__(256)
pack_m16_kernel(uint8_t *__restrict__ codes, int64_t stride, int64_t n_in, int64_t n_out,
                uint8_t *__restrict__ packed, int64_t n_kb, int64_t n_chunks) {
    const int64_t gidx = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (gidx >= n_chunks) return;
    const int lane = (int)(gidx & 63);
    const int64_t blk = gidx >> 6;
    const int64_t kb = blk % n_kb, ct = blk / n_kb;
    const int g = lane >> 4, n = lane & 15;
    const int64_t col = ct * 16 + n;
    uint8_t *p = packed + gidx * 16;
    if (PACK) {
        uint32_t d[4];
#pragma unroll
        for (int q = 0; q < 4; ++q) {
            uint32_t v = 0;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = kb * 64 + 16 * g + 4 * q + e;
                const uint32_t b = (row < n_in && col < n_out) ? (uint32_t)(codes[row * stride + col] ^ 0x80u) : 0u;
                v |= b << (8 * e);
            }
            d[q] = v;
        }
        *reinterpret_cast<uint4 *>(p) = make_uint4(d[0], d[1], d[2], d[3]);
    } else {
        const uint4 v = *reinterpret_cast<const uint4 *>(p);
        const uint32_t d[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
        for (int q = 0; q < 4; ++q)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const int64_t row = kb * 64 + 16 * g + 4 * q + e;
                if (row < n_in && col < n_out) codes[row * stride + col] = (uint8_t)((d[q] >> (8 * e)) ^ 0x80u);
            }
    }
}

}  // namespace rwkv

using namespace rwkv;

extern "C" {

int rwkv_version(void) { return 100; }
const char *rwkv_last_error(void) { return rwkv::g_err; }

int rwkv_quantize_u8(rwkv_stream_t stream, const float *weight, int64_t n_out, int64_t n_in,
                     uint8_t *codes, float *range, double *offset) {
    RWKV_CHECK_ARG(weight && codes && range && offset, "rwkv_quantize_u8: null pointer");
    RWKV_CHECK_ARG(n_out > 0 && n_in > 0, "rwkv_quantize_u8: sizes must be positive");
    RWKV_CHECK_ALIGN(weight, 4);
    RWKV_CHECK_ALIGN(range, 4);
    RWKV_CHECK_ALIGN(offset, 8);
    hipLaunchKernelGGL(quantize_kernel, dim3((unsigned)ceil_div(n_in, 64)), dim3(256), 0,
                       (hipStream_t)stream, weight, n_out, n_in, codes, range, offset);
    RWKV_CHECK_LAUNCH("quantize_kernel");
    return RWKV_OK;
}

size_t rwkv_packed_bytes(int64_t n_in, int64_t n_out) {
    if (n_in <= 0 || n_out <= 0) return 0;
    return (size_t)(ceil_div(n_out, kTileCols) * ceil_div(n_in, kBlockRows) * kBlockBytes);
}

int rwkv_pack_u8(rwkv_stream_t stream, const uint8_t *codes, int64_t codes_stride,
                 int64_t n_in, int64_t n_out, uint8_t *packed) {
    RWKV_CHECK_ARG(codes && packed, "rwkv_pack_u8: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && codes_stride >= n_out, "rwkv_pack_u8: bad sizes");
    RWKV_CHECK_ALIGN(packed, 16);
    const int64_t n_kb = ceil_div(n_in, kBlockRows);
    const int64_t n_chunks = ceil_div(n_out, kTileCols) * n_kb * 64;
    hipLaunchKernelGGL(pack_kernel<true>, dim3((unsigned)ceil_div(n_chunks, 256)), dim3(256), 0,
                       (hipStream_t)stream, const_cast<uint8_t *>(codes), codes_stride, n_in, n_out,
                       packed, n_kb, n_chunks);
    RWKV_CHECK_LAUNCH("pack_kernel");
    return RWKV_OK;
}

int rwkv_unpack_u8(rwkv_stream_t stream, const uint8_t *packed, int64_t n_in, int64_t n_out,
                   uint8_t *codes, int64_t codes_stride) {
    RWKV_CHECK_ARG(codes && packed, "rwkv_unpack_u8: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && codes_stride >= n_out, "rwkv_unpack_u8: bad sizes");
    RWKV_CHECK_ALIGN(packed, 16);
    const int64_t n_kb = ceil_div(n_in, kBlockRows);
    const int64_t n_chunks = ceil_div(n_out, kTileCols) * n_kb * 64;
    hipLaunchKernelGGL(pack_kernel<false>, dim3((unsigned)ceil_div(n_chunks, 256)), dim3(256), 0,
                       (hipStream_t)stream, codes, codes_stride, n_in, n_out,
                       const_cast<uint8_t *>(packed), n_kb, n_chunks);
    RWKV_CHECK_LAUNCH("unpack_kernel");
    return RWKV_OK;
}

int rwkv_dequant_packed(rwkv_stream_t stream, const uint8_t *packed, const float *range,
                        const double *offset, int64_t n_in, int64_t n_out, float *dq) {
    RWKV_CHECK_ARG(packed && range && offset && dq, "rwkv_dequant_packed: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0, "rwkv_dequant_packed: bad sizes");
    const int64_t n = n_in * n_out;
    hipLaunchKernelGGL(dequant_packed_kernel, dim3((unsigned)ceil_div(n, 256)), dim3(256), 0,
                       (hipStream_t)stream, packed, range, offset, n_in, n_out,
                       ceil_div(n_in, kBlockRows), dq);
    RWKV_CHECK_LAUNCH("dequant_packed_kernel");
    return RWKV_OK;
}

size_t rwkv_packed_m16_bytes(int64_t n_in, int64_t n_out) {
    if (n_in <= 0 || n_out <= 0) return 0;
    return (size_t)(ceil_div(n_out, 16) * ceil_div(n_in, 64) * 1024);
}

int rwkv_pack_m16(rwkv_stream_t stream, const uint8_t *codes, int64_t codes_stride,
                  int64_t n_in, int64_t n_out, uint8_t *packed) {
    RWKV_CHECK_ARG(codes && packed, "rwkv_pack_m16: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && codes_stride >= n_out, "rwkv_pack_m16: bad sizes");
    RWKV_CHECK_ALIGN(packed, 16);
    const int64_t n_kb = ceil_div(n_in, 64);
    const int64_t n_chunks = ceil_div(n_out, 16) * n_kb * 64;
    hipLaunchKernelGGL(pack_m16_kernel<true>, dim3((unsigned)ceil_div(n_chunks, 256)), dim3(256), 0,
                       (hipStream_t)stream, const_cast<uint8_t *>(codes), codes_stride, n_in, n_out,
                       packed, n_kb, n_chunks);
    RWKV_CHECK_LAUNCH("pack_m16_kernel");
    return RWKV_OK;
}

int rwkv_unpack_m16(rwkv_stream_t stream, const uint8_t *packed, int64_t n_in, int64_t n_out,
                    uint8_t *codes, int64_t codes_stride) {
    RWKV_CHECK_ARG(codes && packed, "rwkv_unpack_m16: null pointer");
    RWKV_CHECK_ARG(n_in > 0 && n_out > 0 && codes_stride >= n_out, "rwkv_unpack_m16: bad sizes");
    RWKV_CHECK_ALIGN(packed, 16);
    const int64_t n_kb = ceil_div(n_in, 64);
    const int64_t n_chunks = ceil_div(n_out, 16) * n_kb * 64;
    hipLaunchKernelGGL(pack_m16_kernel<false>, dim3((unsigned)ceil_div(n_chunks, 256)), dim3(256), 0,
                       (hipStream_t)stream, codes, codes_stride, n_in, n_out,
                       const_cast<uint8_t *>(packed), n_kb, n_chunks);
    RWKV_CHECK_LAUNCH("unpack_m16_kernel");
    return RWKV_OK;
}

}  // extern "C"
