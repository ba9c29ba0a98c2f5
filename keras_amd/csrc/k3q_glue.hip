// Two small kernels of the decoder harness's glue between the quantized layers, bfloat16:
// RMS normalisation of rows and the SwiGLU gate silu(g) * u.  A decode step runs each of them
// once or twice per block on a few KiB; the point is one short launch each.
#include "k3q_common.h"

namespace k3q {
namespace {

// y[r, :] = bf16( x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w[:] ), float32 arithmetic, one rounding.
// One workgroup of 256 threads per row; D % 8 == 0; a thread keeps up to kMaxChunks 16-byte chunks.
constexpr int kMaxChunks = 4;  // D <= 8192
__global__ __launch_bounds__(256) void rmsnorm_rows(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                   uint16_t* __restrict__ y, int D, int64_t x_stride,
                                                   int64_t y_stride, float eps) {
    __shared__ float part[4];
    const int tid = threadIdx.x;
    const int chunks = D >> 3;
    const v4u* xr = (const v4u*)(x + (int64_t)blockIdx.x * x_stride);
    v4u c[kMaxChunks], g[kMaxChunks];
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ci = tid + i * 256;
        const int cc = ci < chunks ? ci : 0;
        c[i] = xr[cc];
        g[i] = ((const v4u*)w)[cc];
    }
    float ss = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        if (tid + i * 256 < chunks) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = __uint_as_float(c[i][e] << 16), hi = __uint_as_float(c[i][e] & 0xffff0000u);
                ss += lo * lo + hi * hi;
            }
        }
    }
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) ss += __shfl_xor(ss, o, kWave);
    if ((tid & 63) == 0) part[tid >> 6] = ss;
    __syncthreads();
    const float total = (part[0] + part[1]) + (part[2] + part[3]);
    const float rstd = 1.0f / sqrtf(total / (float)D + eps);
    v4u* yr = (v4u*)(y + (int64_t)blockIdx.x * y_stride);
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ci = tid + i * 256;
        if (ci < chunks) {
            v4u o;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                const float lo = __uint_as_float(c[i][e] << 16) * rstd * __uint_as_float(g[i][e] << 16);
                const float hi = __uint_as_float(c[i][e] & 0xffff0000u) * rstd * __uint_as_float(g[i][e] & 0xffff0000u);
                o[e] = pack_bf16x2(lo, hi);
            }
            yr[ci] = o;
        }
    }
}

// y = bf16( bf16(g / (1 + exp(-g))) * u ): the two roundings of silu(g) followed by the multiply
__global__ __launch_bounds__(256) void silu_mul_rows(const uint16_t* __restrict__ g, const uint16_t* __restrict__ u,
                                                    uint16_t* __restrict__ y, int chunks_per_row, int64_t g_stride,
                                                    int64_t u_stride, int64_t y_stride, int64_t total_chunks) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total_chunks) return;
    const int64_t r = t / chunks_per_row;
    const int c = (int)(t - r * chunks_per_row);
    const v4u gv = ((const v4u*)(g + r * g_stride))[c];
    const v4u uv = ((const v4u*)(u + r * u_stride))[c];
    v4u o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float a[2] = {__uint_as_float(gv[e] << 16), __uint_as_float(gv[e] & 0xffff0000u)};
        const float b[2] = {__uint_as_float(uv[e] << 16), __uint_as_float(uv[e] & 0xffff0000u)};
#pragma unroll
        for (int h = 0; h < 2; ++h) a[h] = round_bf16(round_bf16(a[h] / (1.0f + expf(-a[h]))) * b[h]);
        o[e] = pack_bf16x2(a[0], a[1]);
    }
    ((v4u*)(y + r * y_stride))[c] = o;
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_rmsnorm(const void* x, const void* weight, int dtype, int64_t rows, int64_t dim,
                           int64_t x_row_stride, float epsilon, void* y, int64_t y_row_stride, void* stream) {
    if (dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (rows < 0 || dim <= 0 || (dim % 8) != 0 || dim > 8 * 256 * kMaxChunks || rows >= (1 << 30) ||
        (x_row_stride % 8) != 0 || (y_row_stride % 8) != 0 || x_row_stride < dim || y_row_stride < dim)
        return K3Q_ERR_SHAPE;
    if (rows == 0) return K3Q_OK;
    if (!x || !weight || !y) return K3Q_ERR_NULL;
    if (!aligned_to(x, 16) || !aligned_to(weight, 16) || !aligned_to(y, 16)) return K3Q_ERR_ALIGN;
    rmsnorm_rows<<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)weight,
                                                                 (uint16_t*)y, (int)dim, x_row_stride, y_row_stride,
                                                                 epsilon);
    return launch_status();
}

extern "C" int k3q_silu_mul(const void* gate, const void* up, int dtype, int64_t rows, int64_t dim,
                            int64_t gate_row_stride, int64_t up_row_stride, void* y, int64_t y_row_stride,
                            void* stream) {
    if (dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (rows < 0 || dim <= 0 || (dim % 8) != 0 || (gate_row_stride % 8) != 0 || (up_row_stride % 8) != 0 ||
        (y_row_stride % 8) != 0 || gate_row_stride < dim || up_row_stride < dim || y_row_stride < dim ||
        rows * (dim / 8) >= ((int64_t)1 << 38))
        return K3Q_ERR_SHAPE;
    if (rows == 0) return K3Q_OK;
    if (!gate || !up || !y) return K3Q_ERR_NULL;
    if (!aligned_to(gate, 16) || !aligned_to(up, 16) || !aligned_to(y, 16)) return K3Q_ERR_ALIGN;
    const int64_t chunks = rows * (dim / 8);
    silu_mul_rows<<<(unsigned)((chunks + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint16_t*)gate, (const uint16_t*)up, (uint16_t*)y, (int)(dim / 8), gate_row_stride, up_row_stride,
        y_row_stride, chunks);
    return launch_status();
}
