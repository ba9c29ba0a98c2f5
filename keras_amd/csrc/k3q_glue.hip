// Two small kernels of the decoder harness's glue between the quantized layers, bfloat16:
// RMS normalisation of rows and the SwiGLU gate silu(g) * u.  A decode step runs each of them
// once or twice per block on a few KiB; the point is one short launch each.
#include "k3q_common.h"

namespace k3q {
namespace {

// y[r, :] = bf16( x[r, :] * rsqrt(mean(x[r, :]^2) + eps) * w[:] ), float32 arithmetic, one rounding.
// One workgroup of 256 threads per row; D % 8 == 0; a thread keeps up to kMaxChunks 16-byte chunks.
// The sum of squares has a fixed order -- per 16-byte piece, per block of 64 pieces (wave_sum), blocks
// in ascending order -- which the matmul kernels that normalise their input themselves follow too.
constexpr int kMaxChunks = 8;  // D <= 16384
__global__ __launch_bounds__(256) void rmsnorm_rows(const uint16_t* __restrict__ x, const uint16_t* __restrict__ w,
                                                   uint16_t* __restrict__ y, int D, int64_t x_stride,
                                                   int64_t y_stride, float eps) {
    __shared__ float part[4 * kMaxChunks];
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
    // block 4 i + wave holds pieces [64 (4 i + wave), + 64); pieces past the row count zero
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const float ss = wave_sum(tid + i * 256 < chunks ? piece_sum_squares(c[i]) : 0.f);
        if ((tid & 63) == 0) part[4 * i + (tid >> 6)] = ss;
    }
    __syncthreads();
    const int blocks = (chunks + 63) >> 6;
    float total = 0.f;
    for (int b = 0; b < blocks; ++b) total += part[b];
    const float rstd = 1.0f / sqrtf(total / (float)D + eps);
    v4u* yr = (v4u*)(y + (int64_t)blockIdx.x * y_stride);
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ci = tid + i * 256;
        if (ci < chunks) yr[ci] = piece_rms_scale(c[i], g[i], rstd);
    }
}

// y = bf16( bf16(silu(g)) * u ): the two roundings of silu(g) followed by the multiply (piece_silu_mul)
__global__ __launch_bounds__(256) void silu_mul_rows(const uint16_t* __restrict__ g, const uint16_t* __restrict__ u,
                                                    uint16_t* __restrict__ y, int chunks_per_row, int64_t g_stride,
                                                    int64_t u_stride, int64_t y_stride, int64_t total_chunks) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= total_chunks) return;
    const int64_t r = t / chunks_per_row;
    const int c = (int)(t - r * chunks_per_row);
    const v4u gv = ((const v4u*)(g + r * g_stride))[c];
    const v4u uv = ((const v4u*)(u + r * u_stride))[c];
    const v4u o = piece_silu_mul(gv, uv);
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
