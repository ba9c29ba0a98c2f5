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

// The operation in front of int8 layers and their activation quantizer in one launch: h = op(x) as
// k3q_rmsnorm / k3q_silu_mul write it, and q, scale = abs-max quantisation of h as k3q_absmax_quantize
// writes them (same helpers, same order of the sums: same bits).  One workgroup of 256 threads per
// row, the row in registers from the first load to the last store.
template <bool kIntRange>
__global__ __launch_bounds__(256) void input_op_quantize_rows(const uint16_t* __restrict__ x,
                                                             const uint16_t* __restrict__ operand, int kind,
                                                             float op_eps, int D, float eps, float qlo, float qhi,
                                                             uint16_t* __restrict__ h, int8_t* __restrict__ q,
                                                             uint16_t* __restrict__ scale) {
    __shared__ float part[4 * kMaxChunks];
    __shared__ float wmax[4];
    const int tid = threadIdx.x;
    const int chunks = D >> 3;
    const int64_t row = blockIdx.x;
    const v4u* xr = (const v4u*)(x + row * D);
    const v4u* orow = (const v4u*)(operand + (kind == K3Q_INPUT_RMS_NORM ? 0 : row * D));
    v4u c[kMaxChunks], g[kMaxChunks];
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ci = tid + i * 256;
        const int cc = ci < chunks ? ci : 0;
        c[i] = xr[cc];
        g[i] = orow[cc];
    }
    if (kind == K3Q_INPUT_RMS_NORM) {
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) {
            const float ss = wave_sum(tid + i * 256 < chunks ? piece_sum_squares(c[i]) : 0.f);
            if ((tid & 63) == 0) part[4 * i + (tid >> 6)] = ss;
        }
        __syncthreads();
        const int blocks = (chunks + 63) >> 6;
        float total = 0.f;
        for (int b = 0; b < blocks; ++b) total += part[b];
        const float rstd = 1.0f / sqrtf(total / (float)D + op_eps);
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) c[i] = piece_rms_scale(c[i], g[i], rstd);
    } else {
#pragma unroll
        for (int i = 0; i < kMaxChunks; ++i) c[i] = piece_silu_mul(g[i], c[i]);
    }
    // the quantizer on the rounded row: maximum, bf16(qhi / bf16(amax + eps)), bf16 products
    float amax = 0.f;
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        if (tid + i * 256 < chunks) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                amax = fmaxf(amax, fabsf(__uint_as_float(c[i][e] << 16)));
                amax = fmaxf(amax, fabsf(__uint_as_float(c[i][e] & 0xffff0000u)));
            }
        }
    }
    amax = wave_max(amax);
    if ((tid & 63) == 0) wmax[tid >> 6] = amax;
    __syncthreads();
    amax = fmaxf(fmaxf(wmax[0], wmax[1]), fmaxf(wmax[2], wmax[3]));
    const float s = round_bf16(qhi / round_bf16(amax + eps));
    if (tid == 0) scale[row] = (uint16_t)(__float_as_uint(s) >> 16);
    v4u* hr = (v4u*)(h + row * D);
    v2u* qr = (v2u*)(q + row * D);
#pragma unroll
    for (int i = 0; i < kMaxChunks; ++i) {
        const int ci = tid + i * 256;
        if (ci < chunks) {
            hr[ci] = c[i];
            if (kIntRange) {
                qr[ci] = quantize_piece_bf16(c[i], s, qlo, qhi);
            } else {
                u32 b[8];
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    const float f[2] = {__uint_as_float(c[i][e] << 16), __uint_as_float(c[i][e] & 0xffff0000u)};
#pragma unroll
                    for (int hh = 0; hh < 2; ++hh) {
                        float v = rintf(round_bf16(f[hh] * s));
                        v = fminf(fmaxf(v, qlo), qhi);
                        b[2 * e + hh] = (u32)(int)v & 0xffu;
                    }
                }
                const v2u o = {b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24),
                               b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24)};
                qr[ci] = o;
            }
        }
    }
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

extern "C" int k3q_input_op_quantize(const void* x, int dtype, int64_t rows, int64_t dim, const k3q_input_op* pre,
                                     float epsilon, float range_lo, float range_hi, void* h, int8_t* q,
                                     void* scale, void* stream) {
    if (dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (rows < 0 || dim <= 0 || (dim % 8) != 0 || dim > 8 * 256 * kMaxChunks || rows >= (1 << 30)) return K3Q_ERR_SHAPE;
    if (!(range_lo >= -128.f && range_hi <= 127.f && range_lo <= range_hi)) return K3Q_ERR_RANGE;
    if (!pre || (pre->kind != K3Q_INPUT_RMS_NORM && pre->kind != K3Q_INPUT_SILU_GATE)) return K3Q_ERR_SHAPE;
    if (rows == 0) return K3Q_OK;
    if (!x || !pre->operand || !h || !q || !scale) return K3Q_ERR_NULL;
    if (!aligned_to(x, 16) || !aligned_to(pre->operand, 16) || !aligned_to(h, 16) || !aligned_to(q, 8) ||
        !aligned_to(scale, 2))
        return K3Q_ERR_ALIGN;
    const float eps_bf16 = host_round_bf16(epsilon);  // torch rounds the epsilon operand to the tensor dtype
    const bool int_range = range_lo == rintf(range_lo) && range_hi == rintf(range_hi);
    auto kernel = int_range ? input_op_quantize_rows<true> : input_op_quantize_rows<false>;
    kernel<<<(unsigned)rows, 256, 0, (hipStream_t)stream>>>((const uint16_t*)x, (const uint16_t*)pre->operand, pre->kind,
                                                           pre->epsilon, (int)dim, eps_bf16, range_lo, range_hi,
                                                           (uint16_t*)h, q, (uint16_t*)scale);
    return launch_status();
}
