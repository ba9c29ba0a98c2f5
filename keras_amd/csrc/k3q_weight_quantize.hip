// Weight quantizers for kernels that already live on the device: the float32 arithmetic of the
// reference's numpy (`to_numpy=True`) paths, step for step, so that the integers, scales and zero
// points are the bits numpy produces on the host.
//
//   absmax_reduce   abs-max over a run of axes that is not trailing: x [outer, R, inner], one scale
//                   per (outer, inner) -- Dense kernels (axis 0: outer 1, R = input_dim, inner =
//                   units) and EinsumDense kernels (keras/src/quantizers/quantizers.py:95-109)
//   grouped_zp      groups of `block` rows of a [K, N] kernel, per (group, column) scale and zero
//                   point from the group's min / max (quantizers.py:182-234)
//
// What makes the bits equal: every step is one IEEE float32 operation in numpy and here (compiled
// with -ffp-contract=off, `/` is the correctly rounded division, rintf rounds half to even as
// np.round does); bfloat16 inputs are widened first, as the reference's conversion to numpy does.
// The abs-max form reads x from memory twice (a column's maximum needs all of the column before the
// first integer, and the kernel is larger than the chip's caches).  Groups of up to 128 rows keep
// their rows in registers between the min / max and the integers (grouped_zp_held: one read); larger
// groups take the generic two-pass kernel.
#include "k3q_common.h"

namespace k3q {
namespace {

constexpr int kWqX = 64;   // threads along the columns
constexpr int kWqY = 4;    // threads along the reduced rows
constexpr int kWqT = kWqX * kWqY;
constexpr int kWqChunk = 256;  // rows of R per workgroup in the abs-max passes

template <bool kBF16, int kV>
__device__ __forceinline__ void load_vals(const void* x, int64_t idx, float* f) {
    if (kV == 4) {
        if (kBF16) {
            const v2u c = *(const v2u*)((const uint16_t*)x + idx);
            f[0] = __uint_as_float(c[0] << 16);
            f[1] = __uint_as_float(c[0] & 0xffff0000u);
            f[2] = __uint_as_float(c[1] << 16);
            f[3] = __uint_as_float(c[1] & 0xffff0000u);
        } else {
            const v4u c = *(const v4u*)((const u32*)x + idx);
#pragma unroll
            for (int e = 0; e < 4; ++e) f[e] = __uint_as_float(c[e]);
        }
    } else {
        f[0] = raw_to_f32<kBF16>(load_raw<kBF16>(x, idx));
    }
}

template <int kV>
__device__ __forceinline__ void store_q(int8_t* q, int64_t idx, const int* v) {
    if (kV == 4) {
        *(u32*)(q + idx) = (u32)(v[0] & 0xff) | ((u32)(v[1] & 0xff) << 8) | ((u32)(v[2] & 0xff) << 16) |
                           ((u32)(v[3] & 0xff) << 24);
    } else {
        q[idx] = (int8_t)v[0];
    }
}

template <bool kBF16>
__device__ __forceinline__ void store_scale(void* s, int64_t idx, float v) {
    if (kBF16) ((uint16_t*)s)[idx] = (uint16_t)f32_to_bf16_bits(v);
    else ((float*)s)[idx] = v;
}

struct ReduceParams {
    const void* x;
    int8_t* q;
    void* scale;
    u32* amax;  // [outer * inner] bit patterns of the running max of |x| (zeroed by the entry point)
    int64_t R, inner;
    float eps, qlo, qhi;
};

// pass 1: |x| maxima of a chunk of rows, merged into `amax` with an unsigned max of the bit patterns
// (non-negative floats order like their bits)
template <bool kBF16, int kV>
__global__ __launch_bounds__(kWqT) void absmax_reduce_max(ReduceParams p) {
    __shared__ float part[kWqY][kWqX * 4];
    const int tx = threadIdx.x % kWqX, ty = threadIdx.x / kWqX;
    const int64_t col = ((int64_t)blockIdx.x * kWqX + tx) * kV;
    const int64_t o = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * kWqChunk;
    const int64_t r1 = r0 + kWqChunk < p.R ? r0 + kWqChunk : p.R;
    float m[kV];
#pragma unroll
    for (int e = 0; e < kV; ++e) m[e] = 0.f;
    if (col < p.inner) {
        for (int64_t r = r0 + ty; r < r1; r += kWqY) {
            float f[kV];
            load_vals<kBF16, kV>(p.x, (o * p.R + r) * p.inner + col, f);
#pragma unroll
            for (int e = 0; e < kV; ++e) m[e] = fmaxf(m[e], fabsf(f[e]));
        }
    }
#pragma unroll
    for (int e = 0; e < kV; ++e) part[ty][tx * 4 + e] = m[e];
    __syncthreads();
    if (ty == 0 && col < p.inner) {
#pragma unroll
        for (int e = 0; e < kV; ++e) {
            float v = part[0][tx * 4 + e];
#pragma unroll
            for (int y = 1; y < kWqY; ++y) v = fmaxf(v, part[y][tx * 4 + e]);
            atomicMax(p.amax + o * p.inner + col + e, __float_as_uint(v));
        }
    }
}

// pass 2: scale = hi / (amax + eps), q = clip(rint(x * scale))
template <bool kBF16, int kV>
__global__ __launch_bounds__(kWqT) void absmax_reduce_quantize(ReduceParams p) {
    const int tx = threadIdx.x % kWqX, ty = threadIdx.x / kWqX;
    const int64_t col = ((int64_t)blockIdx.x * kWqX + tx) * kV;
    if (col >= p.inner) return;
    const int64_t o = blockIdx.z;
    const int64_t r0 = (int64_t)blockIdx.y * kWqChunk;
    const int64_t r1 = r0 + kWqChunk < p.R ? r0 + kWqChunk : p.R;
    float s[kV];
#pragma unroll
    for (int e = 0; e < kV; ++e) s[e] = p.qhi / (__uint_as_float(p.amax[o * p.inner + col + e]) + p.eps);
    if (blockIdx.y == 0 && ty == 0) {
#pragma unroll
        for (int e = 0; e < kV; ++e) store_scale<kBF16>(p.scale, o * p.inner + col + e, s[e]);
    }
    for (int64_t r = r0 + ty; r < r1; r += kWqY) {
        const int64_t idx = (o * p.R + r) * p.inner + col;
        float f[kV];
        load_vals<kBF16, kV>(p.x, idx, f);
        int v[kV];
#pragma unroll
        for (int e = 0; e < kV; ++e) v[e] = (int)fminf(fmaxf(rintf(f[e] * s[e]), p.qlo), p.qhi);
        store_q<kV>(p.q, idx, v);
    }
}

struct GroupedParams {
    const void* x;
    int8_t* q;
    void* scale;
    int8_t* zero;
    int64_t K, N;
    int block;
    float eps, qmin, qmax, levels;  // levels = qmax - qmin
};

// one workgroup per (column tile, group): min / max of the group's rows (rows past K count as the
// zeros the reference pads with), then scale, zero point and the integers
template <bool kBF16, int kV>
__global__ __launch_bounds__(kWqT) void grouped_zp(GroupedParams p) {
    __shared__ float lo_s[kWqY][kWqX * 4], hi_s[kWqY][kWqX * 4];
    const int tx = threadIdx.x % kWqX, ty = threadIdx.x / kWqX;
    const int64_t col = ((int64_t)blockIdx.x * kWqX + tx) * kV;
    const int64_t g = blockIdx.y;
    const int64_t r0 = g * p.block;
    const bool live = col < p.N;
    float lo[kV], hi[kV];
#pragma unroll
    for (int e = 0; e < kV; ++e) {
        lo[e] = INFINITY;
        hi[e] = -INFINITY;
    }
    if (live) {
        for (int i = ty; i < p.block; i += kWqY) {
            float f[kV];
            if (r0 + i < p.K) {
                load_vals<kBF16, kV>(p.x, (r0 + i) * p.N + col, f);
            } else {
#pragma unroll
                for (int e = 0; e < kV; ++e) f[e] = 0.f;
            }
#pragma unroll
            for (int e = 0; e < kV; ++e) {
                lo[e] = fminf(lo[e], f[e]);
                hi[e] = fmaxf(hi[e], f[e]);
            }
        }
    }
#pragma unroll
    for (int e = 0; e < kV; ++e) {
        lo_s[ty][tx * 4 + e] = lo[e];
        hi_s[ty][tx * 4 + e] = hi[e];
    }
    __syncthreads();
    if (!live) return;
    float scale[kV], zero[kV];
#pragma unroll
    for (int e = 0; e < kV; ++e) {
        float l = lo_s[0][tx * 4 + e], h = hi_s[0][tx * 4 + e];
#pragma unroll
        for (int y = 1; y < kWqY; ++y) {
            l = fminf(l, lo_s[y][tx * 4 + e]);
            h = fmaxf(h, hi_s[y][tx * 4 + e]);
        }
        scale[e] = ((h - l) + p.eps) / p.levels;
        zero[e] = fminf(fmaxf(rintf(-l / scale[e]) + p.qmin, p.qmin), p.qmax);
    }
    if (ty == 0) {
#pragma unroll
        for (int e = 0; e < kV; ++e) {
            store_scale<kBF16>(p.scale, g * p.N + col + e, scale[e]);
            p.zero[g * p.N + col + e] = (int8_t)(int)zero[e];
        }
    }
    for (int i = ty; i < p.block && r0 + i < p.K; i += kWqY) {
        const int64_t idx = (r0 + i) * p.N + col;
        float f[kV];
        load_vals<kBF16, kV>(p.x, idx, f);
        int v[kV];
#pragma unroll
        for (int e = 0; e < kV; ++e)
            v[e] = (int)fminf(fmaxf(rintf(f[e] / scale[e]) + zero[e], p.qmin), p.qmax);
        store_q<kV>(p.q, idx, v);
    }
}

// rintf(x / s) with the division's own rounding, for a column scale s > 0 whose reciprocal
// (correctly rounded) is at hand.  r = x * (1 / s) lies within 3 * 2^-24 |r| of the correctly rounded
// quotient t, so rint(t) = rint(r) unless r is that close to a half-integer; there (and for
// anything that is not a number) the division is done.  The margin used is 2^-20 |r|.
__device__ __forceinline__ float rint_quotient(float x, float s, float inv_s) {
    const float r = x * inv_s;
    float n = rintf(r);
    const float d = fabsf(r - n);
    if (!(0.5f - d > fabsf(r) * 0x1p-20f)) n = rintf(x / s);
    return n;
}

// The same for groups of up to kHeldY * kHeldRows rows with N a multiple of 4.  A thread keeps its
// rows in registers between the two passes, so memory sees x once (the groups resident on the chip
// at one time are far larger than its caches, and the generic kernel's second read comes from
// memory again); the integers come from rint_quotient.  A workgroup walks work items (column
// tile, group) at a stride of the grid and asks for the next item's rows before it works on the
// current one: with one item per workgroup the whole chip alternates between loading and computing
// (the registers allow one or two workgroups per CU), and neither memory nor the vector units see
// more than half of the time.
constexpr int kHeldY = 8, kHeldRows = 16;
template <bool kBF16>
__global__ __launch_bounds__(kWqX * kHeldY) void grouped_zp_held(GroupedParams p, int col_tiles, int items) {
    __shared__ float lo_s[2][kHeldY][kWqX * 4], hi_s[2][kHeldY][kWqX * 4];
    const int tx = threadIdx.x % kWqX, ty = threadIdx.x / kWqX;
    auto load_item = [&](const int item, float (&rows)[kHeldRows][4]) {
        const int64_t g = item / col_tiles;
        const int64_t col = ((int64_t)(item - g * col_tiles) * kWqX + tx) * 4;
        const int64_t r0 = g * p.block;
#pragma unroll
        for (int j = 0; j < kHeldRows; ++j) {
            const int i = ty + j * kHeldY;
            if (item < items && col < p.N && i < p.block && r0 + i < p.K) {
                load_vals<kBF16, 4>(p.x, (r0 + i) * p.N + col, rows[j]);
            } else {  // rows past K count as zeros; rows past the group do not count (skipped below)
#pragma unroll
                for (int e = 0; e < 4; ++e) rows[j][e] = 0.f;
            }
        }
    };
    auto work = [&](const int item, const int par, const float (&rows)[kHeldRows][4]) {
        const int64_t g = item / col_tiles;
        const int64_t col = ((int64_t)(item - g * col_tiles) * kWqX + tx) * 4;
        const int64_t r0 = g * p.block;
        float lo[4], hi[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo[e] = INFINITY;
            hi[e] = -INFINITY;
        }
#pragma unroll
        for (int j = 0; j < kHeldRows; ++j)
            if (ty + j * kHeldY < p.block) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    lo[e] = fminf(lo[e], rows[j][e]);
                    hi[e] = fmaxf(hi[e], rows[j][e]);
                }
            }
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            lo_s[par][ty][tx * 4 + e] = lo[e];
            hi_s[par][ty][tx * 4 + e] = hi[e];
        }
        __syncthreads();  // (the buffers alternate, so the item after the next may overwrite this one's)
        if (col >= p.N) return;
        float scale[4], inv[4], zero[4];
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            float l = lo_s[par][0][tx * 4 + e], h = hi_s[par][0][tx * 4 + e];
#pragma unroll
            for (int y = 1; y < kHeldY; ++y) {
                l = fminf(l, lo_s[par][y][tx * 4 + e]);
                h = fmaxf(h, hi_s[par][y][tx * 4 + e]);
            }
            scale[e] = ((h - l) + p.eps) / p.levels;
            inv[e] = 1.0f / scale[e];
            zero[e] = fminf(fmaxf(rintf(-l / scale[e]) + p.qmin, p.qmin), p.qmax);
        }
        if (ty == 0) {
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                store_scale<kBF16>(p.scale, g * p.N + col + e, scale[e]);
                p.zero[g * p.N + col + e] = (int8_t)(int)zero[e];
            }
        }
#pragma unroll
        for (int j = 0; j < kHeldRows; ++j) {
            const int i = ty + j * kHeldY;
            if (i < p.block && r0 + i < p.K) {
                int v[4];
#pragma unroll
                for (int e = 0; e < 4; ++e)
                    v[e] = (int)__builtin_amdgcn_fmed3f(rint_quotient(rows[j][e], scale[e], inv[e]) + zero[e], p.qmin, p.qmax);
                store_q<4>(p.q, (r0 + i) * p.N + col, v);
            }
        }
    };
    float a[kHeldRows][4], b[kHeldRows][4];
    const int step = gridDim.x;
    int item = blockIdx.x;
    load_item(item, a);
    while (item < items) {  // (uniform over the workgroup: every thread meets every barrier)
        load_item(item + step, b);
        work(item, 0, a);
        item += step;
        if (item >= items) break;
        load_item(item + step, a);
        work(item, 1, b);
        item += step;
    }
}

__global__ void clear_u32(u32* p, int64_t n) {
    const int64_t i = (int64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_weight_absmax_quantize(const void* x, int x_dtype, int64_t outer, int64_t R, int64_t inner,
                                          float epsilon, float range_lo, float range_hi, int8_t* q,
                                          void* scale, void* amax_workspace, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (outer < 0 || R < 0 || inner < 0 || outer > 65535) return K3Q_ERR_SHAPE;
    if (range_lo < -128.f || range_hi > 127.f || range_lo > range_hi) return K3Q_ERR_RANGE;
    if (outer == 0 || inner == 0) return K3Q_OK;
    if (R == 0) return K3Q_ERR_SHAPE;  // the maximum of nothing
    if (!x || !q || !scale || !amax_workspace) return K3Q_ERR_NULL;
    const int64_t chunks = (R + kWqChunk - 1) / kWqChunk;
    if (chunks > 65535) return K3Q_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    ReduceParams p;
    p.x = x;
    p.q = q;
    p.scale = scale;
    p.amax = (u32*)amax_workspace;
    p.R = R;
    p.inner = inner;
    p.eps = epsilon;
    p.qlo = range_lo;
    p.qhi = range_hi;
    const int64_t cells = outer * inner;
    clear_u32<<<(unsigned)((cells + 255) / 256), 256, 0, s>>>(p.amax, cells);
    const bool bf = x_dtype == K3Q_BF16;
    const bool vec = (inner % 4) == 0 && aligned_to(x, bf ? 8 : 16) && aligned_to(q, 4);
    const int v = vec ? 4 : 1;
    dim3 grid((unsigned)((inner + (int64_t)kWqX * v - 1) / ((int64_t)kWqX * v)), (unsigned)chunks, (unsigned)outer);
    if (bf && vec) {
        absmax_reduce_max<true, 4><<<grid, kWqT, 0, s>>>(p);
        absmax_reduce_quantize<true, 4><<<grid, kWqT, 0, s>>>(p);
    } else if (bf) {
        absmax_reduce_max<true, 1><<<grid, kWqT, 0, s>>>(p);
        absmax_reduce_quantize<true, 1><<<grid, kWqT, 0, s>>>(p);
    } else if (vec) {
        absmax_reduce_max<false, 4><<<grid, kWqT, 0, s>>>(p);
        absmax_reduce_quantize<false, 4><<<grid, kWqT, 0, s>>>(p);
    } else {
        absmax_reduce_max<false, 1><<<grid, kWqT, 0, s>>>(p);
        absmax_reduce_quantize<false, 1><<<grid, kWqT, 0, s>>>(p);
    }
    return launch_status();
}

extern "C" int k3q_weight_quantize_grouped(const void* x, int x_dtype, int64_t K, int64_t N, int64_t block_size,
                                           float epsilon, float range_lo, float range_hi, int8_t* q,
                                           void* scale, int8_t* zero, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (K < 0 || N < 0 || block_size <= 0 || block_size > (1 << 20)) return K3Q_ERR_SHAPE;
    if (range_lo < -128.f || range_hi > 127.f || range_lo >= range_hi) return K3Q_ERR_RANGE;
    if (K == 0 || N == 0) return K3Q_OK;
    if (!x || !q || !scale || !zero) return K3Q_ERR_NULL;
    const int64_t groups = (K + block_size - 1) / block_size;
    if (groups > 65535) return K3Q_ERR_SHAPE;
    GroupedParams p;
    p.x = x;
    p.q = q;
    p.scale = scale;
    p.zero = zero;
    p.K = K;
    p.N = N;
    p.block = (int)block_size;
    p.eps = epsilon;
    p.qmin = range_lo;
    p.qmax = range_hi;
    p.levels = range_hi - range_lo;
    const bool bf = x_dtype == K3Q_BF16;
    const bool vec = (N % 4) == 0 && aligned_to(x, bf ? 8 : 16) && aligned_to(q, 4);
    const int v = vec ? 4 : 1;
    dim3 grid((unsigned)((N + (int64_t)kWqX * v - 1) / ((int64_t)kWqX * v)), (unsigned)groups);
    hipStream_t s = (hipStream_t)stream;
    // the held form's quotient needs a finite positive scale and its reciprocal: an epsilon > 0 gives
    // both for any finite kernel
    const int64_t col_tiles = grid.x, items = col_tiles * groups;
    const bool held = vec && block_size <= (int64_t)kHeldY * kHeldRows && epsilon > 0.f && items < (1ll << 30);
    if (held) {
        const unsigned blocks = (unsigned)(items < 256 ? items : 256);  // one resident workgroup per CU
        if (bf) grouped_zp_held<true><<<blocks, kWqX * kHeldY, 0, s>>>(p, (int)col_tiles, (int)items);
        else grouped_zp_held<false><<<blocks, kWqX * kHeldY, 0, s>>>(p, (int)col_tiles, (int)items);
        return launch_status();
    }
    if (bf && vec) grouped_zp<true, 4><<<grid, kWqT, 0, s>>>(p);
    else if (bf) grouped_zp<true, 1><<<grid, kWqT, 0, s>>>(p);
    else if (vec) grouped_zp<false, 4><<<grid, kWqT, 0, s>>>(p);
    else grouped_zp<false, 1><<<grid, kWqT, 0, s>>>(p);
    return launch_status();
}
