// Row-wise abs-max quantizer: x [rows, cols] (float32 or bfloat16) ->
// q int8 [rows, cols] + scale [rows].
//
// HBM-bound: x is read once, q and scale are written once.  A row is held in
// registers between the max reduction and the quantisation, so the nine torch
// passes of the reference collapse into one read and one write.  Every
// arithmetic step is rounded to the tensor dtype exactly as torch rounds it
// (for bfloat16: the epsilon, the sum, the quotient and the product are each
// rounded to bfloat16 before the next step), which is what makes the int8
// output bit-identical to the reference.
#include <type_traits>

#include "k3q_common.h"

namespace k3q {
namespace {

template <int kDtype>
struct Elem;
template <>
struct Elem<K3Q_F32> {
    static constexpr int kBytes = 4;
    static constexpr int kPerChunk = 4;  // elements in a 16-byte chunk
};
template <>
struct Elem<K3Q_BF16> {
    static constexpr int kBytes = 2;
    static constexpr int kPerChunk = 8;
};

// unpack one 16-byte chunk into floats
template <int kDtype>
__device__ __forceinline__ void chunk_to_floats(const v4u& c, float* f) {
    if (kDtype == K3Q_F32) {
#pragma unroll
        for (int i = 0; i < 4; ++i) f[i] = __uint_as_float(c[i]);
    } else {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            f[2 * i] = __uint_as_float(c[i] << 16);
            f[2 * i + 1] = __uint_as_float(c[i] & 0xffff0000u);
        }
    }
}

template <int kDtype>
__device__ __forceinline__ float scale_from_amax(float amax, float eps, float qhi) {
    if (kDtype == K3Q_F32) return qhi / (amax + eps);
    float t = round_bf16(amax + eps);  // eps arrives already rounded to bfloat16
    return round_bf16(qhi / t);
}

template <int kDtype>
__device__ __forceinline__ int quantize_one(float v, float s, float qlo, float qhi) {
    float p = v * s;
    if (kDtype == K3Q_BF16) p = round_bf16(p);
    p = rintf(p);  // round half to even
    p = fminf(fmaxf(p, qlo), qhi);
    return (int)p;
}

// max over the threads that share a row: `kTpr` consecutive threads, kTpr in {64, 256}
template <int kTpr>
__device__ __forceinline__ float row_max(float v, float* lds) {
    v = wave_max(v);
    if (kTpr == kWave) return v;
    const int wave = threadIdx.x / kWave;
    if ((threadIdx.x % kWave) == 0) lds[wave] = v;
    __syncthreads();
    float r = lds[0];
#pragma unroll
    for (int w = 1; w < kTpr / kWave; ++w) r = fmaxf(r, lds[w]);
    return r;
}

// Fast path.  cols % 16 == 0, rows 16-byte aligned.  kTpr threads share a row (a wave, or the whole
// 256-thread block); a thread keeps up to kGroups * kCpg 16-byte pieces of the row in registers,
// piece j of a thread being piece j * kTpr + lane of the row: every load instruction of a wave reads
// 1 KiB contiguous and every store 512 (bfloat16) or 256 (float32) contiguous bytes.  (A thread that
// owned 16 consecutive elements, for the sake of 16-byte stores, made every load instruction touch
// its lines half or a quarter at a time: 4096 x 8192 bfloat16 19.4-20.9 -> 16.8-17.4 us.)
// kFast (bfloat16 rows, integer ends of the range): quantize_piece_bf16, 7 instructions per value
// instead of 11 -- at 4096 x 8192 the kernel's arithmetic is otherwise as long as its memory traffic.
template <int kDtype, int kTpr, int kGroups, bool kFast = false>
__global__ __launch_bounds__(256) void quantize_rows_vec(const char* __restrict__ x, int64_t rows,
                                                         int64_t groups_per_row,
                                                         int64_t x_row_bytes, float eps, float qlo,
                                                         float qhi, int8_t* __restrict__ q,
                                                         void* __restrict__ scale) {
    constexpr int kPer = Elem<kDtype>::kPerChunk;
    constexpr int kCpg = 16 / kPer;  // 16-byte pieces per group of 16 elements
    constexpr int kPieces = kGroups * kCpg;
    constexpr int kRowsPerBlock = 256 / kTpr;
    static_assert(!kFast || kDtype == K3Q_BF16, "the fast form is for bfloat16 rows");
    __shared__ float lds[256 / kWave];
    const int lane = threadIdx.x % kTpr;
    const int64_t row = (int64_t)blockIdx.x * kRowsPerBlock + threadIdx.x / kTpr;
    const bool live = row < rows;
    const v4u* xr = (const v4u*)(x + (live ? row : 0) * x_row_bytes);
    const int pieces = (int)groups_per_row * kCpg;

    // A row that fills every piece of every thread (the usual case: the row length is a multiple of
    // what the block holds at once) runs without per-piece predicates: the compiler then issues the
    // loads back to back and interleaves the pieces' arithmetic instead of one branch per piece.
    auto run = [&](auto full_c) {
        constexpr bool full = decltype(full_c)::value;
        v4u c[kPieces];
        float amax = 0.0f;
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const int pi = j * kTpr + lane;
            if (full || (live && pi < pieces)) c[j] = __builtin_nontemporal_load(xr + pi);
        }
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const int pi = j * kTpr + lane;
            if (full || (live && pi < pieces)) {
                float f[kPer];
                chunk_to_floats<kDtype>(c[j], f);
#pragma unroll
                for (int e = 0; e < kPer; ++e) amax = fmaxf(amax, fabsf(f[e]));
            }
        }
        amax = row_max<kTpr>(amax, lds);
        if (!live) return;
        const float s = scale_from_amax<kDtype>(amax, eps, qhi);
        if (lane == 0) {
            if (kDtype == K3Q_F32)
                ((float*)scale)[row] = s;
            else
                ((uint16_t*)scale)[row] = (uint16_t)(__float_as_uint(s) >> 16);
        }
        int8_t* qr = q + row * groups_per_row * 16;
#pragma unroll
        for (int j = 0; j < kPieces; ++j) {
            const int pi = j * kTpr + lane;
            if (full || pi < pieces) {
                if constexpr (kFast) {
                    __builtin_nontemporal_store(quantize_piece_bf16(c[j], s, qlo, qhi), (v2u*)qr + pi);
                } else {
                    float f[kPer];
                    chunk_to_floats<kDtype>(c[j], f);
                    u32 o[kPer / 4];
#pragma unroll
                    for (int d = 0; d < kPer / 4; ++d) {
                        u32 b0 = (u32)quantize_one<kDtype>(f[4 * d + 0], s, qlo, qhi) & 0xffu;
                        u32 b1 = (u32)quantize_one<kDtype>(f[4 * d + 1], s, qlo, qhi) & 0xffu;
                        u32 b2 = (u32)quantize_one<kDtype>(f[4 * d + 2], s, qlo, qhi) & 0xffu;
                        u32 b3 = (u32)quantize_one<kDtype>(f[4 * d + 3], s, qlo, qhi) & 0xffu;
                        o[d] = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
                    }
                    if constexpr (kPer == 8) {
                        const v2u ov = {o[0], o[1]};
                        __builtin_nontemporal_store(ov, (v2u*)qr + pi);
                    } else {
                        __builtin_nontemporal_store(o[0], (u32*)qr + pi);
                    }
                }
            }
        }
    };
    // (uniform over the block: with several rows per block the last block may hold dead rows)
    const bool all_live = (int64_t)(blockIdx.x + 1) * kRowsPerBlock <= rows;
    if (all_live && pieces == kPieces * kTpr)
        run(std::true_type{});
    else
        run(std::false_type{});
}

// Any shape / alignment, and rows too long for the register-resident path:
// one block per row, two passes over the row (the second one hits L2).
template <int kDtype>
__global__ __launch_bounds__(256) void quantize_rows_generic(const char* __restrict__ x,
                                                             int64_t cols, int64_t x_row_stride,
                                                             float eps, float qlo, float qhi,
                                                             int8_t* __restrict__ q,
                                                             void* __restrict__ scale) {
    __shared__ float lds[256 / kWave];
    const int64_t row = blockIdx.x;
    float amax = 0.0f;
    auto load = [&](int64_t c) -> float {
        if (kDtype == K3Q_F32) return ((const float*)x)[row * x_row_stride + c];
        return bf16_bits_to_f32(((const uint16_t*)x)[row * x_row_stride + c]);
    };
    for (int64_t c = threadIdx.x; c < cols; c += 256) amax = fmaxf(amax, fabsf(load(c)));
    amax = row_max<256>(amax, lds);
    const float s = scale_from_amax<kDtype>(amax, eps, qhi);
    if (threadIdx.x == 0) {
        if (kDtype == K3Q_F32)
            ((float*)scale)[row] = s;
        else
            ((uint16_t*)scale)[row] = (uint16_t)(__float_as_uint(s) >> 16);
    }
    for (int64_t c = threadIdx.x; c < cols; c += 256)
        q[row * cols + c] = (int8_t)quantize_one<kDtype>(load(c), s, qlo, qhi);
}

template <int kDtype, int kTpr, int kGroups>
void launch_vec(const void* x, int64_t rows, int64_t groups_per_row, int64_t row_bytes, float eps,
                float qlo, float qhi, int8_t* q, void* scale, hipStream_t s) {
    constexpr int kRowsPerBlock = 256 / kTpr;
    unsigned blocks = (unsigned)((rows + kRowsPerBlock - 1) / kRowsPerBlock);
    if constexpr (kDtype == K3Q_BF16) {
        if (qlo == rintf(qlo) && qhi == rintf(qhi)) {
            quantize_rows_vec<kDtype, kTpr, kGroups, true><<<blocks, 256, 0, s>>>(
                (const char*)x, rows, groups_per_row, row_bytes, eps, qlo, qhi, q, scale);
            return;
        }
    }
    quantize_rows_vec<kDtype, kTpr, kGroups><<<blocks, 256, 0, s>>>(
        (const char*)x, rows, groups_per_row, row_bytes, eps, qlo, qhi, q, scale);
}

#ifndef K3Q_QUANT_WAVE_ROW_MIN
#define K3Q_QUANT_WAVE_ROW_MIN 1024
#endif
constexpr int64_t kWaveRowMin = K3Q_QUANT_WAVE_ROW_MIN;

template <int kDtype>
int dispatch(const void* x, int64_t rows, int64_t cols, int64_t stride, float eps, float qlo,
             float qhi, int8_t* q, void* scale, hipStream_t s) {
    constexpr int kBytes = Elem<kDtype>::kBytes;
    const bool vec_ok = (cols % 16) == 0 && ((stride * kBytes) % 16) == 0 && aligned_to(x, 16) &&
                        aligned_to(q, 16);
    const int64_t gpr = cols / 16;  // 16-element groups per row
    // A wave per row (no LDS, no barrier) for short rows, where a 256-thread block would idle
    // most of its lanes; longer rows do better spread over a block (fewer registers per
    // thread, more rows in flight per CU).
    if (vec_ok && (gpr <= 64 || (gpr <= 128 && rows >= kWaveRowMin))) {
        if (gpr <= 64)
            launch_vec<kDtype, 64, 1>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
        else
            launch_vec<kDtype, 64, 2>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
    } else if (vec_ok && gpr <= 256 * 8) {
        if (gpr <= 256)
            launch_vec<kDtype, 256, 1>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
        else if (gpr <= 512)
            launch_vec<kDtype, 256, 2>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
        else if (gpr <= 1024)
            launch_vec<kDtype, 256, 4>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
        else
            launch_vec<kDtype, 256, 8>(x, rows, gpr, stride * kBytes, eps, qlo, qhi, q, scale, s);
    } else {
        quantize_rows_generic<kDtype><<<(unsigned)rows, 256, 0, s>>>((const char*)x, cols, stride,
                                                                     eps, qlo, qhi, q, scale);
    }
    return launch_status();
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_absmax_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols,
                                   int64_t x_row_stride, float eps, float qlo, float qhi,
                                   int8_t* q, void* scale, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (rows < 0 || cols < 0 || x_row_stride < cols) return K3Q_ERR_SHAPE;
    if (rows > 0x7fffffff) return K3Q_ERR_SHAPE;
    if (!(qlo >= -128.0f && qhi <= 127.0f && qlo <= qhi)) return K3Q_ERR_RANGE;
    if (rows == 0) return K3Q_OK;
    if (cols == 0) return K3Q_ERR_SHAPE;  // the reference raises on an empty reduction
    if (!x || !q || !scale) return K3Q_ERR_NULL;
    if (!aligned_to(x, x_dtype == K3Q_F32 ? 4 : 2) || !aligned_to(scale, x_dtype == K3Q_F32 ? 4 : 2))
        return K3Q_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    if (x_dtype == K3Q_F32)
        return dispatch<K3Q_F32>(x, rows, cols, x_row_stride, eps, qlo, qhi, q, scale, s);
    // torch rounds the epsilon operand to the tensor dtype before the add
    const float eps_bf16 = host_round_bf16(eps);
    return dispatch<K3Q_BF16>(x, rows, cols, x_row_stride, eps_bf16, qlo, qhi, q, scale, s);
}
