// Streaming weight-only int8 matmul, [N, K] kernel, 1..8 rows of float activations.
//
// A wave owns whole rows of the kernel: per iteration its 64 lanes load 16 bytes each of one
// row (1 KiB contiguous), convert the bytes to float (v_bfe_i32 + v_cvt_f32_i32) and
// multiply-add them into one float accumulator per row of x; the rows of x (at most four per
// pass) sit in LDS in their own dtype, staged once per workgroup.  Two kernel rows, four
// pieces each, are in flight per wave so that enough loads are outstanding to cover HBM latency.  A wave-wide
// sum at the end of a row and the de-scale of the reference's weight-only branch
// (keras/src/layers/core/dense.py:961-983 without the activation quantizer):
// y = T(T(acc) / scale[n]) (+ bias[n]).  No matrix core: at <= 4 rows the conversion and
// the FMAs fit under the time the bytes take to arrive.
#include "k3q_common.h"
#include "k3q_gemv_w8.h"

namespace k3q {
namespace {

constexpr int kThreads = 512;       // 8 waves
constexpr int kRowsPerPass = 4;     // rows of x per launch
constexpr int kLdsBudget = 128 * 1024;

struct W8Params {
    const void* x;       // [rows, K]
    const int8_t* b;     // [N, K]
    const void* scale;   // T [N] or null
    const void* bias;    // T [N] or null
    void* y;             // [rows, N] (row stride N)
    int64_t N, K;
    int rows;            // 1..kRowsPerPass
};

template <bool kBF16>
__device__ __forceinline__ float load_scalar(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

// dot products of 16 weights (one 16-byte load) with the 16 activations of each row of x
template <bool kBF16, int kRows>
__device__ __forceinline__ void fma16(const v4u& w, const char* xs, int64_t row_bytes, int64_t k,
                                      float (&acc)[kRows]) {
    float wf[16];
#pragma unroll
    for (int j = 0; j < 16; ++j)
        wf[j] = (float)(int)__builtin_amdgcn_sbfe((int)w[j >> 2], 8 * (j & 3), 8);
#pragma unroll
    for (int m = 0; m < kRows; ++m) {
        const char* xr = xs + m * row_bytes;
        if (kBF16) {
            const v4u a = *(const v4u*)(xr + 2 * k), c = *(const v4u*)(xr + 2 * k + 16);
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                acc[m] = fmaf(wf[2 * d], __uint_as_float(a[d] << 16), acc[m]);
                acc[m] = fmaf(wf[2 * d + 1], __uint_as_float(a[d] & 0xffff0000u), acc[m]);
                acc[m] = fmaf(wf[8 + 2 * d], __uint_as_float(c[d] << 16), acc[m]);
                acc[m] = fmaf(wf[8 + 2 * d + 1], __uint_as_float(c[d] & 0xffff0000u), acc[m]);
            }
        } else {
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                const v4f a = *(const v4f*)(xr + 4 * k + 16 * q);
#pragma unroll
                for (int d = 0; d < 4; ++d) acc[m] = fmaf(wf[4 * q + d], a[d], acc[m]);
            }
        }
    }
}

template <bool kBF16, int kRows>
__global__ __launch_bounds__(kThreads) void gemv_w8_nk(W8Params p) {
    extern __shared__ __attribute__((aligned(16))) char xs[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    constexpr int kElt = kBF16 ? 2 : 4;
    const int64_t row_bytes = p.K * kElt;
    // the rows of x, as they are (K % 16 == 0: whole 16-byte pieces)
    for (int64_t i = (int64_t)tid * 16; i < kRows * row_bytes; i += kThreads * 16)
        *(v4u*)(xs + i) = *(const v4u*)((const char*)p.x + i);
    __syncthreads();

    const int64_t wave_id = (int64_t)blockIdx.x * (kThreads / 64) + wave;
    const int64_t waves = (int64_t)gridDim.x * (kThreads / 64);
    // two kernel rows per step: n and n + waves
    for (int64_t n = wave_id; n < p.N; n += 2 * waves) {
        const int64_t n2 = n + waves;
        const bool two = n2 < p.N;
        const int8_t* r0 = p.b + n * p.K;
        const int8_t* r1 = p.b + (two ? n2 : n) * p.K;
        float acc0[kRows], acc1[kRows];
#pragma unroll
        for (int m = 0; m < kRows; ++m) acc0[m] = acc1[m] = 0.f;
        // batches of 1 KiB pieces per row (four while x has one or two rows): loads in flight
        // before the first use
        constexpr int kBatch = kRows <= 2 ? 4 : 1;  // more rows of x: registers go to the FMAs
        for (int64_t k0 = (int64_t)lane * 16; k0 < p.K; k0 += kBatch * 64 * 16) {
            v4u w0[kBatch], w1[kBatch];
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int64_t k = k0 + j * 64 * 16;
                if (k < p.K) {
                    w0[j] = *(const v4u*)(r0 + k);
                    w1[j] = *(const v4u*)(r1 + k);
                }
            }
#pragma unroll
            for (int j = 0; j < kBatch; ++j) {
                const int64_t k = k0 + j * 64 * 16;
                if (k < p.K) {
                    fma16<kBF16, kRows>(w0[j], xs, row_bytes, k, acc0);
                    fma16<kBF16, kRows>(w1[j], xs, row_bytes, k, acc1);
                }
            }
        }
#pragma unroll
        for (int m = 0; m < kRows; ++m) {
#pragma unroll
            for (int o = 32; o > 0; o >>= 1) {
                acc0[m] += __shfl_xor(acc0[m], o, kWave);
                acc1[m] += __shfl_xor(acc1[m], o, kWave);
            }
        }
        // lane m finishes row m of x for kernel row n, lane kRows + m for kernel row n2
        const bool second = lane >= kRows;
        if (lane < 2 * kRows && (two || !second)) {
            const int m = lane % kRows;
            float a = 0.f;
#pragma unroll
            for (int q = 0; q < kRows; ++q) a = (q == m) ? (second ? acc1[q] : acc0[q]) : a;
            const int64_t col = second ? n2 : n;
            float r = a;
            if (kBF16) {
                r = round_bf16(r);
                if (p.scale) r = div_round_bf16(r, load_scalar<true>(p.scale, col));
                if (p.bias) r = round_bf16(r + load_scalar<true>(p.bias, col));
                ((uint16_t*)p.y)[m * p.N + col] = (uint16_t)f32_to_bf16_bits(r);
            } else {
                if (p.scale) r = r / load_scalar<false>(p.scale, col);
                if (p.bias) r = r + load_scalar<false>(p.bias, col);
                ((float*)p.y)[m * p.N + col] = r;
            }
        }
    }
}

template <bool kBF16, int kRows>
int launch(const W8Params& p, int grid, size_t lds, hipStream_t s) {
    static const bool raised =
        hipFuncSetAttribute((const void*)gemv_w8_nk<kBF16, kRows>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget) == hipSuccess;
    if (!raised) return K3Q_ERR_LAUNCH;
    gemv_w8_nk<kBF16, kRows><<<grid, kThreads, lds, s>>>(p);
    return launch_status();
}

template <bool kBF16>
int launch_rows(const W8Params& p, int grid, size_t lds, hipStream_t s) {
    switch (p.rows) {
        case 1: return launch<kBF16, 1>(p, grid, lds, s);
        case 2: return launch<kBF16, 2>(p, grid, lds, s);
        case 3: return launch<kBF16, 3>(p, grid, lds, s);
        default: return launch<kBF16, 4>(p, grid, lds, s);
    }
}

}  // namespace

bool gemv_w8_nk_supported(int64_t M, int64_t N, int64_t K, int x_dtype, const void* x, const void* b,
                          const void* y) {
    const int64_t elt = x_dtype == K3Q_BF16 ? 2 : 4;
    const int64_t rows = M < kRowsPerPass ? M : kRowsPerPass;
    return M >= 1 && M <= kGemvW8MaxRows && N >= 1 && (K % 16) == 0 && rows * K * elt <= kLdsBudget &&
           aligned_to(x, 16) && aligned_to(b, 16) && aligned_to(y, elt);
}

int gemv_w8_nk_run(const void* x, int x_dtype, const int8_t* b, int64_t M, int64_t N, int64_t K,
                   const void* scale, const void* bias, void* y, hipStream_t s) {
    const bool bf16 = x_dtype == K3Q_BF16;
    const int64_t elt = bf16 ? 2 : 4;
    // enough workgroups to give every wave two kernel rows at a time, at most two per CU
    int dev = 0, cus = 0;
    if (hipGetDevice(&dev) != hipSuccess ||
        hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || cus <= 0)
        return K3Q_ERR_LAUNCH;
    int64_t grid = (N + 2 * (kThreads / 64) - 1) / (2 * (kThreads / 64));
    if (grid > 2 * cus) grid = 2 * cus;
    for (int64_t m0 = 0; m0 < M; m0 += kRowsPerPass) {
        W8Params p{};
        p.rows = (int)(M - m0 < kRowsPerPass ? M - m0 : kRowsPerPass);
        p.x = (const char*)x + m0 * K * elt;
        p.b = b;
        p.scale = scale;
        p.bias = bias;
        p.y = (char*)y + m0 * N * elt;
        p.N = N;
        p.K = K;
        const size_t lds = (size_t)(p.rows * K * elt);
        const int rc = bf16 ? launch_rows<true>(p, (int)grid, lds, s) : launch_rows<false>(p, (int)grid, lds, s);
        if (rc != K3Q_OK) return rc;
    }
    return K3Q_OK;
}

}  // namespace k3q
