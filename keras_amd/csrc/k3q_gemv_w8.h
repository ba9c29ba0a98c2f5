// Weight-only int8 matmul for decode-sized M with the kernel stored K-contiguous ([N, K], the
// prepacked copy of a Dense kernel or a tied embedding table): float activations against int8
// weights, y = T(T(x . W^T) / scale[n]) (+ bias).  HBM-bound: the kernel is streamed once per
// pass of up to four rows of x.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace k3q {

constexpr int64_t kGemvW8MaxRows = 8;  // two passes; beyond that the MFMA route is faster

bool gemv_w8_nk_supported(int64_t M, int64_t N, int64_t K, int x_dtype, const void* x, const void* b,
                          const void* y);

// x: [M, K] of x_dtype (K3Q_F32 | K3Q_BF16); b: int8 [N, K]; scale / bias: x_dtype [N] or null
int gemv_w8_nk_run(const void* x, int x_dtype, const int8_t* b, int64_t M, int64_t N, int64_t K,
                   const void* scale, const void* bias, void* y, hipStream_t s);

}  // namespace k3q
