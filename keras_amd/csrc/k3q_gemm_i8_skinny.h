// Decode-sized int8 matmul (see k3q_gemm_i8_skinny.hip); called from k3q_gemm_i8.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace k3q {

constexpr int64_t kSkinnyMaxRows = 64;

// shape / alignment the skinny kernel takes: M <= 64, N % 16 == 0, K % 8 == 0, b in [K, N] layout
bool gemm_i8_skinny_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* b);

// scratch for the int32 split-K partials (0 when K is not split)
int64_t gemm_i8_skinny_workspace_bytes(int64_t M, int64_t N, int64_t K);

int gemm_i8_skinny_run(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                       const void* a_scale, const void* b_scale, const void* bias, bool bf16, int flags,
                       void* y, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                       hipStream_t s, bool bias_per_row = false);  // bias_per_row: bias is [M, N]

// the same for a kernel given in [N, K] layout (K contiguous): M <= 64, K % 64 == 0
bool gemm_i8_skinny_nk_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* b);
int64_t gemm_i8_skinny_nk_workspace_bytes(int64_t M, int64_t N, int64_t K);
int gemm_i8_skinny_nk_run(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                          const void* a_scale, const void* b_scale, const void* bias, bool bf16, int flags,
                          void* y, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                          hipStream_t s);

}  // namespace k3q
