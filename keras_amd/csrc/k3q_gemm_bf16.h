// bfloat16 x bfloat16 -> float32 GEMM on the tile machinery of the int8 GEMM
// (k3q_gemm_i8.hip): y[M,N] = T(T(a[M,K] . bt[N,K]^T) / scale[n]) (+ bias), bfloat16 operands.
// Used for prefill-sized int4 matmuls, where bt is the int4 kernel de-quantised into scratch.
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>

namespace k3q {

// K % 64 == 0, N % 4 == 0, 16-byte aligned operands
bool gemm_bf16_nk_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* bt,
                            const void* y);

// scratch for the partial sums of a K split (problems with few tiles and a long K); 0 if none
int64_t gemm_bf16_nk_workspace_bytes(int64_t M, int64_t N, int64_t K);

// b_scale [N] and bias [N] may be null; they and y are bfloat16, or float32 with out_f32 (the
// operands then being high / low bfloat16 parts of float32 values, concatenated along K).
// workspace (may be null: then K is not split) is 16-byte aligned scratch.
int gemm_bf16_nk_run(const void* a, const void* bt, int64_t M, int64_t N, int64_t K,
                     const void* b_scale, const void* bias, void* y, bool out_f32, void* workspace,
                     int64_t workspace_bytes, hipStream_t s);

// out[M, parts * K] (bfloat16) = [xh | xl (| xh)] of float32 x[M, K]: xh = the top 16 bits of
// a value, xl = the rounded remainder; K % 4 == 0 (k3q_gemv_w4.hip)
void split_f32_rows_launch(const float* x, uint16_t* out, int64_t M, int64_t K, int parts,
                           hipStream_t s);

}  // namespace k3q
