/*
 * Test hooks of libk3q.so.  NOT part of the C ABI (include/k3q.h): nothing here is for callers,
 * the prefix is k3qt_, and a binding must not depend on any of it.  The parity tests reach these
 * through keras_amd._lib.TEST_SIGNATURES.
 */
#pragma once
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/*
 * k3q_gemv_w4_fused with the launch plan overridden, so that the
 * parity tests can run every variant of the kernel (dwords per lane, rows per chunk, waves,
 * slice length) at one shape instead of relying on the shapes that select them:
 * plan = {dwords per lane per k row (1|2), 16-row steps per chunk (1|2),
 * waves per workgroup (1..8), rows of K per wave}; entries <= 0 and a null
 * `plan` keep the built-in choice.  The workspace must then hold
 * ceil(K / (waves * rows per wave)) * min(M, 16) * N floats.  No counterpart in the reference.
 */
int k3qt_gemv_w4_plan(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                     const void* w_packed, const void* scale, const void* zero,
                     int64_t block_size, const void* bias, void* y, void* workspace,
                     int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                     const int* plan, void* stream);

#ifdef __cplusplus
}
#endif
