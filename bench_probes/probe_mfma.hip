// Measurement aid, not part of the product library: a loop of nothing but
// v_mfma_i32_32x32x32_i8 on register-resident operands (no LDS, no memory traffic), to read
// what the matrix cores of this board sustain under its power management.  Built into a
// library of its own (libk3q_probe.so); only bench.py loads it.
//
// Operand kinds: 0 all-zero bytes, 1 uniform random bytes, 2 activation-like (small
// magnitudes, as an abs-max quantised normal row has) against uniform random weights.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v16i __attribute__((ext_vector_type(16)));

__device__ inline unsigned mix(unsigned x) {
    x ^= x >> 16;
    x *= 0x7feb352dU;
    x ^= x >> 15;
    x *= 0x846ca68bU;
    x ^= x >> 16;
    return x;
}

// 256 threads = one wave per SIMD; every wave keeps four independent accumulator chains busy.
// clk[0] = shader clocks, clk[1] = 100 MHz reference ticks of workgroup 0, start to end.
__global__ __launch_bounds__(256) void mfma_i8_only(int kind, int iters, int* sink, unsigned long long* clk) {
    const unsigned long long c0 = __builtin_readcyclecounter(), r0 = __builtin_amdgcn_s_memrealtime();
    v4i a[2], b[2];
    for (int i = 0; i < 2; ++i)
        for (int j = 0; j < 4; ++j) {
            const unsigned h = mix(threadIdx.x * 131 + i * 17 + j + blockIdx.x * 7919), h2 = mix(h + 12345);
            unsigned small = 0;
            for (int q = 0; q < 4; ++q) small |= ((unsigned)((((int)((h >> (8 * q)) & 63)) - 32) & 0xff)) << (8 * q);
            a[i][j] = kind == 0 ? 0 : kind == 1 ? (int)h : (int)small;
            b[i][j] = kind == 0 ? 0 : (int)h2;
        }
    v16i c[4];
    for (int i = 0; i < 4; ++i)
        for (int r = 0; r < 16; ++r) c[i][r] = 0;
    for (int it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < 2; ++i)
#pragma unroll
            for (int j = 0; j < 2; ++j)
                c[i * 2 + j] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a[i], b[j], c[i * 2 + j], 0, 0, 0);
    }
    const v16i s = c[0] + c[1] + c[2] + c[3];
    if (s[0] == 0x7ffffff1) sink[0] = s[1];  // keeps the loop alive
    if (threadIdx.x == 0 && blockIdx.x == 0) {
        clk[0] = __builtin_readcyclecounter() - c0;
        clk[1] = __builtin_amdgcn_s_memrealtime() - r0;
    }
}

}  // namespace

// Launches the loop on 1024 workgroups (4 waves each).  `out` is 32 bytes of device memory:
// [0,16) two uint64 clock readings, [16,20) a sink.  Returns the integer operations the launch
// performs (2 per multiply-accumulate), or -1 for a bad argument or a failed launch.
extern "C" double k3q_probe_mfma_i8_only(int kind, int iters, void* out, void* stream) {
    if (kind < 0 || kind > 2 || iters <= 0 || !out) return -1.0;
    mfma_i8_only<<<1024, 256, 0, (hipStream_t)stream>>>(kind, iters, (int*)((char*)out + 16),
                                                       (unsigned long long*)out);
    if (hipGetLastError() != hipSuccess) return -1.0;
    return 1024.0 * 4 * 4 * 65536.0 * iters;
}
