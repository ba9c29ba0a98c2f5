// Measurement aid, not part of the product library (built into bench_probes/libk3q_probe.so;
// only bench.py loads it): what a launch that does nothing but READ a buffer costs on this board, and what a
// launch that does nothing at all costs.  The decode kernels stream a weight matrix once; their
// time per launch is compared with these two.
//
// stream_read: the access pattern of the decode kernels without their arithmetic -- 8 waves per
// workgroup, every wave a contiguous run, 1 KiB per load instruction (16 bytes per lane,
// nontemporal), `kDepth` loads of a wave in flight, a slot requested again as soon as it has been
// consumed.  Each workgroup writes one dword.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef unsigned v4u __attribute__((ext_vector_type(4)));

template <int kDepth>
__global__ __launch_bounds__(512) void stream_read(const v4u* src, int steps, unsigned* out) {
    const int lane = threadIdx.x & 63;
    const int wave = blockIdx.x * 8 + (threadIdx.x >> 6);
    const v4u* p = src + (int64_t)wave * steps * 64 + lane;
    v4u r[kDepth];
#pragma unroll
    for (int d = 0; d < kDepth; ++d) r[d] = __builtin_nontemporal_load(p + (int64_t)d * 64);
    v4u acc = {0u, 0u, 0u, 0u};
    // (steps is a multiple of kDepth, at least two rounds; the last round requests nothing)
    for (int base = kDepth; base < steps; base += kDepth) {
#pragma unroll
        for (int d = 0; d < kDepth; ++d) {
            acc ^= r[d];
            r[d] = __builtin_nontemporal_load(p + (int64_t)(base + d) * 64);
        }
    }
#pragma unroll
    for (int d = 0; d < kDepth; ++d) acc ^= r[d];
    unsigned v = acc[0] ^ acc[1] ^ acc[2] ^ acc[3];
#pragma unroll
    for (int o = 32; o > 0; o >>= 1) v ^= __shfl_xor(v, o, 64);
    __shared__ unsigned part[8];
    if (lane == 0) part[threadIdx.x >> 6] = v;
    __syncthreads();
    if (threadIdx.x == 0) {
        unsigned t = 0;
        for (int q = 0; q < 8; ++q) t ^= part[q];
        out[blockIdx.x] = t;
    }
}

__global__ void nothing(unsigned* out) {
    if (out == (unsigned*)1) out[0] = 0;  // never true
}

}  // namespace

// Reads `bytes` of `src` once with `workgroups` workgroups of 8 waves, `depth` (4, 8 or 16) loads
// of a wave in flight; `out` takes one dword per workgroup.  bytes must split into
// workgroups x 8 waves x depth x 1 KiB pieces, at least two rounds of them.  0, or -1 for a bad
// argument or a failed launch.
extern "C" int k3q_probe_stream_read(const void* src, int64_t bytes, int workgroups, int depth, void* out,
                                     void* stream) {
    if (!src || !out || bytes <= 0 || workgroups <= 0) return -1;
    const int64_t per_wave = bytes / ((int64_t)workgroups * 8);
    if (per_wave * workgroups * 8 != bytes || per_wave % (1024 * (int64_t)depth) || per_wave < 2048 * (int64_t)depth)
        return -1;
    const int steps = (int)(per_wave / 1024);
    hipStream_t s = (hipStream_t)stream;
    if (depth == 4) stream_read<4><<<workgroups, 512, 0, s>>>((const v4u*)src, steps, (unsigned*)out);
    else if (depth == 8) stream_read<8><<<workgroups, 512, 0, s>>>((const v4u*)src, steps, (unsigned*)out);
    else if (depth == 16) stream_read<16><<<workgroups, 512, 0, s>>>((const v4u*)src, steps, (unsigned*)out);
    else return -1;
    return hipGetLastError() == hipSuccess ? 0 : -1;
}

// One workgroup of one wave that does nothing: the cost of a launch itself.
extern "C" int k3q_probe_empty(void* out, void* stream) {
    nothing<<<1, 64, 0, (hipStream_t)stream>>>((unsigned*)out);
    return hipGetLastError() == hipSuccess ? 0 : -1;
}
