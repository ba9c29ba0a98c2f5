// int4 <-> int8 nibble packing along the middle axis of [outer, len, inner].
//
// Both directions are pure HBM streams (1.5 bytes moved per int4 value), so
// the fast paths do nothing but 8- or 16-byte loads, a handful of bit operations
// per dword and 16-byte stores that fill whole cache lines per instruction.  inner == 1 is the "pack along the last axis" case
// (the two nibbles of a byte are neighbours in memory and must be interleaved
// with byte permutes); inner > 1 is the "pack along a leading axis" case (the
// two nibbles go to two different rows, no interleave).
#include "k3q_common.h"

namespace k3q {
namespace {

constexpr int kThreads = 256;
constexpr u32 kLowNibbles = 0x0F0F0F0Fu;

// 4 nibble-valued bytes (0..15) -> 4 sign-extended int4 bytes: (v ^ 8) - 8 per byte.
// v | 0xF0 when bit 3 is set; (v & 8) * 0x1E == 0xF0 and never carries out of the byte.
__device__ __forceinline__ u32 sign_extend_nibbles(u32 v) { return v | ((v & 0x08080808u) * 0x1Eu); }

template <bool kSigned>
__device__ __forceinline__ void split_dword(u32 w, u32& lo, u32& hi) {
    lo = w & kLowNibbles;
    hi = (w >> 4) & kLowNibbles;
    if (kSigned) {
        lo = sign_extend_nibbles(lo);
        hi = sign_extend_nibbles(hi);
    }
}

// ---- unpack, nibbles adjacent along the packed axis (inner == 1) ----------
// A thread turns 8 packed bytes into one 16-byte store, twice: the stores of a wave are then 1 KiB
// of consecutive addresses each (16 packed bytes -> two neighbouring stores per thread would leave
// every store instruction filling half of each cache line, and memory sees the partial writes).
template <bool kSigned>
__global__ __launch_bounds__(kThreads) void unpack_last_vec(const v2u* __restrict__ in,
                                                            v4u* __restrict__ out, int64_t n_half) {
#pragma unroll
    for (int h = 0; h < 2; ++h) {
        const int64_t i = ((int64_t)blockIdx.x * 2 + h) * kThreads + threadIdx.x;
        if (i >= n_half) return;
        const v2u w = __builtin_nontemporal_load(in + i);
        v4u o;
#pragma unroll
        for (int d = 0; d < 2; ++d) {
            u32 lo, hi;
            split_dword<kSigned>(w[d], lo, hi);
            o[2 * d] = byte_perm(hi, lo, 0x05010400u);      // lo0 hi0 lo1 hi1
            o[2 * d + 1] = byte_perm(hi, lo, 0x07030602u);  // lo2 hi2 lo3 hi3
        }
        __builtin_nontemporal_store(o, out + i);
    }
}

// ---- unpack, nibbles go to rows 2j and 2j+1 (inner % 16 == 0) -------------
template <bool kSigned>
__global__ __launch_bounds__(kThreads) void unpack_mid_vec(const v4u* __restrict__ in,
                                                           v4u* __restrict__ out, int64_t outer,
                                                           int64_t plen, int64_t inner16,
                                                           int64_t orig_len) {
    int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    int64_t total = outer * plen * inner16;
    if (t >= total) return;
    int64_t i = t % inner16;
    int64_t j = (t / inner16) % plen;
    int64_t o = t / (inner16 * plen);
    v4u w = __builtin_nontemporal_load(in + t);
    v4u lo, hi;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        u32 l, h;
        split_dword<kSigned>(w[d], l, h);
        lo[d] = l;
        hi[d] = h;
    }
    int64_t row = o * orig_len + 2 * j;
    __builtin_nontemporal_store(lo, out + row * inner16 + i);
    if (2 * j + 1 < orig_len) __builtin_nontemporal_store(hi, out + (row + 1) * inner16 + i);
}

// ---- unpack, any shape: one packed byte per thread ------------------------
template <bool kSigned>
__global__ __launch_bounds__(kThreads) void unpack_generic(const uint8_t* __restrict__ in,
                                                           uint8_t* __restrict__ out, int64_t outer,
                                                           int64_t plen, int64_t inner,
                                                           int64_t orig_len) {
    int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    int64_t total = outer * plen * inner;
    if (t >= total) return;
    int64_t i = t % inner;
    int64_t j = (t / inner) % plen;
    int64_t o = t / (inner * plen);
    if (2 * j >= orig_len) return;  // slice that holds only padding
    u32 b = in[t];
    u32 lo = b & 0x0Fu;
    u32 hi = (b >> 4) & 0x0Fu;
    if (kSigned) {
        lo = (lo ^ 8u) - 8u;
        hi = (hi ^ 8u) - 8u;
    }
    int64_t base = (o * orig_len + 2 * j) * inner + i;
    out[base] = (uint8_t)lo;
    if (2 * j + 1 < orig_len) out[base + inner] = (uint8_t)hi;
}

// ---- pack, inner == 1, even length -----------------------------------------
__global__ __launch_bounds__(kThreads) void pack_last_vec(const v4u* __restrict__ in,
                                                          v4u* __restrict__ out, int64_t n_chunks) {
    int64_t i = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    if (i >= n_chunks) return;
    v4u a = __builtin_nontemporal_load(in + 2 * i);
    v4u b = __builtin_nontemporal_load(in + 2 * i + 1);
    v4u r;
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        u32 w0 = d < 2 ? a[2 * d] : b[2 * (d - 2)];
        u32 w1 = d < 2 ? a[2 * d + 1] : b[2 * (d - 2) + 1];
        u32 even = byte_perm(w1, w0, 0x06040200u);
        u32 odd = byte_perm(w1, w0, 0x07050301u);
        r[d] = (even & kLowNibbles) | ((odd & kLowNibbles) << 4);
    }
    __builtin_nontemporal_store(r, out + i);
}

// ---- pack, rows 2j and 2j+1 (inner % 16 == 0) -------------------------------
__global__ __launch_bounds__(kThreads) void pack_mid_vec(const v4u* __restrict__ in,
                                                         v4u* __restrict__ out, int64_t outer,
                                                         int64_t len, int64_t inner16) {
    int64_t plen = (len + 1) / 2;
    int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    int64_t total = outer * plen * inner16;
    if (t >= total) return;
    int64_t i = t % inner16;
    int64_t j = (t / inner16) % plen;
    int64_t o = t / (inner16 * plen);
    int64_t row = o * len + 2 * j;
    v4u lo = __builtin_nontemporal_load(in + row * inner16 + i);
    v4u hi = {0u, 0u, 0u, 0u};
    if (2 * j + 1 < len) hi = __builtin_nontemporal_load(in + (row + 1) * inner16 + i);
    v4u r;
#pragma unroll
    for (int d = 0; d < 4; ++d) r[d] = (lo[d] & kLowNibbles) | ((hi[d] & kLowNibbles) << 4);
    __builtin_nontemporal_store(r, out + t);
}

// ---- pack, any shape --------------------------------------------------------
__global__ __launch_bounds__(kThreads) void pack_generic(const uint8_t* __restrict__ in,
                                                         uint8_t* __restrict__ out, int64_t outer,
                                                         int64_t len, int64_t inner) {
    int64_t plen = (len + 1) / 2;
    int64_t t = (int64_t)blockIdx.x * kThreads + threadIdx.x;
    int64_t total = outer * plen * inner;
    if (t >= total) return;
    int64_t i = t % inner;
    int64_t j = (t / inner) % plen;
    int64_t o = t / (inner * plen);
    int64_t base = (o * len + 2 * j) * inner + i;
    u32 lo = in[base];
    u32 hi = (2 * j + 1 < len) ? in[base + inner] : 0u;
    out[t] = (uint8_t)((lo & 0x0Fu) | ((hi & 0x0Fu) << 4));
}

inline unsigned blocks_for(int64_t n) { return (unsigned)((n + kThreads - 1) / kThreads); }
constexpr int64_t kMaxThreads = (int64_t)0x7fffffff * kThreads;

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_pack_int4(const void* in, int64_t outer, int64_t len, int64_t inner, void* out,
                             void* stream) {
    if (outer < 0 || len < 0 || inner < 0) return K3Q_ERR_SHAPE;
    int64_t plen = (len + 1) / 2;
    int64_t total = outer * plen * inner;
    if (total == 0) return K3Q_OK;
    if (!in || !out) return K3Q_ERR_NULL;
    if (total > kMaxThreads) return K3Q_ERR_SHAPE;
    hipStream_t s = (hipStream_t)stream;
    bool al = aligned_to(in, 16) && aligned_to(out, 16);
    if (inner == 1 && (len % 2) == 0 && (total % 16) == 0 && al) {
        int64_t n = total / 16;
        pack_last_vec<<<blocks_for(n), kThreads, 0, s>>>((const v4u*)in, (v4u*)out, n);
    } else if (inner > 1 && (inner % 16) == 0 && al) {
        int64_t n = total / 16;
        pack_mid_vec<<<blocks_for(n), kThreads, 0, s>>>((const v4u*)in, (v4u*)out, outer, len,
                                                        inner / 16);
    } else {
        pack_generic<<<blocks_for(total), kThreads, 0, s>>>((const uint8_t*)in, (uint8_t*)out,
                                                            outer, len, inner);
    }
    return launch_status();
}

extern "C" int k3q_unpack_int4(const void* in, int64_t outer, int64_t packed_len, int64_t inner,
                               int64_t orig_len, int is_signed, void* out, void* stream) {
    if (outer < 0 || packed_len < 0 || inner < 0 || orig_len < 0) return K3Q_ERR_SHAPE;
    if (orig_len > 2 * packed_len) return K3Q_ERR_SHAPE;
    int64_t total = outer * packed_len * inner;
    if (total == 0 || orig_len == 0) return K3Q_OK;
    if (!in || !out) return K3Q_ERR_NULL;
    if (total > kMaxThreads) return K3Q_ERR_SHAPE;
    // Slices beyond ceil(orig_len/2) hold only padding and are never unpacked.
    int64_t used_plen = (orig_len + 1) / 2;
    hipStream_t s = (hipStream_t)stream;
    bool al = aligned_to(in, 16) && aligned_to(out, 16);
    bool full = (used_plen == packed_len);
    if (inner == 1 && full && orig_len == 2 * packed_len && (total % 16) == 0 && al) {
        int64_t n = total / 8;  // 8 packed bytes per store
        if (is_signed)
            unpack_last_vec<true><<<blocks_for((n + 1) / 2), kThreads, 0, s>>>((const v2u*)in, (v4u*)out, n);
        else
            unpack_last_vec<false><<<blocks_for((n + 1) / 2), kThreads, 0, s>>>((const v2u*)in, (v4u*)out, n);
    } else if (inner > 1 && (inner % 16) == 0 && full && al) {
        int64_t n = total / 16;
        if (is_signed)
            unpack_mid_vec<true><<<blocks_for(n), kThreads, 0, s>>>(
                (const v4u*)in, (v4u*)out, outer, packed_len, inner / 16, orig_len);
        else
            unpack_mid_vec<false><<<blocks_for(n), kThreads, 0, s>>>(
                (const v4u*)in, (v4u*)out, outer, packed_len, inner / 16, orig_len);
    } else {
        if (is_signed)
            unpack_generic<true><<<blocks_for(total), kThreads, 0, s>>>(
                (const uint8_t*)in, (uint8_t*)out, outer, packed_len, inner, orig_len);
        else
            unpack_generic<false><<<blocks_for(total), kThreads, 0, s>>>(
                (const uint8_t*)in, (uint8_t*)out, outer, packed_len, inner, orig_len);
    }
    return launch_status();
}
