// Shared device helpers for the k3q kernels (gfx950 only).
#pragma once

#include <hip/hip_runtime.h>
#include <stdint.h>
#include <string.h>

#include "../../include/k3q.h"

namespace k3q {

typedef uint32_t u32;
typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef float v16f __attribute__((ext_vector_type(16)));
typedef __bf16 v8bf __attribute__((ext_vector_type(8)));
typedef u32 v4u __attribute__((ext_vector_type(4)));
typedef u32 v2u __attribute__((ext_vector_type(2)));

constexpr int kWave = 64;

__device__ __forceinline__ float bf16_bits_to_f32(u32 h) { return __uint_as_float(h << 16); }

// A float32 / bfloat16 element as raw bits, and back.  Loads issued as raw bits can all be
// in flight before the first conversion waits for one of them.
template <bool kBF16>
__device__ __forceinline__ u32 load_raw(const void* p, int64_t i) {
    if (kBF16) return (u32)((const uint16_t*)p)[i];
    return ((const u32*)p)[i];
}
template <bool kBF16>
__device__ __forceinline__ float raw_to_f32(u32 bits) {
    return __uint_as_float(kBF16 ? bits << 16 : bits);
}

// float -> bfloat16 bits, round to nearest even (NaN stays NaN): one v_cvt_pk_bf16_f32.
__device__ __forceinline__ u32 f32_to_bf16_bits(float f) {
    return (u32)__builtin_bit_cast(unsigned short, (__bf16)f);
}

// two floats -> packed bfloat16 pair (lo in bits 0..15), one conversion instruction
__device__ __forceinline__ u32 pack_bf16x2(float lo, float hi) {
    typedef __bf16 bf2 __attribute__((ext_vector_type(2)));
    typedef float f2 __attribute__((ext_vector_type(2)));
    const f2 v = {lo, hi};
    return __builtin_bit_cast(u32, __builtin_convertvector(v, bf2));
}

// value of f after a round trip through bfloat16
__device__ __forceinline__ float round_bf16(float f) { return (float)(__bf16)f; }

// bfloat16(a / b) for a and b that are themselves bfloat16 values, bit-identical to rounding
// the IEEE float32 quotient.  Such a quotient is never closer than 2^-17 (relative) to the
// midpoint of two bfloat16 values: with 8-bit significands A, B the distance is
// |512 A - (2j+1) B| / (512 B), a non-zero integer over less than 2^17.  a * rcp(b) is within
// 2^-22, so it rounds the same way.  Operands outside [2^-60, 2^60] (where rcp or the product
// could leave the normal range) take the IEEE division.
__device__ __forceinline__ float div_round_bf16(float a, float b) {
    const u32 ea = (__float_as_uint(a) >> 23) & 0xffu, eb = (__float_as_uint(b) >> 23) & 0xffu;
    const bool a_ok = (ea - 67u) <= 120u || (__float_as_uint(a) << 1) == 0u;
    if (__builtin_expect(a_ok && (eb - 67u) <= 120u, 1)) return round_bf16(a * __builtin_amdgcn_rcpf(b));
    return round_bf16(a / b);
}

// Maximum over the 64 lanes of a wave, in every lane.  Data-parallel-primitive moves instead of
// shuffles through the LDS crossbar: six dependent steps at register speed (a shuffle step costs an
// LDS round trip, which a kernel that reduces per 16-byte piece pays many times over).  A lane whose
// source lane is outside its row, or masked, keeps its own value: fmaxf(v, v).  All 64 lanes must be
// active.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move(float v) {
    const int i = __float_as_int(v);
    return __int_as_float(__builtin_amdgcn_update_dpp(i, i, kCtrl, kRowMask, 0xf, false));
}
__device__ __forceinline__ float wave_max(float v) {
    v = fmaxf(v, dpp_move<0xB1, 0xf>(v));   // quad_perm [1,0,3,2]
    v = fmaxf(v, dpp_move<0x4E, 0xf>(v));   // quad_perm [2,3,0,1]
    v = fmaxf(v, dpp_move<0x141, 0xf>(v));  // row_half_mirror: the other quad of each half row
    v = fmaxf(v, dpp_move<0x140, 0xf>(v));  // row_mirror: the other half of each row of 16
    v = fmaxf(v, dpp_move<0x142, 0xa>(v));  // row_bcast15: rows 1 and 3 take in rows 0 and 2
    v = fmaxf(v, dpp_move<0x143, 0xc>(v));  // row_bcast31: rows 2 and 3 take in row 1 (= rows 0, 1)
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Eight bfloat16 values of a 16-byte piece -> eight int8 (two dwords), abs-max quantisation with the
// row's scale s: product, its bfloat16 rounding (one conversion per pair), clip, and rint + int
// conversion in one addition (1.5 * 2^23 + v leaves rint(v), half to even, in the low mantissa bits:
// the byte is its two's complement).  The clip comes BEFORE the rounding, which equals the reference's
// round-then-clip only when the ends of the range are integers: callers check that.
__device__ __forceinline__ v2u quantize_piece_bf16(const v4u& c, float s, float qlo, float qhi) {
    u32 t[8];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const u32 pk = pack_bf16x2(__uint_as_float(c[e] << 16) * s, __uint_as_float(c[e] & 0xffff0000u) * s);
        const float v0 = fminf(fmaxf(__uint_as_float(pk << 16), qlo), qhi);
        const float v1 = fminf(fmaxf(__uint_as_float(pk & 0xffff0000u), qlo), qhi);
        t[2 * e] = __float_as_uint(v0 + 12582912.0f);
        t[2 * e + 1] = __float_as_uint(v1 + 12582912.0f);
    }
    const u32 a0 = __builtin_amdgcn_perm(t[1], t[0], 0x0c0c0400u), a1 = __builtin_amdgcn_perm(t[3], t[2], 0x0c0c0400u);
    const u32 b0 = __builtin_amdgcn_perm(t[5], t[4], 0x0c0c0400u), b1 = __builtin_amdgcn_perm(t[7], t[6], 0x0c0c0400u);
    const v2u o = {a0 | (a1 << 16), b0 | (b1 << 16)};
    return o;
}

// Sum over the 64 lanes of a wave, in every lane, by the same moves (lanes a move does not write
// add zero).  The tree is fixed: pairs, quads, halves of a row, rows of 16, then
// (row 3 + row 2) + (row 1 + row 0) -- kernels that must agree bit for bit on a float sum (a
// normalisation computed alone or inside a matmul kernel) both reduce with this.
template <int kCtrl, int kRowMask>
__device__ __forceinline__ float dpp_move_or_zero(float v) {
    return __int_as_float(__builtin_amdgcn_update_dpp(0, __float_as_int(v), kCtrl, kRowMask, 0xf, false));
}
__device__ __forceinline__ float wave_sum(float v) {
    v += dpp_move_or_zero<0xB1, 0xf>(v);
    v += dpp_move_or_zero<0x4E, 0xf>(v);
    v += dpp_move_or_zero<0x141, 0xf>(v);
    v += dpp_move_or_zero<0x140, 0xf>(v);
    v += dpp_move_or_zero<0x142, 0xa>(v);
    v += dpp_move_or_zero<0x143, 0xc>(v);
    return __int_as_float(__builtin_amdgcn_readlane(__float_as_int(v), 63));
}

// Sum of squares of the eight bfloat16 values of a 16-byte piece, float32, fixed order.
__device__ __forceinline__ float piece_sum_squares(const v4u& c) {
    float q[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(c[e] << 16), hi = __uint_as_float(c[e] & 0xffff0000u);
        q[e] = lo * lo + hi * hi;
    }
    return (q[0] + q[1]) + (q[2] + q[3]);
}

// RMS normalisation of a piece: bf16(x * rstd * w), one rounding of the float32 product.
__device__ __forceinline__ v4u piece_rms_scale(const v4u& x, const v4u& w, float rstd) {
    v4u o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float lo = __uint_as_float(x[e] << 16) * rstd * __uint_as_float(w[e] << 16);
        const float hi = __uint_as_float(x[e] & 0xffff0000u) * rstd * __uint_as_float(w[e] & 0xffff0000u);
        o[e] = pack_bf16x2(lo, hi);
    }
    return o;
}

// SwiGLU gate of a piece: bf16(bf16(silu(g)) * u), silu(g) = g / (1 + 2^(-g log2 e)) with the
// hardware's exp2 and reciprocal (each within an ulp or two of float32: the bfloat16 result differs
// from an exactly rounded one on a fraction of a percent of the elements, by one ulp).
__device__ __forceinline__ v4u piece_silu_mul(const v4u& g, const v4u& u) {
    v4u o;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float a[2] = {__uint_as_float(g[e] << 16), __uint_as_float(g[e] & 0xffff0000u)};
        const float b[2] = {__uint_as_float(u[e] << 16), __uint_as_float(u[e] & 0xffff0000u)};
#pragma unroll
        for (int h = 0; h < 2; ++h) {
            const float s = a[h] * __builtin_amdgcn_rcpf(1.0f + __builtin_amdgcn_exp2f(a[h] * -1.44269504f));
            a[h] = round_bf16(s) * b[h];
        }
        o[e] = pack_bf16x2(a[0], a[1]);
    }
    return o;
}

// byte select: result byte i = byte sel[i] of the 8-byte pool {lo: bytes 0-3, hi: bytes 4-7}
__device__ __forceinline__ u32 byte_perm(u32 hi, u32 lo, u32 sel) {
    return __builtin_amdgcn_perm(hi, lo, sel);
}

inline int launch_status() {
    return hipGetLastError() == hipSuccess ? K3Q_OK : K3Q_ERR_LAUNCH;
}

// host-side: value of f after rounding to bfloat16 (nearest even)
inline float host_round_bf16(float f) {
    uint32_t u;
    ::memcpy(&u, &f, 4);
    u += 0x7fffu + ((u >> 16) & 1u);
    u &= 0xffff0000u;
    ::memcpy(&f, &u, 4);
    return f;
}

inline bool aligned_to(const void* p, size_t a) { return (reinterpret_cast<uintptr_t>(p) % a) == 0; }

}  // namespace k3q
