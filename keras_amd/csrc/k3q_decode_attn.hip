// One new position of causal self-attention against a key / value cache, bfloat16, head
// width 128: rotate the new query and key (rotate-half RoPE, tables indexed by the position),
// write the new key and value rows into the cache at the position, attend over rows
// 0 ... position.  One launch where the decoder step otherwise runs a dozen small ones.
//
// One workgroup per (sequence, head), 8 waves.  A wave instruction covers 4 cache rows
// (16 lanes x 16 bytes per 256-byte row), waves take blocks of 4 rows round-robin; scores go
// through LDS (one float per cache row), softmax in float32, the value sum is reduced over
// the 4 row slots of a wave by lane exchange and over the waves through LDS.
// The position is read from device memory, so a captured graph replays with a new one.
// Two dependent rounds of loads: the position with the new query / key / value rows, then the
// rotation's table entries with the cached rows below the position; the new rows are used from
// LDS, so nothing waits for their stores into the cache to be acknowledged.
#include "k3q_common.h"

namespace k3q {
namespace {

constexpr int kHd = 128;
constexpr int kAW = 8;           // waves per workgroup
constexpr int kAT = 64 * kAW;

struct AttnParams {
    const uint16_t *q, *k, *v;      // [B, H, 128] bfloat16 (one position)
    const uint16_t *cos_t, *sin_t;  // [max_len, 128] bfloat16
    const int64_t* pos;             // device: the position of this step
    uint16_t *kc, *vc;              // [B, H, max_len, 128]
    uint16_t* out;                  // [B, H, 128]
    int* oob;                       // device flag, may be null: set to 1 when the position is outside the cache
    int H, max_len;
    float scale;
};

// every lane of a row of 16 gets the row's sum: x ^ 1, x ^ 2, then the other quad of the half row,
// then the other half (the same pairs, in the same order, as a butterfly over 1, 2, 4, 8)
__device__ __forceinline__ float row16_sum(float v) {
    v += dpp_move<0xB1, 0xf>(v);   // quad_perm [1,0,3,2]
    v += dpp_move<0x4E, 0xf>(v);   // quad_perm [2,3,0,1]
    v += dpp_move<0x141, 0xf>(v);  // row_half_mirror
    v += dpp_move<0x140, 0xf>(v);  // row_mirror
    return v;
}

__global__ __launch_bounds__(kAT) void decode_attention(AttnParams p) {
    extern __shared__ __attribute__((aligned(16))) float attn_lds[];
    float* qs = attn_lds;                   // [128] rotated query, pre-scaled
    float* red = qs + kHd;                  // [2 * kAW]
    float* oacc = red + 2 * kAW;            // [kAW][128]
    uint16_t* knew = (uint16_t*)(oacc + kAW * kHd);  // [128] the new key row as it goes into the cache
    uint16_t* vnew = knew + kHd;            // [128] the new value row
    float* sc = (float*)(vnew + kHd);       // [max_len]
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int bh = blockIdx.x;
    // The loads that do not depend on the position go out together with the position itself:
    // the new query / key elements (with their rotate-half partners) and the new value row.
    const int d = tid & (kHd - 1);
    float x = 0.f, sw = 0.f;
    v4u vrow = {0u, 0u, 0u, 0u};
    if (tid < 2 * kHd) {
        const uint16_t* src = (tid < kHd ? p.q : p.k) + (int64_t)bh * kHd;
        x = bf16_bits_to_f32(src[d]);
        sw = bf16_bits_to_f32(src[d ^ (kHd / 2)]);
    } else if (tid < 2 * kHd + 16) {
        vrow = ((const v4u*)(p.v + (int64_t)bh * kHd))[tid - 2 * kHd];
    }
    // A position outside the cache (the torch ops this stands for raise there): nothing is written
    // to the caches, the output rows are zero and the caller's flag is raised.  Every thread reads
    // the same position, so the whole workgroup leaves here before its first barrier.
    const int64_t pos64 = p.pos[0];
    if (pos64 < 0 || pos64 >= p.max_len) {
        if (tid < kHd) p.out[(int64_t)bh * kHd + tid] = 0;
        if (tid == 0 && p.oob) p.oob[0] = 1;
        return;
    }
    const int pos = (int)pos64;
    const int64_t row0 = (int64_t)bh * p.max_len;  // first cache row of this (sequence, head)

    // ---- second round of loads: the rotation's table entries and the cached rows ----
    // Rows 0 ... pos-1 are in the cache already, so their loads need not wait for the new row to be
    // written: row pos itself is taken from LDS below.  Blocks of 4 cache rows go to the waves
    // round-robin; a wave asks for kU blocks of keys at once and -- for its first kU blocks -- for
    // the value rows too, before the softmax, so that the weighted sum finds them in registers
    // (the value rows do not depend on the scores).
    float cs = 0.f, sn = 0.f;
    if (tid < 2 * kHd) {
        cs = bf16_bits_to_f32(p.cos_t[(int64_t)pos * kHd + d]);
        sn = bf16_bits_to_f32(p.sin_t[(int64_t)pos * kHd + d]);
    }
    const int n = pos + 1;
    const int nblk = (n + 3) >> 2;
    const int sub = lane >> 4, dl = (lane & 15) * 8;
    const int last_old = pos > 0 ? pos - 1 : 0;  // a row that is safe to read for lanes without a cached row
    constexpr int kU = 8;
    v4u kk0[kU], vv0[kU];
    if (wave < nblk) {
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (wave + u * kAW) + sub;
            kk0[u] = *(const v4u*)(p.kc + (row0 + (j < pos ? j : last_old)) * kHd + dl);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (wave + u * kAW) + sub;
            vv0[u] = *(const v4u*)(p.vc + (row0 + (j < pos ? j : last_old)) * kHd + dl);
        }
    }

    // ---- rotate q and k; the new rows go to the cache and, for this launch, to LDS ----
    if (tid < 2 * kHd) {
        // the rounding steps of x * cos + swapped * sin evaluated in bfloat16
        const float r = round_bf16(round_bf16(x * cs) + round_bf16(sw * sn));
        if (tid < kHd) {
            qs[d] = r * p.scale;
        } else {
            const uint16_t bits = (uint16_t)f32_to_bf16_bits(r);
            knew[d] = bits;
            p.kc[(row0 + pos) * kHd + d] = bits;
        }
    } else if (tid < 2 * kHd + 16) {
        const int c = tid - 2 * kHd;
        ((v4u*)vnew)[c] = vrow;
        ((v4u*)(p.vc + (row0 + pos) * kHd))[c] = vrow;
    }
    __syncthreads();

    // ---- scores ----
    float qv[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) qv[e] = qs[dl + e];
    float mx = -INFINITY;
    for (int kb0 = wave; kb0 < nblk; kb0 += kAW * kU) {
        v4u kk[kU];
        if (kb0 == wave) {
#pragma unroll
            for (int u = 0; u < kU; ++u) kk[u] = kk0[u];
        } else {
#pragma unroll
            for (int u = 0; u < kU; ++u) {
                const int j = 4 * (kb0 + u * kAW) + sub;
                kk[u] = *(const v4u*)(p.kc + (row0 + (j < pos ? j : last_old)) * kHd + dl);
            }
        }
        float dot[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (kb0 + u * kAW) + sub;
            if (j == pos) kk[u] = *(const v4u*)(knew + dl);
            dot[u] = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                dot[u] += qv[2 * e] * __uint_as_float(kk[u][e] << 16);
                dot[u] += qv[2 * e + 1] * __uint_as_float(kk[u][e] & 0xffff0000u);
            }
        }
        // sum over the 16 lanes of a row, as lane exchanges inside the vector unit (through LDS
        // permutes the kU dependent chains of four exchanges took 2 us of the launch's 8)
#pragma unroll
        for (int u = 0; u < kU; ++u) dot[u] = row16_sum(dot[u]);
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (kb0 + u * kAW) + sub;
            if (j < n) {
                mx = fmaxf(mx, dot[u]);
                if ((lane & 15) == 0) sc[j] = dot[u];
            }
        }
    }
    mx = wave_max(mx);
    if (lane == 0) red[wave] = mx;
    __syncthreads();
    float gmx = red[0];
#pragma unroll
    for (int w = 1; w < kAW; ++w) gmx = fmaxf(gmx, red[w]);

    // ---- softmax numerators ----
    float part = 0.f;
    for (int j = tid; j < n; j += kAT) {
        const float e = __expf(sc[j] - gmx);
        sc[j] = e;
        part += e;
    }
    part = wave_sum(part);
    if (lane == 0) red[kAW + wave] = part;
    __syncthreads();
    float total = 0.f;
#pragma unroll
    for (int w = 0; w < kAW; ++w) total += red[kAW + w];

    // ---- weighted sum of the value rows ----
    float acc[8];
#pragma unroll
    for (int e = 0; e < 8; ++e) acc[e] = 0.f;
    auto add_row = [&](const v4u& vv, const float w) {
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            acc[2 * e] += w * __uint_as_float(vv[e] << 16);
            acc[2 * e + 1] += w * __uint_as_float(vv[e] & 0xffff0000u);
        }
    };
    if (wave < nblk) {
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (wave + u * kAW) + sub;
            if (j == pos) vv0[u] = *(const v4u*)(vnew + dl);
            add_row(vv0[u], j < n ? sc[j] : 0.f);
        }
    }
    for (int kb0 = wave + kAW * kU; kb0 < nblk; kb0 += kAW * kU) {
        v4u vv[kU];
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (kb0 + u * kAW) + sub;
            vv[u] = *(const v4u*)(p.vc + (row0 + (j < pos ? j : last_old)) * kHd + dl);
        }
#pragma unroll
        for (int u = 0; u < kU; ++u) {
            const int j = 4 * (kb0 + u * kAW) + sub;
            if (j == pos) vv[u] = *(const v4u*)(vnew + dl);
            add_row(vv[u], j < n ? sc[j] : 0.f);
        }
    }
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        acc[e] += __shfl_xor(acc[e], 16, kWave);
        acc[e] += __shfl_xor(acc[e], 32, kWave);
    }
    if (lane < 16) {
#pragma unroll
        for (int e = 0; e < 8; ++e) oacc[wave * kHd + dl + e] = acc[e];
    }
    __syncthreads();
    if (tid < kHd) {
        float o = 0.f;
#pragma unroll
        for (int w = 0; w < kAW; ++w) o += oacc[w * kHd + tid];
        p.out[(int64_t)bh * kHd + tid] = (uint16_t)f32_to_bf16_bits(o / total);
    }
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_decode_attention(const void* q, const void* k, const void* v, int dtype, int64_t B,
                                    int64_t H, int64_t head_dim, int64_t max_len, const void* cos_table,
                                    const void* sin_table, const int64_t* pos, void* k_cache,
                                    void* v_cache, void* out, int* oob_flag, void* stream) {
    if (dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (B < 0 || H <= 0 || head_dim != kHd || max_len <= 0 || max_len > 32768 || B * H >= (1 << 30))
        return K3Q_ERR_SHAPE;
    if (B == 0) return K3Q_OK;
    if (!q || !k || !v || !cos_table || !sin_table || !pos || !k_cache || !v_cache || !out) return K3Q_ERR_NULL;
    if (!aligned_to(v, 16) || !aligned_to(k_cache, 16) || !aligned_to(v_cache, 16) || !aligned_to(pos, 8))
        return K3Q_ERR_ALIGN;
    AttnParams p;
    p.q = (const uint16_t*)q;
    p.k = (const uint16_t*)k;
    p.v = (const uint16_t*)v;
    p.cos_t = (const uint16_t*)cos_table;
    p.sin_t = (const uint16_t*)sin_table;
    p.pos = pos;
    p.kc = (uint16_t*)k_cache;
    p.vc = (uint16_t*)v_cache;
    p.out = (uint16_t*)out;
    p.oob = oob_flag;
    p.H = (int)H;
    p.max_len = (int)max_len;
    p.scale = 0.08838834764831845f;  // 1 / sqrt(128)
    const size_t lds = (size_t)(kHd + 2 * kAW + kAW * kHd + kHd + max_len) * sizeof(float);  // as laid out in the kernel
    if (lds > 64 * 1024) {
        static const bool raised = hipFuncSetAttribute((const void*)decode_attention,
                                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                                       160 * 1024) == hipSuccess;
        if (!raised) return K3Q_ERR_LAUNCH;
    }
    decode_attention<<<(unsigned)(B * H), kAT, lds, (hipStream_t)stream>>>(p);
    return launch_status();
}
