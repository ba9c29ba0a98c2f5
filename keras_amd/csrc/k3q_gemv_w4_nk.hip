// Weight-only int4 matmul for decode-sized M with the kernel stored K-contiguous:
//     y[m, n] = sum_k x[m, k] * W[n, k],   W packed as int8 [N, ceil(K/2)], low nibble = even k.
//
// This is the layout of a tied int4 embedding table [vocab, ceil(dim/2)] when it serves as
// the LM head (ReversibleEmbedding._int4_call with reverse=True,
// keras/src/layers/core/reversible_embedding.py:298-381): the reference transposes the
// table, unpacks it along axis 0, de-quantises it to a float [dim, vocab] matrix and
// multiplies.  Here the packed bytes are read once, in place.
//
//   per-row scale (block_size <= 0):  y = T(T(acc) / scale[n])
//   grouped       (block_size  > 0):  y = T(sum_g scale[n, g] * (acc_g - zero[n, g] * sum_g x))
//
// v_mfma_f32_16x16x32_bf16 takes K-contiguous operands as they are: lane (i = lane%16,
// c = lane/16) loads 16 bytes = 32 consecutive k of weight row n0 + i at k0 + 32c; dword j of
// that load feeds MFMA j.  ((w >> 4p) & 0x000F000F) ^ 0x43084308 is the bfloat16 pair
// (136 + nibble p, 136 + nibble p + 4), so slot 2p / 2p+1 of the lane carry k + p / k + p + 4;
// the x operand is permuted to the same slot order (v_perm).  The +136 offset and, grouped,
// the zero point leave through sum_k x, which is accumulated while x is staged.
//
// x (at most 8 rows per pass) is staged once per workgroup in LDS as bfloat16 (float32 x:
// a high and a low bfloat16 part, two MFMAs) together with its per-128-column sums; the 8
// waves of a workgroup then stream 16 weight rows each with nothing but 16-byte loads.
#include "k3q_common.h"

namespace k3q {
namespace {

constexpr u32 kMagicFlip = 0x43084308u;
constexpr u32 kNibblePair = 0x000F000Fu;
constexpr float kOffset = 136.0f;
constexpr int kRows = 8;          // rows of x per pass, at most (fewer when LDS is short)
constexpr int kWaves = 8;         // 16 weight rows each
constexpr int kStep = 128;        // k per MFMA step: 4 lanes x 32 nibbles per row
constexpr int kUnroll = 4;        // steps whose loads are in flight together
constexpr int kLdsBudget = 144 * 1024;

struct NkParams {
    const void* x;        // [M, K]
    const uint8_t* w;     // [N, row_bytes]
    const void* scale;    // [N] or [N, G]
    const int8_t* zero;   // [N, G]
    void* y;              // [M, N]
    int64_t K, N, row_bytes, G;
    int M, m0;
    int rows;             // rows of x staged per pass (<= kRows); LDS holds rows + 1
    int group_steps;      // steps per group (grouped: block_size / 128)
    int round_acc;        // float32 output of a bfloat16 layer: per-row path rounds acc to bfloat16
};

// LDS of the fast kernel: `parts` arrays of (rows + 1) staged rows, then the per-step sums
inline int64_t lds_bytes(int parts, int rows, int64_t K) {
    return (int64_t)parts * (rows + 1) * (K * 2 + 16) + (int64_t)rows * (K / kStep) * 4;
}

template <bool kBF16>
__device__ __forceinline__ float load_s(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

__device__ __forceinline__ v8bf as_bf(const v4u& v) { return __builtin_bit_cast(v8bf, v); }

// LDS: kParts arrays of (rows + 1) rows of (K + 8) bfloat16 (the last row is zeros and
// serves the MFMA columns that have no x row), then sums [rows][nsteps] as float.
template <bool kXF32, bool kScaleBF16, bool kOutBF16, bool kGrouped>
__global__ __launch_bounds__(kWaves * 64) void gemv_w4_nk(NkParams p) {
    extern __shared__ char lds[];
    constexpr int kParts = kXF32 ? 2 : 1;
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int i = lane & 15;
    const int c = lane >> 4;
    const int M = p.M;
    const int64_t K = p.K;
    const int nsteps = (int)(K / kStep);
    const int xstride = (int)(K * 2 + 16);  // bytes per staged row
    const int rows = p.rows;
    const int part_bytes = (rows + 1) * xstride;
    float* sums = (float*)(lds + kParts * part_bytes);  // [rows][nsteps]

    // ---- stage x: bfloat16 rows, zero rows past M, the zero row, per-step sums ----
    {
        const int64_t chunks_per_row = K / 8;  // 8 elements per chunk
        for (int64_t e = tid; e < (rows + 1) * chunks_per_row; e += kWaves * 64) {
            const int row = (int)(e / chunks_per_row);
            const int64_t k = (e - row * chunks_per_row) * 8;
            v4u hi = {0u, 0u, 0u, 0u}, lo = {0u, 0u, 0u, 0u};
            if (row < M && row < rows) {
                if (kXF32) {
                    const float* src = (const float*)p.x + (int64_t)(p.m0 + row) * K + k;
                    const v4u a = *(const v4u*)src, b = *(const v4u*)(src + 4);
                    u32 h[8], l[8];
#pragma unroll
                    for (int t = 0; t < 8; ++t) {
                        const u32 f = t < 4 ? a[t] : b[t - 4];
                        const u32 top = f & 0xffff0000u;
                        h[t] = top >> 16;
                        l[t] = f32_to_bf16_bits(__uint_as_float(f) - __uint_as_float(top));
                    }
#pragma unroll
                    for (int d = 0; d < 4; ++d) {
                        hi[d] = h[2 * d] | (h[2 * d + 1] << 16);
                        lo[d] = l[2 * d] | (l[2 * d + 1] << 16);
                    }
                } else {
                    hi = *(const v4u*)((const uint16_t*)p.x + (int64_t)(p.m0 + row) * K + k);
                }
            }
            *(v4u*)(lds + row * xstride + k * 2) = hi;
            if (kXF32) *(v4u*)(lds + part_bytes + row * xstride + k * 2) = lo;
        }
        __syncthreads();
        // sums of the staged values (what the matrix core will multiply), one thread per (row, step)
        for (int e = tid; e < rows * nsteps; e += kWaves * 64) {
            const int row = e / nsteps, st = e - row * nsteps;
            float acc = 0.f;
            for (int part = 0; part < kParts; ++part) {
                const v4u* src = (const v4u*)(lds + part * part_bytes + row * xstride + st * kStep * 2);
                for (int q = 0; q < kStep / 8; ++q) {
                    const v4u v = src[q];
#pragma unroll
                    for (int d = 0; d < 4; ++d)
                        acc += __uint_as_float(v[d] << 16) + __uint_as_float(v[d] & 0xffff0000u);
                }
            }
            sums[row * nsteps + st] = acc;
        }
        __syncthreads();
    }

    const int64_t n0 = ((int64_t)blockIdx.x * kWaves + wave) * 16;
    if (n0 >= p.N) return;
    int64_t nrow = n0 + i;
    if (nrow >= p.N) nrow = p.N - 1;  // loads stay in bounds; such rows are never stored
    const uint8_t* wrow = p.w + nrow * p.row_bytes + 16 * c;
    // x operand of this lane: row i (the zero row for i >= kRows), k offset 32c
    const char* xlane = lds + (i < rows ? i : rows) * xstride + 64 * c;
    const int srow = i < rows ? i : 0;  // sums row (columns i >= rows are never stored)

    v4f acc = {0.f, 0.f, 0.f, 0.f};
    v4f tot = {0.f, 0.f, 0.f, 0.f};
    float gsum = 0.f;  // sum of x over the steps accumulated in `acc`

    // rows of this lane's four outputs
    int64_t orow[4];
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        orow[r] = n0 + 4 * c + r;
        if (orow[r] >= p.N) orow[r] = p.N - 1;
    }

    // grouped: scale and zero point of (output row r, group of step u), fetched with the
    // batch's weights so that the flush never waits on memory
    float sv[kGrouped ? kUnroll : 1][4], zv[kGrouped ? kUnroll : 1][4];
    auto flush = [&](int u) {
#pragma unroll
        for (int r = 0; r < 4; ++r) {
            tot[r] += sv[u][r] * (acc[r] - (kOffset + zv[u][r]) * gsum);
            acc[r] = 0.f;
        }
        gsum = 0.f;
    };

    for (int s0 = 0; s0 < nsteps; s0 += kUnroll) {
        v4u wv[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int st = s0 + u < nsteps ? s0 + u : nsteps - 1;
            wv[u] = __builtin_nontemporal_load((const v4u*)(wrow + (int64_t)st * (kStep / 2)));
            if (kGrouped) {
                const int64_t g = st / p.group_steps;
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    sv[u][r] = load_s<kScaleBF16>(p.scale, orow[r] * p.G + g);
                    zv[u][r] = (float)p.zero[orow[r] * p.G + g];
                }
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int st = s0 + u;
            if (st >= nsteps) break;
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                v4u av;
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) av[pp] = ((wv[u][j] >> (4 * pp)) & kNibblePair) ^ kMagicFlip;
#pragma unroll
                for (int part = 0; part < kParts; ++part) {
                    const v4u xr = *(const v4u*)(xlane + part * part_bytes + (st * kStep + 8 * j) * 2);
                    // (x0,x1),(x2,x3),(x4,x5),(x6,x7) -> (x0,x4),(x1,x5),(x2,x6),(x3,x7)
                    v4u xb;
                    xb[0] = byte_perm(xr[2], xr[0], 0x05040100u);
                    xb[1] = byte_perm(xr[2], xr[0], 0x07060302u);
                    xb[2] = byte_perm(xr[3], xr[1], 0x05040100u);
                    xb[3] = byte_perm(xr[3], xr[1], 0x07060302u);
                    acc = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(av), as_bf(xb), acc, 0, 0, 0);
                }
            }
            gsum += sums[srow * nsteps + st];
            if (kGrouped && ((st + 1) % p.group_steps == 0 || st == nsteps - 1))
                flush(u);
        }
    }

    // lane holds outputs (m = i, n = n0 + 4c + r)
    if (i >= M || i >= rows) return;
    const int64_t nfirst = n0 + 4 * c;
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        if (nfirst + r >= p.N) continue;
        float v;
        if (kGrouped) {
            v = tot[r];
        } else {
            v = acc[r] - kOffset * gsum;
            const float s = load_s<kScaleBF16>(p.scale, nfirst + r);
            if (kOutBF16) {
                v = round_bf16(v) / s;
            } else {
                if (p.round_acc) v = round_bf16(v);
                v = v / s;
            }
        }
        const int64_t o = (int64_t)(p.m0 + i) * p.N + nfirst + r;
        if (kOutBF16)
            ((uint16_t*)p.y)[o] = (uint16_t)f32_to_bf16_bits(v);
        else
            ((float*)p.y)[o] = v;
    }
}

// Any shape: one thread per output, fp32 FMA chain over K.
template <bool kXF32, bool kScaleBF16, bool kOutBF16, bool kGrouped>
__global__ __launch_bounds__(256) void gemv_w4_nk_generic(NkParams p, int64_t block_size) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (n >= p.N) return;
    const uint8_t* wr = p.w + n * p.row_bytes;
    auto xat = [&](int64_t k) {
        if (kXF32) return ((const float*)p.x)[(int64_t)(p.m0 + m) * p.K + k];
        return bf16_bits_to_f32(((const uint16_t*)p.x)[(int64_t)(p.m0 + m) * p.K + k]);
    };
    auto wat = [&](int64_t k) {
        const u32 byte = wr[k >> 1];
        const u32 nib = (k & 1) ? (byte >> 4) : (byte & 0xfu);
        return (float)((int)(nib ^ 8u) - 8);
    };
    float total = 0.f;
    if (kGrouped) {
        for (int64_t k0 = 0; k0 < p.K; k0 += block_size) {
            const int64_t g = k0 / block_size;
            const float s = load_s<kScaleBF16>(p.scale, n * p.G + g);
            const float z = (float)p.zero[n * p.G + g];
            const int64_t k1 = k0 + block_size < p.K ? k0 + block_size : p.K;
            float acc = 0.f;
            for (int64_t k = k0; k < k1; ++k) acc = fmaf(xat(k), wat(k) - z, acc);
            total = fmaf(acc, s, total);
        }
    } else {
        for (int64_t k = 0; k < p.K; ++k) total = fmaf(xat(k), wat(k), total);
        const float s = load_s<kScaleBF16>(p.scale, n);
        if (kOutBF16)
            total = round_bf16(total) / s;
        else
            total = (p.round_acc ? round_bf16(total) : total) / s;
    }
    const int64_t o = (int64_t)(p.m0 + m) * p.N + n;
    if (kOutBF16)
        ((uint16_t*)p.y)[o] = (uint16_t)f32_to_bf16_bits(total);
    else
        ((float*)p.y)[o] = total;
}

template <bool kXF32, bool kScaleBF16, bool kOutBF16, bool kGrouped>
int run_typed(NkParams p, int64_t M, bool fast, int64_t block_size, hipStream_t s) {
    if (fast) {
        const size_t lds = (size_t)lds_bytes(kXF32 ? 2 : 1, p.rows, p.K);
        static const bool raised = [] {
            return hipFuncSetAttribute((const void*)gemv_w4_nk<kXF32, kScaleBF16, kOutBF16, kGrouped>,
                                       hipFuncAttributeMaxDynamicSharedMemorySize,
                                       kLdsBudget) == hipSuccess;
        }();
        (void)raised;
        const unsigned blocks = (unsigned)((p.N + 16 * kWaves - 1) / (16 * kWaves));
        for (int64_t m0 = 0; m0 < M; m0 += p.rows) {
            p.m0 = (int)m0;
            p.M = (int)(M - m0 < p.rows ? M - m0 : p.rows);
            gemv_w4_nk<kXF32, kScaleBF16, kOutBF16, kGrouped><<<blocks, kWaves * 64, lds, s>>>(p);
        }
    } else {
        for (int64_t m0 = 0; m0 < M; m0 += 65535) {
            p.m0 = (int)m0;
            p.M = (int)(M - m0 < 65535 ? M - m0 : 65535);
            dim3 grid((unsigned)((p.N + 255) / 256), (unsigned)p.M);
            gemv_w4_nk_generic<kXF32, kScaleBF16, kOutBF16, kGrouped><<<grid, 256, 0, s>>>(p, block_size);
        }
    }
    return launch_status();
}

template <bool kGrouped>
int run_grouped(const NkParams& p, int64_t M, int x_dtype, int scale_dtype, bool fast,
                int64_t block_size, hipStream_t s) {
    if (x_dtype == K3Q_F32) {
        if (scale_dtype == K3Q_F32) return run_typed<true, false, false, kGrouped>(p, M, fast, block_size, s);
        return run_typed<true, true, false, kGrouped>(p, M, fast, block_size, s);
    }
    if (scale_dtype == K3Q_F32) return run_typed<false, false, false, kGrouped>(p, M, fast, block_size, s);
    return run_typed<false, true, true, kGrouped>(p, M, fast, block_size, s);
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_gemv_w4_nk(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                              const int8_t* w_packed, const void* scale, int scale_dtype,
                              const int8_t* zero, int64_t block_size, void* y, void* stream) {
    if ((x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) ||
        (scale_dtype != K3Q_F32 && scale_dtype != K3Q_BF16))
        return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!x || !w_packed || !scale || !y) return K3Q_ERR_NULL;
    const bool grouped = block_size > 0;
    if (grouped && !zero) return K3Q_ERR_NULL;
    const bool out_bf16 = x_dtype == K3Q_BF16 && scale_dtype == K3Q_BF16;
    if (!aligned_to(x, x_dtype == K3Q_F32 ? 4 : 2) || !aligned_to(scale, scale_dtype == K3Q_F32 ? 4 : 2) ||
        !aligned_to(y, out_bf16 ? 2 : 4))
        return K3Q_ERR_ALIGN;

    NkParams p{};
    p.x = x;
    p.w = (const uint8_t*)w_packed;
    p.scale = scale;
    p.zero = zero;
    p.y = y;
    p.K = K;
    p.N = N;
    p.row_bytes = (K + 1) / 2;
    p.G = grouped ? (K + block_size - 1) / block_size : 1;
    p.group_steps = grouped ? (int)(block_size / kStep) : 1;
    // float32 result of a bfloat16 input with float32 scales: the reference casts the matmul
    // result to bfloat16 before the (promoting) division
    p.round_acc = (x_dtype == K3Q_BF16 && scale_dtype == K3Q_F32 && !grouped) ? 1 : 0;
    const int parts = x_dtype == K3Q_F32 ? 2 : 1;
    int rows = (int)(M < kRows ? M : kRows);
    while (rows > 1 && lds_bytes(parts, rows, K) > kLdsBudget) --rows;
    p.rows = rows;
    const bool fast = (K % kStep) == 0 && (!grouped || (block_size % kStep) == 0) &&
                      lds_bytes(parts, rows, K) <= kLdsBudget && aligned_to(x, 16) &&
                      aligned_to(w_packed, 16);
    hipStream_t s = (hipStream_t)stream;
    if (grouped) return run_grouped<true>(p, M, x_dtype, scale_dtype, fast, block_size, s);
    return run_grouped<false>(p, M, x_dtype, scale_dtype, fast, block_size, s);
}
