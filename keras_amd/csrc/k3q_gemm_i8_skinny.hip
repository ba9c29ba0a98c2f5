// int8 x int8 -> int32 matmul for decode-sized M (<= 64 rows), with the Dense de-scale.
//
// HBM-bound on the weights, so the int8 kernel is read ONCE, in the [K, N] layout the layer
// stores (no shadow copy), with 16-byte loads that are contiguous along N.  As in the int4
// kernel, the matrix core is fed operands whose "K slots" mix k and n:
//   v_mfma_i32_32x32x32_i8 gives each lane (i = lane%32, g = lane/32) 16 byte-slots of row i.
//   The lane loads 16 bytes (columns n0+16i .. +15) of four consecutive k rows.  MFMA c
//   (c = 0..3) takes dword c of each of the four loads: slot (t, b) of row i is
//   W[k0 + 4g + t][n0 + 16i + 4c + b], i.e. four k values of four different columns.
//   The activation operand has 32 columns = 4 column groups x 8 rows of x; column (bb, m)
//   carries xq[m][k0 + 4g + t] in slot (t, bb) and zero elsewhere, so D[i][(bb, m)] is the
//   exact int32 partial dot product of x row m with column n0 + 16i + 4c + bb.
// Three quarters of the MFMA multiplies zeros; at <= 64 rows the matrix core has an order of
// magnitude of headroom over HBM.
//
// Split-K: as in the int4 kernel (waves of a workgroup through LDS, workgroups through int32
// partials and a second kernel).  Integer partial sums make the result exact whatever the
// split.
#include "k3q_common.h"
#include "k3q_gemm_i8_skinny.h"

namespace k3q {
namespace {

constexpr int kNB = 512;        // columns per workgroup: 32 lanes x 16 bytes
constexpr int kStepK = 8;       // k rows per MFMA step: 2 lane groups x 4 rows
constexpr int kMaxWaves = 8;
constexpr int kRowStride = kNB + 4;  // ints per x row in the LDS slab: the pad spreads rows over banks

struct SkinnyParams {
    const int8_t* xq;      // [M, K]
    const int8_t* w;       // [K, N]
    const void* a_scale;   // T [M] or null
    const void* b_scale;   // T [N] or null
    const void* bias;      // T [N] or null
    int64_t bias_stride;   // elements from one row's bias to the next: 0 (one bias for all rows)
                           // or N (an [M, N] addend, e.g. a residual)
    void* y;               // T [M, N] or null
    int32_t* acc_out;      // [M, N] or null
    int32_t* part;         // [KS, M, N]
    int64_t K, N;
    int M;                 // rows in this launch
    int m0;                // first row of this launch
    int klen;              // rows of K per wave
    int exact;             // bit 1: bfloat16 output; bit 2: round the accumulator to bfloat16 first
};

template <bool kBF16>
__device__ __forceinline__ float load_t(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

// epilogue of one output with its scales and bias already in registers (bias 0 without one)
template <bool kBF16>
__device__ __forceinline__ void finish_vals(const SkinnyParams& p, int m, int64_t n, int acc, float sa,
                                            float sb, float bias) {
    const int64_t row = p.m0 + m;
    if (p.acc_out) p.acc_out[row * p.N + n] = acc;
    if (!p.y) return;
    float r;
    if (kBF16) {
        // decode-sized outputs always take the reference's rounding chain
        r = round_bf16(round_bf16((float)acc) / round_bf16(sb * sa));
        if (p.bias) r = round_bf16(r + bias);
        ((uint16_t*)p.y)[row * p.N + n] = (uint16_t)f32_to_bf16_bits(r);
    } else {
        const float accf = (p.exact & 4) ? round_bf16((float)acc) : (float)acc;
        r = accf / (sb * sa);
        if (p.bias) r = r + bias;
        ((float*)p.y)[row * p.N + n] = r;
    }
}

template <bool kBF16>
__device__ __forceinline__ void finish(const SkinnyParams& p, int m, int64_t n, int acc) {
    const float sa = (p.y && p.a_scale) ? load_t<kBF16>(p.a_scale, p.m0 + m) : 1.0f;
    const float sb = (p.y && p.b_scale) ? load_t<kBF16>(p.b_scale, n) : 1.0f;
    const float bias = (p.y && p.bias) ? load_t<kBF16>(p.bias, (int64_t)(p.m0 + m) * p.bias_stride + n) : 0.0f;
    finish_vals<kBF16>(p, m, n, acc, sa, sb, bias);
}

// kSteps: 8-row steps per chunk.  kSets: 8-row groups of x handled per pass (1 or 2).
template <int kSteps, int kSets>
__global__ __launch_bounds__(kMaxWaves * 64) void gemm_i8_skinny(SkinnyParams p) {
    extern __shared__ int red[];  // [M][kRowStride], all waves add into it
    constexpr int kChunk = kSteps * kStepK;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int nwaves = blockDim.x >> 6;
    const int i = lane & 31;        // weight lane: columns 16i..16i+15; x lane: column (bb, m)
    const int g = lane >> 5;
    const int bb = (lane >> 3) & 3;  // column group of this lane's x operand
    const int mrow = lane & 7;
    const int per_xcd = gridDim.x / 8;
    const int cb = (blockIdx.x % 8) * per_xcd + blockIdx.x / 8;
    const int64_t nb = (int64_t)cb * kNB;
    if (nb >= p.N) return;  // grid.x is padded to a multiple of 8
    const int64_t kw0 = ((int64_t)blockIdx.y * nwaves + wave) * p.klen;
    const int nchunks = p.klen / kChunk;
    const int M = p.M;

    int64_t ncol = nb + 16 * i;
    if (ncol >= p.N) ncol = p.N - 16;  // N % 16 == 0; results of these lanes are never stored
    u32 loff[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) loff[t] = (u32)((4 * g + t) * p.N + ncol);
    u32 xoff[kSets], xmask[kSets];
#pragma unroll
    for (int st = 0; st < kSets; ++st) {
        const int m = mrow + 8 * st;
        xmask[st] = m < M ? 0xffffffffu : 0u;
        xoff[st] = (u32)((m < M ? m : M - 1) * p.K + 4 * g);
    }
    const int8_t* xbase = p.xq + (int64_t)p.m0 * p.K;

    v4u wreg[2][kSteps][4];
    u32 xraw[2][kSteps][kSets];
    auto load_chunk = [&](int b, int c) {
        const int64_t kc = kw0 + (int64_t)c * kChunk;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int64_t ks = kc + kStepK * s;
            const int64_t kk = ks < p.K ? ks : p.K - kStepK;  // K % 8 == 0
            const int8_t* rb = p.w + kk * p.N;
#pragma unroll
            for (int t = 0; t < 4; ++t) wreg[b][s][t] = __builtin_nontemporal_load((const v4u*)(rb + loff[t]));
#pragma unroll
            for (int st = 0; st < kSets; ++st) xraw[b][s][st] = *(const u32*)(xbase + kk + xoff[st]);
        }
    };

    v16i acc[kSets][4];
#pragma unroll
    for (int st = 0; st < kSets; ++st)
#pragma unroll
        for (int c = 0; c < 4; ++c)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[st][c][r] = 0;

    auto compute_chunk = [&](int b, int c) {
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const bool kvalid = kw0 + (int64_t)c * kChunk + kStepK * s < p.K;
            v4i xb[kSets];
#pragma unroll
            for (int st = 0; st < kSets; ++st) {
                const u32 d = xraw[b][s][st] & (kvalid ? xmask[st] : 0u);
#pragma unroll
                for (int t = 0; t < 4; ++t) xb[st][t] = (int)(((d >> (8 * t)) & 0xffu) << (8 * bb));
            }
#pragma unroll
            for (int cc = 0; cc < 4; ++cc) {
                const v4i av = {(int)wreg[b][s][0][cc], (int)wreg[b][s][1][cc], (int)wreg[b][s][2][cc],
                                (int)wreg[b][s][3][cc]};
#pragma unroll
                for (int st = 0; st < kSets; ++st)
                    acc[st][cc] = __builtin_amdgcn_mfma_i32_32x32x32_i8(av, xb[st], acc[st][cc], 0, 0, 0);
            }
        }
    };

    load_chunk(0, 0);
    // the waves of the workgroup meet in one int32 slab through LDS atomic adds: integer sums
    // do not depend on the order, so this stays deterministic
    // (bare barrier after an LDS-only wait: a full __syncthreads would also wait for the
    // loads just issued)
    for (int idx = threadIdx.x; idx < M * kRowStride; idx += blockDim.x) red[idx] = 0;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
#pragma unroll 1
    for (int c = 0; c < nchunks; c += 2) {
        if (c + 1 < nchunks) load_chunk(1, c + 1);
        compute_chunk(0, c);
        if (c + 2 < nchunks) load_chunk(0, c + 2);
        if (c + 1 < nchunks) compute_chunk(1, c + 1);
    }

    // lane (j = lane%32, gq = lane/32) holds D[row 8*(r/4) + 4*gq + r%4][col j]:
    //   column n_local = 16*row + 4*c + j/8,  x row m = j%8 + 8*set
#pragma unroll
    for (int st = 0; st < kSets; ++st) {
        const int m = mrow + 8 * st;
        if (m < M) {
            int* dst = red + m * kRowStride;
#pragma unroll
            for (int c = 0; c < 4; ++c)
#pragma unroll
                for (int r = 0; r < 16; ++r) {
                    const int row = 8 * (r >> 2) + 4 * g + (r & 3);
                    __hip_atomic_fetch_add(dst + 16 * row + 4 * c + bb, acc[st][c][r], __ATOMIC_RELAXED,
                                           __HIP_MEMORY_SCOPE_WORKGROUP);
                }
        }
    }
    __syncthreads();

    const int KS = gridDim.y;
    for (int idx = threadIdx.x; idx < M * (kNB / 4); idx += blockDim.x) {
        const int m = idx / (kNB / 4);
        const int nl = (idx % (kNB / 4)) * 4;
        const v4i sum = *(const v4i*)(red + m * kRowStride + nl);
        const int64_t n = nb + nl;
        if (n < p.N) {  // N % 16 == 0: all four columns in or out
            if (KS == 1) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    if (p.exact & 2)
                        finish<true>(p, m, n + e, sum[e]);
                    else
                        finish<false>(p, m, n + e, sum[e]);
                }
            } else {
                *(v4i*)(p.part + ((int64_t)blockIdx.y * M + m) * p.N + n) = sum;
            }
        }
    }
}

template <bool kBF16>
__global__ __launch_bounds__(256) void gemm_i8_skinny_reduce(SkinnyParams p, int KS) {
    const int64_t n = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const int m = blockIdx.y;
    if (n >= p.N) return;
    // scales and bias first, then eight partials in flight before the first add (left alone,
    // the scheduler pairs every load with its add: one memory round trip per partial)
    const bool want_y = p.y != nullptr;
    u32 sa_raw = 0, sb_raw[4] = {0, 0, 0, 0}, bi_raw[4] = {0, 0, 0, 0};
    if (want_y) {
        if (p.a_scale) sa_raw = load_raw<kBF16>(p.a_scale, p.m0 + m);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (p.b_scale) sb_raw[e] = load_raw<kBF16>(p.b_scale, n + e);
            if (p.bias) bi_raw[e] = load_raw<kBF16>(p.bias, (int64_t)(p.m0 + m) * p.bias_stride + n + e);
        }
    }
    const int32_t* src = p.part + (int64_t)m * p.N + n;
    const int64_t stride = (int64_t)p.M * p.N;
    v4i sum = {0, 0, 0, 0};
    for (int ks = 0; ks < KS; ks += 8) {
        v4i t[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            t[u] = v4i{0, 0, 0, 0};
            if (ks + u < KS) t[u] = *(const v4i*)(src + (ks + u) * stride);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 8; ++u) sum += t[u];
    }
#pragma unroll
    for (int e = 0; e < 4; ++e)
        finish_vals<kBF16>(p, m, n + e, sum[e], p.a_scale ? raw_to_f32<kBF16>(sa_raw) : 1.0f,
                           p.b_scale ? raw_to_f32<kBF16>(sb_raw[e]) : 1.0f, raw_to_f32<kBF16>(bi_raw[e]));
}

// ---- [N, K] kernel layout (K contiguous): tied embedding tables, prepacked kernels ----
//
// v_mfma_i32_16x16x64_i8 takes this layout as it is: lane (i = lane%16, c = lane/16) supplies
// 16 consecutive k bytes (chunk c of a 64-byte step) of weight row n0 + i as the first
// operand and of x row i as the second; D[4c + r][i] is then the int32 dot product of
// weight row n0 + 4c + r with x row i.  A wave owns kTiles tiles of 16 weight rows and walks
// its K slice in batches of kUnroll steps whose loads are all issued before the first MFMA;
// waves never talk to each other (no LDS, no barrier).  K is split over blockIdx.y only when
// N alone gives too few waves; partials are int32 and summed by gemm_i8_skinny_reduce.
constexpr int kNkUnroll = 8;

template <int kTiles>
__global__ __launch_bounds__(256) void gemm_i8_skinny_nk(SkinnyParams p) {
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const int i = lane & 15;
    const int c = lane >> 4;
    const int M = p.M;
    const int64_t n0 = ((int64_t)blockIdx.x * 4 + wave) * (16 * kTiles);
    if (n0 >= p.N) return;
    const int64_t k_begin = (int64_t)blockIdx.y * p.klen;
    int64_t k_end = k_begin + p.klen;
    if (k_end > p.K) k_end = p.K;

    const int8_t* wrow[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
        int64_t n = n0 + 16 * t + i;
        if (n >= p.N) n = p.N - 1;  // loads stay in bounds; these rows are never stored
        wrow[t] = p.w + n * p.K + 16 * c;
    }
    const int8_t* xrow = p.xq + (int64_t)(p.m0 + (i < M ? i : M - 1)) * p.K + 16 * c;
    const u32 xmask = i < M ? 0xffffffffu : 0u;

    v4i acc[kTiles];
#pragma unroll
    for (int t = 0; t < kTiles; ++t) acc[t] = v4i{0, 0, 0, 0};

    // two register buffers of kNkUnroll steps each: the next batch is requested before the
    // current one is consumed, so a wave always has loads in flight
    v4u wv[2][kNkUnroll][kTiles], xv[2][kNkUnroll];
    constexpr int64_t kBatch = 64 * kNkUnroll;
    auto load_batch = [&](int b, int64_t k0) {
#pragma unroll
        for (int u = 0; u < kNkUnroll; ++u) {
            // steps past the slice end re-read the last valid step and meet a zero x operand
            const int64_t k = k0 + 64 * u < k_end ? k0 + 64 * u : k_end - 64;
#pragma unroll
            for (int t = 0; t < kTiles; ++t)
                wv[b][u][t] = __builtin_nontemporal_load((const v4u*)(wrow[t] + k));
            xv[b][u] = *(const v4u*)(xrow + k);
        }
    };
    auto compute_batch = [&](int b, int64_t k0) {
#pragma unroll
        for (int u = 0; u < kNkUnroll; ++u) {
            const u32 m = k0 + 64 * u < k_end ? xmask : 0u;
            const v4u xm = {xv[b][u][0] & m, xv[b][u][1] & m, xv[b][u][2] & m, xv[b][u][3] & m};
#pragma unroll
            for (int t = 0; t < kTiles; ++t)
                acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(
                    __builtin_bit_cast(v4i, wv[b][u][t]), __builtin_bit_cast(v4i, xm), acc[t], 0, 0, 0);
        }
    };
    // Rows are K bytes apart, typically a multiple of every channel interleave, so waves that
    // walk K in step would all sit on the same memory channels at the same time.  Integer
    // sums do not care about order: each wave starts at its own batch and wraps around.
    const int nbatch = (int)((k_end - k_begin + kBatch - 1) / kBatch);
    const int rot = (int)(((int64_t)blockIdx.x * 4 + wave) % nbatch);
    auto batch_k = [&](int j) {
        int r = j + rot;
        if (r >= nbatch) r -= nbatch;
        return k_begin + (int64_t)r * kBatch;
    };
    load_batch(0, batch_k(0));
#pragma unroll 1
    for (int j = 0; j < nbatch; j += 2) {
        if (j + 1 < nbatch) load_batch(1, batch_k(j + 1));
        compute_batch(0, batch_k(j));
        if (j + 2 < nbatch) load_batch(0, batch_k(j + 2));
        if (j + 1 < nbatch) compute_batch(1, batch_k(j + 1));
    }

    // lane holds rows n0 + 16t + 4c + r (r = 0..3) of x row i
    if (i >= M) return;
    const int KS = gridDim.y;
#pragma unroll
    for (int t = 0; t < kTiles; ++t) {
        const int64_t n = n0 + 16 * t + 4 * c;
        if (KS > 1) {
            if (n + 3 < p.N) {
                *(v4i*)(p.part + ((int64_t)blockIdx.y * M + i) * p.N + n) = acc[t];
            } else {
#pragma unroll
                for (int r = 0; r < 4; ++r)
                    if (n + r < p.N) p.part[((int64_t)blockIdx.y * M + i) * p.N + n + r] = acc[t][r];
            }
        } else {
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                if (n + r >= p.N) continue;
                if (p.exact & 2)
                    finish<true>(p, i, n + r, acc[t][r]);
                else
                    finish<false>(p, i, n + r, acc[t][r]);
            }
        }
    }
}

struct NkPlan {
    int tiles;    // 16-row tiles per wave
    int ks;       // K slices (blockIdx.y)
    int64_t klen; // bytes of K per slice, a multiple of 64
};

NkPlan make_nk_plan(int64_t N, int64_t K) {
    NkPlan pl{};
    pl.tiles = 1;
    const int64_t waves = (N + 16 * pl.tiles - 1) / (16 * pl.tiles);
    int64_t ks = 1;
    // aim at >= 2048 waves (8 per CU), keep at least 512 bytes of K per slice
    // (the reduction kernel works on groups of four columns)
    while ((N % 4) == 0 && waves * ks < 2048 && K / (ks * 2) >= 512) ks *= 2;
    int64_t klen = (K / ks + 63) / 64 * 64;
    pl.ks = (int)((K + klen - 1) / klen);
    pl.klen = klen;
    return pl;
}

struct Plan {
    int steps, sets, rows, waves, klen, ks;
};

Plan make_plan(int64_t M, int64_t K, int64_t N) {
    Plan pl{};
    pl.sets = M > 8 ? 2 : 1;
    pl.rows = 8 * pl.sets;
    const int rows_used = (int)(M < pl.rows ? M : pl.rows);
    int steps = pl.sets == 2 ? 2 : 4;
    while (steps > 1 && (K % (steps * kStepK)) != 0) steps >>= 1;
    pl.steps = steps;
    const int chunk = steps * kStepK;
    const int64_t nblocks = (N + kNB - 1) / kNB;
    int waves = kMaxWaves;
    (void)rows_used;
    int64_t klen = K * nblocks / (256 * (int64_t)waves);  // about one workgroup per CU
    klen = klen / chunk * chunk;
    if (klen < chunk) klen = chunk;
    if (klen > K) klen = (K + chunk - 1) / chunk * chunk;
    pl.klen = (int)klen;
    const int64_t slices = (K + klen - 1) / klen;
    while (waves > 1 && waves / 2 >= slices) waves >>= 1;
    pl.waves = waves;
    pl.ks = (int)((slices + waves - 1) / waves);
    return pl;
}

template <int kSets>
void launch_steps(int steps, const SkinnyParams& p, dim3 grid, int threads, size_t lds, hipStream_t s) {
    switch (steps) {
        case 4: gemm_i8_skinny<4, kSets><<<grid, threads, lds, s>>>(p); break;
        case 2: gemm_i8_skinny<2, kSets><<<grid, threads, lds, s>>>(p); break;
        default: gemm_i8_skinny<1, kSets><<<grid, threads, lds, s>>>(p); break;
    }
}

}  // namespace

bool gemm_i8_skinny_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* b) {
    return M > 0 && M <= kSkinnyMaxRows && (N % 16) == 0 && (K % kStepK) == 0 && aligned_to(a, 4) &&
           aligned_to(b, 16);
}

int64_t gemm_i8_skinny_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || M > kSkinnyMaxRows) return 0;
    const Plan pl = make_plan(M, K, N);
    if (pl.ks <= 1) return 0;
    const int64_t rows = M < pl.rows ? M : pl.rows;
    return (int64_t)pl.ks * rows * N * 4;
}

bool gemm_i8_skinny_nk_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* b) {
    return M > 0 && M <= kSkinnyMaxRows && N > 0 && (K % 64) == 0 && aligned_to(a, 16) &&
           aligned_to(b, 16);
}

int64_t gemm_i8_skinny_nk_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || M > kSkinnyMaxRows || (K % 64) != 0) return 0;
    const NkPlan pl = make_nk_plan(N, K);
    if (pl.ks <= 1) return 0;
    return (int64_t)pl.ks * (M < 16 ? M : 16) * N * 4;
}

int gemm_i8_skinny_nk_run(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                          const void* a_scale, const void* b_scale, const void* bias, bool bf16, int flags,
                          void* y, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                          hipStream_t s) {
    SkinnyParams p{};
    p.xq = a;
    p.w = b;
    p.a_scale = a_scale;
    p.b_scale = b_scale;
    p.bias = bias;
    p.y = y;
    p.acc_out = acc_out;
    p.K = K;
    p.N = N;
    p.exact = (bf16 ? 2 : 0) | ((flags & 2) ? 4 : 0);
    const NkPlan pl = make_nk_plan(N, K);
    if (pl.ks > 1) {
        const int64_t need = (int64_t)pl.ks * (M < 16 ? M : 16) * N * 4;
        if (!workspace || workspace_bytes < need) return K3Q_ERR_WORKSPACE;
        if (!aligned_to(workspace, 16)) return K3Q_ERR_ALIGN;
        p.part = (int32_t*)workspace;
    }
    p.klen = (int)pl.klen;
    const int64_t waves = (N + 16 * pl.tiles - 1) / (16 * pl.tiles);
    for (int64_t m0 = 0; m0 < M; m0 += 16) {
        const int rows = (int)((M - m0 < 16) ? M - m0 : 16);
        p.m0 = (int)m0;
        p.M = rows;
        dim3 grid((unsigned)((waves + 3) / 4), (unsigned)pl.ks);
        if (pl.tiles == 2)
            gemm_i8_skinny_nk<2><<<grid, 256, 0, s>>>(p);
        else
            gemm_i8_skinny_nk<1><<<grid, 256, 0, s>>>(p);
        if (pl.ks > 1) {
            dim3 rgrid((unsigned)((N / 4 + 255) / 256), rows);
            if (bf16)
                gemm_i8_skinny_reduce<true><<<rgrid, 256, 0, s>>>(p, pl.ks);
            else
                gemm_i8_skinny_reduce<false><<<rgrid, 256, 0, s>>>(p, pl.ks);
        }
    }
    return launch_status();
}

int gemm_i8_skinny_run(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                       const void* a_scale, const void* b_scale, const void* bias, bool bf16, int flags,
                       void* y, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                       hipStream_t s, bool bias_per_row) {
    SkinnyParams p{};
    p.xq = a;
    p.w = b;
    p.a_scale = a_scale;
    p.b_scale = b_scale;
    p.bias = bias;
    p.bias_stride = (bias && bias_per_row) ? N : 0;
    p.y = y;
    p.acc_out = acc_out;
    p.K = K;
    p.N = N;
    p.exact = (bf16 ? 2 : 0) | ((flags & 2) ? 4 : 0);
    const Plan pl = make_plan(M, K, N);
    const int64_t nblocks = (N + kNB - 1) / kNB;
    const int rows_max = (int)(M < pl.rows ? M : pl.rows);
    if (pl.ks > 1) {
        const int64_t need = (int64_t)pl.ks * rows_max * N * 4;
        if (!workspace || workspace_bytes < need) return K3Q_ERR_WORKSPACE;
        if (!aligned_to(workspace, 16)) return K3Q_ERR_ALIGN;
        p.part = (int32_t*)workspace;
    }
    p.klen = pl.klen;
    for (int64_t m0 = 0; m0 < M; m0 += pl.rows) {
        const int rows = (int)((M - m0 < pl.rows) ? M - m0 : pl.rows);
        p.m0 = (int)m0;
        p.M = rows;
        dim3 grid((unsigned)((nblocks + 7) / 8 * 8), (unsigned)pl.ks);
        const int threads = pl.waves * 64;
        const size_t lds = (size_t)rows * kRowStride * sizeof(int);
        if (rows > 8)
            launch_steps<2>(pl.steps, p, grid, threads, lds, s);
        else
            launch_steps<1>(pl.steps, p, grid, threads, lds, s);
        if (pl.ks > 1) {
            dim3 rgrid((unsigned)((N / 4 + 255) / 256), rows);
            if (bf16)
                gemm_i8_skinny_reduce<true><<<rgrid, 256, 0, s>>>(p, pl.ks);
            else
                gemm_i8_skinny_reduce<false><<<rgrid, 256, 0, s>>>(p, pl.ks);
        }
    }
    return launch_status();
}

}  // namespace k3q
