// Weight-only int4 skinny matmul (decode sizes): y[M,N] = x[M,K] . W4[K,N].
//
// W4 is the Dense int4 kernel exactly as the layer stores it: int8 bytes
// [K, ceil(N/2)], low nibble = even output column, high nibble = odd column.
// The kernel is HBM-bound on those bytes, so the design rule is: every packed
// byte is fetched once, with 16-byte loads that are contiguous along N, goes
// straight into registers, and is never re-laid-out in memory.
//
// How nibbles that are contiguous along N reach a matrix core that wants
// operands contiguous along K:
//   v_mfma_f32_16x16x32_bf16 computes D[i,j] = sum_s A[i,s] * B[s,j] over 32
//   "slots" s.  Lane (i = lane%16, g = lane/16) supplies slots 8g..8g+7 of row
//   i as four dwords of two bf16 each.  A lane loads 16 bytes (32 columns) of
//   four consecutive k rows.  For dword q (8 columns) and nibble position p in
//   0..3, ((w >> 4p) & 0x000F000F) | 0x43004300 is, with no further work, the
//   bf16 pair (128 + nibble p, 128 + nibble p+4): two DIFFERENT output columns
//   of the same k.  Those two values are placed in an even and an odd slot, and
//   the x operand is built so that column j < 8 of B carries x only in even
//   slots and column j >= 8 only in odd slots.  D[i, j<8] is then the partial
//   dot product for column (p), D[i, j>=8] the one for column (p + 4), for row
//   m = j % 8 of x.  Half of the MFMA work multiplies zeros; the matrix core
//   has >3x headroom over HBM here, so that is free, and the conversion costs
//   one VALU op per weight.
//   Nibbles are XOR-ed with 8 first, so the bf16 value is (signed nibble + 136);
//   an extra MFMA against an all-ones A accumulates sum_k x, and the offset is
//   removed as acc - 136 * sum_x (grouped: scale * (acc - (136 + zero) * sum_x)
//   per group, which also folds the zero point).
//
// Split-K: wave w of workgroup (nb, ks) owns `klen` consecutive rows of K for
// the 128 * kVec columns of block nb and walks them in register double-buffered
// chunks of kSteps * 16 rows.  Waves of a workgroup are reduced through LDS,
// workgroups through fp32 partials in `workspace` that a second, tiny kernel
// adds in a fixed order before applying the epilogue: the result does not
// depend on scheduling.  With arrival counters from the caller the second
// kernel is not launched: the workgroup that arrives last at its column
// block's counter sums the partials itself, in the same order (same bits).
// That variant does NOT use device-scope fences -- on this multi-XCD part an
// agent-scope release / acquire is a write-back / invalidate of a whole L2 per
// wave, measured 4-7x slower than the second launch.  It orders the data by
// hand instead: partials are written with write-through stores (sc1), every
// thread waits for the acknowledgement of its own stores (s_waitcnt vmcnt(0)),
// the workgroup's barrier collects those waits, and only then is the arrival
// counted; the last workgroup reads the partials with L2-bypassing loads (sc1).
#include "k3q_common.h"
#include "k3q_gemm_bf16.h"

#include <mutex>

namespace k3q {
namespace {

constexpr u32 kMagicFlip = 0x43084308u;  // bf16 128.0 in both halves, nibble bit 3 flipped
constexpr u32 kNibblePair = 0x000F000Fu;
constexpr u32 kOnes = 0x3F803F80u;
constexpr float kOffset = 136.0f;  // 128 (bf16 magic exponent) + 8 (nibble ^ 8)
constexpr int kMaxWaves = 8;
constexpr int kRedPad = 8;
constexpr int kLdsBudget = 144 * 1024;  // of the 160 KiB a workgroup may use

// gfx9 s_waitcnt immediate for "at most n vector-memory operations outstanding" (loads AND
// stores count in vmcnt on this ISA; expcnt and lgkmcnt are left alone)
constexpr int km_vmcnt(int n) { return (n & 0xF) | ((n >> 4) << 14) | 0x0F70; }

struct GemvParams {
    const void* x;         // [M, K] bf16 or f32
    const uint8_t* w;      // [K, row_bytes]
    const void* scale;     // T [N] or [G, N]
    const int8_t* zero;    // [G, N] or null
    const void* bias;      // T [N] or null
    int64_t bias_stride;   // elements from one row's bias to the next: 0 (one bias for all rows)
                           // or N (an [M, N] addend, e.g. a residual)
    void* y;               // T [M, N]
    float* part;           // [KS, M, N] fp32 partials (KS > 1)
    unsigned* sync;        // arrival counters, one per column block, zero between calls (or null)
    int64_t K, N, row_bytes;
    int M;                 // rows of x in this launch
    int m0;                // first row of x handled by this launch
    int block_size;        // rows of K per group (grouped only)
    int klen;              // rows of K per wave (multiple of the chunk)
    int nwaves;            // waves per workgroup (blockDim.x / 64)
    int per_xcd;           // column blocks per XCD (gridDim.x / 8)
    int ks;                // workgroups along K (gridDim.y)
};

__device__ __forceinline__ v8bf as_bf(const v4u& v) { return __builtin_bit_cast(v8bf, v); }

template <bool kBF16>
__device__ __forceinline__ float load_t(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

// epilogue of Dense._int4_call in the layer dtype T
template <bool kBF16, bool kGrouped>
__device__ __forceinline__ void finish(const GemvParams& p, int m, int64_t n, float sum) {
    float v = sum;
    if (kBF16) {
        v = round_bf16(v);
        if (!kGrouped) v = round_bf16(v / load_t<true>(p.scale, n));
        if (p.bias) v = round_bf16(v + load_t<true>(p.bias, (int64_t)(p.m0 + m) * p.bias_stride + n));
        ((uint16_t*)p.y)[(int64_t)(p.m0 + m) * p.N + n] = (uint16_t)(__float_as_uint(v) >> 16);
    } else {
        if (!kGrouped) v = v / load_t<false>(p.scale, n);
        if (p.bias) v = v + load_t<false>(p.bias, (int64_t)(p.m0 + m) * p.bias_stride + n);
        ((float*)p.y)[(int64_t)(p.m0 + m) * p.N + n] = v;
    }
}

// Partial sums that another workgroup of the same launch reads go around the caches that are
// not coherent across the device (agent-scope accesses), as two 8-byte halves.
__device__ __forceinline__ void store_v4f_device(float* dst, const v4f& v) {
    const v4u b = __builtin_bit_cast(v4u, v);
    __hip_atomic_store((uint64_t*)dst, (uint64_t)b[0] | ((uint64_t)b[1] << 32), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
    __hip_atomic_store((uint64_t*)dst + 1, (uint64_t)b[2] | ((uint64_t)b[3] << 32), __ATOMIC_RELAXED,
                       __HIP_MEMORY_SCOPE_AGENT);
}
template <bool kDevice>
__device__ __forceinline__ v4f load_v4f(const float* src) {
    if (!kDevice) return *(const v4f*)src;
    const uint64_t lo = __hip_atomic_load((const uint64_t*)src, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const uint64_t hi = __hip_atomic_load((const uint64_t*)src + 1, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    const v4u b = {(u32)lo, (u32)(lo >> 32), (u32)hi, (u32)(hi >> 32)};
    return __builtin_bit_cast(v4f, b);
}

// Sum of the KS partials of four adjacent outputs, in one fixed order wherever it is
// computed: four interleaved chains (partial ks goes to chain ks % 4), joined pairwise.
// The loads go out in groups of 16 or 8, then 4 and a remainder, each group in flight as a whole
// before its first add (left alone, the scheduler pairs every load with its add: one memory
// round trip per partial).
template <bool kDevice, int kCount>
__device__ __forceinline__ void add_partials(v4f (&s4)[4], const float* src, int64_t stride) {
    v4f t[kCount];
#pragma unroll
    for (int u = 0; u < kCount; ++u) t[u] = load_v4f<kDevice>(src + u * stride);
    __builtin_amdgcn_sched_barrier(0);
#pragma unroll
    for (int u = 0; u < kCount; ++u) s4[u & 3] += t[u];
}

// kWide: groups of 16 (64 data and 32 address registers: too many inside the main kernel,
// where they cost the per-channel variant its fourth wave per SIMD)
template <bool kDevice, bool kWide>
__device__ __forceinline__ v4f sum_partials(const float* src, int64_t stride, int KS) {
    v4f s4[4];
#pragma unroll
    for (int u = 0; u < 4; ++u) s4[u] = v4f{0.f, 0.f, 0.f, 0.f};
    int ks = 0;
    if (kWide) {
        for (; ks + 16 <= KS; ks += 16) add_partials<kDevice, 16>(s4, src + ks * stride, stride);
    } else {
        for (; ks + 16 <= KS; ks += 8) add_partials<kDevice, 8>(s4, src + ks * stride, stride);
    }
    if (ks + 8 <= KS) {
        add_partials<kDevice, 8>(s4, src + ks * stride, stride);
        ks += 8;
    }
    if (ks + 4 <= KS) {
        add_partials<kDevice, 4>(s4, src + ks * stride, stride);
        ks += 4;
    }
    if (ks < KS) {  // one to three left
        v4f t[3];
#pragma unroll
        for (int u = 0; u < 3; ++u) {
            t[u] = v4f{0.f, 0.f, 0.f, 0.f};
            if (ks + u < KS) t[u] = load_v4f<kDevice>(src + (ks + u) * stride);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 3; ++u) s4[u] += t[u];
    }
    return (s4[0] + s4[1]) + (s4[2] + s4[3]);
}

// finish for four adjacent outputs with the scale and bias loads issued before `sum` is
// needed (`sum` is passed as a callable): in the single-launch K split the loads of the
// partials then overlap them instead of following them.
template <bool kBF16, bool kGrouped, typename SumFn>
__device__ __forceinline__ void finish4_prefetched(const GemvParams& p, int m, int64_t n, SumFn sum_fn) {
    u32 sc_raw[4] = {0, 0, 0, 0}, bi_raw[4] = {0, 0, 0, 0};
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        if (!kGrouped) sc_raw[e] = load_raw<kBF16>(p.scale, n + e);
        if (p.bias) bi_raw[e] = load_raw<kBF16>(p.bias, (int64_t)(p.m0 + m) * p.bias_stride + n + e);
    }
    __builtin_amdgcn_sched_barrier(0);
    const v4f sum = sum_fn();
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        float v = sum[e];
        if (kBF16) {
            v = round_bf16(v);
            if (!kGrouped) v = round_bf16(v / raw_to_f32<true>(sc_raw[e]));
            if (p.bias) v = round_bf16(v + raw_to_f32<true>(bi_raw[e]));
            ((uint16_t*)p.y)[(int64_t)(p.m0 + m) * p.N + n + e] = (uint16_t)(__float_as_uint(v) >> 16);
        } else {
            if (!kGrouped) v = v / raw_to_f32<false>(sc_raw[e]);
            if (p.bias) v = v + raw_to_f32<false>(bi_raw[e]);
            ((float*)p.y)[(int64_t)(p.m0 + m) * p.N + n + e] = v;
        }
    }
}

template <int kVec>
struct Packed {
    u32 d[kVec];
};

template <int kVec>
__device__ __forceinline__ Packed<kVec> load_packed(const uint8_t* p) {
    Packed<kVec> r;
    if (kVec == 2) {
        v2u v = __builtin_nontemporal_load((const v2u*)p);
#pragma unroll
        for (int q = 0; q < kVec; ++q) r.d[q] = v[q];
    } else {
        r.d[0] = __builtin_nontemporal_load((const u32*)p);
    }
    return r;
}

// kVec: dwords (8 columns each) a lane loads per k row; the block is 128*kVec columns.
// kSteps: 16-row K steps per chunk.  kSets: n -> up to 8n rows of bf16 x (n = 1, 2, 4); 2 -> also
// rows of bf16 x, or up to 8 rows of f32 x split into two bf16 parts.
template <int kVec, int kSteps, int kSets, bool kXF32, bool kGrouped>
__device__ __forceinline__ void gemv_w4_body(const GemvParams& p, const int bx, const int by) {
    extern __shared__ float red[];  // [waves][M][kNB + kRedPad]
    // Every kernel argument is fetched now, in one scalar round trip, instead of in four
    // dependent ones spread over the address set-up (0.8 us before the first load otherwise);
    // launch geometry comes with the arguments, not from the dispatch packet.
    asm volatile("" ::"s"(p.x), "s"(p.w), "s"(p.scale), "s"(p.zero), "s"(p.bias), "s"(p.y),
                 "s"(p.part), "s"(p.sync), "s"(p.K), "s"(p.N), "s"(p.row_bytes), "s"(p.M), "s"(p.m0),
                 "s"(p.block_size), "s"(p.klen), "s"(p.nwaves), "s"(p.per_xcd), "s"(p.ks));
    constexpr bool kBF16 = !kXF32;
    constexpr int kAccSets = kXF32 ? 1 : kSets;
    constexpr int kNB = 128 * kVec;
    // LDS row of partial sums: 8 floats of padding put the rows m, m+1, ... that the 16 lanes
    // of a quarter wave store together on disjoint banks (m * 8 + grp * 4 + 0..3)
    constexpr int kRedStride = kNB + kRedPad;
    constexpr int kChunk = kSteps * 16;
    const int lane = threadIdx.x & 63;
    const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform by construction
    const int nwaves = p.nwaves;
    const int i = lane & 15;
    const int g = lane >> 4;
    const int grp = (lane >> 3) & 1;
    const int mrow = lane & 7;
    // Workgroups are dealt round-robin to the 8 XCDs: give each XCD a contiguous range of
    // column blocks, so that blocks which share a 128-byte line of a packed row (kVec == 1)
    // meet in one L2 instead of fetching the line twice.
    const int per_xcd = p.per_xcd;
    const int cb = (bx % 8) * per_xcd + bx / 8;
    const int64_t nb = (int64_t)cb * kNB;
    if (nb >= p.N) return;  // grid.x is padded to a multiple of 8
    const int64_t kw0 = ((int64_t)by * nwaves + wave) * p.klen;
    const int nchunks = p.klen / kChunk;
    const int M = p.M;

    Packed<kVec> wreg[2][kSteps][4];
    constexpr int kRaw = kXF32 ? 1 : kSets;  // raw x loads per step
    v4u xraw[2][kSteps][kRaw];
    int64_t ncol = nb + 8 * kVec * i;
    if (ncol >= p.N) ncol = p.N - 8 * kVec;  // N % (8 * kVec) == 0: stays a valid lane column

    // Addressing: a wave-uniform 64-bit row base per 16-row step plus four per-lane 32-bit
    // byte offsets.  Steps past K (K % 16 == 0) are pointed at the last valid step and get a
    // zero x operand; lane columns past N were pointed at valid columns and are never stored.
    u32 loff[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) loff[t] = (u32)((4 * g + t) * p.row_bytes + (ncol >> 1));
    const int xel = kXF32 ? 4 : 2;
    u32 xoff[kRaw], xmask[kRaw];
#pragma unroll
    for (int r = 0; r < kRaw; ++r) {
        const int m = mrow + 8 * r;
        xmask[r] = m < M ? 0xffffffffu : 0u;
        xoff[r] = (u32)(((m < M ? m : M - 1) * p.K + 4 * g) * xel);  // clamped, masked later
    }
    const char* xbase = (const char*)p.x + (int64_t)p.m0 * p.K * xel;
    auto load_chunk = [&](int b, int c) {
        const int64_t kc = kw0 + (int64_t)c * kChunk;
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int64_t ks = kc + 16 * s;
            const uint8_t* rb = p.w + (ks < p.K ? ks : p.K - 16) * p.row_bytes;
#pragma unroll
            for (int t = 0; t < 4; ++t) wreg[b][s][t] = load_packed<kVec>(rb + loff[t]);
        }
        // raw x values for the same rows; turned into MFMA operands at compute time so that
        // nothing here waits on memory
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            const int64_t ks = kc + 16 * s;
            const char* xs = xbase + (ks < p.K ? ks : 0) * xel;
#pragma unroll
            for (int r = 0; r < kRaw; ++r) {
                if (kXF32) {
                    xraw[b][s][r] = *(const v4u*)(xs + xoff[r]);
                } else {
                    const v2u d = *(const v2u*)(xs + xoff[r]);
                    xraw[b][s][r] = v4u{d[0], d[1], 0u, 0u};
                }
            }
        }
    };

    // B[slot, j] holds x[m(j), k] in even (j < 8) or odd (j >= 8) slots; rows of x past M and
    // steps past K contribute zeros
    auto x_operand = [&](int b, int c, int s, int st) -> v4u {
        const bool kvalid = kw0 + (int64_t)c * kChunk + 16 * s < p.K;
        u32 h[4];
        if (kXF32) {
            const u32 mask = kvalid ? xmask[0] : 0u;
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const u32 f = xraw[b][s][0][t] & mask;
                const u32 hi = f & 0xffff0000u;
                if (st == 0) {
                    h[t] = hi >> 16;
                } else {
                    const float rem = __uint_as_float(f) - __uint_as_float(hi);
                    h[t] = f32_to_bf16_bits(rem);
                }
            }
        } else {
            const u32 mask = kvalid ? xmask[st] : 0u;
            const u32 d0 = xraw[b][s][st][0] & mask, d1 = xraw[b][s][st][1] & mask;
            h[0] = d0 & 0xffffu;
            h[1] = d0 >> 16;
            h[2] = d1 & 0xffffu;
            h[3] = d1 >> 16;
        }
        v4u bv;
#pragma unroll
        for (int t = 0; t < 4; ++t) bv[t] = grp ? (h[t] << 16) : h[t];
        return bv;
    };

    v4f acc[kAccSets][kVec][4];
    v4f accs[kAccSets];
    v4f tot[kGrouped ? kAccSets : 1][kGrouped ? kVec : 1][kGrouped ? 4 : 1];
    auto clear_acc = [&]() {
#pragma unroll
        for (int a = 0; a < kAccSets; ++a) {
            accs[a] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int q = 0; q < kVec; ++q)
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) acc[a][q][pp] = v4f{0.f, 0.f, 0.f, 0.f};
        }
    };
    clear_acc();
    if (kGrouped) {
#pragma unroll
        for (int a = 0; a < kAccSets; ++a)
#pragma unroll
            for (int q = 0; q < kVec; ++q)
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) tot[a][q][pp] = v4f{0.f, 0.f, 0.f, 0.f};
    }
    const v4u ones = {kOnes, kOnes, kOnes, kOnes};

    auto compute_chunk = [&](int b, int c) {
#pragma unroll
        for (int s = 0; s < kSteps; ++s) {
            v4u xb[kSets];
#pragma unroll
            for (int st = 0; st < kSets; ++st) xb[st] = x_operand(b, c, s, st);
#pragma unroll
            for (int st = 0; st < kSets; ++st) {
                const int a = kXF32 ? 0 : st;
                accs[a] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf(ones), as_bf(xb[st]),
                                                                  accs[a], 0, 0, 0);
            }
#pragma unroll
            for (int q = 0; q < kVec; ++q) {
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    v4u av;
                    // (nibble ^ 8) | 0x4300 per half, as one and-xor (v_bitop3_b32)
#pragma unroll
                    for (int t = 0; t < 4; ++t)
                        av[t] = ((wreg[b][s][t].d[q] >> (4 * pp)) & kNibblePair) ^ kMagicFlip;
#pragma unroll
                    for (int st = 0; st < kSets; ++st) {
                        const int a = kXF32 ? 0 : st;
                        acc[a][q][pp] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                            as_bf(av), as_bf(xb[st]), acc[a][q][pp], 0, 0, 0);
                    }
                }
            }
        }
    };

    // lane (j = lane%16, gq = lane/16) holds D[row 4*gq + r][col j]:
    //   column n_local = 8*kVec*(4*gq + r) + 8*q + pp + 4*grp,  x row m = (j % 8) + 8*set
    // grouped: the scales and zero points of the current group are fetched ahead of time (at
    // kernel start / right after the previous flush), so that the flush finds them in
    // registers instead of waiting on memory once per group.
    constexpr int kGq = kGrouped ? kVec : 1;
    constexpr int kGr = kGrouped ? 4 : 1;
    v4u gsc[kGr][kGq];  // four scales: 8 bytes (bf16) or 16 bytes (f32)
    u32 gzp[kGr][kGq];  // four int8 zero points
    const int64_t ngroups = kGrouped ? (p.K + p.block_size - 1) / p.block_size : 1;
    auto load_group = [&](int64_t gi) {
        if (!kGrouped) return;
        if (gi > ngroups - 1) gi = ngroups - 1;
#pragma unroll
        for (int r = 0; r < kGr; ++r) {
#pragma unroll
            for (int q = 0; q < kGq; ++q) {
                int64_t n = nb + 8 * kVec * (4 * g + r) + 8 * q + 4 * grp;
                if (n >= p.N) n = p.N - 4;  // N % 8 == 0: a valid, aligned stand-in, never stored
                const int64_t o = gi * p.N + n;
                gzp[r][q] = *(const u32*)(p.zero + o);
                if (kBF16) {
                    const v2u t = *(const v2u*)((const uint16_t*)p.scale + o);
                    gsc[r][q] = v4u{t[0], t[1], 0u, 0u};
                } else {
                    gsc[r][q] = *(const v4u*)((const float*)p.scale + o);
                }
            }
        }
    };
    // fold this group's scale and zero point into the running totals
    auto flush_group = [&](int64_t gi) {
#pragma unroll
        for (int r = 0; r < kGr; ++r) {
#pragma unroll
            for (int q = 0; q < kGq; ++q) {
                float sc[4], zp[4];
#pragma unroll
                for (int pp = 0; pp < 4; ++pp) {
                    if (kBF16) {
                        const u32 w = gsc[r][q][pp >> 1];
                        sc[pp] = __uint_as_float((pp & 1) ? (w & 0xffff0000u) : (w << 16));
                    } else {
                        sc[pp] = __uint_as_float(gsc[r][q][pp]);
                    }
                    zp[pp] = (float)(int)(int8_t)(gzp[r][q] >> (8 * pp));
                }
#pragma unroll
                for (int a = 0; a < kAccSets; ++a)
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
                        tot[a][q][pp][r] += sc[pp] * (acc[a][q][pp][r] - (kOffset + zp[pp]) * accs[a][r]);
            }
        }
        clear_acc();
        load_group(gi + 1);
    };
    auto after_chunk = [&](int c) {
        if (!kGrouped) return;
        const int64_t kend = kw0 + (int64_t)(c + 1) * kChunk;  // first row after this chunk
        if (kend - kChunk >= p.K) return;                       // chunk entirely past K
        if ((kend % p.block_size) == 0 || c == nchunks - 1 || kend >= p.K)
            flush_group((kend - 1 < p.K ? kend - 1 : p.K - 1) / p.block_size);
    };

    load_chunk(0, 0);
    if (kGrouped) load_group((kw0 < p.K ? kw0 : p.K - 1) / p.block_size);
#pragma unroll 1
    for (int c = 0; c < nchunks; c += 2) {
        if (c + 1 < nchunks) load_chunk(1, c + 1);
        compute_chunk(0, c);
        after_chunk(c);
        if (c + 2 < nchunks) load_chunk(0, c + 2);
        if (c + 1 < nchunks) {
            compute_chunk(1, c + 1);
            after_chunk(c + 1);
        }
    }

    // ---- remove the +136 offset (per-channel) and park this wave's partial in LDS ----
#pragma unroll
    for (int a = 0; a < kAccSets; ++a) {
        const int m = mrow + 8 * a;
        if (m < M) {
            float* dst = red + ((size_t)wave * M + m) * kRedStride;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
#pragma unroll
                for (int q = 0; q < kVec; ++q) {
                    const int nl = 8 * kVec * (4 * g + r) + 8 * q + 4 * grp;
                    v4f o;
#pragma unroll
                    for (int pp = 0; pp < 4; ++pp)
                        o[pp] = kGrouped ? tot[a][q][pp][r] : acc[a][q][pp][r] - kOffset * accs[a][r];
                    *(v4f*)(dst + nl) = o;
                }
            }
        }
    }
    __syncthreads();

    // ---- reduce the waves of this workgroup, four columns per thread ----
    const int KS = p.ks;
    for (int idx = threadIdx.x; idx < M * (kNB / 4); idx += nwaves * 64) {
        const int m = idx / (kNB / 4);
        const int nl = (idx % (kNB / 4)) * 4;
        v4f sum = {0.f, 0.f, 0.f, 0.f};
        for (int w = 0; w < nwaves; ++w) sum += *(const v4f*)(red + ((size_t)w * M + m) * kRedStride + nl);
        const int64_t n = nb + nl;
        if (n < p.N) {  // N % 8 == 0 on this path: all four columns in or out
            if (KS == 1) {
#pragma unroll
                for (int e = 0; e < 4; ++e) finish<kBF16, kGrouped>(p, m, n + e, sum[e]);
            } else {
                float* dst = p.part + ((int64_t)by * M + m) * p.N + n;
                if (p.sync) store_v4f_device(dst, sum);
                else *(v4f*)dst = sum;
            }
        }
    }
    // ---- K split finished in this launch ----
    // The workgroup that arrives last at its column block's counter sums the KS partials (in
    // the order of the split, whoever comes last) and applies the epilogue; it leaves the
    // counter at zero for the next call.
    if (KS == 1 || p.sync == nullptr) return;
    // The partials were stored write-through (sc1), around the caches that are not coherent
    // across the device; a store leaves vmcnt only when the memory side has acknowledged it.
    // Every thread waits for its own stores here, explicitly: a workgroup-scope release fence
    // does NOT wait for vector-memory stores on this target (it only orders LDS), and a
    // device-scope release would write back the whole L2 once per wave (54 us per call
    // instead of 12).  The barrier then joins the waits of all threads, and only after it is
    // the arrival counted, so the counter cannot run ahead of any partial of this workgroup.
    __builtin_amdgcn_s_waitcnt(km_vmcnt(0));
    asm volatile("" ::: "memory");
    __syncthreads();
    int* flag = (int*)red;
    if (threadIdx.x == 0) flag[0] = atomicAdd(p.sync + cb, 1u) == (unsigned)(KS - 1);
    __syncthreads();
    const bool last = flag[0] != 0;
    if (!last) return;
    __builtin_amdgcn_fence(__ATOMIC_ACQUIRE, "workgroup");  // no load below moves above the count
    const int items = M * (kNB / 4);
    for (int idx = threadIdx.x; idx < items; idx += nwaves * 64) {
        const int m = idx / (kNB / 4);
        const int64_t n = nb + (idx % (kNB / 4)) * 4;
        if (n >= p.N) continue;
        finish4_prefetched<kBF16, kGrouped>(p, m, n, [&]() {
            return sum_partials<true, false>(p.part + (int64_t)m * p.N + n, (int64_t)M * p.N, KS);
        });
    }
    if (threadIdx.x == 0) atomicExch(p.sync + cb, 0u);
}

template <int kVec, int kSteps, int kSets, bool kXF32, bool kGrouped>
__global__ __launch_bounds__(kMaxWaves * 64) void gemv_w4_mfma(GemvParams p) {
    gemv_w4_body<kVec, kSteps, kSets, kXF32, kGrouped>(p, blockIdx.x, blockIdx.y);
}

// Several kernels against one x in one launch (the query / key / value projections of an
// attention block, the gate / up projections of a gated MLP): the column blocks of the
// problems lie side by side along blockIdx.x, each problem with its own operands, partials
// and arrival counters; the K split (blockIdx.y) is the largest of theirs.
constexpr int kMaxProblems = 4;
struct GemvMulti {
    GemvParams p[kMaxProblems];
    int first[kMaxProblems + 1];  // first blockIdx.x of each problem (multiples of 8), then the end
    int count;
};

template <int kVec, int kSteps, int kSets, bool kXF32, bool kGrouped>
__global__ __launch_bounds__(kMaxWaves * 64) void gemv_w4_mfma_multi(GemvMulti mp) {
    const int bx = blockIdx.x;
    int i = 0;
    while (i + 1 < mp.count && bx >= mp.first[i + 1]) ++i;
    const GemvParams& p = mp.p[i];
    if ((int)blockIdx.y >= p.ks) return;
    gemv_w4_body<kVec, kSteps, kSets, kXF32, kGrouped>(p, bx - mp.first[i], blockIdx.y);
}

// Second pass when K is split over workgroups: sum the KS partials of every output in a
// fixed order and apply the epilogue.  A kernel boundary is the cheapest device-wide
// ordering point between the partial stores and these loads.
template <bool kBF16, bool kGrouped>
__global__ __launch_bounds__(256) void gemv_w4_reduce(GemvParams p, int KS) {
    const int64_t n = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;
    const int m = blockIdx.y;
    if (n >= p.N) return;
    finish4_prefetched<kBF16, kGrouped>(p, m, n, [&]() {
        return sum_partials<false, true>(p.part + (int64_t)m * p.N + n, (int64_t)p.M * p.N, KS);
    });
}

// Any shape: one thread per output, fp32 FMA chain over K.  Used when N is not a
// multiple of 8, K not a multiple of 16, or the group size does not tile.
template <bool kBF16, bool kGrouped>
__global__ __launch_bounds__(256) void gemv_w4_generic(GemvParams p) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int m = blockIdx.y;
    if (n >= p.N) return;
    const int shift = (n & 1) ? 4 : 0;
    const uint8_t* wp = p.w + (n >> 1);
    float total = 0.f;
    if (kGrouped) {
        for (int64_t k0 = 0; k0 < p.K; k0 += p.block_size) {
            const int64_t gi = k0 / p.block_size;
            const float sc = load_t<kBF16>(p.scale, gi * p.N + n);
            const float zp = (float)p.zero[gi * p.N + n];
            float acc = 0.f;
            const int64_t k1 = (k0 + p.block_size < p.K) ? k0 + p.block_size : p.K;
            for (int64_t k = k0; k < k1; ++k) {
                const int u = (wp[k * p.row_bytes] >> shift) & 0xF;
                const float wv = (float)((u ^ 8) - 8) - zp;
                acc = fmaf(load_t<kBF16>(p.x, (int64_t)(p.m0 + m) * p.K + k), wv, acc);
            }
            total = fmaf(acc, sc, total);
        }
    } else {
        for (int64_t k = 0; k < p.K; ++k) {
            const int u = (wp[k * p.row_bytes] >> shift) & 0xF;
            total = fmaf(load_t<kBF16>(p.x, (int64_t)(p.m0 + m) * p.K + k), (float)((u ^ 8) - 8), total);
        }
    }
    finish<kBF16, kGrouped>(p, m, n, total);
}

// Prefill-sized M: the packed kernel is de-quantised once per call into a bfloat16 [N, K]
// scratch matrix (K contiguous, what the MFMA GEMM consumes) and the product runs on the
// matrix cores at full tile size.  Per-channel: the scratch holds the plain nibble values
// (exact) and the GEMM epilogue divides by the scale, as the reference's matmul + divide does;
// grouped: it holds T((w - zero) * scale), rounded to bfloat16 per weight exactly as the
// reference's de-quantised kernel is.
constexpr int kDqK = 64;    // tile of a workgroup: 64 rows of K x 256 columns, so that both the
constexpr int kDqN = 256;   // packed rows read and the [n][k] rows written are whole 128-byte lines
constexpr int kDqRouteK = 128, kDqRouteN = 64;  // shapes the route takes: K % 128 == 0, N % 64 == 0

// kF32 = false: bfloat16 scales, out[N][K] = T(w) or T((w - zero) * scale), rounded per weight
// exactly as the reference's de-quantised kernel is.
// kF32 = true: float32 scales, output rows of `parts` segments of K values for the float32
// route below: [w | w] (per-channel, exact) or [wh | wh | wl] of w = (nibble - zero) * scale.
//
// Phase 1, thread = (row pair rp, 32-column chunk c): two 16-byte loads (rows 2rp, 2rp + 1),
// each column's pair of values packed into one dword and written to the LDS tile [n][k]
// (128 bytes of k per column, 16-byte chunks XOR-swizzled by the column so that phase 2's
// reads spread over the banks).  Phase 2, thread = (column, 16-byte chunk of k): eight lanes
// store one 128-byte piece of an output row.
template <bool kGrouped, bool kF32>
__global__ __launch_bounds__(256) void dequant_w4_nk(const uint8_t* __restrict__ w,
                                                     const void* __restrict__ scale,
                                                     const int8_t* __restrict__ zero,
                                                     uint16_t* __restrict__ out, int64_t K, int64_t N,
                                                     int block_size) {
    constexpr bool kLow = kGrouped && kF32;  // a low part exists
    constexpr int kParts = kF32 ? (kGrouped ? 3 : 2) : 1;
    __shared__ __attribute__((aligned(16))) u32 thi[kDqN * 32];
    __shared__ __attribute__((aligned(16))) u32 tlo[kLow ? kDqN * 32 : 4];
    const int64_t k0 = (int64_t)blockIdx.y * kDqK;
    const int64_t n0 = (int64_t)blockIdx.x * kDqN;
    {
        const int rp = threadIdx.x & 31, c = threadIdx.x >> 5;
        const int64_t k = k0 + 2 * rp, n = n0 + 32 * c;
        if (n < N) {  // N % 32 == 0: a chunk is inside or outside as a whole
            const v4u p0 = *(const v4u*)(w + k * (N / 2) + n / 2);
            const v4u p1 = *(const v4u*)(w + (k + 1) * (N / 2) + n / 2);
            const int64_t g = kGrouped ? k / block_size : 0;  // block_size is even: one group for both rows
#pragma unroll
            for (int q = 0; q < 4; ++q) {
                float sc[8], zp[8];
                if (kGrouped) {
                    const v2u zv = *(const v2u*)(zero + g * N + n + 8 * q);
#pragma unroll
                    for (int e = 0; e < 8; ++e) zp[e] = (float)(int)(int8_t)(zv[e >> 2] >> (8 * (e & 3)));
                    if (kF32) {
                        const v4f s0 = *(const v4f*)((const float*)scale + g * N + n + 8 * q);
                        const v4f s1 = *(const v4f*)((const float*)scale + g * N + n + 8 * q + 4);
#pragma unroll
                        for (int e = 0; e < 4; ++e) {
                            sc[e] = s0[e];
                            sc[4 + e] = s1[e];
                        }
                    } else {
                        const v4u sv = *(const v4u*)((const uint16_t*)scale + g * N + n + 8 * q);
#pragma unroll
                        for (int d = 0; d < 4; ++d) {
                            sc[2 * d] = __uint_as_float(sv[d] << 16);
                            sc[2 * d + 1] = __uint_as_float(sv[d] & 0xffff0000u);
                        }
                    }
                }
#pragma unroll
                for (int e = 0; e < 8; ++e) {
                    // low nibble = even column; sign-extended 4-bit field
                    float v0 = (float)(int)__builtin_amdgcn_sbfe((int)p0[q], 4 * e, 4);  // the builtin's type is unsigned
                    float v1 = (float)(int)__builtin_amdgcn_sbfe((int)p1[q], 4 * e, 4);
                    if (kGrouped) {  // the difference is exact, the product rounds once
                        v0 = (v0 - zp[e]) * sc[e];
                        v1 = (v1 - zp[e]) * sc[e];
                    }
                    const int nl = 32 * c + 8 * q + e;
                    const int at = nl * 32 + (rp ^ (((nl >> 1) & 7) << 2));
                    if (kLow) {
                        const u32 t0 = __float_as_uint(v0) & 0xffff0000u, t1 = __float_as_uint(v1) & 0xffff0000u;
                        thi[at] = (t0 >> 16) | t1;
                        tlo[at] = pack_bf16x2(v0 - __uint_as_float(t0), v1 - __uint_as_float(t1));
                    } else {
                        thi[at] = pack_bf16x2(v0, v1);
                    }
                }
            }
        }
    }
    __syncthreads();
#pragma unroll
    for (int i = 0; i < 8; ++i) {
        const int nl = (threadIdx.x >> 3) + 32 * i, j = threadIdx.x & 7;
        if (n0 + nl >= N) continue;
        const int at = nl * 32 + ((j ^ ((nl >> 1) & 7)) << 2);
        const v4u hi = *(const v4u*)(thi + at);
        uint16_t* dst = out + (n0 + nl) * kParts * K + k0 + 8 * j;
        *(v4u*)dst = hi;
        if (kF32) *(v4u*)(dst + K) = hi;
        if (kLow) *(v4u*)(dst + 2 * K) = *(const v4u*)(tlo + at);
    }
}

// Below this the 16-row decode passes are faster (K = N = 4096: 51 us at 64 rows; at 128 rows
// the passes take 96 us, de-quantise + GEMM 67 us).
// ---- float32 inputs on the same route -------------------------------------------------
// A float32 value is the sum of two bfloat16 values to 2^-17: hi = its top 16 bits, lo = the
// rounded remainder.  With x = xh + xl and w = wh + wl,  x.w = xh.wh + xl.wh + xh.wl (+ 2^-18),
// which is ONE bfloat16 GEMM over a K axis of three segments: a = [xh | xl | xh],
// b = [wh | wh | wl].  Per-channel kernels are small integers (wl = 0): two segments.
__global__ __launch_bounds__(256) void split_f32_rows(const float* __restrict__ x,
                                                      uint16_t* __restrict__ out, int64_t M,
                                                      int64_t K, int parts) {
    const int64_t i = ((int64_t)blockIdx.x * 256 + threadIdx.x) * 4;  // 4 elements per thread
    if (i >= M * K) return;
    const int64_t m = i / K, k = i - m * K;
    const v4u f = *(const v4u*)(x + i);
    u32 hi[4], lo[4];
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const u32 top = f[e] & 0xffff0000u;
        hi[e] = top >> 16;
        lo[e] = f32_to_bf16_bits(__uint_as_float(f[e]) - __uint_as_float(top));
    }
    const v2u h2 = {hi[0] | (hi[1] << 16), hi[2] | (hi[3] << 16)};
    const v2u l2 = {lo[0] | (lo[1] << 16), lo[2] | (lo[3] << 16)};
    uint16_t* row = out + m * parts * K + k;
    *(v2u*)row = h2;
    *(v2u*)(row + K) = l2;
    if (parts == 3) *(v2u*)(row + 2 * K) = h2;
}

// From here on the route wins: the row passes cost per 32 rows (bfloat16; K = N = 4096: 17 us
// each) or per 8 rows (float32: 10 us each), the route's cost is nearly flat in M up to a few
// hundred rows (the de-quantisation of the whole kernel, and a GEMM that splits K while its
// tiles are few): 31 us at 128 bfloat16 rows, 56 us at 128 float32 rows.
// The float32 route writes six bytes per weight before its GEMM starts, so on large kernels
// it needs more rows to win (4096 x 14336: 167 us flat against 2.1 us per row in passes).
constexpr int64_t kGemmMinRowsBF16 = 65, kGemmMinRowsF32 = 48, kGemmMinRowsF32Large = 80;

inline bool gemm_route_ok(bool f32, int64_t M, int64_t K, int64_t N) {
    const int64_t min_rows = !f32 ? kGemmMinRowsBF16
                                  : (K * N > (int64_t(1) << 25) ? kGemmMinRowsF32Large : kGemmMinRowsF32);
    return M >= min_rows && (K % kDqRouteK) == 0 && (N % kDqRouteN) == 0;
}

// scratch of the GEMM route: the de-quantised kernel and, for float32 inputs, the split rows
inline int64_t gemm_route_bytes(bool f32, bool grouped, int64_t M, int64_t K, int64_t N) {
    if (!f32) return N * K * 2;
    const int64_t parts = grouped ? 3 : 2;
    return (N + M) * parts * K * 2;
}

// what the GEMM itself may use beyond that (partials of a K split)
inline int64_t gemm_route_extra_bytes(bool f32, bool grouped, int64_t M, int64_t K, int64_t N) {
    const int64_t parts = f32 ? (grouped ? 3 : 2) : 1;
    return gemm_bf16_nk_workspace_bytes(M, N, parts * K);
}

struct Plan {
    bool fast;
    int vec;     // dwords per lane per k row
    int steps;   // 16-row steps per chunk
    int sets;
    int rows;    // rows of x per launch
    int waves;   // waves per workgroup
    int klen;    // rows of K per wave
    int ks;      // workgroups along K
};

constexpr int kTargetWorkgroups = 256;  // one per CU


// plan_override (may be null): {vec, steps, waves, klen}; entries <= 0 keep the heuristic.
Plan make_plan(int x_dtype, int64_t M, int64_t K, int64_t N, int64_t block_size,
               const int* plan_override) {
    Plan pl{};
    const bool grouped = block_size > 0;
    pl.fast = (N % 8) == 0 && (K % 16) == 0 && (!grouped || block_size % 16 == 0);
    if (!pl.fast) return pl;
    const bool f32 = x_dtype == K3Q_F32;
    // rows of x per pass: 8 per row set; bfloat16 takes up to four sets (32 rows), so that
    // 17..127 rows need a half to a quarter of the passes over the kernel
    pl.rows = f32 ? 8 : (M > 16 ? 32 : M > 8 ? 16 : 8);
    pl.sets = f32 ? 2 : pl.rows / 8;
    const int rows_used = (int)(M < pl.rows ? M : pl.rows);

    // Measured on MI355X at K = N = 8192: 8 waves per workgroup, 8-byte loads per lane and
    // one or two workgroups per CU beat wider loads and finer K splits.  Narrow or small
    // kernels (N <= 4096, or under 2^25 weights) do better with 4-byte loads, i.e. twice the
    // column blocks and half the K split (Llama-7B-sized decoder step: 4.91 -> 4.76 ms).
    int vec = ((grouped && pl.sets == 2) || pl.sets == 4) ? 1 : 2;
    if (vec == 2 && (N <= 4096 || N * K < ((int64_t)1 << 25))) vec = 1;
    if (plan_override && plan_override[0] > 0) vec = plan_override[0];
    while (vec > 1 && (N % (8 * vec)) != 0) vec >>= 1;
    if (vec != 1 && vec != 2) vec = vec > 2 ? 2 : 1;  // 16-byte loads per lane lost every sweep
    if (pl.sets == 4) vec = 1;                       // the only width built for four row sets
    pl.vec = vec;

    int steps = 2;
    if (plan_override && plan_override[1] > 0) steps = plan_override[1];
    if (steps != 1 && steps != 2) steps = 2;
    if ((K % 32) != 0 || (grouped && (block_size % 32) != 0)) steps = 1;
    if (grouped && pl.sets == 4) steps = 1;  // two steps would spill registers
    pl.steps = steps;
    const int chunk = steps * 16;

    const int nb_cols = 128 * vec;
    const int64_t nblocks = (N + nb_cols - 1) / nb_cols;
    int waves = kMaxWaves;
    while (waves > 1 && (int64_t)waves * rows_used * (nb_cols + kRedPad) * 4 > kLdsBudget) waves >>= 1;
    if (plan_override && plan_override[2] > 0 && plan_override[2] <= waves) waves = plan_override[2];

    // rows of K per wave: the slice length that gives about one workgroup per CU
    // Per-channel scales and one row set: two workgroups per CU, so that one workgroup's
    // cross-wave reduction overlaps the other's loads (11.4 vs 12.8 us at M = 1).
    const int target = (!grouped && pl.sets == 1) ? 2 * kTargetWorkgroups : kTargetWorkgroups;
    int64_t klen = K * nblocks / ((int64_t)target * waves);
    klen = klen / chunk * chunk;
    if (klen < chunk) klen = chunk;
    // at least two chunks per wave (so that loads and MFMAs overlap) while that still leaves
    // one workgroup per CU
    if (!grouped && klen < 2 * chunk && K * nblocks / (2 * chunk * (int64_t)waves) >= kTargetWorkgroups)
        klen = 2 * chunk;
    if (grouped) {
        // a slice that straddles group boundaries pays an extra flush per wave: snap to a
        // multiple of the group size, or to a fraction of it (14 us instead of 21 us at
        // K = 4096, N = 14336, where the formula above gives 96 rows for groups of 128)
        if (4 * klen >= 3 * block_size) {
            klen = (klen + block_size / 2) / block_size * block_size;
        } else {
            int64_t frac = block_size;
            while (frac / 2 >= chunk && (frac / 2) % chunk == 0 && 3 * (frac / 2) >= 2 * klen &&
                   frac > klen)
                frac /= 2;
            klen = frac;
        }
    }
    if (target == kTargetWorkgroups) {
        // a few workgroups more than CUs run as a second round on some CUs and hold the launch
        // back (weights cold in HBM; K = 4096, N = 11008, groups of 128: 16.4 us, 12.1 us once
        // the launch fits one round; K = 5120, N = 13824: 21.4 / 18.0): lengthen the slices
        const int64_t step = grouped ? (klen >= block_size ? block_size : klen) : chunk;
        auto workgroups = [&](int64_t kl) {
            const int64_t slices = (K + kl - 1) / kl;
            return nblocks * ((slices + waves - 1) / waves);
        };
        while (workgroups(klen) > kTargetWorkgroups && workgroups(klen) < 7 * kTargetWorkgroups / 4 &&
               klen + step <= K)
            klen += step;
    }
    if (plan_override && plan_override[3] > 0) klen = (plan_override[3] + chunk - 1) / chunk * chunk;
    if (klen > K) klen = (K + chunk - 1) / chunk * chunk;
    pl.klen = (int)klen;
    const int64_t slices = (K + klen - 1) / klen;
    while (waves > 1 && waves / 2 >= slices) waves >>= 1;
    pl.waves = waves;
    pl.ks = (int)((slices + waves - 1) / waves);
    return pl;
}

// `multi` (may be null): the multi-problem launch; otherwise `p` alone
template <int kVec, int kSteps, int kSets, bool kXF32>
void launch4(const GemvParams& p, const GemvMulti* multi, bool grouped, dim3 grid, int threads,
             size_t lds, hipStream_t s) {
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    static const bool raised = [] {
        bool ok = true;
        const void* kernels[4] = {
            (const void*)gemv_w4_mfma<kVec, kSteps, kSets, kXF32, true>,
            (const void*)gemv_w4_mfma<kVec, kSteps, kSets, kXF32, false>,
            (const void*)gemv_w4_mfma_multi<kVec, kSteps, kSets, kXF32, true>,
            (const void*)gemv_w4_mfma_multi<kVec, kSteps, kSets, kXF32, false>};
        for (const void* k : kernels)
            ok = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, kLdsBudget) ==
                     hipSuccess && ok;
        return ok;
    }();
    (void)raised;
    if (multi) {
        if (grouped)
            gemv_w4_mfma_multi<kVec, kSteps, kSets, kXF32, true><<<grid, threads, lds, s>>>(*multi);
        else
            gemv_w4_mfma_multi<kVec, kSteps, kSets, kXF32, false><<<grid, threads, lds, s>>>(*multi);
    } else if (grouped) {
        gemv_w4_mfma<kVec, kSteps, kSets, kXF32, true><<<grid, threads, lds, s>>>(p);
    } else {
        gemv_w4_mfma<kVec, kSteps, kSets, kXF32, false><<<grid, threads, lds, s>>>(p);
    }
}

template <int kVec, int kSteps>
void launch2(int sets, bool f32, const GemvParams& p, const GemvMulti* multi, bool grouped, dim3 grid,
             int threads, size_t lds, hipStream_t s) {
    if (f32) {
        launch4<kVec, kSteps, 2, true>(p, multi, grouped, grid, threads, lds, s);
    } else if (sets == 4) {
        // four row sets only with 4-byte loads per lane (register budget)
        if constexpr (kVec == 1) launch4<1, kSteps, 4, false>(p, multi, grouped, grid, threads, lds, s);
    } else if (sets == 2) {
        launch4<kVec, kSteps, 2, false>(p, multi, grouped, grid, threads, lds, s);
    } else {
        launch4<kVec, kSteps, 1, false>(p, multi, grouped, grid, threads, lds, s);
    }
}

void launch_plan(const Plan& pl, int sets, bool f32, const GemvParams& p, const GemvMulti* multi,
                 bool grouped, dim3 grid, int threads, size_t lds, hipStream_t s) {
    const int key = pl.vec * 10 + pl.steps;
    switch (key) {
        case 22: launch2<2, 2>(sets, f32, p, multi, grouped, grid, threads, lds, s); break;
        case 21: launch2<2, 1>(sets, f32, p, multi, grouped, grid, threads, lds, s); break;
        case 12: launch2<1, 2>(sets, f32, p, multi, grouped, grid, threads, lds, s); break;
        default: launch2<1, 1>(sets, f32, p, multi, grouped, grid, threads, lds, s); break;
    }
}

int run_gemv_w4(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N, const void* w_packed,
                const void* scale, const void* zero, int64_t block_size, const void* bias, void* y,
                void* workspace, int64_t workspace_bytes, const int* plan_override, void* counters,
                int64_t counters_bytes, hipStream_t s, bool bias_per_row = false) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!x || !w_packed || !scale || !y) return K3Q_ERR_NULL;
    const bool grouped = block_size > 0;
    if (grouped && !zero) return K3Q_ERR_NULL;
    const bool f32 = x_dtype == K3Q_F32;
    const size_t el = f32 ? 4 : 2;
    if (!aligned_to(x, el) || !aligned_to(scale, el) || !aligned_to(y, el) ||
        (bias && !aligned_to(bias, el)))
        return K3Q_ERR_ALIGN;

    GemvParams p{};
    p.x = x;
    p.w = (const uint8_t*)w_packed;
    p.scale = scale;
    p.zero = (const int8_t*)zero;
    p.bias = bias;
    p.bias_stride = (bias && bias_per_row) ? N : 0;
    p.y = y;
    p.K = K;
    p.N = N;
    p.row_bytes = (N + 1) / 2;
    p.block_size = grouped ? (int)block_size : 0;

    // (the tile GEMM's epilogue knows one bias row only: a per-row addend stays on the decode
    // kernels, whose entry point admits decode sizes only)
    if (!plan_override && !bias_per_row && gemm_route_ok(f32, M, K, N) && workspace &&
        workspace_bytes >= gemm_route_bytes(f32, grouped, M, K, N) && aligned_to(workspace, 16) &&
        aligned_to(w_packed, 16) && aligned_to(scale, 16) && (!zero || aligned_to(zero, 16)) &&
        aligned_to(x, 16) && aligned_to(y, 16)) {
        dim3 grid((unsigned)((N + kDqN - 1) / kDqN), (unsigned)(K / kDqK));
        if (!f32) {
            if (grouped)
                dequant_w4_nk<true, false><<<grid, 256, 0, s>>>(
                    (const uint8_t*)w_packed, scale, (const int8_t*)zero, (uint16_t*)workspace, K, N,
                    (int)block_size);
            else
                dequant_w4_nk<false, false><<<grid, 256, 0, s>>>(
                    (const uint8_t*)w_packed, nullptr, nullptr, (uint16_t*)workspace, K, N, 0);
            if (!gemm_bf16_nk_supported(M, N, K, x, workspace, y)) return K3Q_ERR_SHAPE;
            const int64_t used = gemm_route_bytes(false, grouped, M, K, N);
            return gemm_bf16_nk_run(x, workspace, M, N, K, grouped ? nullptr : scale, bias, y, false,
                                    (char*)workspace + used, workspace_bytes - used, s);
        }
        const int parts = grouped ? 3 : 2;
        uint16_t* wt = (uint16_t*)workspace;            // [N, parts * K]
        uint16_t* xs = wt + (int64_t)N * parts * K;      // [M, parts * K]
        if (grouped)
            dequant_w4_nk<true, true><<<grid, 256, 0, s>>>(
                (const uint8_t*)w_packed, scale, (const int8_t*)zero, wt, K, N, (int)block_size);
        else
            dequant_w4_nk<false, true><<<grid, 256, 0, s>>>(
                (const uint8_t*)w_packed, nullptr, nullptr, wt, K, N, 0);
        split_f32_rows_launch((const float*)x, xs, M, K, parts, s);
        if (!gemm_bf16_nk_supported(M, N, (int64_t)parts * K, xs, wt, y)) return K3Q_ERR_SHAPE;
        const int64_t used = gemm_route_bytes(true, grouped, M, K, N);
        return gemm_bf16_nk_run(xs, wt, M, N, (int64_t)parts * K, grouped ? nullptr : scale, bias, y,
                                true, (char*)workspace + used, workspace_bytes - used, s);
    }
    Plan pl = make_plan(x_dtype, M, K, N, block_size, plan_override);
    // vector loads of x rows, packed rows, scales and zero points
    if (pl.fast && (!aligned_to(x, 16) || !aligned_to(w_packed, 16) || !aligned_to(scale, 16) ||
                    (zero && !aligned_to(zero, 4))))
        pl.fast = false;
    if (!pl.fast) {
        for (int64_t m0 = 0; m0 < M; m0 += 65535) {
            const int rows = (int)((M - m0 < 65535) ? M - m0 : 65535);
            p.m0 = (int)m0;
            p.M = rows;
            dim3 grid((unsigned)((N + 255) / 256), rows);
            if (f32) {
                if (grouped)
                    gemv_w4_generic<false, true><<<grid, 256, 0, s>>>(p);
                else
                    gemv_w4_generic<false, false><<<grid, 256, 0, s>>>(p);
            } else {
                if (grouped)
                    gemv_w4_generic<true, true><<<grid, 256, 0, s>>>(p);
                else
                    gemv_w4_generic<true, false><<<grid, 256, 0, s>>>(p);
            }
        }
        return launch_status();
    }

    const int nb_cols = 128 * pl.vec;
    const int64_t nblocks = (N + nb_cols - 1) / nb_cols;
    const int rows_max = (int)(M < pl.rows ? M : pl.rows);
    if (pl.ks > 1) {
        const int64_t need = (int64_t)pl.ks * rows_max * N * 4;
        if (!workspace || workspace_bytes < need) return K3Q_ERR_WORKSPACE;
        if (!aligned_to(workspace, 16)) return K3Q_ERR_ALIGN;
        p.part = (float*)workspace;
        // with arrival counters (zero between calls) the K split is summed in the same launch,
        // while the last workgroup of a column block has one output quad per thread at most
        // (K = N = 8192, 16 rows, per-channel: 19.0 us with two quads per thread, 17.3 us with the
        // second kernel; Llama-7B-sized decoder step: 4.67 ms against 4.92 ms)
        if (counters && counters_bytes >= nblocks * 4 && aligned_to(counters, 4) &&
            ((pl.sets < 4 && rows_max * (nb_cols / 4) <= pl.waves * 64) || plan_override))
            p.sync = (unsigned*)counters;
    }
    p.klen = pl.klen;
    for (int64_t m0 = 0; m0 < M; m0 += pl.rows) {
        const int rows = (int)((M - m0 < pl.rows) ? M - m0 : pl.rows);
        p.m0 = (int)m0;
        p.M = rows;
        dim3 grid((unsigned)((nblocks + 7) / 8 * 8), (unsigned)pl.ks);
        const int threads = pl.waves * 64;
        p.nwaves = pl.waves;
        p.per_xcd = (int)(grid.x / 8);
        p.ks = pl.ks;
        const size_t lds = (size_t)pl.waves * rows * (nb_cols + kRedPad) * sizeof(float);
        const int sets = f32 ? 2 : (rows > 16 ? 4 : rows > 8 ? 2 : 1);
        launch_plan(pl, sets, f32, p, nullptr, grouped, grid, threads, lds, s);
        if (pl.ks > 1 && !p.sync) {
            dim3 rgrid((unsigned)((N / 4 + 255) / 256), rows);
            if (f32) {
                if (grouped)
                    gemv_w4_reduce<false, true><<<rgrid, 256, 0, s>>>(p, pl.ks);
                else
                    gemv_w4_reduce<false, false><<<rgrid, 256, 0, s>>>(p, pl.ks);
            } else {
                if (grouped)
                    gemv_w4_reduce<true, true><<<rgrid, 256, 0, s>>>(p, pl.ks);
                else
                    gemv_w4_reduce<true, false><<<rgrid, 256, 0, s>>>(p, pl.ks);
            }
        }
    }
    return launch_status();
}

// One launch for several decode-sized problems that share x; returns false when their
// plans do not allow it (the caller then runs them one by one).
struct MultiProblem {
    int64_t N;
    const void* w_packed;
    const void* scale;
    const void* zero;
    const void* bias;
    void* y;
};

bool try_gemv_w4_multi(const void* x, int x_dtype, int64_t M, int64_t K, int count,
                       const MultiProblem* pr, int64_t block_size, char* workspace,
                       const int64_t* ws_offset, unsigned* counters, const int64_t* cnt_offset,
                       hipStream_t s, int* rc) {
    if (count < 2 || count > kMaxProblems) return false;
    const bool grouped = block_size > 0;
    const bool f32 = x_dtype == K3Q_F32;
    // One plan for all of them, made for a kernel as wide as the problems together: the launch
    // is then cut into about one workgroup per CU overall, not per problem.
    int64_t n_total = 0;
    for (int i = 0; i < count; ++i) n_total += pr[i].N;
    const Plan pl0 = make_plan(x_dtype, M, K, n_total, block_size, nullptr);
    if (!pl0.fast || M > pl0.rows || pl0.sets >= 4) return false;
    const int nb_cols = 128 * pl0.vec;
    // the last workgroup of a column block sums the K split: one output quad per thread
    if (pl0.ks > 1 && (int)M * (nb_cols / 4) > pl0.waves * 64) return false;
    GemvMulti mp{};
    int next_block = 0;
    const size_t lds = (size_t)pl0.waves * M * (nb_cols + kRedPad) * sizeof(float);
    for (int i = 0; i < count; ++i) {
        if ((pr[i].N % (8 * pl0.vec)) != 0) return false;
        if (!aligned_to(pr[i].w_packed, 16) || !aligned_to(pr[i].scale, 16) ||
            (pr[i].zero && !aligned_to(pr[i].zero, 4)))
            return false;
        const int64_t nblocks = (pr[i].N + nb_cols - 1) / nb_cols;
        if (pl0.ks > 1 && ((int64_t)pl0.ks * M * pr[i].N * 4 > ws_offset[i + 1] - ws_offset[i] ||
                           nblocks * 4 > cnt_offset[i + 1] - cnt_offset[i]))
            return false;
        GemvParams& p = mp.p[i];
        p.x = x;
        p.w = (const uint8_t*)pr[i].w_packed;
        p.scale = pr[i].scale;
        p.zero = (const int8_t*)pr[i].zero;
        p.bias = pr[i].bias;
        p.y = pr[i].y;
        p.K = K;
        p.N = pr[i].N;
        p.row_bytes = (pr[i].N + 1) / 2;
        p.block_size = grouped ? (int)block_size : 0;
        p.M = (int)M;
        p.m0 = 0;
        p.klen = pl0.klen;
        p.nwaves = pl0.waves;
        p.ks = pl0.ks;
        const int gx = (int)((nblocks + 7) / 8 * 8);
        p.per_xcd = gx / 8;
        if (pl0.ks > 1) {
            p.part = (float*)(workspace + ws_offset[i]);
            p.sync = counters + cnt_offset[i] / 4;
        }
        mp.first[i] = next_block;
        next_block += gx;
    }
    const int max_ks = pl0.ks;
    mp.first[count] = next_block;
    mp.count = count;
    dim3 grid((unsigned)next_block, (unsigned)max_ks);
    const int sets = f32 ? 2 : (M > 16 ? 4 : M > 8 ? 2 : 1);
    launch_plan(pl0, sets, f32, mp.p[0], &mp, grouped, grid, pl0.waves * 64, lds, s);
    *rc = launch_status();
    return true;
}

// ---- 33 ... 256 rows from a K-contiguous copy of the int4 kernel --------------------------
// The stored kernel has N contiguous, an MFMA operand wants K contiguous.  With a copy of the
// kernel laid out [N, K/2] -- eight consecutive k of a column per dword, the even ones in the
// low half-word's nibbles and the odd ones in the high half-word's -- a lane's 16-byte load IS
// its operand of four MFMA steps: `(d >> 4p) & 0x000F000F` is the nibble pair (k = 2p, 2p + 1),
// and `^ 0x00080008 | 0x43004300` turns it into the bfloat16 pair (136 + q).  Nothing is
// de-quantised in memory; the kernel is read once, as int4.  The offset, the zero point and
// the scale are taken out per group of K with the sums of x over that group, as the decode
// kernel does: tot += scale * (acc - (136 + zero) * sum_k x).
constexpr int kKmBM = 128, kKmBN = 256, kKmStage = 64;  // tile; values of K per stage
constexpr int kKmThreads = 512;                        // 8 waves: 2 (M) x 4 (N), 64 x 64 each
constexpr u32 kKmNibbles = 0x000F000Fu, kKmFlip = 0x00080008u, kKmExp = 0x43004300u;

__device__ __forceinline__ int km_swz(int row) { return (row & 6) | ((row ^ (row >> 3)) & 1); }

struct KmParams {
    const uint16_t* x;      // [M, K] bf16
    const uint8_t* shadow;  // [N, K/2]
    const void* scale;      // bf16 [G, N] (grouped) or unused
    const int8_t* zero;     // [G, N] (grouped)
    const v2u* sx;          // [K / gsize, M] sums of x over each group of K, as three bfloat16 parts
    float* part;            // [KS, M, N]
    int64_t M, N, K;
    int gsize;              // values of K per group (multiple of kKmStage)
    int klen;               // values of K per split (multiple of gsize)
    int strip;              // 1: `shadow` is the strip-linear copy of the decode kernels (k3q_w4s_pack), see below
    int units;              // (strip) K / 128
};

// sx[g][m] = sum of x[m, g*gsize .. (g+1)*gsize): one wave per (g, m), fixed order.  Stored as
// three bfloat16 parts {hi, lo, lolo, 0} whose sum is the float32 sum (each part rounds what the
// ones before left over), so that an MFMA step can multiply it by a kernel-side constant
__global__ __launch_bounds__(256) void km_group_sums(const uint16_t* __restrict__ x, v2u* __restrict__ sx,
                                                     int64_t M, int64_t K, int gsize) {
    const int lane = threadIdx.x & 63;
    const int64_t m = (int64_t)blockIdx.y * 4 + (threadIdx.x >> 6);
    const int64_t g = blockIdx.x;
    if (m >= M) return;
    const uint16_t* row = x + m * K + g * gsize;
    float sum = 0.f;
    for (int k = lane * 2; k < gsize; k += 128) {
        const u32 d = *(const u32*)(row + k);
        sum += bf16_bits_to_f32(d & 0xffffu) + bf16_bits_to_f32(d >> 16);
    }
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) sum += __shfl_xor(sum, off, 64);
    if (lane == 0) {
        const u32 hi = f32_to_bf16_bits(sum);
        const float r1 = sum - bf16_bits_to_f32(hi);
        const u32 lo = f32_to_bf16_bits(r1);
        const u32 lolo = f32_to_bf16_bits(r1 - bf16_bits_to_f32(lo));
        v2u o;
        o[0] = hi | (lo << 16);
        o[1] = lolo;
        sx[g * M + m] = o;
    }
}

// Everything the loop consumes arrives by LDS-DMA (global_load_lds), nothing through
// registers: the compiler then places no waits of its own in the loop (a register load there
// made it wait for every outstanding operation at each use, which serialised the pipeline:
// 3 us per stage), and the one s_waitcnt per stage is written by hand.
// kDepth: stages in flight or in use.  Per stage a slot holds the x tile (128 rows x 128 B,
// chunk-swizzled), the kernel rows (256 rows x 32 B) and the group's parameters (256 scales,
// 256 zero points, 128 sums of x of 8 bytes); every wave issues four DMA instructions per stage.
constexpr int kKmXBytes = kKmBM * 128, kKmWBytes = kKmBN * 32, kKmParBytes = 2048;
constexpr int kKmSlotBytes = kKmXBytes + kKmWBytes + kKmParBytes;
constexpr int kKmParScale = 0, kKmParZero = 512, kKmParSx = 768, kKmParSpare = 1792;

// kGroupStages: stages per group of K when that is 1, 2 or 4 (groups of 64, 128, 256), else 0.
// Known at compile time, the first MFMAs of a group take a zero accumulator operand and the
// 64 accumulators are never cleared; with 0 the group ends are found at run time.
// kNB: blocks of 32 kernel rows per wave: 2 (tiles of 128 x 256) or 1 (128 x 128, for kernels so
// narrow that wide tiles leave CUs idle even at eight splits).
// kWM: waves along M: 2 (tiles of 128 rows) or 1 (64 rows, eight waves side by side, kNB = 1).
template <bool kGrouped, int kDepth, int kGroupStages, int kWM, int kNB>
__global__ __launch_bounds__(kKmThreads) void gemm_w4_kmajor(KmParams p) {
    constexpr int kWaveN = 32 * kNB, kBN = kWaveN * (8 / kWM), kBM = 64 * kWM;
    extern __shared__ char km_lds[];
    constexpr int kXOps = kWM;               // x-tile DMA instructions a wave issues per stage
    constexpr int kOpsPerStage = kXOps + 2;  // DMA instructions a wave issues per stage
    const int tid = threadIdx.x, lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wm = kWM == 2 ? wave >> 2 : 0, wn = kWM == 2 ? (wave & 3) : wave;
    const int i = lane & 31, g = lane >> 5;
    const int64_t n0 = (int64_t)blockIdx.x * kBN, m0 = (int64_t)blockIdx.y * kBM;
    const int64_t k_begin = (int64_t)blockIdx.z * p.klen;
    const int64_t k_end = k_begin + p.klen < p.K ? k_begin + p.klen : p.K;
    const int stages = (int)((k_end - k_begin) / kKmStage);

    // x tile: instruction d of a stage fills LDS bytes [d * 1024, +1024) = 8 rows, the lane's
    // 16 bytes at lane * 16; the chunk swizzle is applied on the source side.  A wave issues
    // instructions kXOps * wave ... kXOps * wave + kXOps - 1.
    const char* a_src[kXOps];
#pragma unroll
    for (int j = 0; j < kXOps; ++j) {
        const int row = (kXOps * wave + j) * 8 + (lane >> 3);
        const int ch = (lane & 7) ^ km_swz(row);
        int64_t grow = m0 + row;
        if (grow >= p.M) grow = p.M - 1;
        // (strip: position 4 g + s of the stage's x row holds chunk 4 s + 2 h + g of the unit's sixteen)
        a_src[j] = (const char*)(p.x + grow * p.K + k_begin) + (p.strip ? 4 * (ch & 3) + (ch >> 2) : ch) * 16;
    }
    // The same kernel reads the decode kernels' strip-linear copy instead of a K-contiguous one
    // (p.strip): [strip = n / 16][unit = k / 128][lane' = i + 16 g'][4 dwords], dword s of lane' the
    // eight k = 128 unit + 32 s + 8 g' + e.  A stage is then HALF A UNIT in another sense than 64
    // consecutive k: stage h of a unit takes the pieces g' = 2 h and 2 h + 1 of every column -- a
    // column's two 16-byte pieces of the stage, 512 contiguous bytes per strip and instruction --
    // i.e. the sixteen k = 32 s + 16 h ... + 15 for s = 0 ... 3.  MFMA step s of the stage contracts
    // exactly those sixteen (lanes 0 ... 31 the first eight, lanes 32 ... 63 the second), so only the
    // SOURCE addresses change: the kernel rows advance by 512 bytes per stage, and the x tile takes
    // the matching four runs of 32 bytes of the unit's 256 (advancing by 32, then by 224).  A sum
    // over a group of 128 (= a unit) does not care in which order its k arrive; groups of 64 would
    // be split across stages and keep the K-contiguous copy.
    int x_step = p.strip ? 32 : 128;
    const int w_step = p.strip ? 512 : 32;
    // kernel rows: one instruction per wave and stage = 32 rows x 32 bytes, two lanes per row
    const char* w_src;
    {
        // (narrow tiles: waves 4 ... 7 fetch the rows of waves 0 ... 3 again, into the unused half)
        int64_t n = n0 + (kBN == 128 ? (wave & 3) : wave) * 32 + (lane >> 1);
        if (n >= p.N) n = p.N - 1;
        if (p.strip)
            w_src = (const char*)p.shadow + ((n >> 4) * p.units + k_begin / 128) * 1024 + (n & 15) * 16 + (lane & 1) * 256;
        else
            w_src = (const char*)p.shadow + n * (p.K / 2) + k_begin / 2 + (lane & 1) * 16;
    }
    // group parameters, four bytes per lane: waves 0, 1 the scales, wave 2 the zero points,
    // waves 3 ... 6 the sums of x (two dwords per row); the last fetches a spare copy so that
    // every wave counts alike (per-channel kernels: waves 0 ... 2 as well)
    const char* par_base;
    int64_t par_step;   // bytes from one group to the next
    int par_dst;
    {
        const int w = wave;
        if (kGrouped && w < 2) {
            int64_t n = n0 + w * 128 + lane * 2;
            if (n > p.N - 2) n = p.N - 2;
            par_base = (const char*)p.scale + n * 2;
            par_step = p.N * 2;
            par_dst = kKmParScale + w * 256;
        } else if (kGrouped && w == 2) {
            int64_t n = n0 + lane * 4;
            if (n > p.N - 4) n = p.N - 4;
            par_base = (const char*)p.zero + n;
            par_step = p.N;
            par_dst = kKmParZero;
        } else {
            const bool sums = w >= 3 && w <= 6;
            const int dw = sums ? (w - 3) * 64 + lane : lane;  // dword of the tile's 128 x 2
            int64_t m = m0 + (dw >> 1);
            if (m >= p.M) m = p.M - 1;
            par_base = (const char*)(p.sx + m) + (dw & 1) * 4;
            par_step = p.M * 8;
            par_dst = sums ? kKmParSx + (w - 3) * 256 : (w == 7 ? kKmParSpare : w * 256);
        }
    }
    int a_row[2];
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) a_row[mb] = wm * 64 + mb * 32 + i;

    v16f acc[kNB][2], tot[kNB][2];
#pragma unroll
    for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
        for (int mb = 0; mb < 2; ++mb)
#pragma unroll
            for (int r = 0; r < 16; ++r) acc[nb][mb][r] = tot[nb][mb][r] = 0.f;
    v16f zero16;
#pragma unroll
    for (int r = 0; r < 16; ++r) zero16[r] = 0.f;

    // stages are issued in order, one after the other: the sources advance by a stage each time
    // and the parameter source by a group every `group_stages` stages (no per-stage address
    // arithmetic: a 64-bit division per stage cost more scalar instructions than the MFMAs)
    const int group_stages = p.gsize / kKmStage;
    const char* par_src = par_base + (k_begin / p.gsize) * par_step;
    int issued_in_group = 0;
    auto issue = [&](int slot) {
        char* base = km_lds + slot * kKmSlotBytes;
#pragma unroll
        for (int j = 0; j < kXOps; ++j) {
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)a_src[j],
                (__attribute__((address_space(3))) void*)(base + (kXOps * wave + j) * 1024), 16, 0, 0);
            a_src[j] += x_step;
        }
        if (p.strip) x_step = 256 - x_step;
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)w_src,
            (__attribute__((address_space(3))) void*)(base + kKmXBytes + wave * 1024), 16, 0, 0);
        w_src += w_step;
        __builtin_amdgcn_global_load_lds(
            (const __attribute__((address_space(1))) void*)par_src,
            (__attribute__((address_space(3))) void*)(base + kKmXBytes + kKmWBytes + par_dst), 4, 0, 0);
        if (++issued_in_group == group_stages) {
            issued_in_group = 0;
            par_src += par_step;
        }
    };
#pragma unroll
    for (int d = 0; d < kDepth - 1; ++d)
        if (d < stages) issue(d);

    int done_in_group = 0;
    for (int st0 = 0; st0 < stages; st0 += kDepth) {
#pragma unroll
        for (int u = 0; u < kDepth; ++u) {
            const int st = st0 + u;
            if (st >= stages) break;
            // stage st has landed once at most the operations of the stages issued after it are
            // outstanding; near the end fewer were issued: wait for everything
            if (st + kDepth - 2 < stages)
                __builtin_amdgcn_s_waitcnt(km_vmcnt(kOpsPerStage * (kDepth - 2)));
            else
                __builtin_amdgcn_s_waitcnt(km_vmcnt(0));
            // s_barrier without a fence (a fence would drain the DMA of the stages in flight):
            // every wave's part of the slot is there; slot u - 1 is free
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (st + kDepth - 1 < stages) issue((u + kDepth - 1) % kDepth);
            const char* cur = km_lds + u * kKmSlotBytes;
            v4u wq[kNB];  // this lane's 32 values of K of its two kernel rows: chunk 4g + s at step s
#pragma unroll
            for (int nb = 0; nb < kNB; ++nb)
                wq[nb] = *(const v4u*)(cur + kKmXBytes + (wn * kWaveN + nb * 32 + i) * 32 + g * 16);
            // (kDepth is a multiple of kGroupStages and a split starts on a group: u tells)
            constexpr bool kStatic = kGroupStages > 0;
            const bool group_first = kStatic && (u % (kStatic ? kGroupStages : 1)) == 0;
#pragma unroll
            for (int s = 0; s < 4; ++s) {
                v4u xa[2], wb[kNB];
#pragma unroll
                for (int mb = 0; mb < 2; ++mb)
                    xa[mb] = *(const v4u*)(cur + a_row[mb] * 128 + (((4 * g + s) ^ km_swz(a_row[mb])) << 4));
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
                    const u32 d = wq[nb][s];
#pragma unroll
                    for (int q = 0; q < 4; ++q) wb[nb][q] = (((d >> (4 * q)) & kKmNibbles) ^ kKmFlip) | kKmExp;
                }
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb)
                        acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                            as_bf(wb[nb]), as_bf(xa[mb]), (group_first && s == 0) ? zero16 : acc[nb][mb], 0, 0, 0);
            }
            // end of a group of K (or of this split): fold offset, zero point and scale
            bool group_last;
            if (kStatic) {
                group_last = (u % (kStatic ? kGroupStages : 1)) == (kStatic ? kGroupStages : 1) - 1;
            } else {
                group_last = ++done_in_group == group_stages || st + 1 == stages;
                if (group_last) done_in_group = 0;
            }
            if (group_last) {
                const char* par = cur + kKmXBytes + kKmWBytes;
                // acc -= (136 + zero) * sum(x) as one more MFMA step: k = 0 ... 2 carry -128 on the
                // kernel side, k = 3 ... 5 carry -(8 + zero) (any int8 zero point is exact in
                // bfloat16), both against the three bfloat16 parts of the sum of x; products of
                // two bfloat16 are exact in float32, so the cancellation happens in the accumulator
                v4u xs[2], wz[kNB];
#pragma unroll
                for (int mb = 0; mb < 2; ++mb) {
                    v2u raw = *(const v2u*)(par + kKmParSx + a_row[mb] * 8);
                    if (g) raw[0] = raw[1] = 0;  // lanes 32 ... 63 hold k = 8 ... 15: nothing there
                    xs[mb][0] = raw[0];                                   // hi, lo
                    xs[mb][1] = (raw[1] & 0xffffu) | (raw[0] << 16);      // lolo, hi
                    xs[mb][2] = (raw[0] >> 16) | (raw[1] << 16);          // lo, lolo
                    xs[mb][3] = 0;
                }
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
                    int zp = 0;
                    if (kGrouped) zp = *(const int8_t*)(par + kKmParZero + wn * kWaveN + nb * 32 + i);
                    const u32 cz = __float_as_uint(-(float)(8 + zp)) >> 16;
                    wz[nb][0] = 0xC300C300u;                              // -128, -128
                    wz[nb][1] = 0xC300u | (cz << 16);                     // -128, -(8 + zero)
                    wz[nb][2] = cz | (cz << 16);
                    wz[nb][3] = 0;
                }
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb)
#pragma unroll
                    for (int mb = 0; mb < 2; ++mb)
                        acc[nb][mb] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(as_bf(wz[nb]), as_bf(xs[mb]),
                                                                              acc[nb][mb], 0, 0, 0);
#pragma unroll
                for (int nb = 0; nb < kNB; ++nb) {
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        float sc[4] = {1.f, 1.f, 1.f, 1.f};
                        if (kGrouped) {
                            const int nl = wn * kWaveN + nb * 32 + 8 * rg + 4 * g;
                            const v2u sraw = *(const v2u*)(par + kKmParScale + nl * 2);
#pragma unroll
                            for (int e = 0; e < 4; ++e) {
                                const u32 w = sraw[e >> 1];
                                sc[e] = __uint_as_float((e & 1) ? (w & 0xffff0000u) : (w << 16));
                            }
                        }
#pragma unroll
                        for (int e = 0; e < 4; ++e)
#pragma unroll
                            for (int mb = 0; mb < 2; ++mb) {
                                const int r = 4 * rg + e;
                                tot[nb][mb][r] = __builtin_fmaf(sc[e], acc[nb][mb][r], tot[nb][mb][r]);
                                if (!kStatic) acc[nb][mb][r] = 0.f;
                            }
                    }
                }
            }
        }
    }

    // raw sums of this split; gemv_w4_reduce adds the splits and applies the epilogue
#pragma unroll
    for (int mb = 0; mb < 2; ++mb) {
        const int64_t m = m0 + a_row[mb];
        if (m >= p.M) continue;
#pragma unroll
        for (int nb = 0; nb < kNB; ++nb) {
            if (n0 + wn * kWaveN + nb * 32 >= p.N) continue;  // N % 32 == 0: a block is in or out as a whole
#pragma unroll
            for (int rg = 0; rg < 4; ++rg) {
                const int64_t n = n0 + wn * kWaveN + nb * 32 + 8 * rg + 4 * g;
                v4f o;
#pragma unroll
                for (int e = 0; e < 4; ++e) o[e] = tot[nb][mb][4 * rg + e];
                *(v4f*)(p.part + ((int64_t)blockIdx.z * p.M + m) * p.N + n) = o;
            }
        }
    }
}

// shapes and sizes the K-contiguous route takes
inline bool kmajor_ok(int64_t M, int64_t K, int64_t N, int64_t block_size) {
    const int64_t gsize = block_size > 0 ? block_size : 128;
    return M >= 17 && M <= 512 && (K % 128) == 0 && (N % 32) == 0 && (gsize % kKmStage) == 0 &&
           (K % gsize) == 0;
}

struct KmPlan {
    int ks;
    int64_t klen;
    int bn;  // tile width: 256, or 128 where 256 would leave CUs idle even at eight splits
    int bm;  // tile rows: 128, or 64 (with 256 columns) up to 64 rows
};

inline KmPlan kmajor_plan(int64_t M, int64_t K, int64_t N, int64_t gsize) {
    const int bm = M <= 64 ? 64 : kKmBM;
    const int64_t m_tiles = (M + bm - 1) / bm;
    const int bn = (bm == kKmBM && m_tiles * ((N + kKmBN - 1) / kKmBN) * 8 < kTargetWorkgroups) ? kKmBN / 2
                                                                                               : kKmBN;
    const int64_t tiles = m_tiles * ((N + bn - 1) / bn);
    // about one workgroup per CU, at most eight splits (every split writes and the reduction
    // reads M x N floats: at 128 rows one split of a 4096 x 14336 kernel is a quarter of the
    // kernel's own bytes), at least eight stages per split
    // (one workgroup fits a CU: the launch must not spill into a second round)
    int64_t ks = kTargetWorkgroups / tiles;
    if (ks < 1) ks = 1;
    if (ks > 8) ks = 8;
    const int64_t unit = gsize > 2 * kKmStage ? gsize : 2 * kKmStage;  // a split is whole groups
    int64_t klen = (K / ks + unit - 1) / unit * unit;
    if (klen < 8 * kKmStage) klen = (8 * kKmStage + unit - 1) / unit * unit;
    if (klen > K) klen = K;
    KmPlan pl;
    pl.bn = bn;
    pl.bm = bm;
    pl.klen = klen;
    pl.ks = (int)((K + klen - 1) / klen);
    return pl;  // rounding klen up can only lower the split count
}

}  // namespace

void split_f32_rows_launch(const float* x, uint16_t* out, int64_t M, int64_t K, int parts,
                           hipStream_t s) {
    split_f32_rows<<<(unsigned)((M * K / 4 + 255) / 256), 256, 0, s>>>(x, out, M, K, parts);
}

}  // namespace k3q

using namespace k3q;

extern "C" int64_t k3q_gemv_w4_workspace_bytes(int64_t M, int64_t K, int64_t N) {
    if (M <= 0 || K <= 0 || N <= 0) return 0;
    // the largest partial buffer the built-in plans ask for (the plan depends on
    // the dtype and on whether the kernel is grouped; take the maximum over those)
    int64_t part = 0;
    const int64_t groupings[3] = {-1, 128, 32};
    for (int dt = 0; dt < 2; ++dt)
        for (int gi = 0; gi < 3; ++gi) {
            const Plan pl = make_plan(dt, M, K, N, groupings[gi], nullptr);
            if (!pl.fast || pl.ks <= 1) continue;
            const int64_t rows = M < pl.rows ? M : pl.rows;
            const int64_t b = (int64_t)pl.ks * rows * N * 4;
            if (b > part) part = b;
        }
    // prefill sizes: room for the bfloat16 [N, K] copy of the de-quantised kernel
    for (int f32 = 0; f32 < 2; ++f32)
        if (gemm_route_ok(f32, M, K, N)) {
            const int64_t need = gemm_route_bytes(f32, true, M, K, N) +
                                 gemm_route_extra_bytes(f32, true, M, K, N);
            if (need > part) part = need;
        }
    return part;
}

extern "C" int k3q_gemv_w4(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                           const void* w_packed, const void* scale, const void* zero,
                           int64_t block_size, const void* bias, void* y, void* workspace,
                           int64_t workspace_bytes, void* stream) {
    return run_gemv_w4(x, x_dtype, M, K, N, w_packed, scale, zero, block_size, bias, y, workspace,
                       workspace_bytes, nullptr, nullptr, 0, (hipStream_t)stream);
}

extern "C" int64_t k3q_gemv_w4_counters_bytes(int64_t N) {
    return N <= 0 ? 0 : (N + 127) / 128 * 4;
}

extern "C" int k3q_gemv_w4_fused(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                 const void* w_packed, const void* scale, const void* zero,
                                 int64_t block_size, const void* bias, void* y, void* workspace,
                                 int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                                 void* stream) {
    return run_gemv_w4(x, x_dtype, M, K, N, w_packed, scale, zero, block_size, bias, y, workspace,
                       workspace_bytes, nullptr, counters, counters_bytes, (hipStream_t)stream);
}

extern "C" int k3q_gemv_w4_addend(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                  const void* w_packed, const void* scale, const void* zero,
                                  int64_t block_size, const void* addend, void* y, void* workspace,
                                  int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                                  void* stream) {
    if (M > 64) return K3Q_ERR_SHAPE;
    if (M > 0 && !addend) return K3Q_ERR_NULL;
    return run_gemv_w4(x, x_dtype, M, K, N, w_packed, scale, zero, block_size, addend, y, workspace,
                       workspace_bytes, nullptr, counters, counters_bytes, (hipStream_t)stream, true);
}

extern "C" int k3qt_gemv_w4_plan(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                const void* w_packed, const void* scale, const void* zero,
                                int64_t block_size, const void* bias, void* y, void* workspace,
                                int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                                const int* plan, void* stream) {
    return run_gemv_w4(x, x_dtype, M, K, N, w_packed, scale, zero, block_size, bias, y, workspace,
                       workspace_bytes, plan, counters, counters_bytes, (hipStream_t)stream);
}

extern "C" int k3q_gemv_w4_multi(const void* x, int x_dtype, int64_t M, int64_t K, int count,
                                 const k3q_gemv_w4_problem* problems, int64_t block_size,
                                 void* workspace, int64_t workspace_bytes, void* counters,
                                 int64_t counters_bytes, void* stream) {
    if (count < 0) return K3Q_ERR_SHAPE;
    if (count == 0) return K3Q_OK;
    if (!problems) return K3Q_ERR_NULL;
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0) return K3Q_ERR_SHAPE;
    // every problem has its own slice of the workspace and of the counters
    constexpr int kMaxCount = 16;
    if (count > kMaxCount) return K3Q_ERR_SHAPE;
    int64_t ws_offset[kMaxCount + 1], cnt_offset[kMaxCount + 1];
    MultiProblem pr[kMaxCount];
    ws_offset[0] = cnt_offset[0] = 0;
    const size_t el = x_dtype == K3Q_F32 ? 4 : 2;
    for (int i = 0; i < count; ++i) {
        const k3q_gemv_w4_problem& q = problems[i];
        if (q.N <= 0) return K3Q_ERR_SHAPE;
        if (M > 0 && (!x || !q.w_packed || !q.scale || !q.y || (block_size > 0 && !q.zero)))
            return K3Q_ERR_NULL;
        if (!aligned_to(q.scale, el) || !aligned_to(q.y, el) || (q.bias && !aligned_to(q.bias, el)))
            return K3Q_ERR_ALIGN;
        pr[i] = MultiProblem{q.N, q.w_packed, q.scale, q.zero, q.bias, q.y};
        ws_offset[i + 1] = ws_offset[i] + (k3q_gemv_w4_workspace_bytes(M, K, q.N) + 255) / 256 * 256;
        cnt_offset[i + 1] = cnt_offset[i] + k3q_gemv_w4_counters_bytes(q.N);
    }
    if (M == 0) return K3Q_OK;
    const bool ws_ok = workspace && aligned_to(workspace, 16) && workspace_bytes >= ws_offset[count];
    const bool cnt_ok = counters && aligned_to(counters, 4) && counters_bytes >= cnt_offset[count];
    hipStream_t s = (hipStream_t)stream;
    int rc = K3Q_OK;
    if (ws_ok && cnt_ok && aligned_to(x, 16) &&
        try_gemv_w4_multi(x, x_dtype, M, K, count, pr, block_size, (char*)workspace, ws_offset,
                          (unsigned*)counters, cnt_offset, s, &rc))
        return rc;
    for (int i = 0; i < count; ++i) {
        // one after the other on the stream: each may use all of the workspace and counters
        rc = run_gemv_w4(x, x_dtype, M, K, pr[i].N, pr[i].w_packed, pr[i].scale, pr[i].zero, block_size,
                         pr[i].bias, pr[i].y, ws_ok ? workspace : nullptr, ws_ok ? workspace_bytes : 0,
                         nullptr, cnt_ok ? counters : nullptr, cnt_ok ? counters_bytes : 0, s);
        if (rc != K3Q_OK) return rc;
    }
    return K3Q_OK;
}

namespace k3q {
namespace {
// One thread per dword of the K-contiguous copy; threads of a wave take neighbouring columns,
// so the reads of the stored kernel (row-major [K, ceil(N/2)]) are contiguous per row.
__global__ __launch_bounds__(256) void w4_kmajor_pack(const uint8_t* __restrict__ w, u32* __restrict__ out,
                                                     int64_t K8, int64_t N) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (t >= K8 * N) return;
    const int64_t n = t % N, j = t / N;
    const int64_t row_bytes = (N + 1) / 2;
    const int shift = (int)(n & 1) * 4;
    u32 d = 0;
#pragma unroll
    for (int e = 0; e < 8; ++e) {
        const u32 nib = (w[(8 * j + e) * row_bytes + n / 2] >> shift) & 0xFu;
        d |= nib << ((e & 1) * 16 + (e >> 1) * 4);
    }
    out[n * K8 + j] = d;
}
}  // namespace
}  // namespace k3q

extern "C" int k3q_w4_kmajor_pack(const int8_t* w_packed, int64_t K, int64_t N, int32_t* w_kmajor, void* stream) {
    if (K <= 0 || N <= 0 || (K % 8) != 0 || (K / 8) * N >= ((int64_t)1 << 39)) return K3Q_ERR_SHAPE;
    if (!w_packed || !w_kmajor) return K3Q_ERR_NULL;
    if (!aligned_to(w_kmajor, 4)) return K3Q_ERR_ALIGN;
    const int64_t dwords = (K / 8) * N;
    k3q::w4_kmajor_pack<<<(unsigned)((dwords + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint8_t*)w_packed, (u32*)w_kmajor, K / 8, N);
    return launch_status();
}

extern "C" int64_t k3q_gemm_w4_kmajor_workspace_bytes(int64_t M, int64_t K, int64_t N, int64_t block_size) {
    if (!kmajor_ok(M, K, N, block_size)) return 0;
    const int64_t gsize = block_size > 0 ? block_size : 128;
    const KmPlan pl = kmajor_plan(M, K, N, gsize);
    return ((K / gsize) * M * 8 + 255) / 256 * 256 + (int64_t)pl.ks * M * N * 4;
}

static int run_gemm_w4_tiles(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                             const void* w_kmajor, bool strip, const void* scale, const void* zero,
                             int64_t block_size, const void* bias, void* y, void* workspace,
                             int64_t workspace_bytes, void* stream) {
    if (x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!x || !w_kmajor || !scale || !y) return K3Q_ERR_NULL;
    const bool grouped = block_size > 0;
    if (grouped && !zero) return K3Q_ERR_NULL;
    if (!kmajor_ok(M, K, N, block_size)) return K3Q_ERR_SHAPE;
    if (strip && block_size > 0 && (block_size % 128) != 0) return K3Q_ERR_SHAPE;
    if (!aligned_to(x, 16) || !aligned_to(w_kmajor, 16) || !aligned_to(scale, 8) ||
        (zero && !aligned_to(zero, 4)) || !aligned_to(y, 8) || (bias && !aligned_to(bias, 2)))
        return K3Q_ERR_ALIGN;
    const int64_t need = k3q_gemm_w4_kmajor_workspace_bytes(M, K, N, block_size);
    if (!workspace || workspace_bytes < need) return K3Q_ERR_WORKSPACE;
    if (!aligned_to(workspace, 16)) return K3Q_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    int64_t gsize = grouped ? block_size : 128;
    const KmPlan pl = kmajor_plan(M, K, N, gsize);
    // per-channel kernels need the offset taken out only once per split
    if (!grouped && (K % pl.klen) == 0) gsize = pl.klen;
    v2u* sx = (v2u*)workspace;
    float* part = (float*)((char*)workspace + ((K / gsize) * M * 8 + 255) / 256 * 256);
    km_group_sums<<<dim3((unsigned)(K / gsize), (unsigned)((M + 3) / 4)), 256, 0, s>>>(
        (const uint16_t*)x, sx, M, K, (int)gsize);
    KmParams kp{};
    kp.x = (const uint16_t*)x;
    kp.shadow = (const uint8_t*)w_kmajor;
    kp.scale = scale;
    kp.zero = (const int8_t*)zero;
    kp.sx = sx;
    kp.part = part;
    kp.M = M;
    kp.N = N;
    kp.K = K;
    kp.gsize = (int)gsize;
    kp.klen = (int)pl.klen;
    kp.strip = strip ? 1 : 0;
    kp.units = (int)(K / 128);
    dim3 grid((unsigned)((N + pl.bn - 1) / pl.bn), (unsigned)((M + pl.bm - 1) / pl.bm), (unsigned)pl.ks);
    constexpr int kDepth = 4;
    const size_t lds = (size_t)kDepth * kKmSlotBytes;
    using KmKernel = void (*)(KmParams);
#define K3Q_KM_ROW(G, WM, NB)                                                               \
    {gemm_w4_kmajor<G, kDepth, 0, WM, NB>, gemm_w4_kmajor<G, kDepth, 1, WM, NB>,             \
     gemm_w4_kmajor<G, kDepth, 2, WM, NB>, gemm_w4_kmajor<G, kDepth, 4, WM, NB>}
    // tile shapes: 128 x 128, 128 x 256, 64 x 256
    static const KmKernel kernels[2][3][4] = {
        {K3Q_KM_ROW(false, 2, 1), K3Q_KM_ROW(false, 2, 2), K3Q_KM_ROW(false, 1, 1)},
        {K3Q_KM_ROW(true, 2, 1), K3Q_KM_ROW(true, 2, 2), K3Q_KM_ROW(true, 1, 1)}};
#undef K3Q_KM_ROW
    static const bool raised = [] {
        bool ok = true;
        for (int a = 0; a < 2; ++a)
            for (int b = 0; b < 3; ++b)
                for (int c = 0; c < 4; ++c)
                    ok = hipFuncSetAttribute((const void*)kernels[a][b][c],
                                             hipFuncAttributeMaxDynamicSharedMemorySize,
                                             kLdsBudget) == hipSuccess && ok;
        return ok;
    }();
    (void)raised;
    const int gs = (int)(gsize / kKmStage);
    const int variant = gs == 1 ? 1 : gs == 2 ? 2 : gs == 4 ? 3 : 0;
    const int shape = pl.bm == 64 ? 2 : pl.bn == kKmBN ? 1 : 0;
    kernels[grouped ? 1 : 0][shape][variant]<<<grid, kKmThreads, lds, s>>>(kp);
    // the decode kernel's second pass: sums the splits in order, applies scale and bias
    GemvParams gp{};
    gp.scale = scale;
    gp.bias = bias;
    gp.y = y;
    gp.part = part;
    gp.N = N;
    gp.M = (int)M;
    gp.m0 = 0;
    dim3 rgrid((unsigned)((N / 4 + 255) / 256), (unsigned)M);
    if (grouped)
        gemv_w4_reduce<true, true><<<rgrid, 256, 0, s>>>(gp, pl.ks);
    else
        gemv_w4_reduce<true, false><<<rgrid, 256, 0, s>>>(gp, pl.ks);
    return launch_status();
}

extern "C" int k3q_gemm_w4_kmajor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                  const void* w_kmajor, const void* scale, const void* zero,
                                  int64_t block_size, const void* bias, void* y, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
    return run_gemm_w4_tiles(x, x_dtype, M, K, N, w_kmajor, false, scale, zero, block_size, bias, y, workspace,
                             workspace_bytes, stream);
}

extern "C" int k3q_gemm_w4_strip(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                 const void* w_strip, const void* scale, const void* zero,
                                 int64_t block_size, const void* bias, void* y, void* workspace,
                                 int64_t workspace_bytes, void* stream) {
    return run_gemm_w4_tiles(x, x_dtype, M, K, N, w_strip, true, scale, zero, block_size, bias, y, workspace,
                             workspace_bytes, stream);
}

// ---- the decode-sized call for callers that cannot allocate -----------------------------
// The K split's partial sums and arrival counters live in a file-scope device array instead
// of a caller's workspace.  Every device the library runs on holds its own copy of the array
// (until the process ends); its address on a device comes from hipGetSymbolAddress, asked
// once per device with that device current -- the array's name is a host-side stand-in in
// host code, not a device address.
namespace k3q {
namespace {
constexpr int64_t kStaticCounterBytes = 64 * 1024;          // column blocks of N <= 2^21
constexpr int64_t kStaticPartialBytes = 16 * 1024 * 1024;   // K split x rows x N floats
static __device__ __align__(256) unsigned char scratch[kStaticCounterBytes + kStaticPartialBytes];

constexpr int kStaticMaxDevices = 64;
unsigned char* g_scratch_ptr[kStaticMaxDevices];  // per device, null until asked for
std::mutex g_scratch_mutex;

__global__ void clear_words(unsigned* p, int n) {
    const int i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) p[i] = 0u;
}

// Address of this device's copy of `scratch` ("this device" = the current one, which a launch on
// `s` requires to be the device of `s` anyway).  The look-up happens on the first call on a device
// and that call may already be under stream capture: the symbol query is not a stream operation,
// so the thread's capture mode is relaxed around it (under the strict modes a capture refuses
// every call that is not known to be safe, and is invalidated by it).  On a first call outside
// capture the counters are also cleared on `s` by a fill kernel; a first call under capture relies
// on what the language guarantees -- a `__device__` array without initialiser is zero when the
// code object is loaded -- and adds no node of its own to the caller's graph.  Every call leaves
// the counters at zero again.
int static_scratch(hipStream_t s, unsigned char** out) {
    int dev = -1;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= kStaticMaxDevices) return K3Q_ERR_LAUNCH;
    std::lock_guard<std::mutex> lock(g_scratch_mutex);
    if (!g_scratch_ptr[dev]) {
        hipStreamCaptureStatus capturing = hipStreamCaptureStatusNone;
        if (hipStreamIsCapturing(s, &capturing) != hipSuccess) return K3Q_ERR_LAUNCH;
        hipStreamCaptureMode mode = hipStreamCaptureModeRelaxed;
        if (hipThreadExchangeStreamCaptureMode(&mode) != hipSuccess) return K3Q_ERR_LAUNCH;
        unsigned char* ptr = nullptr;
        const hipError_t found = hipGetSymbolAddress((void**)&ptr, HIP_SYMBOL(scratch));
        if (hipThreadExchangeStreamCaptureMode(&mode) != hipSuccess) return K3Q_ERR_LAUNCH;
        if (found != hipSuccess || !ptr) return K3Q_ERR_LAUNCH;
        if (capturing == hipStreamCaptureStatusNone) {
            const int words = (int)(kStaticCounterBytes / 4);
            clear_words<<<(words + 255) / 256, 256, 0, s>>>((unsigned*)ptr, words);
            if (hipGetLastError() != hipSuccess) return K3Q_ERR_LAUNCH;
        }
        g_scratch_ptr[dev] = ptr;
    }
    *out = g_scratch_ptr[dev];
    return K3Q_OK;
}
}  // namespace
}  // namespace k3q

extern "C" int64_t k3q_gemv_w4_static_max_bytes(void) { return kStaticPartialBytes; }

extern "C" int k3q_gemv_w4_static(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                                  const void* w_packed, const void* scale, const void* zero,
                                  int64_t block_size, const void* bias, void* y, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M > 16) return K3Q_ERR_SHAPE;  // decode sizes only: larger M needs scratch that scales with N * K
    if (M == 0) return K3Q_OK;
    if (!x || !w_packed || !scale || !y) return K3Q_ERR_NULL;
    if (block_size > 0 && !zero) return K3Q_ERR_NULL;
    // the plan is the one k3q_gemv_w4_fused makes: same kernels, same partials, same order
    const Plan pl = make_plan(x_dtype, M, K, N, block_size, nullptr);
    const int64_t rows = M < pl.rows ? M : pl.rows;
    const int64_t need = (pl.fast && pl.ks > 1) ? (int64_t)pl.ks * rows * N * 4 : 0;
    if (need > kStaticPartialBytes || k3q_gemv_w4_counters_bytes(N) > kStaticCounterBytes)
        return K3Q_ERR_WORKSPACE;
    unsigned char* base = nullptr;
    const int rc = static_scratch((hipStream_t)stream, &base);
    if (rc != K3Q_OK) return rc;
    return run_gemv_w4(x, x_dtype, M, K, N, w_packed, scale, zero, block_size, bias, y,
                       base + kStaticCounterBytes, kStaticPartialBytes, nullptr, base,
                       kStaticCounterBytes, (hipStream_t)stream);
}
