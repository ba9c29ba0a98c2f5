// Decode-sized int8 Dense forward in one launch, from a strip-linear copy of the int8 kernel:
//     q, sa = abs_max_quantize(x, axis=-1)          (x: up to 16 bfloat16 rows)
//     y[m,n] = bf16( bf16(acc[m,n]) / bf16(sa[m] * sb[n]) ) (+ bias),  acc = sum_k q[m,k] * w[k,n]
// with every rounding step of the reference's op sequence (the bit-exact epilogue of the tile GEMM).
//
// Copy layout ("w8s"): [strip = n / 16][unit = k / 64][lane = 64][16 bytes], 1 KiB per
// (strip, unit); lane = i + 16 g holds column n = 16 strip + i, bytes k = 64 unit + 16 g + (0..15):
// the B operand of v_mfma_i32_16x16x64_i8 as it lies, a wave instruction reads 1 KiB contiguous.
// The strip count is padded to even with zero strips.
//
// Workgroup: 8 waves.  A workgroup owns groups of kSW strips and all of K for them: wave q takes
// a contiguous slice of the units, so no partial sums leave the workgroup.  Every workgroup
// quantises x itself (x is a few KiB to a few hundred KiB and comes from L2): row maxima through
// LDS, the int8 rows into LDS, the scales stay there for the epilogue.  The weights go through
// a register ring of kD units per strip that is refilled right after a unit is consumed and
// runs on across group boundaries (a workgroup with several groups streams without a gap).
#include <mutex>
#include <set>

#include "k3q_common.h"

namespace k3q {
namespace {

constexpr int kQ = 8;            // waves per workgroup
constexpr int kT = 64 * kQ;
constexpr int kMaxRows8 = 16;
constexpr int kResident8 = 256;  // workgroups the chip holds at once (one per CU)

struct W8sParams {
    const uint16_t* x;      // [M, K] bfloat16 (quantised in the kernel), or
    const int8_t* xq;       // [M, K] int8 with
    const uint16_t* xs;     // [M] bfloat16 scales (already quantised rows)
    const v4i* w;           // strip-linear copy
    const uint16_t* scale;  // [N] bfloat16 kernel scale
    const uint16_t* bias;   // [N] or [M, N] bfloat16, or null
    uint16_t* y;            // [M, N] bfloat16
    int64_t bias_stride;    // 0: one row for all, N: a row per row of x
    int M, K, N;
    int units;              // K / 64
    int groups;             // strip groups (kSW strips each)
    int row_magic;          // ceil(2^32 / (K / 8)): piece -> row
    float eps, qlo, qhi;    // quantizer settings (eps already rounded to bfloat16)
    // an operation on x before it is quantised (kernels built with kPre only):
    int pre_kind;            // 1: rms_norm(x) * pre_op (bf16 [K]); 2: silu(pre_op) * x (pre_op bf16 [M, K])
    float pre_eps;           // rms_norm's epsilon
    const uint16_t* pre_op;
};

__device__ __forceinline__ float scale_from_amax_bf16(float amax, float eps, float qhi) {
    return round_bf16(qhi / round_bf16(amax + eps));
}
// y = T(T(acc) / T(sa * sb)) (+ bias), T = bfloat16: the reference's sequence, every step rounded
__device__ __forceinline__ float descale_exact_bf16(int acc, float sa, float sb, float bv, bool has_bias) {
    const float os = round_bf16(sb * sa);
    float r = round_bf16(round_bf16((float)acc) / os);  // (a few values per lane: the plain division is the faster form here)
    if (has_bias) r = round_bf16(r + bv);
    return r;
}

// kNP: 16-byte pieces of x a thread keeps in registers between the row maxima and the
// quantisation (0: it reads them twice); -1: the rows arrive quantised (p.xq, p.xs).
// kPre (kNP > 0 only): the rows are transformed before they are quantised (p.pre_kind): rms_norm with
// a gain, the bits of k3q_rmsnorm, or multiplied by silu of a second input, the bits of k3q_silu_mul.
template <int kSW, int kD, int kNP, bool kPre = false>
__device__ __forceinline__ void gemv_w8s_body(const W8sParams& p, const int block, const int n_blocks) {
    extern __shared__ __attribute__((aligned(16))) char w8s_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int q = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int M = p.M, K = p.K;
    const int pitch = K + 16;
    // LDS: x rows as int8 | row maxima (uint bits) | row scales | reduction buffers
    char* xs = w8s_lds;
    u32* rowmax = (u32*)(w8s_lds + ((M * pitch + 255) & ~255));
    float* sa = (float*)(rowmax + kMaxRows8);
    const int mq = (M + 3) >> 2;  // accumulator row quads that hold rows of x
    int* red = (int*)(sa + kMaxRows8);
    const int red_one = kQ * kSW * mq * 16 * 4;  // ints per buffer

    // ---- this wave's slice of the units: blocks of kD units, the first waves take one more ----
    const int blocks = p.units / kD;
    const int per = blocks / kQ, extra = blocks - per * kQ;
    const int b0 = q * per + (q < extra ? q : extra);
    const int my_units = (per + (q < extra ? 1 : 0)) * kD;
    const int u_begin = b0 * kD;

    // ---- the weight stream: the load cursor (group, first unit of a block) runs one block of
    // kD units ahead of the consumer, across group boundaries ----
    const int stride = n_blocks;
    int lg = block, lu = u_begin;
    const int last_group = p.groups - 1;
    // Workgroups are dealt round-robin to the 8 XCDs, so XCD x would take the strip groups x, x + 8, ...:
    // addresses a fixed distance apart, and with groups of 256 KiB (K = 8192, two strips) that lands an
    // XCD's whole stream on a fraction of the memory channels (measured: odd XCDs finished 1 us after
    // even ones, 15.2 us per call).  Rotating the assignment within every row of eight groups (XCD x
    // takes group 8 i + (x + i) % 8) spreads each XCD's addresses again: 13.2 us, and 42.9 -> 39.9 us at
    // N = 28672.  Smaller groups do not alias and keep the plain order (the rotation costs them 0.1 us).
    const bool rotate = p.units * kSW >= 256;
    auto place = [&](const int gi) {
        return rotate && (gi | 7) < p.groups ? (gi & ~7) | ((gi + (gi >> 3)) & 7) : gi;
    };
    const v4i* nb[kSW];  // this lane's pieces of the block at the cursor, unit by unit 64 entries apart
    auto at_cursor = [&]() {
        const int g2 = place(lg < last_group ? lg : last_group);  // past the end: a valid address, never used
#pragma unroll
        for (int t = 0; t < kSW; ++t) nb[t] = p.w + ((int64_t)(g2 * kSW + t) * p.units + lu) * 64 + lane;
    };
    auto advance = [&]() {
        lu += kD;
        if (lu == u_begin + my_units) {
            lu = u_begin;
            lg += stride;
        }
        at_cursor();
    };
    v4i W[kD][kSW];
    auto refill = [&](int d) {
#pragma unroll
        for (int t = 0; t < kSW; ++t) W[d][t] = __builtin_nontemporal_load(nb[t] + d * 64);
    };
    at_cursor();
    // Every wave's first x requests go out before any wave's weight requests: a compute unit's
    // memory pipeline serves requests in the order they were issued, and x behind 64 KiB of another
    // wave's weights reaches LDS that much later.  (A bare barrier: nothing is waited for.)
    auto x_before_weights = []() {
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    };

    // ---- stage x ----
    if constexpr (kNP < 0) {
        // rows already quantised: copy them (16 int8 per piece) and their scales into LDS
        const int pieces = M * (K >> 4);
        constexpr int kCP = 4;  // pieces in flight per thread and round
        v4u c[kCP];
        auto copy_load = [&](int base) {
#pragma unroll
            for (int i = 0; i < kCP; ++i) {
                const int pi = base + i * kT + tid;
                c[i] = ((const v4u*)p.xq)[pi < pieces ? pi : pieces - 1];
            }
        };
        auto copy_store = [&](int base) {
#pragma unroll
            for (int i = 0; i < kCP; ++i) {
                const int pi = base + i * kT + tid;
                if (pi < pieces) {
                    const int row = (int)__umulhi((u32)pi, (u32)p.row_magic);  // magic of K / 16 here
                    const int col = (pi - row * (K >> 4)) << 4;
                    *(v4u*)(xs + row * pitch + col) = c[i];
                }
            }
        };
        copy_load(0);
        x_before_weights();
#pragma unroll
        for (int d = 0; d < kD; ++d) refill(d);
        advance();
        copy_store(0);
        for (int base = kCP * kT; base < pieces; base += kCP * kT) {
            copy_load(base);
            copy_store(base);
        }
        if (tid < M) sa[tid] = bf16_bits_to_f32(p.xs[tid]);
    } else {
        // row maxima, scales, int8 rows: abs_max_quantize of the rows inside the workgroup
        const int pieces = M * (K >> 3);  // 16-byte pieces of x (8 values)
        if (tid < kMaxRows8) rowmax[tid] = 0u;
        static_assert(!kPre || kNP > 0, "the transform works on the pieces kept in registers");
        v4u xr[kNP > 0 ? kNP : 1];
        v4u xop[kPre ? kNP : 1];
        if (kNP > 0) {
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                const int pi = tid + i * kT;
                const int pc = pi < pieces ? pi : pieces - 1;
                xr[i] = ((const v4u*)p.x)[pc];
                if constexpr (kPre) {  // the gain's piece of this column, or the second input's piece
                    const int row = (int)__umulhi((u32)pc, (u32)p.row_magic);
                    xop[i] = ((const v4u*)p.pre_op)[p.pre_kind == 1 ? pc - row * (K >> 3) : pc];
                }
            }
            x_before_weights();
        }
#pragma unroll
        for (int d = 0; d < kD; ++d) refill(d);
        advance();
        __syncthreads();  // rowmax cleared
        if constexpr (kPre) {
            if (p.pre_kind == 1) {
                // sums of squares per piece, per block of 64 pieces (a wave's pieces of one turn), blocks
                // in ascending order: the order of k3q_rmsnorm.  The reduction buffers are free until
                // the first group ends.
                float* blk = (float*)red;  // [M][blocks per row], then [M] reciprocal root mean squares
                const int per_row = K >> 3, nblk = per_row >> 6;
#pragma unroll
                for (int i = 0; i < kNP; ++i) {
                    const int first = tid + i * kT - lane;
                    if (first < pieces) {
                        const float ss = wave_sum(piece_sum_squares(xr[i]));
                        const int m = (int)__umulhi((u32)first, (u32)p.row_magic);
                        if (lane == 0) blk[m * nblk + ((first - m * per_row) >> 6)] = ss;
                    }
                }
                __syncthreads();
                float* rstd = blk + M * nblk;
                if (tid < M) {
                    float total = 0.f;
                    for (int b = 0; b < nblk; ++b) total += blk[tid * nblk + b];
                    rstd[tid] = 1.0f / sqrtf(total / (float)K + p.pre_eps);
                }
                __syncthreads();
#pragma unroll
                for (int i = 0; i < kNP; ++i) {
                    const int pi = tid + i * kT;
                    if (pi < pieces)
                        xr[i] = piece_rms_scale(xr[i], xop[i], rstd[(int)__umulhi((u32)pi, (u32)p.row_magic)]);
                }
            } else {
#pragma unroll
                for (int i = 0; i < kNP; ++i) xr[i] = piece_silu_mul(xop[i], xr[i]);
            }
        }
        auto piece_amax = [](const v4u& c) {
            float a = 0.f;
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                a = fmaxf(a, fabsf(__uint_as_float(c[e] << 16)));
                a = fmaxf(a, fabsf(__uint_as_float(c[e] & 0xffff0000u)));
            }
            return a;
        };
        // a wave's 64 consecutive pieces lie in one row (K % 512 == 0): one LDS atomic per wave and turn
        auto fold_amax = [&](int pi, float a) {
            a = wave_max(a);
            const int row = (int)__umulhi((u32)(pi < pieces ? pi : pieces - 1), (u32)p.row_magic);
            if (lane == 0 && pi < pieces) atomicMax(rowmax + row, __float_as_uint(a));
        };
        if (kNP > 0) {
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                const int pi = tid + i * kT;
                if (pi - lane < pieces) fold_amax(pi, piece_amax(xr[i]));
            }
        } else {
            for (int base = 0; base < pieces; base += kT) {
                const int pi = base + tid;
                const v4u c = ((const v4u*)p.x)[pi < pieces ? pi : pieces - 1];
                if (pi - lane < pieces) fold_amax(pi, piece_amax(c));
            }
        }
        __syncthreads();
        if (tid < M) sa[tid] = scale_from_amax_bf16(__uint_as_float(rowmax[tid]), p.eps, p.qhi);
        __syncthreads();
        // (quantize_piece_bf16: the clip before the rounding, exact between the integer ends of the range
        // that the entry point insists on)
        auto quantize_piece = [&](int pi, const v4u& c) {
            const int row = (int)__umulhi((u32)pi, (u32)p.row_magic);
            const int col = (pi - row * (K >> 3)) << 3;
            *(v2u*)(xs + row * pitch + col) = quantize_piece_bf16(c, sa[row], p.qlo, p.qhi);
        };
        if (kNP > 0) {
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                const int pi = tid + i * kT;
                if (pi < pieces) quantize_piece(pi, xr[i]);
            }
        } else {
            for (int base = 0; base < pieces; base += kT) {
                const int pi = base + tid;
                const v4u c = ((const v4u*)p.x)[pi < pieces ? pi : pieces - 1];
                if (pi < pieces) quantize_piece(pi, c);
            }
        }
    }
    __syncthreads();

    // ---- groups of strips ----
    const int i16 = lane & 15, g = lane >> 4;
    const bool row_live = i16 < M;
    const char* xrow = xs + (row_live ? i16 : 0) * pitch + 16 * g;
    const bool has_bias = p.bias != nullptr;
    int turn = 0;
    for (int grp = block; grp < p.groups; grp += stride, ++turn) {
        // epilogue operands of this group, asked for before the group's units (loads return in
        // order: asked for late they would wait for the next group's first units)
        const int n0 = place(grp) * kSW * 16;
        u32 sb_raw[kSW], bias_raw[kSW][4];
#pragma unroll
        for (int t = 0; t < kSW; ++t) {
            const int n = n0 + t * 16 + i16;
            const int nn = n < p.N ? n : p.N - 1;
            sb_raw[t] = p.scale[nn];
            const uint16_t* bp = has_bias ? p.bias : p.scale;
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                const int m = 4 * g + r;
                bias_raw[t][r] = bp[(has_bias && m < M ? (int64_t)m * p.bias_stride : 0) + nn];
            }
        }
        v4i acc[kSW];
#pragma unroll
        for (int t = 0; t < kSW; ++t) acc[t] = v4i{0, 0, 0, 0};
        v4i a_next = *(const v4i*)(xrow + u_begin * 64);
        for (int u = u_begin; u < u_begin + my_units; u += kD) {
#pragma unroll
            for (int d = 0; d < kD; ++d) {
                v4i a = a_next;
                if (!row_live) a = v4i{0, 0, 0, 0};
                // (the read past this wave's slice stays inside the row's padding or the next row)
                a_next = *(const v4i*)(xrow + (u + d + 1) * 64);
#pragma unroll
                for (int t = 0; t < kSW; ++t)
                    acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a, W[d][t], acc[t], 0, 0, 0);
                refill(d);
                __builtin_amdgcn_sched_barrier(0);  // the refill stays here: right behind its unit's last use
            }
            advance();
        }
        // ---- sum the waves' slices (exact integers), de-scale, store ----
        int* rbuf = red + (turn & 1) * red_one;
        if (g < mq) {
#pragma unroll
            for (int t = 0; t < kSW; ++t) *(v4i*)(rbuf + (((q * kSW + t) * mq + g) * 16 + i16) * 4) = acc[t];
        }
        __syncthreads();
        if (q < kSW && g < mq) {
            v4i tot = v4i{0, 0, 0, 0};
#pragma unroll
            for (int qq = 0; qq < kQ; ++qq) tot += *(const v4i*)(rbuf + (((qq * kSW + q) * mq + g) * 16 + i16) * 4);
            u32 sbq = sb_raw[0];
            u32 bq[4];
#pragma unroll
            for (int r = 0; r < 4; ++r) bq[r] = bias_raw[0][r];
#pragma unroll
            for (int t = 1; t < kSW; ++t) {
                if (q == t) {
                    sbq = sb_raw[t];
#pragma unroll
                    for (int r = 0; r < 4; ++r) bq[r] = bias_raw[t][r];
                }
            }
            const int n = n0 + q * 16 + i16;
            if (n < p.N) {
                const float sb = bf16_bits_to_f32(sbq);
#pragma unroll
                for (int r = 0; r < 4; ++r) {
                    const int m = 4 * g + r;
                    if (m < M) {
                        const float yv = descale_exact_bf16(tot[r], sa[m], sb, bf16_bits_to_f32(bq[r]), has_bias);
                        p.y[(int64_t)m * p.N + n] = (uint16_t)f32_to_bf16_bits(yv);
                    }
                }
            }
        }
        // (the next group's partials go to the other buffer: no second barrier)
    }
}

template <int kSW, int kD, int kNP>
__global__ __launch_bounds__(kT) void gemv_w8s(W8sParams p) {
    gemv_w8s_body<kSW, kD, kNP>(p, (int)blockIdx.x, (int)gridDim.x);
}

// Up to kMaxProblems8 kernels against one x in one launch (the query / key / value projections of
// an attention block, gate / up of an MLP): workgroups [first[i], first[i+1]) work on problem i,
// every workgroup stages (and, fused, quantises) x as in the single launch.
constexpr int kMaxProblems8 = 4;
struct W8sMulti {
    W8sParams p[kMaxProblems8];
    int first[kMaxProblems8 + 1];
    int count;
};
template <int kSW, int kD, int kNP>
__global__ __launch_bounds__(kT) void gemv_w8s_multi(W8sMulti mp) {
    const int bx = blockIdx.x;
    int i = 0;
    while (i + 1 < mp.count && bx >= mp.first[i + 1]) ++i;
    gemv_w8s_body<kSW, kD, kNP>(mp.p[i], bx - mp.first[i], mp.first[i + 1] - mp.first[i]);
}

template <int kSW, int kD, int kNP>
__global__ __launch_bounds__(kT) void gemv_w8s_pre(W8sMulti mp) {
    const int bx = blockIdx.x;
    int i = 0;
    while (i + 1 < mp.count && bx >= mp.first[i + 1]) ++i;
    gemv_w8s_body<kSW, kD, kNP, true>(mp.p[i], bx - mp.first[i], mp.first[i + 1] - mp.first[i]);
}

// One thread per 16-byte lane entry of the copy.  w: the stored int8 kernel, row-major [K, N].
__global__ __launch_bounds__(256) void w8s_pack(const int8_t* __restrict__ w, v4u* __restrict__ out, int64_t K,
                                               int64_t N, int64_t strips) {
    const int64_t t = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t units = K / 64;
    if (t >= strips * units * 64) return;
    const int lane = (int)(t & 63);
    const int64_t u = (t >> 6) % units, s = (t >> 6) / units;
    const int64_t n = s * 16 + (lane & 15);
    const int64_t k0 = u * 64 + (lane >> 4) * 16;
    v4u o = {0, 0, 0, 0};
    if (n < N) {
#pragma unroll
        for (int e = 0; e < 16; ++e) o[e >> 2] |= ((u32)(uint8_t)w[(k0 + e) * N + n]) << (8 * (e & 3));
    }
    out[t] = o;
}

int64_t strips_padded8(int64_t N) { return ((N + 15) / 16 + 1) / 2 * 2; }

struct W8sPlan {
    bool ok;
    int sw, d, np;
    int64_t groups, blocks;
    int64_t resident;  // workgroups of this kernel form the chip holds at once (256 or 512)
    size_t lds;
};

// shared: the plan is for a launch that several problems share
W8sPlan w8s_plan(int64_t M, int64_t K, int64_t N, bool shared = false) {
    W8sPlan pl{};
    // a wave's 64 pieces of x stay inside a row (K % 512), whole strips (N % 16)
    if (M < 1 || M > kMaxRows8 || K < 1024 || (K % 512) != 0 || (N % 16) != 0 || N < 16) return pl;
    const int64_t units = K / 64, strips = N / 16;
    if (strips < 192) return pl;  // all of K stays inside a workgroup: the strips alone fill the chip
    pl.d = (units / 4 >= 2 * kQ) ? 4 : 2;
    if ((units % pl.d) != 0 || units / pl.d < kQ) return pl;
    pl.sw = strips >= 2 * kResident8 ? 2 : 1;
    pl.resident = kResident8;
    // The kernels with few pieces of x per thread stay well within 128 registers, so two workgroups
    // fit a CU: a shared launch of up to 1024 strips per problem then runs one strip per wave on 512
    // resident workgroups (twice the requests in flight; x small enough for two workgroups' LDS).
    if (shared && strips < 4 * kResident8 && M * K / 8 <= 4 * kT &&
        (size_t)((M * (K + 16) + 255) & ~255) + 2 * kMaxRows8 * 4 + 2 * (size_t)kQ * ((M + 3) / 4) * 16 * 4 * 4 <= 80 * 1024) {
        pl.sw = 1;
        pl.resident = 2 * kResident8;
    }
    pl.groups = (strips + pl.sw - 1) / pl.sw;
    const int64_t turns = (pl.groups + pl.resident - 1) / pl.resident;
    pl.blocks = (pl.groups + turns - 1) / turns;
    const int64_t pieces = M * K / 8;
    pl.np = pieces <= kT ? 1 : pieces <= 4 * kT ? 4 : pieces <= 16 * kT ? 16 : 0;
    const size_t red_one = (size_t)kQ * pl.sw * ((M + 3) / 4) * 16 * 4 * 4;
    pl.lds = (size_t)((M * (K + 16) + 255) & ~255) + 2 * kMaxRows8 * 4 + (turns > 1 ? 2 : 1) * red_one;
    pl.ok = pl.lds <= 160 * 1024;
    return pl;
}

typedef void (*W8sKernel)(W8sParams);
typedef void (*W8sMultiKernel)(W8sMulti);

template <int kSW, int kD>
W8sKernel pick_np8(int np) {
    switch (np) {
        case -1: return gemv_w8s<kSW, kD, -1>;
        case 1: return gemv_w8s<kSW, kD, 1>;
        case 4: return gemv_w8s<kSW, kD, 4>;
        case 16: return gemv_w8s<kSW, kD, 16>;
        default: return gemv_w8s<kSW, kD, 0>;
    }
}

template <int kSW, int kD>
W8sMultiKernel pick_np8_multi(int np) {
    switch (np) {
        case -1: return gemv_w8s_multi<kSW, kD, -1>;
        case 1: return gemv_w8s_multi<kSW, kD, 1>;
        case 4: return gemv_w8s_multi<kSW, kD, 4>;
        case 16: return gemv_w8s_multi<kSW, kD, 16>;
        default: return gemv_w8s_multi<kSW, kD, 0>;
    }
}

template <int kSW, int kD>
W8sMultiKernel pick_np8_pre(int np) {
    switch (np) {
        case 1: return gemv_w8s_pre<kSW, kD, 1>;
        case 4: return gemv_w8s_pre<kSW, kD, 4>;
        case 16: return gemv_w8s_pre<kSW, kD, 16>;
        default: return nullptr;
    }
}

W8sMultiKernel pick_kernel8_pre(const W8sPlan& pl) {
    if (pl.sw == 2) return pl.d == 4 ? pick_np8_pre<2, 4>(pl.np) : pick_np8_pre<2, 2>(pl.np);
    return pl.d == 4 ? pick_np8_pre<1, 4>(pl.np) : pick_np8_pre<1, 2>(pl.np);
}

W8sMultiKernel pick_kernel8_multi(const W8sPlan& pl) {
    if (pl.sw == 2) return pl.d == 4 ? pick_np8_multi<2, 4>(pl.np) : pick_np8_multi<2, 2>(pl.np);
    return pl.d == 4 ? pick_np8_multi<1, 4>(pl.np) : pick_np8_multi<1, 2>(pl.np);
}

W8sKernel pick_kernel8(const W8sPlan& pl) {
    if (pl.sw == 2) return pl.d == 4 ? pick_np8<2, 4>(pl.np) : pick_np8<2, 2>(pl.np);
    return pl.d == 4 ? pick_np8<1, 4>(pl.np) : pick_np8<1, 2>(pl.np);
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int64_t k3q_w8s_shadow_bytes(int64_t K, int64_t N) {
    if (K <= 0 || N <= 0 || (K % 64) != 0) return 0;
    return strips_padded8(N) * (K / 64) * 1024;
}

extern "C" int k3q_w8s_pack(const int8_t* w, int64_t K, int64_t N, void* shadow, void* stream) {
    if (K <= 0 || N <= 0 || (K % 64) != 0) return K3Q_ERR_SHAPE;
    if (!w || !shadow) return K3Q_ERR_NULL;
    if (!aligned_to(shadow, 16)) return K3Q_ERR_ALIGN;
    const int64_t entries = k3q_w8s_shadow_bytes(K, N) / 16;
    w8s_pack<<<(unsigned)((entries + 255) / 256), 256, 0, (hipStream_t)stream>>>(w, (v4u*)shadow, K, N,
                                                                                 strips_padded8(N));
    return launch_status();
}

extern "C" int k3q_dense_i8_w8s_supported(int64_t M, int64_t K, int64_t N) { return w8s_plan(M, K, N).ok ? 1 : 0; }

namespace {
// checks the operands of one problem and fills its kernel parameters
int fill_params8(W8sParams& p, const W8sPlan& pl, const void* x, const int8_t* xq, const void* xs, int64_t M,
                 int64_t K, int64_t N, const void* shadow, const void* kernel_scale, const void* bias,
                 int64_t bias_stride, float epsilon, float range_lo, float range_hi, void* y) {
    if (bias_stride != 0 && bias_stride != N) return K3Q_ERR_SHAPE;
    const bool quantised = xq != nullptr;
    if (!(quantised ? (const void*)xs : x) || !shadow || !kernel_scale || !y) return K3Q_ERR_NULL;
    if (!aligned_to(quantised ? (const void*)xq : x, 16) || !aligned_to(shadow, 16) || !aligned_to(y, 2) ||
        !aligned_to(kernel_scale, 2) || (bias && !aligned_to(bias, 2)) || (xs && !aligned_to(xs, 2)))
        return K3Q_ERR_ALIGN;
    p.x = (const uint16_t*)x;
    p.xq = xq;
    p.xs = (const uint16_t*)xs;
    p.w = (const v4i*)shadow;
    p.scale = (const uint16_t*)kernel_scale;
    p.bias = (const uint16_t*)bias;
    p.y = (uint16_t*)y;
    p.bias_stride = bias ? bias_stride : 0;
    p.M = (int)M;
    p.K = (int)K;
    p.N = (int)N;
    p.units = (int)(K / 64);
    p.groups = (int)pl.groups;
    const uint64_t per_row = (uint64_t)K / (quantised ? 16 : 8);
    p.row_magic = (int)(uint32_t)((((uint64_t)1 << 32) + per_row - 1) / per_row);
    p.eps = host_round_bf16(epsilon);  // torch rounds the epsilon operand to the tensor dtype before the add
    p.qlo = range_lo;
    p.qhi = range_hi;
    return K3Q_OK;
}

// more than 64 KiB of dynamic LDS has to be allowed per kernel, once
int raise_lds(const void* kernel) {
    static std::mutex mu;
    static std::set<const void*> raised;
    std::lock_guard<std::mutex> lock(mu);
    if (!raised.count(kernel)) {
        if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
            return K3Q_ERR_LAUNCH;
        raised.insert(kernel);
    }
    return K3Q_OK;
}

int launch_w8s(const void* x, const int8_t* xq, const void* xs, int64_t M, int64_t K, int64_t N,
               const void* shadow, const void* kernel_scale, const void* bias, int64_t bias_stride,
               float epsilon, float range_lo, float range_hi, void* y, hipStream_t stream) {
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    W8sPlan pl = w8s_plan(M, K, N);
    if (!pl.ok) return K3Q_ERR_SHAPE;
    W8sParams p;
    int rc = fill_params8(p, pl, x, xq, xs, M, K, N, shadow, kernel_scale, bias, bias_stride, epsilon, range_lo,
                          range_hi, y);
    if (rc != K3Q_OK) return rc;
    if (xq) pl.np = -1;
    const W8sKernel kernel = pick_kernel8(pl);
    if ((rc = raise_lds((const void*)kernel)) != K3Q_OK) return rc;
    kernel<<<(unsigned)pl.blocks, kT, pl.lds, stream>>>(p);
    return launch_status();
}
}  // namespace

extern "C" int k3q_dense_i8_w8s(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N, const void* shadow,
                                const void* kernel_scale, const void* bias, int64_t bias_stride, float epsilon,
                                float range_lo, float range_hi, void* y, void* stream) {
    if (x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (!(range_lo >= -128.f && range_hi <= 127.f && range_lo < range_hi)) return K3Q_ERR_SHAPE;
    // (the in-kernel quantizer clips before it rounds: exact only between integer ends)
    if (range_lo != rintf(range_lo) || range_hi != rintf(range_hi)) return K3Q_ERR_RANGE;
    return launch_w8s(x, nullptr, nullptr, M, K, N, shadow, kernel_scale, bias, bias_stride, epsilon, range_lo,
                      range_hi, y, (hipStream_t)stream);
}

extern "C" int k3q_gemm_i8_w8s(const int8_t* a, const void* a_scale, int scale_dtype, int64_t M, int64_t K,
                               int64_t N, const void* shadow, const void* kernel_scale, const void* bias,
                               int64_t bias_stride, void* y, void* stream) {
    if (scale_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M > 0 && !a) return K3Q_ERR_NULL;
    return launch_w8s(nullptr, a, a_scale, M, K, N, shadow, kernel_scale, bias, bias_stride, 0.f, -127.f, 127.f,
                      y, (hipStream_t)stream);
}

namespace {
int w8s_run_shared(const void* x, int x_dtype, const int8_t* a, const void* a_scale, int64_t M, int64_t K,
                   const k3q_input_op* pre, int count, const k3q_w8s_problem* problems, float epsilon,
                   float range_lo, float range_hi, bool bias_rows, void* stream) {
    if (x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (count < 0 || M < 0 || K <= 0) return K3Q_ERR_SHAPE;
    if (!(range_lo >= -128.f && range_hi <= 127.f && range_lo < range_hi)) return K3Q_ERR_SHAPE;
    // (the in-kernel quantizer clips before it rounds: exact only between integer ends)
    if (range_lo != rintf(range_lo) || range_hi != rintf(range_hi)) return K3Q_ERR_RANGE;
    if (count == 0 || M == 0) return K3Q_OK;
    if (!problems) return K3Q_ERR_NULL;
    const bool has_pre = pre != nullptr && pre->kind != K3Q_INPUT_NONE;
    if (has_pre) {
        if (a || !x) return K3Q_ERR_NULL;  // the transform works on bfloat16 rows
        if (pre->kind != K3Q_INPUT_RMS_NORM && pre->kind != K3Q_INPUT_SILU_GATE) return K3Q_ERR_SHAPE;
        if (!pre->operand) return K3Q_ERR_NULL;
        if (!aligned_to(pre->operand, 16)) return K3Q_ERR_ALIGN;
    }
    int at = 0;
    while (at < count) {
        // problems whose plans agree share a launch, up to kMaxProblems8 at a time
        W8sMulti mp{};
        W8sPlan pl0{};
        int64_t groups[kMaxProblems8], total = 0;
        size_t lds_two = 0, lds_red_one = 0;
        int n = 0;
        for (; at + n < count && n < kMaxProblems8; ++n) {
            const k3q_w8s_problem& q = problems[at + n];
            if (q.N <= 0) return K3Q_ERR_SHAPE;
            const W8sPlan pl = w8s_plan(M, K, q.N, count >= 2);
            if (!pl.ok) return K3Q_ERR_SHAPE;
            if (n == 0) {
                pl0 = pl;
                // workgroups of a shared launch may take turns even where a problem alone would not
                lds_red_one = (size_t)kQ * pl.sw * ((M + 3) / 4) * 16 * 4 * 4;
                lds_two = (size_t)((M * (K + 16) + 255) & ~255) + 2 * kMaxRows8 * 4 + 2 * lds_red_one;
            } else if (pl.sw != pl0.sw || pl.d != pl0.d || pl.resident != pl0.resident) {
                break;
            }
            const int rc = fill_params8(mp.p[n], pl, x, a, a_scale, M, K, q.N, q.shadow, q.kernel_scale, q.bias,
                                        bias_rows ? q.N : 0, epsilon, range_lo, range_hi, q.y);
            if (rc != K3Q_OK) return rc;
            if (has_pre) {
                // the pieces stay in registers, and the block sums fit the first reduction buffer
                if (pl.np <= 0 || M * (K / 512 + 1) > 512 * ((M + 3) / 4) * pl.sw) return K3Q_ERR_SHAPE;
                mp.p[n].pre_kind = pre->kind;
                mp.p[n].pre_eps = pre->epsilon;
                mp.p[n].pre_op = (const uint16_t*)pre->operand;
            }
            groups[n] = pl.groups;
            total += pl.groups;
        }
        // the launch as a whole is cut for the chip: about kResident8 workgroups, each problem its share;
        // workgroups that take turns need both reduction buffers, and where those do not fit beside x
        // the first problem goes alone, with its own plan
        int64_t turns = (total + pl0.resident - 1) / pl0.resident;
        size_t lds = turns > 1 ? lds_two : lds_two - lds_red_one;
        if (lds > (size_t)160 * 1024) {
            n = 1;
            turns = (groups[0] + pl0.resident - 1) / pl0.resident;
            lds = pl0.lds;
        }
        int next_block = 0;
        for (int i = 0; i < n; ++i) {
            mp.first[i] = next_block;
            next_block += (int)((groups[i] + turns - 1) / turns);
        }
        mp.first[n] = next_block;
        mp.count = n;
        if (a) pl0.np = -1;
        int rc;
        if (has_pre) {
            const W8sMultiKernel kernel = pick_kernel8_pre(pl0);
            if (!kernel) return K3Q_ERR_SHAPE;
            if ((rc = raise_lds((const void*)kernel)) != K3Q_OK) return rc;
            kernel<<<(unsigned)next_block, kT, lds, (hipStream_t)stream>>>(mp);
        } else if (n == 1) {
            const W8sKernel kernel = pick_kernel8(pl0);
            if ((rc = raise_lds((const void*)kernel)) != K3Q_OK) return rc;
            kernel<<<(unsigned)next_block, kT, lds, (hipStream_t)stream>>>(mp.p[0]);
        } else {
            const W8sMultiKernel kernel = pick_kernel8_multi(pl0);
            if ((rc = raise_lds((const void*)kernel)) != K3Q_OK) return rc;
            kernel<<<(unsigned)next_block, kT, lds, (hipStream_t)stream>>>(mp);
        }
        if ((rc = launch_status()) != K3Q_OK) return rc;
        at += n;
    }
    return K3Q_OK;
}
}  // namespace

extern "C" int k3q_dense_i8_w8s_multi(const void* x, int x_dtype, const int8_t* a, const void* a_scale, int64_t M,
                                      int64_t K, int count, const k3q_w8s_problem* problems, float epsilon,
                                      float range_lo, float range_hi, void* stream) {
    return w8s_run_shared(x, x_dtype, a, a_scale, M, K, nullptr, count, problems, epsilon, range_lo, range_hi, false,
                          stream);
}

extern "C" int k3q_dense_i8_w8s_pre(const void* x, int x_dtype, int64_t M, int64_t K, const k3q_input_op* pre,
                                    int count, const k3q_w8s_problem* problems, float epsilon, float range_lo,
                                    float range_hi, int bias_rows, void* stream) {
    return w8s_run_shared(x, x_dtype, nullptr, nullptr, M, K, pre, count, problems, epsilon, range_lo, range_hi,
                          bias_rows != 0, stream);
}
