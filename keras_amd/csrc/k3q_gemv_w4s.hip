// Weight-only int4 decode matmul from a strip-linear copy of the kernel: y[M,N] = x[M,K] . W4[K,N], M <= 16.
//
// The layer's stored kernel ([K, ceil(N/2)] bytes, two output columns per byte) makes a workgroup
// read 128-byte pieces at a 4 KiB stride and needs a split of K over workgroups to fill the chip.
// This kernel reads a second copy, laid out for the decode access pattern and made once per layer
// (k3q_w4s_pack):
//
//   [strip = n / 16][unit = k / 128][lane = 64][dword = 4]            1 KiB per (strip, unit)
//   lane = i + 16 g holds column n = 16 strip + i; its dword s holds the 8 nibbles of
//   k = 128 unit + 32 s + 8 g + e, e = 2t at bits [4t, 4t + 4), e = 2t + 1 at bits [16 + 4t, ...).
//
// A wave's 16-byte-per-lane load of one unit is then 1 KiB of contiguous memory AND, dword by
// dword, the A operand of four v_mfma_f32_16x16x32_bf16 steps: ((d >> 4t) & 0x000F000F) ^ 0x43084308
// is the bfloat16 pair (136 + w[k = ..2t], 136 + w[k = ..2t+1]) of column i.  A strip's units follow
// each other in memory, so a wave streams a contiguous run and a workgroup (one or two strips, all
// of K) a contiguous region; nothing is exchanged between workgroups, no partial sums leave the CU.
//
// x is staged once per workgroup in LDS (rows padded by 16 bytes: the sixteen lanes of a B-operand
// read then hit disjoint banks) and read back as MFMA B operands, reused for both strips of a wave.
// An all-ones A operand accumulates the sum of x over the same k, which removes the +136 offset
// (grouped: the zero point as well, per group of 128 = one unit).
//
// Scheduling facts this kernel is built on (measured on MI355X):
//  * the waits the compiler places around loads that are issued conditionally, or around LDS-DMA
//    mixed with register loads, drain the whole queue: every load here is unconditional (addresses
//    clamped instead) and goes through registers;
//  * a slot of the weight ring is refilled right after its conversion, which is interleaved with the
//    previous unit's MFMAs (sched_group_barrier), so that the request stream never waits for the
//    matrix pipe;
//  * x is requested before any weight: requested after them it would arrive behind the whole first
//    burst of weights (the memory system serves a launch's first requests roughly in order).
#include "k3q_common.h"

#include <mutex>
#include <set>
#include <type_traits>

namespace k3q {
namespace {

constexpr int kQ = 8;            // waves per workgroup = slices of K
constexpr int kT = kQ * 64;      // threads
constexpr int kMaxRows = 16;     // rows of x
constexpr int kMaxPieces = 16;   // 16-byte pieces of x a thread stages: M * K <= 16 * 8 * kT
constexpr int kRedStride = 20;   // floats per (row, strip) line of the cross-wave reduction
constexpr int kMaxProblems = 4;

struct W4sParams {
    const uint16_t* x;       // [M, K] bf16
    const v4u* w;            // strip-linear copy
    const uint16_t* scale;   // per-channel: bf16 [N]
    const uint8_t* gparams;  // grouped/128: [strip][unit][4][{4 bf16 scales, 4 (zero + 128)}] = 48 B
    const uint16_t* bias;    // bf16 [N] or [M, N], or null
    uint16_t* y;             // [M, N] bf16
    int64_t bias_stride;     // 0 or N
    int M, K, N, units;      // units = K / 128
    int row_magic;           // ceil(2^32 / pieces per staged row): piece -> row without a division
    int slice_magic;         // (x staged in two parts) ceil(2^32 / pieces of a slice's first part); row_magic: of a row's
    int row_magic2, slice_magic2;  // the same for the second part
    int own_magic[2];        // (waves stage their own slices) ceil(2^32 / pieces per row of a slice): short, long slice
    int own;                 // 1: every wave stages its own slice of x; 0: the workgroup's threads share all of x
    // an operation on x on its way into LDS (kernels built with kPre only):
    int pre_kind;             // 1: rms_norm(x) * pre_op (bf16 [K]); 2: silu(pre_op) * x (pre_op bf16 [M, K])
    float pre_eps;            // rms_norm's epsilon
    const uint16_t* pre_op;
};

struct W4sMulti {
    W4sParams p[kMaxProblems];
    int first[kMaxProblems + 1];  // first blockIdx.x of each problem, then the end
    int count;
};

__device__ __forceinline__ v8bf as_bf8(const v4u& v) { return __builtin_bit_cast(v8bf, v); }
__device__ __forceinline__ float bf_lo(u32 d) { return __uint_as_float(d << 16); }
__device__ __forceinline__ float bf_hi(u32 d) { return __uint_as_float(d & 0xffff0000u); }

// kSW strips per wave (2: the x fragments serve two strips), ring of kD units (2 or 4), kNP staged
// pieces of x per thread, kGrouped: groups of 128 with zero points.
// A workgroup takes strip groups `block`, `block + stride`, ... one after the other as ONE stream of
// units: the ring runs across the boundary (the last bodies of a group convert and request the
// first units of the next), so that a workgroup pays the memory latency once, not once per group.
// kHalves: x does not fit LDS as a whole (9 ... 16 rows of a long K): every wave's slice is cut in two,
// LDS holds the first halves, then -- once every wave is through with them -- the second halves
// (one turn per workgroup only: the launch plan sees to it).
// kPre: x is transformed on its way into LDS (p.pre_kind): the rows are normalised (rms_norm with a
// gain, as k3q_rmsnorm does, same bits) or multiplied by silu of a second input (as k3q_silu_mul).
// Every workgroup repeats the transform on all of x -- a few hundred float operations per thread,
// against a launch and a round trip through memory for the separate kernel.
template <int kSW, int kD, int kNP, bool kGrouped, bool kHalves, bool kPre = false>
__device__ __forceinline__ void gemv_w4s_body(const W4sParams& p, const int block, const int stride) {
    extern __shared__ __attribute__((aligned(16))) char w4s_lds[];
    const int tid = threadIdx.x, lane = tid & 63;
    const int q = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int units = p.units;
    const int M = p.M, K = p.K;
    const int j = lane & 15, g = lane >> 4;
    const int jj = j < M ? j : M - 1;
    const int groups = (p.N / 16 + kSW - 1) / kSW;
    // slices of K: whole blocks of kD units, the first (blocks % kQ) waves take one more
    const int blocks = units / kD;
    const int base = blocks / kQ, extra = blocks - base * kQ;
    const int U = (base + (q < extra ? 1 : 0)) * kD;
    const int u0 = (q * base + (q < extra ? q : extra)) * kD;
    const int R = U / kD;  // >= 2 (the launch plan sees to it)
    // kHalves: LDS holds the first Rh rounds' worth of every wave's slice, then the rest (the two parts
    // are equal when the slice has an even number of rounds)
    const int Rh = kHalves ? (R + 1) / 2 : R;
    const int Uh = Rh * kD;    // units of a slice whose x is in LDS at a time (the first part)
    const int Uh2 = U - Uh;    // (kHalves) the second part
    const int pitch = (kHalves ? kQ * Uh * 256 : K * 2) + 16;
    // (two buffers, one per parity of the turn, when a workgroup takes several turns)
    float* red = (float*)(w4s_lds + ((M * pitch + 255) & ~255));

    // ---- x into registers first (every load unconditional: pieces past the end re-read piece 0) ----
    // Whole rows (kHalves: half h of every wave's slice, row m = [slice 0 | slice 1 | ...]), spread over
    // the workgroup's threads -- or, for a small x (p.own), every wave loads and stores ITS OWN slice of
    // every row, the only part of x it reads back: nothing is exchanged between waves then, and no
    // barrier stands between a wave's x (the oldest requests in its queue) and its first weights.
    // (Measured: worth 0.3 us up to 32 KiB of x, a loss beyond.)
    static_assert(!(kPre && kHalves), "no transform of x staged in halves");
    const bool own = !kHalves && !kPre && p.own;
    const int per_row = own ? U * 16 : K >> 3;  // (kHalves: per part, below)
    const int pieces = M * per_row;
    const u32 row_magic = own ? (u32)p.own_magic[q < extra ? 1 : 0] : (u32)p.row_magic;
    const int own_col = own ? u0 * 16 : 0;  // first piece of the wave's slice within a row
    const int row_pieces = K >> 3;
    v4u xst[kNP];
    v4u xop[kPre ? kNP : 1];
    auto stage_load = [&](const int h) {
        if constexpr (kHalves) {
            // part h of every wave's slice: row m of LDS = [slice 0's part | slice 1's part | ...]
            const int uw = h ? Uh2 : Uh, part_row = kQ * uw * 16, part_pieces = M * part_row;
            const u32 rm = (u32)(h ? p.row_magic2 : p.row_magic), sm = (u32)(h ? p.slice_magic2 : p.slice_magic);
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                int pi = i * kT + tid;
                pi = pi < part_pieces ? pi : 0;
                const int m = (int)__umulhi((unsigned)pi, rm);
                const int c = pi - m * part_row;
                const int qq = (int)__umulhi((unsigned)c, sm);  // c / (uw * 16): the slice
                const int cc = c - qq * (uw * 16);
                xst[i] = *(const v4u*)(p.x + (int64_t)m * K + (int64_t)(qq * U + (h ? Uh : 0)) * 128 + cc * 8);
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < kNP; ++i) {
            int pi = own ? i * 64 + lane : i * kT + tid;
            pi = pi < pieces ? pi : 0;
            const int m = (int)__umulhi((unsigned)pi, row_magic);
            const int c = pi - m * per_row;
            {
                xst[i] = *(const v4u*)(p.x + ((int64_t)m * row_pieces + own_col + c) * 8);
                if constexpr (kPre)  // the gain's piece of this column, or the second input's piece
                    xop[i] = *(const v4u*)(p.pre_op + (p.pre_kind == 1 ? (int64_t)c : (int64_t)m * row_pieces + c) * 8);
            }
        }
    };
    auto stage_store = [&](const int h) {
        if constexpr (kHalves) {
            const int part_row = kQ * (h ? Uh2 : Uh) * 16, part_pieces = M * part_row;
            const u32 rm = (u32)(h ? p.row_magic2 : p.row_magic);
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                const int pi = i * kT + tid;
                if (pi < part_pieces) {
                    const int m = (int)__umulhi((unsigned)pi, rm);
                    *(v4u*)(w4s_lds + m * pitch + (pi - m * part_row) * 16) = xst[i];
                }
            }
            return;
        }
#pragma unroll
        for (int i = 0; i < kNP; ++i) {
            const int pi = own ? i * 64 + lane : i * kT + tid;
            if (pi < pieces) {
                const int m = (int)__umulhi((unsigned)pi, row_magic);
                const int c = pi - m * per_row;
                *(v4u*)(w4s_lds + m * pitch + (own_col + c) * 16) = xst[i];
            }
        }
    };
    stage_load(0);
    __builtin_amdgcn_sched_barrier(0);
    // weights and grouped parameters of a strip group at this wave's slice: wave-uniform bases (scalar
    // registers), the lane's part is added at the load
    // Strip groups are dealt to the XCDs in rotation (XCD x takes group 8 i + (x + i) % 8 instead of
    // x + 8 i): with the plain order an XCD's whole stream has the three address bits above the group
    // size fixed, and where those are bits 18 ... 23 it sits on a fraction of the memory channels (a
    // read-only launch of 256 KiB chunks: 12.1 us against 11.4 rotated).  Measured here: two strips
    // per wave gain (gate + up of 4096 x 14336: 10.2 -> 9.6 us), one strip per wave loses 0.3 us,
    // so only the former rotate.
    const bool rotate = kSW == 2;
    auto place = [&](const int gi) {
        return rotate && (gi | 7) < groups ? (gi & ~7) | ((gi + (gi >> 3)) & 7) : gi;
    };
    auto w_base = [&](const int grp, const int t) {
        return (const char*)p.w + ((int64_t)(place(grp) * kSW + t) * units + u0) * 1024;
    };
    auto z_base = [&](const int grp, const int t) {
        return (const char*)p.gparams + ((int64_t)(place(grp) * kSW + t) * units + u0) * 48;
    };
    const unsigned lane_w = lane * 16u, lane_z = 12u * g;  // (unsigned: a scalar base + a 32-bit lane offset is one address form)
    // The weight stream of a wave: unit after unit of its slice, group after group of the workgroup.
    // The cursor (group, unit) is where the next request goes; the ring is refilled in stream order,
    // so a request needs no index, and the stream may run any number of groups ahead of the sums (a
    // slice as short as the ring is one round per group).  Past the workgroup's last group the cursor
    // stays on it: requested, never used.
    int cg = block, cu = 0;
    const char* cw[kSW];  // where the next request of a strip goes: advanced by a unit per request
    const char* cz[kSW];
    auto at_group = [&]() {
#pragma unroll
        for (int t = 0; t < kSW; ++t) {
            cw[t] = w_base(cg, t);
            cz[t] = z_base(cg, t);
        }
    };
    at_group();
    v4u W[kD][kSW];
    u32 Z[kGrouped ? kD : 1][kSW][3];
    auto fetch = [&](const int d) {
#pragma unroll
        for (int t = 0; t < kSW; ++t) {
            W[d][t] = __builtin_nontemporal_load((const v4u*)(cw[t] + lane_w));
            cw[t] += 1024;
        }
        if constexpr (kGrouped) {
#pragma unroll
            for (int t = 0; t < kSW; ++t) {
                const u32* z = (const u32*)(cz[t] + lane_z);
                Z[d][t][0] = z[0];
                Z[d][t][1] = z[1];
                Z[d][t][2] = z[2];
                cz[t] += 48;
            }
        }
        if (++cu == U) {
            cu = 0;
            cg = cg + stride < groups ? cg + stride : cg;
            at_group();
        }
    };
#pragma unroll
    for (int d = 0; d < kD; ++d) fetch(d);
    __builtin_amdgcn_sched_barrier(0);
    if constexpr (kPre) {
        if (p.pre_kind == 1) {
            // sums of squares: per piece, per block of 64 pieces (a wave's pieces of one turn: K % 512 == 0),
            // blocks in ascending order -- the order of k3q_rmsnorm
            float* blk = red;  // [M][blocks per row], then [M] reciprocal root mean squares
            const int nblk = per_row >> 6;
#pragma unroll
            for (int i = 0; i < kNP; ++i) {
                const int first = i * kT + tid - lane;
                if (first < pieces) {
                    const float ss = wave_sum(piece_sum_squares(xst[i]));
                    const int m = (int)__umulhi((unsigned)first, row_magic);
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
                const int pi = i * kT + tid;
                if (pi < pieces) xst[i] = piece_rms_scale(xst[i], xop[i], rstd[(int)__umulhi((unsigned)pi, row_magic)]);
            }
        } else {
#pragma unroll
            for (int i = 0; i < kNP; ++i) xst[i] = piece_silu_mul(xop[i], xst[i]);
        }
    }
    // ---- x into LDS: the stores wait for the x loads only (they are the older ones) ----
    stage_store(0);
    if (!own) __syncthreads();  // (own slices: a wave reads back only what it wrote itself)

    const char* xrow = w4s_lds + jj * pitch + (kHalves ? q * Uh : u0) * 256 + g * 16;  // (kHalves: of the part in LDS)
    const v4u ones = {0x3F803F80u, 0x3F803F80u, 0x3F803F80u, 0x3F803F80u};
    const v4f zero4 = {0.f, 0.f, 0.f, 0.f};
    // (three MFMAs per step with kSW = 2, two with one strip: a strip's own chain has the others between
    // its links, which is enough for the matrix pipe's latency)
    v4f acc[2][kSW], accs[2], tot[kSW];
    u32 Zk[2][kSW][3];
    v4u av[2][kSW][4], xf[2][4];

    auto cvt1 = [&](const u32 w, v4u& out) {
#pragma unroll
        for (int e = 0; e < 4; ++e) out[e] = ((w >> (4 * e)) & 0x000F000Fu) ^ 0x43084308u;
    };
    auto read_x = [&](const int b, const int i) {
#pragma unroll
        for (int s = 0; s < 4; ++s) xf[b][s] = *(const v4u*)(xrow + i * 256 + s * 64);
    };
    // grouped: tot += scale * (acc - (136 + zero) * sum(x)) for the unit in buffers a
    auto fold = [&](const int a) {
#pragma unroll
        for (int t = 0; t < kSW; ++t)
#pragma unroll
            for (int r = 0; r < 4; ++r) {
                // (136 + zero) * sum(x) = (zero + 128) * sum(x) + 8 * sum(x); the byte converts in one operation
                const float sc = (r & 1) ? bf_hi(Zk[a][t][r >> 1]) : bf_lo(Zk[a][t][r >> 1]);
                const float zu = (float)((Zk[a][t][2] >> (8 * r)) & 0xffu);
                const float d = __builtin_fmaf(-zu, accs[a][r], acc[a][t][r] - 8.0f * accs[a][r]);
                tot[t][r] = __builtin_fmaf(sc, d, tot[t][r]);
            }
    };
    // Unit i of the group (slot d, buffers b = d & 1): its MFMAs, interleaved with the conversion of
    // the unit after it (slot dn; after the group's last unit: the next group's first).  Halfway, the
    // fold of unit i - 1, whose MFMAs are long done; after it that unit's parameter buffer takes those
    // of the unit after.  Then slot dn is requested again: unit i + 1 + kD, from the next group if past
    // the end of this one.
    // x_later: the unit after this one needs the other half of x: its fragments are read by the caller
    auto body = [&](auto d_c, const int i, auto has_next_c, auto do_refill_c, const bool fold_prev,
                    auto x_later_c) {
        constexpr int d = decltype(d_c)::value;
        constexpr bool has_next = decltype(has_next_c)::value, do_refill = decltype(do_refill_c)::value;
        constexpr bool x_later = decltype(x_later_c)::value;
        constexpr int b = d & 1, dn = (d + 1) % kD;
        constexpr int ab = kGrouped ? b : 0;
        if (has_next && !x_later) {
            int nx = i + 1 < U ? i + 1 : 0;
            if (kHalves) nx = nx >= Uh ? nx - Uh : nx;
            read_x(b ^ 1, nx);
        }
#pragma unroll
        for (int s = 0; s < 4; ++s) {
            const bool fresh = kGrouped && s == 0;  // (constant once unrolled)
            accs[ab] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(as_bf8(ones), as_bf8(xf[b][s]),
                                                               fresh ? zero4 : accs[ab], 0, 0, 0);
#pragma unroll
            for (int t = 0; t < kSW; ++t)
                acc[ab][t] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                    as_bf8(av[b][t][s]), as_bf8(xf[b][s]), fresh ? zero4 : acc[ab][t], 0, 0, 0);
            if (has_next) {
#pragma unroll
                for (int t = 0; t < kSW; ++t) cvt1(W[dn][t][s], av[b ^ 1][t][s]);
            }
            if (s == 1) {
                if (kGrouped && fold_prev) fold(b ^ 1);
                if constexpr (kGrouped && has_next) {
#pragma unroll
                    for (int t = 0; t < kSW; ++t)
#pragma unroll
                        for (int c = 0; c < 3; ++c) Zk[b ^ 1][t][c] = Z[dn][t][c];
                }
            }
        }
        if (has_next) {
            // per step: (1 + kSW) MFMAs against 7 kSW conversions
#pragma unroll
            for (int k = 0; k < 4; ++k) {
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kSW == 2 ? 5 : 4, 0);
                __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                __builtin_amdgcn_sched_group_barrier(0x002, kSW == 2 ? 5 : 3, 0);
                if (kSW == 2) {
                    __builtin_amdgcn_sched_group_barrier(0x008, 1, 0);
                    __builtin_amdgcn_sched_group_barrier(0x002, 4, 0);
                }
            }
        }
        __builtin_amdgcn_sched_barrier(0);
        if (do_refill) fetch(dn);
        __builtin_amdgcn_sched_barrier(0);
    };
    using std::bool_constant;
    using std::integral_constant;
    // last: last round of the last group, nothing follows; turn_c: last round on the first half of x
    auto round = [&](auto last_c, const int r, auto turn_c) {
        constexpr bool last = decltype(last_c)::value;
        const bool_constant<false> no{};
        const int i0 = r * kD;
        body(integral_constant<int, 0>{}, i0, bool_constant<true>{}, bool_constant<!last>{}, r > 0, no);
        if constexpr (kD == 2) {
            body(integral_constant<int, 1>{}, i0 + 1, bool_constant<!last>{}, bool_constant<!last>{}, true, turn_c);
        } else {
            body(integral_constant<int, 1>{}, i0 + 1, bool_constant<true>{}, bool_constant<!last>{}, true, no);
            body(integral_constant<int, 2>{}, i0 + 2, bool_constant<true>{}, bool_constant<!last>{}, true, no);
            body(integral_constant<int, 3>{}, i0 + 3, bool_constant<!last>{}, bool_constant<!last>{}, true, turn_c);
        }
    };

    // prologue: unit 0 converted, its x fragments read, its slot requested again
    read_x(0, 0);
#pragma unroll
    for (int t = 0; t < kSW; ++t)
#pragma unroll
        for (int s = 0; s < 4; ++s) cvt1(W[0][t][s], av[0][t][s]);
    if constexpr (kGrouped) {
#pragma unroll
        for (int t = 0; t < kSW; ++t)
#pragma unroll
            for (int c = 0; c < 3; ++c) Zk[0][t][c] = Z[0][t][c];
    }
    __builtin_amdgcn_sched_barrier(0);
    fetch(0);
    __builtin_amdgcn_sched_barrier(0);

    u32 esc[kSW][2], ebi[kSW][2];
    // a group's set-up: where the group after it lies, fresh sums, and the epilogue's operands
    // requested now rather than at the end of the group's stream
    auto begin = [&](const int grp, const int nxt_grp) {
#pragma unroll
        for (int t = 0; t < kSW; ++t) tot[t] = zero4;
        if (!kGrouped) {  // (grouped: every unit starts its own accumulators)
            accs[0] = zero4;
#pragma unroll
            for (int t = 0; t < kSW; ++t) acc[0][t] = zero4;
        }
#pragma unroll
        for (int t = 0; t < kSW; ++t) {
            int n = (place(grp) * kSW + t) * 16 + 4 * g;
            n = n < p.N ? n : p.N - 4;  // N % 16 == 0: a valid stand-in, never stored
            esc[t][0] = esc[t][1] = 0;
            if (!kGrouped) {
                const v2u v = *(const v2u*)(p.scale + n);
                esc[t][0] = v[0];
                esc[t][1] = v[1];
            }
            // (no bias: the load still happens, from x, and is ignored -- a branch around a load costs
            // the loads behind it their place in the compiler's wait counts)
            const uint16_t* src = p.bias ? p.bias + (int64_t)jj * p.bias_stride + n : p.x;
            const v2u v = *(const v2u*)src;
            ebi[t][0] = v[0];
            ebi[t][1] = v[1];
        }
        __builtin_amdgcn_sched_barrier(0);
    };
    // a group's end: the slices of K meet in LDS, wave t adds them up for strip t (ascending order of the
    // waves, its own sums from its registers) and applies the layer's epilogue: the two strips of a
    // group finish side by side instead of one after the other in wave 0
    auto finish = [&](const int grp, const int turn) {
        if (kGrouped) {
            fold((kD - 1) & 1);
        } else {
#pragma unroll
            for (int t = 0; t < kSW; ++t)
#pragma unroll
                for (int rr = 0; rr < 4; ++rr)
                    tot[t][rr] = acc[0][t][rr] - 136.0f * accs[0][rr];
        }
        float* rbuf = red + (turn & 1) * (kQ * kSW * M * kRedStride);  // rows of x only
        auto slot = [&](const int qq, const int t) { return rbuf + ((qq * kSW + t) * M + j) * kRedStride + 4 * g; };
        if (j < M) {
#pragma unroll
            for (int t = 0; t < kSW; ++t)
                if (q != t) *(v4f*)slot(q, t) = tot[t];
        }
        __syncthreads();
        auto finalize = [&](auto t_c) {
            constexpr int t = decltype(t_c)::value;
            v4f sum = t == 0 ? tot[0] : *(const v4f*)slot(0, t);
#pragma unroll
            for (int qq = 1; qq < kQ; ++qq) {
                if (qq == t) sum += tot[t];
                else sum += *(const v4f*)slot(qq, t);
            }
            const int n = (place(grp) * kSW + t) * 16 + 4 * g;
            if (n >= p.N) return;
            u32 o[4];
#pragma unroll
            for (int rr = 0; rr < 4; ++rr) {
                float v = round_bf16(sum[rr]);
                if (!kGrouped)
                    v = round_bf16(v / ((rr & 1) ? bf_hi(esc[t][rr >> 1]) : bf_lo(esc[t][rr >> 1])));
                if (p.bias) v = round_bf16(v + ((rr & 1) ? bf_hi(ebi[t][rr >> 1]) : bf_lo(ebi[t][rr >> 1])));
                o[rr] = f32_to_bf16_bits(v);
            }
            const v2u ov = {o[0] | (o[1] << 16), o[2] | (o[3] << 16)};
            *(v2u*)(p.y + (int64_t)j * p.N + n) = ov;
        };
        if (j < M) {
            if (q == 0) finalize(std::integral_constant<int, 0>{});
            if constexpr (kSW == 2) {
                if (q == 1) finalize(std::integral_constant<int, 1>{});
            }
        }
    };

    int turn = 0;
    int grp = block;
    // every group but the workgroup's last: all rounds request and convert ahead, into the next group
    for (; grp + stride < groups; grp += stride, ++turn) {
        begin(grp, grp + stride);
        for (int r = 0; r < R; ++r) round(bool_constant<false>{}, r, bool_constant<false>{});
        finish(grp, turn);
    }
    // the last group: its last round has nothing to request or convert (the one request before it that
    // falls past the end re-reads the group's first unit: never used)
    begin(grp, grp);
    if constexpr (kHalves) {
        for (int r = 0; r < Rh - 1; ++r) round(bool_constant<false>{}, r, bool_constant<false>{});
        // the last round on the first halves: the second halves are requested now and written once
        // every wave has read its last fragments of the first (its MFMAs hold them in registers)
        stage_load(1);
        __builtin_amdgcn_sched_barrier(0);
        round(bool_constant<false>{}, Rh - 1, bool_constant<true>{});
        __syncthreads();
        stage_store(1);
        xrow = w4s_lds + jj * pitch + q * Uh2 * 256 + g * 16;
        __syncthreads();
        read_x(0, 0);  // unit Uh, the first of the second part (buffer 0: kD is even)
        for (int r = Rh; r < R - 1; ++r) round(bool_constant<false>{}, r, bool_constant<false>{});
    } else {
        for (int r = 0; r < R - 1; ++r) round(bool_constant<false>{}, r, bool_constant<false>{});
    }
    round(bool_constant<true>{}, R - 1, bool_constant<false>{});
    finish(grp, turn);
}

// One strip per wave and a ring of two: held to 128 registers (four waves per SIMD; they need 129
// unbounded), so that two workgroups fit a CU.  A launch shared by several problems can have a few
// workgroups more than the chip has CUs (three problems of 256 groups in three turns: 3 x 86 = 258);
// with one workgroup per CU the two extra ones would run after all the others (measured: 10.0 ->
// 14.5 us for the query / key / value launch).  The other forms spill under that bound and keep theirs.
template <int kSW, int kD, int kNP, bool kGrouped>
__global__ __launch_bounds__(kT, (kSW == 1 && kD == 2) ? 4 : 1) void gemv_w4s(W4sMulti mp) {
    const int bx = blockIdx.x;
    int i = 0;
    while (i + 1 < mp.count && bx >= mp.first[i + 1]) ++i;
    gemv_w4s_body<kSW, kD, kNP, kGrouped, false>(mp.p[i], bx - mp.first[i], mp.first[i + 1] - mp.first[i]);
}

template <int kSW, int kD, int kNP, bool kGrouped>
__global__ __launch_bounds__(kT, (kSW == 1 && kD == 2 && kNP <= 8) ? 4 : 1) void gemv_w4s_pre(W4sMulti mp) {
    const int bx = blockIdx.x;
    int i = 0;
    while (i + 1 < mp.count && bx >= mp.first[i + 1]) ++i;
    gemv_w4s_body<kSW, kD, kNP, kGrouped, false, true>(mp.p[i], bx - mp.first[i], mp.first[i + 1] - mp.first[i]);
}

// One problem per launch: its parameters ARE the kernel arguments, fetched in one scalar round trip
// (the several-problem kernel first finds its problem, then fetches that problem's parameters: two
// dependent round trips more before the first vector load can be issued).
template <int kSW, int kD, int kNP, bool kGrouped>
__global__ __launch_bounds__(kT) void gemv_w4s_one(W4sParams p) {
    gemv_w4s_body<kSW, kD, kNP, kGrouped, false>(p, blockIdx.x, gridDim.x);
}

// 9 ... 16 rows of a K too long for LDS: x in two halves (two strips per wave, ring of two, one turn)
template <int kSW, bool kGrouped>
__global__ __launch_bounds__(kT) void gemv_w4s_halves(W4sParams p) {
    gemv_w4s_body<kSW, 2, 16, kGrouped, true>(p, blockIdx.x, gridDim.x);
}

// ---- the strip-linear copy ---------------------------------------------------------------
// One thread per dword of the copy; strips past N (the copy holds an even number of strips) are zero.
__global__ __launch_bounds__(256) void w4s_pack(const uint8_t* __restrict__ w, u32* __restrict__ out,
                                                int64_t K, int64_t N, int64_t strips_padded) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t units = K / 128;
    if (idx >= strips_padded * units * 256) return;
    const int s = (int)(idx & 3), lane = (int)((idx >> 2) & 63);
    const int64_t su = idx >> 8, unit = su % units, strip = su / units;
    const int i = lane & 15, g = lane >> 4;
    const int64_t n = strip * 16 + i;
    u32 d = 0;
    if (n < N) {
        const int64_t row_bytes = (N + 1) / 2;
        const int shift = (n & 1) ? 4 : 0;
        const int64_t k0 = unit * 128 + 32 * s + 8 * g;
#pragma unroll
        for (int e = 0; e < 8; ++e) {
            const u32 nib = (w[(k0 + e) * row_bytes + (n >> 1)] >> shift) & 0xFu;
            d |= nib << ((e & 1) ? 16 + 4 * (e >> 1) : 4 * (e >> 1));
        }
    }
    out[idx] = d;
}

// grouped parameters: [strip][unit][c = 4]{scale[4 c .. 4 c + 3] bf16, (zero + 128)[4 c .. 4 c + 3]}
template <bool kBF16>
__global__ __launch_bounds__(256) void w4s_pack_params(const void* __restrict__ scale,
                                                       const int8_t* __restrict__ zero,
                                                       uint8_t* __restrict__ out, int64_t units, int64_t N,
                                                       int64_t strips_padded) {
    const int64_t idx = (int64_t)blockIdx.x * 256 + threadIdx.x;  // (strip, unit, c)
    if (idx >= strips_padded * units * 4) return;
    const int c = (int)(idx & 3);
    const int64_t su = idx >> 2, unit = su % units, strip = su / units;
    u32 rec[3] = {0, 0, 0x80808080u};
    const int64_t n = strip * 16 + 4 * c;
    if (n < N) {  // N % 16 == 0: four columns in or out together
        u32 h[4], z = 0;
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            const int64_t o = unit * N + n + e;
            h[e] = kBF16 ? (u32)((const uint16_t*)scale)[o] : f32_to_bf16_bits(((const float*)scale)[o]);
            z |= ((u32)(uint8_t)(zero[o] ^ 0x80)) << (8 * e);  // zero + 128 as an unsigned byte
        }
        rec[0] = h[0] | (h[1] << 16);
        rec[1] = h[2] | (h[3] << 16);
        rec[2] = z;
    }
    u32* dst = (u32*)(out + idx * 12);
    dst[0] = rec[0];
    dst[1] = rec[1];
    dst[2] = rec[2];
}

inline int64_t strips_padded(int64_t N) { return ((N + 15) / 16 + 1) / 2 * 2; }

struct W4sPlan {
    bool ok;
    bool halves;  // x staged in two halves (9 ... 16 rows of a long K)
    bool own;     // every wave stages its own slice of x (a small x)
    int sw, d, np;
    int64_t groups;  // strip groups (kSW strips each)
    int64_t blocks;  // workgroups: each takes groups block, block + blocks, ...
    int64_t resident;  // workgroups of this kernel form the chip holds at once (256 or 512)
    size_t lds;      // dynamic LDS of a launch of this problem alone
    size_t lds_two;  // the same with both reduction buffers: what a launch needs whose workgroups take turns
};

constexpr int kResident = 256;  // workgroups the chip holds at once: one per CU (registers)

// shared: the plan is for a launch that several problems share (the kernels of such launches are
// held to 128 registers where that costs nothing, the one-problem kernel is not)
W4sPlan w4s_plan(int64_t M, int64_t K, int64_t N, int64_t block_size, bool pre = false, bool shared = false) {
    W4sPlan pl{};
    const bool grouped = block_size > 0;
    if (M < 1 || M > kMaxRows || (K % 128) != 0 || (N % 16) != 0) return pl;
    if (grouped && block_size != 128) return pl;
    const int64_t units = K / 128, strips = N / 16;
    // all of K stays inside a workgroup, so the strips alone have to fill the chip
    if (strips < 192) return pl;
    // every wave walks at least two rounds of the ring
    if ((units % 4) == 0 && units / 4 >= 2 * kQ) pl.d = 4;
    else if ((units % 2) == 0 && units / 2 >= 2 * kQ) pl.d = 2;
    else return pl;
    pl.sw = strips >= 2 * kResident ? 2 : 1;
    pl.resident = kResident;
    // One strip per wave with a ring of two stays within 128 registers, so two workgroups fit a CU --
    // which a short K needs: its ring holds 2 KiB per wave, 16 KiB per workgroup, and 256 workgroups
    // would have 4 MiB in flight.  Up to 1024 strips then go one per wave to 512 resident workgroups
    // (x small enough for two workgroups' LDS, and few enough pieces per thread for that register
    // budget).
    if (shared && pl.d == 2 && strips < 4 * kResident && M * K <= 8 * 8 * kT &&
        (size_t)((M * (K * 2 + 16) + 255) & ~255) + 2 * (size_t)kQ * M * kRedStride * 4 <= 80 * 1024) {
        pl.sw = 1;
        pl.resident = 2 * kResident;
    }
    pl.groups = (strips + pl.sw - 1) / pl.sw;
    // more groups than the chip holds workgroups: each workgroup takes several, one after the other
    const int64_t turns = (pl.groups + pl.resident - 1) / pl.resident;
    pl.blocks = (pl.groups + turns - 1) / turns;
    const size_t red = (size_t)(turns > 1 ? 2 : 1) * kQ * pl.sw * M * kRedStride * 4;
    const int64_t stage_max = (int64_t)kMaxPieces * 8 * kT;  // elements of x a workgroup stages at a time
    const size_t lds_limit = 160 * 1024;
    // x whole in LDS ...
    const size_t red_one = (size_t)kQ * pl.sw * M * kRedStride * 4;
    pl.lds = (size_t)((M * (K * 2 + 16) + 255) & ~255) + red;
    pl.lds_two = pl.lds - red + 2 * red_one;
    if (M * K <= stage_max && pl.lds <= lds_limit) {
        // a small x: every wave stages its own slice of every row (16 pieces per unit and row, over 64 lanes)
        const int64_t ring_blocks = units / pl.d;
        const int64_t longest = (ring_blocks / kQ + (ring_blocks % kQ ? 1 : 0)) * pl.d;  // units of the longest slice
        const int64_t per_lane = (M * longest * 16 + 63) / 64;
        const int64_t pieces = M * K / 8;
        pl.own = !pre && M * K * 2 <= 32 * 1024 && per_lane <= 4;
        if (pl.own) pl.np = per_lane <= 2 ? 2 : 4;
        else pl.np = pieces <= 2 * kT ? 2 : pieces <= 4 * kT ? 4 : pieces <= 8 * kT ? 8 : 16;
        pl.ok = true;
        return pl;
    }
    // ... or in two parts: equal slices of whole rounds of a ring of two, the first part the larger one
    // when the rounds are odd; one turn per workgroup
    const int64_t slice_rounds = units / (2 * kQ);               // rounds of a wave's slice (ring of 2)
    const int64_t first_units = (slice_rounds + 1) / 2 * 2;      // units of a slice in the first part
    pl.lds = (size_t)((M * (kQ * first_units * 256 + 16) + 255) & ~255) + red;
    if (!pre && (units % (2 * kQ)) == 0 && slice_rounds >= 2 && M * kQ * first_units * 128 <= stage_max &&
        pl.lds <= lds_limit && turns == 1) {
        pl.halves = true;
        pl.d = 2;
        pl.np = 16;
        pl.ok = true;
    }
    return pl;
}

struct W4sKernels {
    void (*multi)(W4sMulti);
    void (*one)(W4sParams);
    void (*pre)(W4sMulti);  // with a transform of x on its way into LDS
};

template <int kSW, int kD, bool kGrouped>
W4sKernels pick_np(int np) {
    switch (np) {
        case 2: return {gemv_w4s<kSW, kD, 2, kGrouped>, gemv_w4s_one<kSW, kD, 2, kGrouped>,
                        gemv_w4s_pre<kSW, kD, 2, kGrouped>};
        case 4: return {gemv_w4s<kSW, kD, 4, kGrouped>, gemv_w4s_one<kSW, kD, 4, kGrouped>,
                        gemv_w4s_pre<kSW, kD, 4, kGrouped>};
        case 8: return {gemv_w4s<kSW, kD, 8, kGrouped>, gemv_w4s_one<kSW, kD, 8, kGrouped>,
                        gemv_w4s_pre<kSW, kD, 8, kGrouped>};
        default: return {gemv_w4s<kSW, kD, 16, kGrouped>, gemv_w4s_one<kSW, kD, 16, kGrouped>,
                         gemv_w4s_pre<kSW, kD, 16, kGrouped>};
    }
}

W4sKernels pick_kernel(const W4sPlan& pl, bool grouped) {
    if (pl.sw == 2) {
        if (pl.d == 4) return grouped ? pick_np<2, 4, true>(pl.np) : pick_np<2, 4, false>(pl.np);
        return grouped ? pick_np<2, 2, true>(pl.np) : pick_np<2, 2, false>(pl.np);
    }
    if (pl.d == 4) return grouped ? pick_np<1, 4, true>(pl.np) : pick_np<1, 4, false>(pl.np);
    return grouped ? pick_np<1, 2, true>(pl.np) : pick_np<1, 2, false>(pl.np);
}

int fill_params(W4sParams& p, const W4sPlan& pl, const void* x, int64_t M, int64_t K, int64_t N,
                const void* shadow, const void* scale, const void* gparams, int64_t block_size,
                const void* bias, int64_t bias_stride, void* y) {
    const bool grouped = block_size > 0;
    if (!x || !shadow || !y || (grouped ? !gparams : !scale)) return K3Q_ERR_NULL;
    if (!aligned_to(x, 16) || !aligned_to(shadow, 16) || !aligned_to(y, 8) || (scale && !aligned_to(scale, 8)) ||
        (gparams && !aligned_to(gparams, 4)) || (bias && !aligned_to(bias, 8)))
        return K3Q_ERR_ALIGN;
    p.x = (const uint16_t*)x;
    p.w = (const v4u*)shadow;
    p.scale = (const uint16_t*)scale;
    p.gparams = (const uint8_t*)gparams;
    p.bias = (const uint16_t*)bias;
    p.y = (uint16_t*)y;
    p.bias_stride = bias ? bias_stride : 0;
    p.M = (int)M;
    p.K = (int)K;
    p.N = (int)N;
    p.units = (int)(K / 128);
    const uint64_t per_row = (uint64_t)K / (pl.halves ? 16 : 8);
    p.row_magic = (int)(uint32_t)((((uint64_t)1 << 32) + per_row - 1) / per_row);
    {
        const uint64_t ring_blocks = (uint64_t)(K / 128) / pl.d, base = ring_blocks / kQ;
        for (int e = 0; e < 2; ++e) {
            const uint64_t own = (base + e) * pl.d * 16;  // pieces per row of a slice of base (+ 1) ring blocks
            p.own_magic[e] = own ? (int)(uint32_t)((((uint64_t)1 << 32) + own - 1) / own) : 0;
        }
    }
    p.own = pl.own ? 1 : 0;
    p.slice_magic = p.row_magic2 = p.slice_magic2 = 0;
    if (pl.halves) {
        // pieces per slice and per row of LDS, first and second part
        const uint64_t slice_units = (uint64_t)(K / 128) / kQ, rounds = slice_units / 2;
        const uint64_t first = (rounds + 1) / 2 * 2, second = slice_units - first;
        auto magic = [](uint64_t d) { return (int)(uint32_t)((((uint64_t)1 << 32) + d - 1) / d); };
        p.row_magic = magic(kQ * first * 16);
        p.slice_magic = magic(first * 16);
        p.row_magic2 = magic(kQ * second * 16);
        p.slice_magic2 = magic(second * 16);
    }
    return K3Q_OK;
}

int launch_w4s(const W4sPlan& pl, bool grouped, const W4sMulti& mp, int total_blocks, size_t lds, hipStream_t s,
               bool pre = false) {
    W4sKernels ks = pick_kernel(pl, grouped);
    if (pre && pl.halves) return K3Q_ERR_SHAPE;
    if (pl.halves) {
        if (mp.count != 1) return K3Q_ERR_SHAPE;
        ks.one = pl.sw == 2 ? (grouped ? gemv_w4s_halves<2, true> : gemv_w4s_halves<2, false>)
                            : (grouped ? gemv_w4s_halves<1, true> : gemv_w4s_halves<1, false>);
    }
    const void* kernel = pre ? (const void*)ks.pre : mp.count == 1 ? (const void*)ks.one : (const void*)ks.multi;
    // more than 64 KiB of dynamic LDS has to be allowed per kernel, once
    {
        static std::mutex mu;
        static std::set<const void*> raised;
        std::lock_guard<std::mutex> lock(mu);
        if (!raised.count(kernel)) {
            if (hipFuncSetAttribute(kernel, hipFuncAttributeMaxDynamicSharedMemorySize, 160 * 1024) != hipSuccess)
                return K3Q_ERR_LAUNCH;
            raised.insert(kernel);
        }
    }
    if (pre) ks.pre<<<(unsigned)total_blocks, kT, lds, s>>>(mp);
    else if (mp.count == 1) ks.one<<<(unsigned)total_blocks, kT, lds, s>>>(mp.p[0]);
    else ks.multi<<<(unsigned)total_blocks, kT, lds, s>>>(mp);
    return launch_status();
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int64_t k3q_w4s_shadow_bytes(int64_t K, int64_t N) {
    if (K <= 0 || N <= 0 || (K % 128) != 0) return 0;
    return strips_padded(N) * (K / 128) * 1024;
}

extern "C" int64_t k3q_w4s_params_bytes(int64_t K, int64_t N, int64_t block_size) {
    if (K <= 0 || N <= 0 || (K % 128) != 0 || block_size != 128) return 0;
    return strips_padded(N) * (K / 128) * 48;
}

extern "C" int k3q_w4s_pack(const int8_t* w_packed, int64_t K, int64_t N, void* shadow, void* stream) {
    if (K <= 0 || N <= 0 || (K % 128) != 0) return K3Q_ERR_SHAPE;
    if (!w_packed || !shadow) return K3Q_ERR_NULL;
    if (!aligned_to(shadow, 16)) return K3Q_ERR_ALIGN;
    const int64_t dwords = k3q_w4s_shadow_bytes(K, N) / 4;
    w4s_pack<<<(unsigned)((dwords + 255) / 256), 256, 0, (hipStream_t)stream>>>(
        (const uint8_t*)w_packed, (u32*)shadow, K, N, strips_padded(N));
    return launch_status();
}

extern "C" int k3q_w4s_pack_params(const void* scale, int scale_dtype, const int8_t* zero, int64_t K,
                                   int64_t N, int64_t block_size, void* params, void* stream) {
    if (K <= 0 || N <= 0 || (K % 128) != 0 || (N % 16) != 0 || block_size != 128) return K3Q_ERR_SHAPE;
    if (scale_dtype != K3Q_F32 && scale_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (!scale || !zero || !params) return K3Q_ERR_NULL;
    if (!aligned_to(params, 4)) return K3Q_ERR_ALIGN;
    const int64_t recs = strips_padded(N) * (K / 128) * 4;
    const unsigned grid = (unsigned)((recs + 255) / 256);
    if (scale_dtype == K3Q_BF16)
        w4s_pack_params<true><<<grid, 256, 0, (hipStream_t)stream>>>(scale, zero, (uint8_t*)params, K / 128, N,
                                                                      strips_padded(N));
    else
        w4s_pack_params<false><<<grid, 256, 0, (hipStream_t)stream>>>(scale, zero, (uint8_t*)params, K / 128, N,
                                                                       strips_padded(N));
    return launch_status();
}

extern "C" int k3q_gemv_w4s_supported(int64_t M, int64_t K, int64_t N, int64_t block_size) {
    return w4s_plan(M, K, N, block_size).ok ? 1 : 0;
}

extern "C" int k3q_gemv_w4s(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N, const void* shadow,
                            const void* scale, const void* gparams, int64_t block_size, const void* bias,
                            int64_t bias_stride, void* y, void* stream) {
    if (x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (bias_stride != 0 && bias_stride != N) return K3Q_ERR_SHAPE;
    const W4sPlan pl = w4s_plan(M, K, N, block_size);
    if (!pl.ok) return K3Q_ERR_SHAPE;
    W4sMulti mp{};
    const int rc = fill_params(mp.p[0], pl, x, M, K, N, shadow, scale, gparams, block_size, bias, bias_stride, y);
    if (rc != K3Q_OK) return rc;
    mp.first[0] = 0;
    mp.first[1] = (int)pl.blocks;
    mp.count = 1;
    return launch_w4s(pl, block_size > 0, mp, (int)pl.blocks, pl.lds, (hipStream_t)stream);
}

namespace {

// Problems that share x: launches of up to kMaxProblems problems whose plans agree.  pre: the
// transform of x (null: none); bias_rows: every bias is [M, N] (a row per row of x) instead of [N].
int w4s_run_shared(const void* x, int x_dtype, int64_t M, int64_t K, const k3q_input_op* pre, int count,
                   const k3q_gemv_w4s_problem* problems, int64_t block_size, bool bias_rows, void* stream) {
    if (x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (count < 0 || M < 0 || K <= 0) return K3Q_ERR_SHAPE;
    if (count == 0 || M == 0) return K3Q_OK;
    if (!problems) return K3Q_ERR_NULL;
    const bool has_pre = pre != nullptr && pre->kind != K3Q_INPUT_NONE;
    if (has_pre) {
        if (pre->kind != K3Q_INPUT_RMS_NORM && pre->kind != K3Q_INPUT_SILU_GATE) return K3Q_ERR_SHAPE;
        if (!pre->operand) return K3Q_ERR_NULL;
        if (!aligned_to(pre->operand, 16)) return K3Q_ERR_ALIGN;
        // (the row sums are taken per block of 64 pieces and kept beside the reduction buffers)
        if (pre->kind == K3Q_INPUT_RMS_NORM && ((K % 512) != 0 || K > 65536)) return K3Q_ERR_SHAPE;
    }
    hipStream_t s = (hipStream_t)stream;
    int at = 0;
    while (at < count) {
        W4sMulti mp{};
        W4sPlan pl0{};
        int64_t groups[kMaxProblems], total = 0;
        int n = 0;
        for (; at + n < count && n < kMaxProblems; ++n) {
            const k3q_gemv_w4s_problem& q = problems[at + n];
            if (q.N <= 0) return K3Q_ERR_SHAPE;
            const W4sPlan pl = w4s_plan(M, K, q.N, block_size, has_pre, count >= 2);
            if (!pl.ok || (has_pre && pl.halves)) return K3Q_ERR_SHAPE;
            if (n == 0) pl0 = pl;
            else if (pl.sw != pl0.sw || pl.d != pl0.d || pl.np != pl0.np || pl.own != pl0.own || pl.resident != pl0.resident ||
                     pl.halves || pl0.halves)
                break;
            const int rc = fill_params(mp.p[n], pl, x, M, K, q.N, q.shadow, q.scale, q.gparams, block_size,
                                       q.bias, bias_rows ? q.N : 0, q.y);
            if (rc != K3Q_OK) return rc;
            if (has_pre) {
                mp.p[n].pre_kind = pre->kind;
                mp.p[n].pre_eps = pre->epsilon;
                mp.p[n].pre_op = (const uint16_t*)pre->operand;
            }
            groups[n] = pl.groups;
            total += pl.groups;
        }
        // the launch as a whole is cut for the chip: about kResident workgroups, each problem its share;
        // workgroups that take turns need both reduction buffers, and where those do not fit beside x
        // the first problem goes alone
        int64_t turns = (total + pl0.resident - 1) / pl0.resident;
        size_t lds = turns > 1 ? pl0.lds_two : pl0.lds;
        if (lds > (size_t)160 * 1024) {
            n = 1;
            turns = (groups[0] + pl0.resident - 1) / pl0.resident;
            lds = pl0.lds;
        }
        if (pl0.halves && n != 1) return K3Q_ERR_SHAPE;
        int next_block = 0;
        for (int i = 0; i < n; ++i) {
            mp.first[i] = next_block;
            next_block += (int)((groups[i] + turns - 1) / turns);
        }
        mp.first[n] = next_block;
        mp.count = n;
        const int rc = launch_w4s(pl0, block_size > 0, mp, next_block, lds, s, has_pre);
        if (rc != K3Q_OK) return rc;
        at += n;
    }
    return K3Q_OK;
}

}  // namespace

extern "C" int k3q_gemv_w4s_multi(const void* x, int x_dtype, int64_t M, int64_t K, int count,
                                  const k3q_gemv_w4s_problem* problems, int64_t block_size, void* stream) {
    return w4s_run_shared(x, x_dtype, M, K, nullptr, count, problems, block_size, false, stream);
}

extern "C" int k3q_gemv_w4s_pre(const void* x, int x_dtype, int64_t M, int64_t K, const k3q_input_op* pre, int count,
                                const k3q_gemv_w4s_problem* problems, int64_t block_size, int bias_rows,
                                void* stream) {
    return w4s_run_shared(x, x_dtype, M, K, pre, count, problems, block_size, bias_rows != 0, stream);
}
