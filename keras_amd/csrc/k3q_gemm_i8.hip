// int8 x int8 -> int32 GEMM with the Dense de-scale epilogue fused:
//     y[m,n] = T( acc[m,n] / (a_scale[m] * b_scale[n]) ) (+ bias[n]),  acc = sum_k a[m,k] * b[k,n]
//
// MFMA-bound kernel for prefill-sized M.  Both operands are consumed K-contiguous:
// `a` is [M,K] as the activation quantizer writes it, the weight comes as the
// [N,K] shadow copy that k3q_prepack_kernel_i8 makes once per layer (the layer's
// own [K,N] variable stays what it is).
//
// Workgroup: 512 threads = 8 waves as 4 (N) x 2 (M); tile 256 (M) x 256 (N), 128
// bytes of K per stage (a full cache line per row and request).  Global -> LDS goes
// through the LDS-DMA path (global_load_lds_dwordx4: 64 lanes x 16 bytes land
// lane-linear in LDS, no VGPR staging), two 64 KiB stages.  The LDS tile is
// [row][128 B] with the eight 16-byte chunks of a row XOR-swizzled by row bits, applied on the global side
// of the DMA (a lane fetches the chunk that belongs at its LDS position), so the
// ds_read_b128 fragment reads are bank-conflict free.
//
// MFMA: v_mfma_i32_32x32x32_i8.  The weight tile is the first (row) operand and
// the activation tile the second (column) operand, so a lane ends up with ONE
// output row m and groups of four consecutive n: stores are 8 or 16 bytes wide.
#include <type_traits>

#include "k3q_common.h"
#include "k3q_gemm_bf16.h"
#include "k3q_gemm_i8_skinny.h"
#include "k3q_gemv_w8.h"

namespace k3q {
namespace {

constexpr int kBK = 128;  // bytes of K per stage: one full 128-byte line per row
constexpr int kStages = 2;
constexpr int kKSteps = kBK / 32;  // MFMA K steps per stage
constexpr int kRowChunks = kBK / 16;  // 16-byte chunks per LDS row

// Tile shape of a workgroup: BM rows of a / y, BN rows of the prepacked weight (= columns of
// y), waves laid out WN (along N) x WM (along M).
template <int BM, int BN, int WN_, int WM_>
struct Tile {
    static constexpr int kBM = BM, kBN = BN, kWavesN = WN_, kWavesM = WM_;
    static constexpr int kThreads = 64 * WN_ * WM_;
    static constexpr int kWN = BN / WN_;      // columns per wave
    static constexpr int kWM = BM / WM_;      // rows per wave
    static constexpr int kNBlk = kWN / 32;    // MFMA blocks along N per wave
    static constexpr int kMBlk = kWM / 32;    // MFMA blocks along M per wave
    static constexpr int kATileBytes = BM * kBK;
    static constexpr int kBTileBytes = BN * kBK;
    static constexpr int kStageBytes = kATileBytes + kBTileBytes;
    static constexpr int kLdsBytes = kStages * kStageBytes;
    static constexpr int kDmaA = kATileBytes / 1024;  // DMA instructions (1 KiB each) per A tile
    static constexpr int kDmaB = kBTileBytes / 1024;
    static constexpr int kDmaPerWave = (kDmaA + kDmaB) / (kThreads / 64);
};
// 256 x 256, 8 waves, 128 KiB of LDS: one workgroup per CU; the shape for large problems.
typedef Tile<256, 256, 4, 2> TileLarge;
// 128 x 128, 4 waves, 64 KiB of LDS: two workgroups per CU; used while the large tile would
// leave CUs without work.
typedef Tile<128, 128, 2, 2> TileSmall;

constexpr int kFlagExactEpilogue = 1;
constexpr int kFlagRoundAccBF16 = 2;   // float32 output of a bfloat16 layer: acc is cast to bfloat16 first

struct GemmParams {
    const int8_t* a;        // [M, K]
    const int8_t* bt;       // [N, K]
    const void* a_scale;    // T [M] or null
    const void* b_scale;    // T [N] or null
    const void* bias;       // T [N] or null
    void* y;                // T [M, N] or null
    int32_t* acc_out;       // [M, N] or null
    int64_t M, N, K;
    int64_t row_bytes;      // bytes per row of a and bt: K (int8) or 2K (bfloat16 operands)
    int tiles_m, tiles_n;
    int flags;
    // bt is not [N, K] rows but the strip-linear copy of the int8 decode kernel (k3q_w8s_pack):
    // [strip = n / 16][unit = k / 64][lane' = n % 16 + 16 g][16 bytes k = 64 unit + 16 g ...].  Only the
    // SOURCE addresses of the B tile's DMA change: a row's 16-byte chunk c of stage kt lies at
    // ((strip * units + 2 kt + c / 4) * 64 + n % 16 + 16 (c % 4)) * 16, i.e. a stage is 2 KiB further on.
    int b_strip, b_units;
    // split of K over workgroups (problems with few tiles and a long K): split sp takes the
    // stages [sp * kt_split, min((sp + 1) * kt_split, stages)) and stores its raw
    // accumulators to part[sp][M][N] (int32 or float32); gemm_split_reduce sums them in
    // split order and applies the epilogue
    int splits, kt_split;
    void* part;
    int64_t part_bytes;
};

// 16-byte chunk swizzle of a 128-byte LDS row (8 chunks): chunk c of row r lives at chunk
// c ^ swz(r).  ds_read_b128 of one chunk index over consecutive rows is then bank-conflict
// free whether the LDS services 8 or 16 lanes per clock.
__device__ __forceinline__ int swz(int row) {
    return (row & 6) | ((row ^ (row >> 3)) & 1);
}

// gfx9 s_waitcnt encoding: vmcnt[3:0] | expcnt[6:4] | lgkmcnt[11:8] | vmcnt_hi[15:14]
__device__ __forceinline__ void wait_vmcnt0() { __builtin_amdgcn_s_waitcnt(0x0F70); }
template <int kDmaPerWave>
__device__ __forceinline__ void wait_vmcnt_one_stage() {
    __builtin_amdgcn_s_waitcnt(0x0F70 | (kDmaPerWave & 0xF) | ((kDmaPerWave >> 4) << 14));
}
__device__ __forceinline__ void wait_lgkmcnt0() { __builtin_amdgcn_s_waitcnt(0xC07F); }
__device__ __forceinline__ void bare_barrier() {
    // s_barrier without a fence: a fence would also drain the DMA of the stage in flight
    asm volatile("" ::: "memory");
    __builtin_amdgcn_s_barrier();
    asm volatile("" ::: "memory");
}

template <bool kBF16>
__device__ __forceinline__ float load_t(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

// Operand kinds.  The byte geometry is the same for both: a lane's MFMA fragment is 16
// bytes of one row, a stage is 128 bytes of K per row -- 128 int8 or 64 bfloat16 values.
constexpr int kKindI8 = 0;    // int8 x int8 -> int32, v_mfma_i32_32x32x32_i8
constexpr int kKindBF16 = 1;  // bfloat16 x bfloat16 -> float32, v_mfma_f32_32x32x16_bf16

__device__ __forceinline__ u32 raw_bits(int v) { return (u32)v; }
__device__ __forceinline__ u32 raw_bits(float v) { return __float_as_uint(v); }
__device__ __forceinline__ void from_bits(u32 b, int& v) { v = (int)b; }
__device__ __forceinline__ void from_bits(u32 b, float& v) { v = __uint_as_float(b); }

template <int kKind>
struct Mma;
template <>
struct Mma<kKindI8> {
    typedef v16i Acc;
    static __device__ __forceinline__ Acc run(const v4i& b, const v4i& a, const Acc& c) {
        return __builtin_amdgcn_mfma_i32_32x32x32_i8(b, a, c, 0, 0, 0);
    }
};
template <>
struct Mma<kKindBF16> {
    typedef v16f Acc;
    static __device__ __forceinline__ Acc run(const v4i& b, const v4i& a, const Acc& c) {
        return __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, b),
                                                       __builtin_bit_cast(v8bf, a), c, 0, 0, 0);
    }
};

// De-scale of one int32 accumulator.  kExact: the reference's op sequence, every step rounded
// to T (sa, sb are the scales); otherwise one final rounding (sa, sb are their reciprocals, bv
// is 0 without a bias).  kDiv selects the bfloat16 division: 0 IEEE, 1 reciprocal (the caller
// has checked the scales' range), 2 reciprocal with a range check per element; all three
// give the same bits.
template <bool kBF16, bool kExact, int kDiv>
__device__ __forceinline__ float descale_i8(int acc, float sa, float sb, float bv, bool has_bias,
                                            bool round_acc) {
    float accf = (float)acc;
    if (!kBF16 && round_acc) accf = round_bf16(accf);
    if (!kExact) return (accf * sa) * sb + bv;
    if (kBF16) {
        const float os = round_bf16(sb * sa);
        const float ab = round_bf16(accf);
        float r = kDiv == 0   ? round_bf16(ab / os)
                  : kDiv == 1 ? round_bf16(ab * __builtin_amdgcn_rcpf(os))
                              : div_round_bf16(ab, os);
        if (has_bias) r = round_bf16(r + bv);
        return r;
    }
    float r = accf / (sb * sa);
    if (has_bias) r = r + bv;
    return r;
}

// De-scale of one float accumulator of the bfloat16-operand kind: y = T(T(acc) / scale[n])
// (+ bias); T = bfloat16 or float32.
template <bool kBF16>
__device__ __forceinline__ float descale_f(float acc, float sb, float bv, bool has_s, bool has_b) {
    float r = acc;
    if (kBF16) {
        r = round_bf16(r);
        if (has_s) r = div_round_bf16(r, sb);
        if (has_b) r = round_bf16(r + bv);
    } else {
        if (has_s) r = r / sb;
        if (has_b) r = r + bv;
    }
    return r;
}

// kBStrip: the B operand is the strip-linear copy of the int8 decode kernel (GemmParams::b_strip).
// Read row by row, that copy would make every group of 16 lanes of a DMA instruction touch eight
// cache lines instead of two, so the B tile then lies in LDS as [8-row block][chunk][row] instead
// of [row][chunk]: the eight rows of a block fetch one chunk from 128 contiguous bytes of the copy.
// The chunk position is flipped in every second block (neighbouring blocks then sit in different
// halves of the banks for one fragment read), and a K step is still one XOR on the fragment address.
template <class T, int kKind, bool kBF16, bool kExact, bool kBStrip = false>
__global__ __launch_bounds__(T::kThreads) void gemm_mfma(GemmParams p) {
    constexpr int kBM = T::kBM, kBN = T::kBN, kWavesN = T::kWavesN, kThreads = T::kThreads;
    constexpr int kWN = T::kWN, kWM = T::kWM, kNBlk = T::kNBlk, kMBlk = T::kMBlk;
    constexpr int kATileBytes = T::kATileBytes, kStageBytes = T::kStageBytes;
    constexpr int kDmaA = T::kDmaA, kDmaPerWave = T::kDmaPerWave;
    extern __shared__ __attribute__((aligned(1024))) char lds[];
    const int tid = threadIdx.x;
    const int lane = tid & 63;
    const int wave = __builtin_amdgcn_readfirstlane(tid >> 6);
    const int wn = wave % kWavesN;
    const int wm = wave / kWavesN;

    // ---- tile of this workgroup: XCD-aware order ----
    // Workgroups are dealt round-robin to the 8 XCDs; each XCD walks a contiguous range of
    // the tile list, and the list is ordered in bands of 4 tile rows so that the 32 tiles an
    // XCD runs at a time share A rows and B rows in its L2.
    const int total = p.tiles_m * p.tiles_n * p.splits;  // work items: (tile, split of K)
    const int per_xcd = (total + 7) / 8;
    // A workgroup stays on its CU and walks every (gridDim / 8)-th tile of its XCD's range:
    // the output stores of one tile drain while the next tile's loads are already running.
    const int tl_first = blockIdx.x / 8, tl_step = gridDim.x / 8;
    for (int tl = tl_first; tl < per_xcd; tl += tl_step) {
        const int item = (blockIdx.x % 8) * per_xcd + tl;
        if (item >= total) break;
        if (tl != tl_first) __syncthreads();  // the previous tile's epilogue is done with the LDS
        const int t = item / p.splits, sp = item - t * p.splits;
        constexpr int kBand = 4;
        const int band = t / (kBand * p.tiles_n);
        const int band_rows = min(kBand, p.tiles_m - band * kBand);
        const int within = t - band * kBand * p.tiles_n;
        const int tile_m = band * kBand + within % band_rows;
        const int tile_n = within / band_rows;
        const int64_t m0 = (int64_t)tile_m * kBM;
        const int64_t n0 = (int64_t)tile_n * kBN;

        // ---- DMA source addresses ----
        // DMA instruction d of this wave fills LDS bytes [(wave * kDmaPerWave + d) * 1024, +1024) of
        // the stage: 8 rows x 128 B.  The first kDmaA instructions of a stage are the A tile, the
        // rest the B tile.
        const char* src[kDmaPerWave];
#pragma unroll
        for (int d = 0; d < kDmaPerWave; ++d) {
            const int inst = wave * kDmaPerWave + d;
            const bool is_b = inst >= kDmaA;
            const bool strip_b = kBStrip && is_b;
            const int blk = is_b ? inst - kDmaA : inst;  // the 8-row block this instruction fills
            const int row = blk * 8 + (strip_b ? lane & 7 : lane / kRowChunks);
            const int chunk = strip_b ? (lane >> 3) ^ (blk & 1) : (lane & (kRowChunks - 1)) ^ swz(row);
            int64_t grow = (is_b ? n0 : m0) + row;
            const int64_t lim = (is_b ? p.N : p.M) - 1;
            grow = grow < lim ? grow : lim;
            if (strip_b)
                src[d] = (const char*)p.bt + ((grow >> 4) * p.b_units + (chunk >> 2)) * 1024 +
                         ((grow & 15) + 16 * (chunk & 3)) * 16 + (int64_t)sp * p.kt_split * 2048;
            else
                src[d] = (const char*)(is_b ? p.bt : p.a) + grow * p.row_bytes + chunk * 16 +
                         (int64_t)sp * p.kt_split * kBK;
        }
        // (all DMA instructions of a wave belong to the same operand: kDmaA is a multiple of kDmaPerWave)
        static_assert(kDmaA % kDmaPerWave == 0, "a wave's DMA instructions fill one operand");
        const int kstep = (kBStrip && wave * kDmaPerWave >= kDmaA) ? 2048 : kBK;
        auto issue_stage = [&](int kt) {
            char* dst = lds + (kt % kStages) * kStageBytes + wave * kDmaPerWave * 1024;
#pragma unroll
            for (int d = 0; d < kDmaPerWave; ++d) {
                __builtin_amdgcn_global_load_lds(
                    (const __attribute__((address_space(1))) void*)(src[d] + (int64_t)kt * kstep),
                    (__attribute__((address_space(3))) void*)(dst + d * 1024), 16, 0, 0);
            }
        };

        // ---- fragment reads ----
        // MFMA operand lane (i = lane % 32, g = lane / 32) holds row i, bytes [16g, 16g+16) of the
        // 32-byte K step, i.e. logical chunk 2*ks + g of the row.
        const int fi = lane & 31;
        const int fg = lane >> 5;
        // Every 32-row block starts at a multiple of 32 rows, so swz(row) = swz(i) for all of
        // them, and 2*ks + g = (2*ks) ^ g.  The byte address of a fragment is therefore
        // (row base | ((g ^ swz(i)) << 4)) ^ (32 * ks) + block * 32 rows: one register per
        // operand, one XOR per K step, the blocks as immediate offsets.  The stage is a bit of
        // that register, flipped at the hand-over.
        static_assert((kStageBytes & (kStageBytes - 1)) == 0 && kWM % 32 == 0 && kWN % 32 == 0, "addressing");
        const int lane_chunk = (fg ^ swz(fi)) << 4;
        int ra = (wm * kWM + fi) * kBK + lane_chunk;
        int rb = kATileBytes + (wn * kWN + fi) * kBK + lane_chunk;
        if (kBStrip)  // [block][chunk position][row]: chunk 2 ks + g of row i at position (2 ks + g) ^ (block & 1)
            rb = kATileBytes + ((wn * kWN + fi) >> 3) * 1024 + ((fg ^ ((fi >> 3) & 1)) << 7) + (fi & 7) * 16;
        v4i af[2][kMBlk], bf[2][kNBlk];
        auto read_frags = [&](int fb, int ks) {
            const char* pb = lds + (rb ^ ((kBStrip ? 256 : 32) * ks));
#pragma unroll
            for (int nb = 0; nb < kNBlk; ++nb) bf[fb][nb] = *(const v4i*)(pb + nb * 32 * kBK);
            const char* pa = lds + (ra ^ (32 * ks));
#pragma unroll
            for (int mb = 0; mb < kMBlk; ++mb) af[fb][mb] = *(const v4i*)(pa + mb * 32 * kBK);
        };

        typename Mma<kKind>::Acc acc[kNBlk][kMBlk];
#pragma unroll
        for (int nb = 0; nb < kNBlk; ++nb)
#pragma unroll
            for (int mb = 0; mb < kMBlk; ++mb)
#pragma unroll
                for (int r = 0; r < 16; ++r) acc[nb][mb][r] = 0;

        // ---- main loop ----
        // Two LDS stages.  The fragments of K step ks+1 are read in the middle of the MFMAs of
        // step ks; the one barrier per stage sits in the middle of the LAST step's MFMAs, so the
        // matrix core has work queued while waves meet.  At that barrier every wave holds its
        // last fragments of stage kt in registers, so stage kt+2 may be DMA-ed over stage kt, and
        // stage kt+1 (whose DMA every wave has waited for) may be read.
        const int kt_first = sp * p.kt_split;  // this split's stages (all of K without a split)
        const int KT = min(p.kt_split, (int)(p.row_bytes / kBK) - kt_first);
        issue_stage(0);
        if (KT > 1) {
            issue_stage(1);
            wait_vmcnt_one_stage<kDmaPerWave>();
        } else {
            wait_vmcnt0();
        }
        bare_barrier();
        read_frags(0, 0);
        // The DMA of a stage is not issued as one burst: the texture unit takes an instruction
        // per ~16 clocks and the workgroup's 64 would hold every wave (an in-order issuer) away
        // from its MFMAs for up to a thousand clocks.  Instead one DMA instruction follows every
        // kDmaStride-th MFMA, starting at the hand-over (second half of the last K step, into the
        // buffer just released) and ending in the second K step of the next stage, which
        // leaves the last one half a stage to land.
        constexpr int kHalfMmas = kNBlk / 2 * kMBlk;
        constexpr int kDmaStride = 5 * kHalfMmas / kDmaPerWave >= 2 ? 2 : 1;
        static_assert(kKSteps == 4 && 5 * kHalfMmas / kDmaStride >= kDmaPerWave, "DMA slots");
        auto issue_one = [&](int kt, int d) {
            char* dst = lds + (kt % kStages) * kStageBytes + wave * kDmaPerWave * 1024;
            __builtin_amdgcn_global_load_lds(
                (const __attribute__((address_space(1))) void*)(src[d] + (int64_t)kt * kstep),
                (__attribute__((address_space(3))) void*)(dst + d * 1024), 16, 0, 0);
        };
        auto mma_half = [&](int ks, int half, int kt) {
            // halves since the hand-over: 0 = second half of the last step (feeds stage kt+2),
            // 1..4 = the two halves of steps 0 and 1 (feed stage kt+1, begun one stage earlier)
            const int hh = (ks == kKSteps - 1 && half == 1) ? 0 : (ks <= 1 ? 1 + 2 * ks + half : -1);
#pragma unroll
            for (int j = 0; j < kHalfMmas; ++j) {
                const int nb = half * (kNBlk / 2) + j / kMBlk, mb = j % kMBlk;
                acc[nb][mb] = Mma<kKind>::run(bf[ks & 1][nb], af[ks & 1][mb], acc[nb][mb]);
                const int pos = hh * kHalfMmas + j;
                if (hh >= 0 && pos % kDmaStride == kDmaStride - 1 && pos / kDmaStride < kDmaPerWave) {
                    const int target = hh == 0 ? kt + 2 : kt + 1;
                    if ((hh == 0 || kt >= 1) && target < KT) {
                        __builtin_amdgcn_sched_barrier(0);
                        issue_one(target, pos / kDmaStride);
                        __builtin_amdgcn_sched_barrier(0);
                    }
                }
            }
        };
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int ks = 0; ks < kKSteps; ++ks) {
                // first half of this step's MFMAs, then the reads for the next step, then the
                // second half: the reads get half a step of matrix-core time to come back
                __builtin_amdgcn_sched_barrier(0);
                // Raised wave priority from the first MFMA of a step to its last, dropped between
                // steps: measured, 2 % on the exact bfloat16 path at M = 4096, K = N = 8192
                // (233 against 238 us), neutral to 1 % elsewhere; raising it around each half
                // separately, or only around the second, gained less.
                __builtin_amdgcn_s_setprio(1);
                mma_half(ks, 0, kt);
                __builtin_amdgcn_sched_barrier(0);
                if (ks + 1 < kKSteps) {
                    read_frags((ks + 1) & 1, ks + 1);
                } else if (kt + 1 < KT) {
                    wait_vmcnt0();  // own DMA of stage kt+1 has landed (own reads of stage kt are done)
                    bare_barrier();
                    ra ^= kStageBytes;
                    rb ^= kStageBytes;
                    read_frags(0, 0);
                }
                __builtin_amdgcn_sched_barrier(0);
                mma_half(ks, 1, kt);
                __builtin_amdgcn_s_setprio(0);
                __builtin_amdgcn_sched_barrier(0);
            }
        }

        if (p.splits > 1) {
            // raw accumulators of this split, as they lie (16 bytes per lane and column group)
#pragma unroll
            for (int mb = 0; mb < kMBlk; ++mb) {
                const int64_t m = m0 + wm * kWM + mb * 32 + fi;
#pragma unroll
                for (int nb = 0; nb < kNBlk; ++nb)
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        const int64_t n = n0 + wn * kWN + nb * 32 + 8 * rg + 4 * fg;
                        if (m >= p.M || n >= p.N) continue;
                        v4u o;
#pragma unroll
                        for (int e = 0; e < 4; ++e) o[e] = raw_bits(acc[nb][mb][4 * rg + e]);
                        *(v4u*)((u32*)p.part + ((int64_t)sp * p.M + m) * p.N + n) = o;
                    }
            }
            continue;
        }
        // ---- epilogue ----
        // acc[nb][mb][r] is output (m, n) with m = m0 + wm*kWM + mb*32 + lane%32 and
        // n = n0 + wn*kWN + nb*32 + 8*(r/4) + 4*(lane/32) + r%4: a lane owns one row of y per mb
        // and groups of four consecutive columns.
        // Stage the tile's scales and bias in LDS as floats (the main loop is done with it): the
        // per-lane reads below are then cheap and need no large register arrays.
        float* ep = (float*)lds;  // [0,256) b_scale or its reciprocal, [256,512) bias, [512,768) a_scale or reciprocal
        __syncthreads();
        // scales outside [2^-30, 2^30] send the tile to the IEEE division (see div_round_bf16:
        // with both in range, the product of two and an int32 over it stay normal numbers)
        int wide_scale = 0;
        auto out_of_range = [](float v) { return (((__float_as_uint(v) >> 23) & 0xffu) - 97u) > 60u; };
        for (int t = tid; t < kBN; t += kThreads) {
            const int64_t n = n0 + t < p.N ? n0 + t : p.N - 1;
            const float sbv = p.b_scale ? load_t<kBF16>(p.b_scale, n) : 1.0f;
            wide_scale |= out_of_range(sbv);
            ep[t] = kExact ? sbv : 1.0f / sbv;
            ep[kBN + t] = p.bias ? load_t<kBF16>(p.bias, n) : 0.0f;
        }
        for (int t = tid; t < kBM; t += kThreads) {
            const int64_t m = m0 + t < p.M ? m0 + t : p.M - 1;
            const float sav = p.a_scale ? load_t<kBF16>(p.a_scale, m) : 1.0f;
            wide_scale |= out_of_range(sav);
            ep[2 * kBN + t] = kExact ? sav : 1.0f / sav;
        }
        const bool ieee_div = __syncthreads_or(wide_scale) != 0;
        // Output staging.  A lane's accumulators are four consecutive columns of 32 different
        // rows: stored as they are, a wave instruction would touch 32 lines with 8 or 16 bytes
        // each.  Instead every wave passes its 32-row blocks through a private LDS area
        // ([32][kWN] outputs, rows padded by 16 bytes against bank conflicts) and stores them
        // row-contiguous, 16 bytes per lane: whole 128-byte lines per instruction.
        constexpr int kE = kBF16 ? 2 : 4;            // bytes per output
        constexpr int kPitch = kWN * kE + 16;
        constexpr int kChunks = kWN * kE / 16;       // 16-byte chunks per staged row
        constexpr int kRowsPerPass = 64 / kChunks;
        static_assert((2 * kBN + kBM) * 4 <= 4096, "scales and bias fit below the staging areas");
        static_assert(4096 + (kThreads / 64) * 32 * kPitch <= T::kLdsBytes, "staging fits in LDS");
        char* wst = lds + 4096 + wave * (32 * kPitch);
        const bool wide = (((int64_t)p.N * kE) % 16 == 0) && (((uintptr_t)p.y) % 16 == 0);
        const bool quads = (p.N % 4) == 0;  // every row of y (and of acc_out) is 8-byte aligned
        auto stage4 = [&](int nb, int rg, const float (&v)[4]) {
            char* d = wst + fi * kPitch + (nb * 32 + 8 * rg + 4 * fg) * kE;
            if (kBF16) {
                v2u o = {pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3])};
                *(v2u*)d = o;
            } else {
                v4f o = {v[0], v[1], v[2], v[3]};
                *(v4f*)d = o;
            }
        };
        auto flush_rows = [&](int mb) {
            // LDS operations of one wave complete in order: waiting for the writes is enough
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
#pragma unroll
            for (int ps = 0; ps < 32 / kRowsPerPass; ++ps) {
                const int row = ps * kRowsPerPass + lane / kChunks;
                const int chunk = lane % kChunks;
                const v4u d = *(const v4u*)(wst + row * kPitch + chunk * 16);
                const int64_t m = m0 + wm * kWM + mb * 32 + row;
                const int64_t n = n0 + wn * kWN + chunk * (16 / kE);
                if (m >= p.M || n >= p.N) continue;
                char* dst = (char*)p.y + (m * p.N + n) * kE;
                const int valid = (int)min((int64_t)(16 / kE), p.N - n);  // columns of this piece in y
                if (wide && valid == 16 / kE) {
                    *(v4u*)dst = d;
                } else if (quads) {  // rows of y start on 8-byte boundaries
                    v2u lo = {d[0], d[1]}, hi = {d[2], d[3]};
                    *(v2u*)dst = lo;
                    if (valid > 8 / kE) *(v2u*)(dst + 8) = hi;
                } else {  // N % 4 != 0: rows of y start anywhere, element by element
#pragma unroll
                    for (int e = 0; e < 16 / kE; ++e) {
                        if (e >= valid) break;
                        const u32 word = d[e * kE / 4];
                        if (kE == 2)
                            ((uint16_t*)dst)[e] = (uint16_t)(word >> (16 * (e & 1)));
                        else
                            ((u32*)dst)[e] = word;
                    }
                }
            }
            asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");  // reads done before the next block's writes
        };
        if constexpr (kKind == kKindBF16) {
            // float operands (a de-quantised int4 / widened int8 kernel): y = T(T(acc) / scale[n])
            // (+ bias), or with a null scale y = T(acc) (+ bias).  T = bfloat16, or float32 when the
            // operands are the high / low bfloat16 parts of float32 values.
            const bool has_b = p.bias != nullptr, has_s = p.b_scale != nullptr;
#pragma unroll
            for (int mb = 0; mb < kMBlk; ++mb) {
#pragma unroll
                for (int nb = 0; nb < kNBlk; ++nb) {
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        const int nl = wn * kWN + nb * 32 + 8 * rg + 4 * fg;
                        const v4f sb = *(const v4f*)(ep + nl);
                        const v4f bv = *(const v4f*)(ep + kBN + nl);
                        float r[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            r[e] = descale_f<kBF16>((float)acc[nb][mb][4 * rg + e], sb[e], bv[e], has_s, has_b);
                        stage4(nb, rg, r);
                    }
                }
                flush_rows(mb);
            }
            continue;
        }
        const bool has_bias = p.bias != nullptr;
        const bool round_acc = (p.flags & kFlagRoundAccBF16) != 0;
        auto descale = [&](auto rcp_div) {
#pragma unroll
            for (int mb = 0; mb < kMBlk; ++mb) {
                const int ml = wm * kWM + mb * 32 + fi;
                const int64_t m = m0 + ml;
                const float sa = ep[2 * kBN + ml];
#pragma unroll
                for (int nb = 0; nb < kNBlk; ++nb) {
#pragma unroll
                    for (int rg = 0; rg < 4; ++rg) {
                        const int nl = wn * kWN + nb * 32 + 8 * rg + 4 * fg;
                        const int64_t n = n0 + nl;
                        if (p.acc_out && m < p.M && n < p.N) {
                            if (quads) {
                                v4i o = {(int)acc[nb][mb][4 * rg], (int)acc[nb][mb][4 * rg + 1],
                                         (int)acc[nb][mb][4 * rg + 2], (int)acc[nb][mb][4 * rg + 3]};
                                *(v4i*)(p.acc_out + m * p.N + n) = o;
                            } else {
#pragma unroll
                                for (int e = 0; e < 4; ++e)
                                    if (n + e < p.N) p.acc_out[m * p.N + n + e] = (int)acc[nb][mb][4 * rg + e];
                            }
                        }
                        if (!p.y) continue;
                        const v4f sb = *(const v4f*)(ep + nl);
                        const v4f bv = *(const v4f*)(ep + kBN + nl);
                        float v[4];
#pragma unroll
                        for (int e = 0; e < 4; ++e)
                            v[e] = descale_i8<kBF16, kExact, decltype(rcp_div)::value ? 1 : 0>(
                                (int)acc[nb][mb][4 * rg + e], sa, sb[e], bv[e], has_bias, round_acc);
                        stage4(nb, rg, v);
                    }
                }
                if (p.y) flush_rows(mb);
            }
        };
        if constexpr (kExact && kBF16) {
            if (ieee_div) descale(std::false_type{});
            else descale(std::true_type{});
        } else {
            descale(std::false_type{});
        }
    }
}

// Any shape: one thread per output.  b is addressed through strides so that both the
// [K,N] variable layout and the [N,K] shadow copy work.
template <bool kBF16>
__global__ __launch_bounds__(256) void gemm_i8_simple(const int8_t* a, const int8_t* b,
                                                      int64_t b_stride_k, int64_t b_stride_n,
                                                      GemmParams p) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t m = blockIdx.y;
    if (n >= p.N) return;
    int acc = 0;
    for (int64_t k = 0; k < p.K; ++k) acc += (int)a[m * p.K + k] * (int)b[k * b_stride_k + n * b_stride_n];
    if (p.acc_out) p.acc_out[m * p.N + n] = acc;
    if (!p.y) return;
    const float sa = p.a_scale ? load_t<kBF16>(p.a_scale, m) : 1.0f;
    const float sb = p.b_scale ? load_t<kBF16>(p.b_scale, n) : 1.0f;
    float r;
    if (kBF16) {
        r = round_bf16(round_bf16((float)acc) / round_bf16(sb * sa));
        if (p.bias) r = round_bf16(r + load_t<true>(p.bias, n));
        ((uint16_t*)p.y)[m * p.N + n] = (uint16_t)f32_to_bf16_bits(r);
    } else {
        const float accf = (p.flags & kFlagRoundAccBF16) ? round_bf16((float)acc) : (float)acc;
        r = accf / (sb * sa);
        if (p.bias) r = r + load_t<false>(p.bias, n);
        ((float*)p.y)[m * p.N + n] = r;
    }
}

// [K, N] -> [N, out_stride] byte transpose through a padded LDS tile (one-time per layer);
// bytes [K, out_stride) of every output row are zero.  The grid covers out_stride along y.
__global__ __launch_bounds__(256) void transpose_i8(const int8_t* __restrict__ in,
                                                    int8_t* __restrict__ out, int64_t K, int64_t N,
                                                    int64_t out_stride) {
    __shared__ int8_t tile[64][64 + 4];
    const int64_t k0 = (int64_t)blockIdx.y * 64;
    const int64_t n0 = (int64_t)blockIdx.x * 64;
    for (int e = threadIdx.x; e < 64 * 64; e += 256) {
        const int r = e / 64, c = e % 64;
        int8_t v = 0;
        if (k0 + r < K && n0 + c < N) v = in[(k0 + r) * N + n0 + c];
        tile[r][c] = v;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 64 * 64; e += 256) {
        const int r = e / 64, c = e % 64;  // r: n within tile, c: k within tile
        if (n0 + r < N && k0 + c < out_stride) out[(n0 + r) * out_stride + k0 + c] = tile[c][r];
    }
}

// rows of K bytes -> rows of Kpad bytes, zero-filled (Kpad % 16 == 0), 16 output bytes per thread
__global__ __launch_bounds__(256) void pad_rows_i8(const int8_t* __restrict__ in,
                                                   int8_t* __restrict__ out, int64_t rows, int64_t K,
                                                   int64_t Kpad) {
    const int64_t per_row = Kpad / 16;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= rows * per_row) return;
    const int64_t r = i / per_row, c = (i - r * per_row) * 16;
    const int8_t* src = in + r * K + c;
    v4u v = {0u, 0u, 0u, 0u};
    if (c + 16 <= K && (((uintptr_t)src) & 15) == 0) {
        v = *(const v4u*)src;
    } else {
#pragma unroll
        for (int e = 0; e < 16; ++e)
            if (c + e < K) v[e >> 2] |= (u32)(uint8_t)src[e] << (8 * (e & 3));
    }
    *(v4u*)(out + r * Kpad + c) = v;
}

// ---- weight-only int8: the int8 kernel widened to bfloat16 [N, K] in scratch (exact) ----
// [N, K] int8 -> bfloat16 rows of `out_stride` values, 16 values per thread; with `twice` the
// K values of a row are written at +0 and at +K (the [w | w] rows of the float32 route)
__global__ __launch_bounds__(256) void widen_i8_to_bf16(const int8_t* __restrict__ in,
                                                        uint16_t* __restrict__ out, int64_t count16,
                                                        int64_t K, int64_t out_stride, bool twice) {
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= count16) return;
    const v4u v = *(const v4u*)(in + i * 16);
    v4u o[2];
#pragma unroll
    for (int e = 0; e < 16; e += 2) {
        const float lo = (float)(int)(int8_t)(v[e >> 2] >> (8 * (e & 3)));
        const float hi = (float)(int)(int8_t)(v[(e + 1) >> 2] >> (8 * ((e + 1) & 3)));
        o[e >> 3][(e & 7) >> 1] = pack_bf16x2(lo, hi);
    }
    const int64_t n = (i * 16) / K, k = i * 16 - n * K;  // K % 16 == 0: a piece stays in its row
    v4u* dst = (v4u*)(out + n * out_stride + k);
    dst[0] = o[0];
    dst[1] = o[1];
    if (twice) {
        dst = (v4u*)(out + n * out_stride + K + k);
        dst[0] = o[0];
        dst[1] = o[1];
    }
}

// [K, N] int8 -> [N, K] bfloat16 (rows of `out_stride` values, optionally twice) through a
// padded LDS tile
__global__ __launch_bounds__(256) void transpose_widen_i8_to_bf16(const int8_t* __restrict__ in,
                                                                  uint16_t* __restrict__ out,
                                                                  int64_t K, int64_t N,
                                                                  int64_t out_stride, bool twice) {
    __shared__ int8_t tile[64][64 + 4];
    const int64_t k0 = (int64_t)blockIdx.y * 64;
    const int64_t n0 = (int64_t)blockIdx.x * 64;
    for (int e = threadIdx.x; e < 64 * 64; e += 256) {
        const int r = e / 64, c = e % 64;
        int8_t v = 0;
        if (k0 + r < K && n0 + c < N) v = in[(k0 + r) * N + n0 + c];
        tile[r][c] = v;
    }
    __syncthreads();
    for (int e = threadIdx.x; e < 64 * 64; e += 256) {
        const int r = e / 64, c = e % 64;  // r: n within tile, c: k within tile
        if (n0 + r < N && k0 + c < K) {
            const uint16_t h = (uint16_t)f32_to_bf16_bits((float)tile[c][r]);
            out[(n0 + r) * out_stride + k0 + c] = h;
            if (twice) out[(n0 + r) * out_stride + K + k0 + c] = h;
        }
    }
}

// Float x against a bfloat16 kernel [N, parts * K] (parts 3: [wh | wh | wl], the weight is
// wh + wl), any shape: one thread per output, fp32 accumulation.
template <bool kBF16>
__global__ __launch_bounds__(256) void gemm_wbf16_simple(const void* x, const uint16_t* wt, int parts,
                                                         const void* bias, void* y, int64_t N,
                                                         int64_t K) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t m = blockIdx.y;
    if (n >= N) return;
    const uint16_t* w = wt + n * parts * K;
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k) {
        float wv = bf16_bits_to_f32(w[k]);
        if (parts == 3) wv += bf16_bits_to_f32(w[2 * K + k]);
        acc = fmaf(load_t<kBF16>(x, m * K + k), wv, acc);
    }
    if (kBF16) {
        float r = round_bf16(acc);
        if (bias) r = round_bf16(r + load_t<true>(bias, n));
        ((uint16_t*)y)[m * N + n] = (uint16_t)f32_to_bf16_bits(r);
    } else {
        ((float*)y)[m * N + n] = bias ? acc + load_t<false>(bias, n) : acc;
    }
}

// Any shape and dtype: one thread per output, fp32 accumulation.
template <bool kBF16>
__global__ __launch_bounds__(256) void gemm_w8_simple(const void* x, const int8_t* b,
                                                      int64_t b_stride_k, int64_t b_stride_n,
                                                      const void* scale, const void* bias, void* y,
                                                      int64_t N, int64_t K) {
    const int64_t n = (int64_t)blockIdx.x * 256 + threadIdx.x;
    const int64_t m = blockIdx.y;
    if (n >= N) return;
    float acc = 0.f;
    for (int64_t k = 0; k < K; ++k)
        acc = fmaf(load_t<kBF16>(x, m * K + k), (float)b[k * b_stride_k + n * b_stride_n], acc);
    if (kBF16) {
        float r = round_bf16(acc);
        if (scale) r = round_bf16(r / load_t<true>(scale, n));
        if (bias) r = round_bf16(r + load_t<true>(bias, n));
        ((uint16_t*)y)[m * N + n] = (uint16_t)f32_to_bf16_bits(r);
    } else {
        float r = acc;
        if (scale) r = r / load_t<false>(scale, n);
        if (bias) r = r + load_t<false>(bias, n);
        ((float*)y)[m * N + n] = r;
    }
}

// compute units of the current device
inline int cu_count() {
    static int cached[64] = {0};
    int dev = 0;
    if (hipGetDevice(&dev) != hipSuccess || dev < 0 || dev >= 64) return 0;
    if (cached[dev] == 0) {
        int n = 0;
        if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess) n = 0;
        cached[dev] = n > 0 ? n : -1;
    }
    return cached[dev] > 0 ? cached[dev] : 0;
}

// Second kernel of a K split: sums part[0..splits)[m][n] in split order (int32: exact;
// float32: one fixed order) and applies the epilogue of gemm_mfma.  One thread per four
// consecutive columns of a row.
template <int kKind, bool kBF16, bool kExact>
__global__ __launch_bounds__(256) void gemm_split_reduce(GemmParams p) {
    const int64_t quads = p.N / 4;
    const int64_t i = (int64_t)blockIdx.x * 256 + threadIdx.x;
    if (i >= p.M * quads) return;
    const int64_t m = i / quads, n = (i - m * quads) * 4;
    typedef typename std::conditional<kKind == kKindI8, int, float>::type Elem;
    Elem sum[4] = {0, 0, 0, 0};
    // scales and bias as raw bits first, then eight partials, all in flight before the first
    // use (left alone, the scheduler pairs every load with its use: one memory round trip
    // each); the partials are summed in the order of the split
    u32 sa_raw = 0, sb_raw[4] = {0, 0, 0, 0}, bi_raw[4] = {0, 0, 0, 0};
    if (p.y) {
        if (kKind == kKindI8 && p.a_scale) sa_raw = load_raw<kBF16>(p.a_scale, m);
#pragma unroll
        for (int e = 0; e < 4; ++e) {
            if (p.b_scale) sb_raw[e] = load_raw<kBF16>(p.b_scale, n + e);
            if (p.bias) bi_raw[e] = load_raw<kBF16>(p.bias, n + e);
        }
    }
    for (int sp0 = 0; sp0 < p.splits; sp0 += 8) {
        v4u v[8];
#pragma unroll
        for (int u = 0; u < 8; ++u) {
            v[u] = v4u{0u, 0u, 0u, 0u};  // +0 of either type
            if (sp0 + u < p.splits)
                v[u] = *(const v4u*)((const u32*)p.part + ((int64_t)(sp0 + u) * p.M + m) * p.N + n);
        }
        __builtin_amdgcn_sched_barrier(0);
#pragma unroll
        for (int u = 0; u < 8; ++u)
#pragma unroll
            for (int e = 0; e < 4; ++e) {
                Elem t;
                from_bits(v[u][e], t);
                sum[e] += t;
            }
    }
    if constexpr (kKind == kKindI8) {
        if (p.acc_out) {
            v4i o = {(int)sum[0], (int)sum[1], (int)sum[2], (int)sum[3]};
            *(v4i*)(p.acc_out + m * p.N + n) = o;
        }
    }
    if (!p.y) return;
    float r[4];
    const bool has_bias = p.bias != nullptr;
#pragma unroll
    for (int e = 0; e < 4; ++e) {
        const float bv = has_bias ? raw_to_f32<kBF16>(bi_raw[e]) : 0.0f;
        if constexpr (kKind == kKindBF16) {
            const bool has_s = p.b_scale != nullptr;
            r[e] = descale_f<kBF16>((float)sum[e], has_s ? raw_to_f32<kBF16>(sb_raw[e]) : 1.0f, bv,
                                    has_s, has_bias);
        } else {
            float sa = p.a_scale ? raw_to_f32<kBF16>(sa_raw) : 1.0f;
            float sb = p.b_scale ? raw_to_f32<kBF16>(sb_raw[e]) : 1.0f;
            if (!kExact) {
                sa = 1.0f / sa;
                sb = 1.0f / sb;
            }
            r[e] = descale_i8<kBF16, kExact, 2>((int)sum[e], sa, sb, bv, has_bias,
                                                (p.flags & kFlagRoundAccBF16) != 0);
        }
    }
    if (kBF16) {
        v2u o = {pack_bf16x2(r[0], r[1]), pack_bf16x2(r[2], r[3])};
        *(v2u*)((uint16_t*)p.y + m * p.N + n) = o;
    } else {
        v4f o = {r[0], r[1], r[2], r[3]};
        *(v4f*)((float*)p.y + m * p.N + n) = o;
    }
}

// How many ways to split K.  A split pays where the tiles alone leave most of the chip idle
// and K is long.  Cost model fitted to a sweep (128 x 128 tiles, M = 128 .. 1024, K = 2048 ..
// 14336): an unsplit tile walks its stages at 0.65 us each, a split into sp saves
// (1 - 1/sp) of that, costs 4 us for the second kernel and 0.052 us per tile and split for
// writing and reading its 64 KiB of partials, and is taken while tiles * sp still fit on the
// chip at once.  E.g. 32 tiles x 32 stages: 4; 64 x 64: 4; 32 x 112: 8; 128 x 64: 3;
// 128 x 16 or 96 x 32: none.
inline int choose_splits(int64_t tiles, int64_t stages, int resident) {
    int best = 1;
    int64_t best_gain_ns = 0;
    for (int sp = 2; sp <= 8; ++sp) {
        if (tiles * sp > resident || stages / sp < 4) break;
        const int64_t gain_ns = stages * 650 * (sp - 1) / sp - tiles * sp * 52 - 4000;
        if (gain_ns > best_gain_ns) {
            best_gain_ns = gain_ns;
            best = sp;
        }
    }
    return best;
}


// Room for the partials of the largest split the launch may choose (sized for a chip of up
// to 256 CUs; a launch that finds less room splits less).
inline int64_t split_workspace_bytes(int64_t M, int64_t N, int64_t row_bytes) {
    if (M <= 0 || (row_bytes % kBK) != 0 || (N % 4) != 0) return 0;
    const int64_t tiles = ((M + 127) / 128) * ((N + 127) / 128);
    const int splits = choose_splits(tiles, row_bytes / kBK, 512);
    return splits > 1 ? (int64_t)splits * M * N * 4 : 0;
}

template <class T, int kKind, bool kBF16, bool kExact, bool kBStrip = false>
int launch_tile(GemmParams p, hipStream_t s) {
    // more than 64 KiB of dynamic LDS needs the attribute raised once per kernel
    static const bool raised =
        hipFuncSetAttribute((const void*)gemm_mfma<T, kKind, kBF16, kExact, kBStrip>,
                            hipFuncAttributeMaxDynamicSharedMemorySize, T::kLdsBytes) == hipSuccess;
    if (!raised) return K3Q_ERR_LAUNCH;
    p.tiles_m = (int)((p.M + T::kBM - 1) / T::kBM);
    p.tiles_n = (int)((p.N + T::kBN - 1) / T::kBN);
    // one resident set of workgroups (as many as fit on the chip at once, a multiple of the
    // 8 XCDs); each walks its share of the tiles
    const int resident = cu_count() * (T::kLdsBytes <= 64 * 1024 ? 2 : 1) / 8 * 8;
    const int stages = (int)(p.row_bytes / kBK);
    const int64_t tiles = (int64_t)p.tiles_m * p.tiles_n;
    int splits = (p.N % 4) ? 1 : choose_splits(tiles, stages, resident);
    // partials need room and 16-byte rows (no split for N % 4 != 0, above)
    if (splits > 1 && (!p.part || p.part_bytes < (int64_t)splits * p.M * p.N * 4)) {
        const int64_t fit = p.part ? p.part_bytes / (p.M * p.N * 4) : 0;
        splits = fit >= 2 ? (int)fit : 1;
    }
    p.kt_split = (stages + splits - 1) / splits;
    p.splits = (stages + p.kt_split - 1) / p.kt_split;  // no empty split
    const int64_t total = tiles * p.splits;
    int64_t grid = ((total + 7) / 8) * 8;
    if (resident >= 8 && grid > resident) grid = resident;
    gemm_mfma<T, kKind, kBF16, kExact, kBStrip><<<(unsigned)grid, T::kThreads, T::kLdsBytes, s>>>(p);
    if (p.splits > 1) {
        const int64_t threads = p.M * (p.N / 4);
        gemm_split_reduce<kKind, kBF16, kExact><<<(unsigned)((threads + 255) / 256), 256, 0, s>>>(p);
    }
    return launch_status();
}

// The large tile needs about one tile per CU to pay off; below that the small tile (four
// times as many workgroups, two per CU) keeps the chip busy.
constexpr int64_t kLargeTileMinTiles = 224;

template <int kKind, bool kBF16, bool kExact>
int launch_mfma(const GemmParams& p, hipStream_t s) {
    const int64_t large_tiles = ((p.M + 255) / 256) * ((p.N + 255) / 256);
    const bool large = large_tiles >= kLargeTileMinTiles;
    if constexpr (kKind == kKindI8) {
        if (p.b_strip) {
            if (large) return launch_tile<TileLarge, kKind, kBF16, kExact, true>(p, s);
            return launch_tile<TileSmall, kKind, kBF16, kExact, true>(p, s);
        }
    }
    if (large) return launch_tile<TileLarge, kKind, kBF16, kExact>(p, s);
    return launch_tile<TileSmall, kKind, kBF16, kExact>(p, s);
}

}  // namespace

bool gemm_bf16_nk_supported(int64_t M, int64_t N, int64_t K, const void* a, const void* bt,
                            const void* y) {
    return M > 0 && (2 * K) % kBK == 0 && aligned_to(a, 16) && aligned_to(bt, 16) &&
           aligned_to(y, 8) && ((M + 127) / 128) * ((N + 127) / 128) < (1 << 28);
}

int64_t gemm_bf16_nk_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    return split_workspace_bytes(M, N, 2 * K);
}

int gemm_bf16_nk_run(const void* a, const void* bt, int64_t M, int64_t N, int64_t K,
                     const void* b_scale, const void* bias, void* y, bool out_f32, void* workspace,
                     int64_t workspace_bytes, hipStream_t s) {
    GemmParams p{};
    if (workspace && aligned_to(workspace, 16)) {
        p.part = workspace;
        p.part_bytes = workspace_bytes;
    }
    p.a = (const int8_t*)a;
    p.bt = (const int8_t*)bt;
    p.b_scale = b_scale;
    p.bias = bias;
    p.y = y;
    p.M = M;
    p.N = N;
    p.K = K;
    p.row_bytes = 2 * K;
    if (out_f32) return launch_mfma<kKindBF16, false, true>(p, s);
    return launch_mfma<kKindBF16, true, true>(p, s);
}

}  // namespace k3q

using namespace k3q;

extern "C" int64_t k3q_gemm_i8_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (N <= 0 || K <= 0) return 0;
    // decode-sized M with the [K,N] kernel: int32 split-K partials; larger M with the [K,N]
    // kernel: room for the [N,K] copy made per call
    if (M > 0 && M <= kSkinnyMaxRows) {
        // either kernel layout may be passed: room for the larger of the two partial buffers
        const int64_t kn = ((N % 16) == 0 && (K % 8) == 0) ? gemm_i8_skinny_workspace_bytes(M, N, K) : N * K;
        const int64_t nk = gemm_i8_skinny_nk_workspace_bytes(M, N, K);
        return kn > nk ? kn : nk;
    }
    // K not a multiple of the tile's K step: zero-padded copies of both operands, then the
    // partials of a K split
    const int64_t Kpad = (K + kBK - 1) / kBK * kBK;
    if (Kpad != K) return (M + N) * Kpad + split_workspace_bytes(M, N, Kpad);
    // the [N,K] copy (16-byte multiple), then the partials of a K split
    return (N * K + 15) / 16 * 16 + split_workspace_bytes(M, N, K);
}

extern "C" int k3q_prepack_kernel_i8(const int8_t* kernel, int64_t K, int64_t N, int8_t* prepacked,
                                     void* stream) {
    if (K <= 0 || N <= 0) return K3Q_ERR_SHAPE;
    if (!kernel || !prepacked) return K3Q_ERR_NULL;
    dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
    transpose_i8<<<grid, 256, 0, (hipStream_t)stream>>>(kernel, prepacked, K, N, K);
    return launch_status();
}

extern "C" int k3q_gemm_i8_addend(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                                  const void* a_scale, const void* b_scale, const void* addend,
                                  int out_dtype, int flags, void* y, void* workspace,
                                  int64_t workspace_bytes, void* stream) {
    if (out_dtype != K3Q_F32 && out_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || N <= 0 || K <= 0) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!a || !b || !y || !addend) return K3Q_ERR_NULL;
    if (!gemm_i8_skinny_supported(M, N, K, a, b)) return K3Q_ERR_SHAPE;
    return gemm_i8_skinny_run(a, b, M, N, K, a_scale, b_scale, addend, out_dtype == K3Q_BF16, flags, y,
                              nullptr, workspace, workspace_bytes, (hipStream_t)stream, true);
}

extern "C" int k3q_gemm_i8(const int8_t* a, const int8_t* b, int b_layout, int64_t M, int64_t N,
                           int64_t K, const void* a_scale, const void* b_scale, const void* bias,
                           int out_dtype, int flags, void* y, int32_t* acc_out, void* workspace,
                           int64_t workspace_bytes, void* stream) {
    if (out_dtype != K3Q_F32 && out_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || N <= 0 || K <= 0) return K3Q_ERR_SHAPE;
    if (b_layout != 0 && b_layout != 1 && b_layout != 2) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!a || !b || (!y && !acc_out)) return K3Q_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    const bool bf16 = out_dtype == K3Q_BF16;

    GemmParams p{};
    p.a = a;
    p.a_scale = a_scale;
    p.b_scale = b_scale;
    p.bias = bias;
    p.y = y;
    p.acc_out = acc_out;
    p.M = M;
    p.N = N;
    p.K = K;
    p.row_bytes = K;
    p.flags = flags;

    const size_t el = bf16 ? 2 : 4;
    // decode-sized M: bandwidth-bound kernel that reads the [K,N] kernel in place
    if (b_layout == 0 && gemm_i8_skinny_supported(M, N, K, a, b))
        return gemm_i8_skinny_run(a, b, M, N, K, a_scale, b_scale, bias, bf16, flags, y, acc_out,
                                  workspace, workspace_bytes, s);
    // K % 128 != 0 (model widths like 1600 or 960): both operands are copied into scratch with
    // their rows zero-padded to the tile's K step; zeros add nothing, the result is the same
    const int64_t Kpad = (K + kBK - 1) / kBK * kBK;
    const bool padded = Kpad != K;
    bool fast = (padded ? (workspace && aligned_to(workspace, 16) && workspace_bytes >= (M + N) * Kpad)
                        : (aligned_to(a, 16) && aligned_to(b, 16))) &&
                (!y || aligned_to(y, 4 * el)) && (!acc_out || aligned_to(acc_out, 16)) &&
                (!b_scale || aligned_to(b_scale, 16)) && (!bias || aligned_to(bias, 16)) &&
                ((M + 127) / 128) * ((N + 127) / 128) < (1 << 28);
    // [N,K] kernel at decode sizes: the streaming kernel up to 8 rows; beyond that the 128-row
    // tiles (which split K while they are few) are as fast or faster (K = N = 8192, 16 rows:
    // 24 us streamed, 19 us tiled; vocabulary 32000 x 4096, 64 rows: 176 us in passes, 41 us tiled)
    if (b_layout == 1 && gemm_i8_skinny_nk_supported(M, N, K, a, b) &&
        (M <= 8 || !fast))
        return gemm_i8_skinny_nk_run(a, b, M, N, K, a_scale, b_scale, bias, bf16, flags, y, acc_out,
                                     workspace, workspace_bytes, s);
    char* scratch = (workspace && aligned_to(workspace, 16)) ? (char*)workspace : nullptr;
    int64_t scratch_bytes = scratch ? workspace_bytes : 0;
    if (b_layout == 2) {
        // the strip-linear copy of the decode kernel as the tiles' B operand: the tile kernel or nothing
        if (!fast || padded) return K3Q_ERR_SHAPE;
        p.bt = b;
        p.b_strip = 1;
        p.b_units = (int)(K / 64);
    } else if (fast && padded) {
        int8_t* a_pad = (int8_t*)scratch;
        int8_t* b_pad = a_pad + M * Kpad;
        pad_rows_i8<<<(unsigned)((M * (Kpad / 16) + 255) / 256), 256, 0, s>>>(a, a_pad, M, K, Kpad);
        if (b_layout == 0) {
            dim3 grid((unsigned)((N + 63) / 64), (unsigned)(Kpad / 64));
            transpose_i8<<<grid, 256, 0, s>>>(b, b_pad, K, N, Kpad);
        } else {
            pad_rows_i8<<<(unsigned)((N * (Kpad / 16) + 255) / 256), 256, 0, s>>>(b, b_pad, N, K, Kpad);
        }
        p.a = a_pad;
        p.bt = b_pad;
        p.row_bytes = Kpad;
        scratch += (M + N) * Kpad;
        scratch_bytes -= (M + N) * Kpad;
    } else if (fast && b_layout == 0) {
        // needs the [N,K] copy: made here per call when the caller supplies scratch for it
        const int64_t copy_bytes = (N * K + 15) / 16 * 16;
        if (scratch && scratch_bytes >= N * K) {
            int rc = k3q_prepack_kernel_i8(b, K, N, (int8_t*)scratch, stream);
            if (rc != K3Q_OK) return rc;
            p.bt = (const int8_t*)scratch;
            scratch_bytes = scratch_bytes > copy_bytes ? scratch_bytes - copy_bytes : 0;
            scratch += copy_bytes;
        } else {
            fast = false;
        }
    } else {
        p.bt = b;
    }
    p.part = scratch_bytes > 0 ? scratch : nullptr;  // partials of a K split
    p.part_bytes = scratch_bytes;
    if (fast) {
        const bool exact = (flags & kFlagExactEpilogue) != 0;
        if (bf16) return exact ? launch_mfma<kKindI8, true, true>(p, s) : launch_mfma<kKindI8, true, false>(p, s);
        return exact ? launch_mfma<kKindI8, false, true>(p, s) : launch_mfma<kKindI8, false, false>(p, s);
    }

    if (M > 65535) return K3Q_ERR_SHAPE;
    dim3 grid((unsigned)((N + 255) / 256), (unsigned)M);
    const int64_t sk = b_layout == 0 ? N : 1;
    const int64_t sn = b_layout == 0 ? 1 : K;
    if (bf16)
        gemm_i8_simple<true><<<grid, 256, 0, s>>>(a, b, sk, sn, p);
    else
        gemm_i8_simple<false><<<grid, 256, 0, s>>>(a, b, sk, sn, p);
    return launch_status();
}

extern "C" int64_t k3q_gemm_w8_workspace_bytes(int64_t M, int64_t N, int64_t K) {
    if (M <= 0 || N <= 0 || K <= 0) return 0;
    // the kernel widened to bfloat16 (twice, plus the split rows of x, for float32 inputs:
    // sized for that), then the partials of a K split
    return (N + M) * 2 * K * 2 + split_workspace_bytes(M, N, 4 * K);
}

extern "C" int k3q_gemm_w8(const void* x, int x_dtype, const int8_t* b, int b_layout, int64_t M,
                           int64_t N, int64_t K, const void* b_scale, const void* bias, void* y,
                           void* workspace, int64_t workspace_bytes, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || N <= 0 || K <= 0) return K3Q_ERR_SHAPE;
    if (b_layout != 0 && b_layout != 1) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!x || !b || !y) return K3Q_ERR_NULL;
    hipStream_t s = (hipStream_t)stream;
    const bool bf16 = x_dtype == K3Q_BF16;
    // decode sizes on a K-contiguous kernel: streamed in place, nothing widened
    if (b_layout == 1 && gemv_w8_nk_supported(M, N, K, x_dtype, x, b, y) &&
        (!b_scale || aligned_to(b_scale, 4)) && (!bias || aligned_to(bias, 4)))
        return gemv_w8_nk_run(x, x_dtype, b, M, N, K, b_scale, bias, y, s);
    // MFMA route: the kernel widened to bfloat16 in scratch (exact).  float32 x goes there as
    // its high and low bfloat16 parts side by side, [xh | xl] against [w | w]: one bfloat16
    // GEMM over 2K with float32 accumulation and a float32 epilogue (x to 2^-17 relative).
    const int64_t parts = bf16 ? 1 : 2;
    const int64_t wt_bytes = N * parts * K * 2, xs_bytes = bf16 ? 0 : M * parts * K * 2;
    const void* a_op = bf16 ? x : (const void*)((char*)workspace + wt_bytes);
    const bool fast = workspace && workspace_bytes >= wt_bytes + xs_bytes && aligned_to(workspace, 16) &&
                      aligned_to(b, 16) && aligned_to(x, 16) && (K % 64) == 0 &&
                      (!b_scale || aligned_to(b_scale, 4)) &&
                      gemm_bf16_nk_supported(M, N, parts * K, a_op, workspace, y) &&
                      aligned_to(y, bf16 ? 8 : 16);
    if (fast) {
        if (b_layout == 1) {
            const int64_t count16 = N * K / 16;
            widen_i8_to_bf16<<<(unsigned)((count16 + 255) / 256), 256, 0, s>>>(
                b, (uint16_t*)workspace, count16, K, parts * K, !bf16);
        } else {
            dim3 grid((unsigned)((N + 63) / 64), (unsigned)((K + 63) / 64));
            transpose_widen_i8_to_bf16<<<grid, 256, 0, s>>>(b, (uint16_t*)workspace, K, N, parts * K,
                                                            !bf16);
        }
        if (!bf16) split_f32_rows_launch((const float*)x, (uint16_t*)a_op, M, K, 2, s);
        char* rest = (char*)workspace + wt_bytes + xs_bytes;
        return gemm_bf16_nk_run(a_op, workspace, M, N, parts * K, b_scale, bias, y, !bf16, rest,
                                workspace_bytes - wt_bytes - xs_bytes, s);
    }
    if (M > 65535) return K3Q_ERR_SHAPE;
    dim3 grid((unsigned)((N + 255) / 256), (unsigned)M);
    const int64_t sk = b_layout == 0 ? N : 1;
    const int64_t sn = b_layout == 0 ? 1 : K;
    if (bf16)
        gemm_w8_simple<true><<<grid, 256, 0, s>>>(x, b, sk, sn, b_scale, bias, y, N, K);
    else
        gemm_w8_simple<false><<<grid, 256, 0, s>>>(x, b, sk, sn, b_scale, bias, y, N, K);
    return launch_status();
}

extern "C" int64_t k3q_gemm_wbf16_workspace_bytes(int64_t M, int64_t N, int64_t K, int parts) {
    if (M <= 0 || N <= 0 || K <= 0 || parts < 1 || parts > 3) return 0;
    // the split rows of float32 x, then the partials of a K split
    return (parts > 1 ? M * parts * K * 2 : 0) + split_workspace_bytes(M, N, 2 * parts * K);
}

extern "C" int k3q_gemm_wbf16(const void* x, int x_dtype, const uint16_t* wt, int parts, int64_t M,
                              int64_t N, int64_t K, const void* bias, void* y, void* workspace,
                              int64_t workspace_bytes, void* stream) {
    if (x_dtype != K3Q_F32 && x_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (M < 0 || N <= 0 || K <= 0) return K3Q_ERR_SHAPE;
    const bool bf16 = x_dtype == K3Q_BF16;
    if (bf16 ? parts != 1 : (parts != 2 && parts != 3)) return K3Q_ERR_SHAPE;
    if (M == 0) return K3Q_OK;
    if (!x || !wt || !y) return K3Q_ERR_NULL;
    const size_t el = bf16 ? 2 : 4;
    if (!aligned_to(x, el) || !aligned_to(wt, 2) || !aligned_to(y, el) || (bias && !aligned_to(bias, el)))
        return K3Q_ERR_ALIGN;
    hipStream_t s = (hipStream_t)stream;
    const int64_t xs_bytes = bf16 ? 0 : M * parts * K * 2;
    const void* a_op = bf16 ? x : workspace;
    const bool fast = (K % 64) == 0 && aligned_to(x, 16) && (bf16 || (K % 4) == 0) &&
                      (bf16 || (workspace && workspace_bytes >= xs_bytes && aligned_to(workspace, 16))) &&
                      gemm_bf16_nk_supported(M, N, parts * K, a_op, wt, y) &&
                      aligned_to(y, bf16 ? 8 : 16) && (!bias || aligned_to(bias, 4));
    if (fast) {
        if (!bf16) split_f32_rows_launch((const float*)x, (uint16_t*)workspace, M, K, parts, s);
        char* rest = workspace ? (char*)workspace + xs_bytes : nullptr;
        return gemm_bf16_nk_run(a_op, wt, M, N, parts * K, nullptr, bias, y, !bf16, rest,
                                workspace ? workspace_bytes - xs_bytes : 0, s);
    }
    if (M > 65535) return K3Q_ERR_SHAPE;
    dim3 grid((unsigned)((N + 255) / 256), (unsigned)M);
    if (bf16)
        gemm_wbf16_simple<true><<<grid, 256, 0, s>>>(x, wt, parts, bias, y, N, K);
    else
        gemm_wbf16_simple<false><<<grid, 256, 0, s>>>(x, wt, parts, bias, y, N, K);
    return launch_status();
}
