// Quantized embedding lookup: out[t, :] = dequantise(table[ids[t], :]).
//
// Replaces the gather + cast + divide (or grouped subtract / multiply) chain of
// Embedding._int8_call / _int4_call (keras/src/layers/core/embedding.py:521-582):
// one read of the selected int8 / packed-int4 rows, one write of the float rows, no
// unpacked or gathered intermediates in memory.  HBM-bound on the output write.
//
//   int8            out = T(q) / scale[row]
//   int4 per row    out = T(nibble) / scale[row]          (low nibble = even column)
//   int4 grouped    out = (T(nibble) - zero[row, g]) * scale[row, g],  g = column / block
//
// T is the output dtype.  bfloat16 output is only produced when the scales are bfloat16
// too (otherwise the reference's type promotion yields float32); each arithmetic step is
// then rounded to bfloat16 as torch rounds it.  Negative ids wrap once by the vocabulary
// size (keras/src/backend/torch/numpy.py:2005-2017); ids still out of range produce a row
// of zeros and raise the caller's flag word instead of faulting.
#include "k3q_common.h"

namespace k3q {
namespace {

struct EmbParams {
    const void* ids;
    const int8_t* table;
    const void* scale;
    const int8_t* zero;
    void* out;
    int* oob_flag;
    int64_t count, vocab, dim, row_bytes, groups, block_size;
    int64_t parts, part_pieces;  // waves per row and 16-byte output pieces per wave (vector kernel)
};

template <bool kBF16>
__device__ __forceinline__ float scale_at(const void* p, int64_t i) {
    if (kBF16) return bf16_bits_to_f32(((const uint16_t*)p)[i]);
    return ((const float*)p)[i];
}

template <bool kOutBF16>
__device__ __forceinline__ float dequant(float q, float s, float z, bool grouped) {
    if (grouped) {
        const float d = q - z;  // exact: |q - z| <= 255
        return kOutBF16 ? round_bf16(d * s) : d * s;
    }
    return kOutBF16 ? round_bf16(q / s) : q / s;
}

template <typename IdT>
__device__ __forceinline__ int64_t row_of(const EmbParams& p, int64_t t, bool* ok) {
    int64_t r = (int64_t)((const IdT*)p.ids)[t];
    if (r < 0) r += p.vocab;
    *ok = r >= 0 && r < p.vocab;
    if (!*ok) {
        if (p.oob_flag) *(volatile int*)p.oob_flag = 1;
        r = 0;
    }
    return r;
}

// One wave per token.  A lane's piece is whatever de-quantises to one 16-byte store (4
// float32 or 8 bfloat16 outputs, i.e. 2..8 bytes of the table row), so that consecutive
// lanes read consecutive table bytes and every store instruction of the wave writes 1 KiB
// of contiguous output.  Needs dim % piece == 0 and, grouped, block_size % piece == 0.
template <int kBits, bool kScaleBF16, bool kOutBF16, bool kGrouped, typename IdT>
__global__ __launch_bounds__(256) void embedding_rows(EmbParams p) {
    constexpr int kOut = kOutBF16 ? 8 : 4;       // outputs per piece
    constexpr int kIn = kOut * kBits / 8;        // table bytes per piece: 8, 4 or 2
    constexpr int kUnroll = 16;  // a 4096-wide float32 row in one round of loads (4: 143 us for 32768 rows, 8: 128, 16: 124)
    const int lane = threadIdx.x & 63;
    // a row is shared by p.parts waves (more than one only when there are few tokens)
    const int64_t wid = (int64_t)blockIdx.x * 4 + (threadIdx.x >> 6);
    const int64_t t = wid / p.parts;
    if (t >= p.count) return;
    bool ok;
    const int64_t row = row_of<IdT>(p, t, &ok);
    const char* src = (const char*)p.table + row * p.row_bytes;
    const int64_t first = (wid - t * p.parts) * p.part_pieces;
    int64_t pieces = first + p.part_pieces;
    if (pieces > p.dim / kOut) pieces = p.dim / kOut;
    float s_row = 1.0f;
    if (!kGrouped) s_row = scale_at<kScaleBF16>(p.scale, row);
    for (int64_t c0 = first; c0 < pieces; c0 += 64 * kUnroll) {
        uint64_t w[kUnroll];
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t c = c0 + 64 * u + lane;
            w[u] = 0;
            if (c < pieces) {
                if (kIn == 8)
                    w[u] = __builtin_nontemporal_load((const uint64_t*)(src + c * 8));
                else if (kIn == 4)
                    w[u] = __builtin_nontemporal_load((const u32*)(src + c * 4));
                else
                    w[u] = __builtin_nontemporal_load((const uint16_t*)(src + c * 2));
            }
        }
#pragma unroll
        for (int u = 0; u < kUnroll; ++u) {
            const int64_t c = c0 + 64 * u + lane;
            if (c >= pieces) continue;
            const int64_t col = c * kOut;
            float s = s_row, z = 0.0f;
            if (kGrouped) {
                const int64_t gi = row * p.groups + col / p.block_size;
                s = scale_at<kScaleBF16>(p.scale, gi);
                z = (float)p.zero[gi];
            }
            float v[kOut];
#pragma unroll
            for (int e = 0; e < kOut; ++e) {
                float q;
                if (kBits == 8) {
                    q = (float)(int)(int8_t)(w[u] >> (8 * e));
                } else {
                    const u32 nib = (u32)(w[u] >> (4 * e)) & 0xfu;  // low nibble = even column
                    q = (float)((int)(nib ^ 8u) - 8);
                }
                v[e] = ok ? dequant<kOutBF16>(q, s, z, kGrouped) : 0.0f;
            }
            if (kOutBF16) {
                v4u o;
#pragma unroll
                for (int d = 0; d < 4; ++d)
                    o[d] = f32_to_bf16_bits(v[2 * d]) | (f32_to_bf16_bits(v[2 * d + 1]) << 16);
                __builtin_nontemporal_store(o, (v4u*)((uint16_t*)p.out + t * p.dim + col));
            } else {
                v4f o = {v[0], v[1], v[2], v[3]};
                __builtin_nontemporal_store(o, (v4f*)((float*)p.out + t * p.dim + col));
            }
        }
    }
}

// Any dim / block size: one thread per output element.
template <int kBits, bool kScaleBF16, bool kOutBF16, bool kGrouped, typename IdT>
__global__ __launch_bounds__(256) void embedding_generic(EmbParams p) {
    const int64_t t = blockIdx.y;
    bool ok;
    const int64_t row = row_of<IdT>(p, t, &ok);
    for (int64_t col = (int64_t)blockIdx.x * 256 + threadIdx.x; col < p.dim;
         col += (int64_t)gridDim.x * 256) {
        float q;
        if (kBits == 8) {
            q = (float)p.table[row * p.row_bytes + col];
        } else {
            const u32 byte = (uint8_t)p.table[row * p.row_bytes + (col >> 1)];
            const u32 nib = (col & 1) ? (byte >> 4) : (byte & 0xfu);
            q = (float)((int)(nib ^ 8u) - 8);
        }
        float s, z = 0.0f;
        if (kGrouped) {
            const int64_t gi = row * p.groups + col / p.block_size;
            s = scale_at<kScaleBF16>(p.scale, gi);
            z = (float)p.zero[gi];
        } else {
            s = scale_at<kScaleBF16>(p.scale, row);
        }
        const float v = ok ? dequant<kOutBF16>(q, s, z, kGrouped) : 0.0f;
        if (kOutBF16)
            ((uint16_t*)p.out)[t * p.dim + col] = (uint16_t)f32_to_bf16_bits(v);
        else
            ((float*)p.out)[t * p.dim + col] = v;
    }
}

template <int kBits, bool kScaleBF16, bool kOutBF16, bool kGrouped, typename IdT>
void launch(const EmbParams& p, bool vec, hipStream_t s) {
    if (vec) {
        // few tokens (decode): spread each row over several waves, down to 64 pieces a wave
        EmbParams q = p;
        const int64_t pieces = p.dim / (kOutBF16 ? 8 : 4);
        int64_t parts = 1;
        while (p.count * parts < 2048 && pieces / (parts * 2) >= 64) parts *= 2;
        q.parts = parts;
        q.part_pieces = ((pieces + parts - 1) / parts + 63) / 64 * 64;
        embedding_rows<kBits, kScaleBF16, kOutBF16, kGrouped, IdT>
            <<<(unsigned)((p.count * parts + 3) / 4), 256, 0, s>>>(q);
    } else {
        // grid.y is limited to 65535 tokens per launch
        for (int64_t t0 = 0; t0 < p.count; t0 += 65535) {
            EmbParams q = p;
            const int64_t n = p.count - t0 < 65535 ? p.count - t0 : 65535;
            q.ids = (const char*)p.ids + t0 * sizeof(IdT);
            q.out = (char*)p.out + t0 * p.dim * (kOutBF16 ? 2 : 4);
            q.count = n;
            unsigned gx = (unsigned)((p.dim + 255) / 256);
            if (gx > 64) gx = 64;
            embedding_generic<kBits, kScaleBF16, kOutBF16, kGrouped, IdT>
                <<<dim3(gx, (unsigned)n), 256, 0, s>>>(q);
        }
    }
}

template <int kBits, bool kScaleBF16, bool kOutBF16, bool kGrouped>
void launch_ids(const EmbParams& p, int ids_dtype, bool vec, hipStream_t s) {
    if (ids_dtype == K3Q_I64)
        launch<kBits, kScaleBF16, kOutBF16, kGrouped, int64_t>(p, vec, s);
    else
        launch<kBits, kScaleBF16, kOutBF16, kGrouped, int32_t>(p, vec, s);
}

template <int kBits, bool kGrouped>
void launch_types(const EmbParams& p, int ids_dtype, int scale_dtype, int out_dtype, bool vec,
                  hipStream_t s) {
    if (out_dtype == K3Q_BF16)  // implies bfloat16 scales
        launch_ids<kBits, true, true, kGrouped>(p, ids_dtype, vec, s);
    else if (scale_dtype == K3Q_BF16)
        launch_ids<kBits, true, false, kGrouped>(p, ids_dtype, vec, s);
    else
        launch_ids<kBits, false, false, kGrouped>(p, ids_dtype, vec, s);
}

}  // namespace
}  // namespace k3q

using namespace k3q;

extern "C" int k3q_embedding_lookup(const void* ids, int ids_dtype, int64_t count,
                                    const int8_t* table, int64_t vocab, int64_t dim, int bits,
                                    const void* scale, int scale_dtype, const int8_t* zero,
                                    int64_t block_size, int out_dtype, void* out, int* oob_flag,
                                    void* stream) {
    if (ids_dtype != K3Q_I32 && ids_dtype != K3Q_I64) return K3Q_ERR_DTYPE;
    if ((scale_dtype != K3Q_F32 && scale_dtype != K3Q_BF16) ||
        (out_dtype != K3Q_F32 && out_dtype != K3Q_BF16))
        return K3Q_ERR_DTYPE;
    // float32 scales promote the result to float32 in the reference
    if (out_dtype == K3Q_BF16 && scale_dtype != K3Q_BF16) return K3Q_ERR_DTYPE;
    if (bits != 8 && bits != 4) return K3Q_ERR_SHAPE;
    if (count < 0 || vocab <= 0 || dim <= 0) return K3Q_ERR_SHAPE;
    const bool grouped = block_size > 0;
    if (grouped && bits != 4) return K3Q_ERR_SHAPE;
    if (count == 0) return K3Q_OK;
    if (!ids || !table || !scale || !out) return K3Q_ERR_NULL;
    if (grouped && !zero) return K3Q_ERR_NULL;
    const size_t sel = scale_dtype == K3Q_F32 ? 4 : 2, oel = out_dtype == K3Q_F32 ? 4 : 2;
    if (!aligned_to(ids, ids_dtype == K3Q_I64 ? 8 : 4) || !aligned_to(scale, sel) ||
        !aligned_to(out, oel) || (oob_flag && !aligned_to(oob_flag, 4)))
        return K3Q_ERR_ALIGN;

    EmbParams p{};
    p.ids = ids;
    p.table = table;
    p.scale = scale;
    p.zero = zero;
    p.out = out;
    p.oob_flag = oob_flag;
    p.count = count;
    p.vocab = vocab;
    p.dim = dim;
    p.row_bytes = bits == 8 ? dim : (dim + 1) / 2;
    p.block_size = grouped ? block_size : 0;
    p.groups = grouped ? (dim + block_size - 1) / block_size : 0;
    // a piece is one 16-byte store: 4 float32 or 8 bfloat16 outputs
    const int piece = out_dtype == K3Q_BF16 ? 8 : 4;
    const bool vec = (dim % piece) == 0 && aligned_to(table, 8) && aligned_to(out, 16) &&
                     (!grouped || (block_size % piece) == 0);
    hipStream_t s = (hipStream_t)stream;
    if (bits == 8)
        launch_types<8, false>(p, ids_dtype, scale_dtype, out_dtype, vec, s);
    else if (grouped)
        launch_types<4, true>(p, ids_dtype, scale_dtype, out_dtype, vec, s);
    else
        launch_types<4, false>(p, ids_dtype, scale_dtype, out_dtype, vec, s);
    return launch_status();
}
