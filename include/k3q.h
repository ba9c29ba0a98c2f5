/*
 * k3q -- C ABI of the MI355X (gfx950) kernels behind the Keras 3 quantized
 * Dense / EinsumDense forward.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer owned by the caller; nothing is
 *     allocated, freed or retained by the library (scratch memory is passed in
 *     as `workspace`), so the calls are re-entrant and hold no global state;
 *   - `stream` is a hipStream_t passed as void*; kernels are enqueued on it and
 *     the call returns without synchronising;
 *   - the return value is K3Q_OK or a negative K3Q_ERR_* code; nothing is
 *     launched when an argument is rejected;
 *   - dtype codes: K3Q_F32 = 0, K3Q_BF16 = 1; index dtypes K3Q_I32 = 2, K3Q_I64 = 3.
 *
 * The reference (keras-team/keras 3.16.0) has no FFI: these entry points
 * replace chains of torch ops, and each comment cites the chain it replaces.
 */
#ifndef K3Q_H_
#define K3Q_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

#define K3Q_F32 0
#define K3Q_BF16 1
#define K3Q_I32 2
#define K3Q_I64 3

#define K3Q_OK 0
#define K3Q_ERR_NULL (-1)      /* a required pointer is null                    */
#define K3Q_ERR_SHAPE (-2)     /* negative / zero / inconsistent extent          */
#define K3Q_ERR_ALIGN (-3)     /* pointer or stride breaks the stated alignment  */
#define K3Q_ERR_DTYPE (-4)     /* unknown dtype code                             */
#define K3Q_ERR_WORKSPACE (-5) /* workspace missing or smaller than required     */
#define K3Q_ERR_LAUNCH (-6)    /* the HIP runtime refused the launch             */
#define K3Q_ERR_RANGE (-7)     /* value_range outside what the output can hold   */

/* Library version: major * 10000 + minor * 100 + patch. */
int k3q_version(void);

/* Static, human readable text for a K3Q_* code. */
const char* k3q_error_string(int code);

/*
 * Row-wise abs-max quantizer.
 * Replaces the tensor path of keras.quantizers.abs_max_quantize
 * (keras/src/quantizers/quantizers.py:111-120: abs, amax(keepdims), add eps,
 * divide, cast, multiply, round, clip, cast) for a reduction over the trailing
 * `cols` elements of each of `rows` rows:
 *     scale[r] = T(qhi / T(amax_r + T(eps)));  q[r,c] = int8(clip(rne(T(x[r,c]*scale[r])), qlo, qhi))
 * with every step rounded to T = x_dtype, as torch does.
 * x: [rows, cols] with row stride `x_row_stride` elements; q: contiguous
 * [rows, cols] int8; scale: [rows] of x_dtype.
 */
int k3q_absmax_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols,
                        int64_t x_row_stride, float eps, float qlo, float qhi,
                        int8_t* q, void* scale, void* stream);

/*
 * The weight quantizers of `quantize()` for kernels that live on the device.  The reference
 * runs them in numpy on the host (`to_numpy=True`); these repeat its float32 operations one
 * by one, so q, scale and zero are the bits numpy produces (bfloat16 inputs are widened to
 * float32 first and the scale is rounded back to bfloat16 at the end).
 *
 * k3q_weight_absmax_quantize replaces keras/src/quantizers/quantizers.py:95-109 for a reduction
 * over the middle axis of a contiguous x [outer, R, inner] (Dense: axis 0 of [K, N] is outer 1,
 * R = K, inner = N; EinsumDense: its kernel's reduced axes):
 *     scale[o, i] = hi / (max_r |x[o, r, i]| + eps);  q = int8(clip(rint(x * scale), lo, hi))
 * q: [outer, R, inner] int8; scale: [outer, inner] of x_dtype; amax_workspace: outer * inner
 * 32-bit words of scratch (cleared by the call).  outer <= 65535, R <= 65535 * 256.
 *
 * k3q_weight_quantize_grouped replaces the numpy variant of
 * abs_max_quantize_grouped_with_zero_point, quantizers.py:182-234, for x [K, N]: groups of
 * `block_size` rows (the last one zero-padded), per (group, column)
 *     scale = ((max - min) + eps) / (hi - lo);  zero = clip(rint(-min / scale) + lo, lo, hi)
 *     q = int8(clip(rint(x / scale) + zero, lo, hi))
 * q: [K, N] int8; scale: [ceil(K / block_size), N] of x_dtype; zero: the same shape, int8.
 */
int k3q_weight_absmax_quantize(const void* x, int x_dtype, int64_t outer, int64_t R, int64_t inner,
                               float epsilon, float range_lo, float range_hi, int8_t* q, void* scale,
                               void* amax_workspace, void* stream);
int k3q_weight_quantize_grouped(const void* x, int x_dtype, int64_t K, int64_t N, int64_t block_size,
                                float epsilon, float range_lo, float range_hi, int8_t* q, void* scale,
                                int8_t* zero, void* stream);

/*
 * pack_int4 along the middle axis of a contiguous [outer, len, inner] int8 or
 * uint8 tensor -> [outer, ceil(len/2), inner]; byte = (lo & 15) | ((hi & 15) << 4),
 * an odd `len` is padded with one zero slice.
 * Replaces keras.quantizers.pack_int4 (keras/src/quantizers/quantizers.py:715-750).
 */
int k3q_pack_int4(const void* in, int64_t outer, int64_t len, int64_t inner,
                  void* out, void* stream);

/*
 * unpack_int4: [outer, packed_len, inner] -> [outer, orig_len, inner] with
 * orig_len in {2*packed_len - 1, 2*packed_len}; is_signed applies (v ^ 8) - 8.
 * Replaces keras.quantizers.unpack_int4 (keras/src/quantizers/quantizers.py:830-900).
 */
int k3q_unpack_int4(const void* in, int64_t outer, int64_t packed_len, int64_t inner,
                    int64_t orig_len, int is_signed, void* out, void* stream);

/*
 * int8 x int8 -> int32 matmul with the Dense / EinsumDense de-scale fused:
 *     acc[m,n] = sum_k a[m,k] * b[k,n]                       (exact int32)
 *     y[m,n]   = T(T(acc[m,n]) / T(b_scale[n] * a_scale[m]))  (+ bias[n])
 * a: [M,K] int8 (the quantised activations).  b: the layer's int8 kernel, either
 * as the variable stores it, [K,N] (b_layout 0), or as the [N,K] shadow copy made
 * by k3q_prepack_kernel_i8 (b_layout 1), or as the strip-linear copy that the int8 decode
 * kernel streams (k3q_w8s_pack; b_layout 2: MFMA tile kernel only, K % 128 == 0, the same
 * accumulators and bits -- a layer then keeps ONE derived copy of its kernel for every row
 * count; K3Q_ERR_SHAPE where the tile kernel does not apply).  a_scale [M], b_scale [N], bias [N] are
 * of out_dtype; a null scale counts as 1, a null bias as absent.  y: out_dtype
 * [M,N] or null.  acc_out: int32 [M,N] or null (the raw accumulators, for
 * bit-exact checks).  At least one of y / acc_out must be given.
 * flags bit 0 (K3Q_GEMM_EXACT_EPILOGUE): round after every step exactly as the
 * reference's op chain does; otherwise y = T(acc * (1/a_scale) * (1/b_scale) + bias)
 * with one final rounding (differs from the chain by at most the chain's own
 * intermediate roundings).
 * The MFMA kernel needs K % 128 == 0 and 16-byte aligned operands (any N; with
 * N % 4 != 0 the rows of y are stored element by element and K is never split).
 * With K % 128 != 0 (a model width of 1600 or 960) and a `workspace` of
 * k3q_gemm_i8_workspace_bytes (either b_layout) both operands are first copied into it
 * with their rows zero-padded to the next multiple of 128: the same accumulators, bit for
 * bit.  Other shapes run a plain kernel.  With b_layout 0 the MFMA kernel also needs
 * `workspace` (k3q_gemm_i8_workspace_bytes, 16-byte aligned) to hold the [N,K]
 * copy it makes on every call; callers that reuse a kernel should prepack once.
 * flags bit 1 (K3Q_GEMM_ROUND_ACC_BF16, float32 output only): acc is cast to bfloat16
 * before the division, which is what a bfloat16-compute layer with float32 scales
 * computes (ReversibleEmbedding reads its scale without autocast).
 * Decode sizes run bandwidth-bound kernels that stream b in place, always with the
 * exact epilogue: b_layout 0 up to 64 rows (N % 16 == 0, K % 8 == 0; passes of 16
 * rows), b_layout 1 -- e.g. a tied int8 embedding table used as the LM head -- up to
 * 8 rows (K % 64 == 0; up to 64 rows when the MFMA kernel's conditions do not hold).
 * They may split K and then need `workspace` for int32 partials.  The MFMA kernel
 * itself picks 128 x 128 tiles while 256 x 256 tiles would leave CUs idle, and where
 * even those are few and K is long (e.g. M = 128, K = N = 8192) it splits K over
 * workgroups: int32 partials in `workspace` after the [N,K] copy's place
 * (ceil16(N * K) bytes in; with b_layout 1 only that second part is of use and a
 * workspace of k3q_gemm_i8_workspace_bytes - ceil16(N * K) bytes may be passed), summed
 * by a second kernel that applies the epilogue; results are the same bits either way.
 * Without that room K is not split.
 * The reverse projection of ReversibleEmbedding._int8_call
 * (keras/src/layers/core/reversible_embedding.py:272-296) is this call with
 * b = the [vocab, dim] table as stored, b_layout 1 and no bias.
 * Replaces cast, cast, matmul (keras/src/backend/torch/numpy.py:139-157), cast,
 * multiply, divide, add of Dense._int8_call (keras/src/layers/core/dense.py:961-983)
 * and the einsum form in EinsumDense._int8_call
 * (keras/src/layers/core/einsum_dense.py:1072-1084).
 */
#define K3Q_GEMM_EXACT_EPILOGUE 1
#define K3Q_GEMM_ROUND_ACC_BF16 2
int64_t k3q_gemm_i8_workspace_bytes(int64_t M, int64_t N, int64_t K);
int k3q_prepack_kernel_i8(const int8_t* kernel, int64_t K, int64_t N, int8_t* prepacked,
                          void* stream);
int k3q_gemm_i8(const int8_t* a, const int8_t* b, int b_layout, int64_t M, int64_t N, int64_t K,
                const void* a_scale, const void* b_scale, const void* bias, int out_dtype,
                int flags, void* y, int32_t* acc_out, void* workspace, int64_t workspace_bytes,
                void* stream);

/*
 * k3q_gemm_i8 at decode sizes (M <= 64, b as [K, N], N % 16 == 0, K % 8 == 0; anything else
 * K3Q_ERR_SHAPE) for a layer without bias, with an [M, N] addend (the output dtype,
 * row-major, may be y itself) added to the de-scaled product the way a bias is:
 *     y[m, n] = T(T(acc / scales)[m, n] + addend[m, n])
 * which is `residual + layer(x)` of the reference's op sequence
 * (keras/src/layers/core/dense.py:961-983 followed by the caller's add) in the same launch.
 */
int k3q_gemm_i8_addend(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                       const void* a_scale, const void* b_scale, const void* addend, int out_dtype,
                       int flags, void* y, void* workspace, int64_t workspace_bytes, void* stream);

/*
 * Weight-only int8 matmul: float activations, int8 kernel (a Dense int8 layer whose
 * config has no activation quantizer):
 *     y = T(T(x . b) / b_scale[n]) (+ bias)
 * x: [M, K] float32 or bfloat16; b as in k3q_gemm_i8 ([K,N] with b_layout 0, the
 * prepacked [N,K] with b_layout 1); b_scale, bias, y of x_dtype.  Decode sizes (M <= 8,
 * b_layout 1, K % 16 == 0, 16-byte aligned x and b) stream the kernel in place, once per
 * four rows of x, with fp32 accumulation (K = N = 8192, M = 1: 13 us).  Otherwise, with
 * K % 64 == 0, N % 4 == 0 and `workspace` (k3q_gemm_w8_workspace_bytes, 16-byte aligned),
 * the kernel is widened to bfloat16 in scratch (exact) and the MFMA tile kernel runs on it;
 * float32 x goes there as its high and low bfloat16 parts ([xh | xl] against [w | w], float32
 * accumulation and epilogue, x to 2^-17 relative).  Everything else runs a plain kernel
 * with fp32 accumulation.
 * Replaces matmul (float x int8: both cast to the float type,
 * keras/src/backend/torch/numpy.py:139-157), cast, divide, add of Dense._int8_call
 * without inputs_quantizer (keras/src/layers/core/dense.py:961-983).
 */
int64_t k3q_gemm_w8_workspace_bytes(int64_t M, int64_t N, int64_t K);
int k3q_gemm_w8(const void* x, int x_dtype, const int8_t* b, int b_layout, int64_t M, int64_t N,
                int64_t K, const void* b_scale, const void* bias, void* y, void* workspace,
                int64_t workspace_bytes, void* stream);

/*
 * Float matmul against a kernel that exists only de-quantised, stored as bfloat16 [N, parts * K]
 * (K-contiguous rows):  y[m, n] = T(sum_k x[m, k] * w[n, k]) (+ bias[n]).
 *   x bfloat16:  parts = 1, wt = w.
 *   x float32:   parts = 3, wt = [wh | wh | wl] with w = wh + wl (the bfloat16 rounding of a
 *                float32 weight and the rounded remainder); x is split the same way in
 *                `workspace` and the product runs as one bfloat16 GEMM over 3K with float32
 *                accumulation (x and w to about 2^-17 relative).  parts = 2, wt = [w | w], for
 *                weights that are exact in bfloat16.
 * K % 64 == 0 and 16-byte aligned operands run on the MFMA tile kernel (which splits K over
 * workgroups while its tiles are few); anything else on a plain kernel.
 * For EinsumDense int4 kernels whose stored [rows, columns] matrix is a row-major reshape of a
 * kernel with contracted axes that are not leading (e.g. "btd,ndh->btnh"): there a stored
 * column's scale does not belong to one output column, so the reference's own order
 * (de-quantise, reshape, einsum: keras/src/layers/core/einsum_dense.py:1136-1187, :1205-1236)
 * is the only one, with the de-quantised kernel kept by the layer instead of rebuilt per call.
 * workspace: k3q_gemm_wbf16_workspace_bytes(M, N, K, parts) bytes, 16-byte aligned.
 */
int64_t k3q_gemm_wbf16_workspace_bytes(int64_t M, int64_t N, int64_t K, int parts);
int k3q_gemm_wbf16(const void* x, int x_dtype, const uint16_t* wt, int parts, int64_t M, int64_t N,
                   int64_t K, const void* bias, void* y, void* workspace, int64_t workspace_bytes,
                   void* stream);

/*
 * Weight-only int4 matmul, any M (bandwidth-bound kernel tuned for M <= 16; passes of
 * 32 rows (bfloat16) or 8 rows (float32) below prefill sizes; from 65 (float32: 48 to 80) rows on, for
 * K % 128 == 0 and N % 64 == 0, the kernel is de-quantised once per call into `workspace`
 * as bfloat16 [N, K] and the product runs on the MFMA tile kernel (which splits K over
 * workgroups while its tiles are few); float32 x and the float32 de-quantised kernel go
 * there as high + low bfloat16 parts concatenated along K, which keeps float32 accuracy to
 * about 2^-17):
 *     per-channel (block_size <= 0):  y = T(T(x . unpack(w)) / scale[n])   (+ bias)
 *     grouped     (block_size  > 0):  y = T(x . ((unpack(w) - zero[g]) * scale[g]))  (+ bias),  g = k / block_size
 * x: [M, K] of x_dtype, contiguous.  w_packed: the layer's int4 kernel as stored,
 * int8 [K, ceil(N/2)], low nibble = even column.  scale: x_dtype, [N] or
 * [ceil(K/block_size), N].  zero: int8 [ceil(K/block_size), N] (grouped only).
 * bias: x_dtype [N] or null.  y: x_dtype [M, N].  At decode sizes the packed kernel
 * is read once from HBM and is neither unpacked nor de-quantised in memory.
 * Replaces, per call, unpack_int4 + (dequantize_with_sz_map | cast) + matmul +
 * divide of Dense._int4_call (keras/src/layers/core/dense.py:988-1095) and the
 * int4 branch of EinsumDense (keras/src/layers/core/einsum_dense.py:1120-1261).
 *
 * workspace: k3q_gemv_w4_workspace_bytes(M, K, N) bytes, 16-byte aligned, contents
 * irrelevant.  It holds the fp32 partial sums of the K split between the two
 * kernels of a call (decode sizes) or the de-quantised kernel (prefill sizes), so
 * two calls that overlap in time must not share one.  Without it (null / too small)
 * prefill sizes fall back to the passes.
 */
int64_t k3q_gemv_w4_workspace_bytes(int64_t M, int64_t K, int64_t N);
int k3q_gemv_w4(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                const void* w_packed, const void* scale, const void* zero,
                int64_t block_size, const void* bias, void* y, void* workspace,
                int64_t workspace_bytes, void* stream);

/*
 * k3q_gemv_w4 with the K split of decode sizes finished in the same launch instead of by a
 * second kernel (K = N = 8192, one row: one launch less per call).  The workgroups of a column
 * block count their arrivals in `counters` and the one that comes last sums the partials, in
 * the order of the split, so results do not depend on which one that is.
 * counters: k3q_gemv_w4_counters_bytes(N) bytes of device memory, 4-byte aligned, ZERO before
 * the first call; every call leaves them zero again.  Calls ordered on one stream may share
 * them; two calls that overlap in time must not.  Null or too small: as k3q_gemv_w4.
 * No counterpart in the reference (torch's matmul owns its own scratch there).
 */
int64_t k3q_gemv_w4_counters_bytes(int64_t N);
int k3q_gemv_w4_fused(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                      const void* w_packed, const void* scale, const void* zero,
                      int64_t block_size, const void* bias, void* y, void* workspace,
                      int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                      void* stream);

/*
 * k3q_gemv_w4_fused for a layer without bias, with an [M, N] addend (same dtype as x,
 * row-major, may be y itself) that is added to the rounded product the way a bias is:
 *     y[m, n] = T(T(x . W)[m, n] + addend[m, n])
 * which is what `residual + layer(x)` computes in the reference's op sequence
 * (keras/src/layers/core/dense.py:1088-1095 followed by the caller's add), in one launch.
 * Decode sizes only: M <= 64 (K3Q_ERR_SHAPE beyond); runs the decode kernels in passes.
 */
int k3q_gemv_w4_addend(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                       const void* w_packed, const void* scale, const void* zero,
                       int64_t block_size, const void* addend, void* y, void* workspace,
                       int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                       void* stream);

/*
 * k3q_gemv_w4_fused at decode sizes (M <= 16; K3Q_ERR_SHAPE beyond) for callers that cannot
 * allocate device memory or hand a workspace in: code under HIP graph capture, serving loops
 * and harnesses that forbid hipMalloc.  It calls no allocating routine.  The partial sums of
 * the K split and the arrival counters live in a device array inside the library (16 MiB +
 * 64 KiB per GPU the library runs on, held until the process ends) instead of `workspace` /
 * `counters`; the same kernels, the same partials, the same summation order, the same bits.
 * A shape whose K split needs more than k3q_gemv_w4_static_max_bytes() of partials
 * (K split x min(M, 16) x N floats) is rejected with K3Q_ERR_WORKSPACE and nothing is launched.
 * Every call on a GPU shares that GPU's array: calls ordered on one stream are fine, calls
 * that overlap in time on one GPU (two streams, two host threads) race on it.  The current
 * device must be the device of `stream`.  The first call on a device may itself be under stream
 * capture (it adds only the matmul's own nodes to the graph).
 * No counterpart in the reference (torch's matmul owns its own scratch there).
 */
int64_t k3q_gemv_w4_static_max_bytes(void);
int k3q_gemv_w4_static(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                       const void* w_packed, const void* scale, const void* zero,
                       int64_t block_size, const void* bias, void* y, void* stream);

/*
 * Weight-only int4 matmul for up to 16 bfloat16 rows from a strip-linear copy of the kernel: what
 * k3q_gemv_w4 computes (to the order of the fp32 sums), with the kernel streamed as contiguous
 * 1 KiB pieces, all of K inside a workgroup -- no partial sums, no workspace, no counters, and
 * nothing allocated: one launch that reads the copy once.
 *   shadow:  k3q_w4s_shadow_bytes(K, N) bytes made by k3q_w4s_pack from the stored kernel
 *            ([K, ceil(N/2)], low nibble = even column), once per layer.  Layout:
 *            [strip = n / 16][unit = k / 128][lane = 64][dword = 4]; lane i + 16 g holds column
 *            16 strip + i, its dword s the nibbles of k = 128 unit + 32 s + 8 g + e: e = 2t at bits
 *            [4t, 4t + 4), e = 2t + 1 at bits [16 + 4t, 16 + 4t + 4) (two's-complement low four bits);
 *            the strip count is rounded up to an even number with zero strips.
 *   per-channel (block_size <= 0): scale = bfloat16 [N];          y = T(T(x . W) / scale[n]) (+ bias)
 *   grouped (block_size == 128):   gparams = k3q_w4s_params_bytes bytes made by k3q_w4s_pack_params
 *            from scale, zero [K / 128, N]: per (strip, unit) four records {4 bfloat16 scales,
 *            4 bytes zero + 128};                                  y = T(x . ((W - zero) * scale)) (+ bias)
 *   bias: bfloat16 [N] (bias_stride 0) or an [M, N] addend (bias_stride N), or null.
 * Takes (k3q_gemv_w4s_supported): bfloat16 x, 1 <= M <= 16 while the rows fit a workgroup's LDS
 * (M * K <= 65536 values and M * (2 K + 16) bytes + the cross-wave sums within 160 KiB; beyond that x is
 * staged in two parts of every wave's slice, the first the larger, when K % 2048 == 0, K >= 4096, that
 * part fits the same limits and every workgroup has one strip group: N <= 8192),
 * K % 256 == 0, K >= 4096, N % 16 == 0, N >= 3072, block_size <= 0 or == 128; anything else
 * K3Q_ERR_SHAPE (callers keep k3q_gemv_w4 for those).  k3q_gemv_w4s_multi: several kernels against one x (same M, K,
 * block_size), one launch for those whose launch plans agree.
 * Replaces what k3q_gemv_w4 replaces (keras/src/layers/core/dense.py:988-1095,
 * keras/src/layers/core/einsum_dense.py:1120-1261).
 */
typedef struct {
    int64_t N;
    const void* shadow;
    const void* scale;
    const void* gparams;
    const void* bias;
    void* y;
} k3q_gemv_w4s_problem;
int64_t k3q_w4s_shadow_bytes(int64_t K, int64_t N);
int64_t k3q_w4s_params_bytes(int64_t K, int64_t N, int64_t block_size);
int k3q_w4s_pack(const int8_t* w_packed, int64_t K, int64_t N, void* shadow, void* stream);
int k3q_w4s_pack_params(const void* scale, int scale_dtype, const int8_t* zero, int64_t K, int64_t N,
                        int64_t block_size, void* params, void* stream);
int k3q_gemv_w4s_supported(int64_t M, int64_t K, int64_t N, int64_t block_size);
int k3q_gemv_w4s(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N, const void* shadow,
                 const void* scale, const void* gparams, int64_t block_size, const void* bias,
                 int64_t bias_stride, void* y, void* stream);
int k3q_gemv_w4s_multi(const void* x, int x_dtype, int64_t M, int64_t K, int count,
                       const k3q_gemv_w4s_problem* problems, int64_t block_size, void* stream);

/*
 * The decode matmuls with an operation on their input folded in: the rows of x are transformed on
 * their way into the workgroup's LDS, which saves the launch and the round trip through memory of a
 * separate elementwise kernel between two layers of a decoder block.
 *   K3Q_INPUT_RMS_NORM:  x' = T(x * rsqrt(mean(x^2) + epsilon) * operand), operand = the gain,
 *                        bfloat16 [K]; the bits k3q_rmsnorm writes.  K % 512 == 0, K <= 65536.
 *   K3Q_INPUT_SILU_GATE: x' = T(T(silu(operand)) * x), operand = the gate, bfloat16 [M, K], dense;
 *                        the bits k3q_silu_mul(gate = operand, up = x) writes.
 * Every workgroup repeats the transform on all of x: worth it for the few rows of a decode step.
 * k3q_gemv_w4s_pre: as k3q_gemv_w4s_multi (count >= 1 kernels against one x); bias_rows != 0: every
 * problem's bias is an [M, N] addend (a row per row of x) instead of [N].  x whole in LDS only (no
 * staging in halves): K3Q_ERR_SHAPE otherwise.
 * k3q_dense_i8_w8s_pre: as k3q_dense_i8_w8s_multi with x given in bfloat16 (the rows are transformed,
 * then quantised, inside the kernel); same bias_rows.
 * No counterpart in the reference, whose layers each run their own ops
 * (keras/src/layers/core/dense.py:961-986, 988-1095 see the normalised / gated tensor as input).
 */
#define K3Q_INPUT_NONE 0
#define K3Q_INPUT_RMS_NORM 1
#define K3Q_INPUT_SILU_GATE 2
typedef struct {
    int kind;
    float epsilon;
    const void* operand;
} k3q_input_op;
int k3q_gemv_w4s_pre(const void* x, int x_dtype, int64_t M, int64_t K, const k3q_input_op* pre, int count,
                     const k3q_gemv_w4s_problem* problems, int64_t block_size, int bias_rows, void* stream);

/*
 * Weight-only int4 matmul for 17 ... 512 bfloat16 rows from a K-contiguous copy of the kernel:
 * the same result as k3q_gemv_w4 to the order of the fp32 sums, with the kernel read once as
 * int4 (k3q_gemv_w4's route for these sizes writes it out as bfloat16 first: nine times the
 * bytes at 128 rows).
 * w_kmajor: int4 [N, K/2]; dword j of row n holds k = 8j ... 8j+7 of column n, the nibble of
 * k = 8j + 2p at bits [4p, 4p+4) and of k = 8j + 2p + 1 at bits [16+4p, 16+4p+4), each the low
 * four bits of the two's-complement value (k3q_w4_kmajor_pack builds it from the stored
 * [K, ceil(N/2)] kernel, once per layer; K % 8 == 0).  scale, zero, block_size, bias, y as for k3q_gemv_w4.
 * Needs K % 128 == 0, N % 32 == 0, K % block_size == 0 and block_size % 64 == 0 (K3Q_ERR_SHAPE
 * otherwise); workspace: k3q_gemm_w4_kmajor_workspace_bytes bytes, 16-byte aligned.
 * Replaces what k3q_gemv_w4 replaces (keras/src/layers/core/dense.py:988-1095).
 */
int k3q_w4_kmajor_pack(const int8_t* w_packed, int64_t K, int64_t N, int32_t* w_kmajor, void* stream);
int64_t k3q_gemm_w4_kmajor_workspace_bytes(int64_t M, int64_t K, int64_t N, int64_t block_size);
int k3q_gemm_w4_kmajor(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                       const void* w_kmajor, const void* scale, const void* zero, int64_t block_size,
                       const void* bias, void* y, void* workspace, int64_t workspace_bytes,
                       void* stream);

/*
 * k3q_gemm_w4_kmajor from the strip-linear copy that the decode kernels stream (k3q_w4s_pack)
 * instead of a K-contiguous copy of its own: same tiles, same sums in another order of k inside
 * each unit of 128 (results within the float tolerance of k3q_gemm_w4_kmajor, not its bits), so a
 * layer keeps ONE derived copy of its kernel for 1 ... 512 rows.  Same arguments and workspace
 * (k3q_gemm_w4_kmajor_workspace_bytes); block_size <= 0 or a multiple of 128, else K3Q_ERR_SHAPE.
 */
int k3q_gemm_w4_strip(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                      const void* w_strip, const void* scale, const void* zero,
                      int64_t block_size, const void* bias, void* y, void* workspace,
                      int64_t workspace_bytes, void* stream);

/*
 * Several weight-only int4 matmuls against ONE x, each as k3q_gemv_w4_fused computes it (same
 * bits), in one launch when they are decode-sized (M <= 16) and their launch plans agree
 * (e.g. kernels of one shape: the query / key / value projections of an attention block, the
 * gate / up projections of a gated MLP); otherwise one after the other.  A launch costs
 * several microseconds whatever it does, which is most of a decode-sized matmul.
 * problems[i]: the operands of k3q_gemv_w4 that differ per kernel (N, w_packed [K, ceil(N/2)],
 * scale, zero, bias, y [M, N]); block_size is common.  workspace: the sum over i of
 * k3q_gemv_w4_workspace_bytes(M, K, N_i), each rounded up to a multiple of 256; counters: the
 * sum of k3q_gemv_w4_counters_bytes(N_i), zero between calls as for k3q_gemv_w4_fused.
 * No counterpart in the reference, whose layers each call matmul on their own.
 */
typedef struct {
    int64_t N;
    const void* w_packed;
    const void* scale;
    const void* zero;
    const void* bias;
    void* y;
} k3q_gemv_w4_problem;
int k3q_gemv_w4_multi(const void* x, int x_dtype, int64_t M, int64_t K, int count,
                      const k3q_gemv_w4_problem* problems, int64_t block_size, void* workspace,
                      int64_t workspace_bytes, void* counters, int64_t counters_bytes,
                      void* stream);

/*
 * Weight-only int4 matmul for decode-sized M with the kernel stored K-contiguous:
 *     y[m,n] = sum_k x[m,k] * W[n,k],  w_packed int8 [N, ceil(K/2)], low nibble = even k
 *   block_size <= 0: scale [N];                         y = T(T(acc) / scale[n])
 *   block_size  > 0: scale, zero [N, ceil(K/block)];     y = T(x . ((W - zero) * scale))
 * This is a tied int4 embedding table [vocab, ceil(dim/2)] used as the LM head: the reverse
 * branch of ReversibleEmbedding._int4_call without an activation quantizer
 * (keras/src/layers/core/reversible_embedding.py:298-381: transpose, unpack_int4 along
 * axis 0, dequantize_with_sz_map | divide, matmul).  x: [M, K] float32 or bfloat16;
 * y: [M, N], bfloat16 when x and scale are both bfloat16, float32 otherwise (the
 * reference's promotion).  Any M (tuned for M <= 8); the fast kernel needs K % 128 == 0
 * and, grouped, block_size % 128 == 0; other shapes run a plain kernel.
 */
int k3q_gemv_w4_nk(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N,
                   const int8_t* w_packed, const void* scale, int scale_dtype,
                   const int8_t* zero, int64_t block_size, void* y, void* stream);

/*
 * Quantized embedding lookup: out[t, :] = dequantise(table[ids[t], :]), t < count.
 * Replaces the take + cast + divide chain of Embedding._int8_call
 * (keras/src/layers/core/embedding.py:521-541) and the unpack_int4 + take +
 * (divide | dequantize_with_sz_map) chain of Embedding._int4_call (:543-582,
 * keras/src/quantizers/quantizers.py:1631-1668).
 *   bits = 8: table [vocab, dim] int8, scale [vocab];      out = T(q) / scale[row]
 *   bits = 4: table [vocab, ceil(dim/2)] int8, low nibble = even column;
 *     block_size <= 0: scale [vocab];                        out = T(q) / scale[row]
 *     block_size  > 0: scale, zero [vocab, ceil(dim/block)]; out = (T(q) - zero) * scale
 * ids: int32 or int64 (ids_dtype); negative ids wrap once by `vocab`
 * (keras/src/backend/torch/numpy.py:2005-2017).  An id still outside [0, vocab)
 * gives a row of zeros and sets *oob_flag (may be null) to 1 -- the reference
 * raises there; the host mirror turns the flag into the same IndexError.
 * out_dtype follows the reference's promotion: bfloat16 only with bfloat16
 * scales, else float32 (K3Q_ERR_DTYPE otherwise).
 */
int k3q_embedding_lookup(const void* ids, int ids_dtype, int64_t count, const int8_t* table,
                         int64_t vocab, int64_t dim, int bits, const void* scale,
                         int scale_dtype, const int8_t* zero, int64_t block_size, int out_dtype,
                         void* out, int* oob_flag, void* stream);

/*
 * Decode-sized int8 Dense forward in ONE launch, from a strip-linear copy of the int8 kernel:
 * the rows of x (1 ... 16, bfloat16) are abs-max quantised inside the kernel exactly as
 * k3q_absmax_quantize does (same roundings, same int8 values and scales), multiplied exactly
 * (int32 sums of all of K inside a workgroup: no partial sums in memory, no workspace) and
 * de-scaled with the bit-exact bfloat16 epilogue of k3q_gemm_i8 (flags bit 0):
 *     y = bf16(bf16(acc) / bf16(sa * sb)) (+ bias, one more rounding).
 * Same bits as k3q_absmax_quantize followed by k3q_gemm_i8 with K3Q_GEMM_EXACT_EPILOGUE.
 * Replaces the chain keras/src/layers/core/dense.py:956-972 (inputs_quantizer, ops.matmul,
 * cast, divide by the scales, bias add) and einsum_dense.py:1063-1083 for GEMM-shaped
 * equations, for calls of up to 16 rows.
 *
 * shadow (k3q_w8s_pack from the stored [K, N] int8 kernel, once per layer):
 * [strip = n/16][unit = k/64][lane = 64][16 bytes]; lane i + 16 g holds column 16 strip + i,
 * bytes k = 64 unit + 16 g + (0 ... 15); the strip count is padded to even with zero strips;
 * k3q_w8s_shadow_bytes gives its size.  kernel_scale: bfloat16 [N].  bias: bfloat16, N values
 * (bias_stride 0) or M x N (bias_stride N: a row per row of x), or null.
 * epsilon, range_lo, range_hi: the quantizer's settings (1e-7, -127, 127 by default); the range
 * inside [-128, 127] (K3Q_ERR_SHAPE) with integer ends (K3Q_ERR_RANGE: the kernel clips before it
 * rounds, which equals the reference's round-then-clip only between integers; other ranges go
 * through k3q_absmax_quantize + k3q_gemm_i8_w8s).
 * Needs K % 512 == 0, K >= 1024, N % 16 == 0, N >= 3072 and M x K small enough for LDS
 * (k3q_dense_i8_w8s_supported says; K3Q_ERR_SHAPE otherwise).
 *
 * k3q_gemm_i8_w8s is the same kernel for rows that are already quantised (a: int8 [M, K],
 * a_scale: bfloat16 [M], as k3q_absmax_quantize writes them): every workgroup re-quantising
 * all of x costs more than a quantizer launch from about 16 K values of x on, and layers that
 * share their input quantise it once.  Same shapes, same bits.
 */
int64_t k3q_w8s_shadow_bytes(int64_t K, int64_t N);
int k3q_w8s_pack(const int8_t* w, int64_t K, int64_t N, void* shadow, void* stream);
int k3q_dense_i8_w8s_supported(int64_t M, int64_t K, int64_t N);
int k3q_dense_i8_w8s(const void* x, int x_dtype, int64_t M, int64_t K, int64_t N, const void* shadow,
                     const void* kernel_scale, const void* bias, int64_t bias_stride, float epsilon,
                     float range_lo, float range_hi, void* y, void* stream);
int k3q_gemm_i8_w8s(const int8_t* a, const void* a_scale, int scale_dtype, int64_t M, int64_t K, int64_t N,
                    const void* shadow, const void* kernel_scale, const void* bias, int64_t bias_stride,
                    void* y, void* stream);
/*
 * Several int8 layers against ONE x in one launch (the query / key / value projections of an
 * attention block, gate / up of an MLP): each result is what k3q_dense_i8_w8s (a == NULL: the rows
 * are quantised in the kernel) or k3q_gemm_i8_w8s (a, a_scale: rows already quantised) gives for
 * that problem alone, bit for bit; problems whose launch plans differ run in launches of their own.
 * bias: N values or NULL.  No counterpart in the reference (its layers each run their own matmul).
 */
typedef struct {
    int64_t N;
    const void* shadow;       /* k3q_w8s_pack of the layer's [K, N] kernel */
    const void* kernel_scale; /* bfloat16 [N] */
    const void* bias;         /* bfloat16 [N] or NULL */
    void* y;                  /* bfloat16 [M, N] */
} k3q_w8s_problem;
int k3q_dense_i8_w8s_multi(const void* x, int x_dtype, const int8_t* a, const void* a_scale, int64_t M, int64_t K,
                           int count, const k3q_w8s_problem* problems, float epsilon, float range_lo,
                           float range_hi, void* stream);
/* with an operation on x before it is quantised: see k3q_gemv_w4s_pre */
int k3q_dense_i8_w8s_pre(const void* x, int x_dtype, int64_t M, int64_t K, const k3q_input_op* pre, int count,
                         const k3q_w8s_problem* problems, float epsilon, float range_lo, float range_hi,
                         int bias_rows, void* stream);

/*
 * The operation and the activation quantizer of the int8 layers behind it in one launch, for any
 * number of bfloat16 rows (dim % 8 == 0, dim <= 16384, x / operand / h dense): h = op(x) with the
 * bits of k3q_rmsnorm / k3q_silu_mul, and q, scale = abs-max quantisation of h over the last axis
 * with the bits of k3q_absmax_quantize (scale bfloat16 [rows]).  Used where the decode kernels do
 * not fold the operation in themselves (more than a few rows): one launch instead of two, and h
 * is not read back.  No counterpart in the reference.
 */
int k3q_input_op_quantize(const void* x, int dtype, int64_t rows, int64_t dim, const k3q_input_op* pre,
                          float epsilon, float range_lo, float range_hi, void* h, int8_t* q, void* scale,
                          void* stream);

/*
 * One new position of causal self-attention against a key / value cache (the decoder
 * harness's step between the quantized projections): rotate-half RoPE of the new query and
 * key with the table rows of *pos, the new key and value rows written into the caches at
 * *pos, softmax(q . K^T / sqrt(128)) . V over cache rows 0 ... *pos.  bfloat16, head width 128.
 * q, k, v, out: [B, H, 128]; cos_table, sin_table: [max_len, 128] (sin with the sign of the
 * rotated half folded in); k_cache, v_cache: [B, H, max_len, 128]; pos: one int64 in device
 * memory, read by the kernel (a captured graph replays with the value it then holds).
 * A position outside [0, max_len) writes nothing to the caches, gives zero output rows and sets
 * *oob_flag (one int32 in device memory, may be null; the kernel never clears it) to 1: the torch
 * ops this stands for raise there, and the caller checks the flag when it next synchronises.
 * No counterpart in the reference's quantized layers: it stands for the torch ops (two
 * multiplies and an add per rotation, two index_copy, scaled_dot_product_attention) that a
 * Keras decoder runs between its Dense / EinsumDense calls.
 */
int k3q_decode_attention(const void* q, const void* k, const void* v, int dtype, int64_t B, int64_t H,
                         int64_t head_dim, int64_t max_len, const void* cos_table, const void* sin_table,
                         const int64_t* pos, void* k_cache, void* v_cache, void* out, int* oob_flag,
                         void* stream);

/*
 * Two more pieces of the decoder harness's glue (no counterpart in the quantized layers; they
 * stand for `rms_norm` and `silu(gate) * up` between the Dense calls of a decoder block), bfloat16:
 * k3q_rmsnorm: y[r, :] = bf16(x[r, :] * rsqrt(mean(x[r, :]^2) + epsilon) * weight[:]), float32
 * arithmetic and one rounding; dim % 8 == 0, dim <= 16384; row strides in elements (% 8 == 0).
 * k3q_silu_mul: y = bf16(bf16(g / (1 + exp(-g))) * u) element by element, rows given by strides.
 */
int k3q_rmsnorm(const void* x, const void* weight, int dtype, int64_t rows, int64_t dim, int64_t x_row_stride,
                float epsilon, void* y, int64_t y_row_stride, void* stream);
int k3q_silu_mul(const void* gate, const void* up, int dtype, int64_t rows, int64_t dim, int64_t gate_row_stride,
                 int64_t up_row_stride, void* y, int64_t y_row_stride, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* K3Q_H_ */
