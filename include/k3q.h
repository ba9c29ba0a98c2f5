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
 *   - dtype codes: K3Q_F32 = 0, K3Q_BF16 = 1.
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

#ifdef __cplusplus
}
#endif
#endif /* K3Q_H_ */
