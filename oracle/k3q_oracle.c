/*
 * Plain-C restatement of the integer / rounding-critical parts of the Keras 3
 * quantized Dense path.  TEST INFRASTRUCTURE ONLY: loaded by tests/, by
 * __graft_entry__.smoke() and by the cpu_baseline leg of bench.py; never by
 * the keras_amd package.
 *
 * It is a second, independent statement of the same algorithms that
 * oracle/keras_cpu_path.py states with torch primitives: the two are checked
 * against each other and against the reference's known-answer vectors, so a
 * mistake in either one shows up as a disagreement.
 *
 * Reference (keras-team/keras 3.16.0):
 *   abs_max_quantize          keras/src/quantizers/quantizers.py:111-120
 *   pack_int4 / unpack_int4   keras/src/quantizers/quantizers.py:700-750, 830-900
 *   int8 matmul on CPU        keras/src/backend/torch/numpy.py:139-157
 *   Dense._int8_call          keras/src/layers/core/dense.py:961-986
 *   Dense._int4_call          keras/src/layers/core/dense.py:1003-1084
 *
 * Build: see oracle/Makefile  (gcc -O3 -fopenmp -shared -fPIC).
 */
#include <math.h>
#include <stdint.h>
#include <string.h>

/* ---- bfloat16 helpers: round-to-nearest-even on the upper 16 bits ---- */
static inline float bf16_to_f32(uint16_t h) {
    uint32_t u = (uint32_t)h << 16;
    float f;
    memcpy(&f, &u, 4);
    return f;
}
static inline uint16_t f32_to_bf16(float f) {
    uint32_t u;
    memcpy(&u, &f, 4);
    if ((u & 0x7fffffffu) > 0x7f800000u) return (uint16_t)((u >> 16) | 0x40); /* NaN */
    u += 0x7fffu + ((u >> 16) & 1u);
    return (uint16_t)(u >> 16);
}
static inline float round_bf16(float f) { return bf16_to_f32(f32_to_bf16(f)); }

/* round half to even, as torch.round / np.round */
static inline float rne(float v) { return nearbyintf(v); }

/*
 * abs_max_quantize, tensor path, reduction over the last axis of [rows, cols].
 * x_dtype 0: float32 buffers, 1: bfloat16 buffers (uint16 payload).
 * Every arithmetic step is rounded to the tensor dtype, epsilon included
 * (torch casts the 0-dim float32 epsilon tensor to the common dtype first).
 */
void k3q_oracle_absmax_quantize(const void* x, int x_dtype, int64_t rows, int64_t cols,
                                float eps, float qlo, float qhi, int8_t* q, void* scale) {
#pragma omp parallel for schedule(static)
    for (int64_t r = 0; r < rows; ++r) {
        float amax = 0.0f;
        for (int64_t c = 0; c < cols; ++c) {
            float v = x_dtype ? bf16_to_f32(((const uint16_t*)x)[r * cols + c])
                              : ((const float*)x)[r * cols + c];
            float a = fabsf(v);
            if (a > amax || a != a) amax = a;
        }
        float s;
        if (x_dtype) {
            float t = round_bf16(amax + round_bf16(eps));
            s = round_bf16(qhi / t);
            ((uint16_t*)scale)[r] = f32_to_bf16(s);
        } else {
            float t = amax + eps;
            s = qhi / t;
            ((float*)scale)[r] = s;
        }
        for (int64_t c = 0; c < cols; ++c) {
            float v = x_dtype ? bf16_to_f32(((const uint16_t*)x)[r * cols + c])
                              : ((const float*)x)[r * cols + c];
            float p = v * s;
            if (x_dtype) p = round_bf16(p);
            p = rne(p);
            if (p < qlo) p = qlo;
            if (p > qhi) p = qhi;
            q[r * cols + c] = (int8_t)p;
        }
    }
}

/* pack along the middle axis of [outer, len, inner]; out is [outer, ceil(len/2), inner] */
void k3q_oracle_pack_int4(const uint8_t* in, int64_t outer, int64_t len, int64_t inner,
                          uint8_t* out) {
    int64_t plen = (len + 1) / 2;
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t j = 0; j < plen; ++j)
            for (int64_t i = 0; i < inner; ++i) {
                uint8_t lo = in[(o * len + 2 * j) * inner + i];
                uint8_t hi = (2 * j + 1 < len) ? in[(o * len + 2 * j + 1) * inner + i] : 0;
                out[(o * plen + j) * inner + i] = (uint8_t)((lo & 0x0F) | ((hi & 0x0F) << 4));
            }
}

/* unpack along the middle axis of [outer, plen, inner] to [outer, orig_len, inner] */
void k3q_oracle_unpack_int4(const uint8_t* in, int64_t outer, int64_t plen, int64_t inner,
                            int64_t orig_len, int is_signed, uint8_t* out) {
    for (int64_t o = 0; o < outer; ++o)
        for (int64_t l = 0; l < orig_len; ++l)
            for (int64_t i = 0; i < inner; ++i) {
                uint8_t b = in[(o * plen + l / 2) * inner + i];
                uint8_t v = (l & 1) ? ((b >> 4) & 0x0F) : (b & 0x0F);
                if (is_signed) v = (uint8_t)((v ^ 8) - 8);
                out[(o * orig_len + l) * inner + i] = v;
            }
}

/* int8 [M,K] x int8 [K,N] -> int32 [M,N], exact */
__attribute__((target_clones("avx512f", "avx2", "default")))
void k3q_oracle_gemm_i8(const int8_t* a, const int8_t* b, int64_t M, int64_t N, int64_t K,
                        int32_t* c) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m) {
        int32_t* crow = c + m * N;
        for (int64_t n = 0; n < N; ++n) crow[n] = 0;
        for (int64_t k = 0; k < K; ++k) {
            int32_t av = a[m * K + k];
            if (av == 0) continue;
            const int8_t* brow = b + k * N;
            for (int64_t n = 0; n < N; ++n) crow[n] += av * (int32_t)brow[n];
        }
    }
}

/*
 * De-scale epilogue of Dense._int8_call:  y = T(T(acc) / T(ks[n]*s_in[m])) (+ T bias).
 * dtype 0 float32, 1 bfloat16 (scales, bias and y are uint16 payloads then).
 */
void k3q_oracle_descale(const int32_t* acc, int64_t M, int64_t N, int dtype,
                        const void* s_in, const void* ks, const void* bias, void* y) {
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            if (dtype) {
                float si = bf16_to_f32(((const uint16_t*)s_in)[m]);
                float kn = bf16_to_f32(((const uint16_t*)ks)[n]);
                float os = round_bf16(kn * si);
                float v = round_bf16((float)acc[m * N + n]);
                v = round_bf16(v / os);
                if (bias) v = round_bf16(v + bf16_to_f32(((const uint16_t*)bias)[n]));
                ((uint16_t*)y)[m * N + n] = f32_to_bf16(v);
            } else {
                float os = ((const float*)ks)[n] * ((const float*)s_in)[m];
                float v = (float)acc[m * N + n];
                v = v / os;
                if (bias) v = v + ((const float*)bias)[n];
                ((float*)y)[m * N + n] = v;
            }
        }
}

/*
 * int4 weight-only Dense, evaluated in double precision: the value the float
 * paths approximate.  Used only for tolerance checks (never bit-exact).
 *   per-channel (block_size <= 0): y = (sum_k x[m,k] * q[k,n]) / scale[n]
 *   grouped:                       y = sum_k x[m,k] * (q[k,n] - zero[g,n]) * scale[g,n]
 * w_packed is [K, ceil(N/2)], low nibble = even column.
 */
void k3q_oracle_w4_matmul_f64(const float* x, int64_t M, int64_t K, int64_t N,
                              const uint8_t* w_packed, const float* scale, const int8_t* zero,
                              int64_t block_size, const float* bias, double* y) {
    int64_t pn = (N + 1) / 2;
#pragma omp parallel for schedule(static)
    for (int64_t m = 0; m < M; ++m)
        for (int64_t n = 0; n < N; ++n) {
            double acc = 0.0;
            for (int64_t k = 0; k < K; ++k) {
                uint8_t b = w_packed[k * pn + n / 2];
                int v = (n & 1) ? ((b >> 4) & 0x0F) : (b & 0x0F);
                v = (v ^ 8) - 8;
                if (block_size > 0) {
                    int64_t g = k / block_size;
                    acc += (double)x[m * K + k] * (double)(v - zero[g * N + n]) *
                           (double)scale[g * N + n];
                } else {
                    acc += (double)x[m * K + k] * (double)v;
                }
            }
            if (block_size <= 0) acc /= (double)scale[n];
            if (bias) acc += (double)bias[n];
            y[m * N + n] = acc;
        }
}
