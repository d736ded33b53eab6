/*
 * TEST INFRASTRUCTURE ONLY -- see oracle.h. CPU restatement of Bolt's x86 AVX-512-VNNI
 * quantized matrix-product path. Never linked into or called from the product.
 *
 * Pinning status (tests/test_oracle_vs_ref.py, tests/test_golden.py):
 *   size queries, offsetC, GEMM, GEMV (both signedness variants), quantize F32->U8_Q / I8,
 *   I32->U8_Q / I8, U8_Q->I8, bias fold, dequantize, requantize, int8 convolution:
 *     pinned bit-for-bit against the reference's own compiled sources (oracle/_ref) on seeded
 *     and hand-built tie / saturation inputs, and against the golden vectors committed from
 *     those runs.
 *   per-output-channel epilogue: not in the reference; pinned by reduction to the per-tensor
 *     reference result when all channel scales are equal.
 *   BNN convolution: the reference path is ARMv8.2-fp16 only and cannot be built here; the
 *     integer sums are pinned by a brute-force +-1 / {0,1} convolution (orc_bnn_conv_bruteforce)
 *     and the popcount identity.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

#define ALIGN_UP(x, a) (((x) + (a)-1) / (a) * (a))

/* vcvtps2dq: round to nearest even; NaN / out of range -> 0x80000000 ("integer indefinite") */
static inline int32_t rne_i32(float v)
{
    if (!(v >= -2147483648.0f && v < 2147483648.0f)) {
        return INT32_MIN;
    }
    return (int32_t)lrintf(v); /* default rounding mode = FE_TONEAREST */
}

/* vpmovusdb: saturate the dword read as an UNSIGNED number -> negatives become 255 */
static inline uint8_t usat8_u(int32_t v)
{
    return ((uint32_t)v > 255u) ? 255 : (uint8_t)v;
}

/* vpmovsdb: signed saturation to [-128, 127] */
static inline int8_t ssat8(int32_t v)
{
    return (int8_t)(v < -128 ? -128 : (v > 127 ? 127 : v));
}

static inline int32_t wrap_add(int32_t a, int32_t b)
{
    return (int32_t)((uint32_t)a + (uint32_t)b);
}

/* ------------------------------------------------------------------------------------
 * Size queries
 * ---------------------------------------------------------------------------------- */

/* compute/blas_enhance/src/cpu/x86/int8/avx512/mmm_avx512_vnni.cpp:22-40 */
void orc_mmm_transform_rhs_bytes(uint32_t N, uint32_t K, int packed, uint32_t *bytes, uint32_t *rhsBytes)
{
    uint32_t matrix = 0, pad = 0;
    if (!packed) {
        pad += N * 4;
        matrix = ALIGN_UP(N, 16) * ALIGN_UP(K, 8);
        pad += matrix + 64;
    }
    if (rhsBytes) {
        *rhsBytes = matrix;
    }
    if (bytes) {
        *bytes = pad;
    }
}

/* mmm_avx512_vnni.cpp:42-58 */
uint32_t orc_mmm_tmp_bytes(uint32_t N, uint32_t M, uint32_t K, int transA, int packedB)
{
    uint32_t bytes = 0;
    orc_mmm_transform_rhs_bytes(N, K, packedB, &bytes, 0);
    if (!transA) {
        bytes += 32 * K;
        if (K % 8 != 0) {
            bytes += ALIGN_UP(M, 24) * 8;
        }
    } else {
        uint32_t kb = ALIGN_UP(K, 8);
        bytes += ALIGN_UP(M, 24) * (kb < 4096 ? kb : 4096);
    }
    bytes += N * 4;
    bytes += 64;
    return bytes;
}

/* compute/blas_enhance/src/cpu/x86/mvm.cpp:23-42 (also used as the mvm tmp-bytes, :77-100) */
uint32_t orc_mvm_transform_weight_bytes(uint32_t N, uint32_t K, int wdt, int packed)
{
    uint32_t bytes = 0;
    if (wdt == ORC_I8) {
        bytes += N * 4;
    }
    if (wdt == ORC_U8Q) {
        if (K % 32 != 0) {
            bytes += 32 * (N + 1);
        }
    }
    if (!packed) {
        bytes += ALIGN_UP(N, 16) * ALIGN_UP(K, 8); /* 1 byte per element for both dtypes */
        bytes += 32;
    }
    return bytes;
}

/* ------------------------------------------------------------------------------------
 * Compensation vector: mmm_avx512_vnni.cpp:81-87,112-118; mvm_avx512_vnni.cpp:73-79,121-127
 * ---------------------------------------------------------------------------------- */
void orc_offsetC(const int8_t *W, uint32_t K, uint32_t N, int w_is_NK, int32_t *out)
{
    for (uint32_t n = 0; n < N; ++n) {
        int32_t s = 0;
        for (uint32_t k = 0; k < K; ++k) {
            s += (int32_t)(w_is_NK ? W[(size_t)n * K + k] : W[(size_t)k * N + n]);
        }
        out[n] = s * (-128);
    }
}

/* ------------------------------------------------------------------------------------
 * GEMM/GEMV epilogue: mmm_avx512_vnni.cpp:1796-1808 + blas_common_int8.h:922-925,1195-1200
 *   scale == NULL      : raw int32
 *   scale[0] > 0       : f32 = cvt(acc) * (1.0f / scale[0])
 *   scale[0] < 0       : u8  = usat8_u(rne(cvt(acc) * scale[1]) + 128)   (integer +128)
 * ---------------------------------------------------------------------------------- */
static inline float epi_factor(const float *scale)
{
    return (scale[0] < 0) ? scale[1] : 1.0f / scale[0];
}

static inline void epi_store(int32_t acc, void *C, size_t idx, int cdt, const float *scale, float factor)
{
    if (scale == 0 || cdt == ORC_I32) {
        ((int32_t *)C)[idx] = acc;
    } else if (scale[0] < 0) {
        float f = (float)acc * factor;
        ((uint8_t *)C)[idx] = usat8_u(wrap_add(rne_i32(f), 128));
    } else {
        ((float *)C)[idx] = (float)acc * factor;
    }
}

/*
 * compute/blas_enhance/src/mmm.cpp:150-238 -> cpu/x86/mmm.cpp:154-186 ->
 * mmm_avx512_vnni.cpp:1760-1891 with the kernel template :1379-1483.
 *   acc = offsetC[n] + C_in[m][n] + sum_k A_u8[m][k] * W_s8[k][n]     (int32, wraps)
 * C_in: the int32 bits already in C for i32 / f32 output (the f32 buffer doubles as the int32
 * parking area between K blocks, :1796-1808); for u8 output the accumulator lives in a zeroed
 * tmp area (:1800-1803) so C_in is 0. DT_I32 output forces scale = NULL (mmm.cpp:222-224).
 */
void orc_mmm_int8(uint32_t M, uint32_t N, uint32_t K, const uint8_t *A, int transA, const int8_t *W,
    int w_is_NK, const int32_t *offsetC, void *C, int cdt, const float *scale)
{
    if (cdt == ORC_I32) {
        scale = 0;
    }
    float factor = scale ? epi_factor(scale) : 0.0f;
#pragma omp parallel for schedule(static)
    for (uint32_t m = 0; m < M; ++m) {
        for (uint32_t n = 0; n < N; ++n) {
            int32_t acc = offsetC[n];
            if (!(scale && scale[0] < 0)) {
                acc = wrap_add(acc, ((int32_t *)C)[(size_t)m * N + n]);
            }
            uint32_t s = 0;
            for (uint32_t k = 0; k < K; ++k) {
                int32_t a = transA ? A[(size_t)k * M + m] : A[(size_t)m * K + k];
                int32_t w = w_is_NK ? W[(size_t)n * K + k] : W[(size_t)k * N + n];
                s += (uint32_t)(a * w);
            }
            acc = wrap_add(acc, (int32_t)s);
            epi_store(acc, C, (size_t)m * N + n, cdt, scale, factor);
        }
    }
}

/* matrix_vector_multiply never looks at the result dtype: the scale pointer alone selects the
 * store (mvm_avx512_vnni.cpp:724-735), unlike matrix_matrix_multiply (mmm.cpp:222-224). */
static inline int mvm_out_type(const float *scale)
{
    return scale ? (scale[0] < 0 ? ORC_U8Q : ORC_F32) : ORC_I32;
}

/*
 * compute/blas_enhance/src/mvm.cpp:132-194 -> cpu/x86/mvm.cpp:102-138 ->
 * mvm_avx512_vnni.cpp:703-759 (kernels :133-666, tail kernel :668-701).
 *   y[n] = offsetC[n] + y_in[n] + sum_k W_s8[n][k] * x_u8[k]
 * u8 output accumulates in a zeroed tmp area (:729-730) so y_in is 0 there.
 * Tail-kernel behaviour (rows n >= N - N%8, :677-700), reproduced as the reference has it:
 *   - y_in is never added (first K block starts from offsetC alone, later blocks reload the
 *     partial sum the kernel itself stored);
 *   - u8 output truncates instead of rounding: t = (int)(cvt(acc)*f + 128); u8 = t > 255 ? 255
 *     : (low byte of t).
 */
void orc_mvm_int8(uint32_t N, uint32_t K, const int8_t *W, int w_is_NK, const uint8_t *x,
    const int32_t *offsetC, void *y, int ydt, const float *scale)
{
    (void)ydt;
    float factor = scale ? epi_factor(scale) : 0.0f;
    uint32_t tail0 = N - N % 8;
    for (uint32_t n = 0; n < N; ++n) {
        int tail = (n >= tail0);
        int32_t acc = offsetC[n];
        if (!tail && !(scale && scale[0] < 0)) {
            acc = wrap_add(acc, ((int32_t *)y)[n]);
        }
        uint32_t s = 0;
        for (uint32_t k = 0; k < K; ++k) {
            int32_t w = w_is_NK ? W[(size_t)n * K + k] : W[(size_t)k * N + n];
            s += (uint32_t)(w * (int32_t)x[k]);
        }
        acc = wrap_add(acc, (int32_t)s);
        if (tail && scale && scale[0] < 0) {
            float f = (float)acc * factor;
            float g = f + 128.0f;
            int32_t t = (!(g >= -2147483648.0f && g < 2147483648.0f)) ? INT32_MIN : (int32_t)g;
            ((uint8_t *)y)[n] = (t > 255) ? 255 : (uint8_t)t;
        } else {
            epi_store(acc, y, n, mvm_out_type(scale), scale, factor);
        }
    }
}

/*
 * u8 matrix x s8 vector (matmul's [M,K]x[K,1] route):
 * compute/blas_enhance/src/cpu/x86/int8/avx512/mvm_avx512_vnni_row.cpp:931-1028.
 *   y[m] = (-128 * sum_k x[k]) + sum_k A_u8[m][k] * x_s8[k]
 * y is OVERWRITTEN: the driver runs a single K block (:1008-1009, blockSizeK = numColumns), so
 * the "accumulate into the stored partial" flag is never set and the previous contents of y are
 * not read (observed on the compiled reference as well). The compensation is computed inside the call (:940-985); tmp's offsetC slot is not read.
 * a_is_KM = 1: A is stored transposed [K][M] (DF_TRANSPOSE, :986-989).
 */
void orc_mvm_u8mat_i8vec(uint32_t M, uint32_t K, const uint8_t *A, int a_is_KM, const int8_t *x, void *y,
    int ydt, const float *scale)
{
    (void)ydt;
    float factor = scale ? epi_factor(scale) : 0.0f;
    int32_t off = 0;
    for (uint32_t k = 0; k < K; ++k) {
        off += x[k];
    }
    off *= -128;
    for (uint32_t m = 0; m < M; ++m) {
        int32_t acc = off; /* y_in is never read: one K block, flags bit 0 stays clear */
        uint32_t s = 0;
        for (uint32_t k = 0; k < K; ++k) {
            int32_t a = a_is_KM ? A[(size_t)k * M + m] : A[(size_t)m * K + k];
            s += (uint32_t)(a * (int32_t)x[k]);
        }
        acc = wrap_add(acc, (int32_t)s);
        epi_store(acc, y, m, mvm_out_type(scale), scale, factor);
    }
}

/* ------------------------------------------------------------------------------------
 * Quantize: compute/tensor/src/cpu/x86/int8/avx512/quantize.cpp
 * ---------------------------------------------------------------------------------- */

/* :21-68 -- max |x| by clearing the sign bit and vmaxps (NaN never wins); 127 / max in fp32 */
float orc_symmetric_scale_f32(const float *x, uint32_t n)
{
    float m = 0.0f;
    for (uint32_t i = 0; i < n; ++i) {
        float a = fabsf(x[i]);
        if (a > m) {
            m = a;
        }
    }
    return (m == 0.0f) ? 1.0f : 127.0f / m;
}

static void resolve_scale(const float *x, uint32_t n, float *scale, int mode)
{
    if (!mode || *scale <= 0) { /* :129-133 */
        float minScale = *scale;
        float dyn = orc_symmetric_scale_f32(x, n);
        *scale = (minScale > dyn) ? minScale : dyn;
    }
}

/* :121-179 -- t = x*s; u = t + 128.0f (separate add); q = clamp(rne(u), 1, 255) */
void orc_quantize_f32_u8(const float *x, uint32_t n, uint8_t *q, float *scale, int mode)
{
    resolve_scale(x, n, scale, mode);
    float s = *scale;
    for (uint32_t i = 0; i < n; ++i) {
        float t = x[i] * s;
        float u = t + 128.0f;
        int32_t v = rne_i32(u);
        v = v < 1 ? 1 : v;
        v = v > 255 ? 255 : v;
        q[i] = (uint8_t)v;
    }
}

/* :181-234 -- q = clamp(rne(x*s), -127, 127) */
void orc_quantize_f32_i8(const float *x, uint32_t n, int8_t *q, float *scale, int mode)
{
    resolve_scale(x, n, scale, mode);
    float s = *scale;
    for (uint32_t i = 0; i < n; ++i) {
        int32_t v = rne_i32(x[i] * s);
        v = v < -127 ? -127 : v;
        v = v > 127 ? 127 : v;
        q[i] = (int8_t)v;
    }
}

/* :271-313 -- byte add of 0x80 */
void orc_u8_to_i8(const uint8_t *x, uint32_t n, int8_t *q)
{
    for (uint32_t i = 0; i < n; ++i) {
        q[i] = (int8_t)(uint8_t)(x[i] + 0x80);
    }
}

/* :70-119 -- vpabsd + vpmaxsd: |INT32_MIN| stays negative and never wins */
static float requant_factor(const int32_t *x, uint32_t n, float *scale)
{
    float raw = 0.0f;
    if (scale[0] < 0 && scale[1] > 0) {
        int32_t m = 0;
        for (uint32_t i = 0; i < n; ++i) {
            int32_t a = (x[i] == INT32_MIN) ? INT32_MIN : (x[i] < 0 ? -x[i] : x[i]);
            if (a > m) {
                m = a;
            }
        }
        raw = (m == 0) ? 1.0f : 127.0f / (float)m;
        scale[0] = scale[1] * raw;
    } else if (scale[0] > 0 && scale[1] > 0) {
        raw = scale[0] / scale[1];
    }
    return raw;
}

/* :315-361 -- q = ssat8(rne(cvt(x) * r)), no -127 clamp */
void orc_quantize_i32_i8(const int32_t *x, uint32_t n, int8_t *q, float *scale)
{
    float r = requant_factor(x, n, scale);
    for (uint32_t i = 0; i < n; ++i) {
        q[i] = ssat8(rne_i32((float)x[i] * r));
    }
}

/* :364-416 -- q = usat8_u(rne(cvt(x) * r + 128.0f)) (fp32 add BEFORE rounding) */
void orc_quantize_i32_u8(const int32_t *x, uint32_t n, uint8_t *q, float *scale)
{
    float r = requant_factor(x, n, scale);
    for (uint32_t i = 0; i < n; ++i) {
        float t = (float)x[i] * r;
        float u = t + 128.0f;
        q[i] = usat8_u(rne_i32(u));
    }
}

/* :236-269 -- out[n] = (I32)(round(bias[n]*s) [+ offsetC[n]]); C round(): half away from zero.
 * bias == NULL: copy offsetC (packed filter) or zeros (offsetC == NULL). */
void orc_bias_offsetC(const float *bias, uint32_t N, const int32_t *offsetC, const float *scale, int32_t *out)
{
    for (uint32_t i = 0; i < N; ++i) {
        if (!bias) {
            out[i] = offsetC ? offsetC[i] : 0;
            continue;
        }
        float p = bias[i] * scale[0];
        double r = round((double)p);
        if (offsetC) {
            r += (double)offsetC[i];
        }
        out[i] = (int32_t)r;
    }
}

/* compute/tensor/src/cpu/x86/int8/avx512/dequantize.cpp:18-58 -- f = cvt(q) * (1 / s) */
void orc_dequantize_i32_f32(const int32_t *q, uint32_t n, const float *scale, float *out)
{
    float f = 1 / *scale;
    for (uint32_t i = 0; i < n; ++i) {
        out[i] = (float)q[i] * f;
    }
}

/* dequantize.cpp:60-101 -- f = cvt(u8 - 128) * (1 / s) */
void orc_dequantize_u8_f32(const uint8_t *q, uint32_t n, const float *scale, float *out)
{
    float f = 1 / *scale;
    for (uint32_t i = 0; i < n; ++i) {
        out[i] = (float)((int32_t)q[i] - 128) * f;
    }
}

/* compute/tensor/src/cpu/requantize.cpp:20-50 + cpu_functions_template.h:50-55:
 * out = (INT8)(rescale * in) with C truncation toward zero; memcpy when scales are equal. */
void orc_requantize_i8(const int8_t *in, uint32_t n, float inScale, int8_t *out, float outScale)
{
    if (outScale == inScale) {
        memcpy(out, in, n);
        return;
    }
    float r = outScale / inScale;
    for (uint32_t i = 0; i < n; ++i) {
        float v = r * (float)in[i] + 0.0f;
        out[i] = (int8_t)(int32_t)v;
    }
}

/* vector_vector_axpby, fp32 (compute/blas_enhance/src/cpu/x86/fp32/axpby.cpp:16-34): y = fmadd(a, x, y * b) --
 * the product y * b rounded to fp32, then one fused multiply-add. The scalar tail `a * x[i] + b * y[i]` compiles to
 * the same contraction under the reference's -O3 -mfma (checked against the compiled reference for every length). */
void orc_axpby_f32(uint32_t n, float a, const float *x, float b, float *y)
{
    for (uint32_t i = 0; i < n; ++i) {
        volatile float t = y[i] * b;
        y[i] = fmaf(a, x[i], t);
    }
}

/* Per-output-channel dequantisation with fp32 bias: not in the reference (Tensor carries one
 * scale, common/memory/include/tensor.hpp:83-96). Closed form that reduces to the reference's
 * per-tensor epilogue when every scaleW[n] is equal and bias is NULL:
 *   out[m][n] = cvt(acc) * (1.0f / (scaleI[m or 0] * scaleW[n])) (+ bias[n]) */
void orc_dequant_per_channel(const int32_t *acc, uint32_t M, uint32_t N, const float *scaleI,
    const float *scaleW, const float *bias, float *out)
{
    for (uint32_t m = 0; m < M; ++m) {
        for (uint32_t n = 0; n < N; ++n) {
            float s = scaleI[0] * scaleW[n];
            float f = 1.0f / s;
            float v = (float)acc[(size_t)m * N + n] * f;
            if (bias) {
                v = v + bias[n];
            }
            out[(size_t)m * N + n] = v;
        }
    }
}

/*
 * int8 FullyConnected, x86 branch of compute/tensor/src/fully_connected.cpp:372-495.
 *   scaleO = scaleI * scaleW (:396); offsetCBias = round(bias*scaleO) + offsetC (:400-406);
 *   output zeroed (:458); M == 1 -> matrix_vector_multiply else matrix_matrix_multiply (:461-475)
 *   F32 out: scale = &scaleO (:381-382)
 *   U8_Q out with *scaleO_io > 0: scale = {-1, scaleOut / scaleO} (:383-387,408-410)
 *   U8_Q out with *scaleO_io <= 0: int32 result then quantizeI32ToU8 with {-1, scaleO} (:388,477-486)
 *   I32 out: raw accumulators.
 * On return *scaleO_io holds the output tensor's scale (for F32 the compute scale).
 */
void orc_fully_connected_int8(uint32_t M, uint32_t K, uint32_t N, const uint8_t *x, float scaleI,
    const int8_t *W_NK, float scaleW, const float *bias, void *out, int odt, float *scaleO_io)
{
    float scaleO = scaleI * scaleW;
    int32_t *off = (int32_t *)malloc(sizeof(int32_t) * N);
    int32_t *offb = (int32_t *)malloc(sizeof(int32_t) * N);
    orc_offsetC(W_NK, K, N, 1, off);
    orc_bias_offsetC(bias, N, off, &scaleO, offb);
    float sarr[2] = {-1, -1};
    const float *scale = 0;
    int cdt = odt;
    void *dst = out;
    int32_t *i32tmp = 0;
    if (odt == ORC_F32) {
        scale = &scaleO;
    } else if (odt == ORC_U8Q) {
        if (*scaleO_io > 0) {
            sarr[1] = *scaleO_io / scaleO;
            scale = sarr;
        } else {
            cdt = ORC_I32;
            i32tmp = (int32_t *)malloc(sizeof(int32_t) * (size_t)M * N);
            dst = i32tmp;
        }
    }
    size_t esz = (cdt == ORC_U8Q) ? 1 : 4;
    memset(dst, 0, esz * (size_t)M * N);
    if (M == 1) {
        orc_mvm_int8(N, K, W_NK, 1, x, offb, dst, cdt, scale);
    } else {
        orc_mmm_int8(M, N, K, x, 0, W_NK, 1, offb, dst, cdt, scale);
    }
    if (i32tmp) {
        float sc[2] = {*scaleO_io, scaleO};
        orc_quantize_i32_u8(i32tmp, M * N, (uint8_t *)out, sc);
        *scaleO_io = sc[0];
        free(i32tmp);
    } else if (odt == ORC_F32 || odt == ORC_I32) {
        *scaleO_io = scaleO;
    }
    free(off);
    free(offb);
}
