/* TEST INFRASTRUCTURE ONLY -- CPU restatement of the reference's int8 deconvolution (transposed
 * convolution) on x86, used by tests/ to check the GPU path. Never linked into the product.
 *
 * Reference: compute/tensor/src/cpu/deconvolution.cpp
 *   - deconvolution_gemm (:252-365), taken for DF_NCHW inputs (CONVOLUTION_ALGORITHM_IM2COL_GEMM, :52-53)
 *   - deconvolution_pointwise_x86 (compute/tensor/src/cpu/x86/deconvolution.cpp:130-257), taken for
 *     DF_NCHWC8 / DF_NCHWC16 inputs (CONVOLUTION_ALGORITHM_POINTWISE, :47-50)
 *   - overlap-and-crop: compute/tensor/src/cpu/x86/fp32/transform_functions_fp32.h:221-280 (gemm form),
 *     :348-409 (pointwise, overlapping taps), :411-463 (pointwise, kernel == stride)
 * Both forms first multiply every input pixel's channel vector with the [ic] x [oc * fh * fw] filter
 * matrix (u8 x s8, int32) and then add each product column into the output pixel it lands on:
 *   col[n, kh, kw][o, jh, jw] = sum_c (in_u8[n, c, kh, kw] - 128) * w[c][o][jh][jw]
 *   lands on (oh, ow) = (kh * sh + jh - pad_top, kw * sw + jw - pad_left) when inside the output.
 * What differs is where bias, activation and the change of data type sit:
 *   IM2COL_GEMM: acc = round(sI*sW*b[o]) + sum col; ReLU on int32; then F32 = cvt(acc) * (1 / (sI*sW)), or
 *                u8 = requantised with {scale[1], sI*sW} (dynamic when scale[1] <= 0); scale[2] becomes sI*sW
 *                when the output is quantised (:355-357).
 *   POINTWISE, kernel == stride (every output pixel has exactly one tap): the 1x1 convolution itself
 *                folds the bias and writes u8 with a dynamic scale taken over ALL columns (cropped ones
 *                included); F32 output is that u8 dequantised; ReLU last (u8: max(q, 128)).
 *   POINTWISE, overlapping taps: u8 output: int32 sums + round(sI*sW*b), dynamic requantisation
 *                (scale[2] = sI*sW, scale[1] = sI*sW*r), ReLU last; F32 output: every column is first
 *                dequantised, cvt(col) * (1 / (sI*sW)), and the fp32 terms are added onto b[o] in
 *                ascending (kh, kw) order; ReLU last; scale[1] = sI*sW.
 */
#include <math.h>
#include <stdint.h>
#include <stdlib.h>
#include <string.h>
#include "oracle.h"

static inline size_t in_index(const orc_deconv_desc *d, uint32_t n, uint32_t c, uint32_t h, uint32_t w)
{
    if (d->in_c == 0) {
        return (((size_t)n * d->ic + c) * d->ih + h) * d->iw + w;
    }
    const uint32_t x = (uint32_t)d->in_c;
    return ((((size_t)n * (d->ic / x) + c / x) * d->ih + h) * d->iw + w) * x + c % x;
}

static inline size_t out_index(const orc_deconv_desc *d, uint32_t n, uint32_t o, uint32_t h, uint32_t w)
{
    const uint32_t x = (uint32_t)d->out_c;
    return ((((size_t)n * (d->oc / x) + o / x) * d->oh + h) * d->ow + w) * x + o % x;
}

/* col[((n*ih + kh)*iw + kw)][(jh*fw + jw)*oc + o] */
static int32_t *product_columns(const orc_deconv_desc *d, const uint8_t *in, const int8_t *filter)
{
    const uint32_t taps = d->fh * d->fw;
    const size_t cols = (size_t)taps * d->oc;
    int32_t *col = (int32_t *)calloc((size_t)d->n * d->ih * d->iw * cols, sizeof(int32_t));
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t kh = 0; kh < d->ih; ++kh) {
            for (uint32_t kw = 0; kw < d->iw; ++kw) {
                int32_t *row = col + (((size_t)n * d->ih + kh) * d->iw + kw) * cols;
                for (uint32_t c = 0; c < d->ic; ++c) {
                    const int32_t v = (int32_t)in[in_index(d, n, c, kh, kw)] - 128;
                    for (uint32_t o = 0; o < d->oc; ++o) {
                        for (uint32_t j = 0; j < taps; ++j) {
                            row[(size_t)j * d->oc + o] += v * filter[((size_t)c * d->oc + o) * taps + j];
                        }
                    }
                }
            }
        }
    }
    return col;
}

void orc_deconv_int8(const orc_deconv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias, float *scale,
    void *out)
{
    const uint32_t taps = d->fh * d->fw;
    const size_t cols = (size_t)taps * d->oc;
    const size_t pixels = (size_t)d->n * d->ih * d->iw;
    const size_t total = (size_t)d->n * d->oc * d->oh * d->ow;
    const float sO = scale[0] * scale[2];
    int32_t *col = product_columns(d, in, filter);
    int32_t *bq = (int32_t *)malloc(sizeof(int32_t) * d->oc);
    for (uint32_t o = 0; o < d->oc; ++o) {
        const float p = sO * bias[o];
        bq[o] = (int32_t)round((double)p);
    }
    const int gemm_form = d->in_c == 0;
    const int equal = !gemm_form && d->fh == d->sh && d->fw == d->sw;

    if (equal) {
        /* x86/deconvolution.cpp:157-165,178-194: the convolution output is u8 whatever the tensor asked for */
        for (size_t m = 0; m < pixels; ++m) {
            for (uint32_t j = 0; j < taps; ++j) {
                for (uint32_t o = 0; o < d->oc; ++o) {
                    col[m * cols + (size_t)j * d->oc + o] += bq[o];
                }
            }
        }
        uint8_t *qcol = (uint8_t *)malloc(pixels * cols);
        float s2[2] = {-1.0f, sO};
        orc_quantize_i32_u8(col, (uint32_t)(pixels * cols), qcol, s2); /* the 1x1 convolution's own requantisation */
        scale[1] = s2[0];
        const float inv = 1.0f / scale[1];
        for (uint32_t n = 0; n < d->n; ++n) {
            for (uint32_t kh = 0; kh < d->ih; ++kh) {
                for (uint32_t kw = 0; kw < d->iw; ++kw) {
                    const uint8_t *row = qcol + (((size_t)n * d->ih + kh) * d->iw + kw) * cols;
                    for (uint32_t j = 0; j < taps; ++j) {
                        const int64_t oh = (int64_t)kh * d->sh + j / d->fw - d->pt, ow = (int64_t)kw * d->sw + j % d->fw - d->pl;
                        if (oh < 0 || oh >= (int64_t)d->oh || ow < 0 || ow >= (int64_t)d->ow) {
                            continue;
                        }
                        for (uint32_t o = 0; o < d->oc; ++o) {
                            uint8_t q = row[(size_t)j * d->oc + o];
                            const size_t oi = out_index(d, n, o, (uint32_t)oh, (uint32_t)ow);
                            if (d->odt == ORC_U8Q) {
                                if (d->relu && q < 128) {
                                    q = 128; /* vpmaxub with 0x80, x86_functions_int8.h:32-61 */
                                }
                                ((uint8_t *)out)[oi] = q;
                            } else {
                                float f = (float)((int32_t)q - 128) * inv; /* avx512/dequantize.cpp:62-101 */
                                if (d->relu && !(f > 0.0f)) {
                                    f = 0.0f;
                                }
                                ((float *)out)[oi] = f;
                            }
                        }
                    }
                }
            }
        }
        free(qcol);
        free(col);
        free(bq);
        return;
    }

    if (!gemm_form && d->odt == ORC_F32) {
        /* x86/deconvolution.cpp:166-176,212-227: fp32 columns added onto the bias in (kh, kw) order */
        const float f = 1 / sO;
        scale[1] = sO;
        for (uint32_t n = 0; n < d->n; ++n) {
            for (uint32_t o = 0; o < d->oc; ++o) {
                for (uint32_t oh = 0; oh < d->oh; ++oh) {
                    for (uint32_t ow = 0; ow < d->ow; ++ow) {
                        float a = bias[o];
                        for (uint32_t kh = 0; kh < d->ih; ++kh) {
                            const int64_t jh = (int64_t)oh + d->pt - (int64_t)kh * d->sh;
                            if (jh < 0 || jh >= (int64_t)d->fh) {
                                continue;
                            }
                            for (uint32_t kw = 0; kw < d->iw; ++kw) {
                                const int64_t jw = (int64_t)ow + d->pl - (int64_t)kw * d->sw;
                                if (jw < 0 || jw >= (int64_t)d->fw) {
                                    continue;
                                }
                                const int32_t v = col[(((size_t)n * d->ih + kh) * d->iw + kw) * cols +
                                    (size_t)(jh * d->fw + jw) * d->oc + o];
                                const float t = (float)v * f;
                                a = a + t;
                            }
                        }
                        if (d->relu && !(a > 0.0f)) {
                            a = 0.0f;
                        }
                        ((float *)out)[out_index(d, n, o, oh, ow)] = a;
                    }
                }
            }
        }
        free(col);
        free(bq);
        return;
    }

    /* int32 sums: bias + every column that lands on the pixel (order does not matter) */
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * total);
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t o = 0; o < d->oc; ++o) {
            for (uint32_t oh = 0; oh < d->oh; ++oh) {
                for (uint32_t ow = 0; ow < d->ow; ++ow) {
                    uint32_t a = (uint32_t)bq[o];
                    for (uint32_t jh = 0; jh < d->fh; ++jh) {
                        const int64_t t = (int64_t)oh + d->pt - jh;
                        if (t < 0 || t % d->sh || t / d->sh >= (int64_t)d->ih) {
                            continue;
                        }
                        for (uint32_t jw = 0; jw < d->fw; ++jw) {
                            const int64_t u = (int64_t)ow + d->pl - jw;
                            if (u < 0 || u % d->sw || u / d->sw >= (int64_t)d->iw) {
                                continue;
                            }
                            a += (uint32_t)col[(((size_t)n * d->ih + t / d->sh) * d->iw + u / d->sw) * cols +
                                (size_t)(jh * d->fw + jw) * d->oc + o];
                        }
                    }
                    acc[out_index(d, n, o, oh, ow)] = (int32_t)a;
                }
            }
        }
    }
    free(col);
    free(bq);
    if (gemm_form && d->relu) {
        for (size_t i = 0; i < total; ++i) {
            acc[i] = acc[i] < 0 ? 0 : acc[i]; /* deconvolution.cpp:338-342 */
        }
    }
    if (d->odt == ORC_F32) { /* gemm form only: deconvolution.cpp:346-354 */
        const float f = 1 / sO;
        for (size_t i = 0; i < total; ++i) {
            ((float *)out)[i] = (float)acc[i] * f;
        }
    } else if (d->odt == ORC_I32) {
        memcpy(out, acc, sizeof(int32_t) * total);
    } else {
        float s2[2] = {gemm_form ? scale[1] : -1.0f, sO}; /* deconvolution.cpp:356-357, x86/deconvolution.cpp:243-245 */
        orc_quantize_i32_u8(acc, (uint32_t)total, (uint8_t *)out, s2);
        scale[1] = s2[0];
        scale[2] = sO;
        if (!gemm_form && d->relu) {
            for (size_t i = 0; i < total; ++i) {
                uint8_t *q = (uint8_t *)out + i;
                *q = *q < 128 ? 128 : *q;
            }
        }
    }
    free(acc);
}

/* ------------------------------------------------------------------------------------
 * int8 depthwise convolution as the reference's x86 kernel computes it
 * (compute/tensor/src/cpu/x86/int8/avx512/depthwise_convolution_direct.cpp:441-599): u8 NCHWC16 input,
 * one s8 fh x fw filter per channel, int32 result in NCHWC16:
 *   acc[n, c, y, x] = round(bias[c] * sI * sF) + sum_{kh, kw} (in_u8[n, c, y*sh + kh, x*sw + kw] - 128) * w[c][kh][kw]
 * with ReLU in the integer domain (:125-145). The window is taken from the UNPADDED image at (y*sh, x*sw) (:560-566):
 * paddings and dilation do not enter the gather, so only pad 0 / dilation 1 is a convolution; the restatement covers
 * exactly that. The int32 result is the only defined one: the fp32 epilogue converts the bits of the scale factor
 * instead of the accumulators (:148-166), and a quantised result is left in tmp, never written to the output (:521-525).
 * scale = {input, output (written: sI * sF), filter}.
 * ---------------------------------------------------------------------------------- */
void orc_depthwise_int8_i32(uint32_t n, uint32_t c, uint32_t ih, uint32_t iw, uint32_t fh, uint32_t fw, uint32_t sh,
    uint32_t sw, uint32_t oh, uint32_t ow, const uint8_t *in, const int8_t *filter, const float *bias, float *scale, int relu,
    int32_t *out)
{
    const float s = scale[0] * scale[2];
    scale[1] = s;
    for (uint32_t b = 0; b < n; ++b) {
        for (uint32_t ch = 0; ch < c; ++ch) {
            int32_t bq = 0;
            if (bias) {
                const float p = bias[ch] * s;
                bq = (int32_t)round((double)p); /* avx512/quantize.cpp:236-269 */
            }
            for (uint32_t y = 0; y < oh; ++y) {
                for (uint32_t x = 0; x < ow; ++x) {
                    uint32_t a = (uint32_t)bq;
                    for (uint32_t kh = 0; kh < fh; ++kh) {
                        for (uint32_t kw = 0; kw < fw; ++kw) {
                            const size_t ii = ((((size_t)b * (c / 16) + ch / 16) * ih + (y * sh + kh)) * iw + (x * sw + kw)) * 16 + ch % 16;
                            a += (uint32_t)(((int32_t)in[ii] - 128) * (int32_t)filter[((size_t)ch * fh + kh) * fw + kw]);
                        }
                    }
                    int32_t v = (int32_t)a;
                    if (relu && v < 0) {
                        v = 0;
                    }
                    out[((((size_t)b * (c / 16) + ch / 16) * oh + y) * ow + x) * 16 + ch % 16] = v;
                }
            }
        }
    }
}
