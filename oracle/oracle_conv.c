/*
 * TEST INFRASTRUCTURE ONLY -- see oracle.h. int8 convolution (x86 direct-conv semantics) and
 * 1-bit XNOR / DoReFa convolution restated as plain loops. Never linked into the product.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

static inline int32_t rne_i32_(float v)
{
    if (!(v >= -2147483648.0f && v < 2147483648.0f)) {
        return INT32_MIN;
    }
    return (int32_t)lrintf(v);
}

/* NCHWCx element index, compute/tensor/src/cpu/general/convolution.cpp:98-106 */
static inline size_t nchwcx(uint32_t n, uint32_t c, uint32_t h, uint32_t w, uint32_t C, uint32_t H, uint32_t W, uint32_t x)
{
    return ((((size_t)n * (C / x) + c / x) * H + h) * W + w) * x + c % x;
}

/*
 * Accumulators of the x86 int8 direct convolution,
 * compute/tensor/src/cpu/x86/int8/avx512/convolution_direct.cpp:2584-2809:
 *   acc = offsetC[oc] + round(bias[oc] * scaleI * scaleF) + sum_{c,kh,kw} in_u8 * w_s8
 * with offsetC[oc] = -128 * sum over ALL taps of w (convolution_transform.cpp:38-44) and the padded
 * border reading 128 (transform_functions_int8.h:187-205), i.e.
 *   acc = round(bias * s) + sum_{taps inside the image} (in_u8 - 128) * w
 * Input u8 NCHWC8, filter s8 NCHW, output plain [n][oc][oh][ow].
 */
void orc_conv_int8_acc(const orc_conv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias,
    float scaleI, float scaleF, int32_t *acc)
{
    const float s = scaleI * scaleF; /* :2687 */
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t o = 0; o < d->oc; ++o) {
            int32_t b = 0;
            if (bias) {
                float p = bias[o] * s;
                b = (int32_t)round((double)p); /* avx512/quantize.cpp:259-267 */
            }
            for (uint32_t y = 0; y < d->oh; ++y) {
                for (uint32_t x = 0; x < d->ow; ++x) {
                    uint32_t a = (uint32_t)b;
                    for (uint32_t c = 0; c < d->ic; ++c) {
                        for (uint32_t kh = 0; kh < d->fh; ++kh) {
                            const int64_t ih = (int64_t)y * d->sh + (int64_t)kh * d->dh - d->pt;
                            if (ih < 0 || ih >= (int64_t)d->ih) {
                                continue;
                            }
                            for (uint32_t kw = 0; kw < d->fw; ++kw) {
                                const int64_t iw = (int64_t)x * d->sw + (int64_t)kw * d->dw - d->pl;
                                if (iw < 0 || iw >= (int64_t)d->iw) {
                                    continue;
                                }
                                const int32_t v = (int32_t)in[nchwcx(n, c, (uint32_t)ih, (uint32_t)iw, d->ic, d->ih, d->iw, 8)] - 128;
                                const int32_t w = filter[(((size_t)o * d->ic + c) * d->fh + kh) * d->fw + kw];
                                a += (uint32_t)(v * w);
                            }
                        }
                    }
                    acc[(((size_t)n * d->oc + o) * d->oh + y) * d->ow + x] = (int32_t)a;
                }
            }
        }
    }
}

/* output element index of the x86 path: 16-channel blocks, a trailing 8-channel block when
 * oc % 16 == 8 (convolution_direct.cpp:2758-2769, simdOc = min(16, ocSize)); out_c = 8 gives the
 * plain NCHWC8 the path is also asked for. */
static inline size_t conv_out_index(const orc_conv_desc *d, uint32_t n, uint32_t o, uint32_t r)
{
    const uint32_t x = (uint32_t)d->out_c;
    const uint32_t blk = o / x;
    uint32_t bw = d->oc - blk * x;
    bw = bw < x ? bw : x;
    return (size_t)n * d->oc * d->oh * d->ow + (size_t)blk * x * d->oh * d->ow + (size_t)r * bw + o % x;
}

/*
 * Full operator (convolution_direct.cpp:2676-2706, kernel epilogue :2393-2425, requant :2797-2806).
 *   scale = {input scale, output scale (in / out), filter scale}
 *   ORC_F32: out = cvt(acc) * (1 / (sI*sF)) [+ eltwise], ReLU in fp32; scale[1] = sI*sF
 *   ORC_I32: ReLU in the integer domain, raw accumulators
 *   ORC_U8Q: integer ReLU, then dynamic requantisation over the WHOLE batch tensor:
 *            r = 127 / max|acc| (1 if 0), u8 = usat8_u(rne(cvt(acc) * r + 128.0f)), scale[1] = sI*sF*r
 */
void orc_conv_int8(const orc_conv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias,
    const float *eltwise, float *scale, void *out)
{
    const size_t total = (size_t)d->n * d->oc * d->oh * d->ow;
    const uint32_t ohw = d->oh * d->ow;
    int32_t *acc = (int32_t *)malloc(sizeof(int32_t) * total);
    orc_conv_int8_acc(d, in, filter, bias, scale[0], scale[2], acc);
    const float sO = scale[0] * scale[2];
    scale[1] = sO;
    if (d->odt == ORC_F32) {
        const float f = 1 / sO;
        for (uint32_t n = 0; n < d->n; ++n) {
            for (uint32_t o = 0; o < d->oc; ++o) {
                for (uint32_t r = 0; r < ohw; ++r) {
                    const size_t oi = conv_out_index(d, n, o, r);
                    float v = (float)acc[((size_t)n * d->oc + o) * ohw + r] * f;
                    if (eltwise) {
                        v = v + eltwise[oi];
                    }
                    if (d->relu && !(v > 0.0f)) {
                        v = 0.0f; /* vmaxps(0, v) */
                    }
                    ((float *)out)[oi] = v;
                }
            }
        }
        free(acc);
        return;
    }
    int32_t m = 0;
    for (size_t i = 0; i < total; ++i) {
        if (d->relu && acc[i] < 0) {
            acc[i] = 0;
        }
        const int32_t a = (acc[i] == INT32_MIN) ? INT32_MIN : (acc[i] < 0 ? -acc[i] : acc[i]);
        if (a > m) {
            m = a;
        }
    }
    const float r = (m == 0) ? 1.0f : 127.0f / (float)m;
    if (d->odt == ORC_U8Q) {
        scale[1] = sO * r;
    }
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t o = 0; o < d->oc; ++o) {
            for (uint32_t p = 0; p < ohw; ++p) {
                const int32_t a = acc[((size_t)n * d->oc + o) * ohw + p];
                const size_t oi = conv_out_index(d, n, o, p);
                if (d->odt == ORC_I32) {
                    ((int32_t *)out)[oi] = a;
                } else {
                    const float t = (float)a * r;
                    const float u = t + 128.0f;
                    const int32_t q = rne_i32_(u);
                    ((uint8_t *)out)[oi] = ((uint32_t)q > 255u) ? 255 : (uint8_t)q;
                }
            }
        }
    }
    free(acc);
}

/* ------------------------------------------------------------------------------------
 * 1-bit convolution. The reference path is ARMv8.2 fp16 only
 * (compute/tensor/src/cpu/arm/bnn/convolution_xnor_A76.cpp, convolution_dorefa_A76.cpp; naive form
 * compute/tensor/src/cpu/general/convolution.cpp:141-178,265-284) and cannot be built on x86.
 * ---------------------------------------------------------------------------------- */

/* common/uni/include/data_type.h:203-222 applied to an NCHWC8 tensor: 8 consecutive values (the 8
 * channels of one pixel) make one byte, first value in the MSB; 1 iff x >= threshold (0 for
 * DT_BIN11, 0.5 for DT_BIN01). Result layout [n][c/8][h][w] bytes. */
void orc_bnn_pack_input(const orc_bnn_desc *d, const float *x_nchwc8, uint8_t *bits)
{
    const float thr = d->xnor ? 0.0f : 0.5f;
    const size_t nbytes = (size_t)d->n * (d->ic / 8) * d->ih * d->iw;
    for (size_t i = 0; i < nbytes; ++i) {
        uint8_t b = 0;
        for (int j = 0; j < 8; ++j) {
            if (x_nchwc8[i * 8 + j] >= thr) {
                b |= (uint8_t)(1u << (7 - j));
            }
        }
        bits[i] = b;
    }
}

/*
 * convolution_xnor_A76.cpp:59-106,657-720 / convolution_dorefa_A76.cpp:627-712.
 *   in_bits  [n][ic/8][ih][iw] bytes, padded with 0 bits (transform_functions.h:163-204)
 *   w_bits   DF_NCHWN16C8: byte index ((o/16 * ic/8 + c/8) * fh*fw + hw) * 16 + o%16
 *            (convolution_transform_bnn.h:58-79), MSB = channel c%8 == 0
 *   XNOR:    S = fh*fw*ic - 2 * popcount(x XOR w)       (0 bit = -1, so padding counts as -1)
 *   DoReFa:  S = popcount(x AND w)
 *   out = fma(S, scale[o], bias[o]) (vfmaq in the reference), NCHWC8.
 */
void orc_bnn_conv(const orc_bnn_desc *d, const uint8_t *in_bits, const uint8_t *w_bits, const float *scale,
    const float *bias, int32_t *sums, float *out)
{
    const uint32_t ic8 = d->ic / 8, fhw = d->fh * d->fw;
    const int32_t base = (int32_t)(fhw * d->ic);
#pragma omp parallel for collapse(2) schedule(static)
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t o = 0; o < d->oc; ++o) {
            for (uint32_t y = 0; y < d->oh; ++y) {
                for (uint32_t x = 0; x < d->ow; ++x) {
                    int32_t cnt = 0;
                    for (uint32_t c = 0; c < ic8; ++c) {
                        for (uint32_t kh = 0; kh < d->fh; ++kh) {
                            for (uint32_t kw = 0; kw < d->fw; ++kw) {
                                const int64_t ih = (int64_t)y * d->sh + kh - d->pt;
                                const int64_t iw = (int64_t)x * d->sw + kw - d->pl;
                                uint8_t xb = 0; /* zero-bit padding */
                                if (ih >= 0 && ih < (int64_t)d->ih && iw >= 0 && iw < (int64_t)d->iw) {
                                    xb = in_bits[(((size_t)n * ic8 + c) * d->ih + (size_t)ih) * d->iw + (size_t)iw];
                                }
                                const uint8_t wb =
                                    w_bits[(((size_t)(o / 16) * ic8 + c) * fhw + kh * d->fw + kw) * 16 + o % 16];
                                cnt += __builtin_popcount(d->xnor ? (uint8_t)(xb ^ wb) : (uint8_t)(xb & wb));
                            }
                        }
                    }
                    const int32_t S = d->xnor ? base - 2 * cnt : cnt;
                    const size_t oi = nchwcx(n, o, y, x, d->oc, d->oh, d->ow, 8);
                    if (sums) {
                        sums[oi] = S;
                    }
                    if (out) {
                        out[oi] = fmaf((float)S, scale[o], bias[o]);
                    }
                }
            }
        }
    }
}

/* Independent check of the above: convolution of the +-1 / {0,1} VALUES (plain NCHW floats), pad
 * value -1 (XNOR) / 0 (DoReFa) as in cpu/general/convolution.cpp:272,282. Output plain NCHW. */
void orc_bnn_conv_bruteforce(const orc_bnn_desc *d, const float *x_nchw, const float *w_nchw, int32_t *sums_nchw)
{
    const float thr = d->xnor ? 0.0f : 0.5f;
    const int lo = d->xnor ? -1 : 0;
    for (uint32_t n = 0; n < d->n; ++n) {
        for (uint32_t o = 0; o < d->oc; ++o) {
            for (uint32_t y = 0; y < d->oh; ++y) {
                for (uint32_t x = 0; x < d->ow; ++x) {
                    int32_t s = 0;
                    for (uint32_t c = 0; c < d->ic; ++c) {
                        for (uint32_t kh = 0; kh < d->fh; ++kh) {
                            for (uint32_t kw = 0; kw < d->fw; ++kw) {
                                const int64_t ih = (int64_t)y * d->sh + kh - d->pt;
                                const int64_t iw = (int64_t)x * d->sw + kw - d->pl;
                                int xv = lo;
                                if (ih >= 0 && ih < (int64_t)d->ih && iw >= 0 && iw < (int64_t)d->iw) {
                                    xv = (x_nchw[(((size_t)n * d->ic + c) * d->ih + (size_t)ih) * d->iw + (size_t)iw] >= thr) ? 1 : lo;
                                }
                                const int wv = (w_nchw[(((size_t)o * d->ic + c) * d->fh + kh) * d->fw + kw] >= thr) ? 1 : lo;
                                s += xv * wv;
                            }
                        }
                    }
                    sums_nchw[(((size_t)n * d->oc + o) * d->oh + y) * d->ow + x] = s;
                }
            }
        }
    }
}
