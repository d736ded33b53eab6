/*
 * TEST INFRASTRUCTURE ONLY -- see oracle.h. Quantised pooling and concatenation restated as plain
 * loops. Never linked into the product.
 * Pinned by tests/test_oracle_pool.py against the reference's own pooling_uint8 / concat_cpu built into
 * oracle/_ref (whole tensors, every mode), against a textbook floor-mean on inputs where the fixed-point
 * form is exact, and against numpy's maximum / concatenate.
 */
#include "oracle.h"
#include <string.h>

/* compute/tensor/src/cpu/x86/int8/avx512/pooling_int8.cpp:316-429 (pooling_uint8) with the arithmetic of
 * pooling_c16_max_w1 (:113-148) and pooling_c16_mean_w1 (:278-314). in / out: u8 [n][c/16][h][w][16].
 * scale[0] is read, scale[1] written (:366-370). Returns 0, or 1 for what the reference rejects. */
int orc_pooling_u8_c16(const orc_pool_desc *d, const uint8_t *in, uint8_t *out, float *scale)
{
    if (d->c % 16 || d->pt >= d->kh || d->pl >= d->kw) {
        return 1;
    }
    const int32_t shift = 65536;
    const int32_t factor = (int32_t)((uint32_t)shift / (d->kh * d->kw)); /* :361 */
    if (factor < 1) {
        return 1;
    }
    if (scale) {
        if (!d->mean) {
            scale[1] = scale[0];
        } else {
            scale[1] = scale[0] * (float)factor * (float)(d->kw * d->kh) / (float)shift; /* :369 */
        }
    }
    const size_t planes = (size_t)d->n * (d->c / 16);
    for (size_t p = 0; p < planes; ++p) {
        const uint8_t *ip = in + p * d->ih * d->iw * 16;
        uint8_t *op = out + p * d->oh * d->ow * 16;
        for (uint32_t h = 0; h < d->oh; ++h) {
            for (uint32_t w = 0; w < d->ow; ++w) {
                int hs = (int)(h * d->sh) - (int)d->pt, ws = (int)(w * d->sw) - (int)d->pl; /* :385-390 */
                int he = hs + (int)d->kh < (int)d->ih ? hs + (int)d->kh : (int)d->ih;
                int we = ws + (int)d->kw < (int)d->iw ? ws + (int)d->kw : (int)d->iw;
                if (hs < 0) {
                    hs = 0;
                }
                if (ws < 0) {
                    ws = 0;
                }
                const int kh = he - hs, kw = we - ws;
                if (kh <= 0 || kw <= 0) {
                    return 1; /* the reference's loops are not defined for an empty window */
                }
                int32_t pool = factor; /* count_include_pad, :377 */
                if (!d->count_include_pad) {
                    pool = (int32_t)((uint32_t)shift / (uint32_t)(kh * kw)); /* :398-400 */
                }
                for (int c = 0; c < 16; ++c) {
                    if (!d->mean) {
                        uint8_t m = 0;
                        for (int y = hs; y < he; ++y) {
                            for (int x = ws; x < we; ++x) {
                                uint8_t v = ip[((size_t)y * d->iw + x) * 16 + c];
                                m = v > m ? v : m; /* vpmaxub */
                            }
                        }
                        op[((size_t)h * d->ow + w) * 16 + c] = m;
                    } else {
                        int32_t acc = -128 * kh * kw; /* :283-287 */
                        for (int y = hs; y < he; ++y) {
                            for (int x = ws; x < we; ++x) {
                                acc += ip[((size_t)y * d->iw + x) * 16 + c]; /* vpmovzxbd + vpaddd */
                            }
                        }
                        uint32_t prod = (uint32_t)acc * (uint32_t)pool; /* vpmulld: low 32 bits */
                        uint32_t r = (prod >> 16) + 128u;               /* vpsrld (logical), vpaddd */
                        op[((size_t)h * d->ow + w) * 16 + c] = r > 255u ? 255 : (uint8_t)r; /* vpmovusdb */
                    }
                }
            }
        }
    }
    return 0;
}

/* compute/tensor/src/cpu/concat.cpp:164-189 (concat_cpu, DT_I8 with scales) for inputs that are already in
 * the output's layout: *oscale = min of the input scales (cpu_functions_template.h:282-296), every input
 * requantised to it (orc_requantize_i8), then `loops` rows of len[j] bytes interleaved (concat.cpp:40-46).
 * scales == NULL: plain byte concatenation. */
void orc_concat_i8(uint32_t num, const int8_t *const *in, const uint32_t *len, const float *scales, uint32_t loops,
    int8_t *out, float *oscale)
{
    float mn = 0;
    if (scales && num) {
        mn = scales[0];
        for (uint32_t j = 1; j < num; ++j) {
            mn = scales[j] < mn ? scales[j] : mn;
        }
        if (oscale) {
            *oscale = mn;
        }
    }
    size_t stride = 0;
    for (uint32_t j = 0; j < num; ++j) {
        stride += len[j];
    }
    size_t off = 0;
    for (uint32_t j = 0; j < num; ++j) {
        for (uint32_t i = 0; i < loops; ++i) {
            const int8_t *s = in[j] + (size_t)i * len[j];
            int8_t *dst = out + (size_t)i * stride + off;
            if (scales) {
                orc_requantize_i8(s, len[j], scales[j], dst, mn);
            } else {
                memcpy(dst, s, len[j]);
            }
        }
        off += len[j];
    }
}
