/* TEST INFRASTRUCTURE ONLY -- CPU restatement of the weight-storage arithmetic of Bolt's post-training quantisation
 * tool and of the matching load-time expansion, used by tests/ to check the GPU path. Never linked into the product.
 *
 *   storage quantisation : model_tools/src/model_data_type_converter.cpp:22-103
 *                          (ws_datatype_converter_bnn / _int8 / _int4, roundNearestEven)
 *   load-time expansion  : common/model_spec/src/model_deserialize.cpp:162-222
 *                          (dequantize_int8_weight, dequantize_int4_weight, dequantize_int4_int8, dequantize_int4_u8_q)
 */
#include <math.h>
#include <stdint.h>
#include "oracle.h"

/* roundNearestEven (:48-58): C round(), then ties pulled back to the even neighbour -- round-to-nearest-even of a
 * float, which nearbyintf gives under the default FE_TONEAREST mode */
static int8_t rne_i8(float v)
{
    return (int8_t)nearbyintf(v);
}

static float max_abs(const float *w, int n)
{
    float m = 0;
    for (int i = 0; i < n; ++i) {
        const float a = fabsf(w[i]);
        if (a > m) {
            m = a;
        }
    }
    return m;
}

/* :60-75: scale = max(127.0 / max|w| (a double quotient), caller's scale), stored as float; q = rne(w * scale) */
void orc_ws_convert_int8(const float *w, int n, int8_t *q, float *scale)
{
    const float m = max_abs(w, n);
    const double dyn = 127.0 / (double)m;
    *scale = (float)(dyn > (double)*scale ? dyn : (double)*scale);
    for (int i = 0; i < n; ++i) {
        const float p = w[i] * *scale;
        q[i] = rne_i8(p);
    }
}

/* :77-103 for an even count: nibble = rne((float)(w * 7.0 / max|w|)) + 7, the product and quotient in double; element i
 * in the low (even i) or high (odd i) half of byte i / 2; scale = max(7.0 / max|w|, caller's scale) */
void orc_ws_convert_int4(const float *w, int n, int8_t *q, float *scale)
{
    const float m = max_abs(w, n);
    const double dyn = 7.0 / (double)m;
    *scale = (float)(dyn > (double)*scale ? dyn : (double)*scale);
    for (int i = 0; i + 1 < n; i += 2) {
        const int8_t t0 = (int8_t)(rne_i8((float)((double)w[i] * 7.0 / (double)m)) + 7);
        const int8_t t1 = (int8_t)(rne_i8((float)((double)w[i + 1] * 7.0 / (double)m)) + 7);
        q[i / 2] = (int8_t)((t1 << 4) | t0);
    }
}

/* :22-46: one bit per weight, set when w > 0, first weight in the top bit; returns the first positive weight (the
 * common magnitude of a binary filter), or the last weight if none is positive, or 1 for an empty tensor */
float orc_ws_convert_bnn(const float *w, int n, uint8_t *bits)
{
    for (int i = 0; i < n; i += 8) {
        uint8_t b = 0;
        for (int j = 0; j < 8; ++j) {
            if (w[i + j] > 0) {
                b |= (uint8_t)(1u << (7 - j));
            }
        }
        bits[i / 8] = b;
    }
    float scale = 1;
    for (int i = 0; i < n; ++i) {
        scale = w[i];
        if (scale > 0) {
            break;
        }
    }
    return scale;
}

/* model_deserialize.cpp:162-185: d = (1 / scale) * q through a 255-entry table, the product in float */
void orc_dequantize_int8_weight(int n, float scale, const int8_t *q, float *d)
{
    const float factor = 1 / scale;
    for (int i = 0; i < n; ++i) {
        d[i] = factor * (float)(int)q[i];
    }
}

/* :187-208 */
void orc_dequantize_int4_weight(int n, float scale, const int8_t *q, float *d)
{
    const float factor = 1 / scale;
    for (int i = 0; i < n; ++i) {
        const int nib = (q[i / 2] >> ((i % 2) * 4)) & 0xF;
        d[i] = factor * (float)(nib - 7);
    }
}

/* :210-215 */
void orc_dequantize_int4_int8(int n, const int8_t *q, int8_t *d)
{
    for (int i = 0; i < n; ++i) {
        d[i] = (int8_t)(((q[i / 2] >> ((i % 2) * 4)) & 0xF) - 7);
    }
}

/* :217-222 */
void orc_dequantize_int4_u8q(int n, const int8_t *q, uint8_t *d)
{
    for (int i = 0; i < n; ++i) {
        d[i] = (uint8_t)(((q[i / 2] >> ((i % 2) * 4)) & 0xF) + 121);
    }
}
