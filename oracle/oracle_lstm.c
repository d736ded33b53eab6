/*
 * TEST INFRASTRUCTURE ONLY -- see oracle.h. The int8 LSTM cell restated as plain loops. Never linked into
 * the product.
 * Pinned by tests/test_oracle_lstm.py: the quantised [x | h] bytes and the integer products come from
 * orc_quantize_f32_u8 / orc_mvm_int8 (pinned bit for bit elsewhere); the whole cell is compared with the
 * reference's own compiled lstmcell_int8 (oracle/_ref) to 2e-6, the difference being the reference's
 * polynomial exp in its 8-wide loop against libm here, and with an independent float64 numpy cell.
 */
#include "oracle.h"
#include <math.h>
#include <stdlib.h>
#include <string.h>

/* compute/tensor/src/cpu/x86/int8/lstm.cpp:20-179. W: s8 [4*column][xdim+hdim] row-major (the matrix the reference
 * packs), gate order i, g, f, o (:118-121); gates as the scalar tail computes them (:151-161). column = hdim without a
 * projection (Wp NULL); with one, column = num_projection, the gates give column values per row and the hidden state
 * is Wp times those (:170-173, mvm_nkn32_with_bias in cpu/x86/fp32/mvm_nkn32.h:19-140: Wp is fp32 [hdim/32][column][32],
 * every output one chain of fused multiply-adds over k ascending from 0). state row m: [C (column) | H (hdim)].
 * scale = {activation scale or <= 0, weight scale}. */
void orc_lstmcell_int8_proj(uint32_t batch, uint32_t xdim, uint32_t hdim, uint32_t column, const float *x, uint32_t x_stride,
    const int8_t *W, const float *Wp, const float *bias, uint32_t bias_stride, const float *scale, float *state,
    float forget_bias, float zoneout_cell, float zoneout_output, float *out, uint32_t out_stride)
{
    const uint32_t K = xdim + hdim, N = 4 * column;
    float *xh = (float *)malloc(sizeof(float) * K);
    float *inter = (float *)malloc(sizeof(float) * N);
    float *act = (float *)malloc(sizeof(float) * column);
    uint8_t *q = (uint8_t *)malloc(K);
    int32_t *offsetC = (int32_t *)malloc(sizeof(int32_t) * N);
    orc_offsetC(W, K, N, 1, offsetC); /* the vector behind the packed weight, :110 */
    for (uint32_t m = 0; m < batch; ++m) {
        float *stC = state + (size_t)m * (column + hdim), *stH = stC + column;
        memcpy(xh, x + (size_t)m * x_stride, sizeof(float) * xdim); /* :93-95 */
        memcpy(xh + xdim, stH, sizeof(float) * hdim);
        float iScale = scale[0];
        orc_quantize_f32_u8(xh, K, q, &iScale, 1); /* :106 */
        float oScale = iScale * scale[1];          /* :107 */
        memset(inter, 0, sizeof(float) * N);
        orc_mvm_int8(N, K, W, 1, q, offsetC, inter, ORC_F32, &oScale); /* :109-112 */
        const float *b = bias + (size_t)m * bias_stride;
        for (uint32_t n = 0; n < N; ++n) {
            inter[n] = inter[n] + b[n]; /* :114 */
        }
        for (uint32_t h = 0; h < column; ++h) { /* :151-161 */
            float C_s = stC[h];
            float I_s = (float)(1.0 / (1.0 + exp(-inter[h])));
            float F_s = (float)(1.0 / (1.0 + exp(-(inter[h + 2 * column] + forget_bias))));
            float O_s = (float)(1.0 / (1.0 + exp(-inter[h + 3 * column])));
            float G_s = (float)tanh(inter[h + column]);
            float C_n = C_s * F_s + I_s * G_s;
            act[h] = (float)(O_s * tanh(C_n));
            if (zoneout_cell != 0) { /* :164-168 */
                stC[h] = C_n * (1 - zoneout_cell) + C_s * zoneout_cell;
            } else {
                stC[h] = C_n;
            }
        }
        for (uint32_t h = 0; h < hdim; ++h) {
            float value;
            if (Wp) { /* :170-173 */
                float acc = 0.0f;
                for (uint32_t k = 0; k < column; ++k) {
                    acc = fmaf(act[k], Wp[((size_t)(h / 32) * column + k) * 32 + h % 32], acc);
                }
                value = acc;
            } else {
                value = act[h];
            }
            out[(size_t)m * out_stride + h] = value;
            if (zoneout_output != 0) { /* :175-178 */
                stH[h] = value * (1 - zoneout_output) + stH[h] * zoneout_output;
            } else {
                stH[h] = value;
            }
        }
    }
    free(xh);
    free(inter);
    free(act);
    free(q);
    free(offsetC);
}

void orc_lstmcell_int8(uint32_t batch, uint32_t xdim, uint32_t hdim, const float *x, uint32_t x_stride,
    const int8_t *W, const float *bias, uint32_t bias_stride, const float *scale, float *state, float forget_bias,
    float zoneout_cell, float zoneout_output, float *out, uint32_t out_stride)
{
    orc_lstmcell_int8_proj(batch, xdim, hdim, hdim, x, x_stride, W, NULL, bias, bias_stride, scale, state, forget_bias,
        zoneout_cell, zoneout_output, out, out_stride);
}
