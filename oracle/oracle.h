/*
 * TEST INFRASTRUCTURE ONLY -- CPU restatement of Bolt's x86 AVX-512-VNNI quantized
 * matrix-product path, used as the parity checker for the gfx950 kernels.
 *
 * Only tests/, __graft_entry__.smoke() and the cpu_baseline leg of bench.py may load the
 * library built from this file. The product (bolt_amd/) never links, imports or calls it.
 *
 * Every function cites the reference lines it restates. Plain C, scalar, exact int32
 * (two's-complement wrap) accumulation; fp32 steps are written as separate multiply / add
 * and compiled with -ffp-contract=off so they round exactly like the reference's
 * vmulps / vaddps / vcvtps2dq sequences.
 */
#ifndef BOLT_ORACLE_H
#define BOLT_ORACLE_H
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* output-type selector shared by the GEMM/GEMV oracles (values = Bolt DataType) */
enum { ORC_I32 = 3, ORC_F32 = 6, ORC_U8Q = 10, ORC_I8 = 1 };

/* ---- size queries ------------------------------------------------------------------ */
void orc_mmm_transform_rhs_bytes(uint32_t N, uint32_t K, int packed, uint32_t *bytes, uint32_t *rhsBytes);
uint32_t orc_mmm_tmp_bytes(uint32_t N, uint32_t M, uint32_t K, int transA, int packedB);
uint32_t orc_mvm_transform_weight_bytes(uint32_t N, uint32_t K, int wdt, int packed);

/* ---- weight compensation vector ---------------------------------------------------- */
/* w_is_NK = 1: W stored [N][K]; 0: stored [K][N]. out[n] = -128 * sum_k W[k][n]. */
void orc_offsetC(const int8_t *W, uint32_t K, uint32_t N, int w_is_NK, int32_t *out);

/* ---- GEMM / GEMV ------------------------------------------------------------------- */
void orc_mmm_int8(uint32_t M, uint32_t N, uint32_t K, const uint8_t *A, int transA, const int8_t *W,
    int w_is_NK, const int32_t *offsetC, void *C, int cdt, const float *scale);
void orc_mvm_int8(uint32_t N, uint32_t K, const int8_t *W, int w_is_NK, const uint8_t *x,
    const int32_t *offsetC, void *y, int ydt, const float *scale);
void orc_mvm_u8mat_i8vec(uint32_t M, uint32_t K, const uint8_t *A, int a_is_KM, const int8_t *x, void *y,
    int ydt, const float *scale);

/* ---- quantize / dequantize / requantize ------------------------------------------- */
float orc_symmetric_scale_f32(const float *x, uint32_t n);
void orc_quantize_f32_u8(const float *x, uint32_t n, uint8_t *q, float *scale, int mode);
void orc_quantize_f32_i8(const float *x, uint32_t n, int8_t *q, float *scale, int mode);
void orc_u8_to_i8(const uint8_t *x, uint32_t n, int8_t *q);
void orc_quantize_i32_i8(const int32_t *x, uint32_t n, int8_t *q, float *scale);
void orc_quantize_i32_u8(const int32_t *x, uint32_t n, uint8_t *q, float *scale);
void orc_bias_offsetC(const float *bias, uint32_t N, const int32_t *offsetC, const float *scale, int32_t *out);
void orc_dequantize_i32_f32(const int32_t *q, uint32_t n, const float *scale, float *out);
void orc_dequantize_u8_f32(const uint8_t *q, uint32_t n, const float *scale, float *out);
void orc_requantize_i8(const int8_t *in, uint32_t n, float inScale, int8_t *out, float outScale);

/* ---- per-output-channel epilogue (superset of the reference, closed form) --------- */
void orc_axpby_f32(uint32_t n, float a, const float *x, float b, float *y);
void orc_dequant_per_channel(const int32_t *acc, uint32_t M, uint32_t N, const float *scaleI,
    const float *scaleW, const float *bias, float *out);

/* ---- int8 FullyConnected (x86 branch) ---------------------------------------------- */
void orc_fully_connected_int8(uint32_t M, uint32_t K, uint32_t N, const uint8_t *x, float scaleI,
    const int8_t *W_NK, float scaleW, const float *bias, void *out, int odt, float *scaleO);

/* ---- int8 convolution (x86 direct-conv semantics, any kernel/stride/pad) ---------- */
typedef struct {
    uint32_t n, ic, ih, iw;      /* input  u8, NCHWC8            */
    uint32_t oc, fh, fw;         /* filter s8, NCHW [oc,ic,fh,fw] */
    uint32_t sh, sw, pt, pb, pl, pr, dh, dw;
    uint32_t oh, ow;
    int relu;                    /* ACTIVATION_RELU               */
    int odt;                     /* ORC_I32 / ORC_F32 / ORC_U8Q   */
    int out_c;                   /* channel block of the output layout: 8 or 16 */
} orc_conv_desc;
void orc_conv_int8_acc(const orc_conv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias,
    float scaleI, float scaleF, int32_t *acc /* NCHW-plain [n][oc][oh][ow] */);
void orc_conv_int8(const orc_conv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias,
    const float *eltwise, float *scale /* [in, out, filter] */, void *out);

/* ---- int8 deconvolution (oracle_deconv.c) ---------------------------------------------- */
typedef struct {
    uint32_t n, ic, ih, iw;      /* input u8: in_c = 0 plain NCHW, 8 / 16 = NCHWC8 / NCHWC16 */
    uint32_t oc, fh, fw;         /* filter s8 [ic][oc][fh][fw] */
    uint32_t sh, sw, pt, pb, pl, pr;
    uint32_t oh, ow;
    int in_c;
    int out_c;                   /* channel block of the output layout: 16, or 8 when oc == 8 */
    int relu;
    int odt;                     /* ORC_F32 / ORC_U8Q (ORC_I32: raw sums of the gemm form) */
} orc_deconv_desc;
void orc_deconv_int8(const orc_deconv_desc *d, const uint8_t *in, const int8_t *filter, const float *bias,
    float *scale /* [in, out, filter]; left as the reference leaves the caller's array */, void *out);

/* int8 depthwise convolution, int32 result, no padding (oracle_deconv.c) */
void orc_depthwise_int8_i32(uint32_t n, uint32_t c, uint32_t ih, uint32_t iw, uint32_t fh, uint32_t fw, uint32_t sh,
    uint32_t sw, uint32_t oh, uint32_t ow, const uint8_t *in, const int8_t *filter /* [c][fh][fw] */, const float *bias,
    float *scale /* [in, out, filter] */, int relu, int32_t *out);

/* ---- weight storage of the post-training quantisation tool (oracle_ptq.c) ----------------- */
void orc_ws_convert_int8(const float *w, int n, int8_t *q, float *scale /* in: floor, out: scale used */);
void orc_ws_convert_int4(const float *w, int n /* even */, int8_t *q, float *scale);
float orc_ws_convert_bnn(const float *w, int n /* multiple of 8 */, uint8_t *bits);
void orc_dequantize_int8_weight(int n, float scale, const int8_t *q, float *d);
void orc_dequantize_int4_weight(int n, float scale, const int8_t *q, float *d);
void orc_dequantize_int4_int8(int n, const int8_t *q, int8_t *d);
void orc_dequantize_int4_u8q(int n, const int8_t *q, uint8_t *d);

/* ---- 1-bit convolution ------------------------------------------------------------- */
typedef struct {
    uint32_t n, ic, ih, iw, oc, fh, fw, sh, sw, pt, pb, pl, pr, oh, ow;
    int xnor; /* 1 = DT_BIN11 (+-1, pad bit 0 = -1); 0 = DT_BIN01 ({0,1}, pad 0) */
} orc_bnn_desc;
void orc_bnn_pack_input(const orc_bnn_desc *d, const float *x_nchwc8, uint8_t *bits);
void orc_bnn_conv(const orc_bnn_desc *d, const uint8_t *in_bits, const uint8_t *w_bits_nchwn16c8,
    const float *scale, const float *bias, int32_t *sums_nchwc8, float *out_nchwc8);
void orc_bnn_conv_bruteforce(const orc_bnn_desc *d, const float *x_nchw, const float *w_nchw,
    int32_t *sums_nchw);

/* ---- u8 pooling (NCHWC16) and s8 concatenation ------------------------------------- */
typedef struct {
    uint32_t n, c, ih, iw, oh, ow;
    uint32_t kh, kw, sh, sw, pt, pl;
    int mean;              /* 0 = POOLING_MAX, 1 = POOLING_MEAN */
    int count_include_pad;
} orc_pool_desc;
int orc_pooling_u8_c16(const orc_pool_desc *d, const uint8_t *in, uint8_t *out, float *scale /* [in, out] */);
void orc_concat_i8(uint32_t num, const int8_t *const *in, const uint32_t *len, const float *scales, uint32_t loops,
    int8_t *out, float *oscale);

/* ---- int8 LSTM cell ---------------------------------------------------------------- */
void orc_lstmcell_int8_proj(uint32_t batch, uint32_t xdim, uint32_t hdim, uint32_t column, const float *x, uint32_t x_stride,
    const int8_t *W, const float *Wp, const float *bias, uint32_t bias_stride, const float *scale, float *state,
    float forget_bias, float zoneout_cell, float zoneout_output, float *out, uint32_t out_stride);
void orc_lstmcell_int8(uint32_t batch, uint32_t xdim, uint32_t hdim, const float *x, uint32_t x_stride,
    const int8_t *W, const float *bias, uint32_t bias_stride, const float *scale, float *state, float forget_bias,
    float zoneout_cell, float zoneout_output, float *out, uint32_t out_stride);

#ifdef __cplusplus
}
#endif
#endif
