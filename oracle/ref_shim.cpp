// TEST INFRASTRUCTURE ONLY. Flat C entry points over the reference's own x86 AVX-512-VNNI
// objects, compiled where they lie under /root/reference by oracle/Makefile into
// oracle/_ref/libboltref.so. Used (a) to write the golden vectors under tests/golden/ and
// to pin oracle/oracle.c against the real reference, and (b) as the "reference" CPU
// baseline in bench.py when the host CPU has avx512_vnni. Nothing in the product path may
// load this file's output.
//
// Each wrapper builds the TensorDesc arguments exactly as the reference's own unit tests do
// (compute/blas_enhance/tests/test_mmm.cpp:30-90, test_mvm.cpp:30-90) and forwards to the
// public function; no arithmetic happens here.
#include <omp.h>
#include <cstdint>
#include <cstring>
#include "blas_enhance.h"
#include "tensor_desc.h"
#include "parameter_spec.h"
#include "cpu/x86/int8/tensor_computing_int8.h"
#include "cpu/tensor_computing_cpu.h"
#include <vector>

// internal (non-public) reference prototypes, compute/tensor/src/cpu/x86/tensor_computing_x86.h
EE quantize_x86(TensorDesc dDesc, const void *data, TensorDesc *qDesc, void *qData, F32 *scale, int mode);
EE dequantize_x86(TensorDesc qDesc, void *qData, const F32 *scale, TensorDesc bDesc, void *bData,
    TensorDesc dDesc, void *dData);
EE quantize_bias_offsetC(const void *bias, TensorDesc biasDesc, DataType qType, const void *filter,
    TensorDesc filterDesc, const F32 *scale, void *offsetCBias);
EE requantize_cpu(TensorDesc inputDesc, INT8 *input, F32 inputScale, TensorDesc outputDesc,
    INT8 *output, F32 outputScale, Arch arch);

extern int OMP_NUM_THREADS;

// bfmt: 0 = DF_NORMAL [K,N], 1 = DF_TRANSPOSE [N,K], 2 = packed DF_NKNxKx (logical [K,N])
static TensorDesc rhs_desc(int bfmt, U32 K, U32 N)
{
    if (bfmt == 0) {
        return tensor2df(DT_I8, DF_NORMAL, K, N);
    }
    if (bfmt == 1) {
        return tensor2df(DT_I8, DF_TRANSPOSE, N, K);
    }
    return tensor2df(DT_I8, DF_NKNxKx, K, N);
}

// wfmt: 0 = DF_NORMAL [N,K], 1 = DF_TRANSPOSE [K,N], 2 = packed DF_NKN32K4 (logical [N,K])
static TensorDesc mvm_desc(int wfmt, U32 N, U32 K, DataType dt)
{
    if (wfmt == 0) {
        return tensor2df(dt, DF_NORMAL, N, K);
    }
    if (wfmt == 1) {
        return tensor2df(dt, DF_TRANSPOSE, K, N);
    }
    return tensor2df(dt, matrix_vector_multiply_weight_format(dt), N, K);
}

extern "C" {

void ref_set_threads(int n)
{
    OMP_NUM_THREADS = n;
}

// y = a * x + b * y, fp32 (compute/blas_enhance/src/axpby.cpp:24-60)
int ref_axpby_f32(U32 n, float a, const float *x, float b, float *y)
{
    return vector_vector_axpby(a, tensor1d(DT_F32, n), x, b, tensor1d(DT_F32, n), y, X86_AVX512);
}

int ref_mmm_transform_rhs_bytes(int bfmt, U32 K, U32 N, U32 *bytes, U32 *rhsBytes)
{
    return matrix_matrix_multiply_transform_rhs_bytes(rhs_desc(bfmt, K, N), bytes, rhsBytes, X86_AVX512);
}

// out_desc: {df, nDims, dims[0], dims[1]} of the transformed descriptor
int ref_mmm_transform_rhs(int bfmt, U32 K, U32 N, const void *src, void *dst, U32 *out_desc)
{
    TensorDesc t;
    memset(&t, 0xff, sizeof(t));
    EE e = matrix_matrix_multiply_transform_rhs(rhs_desc(bfmt, K, N), src, &t, dst, X86_AVX512);
    out_desc[0] = t.df;
    out_desc[1] = t.nDims;
    out_desc[2] = t.dims[0];
    out_desc[3] = t.dims[1];
    return e;
}

int ref_mmm_tmp_bytes(int transA, int bfmt, U32 M, U32 K, U32 N, U32 *bytes)
{
    TensorDesc a = transA ? tensor2df(DT_U8_Q, DF_TRANSPOSE, K, M) : tensor2df(DT_U8_Q, DF_NORMAL, M, K);
    return matrix_matrix_multiply_tmp_bytes(a, rhs_desc(bfmt, K, N), bytes, X86_AVX512);
}

// cdt: DataType of C (DT_I32 / DT_F32 / DT_U8_Q)
int ref_mmm(int transA, int bfmt, U32 M, U32 K, U32 N, const void *A, const void *B, U32 tmpBytes,
    void *tmp, int cdt, void *C, const float *scale)
{
    TensorDesc a = transA ? tensor2df(DT_U8_Q, DF_TRANSPOSE, K, M) : tensor2df(DT_U8_Q, DF_NORMAL, M, K);
    TensorDesc c = tensor2df((DataType)cdt, DF_NORMAL, M, N);
    return matrix_matrix_multiply(a, A, rhs_desc(bfmt, K, N), B, tmpBytes, tmp, c, C, scale, X86_AVX512);
}

int ref_mvm_transform_weight_bytes(int wfmt, int wdt, U32 N, U32 K, U32 *bytes)
{
    return matrix_vector_multiply_transform_weight_bytes(mvm_desc(wfmt, N, K, (DataType)wdt), bytes, X86_AVX512);
}

int ref_mvm_transform_weight(int wfmt, U32 N, U32 K, const void *src, void *dst, U32 *out_desc)
{
    TensorDesc t;
    memset(&t, 0xff, sizeof(t));
    EE e = matrix_vector_multiply_transform_weight(mvm_desc(wfmt, N, K, DT_I8), src, &t, dst, X86_AVX512);
    out_desc[0] = t.df;
    out_desc[1] = t.nDims;
    out_desc[2] = t.dims[0];
    out_desc[3] = t.dims[1];
    return e;
}

int ref_mvm_tmp_bytes(int wfmt, int wdt, U32 N, U32 K, U32 *bytes)
{
    DataType vdt = ((DataType)wdt == DT_I8) ? DT_U8_Q : DT_I8;
    return matrix_vector_multiply_tmp_bytes(mvm_desc(wfmt, N, K, (DataType)wdt), tensor1d(vdt, K), bytes, X86_AVX512);
}

// wdt = DT_I8: s8 matrix x u8 vector; wdt = DT_U8_Q: u8 matrix (DF_NORMAL [N,K]) x s8 vector
int ref_mvm(int wfmt, int wdt, U32 N, U32 K, const void *W, const void *x, U32 tmpBytes, void *tmp,
    int rdt, void *y, const float *scale)
{
    DataType vdt = ((DataType)wdt == DT_I8) ? DT_U8_Q : DT_I8;
    return matrix_vector_multiply(mvm_desc(wfmt, N, K, (DataType)wdt), W, tensor1d(vdt, K), x, tmpBytes,
        tmp, tensor1d((DataType)rdt, N), y, scale, X86_AVX512);
}

int ref_quantize(int ddt, const void *data, U32 n, int qdt, void *q, float *scale, int mode)
{
    TensorDesc d = tensor1d((DataType)ddt, n);
    TensorDesc qd = tensor1d((DataType)qdt, n);
    return quantize_x86(d, data, &qd, q, scale, mode);
}

int ref_dequantize(int qdt, void *q, U32 n, const float *scale, float *out)
{
    TensorDesc qd = tensor1d((DataType)qdt, n);
    TensorDesc dd = tensor1d(DT_F32, n);
    TensorDesc bd = tensor1d(DT_F32, 0);
    return dequantize_x86(qd, q, scale, bd, nullptr, dd, out);
}

// packed_filter = 1: `offsetC` holds the compensation vector of a packed weight blob and is
// added; 0: native-format filter, the vector is not added (avx512/quantize.cpp:244,259-262).
int ref_quantize_bias_offsetC(const float *bias, U32 N, const int32_t *offsetC, int packed_filter,
    const float *scale, int32_t *out)
{
    TensorDesc bd = tensor1d(DT_F32, N);
    TensorDesc fd = tensor2df(DT_I8, packed_filter ? DF_NKNxKx : DF_NORMAL, N, N);
    return quantize_bias_offsetC(bias, bd, DT_I32, offsetC, fd, scale, out);
}

int ref_requantize(const int8_t *in, U32 n, float inScale, int8_t *out, float outScale)
{
    TensorDesc d = tensor1d(DT_I8, n);
    return requantize_cpu(d, (INT8 *)in, inScale, d, out, outScale, X86_AVX512);
}

// int8 convolution through the reference's own sequence (compute/tensor/tests/test_convolution_int8.cpp:59-161):
// transform_filter -> tmp bytes -> convolution_int8. Input u8 (DT_U8_Q) in `idf` (DF_NCHWC8 = 2 or
// DF_NCHWC16 = 41), filter s8 NCHW, fp32 bias, optional fp32 eltwise input laid out like the output.
// alg: 1 = CONVOLUTION_ALGORITHM_DIRECT, 0 = POINTWISE. scale[3] = {input, output (in/out), filter}.
// odt: DT_F32 or DT_U8_Q; output layout is what the reference writes (NCHWC16, tail block C8).
int ref_conv_int8(U32 n, U32 ic, U32 ih, U32 iw, int idf, U32 oc, U32 fh, U32 fw, U32 sh, U32 sw, U32 pt, U32 pb,
    U32 pl, U32 pr, U32 dh, U32 dw, U32 oh, U32 ow, int alg, const uint8_t *in, const int8_t *filter, const float *bias,
    const float *eltwise, float *scale, int relu, int odt, void *out)
{
    ConvolutionParamSpec p = createConvolutionParamSpec(
        1, 1, fh, fw, 1, sh, sw, 0, 0, pt, pb, pl, pr, 1, dh, dw, oc, CONVOLUTION_DEPTHWISE_POINTWISE);
    ConvolutionForwardAlgorithm a = (ConvolutionForwardAlgorithm)alg;
    TensorDesc inputDesc = tensor4df(DT_U8_Q, (DataFormat)idf, n, ic, ih, iw);
    TensorDesc filterDesc = tensor4df(DT_I8, DF_NCHW, oc, ic, fh, fw);
    TensorDesc biasDesc = tensor1d(DT_F32, oc);
    TensorDesc outputDesc = tensor4df((DataType)odt, DF_NCHWC16, n, oc, oh, ow);
    U32 fcPad = (ic + 15) / 16 * 16;
    U32 ftmBytes = oc * fcPad * fh * fw + oc * 4 + 32;  // cpu/x86/convolution.cpp:105-170
    INT8 *ftm = (INT8 *)calloc(ftmBytes + 64, 1);
    TensorDesc ftmDesc;
    EE e = convolution_transform_filter_int8(filterDesc, filter, p, a, &ftmDesc, ftm);
    if (e != SUCCESS) {
        free(ftm);
        return 1000 + e;
    }
    U32 tmpBytes = 0;
    e = convolution_infer_forward_tmp_bytes_int8(inputDesc, ftmDesc, outputDesc, p, a, &tmpBytes);
    if (e != SUCCESS) {
        free(ftm);
        return 2000 + e;
    }
    void *tmp = calloc((size_t)tmpBytes + n * oc * oh * ow * 4 + 4096, 1);
    ActivationParamSpec act;
    act.mode = relu ? ACTIVATION_RELU : ACTIVATION_NULL;
    e = convolution_int8(inputDesc, (UINT8 *)in, (F32 *)eltwise, ftmDesc, ftm, p, a, biasDesc, bias, tmpBytes, tmp,
        outputDesc, out, scale, act, X86_AVX512);
    free(tmp);
    free(ftm);
    return e;
}

// The same convolution timed for a CPU baseline: filter transform and buffers once, then `reps` calls of
// convolution_int8 between two clock readings (scale[1] is reset to -1 before each call: dynamic output scale).
// *seconds receives the time of the calls alone.
int ref_conv_int8_loop(U32 n, U32 ic, U32 ih, U32 iw, int idf, U32 oc, U32 fh, U32 fw, U32 sh, U32 sw, U32 pt, U32 pb,
    U32 pl, U32 pr, U32 oh, U32 ow, int alg, const uint8_t *in, const int8_t *filter, const float *bias, float *scale,
    int relu, int odt, void *out, int reps, double *seconds)
{
    ConvolutionParamSpec p = createConvolutionParamSpec(
        1, 1, fh, fw, 1, sh, sw, 0, 0, pt, pb, pl, pr, 1, 1, 1, oc, CONVOLUTION_DEPTHWISE_POINTWISE);
    ConvolutionForwardAlgorithm a = (ConvolutionForwardAlgorithm)alg;
    TensorDesc inputDesc = tensor4df(DT_U8_Q, (DataFormat)idf, n, ic, ih, iw);
    TensorDesc filterDesc = tensor4df(DT_I8, DF_NCHW, oc, ic, fh, fw);
    TensorDesc biasDesc = tensor1d(DT_F32, oc);
    TensorDesc outputDesc = tensor4df((DataType)odt, DF_NCHWC16, n, oc, oh, ow);
    U32 fcPad = (ic + 15) / 16 * 16;
    U32 ftmBytes = oc * fcPad * fh * fw + oc * 4 + 32;
    INT8 *ftm = (INT8 *)calloc(ftmBytes + 64, 1);
    TensorDesc ftmDesc;
    EE e = convolution_transform_filter_int8(filterDesc, filter, p, a, &ftmDesc, ftm);
    U32 tmpBytes = 0;
    if (e == SUCCESS) {
        e = convolution_infer_forward_tmp_bytes_int8(inputDesc, ftmDesc, outputDesc, p, a, &tmpBytes);
    }
    if (e != SUCCESS) {
        free(ftm);
        return 1000 + e;
    }
    void *tmp = calloc((size_t)tmpBytes + (size_t)n * oc * oh * ow * 4 + 4096, 1);
    ActivationParamSpec act;
    act.mode = relu ? ACTIVATION_RELU : ACTIVATION_NULL;
    const float sI = scale[0], sF = scale[2];
    const double t0 = omp_get_wtime();
    for (int r = 0; r < reps && e == SUCCESS; ++r) {
        scale[0] = sI;
        scale[1] = -1;
        scale[2] = sF;
        e = convolution_int8(inputDesc, (UINT8 *)in, nullptr, ftmDesc, ftm, p, a, biasDesc, bias, tmpBytes, tmp, outputDesc, out,
            scale, act, X86_AVX512);
    }
    *seconds = omp_get_wtime() - t0;
    free(tmp);
    free(ftm);
    return e;
}

// u8 pooling on NCHWC16 (compute/tensor/src/cpu/x86/int8/avx512/pooling_int8.cpp:316). scale[2] = {in, out}.
int ref_pooling_u8(U32 n, U32 c, U32 ih, U32 iw, U32 oh, U32 ow, U32 kh, U32 kw, U32 sh, U32 sw, U32 pt, U32 pl,
    int mean, int count_include_pad, const uint8_t *in, uint8_t *out, float *scale)
{
    PoolingParamSpec p;
    memset(&p, 0, sizeof(p));
    p.kernel_t = 1;
    p.kernel_h = kh;
    p.kernel_w = kw;
    p.stride_t = 1;
    p.stride_h = sh;
    p.stride_w = sw;
    p.pad_top = pt;
    p.pad_left = pl;
    p.mode = mean ? POOLING_MEAN : POOLING_MAX;
    p.count_include_pad = count_include_pad != 0;
    TensorDesc inputDesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, ih, iw);
    TensorDesc outputDesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, oh, ow);
    return pooling_uint8(inputDesc, in, p, outputDesc, out, scale);
}

// s8 concatenation with a common scale (compute/tensor/src/cpu/concat.cpp:164). Inputs are 4-D tensors in `df`
// that differ in dims[axis_from_outermost]; they are rescaled in place by the reference, so pass copies.
int ref_concat_i8(U32 num, const U32 *dims4 /* num x {n,c,h,w} */, int df, int axis, int8_t **in, float *scales,
    const U32 *odims4, int8_t *out, float *oscale)
{
    std::vector<TensorDesc> descs;
    std::vector<void *> ptrs;
    for (U32 j = 0; j < num; ++j) {
        descs.push_back(tensor4df(DT_I8, (DataFormat)df, dims4[4 * j], dims4[4 * j + 1], dims4[4 * j + 2],
            dims4[4 * j + 3]));
        ptrs.push_back(in[j]);
    }
    TensorDesc od = tensor4df(DT_I8, (DataFormat)df, odims4[0], odims4[1], odims4[2], odims4[3]);
    ConcatParamSpec p;
    p.axis = axis;
    p.num_concat = (I32)num;
    return concat_cpu(descs, ptrs, scales, p, nullptr, od, out, oscale, X86_AVX512);
}

// int8 LSTM cell (compute/tensor/src/cpu/x86/int8/lstm.cpp:20). W: s8 [4*hdim][xdim+hdim] row-major, packed here
// with the reference's own matrix_vector_multiply_transform_weight. state rows [C | H]; scale = {activation, weight}.
// column = hdim and Wp = nullptr: no projection; else column = num_projection, W is [4 * column][K] and Wp the fp32
// projection matrix in the DF_NKN32 layout the cell reads it in, [hdim / 32][column][32] (lstm.cpp:170-173)
int ref_lstmcell_int8_proj(U32 batch, U32 xdim, U32 hdim, U32 column, const float *x, U32 x_stride, const int8_t *W,
    const float *Wp, const float *bias, float *scale, float *state, float forget_bias, float zoneout_cell,
    float zoneout_output, float *out, U32 out_stride)
{
    const U32 N = 4 * column, K = xdim + hdim;
    TensorDesc wDesc = tensor2df(DT_I8, DF_NORMAL, N, K);
    U32 bytes = 0;
    EE e = matrix_vector_multiply_transform_weight_bytes(wDesc, &bytes, X86_AVX512);
    if (e != SUCCESS) {
        return 1000 + e;
    }
    INT8 *blob = (INT8 *)calloc((size_t)bytes + 64, 1);
    TensorDesc tDesc;
    e = matrix_vector_multiply_transform_weight(wDesc, W, &tDesc, blob, X86_AVX512);
    if (e != SUCCESS) {
        free(blob);
        return 2000 + e;
    }
    RNNParamSpec p;
    memset(&p, 0, sizeof(p));
    p.mode = RNN_LSTM;
    p.num_outputs = hdim;
    p.steps = -1;
    p.num_projection = Wp ? column : 0;
    p.zoneout_cell = zoneout_cell;
    p.zoneout_output = zoneout_output;
    p.bi_direction = false;
    p.forget_bias = forget_bias;
    p.activation_type = ACTIVATION_TANH;
    TensorDesc xDesc = tensor2df(DT_F32, DF_NORMAL, batch, xdim);
    TensorDesc hDesc = tensor2df(DT_F32, DF_NORMAL, batch, hdim);
    TensorDesc fDesc = tensor2df(DT_I8, DF_NKN32, N, K);
    TensorDesc bDesc = tensor1d(DT_F32, N);
    const void *filters[2] = {blob, Wp};
    const void *biases[2] = {bias, nullptr};
    U32 tmpBytes = (K + N) * 4 + K + 256;
    void *tmp = calloc(tmpBytes, 1);
    // out_stride doubles as batchStrideH, so the reference reads bias row m at m * (out_stride / hdim) * N
    e = lstmcell_int8(xDesc, x, &fDesc, filters, &bDesc, biases, scale, state, tmpBytes, tmp, p, x_stride, out_stride,
        hDesc, out, X86_AVX512);
    free(tmp);
    free(blob);
    return e;
}

int ref_lstmcell_int8(U32 batch, U32 xdim, U32 hdim, const float *x, U32 x_stride, const int8_t *W, const float *bias,
    float *scale, float *state, float forget_bias, float zoneout_cell, float zoneout_output, float *out, U32 out_stride)
{
    return ref_lstmcell_int8_proj(batch, xdim, hdim, hdim, x, x_stride, W, nullptr, bias, scale, state, forget_bias,
        zoneout_cell, zoneout_output, out, out_stride);
}

}  // extern "C"
