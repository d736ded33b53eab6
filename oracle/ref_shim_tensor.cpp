// TEST INFRASTRUCTURE ONLY. Flat C entry points over the reference's Tensor-level operators
// (compute/tensor/src/{fully_connected,matmul,convolution}.cpp) and over the fp32 neighbours of an
// encoder layer (compute/tensor/src/cpu/x86/fp32/{layer_norm,softmax}.cpp, x86_functions_fp32.h),
// compiled where they lie under /root/reference by oracle/Makefile into oracle/_ref/libboltref.so.
// They pin the ORCHESTRATION rows (tmp layout, scale plumbing, which BLAS route runs) and the size /
// format queries of the convolution, and write golden vectors. Nothing in the product may load this.
//
// Tensors are built the way the reference's own tests and engine build them
// (compute/tensor/tests/test_convolution_int8.cpp:59-161,
// inference/engine/include/cpu/fully_connected_cpu.hpp:192-252); no arithmetic happens here.
#include <cstdint>
#include <cstring>
#include <vector>
#include "tensor_computing.h"
#include "blas_enhance.h"
#include "cpu/x86/fp32/tensor_computing_fp32.h"
#include "cpu/x86/int8/tensor_computing_int8.h"
#include "cpu/x86/fp32/x86_functions_fp32.h"

static ArchInfo g_arch = {X86_AVX512, nullptr};

static Tensor make(TensorDesc d, const void *src)
{
    Tensor t = Tensor::alloc_sized<CPUMem>(d);
    if (src) {
        memcpy(get_ptr_from_tensor(t, CPU_GENERAL), src, tensorNumBytes(d));
    }
    return t;
}

static void put_desc(TensorDesc d, U32 *out)  // {dt, df, nDims, dims[0..5]}
{
    out[0] = d.dt;
    out[1] = d.df;
    out[2] = d.nDims;
    for (U32 i = 0; i < 6; ++i) {
        out[3 + i] = i < d.nDims ? d.dims[i] : 0;
    }
}

extern "C" {

// int8 FullyConnected exactly as the engine runs it: weight s8 [N, K] packed with
// matrix_vector_multiply_transform_weight (mvm != 0) or matrix_matrix_multiply_transform_rhs
// (fully_connected_cpu.hpp:231-248), then fully_connected_infer_forward_tmp_bytes and fully_connected().
// x: u8 [M, K] with scale scaleI. odt: DT_F32 / DT_U8_Q / DT_I32 ... scaleO_io: in = the output tensor's scale
// before the call (<= 0: unknown), out = its scale after the call. Returns the EE code.
int ref_fc_tensor(U32 M, U32 K, U32 N, const uint8_t *x, float scaleI, const int8_t *W_NK, float scaleW,
    const float *bias, int mvm, int odt, void *out, float *scaleO_io, U32 *tmpBytesOut)
{
    TensorDesc fDesc = tensor2df(DT_I8, mvm ? DF_NORMAL : DF_TRANSPOSE, N, K);
    U32 tBytes = 0;
    TensorDesc tDesc;
    Tensor wtm;
    if (mvm) {
        EE e = matrix_vector_multiply_transform_weight_bytes(fDesc, &tBytes, X86_AVX512);
        if (e != SUCCESS) {
            return 1000 + e;
        }
        wtm = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, tBytes));
        e = matrix_vector_multiply_transform_weight(fDesc, W_NK, &tDesc, get_ptr_from_tensor(wtm, CPU_GENERAL), X86_AVX512);
        if (e != SUCCESS) {
            return 1100 + e;
        }
    } else {
        EE e = matrix_matrix_multiply_transform_rhs_bytes(fDesc, &tBytes, nullptr, X86_AVX512);
        if (e != SUCCESS) {
            return 1200 + e;
        }
        wtm = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, tBytes));
        e = matrix_matrix_multiply_transform_rhs(fDesc, W_NK, &tDesc, get_ptr_from_tensor(wtm, CPU_GENERAL), X86_AVX512);
        if (e != SUCCESS) {
            return 1300 + e;
        }
    }
    wtm.resize(tDesc);
    wtm.set_scale(scaleW);
    Tensor in = make(tensor2df(DT_U8_Q, DF_NORMAL, M, K), x);
    in.set_scale(scaleI);
    Tensor b;
    if (bias) {
        b = make(tensor1d(DT_F32, N), bias);
    }
    Tensor o = Tensor::alloc_sized<CPUMem>(tensor2df((DataType)odt, DF_NORMAL, M, N));
    o.set_scale(*scaleO_io);
    U32 bytes = 0;
    EE e = fully_connected_infer_forward_tmp_bytes(in, wtm, o, &bytes, &g_arch);
    if (e != SUCCESS) {
        return 2000 + e;
    }
    if (tmpBytesOut) {
        *tmpBytesOut = bytes;
    }
    Tensor tmp = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, bytes + 64));
    memset(get_ptr_from_tensor(tmp, CPU_GENERAL), 0xa5, bytes + 64);
    std::vector<Tensor> tmps(1, tmp);
    e = fully_connected(in, wtm, b, tmps, o, &g_arch);
    memcpy(out, get_ptr_from_tensor(o, CPU_GENERAL), tensorNumBytes(o.get_desc()));
    *scaleO_io = o.get_scale();
    return e;
}

// matmul() on fp32 or pre-quantised operands (compute/tensor/src/matmul.cpp:302-576). Shapes are given outermost
// first (na / nb / nc entries), as DF_NCHW tensors like the engine's MatMul operands. adt / bdt: DT_F32, DT_U8_Q,
// DT_I8; cdt: DT_F32. scaleA / scaleB: the operand tensors' scales (ignored by the reference for fp32 operands
// unless positive: quantize_cpu treats them as lower bounds).
int ref_matmul_tensor(int adt, const U32 *ashape, U32 na, int transposeA, const void *A, float scaleA, int bdt,
    const U32 *bshape, U32 nb, int transposeB, const void *B, float scaleB, int cdt, const U32 *cshape, U32 nc,
    void *C, U32 *tmpBytesOut)
{
    auto desc = [](int dt, const U32 *shape, U32 n) {
        TensorDesc d;
        d.dt = (DataType)dt;
        d.df = DF_NCHW;
        d.nDims = n;
        for (U32 i = 0; i < n; ++i) {
            d.dims[i] = shape[n - 1 - i];
        }
        return d;
    };
    Tensor a = make(desc(adt, ashape, na), A), b = make(desc(bdt, bshape, nb), B);
    a.set_scale(scaleA);
    b.set_scale(scaleB);
    Tensor c = Tensor::alloc_sized<CPUMem>(desc(cdt, cshape, nc));
    c.set_scale(-1);
    U32 bytes = 0;
    EE e = matmul_infer_forward_tmp_bytes(a, transposeA != 0, b, transposeB != 0, c, &bytes, &g_arch);
    if (e != SUCCESS) {
        return 2000 + e;
    }
    if (tmpBytesOut) {
        *tmpBytesOut = bytes;
    }
    Tensor tmp = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, bytes + 64));
    std::vector<Tensor> tmps(1, tmp);
    Tensor bias;
    e = matmul(a, transposeA != 0, b, transposeB != 0, bias, tmps, c, &g_arch);
    memcpy(C, get_ptr_from_tensor(c, CPU_GENERAL), tensorNumBytes(c.get_desc()));
    return e;
}

// The convolution's query functions through the public Tensor API (compute/tensor/src/convolution.cpp:28-317):
// output desc for a u8 input (targetDataType = DT_U8_Q), forward algorithm, transformed-filter bytes and desc,
// tmp bytes. q[0..8] = output desc, q[9] = algorithm, q[10] = filter bytes, q[11..19] = ftm desc, q[20] = tmp bytes.
int ref_conv_queries(U32 n, U32 ic, U32 ih, U32 iw, int idf, U32 oc, U32 fh, U32 fw, U32 sh, U32 sw, U32 pt, U32 pb,
    U32 pl, U32 pr, U32 dh, U32 dw, int relu, U32 *q)
{
    ConvolutionParamSpec p = createConvolutionParamSpec(
        1, 1, fh, fw, 1, sh, sw, 0, 0, pt, pb, pl, pr, 1, dh, dw, oc, CONVOLUTION_DEPTHWISE_POINTWISE);
    Tensor in, filter, out;
    in.resize(tensor4df(DT_U8_Q, (DataFormat)idf, n, ic, ih, iw));
    TensorDesc fd = tensor4df(DT_I8, DF_NCHW, oc, ic, fh, fw);
    filter = Tensor::alloc_sized<CPUMem>(fd);
    memset(get_ptr_from_tensor(filter, CPU_GENERAL), 1, tensorNumBytes(fd));
    EE e = convolution_infer_output_size(&in, filter, p, &out, DT_U8_Q, &g_arch);
    if (e != SUCCESS) {
        return 1000 + e;
    }
    put_desc(out.get_desc(), q);
    ActivationParamSpec act;
    act.mode = relu ? ACTIVATION_RELU : ACTIVATION_NULL;
    ConvolutionForwardAlgorithm alg = CONVOLUTION_ALGORITHM_NULL;
    e = convolution_infer_forward_algorithm(in, filter, out, p, CONVOLUTION_FASTEST, &alg, DT_U8_Q, act, &g_arch);
    if (e != SUCCESS) {
        return 2000 + e;
    }
    q[9] = alg;
    U32 fb = 0;
    e = convolution_transform_filter_bytes(filter, p, alg, &fb, &g_arch);
    if (e != SUCCESS) {
        return 3000 + e;
    }
    q[10] = fb;
    Tensor ftm = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, fb + 64)), tmp;
    e = convolution_transform_filter(filter, p, alg, tmp, &ftm, &g_arch);
    if (e != SUCCESS) {
        return 4000 + e;
    }
    put_desc(ftm.get_desc(), q + 11);
    U32 tb = 0;
    e = convolution_infer_forward_tmp_bytes(in, ftm, out, p, alg, &tb, &g_arch);
    if (e != SUCCESS) {
        return 5000 + e;
    }
    q[20] = tb;
    return 0;
}

// int8 deconvolution through the public Tensor API in the engine's order (inference/engine/include/cpu/deconvolution_cpu.hpp:
// infer_output_size -> infer_forward_algorithm -> transform_filter_bytes -> transform_filter -> infer_forward_tmp_bytes ->
// deconvolution). Input u8 (DT_U8_Q) in `idf` (DF_NCHW = 0 -> IM2COL_GEMM, DF_NCHWC8 = 2 / DF_NCHWC16 = 41 -> POINTWISE),
// filter s8 [ic][oc][fh][fw], fp32 bias [oc]. scale[3] = {input, output (in/out), filter} is the caller's array and comes
// back as the reference leaves it. q[0..8] = output desc, q[9] = algorithm, q[10] = filter bytes, q[11..19] = ftm desc,
// q[20] = tmp bytes. `out` must hold n * oc * oh * ow elements of odt.
int ref_deconv_int8(U32 n, U32 ic, U32 ih, U32 iw, int idf, U32 oc, U32 fh, U32 fw, U32 sh, U32 sw, U32 pt, U32 pb, U32 pl,
    U32 pr, const uint8_t *in, const int8_t *filter, const float *bias, float *scale, int relu, int odt, void *out, U32 *q)
{
    ConvolutionParamSpec p = createConvolutionParamSpec(
        1, 1, fh, fw, 1, sh, sw, 0, 0, pt, pb, pl, pr, 1, 1, 1, oc, CONVOLUTION_DECONVOLUTION);
    TensorDesc id = tensor4df(DT_U8_Q, (DataFormat)idf, n, ic, ih, iw);
    Tensor input = make(id, in);
    TensorDesc fd = tensor4df(DT_I8, DF_NCHW, ic, oc, fh, fw);
    Tensor filt = make(fd, filter);
    Tensor output;
    EE e = deconvolution_infer_output_size(&input, filt, p, &output, (DataType)odt, &g_arch);
    if (e != SUCCESS) {
        return 1000 + e;
    }
    put_desc(output.get_desc(), q);
    ActivationParamSpec act;
    act.mode = relu ? ACTIVATION_RELU : ACTIVATION_NULL;
    ConvolutionForwardAlgorithm alg = CONVOLUTION_ALGORITHM_NULL;
    e = deconvolution_infer_forward_algorithm(input, filt, output, p, CONVOLUTION_FASTEST, &alg, (DataType)odt, act, &g_arch);
    if (e != SUCCESS) {
        return 2000 + e;
    }
    q[9] = alg;
    U32 fb = 0;
    e = deconvolution_transform_filter_bytes(filt, p, alg, &fb, &g_arch);
    if (e != SUCCESS) {
        return 3000 + e;
    }
    q[10] = fb;
    Tensor ftm = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, fb + 64)), none;
    e = deconvolution_transform_filter(filt, p, alg, none, &ftm, &g_arch);
    if (e != SUCCESS) {
        return 4000 + e;
    }
    put_desc(ftm.get_desc(), q + 11);
    U32 tb = 0;
    e = deconvolution_infer_forward_tmp_bytes(input, ftm, output, p, alg, &tb, &g_arch);
    if (e != SUCCESS) {
        return 5000 + e;
    }
    q[20] = tb;
    // The POINTWISE route runs a 1x1 convolution inside whose own tmp needs (the int32 results ahead of its
    // requantisation, x86/int8/convolution.cpp:40-93) are not part of deconvolution_infer_forward_tmp_bytes
    // (cpu/deconvolution.cpp:195-222); the engine hides that by sizing one tmp as the maximum over all operators.
    // Here the buffer gets that much slack so the reference does not write past it.
    const size_t slack = (size_t)n * ih * iw * oc * fh * fw * 8 + (1u << 20);
    Tensor tmp = Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, tb + slack));
    memset(get_ptr_from_tensor(tmp, CPU_GENERAL), 0, tb + slack);
    Tensor biasT = make(tensor1d(DT_F32, oc), bias);
    output.alloc();
    e = deconvolution(input, ftm, p, alg, scale, biasT, tmp, output, act, &g_arch);
    if (e != SUCCESS) {
        return 6000 + e;
    }
    memcpy(out, get_ptr_from_tensor(output, CPU_GENERAL), tensorNumBytes(output.get_desc()));
    return 0;
}

// int8 depthwise convolution, inner form (compute/tensor/src/cpu/x86/int8/avx512/depthwise_convolution_direct.cpp:441-599)
// with no pointwise stage: depthwise_convolution_transform_filter_int8 then depthwise_pointwise_convolution_int8.
// Input u8 NCHWC16, filter s8 [1][c][fh][fw] (DF_NCHW), fp32 bias [c]; odt DT_I32 or DT_F32; output NCHWC16.
// The public depthwise_convolution() route hands this function a null scale array (cpu/x86/depthwise_convolution.cpp:
// 107-113), which it dereferences; so it is only callable directly.
int ref_depthwise_int8(U32 n, U32 c, U32 ih, U32 iw, U32 fh, U32 fw, U32 sh, U32 sw, U32 pt, U32 pb, U32 pl, U32 pr, U32 oh,
    U32 ow, const uint8_t *in, const int8_t *filter, const float *bias, float *scale, int relu, int odt, void *out)
{
    ConvolutionParamSpec p = createConvolutionParamSpec(
        c, 1, fh, fw, 1, sh, sw, 0, 0, pt, pb, pl, pr, c, 1, 1, c, CONVOLUTION_DEPTHWISE);
    TensorDesc id = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, ih, iw);
    TensorDesc fd = tensor4df(DT_I8, DF_NCHW, 1, c, fh, fw);
    TensorDesc od = tensor4df((DataType)odt, DF_NCHWC16, n, c, oh, ow);
    U32 fsz = (fh * fw + 3) / 4 * 4;
    std::vector<INT8> ftm((size_t)fsz * c + c * 4 + 4096, 0);
    TensorDesc ftmDesc;
    EE e = depthwise_convolution_transform_filter_int8(fd, filter, &ftmDesc, ftm.data());
    if (e != SUCCESS) {
        return 1000 + e;
    }
    std::vector<uint8_t> tmp((size_t)n * c * oh * ow * 4 + (size_t)c * 4 + (size_t)fsz * 16 * 16 + (1u << 20), 0);
    ActivationParamSpec act, none;
    act.mode = relu ? ACTIVATION_RELU : ACTIVATION_NULL;
    none.mode = ACTIVATION_NULL;
    TensorDesc blank;
    e = depthwise_pointwise_convolution_int8(id, (UINT8 *)in, nullptr, ftmDesc, ftm.data(), blank, nullptr, p,
        tensor1d(DT_F32, c), bias, blank, nullptr, (U32)tmp.size(), tmp.data(), od, out, scale, act, none);
    return e;
}

// The reference's transformed depthwise filter (x86/int8/depthwise_convolution_transform.cpp:17-69): blob must hold
// ALIGN(fh * fw, 4) * c + c * 4 bytes; desc9 = its desc.
int ref_depthwise_transform_filter(U32 c, U32 fh, U32 fw, const int8_t *filter, int8_t *blob, U32 *desc9)
{
    TensorDesc fd = tensor4df(DT_I8, DF_NCHW, 1, c, fh, fw), ftm;
    EE e = depthwise_convolution_transform_filter_int8(fd, filter, &ftm, blob);
    put_desc(ftm, desc9);
    return e;
}

// fp32 neighbours of the int8 GEMMs inside an encoder layer
int ref_layer_norm_f32(U32 rows, U32 H, const float *in, const float *gamma, const float *beta, float *out)
{
    LayerNormParamSpec p;
    memset(&p, 0, sizeof(p));
    p.axis = -1;
    TensorDesc d = tensor2df(DT_F32, DF_NORMAL, rows, H);
    return layer_norm_fp32(d, (F32 *)in, p, (F32 *)gamma, (F32 *)beta, d, out);
}

int ref_softmax_f32(U32 rows, U32 len, const float *in, float *out)
{
    TensorDesc d = tensor2df(DT_F32, DF_NORMAL, rows, len);
    return softmax_fp32(d, in, -1, d, out);
}

// n must be a multiple of 8: the reference's GELU loop has no tail (x86_functions_fp32.h:135)
int ref_gelu_f32(U32 n, const float *in, float *out)
{
    ActivationParamSpec a;
    memset(&a, 0, sizeof(a));
    a.mode = ACTIVATION_GELU;
    return activation_fp32((F32 *)in, n, a, out);
}

}  // extern "C"
