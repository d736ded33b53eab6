// C-ABI entry points of the int8 deconvolution: argument validation, the reference's scale-array conventions, host <->
// device staging for the host-pointer mode, and the sequence 1x1 convolution -> gather (deconv.hip).
#include <cstring>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

namespace {

struct DeconvShape {
    U32 n, ic, ih, iw, oc, fh, fw, oh, ow, sh, sw, pt, pb, pl, pr;
    U32 taps, ocx;  // fh * fw, and the 1x1 convolution's output channels taps * oc
    bool gemm;      // IM2COL_GEMM route (plain NCHW input), else POINTWISE (NCHWC16 input)
    bool equal;     // POINTWISE with kernel == stride
    ConvShape cs;   // the inner 1x1 convolution
    size_t off_bias, off_col, off_acc, off_c8, total_tmp;
};

size_t up256(size_t b)
{
    return (b + 255) / 256 * 256;
}

EE deconv_shape(TensorDesc inputDesc, TensorDesc outputDesc, const ConvolutionParamSpec &p, ConvolutionForwardAlgorithm alg,
    DeconvShape *s)
{
    U32 on;
    if (get4d(inputDesc, &s->n, &s->ic, &s->ih, &s->iw) != SUCCESS || get4d(outputDesc, &on, &s->oc, &s->oh, &s->ow) != SUCCESS) {
        return NOT_MATCH;
    }
    if (alg == CONVOLUTION_ALGORITHM_GROUP_DECONV || p.group != 1) {
        return NOT_SUPPORTED;  // depthwise deconvolution is an fp32 path in the reference
    }
    if (alg != CONVOLUTION_ALGORITHM_IM2COL_GEMM && alg != CONVOLUTION_ALGORITHM_POINTWISE) {
        return NOT_SUPPORTED;
    }
    s->gemm = alg == CONVOLUTION_ALGORITHM_IM2COL_GEMM;
    if (inputDesc.dt != DT_U8_Q) {
        return NOT_SUPPORTED;
    }
    if (s->gemm ? inputDesc.df != DF_NCHW : inputDesc.df != DF_NCHWC16) {
        // DF_NCHWC8 inputs: the reference writes its bias rows in blocks of 8 channels under a 16-channel output
        // (cpu/x86/deconvolution.cpp:143,215-226) -- no defined result to reproduce
        return NOT_SUPPORTED;
    }
    if (outputDesc.df != DF_NCHWC16 || (outputDesc.dt != DT_U8_Q && outputDesc.dt != DT_F32)) {
        return NOT_SUPPORTED;
    }
    s->fh = p.kernel_h;
    s->fw = p.kernel_w;
    s->sh = p.stride_h;
    s->sw = p.stride_w;
    s->pt = p.pad_top;
    s->pb = p.pad_bottom;
    s->pl = p.pad_left;
    s->pr = p.pad_right;
    const U32 dh = p.dilatedRate_h ? p.dilatedRate_h : 1, dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (on != s->n || s->fh == 0 || s->fw == 0 || s->sh == 0 || s->sw == 0 || dh != 1 || dw != 1) {
        return NOT_MATCH;
    }
    if (s->oc % 16 != 0 || s->ic % (s->gemm ? 8 : 16) != 0 || s->n == 0 || s->ih == 0 || s->iw == 0 || s->oh == 0 ||
        s->ow == 0) {
        return NOT_SUPPORTED;
    }
    s->taps = s->fh * s->fw;
    s->equal = !s->gemm && s->fh == s->sh && s->fw == s->sw;
    if (s->equal && ((uint64_t)s->oh + s->pt > (uint64_t)s->sh * s->ih || (uint64_t)s->ow + s->pl > (uint64_t)s->sw * s->iw)) {
        return NOT_SUPPORTED;  // output pixels no column lands on: the reference leaves them unwritten
    }
    const uint64_t ocx = (uint64_t)s->taps * s->oc;
    const uint64_t M = (uint64_t)s->n * s->ih * s->iw, total = (uint64_t)s->n * s->oc * s->oh * s->ow;
    if (ocx > 0x7fffffffull || M > 0x7fffffffull || total > 0xffffffffull || M * ocx > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    s->ocx = (U32)ocx;
    ConvShape &c = s->cs;
    memset(&c, 0, sizeof(c));
    c.n = s->n;
    c.ic = s->ic;
    c.ih = c.oh = c.Hp = s->ih;
    c.iw = c.ow = c.Wp = s->iw;
    c.oc = s->ocx;
    c.fh = c.fw = c.sh = c.sw = c.dh = c.dw = 1;
    c.ICp = align_up(s->ic, 16);
    c.Kp = align_up(c.ICp, 64);
    c.N16 = align_up(s->ocx, 16);
    size_t off;
    size_t b = up256(conv_tmp_layout(c, &off));
    s->off_bias = b;
    b += up256((size_t)s->ocx * 4);
    s->off_col = b;
    b += up256((size_t)M * s->ocx * (s->equal ? 1 : 4));
    s->off_acc = b;
    if (outputDesc.dt == DT_U8_Q && !s->equal) {
        b += up256((size_t)total * 4);
    }
    s->off_c8 = b;
    if (s->gemm) {
        b += up256((size_t)s->n * s->ic * s->ih * s->iw);
    }
    s->total_tmp = b + 32;
    return SUCCESS;
}

size_t deconv_blob_bytes(U32 ic, U32 ocx)
{
    return (size_t)ocx * 4 + (size_t)align_up(ocx, 16) * align_up(align_up(ic, 16), 64);
}

// all pointers device; scale is the caller's host array
EE deconv_device(const DeconvShape &s, const void *input, const void *filter, const void *bias, void *tmp, DataType odt,
    void *output, F32 *sc, int relu)
{
    Ctx &c = ctx();
    U8 *t = (U8 *)tmp;
    float *convBias = (float *)(t + s.off_bias);
    void *col = t + s.off_col;
    const F32 sO = sc[0] * sc[2];
    const void *in = input;
    DataFormat idf = DF_NCHWC16;
    if (s.gemm) {
        HIP_TRY(launch_nchw_to_c8_u8((const uint8_t *)input, s.n, s.ic, s.ih * s.iw, t + s.off_c8, c.stream));
        in = t + s.off_c8;
        idf = DF_NCHWC8;
    }
    DeconvArgs g;
    g.col = col;
    g.out = output;
    g.n = s.n;
    g.oc = s.oc;
    g.ih = s.ih;
    g.iw = s.iw;
    g.oh = s.oh;
    g.ow = s.ow;
    g.fh = s.fh;
    g.fw = s.fw;
    g.sh = s.sh;
    g.sw = s.sw;
    g.pt = s.pt;
    g.pl = s.pl;
    g.bias = (const float *)bias;
    g.scaleO = sO;
    g.relu = relu;
    F32 s3[3] = {sc[0], sc[1], sc[2]};
    if (s.equal) {
        // cpu/x86/deconvolution.cpp:157-165: the bias goes into the convolution, once per tap, and the convolution
        // writes u8 with its own dynamic scale whatever the output tensor's type is
        HIP_TRY(launch_repeat_f32((const float *)bias, s.oc, s.ocx, convBias, c.stream));
        EE e = conv_device(s.cs, idf, in, nullptr, filter, convBias, tmp, DT_U8_Q, DF_NCHWC16, col, s3, 0);
        if (e != SUCCESS) {
            return e;
        }
        sc[1] = s3[1];
        g.mode = odt == DT_U8_Q ? DECONV_U8 : DECONV_F32_FROM_U8;
        g.factor = 1.0f / sc[1];
        HIP_TRY(launch_deconv_gather(g, c.stream));
        return SUCCESS;
    }
    HIP_TRY(launch_fill_u32((uint32_t *)convBias, s.ocx, 0, c.stream));
    EE e = conv_device(s.cs, idf, in, nullptr, filter, convBias, tmp, DT_I32, DF_NCHWC16, col, s3, 0);
    if (e != SUCCESS) {
        return e;
    }
    g.factor = 1 / sO;
    if (odt == DT_F32) {
        if (s.gemm) {
            g.mode = DECONV_F32_DEQ;  // integer ReLU, then one dequantisation (cpu/deconvolution.cpp:338-354)
        } else {
            g.mode = DECONV_F32_SUM;  // cpu/x86/deconvolution.cpp:166-176,212-227
            sc[1] = sO;
        }
        HIP_TRY(launch_deconv_gather(g, c.stream));
        return SUCCESS;
    }
    // u8: int32 sums into tmp with their max, then the requantisation of quantizeI32ToU8 (avx512/quantize.cpp:364-416)
    g.mode = DECONV_I32;
    g.out = t + s.off_acc;
    g.absmax = c.ws;
    g.relu = s.gemm ? relu : 0;
    HIP_TRY(launch_fill_u32(c.ws, kWsWords, 0, c.stream));
    HIP_TRY(launch_deconv_gather(g, c.stream));
    const F32 s0 = s.gemm ? sc[1] : -1.0f;  // cpu/deconvolution.cpp:356-357; cpu/x86/deconvolution.cpp:243-245
    const uint32_t total = s.n * s.oc * s.oh * s.ow;
    const bool dynamic = s0 < 0 && sO > 0;
    if (dynamic) {
        arm_scale(c);
    }
    HIP_TRY(launch_requant_i32((const int32_t *)(t + s.off_acc), total, output, 1, c.ws, s0, sO, dynamic ? c.hscale_dev : nullptr,
        c.stream));
    if (!s.gemm && relu) {
        HIP_TRY(launch_relu_u8((uint8_t *)output, total, c.stream));
    }
    sc[2] = sO;
    if (dynamic) {
        return take_scale(c, &sc[1]);
    }
    return SUCCESS;
}

}  // namespace

extern "C" {

EE deconvolution_infer_output_size_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, ConvolutionParamSpec p,
    TensorDesc *outputDesc, DataType targetDataType, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!outputDesc) {
        return NULL_POINTER;
    }
    U32 in, ic, ih, iw, fn, fc, fh, fw;
    if (get4d(inputDesc, &in, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (fn != 1 && fn != ic) {
        return NOT_MATCH;  // deconvolution.cpp:37
    }
    if (fh < 1 || fw < 1) {
        return NOT_SUPPORTED;
    }
    U32 oh, ow;
    if (p.round_mode == ROUND_TF_SAME) {
        oh = p.stride_h * ih;
        ow = p.stride_w * iw;
    } else {
        oh = fh + p.stride_h * (ih - 1) - p.pad_top - p.pad_bottom + p.output_pad_h;
        ow = fw + p.stride_w * (iw - 1) - p.pad_left - p.pad_right + p.output_pad_w;
    }
    const DataFormat odf = (inputDesc.dt == DT_U8_Q && fc > 8) ? DF_NCHWC16 : DF_NCHWC8;  // :57-64, AVX-512 build
    *outputDesc = tensor4df(targetDataType, odf, in, fc, oh, ow);
    return fc % 8 != 0 ? NOT_SUPPORTED : SUCCESS;  // :88-91
}

EE deconvolution_infer_forward_algorithm_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm, DataType targetDataType,
    Arch arch)
{
    (void)outputDesc;
    (void)p;
    (void)policy;
    (void)targetDataType;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!algorithm) {
        return NULL_POINTER;
    }
    U32 in, ic, ih, iw, fn, fc, fh, fw;
    if (get4d(inputDesc, &in, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (fn == 1 && ic != fn) {
        *algorithm = CONVOLUTION_ALGORITHM_GROUP_DECONV;  // cpu/deconvolution.cpp:43-46
    } else if (inputDesc.df == DF_NCHWC8 || inputDesc.df == DF_NCHWC16) {
        *algorithm = CONVOLUTION_ALGORITHM_POINTWISE;  // :47-51
    } else {
        *algorithm = CONVOLUTION_ALGORITHM_IM2COL_GEMM;
    }
    return SUCCESS;
}

EE deconvolution_transform_filter_bytes_gfx950(TensorDesc filterDesc, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)p;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    if (algorithm != CONVOLUTION_ALGORITHM_IM2COL_GEMM && algorithm != CONVOLUTION_ALGORITHM_POINTWISE) {
        return NOT_SUPPORTED;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_I8) {
        return NOT_SUPPORTED;
    }
    const uint64_t ocx = (uint64_t)fc * fh * fw;
    if (ocx > 0x7fffffffull || deconv_blob_bytes(fn, (U32)ocx) + 32 > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    // the reference's ALIGN(fn, 16) * fc * fh * fw + 32 + fc * fh * fw * 4 (cpu/deconvolution.cpp:140-149) with the
    // reduction length rounded up to 64 for the matrix cores
    *bytes = (U32)(deconv_blob_bytes(fn, (U32)ocx) + 32);
    return SUCCESS;
}

EE deconvolution_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, TensorDesc *ftmDesc, void *filterTransformed, Arch arch)
{
    (void)p;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;
    }
    if (algorithm != CONVOLUTION_ALGORITHM_IM2COL_GEMM && algorithm != CONVOLUTION_ALGORITHM_POINTWISE) {
        return NOT_MATCH;  // x86/int8/deconvolution_transform.cpp:118-120
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHW) {
        return NOT_SUPPORTED;
    }
    const U32 taps = fh * fw, ocx = fc * taps;
    const U32 Kp = align_up(align_up(fn, 16), 64);
    I32 *offsetC = (I32 *)filterTransformed;
    INT8 *mat = (INT8 *)filterTransformed + (size_t)ocx * 4;
    if (arch == AMD_GFX950) {
        const INT8 *src = (const INT8 *)filter;
        memset(mat, 0, (size_t)align_up(ocx, 16) * Kp);
        for (U32 n = 0; n < ocx; ++n) {
            const U32 tap = n / fc, o = n % fc;
            I32 sum = 0;
            for (U32 c = 0; c < fn; ++c) {
                const INT8 v = src[((size_t)c * fc + o) * taps + tap];
                sum += v;
                mat[mmm_packed_offset(n, c, Kp)] = v;
            }
            offsetC[n] = -128 * sum;
        }
    } else {
        EE e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        if (((uintptr_t)filterTransformed & 15) != 0) {
            return fail(NOT_SUPPORTED, "device filter blob must be 16-byte aligned");
        }
        Ctx &c = ctx();
        // rows of the last 16-row block beyond ocx and bytes beyond ic stay zero: clear the matrix first
        HIP_TRY(launch_fill_u32((uint32_t *)mat, (uint32_t)((size_t)align_up(ocx, 16) * Kp / 4), 0, c.stream));
        HIP_TRY(launch_deconv_pack_filter((const int8_t *)filter, fn, fc, taps, (int32_t *)offsetC, (int8_t *)mat, c.stream));
    }
    if (algorithm == CONVOLUTION_ALGORITHM_IM2COL_GEMM) {
        *ftmDesc = tensor2df(DT_I8, DF_NKNxKx, fn, ocx);  // what matrix_matrix_multiply_transform_rhs returns (:166-169)
    } else {
        // x86/int8/deconvolution_transform.cpp:88-93
        *ftmDesc = tensor4df(DT_I8, DF_NCHWC2NxC4, align_up(ocx, 4), align_up(fn, 16), 1, 1);
    }
    return SUCCESS;
}

EE deconvolution_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)filterDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    DeconvShape s;
    EE e = deconv_shape(inputDesc, outputDesc, p, algorithm, &s);
    if (e != SUCCESS) {
        return e;
    }
    if (s.total_tmp > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)s.total_tmp;
    return SUCCESS;
}

EE deconvolution_gfx950(TensorDesc inputDesc, void *input, TensorDesc filterDesc, const void *filter,
    ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, TensorDesc scaleDesc, void *scale, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, ActivationParamSpec activationDesc,
    Arch arch)
{
    (void)scaleDesc;
    (void)biasDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !bias || !tmp || !scale) {
        return NULL_POINTER;  // cpu/deconvolution.cpp:504-507
    }
    if (activationDesc.mode != ACTIVATION_NULL && activationDesc.mode != ACTIVATION_RELU) {
        return NOT_SUPPORTED;
    }
    DeconvShape s;
    EE e = deconv_shape(inputDesc, outputDesc, p, algorithm, &s);
    if (e != SUCCESS) {
        return e;
    }
    // the transformed filter's desc must describe this problem: [K = ic, N = taps * oc] or [n = ALIGN(taps * oc, 4), c = ALIGN(ic, 16)]
    if (filterDesc.dt != DT_I8) {
        return NOT_MATCH;
    }
    if (s.gemm ? (filterDesc.df != DF_NKNxKx || filterDesc.nDims != 2 || filterDesc.dims[0] != s.ocx || filterDesc.dims[1] != s.ic)
               : (filterDesc.df != DF_NCHWC2NxC4 || filterDesc.nDims != 4 || filterDesc.dims[3] != align_up(s.ocx, 4) ||
                     filterDesc.dims[2] != align_up(s.ic, 16))) {
        return NOT_MATCH;
    }
    if (tmpBytes < s.total_tmp) {
        return NOT_MATCH;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    const int relu = activationDesc.mode == ACTIVATION_RELU;
    const DataType odt = outputDesc.dt;
    if (arch == AMD_GFX950_DEVICE) {
        if (((uintptr_t)tmp & 15) || ((uintptr_t)filter & 15) || ((uintptr_t)output & 15) || ((uintptr_t)input & 15) ||
            ((uintptr_t)bias & 15)) {
            return fail(NOT_SUPPORTED, "device tmp / filter / input / output / bias must be 16-byte aligned");
        }
        return deconv_device(s, input, filter, bias, tmp, odt, output, (F32 *)scale, relu);
    }
    Ctx &cx = ctx();
    Stage st;
    const size_t inB = (size_t)s.n * s.ic * s.ih * s.iw;
    const size_t fB = deconv_blob_bytes(s.ic, s.ocx);
    const size_t outB = (size_t)s.n * s.oc * s.oh * s.ow * (odt == DT_U8_Q ? 1 : 4);
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = st.get((size_t)s.oc * 4), *dT = st.get(s.total_tmp), *dO = st.get(outB);
    if (!dIn || !dF || !dB || !dT || !dO) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, input, inB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dF, filter, fB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dB, bias, (size_t)s.oc * 4, hipMemcpyHostToDevice, cx.stream));
    e = deconv_device(s, dIn, dF, dB, dT, odt, dO, (F32 *)scale, relu);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(output, dO, outB, hipMemcpyDeviceToHost, cx.stream));
    HIP_TRY(hipStreamSynchronize(cx.stream));
    return SUCCESS;
}

}  // extern "C"
