// C-ABI entry points of the int8 convolution (size / algorithm queries, filter transform, tmp bytes, the convolution
// itself with its device-pointer core, which the deconvolution and the per-channel / asynchronous forms share) and of
// the 1-bit convolution. Argument validation, Bolt's tmp / scale conventions, host <-> device staging; no arithmetic
// on tensor data happens on the CPU.
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

extern "C" {

// ---- int8 convolution (compute/tensor/src/cpu/x86/int8/convolution.cpp:97-150) ---------------------
extern "C++" {
namespace bgapi {

EE get4d(TensorDesc d, U32 *n, U32 *c, U32 *h, U32 *w)
{
    if (d.nDims != 4) {
        return NOT_MATCH;
    }
    *w = d.dims[0];
    *h = d.dims[1];
    *c = d.dims[2];
    *n = d.dims[3];
    // every 4-D operator sizes its buffers and addresses its elements in 32 bits, as the reference's interface does
    // (tensorNumElements, U32 byte counts): a tensor of 2^32 elements or more is refused rather than wrapped
    if ((uint64_t)d.dims[0] * d.dims[1] >= (1ull << 32) || (uint64_t)d.dims[0] * d.dims[1] * d.dims[2] >= (1ull << 32) ||
        (uint64_t)d.dims[0] * d.dims[1] * d.dims[2] * d.dims[3] >= (1ull << 32)) {
        return NOT_SUPPORTED;
    }
    return SUCCESS;
}

EE conv_shape(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, const ConvolutionParamSpec &p,
    ConvShape *s)
{
    U32 on, fc;
    const EE ei = get4d(inputDesc, &s->n, &s->ic, &s->ih, &s->iw), ef = get4d(filterDesc, &s->oc, &fc, &s->fh, &s->fw);
    const EE eo = get4d(outputDesc, &on, &s->oc, &s->oh, &s->ow);
    if (ei == NOT_SUPPORTED || ef == NOT_SUPPORTED || eo == NOT_SUPPORTED) {
        return NOT_SUPPORTED;  // a tensor too large for 32-bit sizes
    }
    if (ei != SUCCESS || ef != SUCCESS || eo != SUCCESS) {
        return NOT_MATCH;
    }
    if (p.group != 1) {
        return NOT_SUPPORTED;  // depthwise / grouped int8 convolution is a different reference kernel
    }
    // a transformed filter's desc carries the channel count rounded up to 16 (convolution_transform.cpp:70-87)
    if ((fc != s->ic && fc != align_up(s->ic, 16)) || on != s->n || s->ic % 8 != 0 || s->oc % 8 != 0) {
        return NOT_MATCH;
    }
    s->sh = p.stride_h;
    s->sw = p.stride_w;
    s->pt = p.pad_top;
    s->pb = p.pad_bottom;
    s->pl = p.pad_left;
    s->pr = p.pad_right;
    s->dh = p.dilatedRate_h ? p.dilatedRate_h : 1;
    s->dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (s->sh == 0 || s->sw == 0) {
        return NOT_MATCH;
    }
    s->Hp = s->ih + s->pt + s->pb;
    s->Wp = s->iw + s->pl + s->pr;
    s->ICp = align_up(s->ic, 16);
    s->Kp = align_up(s->fh * s->fw * s->ICp, 64);
    s->N16 = align_up(s->oc, 16);
    const U32 eh = (s->fh - 1) * s->dh + 1, ew = (s->fw - 1) * s->dw + 1;
    if (s->Hp < eh || s->Wp < ew || (s->Hp - eh) / s->sh + 1 < s->oh || (s->Wp - ew) / s->sw + 1 < s->ow) {
        return NOT_MATCH;  // the output must fit the padded input (every gather stays inside it)
    }
    // the kernels address the image (the caller's, and the padded copy in tmp) with 32-bit byte offsets; the reference's
    // own tmp-bytes interface is 32-bit as well
    if ((uint64_t)s->n * s->ic * s->ih * s->iw >= (1ull << 32) || (uint64_t)s->n * s->Hp * s->Wp * s->ICp >= (1ull << 32)) {
        return NOT_SUPPORTED;
    }
    return SUCCESS;
}

size_t conv_padded_bytes(const ConvShape &s)
{
    return ((size_t)s.n * s.Hp * s.Wp * s.ICp + 255) / 256 * 256;
}

// tmp = [padded s8 image][offsetC + folded bias, oc int32]
size_t conv_tmp_layout(const ConvShape &s, size_t *off)
{
    size_t b = (conv_padded_bytes(s) + 255) / 256 * 256;
    *off = b;
    b += (size_t)s.oc * 4;
    return b + 32;
}

void conv_pack_filter_host(const INT8 *src, const ConvShape &s, I32 *offsetC, INT8 *dst)
{
    const U32 fhw = s.fh * s.fw;
    memset(dst, 0, (size_t)s.N16 * s.Kp);
    for (U32 n = 0; n < s.oc; ++n) {
        I32 sum = 0;
        for (U32 c = 0; c < s.ic; ++c) {
            for (U32 t = 0; t < fhw; ++t) {
                const INT8 v = src[((size_t)n * s.ic + c) * fhw + t];
                sum += v;
                dst[mmm_packed_offset(n, t * s.ICp + c, s.Kp)] = v;
            }
        }
        offsetC[n] = -128 * sum;
    }
}

// all pointers device
EE conv_device(const ConvShape &s, DataFormat idf, const void *input, const void *eltwise, const void *filter,
    const void *bias, void *tmp, DataType odt, DataFormat odf, void *output, F32 *scale, int relu)
{
    Ctx &c = ctx();
    size_t offOff;
    conv_tmp_layout(s, &offOff);
    U8 *t = (U8 *)tmp;
    const F32 scaleO = scale[0] * scale[2];  // convolution_direct.cpp:2687
    // The filter-panel kernel (few output channels, short K) gathers from the caller's tensor itself when the channel
    // count is a multiple of 16; every other shape first re-lays the input as a zero-padded s8 image in tmp. The
    // in-place gather costs the kernel about as much as half a padding pass (bounds tests, and two 8-byte loads per
    // fragment from NCHWC8), so by default (1) it is taken where the convolution runs once -- int32 and fp32
    // results -- and not for u8 results, whose two passes share one padded image; 2 takes it always.
    const bool gather_ok = conv_panel_ok(s.oc, s.Kp) && s.ic % 16 == 0 && (((uintptr_t)input) & 15) == 0;
    // u8 result in ONE pass of the filter-panel kernel when all its workgroups are resident at once: they agree on
    // max|acc| with the accumulators still in registers and requantise from there. The convolution then runs once,
    // so it also gathers from the caller's tensor in place where it can.
    const uint32_t M_pix = s.n * s.oh * s.ow;
    bool onepass = odt == DT_U8_Q && g_conv_onepass && conv_panel_ok(s.oc, s.Kp) &&
        conv_panel_grid(M_pix) <= conv_onepass_max_grid(s.Kp);
    const bool direct = g_conv_direct && (g_conv_direct == 2 || odt != DT_U8_Q || onepass) && gather_ok;
    if (!direct) {
        HIP_TRY(launch_conv_pad((const uint8_t *)input, s.n, s.ic, s.ih, s.iw, idf == DF_NCHWC16 ? 16 : 8, s.pt, s.pb, s.pl,
            s.pr, (int8_t *)t, c.stream, odt == DT_U8_Q ? c.ws : nullptr));  // u8 results: also clears the max slots
    }
    // filter blob = [offsetC oc*4][packed matrix] (convolution_transform.cpp:36-44 keeps the vector in front)
    const int32_t *offC = (const int32_t *)filter;
    const int8_t *mat = (const int8_t *)filter + (size_t)s.oc * 4;
    // offsetC + round(bias * scaleO) (convolution_direct.cpp:2687-2700) is formed inside the kernel for the columns
    // it owns: no separate launch
    GemmArgs g;
    memset(&g, 0, sizeof(g));
    g.A = direct ? (const uint8_t *)input : (const uint8_t *)t;
    if (direct) {
        g.conv.in_c = idf == DF_NCHWC16 ? 16 : 8;
        g.conv.H = s.ih;
        g.conv.W = s.iw;
        g.conv.IC = s.ic;
        g.conv.pt = s.pt;
        g.conv.pl = s.pl;
    }
    g.Bp = mat;
    g.M = s.n * s.oh * s.ow;
    g.N = s.oc;
    g.K = s.Kp;
    g.ob = offC;
    g.comp = offC;
    g.fold_bias = (const float *)bias;
    g.fold_scale = scaleO;
    g.conv.OHW = s.oh * s.ow;
    g.conv.OW = s.ow;
    g.conv.sh = s.sh;
    g.conv.sw = s.sw;
    g.conv.Hp = s.Hp;
    g.conv.Wp = s.Wp;
    g.conv.ICp = s.ICp;
    g.conv.fh = s.fh;
    g.conv.fw = s.fw;
    g.conv.dh = s.dh;
    g.conv.dw = s.dw;
    g.conv.out_c = (odf == DF_NCHWC8) ? 8 : 16;
    g.conv.relu = relu;
    if (odt == DT_F32) {
        g.C = output;
        g.epi.mode = EPI_F32;
        g.epi.factor = 1 / scaleO;  // :2700-2703
        g.conv.eltwise = (const float *)eltwise;
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        scale[1] = scaleO;
        return SUCCESS;
    }
    g.epi.mode = EPI_I32;
    if (odt == DT_I32) {
        g.C = output;
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        scale[1] = scaleO;
        return SUCCESS;
    }
    // u8 with the tensor-wide dynamic output scale (:2797-2806). The reference parks int32 accumulators
    // in tmp, takes their abs-max and requantises; here the convolution runs twice instead -- once
    // folding max|acc| into the scratch slots without storing anything, once writing u8 with the scale
    // that maximum gives. The arithmetic per element is the same; the int32 tensor (4 bytes per output,
    // written and read back) never exists, which is worth more than the repeated matrix work.
    if (onepass) {
        g.C = output;
        g.epi.mode = EPI_U8;
        g.conv.scaleO = scaleO;
        g.conv.dscale_out = c.hscale_dev;
        g.sync = c.fsync.next(conv_panel_grid(M_pix));
        arm_scale(c);
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        bool gave_up = false;
        EE te = take_scale(c, &scale[1], &gave_up);
        if (te != SUCCESS || !gave_up) {
            return te;
        }
        // the bounded wait of the one-pass form expired (the CUs were held by other work): nothing was stored;
        // the two passes below redo the convolution
        g_fused_fallbacks.fetch_add(1);
        memset(&g.sync, 0, sizeof(g.sync));
        g.epi.mode = EPI_I32;
        g.conv.dscale_out = nullptr;
    }
    g.C = nullptr;
    g.conv.absmax = c.ws;
    if (direct || onepass) {  // otherwise the padding kernel has cleared the slots
        HIP_TRY(launch_fill_u32(c.ws, kWsWords, 0, c.stream));
    }
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    g.C = output;
    g.epi.mode = EPI_U8;
    g.conv.scaleO = scaleO;
    g.conv.dscale_out = c.hscale_dev;  // the new output scale goes straight into pinned host memory
    arm_scale(c);
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    return take_scale(c, &scale[1]);
}

}  // namespace bgapi
}  // extern "C++"

EE convolution_infer_output_size_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, ConvolutionParamSpec p,
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
        return NOT_SUPPORTED;  // 5-D (3-D convolution) is not on the int8 path
    }
    EE ret = SUCCESS;
    if (fh < 1 || fw < 1) {
        ret = NOT_SUPPORTED;
    }
    const U32 dh = p.dilatedRate_h ? p.dilatedRate_h : 1, dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (p.stride_h == 0 || p.stride_w == 0) {
        return NOT_MATCH;
    }
    const I32 fhD = (I32)((fh - 1) * dh + 1), fwD = (I32)((fw - 1) * dw + 1);
    I32 oh, ow;
    switch (p.round_mode) {  // convolution.cpp:62-82
        case ROUND_SAME_UPPER:
            oh = (I32)((ih + p.stride_h - 1) / p.stride_h);
            ow = (I32)((iw + p.stride_w - 1) / p.stride_w);
            break;
        case ROUND_SAME_LOWER:
            oh = (I32)(ih / p.stride_h);
            ow = (I32)(iw / p.stride_w);
            break;
        default: {
            // unsigned arithmetic like the reference's (U32 operands): a window larger than the padded image wraps
            const U32 th = ih + p.pad_top + p.pad_bottom - (U32)fhD, tw = iw + p.pad_left + p.pad_right - (U32)fwD;
            oh = (I32)(th / p.stride_h + 1);
            ow = (I32)(tw / p.stride_w + 1);
            break;
        }
    }
    if (oh < 0 || ow < 0) {
        ret = NOT_MATCH;
    }
    if (fn % 8 != 0) {
        return NOT_SUPPORTED;  // :93-95
    }
    DataFormat odf = DF_NCHWC8;
    if (targetDataType == DT_U8_Q && fn != 8) {
        odf = DF_NCHWC16;  // :97-101
    }
    *outputDesc = tensor4df(targetDataType, odf, in, fn, (U32)oh, (U32)ow);
    return ret;
}

EE convolution_infer_forward_algorithm_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm, DataType targetDataType,
    ActivationParamSpec activationDesc, Arch arch)
{
    (void)outputDesc;
    (void)p;
    (void)policy;
    (void)activationDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!algorithm) {
        return NULL_POINTER;
    }
    if (*algorithm != CONVOLUTION_ALGORITHM_NULL) {
        return SUCCESS;  // cpu/x86/convolution.cpp:39-41
    }
    if (targetDataType != DT_U8_Q && targetDataType != DT_I8) {
        return NOT_SUPPORTED;  // only the quantised convolution runs here
    }
    U32 in, ic, ih, iw, fn, fc, fh, fw;
    if (get4d(inputDesc, &in, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_SUPPORTED;
    }
    *algorithm = (fh == 1 && fw == 1) ? CONVOLUTION_ALGORITHM_POINTWISE : CONVOLUTION_ALGORITHM_DIRECT;  // :79-82, :101
    return SUCCESS;
}

EE convolution_transform_filter_bytes_gfx950(TensorDesc filterDesc, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (p.group != 1 || filterDesc.dt != DT_I8) {
        return NOT_SUPPORTED;
    }
    *bytes = fn * 4 + align_up(fn, 16) * align_up(fh * fw * align_up(fc, 16), 64) + 32;
    return SUCCESS;
}

EE convolution_transform_filter_gfx950(TensorDesc filterDesc, const void *filter, ConvolutionParamSpec p,
    ConvolutionForwardAlgorithm algorithm, TensorDesc *ftmDesc, void *filterTransformed, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;
    }
    if (filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHW || p.group != 1) {
        return NOT_SUPPORTED;
    }
    ConvShape s;
    memset(&s, 0, sizeof(s));
    if (get4d(filterDesc, &s.oc, &s.ic, &s.fh, &s.fw) != SUCCESS) {
        return NOT_MATCH;
    }
    s.ICp = align_up(s.ic, 16);
    s.Kp = align_up(s.fh * s.fw * s.ICp, 64);
    s.N16 = align_up(s.oc, 16);
    if (arch == AMD_GFX950) {
        conv_pack_filter_host((const INT8 *)filter, s, (I32 *)filterTransformed, (INT8 *)filterTransformed + (size_t)s.oc * 4);
    } else {
        EE e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        HIP_TRY(launch_conv_pack_filter((const int8_t *)filter, s.oc, s.ic, s.fh, s.fw, (int32_t *)filterTransformed,
            (int8_t *)filterTransformed + (size_t)s.oc * 4, ctx().stream));
    }
    *ftmDesc = filterDesc;
    ftmDesc->df = DF_NCHWC2NxC4;  // convolution_transform.cpp:207-211
    ftmDesc->dims[2] = s.ICp;      // channels rounded up to the 16 of the packed layout (:70-87)
    return SUCCESS;
}

EE convolution_infer_forward_tmp_bytes_gfx950(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, U32 *bytes, Arch arch)
{
    (void)algorithm;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    ConvShape s;
    EE e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    size_t off;
    const size_t total = conv_tmp_layout(s, &off);
    if (total > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)total;
    return SUCCESS;
}

EE convolution_gfx950(TensorDesc inputDesc, const void *input, const void *eltwiseInput, TensorDesc filterDesc,
    const void *filter, ConvolutionParamSpec p, ConvolutionForwardAlgorithm algorithm, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, F32 *scale,
    ActivationParamSpec activationDesc, Arch arch)
{
    (void)algorithm;
    (void)biasDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !bias || !tmp || !scale) {
        return NULL_POINTER;  // x86/int8/convolution.cpp:114-117
    }
    if (outputDesc.df != DF_NCHWC16 && outputDesc.df != DF_NCHWC8) {
        return NOT_MATCH;  // :128-130
    }
    if (inputDesc.dt != DT_U8_Q || filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHWC2NxC4) {
        return NOT_MATCH;  // convolution_direct.cpp:2613-2615 (activations arrive quantised on this path)
    }
    if (inputDesc.df != DF_NCHWC8 && inputDesc.df != DF_NCHWC16) {
        return NOT_SUPPORTED;
    }
    const DataType odt = outputDesc.dt;
    if (odt != DT_F32 && odt != DT_U8_Q && odt != DT_I32) {
        return NOT_SUPPORTED;
    }
    if (activationDesc.mode != ACTIVATION_NULL && activationDesc.mode != ACTIVATION_RELU) {
        return NOT_SUPPORTED;
    }
    if (eltwiseInput && odt != DT_F32) {
        return NOT_SUPPORTED;
    }
    ConvShape s;
    EE e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    size_t off;
    const size_t need = conv_tmp_layout(s, &off);
    if (tmpBytes < need) {
        return NOT_MATCH;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    const int relu = (activationDesc.mode == ACTIVATION_RELU);
    if (arch == AMD_GFX950_DEVICE) {
        if (((uintptr_t)tmp & 15) || ((uintptr_t)filter & 15) || ((uintptr_t)output & 15) || ((uintptr_t)input & 7)) {
            return fail(NOT_SUPPORTED, "device tmp / filter / output must be 16-byte aligned, input 8-byte aligned");
        }
        return conv_device(s, inputDesc.df, input, eltwiseInput, filter, bias, tmp, odt, outputDesc.df, output, scale,
            relu);
    }
    Ctx &cx = ctx();
    Stage st;
    const size_t inB = (size_t)s.n * s.ic * s.ih * s.iw;
    const size_t fB = (size_t)s.oc * 4 + (size_t)s.N16 * s.Kp;
    const size_t outN = (size_t)s.n * s.oc * s.oh * s.ow;
    const size_t outB = outN * (odt == DT_U8_Q ? 1 : 4);
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = st.get((size_t)s.oc * 4), *dT = st.get(need), *dO = st.get(outB);
    void *dE = eltwiseInput ? st.get(outN * 4) : nullptr;
    if (!dIn || !dF || !dB || !dT || !dO || (eltwiseInput && !dE)) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, input, inB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dF, filter, fB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dB, bias, (size_t)s.oc * 4, hipMemcpyHostToDevice, cx.stream));
    if (dE) {
        HIP_TRY(hipMemcpyAsync(dE, eltwiseInput, outN * 4, hipMemcpyHostToDevice, cx.stream));
    }
    e = conv_device(s, inputDesc.df, dIn, dE, dF, dB, dT, odt, outputDesc.df, dO, scale, relu);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(output, dO, outB, hipMemcpyDeviceToHost, cx.stream));
    HIP_TRY(hipStreamSynchronize(cx.stream));
    return SUCCESS;
}

// ---- 1-bit convolution (compute/tensor/src/cpu/arm/bnn/convolution.cpp:16-72) ----------------------
// Transformed-filter blob: [bit-packed filter, fn * fc * fh * fw / 8 bytes rounded up to 256 (the vector-ALU
// route)][the same filter expanded to int8 in the GEMM's packed right-hand-side layout, K = fh * fw * fc padded
// to 64 (the matrix-core route)]
static size_t bnn_blob_bits_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return ((size_t)fn * fc * fh * fw / 8 + 255) / 256 * 256;
}

static size_t bnn_blob_i8_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return ((size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16) + 255) / 256 * 256;
}

// ... followed by the filter as E2M1 pairs (K bytes = fh * fw * fc / 2 padded to 64) for the fp4 form of that route
static size_t bnn_blob_bytes(U32 fn, U32 fc, U32 fh, U32 fw)
{
    return bnn_blob_bits_bytes(fn, fc, fh, fw) + bnn_blob_i8_bytes(fn, fc, fh, fw) +
        (size_t)align_up(fh * fw * fc / 2, 64) * align_up(fn, 16);
}

EE convolution_transform_filter_bytes_bnn_gfx950(TensorDesc filterDesc, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_BIN01 && filterDesc.dt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    const size_t b = bnn_blob_bytes(fn, fc, fh, fw);
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE convolution_transform_filter_bnn_gfx950(TensorDesc filterDesc, const void *filter, TensorDesc *ftmDesc,
    void *filterTransformed, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;  // convolution_transform_bnn.h:38-40
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_BIN01 && filterDesc.dt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    if (filterDesc.df != DF_NCHW && filterDesc.df != DF_NCHWN16C8) {
        return NOT_MATCH;  // :83-84
    }
    if (fn % 32 != 0 || fc % 32 != 0) {
        return NOT_SUPPORTED;  // kernel structure of the reference (convolution_xnor_A76.cpp:109,665)
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    const size_t bytes = (size_t)fn * fc * fh * fw / 8, bits = bnn_blob_bits_bytes(fn, fc, fh, fw),
                 total = bnn_blob_bytes(fn, fc, fh, fw);
    const int fmt = (filterDesc.df == DF_NCHWN16C8) ? 1 : 0;
    const int xnor = (filterDesc.dt == DT_BIN11);
    if (arch == AMD_GFX950) {
        Stage st;
        void *a = st.get(bytes);
        U8 *b = (U8 *)st.get(total);
        if (!a || !b) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, filter, bytes, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemsetAsync(b, 0, bits, c.stream));
        HIP_TRY(launch_bnn_pack_filter((const uint8_t *)a, fmt, fn, fc, fh * fw, (uint32_t *)b, c.stream));
        HIP_TRY(launch_bnn_expand_filter((const uint32_t *)b, fn, fc, fh * fw, xnor, (int8_t *)(b + bits), c.stream));
        HIP_TRY(hipMemsetAsync(b + bits + (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), 0,
            bnn_blob_i8_bytes(fn, fc, fh, fw) - (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), c.stream));
        HIP_TRY(launch_bnn_expand_filter_fp4((const uint32_t *)b, fn, fc, fh * fw, xnor,
            b + bits + bnn_blob_i8_bytes(fn, fc, fh, fw), c.stream));
        HIP_TRY(hipMemcpyAsync(filterTransformed, b, total, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    } else {
        if (((uintptr_t)filterTransformed & 15) != 0) {
            return fail(NOT_SUPPORTED, "device filterTransformed must be 16-byte aligned");
        }
        U8 *b = (U8 *)filterTransformed;
        if (bits > bytes / 4 * 4) {  // the padding behind the bits, so that equal filters give equal blobs
            HIP_TRY(launch_fill_u32((uint32_t *)(b + bytes / 4 * 4), (U32)((bits - bytes / 4 * 4) / 4), 0, c.stream));
        }
        HIP_TRY(launch_bnn_pack_filter((const uint8_t *)filter, fmt, fn, fc, fh * fw, (uint32_t *)b, c.stream));
        HIP_TRY(launch_bnn_expand_filter((const uint32_t *)b, fn, fc, fh * fw, xnor, (int8_t *)(b + bits), c.stream));
        const size_t i8 = (size_t)align_up(fh * fw * fc, 64) * align_up(fn, 16), i8p = bnn_blob_i8_bytes(fn, fc, fh, fw);
        if (i8p > i8) {
            HIP_TRY(launch_fill_u32((uint32_t *)(b + bits + i8), (U32)((i8p - i8) / 4), 0, c.stream));
        }
        HIP_TRY(launch_bnn_expand_filter_fp4((const uint32_t *)b, fn, fc, fh * fw, xnor, b + bits + i8p, c.stream));
    }
    *ftmDesc = filterDesc;
    ftmDesc->df = DF_NCHWN16C8;  // the tag the operator layer checks; the byte order inside is this library's
    return SUCCESS;
}

EE convolution_infer_forward_tmp_bytes_bnn_gfx950(TensorDesc inputDesc, ConvolutionParamSpec p, U32 *bytes, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    U32 n, ic, ih, iw;
    if (get4d(inputDesc, &n, &ic, &ih, &iw) != SUCCESS) {
        return NOT_MATCH;
    }
    const size_t Hp = ih + p.pad_top + p.pad_bottom, Wp = iw + p.pad_left + p.pad_right;
    // vector-ALU route: the bit-packed padded image. Matrix-core route: the image expanded to one byte per value.
    const size_t bits = (size_t)n * Hp * Wp * (ic / 8) + 32;
    const size_t img = (size_t)n * Hp * Wp * ic + 32;
    const size_t b = std::max(bits, img);
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE convolution_bnn_gfx950(TensorDesc inputDesc, const void *input, TensorDesc filterDesc, const void *filter,
    ConvolutionParamSpec p, TensorDesc scaleDesc, const void *scale, TensorDesc biasDesc, const void *bias, U32 tmpBytes,
    void *tmp, TensorDesc outputDesc, void *output, ActivationParamSpec activationDesc, Arch arch)
{
    (void)scaleDesc;
    (void)biasDesc;
    (void)activationDesc;  // ignored by the reference as well (bnn/convolution.cpp:35)
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !scale || !bias || !tmp) {
        return NULL_POINTER;  // bnn/convolution.cpp:32-35
    }
    U32 n, ic, ih, iw, fn, fc, fh, fw, on, oc, oh, ow;
    if (get4d(inputDesc, &n, &ic, &ih, &iw) != SUCCESS || get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS ||
        get4d(outputDesc, &on, &oc, &oh, &ow) != SUCCESS) {
        return NOT_MATCH;
    }
    const DataType fdt = filterDesc.dt, idt = inputDesc.dt, odt = outputDesc.dt;
    if (fdt != DT_BIN01 && fdt != DT_BIN11) {
        return NOT_SUPPORTED;
    }
    // fp32 stands where the reference has fp16; bit-packed activations of the filter's type are also taken
    if ((idt != DT_F32 && idt != fdt) || (odt != DT_F32 && odt != DT_I32)) {
        return NOT_MATCH;
    }
    if ((idt == DT_F32 && inputDesc.df != DF_NCHWC8) || outputDesc.df != DF_NCHWC8 || filterDesc.df != DF_NCHWN16C8) {
        return NOT_MATCH;  // :45-53
    }
    if (fc != ic || fn != oc || on != n || ic % 32 != 0 || oc % 32 != 0 || p.group != 1 || p.stride_h == 0 ||
        p.stride_w == 0) {
        return NOT_MATCH;
    }
    if ((p.dilatedRate_h > 1) || (p.dilatedRate_w > 1)) {
        return NOT_SUPPORTED;
    }
    const U32 Hp = ih + p.pad_top + p.pad_bottom, Wp = iw + p.pad_left + p.pad_right;
    if (Hp < fh || Wp < fw || (Hp - fh) / p.stride_h + 1 < oh || (Wp - fw) / p.stride_w + 1 < ow) {
        return NOT_MATCH;
    }
    U32 need = 0;
    EE e = convolution_infer_forward_tmp_bytes_bnn_gfx950(inputDesc, p, &need, arch);
    if (e != SUCCESS) {
        return e;
    }
    if (tmpBytes < need) {
        return NOT_MATCH;
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    Stage st;
    const size_t inB = (idt == DT_F32) ? (size_t)n * ic * ih * iw * 4 : (size_t)n * ic * ih * iw / 8;
    const size_t fB = bnn_blob_bytes(oc, ic, fh, fw);
    const size_t outN = (size_t)n * oc * oh * ow;
    const void *dIn = input, *dF = filter, *dS = scale, *dB = bias;
    void *dT = tmp, *dO = output;
    if (arch == AMD_GFX950) {
        void *a = st.get(inB), *f = st.get(fB), *s = st.get((size_t)oc * 4), *b = st.get((size_t)oc * 4);
        dT = st.get(need);
        dO = st.get(outN * 4);
        if (!a || !f || !s || !b || !dT || !dO) {
            return fail(ALLOC_FAILED, "device staging");
        }
        HIP_TRY(hipMemcpyAsync(a, input, inB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(f, filter, fB, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(s, scale, (size_t)oc * 4, hipMemcpyHostToDevice, c.stream));
        HIP_TRY(hipMemcpyAsync(b, bias, (size_t)oc * 4, hipMemcpyHostToDevice, c.stream));
        dIn = a;
        dF = f;
        dS = s;
        dB = b;
    } else if (!aligned4(tmp) || ((uintptr_t)output & 15) || !aligned4(filter)) {
        return fail(NOT_SUPPORTED, "device tmp / filter must be 4-byte aligned, output 16-byte aligned");
    }
    const int xnor = (fdt == DT_BIN11);
    if (g_bnn_mfma && (((uintptr_t)dT | (uintptr_t)dF) & 15) == 0) {
        // matrix-core route: the image expanded to int8 (or E2M1 pairs), the filter already expanded in the blob,
        // then the implicit-GEMM convolution with fma(S, scale, bias) (or the raw sums) as its epilogue
        const bool fp4 = g_bnn_mfma == 2 && conv_fp4_ok(n * oh * ow, oc);
        int8_t *img = (int8_t *)dT;
        const int8_t *flt = (const int8_t *)dF + bnn_blob_bits_bytes(oc, ic, fh, fw) + (fp4 ? bnn_blob_i8_bytes(oc, ic, fh, fw) : 0);
        if (fp4) {
            HIP_TRY(launch_bnn_expand_input_fp4(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left,
                p.pad_right, xnor ? 0.0f : 0.5f, xnor, (uint8_t *)img, c.stream));
        } else {
            HIP_TRY(launch_bnn_expand_input(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left,
                p.pad_right, xnor ? 0.0f : 0.5f, xnor, img, c.stream));
        }
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = (const uint8_t *)img;
        g.Bp = flt;
        g.M = n * oh * ow;
        g.N = oc;
        g.K = fp4 ? align_up(fh * fw * ic / 2, 64) : align_up(fh * fw * ic, 64);  // in operand bytes
        g.fp4 = fp4 ? 1 : 0;
        g.ob = (const int32_t *)flt;  // ob == comp: no offset, the sums are exact as they are
        g.comp = (const int32_t *)flt;
        g.C = dO;
        g.conv.OHW = oh * ow;
        g.conv.OW = ow;
        g.conv.sh = p.stride_h;
        g.conv.sw = p.stride_w;
        g.conv.Hp = Hp;
        g.conv.Wp = Wp;
        g.conv.ICp = fp4 ? ic / 2 : ic;  // bytes per pixel
        g.conv.fh = fh;
        g.conv.fw = fw;
        g.conv.dh = 1;
        g.conv.dw = 1;
        g.conv.out_c = 8;
        if (odt == DT_I32) {
            g.epi.mode = EPI_I32;
        } else {
            g.epi.mode = EPI_F32_CH;
            g.epi.scaleW = (const float *)dS;
            g.epi.bias = (const float *)dB;
        }
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        if (arch == AMD_GFX950) {
            HIP_TRY(hipMemcpyAsync(output, dO, outN * 4, hipMemcpyDeviceToHost, c.stream));
            HIP_TRY(hipStreamSynchronize(c.stream));
        }
        return SUCCESS;
    }
    HIP_TRY(launch_bnn_pack_input(dIn, idt == DT_F32, n, ic, ih, iw, p.pad_top, p.pad_bottom, p.pad_left, p.pad_right,
        xnor ? 0.0f : 0.5f, (uint32_t *)dT, c.stream));
    BnnArgs a;
    memset(&a, 0, sizeof(a));
    a.x = (const uint32_t *)dT;
    a.w = (const uint32_t *)dF;
    a.M = n * oh * ow;
    a.OHW = oh * ow;
    a.OW = ow;
    a.sh = p.stride_h;
    a.sw = p.stride_w;
    a.Hp = Hp;
    a.Wp = Wp;
    a.IC = ic;
    a.OC = oc;
    a.fh = fh;
    a.fw = fw;
    a.scale = (const float *)dS;
    a.bias = (const float *)dB;
    if (odt == DT_I32) {
        a.sums = (int32_t *)dO;
    } else {
        a.out = (float *)dO;
    }
    HIP_TRY(launch_bnn_conv(a, xnor, c.stream));
    if (arch == AMD_GFX950) {
        HIP_TRY(hipMemcpyAsync(output, dO, outN * 4, hipMemcpyDeviceToHost, c.stream));
        HIP_TRY(hipStreamSynchronize(c.stream));
    }
    return SUCCESS;
}

}  // extern "C"
