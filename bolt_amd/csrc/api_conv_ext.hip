// C-ABI: the two forms of the int8 convolution that the reference does not have.
//
//  * per-output-channel filter scales (bolt_gfx950_convolution_int8_perchannel): the reference's kernels carry ONE
//    scale for the whole filter (compute/tensor/src/cpu/x86/int8/avx512/convolution_direct.cpp:2406-2422, 2687-2692);
//    a filter quantised channel by channel needs  f = cvt(acc) * (1.0f / (sI * sW[oc])) + bias[oc], ReLU, and then
//    either the fp32 values or their quantisation with ONE output scale (static, or 127 / max|f| over the tensor).
//  * asynchronous calls with device-resident scales (bolt_gfx950_convolution_async): the reference returns a new
//    output scale through a host pointer (scale[1]), so a chain of quantised convolutions waits for the device after
//    every layer; here the input scale is read from, and the output scale left in, device memory.
//
// Both run the kernels of convolution_gfx950 (gemm.hip: conv_u8s8_panel_kernel, gemm_u8s8_dma_kernel<..., CONV>); what
// differs is the epilogue (EPI_CONV_CH) and where the scales live. A dynamic u8 result runs in ONE pass of the filter-
// panel kernel where all its workgroups are resident at once (they agree on the tensor-wide maximum with their values
// in registers; if that agreement is abandoned the synchronous forms redo the call in two passes from the host, and the
// asynchronous form -- given a tmp with spill room -- finishes on the device), and otherwise in two passes: the first
// only folds the maximum into scratch slots, the second stores. Nothing in the asynchronous form waits for the host.
#include "api_internal.h"

using namespace bg;
using namespace bgapi;

namespace {

struct ConvExt {
    const float *dscaleI = nullptr;   // input scale in device memory (asynchronous form), else scaleI
    float scaleI = 0;
    const float *scaleW = nullptr;    // per-output-channel filter scales [oc] (device); null: one scale, filterScale
    float filterScale = 0;
    float staticOut = 0;              // u8 result: > 0 = quantise with this scale, else dynamic
    float *dscaleO = nullptr;         // device word that receives the output scale; null: the context's pinned word
    // where a one-pass u8 launch may park its values should its grid-wide agreement be abandoned (asynchronous form:
    // 4 bytes per output element); null in the synchronous forms, which hand an abandoned launch back to the host
    void *spill = nullptr;
    bool host_waits = false;          // synchronous form: the scale is taken from the pinned word, a NaN there = redo
    F32 *host_scale = nullptr;        //   ... and handed back here
};

size_t conv_out_elems(const ConvShape &s)
{
    return (size_t)s.n * s.oc * s.oh * s.ow;
}

// tmp of the asynchronous form: the synchronous call's, then room for one 32-bit value per output element
size_t conv_async_tmp_layout(const ConvShape &s, size_t *spill_off)
{
    size_t off;
    const size_t base = (conv_tmp_layout(s, &off) + 255) / 256 * 256;
    *spill_off = base;
    return base + conv_out_elems(s) * 4;
}

// the context's two arrays of max slots, clear before the first two-pass call (and after one that failed half way)
EE conv_ws_ready(Ctx &c)
{
    if (c.conv_ws_dirty) {
        HIP_TRY(launch_fill_u32(c.conv_ws[0], 2 * kWsWords, 0, c.stream));
        c.conv_ws_dirty = false;
    }
    return SUCCESS;
}

// all pointers device
EE conv_device_ext(const ConvShape &s, DataFormat idf, const void *input, const void *eltwise, const void *filter,
    const void *bias, void *tmp, DataType odt, DataFormat odf, void *output, int relu, const ConvExt &x)
{
    Ctx &c = ctx();
    U8 *t = (U8 *)tmp;
    const bool direct = conv_panel_ok(s.oc, s.Kp) && s.ic % 16 == 0 && (((uintptr_t)input) & 15) == 0;
    if (!direct) {
        HIP_TRY(launch_conv_pad((const uint8_t *)input, s.n, s.ic, s.ih, s.iw, idf == DF_NCHWC16 ? 16 : 8, s.pt, s.pb, s.pl,
            s.pr, (int8_t *)t, c.stream, nullptr));
    }
    const int32_t *offC = (const int32_t *)filter;
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
    g.Bp = (const int8_t *)filter + (size_t)s.oc * 4;
    g.M = s.n * s.oh * s.ow;
    g.N = s.oc;
    g.K = s.Kp;
    g.ob = offC;
    g.comp = offC;
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
    g.conv.dscaleI = x.dscaleI;
    g.conv.scaleI = x.scaleI;
    g.conv.dscale_out = x.dscaleO;
    const bool per_channel = x.scaleW != nullptr;
    if (per_channel) {
        g.epi.mode = EPI_CONV_CH;
        g.epi.scaleW = x.scaleW;
        g.epi.bias = (const float *)bias;
    } else {
        // one filter scale: the reference's arithmetic (bias folded into the integer offset with the accumulators'
        // scale, convolution_direct.cpp:2687-2700), that scale formed on the device when the input scale lives there
        g.fold_bias = (const float *)bias;
        g.conv.filter_scale = x.filterScale;
        g.conv.scaleO = x.scaleI * x.filterScale;
        g.fold_scale = g.conv.scaleO;
    }
    if (odt == DT_F32 || odt == DT_I32) {
        g.C = output;
        if (per_channel) {
            g.conv.ch_out = CONV_CH_F32;
            g.conv.eltwise = (const float *)eltwise;
        } else if (odt == DT_F32) {
            g.epi.mode = EPI_F32;
            g.epi.factor = 1 / g.conv.scaleO;
            g.conv.eltwise = (const float *)eltwise;
        } else {
            g.epi.mode = EPI_I32;
        }
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        return SUCCESS;
    }
    // u8 result with one output scale
    if (per_channel && x.staticOut > 0) {
        g.C = output;
        g.conv.ch_out = CONV_CH_U8;
        g.epi.factor = x.staticOut;
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        return SUCCESS;
    }
    EE e = conv_ws_ready(c);
    if (e != SUCCESS) {
        return e;
    }
    // ONE pass where the filter-panel kernel runs and all its workgroups are resident at once: they agree on the
    // tensor-wide maximum with their values still in registers (the convolution is computed once instead of twice)
    const uint32_t M_pix = s.n * s.oh * s.ow;
    const bool onepass = direct && conv_panel_grid(M_pix) <= conv_onepass_max_grid(s.Kp) && (x.host_waits || x.spill);
    if (onepass) {
        g.C = output;
        g.C32 = (float *)x.spill;
        g.conv.absmax = c.conv_ws[c.conv_ws_next];  // touched only if the agreement is abandoned; left clear again
        g.sync = c.fsync.next(conv_panel_grid(M_pix));
        if (per_channel) {
            g.conv.ch_out = CONV_CH_U8;
            g.epi.factor = 0;
        } else {
            g.epi.mode = EPI_U8;
        }
        HIP_TRY(launch_conv_u8s8(g, c.stream));
        if (!x.host_waits) {
            return SUCCESS;
        }
        bool gave_up = false;
        float got = 0;
        EE te = take_scale(c, &got, &gave_up);
        if (te != SUCCESS) {
            return te;
        }
        if (!gave_up) {
            *x.host_scale = got;
            return SUCCESS;
        }
        // the bounded wait expired (other work held the CUs): nothing was stored, the two passes below redo it
        g_fused_fallbacks.fetch_add(1);
        memset(&g.sync, 0, sizeof(g.sync));
        arm_scale(c);
    }
    uint32_t *mine = c.conv_ws[c.conv_ws_next], *other = c.conv_ws[c.conv_ws_next ^ 1];
    c.conv_ws_dirty = true;  // until both passes are enqueued
    g.conv.absmax = mine;
    float *publish = g.conv.dscale_out;
    g.conv.dscale_out = nullptr;
    g.C = nullptr;
    if (per_channel) {
        g.conv.ch_out = CONV_CH_MAX;
    } else {
        g.epi.mode = EPI_I32;  // abs-max pass: nothing stored
    }
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    g.C = output;
    g.conv.dscale_out = publish;
    g.clear_ws = other;
    if (per_channel) {
        g.conv.ch_out = CONV_CH_U8;
        g.epi.factor = 0;
    } else {
        g.epi.mode = EPI_U8;
    }
    HIP_TRY(launch_conv_u8s8(g, c.stream));
    c.conv_ws_next ^= 1;
    c.conv_ws_dirty = false;
    return x.host_waits ? take_scale(c, x.host_scale) : SUCCESS;
}

EE check_common(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc, ActivationParamSpec act,
    const void *eltwiseInput, bool allow_i32)
{
    if (outputDesc.df != DF_NCHWC16 && outputDesc.df != DF_NCHWC8) {
        return NOT_MATCH;
    }
    if (inputDesc.dt != DT_U8_Q || filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHWC2NxC4) {
        return NOT_MATCH;
    }
    if (inputDesc.df != DF_NCHWC8 && inputDesc.df != DF_NCHWC16) {
        return NOT_SUPPORTED;
    }
    const DataType odt = outputDesc.dt;
    if (odt != DT_F32 && odt != DT_U8_Q && !(allow_i32 && odt == DT_I32)) {
        return NOT_SUPPORTED;
    }
    if (act.mode != ACTIVATION_NULL && act.mode != ACTIVATION_RELU) {
        return NOT_SUPPORTED;
    }
    if (eltwiseInput && odt != DT_F32) {
        return NOT_SUPPORTED;
    }
    return SUCCESS;
}

}  // namespace

extern "C" {

EE bolt_gfx950_convolution_int8_perchannel(TensorDesc inputDesc, const void *input, const void *eltwiseInput,
    TensorDesc filterDesc, const void *filter, ConvolutionParamSpec p, const F32 *scaleW, TensorDesc biasDesc,
    const void *bias, U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *output, F32 *scale,
    ActivationParamSpec activationDesc, Arch arch)
{
    (void)biasDesc;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!input || !filter || !output || !tmp || !scale || !scaleW) {
        return NULL_POINTER;
    }
    EE e = check_common(inputDesc, filterDesc, outputDesc, activationDesc, eltwiseInput, false);
    if (e != SUCCESS) {
        return e;
    }
    if (!(scale[0] > 0)) {
        return fail(NOT_MATCH, "the input scale (scale[0]) must be positive");
    }
    ConvShape s;
    e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
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
    Ctx &cx = ctx();
    const DataType odt = outputDesc.dt;
    const int relu = (activationDesc.mode == ACTIVATION_RELU);
    ConvExt x;
    x.scaleI = scale[0];
    x.staticOut = (odt == DT_U8_Q && scale[1] > 0) ? scale[1] : 0.0f;
    const bool dynamic = odt == DT_U8_Q && !(x.staticOut > 0);
    if (dynamic) {
        x.dscaleO = cx.hscale_dev;  // the new output scale goes straight into pinned host memory
        x.host_waits = true;
        x.host_scale = &scale[1];
    }
    if (arch == AMD_GFX950_DEVICE) {
        if (((uintptr_t)tmp & 15) || ((uintptr_t)filter & 15) || ((uintptr_t)output & 15) || ((uintptr_t)input & 7)) {
            return fail(NOT_SUPPORTED, "device tmp / filter / output must be 16-byte aligned, input 8-byte aligned");
        }
        x.scaleW = scaleW;
        if (dynamic) {
            arm_scale(cx);
        }
        return conv_device_ext(s, inputDesc.df, input, eltwiseInput, filter, bias, tmp, odt, outputDesc.df, output, relu, x);
    }
    Stage st;
    const size_t inB = (size_t)s.n * s.ic * s.ih * s.iw;
    const size_t fB = (size_t)s.oc * 4 + (size_t)s.N16 * s.Kp;
    const size_t outN = (size_t)s.n * s.oc * s.oh * s.ow;
    const size_t outB = outN * (odt == DT_U8_Q ? 1 : 4);
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = bias ? st.get((size_t)s.oc * 4) : nullptr, *dT = st.get(need);
    void *dO = st.get(outB), *dW = st.get((size_t)s.oc * 4);
    void *dE = eltwiseInput ? st.get(outN * 4) : nullptr;
    if (!dIn || !dF || (bias && !dB) || !dT || !dO || !dW || (eltwiseInput && !dE)) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, input, inB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dF, filter, fB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dW, scaleW, (size_t)s.oc * 4, hipMemcpyHostToDevice, cx.stream));
    if (dB) {
        HIP_TRY(hipMemcpyAsync(dB, bias, (size_t)s.oc * 4, hipMemcpyHostToDevice, cx.stream));
    }
    if (dE) {
        HIP_TRY(hipMemcpyAsync(dE, eltwiseInput, outN * 4, hipMemcpyHostToDevice, cx.stream));
    }
    x.scaleW = (const float *)dW;
    if (dynamic) {
        arm_scale(cx);
    }
    e = conv_device_ext(s, inputDesc.df, dIn, dE, dF, dB, dT, odt, outputDesc.df, dO, relu, x);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(output, dO, outB, hipMemcpyDeviceToHost, cx.stream));
    HIP_TRY(hipStreamSynchronize(cx.stream));
    return SUCCESS;
}

EE bolt_gfx950_convolution_async_tmp_bytes(TensorDesc inputDesc, TensorDesc filterDesc, TensorDesc outputDesc,
    ConvolutionParamSpec p, U32 *bytes)
{
    if (!bytes) {
        return NULL_POINTER;
    }
    ConvShape s;
    EE e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
    if (e != SUCCESS) {
        return e;
    }
    size_t spill_off;
    const size_t total = conv_async_tmp_layout(s, &spill_off);
    if (total > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)total;
    return SUCCESS;
}

EE bolt_gfx950_convolution_async(TensorDesc inputDesc, const void *input, const void *eltwiseInput, TensorDesc filterDesc,
    const void *filter, ConvolutionParamSpec p, TensorDesc biasDesc, const void *bias, U32 tmpBytes, void *tmp,
    TensorDesc outputDesc, void *output, const float *dscaleI, F32 filterScale, const F32 *scaleW, float *dscaleO,
    F32 staticOutputScale, ActivationParamSpec activationDesc)
{
    (void)biasDesc;
    if (!input || !filter || !output || !tmp || !dscaleI) {
        return NULL_POINTER;
    }
    if (!scaleW && !bias) {
        return NULL_POINTER;  // the one-scale form folds the bias as the reference does and needs one (x86/int8/convolution.cpp:114-117)
    }
    EE e = check_common(inputDesc, filterDesc, outputDesc, activationDesc, eltwiseInput, !scaleW);
    if (e != SUCCESS) {
        return e;
    }
    const DataType odt = outputDesc.dt;
    if (odt == DT_U8_Q && !dscaleO) {
        return NULL_POINTER;
    }
    if (!scaleW && !(filterScale > 0)) {
        return fail(NOT_MATCH, "the filter scale must be positive");
    }
    if (staticOutputScale > 0 && !(scaleW && odt == DT_U8_Q)) {
        return fail(NOT_SUPPORTED, "a static output scale applies to the per-channel form with a u8 result");
    }
    ConvShape s;
    e = conv_shape(inputDesc, filterDesc, outputDesc, p, &s);
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
    if (((uintptr_t)tmp & 15) || ((uintptr_t)filter & 15) || ((uintptr_t)output & 15) || ((uintptr_t)input & 7)) {
        return fail(NOT_SUPPORTED, "device tmp / filter / output must be 16-byte aligned, input 8-byte aligned");
    }
    ConvExt x;
    x.dscaleI = dscaleI;
    x.scaleW = scaleW;
    x.filterScale = filterScale;
    x.staticOut = staticOutputScale;
    x.dscaleO = dscaleO;
    size_t spill_off;
    if (tmpBytes >= conv_async_tmp_layout(s, &spill_off)) {
        x.spill = (U8 *)tmp + spill_off;  // room for the one-pass form's parking area
    }
    return conv_device_ext(s, inputDesc.df, input, eltwiseInput, filter, bias, tmp, odt, outputDesc.df, output,
        activationDesc.mode == ACTIVATION_RELU, x);
}

}  // extern "C"
