// C-ABI entry points of the int8 depthwise convolution (the part of the reference's unfinished x86 path that has a
// defined result): filter transform in the reference's own blob layout, and the int32-result convolution.
#include <cstring>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

extern "C" {

EE depthwise_convolution_transform_filter_bytes_int8_gfx950(TensorDesc filterDesc, U32 *bytes, Arch arch)
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
    if (filterDesc.dt != DT_I8 || fn != 1) {
        return NOT_SUPPORTED;
    }
    // depthwise_pointwise_convolution.cpp:197-205: ALIGN(fh * fw, 4) * fn * fc + 32 + fc * 4
    const uint64_t b = (uint64_t)align_up(fh * fw, 4) * fn * fc + 32 + (uint64_t)fc * 4;
    if (b > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    *bytes = (U32)b;
    return SUCCESS;
}

EE depthwise_convolution_transform_filter_int8_gfx950(TensorDesc filterDesc, const INT8 *filter, TensorDesc *ftmDesc,
    INT8 *filterTransformed, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!filter || !ftmDesc || !filterTransformed) {
        return NULL_POINTER;
    }
    U32 fn, fc, fh, fw;
    if (get4d(filterDesc, &fn, &fc, &fh, &fw) != SUCCESS) {
        return NOT_MATCH;
    }
    if (filterDesc.dt != DT_I8 || filterDesc.df != DF_NCHW || fn != 1 || fc % 16 != 0) {
        return NOT_SUPPORTED;
    }
    const U32 taps = fh * fw, tp = align_up(taps, 4);
    const size_t blobBytes = (size_t)fc * 4 + (size_t)tp * fc;
    std::vector<INT8> hostBlob;
    INT8 *dst = filterTransformed;
    const INT8 *src = filter;
    std::vector<INT8> hostSrc;
    if (arch == AMD_GFX950_DEVICE) {
        // load-time, a few KB: pack on the host and copy the blob over
        EE e = ensure_init();
        if (e != SUCCESS) {
            return e;
        }
        hostSrc.resize((size_t)fc * taps);
        HIP_TRY(hipMemcpyAsync(hostSrc.data(), filter, hostSrc.size(), hipMemcpyDeviceToHost, ctx().stream));
        HIP_TRY(hipStreamSynchronize(ctx().stream));
        src = hostSrc.data();
        hostBlob.resize(blobBytes);
        dst = hostBlob.data();
    }
    // x86/int8/depthwise_convolution_transform.cpp:37-66: [offsetC fc*4][per 16 channels: [tap / 4][channel][tap % 4]]
    I32 *offsetC = (I32 *)dst;
    INT8 *mat = dst + (size_t)fc * 4;
    memset(mat, 0, (size_t)tp * fc);
    for (U32 c = 0; c < fc; ++c) {
        I32 sum = 0;
        for (U32 t = 0; t < taps; ++t) {
            const INT8 v = src[(size_t)c * taps + t];
            sum += v;
            mat[(size_t)(c / 16) * 16 * tp + (size_t)(t / 4) * 64 + (c % 16) * 4 + t % 4] = v;
        }
        offsetC[c] = -128 * sum;
    }
    if (arch == AMD_GFX950_DEVICE) {
        HIP_TRY(hipMemcpyAsync(filterTransformed, hostBlob.data(), blobBytes, hipMemcpyHostToDevice, ctx().stream));
        HIP_TRY(hipStreamSynchronize(ctx().stream));
    }
    *ftmDesc = tensor4df(DT_I8, DF_NCHWN8HW4, fc, 1, fh, fw);  // :21,34 (the tag the reference uses for this layout)
    return SUCCESS;
}

EE depthwise_pointwise_convolution_int8_gfx950(TensorDesc inputDesc, UINT8 *inArray, F32 *eltwiseInput,
    TensorDesc dwFilterDesc, const INT8 *dwFilterArray, TensorDesc pwFilterDesc, const INT8 *pwFilterArray,
    ConvolutionParamSpec p, TensorDesc dwBiasDesc, const F32 *dwBiasArray, TensorDesc pwBiasDesc, const F32 *pwBiasArray,
    U32 tmpBytes, void *tmp, TensorDesc outputDesc, void *outArray, F32 *scale, ActivationParamSpec dwAct,
    ActivationParamSpec pwAct, Arch arch)
{
    (void)pwFilterDesc;
    (void)dwBiasDesc;
    (void)pwBiasDesc;
    (void)pwBiasArray;
    (void)tmpBytes;
    (void)tmp;
    (void)pwAct;
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!inArray || !dwFilterArray || !outArray || !scale) {
        return NULL_POINTER;
    }
    // What the reference's kernel defines (depthwise_convolution_direct.cpp:441-599): int32 results of the depthwise
    // stage alone. Its fp32 epilogue converts the scale factor's bits instead of the accumulators (:148-166), a
    // quantised result stays in tmp (:521-525) and the pointwise stage is never run -- none of those has a result to match.
    if (pwFilterArray || eltwiseInput || outputDesc.dt != DT_I32) {
        return NOT_SUPPORTED;
    }
    if (inputDesc.dt != DT_U8_Q || inputDesc.df != DF_NCHWC16 || outputDesc.df != DF_NCHWC16 || dwFilterDesc.dt != DT_I8 ||
        dwFilterDesc.df != DF_NCHWN8HW4) {
        return NOT_MATCH;  // :472-474
    }
    if (dwAct.mode != ACTIVATION_NULL && dwAct.mode != ACTIVATION_RELU) {
        return NOT_SUPPORTED;
    }
    DepthwiseArgs a;
    U32 on, oc, fn, fc;
    if (get4d(inputDesc, &a.n, &a.c, &a.ih, &a.iw) != SUCCESS || get4d(outputDesc, &on, &oc, &a.oh, &a.ow) != SUCCESS ||
        get4d(dwFilterDesc, &fn, &fc, &a.fh, &a.fw) != SUCCESS) {
        return NOT_MATCH;
    }
    const U32 dh = p.dilatedRate_h ? p.dilatedRate_h : 1, dw = p.dilatedRate_w ? p.dilatedRate_w : 1;
    if (on != a.n || oc != a.c || (fn != a.c && fc != a.c) || a.c % 16 != 0 || p.stride_h == 0 || p.stride_w == 0) {
        return NOT_MATCH;
    }
    if (p.pad_top || p.pad_bottom || p.pad_left || p.pad_right || dh != 1 || dw != 1) {
        // the reference's gather ignores both (:560-566): with them set its result is not a convolution
        return NOT_SUPPORTED;
    }
    a.sh = p.stride_h;
    a.sw = p.stride_w;
    if (a.oh == 0 || a.ow == 0 || (uint64_t)(a.oh - 1) * a.sh + a.fh > a.ih || (uint64_t)(a.ow - 1) * a.sw + a.fw > a.iw) {
        return NOT_MATCH;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &cx = ctx();
    a.scaleO = scale[0] * scale[2];
    a.relu = dwAct.mode == ACTIVATION_RELU;
    const size_t inB = (size_t)a.n * a.c * a.ih * a.iw, outB = (size_t)a.n * a.c * a.oh * a.ow * 4;
    const size_t fB = (size_t)a.c * 4 + (size_t)align_up(a.fh * a.fw, 4) * a.c;
    if (arch == AMD_GFX950_DEVICE) {
        if (((uintptr_t)inArray & 15) || ((uintptr_t)dwFilterArray & 15) || ((uintptr_t)outArray & 15) ||
            ((uintptr_t)dwBiasArray & 3)) {
            return fail(NOT_SUPPORTED, "device input / filter / output must be 16-byte aligned");
        }
        a.in = inArray;
        a.offsetC = (const int32_t *)dwFilterArray;
        a.filter = (const int8_t *)dwFilterArray + (size_t)a.c * 4;
        a.bias = dwBiasArray;
        a.out = (int32_t *)outArray;
        HIP_TRY(launch_depthwise_u8s8_i32(a, cx.stream));
        scale[1] = a.scaleO;  // :507
        return SUCCESS;
    }
    Stage st;
    void *dIn = st.get(inB), *dF = st.get(fB), *dB = dwBiasArray ? st.get((size_t)a.c * 4) : nullptr, *dO = st.get(outB);
    if (!dIn || !dF || !dO || (dwBiasArray && !dB)) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, inArray, inB, hipMemcpyHostToDevice, cx.stream));
    HIP_TRY(hipMemcpyAsync(dF, dwFilterArray, fB, hipMemcpyHostToDevice, cx.stream));
    if (dB) {
        HIP_TRY(hipMemcpyAsync(dB, dwBiasArray, (size_t)a.c * 4, hipMemcpyHostToDevice, cx.stream));
    }
    a.in = (const uint8_t *)dIn;
    a.offsetC = (const int32_t *)dF;
    a.filter = (const int8_t *)dF + (size_t)a.c * 4;
    a.bias = (const float *)dB;
    a.out = (int32_t *)dO;
    HIP_TRY(launch_depthwise_u8s8_i32(a, cx.stream));
    HIP_TRY(hipMemcpyAsync(outArray, dO, outB, hipMemcpyDeviceToHost, cx.stream));
    HIP_TRY(hipStreamSynchronize(cx.stream));
    scale[1] = a.scaleO;
    return SUCCESS;
}

}  // extern "C"
