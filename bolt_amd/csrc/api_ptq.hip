// C-ABI entry points for the weight-storage arithmetic of the post-training quantisation tool and for the load-time
// expansion of stored weights, plus the engine's rule that turns an operator's stored QuantSpec records into the
// scale array its int8 operators are called with.
#include <cstring>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

namespace {

// stage in / run / stage out for an element-wise call: `run` gets device pointers
template <typename F>
EE elementwise(Arch arch, const void *in, size_t inB, void *out, size_t outB, F run)
{
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    if (arch == AMD_GFX950_DEVICE) {
        return run(in, out);
    }
    Ctx &c = ctx();
    Stage st;
    void *dIn = st.get(inB), *dOut = st.get(outB);
    if (!dIn || !dOut) {
        return fail(ALLOC_FAILED, "device staging");
    }
    HIP_TRY(hipMemcpyAsync(dIn, in, inB, hipMemcpyHostToDevice, c.stream));
    e = run(dIn, dOut);
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(hipMemcpyAsync(out, dOut, outB, hipMemcpyDeviceToHost, c.stream));
    HIP_TRY(hipStreamSynchronize(c.stream));
    return SUCCESS;
}

}  // namespace

extern "C" {

EE ws_datatype_converter_int8_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!originalPtr || !targetPtr || !scale) {
        return NULL_POINTER;
    }
    if (paramNum <= 0) {
        return NOT_MATCH;
    }
    const uint32_t n = (uint32_t)paramNum;
    const float floor_ = *scale;
    return elementwise(arch, originalPtr, (size_t)n * 4, targetPtr, n, [&](const void *in, void *out) -> EE {
        Ctx &c = ctx();
        arm_scale(c);
        HIP_TRY(launch_ws_int8((const float *)in, n, (int8_t *)out, c.ws, floor_, c.hscale_dev, c.stream));
        return take_scale(c, scale);
    });
}

EE ws_datatype_converter_int4_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!originalPtr || !targetPtr || !scale) {
        return NULL_POINTER;
    }
    if (paramNum <= 0) {
        return NOT_MATCH;
    }
    if (paramNum % 2) {
        // the reference stores the odd trailing element one byte too far and without its +7 offset
        // (model_data_type_converter.cpp:99-101): not a format anything reads back
        return NOT_SUPPORTED;
    }
    const uint32_t n = (uint32_t)paramNum;
    const float floor_ = *scale;
    return elementwise(arch, originalPtr, (size_t)n * 4, targetPtr, n / 2, [&](const void *in, void *out) -> EE {
        Ctx &c = ctx();
        arm_scale(c);
        HIP_TRY(launch_ws_int4((const float *)in, n, (int8_t *)out, c.ws, floor_, c.hscale_dev, c.stream));
        return take_scale(c, scale);
    });
}

EE ws_datatype_converter_bnn_gfx950(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!originalPtr || !targetPtr || !scale) {
        return NULL_POINTER;
    }
    if (paramNum <= 0 || paramNum % 8) {
        return NOT_MATCH;  // the reference reads whole groups of 8 (:26-37)
    }
    const uint32_t n = (uint32_t)paramNum;
    return elementwise(arch, originalPtr, (size_t)n * 4, targetPtr, n / 8, [&](const void *in, void *out) -> EE {
        Ctx &c = ctx();
        arm_scale(c);
        HIP_TRY(launch_ws_bnn((const float *)in, n, (uint8_t *)out, c.ws, c.hscale_dev, c.stream));
        return take_scale(c, scale);
    });
}

static EE expand(int num, F32 scale, const void *q, int src4, int dst, void *d, Arch arch)
{
    if (!IS_GFX950(arch)) {
        return NOT_SUPPORTED;
    }
    if (!q || !d) {
        return NULL_POINTER;
    }
    if (num <= 0) {
        return NOT_MATCH;
    }
    const uint32_t n = (uint32_t)num;
    const size_t inB = src4 ? (n + 1) / 2 : n, outB = (size_t)n * (dst == 0 ? 4 : 1);
    return elementwise(arch, q, inB, d, outB, [&](const void *in, void *out) -> EE {
        HIP_TRY(launch_ws_expand((const int8_t *)in, n, src4, dst, scale, out, ctx().stream));
        return SUCCESS;
    });
}

EE dequantize_int8_weight_gfx950(int num, F32 scale, INT8 *q, F32 *d, Arch arch)
{
    return expand(num, scale, q, 0, 0, d, arch);
}

EE dequantize_int4_weight_gfx950(int num, F32 scale, INT8 *q, F32 *d, Arch arch)
{
    return expand(num, scale, q, 1, 0, d, arch);
}

EE dequantize_int4_int8_gfx950(int num, INT8 *q, INT8 *d, Arch arch)
{
    return expand(num, 1.0f, q, 1, 1, d, arch);
}

EE dequantize_int4_u8_q_gfx950(int num, INT8 *q, UINT8 *d, Arch arch)
{
    // nibble + 121 = (nibble - 7) + 128
    return expand(num, 1.0f, q, 1, 2, d, arch);
}

EE bolt_gfx950_operator_scales(int operatorKind, const QuantSpec *featureScale, U32 numQuantFeature, DataType inputDataType,
    DataType outputDataType, F32 inputTensorScale, F32 filterScale, F32 scales[3], int *labelledNoQuant)
{
    if (!scales || (numQuantFeature && !featureScale)) {
        return NULL_POINTER;
    }
    if (operatorKind != BOLT_GFX950_OP_CONVOLUTION && operatorKind != BOLT_GFX950_OP_FULLY_CONNECTED &&
        operatorKind != BOLT_GFX950_OP_DECONVOLUTION) {
        return NOT_SUPPORTED;
    }
    for (U32 i = 0; i < numQuantFeature; ++i) {
        if (featureScale[i].num_scale < 1 || !featureScale[i].scale) {
            return NOT_MATCH;
        }
    }
    const bool inQuantised = inputDataType == DT_I8 || inputDataType == DT_U8_Q;
    const bool outQuantised = outputDataType == DT_I8 || outputDataType == DT_U8_Q;
    const F32 first = numQuantFeature ? featureScale[0].scale[0] : 0.0f;
    const F32 last = numQuantFeature ? featureScale[numQuantFeature - 1].scale[0] : 0.0f;
    scales[0] = inputTensorScale;
    scales[2] = filterScale;
    if (operatorKind == BOLT_GFX950_OP_CONVOLUTION) {
        // inference/engine/include/cpu/convolution_cpu.hpp:143-157: one record is enough for the calibrated input scale;
        // the last record is the output scale whatever the output type, -2 there (or no record) leaves it dynamic
        if (!inQuantised && numQuantFeature > 0 && first > 0) {
            scales[0] = first;
        }
        scales[1] = (numQuantFeature > 0 && last != -2) ? last : -1.0f;
    } else {
        // fully_connected_cpu.hpp:92-103 and deconvolution_cpu.hpp:70-84: the calibrated input scale needs MORE than one
        // record (a single record is the output's), the output scale is set only for a quantised output type, and the
        // last record goes through as it is (-2 included)
        if (!inQuantised && numQuantFeature > 1 && first > 0) {
            scales[0] = first;
        }
        if (outQuantised) {
            scales[1] = numQuantFeature > 0 ? last : -1.0f;
        } else {
            // FullyConnected leaves the output tensor's scale alone (reported as -1: nothing to set); the deconvolution's
            // `F32 scales[3] = {-1}` leaves a zero in slot 1 (deconvolution_cpu.hpp:65)
            scales[1] = operatorKind == BOLT_GFX950_OP_DECONVOLUTION ? 0.0f : -1.0f;
        }
    }
    if (labelledNoQuant) {
        // inference/engine/include/operator.hpp:164-169: a first record of 0 labels the operator as not quantised
        *labelledNoQuant = (numQuantFeature != 0 && first == 0) ? 1 : 0;
    }
    return SUCCESS;
}

}  // extern "C"
