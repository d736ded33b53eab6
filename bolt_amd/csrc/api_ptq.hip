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

EE bolt_gfx950_operator_scales(const QuantSpec *featureScale, U32 numQuantFeature, DataType inputDataType,
    F32 inputTensorScale, F32 filterScale, F32 scales[3], int *labelledNoQuant)
{
    if (!scales || (numQuantFeature && !featureScale)) {
        return NULL_POINTER;
    }
    for (U32 i = 0; i < numQuantFeature; ++i) {
        if (featureScale[i].num_scale < 1 || !featureScale[i].scale) {
            return NOT_MATCH;
        }
    }
    // inference/engine/include/cpu/convolution_cpu.hpp:143-157 (fully_connected_cpu.hpp and deconvolution_cpu.hpp:65-84
    // apply the same rule): the input scale is the producing tensor's unless the input still has to be quantised and
    // the record carries a positive calibrated scale; the output scale is the last record's, -2 meaning "leave it to
    // the operator" (dynamic, -1)
    scales[0] = inputTensorScale;
    if (inputDataType != DT_I8 && inputDataType != DT_U8_Q && numQuantFeature > 0 && featureScale[0].scale[0] > 0) {
        scales[0] = featureScale[0].scale[0];
    }
    if (numQuantFeature > 0 && featureScale[numQuantFeature - 1].scale[0] != -2) {
        scales[1] = featureScale[numQuantFeature - 1].scale[0];
    } else {
        scales[1] = -1;
    }
    scales[2] = filterScale;
    if (labelledNoQuant) {
        // inference/engine/include/operator.hpp:164-169: a first record of 0 labels the operator as not quantised
        *labelledNoQuant = (numQuantFeature != 0 && featureScale[0].scale[0] == 0) ? 1 : 0;
    }
    return SUCCESS;
}

}  // extern "C"
