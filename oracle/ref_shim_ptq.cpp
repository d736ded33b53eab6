// TEST INFRASTRUCTURE ONLY. Flat C entry points over the weight-storage arithmetic of the reference's post-training
// quantisation tool (model_tools/src/model_data_type_converter.cpp:22-103) and the load-time expansion of such weights
// (common/model_spec/src/model_deserialize.cpp:162-222), compiled where they lie under /root/reference by
// oracle/Makefile into oracle/_ref/libboltref.so. No arithmetic happens here. Nothing in the product may load this.
#include <cstdint>
#include <cstdlib>
#include <cstring>
#include "data_type.h"
#include "model_spec.h"

// defined (without a header of their own) in the two reference sources named above
F32 ws_datatype_converter_bnn(U8 *originalPtr, U8 *targetPtr, int paramNum);
void ws_datatype_converter_int8(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale);
void ws_datatype_converter_int4(U8 *originalPtr, U8 *targetPtr, int paramNum, F32 *scale);
template <DataType dt, typename T>
void dequantize_int8_weight(int num, F32 scale, INT8 *q, T *d);
template <DataType dt, typename T>
void dequantize_int4_weight(int num, F32 scale, INT8 *q, T *d);
void dequantize_int4_int8(int num, INT8 *q, INT8 *d);
void dequantize_int4_u8_q(int num, INT8 *q, UINT8 *d);
extern template void dequantize_int8_weight<DT_F32, F32>(int, F32, INT8 *, F32 *);

// the model loader's own expansion of a stored weight (common/model_spec/src/model_deserialize.cpp:270-331), which it
// applies to every WeightSpec whose stored type the target cannot compute in (:400-470)
void TransWeightFromI4ToF32(WeightSpec *ptr, INT8 *src);
void TransWeightFromI4ToI8(WeightSpec *ptr, INT8 *src);
void TransWeightFromI4ToU8(WeightSpec *ptr, INT8 *src);
void TransWeightFromI8ToF32(WeightSpec *ptr, INT8 *src);

extern "C" {

// kind 0: stored int8 -> fp32, 1: stored int4 -> fp32, 2: stored int4 -> s8, 3: stored int4 -> u8 (zero point 128).
// stored: the weight bytes as the .bolt file holds them; *scale: the WeightSpec's one weight scale (in / out: the
// loader zeroes it when it hands back fp32). Returns the loader's new bytes_of_weight; the expanded weight is copied
// to out (which must hold that many bytes).
unsigned ref_loader_expand_weight(int kind, const int8_t *stored, unsigned stored_bytes, float *scale, void *out)
{
    WeightSpec ws;
    memset(ws.op_name, 0, sizeof(ws.op_name));
    QuantSpec q;
    q.num_scale = 1;
    q.scale = scale;
    ws.mdt = kind == 0 ? DT_I8 : DT_I4;
    ws.bytes_of_weight = stored_bytes;
    ws.weight = nullptr;
    ws.num_quant_scale = 1;
    ws.weight_scale = &q;
    switch (kind) {
        case 0:
            TransWeightFromI8ToF32(&ws, (INT8 *)stored);
            break;
        case 1:
            TransWeightFromI4ToF32(&ws, (INT8 *)stored);
            break;
        case 2:
            TransWeightFromI4ToI8(&ws, (INT8 *)stored);
            break;
        default:
            TransWeightFromI4ToU8(&ws, (INT8 *)stored);
            break;
    }
    memcpy(out, ws.weight, ws.bytes_of_weight);
    operator delete(ws.weight);  // mt_malloc is operator new (model_common.h:21-24)
    return ws.bytes_of_weight;
}

float ref_ws_convert_bnn(const float *w, int n, uint8_t *bits)
{
    return ws_datatype_converter_bnn((U8 *)w, bits, n);
}

void ref_ws_convert_int8(const float *w, int n, int8_t *q, float *scale)
{
    ws_datatype_converter_int8((U8 *)w, (U8 *)q, n, scale);
}

void ref_ws_convert_int4(const float *w, int n, int8_t *q, float *scale)
{
    ws_datatype_converter_int4((U8 *)w, (U8 *)q, n, scale);
}

void ref_dequantize_int8_weight(int n, float scale, const int8_t *q, float *d)
{
    dequantize_int8_weight<DT_F32, F32>(n, scale, (INT8 *)q, d);
}

void ref_dequantize_int4_int8(int n, const int8_t *q, int8_t *d)
{
    dequantize_int4_int8(n, (INT8 *)q, d);
}

void ref_dequantize_int4_u8q(int n, const int8_t *q, uint8_t *d)
{
    dequantize_int4_u8_q(n, (INT8 *)q, d);
}
}
