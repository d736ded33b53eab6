// TEST INFRASTRUCTURE ONLY. Flat C entry points over the weight-storage arithmetic of the reference's post-training
// quantisation tool (model_tools/src/model_data_type_converter.cpp:22-103) and the load-time expansion of such weights
// (common/model_spec/src/model_deserialize.cpp:162-222), compiled where they lie under /root/reference by
// oracle/Makefile into oracle/_ref/libboltref.so. No arithmetic happens here. Nothing in the product may load this.
#include <cstdint>
#include "data_type.h"

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

extern "C" {

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
