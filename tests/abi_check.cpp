// Compile-time check of include/bolt_gfx950.h and include/bolt_types.h against the reference's own headers.
// Built (syntax only) by `make -C oracle abi`, which tests/test_abi_check.py runs where /root/reference exists.
//
//  1. The prototypes, taken with BOLT_GFX950_NO_TYPES over the reference's types, must have exactly the argument
//     list of the function they replace (blas_enhance.h: identical; the inner tensor_computing forms: identical, or
//     identical plus a trailing Arch where the reference's per-architecture function has none).
//  2. Our stand-alone type header must describe the same bytes: struct sizes, field offsets and every enum value used.
#include <cstddef>
#include <cstdint>
#include <cstring>
#include <stdbool.h>
#include <stdint.h>
#include <string.h>
#include <type_traits>

#include "blas_enhance.h"
#include "tensor_computing.h"
#include "cpu/tensor_computing_cpu.h"
#include "cpu/x86/tensor_computing_x86.h"
#include "cpu/x86/int8/tensor_computing_int8.h"
#include "parameter_spec.h"

#define BOLT_GFX950_NO_TYPES
#include "bolt_gfx950.h"
#undef BOLT_GFX950_NO_TYPES

namespace ours {
#include "bolt_types.h"
}

template <class F>
struct add_arch;
template <class Ret, class... A>
struct add_arch<Ret (*)(A...)> {
    typedef Ret (*type)(A..., Arch);
};

#define SAME(ref, mine) static_assert(std::is_same<decltype(&ref), decltype(&mine)>::value, #mine " differs from " #ref)
#define SAME_PLUS_ARCH(ref, mine) \
    static_assert(std::is_same<add_arch<decltype(&ref)>::type, decltype(&mine)>::value, #mine " is not " #ref " + Arch")

// ---- compute/blas_enhance/include/blas_enhance.h:25-85: all eleven ------------------------------------------------
SAME(vector_vector_axpby, vector_vector_axpby_gfx950);
SAME(matrix_matrix_multiply_tmp_bytes, matrix_matrix_multiply_tmp_bytes_gfx950);
SAME(matrix_matrix_multiply, matrix_matrix_multiply_gfx950);
SAME(matrix_vector_multiply_tmp_bytes, matrix_vector_multiply_tmp_bytes_gfx950);
SAME(matrix_vector_multiply, matrix_vector_multiply_gfx950);
SAME(matrix_matrix_multiply_rhs_format, matrix_matrix_multiply_rhs_format_gfx950);
SAME(matrix_matrix_multiply_transform_rhs_bytes, matrix_matrix_multiply_transform_rhs_bytes_gfx950);
SAME(matrix_matrix_multiply_transform_rhs, matrix_matrix_multiply_transform_rhs_gfx950);
SAME(matrix_vector_multiply_weight_format, matrix_vector_multiply_weight_format_gfx950);
SAME(matrix_vector_multiply_transform_weight_bytes, matrix_vector_multiply_transform_weight_bytes_gfx950);
SAME(matrix_vector_multiply_transform_weight, matrix_vector_multiply_transform_weight_gfx950);

// ---- inner (TensorDesc + pointer) forms of tensor_computing ---------------------------------------------------------
SAME_PLUS_ARCH(quantize_x86, quantize_gfx950);                       // cpu/x86/tensor_computing_x86.h
SAME_PLUS_ARCH(dequantize_x86, dequantize_gfx950);
SAME_PLUS_ARCH(quantize_bias_offsetC, quantize_bias_offsetC_gfx950);
SAME(requantize_cpu, requantize_gfx950);                             // cpu/tensor_computing_cpu.h
SAME_PLUS_ARCH(convolution_transform_filter_bytes_x86, convolution_transform_filter_bytes_gfx950);
SAME_PLUS_ARCH(convolution_transform_filter_x86, convolution_transform_filter_gfx950);
SAME_PLUS_ARCH(convolution_infer_forward_tmp_bytes_x86, convolution_infer_forward_tmp_bytes_gfx950);
SAME(deconvolution_infer_forward_algorithm_cpu, deconvolution_infer_forward_algorithm_gfx950);  // cpu/tensor_computing_cpu.h:200-246
SAME(deconvolution_transform_filter_bytes_cpu, deconvolution_transform_filter_bytes_gfx950);
SAME(deconvolution_transform_filter_cpu, deconvolution_transform_filter_gfx950);
SAME(deconvolution_infer_forward_tmp_bytes_cpu, deconvolution_infer_forward_tmp_bytes_gfx950);
SAME(deconvolution_cpu, deconvolution_gfx950);
SAME_PLUS_ARCH(depthwise_convolution_transform_filter_int8, depthwise_convolution_transform_filter_int8_gfx950);
SAME_PLUS_ARCH(depthwise_pointwise_convolution_int8, depthwise_pointwise_convolution_int8_gfx950);

SAME_PLUS_ARCH(pooling_x86, pooling_gfx950);                          // cpu/x86/tensor_computing_x86.h:191-197
SAME(rnncell_x86, rnncell_gfx950);                                   // cpu/x86/tensor_computing_x86.h:166-181
SAME(rnncell_infer_forward_tmp_bytes_cpu, rnncell_infer_forward_tmp_bytes_gfx950);

// Twins that std::is_same cannot hold against a reference prototype, and why:
//  * fully_connected_gfx950, fully_connected_infer_forward_tmp_bytes_gfx950, matmul_gfx950,
//    matmul_infer_forward_tmp_bytes_gfx950: the reference has only the Tensor-class forms of these
//    (tensor_computing.h); the x86 int8 branch inside them is not a function of its own. The C forms take the
//    unwrapped descs, pointers and scales; include/bolt_gfx950_tensor.hpp puts the reference's Tensor argument
//    lists back on top, and tests/glue_test.cpp compiles those against tensor_computing.h.
//  * convolution_gfx950: convolution_x86 carries a scaleDesc and an untyped scale pointer between algorithm and
//    biasDesc; the C form takes F32 *scale after output, const input pointers, and no scaleDesc.
//  * convolution_infer_output_size_gfx950, convolution_infer_forward_algorithm_gfx950,
//    deconvolution_infer_output_size_gfx950: the reference's forms take Tensor * / ArchInfo_t.
//  * concat_gfx950, concat_infer_forward_tmp_bytes_gfx950: concat_cpu takes std::vector by value, which has no C form;
//    the twin takes a count and two arrays.
//  * rnn_transform_filter_gfx950, rnn_transform_filter_bytes_gfx950: the reference's forms take arrays of descs and
//    pointers (the int8 weight and the fp32 projection together); the twin transforms the int8 weight alone.
//  * convolution_*_bnn_gfx950: the reference's 1-bit convolution is declared in the ARM header
//    (cpu/arm/tensor_computing_arm.h), which does not compile for x86.
//  * ws_datatype_converter_*_gfx950, dequantize_int8_weight_gfx950, dequantize_int4_*_gfx950: the reference declares
//    these in no header (model_data_type_converter.cpp, model_deserialize.cpp); oracle/ref_shim_ptq.cpp repeats their
//    declarations and links them, so a changed argument list fails that link.
//  * depthwise_convolution_transform_filter_bytes_int8_gfx950 and every bolt_gfx950_* entry point: no counterpart.

// ---- plain-data types ---------------------------------------------------------------------------------------------
#define SIZE(T) static_assert(sizeof(ours::T) == sizeof(::T), "sizeof " #T)
#define FIELD(T, f) static_assert(offsetof(ours::T, f) == offsetof(::T, f), "offset of " #T "." #f)
#define VALUE(v) static_assert((long long)ours::v == (long long)::v, "value of " #v)

SIZE(TensorDesc);
FIELD(TensorDesc, dt);
FIELD(TensorDesc, df);
FIELD(TensorDesc, nDims);
FIELD(TensorDesc, dims);
static_assert(sizeof(::TensorDesc) == 92, "TensorDesc is 92 bytes");
SIZE(ActivationParamSpec);
FIELD(ActivationParamSpec, mode);
FIELD(ActivationParamSpec, value);
SIZE(ConvolutionParamSpec);
FIELD(ConvolutionParamSpec, num_outputs);
FIELD(ConvolutionParamSpec, kernel_h);
FIELD(ConvolutionParamSpec, stride_h);
FIELD(ConvolutionParamSpec, pad_top);
FIELD(ConvolutionParamSpec, pad_right);
FIELD(ConvolutionParamSpec, group);
FIELD(ConvolutionParamSpec, dilatedRate_h);
FIELD(ConvolutionParamSpec, convolution_type);
static_assert(sizeof(ours::QuantSpec) == sizeof(QuantSpec) && offsetof(ours::QuantSpec, scale) == offsetof(QuantSpec, scale), "QuantSpec");
FIELD(ConvolutionParamSpec, round_mode);
SIZE(PoolingParamSpec);
FIELD(PoolingParamSpec, mode);
FIELD(PoolingParamSpec, kernel_h);
FIELD(PoolingParamSpec, stride_h);
FIELD(PoolingParamSpec, pad_top);
FIELD(PoolingParamSpec, round_mode);
FIELD(PoolingParamSpec, count_include_pad);
SIZE(ConcatParamSpec);
FIELD(ConcatParamSpec, axis);
SIZE(RNNParamSpec);
FIELD(RNNParamSpec, mode);
FIELD(RNNParamSpec, num_outputs);
FIELD(RNNParamSpec, num_projection);
FIELD(RNNParamSpec, forget_bias);
FIELD(RNNParamSpec, zoneout_output);
FIELD(RNNParamSpec, activation_type);
SIZE(DataType);
SIZE(DataFormat);
SIZE(EE);
SIZE(Arch);

VALUE(DT_U8); VALUE(DT_I8); VALUE(DT_U32); VALUE(DT_I32); VALUE(DT_F16); VALUE(DT_F32); VALUE(DT_BIN01); VALUE(DT_BIN11);
VALUE(DT_F32_8Q); VALUE(DT_U8_Q);
VALUE(DF_NCHW); VALUE(DF_NCHWC8); VALUE(DF_NCHWN8C4); VALUE(DF_NCHWN16C8); VALUE(DF_TRANSPOSE); VALUE(DF_NORMAL);
VALUE(DF_MTK); VALUE(DF_MKT); VALUE(DF_NK); VALUE(DF_NKN32); VALUE(DF_NKN32K4); VALUE(DF_NHWC); VALUE(DF_NKNxKx);
VALUE(DF_NCHWC16); VALUE(DF_NCHWC2NxC4); VALUE(DF_SCALAR);
VALUE(SUCCESS); VALUE(NULL_POINTER); VALUE(NOT_MATCH); VALUE(NOT_FOUND); VALUE(ALLOC_FAILED); VALUE(NOT_IMPLEMENTED);
VALUE(NOT_SUPPORTED); VALUE(GCL_ERROR); VALUE(FILE_ERROR); VALUE(UNKNOWN);
VALUE(CPU_GENERAL); VALUE(X86_AVX512);
VALUE(ACTIVATION_NULL); VALUE(ACTIVATION_RELU); VALUE(ACTIVATION_GELU); VALUE(ACTIVATION_TANH);
VALUE(CONVOLUTION_ALGORITHM_POINTWISE); VALUE(CONVOLUTION_ALGORITHM_DIRECT); VALUE(CONVOLUTION_ALGORITHM_NULL);
VALUE(CONVOLUTION_FASTEST); VALUE(CONVOLUTION_DEPTHWISE_POINTWISE);
VALUE(ROUND_CEIL); VALUE(ROUND_SAME_UPPER); VALUE(ROUND_SAME_LOWER);
VALUE(POOLING_MAX); VALUE(POOLING_MEAN);
VALUE(RNN_LSTM);
// the two Arch values this library appends must not collide with any of the reference's
static_assert((int)ours::AMD_GFX950 > (int)::ARM_A55 && (int)ours::AMD_GFX950 > (int)::X86_AVX512 &&
        (int)ours::AMD_GFX950 > (int)::MALI && (int)ours::AMD_GFX950 > (int)::QUALCOMM,
    "AMD_GFX950 collides with a reference Arch value");

int main()
{
    return 0;
}
