"""ctypes binding of libbolt_gfx950.so, mirroring include/bolt_types.h and include/bolt_gfx950.h.

The library is the product; this module only declares its C-ABI. There is no CPU fallback: if the
shared library is missing, importing `lib()` raises.
"""
import ctypes as C
import os

HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(HERE, "libbolt_gfx950.so")

# DataType (common/uni/include/data_type.h:67-85)
DT_U8, DT_I8, DT_U32, DT_I32, DT_F16, DT_F16_8Q, DT_F32, DT_BIN01, DT_BIN11, DT_F32_8Q, DT_U8_Q = range(11)
# DataFormat (common/uni/include/tensor_desc.h:33-78)
DF_NCHW, DF_NCHWC8, DF_NCHWN16C8 = 0, 2, 9
DF_TRANSPOSE, DF_NORMAL, DF_NK, DF_NKN32K4, DF_NKNxKx, DF_NCHWC16, DF_NCHWC2NxC4 = 13, 14, 17, 21, 39, 41, 42
# EE (common/uni/include/error.h:159-170)
SUCCESS, NULL_POINTER, NOT_MATCH, NOT_FOUND, ALLOC_FAILED = 0, 1, 2, 3, 4
NOT_IMPLEMENTED, NOT_SUPPORTED, UNKNOWN = 50, 51, 99
# Arch (common/uni/include/sys.h:44-55, two values appended)
CPU_GENERAL, X86_AVX512, AMD_GFX950, AMD_GFX950_DEVICE = 1, 9, 11, 12

DIM_LEN = 20


class TensorDesc(C.Structure):
    _pack_ = 8
    _fields_ = [("dt", C.c_uint32), ("df", C.c_uint32), ("nDims", C.c_uint32), ("dims", C.c_uint32 * DIM_LEN)]

    def __repr__(self):
        return "TensorDesc(dt=%d, df=%d, dims=%s)" % (self.dt, self.df, list(self.dims[:self.nDims])[::-1])


assert C.sizeof(TensorDesc) == 92


def tensor4df(dt, df, n, c, h, w):
    d = TensorDesc()
    d.dt, d.df, d.nDims = dt, df, 4
    d.dims[0], d.dims[1], d.dims[2], d.dims[3] = w, h, c, n
    return d


def tensor_num_bytes(d):
    """tensorNumBytes (tensor_desc.h) for byte-sized and wider element types."""
    n = 1
    for i in range(d.nDims):
        n *= d.dims[i]
    return n * {DT_U8: 1, DT_I8: 1, DT_U32: 4, DT_I32: 4, DT_F16: 2, DT_F32: 4, DT_U8_Q: 1}[d.dt]


def tensor2df(dt, df, rows, cols):
    d = tensor4df(dt, df, 1, 1, rows, cols)
    d.nDims = 2
    return d


def tensor1d(dt, n):
    d = tensor4df(dt, DF_NCHW, 1, 1, 1, n)
    d.nDims = 1
    return d


class ConvolutionParamSpec(C.Structure):
    """common/uni/include/parameter_spec.h:259-286"""
    _pack_ = 8
    _fields_ = [(k, C.c_uint32) for k in (
        "num_outputs", "kernel_t", "kernel_h", "kernel_w", "stride_t", "stride_h", "stride_w", "pad_before", "pad_after",
        "pad_top", "pad_bottom", "pad_left", "pad_right", "group", "dilatedRate_t", "dilatedRate_h", "dilatedRate_w",
        "num_outputs_origin", "convolution_type", "dw_activation_type", "pw_activation_type")] + [
        ("activation_spec", C.c_float * 2), ("round_mode", C.c_uint32), ("output_pad_t", C.c_uint32),
        ("output_pad_h", C.c_uint32), ("output_pad_w", C.c_uint32)]


class ActivationParamSpec(C.Structure):
    """common/uni/include/parameter_spec.h:179-183"""
    _pack_ = 8
    _fields_ = [("mode", C.c_uint32), ("value", C.c_float * 4)]


assert C.sizeof(ConvolutionParamSpec) == 108 and C.sizeof(ActivationParamSpec) == 20
ACTIVATION_NULL, ACTIVATION_RELU = 0, 1
CONVOLUTION_ALGORITHM_POINTWISE, CONVOLUTION_ALGORITHM_DIRECT, CONVOLUTION_ALGORITHM_BNN = 0, 1, 6
CONVOLUTION_ALGORITHM_IM2COL_GEMM, CONVOLUTION_ALGORITHM_GROUP_DECONV, CONVOLUTION_ALGORITHM_NULL = 2, 8, 9


def conv_param_spec(oc, fh, fw, stride, pad, dilation=1, group=1):
    """createConvolutionParamSpec (parameter_spec.h:878-920) for the 2-D case."""
    p = ConvolutionParamSpec()
    p.num_outputs, p.kernel_t, p.kernel_h, p.kernel_w = oc, 1, fh, fw
    p.stride_t, p.stride_h, p.stride_w = 1, stride, stride
    p.pad_top = p.pad_bottom = p.pad_left = p.pad_right = pad
    p.group, p.dilatedRate_t, p.dilatedRate_h, p.dilatedRate_w = group, 1, dilation, dilation
    p.num_outputs_origin = oc
    p.convolution_type = 3  # CONVOLUTION_DEPTHWISE_POINTWISE, what the reference's tests pass
    return p


class PoolingParamSpec(C.Structure):
    """common/uni/include/parameter_spec.h:285-301"""
    _fields_ = [(k, C.c_uint32) for k in (
        "kernel_t", "kernel_h", "kernel_w", "stride_t", "stride_h", "stride_w", "pad_before", "pad_after", "pad_top",
        "pad_bottom", "pad_left", "pad_right", "round_mode", "mode")] + [("count_include_pad", C.c_bool)]


class ConcatParamSpec(C.Structure):
    """common/uni/include/parameter_spec.h:451-454"""
    _fields_ = [("axis", C.c_int32), ("num_concat", C.c_int32)]


assert C.sizeof(PoolingParamSpec) == 60 and C.sizeof(ConcatParamSpec) == 8
POOLING_MAX, POOLING_MEAN = 0, 1


def pooling_param_spec(mode, kh, kw, sh, sw, pt, pb, pl, pr, count_include_pad=False, round_mode=0):
    """createPoolingParamSpec (parameter_spec.h:936-970) for the 2-D case."""
    p = PoolingParamSpec()
    p.kernel_t, p.kernel_h, p.kernel_w = 1, kh, kw
    p.stride_t, p.stride_h, p.stride_w = 1, sh, sw
    p.pad_top, p.pad_bottom, p.pad_left, p.pad_right = pt, pb, pl, pr
    p.round_mode, p.mode, p.count_include_pad = round_mode, mode, bool(count_include_pad)
    return p


class RNNParamSpec(C.Structure):
    """common/uni/include/parameter_spec.h:380-393"""
    _fields_ = [("mode", C.c_uint32), ("num_outputs", C.c_uint32), ("steps", C.c_int32), ("num_projection", C.c_int32),
                ("zoneout_cell", C.c_float), ("zoneout_output", C.c_float), ("bi_direction", C.c_bool),
                ("forget_bias", C.c_float), ("activation_type", C.c_uint32)]


assert C.sizeof(RNNParamSpec) == 36
RNN_LSTM, ACTIVATION_TANH, DF_NKN32, DF_NKNx_NKN32 = 1, 6, 19, 40


_vp, _u32, _f32p, _u32p = C.c_void_p, C.c_uint32, C.POINTER(C.c_float), C.POINTER(C.c_uint32)
_TDp = C.POINTER(TensorDesc)

# name -> (restype, argtypes); every symbol include/bolt_gfx950.h declares
class BoltEncoderLayerInt8(C.Structure):
    _fields_ = ([(n, C.c_uint32) for n in ("batch", "seq", "hidden", "heads", "ffn")] +
                [(n, C.c_void_p) for n in ("wqkv", "wo", "w1", "w2")] +
                [(n, C.POINTER(C.c_float)) for n in ("sqkv", "so", "s1", "s2", "bqkv", "bo", "b1", "b2", "ln1_gamma",
                                                     "ln1_beta", "ln2_gamma", "ln2_beta")])


SIGNATURES = {
    "bolt_gfx950_init": (C.c_int, []),
    "bolt_gfx950_get_counter": (C.c_int, [C.c_char_p, C.POINTER(C.c_ulonglong)]),
    "vector_vector_axpby_gfx950": (C.c_int, [C.c_float, TensorDesc, _vp, C.c_float, TensorDesc, _vp, C.c_int]),
    "convolution_infer_output_size_gfx950": (C.c_int, [TensorDesc, TensorDesc, ConvolutionParamSpec, _TDp, C.c_int,
                                                       C.c_int]),
    "convolution_infer_forward_algorithm_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, ConvolutionParamSpec,
                                                             C.c_int, C.POINTER(C.c_int), C.c_int, ActivationParamSpec,
                                                             C.c_int]),
    "bolt_gfx950_set_stream": (C.c_int, [_vp]),
    "bolt_gfx950_synchronize": (C.c_int, []),
    "bolt_gfx950_last_error": (C.c_char_p, []),
    "bolt_gfx950_set_option": (C.c_int, [C.c_char_p, C.c_int]),
    "bolt_gfx950_malloc": (_vp, [C.c_size_t]),
    "bolt_gfx950_free": (None, [_vp]),
    "bolt_gfx950_memcpy_h2d": (C.c_int, [_vp, _vp, C.c_size_t]),
    "bolt_gfx950_memcpy_d2h": (C.c_int, [_vp, _vp, C.c_size_t]),
    "bolt_gfx950_memcpy_d2d": (C.c_int, [_vp, _vp, C.c_size_t]),
    "bolt_gfx950_timer_start": (C.c_int, []),
    "bolt_gfx950_timer_stop": (C.c_int, [_f32p]),
    "matrix_matrix_multiply_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, _u32p, C.c_int]),
    "matrix_matrix_multiply_gfx950": (C.c_int, [TensorDesc, _vp, TensorDesc, _vp, _u32, _vp, TensorDesc, _vp, _vp,
                                                C.c_int]),
    "matrix_matrix_multiply_rhs_format_gfx950": (C.c_int, [C.c_int]),
    "matrix_matrix_multiply_transform_rhs_bytes_gfx950": (C.c_int, [TensorDesc, _u32p, _u32p, C.c_int]),
    "matrix_matrix_multiply_transform_rhs_gfx950": (C.c_int, [TensorDesc, _vp, _TDp, _vp, C.c_int]),
    "matrix_vector_multiply_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, _u32p, C.c_int]),
    "matrix_vector_multiply_gfx950": (C.c_int, [TensorDesc, _vp, TensorDesc, _vp, _u32, _vp, TensorDesc, _vp, _vp,
                                                C.c_int]),
    "matrix_vector_multiply_weight_format_gfx950": (C.c_int, [C.c_int]),
    "matrix_vector_multiply_transform_weight_bytes_gfx950": (C.c_int, [TensorDesc, _u32p, C.c_int]),
    "matrix_vector_multiply_transform_weight_gfx950": (C.c_int, [TensorDesc, _vp, _TDp, _vp, C.c_int]),
    "quantize_gfx950": (C.c_int, [TensorDesc, _vp, _TDp, _vp, _vp, C.c_int, C.c_int]),
    "dequantize_gfx950": (C.c_int, [TensorDesc, _vp, _vp, TensorDesc, _vp, TensorDesc, _vp, C.c_int]),
    "quantize_bias_offsetC_gfx950": (C.c_int, [_vp, TensorDesc, C.c_int, _vp, TensorDesc, _vp, _vp, C.c_int]),
    "requantize_gfx950": (C.c_int, [TensorDesc, _vp, C.c_float, TensorDesc, _vp, C.c_float, C.c_int]),
    "fully_connected_infer_forward_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, _u32p, C.c_int]),
    "fully_connected_gfx950": (C.c_int, [TensorDesc, _vp, C.c_float, TensorDesc, _vp, C.c_float, TensorDesc, _vp, _u32,
                                         _vp, TensorDesc, _vp, _f32p, C.c_int]),
    "matmul_infer_forward_tmp_bytes_gfx950": (C.c_int, [TensorDesc, C.c_bool, TensorDesc, C.c_bool, TensorDesc, _u32p,
                                                        C.c_int]),
    "matmul_gfx950": (C.c_int, [TensorDesc, C.c_bool, _vp, C.c_float, TensorDesc, C.c_bool, _vp, C.c_float, _u32, _vp,
                                TensorDesc, _vp, C.c_int]),
    "convolution_transform_filter_bytes_gfx950": (C.c_int, [TensorDesc, ConvolutionParamSpec, C.c_int, _u32p, C.c_int]),
    "convolution_transform_filter_gfx950": (C.c_int, [TensorDesc, _vp, ConvolutionParamSpec, C.c_int, _TDp, _vp,
                                                      C.c_int]),
    "convolution_infer_forward_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, ConvolutionParamSpec,
                                                             C.c_int, _u32p, C.c_int]),
    "convolution_gfx950": (C.c_int, [TensorDesc, _vp, _vp, TensorDesc, _vp, ConvolutionParamSpec, C.c_int, TensorDesc,
                                     _vp, _u32, _vp, TensorDesc, _vp, _f32p, ActivationParamSpec, C.c_int]),
    "deconvolution_infer_output_size_gfx950": (C.c_int, [TensorDesc, TensorDesc, ConvolutionParamSpec, _TDp, C.c_int,
                                                         C.c_int]),
    "deconvolution_infer_forward_algorithm_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, ConvolutionParamSpec,
                                                               C.c_int, C.POINTER(C.c_int), C.c_int, C.c_int]),
    "deconvolution_transform_filter_bytes_gfx950": (C.c_int, [TensorDesc, ConvolutionParamSpec, C.c_int, _u32p, C.c_int]),
    "deconvolution_transform_filter_gfx950": (C.c_int, [TensorDesc, _vp, ConvolutionParamSpec, C.c_int, _TDp, _vp,
                                                        C.c_int]),
    "deconvolution_infer_forward_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, ConvolutionParamSpec,
                                                               C.c_int, _u32p, C.c_int]),
    "deconvolution_gfx950": (C.c_int, [TensorDesc, _vp, TensorDesc, _vp, ConvolutionParamSpec, C.c_int, TensorDesc, _vp,
                                       TensorDesc, _vp, _u32, _vp, TensorDesc, _vp, ActivationParamSpec, C.c_int]),
    "depthwise_convolution_transform_filter_bytes_int8_gfx950": (C.c_int, [TensorDesc, _u32p, C.c_int]),
    "depthwise_convolution_transform_filter_int8_gfx950": (C.c_int, [TensorDesc, _vp, _TDp, _vp, C.c_int]),
    "depthwise_pointwise_convolution_int8_gfx950": (C.c_int, [TensorDesc, _vp, _vp, TensorDesc, _vp, TensorDesc, _vp,
                                                              ConvolutionParamSpec, TensorDesc, _vp, TensorDesc, _vp, _u32,
                                                              _vp, TensorDesc, _vp, _f32p, ActivationParamSpec,
                                                              ActivationParamSpec, C.c_int]),
    "ws_datatype_converter_int8_gfx950": (C.c_int, [_vp, _vp, C.c_int, _f32p, C.c_int]),
    "ws_datatype_converter_int4_gfx950": (C.c_int, [_vp, _vp, C.c_int, _f32p, C.c_int]),
    "ws_datatype_converter_bnn_gfx950": (C.c_int, [_vp, _vp, C.c_int, _f32p, C.c_int]),
    "dequantize_int8_weight_gfx950": (C.c_int, [C.c_int, C.c_float, _vp, _vp, C.c_int]),
    "dequantize_int4_weight_gfx950": (C.c_int, [C.c_int, C.c_float, _vp, _vp, C.c_int]),
    "dequantize_int4_int8_gfx950": (C.c_int, [C.c_int, _vp, _vp, C.c_int]),
    "dequantize_int4_u8_q_gfx950": (C.c_int, [C.c_int, _vp, _vp, C.c_int]),
    "bolt_gfx950_operator_scales": (C.c_int, [C.c_int, _vp, _u32, C.c_int, C.c_int, C.c_float, C.c_float, _f32p, C.POINTER(C.c_int)]),
    "convolution_transform_filter_bytes_bnn_gfx950": (C.c_int, [TensorDesc, _u32p, C.c_int]),
    "convolution_transform_filter_bnn_gfx950": (C.c_int, [TensorDesc, _vp, C.POINTER(TensorDesc), _vp, C.c_int]),
    "convolution_infer_forward_tmp_bytes_bnn_gfx950": (C.c_int, [TensorDesc, ConvolutionParamSpec, _u32p, C.c_int]),
    "convolution_bnn_gfx950": (C.c_int, [TensorDesc, _vp, TensorDesc, _vp, ConvolutionParamSpec, TensorDesc, _vp,
                                         TensorDesc, _vp, _u32, _vp, TensorDesc, _vp, ActivationParamSpec, C.c_int]),
    "pooling_gfx950": (C.c_int, [TensorDesc, _vp, PoolingParamSpec, _vp, TensorDesc, _vp, _vp, C.c_int]),
    "concat_infer_forward_tmp_bytes_gfx950": (C.c_int, [_u32, _TDp, TensorDesc, _u32p, C.c_int]),
    "concat_gfx950": (C.c_int, [_u32, _TDp, C.POINTER(_vp), _f32p, ConcatParamSpec, _vp, TensorDesc, _vp, _f32p,
                                C.c_int]),
    "rnncell_infer_forward_tmp_bytes_gfx950": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, RNNParamSpec, _u32p, C.c_int]),
    "rnn_transform_filter_bytes_gfx950": (C.c_int, [TensorDesc, RNNParamSpec, _u32p, C.c_int]),
    "rnn_transform_filter_gfx950": (C.c_int, [TensorDesc, _vp, RNNParamSpec, _TDp, _vp, C.c_int]),
    "rnncell_gfx950": (C.c_int, [TensorDesc, _vp, _TDp, C.POINTER(_vp), _TDp, C.POINTER(_vp), _f32p, _vp, _u32, _vp,
                                 RNNParamSpec, _u32, _u32, TensorDesc, _vp, C.c_int]),
    "bolt_gfx950_encoder_layer_int8_workspace_bytes": (C.c_int, [C.POINTER(BoltEncoderLayerInt8),
                                                                 C.POINTER(C.c_size_t)]),
    "bolt_gfx950_encoder_layer_int8_workspace_layout": (C.c_int, [C.POINTER(BoltEncoderLayerInt8),
                                                                  C.POINTER(C.c_size_t)]),
    "bolt_gfx950_encoder_layer_int8": (C.c_int, [C.POINTER(BoltEncoderLayerInt8), _vp, _vp, _vp, C.c_size_t]),
    "bolt_gfx950_encoder_stack_int8_workspace_bytes": (C.c_int, [C.POINTER(BoltEncoderLayerInt8), _u32,
                                                                 C.POINTER(C.c_size_t)]),
    "bolt_gfx950_encoder_stack_int8": (C.c_int, [C.POINTER(BoltEncoderLayerInt8), _u32, _vp, _vp, _vp, C.c_size_t]),
    "bolt_gfx950_attention_f32": (C.c_int, [_vp, _u32, _u32, _u32, _u32, _vp]),
    "bolt_gfx950_add_layernorm_f32": (C.c_int, [_vp, _vp, _vp, _vp, _u32, _u32, _vp]),
    "bolt_gfx950_gelu_f32": (C.c_int, [_vp, C.c_size_t]),
    "bolt_gfx950_quantize_f32_async": (C.c_int, [_vp, _u32, C.c_int, _vp, _vp, C.c_int]),
    "bolt_gfx950_quantize_f32_noalloc": (C.c_int, [_vp, _u32, C.c_int, _vp, _vp, C.c_int]),
    "bolt_gfx950_mmm_int8_perchannel": (C.c_int, [_u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "bolt_gfx950_mmm_int8_perchannel_u8": (C.c_int, [_u32, _u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp, C.c_float]),
    "bolt_gfx950_convolution_int8_perchannel": (C.c_int, [TensorDesc, _vp, _vp, TensorDesc, _vp, ConvolutionParamSpec, _vp,
                                                          TensorDesc, _vp, _u32, _vp, TensorDesc, _vp, _f32p,
                                                          ActivationParamSpec, C.c_int]),
    "bolt_gfx950_convolution_async_tmp_bytes": (C.c_int, [TensorDesc, TensorDesc, TensorDesc, ConvolutionParamSpec, _u32p]),
    "bolt_gfx950_convolution_async": (C.c_int, [TensorDesc, _vp, _vp, TensorDesc, _vp, ConvolutionParamSpec, TensorDesc, _vp,
                                                _u32, _vp, TensorDesc, _vp, _vp, C.c_float, _vp, _vp, C.c_float,
                                                ActivationParamSpec]),
    "bolt_gfx950_mvm_int8_perchannel": (C.c_int, [_u32, _u32, _vp, _vp, _vp, _vp, _vp, _vp, _vp]),
    "bolt_gfx950_mvm_int8_strided_batch": (C.c_int, [_u32, _u32, _u32, _vp, C.c_size_t, _u32, _vp, _vp, _vp, _vp,
                                                     _vp]),
}

_lib = None


def lib():
    """The loaded C-ABI library with argtypes set. Raises if it has not been built."""
    global _lib
    if _lib is None:
        if not os.path.exists(LIB_PATH):
            raise RuntimeError(
                "%s is missing: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
                "(there is no CPU fallback)" % LIB_PATH)
        L = C.CDLL(LIB_PATH)
        for name, (res, args) in SIGNATURES.items():
            fn = getattr(L, name)
            fn.restype = res
            fn.argtypes = args
        _lib = L
    return _lib


class BoltError(RuntimeError):
    pass


def check(code, what=""):
    if code != SUCCESS:
        msg = lib().bolt_gfx950_last_error()
        raise BoltError("%s failed with EE=%d (%s)" % (what, code, (msg or b"").decode()))
