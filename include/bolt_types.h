/*
 * Plain-data types shared across the C-ABI of the gfx950 quantized matrix-product library.
 *
 * Every enum value, field order and struct size below is binary-compatible with the
 * corresponding Bolt type, so a TensorDesc built by Bolt's own tensor2df()/tensor4df()
 * can be handed to this library unchanged:
 *   DataType    <- common/uni/include/data_type.h:67-85
 *   DataFormat  <- common/uni/include/tensor_desc.h:33-78  (implicit values, DF_NCHW = 0)
 *   TensorDesc  <- common/uni/include/tensor_desc.h:92-99  (#pragma pack(8), DIM_LEN 20)
 *   EE          <- common/uni/include/error.h:159-170
 *   Arch        <- common/uni/include/sys.h:44-55           (two values appended)
 *
 * dims[] is innermost-first: a 2-D [rows, cols] matrix has dims[0] = cols, dims[1] = rows;
 * a 4-D NCHW tensor has dims = {w, h, c, n}.
 */
#ifndef BOLT_GFX950_TYPES_H
#define BOLT_GFX950_TYPES_H

#include <stdbool.h>
#include <stdint.h>
#include <string.h>

#ifdef __cplusplus
extern "C" {
#endif

typedef int8_t INT8;
typedef uint8_t UINT8;
typedef uint8_t U8;
typedef int32_t I32;
typedef uint32_t U32;
typedef float F32;

#define DIM_LEN 20

typedef enum {
    DT_U8 = 0,
    DT_I8 = 1,
    DT_U32 = 2,
    DT_I32 = 3,
    DT_F16 = 4,
    DT_F16_8Q = 5,
    DT_F32 = 6,
    DT_BIN01 = 7, /* 1-bit, values {0,1}   (DoReFa) */
    DT_BIN11 = 8, /* 1-bit, values {-1,+1} (XNOR)   */
    DT_F32_8Q = 9,
    DT_U8_Q = 10, /* quantized activation stored as int8 + 128 */
    DT_I64 = 11,
    DT_U64 = 12,
    DT_F64 = 13,
    DT_BF16 = 14,
    DT_I4 = 15,
    DT_NUM = 16,
    DT_FORCE_U32 = 0x7fffffff
} DataType;

typedef enum {
    DF_NCHW = 0,
    DF_NCHWN16 = 1,
    DF_NCHWC8 = 2,
    DF_HWNCN16 = 3,
    DF_NHWCN16 = 4,
    DF_NHWCN8 = 5,
    DF_HWNCN8C4 = 6,
    DF_NCHWN8C4 = 7,
    DF_NCHWN8HW4 = 8,
    DF_NCHWN16C8 = 9, /* BNN filter */
    DF_NCHWCxN32 = 10,
    DF_NCHWCxN24 = 11,
    DF_NCHWC24 = 12,
    DF_TRANSPOSE = 13,
    DF_NORMAL = 14,
    DF_MTK = 15,
    DF_MKT = 16,
    DF_NK = 17,
    DF_NKN16 = 18,
    DF_NKN32 = 19,
    DF_NKN64 = 20,
    DF_NKN32K4 = 21, /* packed int8 matrix_vector_multiply weight */
    DF_NCHWC4 = 22,
    DF_NCHWC3 = 23,
    DF_NHWC = 24,
    DF_NCHWN4C4 = 25,
    DF_NCHWN4 = 26,
    DF_HWCN = 27,
    DF_NCWHN4C4 = 28,
    DF_NHWCN4 = 29,
    DF_CHWNC4 = 30,
    DF_CHWNC8 = 31,
    DF_CHWNC16 = 32,
    DF_CHWC8_NCN8 = 33,
    DF_RGB = 34,
    DF_HWNCN8 = 35,
    DF_NKN24 = 36,
    DF_NKN12 = 37,
    DF_NKN8 = 38,
    DF_NKNxKx = 39, /* packed int8 matrix_matrix_multiply right-hand side */
    DF_NKNx_NKN32 = 40,
    DF_NCHWC16 = 41,
    DF_NCHWC2NxC4 = 42, /* packed int8 convolution filter */
    DF_SCALAR = 43,
    DF_FORCE_U32 = 0x7fffffff
} DataFormat;

#pragma pack(8)
typedef struct TensorDesc {
    DataType dt;
    DataFormat df;
    U32 nDims;
    U32 dims[DIM_LEN];
} TensorDesc;
#pragma pack()

typedef enum {
    SUCCESS = 0,
    NULL_POINTER = 1,
    NOT_MATCH = 2,
    NOT_FOUND = 3,
    ALLOC_FAILED = 4,
    NOT_IMPLEMENTED = 50,
    NOT_SUPPORTED = 51,
    GCL_ERROR = 52,
    FILE_ERROR = 53,
    UNKNOWN = 99
} EE;

typedef enum {
    CPU_GENERAL = 1,
    MALI = 2,
    ARM_V7 = 3,
    ARM_V8 = 4,
    ARM_A55 = 5,
    ARM_A76 = 6,
    QUALCOMM = 7,
    X86_AVX2 = 8,
    X86_AVX512 = 9,
    X86_AVXVNNI = 10,
    /* Appended for this library. Every data pointer handed over with AMD_GFX950 is a HOST
     * pointer: the call stages operands to the GPU, runs, copies back and returns after
     * completion (strict drop-in for Bolt's CPU operator layer). */
    AMD_GFX950 = 11,
    /* Every data pointer (matrices, vectors, tmp, results) is a DEVICE pointer; kernels are
     * enqueued on the library stream and the call returns without waiting. The `scale`
     * argument and TensorDesc arguments stay host-side. */
    AMD_GFX950_DEVICE = 12
} Arch;

typedef struct {
    Arch arch;
    void *archPara;
} ArchInfo;
typedef ArchInfo *ArchInfo_t;

#define IS_GFX950(arch) ((arch) == AMD_GFX950 || (arch) == AMD_GFX950_DEVICE)

/* Activation / convolution parameter records: common/uni/include/parameter_spec.h */
typedef enum {
    ACTIVATION_NULL = 0,
    ACTIVATION_RELU = 1,
    ACTIVATION_RELU6 = 2,
    ACTIVATION_H_SWISH = 3,
    ACTIVATION_H_SIGMOID = 4,
    ACTIVATION_SIGMOID = 5,
    ACTIVATION_TANH = 6,
    ACTIVATION_GELU = 7,
    ACTIVATION_FORCE_U32 = 0x7fffffff
} ActivationMode;

#pragma pack(8)
typedef struct ActivationParamSpec {
    ActivationMode mode;
    float value[4];
} ActivationParamSpec;
#pragma pack()

typedef enum {
    CONVOLUTION_NO_TMP_MEM = 0,
    CONVOLUTION_FASTEST = 1,
    CONVOLUTION_TUNNING = 2,
    CONVOLUTION_LIBRARY_SEARCH = 3,
    CONVOLUTION_POLICY_FORCE_U32 = 0x7fffffff
} ConvolutionPolicy; /* common/uni/include/parameter_spec.h:150-155 */

typedef enum {
    CONVOLUTION_ALGORITHM_POINTWISE = 0,
    CONVOLUTION_ALGORITHM_DIRECT = 1,
    CONVOLUTION_ALGORITHM_IM2COL_GEMM = 2,
    CONVOLUTION_ALGORITHM_GEMM = 3,
    CONVOLUTION_ALGORITHM_GEMM_ICNCHW = 4,
    CONVOLUTION_ALGORITHM_WINOGRAD = 5,
    CONVOLUTION_ALGORITHM_BNN = 6,
    CONVOLUTION_ALGORITHM_INVGEMM = 7,
    CONVOLUTION_ALGORITHM_GROUP_DECONV = 8,
    CONVOLUTION_ALGORITHM_NULL = 9,
    CONVOLUTION_ALGORITHM_FORCE_U32 = 0x7fffffff
} ConvolutionForwardAlgorithm;

/* common/uni/include/parameter_spec.h:94-101, :25-34, :230-247, :259-286 (all inside #pragma pack(8),
 * every member 4 bytes wide except the 8-byte ActivationSpec union) */
typedef enum {
    CONVOLUTION_POINTWISE = 0,
    CONVOLUTION_DILATION = 1,
    CONVOLUTION_DEPTHWISE = 2,
    CONVOLUTION_DEPTHWISE_POINTWISE = 3,
    CONVOLUTION_DECONVOLUTION = 4,
    CONVOLUTION_DEPTHWISE_DECONVOLUTION = 5,
    CONVOLUTION_MODE_FORCE_U32 = 0x7fffffff
} ConvolutionMode;

typedef enum {
    ROUND_CEIL = 0,
    ROUND_FLOOR = 1,
    ROUND_TF_SAME = 2,
    ROUND_TF_VALID = 3,
    ROUND_PREFER_FLOOR = 4,
    ROUND_PREFER_CEIL = 5,
    ROUND_SAME_UPPER = 6,
    ROUND_SAME_LOWER = 7,
    ROUND_MODE_FORCE_U32 = 0x7fffffff
} RoundMode;

typedef union {
    struct {
        float neg_slope;
    } relu_spec;
    struct {
        float min;
        float max;
    } clip_spec;
} ActivationSpec;

#pragma pack(8)
typedef struct {
    U32 num_outputs;
    U32 kernel_t;
    U32 kernel_h;
    U32 kernel_w;
    U32 stride_t;
    U32 stride_h;
    U32 stride_w;
    U32 pad_before;
    U32 pad_after;
    U32 pad_top;
    U32 pad_bottom;
    U32 pad_left;
    U32 pad_right;
    U32 group;
    U32 dilatedRate_t;
    U32 dilatedRate_h;
    U32 dilatedRate_w;
    U32 num_outputs_origin;
    ConvolutionMode convolution_type;
    ActivationMode dw_activation_type;
    ActivationMode pw_activation_type;
    ActivationSpec activation_spec;
    RoundMode round_mode;
    U32 output_pad_t;
    U32 output_pad_h;
    U32 output_pad_w;
} ConvolutionParamSpec;
#pragma pack()

/* common/uni/include/parameter_spec.h:21 */
typedef enum {
    POOLING_MAX = 0,
    POOLING_MEAN = 1,
    POOLING_MODE_FORCE_U32 = 0x7fffffff
} PoolingMode;

/* common/uni/include/parameter_spec.h:285-301 (60 bytes) */
typedef struct {
    U32 kernel_t;
    U32 kernel_h;
    U32 kernel_w;
    U32 stride_t;
    U32 stride_h;
    U32 stride_w;
    U32 pad_before;
    U32 pad_after;
    U32 pad_top;
    U32 pad_bottom;
    U32 pad_left;
    U32 pad_right;
    RoundMode round_mode;
    PoolingMode mode;
    bool count_include_pad;
} PoolingParamSpec;

/* common/uni/include/parameter_spec.h:451-454 */
typedef struct {
    I32 axis;
    I32 num_concat;
} ConcatParamSpec;

/* common/uni/include/parameter_spec.h:126 */
typedef enum {
    RNN_RNN = 0,
    RNN_LSTM = 1,
    RNN_GRU = 2,
    RNN_GRU_LBR = 3,
    RNN_MODE_FORCE_U32 = 0x7fffffff
} RNNMode;

/* common/uni/include/parameter_spec.h:380-393 (36 bytes) */
typedef struct {
    RNNMode mode;
    U32 num_outputs;
    I32 steps; /* >= 0: multi-step RNN, -1: RNNCell */
    I32 num_projection;
    float zoneout_cell;
    float zoneout_output;
    bool bi_direction;
    float forget_bias;
    ActivationMode activation_type;
} RNNParamSpec;

static inline U32 bolt_align(U32 x, U32 a)
{
    return a == 0 ? 0 : (x + a - 1) / a * a;
}

/* bytes per element, common/uni/include/data_type.h:95-107 (binary types: divide the
 * element count by 8 first). */
static inline U32 bytesOf(DataType dt)
{
    static const U32 bytes[] = {1, 1, 4, 4, 2, 2, 4, 1, 1, 4, 1, 8, 8, 8, 2, 1};
    return ((U32)dt < 16) ? bytes[dt] : 0;
}

static inline TensorDesc tensor4df(DataType dt, DataFormat df, U32 n, U32 c, U32 h, U32 w)
{
    TensorDesc d;
    memset(&d, 0, sizeof(d));
    d.dt = dt;
    d.df = df;
    d.nDims = 4;
    d.dims[0] = w;
    d.dims[1] = h;
    d.dims[2] = c;
    d.dims[3] = n;
    return d;
}

static inline TensorDesc tensor2df(DataType dt, DataFormat df, U32 rows, U32 cols)
{
    TensorDesc d = tensor4df(dt, df, 1, 1, rows, cols);
    d.nDims = 2;
    return d;
}

static inline TensorDesc tensor1d(DataType dt, U32 len)
{
    TensorDesc d = tensor4df(dt, DF_NCHW, 1, 1, 1, len);
    d.nDims = 1;
    return d;
}

static inline U32 tensorNumElements(TensorDesc d)
{
    if (d.nDims == 0) {
        return 0;
    }
    U32 r = 1;
    for (U32 i = 0; i < d.nDims && i < DIM_LEN; i++) {
        r *= d.dims[i];
    }
    return r;
}

static inline U32 tensorNumBytes(TensorDesc d)
{
    if (d.dt == DT_BIN01 || d.dt == DT_BIN11) {
        return tensorNumElements(d) / 8;
    }
    return tensorNumElements(d) * bytesOf(d.dt);
}

#ifdef __cplusplus
}
static_assert(sizeof(TensorDesc) == 92, "TensorDesc must match Bolt's 92-byte record");
static_assert(sizeof(PoolingParamSpec) == 60, "PoolingParamSpec must match Bolt's record");
static_assert(sizeof(RNNParamSpec) == 36, "RNNParamSpec must match Bolt's record");
static_assert(sizeof(DataType) == 4 && sizeof(DataFormat) == 4, "enums are 32-bit in Bolt");
#endif

/* common/uni/include/parameter_spec.h:753-756 (inside #pragma pack(8)): one record of per-tensor quantisation scales
 * as a .bolt model stores them per operator (OperatorSpec::feature_scale) and per weight (WeightSpec::weight_scale) */
typedef struct {
    I32 num_scale;
    F32 *scale;
} QuantSpec;

#endif
