// Header-only C++ glue between Bolt's Tensor-level operator interface and the C-ABI of libbolt_gfx950.so.
//
// Include it INSIDE Bolt (after Bolt's own tensor_computing.h / tensor.hpp, which define Tensor, TensorDesc,
// ArchInfo_t ...). Each function below has the argument list of the reference function of the same name in
// compute/tensor/include/tensor_computing.h and unwraps its Tensors exactly as that function does
// (get_ptr_from_tensor, common/memory/include/tensor_auxiliary.h:26-37; compute/tensor/src/quantize.cpp:19-34,
// dequantize.cpp:25-49, fully_connected.cpp:107-159,307-498, matmul.cpp:203-300,302-576,
// convolution.cpp:28-470, deconvolution.cpp:23-279), then calls the `_gfx950` twin. A dispatcher branch
//     } else if (IS_GFX950(arch)) { ret = bolt_gfx950::fully_connected(in, filter, bias, tmp, out, archInfo); }
// in those reference functions is all the operator classes (FullyConnectedCPU, ConvolutionCPU, MatMulCPU,
// QuantizeLinearCPU) need: they keep their call order bytes -> transform -> tmp bytes -> run.
//
// Arch values: AMD_GFX950 (data pointers are host memory) and AMD_GFX950_DEVICE (data pointers are device memory;
// the Tensors are ordinary CpuMemory tensors whose buffer was set with device_tensor() below, so activations stay
// on the GPU between consecutive quantised operators and nothing changes in the classes that pass Tensors around).
// Until Bolt's own `enum Arch` carries the two values they are defined here.
#ifndef BOLT_GFX950_TENSOR_HPP
#define BOLT_GFX950_TENSOR_HPP

#include <memory>
#include <vector>

#ifndef BOLT_GFX950_NO_TYPES
#define BOLT_GFX950_NO_TYPES
#endif
#include "bolt_gfx950.h"

#ifndef BOLT_GFX950_ARCH_IN_ENUM
static const Arch AMD_GFX950 = (Arch)11;
static const Arch AMD_GFX950_DEVICE = (Arch)12;
#ifndef IS_GFX950
#define IS_GFX950(arch) ((arch) == AMD_GFX950 || (arch) == AMD_GFX950_DEVICE)
#endif
#endif

namespace bolt_gfx950 {

// every tensor on this path is a CpuMemory tensor (its buffer may be device memory, see device_tensor)
inline void *ptr_of(Tensor t)
{
    return ((CpuMemory *)(t.get_memory()))->get_ptr();
}

// A Tensor of the given desc whose buffer is DEVICE memory owned by the tensor (freed with the last copy of it).
inline Tensor device_tensor(TensorDesc desc)
{
    Tensor t(CPUMem);
    t.resize(desc);
    void *p = bolt_gfx950_malloc(tensorNumBytes(desc));
    if (p) {
        ((CpuMemory *)(t.get_memory()))->set_shared_ptr(std::shared_ptr<U8>((U8 *)p, [](U8 *q) { bolt_gfx950_free(q); }));
    }
    // allocation refused: the tensor keeps no buffer (ptr_of() == nullptr) and every call it is handed to returns
    // NULL_POINTER; bolt_gfx950_last_error() has the reason
    return t;
}

inline EE upload(Tensor host, Tensor *dev)
{
    return bolt_gfx950_memcpy_h2d(ptr_of(*dev), ptr_of(host), host.bytes());
}

inline EE download(Tensor dev, Tensor *host)
{
    return bolt_gfx950_memcpy_d2h(ptr_of(*host), ptr_of(dev), dev.bytes());
}

// ---- quantize / dequantize (compute/tensor/src/quantize.cpp:19-34, dequantize.cpp:25-49) ---------------------
inline EE quantize(Tensor input, Tensor *output, F32 *scale, ArchInfo_t archInfo)
{
    TensorDesc qDesc = output->get_desc();
    EE ret = quantize_gfx950(input.get_desc(), ptr_of(input), &qDesc, ptr_of(*output), scale, 0, archInfo->arch);
    output->resize(qDesc);
    return ret;
}

inline EE dequantize(Tensor input, const F32 *scale, Tensor bias, Tensor output, ArchInfo_t archInfo)
{
    return dequantize_gfx950(input.get_desc(), ptr_of(input), scale, bias.get_desc(), ptr_of(bias), output.get_desc(),
        ptr_of(output), archInfo->arch);
}

// ---- FullyConnected (fully_connected.cpp:107-159, 307-498; weight transform fully_connected_cpu.hpp:231-248) ---
inline EE fully_connected_infer_forward_tmp_bytes(
    Tensor inputTensor, Tensor filterTensor, Tensor outputTensor, U32 *bytes, ArchInfo_t archInfo)
{
    return fully_connected_infer_forward_tmp_bytes_gfx950(
        inputTensor.get_desc(), filterTensor.get_desc(), outputTensor.get_desc(), bytes, archInfo->arch);
}

// the engine's FullyConnectedCPU::transform_filter for an s8 weight: GEMV packing when the operator runs row by row
// (mvm), GEMM packing otherwise; the transformed tensor carries the weight's scale
inline EE fully_connected_transform_weight(Tensor weight, bool mvm, Tensor *wtm, ArchInfo_t archInfo)
{
    const Arch arch = archInfo->arch;
    TensorDesc fDesc = weight.get_desc(), tDesc;
    U32 bytes = 0;
    EE ret = mvm ? matrix_vector_multiply_transform_weight_bytes_gfx950(fDesc, &bytes, arch)
                 : matrix_matrix_multiply_transform_rhs_bytes_gfx950(fDesc, &bytes, nullptr, arch);
    if (ret != SUCCESS) {
        return ret;
    }
    *wtm = (arch == AMD_GFX950_DEVICE) ? device_tensor(tensor1d(DT_U8, bytes)) : Tensor::alloc_sized<CPUMem>(tensor1d(DT_U8, bytes));
    ret = mvm ? matrix_vector_multiply_transform_weight_gfx950(fDesc, ptr_of(weight), &tDesc, ptr_of(*wtm), arch)
              : matrix_matrix_multiply_transform_rhs_gfx950(fDesc, ptr_of(weight), &tDesc, ptr_of(*wtm), arch);
    wtm->resize(tDesc);
    wtm->set_scale(weight.get_scale());
    return ret;
}

inline EE fully_connected(Tensor inputTensor, Tensor filterTensor, Tensor biasTensor, std::vector<Tensor> tmpTensors,
    Tensor outputTensor, ArchInfo_t archInfo)
{
    void *bias = ptr_of(biasTensor);
    TensorDesc biasDesc;
    if (bias) {
        biasDesc = biasTensor.get_desc();
    }
    F32 scaleO = outputTensor.get_scale();  // <= 0: unknown, the call computes it (fully_connected.cpp:374,388)
    EE ret = fully_connected_gfx950(inputTensor.get_desc(), ptr_of(inputTensor), inputTensor.get_scale(), filterTensor.get_desc(),
        ptr_of(filterTensor), filterTensor.get_scale(), biasDesc, bias, tmpTensors[0].bytes(), ptr_of(tmpTensors[0]),
        outputTensor.get_desc(), ptr_of(outputTensor), &scaleO, archInfo->arch);
    const DataType odt = outputTensor.get_desc().dt;
    if (ret == SUCCESS && (odt == DT_U8_Q || odt == DT_I8)) {
        outputTensor.set_scale(scaleO);  // :486; an fp32 / int32 output's scale is left alone, as in the reference
    }
    return ret;
}

// ---- matmul (matmul.cpp:203-300, 302-576) ---------------------------------------------------------------------
inline EE matmul_infer_forward_tmp_bytes(Tensor matrixATensor, bool transposeA, Tensor matrixBTensor, bool transposeB,
    Tensor matrixCTensor, U32 *bytes, ArchInfo_t archInfo)
{
    return matmul_infer_forward_tmp_bytes_gfx950(matrixATensor.get_desc(), transposeA, matrixBTensor.get_desc(), transposeB,
        matrixCTensor.get_desc(), bytes, archInfo->arch);
}

inline EE matmul(Tensor matrixATensor, bool transposeA, Tensor matrixBTensor, bool transposeB, Tensor biasTensor,
    std::vector<Tensor> tmpTensors, Tensor matrixCTensor, ArchInfo_t archInfo)
{
    if (biasTensor.bytes() > 0) {
        return NOT_SUPPORTED;  // the int8 branch has no caller with a bias
    }
    return matmul_gfx950(matrixATensor.get_desc(), transposeA, ptr_of(matrixATensor), matrixATensor.get_scale(),
        matrixBTensor.get_desc(), transposeB, ptr_of(matrixBTensor), matrixBTensor.get_scale(), tmpTensors[0].bytes(),
        ptr_of(tmpTensors[0]), matrixCTensor.get_desc(), ptr_of(matrixCTensor), archInfo->arch);
}

// ---- int8 convolution (convolution.cpp:28-470) ------------------------------------------------------------------
inline EE convolution_infer_output_size(Tensor *inputTensor, Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    Tensor *outputTensor, DataType targetDataType, ArchInfo_t archInfo)
{
    TensorDesc outputDesc = outputTensor->get_desc();
    EE ret = convolution_infer_output_size_gfx950(
        inputTensor->get_desc(), filterTensor.get_desc(), convParamSpec, &outputDesc, targetDataType, archInfo->arch);
    if (ret == SUCCESS) {
        outputTensor->resize(outputDesc);
    }
    return ret;
}

inline EE convolution_infer_forward_algorithm(Tensor inputTensor, Tensor filterTensor, Tensor outputTensor,
    ConvolutionParamSpec convParamSpec, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm,
    DataType targetDataType, ActivationParamSpec activationDesc, ArchInfo_t archInfo)
{
    return convolution_infer_forward_algorithm_gfx950(inputTensor.get_desc(), filterTensor.get_desc(), outputTensor.get_desc(),
        convParamSpec, policy, algorithm, targetDataType, activationDesc, archInfo->arch);
}

inline EE convolution_transform_filter_bytes(Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, void *bytes, ArchInfo_t archInfo)
{
    return convolution_transform_filter_bytes_gfx950(filterTensor.get_desc(), convParamSpec, algorithm, (U32 *)bytes, archInfo->arch);
}

inline EE convolution_transform_filter(Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, Tensor tmpTensor, Tensor *ftmTensor, ArchInfo_t archInfo)
{
    (void)tmpTensor;
    TensorDesc ftmDesc = ftmTensor->get_desc();
    EE ret = convolution_transform_filter_gfx950(filterTensor.get_desc(), ptr_of(filterTensor), convParamSpec, algorithm, &ftmDesc,
        ptr_of(*ftmTensor), archInfo->arch);
    if (ret == SUCCESS) {
        ftmTensor->resize(ftmDesc);
    }
    return ret;
}

inline EE convolution_infer_forward_tmp_bytes(Tensor inputTensor, Tensor filterTensor, Tensor outputTensor,
    ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, U32 *bytes, ArchInfo_t archInfo)
{
    return convolution_infer_forward_tmp_bytes_gfx950(inputTensor.get_desc(), filterTensor.get_desc(), outputTensor.get_desc(),
        convParamSpec, algorithm, bytes, archInfo->arch);
}

// scale: F32[3] = {input scale, output scale (written), filter scale}, as ConvolutionCPU hands it over
inline EE convolution(std::vector<Tensor> inputTensors, Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, void *scale, Tensor biasTensor, std::vector<Tensor> tmpTensors,
    Tensor outputTensor, ActivationParamSpec activationDesc, ArchInfo_t archInfo)
{
    void *eltwiseInput = nullptr;
    if (inputTensors.size() > 1) {
        // fused add: only the form the x86 path fuses too, an fp32 tensor laid out like the output (convolution.cpp:398-410)
        TensorDesc e = inputTensors[1].get_desc(), o = outputTensor.get_desc();
        if (tensorNumElements(e) != tensorNumElements(o) || e.df != o.df) {
            return NOT_SUPPORTED;
        }
        eltwiseInput = ptr_of(inputTensors[1]);
    }
    return convolution_gfx950(inputTensors[0].get_desc(), ptr_of(inputTensors[0]), eltwiseInput, filterTensor.get_desc(),
        ptr_of(filterTensor), convParamSpec, algorithm, biasTensor.get_desc(), ptr_of(biasTensor), tmpTensors[0].bytes(),
        ptr_of(tmpTensors[0]), outputTensor.get_desc(), ptr_of(outputTensor), (F32 *)scale, activationDesc, archInfo->arch);
}

// ---- int8 deconvolution (deconvolution.cpp:23-279) ---------------------------------------------------------------
inline EE deconvolution_infer_output_size(Tensor *inputTensor, Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    Tensor *outputTensor, DataType targetDataType, ArchInfo_t archInfo)
{
    TensorDesc outputDesc = outputTensor->get_desc();
    EE ret = deconvolution_infer_output_size_gfx950(
        inputTensor->get_desc(), filterTensor.get_desc(), convParamSpec, &outputDesc, targetDataType, archInfo->arch);
    if (ret == SUCCESS) {
        outputTensor->resize(outputDesc);
    }
    return ret;
}

// activationDesc does not take part in the choice on x86 either (cpu/deconvolution.cpp:23-55)
inline EE deconvolution_infer_forward_algorithm(Tensor inputTensor, Tensor filterTensor, Tensor outputTensor,
    ConvolutionParamSpec convParamSpec, ConvolutionPolicy policy, ConvolutionForwardAlgorithm *algorithm,
    DataType targetDataType, ActivationParamSpec activationDesc, ArchInfo_t archInfo)
{
    (void)activationDesc;
    return deconvolution_infer_forward_algorithm_gfx950(inputTensor.get_desc(), filterTensor.get_desc(),
        outputTensor.get_desc(), convParamSpec, policy, algorithm, targetDataType, archInfo->arch);
}

inline EE deconvolution_transform_filter_bytes(Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, void *bytes, ArchInfo_t archInfo)
{
    return deconvolution_transform_filter_bytes_gfx950(
        filterTensor.get_desc(), convParamSpec, algorithm, (U32 *)bytes, archInfo->arch);
}

inline EE deconvolution_transform_filter(Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, Tensor tmpTensor, Tensor *ftmTensor, ArchInfo_t archInfo)
{
    (void)tmpTensor;
    TensorDesc ftmDesc = ftmTensor->get_desc();
    EE ret = deconvolution_transform_filter_gfx950(filterTensor.get_desc(), ptr_of(filterTensor), convParamSpec, algorithm,
        &ftmDesc, ptr_of(*ftmTensor), archInfo->arch);
    if (ret == SUCCESS) {
        ftmTensor->resize(ftmDesc);
    }
    return ret;
}

inline EE deconvolution_infer_forward_tmp_bytes(Tensor inputTensor, Tensor filterTensor, Tensor outputTensor,
    ConvolutionParamSpec convParamSpec, ConvolutionForwardAlgorithm algorithm, U32 *bytes, ArchInfo_t archInfo)
{
    return deconvolution_infer_forward_tmp_bytes_gfx950(inputTensor.get_desc(), filterTensor.get_desc(),
        outputTensor.get_desc(), convParamSpec, algorithm, bytes, archInfo->arch);
}

// scale: host F32[3]: scale[0] = input scale, scale[1] = output scale (in / out: below 0 = dynamic, rewritten with the
// scale the call chose), scale[2] = filter scale -- the order DeconvolutionCPU::run fills them in
// (deconvolution_cpu.hpp:65-84); the scale descriptor is the filter's, as deconvolution.cpp:255 passes it
inline EE deconvolution(Tensor inputTensor, Tensor filterTensor, ConvolutionParamSpec convParamSpec,
    ConvolutionForwardAlgorithm algorithm, void *scale, Tensor biasTensor, Tensor tmpTensor, Tensor outputTensor,
    ActivationParamSpec activationDesc, ArchInfo_t archInfo)
{
    return deconvolution_gfx950(inputTensor.get_desc(), ptr_of(inputTensor), filterTensor.get_desc(), ptr_of(filterTensor),
        convParamSpec, algorithm, filterTensor.get_desc(), scale, biasTensor.get_desc(), ptr_of(biasTensor), tmpTensor.bytes(),
        ptr_of(tmpTensor), outputTensor.get_desc(), ptr_of(outputTensor), activationDesc, archInfo->arch);
}

}  // namespace bolt_gfx950

#endif  // BOLT_GFX950_TENSOR_HPP
