// Operator classes of Bolt's inference engine for the gfx950 back end: what `Factory::createFullyConnected /
// createConvolution / createMatMul / createQuantizeLinear` return when a model is scheduled on the MI355X.
//
// Each class derives from the engine's own CPU class (inference/engine/include/cpu/fully_connected_cpu.hpp,
// convolution_cpu.hpp, matmul_cpu.hpp, quantizelinear_cpu.hpp) and overrides only what touches tensor DATA:
// `run()`, `transform_filter()`, `infer_tmp_memory_size()`. Everything that is shape or bookkeeping logic --
// `infer_output_tensors_size`, `infer_forward_algorithm`, weight descriptors, the feature-scale records of a quantised
// model -- is the base class's code, run with the operator's arch set to X86_AVX512 for the duration of the call so that
// it answers exactly as on Bolt's x86 int8 path (activations DT_U8_Q, `Operator::get_activation_quant_data_type`,
// operator.hpp:125-136; NCHWC16 outputs). No file under the Bolt checkout is changed.
//
// Memory: the operators work on ordinary CpuMemory tensors. With AMD_GFX950_DEVICE (the default here) the buffers of
// the input / output / tmp tensors must be DEVICE memory (bolt_gfx950::device_tensor), so activations stay on the GPU
// from operator to operator; `transform_filter()` moves the weights and the bias there once, at model load. With
// AMD_GFX950 every buffer is host memory and each call stages through the device (strict drop-in, slow).
//
// Include after Bolt's headers are on the include path (inference/engine/include, compute/tensor/include, ...).
#ifndef BOLT_GFX950_ENGINE_HPP
#define BOLT_GFX950_ENGINE_HPP

#include "cpu/fully_connected_cpu.hpp"
#include "cpu/convolution_cpu.hpp"
#include "cpu/matmul_cpu.hpp"
#include "cpu/quantizelinear_cpu.hpp"

#include "bolt_gfx950_tensor.hpp"

namespace bolt_gfx950 {

// the base class's host-side logic answers as on the x86 int8 path while one of these is alive
struct AsX86 {
    Arch *where;
    Arch keep;
    explicit AsX86(ArchInfo *a) : where(&a->arch), keep(a->arch)
    {
        *where = X86_AVX512;
    }
    ~AsX86()
    {
        *where = keep;
    }
};

// a host tensor's bytes in the memory the operator's arch computes from (a copy on the device, or the tensor itself)
inline Tensor resident(Tensor host, Arch arch)
{
    if (arch != AMD_GFX950_DEVICE || host.bytes() == 0 || ptr_of(host) == nullptr) {
        return host;
    }
    Tensor d = device_tensor(host.get_desc());
    d.set_scale(host.get_scale());
    CHECK_STATUS(upload(host, &d));
    return d;
}

inline Tensor alloc_for(TensorDesc desc, Arch arch)
{
    return arch == AMD_GFX950_DEVICE ? device_tensor(desc) : Tensor::alloc_sized<CPUMem>(desc);
}

// ---- FullyConnected (fully_connected_cpu.hpp:84-250) ------------------------------------------------------------
class FullyConnectedGFX950 : public FullyConnectedCPU {
public:
    FullyConnectedGFX950(DataType dt, FullyConnectedParamSpec p, U32 numInput, Arch arch = AMD_GFX950_DEVICE)
        : FullyConnectedCPU(dt, p, numInput)
    {
        this->archInfo.arch = arch;
    }

    std::shared_ptr<Operator> clone() override
    {
        std::shared_ptr<FullyConnectedGFX950> mem = std::shared_ptr<FullyConnectedGFX950>(
            new FullyConnectedGFX950(this->dt, this->p, this->numInput, this->archInfo.arch));
        *mem = *this;
        return mem;
    }

    EE infer_output_tensors_size(std::vector<Tensor *> inTensors, std::vector<Tensor *> outTensors) override
    {
        AsX86 guard(&this->archInfo);
        return FullyConnectedCPU::infer_output_tensors_size(inTensors, outTensors);
    }

    U32 infer_tmp_memory_size() override
    {
        U32 bytes = 0;
        CHECK_STATUS(bolt_gfx950::fully_connected_infer_forward_tmp_bytes(
            this->inputTensors[0], get_weight_tensor(), this->outputTensors[0], &bytes, &this->archInfo));
        return bytes;
    }

    // fully_connected_cpu.hpp:183-250: a weight that is not int8 yet is quantised with its own scale, then packed for the
    // product the operator will run (GEMV row by row, or GEMM); here both steps run on the device and the packed
    // weight and the bias stay there
    EE transform_filter(const TensorDesc &inputDesc) override
    {
        if (use_nchwc8(inputDesc)) {
            return NOT_SUPPORTED;  // (an NCHWC8 feature map flattened into FullyConnected: the weight reorder of :187-196)
        }
        const Arch arch = this->archInfo.arch;
        Tensor tTensor = this->weightTensors[0];
        TensorDesc desc = tTensor.get_desc();
        if (this->mvm) {
            desc.df = DF_NORMAL;
        }
        tTensor.resize(desc);
        tTensor = resident(tTensor, arch);
        const bool thisIsNoQuant = (featureScale.size() > 1 && featureScale[0].back() == 0);
        if (isQuantMixDataType(this->dt) && !thisIsNoQuant && desc.dt != DT_I8) {
            desc.dt = DT_I8;
            Tensor qTensor = alloc_for(desc, arch);
            F32 scale = -1;
            CHECK_STATUS(bolt_gfx950::quantize(tTensor, &qTensor, &scale, &this->archInfo));
            qTensor.set_scale(scale);
            tTensor = qTensor;
        }
        Tensor wtm;
        CHECK_STATUS(bolt_gfx950::fully_connected_transform_weight(tTensor, this->mvm, &wtm, &this->archInfo));
        this->weightTensors[0] = wtm;
        if (this->biasTensors.size() > 0) {
            this->biasTensors[0] = resident(this->biasTensors[0], arch);
        }
        return SUCCESS;
    }

    using FullyConnectedCPU::transform_filter;

    void run() override
    {
        Tensor weightTensor = get_weight_tensor();
        Tensor biasTensor = get_bias_tensor();
        Tensor outputTensor = this->outputTensors[0];
        // the feature-scale rule of fully_connected_cpu.hpp:92-103
        TensorDesc inputDesc = this->inputTensors[0].get_desc();
        TensorDesc outputDesc = outputTensor.get_desc();
        if (featureScale.size() > 1 && featureScale[0][0] > 0 && DT_I8 != inputDesc.dt && DT_U8_Q != inputDesc.dt) {
            this->inputTensors[0].set_scale(featureScale[0][0]);
        }
        if (DT_I8 == outputDesc.dt || DT_U8_Q == outputDesc.dt) {
            if (featureScale.size() > 0) {
                outputTensor.set_scale((featureScale.back())[0]);
            } else {
                outputTensor.set_scale(-1);
            }
        }
        std::vector<Tensor> tmpTensor(1, this->temp);
        CHECK_STATUS(bolt_gfx950::fully_connected(
            this->inputTensors[0], weightTensor, biasTensor, tmpTensor, outputTensor, &this->archInfo));
    }
};

// ---- Convolution (convolution_cpu.hpp:127-560), the int8 CONVOLUTION_POINTWISE / CONVOLUTION_DILATION types ----------
class ConvolutionGFX950 : public ConvolutionCPU {
public:
    ConvolutionGFX950(DataType dt, ConvolutionParamSpec p, ActivationParamSpec dwActivationParamSpec,
        ActivationParamSpec pwActivationParamSpec, Arch arch = AMD_GFX950_DEVICE)
        : ConvolutionCPU(dt, p, dwActivationParamSpec, pwActivationParamSpec)
    {
        this->archInfo.arch = arch;
    }

    std::shared_ptr<Operator> clone() override
    {
        std::shared_ptr<ConvolutionGFX950> mem = std::shared_ptr<ConvolutionGFX950>(new ConvolutionGFX950(
            this->dt, this->p, this->dwActivationParamSpec, this->pwActivationParamSpec, this->archInfo.arch));
        *mem = *this;
        return mem;
    }

    bool on_this_path() const
    {
        return isQuantMixDataType(this->dt) &&
            (this->p.convolution_type == CONVOLUTION_POINTWISE || this->p.convolution_type == CONVOLUTION_DILATION);
    }

    EE infer_output_tensors_size(std::vector<Tensor *> inTensors, std::vector<Tensor *> outTensors) override
    {
        AsX86 guard(&this->archInfo);
        return ConvolutionCPU::infer_output_tensors_size(inTensors, outTensors);
    }

    EE infer_forward_algorithm(std::shared_ptr<AlgorithmMap> algorithmMap) override
    {
        AsX86 guard(&this->archInfo);
        return ConvolutionCPU::infer_forward_algorithm(algorithmMap);
    }

    U32 infer_tmp_memory_size() override
    {
        if (!on_this_path()) {
            UNI_ERROR_LOG("the gfx950 convolution operator runs quantised pointwise / dilated convolutions only\n");
            return 0;
        }
        Tensor inputTensor = this->inputTensors[0];
        inputTensor.resize(transformDescTo4d(inputTensor.get_desc()));
        Tensor outputTensor = this->outputTensors[0];
        outputTensor.resize(transformDescTo4d(outputTensor.get_desc()));
        U32 bytes = 0;
        CHECK_STATUS(bolt_gfx950::convolution_infer_forward_tmp_bytes(
            inputTensor, this->weightTensors[0], outputTensor, p, this->pwAlg, &bytes, &this->archInfo));
        return bytes;
    }

    // convolution_cpu.hpp:497-521: scales[2] = the filter's scale (its own, when it arrives as fp32 and is quantised
    // here), then the filter in the layout the kernels read; the bias follows the filter to the device
    EE transform_filter() override
    {
        if (!on_this_path()) {
            return NOT_SUPPORTED;
        }
        const Arch arch = this->archInfo.arch;
        Tensor filterTensor = resident(this->weightTensors[0], arch);
        TensorDesc qDesc = filterTensor.get_desc();
        this->scales = std::shared_ptr<F32>((F32 *)operator new(3 * bytesOf(DT_F32)));
        if (qDesc.dt != DT_I8) {
            qDesc.dt = DT_I8;
            Tensor qFilterTensor = alloc_for(qDesc, arch);
            this->scales.get()[2] = -1;
            CHECK_STATUS(bolt_gfx950::quantize(filterTensor, &qFilterTensor, this->scales.get() + 2, &this->archInfo));
            filterTensor = qFilterTensor;
            filterTensor.set_scale(this->scales.get()[2]);
        } else {
            this->scales.get()[2] = filterTensor.get_scale();
        }
        U32 ftmBytes = 0;
        CHECK_STATUS(bolt_gfx950::convolution_transform_filter_bytes(filterTensor, this->p, this->pwAlg, &ftmBytes, &this->archInfo));
        Tensor wtm = alloc_for(tensor1d(DT_U8, ftmBytes), arch);
        CHECK_STATUS(bolt_gfx950::convolution_transform_filter(filterTensor, this->p, this->pwAlg, this->temp, &wtm, &this->archInfo));
        this->weightTensors[0] = wtm;
        this->biasTensors[0] = resident(this->biasTensors[0], arch);
        return SUCCESS;
    }

    void run() override
    {
        if (!on_this_path()) {
            UNI_ERROR_LOG("the gfx950 convolution operator runs quantised pointwise / dilated convolutions only\n");
            return;
        }
        Tensor inputTensor = this->inputTensors[0];
        Tensor outputTensor = this->outputTensors[0];
        TensorDesc oriInputDesc = inputTensor.get_desc();
        inputTensor.resize(transformDescTo4d(oriInputDesc));
        TensorDesc oriOutputDesc = outputTensor.get_desc();
        TensorDesc outputDesc = transformDescTo4d(oriOutputDesc);
        outputTensor.resize(outputDesc);
        // the feature-scale rule of convolution_cpu.hpp:143-157
        F32 *scalePtr = this->scales.get();
        TensorDesc inputDesc = inputTensor.get_desc();
        scalePtr[0] = inputTensor.get_scale();
        if (DT_I8 != inputDesc.dt && DT_U8_Q != inputDesc.dt && featureScale.size() > 0 && featureScale[0][0] > 0) {
            scalePtr[0] = featureScale[0][0];
        }
        if (featureScale.size() > 0 && (featureScale.back())[0] != -2) {
            scalePtr[1] = (featureScale.back())[0];
        } else {
            scalePtr[1] = -1;
        }
        std::vector<Tensor> ins = this->inputTensors;
        ins[0] = inputTensor;
        std::vector<Tensor> tmpTensors(1, this->temp);
        CHECK_STATUS(bolt_gfx950::convolution(ins, this->weightTensors[0], p, this->pwAlg, scalePtr, this->biasTensors[0],
            tmpTensors, outputTensor, this->pwActivationParamSpec, &this->archInfo));
        if (DT_I8 == outputDesc.dt || DT_U8_Q == outputDesc.dt) {
            outputTensor.set_scale(scalePtr[1]);
        }
        inputTensor.resize(oriInputDesc);
        outputTensor.resize(oriOutputDesc);
    }
};

// ---- MatMul (matmul_cpu.hpp:31-87) -----------------------------------------------------------------------------------
class MatMulGFX950 : public MatMulCPU {
public:
    MatMulGFX950(DataType dt, MatMulParamSpec p, Arch arch = AMD_GFX950_DEVICE) : MatMulCPU(dt, p)
    {
        this->archInfo.arch = arch;
    }

    std::shared_ptr<Operator> clone() override
    {
        std::shared_ptr<MatMulGFX950> mem = std::shared_ptr<MatMulGFX950>(new MatMulGFX950(this->dt, this->p, this->archInfo.arch));
        *mem = *this;
        return mem;
    }

    EE infer_output_tensors_size(std::vector<Tensor *> inTensors, std::vector<Tensor *> outTensors) override
    {
        AsX86 guard(&this->archInfo);
        return MatMulCPU::infer_output_tensors_size(inTensors, outTensors);
    }

    U32 infer_tmp_memory_size() override
    {
        U32 bytes = 0;
        CHECK_STATUS(bolt_gfx950::matmul_infer_forward_tmp_bytes(inputTensors[0], this->p.transpose_a, inputTensors[1],
            this->p.transpose_b, outputTensors[0], &bytes, &this->archInfo));
        return bytes;
    }

    void run() override
    {
        Tensor inputTensorA = this->inputTensors[0];
        Tensor inputTensorB = this->inputTensors[1];
        Tensor inputTensorC;
        if (this->inputTensors.size() > 2) {
            inputTensorC = this->inputTensors[2];
        }
        Tensor outputTensor = this->outputTensors[0];
        // matmul_cpu.hpp:42-56
        TensorDesc inputDescA = inputTensorA.get_desc();
        TensorDesc inputDescB = inputTensorB.get_desc();
        if (3 == featureScale.size() && featureScale[0][0] > 0 && DT_I8 != inputDescA.dt && DT_U8_Q != inputDescA.dt) {
            inputTensorA.set_scale(featureScale[0][0]);
        }
        if (3 == featureScale.size() && featureScale[1][0] > 0 && DT_I8 != inputDescB.dt && DT_U8_Q != inputDescB.dt) {
            inputTensorB.set_scale(featureScale[1][0]);
        }
        if (featureScale.size() > 0) {
            outputTensor.set_scale((featureScale.back())[0]);
        }
        std::vector<Tensor> tmpTensor(1, this->temp);
        CHECK_STATUS(bolt_gfx950::matmul(inputTensors[0], this->p.transpose_a, inputTensors[1], this->p.transpose_b,
            inputTensorC, tmpTensor, outputTensors[0], &this->archInfo));
    }
};

// ---- QuantizeLinear (quantizelinear_cpu.hpp:32-72) -------------------------------------------------------------------
class QuantizeLinearGFX950 : public QuantizeLinearCPU {
public:
    QuantizeLinearGFX950(DataType dt, QuantizeLinearParamSpec p, Arch arch = AMD_GFX950_DEVICE) : QuantizeLinearCPU(dt, p)
    {
        this->archInfo.arch = arch;
    }

    std::shared_ptr<Operator> clone() override
    {
        std::shared_ptr<QuantizeLinearGFX950> mem =
            std::shared_ptr<QuantizeLinearGFX950>(new QuantizeLinearGFX950(this->dt, this->p, this->archInfo.arch));
        *mem = *this;
        return mem;
    }

    EE infer_output_tensors_size(std::vector<Tensor *> inTensors, std::vector<Tensor *> outTensors) override
    {
        AsX86 guard(&this->archInfo);
        return QuantizeLinearCPU::infer_output_tensors_size(inTensors, outTensors);
    }

    void run() override
    {
        F32 scale = -1;  // default per layer
        TensorDesc inputDesc = this->inputTensors[0].get_desc();
        TensorDesc outputDesc = this->outputTensors[0].get_desc();
        if (inputDesc.dt == outputDesc.dt) {
            if (this->archInfo.arch == AMD_GFX950_DEVICE) {
                CHECK_STATUS(bolt_gfx950_memcpy_d2d(ptr_of(this->outputTensors[0]), ptr_of(this->inputTensors[0]), tensorNumBytes(inputDesc)));
            } else {
                UNI_MEMCPY(ptr_of(this->outputTensors[0]), ptr_of(this->inputTensors[0]), tensorNumBytes(inputDesc));
            }
            return;
        }
        if (featureScale.size() > 0 && featureScale[0].size() > 0 && featureScale[0][0] > 0) {
            scale = featureScale[0][0];
        }
        if (scale <= 0) {
            scale = this->inputTensors[0].get_scale();
        }
        CHECK_STATUS(bolt_gfx950::quantize(this->inputTensors[0], &this->outputTensors[0], &scale, &this->archInfo));
        this->outputTensors[0].set_scale(scale);
    }
};

}  // namespace bolt_gfx950

// The factory a model scheduled on the MI355X is built with (inference/engine/include/cpu/factory_cpu.hpp:98-218): the
// four operators of this path come from the classes above, every other operator from the CPU factory it derives from.
// Needs all of the engine's operator headers (and, to link, all of Bolt), so it is only compiled where asked for.
#ifdef BOLT_GFX950_WITH_FACTORY
#include "cpu/factory_cpu.hpp"

class FactoryGFX950 : public FactoryCPU {
public:
    explicit FactoryGFX950(Arch arch = AMD_GFX950_DEVICE) : arch(arch)
    {}

    std::shared_ptr<Operator> createConvolution(DataType dt, ConvolutionParamSpec p, ActivationParamSpec dwActivationParamSpec,
        ActivationParamSpec pwActivationParamSpec) override
    {
        const bool ours = isQuantMixDataType(dt) && (p.convolution_type == CONVOLUTION_POINTWISE || p.convolution_type == CONVOLUTION_DILATION);
        if (!ours) {
            return FactoryCPU::createConvolution(dt, p, dwActivationParamSpec, pwActivationParamSpec);
        }
        auto cep = (Convolution *)(new bolt_gfx950::ConvolutionGFX950(dt, p, dwActivationParamSpec, pwActivationParamSpec, arch));
        return std::shared_ptr<Operator>(cep);
    }

    std::shared_ptr<Operator> createFullyConnected(DataType dt, FullyConnectedParamSpec p, U32 numInput) override
    {
        if (!isQuantMixDataType(dt)) {
            return FactoryCPU::createFullyConnected(dt, p, numInput);
        }
        auto cep = (FullyConnected *)(new bolt_gfx950::FullyConnectedGFX950(dt, p, numInput, arch));
        return std::shared_ptr<Operator>(cep);
    }

    std::shared_ptr<Operator> createQuantizeLinear(DataType dt, QuantizeLinearParamSpec p) override
    {
        auto cep = new bolt_gfx950::QuantizeLinearGFX950(dt, p, arch);
        return std::shared_ptr<Operator>(cep);
    }

    std::shared_ptr<Operator> createMatMul(DataType dt, MatMulParamSpec p) override
    {
        if (!isQuantMixDataType(dt)) {
            return FactoryCPU::createMatMul(dt, p);
        }
        auto cep = (MatMul *)(new bolt_gfx950::MatMulGFX950(dt, p, arch));
        return std::shared_ptr<Operator>(cep);
    }

private:
    Arch arch;
};
#endif  // BOLT_GFX950_WITH_FACTORY

#endif  // BOLT_GFX950_ENGINE_HPP
