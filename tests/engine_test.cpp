// The engine's operator classes for the gfx950 back end (include/bolt_gfx950_engine.hpp) next to Bolt's own CPU
// classes, driven the way the engine drives an operator (inference/engine/include/cnn.hpp: create as the factory does,
// factory_cpu.hpp:98-218 -> init_feature_scale -> infer_output_tensors_size -> set_weightspec +
// init_weight_bias_from_model -> set tensors -> infer_forward_algorithm -> transform_filter -> infer_tmp_memory_size +
// set_tmp_memory -> run), the CPU class on X86_AVX512 with host tensors, the gfx950 class on AMD_GFX950_DEVICE with
// every activation in DEVICE memory from the first operator's input to the last operator's output. Compared: the
// descs the two infer, every byte of every intermediate and final tensor, and the scales the tensors carry.
//   1. QuantizeLinear -> FullyConnected (u8 out) -> FullyConnected (fp32 out, a -2 record), fp32 weights quantised at
//      load, with nothing calibrated (all scales dynamic) and with calibrated input scales;
//   2. the same chain at one row (the GEMV route), also with a calibrated (static) output scale;
//   3. Convolution 3x3 + ReLU (u8 out) -> Convolution 1x1 (u8 out), fp32 filters quantised at load, dynamic and
//      calibrated scales;
//   4. MatMul of two quantised tensors (batched, second operand transposed).
// Built by `make -C oracle engine` where the reference checkout is present; the binary lands in oracle/_ref/ and
// tests/test_gpu_engine.py runs it on the GPU box. Exit code 0 = everything equal.
#include <cmath>
#include <cstdio>
#include <cstdlib>
#include <cstring>
#include <vector>

#include "tensor_computing.h"
#include "blas_enhance.h"
#include "bolt_gfx950_engine.hpp"

using bolt_gfx950::ConvolutionGFX950;
using bolt_gfx950::FullyConnectedGFX950;
using bolt_gfx950::MatMulGFX950;
using bolt_gfx950::QuantizeLinearGFX950;

// ENGINE_TEST_CPU_ONLY=1: only Bolt's own classes are driven (no GPU needed; nothing is compared) -- checks the driver
static int g_sides = 2;
static unsigned long long g_seed = 20240701ull;
static unsigned rnd()
{
    g_seed = g_seed * 6364136223846793005ull + 1442695040888963407ull;
    return (unsigned)(g_seed >> 33);
}
static float gauss()
{
    float s = 0;
    for (int i = 0; i < 12; ++i) {
        s += (float)(rnd() & 0xffff) / 65536.0f;
    }
    return s - 6.0f;
}
static void *hp(Tensor t)
{
    return ((CpuMemory *)(t.get_memory()))->get_ptr();
}
static Tensor host_tensor(TensorDesc d)
{
    return Tensor::alloc_sized<CPUMem>(d);
}
static Tensor make(TensorDesc d, bool device)
{
    return device ? bolt_gfx950::device_tensor(d) : host_tensor(d);
}
static Tensor to_device(Tensor h)
{
    Tensor d = bolt_gfx950::device_tensor(h.get_desc());
    d.set_scale(h.get_scale());
    CHECK_STATUS(bolt_gfx950::upload(h, &d));
    return d;
}
static Tensor to_host(Tensor t, bool device)
{
    if (!device) {
        return t;
    }
    Tensor h = host_tensor(t.get_desc());
    CHECK_STATUS(bolt_gfx950::download(t, &h));
    h.set_scale(t.get_scale());
    return h;
}
static bool same_desc(TensorDesc a, TensorDesc b)
{
    if (a.dt != b.dt || a.df != b.df || a.nDims != b.nDims) {
        return false;
    }
    for (U32 i = 0; i < a.nDims; ++i) {
        if (a.dims[i] != b.dims[i]) {
            return false;
        }
    }
    return true;
}
static int same(const char *what, Tensor cpu, Tensor gpu, bool with_scale)
{
    Tensor g = to_host(gpu, true);
    if (!same_desc(cpu.get_desc(), g.get_desc())) {
        printf("MISMATCH (desc): %s\n", what);
        return 1;
    }
    if (cpu.bytes() != g.bytes() || memcmp(hp(cpu), hp(g), cpu.bytes()) != 0) {
        printf("MISMATCH (bytes): %s\n", what);
        return 1;
    }
    if (with_scale && cpu.get_scale() != gpu.get_scale()) {
        printf("MISMATCH (scale %g against %g): %s\n", cpu.get_scale(), gpu.get_scale(), what);
        return 1;
    }
    printf("equal: %s (%u bytes, scale %g)\n", what, cpu.bytes(), with_scale ? cpu.get_scale() : 0.0f);
    return 0;
}

struct Scales {
    std::vector<std::vector<F32>> rec;
    std::vector<QuantSpec> spec;
    void build()
    {
        spec.resize(rec.size());
        for (size_t i = 0; i < rec.size(); ++i) {
            spec[i].num_scale = (int)rec[i].size();
            spec[i].scale = rec[i].data();
        }
    }
};

// the engine's call order for one operator; returns its output tensor
template <class OP>
static Tensor drive(OP &op, std::vector<Tensor> inputs, Scales &fs, WeightSpec *ws, bool device, bool weighted,
    std::shared_ptr<AlgorithmMap> amap)
{
    fs.build();
    if (!fs.spec.empty()) {
        op.init_feature_scale((U32)fs.spec.size(), fs.spec.data());
    }
    std::vector<Tensor *> in;
    for (auto &t : inputs) {
        in.push_back(&t);
    }
    Tensor out;
    std::vector<Tensor *> outp(1, &out);
    CHECK_STATUS(op.infer_output_tensors_size(in, outp));
    Tensor outAlloc = make(out.get_desc(), device);
    outAlloc.set_scale(-1);
    std::vector<Tensor> outs(1, outAlloc);
    op.set_input_tensors(inputs);
    op.set_output_tensors(outs);
    op.set_algorithm_map(amap);
    CHECK_STATUS(op.infer_forward_algorithm(amap));
    (void)ws;
    (void)weighted;
    const U32 bytes = op.infer_tmp_memory_size();
    op.set_tmp_memory(make(tensor1d(DT_U8, bytes > 0 ? bytes : 1), device));
    op.run();
    return op.get_output_tensors()[0];
}

template <class OP>
static Tensor drive_weighted(OP &op, std::vector<Tensor> inputs, Scales &fs, WeightSpec *ws, bool device,
    std::shared_ptr<AlgorithmMap> amap)
{
    fs.build();
    if (!fs.spec.empty()) {
        op.init_feature_scale((U32)fs.spec.size(), fs.spec.data());
    }
    std::vector<Tensor *> in;
    for (auto &t : inputs) {
        in.push_back(&t);
    }
    Tensor out;
    std::vector<Tensor *> outp(1, &out);
    CHECK_STATUS(op.infer_output_tensors_size(in, outp));
    op.set_weightspec(*ws);
    CHECK_STATUS(op.init_weight_bias_from_model(nullptr));
    Tensor outAlloc = make(out.get_desc(), device);
    outAlloc.set_scale(-1);
    std::vector<Tensor> outs(1, outAlloc);
    op.set_input_tensors(inputs);
    op.set_output_tensors(outs);
    op.set_algorithm_map(amap);
    CHECK_STATUS(op.infer_forward_algorithm(amap));
    CHECK_STATUS(op.transform_filter());
    const U32 bytes = op.infer_tmp_memory_size();
    op.set_tmp_memory(make(tensor1d(DT_U8, bytes > 0 ? bytes : 1), device));
    op.run();
    return op.get_output_tensors()[0];
}

static WeightSpec weights_f32(std::vector<F32> &w, std::vector<F32> &b)
{
    WeightSpec ws;
    memset(ws.op_name, 0, sizeof(ws.op_name));
    ws.mdt = DT_F32;
    ws.bytes_of_weight = (U32)(w.size() * 4);
    ws.weight = (U8 *)w.data();
    ws.bytes_of_vec = (U32)(b.size() * 4);
    ws.vec = (U8 *)b.data();
    return ws;
}

static int chain_quantize_fc_fc(U32 M, int mode)
{
    // mode 0: nothing calibrated (every scale dynamic); 1: calibrated input scales; 2: the first FullyConnected also has a
    // calibrated (static) output scale -- one row only: with more rows the reference's in-kernel u8 result advances
    // 4 * N bytes per row and overruns its output (blas_common_int8.h:587-590), so there is nothing to compare with
    const U32 K = 512, N1 = 256, N2 = 128;
    std::vector<F32> w1(N1 * K), b1(N1), w2(N2 * N1), b2(N2);
    for (auto &v : w1) {
        v = 0.05f * gauss();
    }
    for (auto &v : w2) {
        v = 0.05f * gauss();
    }
    for (auto &v : b1) {
        v = 0.1f * gauss();
    }
    for (auto &v : b2) {
        v = 0.1f * gauss();
    }
    Tensor x = host_tensor(tensor2df(DT_F32, DF_NORMAL, M, K));
    for (U32 i = 0; i < M * K; ++i) {
        ((F32 *)hp(x))[i] = gauss();
    }
    x.set_scale(-1);
    int bad = 0;
    Tensor keep[2][3];
    for (int side = 0; side < g_sides; ++side) {
        const bool device = side == 1;
        const Arch arch = device ? AMD_GFX950_DEVICE : X86_AVX512;
        std::shared_ptr<AlgorithmMap> amap(new AlgorithmMap(arch, "m", "d", DT_F32_8Q));
        QuantizeLinearParamSpec qp;
        qp.axis = 0;
        qp.dt = DT_U8_Q;
        FullyConnectedParamSpec p1, p2;
        memset(&p1, 0, sizeof(p1));
        p1.num_outputs = N1;
        p1.num_slices = 1;
        p2 = p1;
        p2.num_outputs = N2;
        Scales sq, s1, s2;
        // FullyConnectedCPU::infer_output_tensors_size reads the last record unconditionally (fully_connected_cpu.hpp:
        // 147): a quantised FullyConnected always carries records; -1 = "no calibrated value, decide at run time",
        // -2 = "this operator's output stays fp32"
        if (mode == 0) {
            s1.rec = {{-1.0f}, {-1.0f}};
            s2.rec = {{-1.0f}, {-2.0f}};
        } else {
            sq.rec = {{20.0f}};
            s1.rec = {{20.0f}, {mode == 2 ? 9.5f : -1.0f}};
            s2.rec = {{9.5f}, {-2.0f}};
        }
        WeightSpec ws1 = weights_f32(w1, b1), ws2 = weights_f32(w2, b2);
        std::vector<Tensor> in(1, device ? to_device(x) : x);
        Tensor q, o1, o2;
        if (device) {
            QuantizeLinearGFX950 ql(DT_F32_8Q, qp);
            FullyConnectedGFX950 f1(DT_F32_8Q, p1, K), f2(DT_F32_8Q, p2, N1);
            q = drive(ql, in, sq, nullptr, true, false, amap);
            o1 = drive_weighted(f1, std::vector<Tensor>(1, q), s1, &ws1, true, amap);
            o2 = drive_weighted(f2, std::vector<Tensor>(1, o1), s2, &ws2, true, amap);
        } else {
            QuantizeLinearCPU ql(DT_F32_8Q, qp);
            ql.set_schedule(arch);
            FullyConnectedCPU f1(DT_F32_8Q, p1, K), f2(DT_F32_8Q, p2, N1);
            f1.set_schedule(arch);
            f2.set_schedule(arch);
            q = drive(ql, in, sq, nullptr, false, false, amap);
            o1 = drive_weighted(f1, std::vector<Tensor>(1, q), s1, &ws1, false, amap);
            o2 = drive_weighted(f2, std::vector<Tensor>(1, o1), s2, &ws2, false, amap);
        }
        keep[side][0] = q;
        keep[side][1] = o1;
        keep[side][2] = o2;
    }
    if (g_sides < 2) {
        return 0;
    }
    char what[160];
    const char *names[3] = {"QuantizeLinear output", "FullyConnected 1 output (u8)", "FullyConnected 2 output"};
    for (int k = 0; k < 3; ++k) {
        snprintf(what, sizeof(what), "operator chain, %u rows, scale mode %d: %s", M, mode, names[k]);
        const DataType dt = keep[0][k].get_desc().dt;
        bad += same(what, keep[0][k], keep[1][k], dt == DT_U8_Q || dt == DT_I8);
    }
    if (keep[0][2].get_desc().dt != DT_F32) {
        printf("MISMATCH: a -2 record must give an fp32 output\n");
        bad += 1;
    }
    return bad;
}

static int chain_conv_conv(int mode)
{
    const U32 n = 2, ic = 32, ih = 14, iw = 14, oc1 = 64, oc2 = 32;
    std::vector<F32> w1(oc1 * ic * 9), b1(oc1), w2(oc2 * oc1), b2(oc2);
    for (auto &v : w1) {
        v = 0.05f * gauss();
    }
    for (auto &v : w2) {
        v = 0.05f * gauss();
    }
    for (auto &v : b1) {
        v = 0.1f * gauss();
    }
    for (auto &v : b2) {
        v = 0.1f * gauss();
    }
    Tensor x = host_tensor(tensor4df(DT_U8_Q, DF_NCHWC8, n, ic, ih, iw));
    for (U32 i = 0; i < n * ic * ih * iw; ++i) {
        ((UINT8 *)hp(x))[i] = (UINT8)(128 + rnd() % 128);
    }
    x.set_scale(31.5f);
    ConvolutionParamSpec c1;
    memset(&c1, 0, sizeof(c1));
    c1.num_outputs = oc1;
    c1.num_outputs_origin = oc1;
    c1.kernel_t = 1;
    c1.kernel_h = 3;
    c1.kernel_w = 3;
    c1.stride_t = 1;
    c1.stride_h = 1;
    c1.stride_w = 1;
    c1.pad_top = c1.pad_bottom = c1.pad_left = c1.pad_right = 1;
    c1.group = 1;
    c1.dilatedRate_t = 1;
    c1.dilatedRate_h = 1;
    c1.dilatedRate_w = 1;
    c1.convolution_type = CONVOLUTION_POINTWISE;
    c1.round_mode = ROUND_FLOOR;
    ConvolutionParamSpec c2 = c1;
    c2.num_outputs = oc2;
    c2.num_outputs_origin = oc2;
    c2.kernel_h = c2.kernel_w = 1;
    c2.pad_top = c2.pad_bottom = c2.pad_left = c2.pad_right = 0;
    ActivationParamSpec relu, none;
    memset(&relu, 0, sizeof(relu));
    memset(&none, 0, sizeof(none));
    relu.mode = ACTIVATION_RELU;
    none.mode = ACTIVATION_NULL;
    int bad = 0;
    Tensor keep[2][2];
    for (int side = 0; side < g_sides; ++side) {
        const bool device = side == 1;
        const Arch arch = device ? AMD_GFX950_DEVICE : X86_AVX512;
        std::shared_ptr<AlgorithmMap> amap(new AlgorithmMap(arch, "m", "d", DT_F32_8Q));
        Scales s1, s2;
        if (mode == 1) {
            s1.rec = {{31.5f}, {-1.0f}};
            s2.rec = {{-1.0f}, {-1.0f}};
        }
        WeightSpec ws1 = weights_f32(w1, b1), ws2 = weights_f32(w2, b2);
        std::vector<Tensor> in(1, device ? to_device(x) : x);
        Tensor o1, o2;
        if (device) {
            ConvolutionGFX950 a(DT_F32_8Q, c1, none, relu), b(DT_F32_8Q, c2, none, none);
            a.set_name("conv1");
            b.set_name("conv2");
            o1 = drive_weighted(a, in, s1, &ws1, true, amap);
            o2 = drive_weighted(b, std::vector<Tensor>(1, o1), s2, &ws2, true, amap);
        } else {
            ConvolutionCPU a(DT_F32_8Q, c1, none, relu), b(DT_F32_8Q, c2, none, none);
            a.set_schedule(arch);
            b.set_schedule(arch);
            a.set_name("conv1");
            b.set_name("conv2");
            o1 = drive_weighted(a, in, s1, &ws1, false, amap);
            o2 = drive_weighted(b, std::vector<Tensor>(1, o1), s2, &ws2, false, amap);
        }
        keep[side][0] = o1;
        keep[side][1] = o2;
    }
    if (g_sides < 2) {
        return 0;
    }
    char what[160];
    snprintf(what, sizeof(what), "convolution chain, scale mode %d: 3x3 + ReLU output (u8)", mode);
    bad += same(what, keep[0][0], keep[1][0], true);
    snprintf(what, sizeof(what), "convolution chain, scale mode %d: 1x1 output (u8)", mode);
    bad += same(what, keep[0][1], keep[1][1], true);
    return bad;
}

static int matmul_op()
{
    const U32 B = 3, M = 48, K = 64, N = 80;
    Tensor a = host_tensor(tensor3df(DT_U8_Q, DF_NORMAL, B, M, K)), b = host_tensor(tensor3df(DT_I8, DF_NORMAL, B, N, K));
    for (U32 i = 0; i < B * M * K; ++i) {
        ((UINT8 *)hp(a))[i] = (UINT8)(1 + rnd() % 255);
    }
    for (U32 i = 0; i < B * N * K; ++i) {
        ((INT8 *)hp(b))[i] = (INT8)((int)(rnd() % 255) - 127);
    }
    a.set_scale(17.0f);
    b.set_scale(23.0f);
    MatMulParamSpec p;
    p.transpose_a = false;
    p.transpose_b = true;
    Tensor keep[2];
    for (int side = 0; side < g_sides; ++side) {
        const bool device = side == 1;
        const Arch arch = device ? AMD_GFX950_DEVICE : X86_AVX512;
        std::shared_ptr<AlgorithmMap> amap(new AlgorithmMap(arch, "m", "d", DT_F32_8Q));
        Scales s;
        s.rec = {{-2.0f}};  // fp32 result
        std::vector<Tensor> in;
        in.push_back(device ? to_device(a) : a);
        in.push_back(device ? to_device(b) : b);
        if (device) {
            MatMulGFX950 m(DT_F32_8Q, p);
            keep[side] = drive(m, in, s, nullptr, true, false, amap);
        } else {
            MatMulCPU m(DT_F32_8Q, p);
            m.set_schedule(arch);
            keep[side] = drive(m, in, s, nullptr, false, false, amap);
        }
    }
    if (g_sides < 2) {
        return 0;
    }
    return same("MatMul operator: batched u8 x s8^T -> fp32", keep[0], keep[1], false);
}

int main()
{
    setvbuf(stdout, nullptr, _IOLBF, 0);
    if (getenv("ENGINE_TEST_CPU_ONLY")) {
        g_sides = 1;
    } else {
        CHECK_STATUS(bolt_gfx950_init());
    }
    int bad = 0;
    bad += chain_quantize_fc_fc(64, 0);
    bad += chain_quantize_fc_fc(64, 1);
    for (int mode = 0; mode < 3; ++mode) {
        bad += chain_quantize_fc_fc(1, mode);
    }
    bad += chain_conv_conv(0);
    bad += chain_conv_conv(1);
    bad += matmul_op();
    if (g_sides == 2) {
        CHECK_STATUS(bolt_gfx950_synchronize());
    }
    printf(bad ? "FAILED: %d mismatches\n" : "engine operators: all equal (%d mismatches)\n", bad);
    return bad ? 1 : 0;
}
