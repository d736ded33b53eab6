// Runs Bolt's own Tensor-level operators (compiled from the reference's sources into oracle/_ref/libboltref.so) and
// the gfx950 library through include/bolt_gfx950_tensor.hpp side by side, Tensor for Tensor, and compares bytes:
//   1. QuantizeLinear -> FullyConnected (u8 out, dynamic scale) -> FullyConnected (fp32 out), the activations staying in
//      DEVICE memory between the three operators (Arch AMD_GFX950_DEVICE: only the layer input goes up and only the final
//      output comes down), and the same chain with host pointers (AMD_GFX950);
//   2. an int8 3x3 convolution with ReLU and a u8 result through the six convolution_* calls;
//   3. an int8 4x4 stride-2 deconvolution with ReLU and a u8 result through the six deconvolution_* calls;
//   4. a batched int8 matmul.
// Built by `make -C oracle glue` where the reference checkout is present (this file includes Bolt's headers); the
// binary lands in oracle/_ref/ and tests/test_gpu_glue.py runs it on the GPU box. Exit code 0 = everything equal.
#include <cmath>
#include <cstdio>
#include <cstring>
#include <vector>

#include "tensor_computing.h"
#include "blas_enhance.h"
#include "bolt_gfx950_tensor.hpp"

static ArchInfo g_x86 = {X86_AVX512, nullptr};
static ArchInfo g_host = {AMD_GFX950, nullptr};
static ArchInfo g_dev = {AMD_GFX950_DEVICE, nullptr};

static unsigned long long g_seed = 20240601ull;
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

static Tensor host_tensor(TensorDesc d)
{
    return Tensor::alloc_sized<CPUMem>(d);
}
static void *hp(Tensor t)
{
    return ((CpuMemory *)(t.get_memory()))->get_ptr();
}
static Tensor to_device(Tensor h)
{
    Tensor d = bolt_gfx950::device_tensor(h.get_desc());
    d.set_scale(h.get_scale());
    CHECK_STATUS(bolt_gfx950::upload(h, &d));
    return d;
}
static int same(const char *what, Tensor a, Tensor b)
{
    if (a.bytes() != b.bytes() || memcmp(hp(a), hp(b), a.bytes()) != 0) {
        printf("MISMATCH: %s\n", what);
        return 1;
    }
    printf("equal: %s (%u bytes)\n", what, a.bytes());
    return 0;
}

// the engine's weight transform for the x86 path (fully_connected_cpu.hpp:231-248)
static Tensor ref_transform_weight(Tensor w)
{
    TensorDesc fDesc = w.get_desc(), tDesc;
    U32 bytes = 0;
    CHECK_STATUS(matrix_matrix_multiply_transform_rhs_bytes(fDesc, &bytes, nullptr, X86_AVX512));
    Tensor wtm = host_tensor(tensor1d(DT_U8, bytes));
    CHECK_STATUS(matrix_matrix_multiply_transform_rhs(fDesc, hp(w), &tDesc, hp(wtm), X86_AVX512));
    wtm.resize(tDesc);
    wtm.set_scale(w.get_scale());
    return wtm;
}

template <class FC, class TMPB>
static Tensor run_fc(FC fc, TMPB tmp_bytes, Tensor in, Tensor wtm, Tensor bias, TensorDesc outDesc, ArchInfo_t a, bool device)
{
    Tensor out = device ? bolt_gfx950::device_tensor(outDesc) : host_tensor(outDesc);
    out.set_scale(-1);
    U32 bytes = 0;
    CHECK_STATUS(tmp_bytes(in, wtm, out, &bytes, a));
    Tensor tmp = device ? bolt_gfx950::device_tensor(tensor1d(DT_U8, bytes)) : host_tensor(tensor1d(DT_U8, bytes));
    std::vector<Tensor> tmps(1, tmp);
    CHECK_STATUS(fc(in, wtm, bias, tmps, out, a));
    return out;
}

static int chain_quantize_fc_fc()
{
    const U32 M = 64, K = 1024, N1 = 512, N2 = 256;
    Tensor x = host_tensor(tensor2df(DT_F32, DF_NORMAL, M, K));
    for (U32 i = 0; i < M * K; ++i) {
        ((F32 *)hp(x))[i] = gauss();
    }
    Tensor w1 = host_tensor(tensor2df(DT_I8, DF_TRANSPOSE, N1, K)), w2 = host_tensor(tensor2df(DT_I8, DF_TRANSPOSE, N2, N1));
    for (U32 i = 0; i < N1 * K; ++i) {
        ((INT8 *)hp(w1))[i] = (INT8)((int)(rnd() % 255) - 127);
    }
    for (U32 i = 0; i < N2 * N1; ++i) {
        ((INT8 *)hp(w2))[i] = (INT8)((int)(rnd() % 255) - 127);
    }
    w1.set_scale(100.0f);
    w2.set_scale(64.0f);
    Tensor b1 = host_tensor(tensor1d(DT_F32, N1)), b2 = host_tensor(tensor1d(DT_F32, N2));
    for (U32 i = 0; i < N1; ++i) {
        ((F32 *)hp(b1))[i] = 0.1f * gauss();
    }
    for (U32 i = 0; i < N2; ++i) {
        ((F32 *)hp(b2))[i] = 0.1f * gauss();
    }
    const TensorDesc qd = tensor2df(DT_U8_Q, DF_NORMAL, M, K), o1d = tensor2df(DT_U8_Q, DF_NORMAL, M, N1),
                     o2d = tensor2df(DT_F32, DF_NORMAL, M, N2);

    // the reference
    Tensor xq = host_tensor(qd);
    F32 sI = -1;
    CHECK_STATUS(quantize(x, &xq, &sI, &g_x86));
    xq.set_scale(sI);
    Tensor r1 = run_fc(fully_connected, fully_connected_infer_forward_tmp_bytes, xq, ref_transform_weight(w1), b1, o1d, &g_x86, false);
    Tensor r2 = run_fc(fully_connected, fully_connected_infer_forward_tmp_bytes, r1, ref_transform_weight(w2), b2, o2d, &g_x86, false);

    int bad = 0;
    for (int device = 0; device < 2; ++device) {
        ArchInfo_t a = device ? &g_dev : &g_host;
        Tensor gx = device ? to_device(x) : x, gb1 = device ? to_device(b1) : b1, gb2 = device ? to_device(b2) : b2;
        Tensor gw1 = device ? to_device(w1) : w1, gw2 = device ? to_device(w2) : w2;
        Tensor gq = device ? bolt_gfx950::device_tensor(qd) : host_tensor(qd);
        F32 gs = -1;
        CHECK_STATUS(bolt_gfx950::quantize(gx, &gq, &gs, a));
        gq.set_scale(gs);
        Tensor t1, t2;
        CHECK_STATUS(bolt_gfx950::fully_connected_transform_weight(gw1, false, &t1, a));
        CHECK_STATUS(bolt_gfx950::fully_connected_transform_weight(gw2, false, &t2, a));
        Tensor g1 = run_fc(bolt_gfx950::fully_connected, bolt_gfx950::fully_connected_infer_forward_tmp_bytes, gq, t1, gb1, o1d, a, device);
        Tensor g2 = run_fc(bolt_gfx950::fully_connected, bolt_gfx950::fully_connected_infer_forward_tmp_bytes, g1, t2, gb2, o2d, a, device);
        CHECK_STATUS(bolt_gfx950_synchronize());
        Tensor h2 = g2;
        if (device) {  // the only transfer back: the final output (the u8 activations of the middle never left the GPU)
            h2 = host_tensor(o2d);
            CHECK_STATUS(bolt_gfx950::download(g2, &h2));
        }
        if (gs != sI || g1.get_scale() != r1.get_scale()) {
            printf("MISMATCH: scales %g / %g, %g / %g\n", gs, sI, g1.get_scale(), r1.get_scale());
            bad = 1;
        }
        bad |= same(device ? "QuantizeLinear -> FC -> FC, device-resident activations" : "QuantizeLinear -> FC -> FC, host pointers", h2, r2);
    }
    return bad;
}

static int conv_u8()
{
    const U32 n = 2, ic = 32, ih = 14, iw = 14, oc = 64, fh = 3, fw = 3;
    ConvolutionParamSpec p = createConvolutionParamSpec(1, 1, fh, fw, 1, 1, 1, 0, 0, 1, 1, 1, 1, 1, 1, 1, oc, CONVOLUTION_DEPTHWISE_POINTWISE);
    ActivationParamSpec act;
    act.mode = ACTIVATION_RELU;
    Tensor in = host_tensor(tensor4df(DT_U8_Q, DF_NCHWC8, n, ic, ih, iw));
    for (U32 i = 0; i < in.bytes(); ++i) {
        ((U8 *)hp(in))[i] = (U8)(128 + rnd() % 100);
    }
    Tensor filter = host_tensor(tensor4df(DT_I8, DF_NCHW, oc, ic, fh, fw));
    for (U32 i = 0; i < filter.bytes(); ++i) {
        ((INT8 *)hp(filter))[i] = (INT8)((int)(rnd() % 255) - 127);
    }
    Tensor bias = host_tensor(tensor1d(DT_F32, oc));
    for (U32 i = 0; i < oc; ++i) {
        ((F32 *)hp(bias))[i] = 0.1f * gauss();
    }
    Tensor outs[2];
    F32 oscale[2];
    for (int which = 0; which < 2; ++which) {
        const bool gpu = which == 1;
        ArchInfo_t a = gpu ? &g_host : &g_x86;
        Tensor out;
        ConvolutionForwardAlgorithm alg = CONVOLUTION_ALGORITHM_NULL;
        U32 fb = 0, tb = 0;
        Tensor tmp0;
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::convolution_infer_output_size(&in, filter, p, &out, DT_U8_Q, a));
            CHECK_STATUS(bolt_gfx950::convolution_infer_forward_algorithm(in, filter, out, p, CONVOLUTION_FASTEST, &alg, DT_U8_Q, act, a));
            CHECK_STATUS(bolt_gfx950::convolution_transform_filter_bytes(filter, p, alg, &fb, a));
        } else {
            CHECK_STATUS(convolution_infer_output_size(&in, filter, p, &out, DT_U8_Q, a));
            CHECK_STATUS(convolution_infer_forward_algorithm(in, filter, out, p, CONVOLUTION_FASTEST, &alg, DT_U8_Q, act, a));
            CHECK_STATUS(convolution_transform_filter_bytes(filter, p, alg, &fb, a));
        }
        out.alloc();
        Tensor ftm = host_tensor(tensor1d(DT_U8, fb));
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::convolution_transform_filter(filter, p, alg, tmp0, &ftm, a));
            CHECK_STATUS(bolt_gfx950::convolution_infer_forward_tmp_bytes(in, ftm, out, p, alg, &tb, a));
        } else {
            CHECK_STATUS(convolution_transform_filter(filter, p, alg, tmp0, &ftm, a));
            CHECK_STATUS(convolution_infer_forward_tmp_bytes(in, ftm, out, p, alg, &tb, a));
        }
        Tensor tmp = host_tensor(tensor1d(DT_U8, tb));
        std::vector<Tensor> ins(1, in), tmps(1, tmp);
        F32 scales[3] = {31.5f, -1.0f, 80.0f};
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::convolution(ins, ftm, p, alg, scales, bias, tmps, out, act, a));
        } else {
            CHECK_STATUS(convolution(ins, ftm, p, alg, scales, bias, tmps, out, act, a));
        }
        outs[which] = out;
        oscale[which] = scales[1];
    }
    int bad = 0;
    TensorDesc d0 = outs[0].get_desc(), d1 = outs[1].get_desc();
    if (memcmp(&d0, &d1, sizeof(TensorDesc)) != 0 && (d0.dt != d1.dt || d0.df != d1.df || d0.nDims != d1.nDims ||
            memcmp(d0.dims, d1.dims, d0.nDims * sizeof(U32)) != 0)) {
        printf("MISMATCH: convolution output descs\n");
        bad = 1;
    }
    if (oscale[0] != oscale[1]) {
        printf("MISMATCH: convolution output scale %g / %g\n", oscale[1], oscale[0]);
        bad = 1;
    }
    return bad | same("int8 3x3 convolution, ReLU, u8 out, through the six convolution_* calls", outs[1], outs[0]);
}

static int deconv_u8()
{
    const U32 n = 2, ic = 32, ih = 9, iw = 7, oc = 32, fh = 4, fw = 4;
    ConvolutionParamSpec p = createConvolutionParamSpec(1, 1, fh, fw, 1, 2, 2, 0, 0, 1, 1, 1, 1, 1, 1, 1, oc, CONVOLUTION_DECONVOLUTION);
    ActivationParamSpec act;
    act.mode = ACTIVATION_RELU;
    Tensor in = host_tensor(tensor4df(DT_U8_Q, DF_NCHW, n, ic, ih, iw));
    for (U32 i = 0; i < in.bytes(); ++i) {
        ((U8 *)hp(in))[i] = (U8)(128 + (int)(rnd() % 200) - 100);
    }
    Tensor filter = host_tensor(tensor4df(DT_I8, DF_NCHW, ic, oc, fh, fw));
    for (U32 i = 0; i < filter.bytes(); ++i) {
        ((INT8 *)hp(filter))[i] = (INT8)((int)(rnd() % 255) - 127);
    }
    Tensor bias = host_tensor(tensor1d(DT_F32, oc));
    for (U32 i = 0; i < oc; ++i) {
        ((F32 *)hp(bias))[i] = 0.1f * gauss();
    }
    Tensor outs[2];
    F32 got[2][3];
    for (int which = 0; which < 2; ++which) {
        const bool gpu = which == 1;
        ArchInfo_t a = gpu ? &g_host : &g_x86;
        Tensor out, tmp0;
        ConvolutionForwardAlgorithm alg = CONVOLUTION_ALGORITHM_NULL;
        U32 fb = 0, tb = 0;
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::deconvolution_infer_output_size(&in, filter, p, &out, DT_U8_Q, a));
            CHECK_STATUS(bolt_gfx950::deconvolution_infer_forward_algorithm(in, filter, out, p, CONVOLUTION_FASTEST, &alg, DT_U8_Q, act, a));
            CHECK_STATUS(bolt_gfx950::deconvolution_transform_filter_bytes(filter, p, alg, &fb, a));
        } else {
            CHECK_STATUS(deconvolution_infer_output_size(&in, filter, p, &out, DT_U8_Q, a));
            CHECK_STATUS(deconvolution_infer_forward_algorithm(in, filter, out, p, CONVOLUTION_FASTEST, &alg, DT_U8_Q, act, a));
            CHECK_STATUS(deconvolution_transform_filter_bytes(filter, p, alg, &fb, a));
        }
        out.alloc();
        Tensor ftm = host_tensor(tensor1d(DT_U8, fb + 64));
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::deconvolution_transform_filter(filter, p, alg, tmp0, &ftm, a));
            CHECK_STATUS(bolt_gfx950::deconvolution_infer_forward_tmp_bytes(in, ftm, out, p, alg, &tb, a));
        } else {
            CHECK_STATUS(deconvolution_transform_filter(filter, p, alg, tmp0, &ftm, a));
            CHECK_STATUS(deconvolution_infer_forward_tmp_bytes(in, ftm, out, p, alg, &tb, a));
            // the reference's figure leaves out what the product inside needs (cpu/deconvolution.cpp:188-250); the engine
            // covers that by sharing one tmp sized as the maximum over all operators
            tb += n * ih * iw * oc * fh * fw * 8 + (1u << 20);
        }
        Tensor tmp = host_tensor(tensor1d(DT_U8, tb));
        memset(hp(tmp), 0, tb);
        F32 scales[3] = {31.5f, 80.0f, -1.0f};
        if (gpu) {
            CHECK_STATUS(bolt_gfx950::deconvolution(in, ftm, p, alg, scales, bias, tmp, out, act, a));
        } else {
            CHECK_STATUS(deconvolution(in, ftm, p, alg, scales, bias, tmp, out, act, a));
        }
        outs[which] = out;
        memcpy(got[which], scales, sizeof(scales));
    }
    int bad = 0;
    TensorDesc d0 = outs[0].get_desc(), d1 = outs[1].get_desc();
    if (d0.dt != d1.dt || d0.df != d1.df || d0.nDims != d1.nDims || memcmp(d0.dims, d1.dims, d0.nDims * sizeof(U32)) != 0) {
        printf("MISMATCH: deconvolution output descs\n");
        bad = 1;
    }
    if (memcmp(got[0], got[1], sizeof(got[0])) != 0) {
        printf("MISMATCH: deconvolution scales %g %g %g / %g %g %g\n", got[1][0], got[1][1], got[1][2], got[0][0], got[0][1],
            got[0][2]);
        bad = 1;
    }
    return bad | same("int8 4x4 stride-2 deconvolution, ReLU, u8 out, through the six deconvolution_* calls", outs[1], outs[0]);
}

static int batched_matmul()
{
    TensorDesc ad = tensor4df(DT_F32, DF_NCHW, 2, 3, 16, 64), bd = tensor4df(DT_F32, DF_NCHW, 2, 3, 24, 64),
               cd = tensor4df(DT_F32, DF_NCHW, 2, 3, 16, 24);
    Tensor A = host_tensor(ad), B = host_tensor(bd);
    for (U32 i = 0; i < A.length(); ++i) {
        ((F32 *)hp(A))[i] = gauss();
    }
    for (U32 i = 0; i < B.length(); ++i) {
        ((F32 *)hp(B))[i] = gauss();
    }
    A.set_scale(-1);
    B.set_scale(-1);
    Tensor outs[2];
    for (int which = 0; which < 2; ++which) {
        Tensor Cm = host_tensor(cd), bias;
        Cm.set_scale(-1);
        U32 bytes = 0;
        if (which) {
            CHECK_STATUS(bolt_gfx950::matmul_infer_forward_tmp_bytes(A, false, B, true, Cm, &bytes, &g_host));
        } else {
            CHECK_STATUS(matmul_infer_forward_tmp_bytes(A, false, B, true, Cm, &bytes, &g_x86));
        }
        std::vector<Tensor> tmps(1, host_tensor(tensor1d(DT_U8, bytes + 64)));
        if (which) {
            CHECK_STATUS(bolt_gfx950::matmul(A, false, B, true, bias, tmps, Cm, &g_host));
        } else {
            CHECK_STATUS(matmul(A, false, B, true, bias, tmps, Cm, &g_x86));
        }
        outs[which] = Cm;
    }
    return same("batched int8 matmul of fp32 operands (quantised inside)", outs[1], outs[0]);
}

int main()
{
    if (bolt_gfx950_init() != SUCCESS) {
        printf("no GPU: %s\n", bolt_gfx950_last_error());
        return 2;
    }
    int bad = chain_quantize_fc_fc();
    bad |= conv_u8();
    bad |= deconv_u8();
    bad |= batched_matmul();
    printf(bad ? "glue FAILED\n" : "glue OK\n");
    return bad;
}
