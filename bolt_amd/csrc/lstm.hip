// int8 LSTM cell around the batched GEMV (compute/tensor/src/cpu/x86/int8/lstm.cpp:20-179):
//   lstm_xh_quant_kernel   per batch row: [x | h] gathered, its own dynamic (or the caller's static) scale,
//                          fp32 -> u8 with the quantiser's arithmetic (lstm.cpp:89-109)
//   lstm_gates_kernel      bias add, gates, cell / hidden state update with zoneout (lstm.cpp:113-176)
//   lstm_project_kernel    with num_projection > 0: hidden state = fp32 projection of the gates' values (lstm.cpp:170-178)
// The matrix-vector products in between are one launch of gemv_s8u8_kernel over all rows.
#include "kernels.h"

namespace bg {

__global__ __launch_bounds__(256) void lstm_xh_quant_kernel(const LstmArgs a)
{
    __shared__ float red[4];
    const uint32_t m = blockIdx.x;
    const float *x = a.x + (size_t)m * a.x_stride;
    const float *h = a.state + (size_t)m * (a.column + a.hdim) + a.column;
    const uint32_t K = a.xdim + a.hdim;
    float mx = 0.0f;
    for (uint32_t k = threadIdx.x; k < K; k += 256) {
        const float v = k < a.xdim ? x[k] : h[k - a.xdim];
        mx = fmaxf(mx, fabsf(v));
    }
    for (int off = 32; off > 0; off >>= 1) {
        mx = fmaxf(mx, __shfl_xor(mx, off));
    }
    if ((threadIdx.x & 63) == 0) {
        red[threadIdx.x >> 6] = mx;
    }
    __syncthreads();
    mx = fmaxf(fmaxf(red[0], red[1]), fmaxf(red[2], red[3]));
    // quantize with mode 1 (avx512/quantize.cpp:129-133): the caller's scale if it is positive, else 127 / max
    float s = a.scale_in;
    if (s <= 0) {
        const float dyn = (mx == 0.0f) ? 1.0f : 127.0f / mx;
        s = (s > dyn) ? s : dyn;
    }
    uint8_t *q = a.quant + (size_t)m * K;
    for (uint32_t k = threadIdx.x; k < K; k += 256) {
        const float v = k < a.xdim ? x[k] : h[k - a.xdim];
        q[k] = (uint8_t)q_u8(v, s);
    }
    if (threadIdx.x == 0) {
        a.dscale[m] = s;
    }
}

__device__ __forceinline__ float sigmoid_f(float v)
{
    return 1.0f / (1.0f + expf(-v));
}

__global__ __launch_bounds__(256) void lstm_gates_kernel(const LstmArgs a)
{
    const uint32_t h = blockIdx.x * 256u + threadIdx.x;
    const uint32_t m = blockIdx.y;
    if (h >= a.column) {
        return;
    }
    const float *g = a.inter + (size_t)m * 4 * a.column;
    const float *b = a.bias + (size_t)m * a.bias_stride;
    float p[4];
    if (a.acc_i32) {
        // the matrix-vector epilogue's arithmetic: cvt(acc) * (1 / (row scale * weight scale))
        const float f = 1.0f / (a.dscale[m] * a.scale_w);
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            p[k] = (float)((const int32_t *)g)[h + k * a.column] * f;
        }
    } else {
#pragma unroll
        for (int k = 0; k < 4; ++k) {
            p[k] = g[h + k * a.column];
        }
    }
    const float gi = p[0] + b[h];
    const float gg = p[1] + b[h + a.column];
    const float gf = p[2] + b[h + 2 * a.column];
    const float go = p[3] + b[h + 3 * a.column];
    float *stC = a.state + (size_t)m * (a.column + a.hdim);
    float *stH = stC + a.column;
    const float c0 = stC[h];
    const float I = sigmoid_f(gi), F = sigmoid_f(gf + a.forget_bias), O = sigmoid_f(go), G = tanhf(gg);
    const float c1 = c0 * F + I * G;
    const float hid = O * tanhf(c1);
    if (a.zoneout_cell != 0) {
        stC[h] = c1 * (1 - a.zoneout_cell) + c0 * a.zoneout_cell;
    } else {
        stC[h] = c1;
    }
    if (a.proj) {
        a.act[(size_t)m * a.column + h] = hid;  // the projection kernel takes it from here (lstm.cpp:128)
        return;
    }
    a.out[(size_t)m * a.out_stride + h] = hid;
    if (a.zoneout_output != 0) {
        stH[h] = hid * (1 - a.zoneout_output) + stH[h] * a.zoneout_output;
    } else {
        stH[h] = hid;
    }
}

// mvm_nkn32_with_bias(hDim / 32, num_projection, filter[1], actOutH, projOut, nullptr) (lstm.cpp:170-173;
// cpu/x86/fp32/mvm_nkn32.h:19-140): every output element is one chain of fused multiply-adds over k ascending from an
// accumulator of 0 -- one thread per element here, in that order, so the sums round as the reference's do. Then the
// hidden state follows the projected value (zoneout on the output, :175-178).
__global__ __launch_bounds__(256) void lstm_project_kernel(const LstmArgs a)
{
    const uint32_t h = blockIdx.x * 256u + threadIdx.x;
    const uint32_t m = blockIdx.y;
    if (h >= a.hdim) {
        return;
    }
    const float *w = a.proj + (size_t)(h / 32) * a.column * 32 + (h % 32);
    const float *v = a.act + (size_t)m * a.column;
    float acc = 0.0f;
    for (uint32_t k = 0; k < a.column; ++k) {
        acc = __builtin_fmaf(v[k], w[(size_t)k * 32], acc);
    }
    a.out[(size_t)m * a.out_stride + h] = acc;
    float *stH = a.state + (size_t)m * (a.column + a.hdim) + a.column;
    if (a.zoneout_output != 0) {
        stH[h] = acc * (1 - a.zoneout_output) + stH[h] * a.zoneout_output;
    } else {
        stH[h] = acc;
    }
}

hipError_t launch_lstm_xh_quant(const LstmArgs &a, hipStream_t st)
{
    hipLaunchKernelGGL(lstm_xh_quant_kernel, dim3(a.batch), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_lstm_gates(const LstmArgs &a, hipStream_t st)
{
    hipLaunchKernelGGL(lstm_gates_kernel, dim3((a.column + 255) / 256, a.batch), dim3(256), 0, st, a);
    return hipGetLastError();
}

hipError_t launch_lstm_project(const LstmArgs &a, hipStream_t st)
{
    hipLaunchKernelGGL(lstm_project_kernel, dim3((a.hdim + 255) / 256, a.batch), dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace bg
