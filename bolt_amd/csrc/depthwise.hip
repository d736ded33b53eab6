// int8 depthwise convolution, int32 result, window taken from the unpadded image.
//
// Bolt x86: compute/tensor/src/cpu/x86/int8/avx512/depthwise_convolution_direct.cpp:441-599 gathers, for every block
// of 16 channels and 16 output pixels, the fh * fw taps of each pixel into groups of four bytes per channel and feeds
// them to vpdpbusd against the filter laid out the same way. Here one thread owns one output pixel and four channels:
// per tap it reads one dword of the NCHWC16 input (its four channels) and, per group of four taps, one 16-byte piece
// of the filter blob (four channels x four taps); everything else is integer multiply-add in registers. The kernel is
// bound by the input re-reads that the caches serve and the 4-byte-per-element int32 store.
#include "device_common.h"
#include "kernels.h"

namespace bg {

__global__ __launch_bounds__(256) void depthwise_u8s8_i32_kernel(DepthwiseArgs a)
{
    const uint32_t CB = a.c / 16;
    const uint64_t total = (uint64_t)a.n * CB * a.oh * a.ow * 4;
    const uint64_t id = (uint64_t)blockIdx.x * 256 + threadIdx.x;
    if (id >= total) {
        return;
    }
    const uint32_t q = (uint32_t)(id & 3);
    uint64_t t = id >> 2;
    const uint32_t x = (uint32_t)(t % a.ow);
    t /= a.ow;
    const uint32_t y = (uint32_t)(t % a.oh);
    t /= a.oh;
    const uint32_t cb = (uint32_t)(t % CB), n = (uint32_t)(t / CB);
    const uint32_t c0 = cb * 16 + q * 4;
    const uint32_t taps = a.fh * a.fw, groups = (taps + 3) / 4;
    // filter blob behind offsetC: per 16-channel block, [tap group][channel 0..15][tap 0..3]
    const int8_t *w = a.filter + (size_t)cb * groups * 64 + q * 16;
    const uint8_t *in = a.in + (((size_t)n * CB + cb) * a.ih * a.iw) * 16 + q * 4;
    int acc[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // offsetC + round(bias * s), formed like quantize_bias_offsetC (avx512/quantize.cpp:236-269)
        const int32_t oc = a.offsetC[c0 + i];
        int32_t b = oc;
        if (a.bias) {
            const float p = a.bias[c0 + i] * a.scaleO;
            b = (int32_t)(round((double)p) + (double)oc);
        }
        acc[i] = b;
    }
    for (uint32_t g = 0; g < groups; ++g) {
        const v4i wv = *(const v4i *)(w + (size_t)g * 64);
        const int wd[4] = {wv.x, wv.y, wv.z, wv.w};  // channel i: four taps, one byte each
#pragma unroll
        for (uint32_t k = 0; k < 4; ++k) {
            const uint32_t tap = g * 4 + k;
            if (tap < taps) {
                const uint32_t kh = tap / a.fw, kw = tap % a.fw;
                const uint32_t px = *(const uint32_t *)(in + ((size_t)(y * a.sh + kh) * a.iw + (x * a.sw + kw)) * 16);
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int u = (int)((px >> (8 * i)) & 0xffu);
                    const int wt = (int)(int8_t)((uint32_t)wd[i] >> (8 * k));
                    acc[i] = (int)((uint32_t)acc[i] + (uint32_t)(u * wt));
                }
            }
        }
    }
    if (a.relu) {
#pragma unroll
        for (int i = 0; i < 4; ++i) {
            acc[i] = acc[i] < 0 ? 0 : acc[i];
        }
    }
    *(v4i *)(a.out + id * 4) = (v4i){acc[0], acc[1], acc[2], acc[3]};
}

hipError_t launch_depthwise_u8s8_i32(const DepthwiseArgs &a, hipStream_t st)
{
    const uint64_t threads = (uint64_t)a.n * (a.c / 16) * a.oh * a.ow * 4;
    if (threads == 0) {
        return hipSuccess;
    }
    if (a.c % 16 || (threads + 255) / 256 > 0x7fffffffull || a.fh == 0 || a.fw == 0 ||
        (uint64_t)(a.oh - 1) * a.sh + a.fh > a.ih || (uint64_t)(a.ow - 1) * a.sw + a.fw > a.iw) {
        return hipErrorInvalidValue;  // every window must lie inside the image
    }
    hipLaunchKernelGGL(depthwise_u8s8_i32_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace bg
