// int8 depthwise convolution, int32 result, window taken from the unpadded image.
//
// Bolt x86: compute/tensor/src/cpu/x86/int8/avx512/depthwise_convolution_direct.cpp:441-599 gathers, for every block
// of 16 channels and 16 output pixels, the fh * fw taps of each pixel into groups of four bytes per channel and feeds
// them to vpdpbusd against the filter laid out the same way. Here one thread owns one output pixel and four channels:
// per tap it reads one dword of the NCHWC16 input (its four channels) and, per group of four taps, one 16-byte piece
// of the filter blob (four channels x four taps -- the layout the reference made for vpdpbusd); the four dwords of a
// tap group are transposed to channel-major with eight v_perm_b32 and each channel's four products are one
// v_dot4_i32_i8. The kernel is bound by the input re-reads that the caches serve and the 4-byte-per-element store.
#include "device_common.h"
#include "kernels.h"

namespace bg {

constexpr uint32_t kPixPerWg = 512;

// F3: the filter is 3 x 3 (known when the kernel is compiled): the nine loads of a pixel are issued together and nothing
// walks the taps; otherwise the tap position is carried along at run time.
template <bool F3>
__global__ __launch_bounds__(256) void depthwise_u8s8_i32_kernel(DepthwiseArgs a)
{
    // blockIdx.x = plane * chunks + chunk: the plane (image, 16-channel block) comes from one scalar division per
    // workgroup, the pixel from one 32-bit division per thread
    const uint32_t CB = a.c / 16;
    // (a workgroup takes kPixPerWg pixels of its plane, 64 at a time: with one pixel per thread-quad the launch is
    // bound by the rate at which workgroups can be started, not by memory)
    const uint32_t opix = a.oh * a.ow, chunks = (opix + kPixPerWg - 1) / kPixPerWg;
    const uint32_t plane = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
    const uint32_t q = threadIdx.x & 3;
    const uint32_t cb = plane % CB, n = plane / CB;
    const uint32_t c0 = cb * 16 + q * 4;
    const uint32_t taps = a.fh * a.fw, groups = (taps + 3) / 4;
    // filter blob behind offsetC: per 16-channel block, [tap group][channel 0..15][tap 0..3]
    const int8_t *w = a.filter + (size_t)cb * groups * 64 + q * 16;
    const uint8_t *in = a.in + (((size_t)n * CB + cb) * a.ih * a.iw) * 16 + q * 4;
    int base[4];
#pragma unroll
    for (int i = 0; i < 4; ++i) {
        // offsetC + round(bias * s), formed like quantize_bias_offsetC (avx512/quantize.cpp:236-269); the inputs are
        // re-biased to s8 below, which takes the offsetC = -128 * sum(w) term out again: acc = round(bias * s) + sum (x - 128) * w
        const int32_t oc = a.offsetC[c0 + i];
        int32_t b = oc;
        if (a.bias) {
            const float p = a.bias[c0 + i] * a.scaleO;
            b = (int32_t)(round((double)p) + (double)oc);
        }
        base[i] = (int)((uint32_t)b - (uint32_t)oc);
    }
    // the channel's taps stay in registers across the workgroup's pixels when there are at most 12 of them (3 x 3 and
    // smaller); larger filters re-read their 16 bytes per tap group from the cache
    v4i wreg[3] = {{0, 0, 0, 0}, {0, 0, 0, 0}, {0, 0, 0, 0}};
    const bool held = groups <= 3;
    if (held) {
#pragma unroll
        for (uint32_t g = 0; g < 3; ++g) {
            if (g < groups) {
                wreg[g] = *(const v4i *)(w + (size_t)g * 64);
            }
        }
    }
    for (uint32_t sub = 0; sub < kPixPerWg / 64; ++sub) {
        const uint32_t pix = chunk * kPixPerWg + sub * 64 + (threadIdx.x >> 2);
        if (pix >= opix) {
            break;  // pixels ascend with sub: nothing further for this thread
        }
        const uint32_t y = pix / a.ow, x = pix % a.ow;
        const size_t id = ((size_t)plane * opix + pix) * 4 + q;  // the output is [plane][pixel][16]
        int acc[4] = {base[0], base[1], base[2], base[3]};
        const uint8_t *row = in + ((size_t)(y * a.sh) * a.iw + x * a.sw) * 16;  // tap (0, 0) of this pixel
        // 4 x 4 byte transpose (taps x channels -> channels x taps) with v_perm_b32, then one v_dot4_i32_i8 per channel
        auto tap_group = [&](const uint32_t (&px)[4], const v4i wv) {
            const uint32_t ab_lo = __builtin_amdgcn_perm(px[1], px[0], 0x05010400u), ab_hi = __builtin_amdgcn_perm(px[1], px[0], 0x07030602u);
            const uint32_t cd_lo = __builtin_amdgcn_perm(px[3], px[2], 0x05010400u), cd_hi = __builtin_amdgcn_perm(px[3], px[2], 0x07030602u);
            const uint32_t ch0 = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x05040100u), ch1 = __builtin_amdgcn_perm(cd_lo, ab_lo, 0x07060302u);
            const uint32_t ch2 = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x05040100u), ch3 = __builtin_amdgcn_perm(cd_hi, ab_hi, 0x07060302u);
            acc[0] = __builtin_amdgcn_sdot4((int)ch0, wv.x, acc[0], false);
            acc[1] = __builtin_amdgcn_sdot4((int)ch1, wv.y, acc[1], false);
            acc[2] = __builtin_amdgcn_sdot4((int)ch2, wv.z, acc[2], false);
            acc[3] = __builtin_amdgcn_sdot4((int)ch3, wv.w, acc[3], false);
        };
        if constexpr (F3) {
            // the nine taps at once; the three that pad the last group repeat tap 8 (their weights are zero)
            uint32_t p9[9];
#pragma unroll
            for (int t = 0; t < 9; ++t) {
                p9[t] = *(const uint32_t *)(row + ((size_t)(t / 3) * a.iw + (t % 3)) * 16) ^ 0x80808080u;
            }
            const uint32_t g0[4] = {p9[0], p9[1], p9[2], p9[3]}, g1[4] = {p9[4], p9[5], p9[6], p9[7]}, g2[4] = {p9[8], p9[8], p9[8], p9[8]};
            tap_group(g0, wreg[0]);
            tap_group(g1, wreg[1]);
            tap_group(g2, wreg[2]);
        } else {
            // tap position carried along (kh, kw wrap at fw): no division inside the loop; everything here is wave-uniform
            uint32_t kh = 0, kw = 0, left = taps;
            for (uint32_t g = 0; g < groups; ++g) {
                // channel i: its four taps of this group, one byte each
                const v4i wv = held ? (g == 0 ? wreg[0] : (g == 1 ? wreg[1] : wreg[2])) : *(const v4i *)(w + (size_t)g * 64);
                // the same four taps of the input: one dword (4 channels) per tap; taps past the end repeat the last one
                // (their weights are zero)
                uint32_t px[4];
#pragma unroll
                for (uint32_t k = 0; k < 4; ++k) {
                    px[k] = *(const uint32_t *)(row + ((size_t)kh * a.iw + kw) * 16) ^ 0x80808080u;
                    if (left > 1) {
                        --left;
                        ++kw;
                        if (kw == a.fw) {
                            kw = 0;
                            ++kh;
                        }
                    }
                }
                tap_group(px, wv);
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
}

hipError_t launch_depthwise_u8s8_i32(const DepthwiseArgs &a, hipStream_t st)
{
    const uint64_t planes = (uint64_t)a.n * (a.c / 16), chunks = ((uint64_t)a.oh * a.ow + kPixPerWg - 1) / kPixPerWg;
    if (planes == 0 || chunks == 0) {
        return hipSuccess;
    }
    if (a.c % 16 || planes * chunks > 0x7fffffffull || (uint64_t)a.oh * a.ow > 0x3fffffffull || a.fh == 0 || a.fw == 0 ||
        (uint64_t)(a.oh - 1) * a.sh + a.fh > a.ih || (uint64_t)(a.ow - 1) * a.sw + a.fw > a.iw) {
        return hipErrorInvalidValue;  // every window must lie inside the image
    }
    if (a.fh == 3 && a.fw == 3) {
        hipLaunchKernelGGL(depthwise_u8s8_i32_kernel<true>, dim3((uint32_t)(planes * chunks)), dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL(depthwise_u8s8_i32_kernel<false>, dim3((uint32_t)(planes * chunks)), dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

}  // namespace bg
