// int8 convolution as implicit GEMM on the matrix cores (no im2col buffer is ever materialised).
//
//   acc[n, oc, oy, ox] = offsetC[oc] + round(bias[oc] * sI * sF) + sum_{c, kh, kw} in_u8 * w_s8,
//   border reads 128          (Bolt x86: compute/tensor/src/cpu/x86/int8/avx512/convolution_direct.cpp:2584-2809)
// = round(bias * s) + sum over taps inside the image of (in_u8 - 128) * w_s8.
//
// Launches:
//   1. conv_pad_kernel      u8 NCHWC8 / NCHWC16 activations -> s8 (x - 128), zero-padded border and
//                           channel tail, in planes of 16 channels: [n][ICp/16][Hp][Wp][16]. After this
//                           the 16 K-bytes a lane feeds to one MFMA are 16 consecutive channels of one
//                           tap -- one contiguous 16-byte load, no bounds checks, no re-bias in the loop --
//                           and the 16 lanes that hold consecutive output pixels of a fragment read
//                           consecutive 16-byte pieces (whole cache lines for unit stride).
//   2. the pipelined GEMM kernel of gemm.hip in convolution mode (rows = output pixels, K ordered
//      (kh, kw, c); each lane steps its (kh, kw, 16-channel chunk) position in registers).
//      Epilogue: folded bias, integer ReLU + running max|acc| (int32 out), dequantise + eltwise +
//      fp32 ReLU (fp32 out), or the tensor-wide dynamic requantisation to u8 from a maximum found by
//      a first, store-free pass; written in the reference's NCHWC16 / NCHWC8 output order.
#include "device_common.h"
#include "kernels.h"
#include "layout.h"

namespace bg {

// One workgroup per (image, 16-channel plane, chunk of 1024 padded pixels), one thread per pixel: a thread
// reads the pixel's 16 (or 8) channels from the NCHWC8 / NCHWC16 input -- consecutive threads read
// consecutive pixels, 8 or 16 contiguous bytes each -- re-biases them to s8 and writes 16 contiguous
// bytes. Border pixels and the channel tail are zero.
__global__ __launch_bounds__(256) void conv_pad_kernel(const uint8_t *__restrict__ in, uint32_t N, uint32_t C, uint32_t H,
    uint32_t W, uint32_t cx, uint32_t pt, uint32_t pl, uint32_t Hp, uint32_t Wp, uint32_t ICp, int8_t *__restrict__ out,
    uint32_t *__restrict__ clear_ws)
{
    // optional: zero the scratch slots that the convolution after this kernel folds max|acc| into (saves a launch)
    if (clear_ws && blockIdx.x == 0 && blockIdx.y == 0 && threadIdx.x < kWsSlots) {
        clear_ws[threadIdx.x * kWsStride] = 0;
    }
    const uint32_t planes = ICp / 16;
    const uint32_t c16 = blockIdx.x % planes, n = blockIdx.x / planes;
    const uint32_t npix = Hp * Wp;
    uint32_t end = (blockIdx.y + 1) * 1024;
    end = end < npix ? end : npix;
    // NCHWCx element (n, c, h, w): (((n * C/x + c/x) * H + h) * W + w) * x + c % x. C % 8 == 0, so the
    // 8 channels starting at a multiple of 8 are contiguous for x = 8 and x = 16; a trailing block of
    // an NCHWC16 tensor with C % 16 == 8 is 8 wide (transform_functions_int8.h:208-222).
    size_t src[2];
    uint32_t bw[2];
    bool have[2];
#pragma unroll
    for (int half = 0; half < 2; ++half) {
        const uint32_t c0 = c16 * 16 + half * 8;
        have[half] = c0 < C;
        const uint32_t blk = c0 / cx;
        uint32_t w_ = (have[half] ? C - blk * cx : cx);
        bw[half] = w_ < cx ? w_ : cx;
        src[half] = (size_t)n * C * H * W + (size_t)blk * cx * H * W + c0 % cx;
    }
    int8_t *dst = out + (size_t)blockIdx.x * npix * 16;
    for (uint32_t pix = blockIdx.y * 1024 + threadIdx.x; pix < end; pix += 256) {
        const uint32_t hp = pix / Wp, wp = pix % Wp;
        v2i lo = {0, 0}, hi = {0, 0};
        if (hp >= pt && hp < pt + H && wp >= pl && wp < pl + W) {
            const size_t p = (size_t)(hp - pt) * W + (wp - pl);
            if (have[0]) {
                lo = *(const v2i *)(in + src[0] + p * bw[0]);
                lo ^= (v2i){(int)0x80808080, (int)0x80808080};
            }
            if (have[1]) {
                hi = *(const v2i *)(in + src[1] + p * bw[1]);
                hi ^= (v2i){(int)0x80808080, (int)0x80808080};
            }
        }
        *(v4i *)(dst + (size_t)pix * 16) = (v4i){lo.x, lo.y, hi.x, hi.y};
    }
}

hipError_t launch_conv_pad(const uint8_t *in, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t cx, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, int8_t *out, hipStream_t st, uint32_t *clear_ws)
{
    const uint32_t Hp = H + pt + pb, Wp = W + pl + pr, ICp = align_up(C, 16);
    const uint64_t np = (uint64_t)N * (ICp / 16), npix = (uint64_t)Hp * Wp;
    if (np == 0 || npix == 0) {
        return hipSuccess;
    }
    if (np > 0x7fffffffull || npix > 0x3fffffffull || (npix + 1023) / 1024 > 65535) {
        return hipErrorInvalidValue;
    }
    hipLaunchKernelGGL(conv_pad_kernel, dim3((uint32_t)np, (uint32_t)((npix + 1023) / 1024)), dim3(256), 0, st, in, N, C, H, W,
        cx, pt, pl, Hp, Wp, ICp, out, clear_ws);
    return hipGetLastError();
}


// Filter s8 NCHW [oc][ic][fh][fw] -> MFMA-fragment layout over K = (kh, kw, c) with c padded to ICp
// and K padded to a multiple of 64, N padded to 16. One thread per 8 packed bytes.
__global__ __launch_bounds__(256) void conv_pack_filter_kernel(const int8_t *__restrict__ src, uint32_t OC, uint32_t IC,
    uint32_t fhw, uint32_t ICp, uint32_t Kp, uint32_t N16, int8_t *__restrict__ dst)
{
    const uint32_t k8 = Kp / 8;
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)N16 * k8) {
        return;
    }
    const uint32_t n = (uint32_t)(id / k8);
    const uint32_t k0 = (uint32_t)(id % k8) * 8;
    uint32_t lo = 0, hi = 0;
    const uint32_t tap = k0 / ICp, c0 = k0 % ICp;
    if (n < OC && tap < fhw) {
        for (uint32_t b = 0; b < 8 && c0 + b < IC; ++b) {
            const uint32_t v = (uint8_t)src[((size_t)n * IC + c0 + b) * fhw + tap];
            if (b < 4) {
                lo |= v << (8 * b);
            } else {
                hi |= v << (8 * (b - 4));
            }
        }
    }
    *(v2i *)(dst + mmm_packed_offset(n, k0, Kp)) = (v2i){(int)lo, (int)hi};
}

// offsetC[oc] = -128 * sum over ALL taps and channels (convolution_transform.cpp:38-44): one wave per oc
__global__ __launch_bounds__(256) void conv_offsetC_kernel(const int8_t *__restrict__ src, uint32_t OC, uint32_t len,
    int32_t *__restrict__ out)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t n = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (n >= OC) {
        return;
    }
    int s = 0;
    for (uint32_t i = lane; i < len; i += 64) {
        s += (int)src[(size_t)n * len + i];
    }
    s = wave_reduce_add(s);
    if (lane == 0) {
        out[n] = s * (-128);
    }
}

hipError_t launch_conv_pack_filter(const int8_t *src, uint32_t OC, uint32_t IC, uint32_t fh, uint32_t fw, int32_t *offsetC,
    int8_t *dst, hipStream_t st)
{
    const uint32_t ICp = align_up(IC, 16), Kp = align_up(fh * fw * ICp, 64), N16 = align_up(OC, 16);
    const uint64_t threads = (uint64_t)N16 * (Kp / 8);
    hipLaunchKernelGGL(conv_pack_filter_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, st, src, OC, IC,
        fh * fw, ICp, Kp, N16, dst);
    hipLaunchKernelGGL(conv_offsetC_kernel, dim3((OC + 3) / 4), dim3(256), 0, st, src, OC, IC * fh * fw, offsetC);
    return hipGetLastError();
}

}  // namespace bg
