// int8 deconvolution (transposed convolution) helpers.
//
// Bolt x86 (compute/tensor/src/cpu/deconvolution.cpp:252-365, compute/tensor/src/cpu/x86/deconvolution.cpp:130-257)
// computes it as one matrix product per input pixel,
//   col[n, kh, kw][jh, jw, o] = sum_c (in_u8[n, c, kh, kw] - 128) * w[c][o][jh][jw],
// followed by an overlap-add of every column onto the output pixel (kh * sh + jh - pad_top, kw * sw + jw - pad_left)
// it lands on. Here the product is the int8 convolution kernel run as a 1x1 convolution with fh * fw * oc output
// channels (the filter is packed once, at load time, in that order), and the overlap-add is a GATHER: one thread per
// output pixel and four channels walks the (at most ceil(fh / sh) * ceil(fw / sw)) columns that land on it, in
// ascending (kh, kw) order -- the order the reference's scatter loop reaches that pixel, which its fp32 form depends
// on -- and applies bias, activation and the change of type in the same pass. No atomics, every output written once.
#include "device_common.h"
#include "kernels.h"
#include "layout.h"

namespace bg {

// filter s8 [ic][oc][taps] -> the convolution's packed matrix with rows n' = tap * oc + o over K = ic (padded to
// ICp = ALIGN(ic, 16), Kp = ALIGN(ICp, 64)). One thread per 8 packed bytes.
__global__ __launch_bounds__(256) void deconv_pack_filter_kernel(const int8_t *__restrict__ src, uint32_t IC, uint32_t OC,
    uint32_t taps, uint32_t Kp, int8_t *__restrict__ dst)
{
    const uint32_t k8 = Kp / 8, rows = taps * OC;
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)rows * k8) {
        return;
    }
    const uint32_t n = (uint32_t)(id / k8), c0 = (uint32_t)(id % k8) * 8;
    const uint32_t tap = n / OC, o = n % OC;
    uint32_t lo = 0, hi = 0;
    for (uint32_t b = 0; b < 8 && c0 + b < IC; ++b) {
        const uint32_t v = (uint8_t)src[((size_t)(c0 + b) * OC + o) * taps + tap];
        if (b < 4) {
            lo |= v << (8 * b);
        } else {
            hi |= v << (8 * (b - 4));
        }
    }
    *(v2i *)(dst + mmm_packed_offset(n, c0, Kp)) = (v2i){(int)lo, (int)hi};
}

// offsetC[tap * oc + o] = -128 * sum_c w[c][o][tap] (x86/int8/deconvolution_transform.cpp:33-63)
__global__ __launch_bounds__(256) void deconv_offsetC_kernel(const int8_t *__restrict__ src, uint32_t IC, uint32_t OC,
    uint32_t taps, int32_t *__restrict__ out)
{
    const uint32_t n = blockIdx.x * blockDim.x + threadIdx.x;
    if (n >= taps * OC) {
        return;
    }
    const uint32_t tap = n / OC, o = n % OC;
    int s = 0;
    for (uint32_t c = 0; c < IC; ++c) {
        s += (int)src[((size_t)c * OC + o) * taps + tap];
    }
    out[n] = s * (-128);
}

hipError_t launch_deconv_pack_filter(const int8_t *src, uint32_t IC, uint32_t OC, uint32_t taps, int32_t *offsetC, int8_t *dst,
    hipStream_t st)
{
    const uint32_t Kp = align_up(align_up(IC, 16), 64), rows = taps * OC;
    const uint64_t threads = (uint64_t)rows * (Kp / 8);
    hipLaunchKernelGGL(deconv_pack_filter_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, st, src, IC, OC, taps,
        Kp, dst);
    hipLaunchKernelGGL(deconv_offsetC_kernel, dim3((rows + 255) / 256), dim3(256), 0, st, src, IC, OC, taps, offsetC);
    return hipGetLastError();
}

// u8 plain NCHW -> NCHWC8: one thread per (image, 8-channel block, pixel), reads 8 bytes HW apart (coalesced across the
// wave), writes 8 contiguous bytes
__global__ __launch_bounds__(256) void nchw_to_c8_u8_kernel(const uint8_t *__restrict__ in, uint32_t planes, uint32_t HW,
    uint8_t *__restrict__ out)
{
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)planes * HW) {
        return;
    }
    const uint32_t p = (uint32_t)(id / HW), pix = (uint32_t)(id % HW);
    const uint8_t *s = in + (size_t)p * 8 * HW + pix;
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (uint32_t b = 0; b < 4; ++b) {
        lo |= (uint32_t)s[(size_t)b * HW] << (8 * b);
        hi |= (uint32_t)s[(size_t)(b + 4) * HW] << (8 * b);
    }
    *(v2i *)(out + id * 8) = (v2i){(int)lo, (int)hi};
}

hipError_t launch_nchw_to_c8_u8(const uint8_t *in, uint32_t N, uint32_t C, uint32_t HW, uint8_t *out, hipStream_t st)
{
    const uint64_t threads = (uint64_t)N * (C / 8) * HW;
    if (threads == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(nchw_to_c8_u8_kernel, dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, st, in, N * (C / 8), HW,
        out);
    return hipGetLastError();
}

// out[i] = src[i % period] (fp32 bias repeated once per tap)
__global__ __launch_bounds__(256) void repeat_f32_kernel(const float *__restrict__ src, uint32_t period, uint32_t n,
    float *__restrict__ out)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        out[i] = src[i % period];
    }
}

hipError_t launch_repeat_f32(const float *src, uint32_t period, uint32_t n, float *out, hipStream_t st)
{
    hipLaunchKernelGGL(repeat_f32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, src, period, n, out);
    return hipGetLastError();
}

// One thread per output pixel and 4 channels (output NCHWC16: [n][oc/16][oh][ow][16]). The columns sit where the 1x1
// convolution wrote them: [n][taps * oc / 16][ih][iw][16], channel tap * oc + o.
template <int MODE>
__global__ __launch_bounds__(256) void deconv_gather_kernel(DeconvArgs a)
{
    __shared__ int red[4];
    // blockIdx.x = plane * chunks + chunk: the plane (image, 16-channel block) comes from one scalar division per
    // workgroup, the pixel from one 32-bit division per thread
    const uint32_t OB = a.oc / 16;
    const uint32_t opix = a.oh * a.ow, chunks = (opix + 63) / 64;
    const uint32_t plane = blockIdx.x / chunks, chunk = blockIdx.x % chunks;
    const uint32_t pix = chunk * 64 + (threadIdx.x >> 2);
    int m = 0;
    if (pix < opix) {
        const uint32_t q = threadIdx.x & 3;
        const uint32_t oh = pix / a.ow, ow = pix % a.ow;
        const uint32_t ob = plane % OB, n = plane / OB;
        const size_t id = ((size_t)plane * opix + pix) * 4 + q;  // the output is [plane][pixel][16]
        const uint32_t o0 = ob * 16 + q * 4;
        const uint32_t planes = a.fh * a.fw * OB;
        // kh with 0 <= oh + pt - kh * sh < fh, inside the image
        const uint32_t yh = oh + a.pt, yw = ow + a.pl;
        const uint32_t kh_lo = yh >= a.fh ? (yh - a.fh + a.sh) / a.sh : 0;
        uint32_t kh_hi = yh / a.sh;
        kh_hi = kh_hi < a.ih - 1 ? kh_hi : a.ih - 1;
        const uint32_t kw_lo = yw >= a.fw ? (yw - a.fw + a.sw) / a.sw : 0;
        uint32_t kw_hi = yw / a.sw;
        kw_hi = kw_hi < a.iw - 1 ? kw_hi : a.iw - 1;
        int ai[4] = {0, 0, 0, 0};
        float af[4] = {0, 0, 0, 0};
        uint32_t qb = 0x80808080u;  // MODE_U8 / MODE_F32_FROM_U8: the one column byte per channel
        if (MODE == DECONV_I32 || MODE == DECONV_F32_DEQ) {
            const v4f b = *(const v4f *)(a.bias + o0);
            // round(sI * sW * b) in double like the reference's C round() on the float product
            ai[0] = (int)round((double)(b.x * a.scaleO));
            ai[1] = (int)round((double)(b.y * a.scaleO));
            ai[2] = (int)round((double)(b.z * a.scaleO));
            ai[3] = (int)round((double)(b.w * a.scaleO));
        } else if (MODE == DECONV_F32_SUM) {
            const v4f b = *(const v4f *)(a.bias + o0);
            af[0] = b.x;
            af[1] = b.y;
            af[2] = b.z;
            af[3] = b.w;
        }
        for (uint32_t kh = kh_lo; kh <= kh_hi; ++kh) {
            const uint32_t jh = yh - kh * a.sh;
            for (uint32_t kw = kw_lo; kw <= kw_hi; ++kw) {
                const uint32_t jw = yw - kw * a.sw;
                const uint32_t plane = (jh * a.fw + jw) * OB + ob;
                const size_t at = ((((size_t)n * planes + plane) * a.ih + kh) * a.iw + kw) * 16 + q * 4;
                if (MODE == DECONV_U8 || MODE == DECONV_F32_FROM_U8) {
                    qb = *(const uint32_t *)((const uint8_t *)a.col + at);
                } else {
                    const v4i c = *(const v4i *)((const int32_t *)a.col + at);
                    if (MODE == DECONV_F32_SUM) {
                        af[0] = af[0] + (float)c.x * a.factor;
                        af[1] = af[1] + (float)c.y * a.factor;
                        af[2] = af[2] + (float)c.z * a.factor;
                        af[3] = af[3] + (float)c.w * a.factor;
                    } else {
                        ai[0] = (int)((uint32_t)ai[0] + (uint32_t)c.x);
                        ai[1] = (int)((uint32_t)ai[1] + (uint32_t)c.y);
                        ai[2] = (int)((uint32_t)ai[2] + (uint32_t)c.z);
                        ai[3] = (int)((uint32_t)ai[3] + (uint32_t)c.w);
                    }
                }
            }
        }
        const size_t oi = id * 4;  // the thread order is the output order
        if (MODE == DECONV_I32 || MODE == DECONV_F32_DEQ) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (a.relu && ai[i] < 0) {
                    ai[i] = 0;
                }
            }
            if (MODE == DECONV_I32) {
                *(v4i *)((int32_t *)a.out + oi) = (v4i){ai[0], ai[1], ai[2], ai[3]};
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const int v = ai[i] == (int)0x80000000 ? ai[i] : (ai[i] < 0 ? -ai[i] : ai[i]);
                    m = v > m ? v : m;
                }
            } else {
                *(v4f *)((float *)a.out + oi) =
                    (v4f){(float)ai[0] * a.factor, (float)ai[1] * a.factor, (float)ai[2] * a.factor, (float)ai[3] * a.factor};
            }
        } else if (MODE == DECONV_F32_SUM) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (a.relu && !(af[i] > 0.0f)) {
                    af[i] = 0.0f;
                }
            }
            *(v4f *)((float *)a.out + oi) = (v4f){af[0], af[1], af[2], af[3]};
        } else if (MODE == DECONV_U8) {
            if (a.relu) {  // max(q, 128) per byte (x86_functions_int8.h:32-61)
                uint32_t r = 0;
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const uint32_t b = (qb >> (8 * i)) & 0xffu;
                    r |= (b < 128u ? 128u : b) << (8 * i);
                }
                qb = r;
            }
            *(uint32_t *)((uint8_t *)a.out + oi) = qb;
        } else {  // DECONV_F32_FROM_U8: cvt(q - 128) * (1 / scale) (avx512/dequantize.cpp:62-101)
            float f[4];
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                f[i] = (float)((int)((qb >> (8 * i)) & 0xffu) - 128) * a.factor;
                if (a.relu && !(f[i] > 0.0f)) {
                    f[i] = 0.0f;
                }
            }
            *(v4f *)((float *)a.out + oi) = (v4f){f[0], f[1], f[2], f[3]};
        }
    }
    if (MODE == DECONV_I32 && a.absmax) {
        ws_block_fold_max(a.absmax, m, red);
    }
}

hipError_t launch_deconv_gather(const DeconvArgs &a, hipStream_t st)
{
    const uint64_t planes = (uint64_t)a.n * (a.oc / 16), chunks = ((uint64_t)a.oh * a.ow + 63) / 64;
    if (planes == 0 || chunks == 0) {
        return hipSuccess;
    }
    if (a.oc % 16 || a.ih == 0 || a.iw == 0 || a.sh == 0 || a.sw == 0 || planes * chunks > 0x7fffffffull ||
        (uint64_t)a.oh * a.ow > 0x3fffffffull) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((uint32_t)(planes * chunks)), block(256);
    switch (a.mode) {
        case DECONV_I32:
            hipLaunchKernelGGL((deconv_gather_kernel<DECONV_I32>), grid, block, 0, st, a);
            break;
        case DECONV_F32_DEQ:
            hipLaunchKernelGGL((deconv_gather_kernel<DECONV_F32_DEQ>), grid, block, 0, st, a);
            break;
        case DECONV_F32_SUM:
            hipLaunchKernelGGL((deconv_gather_kernel<DECONV_F32_SUM>), grid, block, 0, st, a);
            break;
        case DECONV_U8:
            hipLaunchKernelGGL((deconv_gather_kernel<DECONV_U8>), grid, block, 0, st, a);
            break;
        case DECONV_F32_FROM_U8:
            hipLaunchKernelGGL((deconv_gather_kernel<DECONV_F32_FROM_U8>), grid, block, 0, st, a);
            break;
        default:
            return hipErrorInvalidValue;
    }
    return hipGetLastError();
}

// in-place max(q, 128) over u8 (ReLU of a quantised tensor, x86_functions_int8.h:32-61)
__global__ __launch_bounds__(256) void relu_u8_kernel(uint8_t *__restrict__ q, uint32_t n)
{
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x, stride = gridDim.x * blockDim.x;
    const uint32_t n4 = ((uintptr_t)q & 3) ? 0 : n / 4;
    uint32_t *q4 = (uint32_t *)q;
    for (uint32_t i = tid; i < n4; i += stride) {
        const uint32_t v = q4[i];
        // bytes below 0x80 have the top bit clear: replace exactly those
        const uint32_t low = ~v & 0x80808080u;        // 0x80 in every byte that is < 128
        const uint32_t mask = (low >> 7) * 0xffu;     // 0xff in those bytes
        q4[i] = (v & ~mask) | low;
    }
    for (uint32_t i = n4 * 4 + tid; i < n; i += stride) {
        q[i] = q[i] < 128 ? 128 : q[i];
    }
}

hipError_t launch_relu_u8(uint8_t *q, uint32_t n, hipStream_t st)
{
    if (n == 0) {
        return hipSuccess;
    }
    uint32_t blocks = (n / 4 + 255) / 256;
    blocks = blocks < 1 ? 1 : (blocks > 4096 ? 4096 : blocks);
    hipLaunchKernelGGL(relu_u8_kernel, dim3(blocks), dim3(256), 0, st, q, n);
    return hipGetLastError();
}

}  // namespace bg
