// 1-bit (XNOR / DoReFa) convolution. Two routes: on the vector ALU with bit-packed +-1 / {0,1}
// operands, XOR (or AND) and population count; and on the int8 matrix cores with the operands
// expanded to one byte per value (see "matrix-core route" below).
// (Bolt: compute/tensor/src/cpu/arm/bnn/convolution_xnor_A76.cpp:17-724, convolution_dorefa_A76.cpp,
//  naive form compute/tensor/src/cpu/general/convolution.cpp:141-178.)
//   XNOR   (DT_BIN11): bit 1 = +1, bit 0 = -1, padding = bit 0;  S = fh*fw*ic - 2 * popcount(x ^ w)
//   DoReFa (DT_BIN01): bit 1 = 1,  bit 0 = 0,  padding = 0;      S = popcount(x & w)
//   out = fma(S, scale[oc], bias[oc])
//
// Data layout on the GPU: activations are re-laid pixel-major, [n][Hp][Wp][ic/32] dwords (32
// channels per dword, zero-bit border), so one tap of one pixel is ic/32 consecutive dwords.
// Weights are re-laid [oc/32][tap][ic/32][32] dwords: for a fixed (tap, channel dword) the 32
// output channels a wave works on are 32 consecutive dwords, which are wave-uniform and therefore
// fetched with scalar loads. A wave owns 64 output pixels (one per lane) x 32 output channels:
// per activation dword it issues 32 x (v_xor_b32 with an SGPR operand + v_bcnt_u32_b32 with the
// accumulator as addend) = 2 VALU instructions per 32 binary multiply-accumulates per lane.
#include "device_common.h"
#include "kernels.h"
#include "layout.h"

namespace bg {

// fp32 NCHWC8 (or already bit-packed [n][ic/8][h][w] bytes, MSB = first channel of the 8) ->
// pixel-major padded dwords. One thread per output dword.
template <int FROM_F32>
__global__ __launch_bounds__(256) void bnn_pack_input_kernel(const void *__restrict__ in, uint32_t N, uint32_t C, uint32_t H,
    uint32_t W, uint32_t pt, uint32_t pl, uint32_t Hp, uint32_t Wp, float thr, uint32_t *__restrict__ out)
{
    const uint32_t cw = C / 32;
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)N * Hp * Wp * cw) {
        return;
    }
    const uint32_t j = (uint32_t)(id % cw);
    uint64_t p = id / cw;
    const uint32_t wp = (uint32_t)(p % Wp);
    p /= Wp;
    const uint32_t hp = (uint32_t)(p % Hp);
    const uint32_t n = (uint32_t)(p / Hp);
    uint32_t word = 0;
    if (hp >= pt && hp < pt + H && wp >= pl && wp < pl + W) {
        const uint32_t h = hp - pt, w = wp - pl;
#pragma unroll
        for (uint32_t b = 0; b < 4; ++b) {
            const uint32_t c8 = j * 4 + b;
            const size_t pix = (((size_t)n * (C / 8) + c8) * H + h) * W + w;
            uint32_t byte = 0;
            if (FROM_F32) {
                const float *f = (const float *)in + pix * 8;
#pragma unroll
                for (int k = 0; k < 8; ++k) {
                    byte |= (f[k] >= thr) ? (1u << (7 - k)) : 0u;  // common/uni/include/data_type.h:213-221
                }
            } else {
                byte = ((const uint8_t *)in)[pix];
            }
            word |= byte << (8 * b);
        }
    }
    out[id] = word;
}

hipError_t launch_bnn_pack_input(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, float thr, uint32_t *out, hipStream_t st)
{
    const uint32_t Hp = H + pt + pb, Wp = W + pl + pr;
    const uint64_t total = (uint64_t)N * Hp * Wp * (C / 32);
    if (total == 0) {
        return hipSuccess;
    }
    const dim3 grid((uint32_t)((total + 255) / 256));
    if (from_f32) {
        hipLaunchKernelGGL((bnn_pack_input_kernel<1>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, out);
    } else {
        hipLaunchKernelGGL((bnn_pack_input_kernel<0>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, out);
    }
    return hipGetLastError();
}

// Filter bits -> [oc/32][tap][ic/32][32] dwords. src_fmt 0: DF_NCHW bit string, bit position
// ((o * ic + c) * fhw + tap), MSB-first in each byte; 1: DF_NCHWN16C8 bytes
// ((o/16 * ic/8 + c/8) * fhw + tap) * 16 + o%16 (convolution_transform_bnn.h:58-79). One thread per dword.
__global__ __launch_bounds__(256) void bnn_pack_filter_kernel(const uint8_t *__restrict__ src, int src_fmt, uint32_t OC,
    uint32_t IC, uint32_t fhw, uint32_t *__restrict__ dst)
{
    const uint32_t cw = IC / 32;
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)OC * fhw * cw) {
        return;
    }
    const uint32_t o32 = (uint32_t)(id % 32);
    uint64_t r = id / 32;
    const uint32_t j = (uint32_t)(r % cw);
    r /= cw;
    const uint32_t tap = (uint32_t)(r % fhw);
    const uint32_t o = (uint32_t)(r / fhw) * 32 + o32;
    uint32_t word = 0;
    for (uint32_t b = 0; b < 4; ++b) {
        const uint32_t c8 = j * 4 + b;
        uint32_t byte = 0;
        if (src_fmt == 1) {
            byte = src[(((size_t)(o / 16) * (IC / 8) + c8) * fhw + tap) * 16 + o % 16];
        } else {
            for (uint32_t k = 0; k < 8; ++k) {
                const uint64_t bit = ((uint64_t)o * IC + c8 * 8 + k) * fhw + tap;
                const uint32_t v = (src[bit >> 3] >> (7 - (bit & 7))) & 1u;
                byte |= v << (7 - k);
            }
        }
        word |= byte << (8 * b);
    }
    dst[id] = word;
}

hipError_t launch_bnn_pack_filter(const uint8_t *src, int src_fmt, uint32_t OC, uint32_t IC, uint32_t fhw, uint32_t *dst,
    hipStream_t st)
{
    const uint64_t total = (uint64_t)OC * fhw * (IC / 32);
    if (total == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(bnn_pack_filter_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st, src, src_fmt, OC, IC,
        fhw, dst);
    return hipGetLastError();
}

// ---- matrix-core route ----------------------------------------------------------------------------
// +-1 (XNOR) and {0, 1} (DoReFa) are int8 values too, and the int8 matrix cores are five times faster
// than the vector ALU's xor + popcount, so the convolution can run as the int8 implicit GEMM of
// conv.hip / gemm.hip on operands expanded to one byte per value: S = sum a * w directly, the
// padding border is -1 (XNOR: a zero bit) or 0 (DoReFa). The expanded image (n * Hp * Wp * ic
// bytes) and the expanded filter live in tmp; the transformed-filter blob stays bit-packed.

// fp32 NCHWC8 (or bit-packed [n][ic/8][h][w] bytes, MSB = first channel of the 8) -> s8 planes of 16
// channels [n][ic/16][Hp][Wp][16]. One workgroup per (image, plane, chunk of 1024 padded pixels), one
// thread per pixel.
template <int FROM_F32>
__global__ __launch_bounds__(256) void bnn_expand_input_kernel(const void *__restrict__ in, uint32_t N, uint32_t C, uint32_t H,
    uint32_t W, uint32_t pt, uint32_t pl, uint32_t Hp, uint32_t Wp, float thr, int zero, int8_t *__restrict__ out)
{
    const uint32_t planes = C / 16;
    const uint32_t c16 = blockIdx.x % planes, n = blockIdx.x / planes;
    const uint32_t npix = Hp * Wp;
    uint32_t end = (blockIdx.y + 1) * 1024;
    end = end < npix ? end : npix;
    const uint32_t lo = (uint32_t)zero & 0xffu;  // the byte a cleared bit expands to: 0xff (-1) or 0
    const uint32_t border = lo * 0x01010101u;
    // a set bit becomes 0x01; a cleared bit 0xff or 0x00: byte = bit ? 1 : lo, four channels at a time
    int8_t *dst = out + (size_t)blockIdx.x * npix * 16;
    for (uint32_t pix = blockIdx.y * 1024 + threadIdx.x; pix < end; pix += 256) {
        const uint32_t hp = pix / Wp, wp = pix % Wp;
        uint32_t o[4] = {border, border, border, border};
        if (hp >= pt && hp < pt + H && wp >= pl && wp < pl + W) {
            const size_t hw = (size_t)(hp - pt) * W + (wp - pl);
#pragma unroll
            for (int half = 0; half < 2; ++half) {
                const uint32_t c8 = c16 * 2 + half;
                const size_t p = ((size_t)n * (C / 8) + c8) * H * W + hw;
                uint32_t bits = 0;  // bit 7 - k = channel k of the 8
                if (FROM_F32) {
                    const v4f f0 = *(const v4f *)((const float *)in + p * 8), f1 = *(const v4f *)((const float *)in + p * 8 + 4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        bits |= (f0[k] >= thr) ? (1u << (7 - k)) : 0u;  // common/uni/include/data_type.h:213-221
                        bits |= (f1[k] >= thr) ? (1u << (3 - k)) : 0u;
                    }
                } else {
                    bits = ((const uint8_t *)in)[p];
                }
#pragma unroll
                for (int q = 0; q < 2; ++q) {
                    // nibble (channels 4q .. 4q+3, first channel in bit 3) -> one byte per channel: copy the
                    // nibble into every byte, keep bit 3 - k in byte k, turn "non-zero" into 1
                    const uint32_t nib = (bits >> (4 - 4 * q)) & 0xfu;
                    uint32_t t = (nib * 0x01010101u) & 0x01020408u;
                    t = ((t + 0x7f7f7f7fu) >> 7) & 0x01010101u;
                    o[half * 2 + q] = t | ((t ^ 0x01010101u) * lo);  // set bit -> 1, cleared bit -> lo (0xff or 0)
                }
            }
        }
        __builtin_nontemporal_store((v4i){(int)o[0], (int)o[1], (int)o[2], (int)o[3]}, (v4i *)(dst + (size_t)pix * 16));
    }
}

hipError_t launch_bnn_expand_input(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W, uint32_t pt,
    uint32_t pb, uint32_t pl, uint32_t pr, float thr, int xnor, int8_t *out, hipStream_t st)
{
    const uint32_t Hp = H + pt + pb, Wp = W + pl + pr;
    const uint64_t np = (uint64_t)N * (C / 16), npix = (uint64_t)Hp * Wp;
    if (np == 0 || npix == 0) {
        return hipSuccess;
    }
    if (np > 0x7fffffffull || npix > 0x3fffffffull || (npix + 1023) / 1024 > 65535) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((uint32_t)np, (uint32_t)((npix + 1023) / 1024));
    const int zero = xnor ? -1 : 0;
    if (from_f32) {
        hipLaunchKernelGGL((bnn_expand_input_kernel<1>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, zero, out);
    } else {
        hipLaunchKernelGGL((bnn_expand_input_kernel<0>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, zero, out);
    }
    return hipGetLastError();
}

// Transformed filter ([oc/32][tap][ic/32][32] dwords of bits) -> the int8 GEMM's packed right-hand side over
// K = (tap, c), K padded to a multiple of 64 with zeros, N = oc. One thread per 16 output bytes
// (16 consecutive channels of one tap for one output channel).
__global__ __launch_bounds__(256) void bnn_expand_filter_kernel(const uint32_t *__restrict__ src, uint32_t OC, uint32_t IC,
    uint32_t fhw, uint32_t Kp, int zero, int8_t *__restrict__ dst)
{
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t kb_n = Kp / 16;
    if (id >= (uint64_t)OC * kb_n) {
        return;
    }
    const uint32_t kb = (uint32_t)(id % kb_n), n = (uint32_t)(id / kb_n);
    const uint32_t k0 = kb * 16;
    uint32_t o[4] = {0, 0, 0, 0};
    if (k0 < fhw * IC) {
        const uint32_t tap = k0 / IC, c0 = k0 % IC, cw = IC / 32;
        const uint32_t word = src[(((size_t)(n / 32) * fhw + tap) * cw + c0 / 32) * 32 + n % 32];
        const uint32_t lo = (uint32_t)zero & 0xffu;
#pragma unroll
        for (int q = 0; q < 16; ++q) {
            const uint32_t c = (c0 % 32) + q;                       // channel within the dword
            const uint32_t bit = (word >> (8 * (c / 8) + 7 - (c % 8))) & 1u;
            o[q / 4] |= (bit ? 1u : lo) << (8 * (q & 3));
        }
    }
    *(v4i *)(dst + mmm_packed_offset(n, k0, Kp)) = (v4i){(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
}

hipError_t launch_bnn_expand_filter(const uint32_t *src, uint32_t OC, uint32_t IC, uint32_t fhw, int xnor, int8_t *dst,
    hipStream_t st)
{
    const uint32_t Kp = align_up(fhw * IC, 64);
    const uint64_t total = (uint64_t)OC * (Kp / 16);
    if (total == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(bnn_expand_filter_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st, src, OC, IC, fhw, Kp,
        xnor ? -1 : 0, dst);
    return hipGetLastError();
}

// ---- fp4 variant of the matrix-core route -----------------------------------------------------------
// +1, -1 and 0 are E2M1 values (0x2, 0xA, 0x0): two channels per byte, 32 channels per 16-byte chunk, and
// v_mfma_scale_f32_16x16x128_f8f6f4 multiplies twice as many of them per instruction as the int8 form.
// Channel c of a 32-channel group sits in byte c / 2, low nibble first; image and filter use the same order,
// which is all a dot product needs.

// 8 bits (bit 7 - k = channel k) -> 8 nibbles of a dword (nibble k = channel k): set bit -> 0x2, cleared -> lo4
__device__ __forceinline__ uint32_t bnn_bits_to_fp4(uint32_t bits, uint32_t lo4)
{
    uint32_t out = 0;
#pragma unroll
    for (int q = 0; q < 2; ++q) {
        const uint32_t nib = (bits >> (4 - 4 * q)) & 0xfu;       // channels 4q .. 4q+3, first channel in bit 3
        uint32_t t = (nib * 0x1111u) & 0x1248u;                  // nibble j keeps bit 3 - j
        t = ((t + 0x7777u) >> 3) & 0x1111u;                      // non-zero -> 1
        const uint32_t v = (t << 1) | ((t ^ 0x1111u) * lo4);     // 1 -> 0x2, 0 -> lo4
        out |= v << (16 * q);
    }
    return out;
}

// fp32 NCHWC8 or bit-packed input -> fp4 planes of 32 channels [n][ic/32][Hp][Wp][16 bytes]
template <int FROM_F32>
__global__ __launch_bounds__(256) void bnn_expand_input_fp4_kernel(const void *__restrict__ in, uint32_t N, uint32_t C,
    uint32_t H, uint32_t W, uint32_t pt, uint32_t pl, uint32_t Hp, uint32_t Wp, float thr, uint32_t lo4,
    uint8_t *__restrict__ out)
{
    const uint32_t planes = C / 32;
    const uint32_t c32 = blockIdx.x % planes, n = blockIdx.x / planes;
    const uint32_t npix = Hp * Wp;
    uint32_t end = (blockIdx.y + 1) * 1024;
    end = end < npix ? end : npix;
    const uint32_t border = lo4 * 0x11111111u;
    uint8_t *dst = out + (size_t)blockIdx.x * npix * 16;
    for (uint32_t pix = blockIdx.y * 1024 + threadIdx.x; pix < end; pix += 256) {
        const uint32_t hp = pix / Wp, wp = pix % Wp;
        uint32_t o[4] = {border, border, border, border};
        if (hp >= pt && hp < pt + H && wp >= pl && wp < pl + W) {
            const size_t hw = (size_t)(hp - pt) * W + (wp - pl);
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                const uint32_t c8 = c32 * 4 + b;
                const size_t p = ((size_t)n * (C / 8) + c8) * H * W + hw;
                uint32_t bits = 0;  // bit 7 - k = channel k of the 8
                if (FROM_F32) {
                    const v4f f0 = *(const v4f *)((const float *)in + p * 8), f1 = *(const v4f *)((const float *)in + p * 8 + 4);
#pragma unroll
                    for (int k = 0; k < 4; ++k) {
                        bits |= (f0[k] >= thr) ? (1u << (7 - k)) : 0u;  // common/uni/include/data_type.h:213-221
                        bits |= (f1[k] >= thr) ? (1u << (3 - k)) : 0u;
                    }
                } else {
                    bits = ((const uint8_t *)in)[p];
                }
                o[b] = bnn_bits_to_fp4(bits, lo4);
            }
        }
        __builtin_nontemporal_store((v4i){(int)o[0], (int)o[1], (int)o[2], (int)o[3]}, (v4i *)(dst + (size_t)pix * 16));
    }
}

hipError_t launch_bnn_expand_input_fp4(const void *in, int from_f32, uint32_t N, uint32_t C, uint32_t H, uint32_t W,
    uint32_t pt, uint32_t pb, uint32_t pl, uint32_t pr, float thr, int xnor, uint8_t *out, hipStream_t st)
{
    const uint32_t Hp = H + pt + pb, Wp = W + pl + pr;
    const uint64_t np = (uint64_t)N * (C / 32), npix = (uint64_t)Hp * Wp;
    if (np == 0 || npix == 0) {
        return hipSuccess;
    }
    if (np > 0x7fffffffull || npix > 0x3fffffffull || (npix + 1023) / 1024 > 65535) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((uint32_t)np, (uint32_t)((npix + 1023) / 1024));
    const uint32_t lo4 = xnor ? 0xAu : 0x0u;
    if (from_f32) {
        hipLaunchKernelGGL((bnn_expand_input_fp4_kernel<1>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, lo4,
            out);
    } else {
        hipLaunchKernelGGL((bnn_expand_input_fp4_kernel<0>), grid, dim3(256), 0, st, in, N, C, H, W, pt, pl, Hp, Wp, thr, lo4,
            out);
    }
    return hipGetLastError();
}

// Transformed filter bits -> fp4 pairs in the GEMM's packed right-hand-side layout over K bytes = (tap, c / 2),
// padded to a multiple of 64 bytes with zeros. One thread per source dword (32 channels = 16 bytes).
__global__ __launch_bounds__(256) void bnn_expand_filter_fp4_kernel(const uint32_t *__restrict__ src, uint32_t OC, uint32_t IC,
    uint32_t fhw, uint32_t Kp, uint32_t lo4, uint8_t *__restrict__ dst)
{
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t kb_n = Kp / 16;
    if (id >= (uint64_t)OC * kb_n) {
        return;
    }
    const uint32_t kb = (uint32_t)(id % kb_n), n = (uint32_t)(id / kb_n);
    const uint32_t cw = IC / 32;
    uint32_t o[4] = {0, 0, 0, 0};
    if (kb < fhw * cw) {
        const uint32_t tap = kb / cw, j = kb % cw;
        const uint32_t word = src[(((size_t)(n / 32) * fhw + tap) * cw + j) * 32 + n % 32];
#pragma unroll
        for (int b = 0; b < 4; ++b) {
            o[b] = bnn_bits_to_fp4((word >> (8 * b)) & 0xffu, lo4);
        }
    }
    *(v4i *)(dst + mmm_packed_offset(n, kb * 16, Kp)) = (v4i){(int)o[0], (int)o[1], (int)o[2], (int)o[3]};
}

hipError_t launch_bnn_expand_filter_fp4(const uint32_t *src, uint32_t OC, uint32_t IC, uint32_t fhw, int xnor, uint8_t *dst,
    hipStream_t st)
{
    const uint32_t Kp = align_up(fhw * IC / 2, 64);
    const uint64_t total = (uint64_t)OC * (Kp / 16);
    if (total == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(bnn_expand_filter_fp4_kernel, dim3((uint32_t)((total + 255) / 256)), dim3(256), 0, st, src, OC, IC, fhw,
        Kp, xnor ? 0xAu : 0x0u, dst);
    return hipGetLastError();
}

// One wave: 64 output pixels (lane = pixel) x 32 output channels.
template <int XNOR>
__global__ __launch_bounds__(256) void bnn_conv_kernel(BnnArgs a)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    // the four waves of a workgroup share one block of 32 output channels (the same weight stream in
    // the scalar cache) and take 64 pixels each
    const uint32_t ob = blockIdx.y;
    const uint32_t cw = a.IC / 32;
    uint32_t pix = (blockIdx.x * 4 + wave) * 64 + lane;
    if ((blockIdx.x * 4 + wave) * 64 >= a.M) {
        return;
    }
    const bool live = pix < a.M;
    pix = live ? pix : a.M - 1;
    const uint32_t img = pix / a.OHW, r = pix % a.OHW;
    const uint32_t oy = r / a.OW, ox = r % a.OW;
    const uint32_t *xp = a.x + (size_t)((img * a.Hp + oy * a.sh) * a.Wp + ox * a.sw) * cw;
    const uint32_t *wp = a.w + (size_t)ob * a.fh * a.fw * cw * 32;

    int acc[32];
#pragma unroll
    for (int o = 0; o < 32; ++o) {
        acc[o] = 0;
    }
    if ((cw & 3) == 0) {
        // 128 channels (one 16-byte load) per step; the load of the next step is issued before the
        // 4 x 64 VALU instructions of this one, so its latency never stalls the wave. The step
        // counters are wave-uniform (scalar ALU).
        const uint32_t cw4 = cw >> 2, steps = a.fh * a.fw * cw4;
        uint32_t j4 = 0, kw = 0, kh = 0;
        v4i nxt = *(const v4i *)xp;
        // the 32 weights of the next 32-channel group are fetched (scalar loads) while the VALU works
        // through the current group: two SGPR sets in flight
        uint32_t wc[32], wn[32];
#pragma unroll
        for (int o = 0; o < 32; ++o) {
            wc[o] = wp[o];
        }
        for (uint32_t it = 0; it < steps; ++it) {
            const v4i cur = nxt;
            if (++j4 == cw4) {
                j4 = 0;
                if (++kw == a.fw) {
                    kw = 0;
                    ++kh;
                }
            }
            const bool more = it + 1 < steps;
            if (more) {
                nxt = *(const v4i *)(xp + (size_t)(kh * a.Wp + kw) * cw + j4 * 4);
            }
#pragma unroll
            for (int u = 0; u < 4; ++u) {
                const uint32_t xv = (uint32_t)cur[u];
                const uint32_t *wq = (u < 3 || more) ? wp + (u + 1) * 32 : wp;  // past the end: any valid address
#pragma unroll
                for (int o = 0; o < 32; ++o) {
                    wn[o] = wq[o];
                }
#pragma unroll
                for (int o = 0; o < 32; ++o) {
                    acc[o] += __builtin_popcount(XNOR ? (xv ^ wc[o]) : (xv & wc[o]));
                }
#pragma unroll
                for (int o = 0; o < 32; ++o) {
                    wc[o] = wn[o];
                }
            }
            wp += 128;
        }
    } else {
        for (uint32_t kh = 0; kh < a.fh; ++kh) {
            for (uint32_t kw = 0; kw < a.fw; ++kw) {
                const uint32_t *xt = xp + (size_t)(kh * a.Wp + kw) * cw;
                for (uint32_t j = 0; j < cw; ++j) {
                    const uint32_t xv = xt[j];
#pragma unroll
                    for (int o = 0; o < 32; ++o) {
                        const uint32_t wv = wp[o];  // wave-uniform address: scalar load
                        acc[o] += __builtin_popcount(XNOR ? (xv ^ wv) : (xv & wv));
                    }
                    wp += 32;
                }
            }
        }
    }
    if (!live) {
        return;
    }
    const int base = (int)(a.fh * a.fw * a.IC);
#pragma unroll
    for (int o8 = 0; o8 < 4; ++o8) {
        const uint32_t oc0 = ob * 32 + o8 * 8;
        const size_t idx = (((size_t)img * (a.OC / 8) + oc0 / 8) * a.OHW + r) * 8;  // NCHWC8
        int s[8];
#pragma unroll
        for (int k = 0; k < 8; ++k) {
            s[k] = XNOR ? base - 2 * acc[o8 * 8 + k] : acc[o8 * 8 + k];
        }
        if (a.sums) {
            *(v4i *)(a.sums + idx) = (v4i){s[0], s[1], s[2], s[3]};
            *(v4i *)(a.sums + idx + 4) = (v4i){s[4], s[5], s[6], s[7]};
        }
        if (a.out) {
            float f[8];
#pragma unroll
            for (int k = 0; k < 8; ++k) {
                f[k] = __builtin_fmaf((float)s[k], a.scale[oc0 + k], a.bias[oc0 + k]);  // vfmaq in the reference
            }
            *(v4f *)(a.out + idx) = (v4f){f[0], f[1], f[2], f[3]};
            *(v4f *)(a.out + idx + 4) = (v4f){f[4], f[5], f[6], f[7]};
        }
    }
}

hipError_t launch_bnn_conv(const BnnArgs &a, int xnor, hipStream_t st)
{
    if (a.M == 0 || a.OC == 0) {
        return hipSuccess;
    }
    const dim3 grid((a.M + 255) / 256, a.OC / 32);
    if (xnor) {
        hipLaunchKernelGGL((bnn_conv_kernel<1>), grid, dim3(256), 0, st, a);
    } else {
        hipLaunchKernelGGL((bnn_conv_kernel<0>), grid, dim3(256), 0, st, a);
    }
    return hipGetLastError();
}

}  // namespace bg
