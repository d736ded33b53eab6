// Quantised pooling and concatenation: byte work bounded by HBM bandwidth.
//
//   pool_u8_c16_kernel   u8 max / mean pooling on NCHWC16 planes
//                        (compute/tensor/src/cpu/x86/int8/avx512/pooling_int8.cpp:316-429)
//   concat_i8_kernel     one input of a quantised concatenation, rescaled to the common output scale
//                        while it is copied into place (compute/tensor/src/cpu/concat.cpp:40-66,164-189
//                        with the arithmetic of compute/tensor/src/cpu/requantize.cpp:20-50)
//
// A lane owns 16 bytes (one pixel of a 16-channel plane, or 16 consecutive bytes of a row) and moves
// them with one 16-byte load per tap and one 16-byte store.
#include <algorithm>
#include "kernels.h"

namespace bg {

typedef unsigned short u16x2 __attribute__((ext_vector_type(2)));

__device__ __forceinline__ uint32_t pk_max_u16(uint32_t a, uint32_t b)
{
    u16x2 r = __builtin_elementwise_max(__builtin_bit_cast(u16x2, a), __builtin_bit_cast(u16x2, b));
    return __builtin_bit_cast(uint32_t, r);
}

// The sixteen channels of a pixel as packed 16-bit lanes: lo[d] holds bytes 0 and 2 of dword d, hi[d]
// bytes 1 and 3. 16-bit sums hold 257 taps of 255; WIDE keeps 32-bit sums for larger windows.
// KS > 0: the window is at most KS x KS taps (KS = 2, 3): all of them are requested before any is used, taps
// outside the clipped window re-read the first one and are masked out. KS = 0: any window, one tap at a time.
template <bool MEAN, bool WIDE, int KS>
__global__ __launch_bounds__(256) void pool_u8_c16_kernel(const PoolArgs a)
{
    const uint32_t gid = blockIdx.x * 256u + threadIdx.x;
    if (gid >= a.total) {
        return;
    }
    const uint32_t ow = gid % a.OW;
    const uint32_t t = gid / a.OW;
    const uint32_t oh = t % a.OH;
    const uint32_t plane = t / a.OH;

    int hs = (int)(oh * a.sh) - (int)a.pt, ws = (int)(ow * a.sw) - (int)a.pl;
    const int he = min(hs + (int)a.kh, (int)a.IH), we = min(ws + (int)a.kw, (int)a.IW);
    hs = max(hs, 0);
    ws = max(ws, 0);
    const uint32_t kh = (uint32_t)(he - hs), kw = (uint32_t)(we - ws);
    const uint4 *src = (const uint4 *)a.in + ((size_t)plane * a.IH + hs) * a.IW + ws;

    uint32_t lo[4], hi[4];
    uint32_t wide[WIDE ? 16 : 1];
#pragma unroll
    for (int d = 0; d < 4; ++d) {
        lo[d] = hi[d] = 0;   // also the identity of an unsigned maximum
    }
    if (WIDE) {
#pragma unroll
        for (int c = 0; c < 16; ++c) {
            wide[c] = 0;
        }
    }
    uint32_t taps = 0;
    if (KS > 0) {
        uint4 v[KS > 0 ? KS * KS : 1];
#pragma unroll
        for (int y = 0; y < KS; ++y) {
#pragma unroll
            for (int x = 0; x < KS; ++x) {
                const bool ok = (uint32_t)y < kh && (uint32_t)x < kw;
                v[y * KS + x] = src[ok ? (size_t)y * a.IW + x : 0];
            }
        }
#pragma unroll
        for (int y = 0; y < KS; ++y) {
#pragma unroll
            for (int x = 0; x < KS; ++x) {
                const uint32_t keep = ((uint32_t)y < kh && (uint32_t)x < kw) ? 0xffffffffu : 0u;
                const uint32_t w4[4] = {v[y * KS + x].x & keep, v[y * KS + x].y & keep, v[y * KS + x].z & keep,
                    v[y * KS + x].w & keep};
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    const uint32_t l = w4[d] & 0x00ff00ffu, h = (w4[d] >> 8) & 0x00ff00ffu;
                    if (MEAN) {
                        lo[d] += l;
                        hi[d] += h;
                    } else {
                        lo[d] = pk_max_u16(lo[d], l);
                        hi[d] = pk_max_u16(hi[d], h);
                    }
                }
            }
        }
    } else {
    for (uint32_t y = 0; y < kh; ++y) {
        const uint4 *row = src + (size_t)y * a.IW;
        for (uint32_t x = 0; x < kw; ++x) {
            const uint4 v = row[x];
            const uint32_t w4[4] = {v.x, v.y, v.z, v.w};
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                const uint32_t l = w4[d] & 0x00ff00ffu, h = (w4[d] >> 8) & 0x00ff00ffu;
                if (MEAN) {
                    lo[d] += l;   // no carry between the halves while fewer than 258 taps are summed
                    hi[d] += h;
                } else {
                    lo[d] = pk_max_u16(lo[d], l);
                    hi[d] = pk_max_u16(hi[d], h);
                }
            }
            if (MEAN && WIDE && ++taps == 256) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    wide[4 * d + 0] += lo[d] & 0xffffu;
                    wide[4 * d + 1] += hi[d] & 0xffffu;
                    wide[4 * d + 2] += lo[d] >> 16;
                    wide[4 * d + 3] += hi[d] >> 16;
                    lo[d] = hi[d] = 0;
                }
                taps = 0;
            }
        }
    }
    }

    uint32_t o4[4];
    if (MEAN) {
        // pooling_int8.cpp:206-229 -- sum of (u8 - 128), times 65536 / taps, LOGICAL shift by 16, + 128,
        // unsigned saturation to a byte (a negative sum therefore saturates to 255, as vpsrld / vpmovusdb do)
        const uint32_t pool = a.count_include_pad ? a.pool_full : 65536u / (kh * kw);
        const int32_t bias = -128 * (int32_t)(kh * kw);
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            uint32_t s[4] = {lo[d] & 0xffffu, hi[d] & 0xffffu, lo[d] >> 16, hi[d] >> 16};
            uint32_t o = 0;
#pragma unroll
            for (int b = 0; b < 4; ++b) {
                if (WIDE) {
                    s[b] += wide[4 * d + b];
                }
                const uint32_t prod = (uint32_t)((int32_t)s[b] + bias) * pool;
                const uint32_t r = min((prod >> 16) + 128u, 255u);
                o |= r << (8 * b);
            }
            o4[d] = o;
        }
    } else {
#pragma unroll
        for (int d = 0; d < 4; ++d) {
            o4[d] = lo[d] | (hi[d] << 8);
        }
    }
    ((uint4 *)a.out)[gid] = make_uint4(o4[0], o4[1], o4[2], o4[3]);
}

hipError_t launch_pool_u8_c16(const PoolArgs &a, hipStream_t st)
{
    if (a.total == 0) {
        return hipSuccess;
    }
    const dim3 grid((a.total + 255) / 256), block(256);
    const bool wide = a.kh * a.kw > 256;
    const int ks = (a.kh <= 2 && a.kw <= 2) ? 2 : (a.kh <= 3 && a.kw <= 3) ? 3 : 0;
#define BG_POOL(M, W, K) hipLaunchKernelGGL((pool_u8_c16_kernel<M, W, K>), grid, block, 0, st, a)
    if (!a.mean) {
        if (ks == 2) {
            BG_POOL(false, false, 2);
        } else if (ks == 3) {
            BG_POOL(false, false, 3);
        } else {
            BG_POOL(false, false, 0);
        }
    } else if (wide) {
        BG_POOL(true, true, 0);
    } else if (ks == 2) {
        BG_POOL(true, false, 2);
    } else if (ks == 3) {
        BG_POOL(true, false, 3);
    } else {
        BG_POOL(true, false, 0);
    }
#undef BG_POOL
    return hipGetLastError();
}

// ---- concatenation --------------------------------------------------------------------------------
// s8 -> s8 with factor r, the arithmetic of array_scale on DT_I8 (r * v + 0, conversion toward zero)
__device__ __forceinline__ uint32_t rescale4(uint32_t w, float r)
{
    uint32_t o = 0;
#pragma unroll
    for (int b = 0; b < 4; ++b) {
        const float v = r * (float)(int8_t)(w >> (8 * b)) + 0.0f;
        o |= ((uint32_t)(int)v & 0xffu) << (8 * b);
    }
    return o;
}

// rows x len bytes, source rows contiguous, destination rows `ostride` apart. VEC: everything is a multiple
// of 16 bytes and a lane moves 16; otherwise a lane moves one byte.
template <bool VEC, bool SCALE>
__global__ __launch_bounds__(256) void concat_i8_kernel(const uint8_t *__restrict__ in, uint8_t *__restrict__ out,
    uint32_t rows, uint32_t len, size_t ostride, float r)
{
    const uint32_t per_row = VEC ? len / 16 : len;
    const size_t total = (size_t)rows * per_row;
    const size_t step = (size_t)gridDim.x * 256u;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < total; i += step) {
        const uint32_t row = (uint32_t)(i / per_row), col = (uint32_t)(i % per_row);
        if (VEC) {
            v4i v = __builtin_nontemporal_load((const v4i *)in + i);
            if (SCALE) {
#pragma unroll
                for (int d = 0; d < 4; ++d) {
                    v[d] = (int)rescale4((uint32_t)v[d], r);
                }
            }
            __builtin_nontemporal_store(v, (v4i *)(out + (size_t)row * ostride) + col);
        } else {
            uint8_t b = in[i];
            if (SCALE) {
                const float v = r * (float)(int8_t)b + 0.0f;
                b = (uint8_t)(int)v;
            }
            out[(size_t)row * ostride + col] = b;
        }
    }
}

hipError_t launch_concat_i8(const void *in, void *out, uint32_t rows, uint32_t len, size_t ostride, int rescale,
    float r, hipStream_t st)
{
    if (rows == 0 || len == 0) {
        return hipSuccess;
    }
    const bool vec = len % 16 == 0 && ostride % 16 == 0 && ((uintptr_t)in | (uintptr_t)out) % 16 == 0;
    const size_t total = (size_t)rows * (vec ? len / 16 : len);
    const uint32_t blocks = (uint32_t)std::min<size_t>((total + 255) / 256, 256 * 64);
    const dim3 grid(blocks), block(256);
    const uint8_t *src = (const uint8_t *)in;
    uint8_t *dst = (uint8_t *)out;
    if (vec && rescale) {
        hipLaunchKernelGGL((concat_i8_kernel<true, true>), grid, block, 0, st, src, dst, rows, len, ostride, r);
    } else if (vec) {
        hipLaunchKernelGGL((concat_i8_kernel<true, false>), grid, block, 0, st, src, dst, rows, len, ostride, r);
    } else if (rescale) {
        hipLaunchKernelGGL((concat_i8_kernel<false, true>), grid, block, 0, st, src, dst, rows, len, ostride, r);
    } else {
        hipLaunchKernelGGL((concat_i8_kernel<false, false>), grid, block, 0, st, src, dst, rows, len, ostride, r);
    }
    return hipGetLastError();
}

// Up to eight inputs in ONE launch: blockIdx.y selects the input. Every length, offset, the stride and every
// pointer are multiples of 16 bytes (the launcher checks), so each lane moves 16 bytes.
__global__ __launch_bounds__(256) void concat_i8_multi_kernel(const ConcatMulti a)
{
    const uint32_t j = blockIdx.y;
    const uint32_t per_row = a.len[j] / 16;
    const size_t total = (size_t)a.rows * per_row;
    const size_t step = (size_t)gridDim.x * 256u;
    const v4i *in = (const v4i *)a.in[j];
    uint8_t *out = a.out + a.off[j];
    const float r = a.r[j];
    const bool scale = a.rescale[j] != 0;
    for (size_t i = (size_t)blockIdx.x * 256u + threadIdx.x; i < total; i += step) {
        const uint32_t row = (uint32_t)(i / per_row), col = (uint32_t)(i % per_row);
        v4i v = __builtin_nontemporal_load(in + i);
        if (scale) {
#pragma unroll
            for (int d = 0; d < 4; ++d) {
                v[d] = (int)rescale4((uint32_t)v[d], r);
            }
        }
        __builtin_nontemporal_store(v, (v4i *)(out + (size_t)row * a.ostride) + col);
    }
}

bool concat_multi_fits(const ConcatMulti &a)
{
    if (a.num == 0 || a.num > 8 || a.rows == 0 || (a.ostride & 15) || ((uintptr_t)a.out & 15)) {
        return false;
    }
    for (uint32_t j = 0; j < a.num; ++j) {
        if (a.len[j] == 0 || (a.len[j] & 15) || (a.off[j] & 15) || ((uintptr_t)a.in[j] & 15)) {
            return false;
        }
    }
    return true;
}

hipError_t launch_concat_i8_multi(const ConcatMulti &a, hipStream_t st)
{
    uint32_t longest = 0;
    for (uint32_t j = 0; j < a.num; ++j) {
        longest = std::max(longest, a.len[j]);
    }
    const size_t total = (size_t)a.rows * (longest / 16);
    const uint32_t blocks = (uint32_t)std::min<size_t>((total + 255) / 256, 256 * 64 / a.num + 1);
    hipLaunchKernelGGL(concat_i8_multi_kernel, dim3(blocks, a.num), dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace bg
