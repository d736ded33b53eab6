// Weight storage of the post-training quantisation tool and the load-time expansion of stored weights, as device
// kernels: all of it is element-wise, bound by HBM, 16 bytes per lane per access.
//
//   model_tools/src/model_data_type_converter.cpp:22-103  fp32 -> s8 / packed 4-bit / 1-bit, per-tensor scale
//   common/model_spec/src/model_deserialize.cpp:162-222   s8 / 4-bit -> fp32 / s8 / u8
//
// The scale of the s8 and 4-bit forms is max(127.0 / max|w|, caller's scale) with the quotient taken in double and
// stored as float (:71, :89); max|w| comes from the two-pass scratch slots (absmax_f32_kernel).
#include "device_common.h"
#include "kernels.h"

namespace bg {

static inline uint32_t blocks_for(uint64_t threads)
{
    const uint64_t b = (threads + 255) / 256;
    return (uint32_t)(b < 1 ? 1 : (b > 16384 ? 16384 : b));
}

__device__ __forceinline__ float ws_scale(const uint32_t *ws, double full, float floor_)
{
    const float m = __uint_as_float((uint32_t)ws_read_max(ws));
    const double dyn = full / (double)m;
    return (float)(dyn > (double)floor_ ? dyn : (double)floor_);
}

// q = rne(w * scale): roundNearestEven (:48-58) is round-half-away with ties pulled back to even
__global__ __launch_bounds__(256) void ws_int8_kernel(const float *__restrict__ w, uint32_t n, int8_t *__restrict__ q,
    const uint32_t *__restrict__ ws, float floor_, float *__restrict__ ds_out)
{
    const float s = ws_scale(ws, 127.0, floor_);
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    if (tid == 0) {
        *ds_out = s;
    }
    const uint32_t n4 = (((uintptr_t)w & 15) || ((uintptr_t)q & 3)) ? 0 : n / 4;
    const v4f *w4 = (const v4f *)w;
    uint32_t *q4 = (uint32_t *)q;
    for (uint32_t i = tid; i < n4; i += stride) {
        const v4f v = w4[i];
        q4[i] = ((uint32_t)rne_i32(v.x * s) & 0xffu) | (((uint32_t)rne_i32(v.y * s) & 0xffu) << 8) |
            (((uint32_t)rne_i32(v.z * s) & 0xffu) << 16) | (((uint32_t)rne_i32(v.w * s) & 0xffu) << 24);
    }
    for (uint32_t i = n4 * 4 + tid; i < n; i += stride) {
        q[i] = (int8_t)rne_i32(w[i] * s);
    }
}

// byte i = (nibble(2i + 1) << 4) | nibble(2i), nibble = rne((float)(w * 7.0 / max|w|)) + 7 with the product and the
// quotient in double (:91-97)
__global__ __launch_bounds__(256) void ws_int4_kernel(const float *__restrict__ w, uint32_t pairs, int8_t *__restrict__ q,
    const uint32_t *__restrict__ ws, float floor_, float *__restrict__ ds_out)
{
    const float s = ws_scale(ws, 7.0, floor_);
    const double m = (double)__uint_as_float((uint32_t)ws_read_max(ws));
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    if (tid == 0) {
        *ds_out = s;
    }
    for (uint32_t i = tid; i < pairs; i += stride) {
        const float a = w[2 * i], b = w[2 * i + 1];
        const int t0 = rne_i32((float)((double)a * 7.0 / m)) + 7, t1 = rne_i32((float)((double)b * 7.0 / m)) + 7;
        q[i] = (int8_t)((t1 << 4) | t0);
    }
}

// one output byte per thread: bit 7 - j set when w[8 i + j] > 0; also the index of the first positive weight
__global__ __launch_bounds__(256) void ws_bnn_kernel(const float *__restrict__ w, uint32_t bytes, uint8_t *__restrict__ bits,
    uint32_t *__restrict__ first_pos)
{
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    uint32_t first = 0xffffffffu;
    for (uint32_t i = tid; i < bytes; i += stride) {
        uint32_t b = 0;
#pragma unroll
        for (uint32_t j = 0; j < 8; ++j) {
            if (w[8 * i + j] > 0.0f) {
                b |= 1u << (7 - j);
            }
        }
        bits[i] = (uint8_t)b;
        if (b && first == 0xffffffffu) {
            first = 8 * i + (uint32_t)__builtin_clz(b << 24);
        }
    }
    if (first != 0xffffffffu) {
        atomicMin(first_pos, first);
    }
}

// scale = first positive weight, else the last weight, else 1 (:38-45)
__global__ void ws_bnn_scale_kernel(const float *__restrict__ w, uint32_t n, const uint32_t *__restrict__ first_pos,
    float *__restrict__ ds_out)
{
    const uint32_t f = *first_pos;
    *ds_out = n == 0 ? 1.0f : (f < n ? w[f] : w[n - 1]);
}

template <int SRC4, int DST>  // DST 0: fp32 = (1 / scale) * v, 1: s8 = v, 2: u8 = v + 128
__global__ __launch_bounds__(256) void ws_expand_kernel(const int8_t *__restrict__ q, uint32_t n, float scale,
    void *__restrict__ d)
{
    const float factor = 1 / scale;
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    for (uint32_t i = tid; i < n; i += stride) {
        int v;
        if (SRC4) {
            v = (((int)q[i / 2] >> ((i % 2) * 4)) & 0xF) - 7;
        } else {
            v = (int)q[i];
        }
        if (DST == 0) {
            ((float *)d)[i] = factor * (float)v;
        } else if (DST == 1) {
            ((int8_t *)d)[i] = (int8_t)v;
        } else {
            ((uint8_t *)d)[i] = (uint8_t)(v + 128);
        }
    }
}

hipError_t launch_ws_int8(const float *w, uint32_t n, int8_t *q, uint32_t *ws, float floor_, float *ds_out, hipStream_t st)
{
    hipError_t e = launch_absmax_f32(w, n, ws, st);
    if (e != hipSuccess) {
        return e;
    }
    hipLaunchKernelGGL(ws_int8_kernel, dim3(blocks_for(n / 4 + 1)), dim3(256), 0, st, w, n, q, ws, floor_, ds_out);
    return hipGetLastError();
}

hipError_t launch_ws_int4(const float *w, uint32_t n, int8_t *q, uint32_t *ws, float floor_, float *ds_out, hipStream_t st)
{
    hipError_t e = launch_absmax_f32(w, n, ws, st);
    if (e != hipSuccess) {
        return e;
    }
    hipLaunchKernelGGL(ws_int4_kernel, dim3(blocks_for(n / 2)), dim3(256), 0, st, w, n / 2, q, ws, floor_, ds_out);
    return hipGetLastError();
}

hipError_t launch_ws_bnn(const float *w, uint32_t n, uint8_t *bits, uint32_t *ws, float *ds_out, hipStream_t st)
{
    hipError_t e = launch_fill_u32(ws, 1, 0xffffffffu, st);
    if (e != hipSuccess) {
        return e;
    }
    if (n >= 8) {
        hipLaunchKernelGGL(ws_bnn_kernel, dim3(blocks_for(n / 8)), dim3(256), 0, st, w, n / 8, bits, ws);
    }
    hipLaunchKernelGGL(ws_bnn_scale_kernel, dim3(1), dim3(1), 0, st, w, n, ws, ds_out);
    return hipGetLastError();
}

hipError_t launch_ws_expand(const int8_t *q, uint32_t n, int src4, int dst, float scale, void *d, hipStream_t st)
{
    if (n == 0) {
        return hipSuccess;
    }
    const dim3 grid(blocks_for(n)), block(256);
#define BG_EXPAND(S, D) hipLaunchKernelGGL((ws_expand_kernel<S, D>), grid, block, 0, st, q, n, scale, d)
    if (src4) {
        if (dst == 0) {
            BG_EXPAND(1, 0);
        } else if (dst == 1) {
            BG_EXPAND(1, 1);
        } else {
            BG_EXPAND(1, 2);
        }
    } else {
        if (dst != 0) {
            return hipErrorInvalidValue;
        }
        BG_EXPAND(0, 0);
    }
#undef BG_EXPAND
    return hipGetLastError();
}

}  // namespace bg
