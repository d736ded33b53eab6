// HBM-bound element-wise kernels of the quantized path: per-tensor symmetric quantize
// (fp32 -> u8 / s8), int32 -> u8 / s8 requantize, dequantize, bias fold, s8 rescale.
// Numerics follow Bolt's AVX-512 kernels step by step
// (compute/tensor/src/cpu/x86/int8/avx512/quantize.cpp, dequantize.cpp): every fp32 multiply and
// add rounds separately (the translation unit is built with -ffp-contract=off), conversions are
// round-to-nearest-even, narrowing saturates the way vpmovusdb / vpmovsdb do.
//
// Dynamic scales need the tensor-wide |max| before the map pass, so quantize is two launches:
// a grid-stride reduction that folds into one device word with atomicMax (non-negative fp32
// order like their bit patterns), then the map pass, in which every thread derives the scale
// from that word. 16 elements per thread: 4 x 128-bit loads, one 128-bit store.
#include "device_common.h"
#include "kernels.h"

namespace bg {

static inline uint32_t grid_for(uint32_t n, uint32_t per_thread, uint32_t block, uint32_t cap)
{
    uint64_t threads = ((uint64_t)n + per_thread - 1) / per_thread;
    uint64_t blocks = (threads + block - 1) / block;
    if (blocks < 1) {
        blocks = 1;
    }
    if (blocks > cap) {
        blocks = cap;
    }
    return (uint32_t)blocks;
}

__global__ void fill_u32_kernel(uint32_t *p, uint32_t n, uint32_t v)
{
    uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i < n) {
        p[i] = v;
    }
}

hipError_t launch_fill_u32(uint32_t *p, uint32_t n, uint32_t v, hipStream_t st)
{
    hipLaunchKernelGGL(fill_u32_kernel, dim3((n + 255) / 256), dim3(256), 0, st, p, n, v);
    return hipGetLastError();
}

__global__ void mul_scalars_kernel(float *out, const float *a, const float *b)
{
    out[0] = a[0] * b[0];
}

hipError_t launch_mul_scalars(float *out, const float *a, const float *b, hipStream_t st)
{
    hipLaunchKernelGGL(mul_scalars_kernel, dim3(1), dim3(1), 0, st, out, a, b);
    return hipGetLastError();
}

// ---- |max| reductions ---------------------------------------------------------------------------
// avx512/quantize.cpp:21-68: sign bit cleared, vmaxps (a NaN never replaces the running max).
template <int VEC>
__global__ __launch_bounds__(256) void absmax_f32_kernel(const float *__restrict__ x, uint32_t n, uint32_t *ws,
    const uint32_t *only_if)
{
    if (only_if && *only_if == 0) {
        return;
    }
    __shared__ int red[4];
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t stride = gridDim.x * blockDim.x;
    float m = 0.0f;
#define BG_AMAX(v)                 \
    {                              \
        float a_ = fabsf(v);       \
        m = (a_ > m) ? a_ : m;     \
    }
    if (VEC) {
        const uint32_t n4 = n / 4;
        const v4f *x4 = (const v4f *)x;
        uint32_t i = tid;
        for (; i + 3 * stride < n4; i += 4 * stride) {  // four independent 16-byte loads in flight
            v4f a = x4[i], b = x4[i + stride], c = x4[i + 2 * stride], d = x4[i + 3 * stride];
            BG_AMAX(a.x) BG_AMAX(a.y) BG_AMAX(a.z) BG_AMAX(a.w) BG_AMAX(b.x) BG_AMAX(b.y) BG_AMAX(b.z) BG_AMAX(b.w)
            BG_AMAX(c.x) BG_AMAX(c.y) BG_AMAX(c.z) BG_AMAX(c.w) BG_AMAX(d.x) BG_AMAX(d.y) BG_AMAX(d.z) BG_AMAX(d.w)
        }
        for (; i < n4; i += stride) {
            v4f v = x4[i];
            BG_AMAX(v.x) BG_AMAX(v.y) BG_AMAX(v.z) BG_AMAX(v.w)
        }
        for (uint32_t j = n4 * 4 + tid; j < n; j += stride) {
            BG_AMAX(x[j])
        }
    } else {
        for (uint32_t i = tid; i < n; i += stride) {
            BG_AMAX(x[i])
        }
    }
#undef BG_AMAX
    // non-negative floats: integer order == float order
    ws_block_fold_max(ws, (int)__float_as_uint(m), red);
}

hipError_t launch_absmax_f32(const float *x, uint32_t n, uint32_t *ws, hipStream_t st, bool ws_is_clear, const uint32_t *only_if)
{
    hipError_t e = ws_is_clear ? hipSuccess : launch_fill_u32(ws, kWsWords, 0, st);
    if (e != hipSuccess || n == 0) {
        return e;
    }
    // a conditional launch nearly always returns at once: a small grid keeps that cheap (the loops stride over the grid)
    const uint32_t blocks = grid_for(n, 16, 256, only_if ? 256 : 1024);
    if (((uintptr_t)x & 15) == 0) {
        hipLaunchKernelGGL((absmax_f32_kernel<1>), dim3(blocks), dim3(256), 0, st, x, n, ws, only_if);
    } else {
        hipLaunchKernelGGL((absmax_f32_kernel<0>), dim3(blocks), dim3(256), 0, st, x, n, ws, only_if);
    }
    return hipGetLastError();
}

// avx512/quantize.cpp:70-119: vpabsd + vpmaxsd, so |INT32_MIN| stays negative and never wins.
__global__ __launch_bounds__(256) void absmax_i32_kernel(const int32_t *__restrict__ x, uint32_t n, uint32_t *ws)
{
    __shared__ int red[4];
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t stride = gridDim.x * blockDim.x;
    int m = 0;
#define BG_AMAX(v)                                                       \
    {                                                                    \
        int v_ = (v);                                                    \
        int a_ = (v_ == (int)0x80000000) ? v_ : (v_ < 0 ? -v_ : v_);     \
        m = (a_ > m) ? a_ : m;                                           \
    }
    if (((uintptr_t)x & 15) == 0) {
        const uint32_t n4 = n / 4;
        const v4i *x4 = (const v4i *)x;
        uint32_t i = tid;
        for (; i + 3 * stride < n4; i += 4 * stride) {
            v4i a = x4[i], b = x4[i + stride], c = x4[i + 2 * stride], d = x4[i + 3 * stride];
            BG_AMAX(a.x) BG_AMAX(a.y) BG_AMAX(a.z) BG_AMAX(a.w) BG_AMAX(b.x) BG_AMAX(b.y) BG_AMAX(b.z) BG_AMAX(b.w)
            BG_AMAX(c.x) BG_AMAX(c.y) BG_AMAX(c.z) BG_AMAX(c.w) BG_AMAX(d.x) BG_AMAX(d.y) BG_AMAX(d.z) BG_AMAX(d.w)
        }
        for (; i < n4; i += stride) {
            v4i v = x4[i];
            BG_AMAX(v.x) BG_AMAX(v.y) BG_AMAX(v.z) BG_AMAX(v.w)
        }
        for (uint32_t j = n4 * 4 + tid; j < n; j += stride) {
            BG_AMAX(x[j])
        }
    } else {
        for (uint32_t i = tid; i < n; i += stride) {
            BG_AMAX(x[i])
        }
    }
#undef BG_AMAX
    ws_block_fold_max(ws, m, red);
}

hipError_t launch_absmax_i32(const int32_t *x, uint32_t n, uint32_t *ws, hipStream_t st)
{
    hipError_t e = launch_fill_u32(ws, kWsWords, 0, st);
    if (e != hipSuccess || n == 0) {
        return e;
    }
    hipLaunchKernelGGL(absmax_i32_kernel, dim3(grid_for(n, 16, 256, 1024)), dim3(256), 0, st, x, n, ws);
    return hipGetLastError();
}

// ---- fp32 -> u8 / s8 ----------------------------------------------------------------------------
__device__ __forceinline__ unsigned q_i8(float x, float s)
{
    // avx512/quantize.cpp:208-212: vmulps, vcvtps2dq, clamp [-127, 127]
    int v = rne_i32(x * s);
    v = v < -127 ? -127 : v;
    v = v > 127 ? 127 : v;
    return (unsigned)v & 0xffu;
}

template <int TO_U8>
__device__ __forceinline__ unsigned q4(v4f v, float s)
{
    if (TO_U8) {
        return q_u8(v.x, s) | (q_u8(v.y, s) << 8) | (q_u8(v.z, s) << 16) | (q_u8(v.w, s) << 24);
    }
    return q_i8(v.x, s) | (q_i8(v.y, s) << 8) | (q_i8(v.z, s) << 16) | (q_i8(v.w, s) << 24);
}

// avx512/quantize.cpp:129-133 / :189-193: dynamic when !mode or the caller's scale is <= 0;
// the result is max(caller's scale, 127 / max|x|), with 127 / 0 replaced by 1.
__device__ __forceinline__ float resolve_scale(float s_in, int mode, const uint32_t *ws)
{
    if (!mode || s_in <= 0) {
        float m = __uint_as_float((uint32_t)ws_read_max(ws));
        float dyn = (m == 0.0f) ? 1.0f : 127.0f / m;
        return (s_in > dyn) ? s_in : dyn;
    }
    return s_in;
}

// GELU: quantise gelu_tanh(x) instead of x (the max in ws is then that of the activated values)
template <int TO_U8, int VEC, int GELU = 0>
__global__ __launch_bounds__(256) void quantize_f32_kernel(const float *__restrict__ x, uint32_t n,
    uint8_t *__restrict__ q, const uint32_t *__restrict__ ws, float s_in, const float *ds_in, int mode,
    float *ds_out, const uint32_t *only_if)  // ds_in may alias ds_out: the resolved scale is a fixed point of resolve_scale
{
    if (only_if && *only_if == 0) {
        return;
    }
    const float s = resolve_scale(ds_in ? *ds_in : s_in, mode, ws);
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    if (tid == 0 && ds_out) {
        *ds_out = s;
    }
    const uint32_t stride = gridDim.x * blockDim.x;
    if (VEC) {
        // lane-contiguous 16-byte loads (a wave's request = 1 KB of whole lines), four in flight, 4-byte stores
        const uint32_t n4 = n / 4;
        const v4f *x4 = (const v4f *)x;
        int *q4w = (int *)q;
        uint32_t i = tid;
        for (; i + 3 * stride < n4; i += 4 * stride) {
            v4f a = x4[i], b = x4[i + stride], c = x4[i + 2 * stride], d = x4[i + 3 * stride];
            if (GELU) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a[e] = gelu_tanh(a[e]);
                    b[e] = gelu_tanh(b[e]);
                    c[e] = gelu_tanh(c[e]);
                    d[e] = gelu_tanh(d[e]);
                }
            }
            q4w[i] = (int)q4<TO_U8>(a, s);
            q4w[i + stride] = (int)q4<TO_U8>(b, s);
            q4w[i + 2 * stride] = (int)q4<TO_U8>(c, s);
            q4w[i + 3 * stride] = (int)q4<TO_U8>(d, s);
        }
        for (; i < n4; i += stride) {
            v4f a = x4[i];
            if (GELU) {
#pragma unroll
                for (int e = 0; e < 4; ++e) {
                    a[e] = gelu_tanh(a[e]);
                }
            }
            q4w[i] = (int)q4<TO_U8>(a, s);
        }
        for (i = n4 * 4 + tid; i < n; i += stride) {
            const float v = GELU ? gelu_tanh(x[i]) : x[i];
            q[i] = (uint8_t)(TO_U8 ? q_u8(v, s) : q_i8(v, s));
        }
    } else {
        for (uint32_t i = tid; i < n; i += stride) {
            q[i] = (uint8_t)(TO_U8 ? q_u8(x[i], s) : q_i8(x[i], s));
        }
    }
}

hipError_t launch_quantize_f32(const float *x, uint32_t n, void *q, int to_u8, const uint32_t *ws, float s_in,
    const float *ds_in, int mode, float *ds_out, hipStream_t st, int gelu, const uint32_t *only_if)
{
    const bool vec = (((uintptr_t)x | (uintptr_t)q) & 15) == 0;
    const uint32_t blocks = grid_for(n, vec ? 16 : 1, 256, only_if ? 256 : 8192);
    if (gelu) {
        if (!to_u8 || !vec) {
            return hipErrorInvalidValue;  // the fused form exists for aligned u8 output only
        }
        hipLaunchKernelGGL((quantize_f32_kernel<1, 1, 1>), dim3(blocks), dim3(256), 0, st, x, n, (uint8_t *)q, ws, s_in, ds_in,
            mode, ds_out, only_if);
        return hipGetLastError();
    }
#define BG_LAUNCH_Q(U, V)                                                                                        \
    hipLaunchKernelGGL((quantize_f32_kernel<U, V>), dim3(blocks), dim3(256), 0, st, x, n, (uint8_t *)q, ws, s_in, \
        ds_in, mode, ds_out, only_if)
    if (to_u8) {
        if (vec) {
            BG_LAUNCH_Q(1, 1);
        } else {
            BG_LAUNCH_Q(1, 0);
        }
    } else {
        if (vec) {
            BG_LAUNCH_Q(0, 1);
        } else {
            BG_LAUNCH_Q(0, 0);
        }
    }
#undef BG_LAUNCH_Q
    return hipGetLastError();
}

// ---- int32 -> u8 / s8 ---------------------------------------------------------------------------
// avx512/quantize.cpp:315-361 (s8: ssat8(rne(cvt(x) * r))) and :364-416
// (u8: usat8_u(rne(cvt(x) * r + 128.0f)), fp32 add before rounding).
template <int TO_U8>
__global__ __launch_bounds__(256) void requant_i32_kernel(const int32_t *__restrict__ x, uint32_t n,
    uint8_t *__restrict__ q, const uint32_t *__restrict__ ws, float s0, float s1, float *__restrict__ ds_out)
{
    float r = 0.0f;
    float out0 = s0;
    if (s0 < 0 && s1 > 0) {
        int m = ws_read_max(ws);
        r = (m == 0) ? 1.0f : 127.0f / (float)m;
        out0 = s1 * r;
    } else if (s0 > 0 && s1 > 0) {
        r = s0 / s1;
    }
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    if (tid == 0 && ds_out) {
        *ds_out = out0;
    }
    const uint32_t stride = gridDim.x * blockDim.x;
#define BG_RQ(v) ((unsigned)(TO_U8 ? usat8_u(rne_i32((float)(v) * r + 128.0f)) : ssat8(rne_i32((float)(v) * r))) & 0xffu)
#define BG_RQ4(v) (BG_RQ(v.x) | (BG_RQ(v.y) << 8) | (BG_RQ(v.z) << 16) | (BG_RQ(v.w) << 24))
    uint32_t done = 0;
    if ((((uintptr_t)x | (uintptr_t)q) & 15) == 0) {
        const uint32_t n16 = n / 16;
        const v4i *x4 = (const v4i *)x;
        v4i *q16 = (v4i *)q;
        for (uint32_t i = tid; i < n16; i += stride) {
            v4i a = x4[4 * i], b = x4[4 * i + 1], c = x4[4 * i + 2], d = x4[4 * i + 3];
            v4i o = {(int)BG_RQ4(a), (int)BG_RQ4(b), (int)BG_RQ4(c), (int)BG_RQ4(d)};
            q16[i] = o;
        }
        done = n16 * 16;
    }
    for (uint32_t i = done + tid; i < n; i += stride) {
        q[i] = (uint8_t)BG_RQ(x[i]);
    }
#undef BG_RQ4
#undef BG_RQ
}

hipError_t launch_requant_i32(const int32_t *x, uint32_t n, void *q, int to_u8, const uint32_t *ws, float s0,
    float s1, float *ds_out, hipStream_t st)
{
    const uint32_t blocks = grid_for(n, 16, 256, 8192);
    if (to_u8) {
        hipLaunchKernelGGL((requant_i32_kernel<1>), dim3(blocks), dim3(256), 0, st, x, n, (uint8_t *)q, ws, s0, s1,
            ds_out);
    } else {
        hipLaunchKernelGGL((requant_i32_kernel<0>), dim3(blocks), dim3(256), 0, st, x, n, (uint8_t *)q, ws, s0, s1,
            ds_out);
    }
    return hipGetLastError();
}

// ---- dynamic quantisation in one launch, one read ----------------------------------------------------
// The two-pass form reads the tensor twice (max, then quantise) in two launches behind a scratch fill. Here
// every thread keeps its share of the tensor in registers across a grid-wide barrier: load (up to PER groups
// of 4 elements per thread), fold max|x| into the sync area, wait until every workgroup has arrived, take
// the maximum, quantise from the registers, store. The tensor is read once and the call is one launch.
//
// The grid is at most two workgroups of 256 threads per CU and never more than the occupancy the runtime reports
// for the kernel, so every workgroup is running when the first one reaches the barrier; a cooperative launch would have the runtime check that, but costs more than the launches saved.
// The grid-wide maximum goes through grid_max_sync (device_common.h): either every workgroup quantises with one
// maximum, or -- when the bounded wait of one of them expires -- none stores anything and the kernel publishes a NaN
// scale, on which the host runs the two-pass form: never a valid scale over partly written output.
template <int SRC_I32, int TO_U8, int PER>
__global__ __launch_bounds__(256) void quantize_fused_kernel(const void *__restrict__ xin, uint32_t n, uint8_t *__restrict__ q,
    GridSync gs, float s_in, float *ds_out)
{
    __shared__ int sync_lds[18];
    const uint32_t n4 = n / 4;
    const uint32_t tid = blockIdx.x * 256 + threadIdx.x, stride = gridDim.x * 256;
    const v4i *x4 = (const v4i *)xin;
    v4i r[PER];  // lane-contiguous 16-byte loads: a wave's request is 1 KB of whole cache lines
    int tail = 0;
    int m = 0;
    float mf = 0.0f;  // fp32 input: v_max_f32 drops NaNs, as the reference's compare-and-keep does
#define BG_FOLD(bits)                                                                  \
    {                                                                                  \
        int b_ = (bits);                                                               \
        if (SRC_I32) {                                                                 \
            int a_ = (b_ == (int)0x80000000) ? b_ : (b_ < 0 ? -b_ : b_); /* vpabsd: |INT32_MIN| stays negative */ \
            m = a_ > m ? a_ : m;                                                       \
        } else {                                                                       \
            mf = fmaxf(mf, fabsf(__int_as_float(b_)));                                 \
        }                                                                              \
    }
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const uint32_t u = tid + k * stride;
        r[k] = (u < n4) ? x4[u] : (v4i){0, 0, 0, 0};
        BG_FOLD(r[k].x) BG_FOLD(r[k].y) BG_FOLD(r[k].z) BG_FOLD(r[k].w)
    }
    if (n4 * 4 + tid < n) {  // fewer than 4 trailing elements, one each for the first threads
        tail = ((const int *)xin)[n4 * 4 + tid];
        BG_FOLD(tail)
    }
#undef BG_FOLD
    if (!SRC_I32) {
        m = __float_as_int(mf);  // non-negative float: integer order == float order
    }
    const uint32_t outcome = grid_max_sync(gs, m, sync_lds);
    if (outcome == kGridAbandoned) {  // the same for every workgroup of the launch: nothing is stored
        if (tid == 0 && ds_out) {
            *ds_out = __int_as_float(0x7fc00000);
        }
        return;
    }
    const int gmax = (int)outcome;
    float s, published;
    if (SRC_I32) {  // avx512/quantize.cpp:315-416 with scale[0] < 0: r = 127 / max, returned scale = scale[1] * r
        s = (gmax == 0) ? 1.0f : 127.0f / (float)gmax;
        published = s_in * s;
    } else {  // :129-133 / :189-193: max(caller's scale, 127 / max|x|), 127 / 0 replaced by 1
        const float mx = __int_as_float(gmax);
        const float dyn = (mx == 0.0f) ? 1.0f : 127.0f / mx;
        s = (s_in > dyn) ? s_in : dyn;
        published = s;
    }
    if (tid == 0 && ds_out) {
        *ds_out = published;
    }
#define BG_QF(bits)                                                                                        \
    ((unsigned)(SRC_I32 ? (TO_U8 ? usat8_u(rne_i32((float)(bits)*s + 128.0f)) : ssat8(rne_i32((float)(bits)*s))) \
                        : (TO_U8 ? q_u8(__int_as_float(bits), s) : q_i8(__int_as_float(bits), s))) & 0xffu)
#define BG_QF4(v) ((int)(BG_QF(v.x) | (BG_QF(v.y) << 8) | (BG_QF(v.z) << 16) | (BG_QF(v.w) << 24)))
    int *q4 = (int *)q;
#pragma unroll
    for (int k = 0; k < PER; ++k) {
        const uint32_t u = tid + k * stride;
        if (u < n4) {
            q4[u] = BG_QF4(r[k]);
        }
    }
    if (n4 * 4 + tid < n) {
        q[n4 * 4 + tid] = (uint8_t)BG_QF(tail);
    }
#undef BG_QF4
#undef BG_QF
}

// Workgroups the barrier is allowed to span: two per CU, or one where the kernel's registers allow no more
// (0 if the device cannot be asked).
template <int SRC_I32, int TO_U8, int PER>
static uint32_t fused_max_grid()
{
    static int cached = -1;
    if (cached < 0) {
        int dev = 0, cus = 0, per_cu = 0;
        if (hipGetDevice(&dev) != hipSuccess || hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess ||
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&per_cu, quantize_fused_kernel<SRC_I32, TO_U8, PER>, 256, 0) != hipSuccess) {
            cached = 0;
        } else {
            cached = cus * (per_cu >= 2 ? 2 : per_cu);
            cached = cached > (int)kGridSyncMaxBlocks ? (int)kGridSyncMaxBlocks : cached;
        }
    }
    return (uint32_t)cached;
}

template <int SRC_I32, int TO_U8, int PER>
static hipError_t launch_fused(const void *x, uint32_t n, void *q, FusedSync &fs, float s_in, float *ds_out, hipStream_t st,
    bool *taken)
{
    const uint32_t units = n / 4, per_block = 256 * PER;
    uint32_t grid = (units + per_block - 1) / per_block;
    grid = grid ? grid : 1;
    if (grid > fused_max_grid<SRC_I32, TO_U8, PER>()) {
        return hipSuccess;  // *taken stays false
    }
    const GridSync gs = fs.next(grid);
    hipLaunchKernelGGL((quantize_fused_kernel<SRC_I32, TO_U8, PER>), dim3(grid), dim3(256), 0, st, x, n, (uint8_t *)q, gs, s_in,
        ds_out);
    hipError_t e = hipGetLastError();
    if (e != hipSuccess) {
        return e;
    }
    *taken = true;
    return hipSuccess;
}

// Dynamic fp32 -> u8 / s8 (src_i32 = 0; s_in = the caller's scale, <= 0 for none) or int32 -> u8 / s8 (src_i32 = 1;
// s_in = scale of the int32 data) in one launch. *taken = false (and nothing launched) when the
// tensor is larger than the size up to which this form wins (512 K elements), or misaligned: the caller then runs
// the two-pass form.
hipError_t launch_quantize_fused(const void *x, uint32_t n, void *q, int src_i32, int to_u8, FusedSync &fs, float s_in,
    float *ds_out, hipStream_t st, bool *taken)
{
    *taken = false;
    // Measured on MI355X against the two-pass form (whose second read comes from the Infinity Cache): 10.4 against
    // 14.9 us per call at 1 K elements, 12.0 against 15.4 at 64 K, 12.9 against 15.4 at 256 K, 16.3 against 15.4 at
    // 1 M, slower beyond (the barrier's
    // arrivals serialise at one address, about 10 ns each, and nothing overlaps the two phases).
    if (n == 0 || n > (1u << 19) || !fs.slots || ((((uintptr_t)x | (uintptr_t)q) & 15) != 0)) {
        return hipSuccess;
    }
#define BG_TRY(S, U, P)                                                                        \
    {                                                                                          \
        hipError_t e_ = launch_fused<S, U, P>(x, n, q, fs, s_in, ds_out, st, taken);           \
        if (e_ != hipSuccess || *taken) {                                                      \
            return e_;                                                                         \
        }                                                                                      \
    }
#define BG_TRY_PER(S, U)   \
    {                      \
        BG_TRY(S, U, 4)    \
        BG_TRY(S, U, 8)    \
    }
    if (src_i32) {
        if (to_u8) {
            BG_TRY_PER(1, 1)
        } else {
            BG_TRY_PER(1, 0)
        }
    } else if (to_u8) {
        BG_TRY_PER(0, 1)
    } else {
        BG_TRY_PER(0, 0)
    }
#undef BG_TRY_PER
#undef BG_TRY
    return hipSuccess;
}

// avx512/quantize.cpp:271-313
__global__ void u8_to_i8_kernel(const uint8_t *__restrict__ x, uint32_t n, int8_t *__restrict__ q)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        q[i] = (int8_t)(uint8_t)(x[i] + 0x80);
    }
}

hipError_t launch_u8_to_i8(const uint8_t *x, uint32_t n, int8_t *q, hipStream_t st)
{
    hipLaunchKernelGGL(u8_to_i8_kernel, dim3(grid_for(n, 4, 256, 8192)), dim3(256), 0, st, x, n, q);
    return hipGetLastError();
}

// y = a * x + b * y in fp32 (compute/blas_enhance/src/cpu/x86/fp32/axpby.cpp:16-34): the vector body there is
// fmadd(a, x, y * b) -- one multiply rounded, then one fused multiply-add.
__global__ __launch_bounds__(256) void axpby_f32_kernel(uint32_t n, float a, const float *__restrict__ x, float b,
    float *__restrict__ y)
{
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t stride = gridDim.x * blockDim.x;
    uint32_t done = 0;
    if ((((uintptr_t)x | (uintptr_t)y) & 15) == 0) {
        const uint32_t n4 = n / 4;
        const v4f *x4 = (const v4f *)x;
        v4f *y4 = (v4f *)y;
        for (uint32_t i = tid; i < n4; i += stride) {
            const v4f u = x4[i], v = y4[i];
            y4[i] = (v4f){__builtin_fmaf(a, u.x, v.x * b), __builtin_fmaf(a, u.y, v.y * b), __builtin_fmaf(a, u.z, v.z * b),
                __builtin_fmaf(a, u.w, v.w * b)};
        }
        done = n4 * 4;
    }
    for (uint32_t i = done + tid; i < n; i += stride) {
        y[i] = __builtin_fmaf(a, x[i], y[i] * b);
    }
}

hipError_t launch_axpby_f32(uint32_t n, float a, const float *x, float b, float *y, hipStream_t st)
{
    hipLaunchKernelGGL(axpby_f32_kernel, dim3(grid_for(n, 4, 256, 8192)), dim3(256), 0, st, n, a, x, b, y);
    return hipGetLastError();
}

// ---- dequantize: avx512/dequantize.cpp:18-101, f = cvt(q) * (1 / s) -----------------------------
__global__ __launch_bounds__(256) void dequant_i32_kernel(const int32_t *__restrict__ q, uint32_t n, const float *__restrict__ ds,
    float s, float *__restrict__ out)
{
    const float f = 1 / (ds ? *ds : s);
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t stride = gridDim.x * blockDim.x;
    uint32_t done = 0;
    if ((((uintptr_t)q | (uintptr_t)out) & 15) == 0) {
        const uint32_t n4 = n / 4;
        const v4i *q4 = (const v4i *)q;
        v4f *o4 = (v4f *)out;
        uint32_t i = tid;
        for (; i + stride < n4; i += 2 * stride) {  // two independent 16-byte loads in flight
            const v4i a = ld_stream(q4 + i), b = ld_stream(q4 + i + stride);
            st_stream(o4 + i, (v4f){(float)a.x * f, (float)a.y * f, (float)a.z * f, (float)a.w * f});
            st_stream(o4 + i + stride, (v4f){(float)b.x * f, (float)b.y * f, (float)b.z * f, (float)b.w * f});
        }
        for (; i < n4; i += stride) {
            const v4i a = ld_stream(q4 + i);
            o4[i] = (v4f){(float)a.x * f, (float)a.y * f, (float)a.z * f, (float)a.w * f};
        }
        done = n4 * 4;
    }
    for (uint32_t i = done + tid; i < n; i += stride) {
        out[i] = (float)q[i] * f;
    }
}

__global__ void dequant_u8_kernel(const uint8_t *__restrict__ q, uint32_t n, const float *__restrict__ ds, float s,
    float *__restrict__ out)
{
    const float f = 1 / (ds ? *ds : s);
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        out[i] = (float)((int)q[i] - 128) * f;
    }
}

hipError_t launch_dequant_i32(const int32_t *q, uint32_t n, const float *ds, float s, float *out, hipStream_t st)
{
    hipLaunchKernelGGL(dequant_i32_kernel, dim3(grid_for(n, 4, 256, 8192)), dim3(256), 0, st, q, n, ds, s, out);
    return hipGetLastError();
}

hipError_t launch_dequant_u8(const uint8_t *q, uint32_t n, const float *ds, float s, float *out, hipStream_t st)
{
    hipLaunchKernelGGL(dequant_u8_kernel, dim3(grid_for(n, 4, 256, 8192)), dim3(256), 0, st, q, n, ds, s, out);
    return hipGetLastError();
}

// ---- bias fold: avx512/quantize.cpp:236-269 -----------------------------------------------------
// out[n] = (I32)(round(bias[n] * s) + offsetC[n]); round() is half away from zero.
__global__ void bias_offsetC_kernel(const float *__restrict__ bias, uint32_t N, const int32_t *__restrict__ offsetC,
    const float *__restrict__ dsA, float sB, int32_t *__restrict__ out)
{
    const uint32_t i = blockIdx.x * blockDim.x + threadIdx.x;
    if (i >= N) {
        return;
    }
    if (!bias) {
        out[i] = offsetC ? offsetC[i] : 0;
        return;
    }
    const float s = dsA ? (*dsA * sB) : sB;
    float p = bias[i] * s;
    double r = round((double)p);
    if (offsetC) {
        r += (double)offsetC[i];
    }
    out[i] = (int32_t)r;
}

hipError_t launch_bias_offsetC(const float *bias, uint32_t N, const int32_t *offsetC, const float *dsA, float sB,
    int32_t *out, hipStream_t st)
{
    if (N == 0) {
        return hipSuccess;
    }
    hipLaunchKernelGGL(bias_offsetC_kernel, dim3((N + 255) / 256), dim3(256), 0, st, bias, N, offsetC, dsA, sB, out);
    return hipGetLastError();
}

// ---- s8 rescale: compute/tensor/src/cpu/requantize.cpp:20-50 ------------------------------------
__global__ void requantize_i8_kernel(const int8_t *__restrict__ in, uint32_t n, float r, int8_t *__restrict__ out)
{
    const uint32_t stride = gridDim.x * blockDim.x;
    for (uint32_t i = blockIdx.x * blockDim.x + threadIdx.x; i < n; i += stride) {
        float v = r * (float)in[i] + 0.0f;
        out[i] = (int8_t)(int)v;
    }
}

hipError_t launch_requantize_i8(const int8_t *in, uint32_t n, float r, int8_t *out, hipStream_t st)
{
    // 16 bytes per lane through the concatenation kernel (one row) where both pointers allow it; the last
    // n % 16 bytes, or everything when a pointer is not 16-byte aligned, one byte per lane
    uint32_t body = 0;
    if ((((uintptr_t)in | (uintptr_t)out) & 15) == 0) {
        body = n & ~15u;
        if (body) {
            hipError_t e = launch_concat_i8(in, out, 1, body, body, 1, r, st);
            if (e != hipSuccess) {
                return e;
            }
        }
    }
    if (n > body) {
        hipLaunchKernelGGL(requantize_i8_kernel, dim3(grid_for(n - body, 4, 256, 8192)), dim3(256), 0, st, in + body,
            n - body, r, out + body);
    }
    return hipGetLastError();
}

}  // namespace bg
