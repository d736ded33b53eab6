// Device-side helpers shared by the gfx950 kernels: the exact rounding / saturation steps of
// the x86 AVX-512 epilogues the results must match bit-for-bit, and wave64 reductions.
#pragma once
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace bg {

typedef int v4i __attribute__((ext_vector_type(4)));
typedef int v2i __attribute__((ext_vector_type(2)));
typedef int v16i __attribute__((ext_vector_type(16)));
typedef float v4f __attribute__((ext_vector_type(4)));
typedef int v8i __attribute__((ext_vector_type(8)));

constexpr int kWave = 64;

// vcvtps2dq: round to nearest even; NaN and out-of-range give 0x80000000.
__device__ __forceinline__ int rne_i32(float v)
{
    if (!(v >= -2147483648.0f && v < 2147483648.0f)) {
        return (int)0x80000000;
    }
    return (int)__builtin_rintf(v);
}

// vpmovusdb: the dword is saturated as an UNSIGNED number, so every negative becomes 255.
__device__ __forceinline__ unsigned usat8_u(int v)
{
    return ((unsigned)v > 255u) ? 255u : (unsigned)v;
}

// vpmovsdb: signed saturation to [-128, 127].
__device__ __forceinline__ int ssat8(int v)
{
    return v < -128 ? -128 : (v > 127 ? 127 : v);
}

// Output selector of the GEMM / GEMV / conv epilogue.
enum EpiMode : int {
    EPI_I32 = 0,       // raw accumulator
    EPI_F32 = 1,       // cvt(acc) * factor                      (factor = 1.0f / scale[0])
    EPI_U8 = 2,        // usat8_u(rne(cvt(acc) * factor) + 128)  (factor = scale[1])
    EPI_F32_CH = 3,    // cvt(acc) * (1.0f / (sI * sW[n])) + bias[n]   per-output-channel extension
    EPI_U8_TRUNC = 4   // (int)(cvt(acc) * factor + 128.0f), > 255 -> 255, else low byte
};

struct Epilogue {
    int mode = 0;
    float factor = 0;            // EPI_F32 / EPI_U8 when dfactor == nullptr
    const float *dfactor = nullptr;    // optional device scalar: EPI_F32 uses 1.0f / *dfactor, EPI_U8 uses *dfactor
    const float *scaleI = nullptr;     // EPI_F32_CH: device scalar input scale
    const float *scaleW = nullptr;     // EPI_F32_CH: device per-channel weight scales [N]
    const float *bias = nullptr;       // EPI_F32_CH: optional device fp32 bias [N]
};

__device__ __forceinline__ float epi_factor(const Epilogue &e)
{
    if (e.dfactor) {
        float s = *e.dfactor;
        return (e.mode == EPI_F32) ? 1.0f / s : s;
    }
    return e.factor;
}

__device__ __forceinline__ unsigned epi_u8(int acc, float factor)
{
    float f = (float)acc * factor;
    return usat8_u((int)((unsigned)rne_i32(f) + 128u));
}

// fp32 -> u8 around the zero point 128
__device__ __forceinline__ unsigned q_u8(float x, float s)
{
    // avx512/quantize.cpp:150-155: vmulps, vaddps 128.0f, vcvtps2dq {rn}, clamp [1, 255]
    float t = x * s;
    float u = t + 128.0f;
    int v = rne_i32(u);
    v = v < 1 ? 1 : v;
    v = v > 255 ? 255 : v;
    return (unsigned)v;
}

__device__ __forceinline__ unsigned epi_u8_trunc(int acc, float factor)
{
    float f = (float)acc * factor;
    float g = f + 128.0f;
    int t = (!(g >= -2147483648.0f && g < 2147483648.0f)) ? (int)0x80000000 : (int)g;
    return (t > 255) ? 255u : ((unsigned)t & 0xffu);
}

__device__ __forceinline__ float epi_f32_ch(int acc, float sI, float sW, const float *bias, int n)
{
    float s = sI * sW;
    float f = 1.0f / s;
    float v = (float)acc * f;
    if (bias) {
        v = v + bias[n];
    }
    return v;
}

__device__ __forceinline__ int wave_reduce_add(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    return v;
}

__device__ __forceinline__ float wave_reduce_max(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v = fmaxf(v, __shfl_xor(v, off, 64));
    }
    return v;
}

// Load / store for data that a kernel touches exactly once and that is too large to stay cached.
template <typename V>
__device__ __forceinline__ V ld_stream(const V *p)
{
    return __builtin_nontemporal_load(p);
}

template <typename V>
__device__ __forceinline__ void st_stream(V *p, V v)
{
    __builtin_nontemporal_store(v, p);
}

// Offset a product's column n starts from, less the compensation of the u8 -> s8 re-bias: ob[n] - comp[n], or --
// when the caller hands over the fp32 bias instead of a folded vector -- the fold done here exactly as the
// stand-alone kernel does it (round(bias * scale) + offsetC in double, converted to int32;
// avx512/quantize.cpp:236-269), so that no separate launch is needed for it.
__device__ __forceinline__ uint32_t column_base(const int32_t *ob, const int32_t *comp, const float *fold_bias,
    float fold_scale, uint32_t n)
{
    const int32_t c = comp[n];
    if (fold_bias) {
        const float p = fold_bias[n] * fold_scale;
        const int32_t o = (int32_t)(round((double)p) + (double)c);
        return (uint32_t)o - (uint32_t)c;
    }
    return (uint32_t)ob[n] - (uint32_t)c;
}

__device__ __forceinline__ float wave_reduce_sum(float v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        v += __shfl_xor(v, off, 64);
    }
    return v;
}

__device__ __forceinline__ int wave_reduce_max_i(int v)
{
#pragma unroll
    for (int off = 32; off > 0; off >>= 1) {
        int o = __shfl_xor(v, off, 64);
        v = v > o ? v : o;
    }
    return v;
}

// tanh-form GELU: x * 0.5 * (1 + tanh(sqrt(2/pi) * (x + 0.044715 x^3))), with tanh(u/2) written as 1 - 2 / (1 + e^u)
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float c0 = 1.5957691216057308f;  // 2 * sqrt(2 / pi)
    const float u = (c0 * x) * __builtin_fmaf(0.044715f, x * x, 1.0f);
    const float e = __expf(u);
    return (2.0f - 2.0f * __builtin_amdgcn_rcpf(1.0f + e)) * (0.5f * x);  // v_rcp_f32: 1 ulp, far inside the layer's tolerance
}

// ---- tensor-wide max through device scratch words --------------------------------------------------
// Atomics from many workgroups to ONE address serialise at the memory side (the eight XCDs' L2s
// are not coherent with each other), ~10 ns apiece. The running max is therefore spread over
// kWsSlots words, one per 64-byte line; a producer workgroup folds its result into slot
// (workgroup % kWsSlots), every consumer wave reads all slots with one load per lane.
constexpr uint32_t kWsSlots = 64, kWsStride = 16, kWsWords = kWsSlots * kWsStride;

__device__ __forceinline__ void ws_fold_max(uint32_t *ws, uint32_t group, int v)
{
    if (v != 0) {
        atomicMax((int *)ws + (group % kWsSlots) * kWsStride, v);
    }
}

// Workgroup-wide max of non-negative ints, folded into the slot of this workgroup. `red` = one
// LDS word per wave. Values are non-negative floats' bit patterns or non-negative ints, so the
// integer order is the wanted order either way.
__device__ __forceinline__ void ws_block_fold_max(uint32_t *ws, int v, int *red)
{
    v = wave_reduce_max_i(v);
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6, waves = (blockDim.x + 63) >> 6;
    if (lane == 0) {
        red[wave] = v;
    }
    __syncthreads();
    if (threadIdx.x == 0) {
        for (uint32_t w = 1; w < waves; ++w) {
            v = red[w] > v ? red[w] : v;
        }
        ws_fold_max(ws, blockIdx.x + blockIdx.y * gridDim.x, v);
    }
}

__device__ __forceinline__ int ws_read_max(const uint32_t *ws)
{
    return wave_reduce_max_i((int)ws[(threadIdx.x & (kWsSlots - 1)) * kWsStride]);
}

}  // namespace bg
