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
    EPI_U8_TRUNC = 4,  // (int)(cvt(acc) * factor + 128.0f), > 255 -> 255, else low byte
    // y = gelu_tanh(cvt(acc) * (1.0f / (sI * sW[n])) + bias[n]); u8 = quantise(y) with the tensor-wide dynamic scale
    // max(0, 127 / max|y|), the maximum agreed on by all workgroups of the launch while y is still in registers
    EPI_U8_GELU_DYN = 5,
    // per-output-channel extension with a u8 result: q_u8(cvt(acc) * (1.0f / (sI * sW[n])) + bias[n], factor) -- the
    // fp32 value of EPI_F32_CH put through the fp32 -> u8 quantiser with the given (static) output scale
    EPI_U8_CH = 6,
    // int8 convolution with per-output-channel filter scales (GemmArgs::conv.ch_out says what is done with the value):
    // f = cvt(acc) * (1.0f / (sI * sW[oc])) + bias[oc] (+ eltwise), ReLU
    EPI_CONV_CH = 7
};

// what EPI_CONV_CH does with its fp32 values
enum ConvChOut : int {
    CONV_CH_F32 = 0,   // stored as they are
    CONV_CH_U8 = 1,    // q_u8(f, s): s = epi.factor when > 0 (static), else 127 / max|f| from the scratch slots (1 for 0)
    CONV_CH_MAX = 2    // nothing stored: max|f| (its bits, an order-preserving int) folded into the scratch slots
};

struct Epilogue {
    int mode = 0;
    float factor = 0;            // EPI_F32 / EPI_U8 when dfactor == nullptr
    const float *dfactor = nullptr;    // optional device scalar: EPI_F32 uses 1.0f / *dfactor, EPI_U8 uses *dfactor
    const float *scaleI = nullptr;     // EPI_F32_CH / EPI_U8_CH: device scalar input scale
    const float *scaleW = nullptr;     // EPI_F32_CH / EPI_U8_CH / EPI_CONV_CH: device per-channel weight scales [N]
    const float *bias = nullptr;       // EPI_F32_CH / EPI_U8_CH / EPI_CONV_CH: optional device fp32 bias [N]
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

// column_base() for NC columns n[0..NC-1] at once: every load first and none behind a branch (the vector that the
// mode does not use is read from the other one's address), so that all of them are in flight together instead of each
// costing its own trip to memory. Columns whose n is past N must be clamped by the caller (n < N always).
template <int NC>
__device__ __forceinline__ void column_bases(const int32_t *ob, const int32_t *comp, const float *fold_bias, float fold_scale,
    const uint32_t (&n)[NC], uint32_t (&base)[NC])
{
    const bool fold = fold_bias != nullptr;
    const int32_t *obp = fold ? comp : ob;
    const float *fbp = fold ? fold_bias : (const float *)comp;
    int32_t c[NC], o[NC];
    float f[NC];
#pragma unroll
    for (int k = 0; k < NC; ++k) {
        c[k] = comp[n[k]];
        o[k] = obp[n[k]];
        f[k] = fbp[n[k]];
    }
#pragma unroll
    for (int k = 0; k < NC; ++k) {
        const float p = f[k] * fold_scale;
        const int32_t v = fold ? (int32_t)(round((double)p) + (double)c[k]) : o[k];
        base[k] = (uint32_t)v - (uint32_t)c[k];
    }
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

// tanh-form GELU: x * 0.5 * (1 + tanh(sqrt(2/pi) * (x + 0.044715 x^3))). With u = 2 sqrt(2/pi) (x + 0.044715 x^3),
// 0.5 (1 + tanh(u / 2)) = 1 - 1 / (1 + e^u), so gelu(x) = x - x / (1 + e^u): eight instructions, two of them
// transcendental (e^u as 2^(u log2 e) with the factor folded into the constant; v_exp_f32 and v_rcp_f32 are 1 ulp,
// far inside the layer's tolerance). x -> -inf gives e^u = 0 and x - x = 0, x -> +inf gives 1 / inf = 0 and x.
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float c0 = 2.3022082f;  // 2 * sqrt(2 / pi) * log2(e)
    const float u = (c0 * x) * __builtin_fmaf(0.044715f, x * x, 1.0f);
    const float e = __builtin_amdgcn_exp2f(u);
    return __builtin_fmaf(-x, __builtin_amdgcn_rcpf(1.0f + e), x);
}

// fp32 -> u8 around the zero point 128 for values known to satisfy |x * s| <= 127 (1 + 2^-22) -- a tensor quantised
// with the dynamic scale 127 / max|x| of its own maximum: the same bytes as q_u8 in four instructions. The sum with
// 2^23 rounds t + 128 (already rounded to fp32 once, like q_u8's) to the nearest-even integer and leaves it in the
// low mantissa bits; clamping to [1, 255] before that rounding equals clamping after it (both are monotone).
// Returns the word whose low byte is the result. NaN quantises to 1 as in q_u8 (v_med3_f32 drops it).
__device__ __forceinline__ uint32_t q_u8_inrange_bits(float x, float s)
{
    const float t = x * s;
    const float u = t + 128.0f;
    const float w = __builtin_amdgcn_fmed3f(u, 1.0f, 255.0f);
    return __float_as_uint(w + 8388608.0f);
}

// low bytes of four words -> one dword (byte 0 = a)
__device__ __forceinline__ uint32_t pack_low_bytes(uint32_t a, uint32_t b, uint32_t c, uint32_t d)
{
    const uint32_t ab = __builtin_amdgcn_perm(b, a, 0x0c0c0400u);  // byte 0 = a[0], byte 1 = b[0], upper bytes 0
    const uint32_t cd = __builtin_amdgcn_perm(d, c, 0x04000c0cu);  // byte 2 = c[0], byte 3 = d[0], lower bytes 0
    return ab | cd;
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

// ---- grid-wide maximum with a bounded wait ------------------------------------------------------------
// For kernels whose workgroups are all resident at once (the launcher sizes the grid for that) and that must
// agree on one tensor-wide maximum half way through, with their partial results still in registers.
//
// Sync area (device memory, zeroed once when allocated, never cleared afterwards): one 64-bit slot per workgroup
// (at most kGridSyncMaxBlocks) and 64 release words, one per 64-byte line. A launch carries an epoch that grows
// with every launch. Every workgroup stores (epoch << 32 | its maximum) into its own slot -- one store, no atomic
// read-modify-write, nothing to wait for. Workgroup 0 collects: its first wave polls all slots (64 per load
// instruction) until each carries this launch's epoch, takes the maximum and publishes (epoch << 32 | max) in the
// release words; the others poll the release word of their own line. Traffic grows with the number of workgroups,
// not with its square (every workgroup polling every slot cost 5-10 us at 400-1000 workgroups), and no address
// takes more than one store per workgroup (an arrival counter serialises at about 10 ns per workgroup).
//
// The waits are bounded, and the outcome is decided exactly once, by a compare-and-swap on release word 0: the
// collector proposes the maximum, a workgroup whose bound expires (the collector included) proposes "abandoned"
// (epoch << 32 | 0xffffffff); whoever swaps first wins and copies the outcome to the other 63 words; every other
// workgroup -- a loser of the swap too -- acts on that one outcome. So all workgroups of a launch see the same
// maximum, or all see "abandoned" (kGridAbandoned).
// Launches that share a sync area must be ordered on one stream.
constexpr uint32_t kGridSyncMaxBlocks = 1024;
struct GridSync {
    unsigned long long *slots = nullptr;    // kGridSyncMaxBlocks words
    unsigned long long *release = nullptr;  // 64 words, 8 words apart
    uint32_t epoch = 0;        // this launch's tag
    uint32_t blocks = 0;       // workgroups in the launch (gridDim.x, <= kGridSyncMaxBlocks)
    uint32_t spin_limit = 0;   // polling rounds (about a microsecond each) before a waiting workgroup gives up
    unsigned *done = nullptr;  // arrival counter for grid_last_arrival (a spare word of the area; zero between launches)
};
constexpr uint32_t kGridAbandoned = 0xffffffffu;  // never a maximum: those are non-negative floats' bits, ints >= 0 or INT32_MIN

// proposes `value` as this epoch's outcome on release word 0, copies it to the other words if it stands, and returns
// the outcome that stands. Called by lane 0 of a wave.
__device__ __forceinline__ uint32_t grid_sync_decide(unsigned long long *release, uint32_t epoch, uint32_t value)
{
    const unsigned long long mine = ((unsigned long long)epoch << 32) | value;
    unsigned long long cur = __hip_atomic_load(release, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
    while ((uint32_t)(cur >> 32) != epoch) {
        const unsigned long long seen = atomicCAS(release, cur, mine);
        if (seen == cur) {
            for (uint32_t k = 1; k < 64; ++k) {
                __hip_atomic_store(release + k * 8, mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
            }
            return value;
        }
        cur = seen;
    }
    return (uint32_t)cur;
}

// Called by every thread of every workgroup of the launch (uniform control flow) with its own candidate `m`
// (values whose signed-integer order is the wanted order: non-negative floats' bits or ints). `lds`: 18 ints of
// the workgroup's LDS; workgroups of whole waves, at most 16; blockIdx.x numbers the workgroups. Returns the
// grid-wide maximum or kGridAbandoned, the same value in every thread of the grid.
// `tid` = threadIdx.x; a kernel with no register to spare across its main loop hands in a value it has formed afresh.
__device__ __forceinline__ uint32_t grid_max_sync(const GridSync &gs, int m, int *lds, uint32_t tid)
{
    const uint32_t lane = tid & 63, wave = tid >> 6, waves = blockDim.x >> 6;
    m = wave_reduce_max_i(m);
    if (lane == 0) {
        lds[wave] = m;
    }
    __syncthreads();
    if (wave == 0) {
        int mine = (lane < waves) ? lds[lane] : (int)0x80000000;
        mine = wave_reduce_max_i(mine);
        const unsigned long long tag = (unsigned long long)gs.epoch << 32;
        if (lane == 0) {
            __hip_atomic_store(gs.slots + blockIdx.x, tag | (uint32_t)mine, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
        }
        uint32_t spins = 0, outcome = kGridAbandoned;
        if (blockIdx.x == 0) {  // the collector
            for (;;) {
                bool ok = true;
                int v = mine;
                for (uint32_t b = lane; b < gs.blocks; b += 64) {
                    if (b != 0) {  // its own slot needs no trip to memory
                        const unsigned long long t = __hip_atomic_load(gs.slots + b, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                        ok = ok && ((uint32_t)(t >> 32) == gs.epoch);
                        const int tv = (int)(uint32_t)t;
                        v = tv > v ? tv : v;
                    }
                }
                if (__all(ok)) {
                    v = wave_reduce_max_i(v);
                    if (lane == 0) {
                        outcome = grid_sync_decide(gs.release, gs.epoch, (uint32_t)v);
                    }
                    break;
                }
                if (++spins > gs.spin_limit) {
                    if (lane == 0) {
                        outcome = grid_sync_decide(gs.release, gs.epoch, kGridAbandoned);
                    }
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        } else if (lane == 0) {
            for (;;) {
                const unsigned long long t =
                    __hip_atomic_load(gs.release + (blockIdx.x & 63) * 8, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);
                if ((uint32_t)(t >> 32) == gs.epoch) {
                    outcome = (uint32_t)t;
                    break;
                }
                if (++spins > gs.spin_limit) {  // give up, unless the outcome has been decided meanwhile
                    outcome = grid_sync_decide(gs.release, gs.epoch, kGridAbandoned);
                    break;
                }
                __builtin_amdgcn_s_sleep(2);
            }
        }
        if (lane == 0) {
            lds[17] = (int)outcome;
        }
    }
    __syncthreads();
    return (uint32_t)lds[17];
}

__device__ __forceinline__ uint32_t grid_max_sync(const GridSync &gs, int m, int *lds)
{
    return grid_max_sync(gs, m, lds, threadIdx.x);
}


// What a kernel does when grid_max_sync() was abandoned and it cannot leave the job to the host: every workgroup
// first stores its partial result where a second pass can read it, then calls this (all threads); exactly one
// workgroup -- the last to arrive -- gets true and does that second pass alone, the others return. No workgroup
// waits for another, so it works whatever part of the grid is resident. The fences make the others' stores visible
// to the one that continues. `lds`: the 18 ints grid_max_sync used.
__device__ __forceinline__ bool grid_last_arrival(const GridSync &gs, int *lds, uint32_t tid)
{
    __threadfence();
    __syncthreads();
    if (tid == 0) {
        const unsigned prev = __hip_atomic_fetch_add(gs.done, 1u, __ATOMIC_ACQ_REL, __HIP_MEMORY_SCOPE_AGENT);
        const bool last = prev + 1 == gs.blocks;
        if (last) {
            __hip_atomic_store(gs.done, 0u, __ATOMIC_RELAXED, __HIP_MEMORY_SCOPE_AGENT);  // for the next launch on the stream
        }
        lds[16] = last ? 1 : 0;
    }
    __syncthreads();
    const bool last = lds[16] != 0;
    if (last) {
        __threadfence();
    }
    return last;
}

__device__ __forceinline__ bool grid_last_arrival(const GridSync &gs, int *lds)
{
    return grid_last_arrival(gs, lds, threadIdx.x);
}

// Both passes of a dynamic fp32 -> u8 quantisation (scale 127 / max|x|, 1 for an all-zero tensor) by ONE workgroup of
// whole waves (at most 16): the second pass of grid_last_arrival()'s survivor. `red`: 16 floats of LDS.
__device__ __forceinline__ void quantize_f32_u8_alone(const float *x, uint32_t n, uint8_t *q, float *ds_out, float *red, uint32_t tid)
{
    const uint32_t nt = blockDim.x;
    float m = 0.0f;
    for (uint32_t k = tid; k < n; k += nt) {
        const float a_ = fabsf(x[k]);
        m = (a_ > m) ? a_ : m;  // a NaN never replaces the running max (avx512/quantize.cpp:21-68)
    }
    m = wave_reduce_max(m);
    __syncthreads();
    if ((tid & 63) == 0) {
        red[tid >> 6] = m;
    }
    __syncthreads();
    m = red[0];
    for (uint32_t w = 1; w < (nt >> 6); ++w) {
        m = red[w] > m ? red[w] : m;
    }
    const float s = (m == 0.0f) ? 1.0f : 127.0f / m;
    if (tid == 0 && ds_out) {
        *ds_out = s;
    }
    for (uint32_t k = tid; k < n; k += nt) {
        q[k] = (uint8_t)q_u8(x[k], s);
    }
}

__device__ __forceinline__ void quantize_f32_u8_alone(const float *x, uint32_t n, uint8_t *q, float *ds_out, float *red)
{
    quantize_f32_u8_alone(x, n, q, ds_out, red, threadIdx.x);
}

}  // namespace bg
