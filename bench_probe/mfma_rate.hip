// Measurement aid, not part of the reference's interface: the rate the int8 matrix cores sustain on this
// device when nothing else limits them. Every wave keeps an 8 x 4 grid of 16x16 accumulator tiles (the
// GEMM kernel's wave tile) and issues v_mfma_i32_16x16x64_i8 back to back on operands that never leave its
// registers; there is no memory traffic inside the loop. With random operand bits the device lowers its
// clock under the load, with all-zero operands it does not: the two figures bracket what any int8 kernel
// can reach here, and the GEMM figures are read against them.
// Built into its own bench-only library (bench_probe/libbench_probe.so); the product library does not contain it.
#include <hip/hip_runtime.h>
#include <stdint.h>

namespace {

typedef int v4i __attribute__((ext_vector_type(4)));

__device__ __forceinline__ uint32_t probe_mix(uint32_t x)
{
    x ^= x >> 16;
    x *= 0x7feb352du;
    x ^= x >> 15;
    x *= 0x846ca68bu;
    x ^= x >> 16;
    return x;
}

__global__ __launch_bounds__(512) void mfma_i8_rate_kernel(uint32_t iters, int zero, int *sink)
{
    constexpr int TM = 8, TN = 4;
    v4i a[TM], b[TN], acc[TM][TN];
    uint32_t s = probe_mix(threadIdx.x + blockIdx.x * 977u + 1u);
#pragma unroll
    for (int i = 0; i < TM; ++i) {
        for (int c = 0; c < 4; ++c) {
            s = probe_mix(s);
            a[i][c] = zero ? 0 : (int)s;
        }
    }
#pragma unroll
    for (int j = 0; j < TN; ++j) {
        for (int c = 0; c < 4; ++c) {
            s = probe_mix(s);
            b[j][c] = zero ? 0 : (int)s;
        }
    }
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            acc[i][j] = v4i{0, 0, 0, 0};
        }
    }
    for (uint32_t it = 0; it < iters; ++it) {
#pragma unroll
        for (int i = 0; i < TM; ++i) {
#pragma unroll
            for (int j = 0; j < TN; ++j) {
                acc[i][j] = __builtin_amdgcn_mfma_i32_16x16x64_i8(a[i], b[j], acc[i][j], 0, 0, 0);
            }
        }
    }
    int r = 0;
#pragma unroll
    for (int i = 0; i < TM; ++i) {
#pragma unroll
        for (int j = 0; j < TN; ++j) {
            r ^= acc[i][j][0] ^ acc[i][j][1] ^ acc[i][j][2] ^ acc[i][j][3];
        }
    }
    if (sink && r == 0x5eed1234 && iters == 0xffffffffu) {  // never true for a real call: keeps the loop alive
        sink[0] = r;
    }
}

}  // namespace

// TOP/s of v_mfma_i32_16x16x64_i8 issued back to back from registers by 8 waves on every CU: the best of three
// timed launches of a few milliseconds each on the default stream. Returns 0, or a hipError_t value.
extern "C" int bench_probe_mfma_int8_rate(int zero_operands, float *tops)
{
    if (!tops) {
        return (int)hipErrorInvalidValue;
    }
    int dev = 0, cus = 0;
    hipError_t err = hipGetDevice(&dev);
    if (err == hipSuccess) {
        err = hipDeviceGetAttribute(&cus, hipDeviceAttributeMultiprocessorCount, dev);
    }
    if (err != hipSuccess) {
        return (int)err;
    }
    const uint32_t blocks = (uint32_t)cus;
    const uint32_t iters = 8000;  // 2 waves per SIMD x 8000 x 32 x 16 cycles: a few milliseconds
    hipEvent_t e0, e1;
    if ((err = hipEventCreate(&e0)) != hipSuccess || (err = hipEventCreate(&e1)) != hipSuccess) {
        return (int)err;
    }
    float best = 0.0f;
    hipLaunchKernelGGL(mfma_i8_rate_kernel, dim3(blocks), dim3(512), 0, nullptr, iters / 8, zero_operands, (int *)nullptr);
    err = hipGetLastError();
    for (int r = 0; r < 3 && err == hipSuccess; ++r) {
        float ms = 0.0f;
        err = hipEventRecord(e0, nullptr);
        if (err == hipSuccess) {
            hipLaunchKernelGGL(mfma_i8_rate_kernel, dim3(blocks), dim3(512), 0, nullptr, iters, zero_operands, (int *)nullptr);
            err = hipGetLastError();
        }
        if (err == hipSuccess) {
            err = hipEventRecord(e1, nullptr);
        }
        if (err == hipSuccess) {
            err = hipEventSynchronize(e1);
        }
        if (err == hipSuccess) {
            err = hipEventElapsedTime(&ms, e0, e1);
        }
        if (err == hipSuccess && (best == 0.0f || ms < best)) {
            best = ms;
        }
    }
    (void)hipEventDestroy(e0);
    (void)hipEventDestroy(e1);
    if (err != hipSuccess) {
        return (int)err;
    }
    const double ops = (double)blocks * 8.0 * (double)iters * 32.0 * (2.0 * 16 * 16 * 64);
    *tops = (float)(ops / ((double)best * 1e-3) / 1e12);
    return 0;
}
