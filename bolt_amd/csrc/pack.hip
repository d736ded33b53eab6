// Load-time weight transforms (device side): re-order an s8 matrix given with arbitrary element
// strides into the packed layouts described in layout.h and compute the u8-offset compensation
// comp[n] = -128 * sum_k W[k][n] (Bolt: mmm_avx512_vnni.cpp:60-121, mvm_avx512_vnni.cpp:28-131).
#include "device_common.h"
#include "kernels.h"
#include "layout.h"

namespace bg {

// One thread per 8 packed bytes (8 consecutive k of one column); both layouts keep those contiguous.
template <int MMM>
__global__ __launch_bounds__(256) void pack_kernel(const int8_t *__restrict__ src, uint32_t sk, uint32_t sn,
    uint32_t K, uint32_t N, uint32_t Kp, uint32_t N16, int8_t *__restrict__ dst)
{
    const uint32_t k8 = Kp / 8;
    const uint64_t id = (uint64_t)blockIdx.x * blockDim.x + threadIdx.x;
    if (id >= (uint64_t)N16 * k8) {
        return;
    }
    const uint32_t n = (uint32_t)(id / k8);
    const uint32_t k0 = (uint32_t)(id % k8) * 8;
    uint32_t lo = 0, hi = 0;
    if (n < N) {
        for (uint32_t b = 0; b < 8 && k0 + b < K; ++b) {
            uint32_t v = (uint8_t)src[(size_t)(k0 + b) * sk + (size_t)n * sn];
            if (b < 4) {
                lo |= v << (8 * b);
            } else {
                hi |= v << (8 * (b - 4));
            }
        }
    }
    const size_t off = MMM ? mmm_packed_offset(n, k0, Kp) : mvm_packed_offset(n, k0, Kp);
    *(v2i *)(dst + off) = (v2i){(int)lo, (int)hi};
}

// one wave per output column
__global__ __launch_bounds__(256) void comp_kernel(const int8_t *__restrict__ src, uint32_t sk, uint32_t sn, uint32_t K,
    uint32_t N, int32_t *__restrict__ comp)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t n = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (n >= N) {
        return;
    }
    int s = 0;
    for (uint32_t k = lane; k < K; k += 64) {
        s += (int)src[(size_t)k * sk + (size_t)n * sn];
    }
    s = wave_reduce_add(s);
    if (lane == 0) {
        comp[n] = s * (-128);
    }
}

template <int MMM>
static hipError_t launch_pack(const int8_t *src, uint32_t sk, uint32_t sn, uint32_t K, uint32_t N, int8_t *dst,
    int32_t *comp, hipStream_t st)
{
    if (N == 0) {
        return hipSuccess;
    }
    if (K == 0) {
        return launch_fill_u32((uint32_t *)comp, N, 0, st);  // an empty sum: the compensation is zero
    }
    const uint32_t Kp = align_up(K, 8), N16 = align_up(N, 16);
    const uint64_t threads = (uint64_t)N16 * (Kp / 8);
    hipLaunchKernelGGL((pack_kernel<MMM>), dim3((uint32_t)((threads + 255) / 256)), dim3(256), 0, st, src, sk, sn, K,
        N, Kp, N16, dst);
    hipLaunchKernelGGL(comp_kernel, dim3((N + 3) / 4), dim3(256), 0, st, src, sk, sn, K, N, comp);
    return hipGetLastError();
}

hipError_t launch_pack_mmm(const int8_t *src, uint32_t sk, uint32_t sn, uint32_t K, uint32_t N, int8_t *dst,
    int32_t *comp, hipStream_t st)
{
    return launch_pack<1>(src, sk, sn, K, N, dst, comp, st);
}

hipError_t launch_pack_mvm(const int8_t *src, uint32_t sk, uint32_t sn, uint32_t K, uint32_t N, int8_t *dst,
    int32_t *comp, hipStream_t st)
{
    return launch_pack<0>(src, sk, sn, K, N, dst, comp, st);
}

}  // namespace bg
