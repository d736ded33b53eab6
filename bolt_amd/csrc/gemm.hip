// int8 GEMM on the gfx950 matrix cores:
//   C[m][n] = ob[n] + C_in[m][n] + sum_k A_u8[m][k] * B_s8[k][n]      (int32, wraps)
// (Bolt: matrix_matrix_multiply, compute/blas_enhance/src/mmm.cpp:150-238 and
// compute/blas_enhance/src/cpu/x86/int8/avx512/mmm_avx512_vnni.cpp:1760-1891.)
//
// V_MFMA_I32_16X16X64_I8 multiplies signed by signed, so A is re-biased on its way in
// (a ^ 0x80 = a - 128 as s8; padding therefore reads as 0) and the missing 128 * sum_k B[k][n]
// comes back from the compensation vector stored behind the packed matrix:
//   sum_k a_u8 * b = sum_k (a ^ 0x80) * b - comp[n],   comp[n] = -128 * sum_k b[k][n].
//
// Operand mapping of the 16x16x64 instruction as used here: lane l supplies row (A) / column (B)
// l % 16 and the 16 K-bytes of K-group l / 16; the result lane l holds column l % 16, rows
// 4 * (l / 16) + {0,1,2,3}. Any K-permutation applied to A and B alike leaves the sum unchanged,
// so only the lane <-> row/column association matters; the packed B layout (layout.h) hands every
// lane its 16 bytes with one 128-bit load.
#include "device_common.h"
#include "kernels.h"
#include "layout.h"

namespace bg {

typedef int v4i_a1 __attribute__((ext_vector_type(4), aligned(1)));

__device__ __forceinline__ void store_tile(const GemmArgs &a, const v4i &acc, uint32_t m0, uint32_t n, uint32_t g)
{
    if (n >= a.N) {
        return;
    }
    const uint32_t base = (uint32_t)a.ob[n] - (uint32_t)a.comp[n];
    float factor = 0.0f, sI = 0.0f, sW = 0.0f;
    if (a.epi.mode == EPI_F32 || a.epi.mode == EPI_U8) {
        factor = epi_factor(a.epi);
    } else if (a.epi.mode == EPI_F32_CH) {
        sI = *a.epi.scaleI;
        sW = a.epi.scaleW[n];
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t m = m0 + 4 * g + r;
        if (m >= a.M) {
            continue;
        }
        const size_t idx = (size_t)m * a.N + n;
        uint32_t v = (uint32_t)acc[r] + base;
        if (a.add_cin && a.epi.mode != EPI_U8) {
            v += (uint32_t)((const int32_t *)a.C)[idx];
        }
        const int vi = (int)v;
        switch (a.epi.mode) {
            case EPI_I32:
                ((int32_t *)a.C)[idx] = vi;
                break;
            case EPI_F32:
                ((float *)a.C)[idx] = (float)vi * factor;
                break;
            case EPI_U8:
                ((uint8_t *)a.C)[idx] = (uint8_t)epi_u8(vi, factor);
                break;
            case EPI_F32_CH:
                ((float *)a.C)[idx] = epi_f32_ch(vi, sI, sW, a.epi.bias, n);
                break;
            default:
                break;
        }
    }
}

// General kernel: any M, N, K, either A orientation, no alignment assumptions. One wave owns a
// 16 x 64 strip of C (four MFMA tiles sharing the A fragment); operands go straight from global
// memory / L2 to registers.
__global__ __launch_bounds__(256) void gemm_u8s8_general_kernel(GemmArgs a)
{
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t m0 = blockIdx.y * 64 + wave * 16;
    const uint32_t n0 = blockIdx.x * 64;
    if (m0 >= a.M) {
        return;
    }
    const uint32_t Kp = align_up(a.K, 8);
    const uint32_t kfull = Kp >> 4;
    const uint32_t nblocks = align_up(a.N, 16) >> 4;
    const uint32_t m = m0 + i;
    v4i acc[4];
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        acc[t] = (v4i){0, 0, 0, 0};
    }
    for (uint32_t k0 = 0; k0 < Kp; k0 += 64) {
        const uint32_t k = k0 + 16 * g;
        v4i af = {0, 0, 0, 0};
        if (m < a.M && k < a.K) {
            if (!a.transA && k + 16 <= a.K) {
                af = *(const v4i_a1 *)(a.A + (size_t)m * a.lda + k);
                af ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
            } else {
                uint32_t t4[4] = {0, 0, 0, 0};
                for (uint32_t b = 0; b < 16 && k + b < a.K; ++b) {
                    const uint32_t v = a.transA ? a.A[(size_t)(k + b) * a.lda + m] : a.A[(size_t)m * a.lda + k + b];
                    t4[b >> 2] |= (v ^ 0x80u) << (8 * (b & 3));
                }
                af = (v4i){(int)t4[0], (int)t4[1], (int)t4[2], (int)t4[3]};
            }
        }
        const uint32_t kb = k >> 4;
#pragma unroll
        for (int t = 0; t < 4; ++t) {
            const uint32_t nb = (n0 >> 4) + t;
            v4i bf = {0, 0, 0, 0};
            if (nb < nblocks) {
                const int8_t *p = a.Bp + (size_t)nb * 16 * Kp;
                if (kb < kfull) {
                    bf = *(const v4i *)(p + (size_t)kb * 256 + i * 16);
                } else if (kb == kfull && (Kp & 15)) {
                    v2i h = *(const v2i *)(p + (size_t)kfull * 256 + i * 8);
                    bf = (v4i){h.x, h.y, 0, 0};
                }
            }
            acc[t] = __builtin_amdgcn_mfma_i32_16x16x64_i8(af, bf, acc[t], 0, 0, 0);
        }
    }
#pragma unroll
    for (int t = 0; t < 4; ++t) {
        store_tile(a, acc[t], m0, n0 + 16 * t + i, g);
    }
}

hipError_t launch_gemm_u8s8(const GemmArgs &a, hipStream_t st)
{
    if (a.M == 0 || a.N == 0) {
        return hipSuccess;
    }
    dim3 grid((a.N + 63) / 64, (a.M + 63) / 64);
    hipLaunchKernelGGL(gemm_u8s8_general_kernel, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace bg
