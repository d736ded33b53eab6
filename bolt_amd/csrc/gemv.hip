// Bandwidth-bound int8 GEMV for decode shapes:
//   y[n] = ob[n] + y_in[n] + sum_k W_s8[n][k] * x_u8[k]
// (Bolt: matrix_vector_multiply, compute/blas_enhance/src/mvm.cpp:132-194 and the AVX-512 path
// compute/blas_enhance/src/cpu/x86/int8/avx512/mvm_avx512_vnni.cpp:703-759.)
//
// gfx950 has signed x signed dot4 only, so the activation is re-biased in the load path
// (x ^ 0x80 = x - 128 as s8) and the missing 128 * sum_k W[n][k] is added back from the
// compensation vector the weight transform stored behind the packed matrix
// (comp[n] = -128 * sum_k W[n][k]):
//   sum_k W * x_u8 = sum_k W * (x ^ 0x80) - comp[n]
//
// One wave owns ROWS consecutive weight rows; every lane streams 16 contiguous bytes per row per
// 1 KiB slab of K (global_load_dwordx4, a full 1 KiB contiguous per wave instruction), feeds four
// v_dot4c_i32_i8 per load, and the ROWS partial sums are folded with a wave64 butterfly at the
// end. The activation slab is read once per wave and reused for all ROWS rows.
#include "device_common.h"
#include "kernels.h"

namespace bg {

typedef int v4i_a4 __attribute__((ext_vector_type(4), aligned(4)));
typedef int v2i_a4 __attribute__((ext_vector_type(2), aligned(4)));

// XV = 1: x is 4-byte aligned, full 16-byte slabs are read with one vector load.
template <int ROWS, int XV>
__global__ __launch_bounds__(256) void gemv_s8u8_kernel(const int8_t *__restrict__ W, uint32_t ldw,
    const uint8_t *__restrict__ x, uint32_t K, uint32_t N, const int32_t *__restrict__ ob,
    const int32_t *__restrict__ comp, void *__restrict__ y, uint32_t tail0, int add_yin, Epilogue epi,
    GemvBatch bt, const float *__restrict__ fold_bias, float fold_scale)
{
    // strided batch of independent products: slice b uses weight blob b % wcopies, its own
    // activation vector, result vector and (per-channel epilogue) input scale
    if (gridDim.y > 1 || bt.wcopies) {
        const uint32_t b = blockIdx.y;
        const size_t wo = (size_t)(bt.wcopies ? b % bt.wcopies : 0) * bt.wstride;
        W += wo;
        comp = (const int32_t *)((const char *)comp + wo);
        ob = (const int32_t *)((const char *)ob + (bt.ob_in_blob ? wo : 0));
        x += (size_t)b * bt.xstride;
        y = (char *)y + (size_t)b * bt.ystride;
        if (epi.scaleI) {
            epi.scaleI += b;
        }
    }
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint32_t n0 = wave * ROWS;
    if (n0 >= N) {
        return;
    }
    int acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        acc[r] = 0;
    }
    const uint32_t Kp = ldw;  // rows are zero-padded to a multiple of 8
    for (uint32_t kc = 0; kc < Kp; kc += 1024) {
        const uint32_t k = kc + lane * 16;
        v4i xs = {0, 0, 0, 0};
        if (k + 16 <= K && XV) {
            xs = *(const v4i_a4 *)(x + k);
        } else if (k < K) {
            uint32_t t[4] = {0, 0, 0, 0};
            for (uint32_t b = 0; b < 16 && k + b < K; ++b) {
                t[b >> 2] |= (uint32_t)x[k + b] << (8 * (b & 3));
            }
            xs = (v4i){(int)t[0], (int)t[1], (int)t[2], (int)t[3]};
        }
        xs ^= (v4i){(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
        v4i w[ROWS];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            w[r] = (v4i){0, 0, 0, 0};
            const uint32_t n = n0 + r;
            if (n < N) {
                const int8_t *p = W + (size_t)n * ldw + k;
                if (k + 16 <= Kp) {
                    // the weights stream through once: the non-temporal hint keeps them from being
                    // retained in L2 / Infinity Cache and is worth 12 % of read bandwidth on this part
                    w[r] = __builtin_nontemporal_load((const v4i_a4 *)p);
                } else if (k + 8 <= Kp) {
                    v2i_a4 h = *(const v2i_a4 *)p;
                    w[r] = (v4i){h.x, h.y, 0, 0};
                }
            }
        }
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            acc[r] = __builtin_amdgcn_sdot4(w[r].x, xs.x, acc[r], false);
            acc[r] = __builtin_amdgcn_sdot4(w[r].y, xs.y, acc[r], false);
            acc[r] = __builtin_amdgcn_sdot4(w[r].z, xs.z, acc[r], false);
            acc[r] = __builtin_amdgcn_sdot4(w[r].w, xs.w, acc[r], false);
        }
    }
    int mine = 0;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        int s = wave_reduce_add(acc[r]);
        if ((int)lane == r) {
            mine = s;
        }
    }
    const uint32_t n = n0 + lane;
    if (lane < ROWS && n < N) {
        const bool tail = (n >= tail0);
        // int32 two's-complement wrap, as vpdpbusd / vpaddd
        uint32_t a = (uint32_t)mine + column_base(ob, comp, fold_bias, fold_scale, n);
        if (add_yin && !tail && epi.mode != EPI_U8) {
            a += (uint32_t)((const int32_t *)y)[n];
        }
        const int ai = (int)a;
        switch (epi.mode) {
            case EPI_I32:
                ((int32_t *)y)[n] = ai;
                break;
            case EPI_F32:
                ((float *)y)[n] = (float)ai * epi_factor(epi);
                break;
            case EPI_U8:
                ((uint8_t *)y)[n] = (uint8_t)(tail ? epi_u8_trunc(ai, epi_factor(epi)) : epi_u8(ai, epi_factor(epi)));
                break;
            case EPI_F32_CH:
                ((float *)y)[n] = epi_f32_ch(ai, *epi.scaleI, epi.scaleW[n], epi.bias, n);
                break;
            default:
                break;
        }
    }
}

// u8 matrix x s8 vector (matmul's [M,K]x[K,1] route, mvm_avx512_vnni_row.cpp:931-1028):
//   y[m] = -128 * sum_k x[k] + sum_k A_u8[m][k] * x_s8[k]  =  sum_k (A ^ 0x80)_s8 * x_s8
// y is overwritten (the reference runs a single K block and never reloads y).
template <int ROWS>
__global__ __launch_bounds__(256) void gemv_u8s8_kernel(const uint8_t *__restrict__ A, uint32_t lda,
    uint32_t sk, const int8_t *__restrict__ x, uint32_t K, uint32_t M, void *__restrict__ y, Epilogue epi)
{
    // lda / sk: byte strides of A along m and k (sk == 1: row-major [M][K]; lda == 1: stored [K][M])
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    const uint32_t m0 = wave * ROWS;
    if (m0 >= M) {
        return;
    }
    int acc[ROWS];
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        acc[r] = 0;
    }
    for (uint32_t k = lane; k < K; k += 64) {
        const int xv = x[k];
#pragma unroll
        for (int r = 0; r < ROWS; ++r) {
            if (m0 + r < M) {
                const int a = (int)A[(size_t)(m0 + r) * lda + (size_t)k * sk] - 128;
                acc[r] += a * xv;
            }
        }
    }
    int mine = 0;
#pragma unroll
    for (int r = 0; r < ROWS; ++r) {
        int s = wave_reduce_add(acc[r]);
        if ((int)lane == r) {
            mine = s;
        }
    }
    const uint32_t m = m0 + lane;
    if (lane < ROWS && m < M) {
        switch (epi.mode) {
            case EPI_I32:
                ((int32_t *)y)[m] = mine;
                break;
            case EPI_F32:
                ((float *)y)[m] = (float)mine * epi_factor(epi);
                break;
            case EPI_U8:
                ((uint8_t *)y)[m] = (uint8_t)epi_u8(mine, epi_factor(epi));
                break;
            default:
                break;
        }
    }
}

template <int ROWS>
static hipError_t launch_s8u8(const GemvArgs &a, hipStream_t st)
{
    const uint32_t waves = (a.N + ROWS - 1) / ROWS;
    const uint32_t blocks = (waves + 3) / 4;
    const uint32_t tail0 = a.N - a.N % 8;
    const dim3 grid(blocks, a.batch.count ? a.batch.count : 1);
    const bool xv = (((uintptr_t)a.x | (uintptr_t)a.batch.xstride) & 3) == 0;
    if (xv) {
        hipLaunchKernelGGL((gemv_s8u8_kernel<ROWS, 1>), grid, dim3(256), 0, st, a.W, a.ldw, a.x, a.K, a.N, a.ob,
            a.comp, a.y, tail0, a.add_yin, a.epi, a.batch, a.fold_bias, a.fold_scale);
    } else {
        hipLaunchKernelGGL((gemv_s8u8_kernel<ROWS, 0>), grid, dim3(256), 0, st, a.W, a.ldw, a.x, a.K, a.N, a.ob,
            a.comp, a.y, tail0, a.add_yin, a.epi, a.batch, a.fold_bias, a.fold_scale);
    }
    return hipGetLastError();
}

hipError_t launch_gemv_s8u8(const GemvArgs &a, hipStream_t st)
{
    if (a.N == 0) {
        return hipSuccess;
    }
    // enough waves to cover 256 CUs several times over before widening the per-wave row block
    if (a.N >= 16384) {
        return launch_s8u8<4>(a, st);
    }
    if (a.N >= 2048) {
        return launch_s8u8<2>(a, st);
    }
    return launch_s8u8<1>(a, st);
}

__device__ __forceinline__ void gemv_u8s8_store(void *y, uint32_t m, int acc, const Epilogue &epi)
{
    switch (epi.mode) {
        case EPI_I32:
            ((int32_t *)y)[m] = acc;
            break;
        case EPI_F32:
            ((float *)y)[m] = (float)acc * epi_factor(epi);
            break;
        case EPI_U8:
            ((uint8_t *)y)[m] = (uint8_t)epi_u8(acc, epi_factor(epi));
            break;
        default:
            break;
    }
}

// Row-major u8 matrix [M][lda], rows and x 16-byte aligned: one wave per row, 16 bytes per lane and
// step, (a ^ 0x80) as s8 against x with v_dot4; the K tail (K % 16) byte by byte.
__global__ __launch_bounds__(256) void gemv_u8s8_rows_kernel(const uint8_t *__restrict__ A, uint32_t lda,
    const int8_t *__restrict__ x, uint32_t K, uint32_t M, void *__restrict__ y, Epilogue epi)
{
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t m = (blockIdx.x * blockDim.x + threadIdx.x) >> 6;
    if (m >= M) {
        return;
    }
    const uint8_t *row = A + (size_t)m * lda;
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
    int acc = 0;
    const uint32_t K16 = K & ~15u;
    for (uint32_t k = lane * 16; k < K16; k += 1024) {
        v4i a = __builtin_nontemporal_load((const v4i *)(row + k));
        const v4i xv = *(const v4i *)(x + k);
        a ^= flip;
        acc = __builtin_amdgcn_sdot4(a.x, xv.x, acc, false);
        acc = __builtin_amdgcn_sdot4(a.y, xv.y, acc, false);
        acc = __builtin_amdgcn_sdot4(a.z, xv.z, acc, false);
        acc = __builtin_amdgcn_sdot4(a.w, xv.w, acc, false);
    }
    if (K16 + lane < K) {
        acc += ((int)row[K16 + lane] - 128) * (int)x[K16 + lane];
    }
    acc = wave_reduce_add(acc);
    if (lane == 0) {
        gemv_u8s8_store(y, m, acc, epi);
    }
}

// u8 matrix stored [K][ldk] (row k holds all M results' coefficients), 4-byte aligned rows: one lane
// per 4 consecutive results, a dword per lane and k (256 contiguous bytes per wave), x[k] is wave-uniform.
// The K range is split over the 4 waves of a block and the partial sums meet in LDS.
__global__ __launch_bounds__(256) void gemv_u8s8_cols_kernel(const uint8_t *__restrict__ A, uint32_t ldk,
    const int8_t *__restrict__ x, uint32_t K, uint32_t M, void *__restrict__ y, Epilogue epi)
{
    __shared__ int part[4][64][4];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t m = (blockIdx.x * 64 + lane) * 4;
    int acc[4] = {0, 0, 0, 0};
    if (m < M) {
        const uint32_t kper = (K + 3) / 4, k0 = wave * kper, k1 = (k0 + kper < K) ? k0 + kper : K;
        const bool full = m + 4 <= M;
        for (uint32_t k = k0; k < k1; ++k) {
            const uint8_t *p = A + (size_t)k * ldk + m;
            uint32_t w;
            if (full) {
                w = *(const uint32_t *)p;
            } else {
                w = 0x80808080u;  // (0x80 - 128) = 0 for the results past M
                for (uint32_t j = 0; m + j < M; ++j) {
                    w = (w & ~(0xffu << (8 * j))) | ((uint32_t)p[j] << (8 * j));
                }
            }
            const int xv = x[k];
#pragma unroll
            for (int j = 0; j < 4; ++j) {
                acc[j] += ((int)((w >> (8 * j)) & 0xff) - 128) * xv;
            }
        }
    }
#pragma unroll
    for (int j = 0; j < 4; ++j) {
        part[wave][lane][j] = acc[j];
    }
    __syncthreads();
    if (wave == 0 && m < M) {
#pragma unroll
        for (int j = 0; j < 4; ++j) {
            if (m + j < M) {
                gemv_u8s8_store(y, m + j, part[0][lane][j] + part[1][lane][j] + part[2][lane][j] + part[3][lane][j], epi);
            }
        }
    }
}

hipError_t launch_gemv_u8s8(const uint8_t *A, uint32_t lda, uint32_t sk, const int8_t *x, uint32_t K, uint32_t M,
    void *y, const Epilogue &epi, hipStream_t st)
{
    if (M == 0) {
        return hipSuccess;
    }
    if (sk == 1 && K >= 16 && (lda & 15) == 0 && ((((uintptr_t)A | (uintptr_t)x) & 15) == 0)) {
        hipLaunchKernelGGL(gemv_u8s8_rows_kernel, dim3((M + 3) / 4), dim3(256), 0, st, A, lda, x, K, M, y, epi);
        return hipGetLastError();
    }
    if (lda == 1 && M >= 4 && (sk & 3) == 0 && (((uintptr_t)A & 3) == 0)) {
        hipLaunchKernelGGL(gemv_u8s8_cols_kernel, dim3((M + 255) / 256), dim3(256), 0, st, A, sk, x, K, M, y, epi);
        return hipGetLastError();
    }
    const uint32_t blocks = (M + 3) / 4;
    hipLaunchKernelGGL((gemv_u8s8_kernel<1>), dim3(blocks), dim3(256), 0, st, A, lda, sk, x, K, M, y, epi);
    return hipGetLastError();
}

}  // namespace bg
