// Byte layouts of the pre-packed weight blobs, shared by host and device code.
//
// matrix_matrix_multiply right-hand side (tagged DF_NKNxKx), "MFMA-fragment" order:
//   Kp = ALIGN(K, 8), N16 = ALIGN(N, 16); the matrix part is exactly N16 * Kp bytes, the size
//   Bolt's transform_rhs_bytes query grants (mmm_avx512_vnni.cpp:22-40).
//   For each block of 16 output columns (16 * Kp bytes):
//     Kp / 16 fragments of 256 bytes  [n 0..15][k 0..15]   -- lane (n, g) of a 16x16x64 MFMA reads
//                                                             its 16 K-bytes with one 128-bit load and
//                                                             a wave reads 1 KiB contiguous per K tile
//     + one 128-byte fragment [n 0..15][k 0..7] when Kp % 16 == 8
//   Rows n >= N and bytes k >= K are zero.
//   The compensation vector comp[n] = -128 * sum_k B[k][n] (int32) follows at byte N16 * Kp.
//
// matrix_vector_multiply weight (tagged DF_NKN32K4): row-major [N16][Kp], zero padded, then comp[N]
// at byte N16 * Kp (mvm_avx512_vnni.cpp:42-47 places it there as well).
#pragma once
#include <stdint.h>
#ifndef BG_HD
#ifdef __HIPCC__
#define BG_HD __host__ __device__
#else
#define BG_HD
#endif
#endif

namespace bg {

BG_HD inline uint32_t align_up(uint32_t x, uint32_t a)
{
    return (x + a - 1) / a * a;
}

BG_HD inline size_t mmm_packed_offset(uint32_t n, uint32_t k, uint32_t Kp)
{
    const uint32_t nb = n >> 4, j = n & 15, kb = k >> 4, kk = k & 15;
    const size_t base = (size_t)nb * 16 * Kp;
    if (kb < (Kp >> 4)) {
        return base + (size_t)kb * 256 + j * 16 + kk;
    }
    return base + (size_t)(Kp >> 4) * 256 + j * 8 + kk;  // 8-wide tail fragment, kk < 8
}

BG_HD inline size_t mvm_packed_offset(uint32_t n, uint32_t k, uint32_t Kp)
{
    return (size_t)n * Kp + k;
}

}  // namespace bg
