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
#include <type_traits>
#include "kernels.h"
#include "layout.h"

namespace bg {

typedef int v4i_a1 __attribute__((ext_vector_type(4), aligned(1)));

__device__ __forceinline__ void store_tile(const GemmArgs &a, const v4i &acc, uint32_t m0, uint32_t n, uint32_t g)
{
    if (n >= a.N) {
        return;
    }
    const uint32_t base = column_base(a.ob, a.comp, a.fold_bias, a.fold_scale, n);
    float factor = 0.0f, sI = 0.0f, sW = 0.0f;
    if (a.epi.mode == EPI_F32 || a.epi.mode == EPI_U8) {
        factor = epi_factor(a.epi);
    } else if (a.epi.mode == EPI_F32_CH || a.epi.mode == EPI_U8_CH) {
        sI = *a.epi.scaleI;
        sW = a.epi.scaleW[n];
        factor = a.epi.factor;
    }
#pragma unroll
    for (int r = 0; r < 4; ++r) {
        const uint32_t m = m0 + 4 * g + r;
        if (m >= a.M) {
            continue;
        }
        const size_t idx = (size_t)m * a.N + n;
        uint32_t v = (uint32_t)acc[r] + base;
        if (a.add_cin && a.epi.mode != EPI_U8 && a.epi.mode != EPI_U8_CH) {
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
            case EPI_U8_CH:
                ((uint8_t *)a.C)[idx] = (uint8_t)q_u8(epi_f32_ch(vi, sI, sW, a.epi.bias, n), factor);
                break;
            default:
                break;
        }
    }
}

// General kernel: any M, N, K, either A orientation, no alignment assumptions. One wave owns a
// 16 x 64 strip of C (four MFMA tiles sharing the A fragment); operands go straight from global
// memory / L2 to registers.
__global__ __launch_bounds__(256, 2) void gemm_u8s8_general_kernel(GemmArgs a)
{
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t m0 = blockIdx.x * 64 + wave * 16;  // rows along x: a grid's x extent has room for any row count
    const uint32_t n0 = blockIdx.y * 64;
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

// Tiled kernel for K % 16 == 0, row-major A with 16-byte aligned rows.
//
// Block = 4 waves (WM x WN), block tile (WM*TM*16) x (WN*TN*16), K step 128 (two 64-wide MFMA
// K tiles). Both operands are staged in LDS in MFMA-fragment order: one fragment = the 1 KiB that
// the 64 lanes of a 16x16x64 MFMA consume, lane l at byte 16*l, so every fragment read is one
// conflict-free ds_read_b128 per lane. B fragments are a straight copy of the packed global
// layout; A fragments are gathered with the same lane pattern (lane (i, g) reads 16 bytes of row
// i at K offset 16*g) and re-biased (^ 0x80) on the way through registers. Two LDS stages: the
// global loads of K step t+1 are issued before the MFMAs of step t and parked in registers.
template <int WM, int WN, int TM, int TN>
struct GemmTile {
    static constexpr int kBM = WM * TM * 16;
    static constexpr int kBN = WN * TN * 16;
    static constexpr int kBK = 128;
    static constexpr int kAFrags = (kBM / 16) * 2;   // per stage
    static constexpr int kBFrags = (kBN / 16) * 2;
    static constexpr int kWaves = WM * WN;
    static constexpr int kALoads = kAFrags / kWaves;  // fragments loaded per wave
    static constexpr int kBLoads = kBFrags / kWaves;
    static constexpr int kStageBytes = (kAFrags + kBFrags) * 1024;
    static constexpr int kLdsBytes = 2 * kStageBytes;
};

// Epilogue straight from the accumulators. The tiled kernels feed the matrix instruction with the
// operands swapped (B fragment first), so a tile's accumulator is the TRANSPOSE of the usual layout:
// lane (i = lane % 16, g = lane / 16) holds C[row i][cols 4g .. 4g+3] of its 16 x 16 tile, four
// consecutive columns of one row. Every result store and C_in load is then one 16-byte access per
// lane with no pass through LDS; a wave covers 16 rows x 64 bytes per access for a matrix, and for
// a convolution (NCHWC16: a pixel's 16 channels are contiguous, consecutive pixels follow each
// other) one contiguous KiB. The per-column terms (offsetC - compensation, reciprocal channel
// scale, bias) depend only on the lane and the tile column and are set up once.
// FULL: the block tile lies wholly inside C and rows of C are 16-byte granular, so no bounds test, no
// scalar tail and -- what matters -- no control flow: the compiler can then count outstanding memory
// operations exactly instead of draining them (s_waitcnt vmcnt(0)) between row blocks, which would
// serialise every wave on the round trip of its own stores. CIN: 0 = C is not read, 1 = it is,
// 2 = decided at run time (edge tiles).
// 16-byte result store. STREAM: a large matrix result is written once and not read again by this
// kernel; stored normally, every round of tiles leaves 8 MiB of dirty lines per XCD in a 4 MiB L2 and
// pushes out the A and B panels the next tiles of that XCD were sharing (measured: the K loop after
// the first round of tiles runs 10-15 % slower). The non-temporal hint keeps the result out of the way.
template <bool STREAM, typename V>
__device__ __forceinline__ void store_c16(V *p, V v)
{
    if (STREAM) {
        __builtin_nontemporal_store(v, p);
    } else {
        *p = v;
    }
}

// Per-column terms a kernel formed ahead of its K loop and parked in its LDS, one entry per column of the block tile
// (the filter-panel convolution: 64 columns): the epilogue reads its 16 entries from there instead of loading the
// vectors from memory and repeating the arithmetic in every lane. Handed over BY VALUE (a pointer to a struct is kept in
// scratch memory by the compiler). base: offset - compensation with the bias folded in (column_base); qs / bs: the
// per-channel form's reciprocal scale 1.0f / (sI * sW[n]) and bias (0 without one). Null: nothing was formed.
struct ColTerms {
    const uint32_t *base = nullptr;
    const float *qs = nullptr;
    const float *bs = nullptr;
};

// SYNC: the kernel's launches may carry a grid-wide agreement (GemmArgs::sync; the filter-panel convolution only) -- the
// code for it, the parking of values when it is abandoned included, is left out of every other kernel
template <int MODE, bool CONV, int WM, int WN, int TM, int TN, bool FULL, int CIN, bool SYNC = false>
__device__ __forceinline__ void epilogue_rows(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0, const ColTerms pre_base = ColTerms())
{
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const bool use_cin = (CIN == 2) ? (!CONV && a.add_cin && MODE != EPI_U8 && MODE != EPI_U8_CH) : (CIN == 1);
    const bool n_vec = FULL || CONV || ((a.N & 3) == 0);
    int lane_max = 0;

    float factor = 0.0f, sI = 0.0f;
    if (CONV && MODE == EPI_U8) {
        // tensor-wide dynamic requantisation (avx512/quantize.cpp:364-416 after the abs-max of :70-119)
        int mx = 0;
        if (!(SYNC && a.sync.slots)) {
            mx = ws_read_max(a.conv.absmax);
        }
        factor = (mx == 0) ? 1.0f : 127.0f / (float)mx;
        if (blockIdx.x == 0 && threadIdx.x == 0 && a.conv.dscale_out && !(SYNC && a.sync.slots)) {
            *a.conv.dscale_out = conv_acc_scale(a.conv) * factor;
        }
    } else if (MODE == EPI_F32 || MODE == EPI_U8) {
        factor = (CONV && a.conv.dscaleI) ? 1.0f / conv_acc_scale(a.conv) : epi_factor(a.epi);
    } else if (MODE == EPI_F32_CH || MODE == EPI_U8_CH) {
        sI = CONV ? 1.0f : *a.epi.scaleI;
        factor = a.epi.factor;  // EPI_U8_CH: the output scale
    }
    const float fold_scale = (CONV && a.conv.dscaleI) ? conv_acc_scale(a.conv) : a.fold_scale;

    uint32_t base[TN][4];
    float qs[TN][4], bs[TN][4];
    uint32_t cblk_off[TN], cblk_w[TN];
    {
        // every per-column term in one batch of loads, none behind a branch (a load per use would put a trip to memory
        // into each column); columns past N read column N - 1 and are dropped. pre_base: the caller formed the
        // offsets ahead of its K loop, while it was waiting for memory anyway.
        uint32_t nn[TN * 4], flat[TN * 4];
        float sw[TN * 4], bi[TN * 4];
        constexpr bool kCh = (MODE == EPI_F32_CH || MODE == EPI_U8_CH);
        const float *swp = kCh ? a.epi.scaleW : (const float *)a.comp;
        const float *bip = (kCh && a.epi.bias) ? a.epi.bias : (const float *)a.comp;
#pragma unroll
        for (int y = 0; y < TN; ++y) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g + c;
                nn[y * 4 + c] = (FULL || n < a.N) ? n : a.N - 1;
                sw[y * 4 + c] = swp[nn[y * 4 + c]];
                bi[y * 4 + c] = bip[nn[y * 4 + c]];
            }
        }
        if (!pre_base.base) {
            column_bases<TN * 4>(a.ob, a.comp, a.fold_bias, fold_scale, nn, flat);
        }
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const bool ok = FULL || (n + c < a.N);
                base[y][c] = pre_base.base ? pre_base.base[(wn * TN + y) * 16 + 4 * g + c] : (ok ? flat[y * 4 + c] : 0u);
                qs[y][c] = 1.0f;
                bs[y][c] = 0.0f;
                if ((MODE == EPI_F32_CH || MODE == EPI_U8_CH) && ok) {
                    if (CONV) {
                        // 1-bit convolution on the matrix cores: fma(S, scale[oc], bias[oc]), scale used as it is
                        qs[y][c] = sw[y * 4 + c];
                        bs[y][c] = bi[y * 4 + c];
                    } else {
                        qs[y][c] = 1.0f / (sI * sw[y * 4 + c]);
                        bs[y][c] = a.epi.bias ? bi[y * 4 + c] : 0.0f;
                    }
                }
            }
            cblk_off[y] = 0;
            cblk_w[y] = 1;
            if (CONV) {
                // output blocks of out_c channels per pixel (a trailing block may be narrower); 4 channels
                // starting at a multiple of 4 never straddle a block
                const uint32_t xc = a.conv.out_c, blk = n / xc;
                cblk_w[y] = (a.N - blk * xc < xc) ? a.N - blk * xc : xc;
                cblk_off[y] = blk * xc * a.conv.OHW + (n % xc);
            }
        }
    }

    if (SYNC && CONV && MODE == EPI_U8 && a.sync.slots) {
        // one pass: the maximum is agreed on by all workgroups of the launch while the accumulators are still in
        // registers (smem: 18 ints of LDS that no wave of the workgroup is still reading tiles from)
        // The column terms and the ReLU go into the accumulators in place, and the terms are zeroed for the code
        // behind: held beside the accumulators across the exchange, the sums cost 64 more registers than there are.
        int lm = 0;
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
#pragma unroll
                for (int x = 0; x < TM; ++x) {
                    int t = (int)((uint32_t)acc[x][y][c] + base[y][c]);
                    t = (a.conv.relu && t < 0) ? 0 : t;
                    acc[x][y][c] = t;
                    const int av = (t == (int)0x80000000) ? t : (t < 0 ? -t : t);
                    lm = (n + c < a.N && m0 + (wm * TM + x) * 16 + i < a.M && av > lm) ? av : lm;
                }
                base[y][c] = 0u;
            }
        }
        const uint32_t outcome = grid_max_sync(a.sync, lm, (int *)smem);
        if (outcome == kGridAbandoned && !a.C32) {  // nothing is stored; the host sees a NaN scale and runs the two passes
            if (blockIdx.x == 0 && threadIdx.x == 0 && a.conv.dscale_out) {
                *a.conv.dscale_out = __int_as_float(0x7fc00000);
            }
            return;
        }
        if (outcome == kGridAbandoned) {
            // Asynchronous form: no host is waiting, and no workgroup may wait for another any more. Every workgroup
            // parks its int32 values (bias folded, ReLU applied) in C32 -- laid out like the result -- and folds its
            // maximum into the scratch slots; the last one to arrive requantises the whole tensor alone. Slow, and
            // only reached when other work held the CUs.
#pragma unroll
            for (int x = 0; x < TM; ++x) {
                const uint32_t m = m0 + (wm * TM + x) * 16 + i;
                if (m >= a.M) {
                    continue;
                }
                const uint32_t img = m / a.conv.OHW, pix = m - img * a.conv.OHW;
#pragma unroll
                for (int y = 0; y < TN; ++y) {
                    const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
                    if (n >= a.N) {
                        continue;
                    }
                    v4i t;
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        const int v = (int)((uint32_t)acc[x][y][c] + base[y][c]);
                        t[c] = (a.conv.relu && v < 0) ? 0 : v;
                    }
                    *(v4i *)((int32_t *)a.C32 + (size_t)img * a.N * a.conv.OHW + cblk_off[y] + (size_t)pix * cblk_w[y]) = t;
                }
            }
            lm = wave_reduce_max_i(lm);
            if (lane == 0) {
                ws_fold_max(a.conv.absmax, blockIdx.x * 8 + wave, lm);
            }
            if (grid_last_arrival(a.sync, (int *)smem)) {
                const int mx = ws_read_max(a.conv.absmax);
                const float fct = (mx == 0) ? 1.0f : 127.0f / (float)mx;
                if (threadIdx.x == 0 && a.conv.dscale_out) {
                    *a.conv.dscale_out = conv_acc_scale(a.conv) * fct;
                }
                const uint32_t total4 = (a.M * a.N) / 4;  // N is a multiple of 8
                for (uint32_t k = threadIdx.x; k < total4; k += blockDim.x) {
                    const v4i t = ((const v4i *)a.C32)[k];
                    unsigned b[4];
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        b[c] = usat8_u(rne_i32((float)t[c] * fct + 128.0f));
                    }
                    ((uint32_t *)a.C)[k] = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                }
                __syncthreads();  // every wave has read the maximum
                for (uint32_t k = threadIdx.x; k < kWsWords; k += blockDim.x) {
                    a.conv.absmax[k] = 0;  // the slots go back clear
                }
            }
            return;
        }
        factor = ((int)outcome == 0) ? 1.0f : 127.0f / (float)(int)outcome;
        if (blockIdx.x == 0 && threadIdx.x == 0 && a.conv.dscale_out) {
            *a.conv.dscale_out = conv_acc_scale(a.conv) * factor;
        }
    }

    v4i cin[2][TN];
#define BG_LOAD_CIN(xx, buf)                                                              \
    if (use_cin) {                                                                        \
        const uint32_t m_ = m0 + (wm * TM + (xx)) * 16 + i;                               \
        _Pragma("unroll") for (int y = 0; y < TN; ++y)                                    \
        {                                                                                 \
            const uint32_t n_ = n0 + (wn * TN + y) * 16 + 4 * g;                          \
            cin[buf][y] = (v4i){0, 0, 0, 0};                                              \
            if (FULL || (m_ < a.M && n_ < a.N)) {                                         \
                const int32_t *p_ = (const int32_t *)a.C + (size_t)m_ * a.N + n_;         \
                if (FULL || (n_vec && n_ + 4 <= a.N)) {                                   \
                    cin[buf][y] = *(const v4i *)p_;                                       \
                } else {                                                                  \
                    for (int c = 0; c < 4 && n_ + c < a.N; ++c) {                         \
                        cin[buf][y][c] = p_[c];                                           \
                    }                                                                     \
                }                                                                         \
            }                                                                             \
        }                                                                                 \
    }
    BG_LOAD_CIN(0, 0);
#pragma unroll
    for (int x = 0; x < TM; ++x) {
        if (x + 1 < TM) {
            BG_LOAD_CIN(x + 1, (x + 1) & 1);  // the next row block's C_in is in flight while this one is stored
        }
        const uint32_t m = m0 + (wm * TM + x) * 16 + i;
        if (!FULL && m >= a.M) {
            continue;
        }
        size_t rowbase = (size_t)m * a.N;
        uint32_t pix = 0;
        if (CONV) {
            const uint32_t img = m / a.conv.OHW;
            pix = m - img * a.conv.OHW;
            rowbase = (size_t)img * a.N * a.conv.OHW;
        }
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
            if (!FULL && n >= a.N) {
                continue;
            }
            const bool vec = FULL || (n_vec && (n + 4 <= a.N));
            int t[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                t[c] = (int)((uint32_t)acc[x][y][c] + base[y][c] + (use_cin ? (uint32_t)cin[x & 1][y][c] : 0u));  // int32 wrap
            }
            size_t idx = rowbase + n;
            if (CONV) {
                idx = rowbase + cblk_off[y] + (size_t)pix * cblk_w[y];
                if ((MODE == EPI_I32 || MODE == EPI_U8) && a.conv.relu) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        t[c] = t[c] < 0 ? 0 : t[c];  // integer ReLU (convolution_direct.cpp:2406)
                    }
                }
                if (MODE == EPI_I32) {
#pragma unroll
                    for (int c = 0; c < 4; ++c) {
                        if (FULL || n + c < a.N) {
                            const int av = (t[c] == (int)0x80000000) ? t[c] : (t[c] < 0 ? -t[c] : t[c]);
                            lane_max = av > lane_max ? av : lane_max;
                        }
                    }
                }
            }
            if (MODE == EPI_I32) {
                if (CONV && !a.C) {
                    // abs-max pass only
                } else if (vec) {
                    store_c16<false>((v4i *)((int32_t *)a.C + idx), (v4i){t[0], t[1], t[2], t[3]});
                } else {
                    for (int c = 0; c < 4 && n + c < a.N; ++c) {
                        ((int32_t *)a.C)[idx + c] = t[c];
                    }
                }
            } else if (MODE == EPI_U8 || MODE == EPI_U8_CH) {
                unsigned b[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (MODE == EPI_U8_CH) {
                        float f = (float)t[c] * qs[y][c];
                        if (a.epi.bias) {
                            f = f + bs[y][c];
                        }
                        b[c] = q_u8(f, factor);
                    } else {
                        // stand-alone requantisation adds 128.0f before rounding, the GEMM's own u8 mode after
                        b[c] = CONV ? usat8_u(rne_i32((float)t[c] * factor + 128.0f)) : epi_u8(t[c], factor);
                    }
                }
                if (vec) {
                    *(uint32_t *)((uint8_t *)a.C + idx) = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
                } else {
                    for (int c = 0; c < 4 && n + c < a.N; ++c) {
                        ((uint8_t *)a.C)[idx + c] = (uint8_t)b[c];
                    }
                }
            } else {
                float f[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (MODE == EPI_F32) {
                        f[c] = (float)t[c] * factor;
                        if (CONV) {  // cvt * (1/s), + eltwise, fp32 ReLU (convolution_direct.cpp:2410-2422)
                            if (a.conv.eltwise && (FULL || n + c < a.N)) {
                                f[c] = f[c] + a.conv.eltwise[idx + c];
                            }
                            if (a.conv.relu && !(f[c] > 0.0f)) {
                                f[c] = 0.0f;
                            }
                        }
                    } else if (CONV) {
                        f[c] = __builtin_fmaf((float)t[c], qs[y][c], bs[y][c]);  // vfmaq in the reference's 1-bit kernels
                    } else {
                        f[c] = (float)t[c] * qs[y][c];
                        if (a.epi.bias) {
                            f[c] = f[c] + bs[y][c];
                        }
                    }
                }
                if (vec) {
                    store_c16<false>((v4f *)((float *)a.C + idx), (v4f){f[0], f[1], f[2], f[3]});
                } else {
                    for (int c = 0; c < 4 && n + c < a.N; ++c) {
                        ((float *)a.C)[idx + c] = f[c];
                    }
                }
            }
        }
    }
#undef BG_LOAD_CIN
    if (CONV && MODE == EPI_I32 && a.conv.absmax) {
        // max |acc| of the whole output tensor, for the dynamic requantisation that follows
        lane_max = wave_reduce_max_i(lane_max);
        if (lane == 0) {
            ws_fold_max(a.conv.absmax, blockIdx.x * 8 + wave, lane_max);
        }
    }
}

// Full-tile epilogue for 32-bit results of a matrix product, through a wave-private LDS panel.
// Straight from the accumulators a store instruction covers 16 rows x 64 bytes: sixteen half cache
// lines, which the memory pipeline takes several times longer to absorb than whole lines (measured:
// 256 such stores of a CU take 3 us against 1 us for the same bytes as 4 rows x 256 bytes). So each
// wave passes one 16 x 64 block of int32 accumulators at a time through 4.25 KiB of LDS (row pitch
// 272 bytes: both the fragment-order writes and the row-order reads are conflict free) and comes out
// with lane (r = lane / 16, c = lane % 16) holding columns 4c .. 4c+3 of row 4 * it + r: every
// result store and every C_in load is then 4 rows x 256 contiguous bytes, and the per-column terms
// shrink to four values per lane. The panel is private to the wave, so there is no barrier: LDS
// operations of one wave execute in order.
template <int MODE, int WM, int WN, int TM, int TN, int CIN, bool STREAM>
__device__ __forceinline__ void epilogue_rows_lds(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0)
{
    static_assert(TN == 4, "a wave's tile row must be 64 columns = 256 bytes of int32");
    static_assert(MODE == EPI_I32 || MODE == EPI_F32 || MODE == EPI_F32_CH, "32-bit results only");
    constexpr uint32_t kPitch = 272;
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    uint8_t *pan = smem + wave * (16 * kPitch);
    uint8_t *wr = pan + i * kPitch + g * 16;  // + 64 * y
    const uint8_t *rd = pan + g * kPitch + i * 16;  // + 4 * kPitch * it   (here g = row in group, i = column chunk)
    const uint32_t n = n0 + wn * 64 + i * 4;
    const uint32_t row0 = m0 + wm * TM * 16 + g;

    float factor = 0.0f, sI = 0.0f;
    if (MODE == EPI_F32) {
        factor = epi_factor(a.epi);
    } else if (MODE == EPI_F32_CH) {
        sI = *a.epi.scaleI;
    }
    uint32_t base[4];
    float qs[4], bs[4];
    {
        // every per-column term in one batch of loads (a load per use would put a trip to memory into each column)
        const uint32_t nn[4] = {n, n + 1, n + 2, n + 3};
        const float *swp = (MODE == EPI_F32_CH) ? a.epi.scaleW : (const float *)a.comp;
        const float *bip = (MODE == EPI_F32_CH && a.epi.bias) ? a.epi.bias : (const float *)a.comp;
        float sw[4], bi[4];
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            sw[c] = swp[nn[c]];
            bi[c] = bip[nn[c]];
        }
        column_bases<4>(a.ob, a.comp, a.fold_bias, a.fold_scale, nn, base);
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            qs[c] = (MODE == EPI_F32_CH) ? 1.0f / (sI * sw[c]) : 1.0f;
            bs[c] = (MODE == EPI_F32_CH && a.epi.bias) ? bi[c] : 0.0f;
        }
    }
    v4i cin[2][4];
#define BG_LOAD_CIN(xx, buf)                                                                           \
    if (CIN) {                                                                                         \
        _Pragma("unroll") for (int it = 0; it < 4; ++it)                                               \
        {                                                                                              \
            cin[buf][it] = *(const v4i *)((const int32_t *)a.C + (size_t)(row0 + (xx)*16 + it * 4) * a.N + n); \
        }                                                                                              \
    }
    BG_LOAD_CIN(0, 0);
#pragma unroll
    for (int x = 0; x < TM; ++x) {
        if (x + 1 < TM) {
            BG_LOAD_CIN(x + 1, (x + 1) & 1);
        }
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            *(v4i *)(wr + 64 * y) = acc[x][y];
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        v4i t[4];
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            t[it] = *(const v4i *)(rd + 4 * kPitch * it);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
#pragma unroll
        for (int it = 0; it < 4; ++it) {
            const size_t idx = (size_t)(row0 + x * 16 + it * 4) * a.N + n;
            int v[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                v[c] = (int)((uint32_t)t[it][c] + base[c] + (CIN ? (uint32_t)cin[x & 1][it][c] : 0u));  // int32 wrap
            }
            if (MODE == EPI_I32) {
                store_c16<STREAM>((v4i *)((int32_t *)a.C + idx), (v4i){v[0], v[1], v[2], v[3]});
            } else {
                float f[4];
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (MODE == EPI_F32) {
                        f[c] = (float)v[c] * factor;
                    } else {
                        f[c] = (float)v[c] * qs[c];
                        if (a.epi.bias) {
                            f[c] = f[c] + bs[c];
                        }
                    }
                }
                store_c16<STREAM>((v4f *)((float *)a.C + idx), (v4f){f[0], f[1], f[2], f[3]});
            }
        }
    }
#undef BG_LOAD_CIN
}

// Full-tile epilogue for u8 results of a matrix product, through a wave-private LDS panel of 16 rows x 64 bytes
// (pitch 80: the 4-byte writes of the fragment layout and the 16-byte reads of the row layout are both free of bank
// conflicts). Straight from the accumulators a store instruction puts 4 bytes of a different row into every lane,
// 64 pieces for the address unit; from the panel lane 4 r + c stores 16 bytes of row r, a quad = one 64-byte piece.
// CH: the per-output-channel form (EPI_U8_CH), the fp32 value of EPI_F32_CH quantised with the static scale epi.factor.
template <int WM, int WN, int TM, int TN, bool CH = false>
__device__ __forceinline__ void epilogue_rows_lds_u8(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0)
{
    static_assert(TN == 4, "a wave's tile row must be 64 columns");
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const float factor = CH ? a.epi.factor : epi_factor(a.epi);
    uint32_t base[TN * 4];
    float qs[TN * 4], bs[TN * 4];
    {
        uint32_t nn[TN * 4];
        float sw[TN * 4], bi[TN * 4];
        const float *swp = CH ? a.epi.scaleW : (const float *)a.comp;
        const float *bip = (CH && a.epi.bias) ? a.epi.bias : (const float *)a.comp;
#pragma unroll
        for (int y = 0; y < TN; ++y) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                nn[y * 4 + c] = n0 + (wn * TN + y) * 16 + 4 * g + c;
                sw[y * 4 + c] = swp[nn[y * 4 + c]];
                bi[y * 4 + c] = bip[nn[y * 4 + c]];
            }
        }
        column_bases<TN * 4>(a.ob, a.comp, a.fold_bias, a.fold_scale, nn, base);
        const float sI = CH ? *a.epi.scaleI : 1.0f;
#pragma unroll
        for (int k = 0; k < TN * 4; ++k) {
            qs[k] = CH ? 1.0f / (sI * sw[k]) : 1.0f;
            bs[k] = (CH && a.epi.bias) ? bi[k] : 0.0f;
        }
    }
    constexpr uint32_t kPitch = 80;
    uint8_t *pan = smem + wave * (16 * kPitch);
    uint8_t *wr = pan + i * kPitch + g * 4;  // + 16 * y
    const uint8_t *rd = pan + (lane >> 2) * kPitch + (lane & 3) * 16;
    uint8_t *out = (uint8_t *)a.C + (size_t)(m0 + wm * TM * 16 + (lane >> 2)) * a.N + n0 + wn * 64 + (lane & 3) * 16;
#pragma unroll
    for (int x = 0; x < TM; ++x) {
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            unsigned b[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const int t_ = (int)((uint32_t)acc[x][y][c] + base[y * 4 + c]);  // int32 wrap
                if (CH) {
                    float f = (float)t_ * qs[y * 4 + c];
                    if (a.epi.bias) {
                        f = f + bs[y * 4 + c];
                    }
                    b[c] = q_u8(f, factor);
                } else {
                    b[c] = epi_u8(t_, factor);
                }
            }
            *(uint32_t *)(wr + 16 * y) = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        const v4i row = *(const v4i *)rd;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        *(v4i *)(out + (size_t)x * 16 * a.N) = row;
    }
}

// EPI_U8_GELU_DYN: the FullyConnected in front of a GELU whose result the next FullyConnected wants quantised with a
// tensor-wide dynamic scale. Written as separate kernels that is an fp32 matrix stored, read for max|gelu|, and read
// again to be quantised; here the accumulators never leave the registers:
//   y = gelu_tanh(cvt(acc + base) * (1 / (sI * sW[n])) + bias[n])     (kept in the accumulator registers)
//   max|y| over the whole result through grid_max_sync               (every tile's workgroup is resident)
//   u8 = q_u8(y, max(0, 127 / max|y|)), scale published through dscale_out
// -- the arithmetic, element for element, of the per-channel fp32 epilogue, gelu_f32_kernel's maximum and
// quantize_f32_kernel<u8, gelu>. If the grid-wide wait is abandoned every workgroup stores its y as fp32 into C32,
// status becomes 1, and the last workgroup to finish quantises all of C32 by itself (grid_last_arrival): slow, but it
// needs neither another launch nor the host, and the wait only expires when the CUs were held by other work.
// Full 256 x 256 tiles only (the launcher checks).
template <int WM, int WN, int TM, int TN>
__device__ __forceinline__ void epilogue_gelu_sync(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0)
{
    static_assert(TN == 4, "a wave's tile row must be 64 columns");
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t tid = wave * 64 + lane;  // the thread's index, from what the caller formed afresh (see there)
    const uint32_t wm = wave / WN, wn = wave % WN;
    const float sI = *a.epi.scaleI;
    if (a.clear_ws && blockIdx.x == 0) {
        for (uint32_t k = tid; k < kWsWords; k += blockDim.x) {
            a.clear_ws[k] = 0;
        }
    }
    // every per-column term first, in one batch of loads (a load per use would put a trip to memory into each step)
    uint32_t base[TN][4];
    float qs[TN][4], bs[TN][4];
#pragma unroll
    for (int y = 0; y < TN; ++y) {
        const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
        const v4i cb = *(const v4i *)(a.comp + n);
        const v4i ob = *(const v4i *)(a.ob + n);
        const v4f sw = *(const v4f *)(a.epi.scaleW + n);
        const v4f bi = a.epi.bias ? *(const v4f *)(a.epi.bias + n) : (v4f){0.0f, 0.0f, 0.0f, 0.0f};
#pragma unroll
        for (int c = 0; c < 4; ++c) {
            base[y][c] = (uint32_t)ob[c] - (uint32_t)cb[c];
            qs[y][c] = 1.0f / (sI * sw[c]);
            bs[y][c] = bi[c];
        }
    }
    float amax = 0.0f;
#pragma unroll
    for (int x = 0; x < TM; ++x) {
#pragma unroll
        for (int y = 0; y < TN; ++y) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                float f = (float)(int)((uint32_t)acc[x][y][c] + base[y][c]) * qs[y][c];
                if (a.epi.bias) {
                    f = f + bs[y][c];
                }
                const float v = gelu_tanh(f);
                amax = fmaxf(amax, fabsf(v));
                acc[x][y][c] = __float_as_int(v);
            }
        }
    }
    const uint32_t outcome = grid_max_sync(a.sync, (int)__float_as_uint(amax), (int *)smem, tid);
    if (outcome == kGridAbandoned) {
        if (blockIdx.x == 0 && tid == 0) {
            *a.status = 1u;
        }
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            const uint32_t m = m0 + (wm * TM + x) * 16 + i;
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
                *(v4i *)(a.C32 + (size_t)m * a.N + n) = acc[x][y];
            }
        }
        // no workgroup can wait for the others now; the last one to get here quantises the whole result alone
        if (grid_last_arrival(a.sync, (int *)smem, tid)) {
            quantize_f32_u8_alone(a.C32, a.M * a.N, (uint8_t *)a.C, a.dscale_out, (float *)smem, tid);
        }
        return;
    }
    const float mx = __uint_as_float(outcome);
    const float s = (mx == 0.0f) ? 1.0f : 127.0f / mx;  // resolve_scale with no caller's scale: max(0, 127 / max)
    if (blockIdx.x == 0 && tid == 0) {
        *a.status = 0u;
        *a.dscale_out = s;
    }
    // u8 rows through a wave-private LDS panel of 16 rows x 64 bytes (pitch 80: the 4-byte writes of the fragment
    // layout and the 16-byte reads of the row layout are both free of bank conflicts), so that a store instruction
    // covers 16 rows x 64 contiguous bytes instead of 16 rows x 16 bytes. LDS operations of one wave execute in order.
    constexpr uint32_t kPitch = 80;
    uint8_t *pan = smem + 256 + wave * (16 * kPitch);
    uint8_t *wr = pan + i * kPitch + g * 4;                      // + 16 * y
    const uint8_t *rd = pan + (lane >> 2) * kPitch + (lane & 3) * 16;
    uint8_t *out = (uint8_t *)a.C + (size_t)(m0 + wm * TM * 16 + (lane >> 2)) * a.N + n0 + wn * 64 + (lane & 3) * 16;
#pragma unroll
    for (int x = 0; x < TM; ++x) {
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const v4i v = acc[x][y];  // |v * s| <= 127: s comes from the maximum of these very values
            *(uint32_t *)(wr + 16 * y) = pack_low_bytes(q_u8_inrange_bits(__int_as_float(v.x), s), q_u8_inrange_bits(__int_as_float(v.y), s),
                q_u8_inrange_bits(__int_as_float(v.z), s), q_u8_inrange_bits(__int_as_float(v.w), s));
        }
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        const v4i row = *(const v4i *)rd;
        asm volatile("s_waitcnt lgkmcnt(0)" ::: "memory");
        __builtin_amdgcn_wave_barrier();
        *(v4i *)(out + (size_t)x * 16 * a.N) = row;
    }
}

// EPI_CONV_CH: the int8 convolution with one filter scale per OUTPUT CHANNEL. Not in the reference, whose kernels
// carry one scale for the whole filter (convolution_direct.cpp:2406-2422, 2687-2692); the arithmetic is the per-channel
// matrix epilogue's (EPI_F32_CH) with the convolution's own tail:
//   f = cvt(acc + ob[oc] - comp[oc]) * (1.0f / (sI * sW[oc]))   single fp32 operations, reciprocal first
//   f = f + bias[oc]                                             when a bias is given
//   f = f + eltwise[...]                                         fp32 result only, as :2410-2422 place it
//   f = max(f, 0)                                                with ReLU
// and then, by conv.ch_out: stored as fp32; or quantised like a fp32 tensor (q_u8, avx512/quantize.cpp:150-155) with
// the static scale epi.factor or the dynamic one 127 / max|f| from the scratch slots; or only max|f| folded into those
// slots. With every sW[oc] equal, no bias and an fp32 result this is the reference's epilogue bit for bit.
template <int WM, int WN, int TM, int TN, bool SYNC>
__device__ __forceinline__ void epilogue_conv_ch(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0, const ColTerms ct = ColTerms())
{
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const float sI = a.conv.dscaleI ? *a.conv.dscaleI : a.conv.scaleI;
    const int out = a.conv.ch_out;
    uint32_t base[TN][4], cblk_off[TN], cblk_w[TN];
    float qs[TN][4], bs[TN][4];
    if (ct.qs) {
        // formed once per workgroup ahead of the K loop (see ColTerms)
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
            const uint32_t at = (wn * TN + y) * 16 + 4 * g;
            const v4i b4 = *(const v4i *)(ct.base + at);
            const v4f q4 = *(const v4f *)(ct.qs + at), s4 = *(const v4f *)(ct.bs + at);
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                base[y][c] = (uint32_t)b4[c];
                qs[y][c] = q4[c];
                bs[y][c] = s4[c];
            }
            const uint32_t xc = a.conv.out_c, blk = n / xc;
            cblk_w[y] = (a.N - blk * xc < xc) ? a.N - blk * xc : xc;
            cblk_off[y] = blk * xc * a.conv.OHW + (n % xc);
        }
    } else {
        // every per-column term in one batch of loads, none behind a branch; columns past N read column N - 1
        uint32_t nn[TN * 4], flat[TN * 4];
        float sw[TN * 4], bi[TN * 4];
        const float *bip = a.epi.bias ? a.epi.bias : a.epi.scaleW;
#pragma unroll
        for (int y = 0; y < TN; ++y) {
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g + c;
                nn[y * 4 + c] = n < a.N ? n : a.N - 1;
                sw[y * 4 + c] = a.epi.scaleW[nn[y * 4 + c]];
                bi[y * 4 + c] = bip[nn[y * 4 + c]];
            }
        }
        column_bases<TN * 4>(a.ob, a.comp, nullptr, 0.0f, nn, flat);
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                base[y][c] = flat[y * 4 + c];
                qs[y][c] = 1.0f / (sI * sw[y * 4 + c]);
                bs[y][c] = a.epi.bias ? bi[y * 4 + c] : 0.0f;
            }
            const uint32_t xc = a.conv.out_c, blk = n / xc;
            cblk_w[y] = (a.N - blk * xc < xc) ? a.N - blk * xc : xc;
            cblk_off[y] = blk * xc * a.conv.OHW + (n % xc);
        }
    }
    if (SYNC && out == CONV_CH_U8 && a.sync.slots) {
        // ONE pass (filter-panel kernel, every workgroup resident): the fp32 values replace the accumulators in their
        // registers, the workgroups agree on max|f| (smem: 18 ints of LDS nobody reads tiles from), and each quantises
        // its own values. Should that agreement be abandoned: with no spill buffer (synchronous form) nothing is
        // stored and a NaN scale tells the host to run the two passes; with one (C32, asynchronous form) every
        // workgroup parks its fp32 values there and the last to arrive quantises the tensor alone.
        float amax = 0.0f;
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            const uint32_t m = m0 + (wm * TM + x) * 16 + i;
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    float f = (float)(int)((uint32_t)acc[x][y][c] + base[y][c]) * qs[y][c];
                    if (a.epi.bias) {
                        f = f + bs[y][c];
                    }
                    if (a.conv.relu && !(f > 0.0f)) {
                        f = 0.0f;
                    }
                    acc[x][y][c] = __float_as_int(f);
                    const float af = fabsf(f);
                    amax = (m < a.M && n < a.N && af > amax) ? af : amax;  // a NaN never wins, as in the quantiser
                }
            }
        }
        const uint32_t outcome = grid_max_sync(a.sync, (int)__float_as_uint(amax), (int *)smem);
        if (outcome == kGridAbandoned && !a.C32) {
            if (blockIdx.x == 0 && threadIdx.x == 0 && a.conv.dscale_out) {
                *a.conv.dscale_out = __int_as_float(0x7fc00000);
            }
            return;
        }
        const bool parked = outcome == kGridAbandoned;
        const float mxf = __uint_as_float(outcome);
        const float so = (mxf == 0.0f) ? 1.0f : 127.0f / mxf;
        if (!parked && blockIdx.x == 0 && threadIdx.x == 0 && a.conv.dscale_out) {
            *a.conv.dscale_out = so;
        }
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            const uint32_t m = m0 + (wm * TM + x) * 16 + i;
            if (m >= a.M) {
                continue;
            }
            const uint32_t img = m / a.conv.OHW, pix = m - img * a.conv.OHW;
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
                if (n >= a.N) {
                    continue;
                }
                const size_t idx = (size_t)img * a.N * a.conv.OHW + cblk_off[y] + (size_t)pix * cblk_w[y];
                if (parked) {
                    *(v4i *)((int32_t *)a.C32 + idx) = acc[x][y];
                } else {
                    const unsigned b0 = q_u8(__int_as_float(acc[x][y][0]), so), b1 = q_u8(__int_as_float(acc[x][y][1]), so);
                    const unsigned b2 = q_u8(__int_as_float(acc[x][y][2]), so), b3 = q_u8(__int_as_float(acc[x][y][3]), so);
                    *(uint32_t *)((uint8_t *)a.C + idx) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
                }
            }
        }
        if (parked) {
            const int wmax = wave_reduce_max_i((int)__float_as_uint(amax));
            if (lane == 0) {
                ws_fold_max(a.conv.absmax, blockIdx.x * 8 + wave, wmax);
            }
            if (grid_last_arrival(a.sync, (int *)smem)) {
                const float mx = __uint_as_float((uint32_t)ws_read_max(a.conv.absmax));
                const float sl = (mx == 0.0f) ? 1.0f : 127.0f / mx;
                if (threadIdx.x == 0 && a.conv.dscale_out) {
                    *a.conv.dscale_out = sl;
                }
                const uint32_t total4 = (a.M * a.N) / 4;
                for (uint32_t k = threadIdx.x; k < total4; k += blockDim.x) {
                    const v4f t = ((const v4f *)a.C32)[k];
                    ((uint32_t *)a.C)[k] = q_u8(t.x, sl) | (q_u8(t.y, sl) << 8) | (q_u8(t.z, sl) << 16) | (q_u8(t.w, sl) << 24);
                }
                __syncthreads();
                for (uint32_t k = threadIdx.x; k < kWsWords; k += blockDim.x) {
                    a.conv.absmax[k] = 0;
                }
            }
        }
        return;
    }
    float s = 0.0f;
    if (out == CONV_CH_U8) {
        if (a.epi.factor > 0.0f) {
            s = a.epi.factor;
        } else {
            const float mx = __uint_as_float((uint32_t)ws_read_max(a.conv.absmax));
            s = (mx == 0.0f) ? 1.0f : 127.0f / mx;
        }
        if (blockIdx.x == 0 && wave == 0 && lane == 0 && a.conv.dscale_out) {
            *a.conv.dscale_out = s;
        }
    }
    int lane_max = 0;
#pragma unroll
    for (int x = 0; x < TM; ++x) {
        const uint32_t m = m0 + (wm * TM + x) * 16 + i;
        if (m >= a.M) {
            continue;
        }
        const uint32_t img = m / a.conv.OHW, pix = m - img * a.conv.OHW;
        const size_t rowbase = (size_t)img * a.N * a.conv.OHW;
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            const uint32_t n = n0 + (wn * TN + y) * 16 + 4 * g;
            if (n >= a.N) {
                continue;
            }
            const size_t idx = rowbase + cblk_off[y] + (size_t)pix * cblk_w[y];
            float f[4];
#pragma unroll
            for (int c = 0; c < 4; ++c) {
                f[c] = (float)(int)((uint32_t)acc[x][y][c] + base[y][c]) * qs[y][c];
                if (a.epi.bias) {
                    f[c] = f[c] + bs[y][c];
                }
                if (out == CONV_CH_F32 && a.conv.eltwise && n + c < a.N) {
                    f[c] = f[c] + a.conv.eltwise[idx + c];
                }
                if (a.conv.relu && !(f[c] > 0.0f)) {
                    f[c] = 0.0f;
                }
            }
            if (out == CONV_CH_MAX) {
#pragma unroll
                for (int c = 0; c < 4; ++c) {
                    if (n + c < a.N) {
                        const int av = (int)__float_as_uint(fabsf(f[c]));  // a NaN's bits never win against a number's:
                        lane_max = (f[c] == f[c] && av > lane_max) ? av : lane_max;  // the quantiser's maximum skips NaNs too
                    }
                }
            } else if (out == CONV_CH_U8) {
                const unsigned b0 = q_u8(f[0], s), b1 = q_u8(f[1], s), b2 = q_u8(f[2], s), b3 = q_u8(f[3], s);
                *(uint32_t *)((uint8_t *)a.C + idx) = b0 | (b1 << 8) | (b2 << 16) | (b3 << 24);
            } else {
                store_c16<false>((v4f *)((float *)a.C + idx), (v4f){f[0], f[1], f[2], f[3]});
            }
        }
    }
    if (out == CONV_CH_MAX) {
        lane_max = wave_reduce_max_i(lane_max);
        if (lane == 0) {
            ws_fold_max(a.conv.absmax, blockIdx.x * 8 + wave, lane_max);
        }
    }
}

template <int MODE, bool CONV, int WM, int WN, int TM, int TN, bool SYNC = false>
__device__ __forceinline__ void epilogue_mode(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0, const ColTerms pre_base = ColTerms())
{
    const bool full = (m0 + WM * TM * 16 <= a.M) && (n0 + WN * TN * 16 <= a.N) && (CONV || (a.N & 3) == 0);
    const bool cin = !CONV && a.add_cin && MODE != EPI_U8 && MODE != EPI_U8_CH;
    if constexpr (!CONV && MODE != EPI_U8 && MODE != EPI_U8_CH && TN == 4) {
        // smem: the kernel's LDS, free by now and at least 8 waves x 4352 bytes (the DMA kernels); null otherwise
        if (full && smem) {
            if (a.stream_c) {
                if (cin) {
                    epilogue_rows_lds<MODE, WM, WN, TM, TN, 1, true>(a, acc, smem, lane, wave, m0, n0);
                } else {
                    epilogue_rows_lds<MODE, WM, WN, TM, TN, 0, true>(a, acc, smem, lane, wave, m0, n0);
                }
            } else if (cin) {
                epilogue_rows_lds<MODE, WM, WN, TM, TN, 1, false>(a, acc, smem, lane, wave, m0, n0);
            } else {
                epilogue_rows_lds<MODE, WM, WN, TM, TN, 0, false>(a, acc, smem, lane, wave, m0, n0);
            }
            return;
        }
    }
    if constexpr (!CONV && (MODE == EPI_U8 || MODE == EPI_U8_CH) && TN == 4) {
        if (full && smem && (a.N & 15) == 0 && ((uintptr_t)a.C & 15) == 0) {
            epilogue_rows_lds_u8<WM, WN, TM, TN, MODE == EPI_U8_CH>(a, acc, smem, lane, wave, m0, n0);
            return;
        }
    }
    if (full && !cin) {
        epilogue_rows<MODE, CONV, WM, WN, TM, TN, true, 0, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
    } else if (full && MODE != EPI_U8 && MODE != EPI_U8_CH && !CONV) {
        epilogue_rows<MODE, CONV, WM, WN, TM, TN, true, 1, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
    } else {
        epilogue_rows<MODE, CONV, WM, WN, TM, TN, false, 2, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
    }
}

template <int WM, int WN, int TM, int TN, bool CONV = false, bool SYNC = false>
__device__ __forceinline__ void epilogue_panel(const GemmArgs &a, v4i (&acc)[TM][TN], uint8_t *smem, uint32_t lane,
    uint32_t wave, uint32_t m0, uint32_t n0, int lds_bytes, const ColTerms pre_base = ColTerms())
{
    (void)lds_bytes;
    if (CONV) {
        if (a.epi.mode == EPI_I32) {
            epilogue_mode<EPI_I32, true, WM, WN, TM, TN, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
        } else if (a.epi.mode == EPI_U8) {
            epilogue_mode<EPI_U8, true, WM, WN, TM, TN, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
        } else if (a.epi.mode == EPI_F32_CH) {
            epilogue_mode<EPI_F32_CH, true, WM, WN, TM, TN, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
        } else if (a.epi.mode == EPI_CONV_CH) {
            epilogue_conv_ch<WM, WN, TM, TN, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
        } else {
            epilogue_mode<EPI_F32, true, WM, WN, TM, TN, SYNC>(a, acc, smem, lane, wave, m0, n0, pre_base);
        }
        return;
    }
    switch (a.epi.mode) {
        case EPI_I32:
            epilogue_mode<EPI_I32, false, WM, WN, TM, TN>(a, acc, smem, lane, wave, m0, n0);
            break;
        case EPI_F32:
            epilogue_mode<EPI_F32, false, WM, WN, TM, TN>(a, acc, smem, lane, wave, m0, n0);
            break;
        case EPI_U8:
            epilogue_mode<EPI_U8, false, WM, WN, TM, TN>(a, acc, smem, lane, wave, m0, n0);
            break;
        case EPI_U8_CH:
            epilogue_mode<EPI_U8_CH, false, WM, WN, TM, TN>(a, acc, smem, lane, wave, m0, n0);
            break;
        default:
            epilogue_mode<EPI_F32_CH, false, WM, WN, TM, TN>(a, acc, smem, lane, wave, m0, n0);
            break;
    }
}

template <int WM, int WN, int TM, int TN>
__global__ __launch_bounds__(WM *WN * 64, 2) void gemm_u8s8_tiled_kernel(GemmArgs a)
{
    using T = GemmTile<WM, WN, TM, TN>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    const uint32_t m0 = blockIdx.y * T::kBM, n0 = blockIdx.x * T::kBN;
    const uint32_t K = a.K;  // == Kp, multiple of 16
    const uint32_t nblocks = align_up(a.N, 16) >> 4;
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};

    v4i acc[TM][TN];
#pragma unroll
    for (int x = 0; x < TM; ++x) {
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            acc[x][y] = (v4i){0, 0, 0, 0};
        }
    }
    v4i ra[T::kALoads], rb[T::kBLoads];

    // per-lane global addresses of this wave's fragments at k0 = 0
    const uint8_t *pa[T::kALoads];
    const int8_t *pb[T::kBLoads];
    bool va[T::kALoads], vb[T::kBLoads];
#pragma unroll
    for (int q = 0; q < T::kALoads; ++q) {
        const uint32_t f = wave * T::kALoads + q;
        const uint32_t row = m0 + (f >> 1) * 16 + i;
        va[q] = row < a.M;
        pa[q] = a.A + (size_t)(va[q] ? row : 0) * a.lda + (f & 1) * 64 + g * 16;
    }
#pragma unroll
    for (int q = 0; q < T::kBLoads; ++q) {
        const uint32_t f = wave * T::kBLoads + q;
        const uint32_t nb = (n0 >> 4) + (f >> 1);
        vb[q] = nb < nblocks;
        pb[q] = a.Bp + (size_t)(vb[q] ? nb : 0) * 16 * K + (size_t)((f & 1) * 4 + g) * 256 + i * 16;
    }

#define BG_LOAD_GLOBAL(k0)                                                                  \
    {                                                                                       \
        _Pragma("unroll") for (int q = 0; q < T::kALoads; ++q)                              \
        {                                                                                   \
            const uint32_t f = wave * T::kALoads + q;                                       \
            const uint32_t k = (k0) + (f & 1) * 64 + g * 16;                                \
            const bool ok = va[q] && k < K;                                                 \
            /* branch-free: out-of-range lanes read a valid dummy address and are zeroed */ \
            const v4i v = *(const v4i *)(ok ? pa[q] + (k0) : a.A);                          \
            ra[q] = ok ? (v ^ flip) : (v4i){0, 0, 0, 0};                                    \
        }                                                                                   \
        _Pragma("unroll") for (int q = 0; q < T::kBLoads; ++q)                              \
        {                                                                                   \
            const uint32_t f = wave * T::kBLoads + q;                                       \
            const uint32_t k = (k0) + (f & 1) * 64 + g * 16;                                \
            const bool ok = vb[q] && k < K;                                                 \
            const v4i v = *(const v4i *)(ok ? pb[q] + (size_t)(k0) * 16 : a.Bp);            \
            rb[q] = ok ? v : (v4i){0, 0, 0, 0};                                             \
        }                                                                                   \
    }
#define BG_STORE_LDS(stage)                                                                 \
    {                                                                                       \
        uint8_t *sA_ = smem + (stage) * T::kStageBytes;                                     \
        uint8_t *sB_ = sA_ + T::kAFrags * 1024;                                             \
        _Pragma("unroll") for (int q = 0; q < T::kALoads; ++q)                              \
        {                                                                                   \
            *(v4i *)(sA_ + (wave * T::kALoads + q) * 1024 + lane * 16) = ra[q];             \
        }                                                                                   \
        _Pragma("unroll") for (int q = 0; q < T::kBLoads; ++q)                              \
        {                                                                                   \
            *(v4i *)(sB_ + (wave * T::kBLoads + q) * 1024 + lane * 16) = rb[q];             \
        }                                                                                   \
    }

    const uint32_t ksteps = (K + T::kBK - 1) / T::kBK;
    BG_LOAD_GLOBAL(0u);
    BG_STORE_LDS(0);
    __syncthreads();
    for (uint32_t t = 0; t < ksteps; ++t) {
        const int cur = t & 1;
        if (t + 1 < ksteps) {
            BG_LOAD_GLOBAL((t + 1) * T::kBK);
        }
        const uint8_t *sA = smem + cur * T::kStageBytes;
        const uint8_t *sB = sA + T::kAFrags * 1024;
#pragma unroll
        for (int kh = 0; kh < 2; ++kh) {
            v4i fa[TM], fb[TN];
#pragma unroll
            for (int x = 0; x < TM; ++x) {
                fa[x] = *(const v4i *)(sA + (((wm * TM + x) << 1) + kh) * 1024 + lane * 16);
            }
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                fb[y] = *(const v4i *)(sB + (((wn * TN + y) << 1) + kh) * 1024 + lane * 16);
            }
#pragma unroll
            for (int x = 0; x < TM; ++x) {
#pragma unroll
                for (int y = 0; y < TN; ++y) {
                    acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[y], fa[x], acc[x][y], 0, 0, 0);  // B first: transposed accumulator
                }
            }
        }
        if (t + 1 < ksteps) {
            BG_STORE_LDS(cur ^ 1);
        }
        __syncthreads();
    }
#undef BG_LOAD_GLOBAL
#undef BG_STORE_LDS

    epilogue_panel<WM, WN, TM, TN>(a, acc, nullptr, lane, wave, m0, n0, T::kLdsBytes);
}

// Pipelined kernel for K % 64 == 0 (the shapes that matter for throughput).
//
// Same fragment-order LDS staging as above, but the tiles travel global -> LDS directly
// (global_load_lds_dwordx4: every lane supplies its own global address, the 64 x 16 bytes land at
// consecutive LDS addresses = exactly one MFMA fragment), with STAGES K tiles of 64 in flight so
// that HBM / L2 latency is covered by several tiles' worth of MFMAs instead of one. No staging
// registers; A is re-biased (^ 0x80) after the fragment read. One s_barrier per K tile:
//   wait until this wave's share of tile t has landed -> barrier (everyone's share has landed and
//   everyone is done reading tile t-1) -> refill the buffer of tile t-1 with tile t+STAGES-1 ->
//   MFMAs on tile t.
// Rows / column blocks past the matrix edge load a clamped (valid) address; what they produce is
// never stored. Workgroup ids are re-mapped so that each XCD (ids are dealt round-robin over the 8
// XCDs) works on one contiguous band of output tiles and re-uses its A rows / B columns in its L2.
// u8 convolution, second pass: the tensor-wide output scale follows from the maximum the first pass left in the
// scratch slots, and the host is waiting for it. The first wave of the first workgroup publishes it before any
// other work and clears the pointer in this workgroup's copy of the arguments, so that the epilogue (which needs
// the same factor for its own arithmetic) does not store it a second time.
__device__ __forceinline__ void conv_publish_scale(GemmArgs &a, uint32_t wave)
{
    if (a.clear_ws && blockIdx.x == 0) {
        // an array of max slots that no kernel still in flight reads (the caller alternates between two): cleared
        // here for the call that will fold into it next
        for (uint32_t k = threadIdx.x; k < kWsWords; k += blockDim.x) {
            a.clear_ws[k] = 0;
        }
    }
    if (a.conv.dscale_out && a.conv.dscaleI && (a.epi.mode == EPI_F32 || (a.epi.mode == EPI_I32 && a.C))) {
        // asynchronous form, fp32 / int32 result: the scale of the accumulators is what the synchronous call reports
        if (blockIdx.x == 0 && wave == 0 && (threadIdx.x & 63) == 0) {
            *a.conv.dscale_out = conv_acc_scale(a.conv);
        }
        a.conv.dscale_out = nullptr;
    }
    if (a.epi.mode == EPI_U8 && a.conv.dscale_out && !a.sync.slots) {
        if (blockIdx.x == 0 && wave == 0) {
            const int mx = ws_read_max(a.conv.absmax);
            const float factor = (mx == 0) ? 1.0f : 127.0f / (float)mx;
            if ((threadIdx.x & 63) == 0) {
                *a.conv.dscale_out = conv_acc_scale(a.conv) * factor;
            }
        }
        a.conv.dscale_out = nullptr;
    } else if (a.epi.mode == EPI_CONV_CH && a.conv.ch_out == CONV_CH_U8 && a.conv.dscale_out && !a.sync.slots) {
        // the per-channel form: the scale the u8 result is quantised with (given, or from the first pass's max|f|)
        if (blockIdx.x == 0 && wave == 0) {
            float s = a.epi.factor;
            if (!(s > 0.0f)) {
                const float mx = __uint_as_float((uint32_t)ws_read_max(a.conv.absmax));
                s = (mx == 0.0f) ? 1.0f : 127.0f / mx;
            }
            if ((threadIdx.x & 63) == 0) {
                *a.conv.dscale_out = s;
            }
        }
        a.conv.dscale_out = nullptr;
    }
}

template <int WM, int WN, int TM, int TN, int STAGES>
struct GemmDma {
    static constexpr int kBM = WM * TM * 16;
    static constexpr int kBN = WN * TN * 16;
    static constexpr int kWaves = WM * WN;
    static constexpr int kAFrags = kBM / 16;
    static constexpr int kBFrags = kBN / 16;
    static constexpr int kLoads = (kAFrags + kBFrags) / kWaves;  // fragments each wave fetches per K tile
    static constexpr int kStageBytes = (kAFrags + kBFrags) * 1024;
    static constexpr int kLdsBytes = STAGES * kStageBytes;
    static_assert((kAFrags + kBFrags) % kWaves == 0, "fragments must divide evenly over the waves");
};

__device__ __forceinline__ constexpr int vmcnt_imm(int n)
{
    return (n & 0xF) | ((n >> 4) << 14) | (0x7 << 4) | (0xF << 8);  // expcnt / lgkmcnt: no wait
}

typedef const __attribute__((address_space(1))) void *gptr_t;
typedef __attribute__((address_space(3))) void *lptr_t;

// FP4 (1-bit convolution only): the operand bytes hold two E2M1 values each (+1 = 0x2, -1 = 0xA, 0 = 0x0) and the
// products are formed by v_mfma_scale_f32_16x16x128_f8f6f4 -- twice the K per instruction at the same rate, fp32
// accumulation that is exact for these integers; the accumulators are converted to int32 before the epilogue.
// GELU_DYN: the kernel ends in the EPI_U8_GELU_DYN epilogue and nothing else (an instantiation of its own, so that
// the registers that epilogue needs do not burden the others).
template <int WM, int WN, int TM, int TN, int STAGES, int PIPE, bool CONV = false, bool FP4 = false, bool GELU_DYN = false>
// Two waves per SIMD are asked for also where a workgroup has four waves: with a budget of 512 registers per lane
// the compiler keeps the accumulators in AGPRs and spends dozens of v_accvgpr moves per K tile on shuffling them.
__global__ __launch_bounds__(WM *WN * 64 * (PIPE == 8 ? 2 : 1), PIPE == 8 ? 1 : 2) void gemm_u8s8_dma_kernel(GemmArgs a)
{
    using T = GemmDma<WM, WN, TM, TN, STAGES>;
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave_all = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);  // wave-uniform: keep it scalar
    // PIPE == 8: two groups of WM x WN waves work on the same tile, group gidx on the K tiles 2 j + gidx
    const uint32_t gidx = (PIPE == 8) ? wave_all / (WM * WN) : 0u, wave = (PIPE == 8) ? wave_all % (WM * WN) : wave_all;
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t wm = wave / WN, wn = wave % WN;
    if (CONV) {
        conv_publish_scale(a, wave);
    }

    // XCD-aware tile order: hardware deals linear workgroup ids round-robin to the 8 XCDs; give XCD x
    // the x-th contiguous eighth of the tile sequence, and walk that sequence in bands of 8 M-tiles.
    const uint32_t tiles_m = (a.M + T::kBM - 1) / T::kBM, tiles_n = (a.N + T::kBN - 1) / T::kBN;
    const uint32_t total = tiles_m * tiles_n;
    uint32_t pid = blockIdx.x;
    if (total % 8 == 0) {
        pid = (pid % 8) * (total / 8) + pid / 8;
    }
    const uint32_t band = 8 * tiles_n;
    const uint32_t band_id = pid / band;
    const uint32_t band_rows = (tiles_m - band_id * 8 < 8) ? tiles_m - band_id * 8 : 8;
    const uint32_t tm = band_id * 8 + (pid % band) % band_rows;
    const uint32_t tn = (pid % band) / band_rows;
    const uint32_t m0 = tm * T::kBM, n0 = tn * T::kBN;

    const uint32_t K = a.K;
    const uint32_t nblocks = align_up(a.N, 16) >> 4;
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
    // Touch the per-column vectors the epilogue will want (offsetC, compensation) now, so that they sit
    // in this XCD's L2 by then instead of costing an HBM round trip at the end of every block.
    int warm = 0;
    {
        const uint32_t n = n0 + wn * TN * 16 + lane;
        if (lane < TN * 16 && n < a.N) {
            warm = (a.fold_bias ? __float_as_int(a.fold_bias[n]) : a.ob[n]) ^ a.comp[n];
            if (a.epi.scaleW) {
                warm ^= __float_as_int(a.epi.scaleW[n]);
            }
            if (a.epi.bias) {
                warm ^= __float_as_int(a.epi.bias[n]);
            }
        }
    }

    v4i acc[TM][TN];
#pragma unroll
    for (int x = 0; x < TM; ++x) {
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            acc[x][y] = (v4i){0, 0, 0, 0};
        }
    }

    if constexpr (PIPE == 3) {
        // Ping-pong schedule as PIPE == 2, with A requested in whole 128-byte lines. A request laid out like the
        // MFMA operand (lane 16 g + i = 16 bytes of row i) puts a different row into every lane, the address unit
        // takes each lane's 16 bytes as a piece of its own, and such a request takes 2.5 times longer to be
        // accepted than 1 KB made of 8 whole lines (measured in isolation: 1 040 against 410 cycles per 16 KB and
        // CU), which is more than the MFMAs of a K tile take. (The other loops now give a row to the four lanes of
        // a quad, 64 contiguous bytes, which is accepted as fast.) Here a
        // request covers 8 rows x 128 bytes = the K bytes of two consecutive tiles, so A travels in pairs of
        // tiles: three slots of 256 rows x 128 bytes (tile pair p in slot p % 3, requested four tiles ahead
        // at the even tile) next to the four B slots of 16 KB (tile t in slot t % 4, requested three ahead).
        // Inside a slot the 16 rows x 128 bytes of row block r sit at r * 2 KB; lane (8 * row + pos) of a
        // request fetches 16-byte chunk pos ^ sw of its row, sw = (row16 >> 1) & 7 with row16 the row inside
        // the 16-row block, so that the fragment read of K half h (lane (i, g) reads chunk 4 h + g of row i:
        // 16 consecutive lanes = 16 rows) spreads over all 64 banks.
        static_assert(PIPE != 3 || (!CONV && !FP4 && WM * WN == 8 && STAGES == 5 && T::kAFrags == 16 && T::kBFrags == 16),
            "the whole-line loop is written for 256 x 256 matrix tiles in 160 KB of LDS");
        static_assert(PIPE != 3 || (WM == 2 && WN == 4 && TM == 8 && TN == 4), "checked for eight waves of 128 x 64 only");
        constexpr uint32_t kASlot = T::kAFrags * 2048, kBBase = 3 * kASlot, kBSlot = T::kBFrags * 1024;
        constexpr int kQA2 = 2 * T::kAFrags / T::kWaves;  // requests per wave and tile pair
        constexpr int kQB = T::kBFrags / T::kWaves;       // requests per wave and tile
        static_assert(kBBase + 4 * kBSlot == (uint32_t)T::kLdsBytes, "LDS layout");
        uint32_t offA[kQA2], offB[kQB];
#pragma unroll
        for (int q = 0; q < kQA2; ++q) {
            const uint32_t b = wave + q * T::kWaves;  // block of 8 rows
            uint32_t row = m0 + b * 8 + (lane >> 3);
            row = row < a.M ? row : a.M - 1;
            const uint32_t row16 = (b & 1) * 8 + (lane >> 3);
            offA[q] = row * a.lda + (((lane & 7) ^ ((row16 >> 1) & 7)) * 16);
        }
#pragma unroll
        for (int q = 0; q < kQB; ++q) {
            uint32_t nb = (n0 >> 4) + (wave + q * T::kWaves);
            nb = nb < nblocks ? nb : nblocks - 1;
            offB[q] = nb * 16 * K + lane * 16;
        }
        const uint32_t ksteps = K / 64, kpairs = ksteps / 2;  // the launcher checks K % 128 == 0
        const uint32_t rdA = (i >> 3) * 1024 + ((i & 7) * 8 + (g ^ ((i >> 1) & 7))) * 16;
#define BG3_ISSUE_A(aslot, pair, QLO, QHI)                                                                        \
    {                                                                                                             \
        const uint8_t *base_ = a.A + (size_t)((pair) < kpairs ? (pair) : kpairs - 1) * 128;                       \
        _Pragma("unroll") for (int q = (QLO); q < (QHI); ++q)                                                     \
        {                                                                                                         \
            __builtin_amdgcn_global_load_lds((gptr_t)(base_ + offA[q]),                                           \
                (lptr_t)(smem + (aslot)*kASlot + (wave + q * T::kWaves) * 1024), 16, 0, 0);                       \
        }                                                                                                         \
    }
#define BG3_ISSUE_B(tile)                                                                                         \
    {                                                                                                             \
        const uint8_t *base_ = (const uint8_t *)a.Bp + (size_t)((tile) < ksteps ? (tile) : ksteps - 1) * 1024;    \
        _Pragma("unroll") for (int q = 0; q < kQB; ++q)                                                           \
        {                                                                                                         \
            __builtin_amdgcn_global_load_lds((gptr_t)(base_ + offB[q]),                                           \
                (lptr_t)(smem + kBBase + ((tile)&3) * kBSlot + (wave + q * T::kWaves) * 1024), 16, 0, 0);         \
        }                                                                                                         \
    }
        // Every tile requests its B three tiles ahead; the even tile t then also requests the A pair t / 2 + 2
        // (tiles t+4, t+5). Order: A0 B0 B1 A1 B2 | tile 0: B3 A2 | tile 1: B4 | tile 2: B5 A3 | tile 3: B6 | ...
        BG3_ISSUE_A(0u, 0u, 0, kQA2);
        BG3_ISSUE_B(0u);
        BG3_ISSUE_B(1u);
        BG3_ISSUE_A(1u, 1u, 0, kQA2);
        BG3_ISSUE_B(2u);
        v4i fa[TM], fb[TN];
        const bool late = wave >= 4;
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kQA2 + 2 * kQB));  // tile 0 landed: B1, A1, B2 may be outstanding
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (late) {
            __builtin_amdgcn_s_barrier();
        }
        // What must have landed at the start of memory phase t is this wave's share of tile t+1. Even t (HALF 0):
        // the pair of tile t+1 is the one being read, B(t+1) is the youngest request needed, and behind it are a
        // pair and B(t+2). Odd t (HALF 1): tile t+1 opens the pair requested three tiles ago, which precedes
        // B(t+1) in the order; behind B(t+1) are B(t+2) and the pair requested at tile t-1. Either way kQA2 + kQB
        // requests may still be outstanding.
#define BG3_STEP(HALF)                                                                                            \
    {                                                                                                             \
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kQA2 + kQB));                                                        \
        asm volatile("" ::: "memory");                                                                            \
        BG3_ISSUE_B(t + 3);                                                                                       \
        if (!(HALF)) {                                                                                            \
            BG3_ISSUE_A(aslot_req, t / 2 + 2, 0, kQA2);                                                           \
        }                                                                                                         \
        {                                                                                                         \
            const uint8_t *sA_ = smem + aslot * kASlot + (rdA ^ ((HALF)*64));                                     \
            const uint8_t *sB_ = smem + kBBase + (t & 3) * kBSlot;                                                \
            _Pragma("unroll") for (int y = 0; y < TN; ++y)                                                        \
            {                                                                                                     \
                fb[y] = *(const v4i *)(sB_ + (wn * TN + y) * 1024 + lane * 16);                                   \
            }                                                                                                     \
            _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                        \
            {                                                                                                     \
                fa[x] = *(const v4i *)(sA_ + (wm * TM + x) * 2048);                                               \
            }                                                                                                     \
        }                                                                                                         \
        __builtin_amdgcn_s_waitcnt(0xc07f);                                                                       \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                            \
        {                                                                                                         \
            fa[x] ^= flip;                                                                                        \
        }                                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_s_barrier();                                                                             \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        __builtin_amdgcn_s_setprio(1);                                                                            \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                            \
        {                                                                                                         \
            _Pragma("unroll") for (int y = 0; y < TN; ++y)                                                        \
            {                                                                                                     \
                acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[y], fa[x], acc[x][y], 0, 0, 0);              \
            }                                                                                                     \
        }                                                                                                         \
        __builtin_amdgcn_s_setprio(0);                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_s_barrier();                                                                             \
        asm volatile("" ::: "memory");                                                                            \
    }
        uint32_t aslot = 0, aslot_req = 2;  // slot of the pair being read / of the pair requested at the even tile
        for (uint32_t t = 0; t < ksteps; t += 2) {
            BG3_STEP(0);
            ++t;
            BG3_STEP(1);
            --t;
            aslot = aslot == 2 ? 0 : aslot + 1;
            aslot_req = aslot_req == 2 ? 0 : aslot_req + 1;
        }
        if (!late) {
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the clamped refetches
#undef BG3_STEP
#undef BG3_ISSUE_A
#undef BG3_ISSUE_B
    } else if constexpr (PIPE == 4) {
        // Ping-pong schedule as PIPE == 3 (A in whole 128-byte lines, pairs of K tiles, three pair slots of 32 KB), with
        // the B fragments NOT staged through LDS: the packed right-hand side already holds every 16-column x 64-byte
        // fragment as 1 KB in lane order, so each wave loads the TN fragments of its own columns straight into registers
        // three tiles ahead (a ring of three register sets). The two waves that share a column block load the same
        // bytes (the second is served by the CU's cache), which doubles the B requests; in exchange the LDS carries A
        // only -- per K tile and CU 64 KB of fragment reads + 16 KB of arriving A instead of 96 + 32 KB, which at
        // 128 bytes per cycle was as long as the 1024 cycles the tile's MFMAs take.
        static_assert(PIPE != 4 || (!CONV && !FP4 && WM * WN == 8 && STAGES == 3 && T::kAFrags == 16 && T::kBFrags == 16 && TN == 4),
            "the register-B loop is written for 256 x 256 matrix tiles");
        static_assert(PIPE != 4 || (WM == 2 && WN == 4 && TM == 8 && TN == 4), "checked for eight waves of 128 x 64 only");
        constexpr uint32_t kASlot = T::kAFrags * 2048;
        constexpr int kQA2 = 2 * T::kAFrags / T::kWaves;  // A requests per wave and tile pair
        static_assert(3 * kASlot == (uint32_t)T::kLdsBytes, "LDS layout");
        uint32_t offA[kQA2], offB[TN];
#pragma unroll
        for (int q = 0; q < kQA2; ++q) {
            const uint32_t b = wave + q * T::kWaves;  // block of 8 rows
            uint32_t row = m0 + b * 8 + (lane >> 3);
            row = row < a.M ? row : a.M - 1;
            const uint32_t row16 = (b & 1) * 8 + (lane >> 3);
            offA[q] = row * a.lda + (((lane & 7) ^ ((row16 >> 1) & 7)) * 16);
        }
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            uint32_t nb = (n0 >> 4) + wn * TN + y;
            nb = nb < nblocks ? nb : nblocks - 1;
            offB[y] = nb * 16 * K + lane * 16;
        }
        const uint32_t ksteps = K / 64, kpairs = ksteps / 2;  // the launcher checks K % 128 == 0
        const uint32_t rdA = (i >> 3) * 1024 + ((i & 7) * 8 + (g ^ ((i >> 1) & 7))) * 16;
#define BG4_ISSUE_A(aslot, pair)                                                                                  \
    {                                                                                                             \
        const uint8_t *base_ = a.A + (size_t)((pair) < kpairs ? (pair) : kpairs - 1) * 128;                       \
        _Pragma("unroll") for (int q = 0; q < kQA2; ++q)                                                          \
        {                                                                                                         \
            __builtin_amdgcn_global_load_lds((gptr_t)(base_ + offA[q]),                                           \
                (lptr_t)(smem + (aslot)*kASlot + (wave + q * T::kWaves) * 1024), 16, 0, 0);                       \
        }                                                                                                         \
    }
#define BG4_LOAD_B(FB, tile)                                                                                      \
    {                                                                                                             \
        const uint8_t *base_ = (const uint8_t *)a.Bp + (size_t)((tile) < ksteps ? (tile) : ksteps - 1) * 1024;    \
        _Pragma("unroll") for (int y = 0; y < TN; ++y)                                                            \
        {                                                                                                         \
            /* issued as text, so that the compiler's own wait insertion does not see these loads: next to the */ \
            /* LDS-bound requests it would wait for ALL outstanding memory operations before the first use.   */ \
            /* The waits are the explicit vmcnt counts below; nothing reads FB between a load and its wait.    */ \
            /* 32-bit lane offset + wave-uniform 64-bit base in scalar registers: no per-lane address arithmetic */ \
            asm volatile("global_load_dwordx4 %0, %1, %2" : "=&v"(FB[y]) : "v"(offB[y]), "s"(base_) : "memory");  \
        }                                                                                                         \
    }
        // Request order: A0 B0 A1 B1 B2 | tile 0: A2 .. B3 | tile 1: .. B4 | tile 2: A3 .. B5 | ... : the even tile t
        // requests pair t / 2 + 2 in its memory phase, every tile t loads B(t + 3) after its MFMAs into the register
        // set it has just consumed. Behind the request of a pair come B, B, the next pair and one more B before the
        // odd tile that first needs it starts: 2 * kQA2... = kQA2 + 3 * TN requests may then still be outstanding.
        v4i fb0[TN], fb1[TN], fb2[TN], fa[TM];
        BG4_ISSUE_A(0u, 0u);
        BG4_LOAD_B(fb0, 0u);
        BG4_ISSUE_A(1u, 1u);
        BG4_LOAD_B(fb1, 1u);
        BG4_LOAD_B(fb2, 2u);
        const bool late = wave >= 4;
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kQA2 + 2 * TN));  // pair 0 (and B0) landed
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (late) {
            __builtin_amdgcn_s_barrier();
        }
#define BG4_STEP(HALF, FB)                                                                                        \
    {                                                                                                             \
        if (HALF) {                                                                                               \
            __builtin_amdgcn_s_waitcnt(vmcnt_imm(kQA2 + 3 * TN)); /* the pair of tile t + 1 has landed */          \
            asm volatile("" ::: "memory");                                                                        \
        } else {                                                                                                  \
            BG4_ISSUE_A(aslot_req, t / 2 + 2);                                                                    \
        }                                                                                                         \
        {                                                                                                         \
            const uint8_t *sA_ = smem + aslot * kASlot + (rdA ^ ((HALF)*64));                                     \
            _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                        \
            {                                                                                                     \
                fa[x] = *(const v4i *)(sA_ + (wm * TM + x) * 2048);                                               \
            }                                                                                                     \
        }                                                                                                         \
        __builtin_amdgcn_s_waitcnt(0xc07f);                                                                       \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                            \
        {                                                                                                         \
            fa[x] ^= flip;                                                                                        \
        }                                                                                                         \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_s_barrier();                                                                             \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        /* B(t), loaded three tiles ago, is in its registers: behind it came B, a pair and B (in some order) */  \
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(kQA2 + 2 * TN));                                                     \
        asm volatile("" : "+v"(FB[0]), "+v"(FB[1]), "+v"(FB[2]), "+v"(FB[3]));                                    \
        __builtin_amdgcn_s_setprio(1);                                                                            \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                                            \
        {                                                                                                         \
            _Pragma("unroll") for (int y = 0; y < TN; ++y)                                                        \
            {                                                                                                     \
                acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(FB[y], fa[x], acc[x][y], 0, 0, 0);              \
            }                                                                                                     \
        }                                                                                                         \
        __builtin_amdgcn_s_setprio(0);                                                                            \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        BG4_LOAD_B(FB, t + 3);                                                                                    \
        __builtin_amdgcn_sched_barrier(0);                                                                        \
        asm volatile("" ::: "memory");                                                                            \
        __builtin_amdgcn_s_barrier();                                                                             \
        asm volatile("" ::: "memory");                                                                            \
    }
#define BG4_PAIR(FBE, FBO)                                                                                        \
    {                                                                                                             \
        BG4_STEP(0, FBE);                                                                                         \
        ++t;                                                                                                      \
        BG4_STEP(1, FBO);                                                                                         \
        ++t;                                                                                                      \
        aslot = aslot == 2 ? 0 : aslot + 1;                                                                       \
        aslot_req = aslot_req == 2 ? 0 : aslot_req + 1;                                                           \
    }
        uint32_t aslot = 0, aslot_req = 2;  // slot of the pair being read / of the pair requested at the even tile
        uint32_t t = 0;
        while (t + 6 <= ksteps) {  // the register ring comes round every three tiles, the A halves every two
            BG4_PAIR(fb0, fb1);
            BG4_PAIR(fb2, fb0);
            BG4_PAIR(fb1, fb2);
        }
        if (t + 2 <= ksteps) {
            BG4_PAIR(fb0, fb1);
        }
        if (t + 2 <= ksteps) {
            BG4_PAIR(fb2, fb0);
        }
        if (!late) {
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the clamped refetches
        // The last loads of every register set are never consumed. Their destinations must stay allocated until the
        // data has landed (the drain above): a register the compiler handed to something else in between -- an
        // address, an accumulator -- would be overwritten when the load returns.
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            asm volatile("" ::"v"(fb0[y]), "v"(fb1[y]), "v"(fb2[y]));
        }
#undef BG4_PAIR
#undef BG4_STEP
#undef BG4_LOAD_B
#undef BG4_ISSUE_A
    } else {
    // This wave's fragments per K tile: kQA A fragments (16 rows x 64 K-bytes), then B fragments.
    // Addresses are split into a wave-uniform 64-bit base that advances with the tile (scalar
    // registers, scalar ALU) and a 32-bit per-lane offset that never changes, so the loop issues
    // its loads without any per-lane 64-bit arithmetic.
    constexpr int kQA = T::kAFrags / T::kWaves;
    static_assert(T::kAFrags % T::kWaves == 0, "A fragments must divide evenly over the waves");
    uint32_t off[T::kLoads];
#pragma unroll
    for (int q = 0; q < T::kLoads; ++q) {
        if (q < kQA) {
            uint32_t row = m0 + (wave + q * T::kWaves) * 16 + i;
            row = row < a.M ? row : a.M - 1;
            if (CONV) {
                // implicit GEMM: row = output pixel; its receptive field starts at this offset of the
                // padded s8 image (planes of 16 channels); the tap / channel-plane offset comes per K tile
                const uint32_t img = row / a.conv.OHW, r = row % a.conv.OHW;
                const uint32_t oy = r / a.conv.OW, ox = r % a.conv.OW;
                off[q] = ((img * (a.conv.ICp / 16) * a.conv.Hp + oy * a.conv.sh) * a.conv.Wp + ox * a.conv.sw) * 16;
            } else {
                // lane 4 r + c asks for 16 bytes of row r: the four lanes of a quad cover 64 contiguous bytes, which the
                // address unit takes as one piece (with lane = 16 g + i, a lane per row, every lane is a piece of its
                // own and a request takes several times longer to be accepted). Chunk c ^ (r / 4 % 4) rather than c,
                // so that the fragment read below, 16 lanes = 16 rows of one chunk, spreads over all banks.
                const uint32_t r4 = lane >> 2;
                uint32_t rowq = m0 + (wave + q * T::kWaves) * 16 + r4;
                rowq = rowq < a.M ? rowq : a.M - 1;
                off[q] = rowq * a.lda + (((lane & 3) ^ ((r4 >> 2) & 3)) * 16);
            }
        } else {
            uint32_t nb = (n0 >> 4) + (wave + (q - kQA) * T::kWaves);
            nb = nb < nblocks ? nb : nblocks - 1;
            off[q] = nb * 16 * K + lane * 16;
        }
    }
    const uint32_t ksteps = K / 64;
    // where lane (i, g) finds chunk g of row i inside a 1 KB A fragment in LDS (see the request layout above)
    const uint32_t a_rd = CONV ? lane * 16 : i * 64 + ((g ^ ((i >> 2) & 3)) * 16);

// slot: which LDS buffer (slot % STAGES); tile: which K tile to fetch. Past the end of K the
// schedule keeps issuing (slot advances, tile is clamped to the last one) so that the number of
// loads in flight, and with it every vmcnt wait, is the same in every step; the refetched tile
// lands in a buffer nobody reads any more.
#define BG_ISSUE(slot, tile, aoff)                                                                       \
    {                                                                                                    \
        uint8_t *st_ = smem + ((slot) % STAGES) * T::kStageBytes;                                        \
        _Pragma("unroll") for (int q = 0; q < T::kLoads; ++q)                                            \
        {                                                                                                \
            const uint8_t *base_ = (q < kQA) ? a.A + (aoff) : (const uint8_t *)a.Bp + (size_t)(tile)*1024;          \
            const int f_ = (q < kQA) ? (wave + q * T::kWaves) : (T::kAFrags + wave + (q - kQA) * T::kWaves);       \
            __builtin_amdgcn_global_load_lds((gptr_t)(base_ + off[q]), (lptr_t)(st_ + f_ * 1024), 16, 0, 0);         \
        }                                                                                                \
    }
#define BG_CLAMP(tile) ((tile) < ksteps ? (tile) : ksteps - 1)
// Offset of K tile `tile` inside an A row: 64 bytes per tile for a matrix (scalar). For a
// convolution K runs over (kh, kw, c) in 16-channel chunks and this lane's K-group g covers chunk
// 4 * tile + g; its (kh, kw, c16) is carried in registers and stepped by four chunks per tile --
// a table in memory would put a vector load, and with it a wait on every tile fetch in flight,
// into each step. Chunks past the last tap (K padded to 64) read the pixel base; their weights are 0.
#define BG_AOFF(tile) ((size_t)(tile)*64)
    static_assert(!CONV || PIPE == 1 || PIPE == 2, "the convolution walk is wired into the fragment-prefetch and ping-pong loops");
    uint32_t cv_c16 = 0, cv_kw = 0, cv_kh = 0;
    const uint32_t cv_cpc = CONV ? a.conv.ICp / 16 : 1;
    if (CONV) {
        const uint32_t tap = g / cv_cpc;
        cv_c16 = g % cv_cpc;
        cv_kh = tap / a.conv.fw;
        cv_kw = tap % a.conv.fw;
    }
#define BG_CV_OFF()                                                                                            \
    ((cv_kh < a.conv.fh) ? (size_t)(((cv_c16 * a.conv.Hp + cv_kh * a.conv.dh) * a.conv.Wp + cv_kw * a.conv.dw) * 16) \
                         : (size_t)0)
#define BG_CV_ADVANCE()                                      \
    {                                                        \
        cv_c16 += 4;                                         \
        _Pragma("unroll") for (int w_ = 0; w_ < 4; ++w_)     \
        {                                                    \
            const bool wr_ = cv_c16 >= cv_cpc;               \
            cv_c16 -= wr_ ? cv_cpc : 0u;                     \
            cv_kw += wr_ ? 1u : 0u;                          \
            const bool w2_ = cv_kw >= a.conv.fw;             \
            cv_kw = w2_ ? 0u : cv_kw;                        \
            cv_kh += w2_ ? 1u : 0u;                          \
        }                                                    \
    }

#pragma unroll
    for (int s = 0; s < (PIPE == 8 ? 0 : STAGES - 1); ++s) {
        BG_ISSUE((uint32_t)s, BG_CLAMP((uint32_t)s), (CONV ? BG_CV_OFF() : BG_AOFF(BG_CLAMP((uint32_t)s))));
        if (CONV && (uint32_t)s + 1 < ksteps) {
            BG_CV_ADVANCE();
        }
    }
    if constexpr (PIPE == 0) {
        for (uint32_t t = 0; t < ksteps; ++t) {
            // tile t is the oldest batch in flight; up to STAGES-2 younger ones may stay outstanding
            if (t + (STAGES - 2) < ksteps) {
                __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * T::kLoads));
            } else {
                __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
            }
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            if (t + (STAGES - 1) < ksteps) {
                BG_ISSUE(t + (STAGES - 1), t + (STAGES - 1), BG_AOFF(t + (STAGES - 1)));
            }
            const uint8_t *sA = smem + (t % STAGES) * T::kStageBytes;
            const uint8_t *sB = sA + T::kAFrags * 1024;
            v4i fb[TN];
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                fb[y] = *(const v4i *)(sB + (wn * TN + y) * 1024 + lane * 16);
            }
#pragma unroll
            for (int x = 0; x < TM; ++x) {
                v4i fa = *(const v4i *)(sA + (wm * TM + x) * 1024 + a_rd);
                if (!CONV) {
                    fa ^= flip;
                }
#pragma unroll
                for (int y = 0; y < TN; ++y) {
                    acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[y], fa, acc[x][y], 0, 0, 0);  // B first: transposed accumulator
                }
            }
        }
    } else if constexpr (PIPE == 2) {
        // Ping-pong schedule for 8 waves = two per SIMD. Each K tile is split into a memory phase
        // (wait for the tile after next, request a new tile, read this tile's fragments from LDS,
        // re-bias A) and a matrix phase (the TM x TN MFMAs and nothing else), with an s_barrier after
        // each. Waves 4-7 run half a tile behind waves 0-3 (one extra barrier up front, one at the
        // end for the others), so on every SIMD one wave is in its matrix phase while the other is in
        // its memory phase: the matrix pipe never waits for loads, LDS or VALU work of the same wave.
        //   visibility: a wave waits for its share of tile t+1 at the start of its memory phase t and
        //   passes a barrier before any wave reads tile t+1 (memory phase t+1);
        //   reuse: tile t+STAGES-1 is requested in memory phase t into the slot of tile t-1, whose
        //   last readers (the late group's memory phase t-1) finished before the barrier just passed.
        // Every wave executes 2 + 2 * ksteps barriers.
        static_assert(WM * WN == 8, "ping-pong needs two waves per SIMD");
        static_assert(STAGES >= 3, "ping-pong needs at least 3 stages");
        v4i fa[TM], fb[TN];
        const bool late = wave >= 4;
        size_t pp_aoff = CONV ? BG_CV_OFF() : 0;  // convolution: offset of the next tile to request (the walk is one ahead)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * T::kLoads));  // tile 0 landed
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        if (late) {
            __builtin_amdgcn_s_barrier();
        }
        for (uint32_t t = 0; t < ksteps; ++t) {
            // ---- memory phase
            __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * T::kLoads));  // my share of tile t+1 landed
            asm volatile("" ::: "memory");
            BG_ISSUE(t + (STAGES - 1), BG_CLAMP(t + (STAGES - 1)), (CONV ? pp_aoff : BG_AOFF(BG_CLAMP(t + (STAGES - 1)))));
            if (CONV) {
                if (t + STAGES < ksteps) {
                    BG_CV_ADVANCE();
                }
                pp_aoff = BG_CV_OFF();
            }
            {
                const uint8_t *sA_ = smem + (t % STAGES) * T::kStageBytes;
                const uint8_t *sB_ = sA_ + T::kAFrags * 1024;
#pragma unroll
                for (int y = 0; y < TN; ++y) {
                    fb[y] = *(const v4i *)(sB_ + (wn * TN + y) * 1024 + lane * 16);
                }
#pragma unroll
                for (int x = 0; x < TM; ++x) {
                    fa[x] = *(const v4i *)(sA_ + (wm * TM + x) * 1024 + a_rd);
                }
            }
            __builtin_amdgcn_s_waitcnt(0xc07f);  // lgkmcnt(0): fragments in registers before the matrix phase
            if (!CONV) {  // a convolution's image is already s8
#pragma unroll
                for (int x = 0; x < TM; ++x) {
                    fa[x] ^= flip;
                }
            }
            __builtin_amdgcn_sched_barrier(0);  // the re-bias belongs to the memory phase
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
            __builtin_amdgcn_sched_barrier(0);
            // ---- matrix phase
            __builtin_amdgcn_s_setprio(1);
#pragma unroll
            for (int x = 0; x < TM; ++x) {
#pragma unroll
                for (int y = 0; y < TN; ++y) {
                    if constexpr (FP4) {
                        const v8i b8 = {fb[y].x, fb[y].y, fb[y].z, fb[y].w, 0, 0, 0, 0};
                        const v8i a8 = {fa[x].x, fa[x].y, fa[x].z, fa[x].w, 0, 0, 0, 0};
                        const v4f c = __builtin_bit_cast(v4f, acc[x][y]);
                        // cbsz = blgp = 4: both operands E2M1; block scales 2^0 (E8M0 127)
                        acc[x][y] = __builtin_bit_cast(v4i,
                            __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(b8, a8, c, 4, 4, 0, 127, 0, 127));
                    } else {
                        acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[y], fa[x], acc[x][y], 0, 0, 0);
                    }
                }
            }
            __builtin_amdgcn_s_setprio(0);
            __builtin_amdgcn_sched_barrier(0);
            asm volatile("" ::: "memory");
            __builtin_amdgcn_s_barrier();
            asm volatile("" ::: "memory");
        }
        if (!late) {
            __builtin_amdgcn_s_barrier();
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the clamped refetches
    } else if constexpr (PIPE == 8) {
        // Two groups of four waves on one 128 x 128 tile, each running the pinned-order loop of PIPE 7 over every other
        // K tile in a stage ring of its own: every SIMD then holds two waves whose MFMAs fill each other's issue
        // gaps, without a second workgroup (these grids have fewer tiles than the part has CUs). The partial
        // sums meet in LDS after the loop (integer sums: the order does not matter) and group 0 runs the epilogue.
        static_assert(!CONV && !FP4 && STAGES >= 3, "matrix product only");
        static_assert(T::kLoads + TM + TN + TM <= TM * TN, "one slot behind each MFMA");
        uint8_t *ring = smem + gidx * T::kLdsBytes;
        const uint32_t gsteps = ksteps / 2;  // the launcher only comes here with an even number of K tiles
        v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
#define BG8_TILE(j) (2 * ((j) < gsteps ? (j) : gsteps - 1) + gidx) /* K tile of this group's step j, clamped */
#define BG8_REQ(slot_, j_)                                                                   \
    {                                                                                        \
        uint8_t *st_ = ring + ((slot_) % STAGES) * T::kStageBytes;                           \
        const uint32_t tl_ = BG8_TILE(j_);                                                   \
        _Pragma("unroll") for (int q = 0; q < T::kLoads; ++q)                                \
        {                                                                                    \
            const uint8_t *base_ = (q < kQA) ? a.A + (size_t)tl_ * 64 : (const uint8_t *)a.Bp + (size_t)tl_ * 1024; \
            const int f_ = (q < kQA) ? (wave + q * T::kWaves) : (T::kAFrags + wave + (q - kQA) * T::kWaves); \
            __builtin_amdgcn_global_load_lds((gptr_t)(base_ + off[q]), (lptr_t)(st_ + f_ * 1024), 16, 0, 0); \
        }                                                                                    \
    }
#define BG8_STEP(tt, FA, FB, NA, NB)                                                         \
    {                                                                                        \
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * T::kLoads) & 0xf0ff);            \
        asm volatile("" ::: "memory");                                                       \
        __builtin_amdgcn_s_barrier();                                                        \
        asm volatile("" ::: "memory");                                                       \
        const uint32_t rd_ = ((tt) + 1 < gsteps ? (tt) + 1 : gsteps - 1) % STAGES;           \
        const uint8_t *rA_ = ring + rd_ * T::kStageBytes + wm * TM * 1024 + a_rd;            \
        const uint8_t *rB_ = ring + rd_ * T::kStageBytes + (T::kAFrags + wn * TN) * 1024 + lane * 16; \
        uint8_t *st_ = ring + (((tt) + (STAGES - 1)) % STAGES) * T::kStageBytes;             \
        const uint32_t tl_ = BG8_TILE((tt) + (STAGES - 1));                                  \
        __builtin_amdgcn_sched_barrier(0);                                                   \
        _Pragma("unroll") for (int m = 0; m < TM * TN; ++m)                                  \
        {                                                                                    \
            acc[m / TN][m % TN] = __builtin_amdgcn_mfma_i32_16x16x64_i8(FB[m % TN], FA[m / TN], acc[m / TN][m % TN], 0, 0, 0); \
            if (m < TM) {                                                                    \
                NA[m] = *(const v4i *)(rA_ + m * 1024);                                      \
            } else if (m < TM + TN) {                                                        \
                NB[m - TM] = *(const v4i *)(rB_ + (m - TM) * 1024);                          \
            } else if (m < TM + TN + T::kLoads) {                                            \
                const int q = m - TM - TN;                                                   \
                const uint8_t *base_ = (q < kQA) ? a.A + (size_t)tl_ * 64 : (const uint8_t *)a.Bp + (size_t)tl_ * 1024; \
                const int f_ = (q < kQA) ? (wave + q * T::kWaves) : (T::kAFrags + wave + (q - kQA) * T::kWaves); \
                __builtin_amdgcn_global_load_lds((gptr_t)(base_ + off[q]), (lptr_t)(st_ + f_ * 1024), 16, 0, 0); \
            } else if (m >= TM * TN - TM) {                                                  \
                NA[m - (TM * TN - TM)] ^= flip;                                              \
            }                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                               \
        }                                                                                    \
    }
        // (the shared prologue above requested tiles 0 .. STAGES-2 into the first ring for everybody: redo it per group)
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int s_ = 0; s_ < STAGES - 1; ++s_) {
            BG8_REQ((uint32_t)s_, (uint32_t)s_);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * T::kLoads));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            fb0[y] = *(const v4i *)(ring + (T::kAFrags + wn * TN + y) * 1024 + lane * 16);
        }
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            fa0[x] = *(const v4i *)(ring + (wm * TM + x) * 1024 + a_rd) ^ flip;
        }
        uint32_t t = 0;
        for (; t + 1 < gsteps; t += 2) {
            BG8_STEP(t, fa0, fb0, fa1, fb1);
            BG8_STEP(t + 1, fa1, fb1, fa0, fb0);
        }
        if (t < gsteps) {
            BG8_STEP(t, fa0, fb0, fa1, fb1);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();  // nobody reads fragments any more: the rings are free
        asm volatile("" ::: "memory");
        {   // group 1 hands its partial sums over: register r of lane l of wave w at ((w * TM * TN + r) * 64 + l) * 16
            v4i *xch = (v4i *)smem + (size_t)wave * (TM * TN) * 64 + lane;
            if (gidx == 1) {
#pragma unroll
                for (int x = 0; x < TM; ++x) {
#pragma unroll
                    for (int y = 0; y < TN; ++y) {
                        xch[(x * TN + y) * 64] = acc[x][y];
                    }
                }
            }
            __syncthreads();
            if (gidx == 0) {
#pragma unroll
                for (int x = 0; x < TM; ++x) {
#pragma unroll
                    for (int y = 0; y < TN; ++y) {
                        acc[x][y] += xch[(x * TN + y) * 64];
                    }
                }
            }
        }
#undef BG8_STEP
#undef BG8_REQ
#undef BG8_TILE
    } else if constexpr (PIPE == 7) {
        // Fragment prefetch as below, with the program order of a K step written out and pinned: a wave that is alone
        // on its SIMD overlaps nothing by itself, and whatever stands in front of the first MFMA of a step runs with
        // the matrix pipe idle. Here each fragment read, tile request and re-bias sits behind an MFMA and issues while
        // that MFMA executes; the re-bias is applied when a fragment arrives, one step ahead of its use.
        static_assert(!CONV && !FP4 && STAGES >= 3, "matrix product only");
        static_assert(T::kLoads + TM + TN + TM <= TM * TN, "one slot behind each MFMA");
        v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
#define BG7_STEP(tt, FA, FB, NA, NB)                                                         \
    {                                                                                        \
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * T::kLoads) & 0xf0ff);            \
        asm volatile("" ::: "memory");                                                       \
        __builtin_amdgcn_s_barrier();                                                        \
        asm volatile("" ::: "memory");                                                       \
        const uint8_t *rA_ = smem + (BG_CLAMP((tt) + 1) % STAGES) * T::kStageBytes + wm * TM * 1024 + a_rd; \
        const uint8_t *rB_ = smem + (BG_CLAMP((tt) + 1) % STAGES) * T::kStageBytes + (T::kAFrags + wn * TN) * 1024 + lane * 16; \
        uint8_t *st_ = smem + (((tt) + (STAGES - 1)) % STAGES) * T::kStageBytes;             \
        const uint32_t tl_ = BG_CLAMP((tt) + (STAGES - 1));                                  \
        __builtin_amdgcn_sched_barrier(0);                                                   \
        _Pragma("unroll") for (int m = 0; m < TM * TN; ++m)                                  \
        {                                                                                    \
            acc[m / TN][m % TN] = __builtin_amdgcn_mfma_i32_16x16x64_i8(FB[m % TN], FA[m / TN], acc[m / TN][m % TN], 0, 0, 0); \
            if (m < TM) {                                                                    \
                NA[m] = *(const v4i *)(rA_ + m * 1024);                                      \
            } else if (m < TM + TN) {                                                        \
                NB[m - TM] = *(const v4i *)(rB_ + (m - TM) * 1024);                          \
            } else if (m < TM + TN + T::kLoads) {                                            \
                const int q = m - TM - TN;                                                   \
                const uint8_t *base_ = (q < kQA) ? a.A + aoff_next : (const uint8_t *)a.Bp + (size_t)tl_ * 1024; \
                const int f_ = (q < kQA) ? (wave + q * T::kWaves) : (T::kAFrags + wave + (q - kQA) * T::kWaves); \
                __builtin_amdgcn_global_load_lds((gptr_t)(base_ + off[q]), (lptr_t)(st_ + f_ * 1024), 16, 0, 0); \
            } else if (m >= TM * TN - TM) {                                                  \
                NA[m - (TM * TN - TM)] ^= flip; /* the reads are 4+ MFMAs old by now */       \
            }                                                                                \
            __builtin_amdgcn_sched_barrier(0);                                               \
        }                                                                                    \
        aoff_next = BG_AOFF(BG_CLAMP((tt) + STAGES));                                        \
    }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * T::kLoads));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int y = 0; y < TN; ++y) {
            fb0[y] = *(const v4i *)(smem + (T::kAFrags + wn * TN + y) * 1024 + lane * 16);
        }
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            fa0[x] = *(const v4i *)(smem + (wm * TM + x) * 1024 + a_rd) ^ flip;
        }
        uint32_t t = 0;
        size_t aoff_next = BG_AOFF(BG_CLAMP(t + (STAGES - 1)));
        for (; t + 1 < ksteps; t += 2) {
            BG7_STEP(t, fa0, fb0, fa1, fb1);
            BG7_STEP(t + 1, fa1, fb1, fa0, fb0);
        }
        if (t < ksteps) {
            BG7_STEP(t, fa0, fb0, fa1, fb1);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));
#undef BG7_STEP
    } else {
        // Fragment-prefetch schedule: the fragments of tile t+1 are read from LDS into a second
        // register set while the MFMAs of tile t run, so no MFMA ever waits for an LDS read. That
        // needs tile t+1 landed before step t starts: one tile more "landed ahead" than above.
        static_assert(STAGES >= 3, "fragment prefetch needs at least 3 stages");
        v4i fa0[TM], fb0[TN], fa1[TM], fb1[TN];
#define BG_READ_FRAGS(tile, FA, FB)                                                          \
    {                                                                                        \
        const uint8_t *sA_ = smem + ((tile) % STAGES) * T::kStageBytes;                      \
        const uint8_t *sB_ = sA_ + T::kAFrags * 1024;                                        \
        _Pragma("unroll") for (int y = 0; y < TN; ++y)                                       \
        {                                                                                    \
            FB[y] = *(const v4i *)(sB_ + (wn * TN + y) * 1024 + lane * 16);                  \
        }                                                                                    \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                       \
        {                                                                                    \
            FA[x] = *(const v4i *)(sA_ + (wm * TM + x) * 1024 + a_rd); /* raw u8 */           \
        }                                                                                    \
    }
#define BG_STEP(tt, FA, FB, NA, NB)                                                          \
    {                                                                                        \
        /* this wave's share of tile tt+1 has landed (younger tiles may stay in flight), and */ \
        /* the fragment reads issued one step ago (FA / FB) are complete                     */ \
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 3) * T::kLoads) & 0xf0ff);            \
        asm volatile("" ::: "memory");                                                       \
        __builtin_amdgcn_s_barrier();                                                        \
        asm volatile("" ::: "memory");                                                       \
        BG_ISSUE((tt) + (STAGES - 1), BG_CLAMP((tt) + (STAGES - 1)), aoff_next);             \
        if (CONV) {                                                                          \
            if ((tt) + STAGES < ksteps) {                                                    \
                BG_CV_ADVANCE();                                                             \
            }                                                                                \
            aoff_next = BG_CV_OFF();                                                         \
        } else {                                                                             \
            aoff_next = BG_AOFF(BG_CLAMP((tt) + STAGES));                                    \
        }                                                                                    \
        BG_READ_FRAGS(BG_CLAMP((tt) + 1), NA, NB);                                           \
        _Pragma("unroll") for (int x = 0; x < TM; ++x)                                       \
        {                                                                                    \
            const v4i fx_ = CONV ? FA[x] : (FA[x] ^ flip); /* re-bias at use: the read stays in flight */ \
            _Pragma("unroll") for (int y = 0; y < TN; ++y)                                   \
            {                                                                                \
                acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(FB[y], fx_, acc[x][y], 0, 0, 0); \
            }                                                                                \
        }                                                                                    \
        /* issue order for the scheduler: the tile fetches first, then one LDS fragment read */ \
        /* slipped in after every second MFMA, so the reads ride under the matrix pipeline   */ \
        __builtin_amdgcn_sched_group_barrier(0x020, T::kLoads, 0);                           \
        _Pragma("unroll") for (int r_ = 0; r_ < TM + TN; ++r_)                               \
        {                                                                                    \
            __builtin_amdgcn_sched_group_barrier(0x008, 2, 0);                               \
            __builtin_amdgcn_sched_group_barrier(0x100, 1, 0);                               \
        }                                                                                    \
        __builtin_amdgcn_sched_group_barrier(0x008, (TM * TN > 2 * (TM + TN)) ? TM * TN - 2 * (TM + TN) : 0, 0); \
    }
        // tile 0 landed everywhere
        __builtin_amdgcn_s_waitcnt(vmcnt_imm((STAGES - 2) * T::kLoads));
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
        BG_READ_FRAGS(0u, fa0, fb0);
        size_t aoff_next = CONV ? BG_CV_OFF() : BG_AOFF(BG_CLAMP((uint32_t)(STAGES - 1)));
        uint32_t t = 0;
        for (; t + 1 < ksteps; t += 2) {
            BG_STEP(t, fa0, fb0, fa1, fb1);
            BG_STEP(t + 1, fa1, fb1, fa0, fb0);
        }
        if (t < ksteps) {  // odd tile count: the register sets are back in their initial roles
            BG_STEP(t, fa0, fb0, fa1, fb1);
        }
        __builtin_amdgcn_s_waitcnt(vmcnt_imm(0));  // drain the clamped refetches before the buffers are reused
#undef BG_STEP
#undef BG_READ_FRAGS
    }
#undef BG_ISSUE
#undef BG_CLAMP
#undef BG_AOFF
#undef BG_CV_OFF
#undef BG_CV_ADVANCE
    }  // PIPE != 3
    asm volatile("" ::"v"(warm));  // keeps the warming loads alive; the value itself is not used
    if constexpr (FP4) {
        static_assert(!FP4 || PIPE == 2, "the fp4 product is wired into the ping-pong loop");
#pragma unroll
        for (int x = 0; x < TM; ++x) {
#pragma unroll
            for (int y = 0; y < TN; ++y) {
                const v4f c = __builtin_bit_cast(v4f, acc[x][y]);
                acc[x][y] = (v4i){(int)c.x, (int)c.y, (int)c.z, (int)c.w};  // exact: sums of +-1 and 0/1 products
            }
        }
    }
    if (!CONV) {
        // the matrix epilogue stages results through LDS: every wave's tile fetches have landed (each
        // drained its own above) and every wave has read its last fragments before anyone writes there
        static_assert(CONV || T::kLdsBytes >= WM * WN * 16 * 272, "LDS too small for the epilogue panels");
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
    }
    if (PIPE == 8 && gidx == 1) {
        return;  // its sums are in group 0's accumulators
    }
    if constexpr (GELU_DYN) {
        // the lane index formed afresh (from the execution mask) rather than kept in a register across the K loop: with the
        // register-B loop this instantiation has none to spare, and the loops with hand-counted loads must not spill
        const uint32_t lane_e = __builtin_amdgcn_mbcnt_hi(~0u, __builtin_amdgcn_mbcnt_lo(~0u, 0u));
        epilogue_gelu_sync<WM, WN, TM, TN>(a, acc, smem, lane_e, wave, m0, n0);
    } else {
        epilogue_panel<WM, WN, TM, TN, CONV>(a, acc, smem, lane, wave, m0, n0, T::kLdsBytes);
    }
}

// Convolution with few output channels (N <= 64) and a filter panel that fits in LDS (K <= 1024).
// With one 64-channel panel every wave's pixel rows are its own, so staging A through LDS buys nothing
// and the shared pipeline pays a barrier per K tile for it. Here the whole packed filter panel is
// fetched into LDS once per block (K x 64 bytes, fragment order), and after one barrier the four
// waves run independently: each owns TM x 16 pixels, gathers its A fragments from the padded image
// straight into registers three K tiles ahead (the compiler tracks those loads), reads the four B
// fragments of a tile from LDS and issues TM x 4 MFMAs. LDS traffic is a third of the shared
// pipeline's and there is no barrier inside the K loop.
//
// DIRECT: A is the caller's u8 tensor (NCHWC8 or NCHWC16) instead of the padded s8 image, so no padding pass runs
// before the kernel. A lane's 16 channels of a tap are one 16-byte load (NCHWC16) or two 8-byte loads from
// neighbouring channel blocks (NCHWC8); taps that fall outside the image, and the chunks that pad K to 64, read a
// constant block of 0x80 instead, and every fragment is re-biased (^ 0x80) before use, which turns those into the
// zeros the padded image holds.
__device__ __attribute__((aligned(16))) const uint8_t kConvPad128[16] = {128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128, 128};

template <int TM, bool DIRECT>
__global__ __launch_bounds__(256, 2) void conv_u8s8_panel_kernel(GemmArgs a)
{
    extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
    __shared__ int sync_lds[18];  // the one-pass u8 form's grid-wide maximum (the waves read the panel at their own pace)
    constexpr int P = 5;  // K tiles of A in flight per wave
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t m0 = blockIdx.x * (4 * TM * 16);
    const uint32_t K = a.K, ksteps = K / 64;
    const uint32_t nblocks = align_up(a.N, 16) >> 4;
    conv_publish_scale(a, wave);

    // the filter panel: fragment (tile t, column block y) at smem + (4 t + y) KiB
    for (uint32_t f = wave; f < 4 * ksteps; f += 4) {
        const uint32_t t = f >> 2, y = f & 3;
        const uint32_t nb = y < nblocks ? y : nblocks - 1;
        const uint8_t *src = (const uint8_t *)a.Bp + (size_t)nb * 16 * K + (size_t)t * 1024 + lane * 16;
        __builtin_amdgcn_global_load_lds((gptr_t)src, (lptr_t)(smem + f * 1024), 16, 0, 0);
    }

    // The loads below name the global address space: a pointer chosen between the image and the constant block would
    // otherwise be loaded from as a flat pointer, and flat loads cannot be counted in order, so every K tile would
    // wait for all the tiles requested after it as well.
    typedef const __attribute__((address_space(1))) uint8_t *gbytes_t;
    typedef const __attribute__((address_space(1))) v4i *gv4i_t;
    typedef const __attribute__((address_space(1))) v2i *gv2i_t;
    const gbytes_t gA = (gbytes_t)a.A, gPad = (gbytes_t)kConvPad128;
    const uint32_t cpc = a.conv.ICp / 16;  // 16-channel planes of the image
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
    const uint32_t ic_bytes = DIRECT ? a.conv.in_c : 16;  // bytes per pixel inside a channel block
    const uint32_t plane8 = a.conv.H * a.conv.W * 8;
    // ---- per-pixel terms ----------------------------------------------------------------------------------
    uint32_t off[TM];   // padded image: byte offset of the pixel's receptive field; DIRECT: of pixel (iy0, ix0), may be "negative"
    int32_t iy0[TM], ix0[TM];  // DIRECT: input row / column of tap (0, 0)
    auto pixel_terms = [&]() {
#pragma unroll
        for (int x = 0; x < TM; ++x) {
            uint32_t row = m0 + (wave * TM + x) * 16 + i;
            row = row < a.M ? row : a.M - 1;
            const uint32_t img = row / a.conv.OHW, r = row % a.conv.OHW;
            const uint32_t oy = r / a.conv.OW, ox = r % a.conv.OW;
            if (DIRECT) {
                iy0[x] = (int32_t)(oy * a.conv.sh) - (int32_t)a.conv.pt;
                ix0[x] = (int32_t)(ox * a.conv.sw) - (int32_t)a.conv.pl;
                off[x] = img * a.conv.IC * a.conv.H * a.conv.W +
                    (uint32_t)(iy0[x] * (int32_t)a.conv.W + ix0[x]) * ic_bytes;  // wraps for border pixels; used only when in range
            } else {
                off[x] = ((img * cpc * a.conv.Hp + oy * a.conv.sh) * a.conv.Wp + ox * a.conv.sw) * 16;
            }
        }
    };

    // ---- per-column terms of the epilogue ------------------------------------------------------------------------
    // offsetC - compensation with the bias folded in (column_base's arithmetic) and, for per-channel filter scales, the
    // reciprocal scale and the bias of each of the (at most 64) output channels: formed ONCE per workgroup by its first
    // 64 threads, while the filter panel and the first tiles are on their way, and parked in LDS; the barrier in front
    // of the K loop publishes them. The epilogue then reads its 16 entries per lane from there -- no loads from memory
    // and no double-precision rounding or division on the critical path behind the K loop, and no registers held
    // across it.
    __shared__ __attribute__((aligned(16))) uint32_t col_base[64];
    __shared__ __attribute__((aligned(16))) float col_qs[64], col_bs[64];
    auto column_terms = [&]() {
        if (threadIdx.x < 64) {
            const uint32_t n = threadIdx.x, nc = n < a.N ? n : a.N - 1;
            const float fold_scale_ = a.conv.dscaleI ? conv_acc_scale(a.conv) : a.fold_scale;
            col_base[n] = (n < a.N) ? column_base(a.ob, a.comp, a.fold_bias, fold_scale_, nc) : 0u;
            float q_ = 1.0f, b_ = 0.0f;
            if (a.epi.mode == EPI_CONV_CH) {
                const float sI_ = a.conv.dscaleI ? *a.conv.dscaleI : a.conv.scaleI;
                q_ = 1.0f / (sI_ * a.epi.scaleW[nc]);
                b_ = a.epi.bias ? a.epi.bias[nc] : 0.0f;
            }
            col_qs[n] = q_;
            col_bs[n] = b_;
        }
    };
    ColTerms pre_base;
    pre_base.base = col_base;
    if (a.epi.mode == EPI_CONV_CH) {
        pre_base.qs = col_qs;
        pre_base.bs = col_bs;
    }

    // this lane's K-group g covers 16-channel chunk 4 * tile + g; its (kh, kw, c16) is stepped in registers
    uint32_t c16 = g % cpc, kw = (g / cpc) % a.conv.fw, kh = (g / cpc) / a.conv.fw, at = 0;  // at: tile the walk points to
    auto tap_offset = [&]() -> uint32_t {
        if (DIRECT) {  // channel block(s) of chunk c16, then the tap's row / column inside the plane
            return ((16 / ic_bytes) * c16 * a.conv.H * a.conv.W + kh * a.conv.dh * a.conv.W + kw * a.conv.dw) * ic_bytes;
        }
        return (kh < a.conv.fh) ? ((c16 * a.conv.Hp + kh * a.conv.dh) * a.conv.Wp + kw * a.conv.dw) * 16 : 0u;
    };
    auto advance = [&]() {
        const uint32_t mv = (at + 1 < ksteps) ? 1u : 0u;  // past the last tile the walk stays put: the refetch is never used
        at += mv;
        c16 += 4 * mv;
#pragma unroll
        for (int w_ = 0; w_ < 4; ++w_) {
            const bool wr_ = c16 >= cpc;
            c16 -= wr_ ? cpc : 0u;
            kw += wr_ ? 1u : 0u;
            const bool w2_ = kw >= a.conv.fw;
            kw = w2_ ? 0u : kw;
            kh += w2_ ? 1u : 0u;
        }
    };

    v4i acc[TM][4];
    // The rest once per input layout (IN16: a pixel's 16 channels are one 16-byte access; else two 8-byte accesses to
    // neighbouring channel blocks) so that no branch separates the loads of a tile from each other. The main loop takes
    // P tiles per round with no condition inside: then the compiler counts the loads still in flight behind a tile's
    // own instead of waiting for all of them. Tiles past the end are requested again from the last tap and dropped.
    auto k_loop = [&](auto in16_tag) {
        constexpr bool IN16 = decltype(in16_tag)::value;
        // one fragment: the lane's 16 channels of pixel x at the current tap
        auto gather = [&](int x, uint32_t o) -> v4i {
            if (!DIRECT) {
                return *(gv4i_t)(gA + off[x] + o);
            }
            const uint32_t iy = (uint32_t)(iy0[x] + (int32_t)(kh * a.conv.dh)), ix = (uint32_t)(ix0[x] + (int32_t)(kw * a.conv.dw));
            const bool ok = kh < a.conv.fh && iy < a.conv.H && ix < a.conv.W;
            const gbytes_t p = ok ? gA + (uint32_t)(off[x] + o) : gPad;
            if (IN16) {
                return *(gv4i_t)p;
            }
            const gbytes_t p2 = ok ? p + plane8 : gPad;  // the next block of 8 channels
            const v2i lo = *(gv2i_t)p, hi = *(gv2i_t)p2;
            return (v4i){lo.x, lo.y, hi.x, hi.y};
        };
        v4i fa[P][TM];
        auto first_tiles = [&]() {
#pragma unroll
            for (int s_ = 0; s_ < P; ++s_) {
                const uint32_t o = tap_offset();
#pragma unroll
                for (int x = 0; x < TM; ++x) {
                    fa[s_][x] = gather(x, o);
                }
                advance();
            }
        };
        // order: the A tiles first (the long pole), the epilogue's column terms behind them, their arithmetic while
        // all of it is on its way
        pixel_terms();
        first_tiles();
        column_terms();
        __builtin_amdgcn_s_waitcnt(0);  // vmcnt(0) lgkmcnt(0): the panel (and the first A tiles) have landed, the column terms are written
        asm volatile("" ::: "memory");
        __builtin_amdgcn_s_barrier();
        asm volatile("" ::: "memory");
#pragma unroll
        for (int x = 0; x < TM; ++x) {
#pragma unroll
            for (int y = 0; y < 4; ++y) {
                acc[x][y] = (v4i){0, 0, 0, 0};
            }
        }
        auto tile = [&](uint32_t t, int u) {
            const uint8_t *sB = smem + (size_t)t * 4096 + lane * 16;
            v4i fb[4];
#pragma unroll
            for (int y = 0; y < 4; ++y) {
                fb[y] = *(const v4i *)(sB + y * 1024);
            }
#pragma unroll
            for (int x = 0; x < TM; ++x) {
                const v4i fx = DIRECT ? (fa[u][x] ^ flip) : fa[u][x];
#pragma unroll
                for (int y = 0; y < 4; ++y) {
                    acc[x][y] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb[y], fx, acc[x][y], 0, 0, 0);
                }
            }
        };
        uint32_t t = 0;
        for (; t + P <= ksteps; t += P) {
#pragma unroll
            for (int u = 0; u < P; ++u) {
                tile(t + u, u);
                const uint32_t o = tap_offset();
#pragma unroll
                for (int x = 0; x < TM; ++x) {
                    fa[u][x] = gather(x, o);
                }
                advance();
            }
        }
#pragma unroll
        for (int u = 0; u < P - 1; ++u) {  // what is left of K: its tiles were requested by the last full round
            if (t + u < ksteps) {
                tile(t + u, u);
            }
        }
    };
    if (a.conv.in_c == 16) {
        k_loop(std::true_type{});
    } else {
        k_loop(std::false_type{});
    }
    epilogue_panel<4, 1, TM, 4, true, true>(a, acc, (uint8_t *)sync_lds, lane, wave, m0, 0u, 0, pre_base);
}

// Skinny kernel for few rows (FullyConnected at small batch: M <= 64 per block, any N, K % 64 == 0).
// The weight panel is the traffic, so a block owns ONE 16-column panel of B for up to 64 rows of A and
// its 8 waves split K between them: each wave streams its K range straight from global memory / L2 into
// registers (B fragment = 1 KiB contiguous in the packed layout, A fragments = 16 rows x 64 bytes), one
// step ahead of the MFMAs, and the 8 partial accumulators meet in LDS. No barrier inside the K loop.
__global__ __launch_bounds__(512) void gemm_u8s8_skinny_kernel(GemmArgs a)
{
    __shared__ v4i part[7][4][64];
    const uint32_t lane = threadIdx.x & 63;
    const uint32_t wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t i = lane & 15, g = lane >> 4;
    const uint32_t n0 = blockIdx.x * 16, m0 = blockIdx.y * 64;
    const uint32_t ksteps = a.K / 64;
    const v4i flip = {(int)0x80808080, (int)0x80808080, (int)0x80808080, (int)0x80808080};
    // this wave's share of the K steps: a contiguous run
    const uint32_t per = (ksteps + 7) / 8;
    const uint32_t s0 = wave * per, s1 = (s0 + per < ksteps) ? s0 + per : ksteps;

    const uint8_t *ap[4];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        uint32_t row = m0 + x * 16 + i;
        row = row < a.M ? row : a.M - 1;  // rows past the end are computed and dropped
        ap[x] = a.A + (size_t)row * a.lda + g * 16;
    }
    const int8_t *bp = a.Bp + (size_t)(n0 >> 4) * 16 * a.K + lane * 16;

    v4i acc[4][1];
#pragma unroll
    for (int x = 0; x < 4; ++x) {
        acc[x][0] = (v4i){0, 0, 0, 0};
    }
    if (s0 < s1) {
        v4i fb = *(const v4i *)(bp + (size_t)s0 * 1024);
        v4i fa[4];
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            fa[x] = *(const v4i *)(ap[x] + (size_t)s0 * 64);
        }
        for (uint32_t s = s0; s < s1; ++s) {
            const uint32_t sn = (s + 1 < s1) ? s + 1 : s;  // the last step refetches itself: no branch around the loads
            const v4i nb = *(const v4i *)(bp + (size_t)sn * 1024);
            v4i na[4];
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                na[x] = *(const v4i *)(ap[x] + (size_t)sn * 64);
            }
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                acc[x][0] = __builtin_amdgcn_mfma_i32_16x16x64_i8(fb, fa[x] ^ flip, acc[x][0], 0, 0, 0);
            }
            fb = nb;
#pragma unroll
            for (int x = 0; x < 4; ++x) {
                fa[x] = na[x];
            }
        }
    }
    if (wave != 0) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            part[wave - 1][x][lane] = acc[x][0];
        }
    }
    __syncthreads();
    if (wave != 0) {
        return;
    }
#pragma unroll
    for (int w = 0; w < 7; ++w) {
#pragma unroll
        for (int x = 0; x < 4; ++x) {
            acc[x][0] += part[w][x][lane];
        }
    }
    epilogue_panel<1, 1, 4, 1>(a, acc, nullptr, lane, 0u, m0, n0, 0);
}

template <int WM, int WN, int TM, int TN, int STAGES, int PIPE = 0, bool CONV = false, bool FP4 = false, bool GELU_DYN = false>
static hipError_t launch_dma(const GemmArgs &a, hipStream_t st)
{
    using T = GemmDma<WM, WN, TM, TN, STAGES>;
    static bool attr_set = false;
    auto kern = gemm_u8s8_dma_kernel<WM, WN, TM, TN, STAGES, PIPE, CONV, FP4, GELU_DYN>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, T::kLdsBytes * (PIPE == 8 ? 2 : 1));
        if (e != hipSuccess) {
            return e;
        }
        attr_set = true;
    }
    const uint32_t tiles = ((a.N + T::kBN - 1) / T::kBN) * ((a.M + T::kBM - 1) / T::kBM);
    GemmArgs b = a;
    // a result much larger than the L2s (8 x 4 MiB) is written in several rounds of tiles: keep it from
    // displacing the operand panels (measured at 8192^3: 6 % faster; at 64 MiB and below: level or slower)
    b.stream_c = !CONV && (uint64_t)a.M * a.N * 4 > ((uint64_t)96 << 20);
    hipLaunchKernelGGL(kern, dim3(tiles), dim3(WM * WN * 64 * (PIPE == 8 ? 2 : 1)), T::kLdsBytes * (PIPE == 8 ? 2 : 1), st, b);
    return hipGetLastError();
}

template <int WM, int WN, int TM, int TN>
static hipError_t launch_tiled(const GemmArgs &a, hipStream_t st)
{
    using T = GemmTile<WM, WN, TM, TN>;
    static bool attr_set = false;
    auto kern = gemm_u8s8_tiled_kernel<WM, WN, TM, TN>;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)kern, hipFuncAttributeMaxDynamicSharedMemorySize, T::kLdsBytes);
        if (e != hipSuccess) {
            return e;
        }
        attr_set = true;
    }
    dim3 grid((a.N + T::kBN - 1) / T::kBN, (a.M + T::kBM - 1) / T::kBM);
    hipLaunchKernelGGL(kern, grid, dim3(WM * WN * 64), T::kLdsBytes, st, a);
    return hipGetLastError();
}

// whether a block may use 160 KB of LDS on the current device (asked once)
static bool lds_160k()
{
    static int have = -1;
    if (have < 0) {
        int dev = 0, bytes = 0;
        have = (hipGetDevice(&dev) == hipSuccess &&
                   hipDeviceGetAttribute(&bytes, hipDeviceAttributeMaxSharedMemoryPerBlock, dev) == hipSuccess && bytes >= 160 * 1024)
            ? 1
            : 0;
    }
    return have == 1;
}

static int g_conv_panel = 4;  // test hook: 0 = shared pipeline only, 2 / 4 = pixel blocks per wave of the panel kernel

void conv_force_panel(int v)
{
    g_conv_panel = v;
}

// the fp4 product exists in the 256 x 256 ping-pong instantiation only: take it where that kernel is the choice anyway
bool conv_fp4_ok(uint32_t M, uint32_t N)
{
    return N >= 256 && (uint64_t)((M + 255) / 256) * ((N + 255) / 256) >= 128;
}

bool conv_panel_ok(uint32_t N, uint32_t K)
{
    return N <= 64 && K % 64 == 0 && K <= 1024 && g_conv_panel != 0;
}

// Workgroups of the filter-panel kernel that are resident at once: two per CU where the kernel's registers and its
// K x 64 bytes of LDS allow (0 if the device cannot be asked), never more than a grid sync spans.
uint32_t conv_onepass_max_grid(uint32_t K)
{
    static int cus = -1, per_cu_regs = 0;
    if (cus < 0) {
        int dev = 0, n = 0, occ = 0;
        if (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess &&
            hipOccupancyMaxActiveBlocksPerMultiprocessor(&occ, conv_u8s8_panel_kernel<4, true>, 256, 65536) == hipSuccess) {
            cus = n;
            per_cu_regs = occ;  // with the largest panel (64 KB): a lower bound for smaller ones
        } else {
            cus = 0;
        }
    }
    (void)K;
    const uint32_t per_cu = per_cu_regs >= 2 ? 2u : (uint32_t)per_cu_regs;
    const uint32_t g = (uint32_t)cus * per_cu;
    return g > kGridSyncMaxBlocks ? kGridSyncMaxBlocks : g;
}

// the grid launch_conv_u8s8 gives the filter-panel kernel for M output pixels
uint32_t conv_panel_grid(uint32_t M)
{
    return (g_conv_panel == 2) ? (M + 127) / 128 : (M + 255) / 256;
}

// Implicit-GEMM convolution: same pipeline, A rows are output pixels gathered from the padded image.
hipError_t launch_conv_u8s8(const GemmArgs &a, hipStream_t st)
{
    if (a.M == 0 || a.N == 0) {
        return hipSuccess;
    }
    if (conv_panel_ok(a.N, a.K)) {
        // one filter panel, small enough to sit in LDS: no barrier in the K loop (see the kernel)
        static bool attr_set = false;
        if (!attr_set) {
            const void *kerns[4] = {(const void *)conv_u8s8_panel_kernel<2, false>, (const void *)conv_u8s8_panel_kernel<4, false>,
                (const void *)conv_u8s8_panel_kernel<2, true>, (const void *)conv_u8s8_panel_kernel<4, true>};
            for (const void *k : kerns) {
                hipError_t e = hipFuncSetAttribute(k, hipFuncAttributeMaxDynamicSharedMemorySize, 65536);
                if (e != hipSuccess) {
                    return e;
                }
            }
            attr_set = true;
        }
        const bool direct = a.conv.in_c != 0;
        const uint32_t grid = (g_conv_panel == 2) ? (a.M + 127) / 128 : (a.M + 255) / 256;
        if (a.sync.slots && (a.sync.blocks != grid || grid > conv_onepass_max_grid(a.K))) {
            return hipErrorInvalidValue;  // the one-pass form needs every workgroup resident at once
        }
        const uint32_t lds = a.K * 64;
        if (g_conv_panel == 2) {
            if (direct) {
                hipLaunchKernelGGL((conv_u8s8_panel_kernel<2, true>), dim3(grid), dim3(256), lds, st, a);
            } else {
                hipLaunchKernelGGL((conv_u8s8_panel_kernel<2, false>), dim3(grid), dim3(256), lds, st, a);
            }
        } else if (direct) {
            hipLaunchKernelGGL((conv_u8s8_panel_kernel<4, true>), dim3(grid), dim3(256), lds, st, a);
        } else {
            hipLaunchKernelGGL((conv_u8s8_panel_kernel<4, false>), dim3(grid), dim3(256), lds, st, a);
        }
        return hipGetLastError();
    }
    if (a.conv.in_c != 0) {
        return hipErrorInvalidValue;  // only the filter-panel kernel gathers from the caller's tensor
    }
    if (a.N <= 64) {
        // Few output channels: nowhere near MFMA-bound, the time is load latency, so what matters is
        // waves per CU and that the grid fits the chip in ONE round (every block lives about as long as
        // the whole kernel). 128-pixel blocks of 4 waves sit three to a CU (768 at once), 256-pixel
        // blocks two to a CU (512 at once).
        const uint32_t b128 = (a.M + 127) / 128, b256 = (a.M + 255) / 256;
        if (b128 <= 768 || b256 > 512) {
            return launch_dma<4, 1, 2, 4, 4, true, true>(a, st);
        }
        return launch_dma<4, 1, 4, 4, 4, true, true>(a, st);
    }
    if (a.fp4) {
        if (!conv_fp4_ok(a.M, a.N)) {
            return hipErrorInvalidValue;
        }
        return launch_dma<2, 4, 8, 4, 4, 2, true, true>(a, st);
    }
    if (a.N >= 256 && (uint64_t)((a.M + 255) / 256) * ((a.N + 255) / 256) >= 128) {
        return launch_dma<2, 4, 8, 4, 4, 2, true>(a, st);     // 256 pixels x 256 channels, ping-pong K loop
    }
    return launch_dma<2, 2, 8, 4, 4, true, true>(a, st);      // 256 pixels x 128 channels
}

static int g_force_tile = -1;  // test hook: -1 = heuristic

// Whether the GELU-and-quantise epilogue (EPI_U8_GELU_DYN) can run for this product: full 256 x 256 tiles of a pipelined
// kernel, few enough of them that each gets a CU of its own at once (160 KB of LDS per workgroup: one per CU).
bool gemm_gelu_dyn_fits(uint32_t M, uint32_t N, uint32_t K)
{
    static int cus = -1;
    if (cus < 0) {
        int dev = 0, n = 0;
        cus = (hipGetDevice(&dev) == hipSuccess && hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) == hipSuccess) ? n : 0;
    }
    if (M == 0 || N == 0 || M % 256 != 0 || N % 256 != 0 || K % 64 != 0 || K < 64) {
        return false;
    }
    const uint64_t tiles = (uint64_t)(M / 256) * (N / 256);
    return tiles >= 128 && tiles <= (uint64_t)cus && g_force_tile < 0;
}

void gemm_force_tile(int t)
{
    g_force_tile = t;
}

hipError_t launch_gemm_u8s8(const GemmArgs &a, hipStream_t st)
{
    if (a.M == 0 || a.N == 0) {
        return hipSuccess;
    }
    // the tiled kernels address both operands with 32-bit byte offsets from a 64-bit base: operands of 4 GiB and more go
    // to the general kernel, which indexes with 64 bits
    const bool fits32 = (uint64_t)a.M * a.lda < (1ull << 32) && (uint64_t)align_up(a.N, 16) * align_up(a.K, 8) < (1ull << 32);
    const bool tiled_ok = !a.transA && (a.K % 16 == 0) && (a.lda % 16 == 0) && (((uintptr_t)a.A & 15) == 0) &&
        (((uintptr_t)a.Bp & 15) == 0) && a.K >= 64 && fits32;
    int tile = 0;
    if (tiled_ok) {
        const uint64_t b256 = (uint64_t)((a.M + 255) / 256) * ((a.N + 255) / 256);
        const uint64_t b128 = (uint64_t)((a.M + 127) / 128) * ((a.N + 127) / 128);
        // measured on MI355X: 256 x 256 / 8 waves wins once it fills most of the 256 CUs; below
        // that 128 x 128 tiles keep more CUs busy; tiny problems go to the general kernel
        const bool k64 = (a.K % 64 == 0);
        if (b256 >= 128 && k64) {
            // ping-pong: 12 % faster than the fragment-prefetch loop at 8192^3, level elsewhere; with A requested in
            // whole lines another 4 % at 8192^3 and level at 4096^3 (needs K % 128 == 0 and 160 KB of LDS)
            tile = (a.K % 128 == 0) ? 12 : 11;
            // within one round of tiles the register-B form is level or ahead (4096^3, the encoder's FFN shapes); from
            // two rounds on the LDS form is (8192 x 4096 x 4096: 122.5 against 128.5 us)
            if (tile == 12 && b256 <= 256) {
                tile = 13;
            }
            // 256 x 256 tiles that leave CUs idle while the 128 x 128 ones come out at exactly two per CU: the smaller
            // tiles win by 20-29 % (2048 x 4096 x 4096 39.8 against 47.2 us, 8192 x 1024 x 1024 16.4 against 20.6,
            // 4096 x 2048 x 2048 25.0 against 29.5); with a ragged last round (576 tiles: 3072^3, 4096 x 768 x 2304)
            // they are level or behind
            if (b256 < 256 && b128 <= 512 && a.epi.mode != EPI_U8_GELU_DYN) {  // (that epilogue needs the large tiles)
                tile = 15;
            }
            // several rounds of large tiles with a short K spend half their time in prologues and epilogues; two small
            // workgroups per CU overlap those with each other's K loops (8192 x 1024 x 4096 53.2 against 58.9 us,
            // 8192 x 768 x 2304 28.7 against 34.0)
            if (b256 > 256 && a.K <= 1024 && a.epi.mode != EPI_U8_GELU_DYN) {
                tile = 15;
            }
        } else if (b128 >= 32 || (a.M >= 128 && a.N >= 128)) {
            tile = k64 ? 15 : 2;  // 15 against 10 (the compiler's order): 8.4 / 17.9 / 14.1 against 9.5 / 20.0 / 16.4 us at 4096 x 768 x 768, 4096 x 3072 x 768, 2048^3
            // long K on a grid that leaves CUs idle: two wave groups per tile on alternate K tiles (17.0 against 18.1 us at
            // 4096 x 3072 x 768; slower for short K and for grids of several rounds)
            if (tile == 15 && a.K % 128 == 0 && ((a.K >= 2048 && b128 <= 224) || (a.K >= 4096 && b128 <= 256))) {
                tile = 16;
            }
        }
    }
    if (g_force_tile >= 0 && (tiled_ok || g_force_tile == 0)) {
        tile = g_force_tile;
    }
    const bool dma_ok = tiled_ok && (a.K % 64 == 0);
    if (tile >= 3 && !dma_ok) {
        tile = tiled_ok ? 2 : 0;
    }
    if (tile == 2 && (a.M + 127) / 128 > 65535u) {
        tile = 0;  // the register-staged kernel counts its row tiles along the grid's y extent
    }
    if (tile == 13 && a.K % 128 != 0) {
        tile = 11;
    }
    if (tile == 12 && (a.K % 128 != 0 || !lds_160k())) {
        tile = 11;
    }
    if (a.epi.mode == EPI_U8_GELU_DYN) {
        // every tile's workgroup must be running when the first one waits for the others: full 256 x 256 tiles, one
        // workgroup per CU, and the sync area, status word and fallback buffer in place
        if ((tile != 11 && tile != 12 && tile != 13) || !gemm_gelu_dyn_fits(a.M, a.N, a.K) || !a.sync.slots || !a.status || !a.C32 || !a.dscale_out ||
            !a.epi.scaleI || !a.epi.scaleW || a.sync.blocks == 0 || a.sync.blocks > kGridSyncMaxBlocks) {
            return hipErrorInvalidValue;
        }
        if (tile == 13) {
            return launch_dma<2, 4, 8, 4, 3, 4, false, false, true>(a, st);
        }
        if (tile == 12) {
            return launch_dma<2, 4, 8, 4, 5, 3, false, false, true>(a, st);
        }
        return launch_dma<2, 4, 8, 4, 4, 2, false, false, true>(a, st);
    }
    // Few rows: the kernel that gives a 16-column weight panel to a workgroup and splits K over its 8 waves beats the
    // 128 x 128 tiles while it has at most one workgroup per CU -- 16 x 4096 x 4096 7.2 against 16.2 us, 256 x 3072 x 768
    // 8.8 against 13.1, 256 x 4096 x 1024 10.8 against 15.6 -- and loses beyond (256 x 4096 x 4096: 34.7 against 16.9).
    // Both sides are priced from measurements: 5.8 us + 21 ns per K tile and 16-row block of a workgroup's 64 rows
    // against 4.5 us + 0.18 us per K tile and round of 128 x 128 tiles.
    if (g_force_tile < 0 && dma_ok && (tile == 15 || tile == 16) && a.epi.mode != EPI_U8_GELU_DYN) {
        const uint64_t wgs = (uint64_t)((a.N + 15) / 16) * ((a.M + 63) / 64);
        if (wgs <= 256) {
            const uint32_t rows16 = (a.M + 15) / 16 < 4 ? (a.M + 15) / 16 : 4, ks = a.K / 64;
            const uint64_t b128 = (uint64_t)((a.M + 127) / 128) * ((a.N + 127) / 128);
            const float few = 5.8f + 0.0214f * (float)ks * (float)rows16;
            const float tiled = 4.5f + 0.18f * (float)ks * (float)((b128 + 255) / 256);
            if (few < tiled) {
                hipLaunchKernelGGL(gemm_u8s8_skinny_kernel, dim3((a.N + 15) / 16, (a.M + 63) / 64), dim3(512), 0, st, a);
                return hipGetLastError();
            }
        }
    }
    switch (tile) {
        case 2:
            return launch_tiled<2, 2, 4, 4>(a, st);  // 128 x 128
        case 7:
            return launch_dma<2, 4, 8, 4, 4, true>(a, st);  // 256 x 256, 8 waves, fragment prefetch
        case 10:
            return launch_dma<2, 2, 4, 4, 4, true>(a, st);  // 128 x 128, fragment prefetch
        case 11:
            return launch_dma<2, 4, 8, 4, 4, 2>(a, st);  // 256 x 256, 8 waves, ping-pong memory / matrix phases
        case 12:
            return launch_dma<2, 4, 8, 4, 5, 3>(a, st);  // the same with A requested in whole 128-byte lines (160 KB of LDS)
        case 13:
            return launch_dma<2, 4, 8, 4, 3, 4>(a, st);  // as 12 with the B fragments loaded straight into registers (96 KB of LDS)
        case 15:
            return launch_dma<2, 2, 4, 4, 4, 7>(a, st);  // 128 x 128, fragment prefetch in a pinned program order
        case 16:
            if (a.K % 128 != 0) {
                return launch_dma<2, 2, 4, 4, 4, 7>(a, st);
            }
            return launch_dma<2, 2, 4, 4, 4, 8>(a, st);  // the same by two groups of four waves on alternate K tiles
        default:
            break;
    }
    if (tile == 0 && g_force_tile < 0 && dma_ok && a.M <= 256) {
        // few rows: one 16-column weight panel per block, K split over its 8 waves
        hipLaunchKernelGGL(gemm_u8s8_skinny_kernel, dim3((a.N + 15) / 16, (a.M + 63) / 64), dim3(512), 0, st, a);
        return hipGetLastError();
    }
    if (g_force_tile == 14 && dma_ok) {
        hipLaunchKernelGGL(gemm_u8s8_skinny_kernel, dim3((a.N + 15) / 16, (a.M + 63) / 64), dim3(512), 0, st, a);
        return hipGetLastError();
    }
    if ((a.N + 63) / 64 > 65535u) {
        return hipErrorInvalidValue;  // more than 4 M columns: beyond a grid's y extent
    }
    dim3 grid((a.M + 63) / 64, (a.N + 63) / 64);
    hipLaunchKernelGGL(gemm_u8s8_general_kernel, grid, dim3(256), 0, st, a);
    return hipGetLastError();
}

}  // namespace bg
