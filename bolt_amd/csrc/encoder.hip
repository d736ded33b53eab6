// fp32 neighbours of the int8 GEMMs inside a BERT-style encoder layer: scaled-dot-product
// attention, residual + LayerNorm, tanh-GELU. Each producer also folds max|out| into the scratch
// slots, so the dynamic per-tensor quantisation that follows needs no abs-max pass of its own.
//   LayerNorm  compute/tensor/src/cpu/x86/fp32/layer_norm.cpp:21-67 (eps 1e-6 inside the sqrt,
//              population variance, alpha * ((x - mean) / std) + beta)
//   GELU       compute/tensor/src/cpu/x86/fp32/x86_functions_fp32.h:127-149
//              (0.5 x (2 - 2 / (1 + exp(2 sqrt(2/pi) x (1 + 0.044715 x^2)))))
//   softmax    compute/tensor/src/cpu/x86/fp32/softmax.cpp (max-subtracted exp, sum, divide)
#include "device_common.h"
#include "kernels.h"

namespace bg {

// Optional duty of the first workgroup: zero the scratch slots of a maximum that has been consumed, so that the
// next producer of those slots finds them clear without a launch of its own.
__device__ __forceinline__ void clear_slots(uint32_t *clear)
{
    if (clear && blockIdx.x == 0 && blockIdx.y == 0 && blockIdx.z == 0 && threadIdx.x < kWsSlots) {
        clear[threadIdx.x * kWsStride] = 0;
    }
}

// ---- attention ------------------------------------------------------------------------------------
// qkv: [batch * S][3 * H] fp32 rows (Q | K | V), head h owns columns h*64 .. h*64+63 of each third.
// fp32 matrix cores (v_mfma_f32_16x16x4_f32): a workgroup owns 64 * NT queries of one (batch, head), each of its
// four waves 16 * NT of them, and walks the keys in chunks of 16 * KT. A chunk's K and V rows (64 floats each) are
// brought into LDS once per workgroup with whole-line loads (16 lanes per 256-byte row) and read from there by
// all four waves; rows are 68 floats apart, which keeps both the 16-byte K reads (16 different rows per
// quarter wave) and the 4-byte V reads (4 rows x 16 consecutive floats) free of bank conflicts.
//   scores^T = K . Q^T   : M = key, N = query, contraction over d. A lane (c = lane % 16, g = lane / 16)
//                          feeds K[key c][16 s + 4 g + t] and Q[query c][16 s + 4 g + t] for step (s, t):
//                          one 16-byte load covers four steps, and both operands permute d the same way.
//   the accumulator of key tile kt then holds score(key 16 kt + 4 g + i, query c), i = 0..3, so the
//   softmax statistics of a query are an in-lane reduction plus two cross-lane steps (xor 16, 32);
//   out^T = V^T . P^T    : M = d, N = query, contraction over keys in the order the accumulators
//                          already have them: step (kt, t) takes P from element t of tile kt and
//                          V[key 16 kt + 4 g + t][d c] -- no transposition through LDS.
// Chunks are merged with the streaming (running max / running sum) form of the max-subtracted softmax.
typedef float v4f_t __attribute__((ext_vector_type(4)));

// NT: query tiles of 16 per wave (a workgroup owns 64 * NT queries); KT: key tiles of 16 per chunk.
template <int D, int NT, int KT>
__global__ __launch_bounds__(256, 2) void attention_f32_kernel(const float *__restrict__ qkv, uint32_t S, uint32_t H,
    float qscale, float *__restrict__ ctx, uint32_t *ws, uint32_t *clear)
{
    clear_slots(clear);
    static_assert(D == 64, "head size 64");
    const uint32_t lane = threadIdx.x & 63, wave = __builtin_amdgcn_readfirstlane(threadIdx.x >> 6);
    const uint32_t c = lane & 15, g = lane >> 4;
    const uint32_t h = blockIdx.y, b = blockIdx.z;
    const uint32_t q0 = blockIdx.x * (64 * NT) + wave * (16 * NT);
    const bool active = q0 < S;  // a wave past the end of the sequence still helps to load the chunks
    extern __shared__ __attribute__((aligned(16))) float att_smem[];
    constexpr uint32_t kRow = 68;  // floats between rows in LDS
    float *sK = att_smem, *sV = att_smem + KT * 16 * kRow;
    const size_t ld = 3 * (size_t)H;
    const float *Qb = qkv + (size_t)b * S * ld + (size_t)h * D;
    const float *Kb = Qb + H, *Vb = Qb + 2 * (size_t)H;

    v4f_t qf[NT][4];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        uint32_t q = q0 + nt * 16 + c;
        q = q < S ? q : S - 1;
#pragma unroll
        for (int s4 = 0; s4 < 4; ++s4) {
            v4f_t v = *(const v4f_t *)(Qb + (size_t)q * ld + 16 * s4 + 4 * g);
            qf[nt][s4] = v * qscale;
        }
    }
    v4f_t o[4][NT];
#pragma unroll
    for (int mt = 0; mt < 4; ++mt) {
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            o[mt][nt] = (v4f_t){0.0f, 0.0f, 0.0f, 0.0f};
        }
    }
    float m[NT], l[NT];
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        m[nt] = -INFINITY;
        l[nt] = 0.0f;
    }

    for (uint32_t k0 = 0; k0 < S; k0 += KT * 16) {
        if (k0) {
            __syncthreads();  // everyone is done with the previous chunk
        }
        {   // chunk -> LDS: KT * 256 pieces of 16 bytes per matrix, KT per thread; rows past the end repeat the last one
#pragma unroll
            for (int r = 0; r < KT; ++r) {
                const uint32_t piece = threadIdx.x + r * 256, row = piece >> 4, col = (piece & 15) * 4;
                uint32_t key = k0 + row;
                key = key < S ? key : S - 1;
                const v4f_t kv = *(const v4f_t *)(Kb + (size_t)key * ld + col);
                const v4f_t vv = *(const v4f_t *)(Vb + (size_t)key * ld + col);
                *(v4f_t *)(sK + row * kRow + col) = kv;
                *(v4f_t *)(sV + row * kRow + col) = vv;
            }
        }
        __syncthreads();
        if (!active) {
            continue;
        }
        v4f_t s[KT][NT];
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int nt = 0; nt < NT; ++nt) {
                s[kt][nt] = (v4f_t){0.0f, 0.0f, 0.0f, 0.0f};
            }
            const float *kp = sK + (kt * 16 + c) * kRow + 4 * g;
#pragma unroll
            for (int s4 = 0; s4 < 4; ++s4) {
                const v4f_t kf = *(const v4f_t *)(kp + 16 * s4);
#pragma unroll
                for (int t = 0; t < 4; ++t) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        s[kt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(kf[t], qf[nt][s4][t], s[kt][nt], 0, 0, 0);
                    }
                }
            }
        }
        // keys past the end of the sequence do not take part
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int i = 0; i < 4; ++i) {
                if (k0 + kt * 16 + 4 * g + i >= S) {
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        s[kt][nt][i] = -INFINITY;
                    }
                }
            }
        }
#pragma unroll
        for (int nt = 0; nt < NT; ++nt) {
            float mx = m[nt];
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
                mx = fmaxf(mx, fmaxf(fmaxf(s[kt][nt][0], s[kt][nt][1]), fmaxf(s[kt][nt][2], s[kt][nt][3])));
            }
            mx = fmaxf(mx, __shfl_xor(mx, 16, 64));
            mx = fmaxf(mx, __shfl_xor(mx, 32, 64));
            const float corr = __expf(m[nt] - mx);  // exp(-inf) = 0 on the first chunk
            float sum = 0.0f;
#pragma unroll
            for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
                for (int i = 0; i < 4; ++i) {
                    const float p = __expf(s[kt][nt][i] - mx);
                    s[kt][nt][i] = p;
                    sum += p;
                }
            }
            sum += __shfl_xor(sum, 16, 64);
            sum += __shfl_xor(sum, 32, 64);
            l[nt] = l[nt] * corr + sum;
            m[nt] = mx;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                o[mt][nt] = o[mt][nt] * corr;
            }
        }
#pragma unroll
        for (int kt = 0; kt < KT; ++kt) {
#pragma unroll
            for (int t = 0; t < 4; ++t) {
                const float *vp = sV + (kt * 16 + 4 * g + t) * kRow + c;  // rows past the end: probability 0
#pragma unroll
                for (int mt = 0; mt < 4; ++mt) {
                    const float vv = vp[16 * mt];
#pragma unroll
                    for (int nt = 0; nt < NT; ++nt) {
                        o[mt][nt] = __builtin_amdgcn_mfma_f32_16x16x4f32(vv, s[kt][nt][t], o[mt][nt], 0, 0, 0);
                    }
                }
            }
        }
    }
    if (!active) {
        return;
    }
    float amax = 0.0f;
#pragma unroll
    for (int nt = 0; nt < NT; ++nt) {
        const uint32_t q = q0 + nt * 16 + c;
        const float inv = 1.0f / l[nt];
        if (q < S) {
            float *op = ctx + ((size_t)b * S + q) * H + (size_t)h * D + 4 * g;
#pragma unroll
            for (int mt = 0; mt < 4; ++mt) {
                const v4f_t v = o[mt][nt] * inv;
                *(v4f_t *)(op + 16 * mt) = v;
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v[0]), fabsf(v[1])), fmaxf(fabsf(v[2]), fabsf(v[3]))));
            }
        }
    }
    if (ws) {
        const int bits = wave_reduce_max_i((int)__float_as_uint(amax));
        if (lane == 0) {
            ws_fold_max(ws, (blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z)) * 4 + wave, bits);
        }
    }
}

hipError_t launch_attention_f32(const float *qkv, uint32_t batch, uint32_t S, uint32_t H, uint32_t heads, float *ctx,
    uint32_t *ws, hipStream_t st, uint32_t *clear)
{
    if (batch == 0 || S == 0 || heads == 0) {
        return hipSuccess;
    }
    if (H != heads * 64) {
        return hipErrorInvalidValue;
    }
    // 16 queries per wave and 64 keys per chunk: 64-query workgroups, three of which share a CU (35 KB of LDS each).
    // At BERT-base (seq 128, 12 heads, batch 32) that is 768 workgroups = 3 waves on every SIMD; with 32 queries
    // per wave the 384 workgroups leave half the CUs with twice the work of the other half.
    constexpr int NT = 1, KT = 4;
    const dim3 grid((S + 64 * NT - 1) / (64 * NT), heads, batch);
    constexpr uint32_t lds = 2 * KT * 16 * 68 * sizeof(float);  // K and V chunk, rows 68 floats apart
    static bool attr_set = false;
    if (!attr_set) {
        hipError_t e = hipFuncSetAttribute((const void *)attention_f32_kernel<64, NT, KT>, hipFuncAttributeMaxDynamicSharedMemorySize, lds);
        if (e != hipSuccess) {
            return e;
        }
        attr_set = true;
    }
    hipLaunchKernelGGL((attention_f32_kernel<64, NT, KT>), grid, dim3(256), lds, st, qkv, S, H, 0.125f, ctx, ws, clear);
    return hipGetLastError();
}

// ---- residual + LayerNorm ---------------------------------------------------------------------------
// out[row] = gamma * ((x - mean) / sqrt(var + 1e-6)) + beta with x = a[row] + b[row]; one wave per row,
// the row stays in registers (V4 float4 per lane, H <= 256 * V4).
template <int V4>
__global__ __launch_bounds__(256) void add_layernorm_kernel(const float *__restrict__ a, const float *__restrict__ b,
    const float *__restrict__ gamma, const float *__restrict__ beta, uint32_t rows, uint32_t H, float *__restrict__ out,
    uint32_t *ws, uint32_t *clear)
{
    clear_slots(clear);
    __shared__ int red[4];
    const uint32_t lane = threadIdx.x & 63, wave = threadIdx.x >> 6;
    const uint32_t row = blockIdx.x * 4 + wave;
    const uint32_t h4 = H / 4;
    float amax = 0.0f;
    if (row < rows) {
        const v4f *ap = (const v4f *)(a + (size_t)row * H);
        const v4f *bp = b ? (const v4f *)(b + (size_t)row * H) : nullptr;
        v4f x[V4];
        float sum = 0.0f;
#pragma unroll
        for (int i = 0; i < V4; ++i) {
            const uint32_t c = lane + 64 * i;
            v4f v = {0.0f, 0.0f, 0.0f, 0.0f};
            if (c < h4) {
                v = ap[c];
                if (bp) {
                    v4f w = bp[c];
                    v.x += w.x;
                    v.y += w.y;
                    v.z += w.z;
                    v.w += w.w;
                }
            }
            x[i] = v;
            sum += (v.x + v.y) + (v.z + v.w);
        }
        const float mean = wave_reduce_sum(sum) / (float)H;
        float sq = 0.0f;
#pragma unroll
        for (int i = 0; i < V4; ++i) {
            if (lane + 64 * i < h4) {
                const float d0 = x[i].x - mean, d1 = x[i].y - mean, d2 = x[i].z - mean, d3 = x[i].w - mean;
                sq += (d0 * d0 + d1 * d1) + (d2 * d2 + d3 * d3);
            }
        }
        const float var = wave_reduce_sum(sq) / (float)H;
        const float sd = sqrtf(var + 1e-6f);
        v4f *op = (v4f *)(out + (size_t)row * H);
#pragma unroll
        for (int i = 0; i < V4; ++i) {
            const uint32_t c = lane + 64 * i;
            if (c < h4) {
                const v4f g = ((const v4f *)gamma)[c], be = ((const v4f *)beta)[c];
                v4f y;
                y.x = __builtin_fmaf(g.x, (x[i].x - mean) / sd, be.x);
                y.y = __builtin_fmaf(g.y, (x[i].y - mean) / sd, be.y);
                y.z = __builtin_fmaf(g.z, (x[i].z - mean) / sd, be.z);
                y.w = __builtin_fmaf(g.w, (x[i].w - mean) / sd, be.w);
                op[c] = y;
                amax = fmaxf(amax, fmaxf(fmaxf(fabsf(y.x), fabsf(y.y)), fmaxf(fabsf(y.z), fabsf(y.w))));
            }
        }
    }
    if (ws) {
        ws_block_fold_max(ws, (int)__float_as_uint(amax), red);
    }
}

hipError_t launch_add_layernorm(const float *a, const float *b, const float *gamma, const float *beta, uint32_t rows,
    uint32_t H, float *out, uint32_t *ws, hipStream_t st, uint32_t *clear)
{
    if (rows == 0) {
        return hipSuccess;
    }
    if (H % 4 != 0 || H > 2048) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((rows + 3) / 4);
    const uint32_t v4 = (H / 4 + 63) / 64;
#define BG_LN(V) hipLaunchKernelGGL((add_layernorm_kernel<V>), grid, dim3(256), 0, st, a, b, gamma, beta, rows, H, out, ws, clear)
    if (v4 <= 1) {
        BG_LN(1);
    } else if (v4 <= 2) {
        BG_LN(2);
    } else if (v4 <= 3) {
        BG_LN(3);
    } else if (v4 <= 4) {
        BG_LN(4);
    } else {
        BG_LN(8);
    }
#undef BG_LN
    return hipGetLastError();
}

// ---- GELU (in place, or only its max|.|) ----------------------------------------------------------------
// STORE = false leaves x as it is and only folds max|gelu(x)| into ws: the quantiser that follows applies the
// same gelu_tanh to what it reads, so the activated tensor is never written.
template <bool STORE>
__global__ __launch_bounds__(256) void gelu_f32_kernel(float *__restrict__ x, uint32_t n4, uint32_t *ws, uint32_t *clear)
{
    clear_slots(clear);
    __shared__ int red[4];
    const uint32_t tid = blockIdx.x * blockDim.x + threadIdx.x;
    const uint32_t stride = gridDim.x * blockDim.x;
    float amax = 0.0f;
    v4f *x4 = (v4f *)x;
    for (uint32_t i = tid; i < n4; i += stride) {
        v4f v = x4[i];
        v.x = gelu_tanh(v.x);
        v.y = gelu_tanh(v.y);
        v.z = gelu_tanh(v.z);
        v.w = gelu_tanh(v.w);
        if (STORE) {
            x4[i] = v;
        }
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    if (ws) {
        ws_block_fold_max(ws, (int)__float_as_uint(amax), red);
    }
}

hipError_t launch_gelu_f32(float *x, size_t n, uint32_t *ws, hipStream_t st, bool store, uint32_t *clear)
{
    if (n == 0) {
        return hipSuccess;
    }
    if (n % 4 != 0 || n / 4 > 0xffffffffull) {
        return hipErrorInvalidValue;
    }
    const uint32_t n4 = (uint32_t)(n / 4);
    uint32_t blocks = (n4 + 255) / 256;
    blocks = blocks > 4096 ? 4096 : blocks;
    if (store) {
        hipLaunchKernelGGL(gelu_f32_kernel<true>, dim3(blocks), dim3(256), 0, st, x, n4, ws, clear);
    } else {
        hipLaunchKernelGGL(gelu_f32_kernel<false>, dim3(blocks), dim3(256), 0, st, x, n4, ws, clear);
    }
    return hipGetLastError();
}

}  // namespace bg
