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

// ---- attention ------------------------------------------------------------------------------------
// qkv: [batch * S][3 * H] fp32 rows (Q | K | V), head h owns columns h*64 .. h*64+63 of each third.
// One wave = 64 query rows of one (batch, head); a lane keeps its query row and its output row in
// registers. Key / value rows are the same for every lane of the wave, so they come in through the
// scalar cache and feed v_fmac as SGPR operands; the dot products run over d = 0..63 in order.
// Softmax is the streaming form over blocks of 16 keys (running max and sum), mathematically the
// max-subtracted softmax of the reference.
template <int D>
__global__ __launch_bounds__(64) void attention_f32_kernel(const float *__restrict__ qkv, uint32_t S, uint32_t H,
    float qscale, float *__restrict__ ctx, uint32_t *ws)
{
    const uint32_t lane = threadIdx.x;
    const uint32_t h = blockIdx.y, b = blockIdx.z;
    uint32_t r = blockIdx.x * 64 + lane;
    const bool live = r < S;
    r = live ? r : S - 1;
    const size_t ld = 3 * (size_t)H;
    const float *base = qkv + (size_t)b * S * ld + (size_t)h * D;
    float q[D], o[D];
    {
        const v4f *qp = (const v4f *)(base + (size_t)r * ld);
#pragma unroll
        for (int d4 = 0; d4 < D / 4; ++d4) {
            v4f v = qp[d4];
            q[4 * d4] = v.x * qscale;
            q[4 * d4 + 1] = v.y * qscale;
            q[4 * d4 + 2] = v.z * qscale;
            q[4 * d4 + 3] = v.w * qscale;
        }
    }
#pragma unroll
    for (int d = 0; d < D; ++d) {
        o[d] = 0.0f;
    }
    float m = -INFINITY, l = 0.0f;
    constexpr int JB = 16;
    for (uint32_t j0 = 0; j0 < S; j0 += JB) {
        float s[JB];
        float mx = m;
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) {
            const uint32_t j = (j0 + jj < S) ? j0 + jj : S - 1;
            const float *kp = base + H + (size_t)j * ld;  // wave-uniform address
            float acc = 0.0f;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                acc = __builtin_fmaf(q[d], kp[d], acc);
            }
            s[jj] = (j0 + jj < S) ? acc : -INFINITY;
            mx = fmaxf(mx, s[jj]);
        }
        const float corr = __expf(m - mx);  // exp(-inf) = 0 on the first block
        l *= corr;
#pragma unroll
        for (int d = 0; d < D; ++d) {
            o[d] *= corr;
        }
#pragma unroll
        for (int jj = 0; jj < JB; ++jj) {
            const uint32_t j = (j0 + jj < S) ? j0 + jj : S - 1;
            const float p = __expf(s[jj] - mx);
            l += p;
            const float *vp = base + 2 * (size_t)H + (size_t)j * ld;
#pragma unroll
            for (int d = 0; d < D; ++d) {
                o[d] = __builtin_fmaf(p, vp[d], o[d]);
            }
        }
        m = mx;
    }
    const float inv = 1.0f / l;
    float amax = 0.0f;
    v4f *op = (v4f *)(ctx + ((size_t)b * S + r) * H + (size_t)h * D);
#pragma unroll
    for (int d4 = 0; d4 < D / 4; ++d4) {
        v4f v = {o[4 * d4] * inv, o[4 * d4 + 1] * inv, o[4 * d4 + 2] * inv, o[4 * d4 + 3] * inv};
        if (live) {
            op[d4] = v;
            amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
        }
    }
    if (ws) {
        const int bits = wave_reduce_max_i((int)__float_as_uint(amax));
        if (lane == 0) {
            ws_fold_max(ws, blockIdx.x + gridDim.x * (blockIdx.y + gridDim.y * blockIdx.z), bits);
        }
    }
}

hipError_t launch_attention_f32(const float *qkv, uint32_t batch, uint32_t S, uint32_t H, uint32_t heads, float *ctx,
    uint32_t *ws, hipStream_t st)
{
    if (batch == 0 || S == 0 || heads == 0) {
        return hipSuccess;
    }
    if (H != heads * 64) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((S + 63) / 64, heads, batch);
    hipLaunchKernelGGL((attention_f32_kernel<64>), grid, dim3(64), 0, st, qkv, S, H, 0.125f, ctx, ws);
    return hipGetLastError();
}

// ---- residual + LayerNorm ---------------------------------------------------------------------------
// out[row] = gamma * ((x - mean) / sqrt(var + 1e-6)) + beta with x = a[row] + b[row]; one wave per row,
// the row stays in registers (V4 float4 per lane, H <= 256 * V4).
template <int V4>
__global__ __launch_bounds__(256) void add_layernorm_kernel(const float *__restrict__ a, const float *__restrict__ b,
    const float *__restrict__ gamma, const float *__restrict__ beta, uint32_t rows, uint32_t H, float *__restrict__ out,
    uint32_t *ws)
{
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
    uint32_t H, float *out, uint32_t *ws, hipStream_t st)
{
    if (rows == 0) {
        return hipSuccess;
    }
    if (H % 4 != 0 || H > 2048) {
        return hipErrorInvalidValue;
    }
    const dim3 grid((rows + 3) / 4);
    const uint32_t v4 = (H / 4 + 63) / 64;
#define BG_LN(V) hipLaunchKernelGGL((add_layernorm_kernel<V>), grid, dim3(256), 0, st, a, b, gamma, beta, rows, H, out, ws)
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

// ---- GELU (in place) ----------------------------------------------------------------------------------
__device__ __forceinline__ float gelu_tanh(float x)
{
    const float c0 = 1.5957691216057308f;  // 2 * sqrt(2 / pi)
    const float u = (c0 * x) * __builtin_fmaf(0.044715f, x * x, 1.0f);
    const float e = __expf(u);
    return (2.0f - 2.0f / (1.0f + e)) * (0.5f * x);
}

__global__ __launch_bounds__(256) void gelu_f32_kernel(float *__restrict__ x, uint32_t n4, uint32_t *ws)
{
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
        x4[i] = v;
        amax = fmaxf(amax, fmaxf(fmaxf(fabsf(v.x), fabsf(v.y)), fmaxf(fabsf(v.z), fabsf(v.w))));
    }
    if (ws) {
        ws_block_fold_max(ws, (int)__float_as_uint(amax), red);
    }
}

hipError_t launch_gelu_f32(float *x, size_t n, uint32_t *ws, hipStream_t st)
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
    hipLaunchKernelGGL(gelu_f32_kernel, dim3(blocks), dim3(256), 0, st, x, n4, ws);
    return hipGetLastError();
}

}  // namespace bg
