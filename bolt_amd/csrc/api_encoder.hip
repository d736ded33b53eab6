// C-ABI entry points of the BERT-style int8 encoder layer and stack (device pointers, asynchronous) and of its fp32
// neighbours (attention, add + LayerNorm, GELU).
#include <hip/hip_runtime.h>
#include <algorithm>
#include <atomic>
#include <cstdio>
#include <cstring>
#include <string>
#include <vector>

#include "api_internal.h"

using namespace bg;
using namespace bgapi;

extern "C" {

// ---- BERT-style int8 encoder layer --------------------------------------------------------------------
namespace {
struct EncoderPlan {
    size_t ws, scales, xq, xq2, qkv, ctx, ao, h1, f, o, total;
};

EncoderPlan encoder_plan(const BoltEncoderLayerInt8 &L)
{
    const size_t T = (size_t)L.batch * L.seq, H = L.hidden, F = L.ffn;
    EncoderPlan p;
    size_t off = 0;
    auto take = [&](size_t bytes) {
        size_t at = off;
        off += (bytes + 255) / 256 * 256;
        return at;
    };
    p.ws = take(4 * kWsWords * sizeof(uint32_t));
    p.scales = take(64);
    p.xq = take(T * H);   // u8 input of the three FullyConnected layers that read [T, H]
    p.xq2 = take(T * F);  // u8 input of the last one, [T, F] (written while the one before it still reads xq)
    p.qkv = take(T * 3 * H * 4);
    p.ctx = take(T * H * 4);
    p.ao = take(T * H * 4);
    p.h1 = take(T * H * 4);
    p.f = take(T * F * 4);
    p.o = take(T * H * 4);
    p.total = off;
    return p;
}

EE encoder_check(const BoltEncoderLayerInt8 *L)
{
    if (!L) {
        return NULL_POINTER;
    }
    if (!L->wqkv || !L->wo || !L->w1 || !L->w2 || !L->sqkv || !L->so || !L->s1 || !L->s2 || !L->ln1_gamma || !L->ln1_beta ||
        !L->ln2_gamma || !L->ln2_beta) {
        return NULL_POINTER;
    }
    if (L->batch == 0 || L->seq == 0 || L->heads == 0 || L->hidden != L->heads * 64 || L->ffn == 0 || L->ffn % 4 != 0 ||
        L->hidden > 2048) {
        return NOT_SUPPORTED;
    }
    if ((uint64_t)L->batch * L->seq * (L->ffn > 3 * L->hidden ? L->ffn : 3 * L->hidden) > 0xffffffffull) {
        return NOT_SUPPORTED;
    }
    return SUCCESS;
}
}  // namespace

EE bolt_gfx950_encoder_layer_int8_workspace_bytes(const BoltEncoderLayerInt8 *layer, size_t *bytes)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!bytes) {
        return NULL_POINTER;
    }
    *bytes = encoder_plan(*layer).total;
    return SUCCESS;
}

EE bolt_gfx950_encoder_layer_int8_workspace_layout(const BoltEncoderLayerInt8 *layer, size_t *offsets)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!offsets) {
        return NULL_POINTER;
    }
    const EncoderPlan p = encoder_plan(*layer);
    offsets[0] = p.qkv;
    offsets[1] = p.ctx;
    offsets[2] = p.ao;
    offsets[3] = p.h1;
    offsets[4] = p.f;
    offsets[5] = p.o;
    return SUCCESS;
}

// One layer's launches. input_max_ready: the scratch slots already hold max|hidden| (the LayerNorm that produced
// `hidden` folded it), so no abs-max pass runs; fold_out_max: the last LayerNorm folds max|out| into those slots for
// the layer that follows.
static EE encoder_run(const BoltEncoderLayerInt8 &L, const EncoderPlan &p, const float *hidden, float *out, void *workspace,
    bool input_max_ready, bool fold_out_max)
{
    hipStream_t st = ctx().stream;
    U8 *w = (U8 *)workspace;
    const U32 T = L.batch * L.seq, H = L.hidden, F = L.ffn;
    float *sc = (float *)(w + p.scales);
    uint8_t *xq = w + p.xq, *xq2 = w + p.xq2;
    float *qkv = (float *)(w + p.qkv), *cx = (float *)(w + p.ctx), *ao = (float *)(w + p.ao), *h1 = (float *)(w + p.h1),
          *f = (float *)(w + p.f), *o = (float *)(w + p.o);

    auto gemm = [&](const uint8_t *A, const void *blob, U32 N, U32 K, const float *dsI, const float *sW, const float *bias,
                    float *C) -> hipError_t {
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = A;
        g.lda = K;
        g.Bp = (const int8_t *)blob;
        g.M = T;
        g.N = N;
        g.K = K;
        g.comp = (const int32_t *)((const U8 *)blob + packed_matrix_bytes(N, K));
        g.ob = g.comp;  // no folded bias: the fp32 bias is added in the epilogue
        g.C = C;
        g.epi.mode = EPI_F32_CH;
        g.epi.scaleI = dsI;
        g.epi.scaleW = sW;
        g.epi.bias = bias;
        return launch_gemm_u8s8(g, st);
    };

    // The four running maxima live in slots the library owns and keeps clear between calls: each array is zeroed
    // by the first workgroup of a kernel that runs after the maximum's only reader and before its next producer
    // (one layer call later). A call that fails half way leaves them in an unknown state, so they are refilled
    // before the next one.
    Ctx &c = ctx();
    uint32_t *ws0 = c.enc_ws, *ws1 = ws0 + kWsWords, *ws2 = ws1 + kWsWords, *ws3 = ws2 + kWsWords;
    if (!input_max_ready) {
        if (c.enc_ws_dirty) {
            HIP_TRY(launch_fill_u32(ws0, 4 * kWsWords, 0, st));
        }
        c.enc_ws_dirty = true;
        HIP_TRY(launch_absmax_f32(hidden, T * H, ws0, st, true));
    }
    // x -> u8 (dynamic per-tensor scale), one quantisation shared by Q, K and V
    HIP_TRY(launch_quantize_f32(hidden, T * H, xq, 1, ws0, 0.0f, nullptr, 0, sc + 0, st));
    HIP_TRY(gemm(xq, L.wqkv, 3 * H, H, sc + 0, L.sqkv, L.bqkv, qkv));
    HIP_TRY(launch_attention_f32(qkv, L.batch, L.seq, H, L.heads, cx, ws1, st, ws0));
    HIP_TRY(launch_quantize_f32(cx, T * H, xq, 1, ws1, 0.0f, nullptr, 0, sc + 1, st));
    HIP_TRY(gemm(xq, L.wo, H, H, sc + 1, L.so, L.bo, ao));
    HIP_TRY(launch_add_layernorm(hidden, ao, L.ln1_gamma, L.ln1_beta, T, H, h1, ws2, st, ws1));
    HIP_TRY(launch_quantize_f32(h1, T * H, xq, 1, ws2, 0.0f, nullptr, 0, sc + 2, st));
    // (the fused kernel is one of the tiled ones: it needs what launch_gemm_u8s8 asks of those -- operands on 16-byte
    // boundaries -- and reads the per-column vectors 16 bytes at a time; anything else takes the unfused sequence)
    const bool fused_aligned = ((((uintptr_t)L.w1) | ((uintptr_t)xq) | ((uintptr_t)L.s1) | ((uintptr_t)L.b1)) & 15) == 0;
    if (g_encoder_fused && fused_aligned && gemm_gelu_dyn_fits(T, F, H)) {
        // FullyConnected + GELU + dynamic quantisation in one launch: the accumulators stay in registers across a
        // grid-wide agreement on max|gelu|; the [T, F] fp32 tensor is never written. Should that agreement be abandoned
        // (the CUs were held by other work), the kernel leaves the activated values in f, sets the status word, and
        // its last workgroup quantises them alone.
        uint32_t *status = (uint32_t *)(sc + 8);
        const uint32_t tiles = (T / 256) * (F / 256);
        GemmArgs g;
        memset(&g, 0, sizeof(g));
        g.A = xq;
        g.lda = H;
        g.Bp = (const int8_t *)L.w1;
        g.M = T;
        g.N = F;
        g.K = H;
        g.comp = (const int32_t *)((const U8 *)L.w1 + packed_matrix_bytes(F, H));
        g.ob = g.comp;
        g.C = xq2;
        g.epi.mode = EPI_U8_GELU_DYN;
        g.epi.scaleI = sc + 2;
        g.epi.scaleW = L.s1;
        g.epi.bias = L.b1;
        g.sync = c.fsync.next(tiles);
        g.dscale_out = sc + 3;
        g.status = status;
        g.C32 = f;
        g.clear_ws = ws2;  // consumed by the quantiser in front of this product
        hipError_t he = launch_gemm_u8s8(g, st);
        if (he != hipSuccess) {
            return fail(UNKNOWN, "launch_gemm_u8s8 (GELU epilogue)", he);
        }
    } else {
        HIP_TRY(gemm(xq, L.w1, F, H, sc + 2, L.s1, L.b1, f));
        // GELU: one pass takes max|gelu(f)| without writing anything, the quantiser applies the same gelu to what it reads
        HIP_TRY(launch_gelu_f32(f, (size_t)T * F, ws3, st, false, ws2));
        HIP_TRY(launch_quantize_f32(f, T * F, xq2, 1, ws3, 0.0f, nullptr, 0, sc + 3, st, 1));
    }
    HIP_TRY(gemm(xq2, L.w2, H, F, sc + 3, L.s2, L.b2, o));
    // (ws0 was consumed by the first quantiser and cleared by the attention kernel: free for the next layer's maximum)
    HIP_TRY(launch_add_layernorm(h1, o, L.ln2_gamma, L.ln2_beta, T, H, out, fold_out_max ? ws0 : nullptr, st, ws3));
    return SUCCESS;
}

EE bolt_gfx950_encoder_layer_int8(const BoltEncoderLayerInt8 *layer, const float *hidden, float *out, void *workspace,
    size_t workspaceBytes)
{
    EE e = encoder_check(layer);
    if (e != SUCCESS) {
        return e;
    }
    if (!hidden || !out || !workspace) {
        return NULL_POINTER;
    }
    const BoltEncoderLayerInt8 &L = *layer;
    const EncoderPlan p = encoder_plan(L);
    if (workspaceBytes < p.total) {
        return NOT_MATCH;
    }
    if (((uintptr_t)workspace & 255) || ((uintptr_t)hidden & 15) || ((uintptr_t)out & 15)) {
        return fail(NOT_SUPPORTED, "workspace must be 256-byte aligned, hidden / out 16-byte aligned");
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    Ctx &c = ctx();
    e = encoder_run(L, p, hidden, out, workspace, false, false);
    if (e != SUCCESS) {
        return e;
    }
    c.enc_ws_dirty = false;
    return SUCCESS;
}

EE bolt_gfx950_encoder_stack_int8(const BoltEncoderLayerInt8 *layers, U32 numLayers, const float *hidden, float *out,
    void *workspace, size_t workspaceBytes)
{
    if (!layers || !hidden || !out || !workspace) {
        return NULL_POINTER;
    }
    if (numLayers == 0) {
        return NOT_SUPPORTED;
    }
    size_t need = 0;
    EE e = bolt_gfx950_encoder_stack_int8_workspace_bytes(layers, numLayers, &need);
    if (e != SUCCESS) {
        return e;
    }
    if (workspaceBytes < need) {
        return NOT_MATCH;
    }
    if (((uintptr_t)workspace & 255) || ((uintptr_t)hidden & 15) || ((uintptr_t)out & 15)) {
        return fail(NOT_SUPPORTED, "workspace must be 256-byte aligned, hidden / out 16-byte aligned");
    }
    e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    // the layers share one layer's workspace (the largest); behind it two [T, hidden] fp32 buffers take the
    // activations from layer to layer
    size_t one = 0;
    for (U32 i = 0; i < numLayers; ++i) {
        const size_t t = encoder_plan(layers[i]).total;
        one = t > one ? t : one;
    }
    const size_t act = ((size_t)layers[0].batch * layers[0].seq * layers[0].hidden * 4 + 255) / 256 * 256;
    float *pp[2] = {(float *)((U8 *)workspace + one), (float *)((U8 *)workspace + one + act)};
    Ctx &c = ctx();
    const float *in = hidden;
    for (U32 i = 0; i < numLayers; ++i) {
        const bool last = i + 1 == numLayers;
        float *o = last ? out : pp[i & 1];
        e = encoder_run(layers[i], encoder_plan(layers[i]), in, o, workspace, i != 0, !last);
        if (e != SUCCESS) {
            return e;
        }
        in = o;
    }
    c.enc_ws_dirty = false;
    return SUCCESS;
}

EE bolt_gfx950_encoder_stack_int8_workspace_bytes(const BoltEncoderLayerInt8 *layers, U32 numLayers, size_t *bytes)
{
    if (!layers || !bytes) {
        return NULL_POINTER;
    }
    if (numLayers == 0) {
        return NOT_SUPPORTED;
    }
    size_t one = 0;
    for (U32 i = 0; i < numLayers; ++i) {
        EE e = encoder_check(&layers[i]);
        if (e != SUCCESS) {
            return e;
        }
        if (layers[i].batch != layers[0].batch || layers[i].seq != layers[0].seq || layers[i].hidden != layers[0].hidden) {
            return NOT_MATCH;  // the activations keep their shape from layer to layer
        }
        const size_t t = encoder_plan(layers[i]).total;
        one = t > one ? t : one;
    }
    const size_t act = ((size_t)layers[0].batch * layers[0].seq * layers[0].hidden * 4 + 255) / 256 * 256;
    *bytes = one + 2 * act;
    return SUCCESS;
}

EE bolt_gfx950_attention_f32(const float *qkv, U32 batch, U32 seq, U32 hidden, U32 heads, float *context)
{
    if (!qkv || !context) {
        return NULL_POINTER;
    }
    if (heads == 0 || hidden != heads * 64) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_attention_f32(qkv, batch, seq, hidden, heads, context, nullptr, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_add_layernorm_f32(const float *a, const float *b, const float *gamma, const float *beta, U32 rows,
    U32 hidden, float *out)
{
    if (!a || !gamma || !beta || !out) {
        return NULL_POINTER;
    }
    if (hidden % 4 != 0 || hidden > 2048) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_add_layernorm(a, b, gamma, beta, rows, hidden, out, nullptr, ctx().stream));
    return SUCCESS;
}

EE bolt_gfx950_gelu_f32(float *x, size_t n)
{
    if (!x) {
        return NULL_POINTER;
    }
    if (n % 4 != 0) {
        return NOT_SUPPORTED;
    }
    EE e = ensure_init();
    if (e != SUCCESS) {
        return e;
    }
    HIP_TRY(launch_gelu_f32(x, n, nullptr, ctx().stream));
    return SUCCESS;
}

}  // extern "C"
