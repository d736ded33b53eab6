"""TEST INFRASTRUCTURE ONLY -- CPU restatement (numpy) of one BERT-style int8 encoder layer as Bolt's
x86 path computes it, used by tests/ and bench.py to check the GPU path. Never imported by the product.

Pieces and the reference code each follows:
  * dynamic per-tensor activation quantisation F32 -> U8_Q: quantize_x86
    (compute/tensor/src/cpu/x86/int8/avx512/quantize.cpp:21-68,121-179) -- delegated to oracle.c
  * int8 FullyConnected: u8 x s8 with int32 accumulation
    (compute/blas_enhance/src/cpu/x86/int8/avx512/mmm_avx512_vnni.cpp:1760-1891); accumulators are taken
    here as the exact integer product (float64 matmul of integers < 2^53, the closed form the C oracle
    is itself pinned against), dequantised per output channel: cvt(acc) * (1.0f / (sI * sW[n])) + b[n]
  * attention: softmax(Q K^T / sqrt(64)) V in fp32 (compute/tensor/src/cpu/x86/fp32/softmax.cpp)
  * LayerNorm: compute/tensor/src/cpu/x86/fp32/layer_norm.cpp:21-67 (population variance, eps 1e-6)
  * GELU: compute/tensor/src/cpu/x86/fp32/x86_functions_fp32.h:127-149 (tanh form through exp)
fp32 reductions are done in float64 and rounded once; the layer output is compared with a 1e-3
relative tolerance, which the summation-order differences (1e-6) do not touch.
"""
import numpy as np

F = np.float32


def quantize_weight_per_channel(W):
    """W: fp32 [N, K] -> (s8 [N, K], scale [N]) with scale[n] = 127 / max|W[n]| (quantised = real * scale)."""
    W = np.asarray(W, F)
    m = np.abs(W).max(axis=1)
    with np.errstate(divide="ignore"):
        s = np.where(m > 0, F(127.0) / m, F(1.0)).astype(F)
    q = np.clip(np.rint(W * s[:, None]), -127, 127).astype(np.int8)
    return q, s


def int8_fc(oracle, x, Wq, sW, bias):
    """x fp32 [T, K] -> dynamic u8 quantisation -> exact integer product -> per-channel dequantisation."""
    from checkers import DT_U8_Q
    xq, sI = oracle.quantize_f32(np.ascontiguousarray(x, F).reshape(-1), DT_U8_Q)
    xq = xq.reshape(x.shape)
    acc = ((xq.astype(np.float64) - 128.0) @ Wq.T.astype(np.float64)).astype(np.int64)
    assert np.abs(acc).max() < 2 ** 31
    return oracle.dequant_per_channel(acc.astype(np.int32), sI, sW, bias), xq, sI


def layer_norm(x, gamma, beta):
    x64 = x.astype(np.float64)
    mean = x64.mean(axis=1, keepdims=True).astype(F)
    var = ((x64 - mean) ** 2).mean(axis=1, keepdims=True).astype(F)
    sd = np.sqrt(var + F(1e-6), dtype=F)
    return (gamma * ((x - mean) / sd) + beta).astype(F)


def gelu(x):
    x = x.astype(F)
    u = (F(1.5957691216057308) * x) * (F(0.044715) * x * x + F(1.0))
    with np.errstate(over="ignore"):
        e = np.exp(u.astype(np.float64)).astype(F)
    return ((F(2.0) - F(2.0) / (F(1.0) + e)) * (F(0.5) * x)).astype(F)


def attention(qkv, batch, seq, hidden, heads):
    d = hidden // heads
    q, k, v = (qkv[:, i * hidden:(i + 1) * hidden].reshape(batch, seq, heads, d).transpose(0, 2, 1, 3).astype(np.float64)
               for i in range(3))
    s = (q * 0.125 if d == 64 else q / np.sqrt(d)) @ k.transpose(0, 1, 3, 2)
    s -= s.max(axis=-1, keepdims=True)
    p = np.exp(s)
    p /= p.sum(axis=-1, keepdims=True)
    ctx = p @ v
    return ctx.transpose(0, 2, 1, 3).reshape(batch * seq, hidden).astype(F)


def encoder_layer(oracle, x, P, batch, seq, hidden, heads):
    """P: dict with wqkv/wo/w1/w2 (s8 [N, K]), sqkv/so/s1/s2, bqkv/bo/b1/b2, ln1_g/ln1_b/ln2_g/ln2_b.
    Returns (out, intermediates)."""
    x = np.ascontiguousarray(x, F)
    qkv, _, _ = int8_fc(oracle, x, P["wqkv"], P["sqkv"], P["bqkv"])
    ctx = attention(qkv, batch, seq, hidden, heads)
    ao, _, _ = int8_fc(oracle, ctx, P["wo"], P["so"], P["bo"])
    h1 = layer_norm(x + ao, P["ln1_g"], P["ln1_b"])
    f, _, _ = int8_fc(oracle, h1, P["w1"], P["s1"], P["b1"])
    f = gelu(f)
    o, _, _ = int8_fc(oracle, f, P["w2"], P["s2"], P["b2"])
    out = layer_norm(h1 + o, P["ln2_g"], P["ln2_b"])
    return out, {"qkv": qkv, "ctx": ctx, "h1": h1, "f": f}
