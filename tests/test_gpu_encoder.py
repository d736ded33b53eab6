"""BERT-style int8 encoder layer on the GPU against the numpy restatement in oracle/encoder_layer.py.
Tolerance of the layer output: 1e-3 relative (max |diff| / max |want|), the bar the path states for
the full layer; the fp32 pieces on their own are held to 2e-5."""
import os
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

sys.path.insert(0, os.path.join(os.path.dirname(os.path.abspath(__file__)), "..", "oracle"))
import encoder_layer as ref_layer  # noqa: E402
from bolt_amd import capi  # noqa: E402
from bolt_amd.host_encoder import EncoderLayer  # noqa: E402

LAYER_RTOL = 1e-3


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def rel(got, want):
    return float(np.abs(got.astype(np.float64) - want).max() / np.abs(want).max())


def make_params(rng, hidden, ffn, with_bias=True):
    P = {}
    for name, N, K in (("qkv", 3 * hidden, hidden), ("o", hidden, hidden), ("1", ffn, hidden), ("2", hidden, ffn)):
        W = (rng.standard_normal((N, K)) * 0.02).astype(np.float32)
        P["w" + name], P["s" + name] = ref_layer.quantize_weight_per_channel(W)
        P["b" + name] = (rng.standard_normal(N) * 0.02).astype(np.float32) if with_bias else None
    for k in ("ln1", "ln2"):
        P[k + "_g"] = (1.0 + 0.1 * rng.standard_normal(hidden)).astype(np.float32) if with_bias else np.ones(hidden, np.float32)
        P[k + "_b"] = (0.1 * rng.standard_normal(hidden)).astype(np.float32) if with_bias else np.zeros(hidden, np.float32)
    return P


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


@pytest.mark.parametrize("shape", [(1, 1, 64, 1), (2, 24, 128, 2), (3, 70, 192, 3), (2, 128, 768, 12)])
def test_attention(torch_mod, shape):
    torch = torch_mod
    batch, seq, hidden, heads = shape
    rng = np.random.default_rng(sum(shape))
    qkv = rng.standard_normal((batch * seq, 3 * hidden)).astype(np.float32)
    want = ref_layer.attention(qkv, batch, seq, hidden, heads)
    out = torch.zeros((batch * seq, hidden), dtype=torch.float32, device="cuda")
    dq = dev(torch, qkv)
    capi.check(capi.lib().bolt_gfx950_attention_f32(dq.data_ptr(), batch, seq, hidden, heads, out.data_ptr()), "attention")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert rel(out.cpu().numpy(), want) < 2e-5


@pytest.mark.parametrize("rows,hidden", [(1, 4), (5, 64), (7, 252), (33, 768), (9, 1024), (4, 2048)])
def test_add_layernorm(torch_mod, rows, hidden):
    torch = torch_mod
    rng = np.random.default_rng(rows + hidden)
    a = rng.standard_normal((rows, hidden)).astype(np.float32) * 3
    b = rng.standard_normal((rows, hidden)).astype(np.float32)
    g = rng.standard_normal(hidden).astype(np.float32)
    be = rng.standard_normal(hidden).astype(np.float32)
    out = torch.zeros((rows, hidden), dtype=torch.float32, device="cuda")
    L = capi.lib()
    da, db, dg, dbe = dev(torch, a), dev(torch, b), dev(torch, g), dev(torch, be)    # kept alive across the calls
    capi.check(L.bolt_gfx950_add_layernorm_f32(da.data_ptr(), db.data_ptr(), dg.data_ptr(), dbe.data_ptr(), rows, hidden,
                                               out.data_ptr()), "ln")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert rel(out.cpu().numpy(), ref_layer.layer_norm(a + b, g, be)) < 2e-5
    capi.check(L.bolt_gfx950_add_layernorm_f32(da.data_ptr(), None, dg.data_ptr(), dbe.data_ptr(), rows, hidden,
                                               out.data_ptr()), "ln")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert rel(out.cpu().numpy(), ref_layer.layer_norm(a, g, be)) < 2e-5
    assert L.bolt_gfx950_add_layernorm_f32(None, None, None, None, rows, hidden, None) == capi.NULL_POINTER


def test_gelu(torch_mod):
    torch = torch_mod
    x = np.concatenate([np.linspace(-12, 12, 4001, dtype=np.float32)[:4000], np.array([-100, 100, 0, -0.0], np.float32)])
    t = dev(torch, x)
    capi.check(capi.lib().bolt_gfx950_gelu_f32(t.data_ptr(), x.size), "gelu")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    got = t.cpu().numpy()
    want = ref_layer.gelu(x)
    assert np.abs(got - want).max() < 2e-5 and got[-4] == 0.0 and got[-3] == 100.0


@pytest.mark.parametrize("cfg", [(2, 24, 128, 2, 256, True), (1, 128, 256, 4, 512, False), (3, 50, 192, 3, 384, True)])
def test_encoder_layer_small(torch_mod, oracle, cfg):
    torch = torch_mod
    batch, seq, hidden, heads, ffn, with_bias = cfg
    print("encoder", cfg, flush=True)
    rng = np.random.default_rng(sum(cfg[:5]))
    P = make_params(rng, hidden, ffn, with_bias)
    x = rng.standard_normal((batch * seq, hidden)).astype(np.float32)
    want, _ = ref_layer.encoder_layer(oracle, x, P, batch, seq, hidden, heads)
    layer = EncoderLayer(torch, batch, seq, hidden, heads, ffn, P)
    got = layer(dev(torch, x))
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    r = rel(got.cpu().numpy(), want)
    print("rel", r, flush=True)
    assert r < LAYER_RTOL
    # a second call on the same workspace gives the same bytes (scratch slots are re-zeroed every call)
    again = layer(dev(torch, x))
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(got, again)


def rel_l2(got, want):
    return float(np.linalg.norm(got.astype(np.float64) - want) / np.linalg.norm(want.astype(np.float64)))


def test_encoder_layer_bert_base(torch_mod, oracle):
    """BASELINE configs[3]: hidden 768, 12 heads, FFN 3072, seq 128, batch 32, weights N(0, 0.02), biases 0,
    LayerNorm gamma 1 / beta 0, hidden states N(0, 1).

    Stage by stage, each stage of the oracle fed with the GPU's own input to that stage: the four int8
    FullyConnected stages (quantise + GEMM + per-channel dequantise) must be bit-exact, the fp32 stages
    within 2e-5. End to end against the oracle run on its own: 1e-3 relative in the L2 norm. Individual
    elements can differ by more: a 1-ulp fp32 difference ahead of a quantiser occasionally moves one
    activation by one int8 step (here max|act|/127 of the GELU output, times one weight), so the max-norm is
    held to 1e-2 and the fraction of elements off by more than 1e-3 of max|out| to 1e-3."""
    torch = torch_mod
    batch, seq, hidden, heads, ffn = 32, 128, 768, 12, 3072
    rng = np.random.default_rng(20240604)
    P = make_params(rng, hidden, ffn, with_bias=False)
    x = rng.standard_normal((batch * seq, hidden)).astype(np.float32)
    layer = EncoderLayer(torch, batch, seq, hidden, heads, ffn, P)
    L = capi.lib()
    dx = dev(torch, x)
    # separate kernels first: that form keeps every fp32 intermediate for the stage-wise checks below
    capi.check(L.bolt_gfx950_set_option(b"encoder_fused", 0), "set_option")
    try:
        got = layer(dx)
        capi.check(L.bolt_gfx950_synchronize(), "sync")
    finally:
        capi.check(L.bolt_gfx950_set_option(b"encoder_fused", 1), "set_option")
    mid = {k: v.cpu().numpy() for k, v in layer.intermediates().items()}
    # the default form (FullyConnected + GELU + quantisation in one launch) does the same arithmetic element for
    # element: the layer output must be the same bytes -- also when its grid-wide wait is forced to give up from the
    # host (a bound of one poll), which sends it through its two-pass fallback
    fused = layer(dx)
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert torch.equal(fused, got), "fused FullyConnected + GELU + quantise differs from the separate kernels"
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 1), "set_option")
    try:
        for rep in range(3):
            forced = layer(dx)
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            assert torch.equal(forced, got), "fallback of the fused form differs (repetition %d)" % rep
    finally:
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 0), "set_option")
    again = layer(dx)
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert torch.equal(again, got)
    got = got.cpu().numpy()

    def same_bits(a, b):
        return np.array_equal(a.view(np.int32), b.view(np.int32))
    assert same_bits(mid["qkv"], ref_layer.int8_fc(oracle, x, P["wqkv"], P["sqkv"], P["bqkv"])[0])
    assert rel(mid["ctx"], ref_layer.attention(mid["qkv"], batch, seq, hidden, heads)) < 2e-5
    assert same_bits(mid["attn_out"], ref_layer.int8_fc(oracle, mid["ctx"], P["wo"], P["so"], P["bo"])[0])
    assert rel(mid["h1"], ref_layer.layer_norm(x + mid["attn_out"], P["ln1_g"], P["ln1_b"])) < 2e-5
    assert same_bits(mid["ffn_pre"], ref_layer.int8_fc(oracle, mid["h1"], P["w1"], P["s1"], P["b1"])[0])
    # the layer never stores the activated values (its quantiser applies GELU to what it reads): take them from the
    # stand-alone GELU entry point, which runs the same device function
    act = dev(torch, mid["ffn_pre"].copy())
    capi.check(capi.lib().bolt_gfx950_gelu_f32(act.data_ptr(), act.numel()), "gelu")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    act = act.cpu().numpy()
    assert rel(act, ref_layer.gelu(mid["ffn_pre"])) < 2e-5
    assert same_bits(mid["ffn_out"], ref_layer.int8_fc(oracle, act, P["w2"], P["s2"], P["b2"])[0])
    assert rel(got, ref_layer.layer_norm(mid["h1"] + mid["ffn_out"], P["ln2_g"], P["ln2_b"])) < 2e-5

    want, _ = ref_layer.encoder_layer(oracle, x, P, batch, seq, hidden, heads)
    r2, rmax = rel_l2(got, want), rel(got, want)
    frac = float((np.abs(got - want) > 1e-3 * np.abs(want).max()).mean())
    print("bert-base layer: rel L2 %.3g, max-norm %.3g, fraction off by > 1e-3: %.3g" % (r2, rmax, frac), flush=True)
    assert r2 < LAYER_RTOL and rmax < 1e-2 and frac < 1e-3


def test_encoder_layer_calls_do_not_leak_maxima(torch_mod):
    """The layer's running maxima live in scratch slots that are cleared inside the layer's own kernels rather than
    by a launch of their own: a call on small activations must give the same bits before and after a call on
    activations a hundred times larger."""
    torch = torch_mod
    batch, seq, hidden, heads, ffn = 2, 64, 256, 4, 512
    rng = np.random.default_rng(11)
    P = make_params(rng, hidden, ffn, with_bias=True)
    x = rng.standard_normal((batch * seq, hidden)).astype(np.float32)
    layer = EncoderLayer(torch, batch, seq, hidden, heads, ffn, P)
    small, big = dev(torch, 0.05 * x), dev(torch, 5.0 * x + 3.0)
    a = layer(small).clone()
    layer(big)
    b = layer(small).clone()
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(a, b)


def test_encoder_errors(torch_mod):
    L = capi.lib()
    spec = capi.BoltEncoderLayerInt8()
    n = capi.C.c_size_t(0)
    assert L.bolt_gfx950_encoder_layer_int8_workspace_bytes(None, capi.C.byref(n)) == capi.NULL_POINTER
    assert L.bolt_gfx950_encoder_layer_int8_workspace_bytes(capi.C.byref(spec), capi.C.byref(n)) == capi.NULL_POINTER


def test_encoder_layer_fused_ffn_other_shape(torch_mod):
    """Another shape that takes the one-launch FullyConnected + GELU + quantise (4096 tokens x FFN 2048 = 128 tiles of
    256 x 256, biases present): same bytes as the separate kernels."""
    torch = torch_mod
    batch, seq, hidden, heads, ffn = 16, 256, 256, 4, 2048
    rng = np.random.default_rng(77)
    P = make_params(rng, hidden, ffn, with_bias=True)
    x = dev(torch, rng.standard_normal((batch * seq, hidden)).astype(np.float32))
    layer = EncoderLayer(torch, batch, seq, hidden, heads, ffn, P)
    L = capi.lib()
    capi.check(L.bolt_gfx950_set_option(b"encoder_fused", 0), "set_option")
    try:
        plain = layer(x).clone()
        capi.check(L.bolt_gfx950_synchronize(), "sync")
    finally:
        capi.check(L.bolt_gfx950_set_option(b"encoder_fused", 1), "set_option")
    fused = layer(x)
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert torch.equal(fused, plain)


@pytest.mark.gpu
def test_encoder_stack_equals_layer_by_layer(torch_mod):
    """bolt_gfx950_encoder_stack_int8 over three layers with different weights (two FFN widths, so the layers' workspaces
    differ) gives, bit for bit, what three single-layer calls give: the maximum the LayerNorm at the end of a layer
    folds for the next one is the maximum that layer's own abs-max pass would have found. Run twice, and once after
    a single-layer call in between, so that slots left over from one form cannot leak into the other."""
    from bolt_amd.host_encoder import EncoderStack
    torch = torch_mod
    batch, seq, hidden, heads = 8, 96, 256, 4
    rng = np.random.default_rng(4242)
    layers = []
    for ffn in (1024, 512, 1024):
        layers.append(EncoderLayer(torch, batch, seq, hidden, heads, ffn, make_params(rng, hidden, ffn, with_bias=True)))
    x = dev(torch, rng.standard_normal((batch * seq, hidden)).astype(np.float32))
    want = x
    for l in layers:
        want = l(want).clone()
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    stack = EncoderStack(torch, layers)
    for rep in range(2):
        got = stack(x)
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        assert torch.equal(got, want), "stack differs from layer-by-layer (repetition %d)" % rep
        layers[1](x)   # a single-layer call between two stack calls
    one = EncoderStack(torch, layers[:1])
    assert torch.equal(one(x), layers[0](x))
    n = capi.C.c_size_t(0)
    assert capi.lib().bolt_gfx950_encoder_stack_int8_workspace_bytes(stack.specs, 0, capi.C.byref(n)) == capi.NOT_SUPPORTED
