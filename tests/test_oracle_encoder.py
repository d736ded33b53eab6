"""Pins oracle/encoder_layer.py (the numpy restatement of the fp32 neighbours of the int8 GEMMs in an encoder
layer) on the CPU, so that a wrong epsilon, variance formula, GELU form, softmax scale or weight-quantisation rule
fails here and not only against the GPU:

  * against the reference's own compiled kernels (oracle/_ref: layer_norm.cpp, softmax.cpp and the GELU of
    x86_functions_fp32.h) where that library can run, and against the bytes it returned, committed in
    tests/golden/encoder_fp32.npz, everywhere else;
  * against torch's CPU implementations and closed forms (hand-computed rows, uniform scores, known points).

Tolerances: the reference evaluates exp with a degree-5 polynomial (x86_avx2_expand.h:60-111, ~2e-7 relative) and
sums in fp32 lanes; the oracle sums in float64 and rounds once. 2e-6 of the output's magnitude separates those and is
40x below the next plausible mistake (eps 1e-5 instead of 1e-6 moves a unit-variance row by 4.5e-6 relative, see the
low-variance rows below where it moves it by 70 %)."""
import os
import sys

import numpy as np
import pytest

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
sys.path.insert(0, os.path.join(ROOT, "oracle"))

import encoder_layer as E  # noqa: E402
from checkers import DT_I8  # noqa: E402
from checkers_tensor import RefTensor  # noqa: E402

GOLD = os.path.join(ROOT, "tests", "golden", "encoder_fp32.npz")
F = np.float32


def ln_inputs():
    rng = np.random.default_rng(20240611)
    x = (rng.standard_normal((48, 768)) * 2.0 + 0.3).astype(F)
    x[5] = F(3.0) + (rng.standard_normal(768) * 1e-3).astype(F)   # variance 1e-6: the epsilon decides the result
    x[6] = F(-1.5)                                                # zero variance: out = beta
    g = rng.standard_normal(768).astype(F)
    b = rng.standard_normal(768).astype(F)
    return x, g, b


def gelu_inputs():
    rng = np.random.default_rng(20240612)
    x = np.concatenate([(rng.standard_normal(4072) * 3.0).astype(F),
                        np.array([0.0, -0.0, 1.0, -1.0, 0.5, -0.5, 8.0, -8.0, 20.0, -20.0, 1e-4, -1e-4, 3.0, -3.0, 2.0,
                                  -2.0, 60.0, -60.0, 0.1, -0.1, 5.0, -5.0, 12.0, -12.0], F)])
    return x


def softmax_inputs():
    rng = np.random.default_rng(20240613)
    s = (rng.standard_normal((96, 128)) * 4.0).astype(F)
    s[3] = 0.0            # uniform
    s[4, 7] = 60.0        # one dominant score
    return s


@pytest.fixture(scope="module")
def reft():
    if not RefTensor.available():
        pytest.skip("oracle/_ref/libboltref.so not built or host lacks avx512_vnni")
    return RefTensor()


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def close(a, b, tol):
    return float(np.abs(a.astype(np.float64) - b.astype(np.float64)).max()) <= tol * max(1.0, float(np.abs(b).max()))


# ---- LayerNorm ------------------------------------------------------------------------------------------------
def ln_close(got, want):
    """Rows of ordinary variance to 2e-6; row 5 (mean 3, variance 1e-6) is ill-conditioned in fp32 -- the
    reference's fp32 mean is off by an ulp of 3, a third of a per cent of that row's standard deviation -- and is
    held to 1e-3 of its magnitude, still 700 times tighter than what a wrong epsilon does to it."""
    rest = np.ones(got.shape[0], bool)
    rest[5] = False
    return close(got[rest], want[rest], 2e-6) and close(got[5], want[5], 1e-3)


def test_layer_norm_vs_reference(reft):
    x, g, b = ln_inputs()
    assert ln_close(E.layer_norm(x, g, b), reft.layer_norm(x, g, b))


def test_layer_norm_vs_golden(gold):
    x, g, b = ln_inputs()
    assert np.array_equal(x, gold["ln_x"])
    assert ln_close(E.layer_norm(x, g, b), gold["ln_y"])


def test_layer_norm_closed_forms():
    import torch
    x, g, b = ln_inputs()
    want = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (768,), torch.from_numpy(g).double(),
                                          torch.from_numpy(b).double(), eps=1e-6).numpy()
    got = E.layer_norm(x, g, b)
    assert ln_close(got, want)
    # the epsilon is 1e-6 (layer_norm.cpp:19), not torch's default 1e-5: row 5 has variance ~1e-6
    other = torch.nn.functional.layer_norm(torch.from_numpy(x).double(), (768,), torch.from_numpy(g).double(),
                                           torch.from_numpy(b).double(), eps=1e-5).numpy()
    assert np.abs(other[5] - want[5]).max() > 0.1 * np.abs(want[5]).max()
    assert np.array_equal(got[6], b)                       # zero variance: (x - mean) = 0 exactly
    # hand-computed row: x = [1, 2, 3, 6]: mean 3, population variance 3.5 (the unbiased one would be 14 / 3)
    row = np.array([[1.0, 2.0, 3.0, 6.0]], F)
    y = E.layer_norm(row, np.array([1, 1, 2, 2], F), np.array([0, 1, 0, -1], F))
    sd = np.sqrt(3.5 + 1e-6)
    assert np.allclose(y[0], [-2 / sd, -1 / sd + 1, 0.0, 2 * 3 / sd - 1], rtol=0, atol=1e-6)


# ---- GELU -----------------------------------------------------------------------------------------------------
def test_gelu_vs_reference(reft):
    x = gelu_inputs()
    got, want = E.gelu(x), reft.gelu(x)
    assert float(np.abs(got - want).max()) <= 2e-6 * float(np.abs(want).max())
    assert float((np.abs(got - want) / np.maximum(np.abs(want), 1e-2)).max()) <= 5e-5   # the reference's exp polynomial


def test_gelu_vs_golden(gold):
    x = gelu_inputs()
    assert np.array_equal(x, gold["gelu_x"])
    assert float(np.abs(E.gelu(x) - gold["gelu_y"]).max()) <= 2e-6 * float(np.abs(gold["gelu_y"]).max())


def test_gelu_closed_forms():
    import torch
    x = gelu_inputs()
    got = E.gelu(x)
    want = torch.nn.functional.gelu(torch.from_numpy(x).double(), approximate="tanh").numpy()
    assert float(np.abs(got - want).max()) <= 1e-6 * float(np.abs(want).max())
    erf = torch.nn.functional.gelu(torch.from_numpy(x).double()).numpy()
    assert float(np.abs(erf - want).max()) > 1e-4          # the erf form is a different function at this tolerance
    pts = dict(zip(x[-24:].tolist(), got[-24:].tolist()))
    assert pts[0.0] == 0.0 and pts[20.0] == 20.0 and pts[60.0] == 60.0 and abs(pts[-20.0]) == 0.0
    assert abs(pts[1.0] - 0.8411919906082768) < 1e-6 and abs(pts[-1.0] + 0.15880800939172324) < 1e-6


# ---- softmax and attention ------------------------------------------------------------------------------------
def oracle_softmax(s):
    """The softmax inside E.attention, exposed through a single head of dimension 64: with V = identity on the first
    `keys` coordinates the context rows are the probabilities themselves."""
    rows, keys = s.shape
    assert keys <= 64 and rows <= keys
    q = np.zeros((keys, 64), F)
    k = np.zeros((keys, 64), F)
    v = np.zeros((keys, 64), F)
    q[:rows, :keys] = s * F(8.0)                 # attention scales q by 1/8 for a head of 64
    k[:, :keys] = np.eye(keys, dtype=F)
    v[:, :keys] = np.eye(keys, dtype=F)
    qkv = np.concatenate([q, k, v], axis=1)
    return E.attention(qkv, 1, keys, 64, 1)[:rows, :keys]


def test_softmax_vs_reference(reft):
    s = softmax_inputs()
    want = reft.softmax(s)
    p = np.exp(s.astype(np.float64) - s.max(axis=1, keepdims=True))
    p /= p.sum(axis=1, keepdims=True)
    assert float(np.abs(want - p).max()) <= 1e-6           # the reference is a softmax over the last axis, max-subtracted
    small = s[:32, :64] / F(4.0)
    assert float(np.abs(oracle_softmax(small) - reft.softmax(small)).max()) <= 1e-6


def test_softmax_vs_golden(gold):
    s = softmax_inputs()
    assert np.array_equal(s, gold["softmax_x"])
    small = s[:32, :64] / F(4.0)
    assert float(np.abs(oracle_softmax(small) - gold["softmax_small_y"]).max()) <= 1e-6


def test_attention_closed_forms():
    import torch
    rng = np.random.default_rng(20240614)
    batch, seq, hidden, heads = 2, 40, 192, 3
    qkv = rng.standard_normal((batch * seq, 3 * hidden)).astype(F)
    got = E.attention(qkv, batch, seq, hidden, heads)
    t = torch.from_numpy(qkv).double().reshape(batch, seq, 3, heads, 64)
    q, k, v = (t[:, :, i].permute(0, 2, 1, 3) for i in range(3))
    p = torch.softmax(q @ k.transpose(-1, -2) / 8.0, dim=-1)        # scale 1 / sqrt(head size)
    want = (p @ v).permute(0, 2, 1, 3).reshape(batch * seq, hidden).numpy()
    assert float(np.abs(got - want).max()) <= 1e-6
    unscaled = (torch.softmax(q @ k.transpose(-1, -2), dim=-1) @ v).permute(0, 2, 1, 3).reshape(batch * seq, hidden)
    assert float(np.abs(unscaled.numpy() - want).max()) > 1e-2      # a dropped 1/8 shows
    # uniform scores (all keys equal): every context row is the mean of V over the keys of its own batch and head
    qkv2 = qkv.copy()
    qkv2[:, hidden:2 * hidden] = qkv2[0, hidden:2 * hidden]
    got2 = E.attention(qkv2, batch, seq, hidden, heads)
    vmean = qkv2[:, 2 * hidden:].reshape(batch, seq, hidden).astype(np.float64).mean(axis=1)
    assert float(np.abs(got2.reshape(batch, seq, hidden) - vmean[:, None, :]).max()) <= 1e-6


# ---- per-channel weight quantisation --------------------------------------------------------------------------
def test_quantize_weight_per_channel(oracle):
    rng = np.random.default_rng(20240615)
    W = (rng.standard_normal((37, 200)) * 0.02).astype(F)
    W[3] = 0.0
    W[4, 9] = 1.0
    tie = np.arange(-126, 127, dtype=F)[:200] + F(0.5)
    W[5] = tie
    W[5, 0] = 127.0          # scale exactly 1: the rest of the row sits on .5 ties -> round half to even
    q, s = E.quantize_weight_per_channel(W)
    for n in range(W.shape[0]):
        wq, ws = oracle.quantize_f32(W[n], DT_I8)     # quantizeF32ToI8 per row (avx512/quantize.cpp:181-234)
        assert s[n] == ws and np.array_equal(q[n], wq), n
    assert s[3] == 1.0 and not q[3].any() and s[5] == 1.0
    assert np.array_equal(q[5, 1:5], np.array([-124, -124, -122, -122], np.int8))
