"""Pins the CPU oracle against the committed golden vectors: bytes the reference's own compiled x86
AVX-512-VNNI path returned for seeded inputs (written by tests/golden/make_golden.py). Needs neither
the reference nor a GPU, so it also runs where oracle/_ref cannot."""
import os

import numpy as np
import pytest

from checkers import DT_F32, DT_I8, DT_I32, DT_U8_Q
from checkers_conv import ConvOracle

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden")


def load(name):
    return np.load(os.path.join(GOLD, name + ".npz"), allow_pickle=False)


def same(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.shape == b.shape and a.dtype == b.dtype and a.tobytes() == b.tobytes()


def test_sizes(oracle):
    g = load("sizes")
    for N, K, b, r, bp, rp, wv, wvp, tv, tvp, wu in g["pack"]:
        assert oracle.mmm_transform_rhs_bytes(N, K) == (b, r)
        assert oracle.mmm_transform_rhs_bytes(N, K, packed=True) == (bp, rp)
        assert oracle.mvm_transform_weight_bytes(N, K) == wv == tv
        assert oracle.mvm_transform_weight_bytes(N, K, packed=True) == wvp
        assert oracle.mvm_transform_weight_bytes(N, K, DT_U8_Q, packed=False) == wu
    for N, K, M, tA, pk, want in g["mmm_tmp"]:
        assert oracle.mmm_tmp_bytes(N, M, K, bool(tA), bool(pk)) == want


def test_mmm(oracle):
    g = load("mmm")
    for i, (M, K, N) in enumerate(g["shapes"]):
        A, W, off, ob, cin, s = g[f"A{i}"], g[f"W{i}"], g[f"offsetC{i}"], g[f"ob{i}"], g[f"cin{i}"], g[f"s{i}"]
        assert same(oracle.offsetC(W, True), off)
        assert same(oracle.bias_offsetC(g[f"bias{i}"], off, s), ob)
        assert same(oracle.mmm(A, W, ob, cin, DT_I32), g[f"i32_{i}"])
        assert same(oracle.mmm(A, W, ob, np.zeros((M, N), np.float32), DT_F32, scale=[s]), g[f"f32_{i}"])
        if f"i32_tA_{i}" in g.files:      # the reference's transposed-A route is only a product for K <= 4096
            assert same(oracle.mmm(np.ascontiguousarray(A.T), W, off, cin, DT_I32, transA=True), g[f"i32_tA_{i}"])
        assert same(oracle.mmm(A, W, off, cin, DT_I32), g[f"i32_unpacked_{i}"])
        assert same(oracle.mmm(A, W, ob, np.zeros((M, N), np.uint8), DT_U8_Q, scale=[-1.0, g[f"u8scale{i}"]]),
                    g[f"u8_{i}"])


def test_mvm(oracle):
    g = load("mvm")
    for i, (N, K) in enumerate(g["shapes"]):
        W, x, off, yin, s = g[f"W{i}"], g[f"x{i}"], g[f"offsetC{i}"], g[f"yin{i}"], g[f"s{i}"]
        assert same(oracle.mvm(W, x, off, yin, DT_I32), g[f"i32_{i}"])
        assert same(oracle.mvm(W, x, off, np.zeros(N, np.float32), DT_F32, scale=[s]), g[f"f32_{i}"])
        assert same(oracle.mvm(W, x, off, yin, DT_I32), g[f"i32_unpacked_{i}"])
        assert same(oracle.mvm(W, x, off, yin, DT_I32), g[f"i32_unpackedT_{i}"])
        assert same(oracle.mvm(W, x, off, np.zeros(N, np.uint8), DT_U8_Q, scale=[-1.0, g[f"u8scale{i}"]]), g[f"u8_{i}"])
        assert same(oracle.mvm_u8mat(g[f"uA{i}"], g[f"uv{i}"], yin, DT_I32), g[f"u8mat_i32_{i}"])


def test_quantize_family(oracle):
    g = load("quantize")
    for i, n in enumerate(g["ns"]):
        x, acc, u = g[f"x{i}"], g[f"acc{i}"], g[f"u{i}"]
        for nm, qdt in (("u8", DT_U8_Q), ("i8", DT_I8)):
            for tag, sc, mode in (("dyn", -1.0, 0), ("static", 20.0, 1), ("floor", 1000.0, 0)):
                q, s = oracle.quantize_f32(x, qdt, sc, mode)
                assert same(q, g[f"{nm}_{tag}_{i}"]) and s == g[f"{nm}_{tag}_s{i}"][0], (nm, tag, n)
            for tag, s0 in (("i32dyn", -1.0), ("i32static", 0.02)):
                q, s = oracle.quantize_i32(acc, qdt, [s0, 37.5])
                assert same(q, g[f"{nm}_{tag}_{i}"]) and same(s, g[f"{nm}_{tag}_s{i}"]), (nm, tag, n)
        assert same(oracle.u8_to_i8(u), g[f"u_to_i8_{i}"])
        assert same(oracle.dequantize(acc, DT_I32, 37.5), g[f"deq_i32_{i}"])
        assert same(oracle.dequantize(u, DT_U8_Q, 11.25), g[f"deq_u8_{i}"])
        assert same(oracle.bias_offsetC(g[f"b{i}"], g[f"o{i}"], 123.456), g[f"bias_offsetC_{i}"])
        assert same(oracle.bias_offsetC(g[f"b{i}"], None, 123.456), g[f"bias_only_{i}"])
        assert same(oracle.requantize(g[f"r{i}"], 10.0, 7.3), g[f"requant_{i}"])
    for nm, qdt in (("u8", DT_U8_Q), ("i8", DT_I8)):
        q, s = oracle.quantize_f32(g["ties"], qdt)
        assert s == 1.0 == g[f"ties_{nm}_s"][0] and same(q, g[f"ties_{nm}"])
    assert same(oracle.bias_offsetC(g["bias_ties"], None, 8.0), g["bias_ties_out"])


def test_conv_int8(oracle):
    co = ConvOracle(oracle)
    g = load("conv_int8")
    for i, case in enumerate(g["cases"]):
        n, ic, ih, iw, oc, fh, fw, stride, pad = (int(v) for v in case)
        for relu in (0, 1):
            for nm, odt in (("u8", DT_U8_Q), ("f32", DT_F32)):
                d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, bool(relu), odt)
                got, gs = co.conv(d, g[f"xq{i}"], g[f"W{i}"], g[f"bias{i}"], [g[f"sI{i}"], -1.0, g[f"sF{i}"]])
                assert same(gs, g[f"{nm}_relu{relu}_scale{i}"]), (case, nm, relu)
                assert same(got, g[f"{nm}_relu{relu}_{i}"]), (case, nm, relu)


def test_pool_and_concat(oracle):
    from checkers_pool import orc_concat, orc_pooling, pool_desc
    g = load("pool_concat")
    for i, case in enumerate(g["pool_cases"]):
        d = pool_desc(tuple(int(v) for v in case))
        y, s = orc_pooling(oracle, d, g[f"pool_x{i}"], 12.75)
        assert same(y, g[f"pool_y{i}"]) and same(np.float32(s), g[f"pool_s{i}"])
    for i in range(int(g["concat_n"])):
        dims = g[f"cat_dims{i}"]
        axis = int(g[f"cat_meta{i}"][1]) % 4
        parts = [g[f"cat_in{i}_{j}"] for j in range(len(dims))]
        lens = [int(np.prod(d[axis:])) for d in dims]
        loops = int(np.prod(dims[0][:axis]))
        y, s = orc_concat(oracle, parts, lens, loops, g[f"cat_scales{i}"])
        assert same(y, g[f"cat_y{i}"]) and same(np.float32(s), g[f"cat_s{i}"])


def test_axpby(oracle):
    from test_oracle_vs_ref import AXPBY_NS, axpby_inputs
    g = load("orchestration")
    for n in AXPBY_NS:
        a, x, b, y = axpby_inputs(n)
        assert same(oracle.axpby(a, x, b, y), g[f"axpby_{n}"])
