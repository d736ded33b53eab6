"""Writes the golden vectors under tests/golden/ by calling the reference's own compiled x86
AVX-512-VNNI path (oracle/_ref/libboltref.so, built by `make -C oracle ref` from the sources under
/root/reference). Run once where that library can run:

    python tests/golden/make_golden.py

Every fixture is data only: seeded inputs and the bytes the reference returned for them, stored as
compressed .npz (numeric arrays, loadable with allow_pickle=False). tests/test_golden.py checks the
CPU oracle against them, tests/test_gpu_golden.py the HIP path, neither needs the reference.
"""
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(HERE))

from checkers import DT_F32, DT_I8, DT_I32, DT_U8_Q, Oracle, Ref  # noqa: E402
from checkers_conv import DF_NCHWC8, ConvOracle, ref_conv, to_nchwc  # noqa: E402
from checkers_pool import pool_desc, ref_concat, ref_pooling  # noqa: E402

SEED = 20240601


def save(name, arrays):
    path = os.path.join(HERE, name + ".npz")
    np.savez_compressed(path, **arrays)
    print(name, len(arrays), "arrays", os.path.getsize(path), "bytes")


def gen_sizes(ref):
    rows = []
    for N in (1, 7, 16, 17, 48, 100, 768, 1024, 3072, 4096):
        for K in (1, 7, 8, 9, 77, 768, 1024, 3072, 4096, 4097):
            b, r = ref.mmm_transform_rhs_bytes(1, K, N)
            bp, rp = ref.mmm_transform_rhs_bytes(2, K, N)
            rows.append([N, K, b, r, bp, rp, ref.mvm_transform_weight_bytes(0, N, K),
                         ref.mvm_transform_weight_bytes(2, N, K), ref.mvm_tmp_bytes(0, N, K),
                         ref.mvm_tmp_bytes(2, N, K), ref.mvm_transform_weight_bytes(0, N, K, DT_U8_Q)])
    tmp = []
    for N in (1, 17, 48, 1024):
        for K in (1, 9, 768, 4097):
            for M in (1, 5, 24, 25, 64, 385):
                for tA in (0, 1):
                    for pk in (0, 1):
                        tmp.append([N, K, M, tA, pk, ref.mmm_tmp_bytes(bool(tA), 2 if pk else 1, M, K, N)])
    save("sizes", {"pack": np.array(rows, np.int64), "mmm_tmp": np.array(tmp, np.int64)})


def gen_mmm(ref, orc):
    rng = np.random.default_rng(SEED + 1)
    out = {}
    shapes = [(1, 1, 1), (3, 9, 17), (8, 64, 48), (25, 77, 100), (7, 130, 33), (24, 256, 64), (33, 40, 31), (5, 4100, 20)]
    out["shapes"] = np.array(shapes, np.int64)
    for i, (M, K, N) in enumerate(shapes):
        A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        blob, rhs, _ = ref.mmm_transform_rhs(1, K, N, W)
        off = blob[rhs:rhs + 4 * N].view(np.int32).copy()
        bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
        s = np.float32(rng.random() * 40 + 5)
        ob = ref.bias_offsetC(bias, off, s)
        cin = rng.integers(-1000, 1000, size=(M, N), dtype=np.int32)
        out[f"A{i}"], out[f"W{i}"], out[f"offsetC{i}"], out[f"bias{i}"], out[f"s{i}"] = A, W, off, bias, s
        out[f"ob{i}"], out[f"cin{i}"] = ob, cin
        out[f"i32_{i}"] = ref.mmm(A, blob, 2, M, K, N, ob, cin, DT_I32)
        out[f"f32_{i}"] = ref.mmm(A, blob, 2, M, K, N, ob, np.zeros((M, N), np.float32), DT_F32, scale=[s])
        # transposed A and unpacked B routes (int32)
        # Transposed A is pinned for K <= 4096 only: from its second K block on the reference transposes
        # out of its own scratch instead of the caller's matrix (mmm_avx512_vnni.cpp:1855-1860: packA = tmp
        # after the first block), so its result for larger K is not the product.
        if K <= 4096:
            out[f"i32_tA_{i}"] = ref.mmm(np.ascontiguousarray(A.T), blob, 2, M, K, N, off, cin, DT_I32, transA=True)
        out[f"i32_unpacked_{i}"] = ref.mmm(A, np.ascontiguousarray(W.T), 0, M, K, N, None, cin, DT_I32)
        # u8 output: one row per call (the reference's row stride for u8 stores is 4 * N)
        f = np.float32(127.0 / max(1, np.abs(out[f"i32_{i}"] - cin).max()))
        out[f"u8scale{i}"] = f
        u8 = np.zeros((M, N), np.uint8)
        for m in range(M):
            u8[m] = ref.mmm(A[m:m + 1], blob, 2, 1, K, N, ob, np.zeros((1, N), np.uint8), DT_U8_Q, scale=[-1.0, f])[0]
        out[f"u8_{i}"] = u8
    save("mmm", out)


def gen_mvm(ref, orc):
    rng = np.random.default_rng(SEED + 2)
    out = {}
    shapes = [(1, 1), (7, 9), (16, 64), (33, 77), (65, 130), (100, 256), (31, 4100), (256, 40)]
    out["shapes"] = np.array(shapes, np.int64)
    for i, (N, K) in enumerate(shapes):
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        x = rng.integers(0, 256, size=K, dtype=np.uint8)
        blob, _ = ref.mvm_transform_weight(0, N, K, W)
        off = (-128 * W.astype(np.int64).sum(axis=1)).astype(np.int32)
        yin = rng.integers(-1000, 1000, size=N, dtype=np.int32)
        s = np.float32(rng.random() * 40 + 5)
        out[f"W{i}"], out[f"x{i}"], out[f"offsetC{i}"], out[f"yin{i}"], out[f"s{i}"] = W, x, off, yin, s
        out[f"i32_{i}"] = ref.mvm(blob, x, 2, N, K, off, yin, DT_I32)
        out[f"f32_{i}"] = ref.mvm(blob, x, 2, N, K, off, np.zeros(N, np.float32), DT_F32, scale=[s])
        out[f"i32_unpacked_{i}"] = ref.mvm(W, x, 0, N, K, None, yin, DT_I32)
        out[f"i32_unpackedT_{i}"] = ref.mvm(np.ascontiguousarray(W.T), x, 1, N, K, None, yin, DT_I32)
        f = np.float32(127.0 / max(1, np.abs(out[f"i32_{i}"] - yin).max()))
        out[f"u8scale{i}"] = f
        out[f"u8_{i}"] = ref.mvm(blob, x, 2, N, K, off, np.zeros(N, np.uint8), DT_U8_Q, scale=[-1.0, f])
        # u8 matrix x s8 vector (row kernel)
        A = rng.integers(0, 256, size=(N, K), dtype=np.uint8)
        v = rng.integers(-127, 128, size=K, dtype=np.int8)
        out[f"uA{i}"], out[f"uv{i}"] = A, v
        out[f"u8mat_i32_{i}"] = ref.mvm(A, v, 0, N, K, None, yin, DT_I32, wdt=DT_U8_Q)
    save("mvm", out)


def tie_table(rng, n):
    """Inputs whose product with the scale lands on or next to .5 so that the rounding mode shows."""
    k = rng.integers(-126, 127, size=n).astype(np.float32)
    eps = rng.choice(np.array([0.0, 2.0 ** -17, -2.0 ** -17], np.float32), size=n)
    x = (k + np.float32(0.5) + eps).astype(np.float32)
    x[0] = 127.0                    # abs-max = 127 -> dynamic scale exactly 1
    return x


def gen_quantize(ref, orc):
    rng = np.random.default_rng(SEED + 3)
    out = {}
    ns = [1, 15, 16, 17, 63, 64, 65, 100, 1000, 4099]
    out["ns"] = np.array(ns, np.int64)
    for i, n in enumerate(ns):
        x = rng.standard_normal(n).astype(np.float32) * np.float32(3.0)
        out[f"x{i}"] = x
        for nm, qdt in (("u8", DT_U8_Q), ("i8", DT_I8)):
            q, s = ref.quantize(x, DT_F32, qdt, [-1.0])
            out[f"{nm}_dyn_{i}"], out[f"{nm}_dyn_s{i}"] = q, s
            q, s = ref.quantize(x, DT_F32, qdt, [20.0], mode=1)
            out[f"{nm}_static_{i}"], out[f"{nm}_static_s{i}"] = q, s
            q, s = ref.quantize(x, DT_F32, qdt, [1000.0], mode=0)     # caller's scale larger than 127/max
            out[f"{nm}_floor_{i}"], out[f"{nm}_floor_s{i}"] = q, s
        acc = rng.integers(-200000, 200000, size=n, dtype=np.int32)
        out[f"acc{i}"] = acc
        for nm, qdt in (("u8", DT_U8_Q), ("i8", DT_I8)):
            q, s = ref.quantize(acc, DT_I32, qdt, [-1.0, 37.5])
            out[f"{nm}_i32dyn_{i}"], out[f"{nm}_i32dyn_s{i}"] = q, s
            q, s = ref.quantize(acc, DT_I32, qdt, [0.02, 37.5])
            out[f"{nm}_i32static_{i}"], out[f"{nm}_i32static_s{i}"] = q, s
        u = rng.integers(0, 256, size=n, dtype=np.uint8)
        out[f"u{i}"] = u
        out[f"u_to_i8_{i}"] = ref.quantize(u, DT_U8_Q, DT_I8, [1.0], check_overrun=False)[0]
        out[f"deq_i32_{i}"] = ref.dequantize(acc, DT_I32, 37.5)
        out[f"deq_u8_{i}"] = ref.dequantize(u, DT_U8_Q, 11.25)
        b = (rng.standard_normal(n) * 0.3).astype(np.float32)
        o = rng.integers(-50000, 50000, size=n, dtype=np.int32)
        out[f"b{i}"], out[f"o{i}"] = b, o
        out[f"bias_offsetC_{i}"] = ref.bias_offsetC(b, o, 123.456)
        out[f"bias_only_{i}"] = ref.bias_offsetC(b, None, 123.456)
        r = rng.integers(-128, 128, size=n, dtype=np.int8)
        out[f"r{i}"] = r
        out[f"requant_{i}"] = ref.requantize(r, 10.0, 7.3)
    t = tie_table(rng, 512)
    out["ties"] = t
    for nm, qdt in (("u8", DT_U8_Q), ("i8", DT_I8)):
        q, s = ref.quantize(t, DT_F32, qdt, [-1.0])
        out[f"ties_{nm}"], out[f"ties_{nm}_s"] = q, s
    b = (rng.integers(-2000, 2000, size=256).astype(np.float32) + np.float32(0.5)) / np.float32(8.0)
    out["bias_ties"] = b
    out["bias_ties_out"] = ref.bias_offsetC(b, None, 8.0)
    save("quantize", out)


def gen_conv(ref, orc):
    co = ConvOracle(orc)
    out = {}
    cases = [(2, 16, 6, 6, 32, 3, 3, 1, 1), (1, 64, 9, 7, 64, 3, 3, 1, 1), (1, 32, 8, 8, 48, 3, 3, 2, 1),
             (1, 16, 7, 7, 40, 3, 3, 1, 0), (1, 24, 6, 5, 24, 5, 5, 1, 2), (1, 8, 6, 6, 8, 3, 3, 1, 1),
             (1, 64, 14, 14, 64, 3, 3, 1, 1)]
    out["cases"] = np.array(cases, np.int64)
    for i, case in enumerate(cases):
        n, ic, ih, iw, oc, fh, fw, stride, pad = case
        rng = np.random.default_rng(SEED + 40 + i)
        x = np.maximum(rng.standard_normal((n, ic, ih, iw)), 0).astype(np.float32)
        xq, s = ref.quantize(to_nchwc(x, 8), DT_F32, DT_U8_Q, [-1.0])
        sI = s[0]
        W = rng.integers(-127, 128, size=(oc, ic, fh, fw), dtype=np.int8)
        bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
        sF = np.float32(80.0)
        out[f"xq{i}"], out[f"sI{i}"], out[f"W{i}"], out[f"bias{i}"], out[f"sF{i}"] = xq.reshape(-1), sI, W, bias, sF
        for relu in (0, 1):
            for nm, odt in (("u8", DT_U8_Q), ("f32", DT_F32)):
                d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, bool(relu), odt)
                got, gs = ref_conv(ref, d, xq.reshape(-1), DF_NCHWC8, W, bias, [sI, -1.0, sF])
                out[f"{nm}_relu{relu}_{i}"], out[f"{nm}_relu{relu}_scale{i}"] = got, gs
    save("conv_int8", out)


def gen_pool(ref):
    """u8 pooling (pooling_uint8) and s8 concatenation (concat_cpu) as the reference computes them."""
    from test_oracle_pool import CONCAT_CASES, POOL_CASES, concat_inputs, concat_layout, pool_input
    out = {"pool_cases": np.array(POOL_CASES, np.int64)}
    for i, case in enumerate(POOL_CASES):
        d = pool_desc(case)
        x = pool_input(case, SEED + 60 + i, relu=(i % 3 != 2))
        y, s = ref_pooling(ref, d, x, 12.75)
        out[f"pool_x{i}"], out[f"pool_y{i}"], out[f"pool_s{i}"] = x, y, np.float32(s)
    out["concat_n"] = np.array(len(CONCAT_CASES), np.int64)
    for i, case in enumerate(CONCAT_CASES):
        df, axis, dims, scales = case
        parts = concat_inputs(case, SEED + 80 + i)
        _, _, odims = concat_layout(case)
        y, s = ref_concat(ref, parts, dims, df, axis, scales, odims)
        out[f"cat_meta{i}"] = np.array([df, axis], np.int64)
        out[f"cat_dims{i}"] = np.array(dims, np.int64)
        out[f"cat_scales{i}"] = np.array(scales, np.float32)
        for j, part in enumerate(parts):
            out[f"cat_in{i}_{j}"] = part
        out[f"cat_y{i}"], out[f"cat_s{i}"] = y, np.float32(s)
    save("pool_concat", out)


def gen_encoder_fp32():
    """fp32 neighbours of the int8 GEMMs in an encoder layer as the reference's x86 kernels compute them:
    layer_norm_fp32, softmax_fp32 and the GELU of activation_fp32."""
    from checkers_tensor import RefTensor
    from test_oracle_encoder import gelu_inputs, ln_inputs, softmax_inputs
    r = RefTensor()
    x, g, b = ln_inputs()
    gx = gelu_inputs()
    s = softmax_inputs()
    small = s[:32, :64] / np.float32(4.0)
    save("encoder_fp32", {"ln_x": x, "ln_g": g, "ln_b": b, "ln_y": r.layer_norm(x, g, b), "gelu_x": gx,
                          "gelu_y": r.gelu(gx), "softmax_x": s, "softmax_y": r.softmax(s),
                          "softmax_small_y": r.softmax(small)})


def gen_orchestration(orc):
    """The reference's Tensor-level callers: fully_connected(), matmul() and the convolution's query functions."""
    from checkers_tensor import RefTensor
    from test_oracle_orchestration import CONV_QUERY_CASES, FC_CASES, MATMUL_CASES, fc_inputs, matmul_inputs
    r = RefTensor()
    out = {}
    for i, case in enumerate(FC_CASES):
        M, K, N, odt, scaleO, mvm, with_bias = case
        x, sI, W, sW, bias = fc_inputs(case, SEED + 100 + i)
        y, so, tb = r.fully_connected(x, sI, W, sW, bias if with_bias else None, odt, scaleO, mvm=bool(mvm))
        out[f"fc_y{i}"], out[f"fc_scale{i}"], out[f"fc_tmp{i}"] = y, np.float32(so), np.int64(tb)
    for i, case in enumerate(MATMUL_CASES):
        a_shape, tA, b_shape, tB = case
        A, B, c_shape = matmul_inputs(case, SEED + 200 + i)
        y, tb = r.matmul(A, DT_F32, tA, -1.0, B, DT_F32, tB, -1.0, c_shape)
        out[f"mm_y{i}"], out[f"mm_tmp{i}"] = y, np.int64(tb)
    rows = []
    for case in CONV_QUERY_CASES:
        q = r.conv_queries(*case)
        rows.append(list(q["out"]) + [q["alg"], q["filter_bytes"]] + list(q["ftm"]) + [q["tmp_bytes"]])
    out["conv_queries"] = np.array(rows, np.int64)
    from test_oracle_vs_ref import AXPBY_NS, axpby_inputs
    ref = Ref(threads=1)
    for n in AXPBY_NS:
        a, x, b, y = axpby_inputs(n)
        out[f"axpby_{n}"] = ref.axpby(a, x, b, y)
    save("orchestration", out)


if __name__ == "__main__":
    if not Ref.available():
        sys.exit("oracle/_ref/libboltref.so is missing or this host has no avx512_vnni")
    ref, orc = Ref(threads=1), Oracle()
    only = set(sys.argv[1:])   # e.g. `make_golden.py encoder_fp32 orchestration` rewrites just those files

    def want(name):
        return not only or name in only
    if want("sizes"):
        gen_sizes(ref)
    if want("mmm"):
        gen_mmm(ref, orc)
    if want("mvm"):
        gen_mvm(ref, orc)
    if want("quantize"):
        gen_quantize(ref, orc)
    if want("conv_int8"):
        gen_conv(ref, orc)
    if want("pool_concat"):
        gen_pool(ref)
    if want("encoder_fp32"):
        gen_encoder_fp32()
    if want("orchestration"):
        gen_orchestration(orc)
