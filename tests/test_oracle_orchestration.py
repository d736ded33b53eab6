"""Pins the ORCHESTRATION rows -- how FullyConnected and matmul sequence the pinned primitives (tmp layout, scale
plumbing, which BLAS route runs) and what the convolution's query functions answer -- against the reference's own
Tensor-level callers compiled into oracle/_ref (fully_connected(), matmul(), convolution_infer_output_size /
_infer_forward_algorithm / _transform_filter_bytes / _transform_filter / _infer_forward_tmp_bytes; built through
oracle/ref_shim_tensor.cpp), and against the bytes they returned, committed in tests/golden/orchestration.npz.
No GPU: the C-ABI's size and format queries run on the host."""
import ctypes as C
import os

import numpy as np
import pytest

from checkers import DT_F32, DT_I8, DT_I32, DT_U8_Q
from checkers_tensor import RefTensor

GOLD = os.path.join(os.path.dirname(os.path.abspath(__file__)), "golden", "orchestration.npz")

# (M, K, N, output type, output tensor scale before the call, weight packed for the GEMV route, bias)
FC_CASES = [
    (64, 1024, 1024, DT_F32, -1.0, 0, 1),     # BASELINE configs[0]
    (24, 256, 160, DT_U8_Q, -1.0, 0, 1),      # unknown output scale: int32 result, then the dynamic requantisation
    (24, 256, 160, DT_I32, -1.0, 0, 1),
    (5, 77, 100, DT_F32, -1.0, 0, 0),         # ragged, no bias
    (1, 1024, 1024, DT_F32, -1.0, 1, 1),      # M = 1 through matrix_vector_multiply
    (1, 1024, 1024, DT_U8_Q, -1.0, 1, 1),
    (1, 1024, 1024, DT_U8_Q, 0.02, 1, 1),     # known output scale: u8 straight from the kernel
    (1, 77, 100, DT_F32, -1.0, 1, 1),
    (1, 256, 64, DT_F32, -1.0, 0, 1),         # M = 1 but the weight carries the GEMM packing: stays a GEMM
]

MATMUL_CASES = [  # (A shape, transposeA, B shape, transposeB), fp32 operands quantised inside
    ((5, 9), False, (9, 7), False),
    ((2, 3, 16, 64), False, (2, 3, 24, 64), True),
    ((4, 33, 20), True, (4, 33, 17), False),
    ((3, 128, 64), False, (64, 48), False),
    ((12, 128, 64), False, (12, 128, 64), True),
    ((1, 64), False, (64, 48), False),
    ((50, 72), False, (72, 1), False),
    ((72, 50), True, (72, 1), False),
    ((2, 3, 1, 64), False, (2, 3, 64, 128), False),
]

# (n, ic, ih, iw, input format, oc, fh, fw, sh, sw, pt, pb, pl, pr)
CONV_QUERY_CASES = [
    (32, 64, 56, 56, 2, 64, 3, 3, 1, 1, 1, 1, 1, 1),      # BASELINE configs[2]
    (1, 16, 6, 6, 2, 32, 3, 3, 1, 1, 1, 1, 1, 1),
    (1, 8, 4, 4, 2, 8, 1, 1, 1, 1, 0, 0, 0, 0),           # fn == 8 keeps NCHWC8
    (2, 24, 9, 9, 41, 40, 3, 3, 2, 2, 1, 1, 1, 1),        # ic % 16 = 8, oc % 16 = 8
    (1, 64, 14, 14, 2, 48, 5, 5, 1, 1, 2, 2, 2, 2),
    (1, 32, 14, 14, 2, 24, 1, 1, 1, 1, 0, 0, 0, 0),
    (4, 128, 28, 28, 41, 256, 3, 3, 2, 2, 0, 1, 0, 1),    # asymmetric padding
    (1, 72, 7, 7, 2, 16, 7, 7, 1, 1, 3, 3, 3, 3),
    (2, 256, 14, 14, 41, 512, 1, 1, 2, 2, 0, 0, 0, 0),
]


def fc_inputs(case, seed):
    M, K, N = case[:3]
    rng = np.random.default_rng(seed)
    x = rng.integers(1, 256, size=(M, K), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    return x, np.float32(31.0 + seed % 7), W, np.float32(100.0), bias


def matmul_inputs(case, seed):
    a_shape, tA, b_shape, tB = case
    rng = np.random.default_rng(seed)
    A = rng.standard_normal(a_shape).astype(np.float32)
    B = rng.standard_normal(b_shape).astype(np.float32)
    M = a_shape[-1] if tA else a_shape[-2]
    N = b_shape[-2] if tB else b_shape[-1]
    lead = a_shape[:-2] if len(a_shape) >= len(b_shape) else b_shape[:-2]
    return A, B, tuple(lead) + (M, N)


SEED = 20240601


@pytest.fixture(scope="module")
def reft():
    if not RefTensor.available():
        pytest.skip("oracle/_ref/libboltref.so not built or host lacks avx512_vnni")
    return RefTensor()


@pytest.fixture(scope="module")
def gold():
    return np.load(GOLD, allow_pickle=False)


def same(a, b):
    a, b = np.ascontiguousarray(a), np.ascontiguousarray(b)
    return a.size == b.size and a.dtype == b.dtype and a.tobytes() == b.tobytes()


def oracle_fc(oracle, case, i):
    M, K, N, odt, scaleO, mvm, with_bias = case
    x, sI, W, sW, bias = fc_inputs(case, SEED + 100 + i)
    return oracle.fully_connected(x, sI, W, sW, bias if with_bias else None, odt, scaleO)


def oracle_mm(oracle, case, i):
    a_shape, tA, b_shape, tB = case
    A, B, c_shape = matmul_inputs(case, SEED + 200 + i)
    f = oracle.matmul_vector if 1 in c_shape[-2:] else oracle.matmul
    return f(A, tA, B, tB, DT_F32)[0]


@pytest.mark.parametrize("i", range(len(FC_CASES)))
def test_fully_connected_vs_reference(oracle, reft, i):
    case = FC_CASES[i]
    M, K, N, odt, scaleO, mvm, with_bias = case
    x, sI, W, sW, bias = fc_inputs(case, SEED + 100 + i)
    want, ws, _ = reft.fully_connected(x, sI, W, sW, bias if with_bias else None, odt, scaleO, mvm=bool(mvm))
    got, gs = oracle_fc(oracle, case, i)
    assert same(got, want), case
    if odt == DT_U8_Q:
        assert gs == ws, case          # the output tensor's scale after the call (:477-486)
    else:
        assert ws == np.float32(scaleO) and gs == sI * sW   # the reference leaves an fp32 / int32 output's scale alone


@pytest.mark.parametrize("i", range(len(FC_CASES)))
def test_fully_connected_vs_golden(oracle, gold, i):
    got, gs = oracle_fc(oracle, FC_CASES[i], i)
    assert same(got, gold[f"fc_y{i}"]), FC_CASES[i]
    if FC_CASES[i][3] == DT_U8_Q:
        assert gs == gold[f"fc_scale{i}"]


@pytest.mark.parametrize("i", range(len(MATMUL_CASES)))
def test_matmul_vs_reference(oracle, reft, i):
    a_shape, tA, b_shape, tB = MATMUL_CASES[i]
    A, B, c_shape = matmul_inputs(MATMUL_CASES[i], SEED + 200 + i)
    want, _ = reft.matmul(A, DT_F32, tA, -1.0, B, DT_F32, tB, -1.0, c_shape)
    assert same(oracle_mm(oracle, MATMUL_CASES[i], i).reshape(-1), want.reshape(-1)), MATMUL_CASES[i]


@pytest.mark.parametrize("i", range(len(MATMUL_CASES)))
def test_matmul_vs_golden(oracle, gold, i):
    assert same(oracle_mm(oracle, MATMUL_CASES[i], i).reshape(-1), gold[f"mm_y{i}"].reshape(-1)), MATMUL_CASES[i]


def test_matmul_prequantised_operands_vs_reference(oracle, reft):
    """Operands handed over as U8_Q / I8 with their scales skip the quantisation (matmul.cpp:401-421)."""
    for i in (0, 1, 3):
        a_shape, tA, b_shape, tB = MATMUL_CASES[i]
        A, B, c_shape = matmul_inputs(MATMUL_CASES[i], SEED + 200 + i)
        qa, sa = oracle.quantize_f32(A.reshape(-1), DT_U8_Q)
        qb, sb = oracle.quantize_f32(B.reshape(-1), DT_I8)
        want, _ = reft.matmul(qa.reshape(a_shape), DT_U8_Q, tA, sa, qb.reshape(b_shape), DT_I8, tB, sb, c_shape)
        assert same(oracle_mm(oracle, MATMUL_CASES[i], i).reshape(-1), want.reshape(-1))


# ---- the C-ABI's host-side queries against the reference's answers ------------------------------------------------
def conv_query_gfx950(case):
    from bolt_amd import capi
    from bolt_amd.capi import (AMD_GFX950, ActivationParamSpec, ConvolutionParamSpec, TensorDesc, tensor4df)
    L = capi.lib()
    n, ic, ih, iw, idf, oc, fh, fw, sh, sw, pt, pb, pl, pr = case
    p = ConvolutionParamSpec()
    p.num_outputs, p.kernel_t, p.kernel_h, p.kernel_w = oc, 1, fh, fw
    p.stride_t, p.stride_h, p.stride_w = 1, sh, sw
    p.pad_top, p.pad_bottom, p.pad_left, p.pad_right = pt, pb, pl, pr
    p.group, p.dilatedRate_t, p.dilatedRate_h, p.dilatedRate_w = 1, 1, 1, 1
    p.convolution_type = 3
    ind = tensor4df(DT_U8_Q, idf, n, ic, ih, iw)
    fd = tensor4df(DT_I8, 0, oc, ic, fh, fw)
    od = TensorDesc()
    assert L.convolution_infer_output_size_gfx950(ind, fd, p, C.byref(od), DT_U8_Q, AMD_GFX950) == 0
    alg = C.c_int(9)
    act = ActivationParamSpec()
    act.mode = 1
    assert L.convolution_infer_forward_algorithm_gfx950(ind, fd, od, p, 1, C.byref(alg), DT_U8_Q, act, AMD_GFX950) == 0
    fb = C.c_uint32(0)
    assert L.convolution_transform_filter_bytes_gfx950(fd, p, alg.value, C.byref(fb), AMD_GFX950) == 0
    W = np.ones((oc, ic, fh, fw), np.int8)
    blob = np.zeros(fb.value, np.uint8)
    ftm = TensorDesc()
    assert L.convolution_transform_filter_gfx950(fd, W.ctypes.data, p, alg.value, C.byref(ftm), blob.ctypes.data,
                                                 AMD_GFX950) == 0
    tb = C.c_uint32(0)
    assert L.convolution_infer_forward_tmp_bytes_gfx950(ind, ftm, od, p, alg.value, C.byref(tb), AMD_GFX950) == 0

    def desc(d):
        return [d.dt, d.df, d.nDims] + [d.dims[i] if i < d.nDims else 0 for i in range(6)]
    return desc(od), alg.value, fb.value, desc(ftm), tb.value, blob


def check_conv_queries(case, want_out, want_alg, want_fb, want_ftm, want_tb):
    n, ic, ih, iw, idf, oc, fh, fw = case[:8]
    out, alg, fb, ftm, tb, blob = conv_query_gfx950(case)
    assert out == list(want_out), (case, out, want_out)       # type, NCHWC16 / NCHWC8 rule, oh, ow
    assert alg == want_alg, case
    assert ftm == list(want_ftm), (case, ftm, want_ftm)       # DF_NCHWC2NxC4, channels rounded up to 16
    icp = (ic + 15) // 16 * 16
    k = fh * fw * icp
    assert want_fb == oc * icp * fh * fw + oc * 4 + 32
    # this back end's blob pads fn to 16 and K to 64: never smaller than the reference's, equal on aligned shapes
    assert fb == oc * 4 + (oc + 15) // 16 * 16 * ((k + 63) // 64 * 64) + 32
    assert fb >= want_fb and (fb == want_fb) == (oc % 16 == 0 and k % 64 == 0), (case, fb, want_fb)
    # offsetC sits at the head of the blob as in the reference (convolution_transform.cpp:36-44): -128 * taps * 1
    assert np.array_equal(blob[:4 * oc].view(np.int32), np.full(oc, -128 * ic * fh * fw, np.int32))
    # tmp holds the padded s8 image + the folded offsets: the reference's query (which parks the int32 result of a u8
    # convolution there, x86/int8/convolution.cpp:40-93) is never smaller on these shapes
    assert tb <= want_tb + 1024, (case, tb, want_tb)


@pytest.mark.parametrize("i", range(len(CONV_QUERY_CASES)))
def test_conv_queries_vs_reference(reft, i):
    case = CONV_QUERY_CASES[i]
    q = reft.conv_queries(*case)
    check_conv_queries(case, q["out"], q["alg"], q["filter_bytes"], q["ftm"], q["tmp_bytes"])


@pytest.mark.parametrize("i", range(len(CONV_QUERY_CASES)))
def test_conv_queries_vs_golden(gold, i):
    row = [int(v) for v in gold["conv_queries"][i]]
    check_conv_queries(CONV_QUERY_CASES[i], row[0:9], row[9], row[10], row[11:20], row[20])


def test_conv_query_arguments():
    from bolt_amd import capi
    from bolt_amd.capi import AMD_GFX950, ActivationParamSpec, ConvolutionParamSpec, TensorDesc, tensor4df
    L = capi.lib()
    p = ConvolutionParamSpec()
    p.kernel_h = p.kernel_w = 3
    p.stride_h = p.stride_w = 1
    p.group = p.dilatedRate_h = p.dilatedRate_w = 1
    ind, fd = tensor4df(DT_U8_Q, 2, 1, 16, 8, 8), tensor4df(DT_I8, 0, 12, 16, 3, 3)
    od = TensorDesc()
    assert L.convolution_infer_output_size_gfx950(ind, fd, p, None, DT_U8_Q, AMD_GFX950) == capi.NULL_POINTER
    assert L.convolution_infer_output_size_gfx950(ind, fd, p, C.byref(od), DT_U8_Q, AMD_GFX950) == capi.NOT_SUPPORTED  # fn % 8
    assert L.convolution_infer_output_size_gfx950(ind, fd, p, C.byref(od), DT_U8_Q, 0) == capi.NOT_SUPPORTED
    fd = tensor4df(DT_I8, 0, 16, 16, 3, 3)
    p.round_mode = 6   # ROUND_SAME_UPPER
    p.stride_h = p.stride_w = 2
    assert L.convolution_infer_output_size_gfx950(ind, fd, p, C.byref(od), DT_F32, AMD_GFX950) == 0
    assert (od.dt, od.df, od.dims[0], od.dims[1], od.dims[2], od.dims[3]) == (DT_F32, 2, 4, 4, 16, 1)
    alg = C.c_int(5)
    act = ActivationParamSpec()
    assert L.convolution_infer_forward_algorithm_gfx950(ind, fd, od, p, 1, C.byref(alg), DT_U8_Q, act, AMD_GFX950) == 0
    assert alg.value == 5      # an algorithm already chosen is kept
    alg = C.c_int(9)
    assert L.convolution_infer_forward_algorithm_gfx950(ind, fd, od, p, 1, C.byref(alg), DT_F32, act,
                                                        AMD_GFX950) == capi.NOT_SUPPORTED


@pytest.mark.parametrize("i", range(len(FC_CASES)))
def test_fc_tmp_bytes_vs_golden(gold, i):
    """fully_connected_infer_forward_tmp_bytes_gfx950 answers what the reference's query answers."""
    from bolt_amd import capi, host
    from bolt_amd.capi import DF_NKN32K4, DF_NKNxKx
    M, K, N, odt, scaleO, mvm, with_bias = FC_CASES[i]
    got = host.fully_connected_tmp_bytes(M, K, N, DF_NKN32K4 if mvm else DF_NKNxKx, odt)
    assert got == int(gold[f"fc_tmp{i}"]), (FC_CASES[i], got, int(gold[f"fc_tmp{i}"]))
