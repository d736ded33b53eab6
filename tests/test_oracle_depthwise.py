"""Pins the int8 depthwise restatement (oracle/oracle_deconv.c: orc_depthwise_int8_i32) bit for bit against the
reference's compiled kernel (oracle/_ref), for the one result that kernel defines -- int32, no padding -- and shows,
against the same compiled code, why the other results are not targets: its fp32 output is not the dequantised sum.
Also holds the gfx950 library's transformed filter (host pointers, no GPU work) byte for byte against the reference's."""
import ctypes as C

import numpy as np
import pytest

from checkers import DT_F32, DT_I32, _p, u32, vp
from checkers_conv import to_nchwc

CASES = [  # n, c, ih, iw, fh, fw, stride
    (1, 16, 6, 6, 3, 3, 1),
    (2, 32, 7, 5, 3, 3, 2),
    (1, 48, 9, 9, 5, 5, 1),
    (1, 16, 5, 8, 2, 3, 1),
    (3, 16, 4, 4, 1, 1, 1),
    (1, 64, 12, 10, 3, 3, 3),
]


def make_case(case, seed):
    n, c, ih, iw, fh, fw, s = case
    rng = np.random.default_rng(seed)
    x = rng.integers(1, 256, size=(n, c, ih, iw), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(c, fh, fw), dtype=np.int8)
    bias = (rng.standard_normal(c) * 0.5).astype(np.float32)
    return x, np.float32(17.25), W, np.float32(33.5), bias, (ih - fh) // s + 1, (iw - fw) // s + 1


def oracle_depthwise(oracle, case, xin, W, bias, scale, relu):
    n, c, ih, iw, fh, fw, s = case
    oh, ow = (ih - fh) // s + 1, (iw - fw) // s + 1
    out = np.zeros(n * c * oh * ow, np.int32)
    sc = np.array(scale, np.float32)
    oracle.lib.orc_depthwise_int8_i32.argtypes = [C.c_uint32] * 10 + [vp, vp, vp, vp, C.c_int, vp]
    oracle.lib.orc_depthwise_int8_i32(n, c, ih, iw, fh, fw, s, s, oh, ow, _p(xin), _p(W), _p(bias), _p(sc), int(relu), _p(out))
    return out, sc


def ref_depthwise(ref, case, xin, W, bias, scale, relu, odt):
    n, c, ih, iw, fh, fw, s = case
    oh, ow = (ih - fh) // s + 1, (iw - fw) // s + 1
    out = np.zeros(n * c * oh * ow + 64, np.int32)
    sc = np.array(scale, np.float32)
    rc = ref.lib.ref_depthwise_int8(u32(n), u32(c), u32(ih), u32(iw), u32(fh), u32(fw), u32(s), u32(s), u32(0), u32(0), u32(0),
                                    u32(0), u32(oh), u32(ow), _p(xin), _p(W), _p(bias), _p(sc), int(relu), odt, _p(out))
    assert rc == 0, rc
    return out[:n * c * oh * ow], sc


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("relu", [False, True])
def test_depthwise_oracle_vs_reference(oracle, ref, case, relu):
    x, sI, W, sF, bias, oh, ow = make_case(case, sum(case))
    xin = to_nchwc(x, 16)
    got, gs = ref_depthwise(ref, case, xin, W, bias, [sI, -1.0, sF], relu, DT_I32)
    want, ws = oracle_depthwise(oracle, case, xin, W, bias, [sI, -1.0, sF], relu)
    assert np.array_equal(gs, ws)
    assert np.array_equal(got, want)


def test_depthwise_oracle_closed_form(oracle):
    """numpy sliding windows, independent of the C loops."""
    case = (2, 32, 7, 6, 3, 2, 2)
    n, c, ih, iw, fh, fw, s = case
    x, sI, W, sF, bias, oh, ow = make_case(case, 3)
    got, _ = oracle_depthwise(oracle, case, to_nchwc(x, 16), W, bias, [sI, -1.0, sF], False)
    want = np.zeros((n, c, oh, ow), np.int64)
    for kh in range(fh):
        for kw in range(fw):
            want += (x[:, :, kh:kh + (oh - 1) * s + 1:s, kw:kw + (ow - 1) * s + 1:s].astype(np.int64) - 128) * W[None, :, kh, kw, None, None]
    want += np.round((np.float32(sI * sF) * bias).astype(np.float64))[None, :, None, None].astype(np.int64)
    assert np.array_equal(got.reshape(n, c // 16, oh, ow, 16).transpose(0, 1, 4, 2, 3).reshape(n, c, oh, ow), want)


def test_reference_fp32_output_is_not_the_dequantised_sum(ref, oracle):
    """Why DT_F32 is not a target: the reference's fp32 epilogue multiplies the accumulators' BITS, read as floats,
    by the converted bits of the factor (depthwise_convolution_direct.cpp:148-166)."""
    case = CASES[0]
    x, sI, W, sF, bias, oh, ow = make_case(case, 1)
    xin = to_nchwc(x, 16)
    f, _ = ref_depthwise(ref, case, xin, W, bias, [sI, -1.0, sF], False, DT_F32)
    acc, _ = oracle_depthwise(oracle, case, xin, W, bias, [sI, -1.0, sF], False)
    sane = acc.astype(np.float32) * np.float32(1.0 / (sI * sF))
    with np.errstate(invalid="ignore"):
        assert not np.allclose(f.view(np.float32), sane, rtol=1e-3, atol=1e-3, equal_nan=False)
    factor_bits = np.float32(np.float32(1.0 / np.float32(sI * sF)).view(np.int32))
    with np.errstate(invalid="ignore", over="ignore"):
        model = acc.view(np.float32) * factor_bits
    same = (f.view(np.float32) == model) | (np.isnan(f.view(np.float32)) & np.isnan(model))
    assert same.all()


@pytest.mark.parametrize("case", CASES)
def test_depthwise_filter_blob_equals_reference(ref, case):
    from bolt_amd import host_conv
    n, c, ih, iw, fh, fw, s = case
    _, _, W, _, _, _, _ = make_case(case, 5)
    blob, ftm = host_conv.depthwise_transform_filter(np.ascontiguousarray(W), c, fh, fw)
    size = (fh * fw + 3) // 4 * 4 * c + c * 4
    want = np.zeros(size + 64, np.int8)
    d9 = np.zeros(9, np.uint32)
    assert ref.lib.ref_depthwise_transform_filter(u32(c), u32(fh), u32(fw), _p(W), _p(want), _p(d9)) == 0
    assert len(blob) == size + 32
    assert np.array_equal(np.asarray(blob[:size]).view(np.int8), want[:size])
    assert [ftm.dt, ftm.df, ftm.nDims] + list(ftm.dims[:4]) == list(d9[:7])
