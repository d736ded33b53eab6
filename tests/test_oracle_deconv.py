"""Pins oracle/oracle_deconv.c bit for bit against the reference's own compiled deconvolution (oracle/_ref,
through deconvolution_infer_output_size ... deconvolution() as the engine calls them), for both routes the x86
build takes with quantised input: IM2COL_GEMM for plain NCHW tensors and POINTWISE for NCHWC16 ones, kernel ==
stride and overlapping taps, u8 (dynamic and, on the GEMM route, static scale) and fp32 outputs, with and without
ReLU, symmetric and one-sided padding. Two independent closed forms guard the restatement itself.

Output channel counts are multiples of 16: with 8 output channels the tensor is NCHWC8 but both routes lay the
bias rows out in blocks of 16 (cpu/deconvolution.cpp:313-328, cpu/x86/deconvolution.cpp:143,215-226), write no
bias row at all and add onto whatever tmp held -- not a defined result, so not a target."""
import numpy as np
import pytest

from checkers import DT_F32, DT_U8_Q
from checkers_deconv import (ALG_IM2COL_GEMM, ALG_POINTWISE, DF_NCHWC8, DF_NCHWC16, DeconvOracle, deconv_desc, lay_input,
                             make_deconv_case, plain_output, ref_deconv)


@pytest.fixture(scope="module")
def do(oracle):
    return DeconvOracle(oracle)


CASES = [  # n, ic, ih, iw, oc, fh, fw, stride, pad
    (1, 16, 4, 4, 16, 2, 2, 2, 0),          # kernel == stride
    (2, 32, 5, 3, 32, 2, 2, 2, 0),
    (1, 16, 3, 5, 16, 3, 3, 3, (1, 1, 1, 1)),  # kernel == stride with cropping
    (1, 16, 4, 4, 16, 3, 3, 2, 1),          # overlapping taps
    (2, 32, 5, 3, 48, 4, 4, 2, 1),
    (1, 48, 6, 6, 32, 4, 4, 2, (1, 1, 2, 0)),
    (1, 16, 5, 4, 16, 3, 3, 1, 1),
    (1, 16, 4, 4, 16, 5, 5, 3, 2),
    (1, 16, 3, 4, 32, 4, 2, 2, (1, 1, 0, 0)),  # overlapping in h only
    (1, 16, 3, 4, 16, 3, 2, (3, 1), 0),      # unequal strides
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("in_c", [0, 16])
@pytest.mark.parametrize("relu", [False, True])
def test_deconv_oracle_vs_reference(do, ref, case, in_c, relu):
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    x, sI, W, sF, bias = make_deconv_case(n, ic, ih, iw, oc, fh, fw, sum(case[:7]))
    xin = lay_input(x, in_c)
    for odt, s1 in ((DT_U8_Q, -1.0), (DT_F32, -1.0), (DT_U8_Q, 0.37)):
        d = deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, in_c, relu, odt)
        got, gs, q = ref_deconv(ref, d, xin, W, bias, [sI, s1, sF])
        want, ws = do.deconv(d, xin, W, bias, [sI, s1, sF])
        assert q["alg"] == (ALG_IM2COL_GEMM if in_c == 0 else ALG_POINTWISE)
        assert list(q["out_desc"][:7]) == [odt, DF_NCHWC16 if oc > 8 else DF_NCHWC8, 4, d.ow, d.oh, oc, n]
        assert np.array_equal(gs, ws), (odt, s1, gs, ws)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (case, in_c, odt, s1)


def test_deconv_oracle_integer_sums_closed_form(do):
    """ORC_I32 sums of the gemm form against numpy: out = round(sI*sW*b) + scatter-add of x^T W."""
    from checkers import DT_I32
    n, ic, ih, iw, oc, fh, fw, stride, pad = 2, 16, 4, 5, 16, 3, 4, 2, 1
    x, sI, W, sF, bias = make_deconv_case(n, ic, ih, iw, oc, fh, fw, 5)
    d = deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, 0, False, DT_I32)
    got, _ = do.deconv(d, x, W, bias, [sI, -1.0, sF])
    full = np.zeros((n, oc, fh + stride * (ih - 1), fw + stride * (iw - 1)), np.int64)
    xs = x.astype(np.int64) - 128
    for kh in range(ih):
        for kw in range(iw):
            contrib = np.einsum("nc,cohw->nohw", xs[:, :, kh, kw], W.astype(np.int64))
            full[:, :, kh * stride:kh * stride + fh, kw * stride:kw * stride + fw] += contrib
    want = full[:, :, pad:pad + d.oh, pad:pad + d.ow] + np.round(np.float32(sI * sF) * bias.astype(np.float64))[None, :, None, None].astype(np.int64)
    assert np.array_equal(plain_output(got, d), want.astype(np.int32))


def test_deconv_oracle_identity_filter(do):
    """1x1 kernel, stride 1, identity-like filter (w[c][o] = 64 when c == o): every output pixel is
    64 * (x - 128) + round(sI*sW*b) before the change of type -- places each layout map."""
    n, ic, ih, iw = 1, 16, 3, 2
    rng = np.random.default_rng(9)
    x = rng.integers(1, 256, size=(n, ic, ih, iw), dtype=np.uint8)
    W = np.zeros((ic, ic, 1, 1), np.int8)
    W[np.arange(ic), np.arange(ic), 0, 0] = 64
    bias = np.arange(ic, dtype=np.float32)
    sI, sF = np.float32(2.0), np.float32(4.0)
    for in_c in (0, 16):
        d = deconv_desc(n, ic, ih, iw, ic, 1, 1, 1, 0, in_c, False, DT_F32)
        got, _ = do.deconv(d, lay_input(x, in_c), W, bias, [sI, -1.0, sF])
        acc = 64 * (x.astype(np.int32) - 128)
        if in_c == 0:   # gemm form: the bias is folded as an integer, then one dequantisation
            want = (acc + np.round(8.0 * bias)[None, :, None, None].astype(np.int32)).astype(np.float32) * np.float32(1 / 8.0)
            assert np.array_equal(plain_output(got, d), want)
        else:           # kernel == stride: u8 round trip, so only to within one step of the dynamic scale
            step = np.abs(acc + 8 * bias[None, :, None, None]).max() / 127.0 / 8.0
            assert np.abs(plain_output(got, d) - (acc / 8.0 + bias[None, :, None, None])).max() <= step * 0.5001


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("in_c", [0, 16])
def test_deconv_queries_match_reference(ref, case, in_c):
    """deconvolution_infer_output_size / _infer_forward_algorithm / _transform_filter (desc) of the gfx950 library, on
    host pointers (no GPU work), against what the reference's own functions answer. The blob and tmp sizes are this
    back end's own and must be at least the reference's blob size."""
    import ctypes as C
    from bolt_amd import capi, host_deconv
    from checkers_deconv import idf_of
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    x, sI, W, sF, bias = make_deconv_case(n, ic, ih, iw, oc, fh, fw, 1)
    for odt in (DT_U8_Q, DT_F32):
        d = deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, in_c, False, odt)
        _, _, q = ref_deconv(ref, d, lay_input(x, in_c), W, bias, [sI, -1.0, sF])
        p = host_deconv.deconv_param_spec(oc, fh, fw, d.sh, d.sw, d.pt, d.pb, d.pl, d.pr)
        idesc, fdesc, odesc, alg = host_deconv.plan(np.zeros(1, np.uint8), idf_of(in_c), n, ic, ih, iw, oc, fh, fw, p, odt)
        assert alg == q["alg"]
        assert [odesc.dt, odesc.df, odesc.nDims] + list(odesc.dims[:4]) == list(q["out_desc"][:7])
        blob, ftm, fbytes = host_deconv.transform_filter(np.ascontiguousarray(W), fdesc, p, alg)
        assert [ftm.dt, ftm.df, ftm.nDims] + list(ftm.dims[:ftm.nDims]) == list(q["ftm_desc"][:3 + ftm.nDims])
        assert fbytes >= q["filter_bytes"]
        if ic % 64 == 0:
            assert fbytes == q["filter_bytes"]
        # offsetC sits in front of the packed matrix in both
        off = np.frombuffer(blob[:oc * fh * fw * 4].tobytes(), np.int32).reshape(fh * fw, oc)
        want = -128 * W.astype(np.int64).sum(axis=0).reshape(oc, fh * fw).T
        assert np.array_equal(off, want)
