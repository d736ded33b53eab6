"""Pins the convolution oracles.

int8 convolution: bit for bit against the reference's own compiled x86 path (oracle/_ref) for u8 and
fp32 outputs, with / without ReLU, several kernel sizes, strides, paddings and channel counts that
exercise the 48 / 32 / 16 / 8 output-channel blocks and the NCHWC8 -> NCHWC16 padding transform.

1-bit convolution: the reference path is ARM fp16 only, so the bit-level oracle is pinned against a
brute-force convolution of the +-1 / {0,1} VALUES (different data path: floats in plain NCHW, no
bit packing), plus the closed forms for all-ones inputs."""
import numpy as np
import pytest

from checkers import DT_F32, DT_I32, DT_U8_Q
from checkers_conv import (DF_NCHWC8, ConvOracle, bnn_pack_filter_nchwn16c8, from_conv_layout, ref_conv, to_nchwc)


@pytest.fixture(scope="module")
def co(oracle):
    return ConvOracle(oracle)


def make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, seed):
    rng = np.random.default_rng(seed)
    x = np.maximum(rng.standard_normal((n, ic, ih, iw)), 0).astype(np.float32)
    xq, sI = oracle.quantize_f32(to_nchwc(x, 8), DT_U8_Q)
    W = rng.integers(-127, 128, size=(oc, ic, fh, fw), dtype=np.int8)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    sF = np.float32(1.0) / np.float32(0.0125)
    return xq, sI, W, sF, bias


CASES = [  # n, ic, ih, iw, oc, fh, fw, stride, pad
    (2, 16, 6, 6, 32, 3, 3, 1, 1),
    (1, 16, 5, 5, 16, 3, 3, 1, 1),
    (1, 64, 9, 7, 64, 3, 3, 1, 1),
    (1, 32, 8, 8, 48, 3, 3, 2, 1),
    (1, 16, 7, 7, 40, 3, 3, 1, 0),
    # ic % 16 != 0 is pinned on one image only: the reference rounds `ic` up to 16 INSIDE its batch loop
    # (convolution_direct.cpp:2737) and then addresses image n at n * ic_rounded * ih * iw, so every
    # image after the first is read from the wrong place.
    (1, 24, 6, 5, 24, 5, 5, 1, 2),
    (1, 8, 6, 6, 8, 3, 3, 1, 1),
]


@pytest.mark.parametrize("case", CASES)
@pytest.mark.parametrize("relu", [False, True])
def test_conv_int8_oracle_vs_reference(oracle, co, ref, case, relu):
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
    for odt in (DT_U8_Q, DT_F32):
        d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, odt)
        got, gs = ref_conv(ref, d, xq, DF_NCHWC8, W, bias, [sI, -1.0, sF])
        want, ws = co.conv(d, xq, W, bias, [sI, -1.0, sF])
        assert np.array_equal(gs, ws), (odt, gs, ws)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (case, odt)


def test_conv_int8_eltwise_fp32(oracle, co, ref):
    n, ic, ih, iw, oc, fh, fw, stride, pad = 1, 16, 6, 6, 32, 3, 3, 1, 1
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 5)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_F32)
    elt = np.random.default_rng(1).standard_normal(n * oc * d.oh * d.ow).astype(np.float32)
    got, _ = ref_conv(ref, d, xq, DF_NCHWC8, W, bias, [sI, -1.0, sF], eltwise=elt)
    want, _ = co.conv(d, xq, W, bias, [sI, -1.0, sF], eltwise=elt)
    assert np.array_equal(got.view(np.int32), want.view(np.int32))


def test_conv_int8_closed_form(oracle, co):
    """Independent of the reference: numpy einsum on the signed values with zero padding."""
    n, ic, ih, iw, oc, fh, fw = 2, 16, 6, 7, 24, 3, 3
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 77)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, 1, 1, False, DT_I32, out_c=8)
    got, _ = co.conv(d, xq, W, bias, [sI, -1.0, sF])
    xs = xq.reshape(n, ic // 8, ih, iw, 8).transpose(0, 1, 4, 2, 3).reshape(n, ic, ih, iw).astype(np.int64) - 128
    xp = np.pad(xs, ((0, 0), (0, 0), (1, 1), (1, 1)))
    acc = np.zeros((n, oc, ih, iw), np.int64)
    for kh in range(3):
        for kw in range(3):
            acc += np.einsum("nchw,oc->nohw", xp[:, :, kh:kh + ih, kw:kw + iw], W[:, :, kh, kw].astype(np.int64))
    b = np.where(bias * (sI * sF) >= 0, np.floor(bias * (sI * sF) + np.float32(0.5)),
                 np.ceil(bias * (sI * sF) - np.float32(0.5))).astype(np.int64)
    acc += b[None, :, None, None]
    assert np.array_equal(from_conv_layout(got, n, oc, ih, iw, 8), acc.astype(np.int32))


@pytest.mark.parametrize("case", CASES[:5])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_perchannel_oracle_reduces_to_the_reference(oracle, co, ref, case, relu):
    """The per-output-channel composition (ConvOracle.conv_perchannel) with every channel scale equal and no bias is the
    reference's own fp32 epilogue (convolution_direct.cpp:2406-2422), bit for bit against the compiled reference; with
    eltwise too. A scale applied as a multiplication instead of a reciprocal, a ReLU before the eltwise sum or a
    transposed output layout fails here."""
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
    zero = np.zeros(oc, np.float32)
    for out_c in (16, 8):
        d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, DT_F32, out_c)
        elt = np.random.default_rng(3).standard_normal(n * oc * d.oh * d.ow).astype(np.float32)
        for e in (None, elt):
            want, _ = (ref_conv(ref, d, xq, DF_NCHWC8, W, zero, [sI, -1.0, sF], eltwise=e) if out_c == 16
                       else co.conv(d, xq, W, zero, [sI, -1.0, sF], eltwise=e))
            got, _ = co.conv_perchannel(oracle, d, xq, W, np.full(oc, sF, np.float32), None, sI, eltwise=e)
            assert np.array_equal(got.view(np.int32), want.view(np.int32)), (case, out_c, e is not None)
            got0, _ = co.conv_perchannel(oracle, d, xq, W, np.full(oc, sF, np.float32), zero, sI, eltwise=e)
            assert np.array_equal(got0.view(np.int32), want.view(np.int32))    # an all-zero bias changes nothing


def test_conv_perchannel_oracle_closed_forms(oracle, co):
    """What the reference cannot pin: (1) with an input that is all zero point the accumulators vanish and the result
    is the bias of each channel, in the output layout; (2) a channel's scale touches that channel only, and doubling it
    halves its values exactly; (3) the u8 form is the pinned quantiser applied to the fp32 form, with the maximum taken
    over the whole tensor (dynamic) or not at all (static)."""
    n, ic, ih, iw, oc, fh, fw = 2, 16, 6, 5, 24, 3, 3
    rng = np.random.default_rng(11)
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 11)
    sw = rng.uniform(40.0, 160.0, oc).astype(np.float32)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, 1, 1, False, DT_F32, 16)
    flat, _ = co.conv_perchannel(oracle, d, np.full_like(xq, 128), W, sw, bias, sI)
    assert np.array_equal(from_conv_layout(flat, n, oc, d.oh, d.ow, 16), np.broadcast_to(bias[None, :, None, None], (n, oc, d.oh, d.ow)))
    base, _ = co.conv_perchannel(oracle, d, xq, W, sw, None, sI)
    sw2 = sw.copy()
    sw2[5] *= 2
    dbl, _ = co.conv_perchannel(oracle, d, xq, W, sw2, None, sI)
    b4, d4 = from_conv_layout(base, n, oc, d.oh, d.ow, 16), from_conv_layout(dbl, n, oc, d.oh, d.ow, 16)
    assert np.array_equal(np.delete(b4, 5, axis=1), np.delete(d4, 5, axis=1))
    assert np.array_equal(d4[:, 5] * 2, b4[:, 5]) and np.any(b4[:, 5] != 0)
    du = co.desc(n, ic, ih, iw, oc, fh, fw, 1, 1, True, DT_U8_Q, 16)
    df = co.desc(n, ic, ih, iw, oc, fh, fw, 1, 1, True, DT_F32, 16)
    f32, _ = co.conv_perchannel(oracle, df, xq, W, sw, bias, sI)
    q, s = co.conv_perchannel(oracle, du, xq, W, sw, bias, sI)
    assert s == np.float32(127.0) / np.abs(f32).max()
    assert np.array_equal(q, np.clip(np.rint(f32 * s + np.float32(128.0)), 1, 255).astype(np.uint8))
    q2, s2 = co.conv_perchannel(oracle, du, xq, W, sw, bias, sI, out_scale=3.5)
    assert s2 == np.float32(3.5)
    assert np.array_equal(q2, np.clip(np.rint(f32 * np.float32(3.5) + np.float32(128.0)), 1, 255).astype(np.uint8))


@pytest.mark.parametrize("xnor", [True, False])
@pytest.mark.parametrize("shape", [(1, 32, 4, 4, 32, 3, 3, 1, 1), (2, 64, 5, 6, 32, 1, 1, 1, 0),
                                   (1, 32, 7, 7, 64, 3, 3, 2, 1)])
def test_bnn_oracle_vs_bruteforce(co, xnor, shape):
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    rng = np.random.default_rng(sum(shape) + xnor)
    if xnor:
        x = np.sign(rng.standard_normal((n, ic, ih, iw))).astype(np.float32)
        x[x == 0] = 1
        w = np.where(rng.random((oc, ic, fh, fw)) < 0.5, -1.0, 1.0).astype(np.float32)
    else:
        x = rng.random((n, ic, ih, iw)).astype(np.float32)
        w = (rng.random((oc, ic, fh, fw)) < 0.5).astype(np.float32)
    d = co.bnn_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, xnor)
    bits = co.bnn_pack_input(d, to_nchwc(x, 8))
    wb = bnn_pack_filter_nchwn16c8(w, xnor)
    scale = rng.uniform(0.5, 1.5, oc).astype(np.float32)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    sums, out = co.bnn_conv(d, bits, wb, scale, bias)
    brute = co.bnn_bruteforce(d, x, w)
    sums_nchw = sums.reshape(n, oc // 8, d.oh, d.ow, 8).transpose(0, 1, 4, 2, 3).reshape(n, oc, d.oh, d.ow)
    assert np.array_equal(sums_nchw, brute)
    want = (sums.astype(np.float64).reshape(n, oc // 8, d.oh, d.ow, 8) * scale.reshape(oc // 8, 1, 1, 8).astype(np.float64)
            + bias.reshape(oc // 8, 1, 1, 8)).astype(np.float32)      # fma = one rounding of the exact value
    assert np.array_equal(out.reshape(want.shape).view(np.int32), want.view(np.int32))


def test_bnn_closed_forms(co):
    n, ic, ih, iw, oc = 1, 32, 5, 5, 32
    d = co.bnn_desc(n, ic, ih, iw, oc, 3, 3, 1, 1, True)
    x = np.ones((n, ic, ih, iw), np.float32)
    w = np.ones((oc, ic, 3, 3), np.float32)
    sums, _ = co.bnn_conv(d, co.bnn_pack_input(d, to_nchwc(x, 8)), bnn_pack_filter_nchwn16c8(w), np.ones(oc, np.float32),
                          np.zeros(oc, np.float32))
    s = sums.reshape(n, oc // 8, 5, 5, 8)
    assert (s[:, :, 1:4, 1:4] == 9 * ic).all()            # interior: every tap +1 * +1
    assert (s[:, :, 0, 0] == (4 - 5) * ic).all()          # corner: 4 taps inside, 5 padded taps count -1
    assert (s[:, :, 0, 1:4] == (6 - 3) * ic).all()        # edge
    d0 = co.bnn_desc(n, ic, ih, iw, oc, 3, 3, 1, 1, False)
    sums0, _ = co.bnn_conv(d0, co.bnn_pack_input(d0, to_nchwc(x, 8)), bnn_pack_filter_nchwn16c8(w, False),
                           np.ones(oc, np.float32), np.zeros(oc, np.float32))
    s0 = sums0.reshape(n, oc // 8, 5, 5, 8)
    assert (s0[:, :, 1:4, 1:4] == 9 * ic).all() and (s0[:, :, 0, 0] == 4 * ic).all()   # DoReFa pads with 0
