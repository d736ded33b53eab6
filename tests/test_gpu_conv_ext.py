"""GPU parity of the two convolution forms the reference does not have (bolt_amd/csrc/api_conv_ext.hip):

* per-output-channel filter scales (bolt_gfx950_convolution_int8_perchannel): against ConvOracle.conv_perchannel -- the
  reference-pinned int32 convolution, three fp32 operations, the reference-pinned fp32 -> u8 quantiser -- bit for bit
  (fp32 bytes, u8 bytes, the returned scale), and against convolution_gfx950 itself when every channel scale is equal;
* asynchronous calls with device-resident scales (bolt_gfx950_convolution_async): every byte and the scale left on
  the device against what the synchronous calls return.

Shapes cover both kernels (filter panel with in-place gather / padded image; shared LDS pipeline for more than 64
channels), ragged pixel counts, channel tails, strides, NCHWC8 and NCHWC16 outputs; BASELINE configs[2] (64 -> 64,
56 x 56, 3 x 3, ReLU, u8 out, per-output-channel scales) on one image against the oracle and at batch 32 through
properties."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_conv  # noqa: E402
from bolt_amd.capi import DF_NCHWC8, DF_NCHWC16, DT_F32, DT_I32, DT_U8_Q  # noqa: E402
from checkers_conv import ConvOracle, from_conv_layout, to_nchwc  # noqa: E402
from test_oracle_conv import make_conv_case  # noqa: E402

CASES = [  # n, ic, ih, iw, oc, fh, fw, stride, pad
    (2, 16, 6, 6, 32, 3, 3, 1, 1),
    (3, 16, 10, 9, 40, 3, 3, 1, 1),
    (2, 24, 6, 5, 24, 5, 5, 1, 2),
    (2, 8, 9, 7, 8, 3, 3, 2, 1),
    (5, 32, 13, 13, 64, 1, 1, 1, 0),
    (3, 48, 7, 11, 72, 3, 3, 1, 1),
    (1, 32, 20, 17, 144, 3, 3, 1, 1),
    (1, 64, 56, 56, 64, 3, 3, 1, 1),
]


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.fixture(scope="module")
def co(oracle):
    return ConvOracle(oracle)


def channel_scales(oc, seed):
    return np.random.default_rng(seed).uniform(50.0, 200.0, oc).astype(np.float32)   # 1 / U(0.005, 0.02)


def put(torch, a, device_mode=True):
    if a is None:
        return None
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a).cuda() if device_mode else a


def run_perchannel(torch, device_mode, xq, idf, W, sw, bias, scale, case, relu, odt, odf=DF_NCHWC16, eltwise=None):
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    p = capi.conv_param_spec(oc, fh, fw, stride, pad)
    blob, ftm = host_conv.transform_filter(put(torch, W, device_mode), oc, ic, fh, fw, p)
    out = host_conv.convolution_perchannel(put(torch, xq, device_mode), idf, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad,
                                           put(torch, sw, device_mode), put(torch, bias, device_mode), scale, relu, odt, odf,
                                           put(torch, eltwise, device_mode))
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return out.cpu().numpy()
    return out


@pytest.mark.parametrize("device_mode", [True, False])
@pytest.mark.parametrize("case", CASES[:7])
def test_conv_perchannel_vs_oracle(torch_mod, oracle, co, device_mode, case):
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
    sw = channel_scales(oc, sum(case))
    for relu in (True, False):
        for odf, out_c in ((DF_NCHWC16, 16), (DF_NCHWC8, 8)):
            for b in (bias, None):
                print("conv perchannel", device_mode, case, relu, out_c, b is not None, flush=True)
                d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, DT_F32, out_c)
                want, _ = co.conv_perchannel(oracle, d, xq, W, sw, b, sI)
                sc = [sI, -7.0]
                got = run_perchannel(torch_mod, device_mode, xq, DF_NCHWC8, W, sw, b, sc, case, relu, DT_F32, odf)
                assert np.array_equal(got.view(np.int32), want.view(np.int32)), (case, relu, out_c)
                assert sc[1] == np.float32(-7.0)                     # an fp32 result leaves the output scale alone
                du = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, DT_U8_Q, out_c)
                for so in (-1.0, 3.25):
                    wq, ws = co.conv_perchannel(oracle, du, xq, W, sw, b, sI, out_scale=so)
                    sc = [sI, so]
                    gq = run_perchannel(torch_mod, device_mode, xq, DF_NCHWC8, W, sw, b, sc, case, relu, DT_U8_Q, odf)
                    assert np.float32(sc[1]) == ws, (case, so, sc, ws)
                    assert np.array_equal(gq, wq), (case, relu, out_c, so)


@pytest.mark.parametrize("case", [CASES[0], CASES[1], CASES[5], CASES[6]])
def test_conv_perchannel_equal_scales_is_the_reference_epilogue(torch_mod, oracle, co, case):
    """Every channel scale equal, no bias (or an all-zero one), fp32 result: the bytes of convolution_gfx950, which the
    other tests hold against the reference. With eltwise as well."""
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, _ = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case) + 1)
    zero = np.zeros(oc, np.float32)
    p = capi.conv_param_spec(oc, fh, fw, stride, pad)
    blob, ftm = host_conv.transform_filter(put(torch_mod, W), oc, ic, fh, fw, p)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_F32)
    elt = np.random.default_rng(2).standard_normal(n * oc * d.oh * d.ow).astype(np.float32)
    for e in (None, elt):
        ref = host_conv.convolution(put(torch_mod, xq), DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad,
                                    put(torch_mod, zero), [sI, -1.0, sF], True, DT_F32, DF_NCHWC16, put(torch_mod, e))
        for b in (None, zero):
            got = host_conv.convolution_perchannel(put(torch_mod, xq), DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride,
                                                   pad, put(torch_mod, np.full(oc, sF, np.float32)), put(torch_mod, b),
                                                   [sI, -1.0], True, DT_F32, DF_NCHWC16, put(torch_mod, e))
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            assert torch_mod.equal(got.view(torch_mod.int32), ref.view(torch_mod.int32)), (case, e is not None, b is not None)


def test_conv_perchannel_nchwc16_input_and_eltwise(torch_mod, oracle, co):
    case = (2, 32, 7, 6, 48, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 9)
    sw = channel_scales(oc, 9)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_F32)
    elt = np.random.default_rng(1).standard_normal(n * oc * d.oh * d.ow).astype(np.float32)
    want, _ = co.conv_perchannel(oracle, d, xq, W, sw, bias, sI, eltwise=elt)
    x16 = to_nchwc(xq.reshape(n, ic // 8, ih, iw, 8).transpose(0, 1, 4, 2, 3).reshape(n, ic, ih, iw), 16)
    for mode in (False, True):
        got = run_perchannel(torch_mod, mode, x16, DF_NCHWC16, W, sw, bias, [sI, -1.0], case, True, DT_F32, eltwise=elt)
        assert np.array_equal(got.view(np.int32), want.view(np.int32))


def test_conv_perchannel_rejects():
    import ctypes as C
    from bolt_amd.capi import ActivationParamSpec, AMD_GFX950, DT_I8, DF_NCHWC2NxC4, tensor1d, tensor4df
    L = capi.lib()
    n, ic, ih, iw, oc = 1, 16, 4, 4, 16
    p = capi.conv_param_spec(oc, 3, 3, 1, 1)
    idesc, odesc = tensor4df(DT_U8_Q, DF_NCHWC8, n, ic, ih, iw), tensor4df(DT_I32, DF_NCHWC16, n, oc, ih, iw)
    fdesc = tensor4df(DT_I8, DF_NCHWC2NxC4, oc, ic, 3, 3)
    buf = np.zeros(1 << 16, np.uint8)
    sw = np.ones(oc, np.float32)
    sc = (C.c_float * 2)(1.0, -1.0)
    act = ActivationParamSpec()
    args = lambda od, swp, s: (idesc, buf.ctypes.data, None, fdesc, buf.ctypes.data, p, swp, tensor1d(DT_F32, oc), None, 1 << 16,
                              buf.ctypes.data, od, buf.ctypes.data, s, act, AMD_GFX950)
    assert L.bolt_gfx950_convolution_int8_perchannel(*args(odesc, sw.ctypes.data, sc)) == capi.NOT_SUPPORTED   # no int32 form
    assert L.bolt_gfx950_convolution_int8_perchannel(*args(tensor4df(DT_F32, DF_NCHWC16, n, oc, ih, iw), None, sc)) == capi.NULL_POINTER
    bad = (C.c_float * 2)(0.0, -1.0)
    assert L.bolt_gfx950_convolution_int8_perchannel(*args(tensor4df(DT_F32, DF_NCHWC16, n, oc, ih, iw), sw.ctypes.data, bad)) == capi.NOT_MATCH


def test_conv_perchannel_config3(torch_mod, oracle, co):
    """BASELINE configs[2] as it is worded: per-output-channel filter scales, fp32 bias, ReLU, u8 result with one
    tensor-wide scale. One image against the oracle; then the batch of 32 through properties: image 5 of the batch
    equals the same image run alone (fp32 form), the u8 tensor is the quantisation of the fp32 tensor with the returned
    scale, that scale is 127 / max, the largest byte is 255 and nothing lies below the zero point."""
    torch = torch_mod
    case = (1, 64, 56, 56, 64, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 20240603)
    sw = channel_scales(oc, 20240603)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_U8_Q)
    want, ws = co.conv_perchannel(oracle, d, xq, W, sw, bias, sI)
    sc = [sI, -1.0]
    got = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, sc, case, True, DT_U8_Q)
    assert np.float32(sc[1]) == ws and np.array_equal(got, want)

    n = 32
    rng = np.random.default_rng(3)
    x = np.maximum(rng.standard_normal((n, ic, ih, iw)), 0).astype(np.float32)
    xq, sI = oracle.quantize_f32(to_nchwc(x, 8), DT_U8_Q)
    xq = xq.reshape(-1)
    case = (n,) + case[1:]
    sc = [sI, -1.0]
    u8 = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, sc, case, True, DT_U8_Q)
    f32 = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, [sI, -1.0], case, True, DT_F32)
    per_in, per_out = ic * ih * iw, oc * ih * iw
    one = run_perchannel(torch, True, xq[5 * per_in:6 * per_in], DF_NCHWC8, W, sw, bias, [sI, -1.0], (1,) + case[1:], True, DT_F32)
    assert np.array_equal(f32[5 * per_out:6 * per_out].view(np.int32), one.view(np.int32))
    d1 = co.desc(1, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_F32)
    want1, _ = co.conv_perchannel(oracle, d1, xq[5 * per_in:6 * per_in], W, sw, bias, sI)
    assert np.array_equal(one.view(np.int32), want1.view(np.int32))
    q, s = oracle.quantize_f32(f32, DT_U8_Q)
    assert np.float32(sc[1]) == s == np.float32(127.0) / f32.max() and np.array_equal(u8, q)
    assert u8.max() == 255 and u8.min() == 128
    # static output scale: one pass, same quantiser
    sc = [sI, 2.5]
    u8s = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, sc, case, True, DT_U8_Q)
    qs, _ = oracle.quantize_f32(f32, DT_U8_Q, 2.5, 1)
    assert np.float32(sc[1]) == np.float32(2.5) and np.array_equal(u8s, qs)


@pytest.mark.parametrize("room", [True, False], ids=["one_pass_room", "two_passes"])
@pytest.mark.parametrize("case", CASES)
def test_conv_async_equals_the_synchronous_calls(torch_mod, oracle, co, case, room):
    """bolt_gfx950_convolution_async with the input scale in device memory: bytes and the scale it leaves on the device
    equal what convolution_gfx950 (one filter scale: u8, fp32, int32) and the per-channel call (fp32, u8 dynamic, u8
    static) return; two calls in a row, the second on other data, so that the alternating maximum slots are used."""
    torch = torch_mod
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    p = capi.conv_param_spec(oc, fh, fw, stride, pad)
    for rep in range(2):
        xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case) + 17 * rep)
        if rep == 1:
            xq = (128 + (xq.astype(np.int32) - 128) // 3).astype(np.uint8)     # smaller maxima than the first call left
        sw = channel_scales(oc, sum(case) + rep)
        blob, ftm = host_conv.transform_filter(put(torch, W), oc, ic, fh, fw, p)
        dx, db, dsw = put(torch, xq), put(torch, bias), put(torch, sw)
        dsi = torch.tensor([float(sI)], dtype=torch.float32, device="cuda")
        for odt in (DT_U8_Q, DT_F32, DT_I32):
            print("conv async per-tensor", case, rep, odt, flush=True)
            sc = [sI, -1.0, sF]
            want = host_conv.convolution(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, db, sc, True, odt)
            dso = torch.tensor([-5.0], dtype=torch.float32, device="cuda")
            got = host_conv.convolution_async(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, db, dsi,
                                              float(sF), None, dso, True, odt, one_pass_room=room)
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (case, rep, odt)
            assert np.float32(dso.item()) == np.float32(sc[1]), (case, odt, dso.item(), sc[1])
        for odt, so in ((DT_F32, 0.0), (DT_U8_Q, 0.0), (DT_U8_Q, 1.75)):
            print("conv async per-channel", case, rep, odt, so, flush=True)
            sc = [sI, so if so > 0 else -1.0]
            want = host_conv.convolution_perchannel(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, dsw, db, sc,
                                                    True, odt)
            dso = torch.tensor([-5.0], dtype=torch.float32, device="cuda")
            got = host_conv.convolution_async(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, db, dsi, 0.0, dsw,
                                              dso, True, odt, static_out=so, one_pass_room=room)
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            assert torch.equal(got.view(torch.uint8), want.view(torch.uint8)), (case, rep, odt, so)
            if odt == DT_U8_Q:
                assert np.float32(dso.item()) == np.float32(sc[1]), (case, so, dso.item(), sc[1])
            else:
                assert dso.item() == -5.0


def test_conv_async_chain_never_touches_the_host(torch_mod, oracle, co):
    """Two quantised convolutions in a row, the second reading its input scale from where the first left its output
    scale, no synchronisation in between: the bytes of the synchronous chain."""
    torch = torch_mod
    n, ic, ih, iw, oc = 4, 32, 14, 14, 32
    p = capi.conv_param_spec(oc, 3, 3, 1, 1)
    xq, sI, W1, sF, b1 = make_conv_case(oracle, n, ic, ih, iw, oc, 3, 3, 41)
    _, _, W2, _, b2 = make_conv_case(oracle, n, oc, ih, iw, oc, 3, 3, 42)
    blob1, ftm1 = host_conv.transform_filter(put(torch, W1), oc, ic, 3, 3, p)
    blob2, ftm2 = host_conv.transform_filter(put(torch, W2), oc, oc, 3, 3, p)
    dx, db1, db2 = put(torch, xq), put(torch, b1), put(torch, b2)
    s1 = [sI, -1.0, sF]
    mid = host_conv.convolution(dx, DF_NCHWC8, n, ic, ih, iw, blob1, ftm1, oc, 3, 3, 1, 1, db1, s1, True, DT_U8_Q)
    s2 = [s1[1], -1.0, sF]
    want = host_conv.convolution(mid, DF_NCHWC16, n, oc, ih, iw, blob2, ftm2, oc, 3, 3, 1, 1, db2, s2, True, DT_U8_Q)
    dsi = torch.tensor([float(sI)], dtype=torch.float32, device="cuda")
    dmid, dout = torch.zeros(1, device="cuda"), torch.zeros(1, device="cuda")
    amid = host_conv.convolution_async(dx, DF_NCHWC8, n, ic, ih, iw, blob1, ftm1, oc, 3, 3, 1, 1, db1, dsi, float(sF), None, dmid,
                                       True, DT_U8_Q)
    got = host_conv.convolution_async(amid, DF_NCHWC16, n, oc, ih, iw, blob2, ftm2, oc, 3, 3, 1, 1, db2, dmid, float(sF), None,
                                      dout, True, DT_U8_Q)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(amid, mid) and torch.equal(got, want)
    assert np.float32(dmid.item()) == np.float32(s1[1]) and np.float32(dout.item()) == np.float32(s2[1])


def test_conv_one_pass_forms_when_their_wait_gives_up(torch_mod, oracle, co):
    """The one-pass u8 forms wait a bounded number of polls for all their workgroups. With the bound forced to one poll
    from the host the launches of more than a few workgroups give up, and every kernel still exits normally:
    the synchronous per-channel call gets a NaN scale and redoes the convolution in two passes (counted); the
    asynchronous calls have no host to fall back on -- their workgroups park their values in tmp and the last one to
    arrive quantises the tensor alone. Same bytes and scales as without the bound, and the maximum slots are left
    clear: a two-pass call right behind still gets its own maximum."""
    import ctypes as C
    torch = torch_mod
    L = capi.lib()
    cases = [(8, 64, 56, 56, 64, 3, 3, 1, 1), (3, 16, 10, 9, 40, 3, 3, 1, 1), (5, 32, 13, 13, 64, 1, 1, 1, 0)]
    want = {}
    for case in cases:
        n, ic, ih, iw, oc, fh, fw, stride, pad = case
        xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
        sw = channel_scales(oc, sum(case))
        d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_U8_Q, 16)
        want[case] = (xq, sI, W, sF, bias, sw, co.conv(d, xq, W, bias, [sI, -1.0, sF]), co.conv_perchannel(oracle, d, xq, W, sw, bias, sI))
    before = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(before)), "counter")

    def run_all(tag):
        for case in cases:
            print("conv one-pass give-up", tag, case, flush=True)
            n, ic, ih, iw, oc, fh, fw, stride, pad = case
            xq, sI, W, sF, bias, sw, (w1, s1), (wc, sc_) = want[case]
            p = capi.conv_param_spec(oc, fh, fw, stride, pad)
            blob, ftm = host_conv.transform_filter(put(torch, W), oc, ic, fh, fw, p)
            dx, db, dsw = put(torch, xq), put(torch, bias), put(torch, sw)
            dsi = torch.tensor([float(sI)], dtype=torch.float32, device="cuda")
            sc = [sI, -1.0]
            got = host_conv.convolution_perchannel(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, dsw, db, sc, True, DT_U8_Q)
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            assert np.float32(sc[1]) == sc_ and np.array_equal(got.cpu().numpy(), wc), (tag, case, "per-channel sync")
            for swp, fs, (wb, wsc) in ((None, float(sF), (w1, s1[1])), (dsw, 0.0, (wc, sc_))):
                for room in (True, False, True):
                    dso = torch.tensor([-5.0], dtype=torch.float32, device="cuda")
                    got = host_conv.convolution_async(dx, DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, db, dsi, fs, swp,
                                                      dso, True, DT_U8_Q, one_pass_room=room)
                    capi.check(L.bolt_gfx950_synchronize(), "sync")
                    assert np.float32(dso.item()) == np.float32(wsc), (tag, case, swp is not None, room, dso.item(), wsc)
                    assert np.array_equal(got.cpu().numpy(), wb), (tag, case, swp is not None, room)
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 1), "set_option")
    try:
        run_all("bound 1")
    finally:
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 0), "set_option")
    after = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(after)), "counter")
    assert after.value > before.value, "no synchronous launch gave up: the test did not exercise the fallback"
    run_all("default bound")
    final = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(final)), "counter")
    assert final.value == after.value


def test_conv_random_shapes_every_form(torch_mod, oracle, co):
    """Twenty seeded random shapes (channels 8-144, filters 1-5, strides, paddings, ragged images) under random kernel
    options, each through every form: the reference's three result types in both output layouts, the per-channel forms
    (fp32, static u8, dynamic u8) and the asynchronous twins with and without room for the one-pass form -- all against
    the CPU checker, bit for bit, scales included."""
    torch = torch_mod
    L = capi.lib()
    rng = np.random.default_rng(20240607)
    try:
        for it in range(20):
            n = int(rng.integers(1, 5))
            ic = int(rng.choice([8, 16, 24, 32, 48, 64]))
            oc = int(rng.choice([8, 16, 24, 32, 40, 48, 64, 72, 96, 144]))
            fh = fw = int(rng.choice([1, 2, 3, 5]))
            stride = int(rng.choice([1, 1, 2]))
            pad = int(rng.integers(0, (fh + 1) // 2 + 1))
            ih = int(rng.integers(max(fh - 2 * pad, 1) + 1, 24))
            iw = int(rng.integers(max(fw - 2 * pad, 1) + 1, 24))
            case = (n, ic, ih, iw, oc, fh, fw, stride, pad)
            relu = bool(rng.random() < 0.6)
            panel, direct, onepass = int(rng.choice([0, 2, 4])), int(rng.choice([0, 1, 2])), int(rng.choice([0, 1]))
            print("conv random", it, case, relu, panel, direct, onepass, flush=True)
            capi.check(L.bolt_gfx950_set_option(b"conv_panel", panel), "set_option")
            capi.check(L.bolt_gfx950_set_option(b"conv_direct", direct), "set_option")
            capi.check(L.bolt_gfx950_set_option(b"conv_onepass", onepass), "set_option")
            xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 977 * it + 5)
            sw = channel_scales(oc, it)
            p = capi.conv_param_spec(oc, fh, fw, stride, pad)
            blob, ftm = host_conv.transform_filter(put(torch, W), oc, ic, fh, fw, p)
            for odf, out_c in ((DF_NCHWC16, 16), (DF_NCHWC8, 8)):
                for odt in (DT_U8_Q, DT_F32, DT_I32):
                    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, odt, out_c)
                    want, ws = co.conv(d, xq, W, bias, [sI, -1.0, sF])
                    sc = [sI, -1.0, sF]
                    got = host_conv.convolution(put(torch, xq), DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad,
                                                put(torch, bias), sc, relu, odt, odf)
                    capi.check(L.bolt_gfx950_synchronize(), "sync")
                    assert np.array_equal(np.array(sc, np.float32), ws), (case, odt, sc, ws)
                    assert np.array_equal(got.cpu().numpy().view(np.uint8), want.view(np.uint8)), (case, odt, out_c)
                d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, DT_F32, out_c)
                want, _ = co.conv_perchannel(oracle, d, xq, W, sw, bias, sI)
                got = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, [sI, -1.0], case, relu, DT_F32, odf)
                assert np.array_equal(got.view(np.int32), want.view(np.int32)), (case, out_c)
                du = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, DT_U8_Q, out_c)
                for so in (-1.0, 2.5):
                    wq, ws = co.conv_perchannel(oracle, du, xq, W, sw, bias, sI, out_scale=so)
                    sc = [sI, so]
                    gq = run_perchannel(torch, True, xq, DF_NCHWC8, W, sw, bias, sc, case, relu, DT_U8_Q, odf)
                    assert np.float32(sc[1]) == ws and np.array_equal(gq, wq), (case, so, out_c)
                    for room in (True, False):
                        dsi = torch.tensor([sI], dtype=torch.float32, device="cuda")
                        dso = torch.zeros(1, dtype=torch.float32, device="cuda")
                        ga = host_conv.convolution_async(put(torch, xq), DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride,
                                                         pad, put(torch, bias), dsi, 0.0, put(torch, sw), dso, relu, DT_U8_Q, odf,
                                                         static_out=(so if so > 0 else 0.0), one_pass_room=room)
                        capi.check(L.bolt_gfx950_synchronize(), "sync")
                        assert np.array_equal(ga.cpu().numpy(), wq) and np.float32(dso.item()) == ws, (case, so, out_c, room)
                want, ws = co.conv(du, xq, W, bias, [sI, -1.0, sF])
                for room in (True, False):
                    dsi = torch.tensor([sI], dtype=torch.float32, device="cuda")
                    dso = torch.zeros(1, dtype=torch.float32, device="cuda")
                    ga = host_conv.convolution_async(put(torch, xq), DF_NCHWC8, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad,
                                                     put(torch, bias), dsi, sF, None, dso, relu, DT_U8_Q, odf, one_pass_room=room)
                    capi.check(L.bolt_gfx950_synchronize(), "sync")
                    assert np.array_equal(ga.cpu().numpy().view(np.uint8), want.view(np.uint8)), (case, out_c, room)
                    assert np.float32(dso.item()) == ws[1], (case, out_c, room)
    finally:
        capi.check(L.bolt_gfx950_set_option(b"conv_panel", 4), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_direct", 1), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_onepass", 1), "set_option")
