"""GPU parity of the int8 convolution against the CPU oracle (itself pinned bit for bit against the
reference's compiled x86 path in test_oracle_conv.py). u8 outputs, the returned dynamic output scale,
int32 accumulators and fp32 outputs are compared bit for bit. Includes a single image of BASELINE
configs[2] (64 -> 64 channels, 56 x 56, 3 x 3, stride 1, pad 1, ReLU, u8 out) against the oracle and
the full batch of 32 through size-independent properties."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_conv  # noqa: E402
from bolt_amd.capi import DF_NCHWC8, DF_NCHWC16, DT_F32, DT_I32, DT_U8_Q  # noqa: E402
from checkers_conv import ConvOracle, from_conv_layout, to_nchwc  # noqa: E402
from test_oracle_conv import CASES, make_conv_case  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.fixture(scope="module")
def co(oracle):
    return ConvOracle(oracle)


def run_conv(torch, device_mode, xq, idf, W, bias, scale, case, relu, odt, odf=DF_NCHWC16, eltwise=None):
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    p = capi.conv_param_spec(oc, fh, fw, stride, pad)

    def put(a):
        if a is None:
            return None
        return torch.from_numpy(np.ascontiguousarray(a)).cuda() if device_mode else np.ascontiguousarray(a)
    blob, ftm = host_conv.transform_filter(put(W), oc, ic, fh, fw, p)
    out = host_conv.convolution(put(xq), idf, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, put(bias), scale, relu,
                                odt, odf, put(eltwise))
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return out.cpu().numpy()
    return out


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CASES + [(2, 24, 6, 5, 24, 5, 5, 1, 2), (3, 16, 10, 9, 72, 3, 3, 1, 1)])
@pytest.mark.parametrize("relu", [False, True])
def test_conv_int8(torch_mod, oracle, co, device_mode, case, relu):
    print("conv", device_mode, case, relu, flush=True)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
    for odt in (DT_U8_Q, DT_F32, DT_I32):
        for odf, out_c in ((DF_NCHWC16, 16), (DF_NCHWC8, 8)):
            d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, odt, out_c)
            want, ws = co.conv(d, xq, W, bias, [sI, -1.0, sF])
            sc = [sI, -1.0, sF]
            got = run_conv(torch_mod, device_mode, xq, DF_NCHWC8, W, bias, sc, case, relu, odt, odf)
            assert np.array_equal(np.array(sc, np.float32), ws), (odt, sc, ws)
            assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (case, odt, out_c)


@pytest.mark.parametrize("onepass", [1, 0], ids=["one_pass", "two_pass"])
@pytest.mark.parametrize("panel,direct", [(0, 0), (2, 0), (2, 2), (4, 0), (4, 2)])
def test_conv_int8_every_kernel(torch_mod, oracle, co, panel, direct, onepass):
    """Convolutions with up to 64 output channels and K <= 1024 have three kernels to choose from: the shared
    LDS pipeline (0) and the filter-panel kernel with 32 (2) or 64 (4) pixels per wave; the filter-panel kernel
    either reads the padded s8 image (direct = 0) or, when the channel count is a multiple of 16, gathers from
    the caller's u8 tensor in place (direct = 2: for every result type). Each is forced in turn on shapes with ragged pixel counts,
    channel tails, strides, a 5 x 5 filter, no padding, and a K that is padded up to 64. u8 results through the
    filter-panel kernel come in one pass (the workgroups agree on the tensor-wide maximum with their accumulators in
    registers; default) or two (maximum only, then the stores)."""
    L = capi.lib()
    try:
        capi.check(L.bolt_gfx950_set_option(b"conv_onepass", onepass), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_panel", panel), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_direct", direct), "set_option")
        for case in [(2, 24, 6, 5, 24, 5, 5, 1, 2), (3, 16, 10, 9, 40, 3, 3, 1, 1), (1, 64, 56, 56, 64, 3, 3, 1, 1),
                     (2, 8, 9, 7, 8, 3, 3, 2, 1), (5, 32, 13, 13, 64, 1, 1, 1, 0), (2, 16, 9, 7, 24, 3, 3, 2, 1),
                     (2, 32, 6, 5, 24, 5, 5, 1, 2), (1, 16, 5, 4, 8, 3, 3, 1, 0), (3, 48, 7, 11, 40, 3, 3, 1, 1)]:
            print("conv kernel", panel, direct, case, flush=True)
            n, ic, ih, iw, oc, fh, fw, stride, pad = case
            xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case) + panel)
            for odt in (DT_U8_Q, DT_F32, DT_I32):
                d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, odt, 16)
                want, ws = co.conv(d, xq, W, bias, [sI, -1.0, sF])
                sc = [sI, -1.0, sF]
                got = run_conv(torch_mod, True, xq, DF_NCHWC8, W, bias, sc, case, True, odt, DF_NCHWC16)
                assert np.array_equal(np.array(sc, np.float32), ws), (odt, sc, ws)
                assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (panel, case, odt)
    finally:
        capi.check(L.bolt_gfx950_set_option(b"conv_panel", 4), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_direct", 1), "set_option")
        capi.check(L.bolt_gfx950_set_option(b"conv_onepass", 1), "set_option")


def test_conv_u8_one_pass_falls_back_when_its_wait_gives_up(torch_mod, oracle, co):
    """The one-pass u8 convolution waits a bounded number of polls for all its workgroups. With the bound forced to one
    poll from the host, launches of more than a few workgroups give up: nothing is stored, the kernel publishes a NaN
    scale and exits normally, and the call redoes the convolution in two passes. Same bytes and scale either way."""
    import ctypes as C
    L = capi.lib()
    before = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(before)), "counter")
    cases = [(8, 64, 56, 56, 64, 3, 3, 1, 1), (3, 16, 10, 9, 40, 3, 3, 1, 1), (5, 32, 13, 13, 64, 1, 1, 1, 0)]
    want = {}
    for case in cases:
        n, ic, ih, iw, oc, fh, fw, stride, pad = case
        xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, sum(case))
        d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_U8_Q, 16)
        want[case] = (xq, sI, W, sF, bias) + co.conv(d, xq, W, bias, [sI, -1.0, sF])
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 1), "set_option")
    try:
        for rep in range(3):
            for case in cases:
                print("conv one-pass fallback", rep, case, flush=True)
                xq, sI, W, sF, bias, out, ws = want[case]
                sc = [sI, -1.0, sF]
                got = run_conv(torch_mod, True, xq, DF_NCHWC8, W, bias, sc, case, True, DT_U8_Q, DF_NCHWC16)
                assert np.array_equal(np.array(sc, np.float32), ws) and np.array_equal(got, out), (rep, case)
    finally:
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 0), "set_option")
    after = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(after)), "counter")
    assert after.value > before.value, "no launch gave up: the test did not exercise the fallback"
    for case in cases:      # and with the default bound the one-pass form completes
        xq, sI, W, sF, bias, out, ws = want[case]
        sc = [sI, -1.0, sF]
        got = run_conv(torch_mod, True, xq, DF_NCHWC8, W, bias, sc, case, True, DT_U8_Q, DF_NCHWC16)
        assert np.array_equal(np.array(sc, np.float32), ws) and np.array_equal(got, out), case
    final = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(final)), "counter")
    assert final.value == after.value


@pytest.mark.parametrize("direct", [2, 0])
def test_conv_int8_nchwc16_input_and_eltwise(torch_mod, oracle, co, direct):
    case = (2, 32, 7, 6, 48, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 9)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_F32)
    elt = np.random.default_rng(1).standard_normal(n * oc * d.oh * d.ow).astype(np.float32)
    want, _ = co.conv(d, xq, W, bias, [sI, -1.0, sF], eltwise=elt)
    # same activations handed over as NCHWC16
    x_nchw = xq.reshape(n, ic // 8, ih, iw, 8).transpose(0, 1, 4, 2, 3).reshape(n, ic, ih, iw)
    x16 = to_nchwc(x_nchw, 16)
    L = capi.lib()
    try:
        capi.check(L.bolt_gfx950_set_option(b"conv_direct", direct), "set_option")
        for mode in (False, True):
            got = run_conv(torch_mod, mode, x16, DF_NCHWC16, W, bias, [sI, -1.0, sF], case, True, DT_F32, eltwise=elt)
            assert np.array_equal(got.view(np.int32), want.view(np.int32))
    finally:
        capi.check(L.bolt_gfx950_set_option(b"conv_direct", 1), "set_option")


def test_conv_config3_single_image(torch_mod, oracle, co):
    case = (1, 64, 56, 56, 64, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    xq, sI, W, sF, bias = make_conv_case(oracle, n, ic, ih, iw, oc, fh, fw, 20240603)
    d = co.desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True, DT_U8_Q)
    want, ws = co.conv(d, xq, W, bias, [sI, -1.0, sF])
    sc = [sI, -1.0, sF]
    got = run_conv(torch_mod, True, xq, DF_NCHWC8, W, bias, sc, case, True, DT_U8_Q)
    assert np.array_equal(np.array(sc, np.float32), ws) and np.array_equal(got, want)


def test_conv_config3_full_batch_properties(torch_mod, oracle, co):
    """Batch 32 at the full shape. Image 5 of the batch run must equal the int32 accumulators of the
    same image run alone (batch independence), the u8 tensor must be the requantisation of those
    accumulators with the tensor-wide scale, and its maximum must be 255 (= 127 + 128)."""
    torch = torch_mod
    n, ic, ih, iw, oc = 32, 64, 56, 56, 64
    rng = np.random.default_rng(3)
    x = np.maximum(rng.standard_normal((n, ic, ih, iw)), 0).astype(np.float32)
    xq, sI = oracle.quantize_f32(to_nchwc(x, 8), DT_U8_Q)
    xq = xq.reshape(-1)
    W = rng.integers(-127, 128, size=(oc, ic, 3, 3), dtype=np.int8)
    bias = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    sF = np.float32(80.0)
    case = (n, ic, ih, iw, oc, 3, 3, 1, 1)
    sc = [sI, -1.0, sF]
    u8 = run_conv(torch, True, xq, DF_NCHWC8, W, bias, sc, case, True, DT_U8_Q)
    acc = run_conv(torch, True, xq, DF_NCHWC8, W, bias, [sI, -1.0, sF], case, True, DT_I32)
    one = run_conv(torch, True, xq[5 * ic * ih * iw:6 * ic * ih * iw], DF_NCHWC8, W, bias, [sI, -1.0, sF],
                   (1,) + case[1:], True, DT_I32)
    per = oc * ih * iw
    assert np.array_equal(acc[5 * per:6 * per], one)
    d1 = co.desc(1, ic, ih, iw, oc, 3, 3, 1, 1, True, DT_I32)
    want1, _ = co.conv(d1, xq[5 * ic * ih * iw:6 * ic * ih * iw], W, bias, [sI, -1.0, sF])
    assert np.array_equal(one, want1)
    q, s = oracle.quantize_i32(acc, DT_U8_Q, [-1.0, float(sI * sF)])
    assert np.float32(sc[1]) == s[0] and np.array_equal(u8, q)
    assert u8.max() == 255 and u8.min() == 128      # ReLU: nothing below the zero point
