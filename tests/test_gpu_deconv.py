"""GPU parity of the int8 deconvolution against the CPU oracle (itself pinned bit for bit against the reference's
compiled deconvolution in test_oracle_deconv.py): both routes (plain NCHW input -> IM2COL_GEMM, NCHWC16 -> POINTWISE),
kernel == stride and overlapping taps, u8 (dynamic, and static on the GEMM route) and fp32 outputs, ReLU on / off,
host- and device-pointer modes. Outputs and the scale array the call leaves behind are compared bit for bit. The
query functions are compared with what the reference answers (golden values recorded from its compiled form)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_deconv  # noqa: E402
from bolt_amd.capi import DF_NCHW, DF_NCHWC16, DT_F32, DT_U8_Q  # noqa: E402
from checkers_deconv import DeconvOracle, deconv_desc, idf_of, lay_input, make_deconv_case  # noqa: E402
from test_oracle_deconv import CASES  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.fixture(scope="module")
def do(oracle):
    return DeconvOracle(oracle)


def run_deconv(torch, device_mode, d, xin, W, bias, scale):
    def put(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda() if device_mode else np.ascontiguousarray(a)
    p = host_deconv.deconv_param_spec(d.oc, d.fh, d.fw, d.sh, d.sw, d.pt, d.pb, d.pl, d.pr)
    x = put(xin)
    idesc, fdesc, odesc, alg = host_deconv.plan(x, idf_of(d.in_c), d.n, d.ic, d.ih, d.iw, d.oc, d.fh, d.fw, p, d.odt)
    assert alg == (2 if d.in_c == 0 else 0)
    assert (odesc.dt, odesc.df, odesc.nDims, list(odesc.dims[:4])) == (d.odt, DF_NCHWC16, 4, [d.ow, d.oh, d.oc, d.n])
    blob, ftm, _ = host_deconv.transform_filter(put(W), fdesc, p, alg)
    out = host_deconv.deconvolution(x, idesc, blob, ftm, p, alg, put(bias), scale, d.relu, odesc)
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return out.cpu().numpy()
    return out


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CASES + [(3, 64, 9, 7, 64, 4, 4, 2, 1), (2, 32, 6, 6, 16, 2, 2, 2, 0)])
@pytest.mark.parametrize("in_c", [0, 16])
@pytest.mark.parametrize("relu", [False, True])
def test_deconv_int8(torch_mod, do, device_mode, case, in_c, relu):
    print("deconv", device_mode, case, in_c, relu, flush=True)
    n, ic, ih, iw, oc, fh, fw, stride, pad = case
    x, sI, W, sF, bias = make_deconv_case(n, ic, ih, iw, oc, fh, fw, sum(case[:7]))
    xin = lay_input(x, in_c)
    for odt, s1 in ((DT_U8_Q, -1.0), (DT_F32, -1.0), (DT_U8_Q, 0.37)):
        d = deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, in_c, relu, odt)
        want, ws = do.deconv(d, xin, W, bias, [sI, s1, sF])
        sc = [sI, s1, sF]
        got = run_deconv(torch_mod, device_mode, d, xin, W, bias, sc)
        assert np.array_equal(np.array(sc, np.float32), ws), (odt, s1, sc, ws)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), (case, in_c, odt, s1)


def test_deconv_upsampling_layer(torch_mod, do):
    """A decoder-sized layer (16 x 64 x 28 x 28 -> 64 channels, 4 x 4 kernel, stride 2, pad 1: 56 x 56 output) on the
    device, u8 output: one image against the oracle, the whole batch through properties (every image of a batch of
    identical images equals the single-image result when the scale is static)."""
    torch = torch_mod
    n, ic, ih, iw, oc, fh, fw, stride, pad = 1, 64, 28, 28, 64, 4, 4, 2, 1
    x, sI, W, sF, bias = make_deconv_case(n, ic, ih, iw, oc, fh, fw, 77)
    xin = lay_input(x, 16)
    d = deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, 16, True, DT_U8_Q)
    want, ws = do.deconv(d, xin, W, bias, [sI, -1.0, sF])
    sc = [sI, -1.0, sF]
    got = run_deconv(torch, True, d, xin, W, bias, sc)
    assert np.array_equal(np.array(sc, np.float32), ws)
    assert np.array_equal(got, want)
    nb = 16
    db = deconv_desc(nb, ic, ih, iw, oc, fh, fw, stride, pad, 16, True, DT_U8_Q)
    scb = [sI, -1.0, sF]
    gotb = run_deconv(torch, True, db, np.tile(xin.reshape(1, -1), (nb, 1)).reshape(-1), W, bias, scb)
    assert np.array_equal(np.array(scb, np.float32), ws)       # same maximum, so the same dynamic scale
    assert all(np.array_equal(gotb.reshape(nb, -1)[i], want) for i in range(nb))


def test_deconv_rejects(torch_mod):
    """What the path does not take: NCHWC8 inputs, channel counts off the blocks, depthwise filters."""
    p = host_deconv.deconv_param_spec(16, 3, 3, 2, 2, 1, 1, 1, 1)
    L = capi.lib()
    import ctypes as C
    b = C.c_uint32(0)
    from bolt_amd.capi import DF_NCHWC8, tensor4df, DT_I8, DF_NCHWC2NxC4, AMD_GFX950
    idesc = tensor4df(DT_U8_Q, DF_NCHWC8, 1, 16, 4, 4)
    odesc = tensor4df(DT_U8_Q, DF_NCHWC16, 1, 16, 7, 7)
    ftm = tensor4df(DT_I8, DF_NCHWC2NxC4, 144, 16, 1, 1)
    assert L.deconvolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, 0, C.byref(b), AMD_GFX950) == capi.NOT_SUPPORTED
    idesc = tensor4df(DT_U8_Q, DF_NCHWC16, 1, 16, 4, 4)
    odesc8 = tensor4df(DT_U8_Q, DF_NCHWC8, 1, 8, 7, 7)
    assert L.deconvolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc8, p, 0, C.byref(b), AMD_GFX950) == capi.NOT_SUPPORTED
    assert L.deconvolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, 8, C.byref(b), AMD_GFX950) == capi.NOT_SUPPORTED
    assert L.deconvolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, 0, C.byref(b), AMD_GFX950) == capi.SUCCESS
