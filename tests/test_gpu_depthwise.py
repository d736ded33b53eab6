"""GPU parity of the int8 depthwise convolution (int32 result, no padding: the one result the reference's kernel
defines) against the CPU oracle, itself pinned against the reference's compiled kernel in test_oracle_depthwise.py.
Host- and device-pointer modes, ReLU on / off, a MobileNet-sized layer; and the argument combinations the reference
computes no defined result for are refused."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_conv  # noqa: E402
from checkers_conv import to_nchwc  # noqa: E402
from test_oracle_depthwise import CASES, make_case, oracle_depthwise  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def run(torch, device_mode, case, xin, W, bias, scale, relu, pad=0):
    n, c, ih, iw, fh, fw, s = case

    def put(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda() if device_mode else np.ascontiguousarray(a)
    blob, ftm = host_conv.depthwise_transform_filter(put(W), c, fh, fw)
    out = host_conv.depthwise_convolution_i32(put(xin), n, c, ih, iw, blob, ftm, fh, fw, s, put(bias), scale, relu, pad)
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return out.cpu().numpy()
    return out


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CASES + [(4, 256, 30, 30, 3, 3, 1)])
@pytest.mark.parametrize("relu", [False, True])
def test_depthwise_int8(torch_mod, oracle, device_mode, case, relu):
    print("depthwise", device_mode, case, relu, flush=True)
    x, sI, W, sF, bias, oh, ow = make_case(case, sum(case))
    xin = to_nchwc(x, 16)
    want, ws = oracle_depthwise(oracle, case, xin, W, bias, [sI, -1.0, sF], relu)
    sc = [sI, -1.0, sF]
    got = run(torch_mod, device_mode, case, xin, W, bias, sc, relu)
    assert np.array_equal(np.array(sc, np.float32), ws)
    assert np.array_equal(got, want)


def test_depthwise_rejects_what_the_reference_leaves_undefined(torch_mod):
    case = CASES[0]
    x, sI, W, sF, bias, oh, ow = make_case(case, 1)
    with pytest.raises(RuntimeError):
        run(torch_mod, False, case, to_nchwc(x, 16), W, bias, [sI, -1.0, sF], False, pad=1)
