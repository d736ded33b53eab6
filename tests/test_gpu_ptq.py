"""GPU parity of the weight-storage converters of the post-training quantisation tool and of the load-time expansion
of stored weights against the CPU oracle (pinned against the reference's compiled functions in test_oracle_ptq.py):
bit for bit, host- and device-pointer modes, including the returned scale, ties and the caller's scale floor, up to a
BERT FFN weight's size (3072 x 768)."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi  # noqa: E402
from checkers import _p, vp  # noqa: E402
from test_oracle_ptq import bind, weights  # noqa: E402

F = np.float32


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def convert(torch, device_mode, name, w, out_bytes, floor):
    L = capi.lib()
    arch = capi.AMD_GFX950_DEVICE if device_mode else capi.AMD_GFX950
    s = (C.c_float * 1)(float(floor))
    if device_mode:
        dw = torch.from_numpy(w).cuda()
        dq = torch.zeros(out_bytes, dtype=torch.uint8, device="cuda")
        capi.check(getattr(L, name)(dw.data_ptr(), dq.data_ptr(), w.size, s, arch), name)
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        return dq.cpu().numpy(), F(s[0])
    q = np.zeros(out_bytes, np.uint8)
    capi.check(getattr(L, name)(w.ctypes.data, q.ctypes.data, w.size, s, arch), name)
    return q, F(s[0])


def expand(torch, device_mode, name, n, q, out_dtype, scale=None):
    L = capi.lib()
    arch = capi.AMD_GFX950_DEVICE if device_mode else capi.AMD_GFX950
    args = [n] + ([float(scale)] if scale is not None else [])
    if device_mode:
        dq = torch.from_numpy(q).cuda()
        dd = torch.zeros(n, dtype={F: torch.float32, np.int8: torch.int8, np.uint8: torch.uint8}[out_dtype], device="cuda")
        capi.check(getattr(L, name)(*args, dq.data_ptr(), dd.data_ptr(), arch), name)
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        return dd.cpu().numpy()
    d = np.zeros(n, out_dtype)
    capi.check(getattr(L, name)(*args, q.ctypes.data, d.ctypes.data, arch), name)
    return d


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("n", [8, 1000, 4096 * 3 + 8, 3072 * 768])
@pytest.mark.parametrize("ties", [False, True])
def test_ws_converters(torch_mod, oracle, device_mode, n, ties):
    print("ws", device_mode, n, ties, flush=True)
    o = bind(oracle.lib, "orc_")
    w = weights(n, n + int(ties), ties)
    for floor in (-1.0, float(F(127.0 / np.abs(w).max() * 1.003))):
        want, ws = np.zeros(n, np.int8), np.array([floor], F)
        o["ws_convert_int8"](_p(w), n, _p(want), _p(ws))
        got, gs = convert(torch_mod, device_mode, "ws_datatype_converter_int8_gfx950", w, n, floor)
        assert gs == ws[0] and np.array_equal(got.view(np.int8), want)
    want4, ws4 = np.zeros(n // 2, np.int8), np.array([-1.0], F)
    o["ws_convert_int4"](_p(w), n, _p(want4), _p(ws4))
    got4, gs4 = convert(torch_mod, device_mode, "ws_datatype_converter_int4_gfx950", w, n // 2, -1.0)
    assert gs4 == ws4[0] and np.array_equal(got4.view(np.int8), want4)
    sign = np.where(w > 0, F(0.5), F(-0.5)).astype(F)
    for arr in (sign, -np.abs(sign)):
        wantb = np.zeros(n // 8, np.uint8)
        wsb = o["ws_convert_bnn"](_p(arr), n, _p(wantb))
        gotb, gsb = convert(torch_mod, device_mode, "ws_datatype_converter_bnn_gfx950", arr, n // 8, 0.0)
        assert gsb == F(wsb) and np.array_equal(gotb, wantb)


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("n", [16, 1001, 3072 * 768])
def test_load_time_expansion(torch_mod, oracle, device_mode, n):
    print("expand", device_mode, n, flush=True)
    o = bind(oracle.lib, "orc_")
    oracle.lib.orc_dequantize_int4_weight.argtypes = [C.c_int, C.c_float, vp, vp]
    rng = np.random.default_rng(n)
    q = rng.integers(-127, 128, size=n, dtype=np.int8)
    scale = F(37.3)
    want = np.zeros(n, F)
    o["dequantize_int8_weight"](n, scale, _p(q), _p(want))
    got = expand(torch_mod, device_mode, "dequantize_int8_weight_gfx950", n, q, F, scale)
    assert np.array_equal(got.view(np.int32), want.view(np.int32))
    nib = rng.integers(0, 15, size=n + n % 2, dtype=np.uint8)
    packed = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8).view(np.int8)
    want4 = np.zeros(n, F)
    oracle.lib.orc_dequantize_int4_weight(n, scale, _p(packed), _p(want4))
    got4 = expand(torch_mod, device_mode, "dequantize_int4_weight_gfx950", n, packed, F, scale)
    assert np.array_equal(got4.view(np.int32), want4.view(np.int32))
    for name, oname, dt in (("dequantize_int4_int8_gfx950", "dequantize_int4_int8", np.int8),
                            ("dequantize_int4_u8_q_gfx950", "dequantize_int4_u8q", np.uint8)):
        w_ = np.zeros(n, dt)
        o[oname](n, _p(packed), _p(w_))
        assert np.array_equal(expand(torch_mod, device_mode, name, n, packed, dt), w_)


def test_ws_converter_rejects(torch_mod):
    L = capi.lib()
    w = np.zeros(9, F)
    q = np.zeros(9, np.uint8)
    s = (C.c_float * 1)(-1.0)
    assert L.ws_datatype_converter_int4_gfx950(w.ctypes.data, q.ctypes.data, 9, s, capi.AMD_GFX950) == capi.NOT_SUPPORTED
    assert L.ws_datatype_converter_bnn_gfx950(w.ctypes.data, q.ctypes.data, 9, s, capi.AMD_GFX950) == capi.NOT_MATCH
    assert L.ws_datatype_converter_int8_gfx950(None, q.ctypes.data, 9, s, capi.AMD_GFX950) == capi.NULL_POINTER


@pytest.mark.parametrize("device_mode", [False, True])
def test_stored_weights_next_to_the_model_loader(torch_mod, device_mode):
    """A weight as a quantised .bolt model stores it (int8 bytes, or two int4 values per byte, with its one scale), expanded
    by the reference's compiled model loader (TransWeightFromI8ToF32 / I4ToF32 / I4ToI8 / I4ToU8,
    common/model_spec/src/model_deserialize.cpp:270-331) and by this library's load-time expanders, side by side: the same
    bytes. Needs oracle/_ref on the box (built where the reference checkout is present)."""
    from checkers import Ref
    if not Ref.available():
        pytest.skip("oracle/_ref not built or host lacks avx512_vnni")
    ref = Ref(threads=1)
    L = ref.lib.ref_loader_expand_weight
    L.argtypes, L.restype = [C.c_int, vp, C.c_uint, vp, vp], C.c_uint
    n = 3072 * 768
    rng = np.random.default_rng(9)
    q8 = rng.integers(-127, 128, size=n, dtype=np.int8)
    nib = rng.integers(0, 15, size=n, dtype=np.uint8)
    q4 = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8).view(np.int8)
    for kind, stored, out_dt, name, scaled in ((0, q8, F, "dequantize_int8_weight_gfx950", True),
                                               (1, q4, F, "dequantize_int4_weight_gfx950", True),
                                               (2, q4, np.int8, "dequantize_int4_int8_gfx950", False),
                                               (3, q4, np.uint8, "dequantize_int4_u8_q_gfx950", False)):
        sc = np.array([51.75], F)
        want = np.zeros(n, out_dt)
        assert L(kind, _p(stored), stored.nbytes, _p(sc), _p(want)) == want.nbytes
        got = expand(torch_mod, device_mode, name, n, stored, out_dt, F(51.75) if scaled else None)
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), name
