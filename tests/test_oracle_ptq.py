"""Pins oracle/oracle_ptq.c (weight-storage quantisation of the post-training quantisation tool and the load-time
expansion of stored weights) bit for bit against the reference's own compiled functions (oracle/_ref), including
ties, the caller's scale floor and the nibble order; plus closed forms that do not go through either."""
import ctypes as C

import numpy as np
import pytest

from checkers import _p, vp

F = np.float32


def bind(lib, prefix):
    f = {}
    for name, args, res in (("ws_convert_int8", [vp, C.c_int, vp, vp], None), ("ws_convert_int4", [vp, C.c_int, vp, vp], None),
                            ("ws_convert_bnn", [vp, C.c_int, vp], C.c_float),
                            ("dequantize_int8_weight", [C.c_int, C.c_float, vp, vp], None),
                            ("dequantize_int4_int8", [C.c_int, vp, vp], None),
                            ("dequantize_int4_u8q", [C.c_int, vp, vp], None)):
        fn = getattr(lib, prefix + name)
        fn.argtypes, fn.restype = args, res
        f[name] = fn
    return f


def weights(n, seed, ties=False):
    rng = np.random.default_rng(seed)
    w = (rng.standard_normal(n) * 0.05).astype(F)
    if ties:   # max|w| = 127 / 4 exactly -> scale 4: products land on k + 0.5
        w = (rng.integers(-508, 509, size=n).astype(F) / F(8.0)).astype(F)
        w[0] = F(31.75)
    return w


@pytest.mark.parametrize("n", [8, 64, 1000, 4096 * 3 + 8])
@pytest.mark.parametrize("ties", [False, True])
@pytest.mark.parametrize("floor", [-1.0, 1.003])
def test_ws_convert_int8_and_int4(oracle, ref, n, ties, floor):
    o, r = bind(oracle.lib, "orc_"), bind(ref.lib, "ref_")
    w = weights(n, n + int(ties), ties)
    if floor > 0:   # a caller's scale a little above 127 / max|w| (7 / max|w|): it wins, and every product still fits
        floor = float(F(127.0 / np.abs(w).max() * floor))
    for name, count in (("ws_convert_int8", n), ("ws_convert_int4", n // 2)):
        qo, qr = np.zeros(n, np.int8), np.zeros(n, np.int8)
        fl = floor if (floor < 0 or name == "ws_convert_int8") else floor * 7.0 / 127.0
        so, sr = np.array([fl], F), np.array([fl], F)
        o[name](_p(w), n, _p(qo), _p(so))
        r[name](_p(w), n, _p(qr), _p(sr))
        assert so[0] == sr[0] and (floor < 0 or so[0] == F(fl)), (name, so, sr)
        assert np.array_equal(qo[:count], qr[:count]), name
    if floor < 0:   # closed forms
        q = np.zeros(n, np.int8)
        s = np.array([floor], F)
        o["ws_convert_int8"](_p(w), n, _p(q), _p(s))
        m = np.abs(w).max()
        assert s[0] == F(127.0) / m and np.abs(q).max() == 127
        assert np.array_equal(q, np.rint((w * s[0]).astype(F)).astype(np.int8))   # numpy rint is round-half-even
        q4 = np.zeros(n // 2, np.int8)
        o["ws_convert_int4"](_p(w), n, _p(q4), _p(s))
        nib = np.rint((w.astype(np.float64) * 7.0 / np.float64(m)).astype(F)).astype(np.int32) + 7
        assert nib.min() >= 0 and nib.max() <= 14 and (nib.max() == 14 or nib.min() == 0)
        assert np.array_equal(q4.view(np.uint8), (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8))


@pytest.mark.parametrize("n", [8, 4096])
def test_ws_convert_bnn(oracle, ref, n):
    o, r = bind(oracle.lib, "orc_"), bind(ref.lib, "ref_")
    for seed, first_positive in ((1, True), (2, False)):
        rng = np.random.default_rng(seed + n)
        w = np.where(rng.random(n) < 0.5, F(0.75), F(-0.75)).astype(F)
        if not first_positive:
            w[:] = -np.abs(w)
        bo, br = np.zeros(n // 8, np.uint8), np.zeros(n // 8, np.uint8)
        so, sr = o["ws_convert_bnn"](_p(w), n, _p(bo)), r["ws_convert_bnn"](_p(w), n, _p(br))
        assert so == sr and np.array_equal(bo, br)
        assert np.array_equal(bo, np.packbits(w > 0))       # MSB-first, like numpy's default bit order
        assert so == (F(0.75) if first_positive else w[-1])


@pytest.mark.parametrize("n", [16, 1000, 65536])
def test_load_time_expansion(oracle, ref, n):
    o, r = bind(oracle.lib, "orc_"), bind(ref.lib, "ref_")
    rng = np.random.default_rng(n)
    q = rng.integers(-127, 128, size=n, dtype=np.int8)
    scale = F(37.3)
    do, dr = np.zeros(n, F), np.zeros(n, F)
    o["dequantize_int8_weight"](n, scale, _p(q), _p(do))
    r["dequantize_int8_weight"](n, scale, _p(q), _p(dr))
    assert np.array_equal(do.view(np.int32), dr.view(np.int32))
    nib = rng.integers(0, 15, size=n, dtype=np.uint8)
    packed = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8).view(np.int8)
    for name, dt in (("dequantize_int4_int8", np.int8), ("dequantize_int4_u8q", np.uint8)):
        a, b = np.zeros(n, dt), np.zeros(n, dt)
        o[name](n, _p(packed), _p(a))
        r[name](n, _p(packed), _p(b))
        assert np.array_equal(a, b)
        assert np.array_equal(a.astype(np.int32), nib.astype(np.int32) + (-7 if dt == np.int8 else 121))
    # int4 -> fp32 has no instantiation in the compiled reference (it is only built for fp16 there): pinned through the
    # two functions above, of which it is the composition -- table[nibble] = (1 / scale) * (nibble - 7)
    oracle.lib.orc_dequantize_int4_weight.argtypes = [C.c_int, C.c_float, vp, vp]
    d4 = np.zeros(n, F)
    oracle.lib.orc_dequantize_int4_weight(n, scale, _p(packed), _p(d4))
    i8 = np.zeros(n, np.int8)
    r["dequantize_int4_int8"](n, _p(packed), _p(i8))
    viaref = np.zeros(n, F)
    r["dequantize_int8_weight"](n, scale, _p(i8), _p(viaref))
    assert np.array_equal(d4.view(np.int32), viaref.view(np.int32))


@pytest.mark.parametrize("n", [16, 1000, 65536])
def test_model_loader_expansion(oracle, ref, n):
    """The model loader itself (common/model_spec/src/model_deserialize.cpp:270-331: TransWeightFromI8ToF32,
    TransWeightFromI4ToF32 / ToI8 / ToU8, applied to a WeightSpec as the .bolt file stores it) against the oracle's four
    expanders: the expanded bytes, the new bytes_of_weight (x 4, x 8, x 2, x 2) and what happens to the stored scale (an
    fp32 result zeroes it). This also pins the int4 -> fp32 expansion, which the compiled reference instantiates only here."""
    o = bind(oracle.lib, "orc_")
    oracle.lib.orc_dequantize_int4_weight.argtypes = [C.c_int, C.c_float, vp, vp]
    L = ref.lib.ref_loader_expand_weight
    L.argtypes, L.restype = [C.c_int, vp, C.c_uint, vp, vp], C.c_uint
    rng = np.random.default_rng(n + 1)
    q8 = rng.integers(-127, 128, size=n, dtype=np.int8)
    nib = rng.integers(0, 15, size=n, dtype=np.uint8)
    q4 = (nib[0::2] | (nib[1::2] << 4)).astype(np.uint8).view(np.int8)
    for kind, stored, out_dt, grow, zeroes in ((0, q8, F, 4, True), (1, q4, F, 8, True), (2, q4, np.int8, 2, False),
                                               (3, q4, np.uint8, 2, False)):
        sc = np.array([37.3], F)
        got = np.zeros(n, out_dt)
        nbytes = L(kind, _p(stored), stored.nbytes, _p(sc), _p(got))
        assert nbytes == stored.nbytes * grow == got.nbytes
        assert sc[0] == (0 if zeroes else F(37.3))
        want = np.zeros(n, out_dt)
        if kind == 0:
            o["dequantize_int8_weight"](n, F(37.3), _p(stored), _p(want))
        elif kind == 1:
            oracle.lib.orc_dequantize_int4_weight(n, F(37.3), _p(stored), _p(want))
        else:
            o["dequantize_int4_int8" if kind == 2 else "dequantize_int4_u8q"](n, _p(stored), _p(want))
        assert np.array_equal(got.view(np.uint8), want.view(np.uint8)), kind


def test_operator_scales_rule():
    """bolt_gfx950_operator_scales (pure host logic) against the three rules of the engine's operator classes, each
    written out here from the header it comes from and evaluated case by case:
      convolution     inference/engine/include/cpu/convolution_cpu.hpp:143-157
      fully connected inference/engine/include/cpu/fully_connected_cpu.hpp:92-103
      deconvolution   inference/engine/include/cpu/deconvolution_cpu.hpp:65-84
    and operator.hpp:164-169 for the no-quant label."""
    from bolt_amd import capi
    from bolt_amd.capi import DT_F32, DT_I8, DT_U8_Q
    CONV, FC, DECONV = 0, 1, 2

    class QuantSpec(C.Structure):
        _fields_ = [("num_scale", C.c_int32), ("scale", C.POINTER(C.c_float))]
    assert C.sizeof(QuantSpec) == 16

    def call(kind, records, idt, odt, in_scale, f_scale=F(50.0)):
        keep = [(C.c_float * len(r))(*r) for r in records]
        arr = (QuantSpec * max(1, len(records)))()
        for i, k in enumerate(keep):
            arr[i].num_scale, arr[i].scale = len(k), C.cast(k, C.POINTER(C.c_float))
        out, noq = (C.c_float * 3)(), C.c_int(-1)
        e = capi.lib().bolt_gfx950_operator_scales(kind, C.cast(arr, C.c_void_p) if records else None, len(records), idt, odt,
                                                   in_scale, f_scale, out, C.byref(noq))
        assert e == capi.SUCCESS
        return [F(v) for v in out], noq.value

    def header_rule(kind, fs, idt, odt, in_scale, f_scale):
        """the three run() bodies, statement by statement"""
        quant = (DT_I8, DT_U8_Q)
        s = [None, None, f_scale]
        s[0] = in_scale
        if kind == CONV:
            if idt not in quant and len(fs) > 0 and fs[0][0] > 0:
                s[0] = F(fs[0][0])
            s[1] = F(fs[-1][0]) if (len(fs) > 0 and fs[-1][0] != -2) else F(-1)
        else:
            if len(fs) > 1 and fs[0][0] > 0 and idt not in quant:
                s[0] = F(fs[0][0])
            if odt in quant:
                s[1] = F(fs[-1][0]) if len(fs) > 0 else F(-1)
            else:
                s[1] = F(0) if kind == DECONV else F(-1)   # `F32 scales[3] = {-1}`: slot 1 starts at 0 / tensor untouched
        return s

    cases = ([], [[12.5], [31.0]], [[12.5], [-2.0]], [[0.0], [31.0]], [[127.0 / 2.5]], [[-2.0]], [[12.5], [7.0], [31.0]])
    for kind in (CONV, FC, DECONV):
        for fs in cases:
            for idt, in_scale in ((DT_F32, F(-1.0)), (DT_U8_Q, F(9.0)), (DT_I8, F(4.5))):
                for odt in (DT_F32, DT_U8_Q, DT_I8):
                    got, noq = call(kind, fs, idt, odt, in_scale)
                    assert got == header_rule(kind, fs, idt, odt, in_scale, F(50.0)), (kind, fs, idt, odt)
                    assert noq == (1 if (fs and fs[0][0] == 0) else 0)
    # the cases the three classes disagree on, spelled out
    one = [[127.0 / 2.5]]                                           # a single positive record (a clip value of 2.5)
    assert call(CONV, one, DT_F32, DT_U8_Q, F(-1.0))[0][:2] == [F(127.0 / 2.5), F(127.0 / 2.5)]    # serves both ends
    assert call(FC, one, DT_F32, DT_U8_Q, F(-1.0))[0][:2] == [F(-1.0), F(127.0 / 2.5)]             # output only
    assert call(DECONV, one, DT_F32, DT_U8_Q, F(-1.0))[0][:2] == [F(-1.0), F(127.0 / 2.5)]
    assert call(CONV, [[12.5], [-2.0]], DT_F32, DT_U8_Q, F(-1.0))[0][1] == F(-1.0)                 # -2 -> dynamic
    assert call(FC, [[12.5], [-2.0]], DT_F32, DT_U8_Q, F(-1.0))[0][1] == F(-2.0)                   # passed through
    assert call(DECONV, [[12.5], [-2.0]], DT_F32, DT_U8_Q, F(-1.0))[0][1] == F(-2.0)
    assert call(CONV, [[12.5], [31.0]], DT_F32, DT_F32, F(-1.0))[0][1] == F(31.0)                  # whatever the output type
    assert call(FC, [[12.5], [31.0]], DT_F32, DT_F32, F(-1.0))[0][1] == F(-1.0)                    # tensor left alone
    assert call(DECONV, [[12.5], [31.0]], DT_F32, DT_F32, F(-1.0))[0][1] == F(0.0)
    assert capi.lib().bolt_gfx950_operator_scales(7, None, 0, DT_F32, DT_F32, F(1.0), F(1.0), (C.c_float * 3)(), None) == capi.NOT_SUPPORTED
