"""ctypes bindings for the pooling / concatenation parts of the CPU checkers (test infrastructure only)."""
import ctypes as C

import numpy as np

from checkers import _p, u32, vp


class PoolDesc(C.Structure):
    _fields_ = [(k, C.c_uint32) for k in ("n", "c", "ih", "iw", "oh", "ow", "kh", "kw", "sh", "sw", "pt", "pl")] + [
        ("mean", C.c_int), ("count_include_pad", C.c_int)]


def pool_out(i, k, s, a, b, ceil):
    v = (i + a + b - k) / s
    return int(np.ceil(v) if ceil else np.floor(v)) + 1


def pool_desc(case):
    """case: n, c, ih, iw, kh, kw, sh, sw, pt, pb, pl, pr, mean, count_include_pad, ceil"""
    n, c, ih, iw, kh, kw, sh, sw, pt, pb, pl, pr, mean, cip, ceil = case
    return PoolDesc(n, c, ih, iw, pool_out(ih, kh, sh, pt, pb, ceil), pool_out(iw, kw, sw, pl, pr, ceil), kh, kw, sh, sw,
                    pt, pl, int(mean), int(cip))


def orc_pooling(oracle, d, x, in_scale):
    L = oracle.lib
    L.orc_pooling_u8_c16.argtypes = [vp, vp, vp, vp]
    L.orc_pooling_u8_c16.restype = C.c_int
    out = np.zeros(d.n * d.c * d.oh * d.ow, np.uint8)
    sc = np.array([in_scale, 0], np.float32)
    e = L.orc_pooling_u8_c16(C.byref(d), _p(x), _p(out), _p(sc))
    assert e == 0
    return out, sc[1]


def ref_pooling(ref, d, x, in_scale):
    out = np.zeros(d.n * d.c * d.oh * d.ow, np.uint8)
    sc = np.array([in_scale, 0], np.float32)
    e = ref.lib.ref_pooling_u8(u32(d.n), u32(d.c), u32(d.ih), u32(d.iw), u32(d.oh), u32(d.ow), u32(d.kh), u32(d.kw),
                               u32(d.sh), u32(d.sw), u32(d.pt), u32(d.pl), d.mean, d.count_include_pad, _p(x), _p(out),
                               _p(sc))
    assert e == 0
    return out, sc[1]


def orc_concat(oracle, parts, lens, loops, scales):
    """parts: s8 arrays of loops * lens[j] bytes. Returns (output, output scale)."""
    L = oracle.lib
    L.orc_concat_i8.argtypes = [u32, vp, vp, vp, u32, vp, vp]
    L.orc_concat_i8.restype = None
    num = len(parts)
    ptrs = (vp * num)(*[p.ctypes.data for p in parts])
    la = np.array(lens, np.uint32)
    out = np.zeros(int(sum(lens)) * loops, np.int8)
    osc = np.zeros(1, np.float32)
    sa = None if scales is None else np.array(scales, np.float32)
    L.orc_concat_i8(num, ptrs, _p(la), _p(sa), loops, _p(out), _p(osc))
    return out, (None if scales is None else osc[0])


def ref_concat(ref, parts, dims, df, axis, scales, odims):
    """dims: per input (n, c, h, w); the reference rescales its inputs in place, so copies are passed."""
    num = len(parts)
    copies = [np.array(p, copy=True) for p in parts]
    ptrs = (vp * num)(*[p.ctypes.data for p in copies])
    da = np.array(dims, np.uint32).reshape(-1)
    oa = np.array(odims, np.uint32)
    out = np.zeros(int(np.prod(odims)), np.int8)
    sa = np.array(scales, np.float32)
    osc = np.zeros(1, np.float32)
    e = ref.lib.ref_concat_i8(u32(num), _p(da), int(df), int(axis), ptrs, _p(sa), _p(oa), _p(out), _p(osc))
    assert e == 0
    return out, osc[0]
