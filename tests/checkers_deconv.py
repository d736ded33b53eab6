"""ctypes bindings for the deconvolution parts of the CPU checkers (test infrastructure only)."""
import ctypes as C

import numpy as np

from checkers import DT_F32, DT_I32, DT_U8_Q, NP_OF, Oracle, _p, u32, vp
from checkers_conv import to_nchwc

DF_NCHW, DF_NCHWC8, DF_NCHWC16 = 0, 2, 41
ALG_POINTWISE, ALG_IM2COL_GEMM = 0, 2


class DeconvDesc(C.Structure):
    _fields_ = [(k, C.c_uint32) for k in ("n", "ic", "ih", "iw", "oc", "fh", "fw", "sh", "sw", "pt", "pb", "pl", "pr",
                                          "oh", "ow")] + [("in_c", C.c_int), ("out_c", C.c_int), ("relu", C.c_int),
                                                          ("odt", C.c_int)]


def deconv_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, in_c, relu, odt):
    """stride / pad: an int or (h, w) / (top, bottom, left, right)."""
    sh, sw = (stride, stride) if np.isscalar(stride) else stride
    pt, pb, pl, pr = (pad,) * 4 if np.isscalar(pad) else pad
    oh = fh + sh * (ih - 1) - pt - pb
    ow = fw + sw * (iw - 1) - pl - pr
    return DeconvDesc(n, ic, ih, iw, oc, fh, fw, sh, sw, pt, pb, pl, pr, oh, ow, in_c, 16 if oc > 8 else 8, int(relu),
                      odt)


def idf_of(in_c):
    return {0: DF_NCHW, 8: DF_NCHWC8, 16: DF_NCHWC16}[in_c]


def lay_input(x_nchw, in_c):
    return np.ascontiguousarray(x_nchw) if in_c == 0 else to_nchwc(x_nchw, in_c)


def plain_output(buf, d):
    """Output tensor (NCHWC16, or NCHWC8 for 8 channels) -> [n][oc][oh][ow]."""
    x = d.out_c
    return buf.reshape(d.n, d.oc // x, d.oh, d.ow, x).transpose(0, 1, 4, 2, 3).reshape(d.n, d.oc, d.oh, d.ow)


class DeconvOracle:
    def __init__(self, oracle=None):
        self.lib = (oracle or Oracle()).lib
        self.lib.orc_deconv_int8.argtypes = [vp, vp, vp, vp, vp, vp]

    def deconv(self, d, in_buf, filt, bias, scale):
        """filt: s8 [ic][oc][fh][fw]. Returns (output in the tensor's layout, scale[3] as the call leaves it)."""
        x = np.ascontiguousarray(in_buf, dtype=np.uint8)
        f = np.ascontiguousarray(filt, dtype=np.int8)
        b = np.ascontiguousarray(bias, dtype=np.float32)
        s = np.array(scale, np.float32).copy()
        out = np.zeros(d.n * d.oc * d.oh * d.ow, NP_OF[d.odt])
        self.lib.orc_deconv_int8(C.byref(d), _p(x), _p(f), _p(b), _p(s), _p(out))
        return out, s


def ref_deconv(ref, d, in_buf, filt, bias, scale):
    """The reference's own deconvolution through its Tensor-level calls. Returns (output, scale[3], queries) with
    queries = {out_desc, alg, filter_bytes, ftm_desc, tmp_bytes}."""
    x = np.ascontiguousarray(in_buf, dtype=np.uint8)
    f = np.ascontiguousarray(filt, dtype=np.int8)
    b = np.ascontiguousarray(bias, dtype=np.float32)
    s = np.array(scale, np.float32).copy()
    total = d.n * d.oc * d.oh * d.ow
    out = np.zeros(total + 64, NP_OF[d.odt])
    q = np.zeros(32, np.uint32)
    rc = ref.lib.ref_deconv_int8(u32(d.n), u32(d.ic), u32(d.ih), u32(d.iw), idf_of(d.in_c), u32(d.oc), u32(d.fh),
                                 u32(d.fw), u32(d.sh), u32(d.sw), u32(d.pt), u32(d.pb), u32(d.pl), u32(d.pr), _p(x), _p(f),
                                 _p(b), _p(s), d.relu, d.odt, _p(out), _p(q))
    assert rc == 0, rc
    return out[:total], s, {"out_desc": q[:9].copy(), "alg": int(q[9]), "filter_bytes": int(q[10]),
                            "ftm_desc": q[11:20].copy(), "tmp_bytes": int(q[20])}


def make_deconv_case(n, ic, ih, iw, oc, fh, fw, seed):
    rng = np.random.default_rng(seed)
    x = rng.integers(1, 256, size=(n, ic, ih, iw), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(ic, oc, fh, fw), dtype=np.int8)
    bias = (rng.standard_normal(oc) * 0.5).astype(np.float32)
    return x, np.float32(23.5), W, np.float32(41.25), bias
