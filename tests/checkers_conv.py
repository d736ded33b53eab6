"""ctypes bindings for the convolution parts of the CPU checkers (test infrastructure only)."""
import ctypes as C

import numpy as np

from checkers import DT_F32, DT_I32, DT_U8_Q, NP_OF, Oracle, Ref, _p, u32, vp

DF_NCHWC8, DF_NCHWC16 = 2, 41


class ConvDesc(C.Structure):
    _fields_ = [(k, C.c_uint32) for k in ("n", "ic", "ih", "iw", "oc", "fh", "fw", "sh", "sw", "pt", "pb", "pl", "pr",
                                          "dh", "dw", "oh", "ow")] + [("relu", C.c_int), ("odt", C.c_int),
                                                                      ("out_c", C.c_int)]


class BnnDesc(C.Structure):
    _fields_ = [(k, C.c_uint32) for k in ("n", "ic", "ih", "iw", "oc", "fh", "fw", "sh", "sw", "pt", "pb", "pl", "pr",
                                          "oh", "ow")] + [("xnor", C.c_int)]


def conv_out_hw(ih, iw, fh, fw, sh, sw, pt, pb, pl, pr, dh=1, dw=1):
    oh = (ih + pt + pb - ((fh - 1) * dh + 1)) // sh + 1
    ow = (iw + pl + pr - ((fw - 1) * dw + 1)) // sw + 1
    return oh, ow


def to_nchwc(x_nchw, c):
    """[n][C][h][w] -> NCHWCc memory order."""
    n, ch, h, w = x_nchw.shape
    return np.ascontiguousarray(x_nchw.reshape(n, ch // c, c, h, w).transpose(0, 1, 3, 4, 2))


def from_conv_layout(buf, n, oc, oh, ow, out_c):
    """Output of the x86 path (blocks of out_c channels, trailing narrower block) -> plain [n][oc][oh][ow]."""
    out = np.empty((n, oc, oh, ow), buf.dtype)
    flat = buf.reshape(n, oc * oh * ow)
    pos = 0
    for b0 in range(0, oc, out_c):
        bw = min(out_c, oc - b0)
        blk = flat[:, pos:pos + bw * oh * ow].reshape(n, oh, ow, bw)
        out[:, b0:b0 + bw] = blk.transpose(0, 3, 1, 2)
        pos += bw * oh * ow
    return out


def to_conv_layout(x_nchw, out_c):
    """plain [n][oc][oh][ow] -> the x86 path's output order (inverse of from_conv_layout), flattened"""
    n, oc, oh, ow = x_nchw.shape
    parts = []
    for b0 in range(0, oc, out_c):
        bw = min(out_c, oc - b0)
        parts.append(x_nchw[:, b0:b0 + bw].transpose(0, 2, 3, 1).reshape(n, oh * ow * bw))
    return np.ascontiguousarray(np.concatenate(parts, axis=1)).reshape(-1)


class ConvOracle:
    def __init__(self, oracle=None):
        self.lib = (oracle or Oracle()).lib
        self.lib.orc_conv_int8_acc.argtypes = [vp, vp, vp, vp, C.c_float, C.c_float, vp]
        self.lib.orc_conv_int8.argtypes = [vp, vp, vp, vp, vp, vp, vp]

    @staticmethod
    def desc(n, ic, ih, iw, oc, fh, fw, stride, pad, relu, odt, out_c=16, dil=1):
        oh, ow = conv_out_hw(ih, iw, fh, fw, stride, stride, pad, pad, pad, pad, dil, dil)
        return ConvDesc(n, ic, ih, iw, oc, fh, fw, stride, stride, pad, pad, pad, pad, dil, dil, oh, ow, int(relu), odt,
                        out_c)

    def conv(self, d, in_nchwc8, filt_nchw, bias, scale, eltwise=None):
        """Returns (output in the x86 layout, scale[3])."""
        x = np.ascontiguousarray(in_nchwc8, dtype=np.uint8)
        f = np.ascontiguousarray(filt_nchw, dtype=np.int8)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        e = None if eltwise is None else np.ascontiguousarray(eltwise, dtype=np.float32)
        s = np.array(scale, np.float32).copy()
        out = np.zeros(d.n * d.oc * d.oh * d.ow, NP_OF[d.odt])
        self.lib.orc_conv_int8(C.byref(d), _p(x), _p(f), _p(b), _p(e), _p(s), _p(out))
        return out, s

    def conv_perchannel(self, oracle, d, in_nchwc8, filt_nchw, scale_w, bias, scale_in, out_scale=-1.0, eltwise=None):
        """The int8 convolution with one filter scale per output channel, which the reference does not have: a
        composition of two pinned pieces with three fp32 numpy operations between them,
          acc  = the reference-pinned int32 convolution (orc_conv_int8_acc through conv(), no bias, no ReLU)
          f    = cvt(acc) * (1.0f / (sI * sW[oc]))  [+ bias[oc]]  [+ eltwise]  [ReLU]
          u8   = the reference-pinned fp32 -> u8 quantiser (orc_quantize_f32_u8): static with out_scale > 0, else dynamic
        d.odt selects DT_F32 or DT_U8_Q. Returns (output in the x86 layout of d.out_c, output scale or None).
        tests/test_oracle_conv.py holds it against the reference's own epilogue (equal scales) and against closed forms."""
        di = ConvDesc.from_buffer_copy(d)
        di.relu, di.odt = 0, DT_I32
        acc, _ = self.conv(di, in_nchwc8, filt_nchw, None, [scale_in, -1.0, 1.0])
        acc = from_conv_layout(acc, d.n, d.oc, d.oh, d.ow, d.out_c)                      # [n][oc][oh][ow]
        sw = np.ascontiguousarray(scale_w, dtype=np.float32)
        r = np.float32(1.0) / (np.float32(scale_in) * sw)                                   # reciprocal first
        f = acc.astype(np.float32) * r[None, :, None, None]
        if bias is not None:
            f = f + np.ascontiguousarray(bias, dtype=np.float32)[None, :, None, None]
        if eltwise is not None:
            f = f + from_conv_layout(np.ascontiguousarray(eltwise, dtype=np.float32), d.n, d.oc, d.oh, d.ow, d.out_c)
        if d.relu:
            f = np.where(f > 0, f, np.float32(0)).astype(np.float32)
        flat = to_conv_layout(f.astype(np.float32), d.out_c)
        if d.odt == DT_F32:
            return flat, None
        if out_scale > 0:
            q, s = oracle.quantize_f32(flat, DT_U8_Q, out_scale, 1)
        else:
            q, s = oracle.quantize_f32(flat, DT_U8_Q)
        return q, s

    def bnn_desc(self, n, ic, ih, iw, oc, fh, fw, stride, pad, xnor):
        oh, ow = conv_out_hw(ih, iw, fh, fw, stride, stride, pad, pad, pad, pad)
        return BnnDesc(n, ic, ih, iw, oc, fh, fw, stride, stride, pad, pad, pad, pad, oh, ow, int(xnor))

    def bnn_pack_input(self, d, x_nchwc8):
        x = np.ascontiguousarray(x_nchwc8, dtype=np.float32)
        bits = np.zeros(d.n * (d.ic // 8) * d.ih * d.iw, np.uint8)
        self.lib.orc_bnn_pack_input(C.byref(d), _p(x), _p(bits))
        return bits

    def bnn_conv(self, d, in_bits, w_bits, scale, bias):
        sums = np.zeros(d.n * d.oc * d.oh * d.ow, np.int32)
        out = np.zeros(d.n * d.oc * d.oh * d.ow, np.float32)
        sc = np.ascontiguousarray(scale, dtype=np.float32)
        bs = np.ascontiguousarray(bias, dtype=np.float32)
        self.lib.orc_bnn_conv(C.byref(d), _p(np.ascontiguousarray(in_bits)), _p(np.ascontiguousarray(w_bits)), _p(sc),
                              _p(bs), _p(sums), _p(out))
        return sums, out

    def bnn_bruteforce(self, d, x_nchw, w_nchw):
        sums = np.zeros((d.n, d.oc, d.oh, d.ow), np.int32)
        self.lib.orc_bnn_conv_bruteforce(C.byref(d), _p(np.ascontiguousarray(x_nchw, dtype=np.float32)),
                                         _p(np.ascontiguousarray(w_nchw, dtype=np.float32)), _p(sums))
        return sums


def bnn_pack_filter_nchwn16c8(w_nchw_pm, xnor=True):
    """+-1 (or 0/1) filter values [oc][ic][fh][fw] -> DF_NCHWN16C8 bytes, MSB = first channel of the 8
    (compute/tensor/src/cpu/arm/bnn/convolution_transform_bnn.h:58-79)."""
    oc, ic, fh, fw = w_nchw_pm.shape
    thr = 0.0 if xnor else 0.5
    bits = (w_nchw_pm >= thr).astype(np.uint8)                        # [oc][ic][fh][fw]
    b = bits.reshape(oc // 16, 16, ic // 8, 8, fh * fw)               # [o][o16][c][c8][hw]
    b = b.transpose(0, 2, 4, 1, 3)                                    # [o][c][hw][o16][c8]
    weights = (1 << (7 - np.arange(8))).astype(np.uint8)
    return np.ascontiguousarray((b * weights).sum(-1).astype(np.uint8)).reshape(-1)


def ref_conv(ref, d, in_buf, idf, filt_nchw, bias, scale, eltwise=None, alg=1):
    """The reference's own compiled convolution_int8 (always writes its NCHWC16 layout)."""
    x = np.ascontiguousarray(in_buf, dtype=np.uint8)
    f = np.ascontiguousarray(filt_nchw, dtype=np.int8)
    b = np.ascontiguousarray(bias, dtype=np.float32)
    e = None if eltwise is None else np.ascontiguousarray(eltwise, dtype=np.float32)
    s = np.array(scale, np.float32).copy()
    out = np.zeros(d.n * d.oc * d.oh * d.ow + 64, NP_OF[d.odt])
    rc = ref.lib.ref_conv_int8(u32(d.n), u32(d.ic), u32(d.ih), u32(d.iw), idf, u32(d.oc), u32(d.fh), u32(d.fw),
                               u32(d.sh), u32(d.sw), u32(d.pt), u32(d.pb), u32(d.pl), u32(d.pr), u32(d.dh), u32(d.dw),
                               u32(d.oh), u32(d.ow), alg, _p(x), _p(f), _p(b), _p(e), _p(s), d.relu, d.odt, _p(out))
    assert rc == 0, rc
    return out[:d.n * d.oc * d.oh * d.ow], s
