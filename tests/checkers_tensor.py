"""ctypes bindings for the reference's Tensor-level operators and fp32 encoder neighbours compiled into
oracle/_ref/libboltref.so (oracle/ref_shim_tensor.cpp). Test infrastructure only."""
import ctypes as C

import numpy as np

from checkers import DT_F32, DT_I8, DT_I32, DT_U8_Q, NP_OF, REF_SO, Ref, _p, u32, vp

F32P = C.POINTER(C.c_float)


class RefTensor:
    @staticmethod
    def available():
        return Ref.available()

    def __init__(self):
        self.lib = C.CDLL(REF_SO)
        L = self.lib
        L.ref_set_threads(1)
        L.ref_fc_tensor.argtypes = [u32, u32, u32, vp, C.c_float, vp, C.c_float, vp, C.c_int, C.c_int, vp, vp, vp]
        L.ref_matmul_tensor.argtypes = [C.c_int, vp, u32, C.c_int, vp, C.c_float, C.c_int, vp, u32, C.c_int, vp,
                                        C.c_float, C.c_int, vp, u32, vp, vp]
        L.ref_conv_queries.argtypes = [u32] * 4 + [C.c_int] + [u32] * 11 + [C.c_int, vp]
        L.ref_layer_norm_f32.argtypes = [u32, u32, vp, vp, vp, vp]
        L.ref_softmax_f32.argtypes = [u32, u32, vp, vp]
        L.ref_gelu_f32.argtypes = [u32, vp, vp]

    def fully_connected(self, x, scaleI, W_NK, scaleW, bias, odt, scaleO=-1.0, mvm=False):
        """Returns (output, output tensor scale after the call, fully_connected_infer_forward_tmp_bytes)."""
        x = np.ascontiguousarray(x, np.uint8)
        W = np.ascontiguousarray(W_NK, np.int8)
        M, K = x.shape
        N = W.shape[0]
        b = None if bias is None else np.ascontiguousarray(bias, np.float32)
        out = np.zeros((M, N), NP_OF[odt])
        s = np.array([scaleO], np.float32)
        tb = np.zeros(1, np.uint32)
        e = self.lib.ref_fc_tensor(M, K, N, _p(x), C.c_float(scaleI), _p(W), C.c_float(scaleW), _p(b), int(mvm), odt,
                                   _p(out), _p(s), _p(tb))
        assert e == 0, e
        return out, s[0], int(tb[0])

    def matmul(self, A, adt, tA, scaleA, B, bdt, tB, scaleB, c_shape, cdt=DT_F32):
        A = np.ascontiguousarray(A, NP_OF[adt])
        B = np.ascontiguousarray(B, NP_OF[bdt])
        sa, sb, sc = (np.array(s, np.uint32) for s in (A.shape, B.shape, c_shape))
        out = np.zeros(c_shape, NP_OF[cdt])
        tb = np.zeros(1, np.uint32)
        e = self.lib.ref_matmul_tensor(adt, _p(sa), sa.size, int(tA), _p(A), C.c_float(scaleA), bdt, _p(sb), sb.size,
                                       int(tB), _p(B), C.c_float(scaleB), cdt, _p(sc), sc.size, _p(out), _p(tb))
        assert e == 0, e
        return out, int(tb[0])

    def conv_queries(self, n, ic, ih, iw, idf, oc, fh, fw, sh, sw, pt, pb, pl, pr, dh=1, dw=1, relu=1):
        """dict(out=(dt, df, nDims, dims...), alg, filter_bytes, ftm=(dt, df, nDims, dims...), tmp_bytes)."""
        q = np.zeros(21, np.uint32)
        e = self.lib.ref_conv_queries(n, ic, ih, iw, idf, oc, fh, fw, sh, sw, pt, pb, pl, pr, dh, dw, int(relu), _p(q))
        assert e == 0, e
        return {"out": tuple(int(v) for v in q[0:9]), "alg": int(q[9]), "filter_bytes": int(q[10]),
                "ftm": tuple(int(v) for v in q[11:20]), "tmp_bytes": int(q[20])}

    def layer_norm(self, x, gamma, beta):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        g, b = np.ascontiguousarray(gamma, np.float32), np.ascontiguousarray(beta, np.float32)
        assert self.lib.ref_layer_norm_f32(x.shape[0], x.shape[1], _p(x), _p(g), _p(b), _p(out)) == 0
        return out

    def softmax(self, x):
        x = np.ascontiguousarray(x, np.float32)
        out = np.empty_like(x)
        assert self.lib.ref_softmax_f32(x.shape[0], x.shape[1], _p(x), _p(out)) == 0
        return out

    def gelu(self, x):
        x = np.ascontiguousarray(x, np.float32)
        assert x.size % 8 == 0
        out = np.empty_like(x)
        assert self.lib.ref_gelu_f32(x.size, _p(x), _p(out)) == 0
        return out
