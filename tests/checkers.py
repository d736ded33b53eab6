"""ctypes bindings for the CPU checkers (test infrastructure, never used by the product).

`Oracle`  -> oracle/liboracle.so        (C restatement, always available after `make -C oracle oracle`)
`Ref`     -> oracle/_ref/libboltref.so  (the reference's own compiled x86 sources; needs avx512_vnni)
"""
import ctypes as C
import os
import subprocess

import numpy as np

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))
ORACLE_SO = os.path.join(ROOT, "oracle", "liboracle.so")
REF_SO = os.path.join(ROOT, "oracle", "_ref", "libboltref.so")

DT_I8, DT_I32, DT_F32, DT_U8_Q = 1, 3, 6, 10
NP_OF = {DT_I8: np.int8, DT_I32: np.int32, DT_F32: np.float32, DT_U8_Q: np.uint8}

u32 = C.c_uint32
vp = C.c_void_p


def _p(a):
    return None if a is None else a.ctypes.data_as(vp)


def host_has_vnni():
    try:
        with open("/proc/cpuinfo") as f:
            return "avx512_vnni" in f.read()
    except OSError:
        return False


def build_oracle():
    if not os.path.exists(ORACLE_SO):
        subprocess.check_call(["make", "-C", os.path.join(ROOT, "oracle"), "oracle"],
                              stdout=subprocess.DEVNULL)


def _scale_arg(scale):
    if scale is None:
        return None, None
    arr = np.array(scale, dtype=np.float32).reshape(-1)
    return arr, _p(arr)


class Oracle:
    def __init__(self):
        build_oracle()
        self.lib = C.CDLL(ORACLE_SO)
        L = self.lib
        L.orc_mmm_tmp_bytes.restype = u32
        L.orc_mmm_tmp_bytes.argtypes = [u32, u32, u32, C.c_int, C.c_int]
        L.orc_mvm_transform_weight_bytes.restype = u32
        L.orc_mvm_transform_weight_bytes.argtypes = [u32, u32, C.c_int, C.c_int]
        L.orc_mmm_transform_rhs_bytes.argtypes = [u32, u32, C.c_int, vp, vp]
        L.orc_symmetric_scale_f32.restype = C.c_float
        L.orc_symmetric_scale_f32.argtypes = [vp, u32]
        L.orc_requantize_i8.argtypes = [vp, u32, C.c_float, vp, C.c_float]
        L.orc_fully_connected_int8.argtypes = [u32, u32, u32, vp, C.c_float, vp, C.c_float, vp, vp,
                                               C.c_int, vp]

    # ---- sizes
    def mmm_transform_rhs_bytes(self, N, K, packed=False):
        b, r = u32(0), u32(0)
        self.lib.orc_mmm_transform_rhs_bytes(N, K, int(packed), C.byref(b), C.byref(r))
        return b.value, r.value

    def mmm_tmp_bytes(self, N, M, K, transA=False, packedB=True):
        return self.lib.orc_mmm_tmp_bytes(N, M, K, int(transA), int(packedB))

    def mvm_transform_weight_bytes(self, N, K, wdt=DT_I8, packed=False):
        return self.lib.orc_mvm_transform_weight_bytes(N, K, wdt, int(packed))

    # ---- blas
    def offsetC(self, W, w_is_NK):
        W = np.ascontiguousarray(W, dtype=np.int8)
        N, K = (W.shape if w_is_NK else W.shape[::-1])
        out = np.empty(N, np.int32)
        self.lib.orc_offsetC(_p(W), u32(K), u32(N), int(w_is_NK), _p(out))
        return out

    def mmm(self, A, W, offsetC, C_in, cdt, scale=None, transA=False, w_is_NK=True):
        """A: u8 [M,K] (or [K,M] if transA); W: s8 [N,K] if w_is_NK else [K,N]."""
        A = np.ascontiguousarray(A, dtype=np.uint8)
        W = np.ascontiguousarray(W, dtype=np.int8)
        M, K = (A.shape[::-1] if transA else A.shape)
        N = W.shape[0] if w_is_NK else W.shape[1]
        out = np.array(C_in, dtype=NP_OF[cdt]).reshape(M, N).copy()
        keep, sp = _scale_arg(scale)
        off = np.ascontiguousarray(offsetC, dtype=np.int32)
        self.lib.orc_mmm_int8(u32(M), u32(N), u32(K), _p(A), int(transA), _p(W), int(w_is_NK), _p(off),
                              _p(out), cdt, sp)
        return out

    def mvm(self, W, x, offsetC, y_in, ydt, scale=None, w_is_NK=True):
        W = np.ascontiguousarray(W, dtype=np.int8)
        x = np.ascontiguousarray(x, dtype=np.uint8)
        N, K = (W.shape if w_is_NK else W.shape[::-1])
        out = np.array(y_in, dtype=NP_OF[ydt]).reshape(N).copy()
        keep, sp = _scale_arg(scale)
        off = np.ascontiguousarray(offsetC, dtype=np.int32)
        self.lib.orc_mvm_int8(u32(N), u32(K), _p(W), int(w_is_NK), _p(x), _p(off), _p(out), ydt, sp)
        return out

    def mvm_u8mat(self, A, x, y_in, ydt, scale=None, a_is_KM=False):
        A = np.ascontiguousarray(A, dtype=np.uint8)
        x = np.ascontiguousarray(x, dtype=np.int8)
        M, K = (A.shape[::-1] if a_is_KM else A.shape)
        out = np.array(y_in, dtype=NP_OF[ydt]).reshape(M).copy()
        keep, sp = _scale_arg(scale)
        self.lib.orc_mvm_u8mat_i8vec(u32(M), u32(K), _p(A), int(a_is_KM), _p(x), _p(out), ydt, sp)
        return out

    # ---- quantize family
    def symmetric_scale(self, x):
        x = np.ascontiguousarray(x, dtype=np.float32)
        return np.float32(self.lib.orc_symmetric_scale_f32(_p(x), u32(x.size)))

    def quantize_f32(self, x, qdt, scale=-1.0, mode=0):
        x = np.ascontiguousarray(x, dtype=np.float32)
        q = np.empty(x.shape, NP_OF[qdt])
        s = np.array([scale], np.float32)
        fn = self.lib.orc_quantize_f32_u8 if qdt == DT_U8_Q else self.lib.orc_quantize_f32_i8
        fn(_p(x), u32(x.size), _p(q), _p(s), int(mode))
        return q, s[0]

    def u8_to_i8(self, x):
        x = np.ascontiguousarray(x, dtype=np.uint8)
        q = np.empty(x.shape, np.int8)
        self.lib.orc_u8_to_i8(_p(x), u32(x.size), _p(q))
        return q

    def quantize_i32(self, x, qdt, scale):
        x = np.ascontiguousarray(x, dtype=np.int32)
        q = np.empty(x.shape, NP_OF[qdt])
        s = np.array(scale, np.float32).copy()
        fn = self.lib.orc_quantize_i32_u8 if qdt == DT_U8_Q else self.lib.orc_quantize_i32_i8
        fn(_p(x), u32(x.size), _p(q), _p(s))
        return q, s

    def bias_offsetC(self, bias, offsetC, scale, N=None):
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        o = None if offsetC is None else np.ascontiguousarray(offsetC, dtype=np.int32)
        N = N or (b.size if b is not None else o.size)
        out = np.empty(N, np.int32)
        s = np.array([scale], np.float32)
        self.lib.orc_bias_offsetC(_p(b), u32(N), _p(o), _p(s), _p(out))
        return out

    def dequantize(self, q, qdt, scale):
        q = np.ascontiguousarray(q, dtype=NP_OF[qdt])
        out = np.empty(q.shape, np.float32)
        s = np.array([scale], np.float32)
        fn = self.lib.orc_dequantize_i32_f32 if qdt == DT_I32 else self.lib.orc_dequantize_u8_f32
        fn(_p(q), u32(q.size), _p(s), _p(out))
        return out

    def requantize(self, x, inScale, outScale):
        x = np.ascontiguousarray(x, dtype=np.int8)
        out = np.empty(x.shape, np.int8)
        self.lib.orc_requantize_i8(_p(x), u32(x.size), C.c_float(inScale), _p(out), C.c_float(outScale))
        return out

    def axpby(self, a, x, b, y):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.array(y, dtype=np.float32).copy()
        self.lib.orc_axpby_f32.argtypes = [u32, C.c_float, vp, C.c_float, vp]
        self.lib.orc_axpby_f32(u32(x.size), C.c_float(a), _p(x), C.c_float(b), _p(out))
        return out

    def dequant_per_channel(self, acc, scaleI, scaleW, bias=None):
        acc = np.ascontiguousarray(acc, dtype=np.int32)
        M, N = acc.shape
        sI = np.array([scaleI], np.float32)
        sW = np.ascontiguousarray(scaleW, dtype=np.float32)
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        out = np.empty((M, N), np.float32)
        self.lib.orc_dequant_per_channel(_p(acc), u32(M), u32(N), _p(sI), _p(sW), _p(b), _p(out))
        return out

    def fully_connected(self, x, scaleI, W_NK, scaleW, bias, odt, scaleO=-1.0):
        x = np.ascontiguousarray(x, dtype=np.uint8)
        W = np.ascontiguousarray(W_NK, dtype=np.int8)
        M, K = x.shape
        N = W.shape[0]
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        out = np.zeros((M, N), NP_OF[odt])
        s = np.array([scaleO], np.float32)
        self.lib.orc_fully_connected_int8(u32(M), u32(K), u32(N), _p(x), C.c_float(scaleI), _p(W),
                                          C.c_float(scaleW), _p(b), _p(out), odt, _p(s))
        return out, s[0]

    def matmul(self, A, tA, B, tB, cdt, scaleA=-1.0, scaleB=-1.0):
        """Batched int8 matmul as the reference's x86 branch composes it (compute/tensor/src/matmul.cpp:367-431,
        495-554) for matrix results: fp32 A -> u8 and fp32 B -> s8 over the WHOLE tensor (scaleA / scaleB are the
        operand tensors' scales, lower bounds of the dynamic ones), scaleO = sA * sB, then per 2-D slice one
        u8 x s8 product starting from zero with cvt(acc) * (1 / scaleO) (cdt DT_F32) or the raw int32 (DT_I32).
        A: [.., M, K] or [.., K, M] if tA; B: [.., K, N] or [.., N, K] if tB. A smaller batch is broadcast.
        Returns (stacked slices, sA, sB)."""
        qa, sa = self.quantize_f32(np.ascontiguousarray(A).reshape(-1), DT_U8_Q, scaleA)
        qb, sb = self.quantize_f32(np.ascontiguousarray(B).reshape(-1), DT_I8, scaleB)
        qa, qb = qa.reshape(A.shape), qb.reshape(B.shape)
        A3 = qa.reshape((-1,) + A.shape[-2:])
        B3 = qb.reshape((-1,) + B.shape[-2:])
        batch = max(A3.shape[0], B3.shape[0])
        outs = []
        s = np.float32(sa) * np.float32(sb)
        for i in range(batch):
            a = A3[i % A3.shape[0]]
            b = B3[i % B3.shape[0]]
            W = b if tB else np.ascontiguousarray(b.T)          # [N, K]
            M = a.shape[1] if tA else a.shape[0]
            N = W.shape[0]
            off = self.offsetC(W, True)
            if cdt == DT_F32:
                outs.append(self.mmm(a, W, off, np.zeros((M, N), np.float32), DT_F32, scale=[s], transA=tA))
            else:
                outs.append(self.mmm(a, W, off, np.zeros((M, N), np.int32), DT_I32, transA=tA))
        return np.stack(outs), sa, sb


    def matmul_vector(self, A, tA, B, tB, cdt):
        """Vector result (one of M, N is 1): A -> I8, B -> U8_Q over the whole tensors, then one
        matrix_vector_multiply per slice (compute/tensor/src/matmul.cpp:374-382, 531-548)."""
        oracle = self
        qa, sa = oracle.quantize_f32(np.ascontiguousarray(A).reshape(-1), DT_I8)
        qb, sb = oracle.quantize_f32(np.ascontiguousarray(B).reshape(-1), DT_U8_Q)
        A3 = qa.reshape((-1,) + A.shape[-2:])
        B3 = qb.reshape((-1,) + B.shape[-2:])
        batch = max(A3.shape[0], B3.shape[0])
        s = np.float32(sa) * np.float32(sb)
        M = A.shape[-1] if tA else A.shape[-2]
        N = B.shape[-2] if tB else B.shape[-1]
        ydt = np.float32 if cdt == DT_F32 else np.int32
        sc = [s] if cdt == DT_F32 else None
        outs = []
        for i in range(batch):
            a = A3[i % A3.shape[0]]
            b = B3[i % B3.shape[0]]
            if M == 1:
                # u8 matrix b ([K, N], or [N, K] if tB) times the s8 vector a
                outs.append(oracle.mvm_u8mat(b, a.reshape(-1), np.zeros(N, ydt), cdt, scale=sc, a_is_KM=not tB))
            else:
                # s8 matrix a ([M, K], or [K, M] if tA) times the u8 vector b
                off = oracle.offsetC(a, not tA)
                outs.append(oracle.mvm(a, b.reshape(-1), off, np.zeros(M, ydt), cdt, scale=sc, w_is_NK=not tA))
        return np.stack(outs), sa, sb


class Ref:
    """The reference's own compiled path. bfmt / wfmt: 0 = DF_NORMAL, 1 = DF_TRANSPOSE, 2 = packed."""

    @staticmethod
    def available():
        return os.path.exists(REF_SO) and host_has_vnni()

    def __init__(self, threads=1):
        self.lib = C.CDLL(REF_SO)
        self.lib.ref_requantize.argtypes = [vp, u32, C.c_float, vp, C.c_float]
        self.lib.ref_set_threads(int(threads))

    def axpby(self, a, x, b, y):
        x = np.ascontiguousarray(x, dtype=np.float32)
        out = np.array(y, dtype=np.float32).copy()
        self.lib.ref_axpby_f32.argtypes = [u32, C.c_float, vp, C.c_float, vp]
        assert self.lib.ref_axpby_f32(u32(x.size), C.c_float(a), _p(x), C.c_float(b), _p(out)) == 0
        return out

    def mmm_transform_rhs_bytes(self, bfmt, K, N):
        b, r = u32(0), u32(0)
        e = self.lib.ref_mmm_transform_rhs_bytes(bfmt, u32(K), u32(N), C.byref(b), C.byref(r))
        assert e == 0
        return b.value, r.value

    def mmm_transform_rhs(self, bfmt, K, N, src):
        src = np.ascontiguousarray(src, dtype=np.int8)
        bytes_, rhs = self.mmm_transform_rhs_bytes(bfmt, K, N)
        dst = np.zeros(bytes_, np.uint8)
        d = (u32 * 4)()
        e = self.lib.ref_mmm_transform_rhs(bfmt, u32(K), u32(N), _p(src), _p(dst), d)
        assert e == 0
        return dst, rhs, list(d)

    def mmm_tmp_bytes(self, transA, bfmt, M, K, N):
        b = u32(0)
        e = self.lib.ref_mmm_tmp_bytes(int(transA), bfmt, u32(M), u32(K), u32(N), C.byref(b))
        assert e == 0
        return b.value

    def mmm(self, A, B, bfmt, M, K, N, offsetC, C_in, cdt, scale=None, transA=False):
        """B is raw ([K,N] / [N,K]) or the packed blob from mmm_transform_rhs. `offsetC` is
        copied to the head of tmp as callers of the reference do (fully_connected.cpp:400-406);
        pass None for unpacked B (the on-the-fly transform writes it itself)."""
        A = np.ascontiguousarray(A, dtype=np.uint8)
        B = np.ascontiguousarray(B)
        tmpBytes = self.mmm_tmp_bytes(transA, bfmt, M, K, N) + M * N * 4 + 64
        tmp = np.zeros(tmpBytes, np.uint8)
        if offsetC is not None:
            tmp[:N * 4] = np.ascontiguousarray(offsetC, dtype=np.int32).view(np.uint8)
        out = np.array(C_in, dtype=NP_OF[cdt]).reshape(M, N).copy()
        keep, sp = _scale_arg(scale)
        e = self.lib.ref_mmm(int(transA), bfmt, u32(M), u32(K), u32(N), _p(A), _p(B), u32(tmpBytes),
                             _p(tmp), cdt, _p(out), sp)
        assert e == 0, e
        return out

    def mvm_transform_weight_bytes(self, wfmt, N, K, wdt=DT_I8):
        b = u32(0)
        e = self.lib.ref_mvm_transform_weight_bytes(wfmt, wdt, u32(N), u32(K), C.byref(b))
        assert e == 0
        return b.value

    def mvm_transform_weight(self, wfmt, N, K, src):
        src = np.ascontiguousarray(src, dtype=np.int8)
        dst = np.zeros(self.mvm_transform_weight_bytes(wfmt, N, K) + 64, np.uint8)
        d = (u32 * 4)()
        e = self.lib.ref_mvm_transform_weight(wfmt, u32(N), u32(K), _p(src), _p(dst), d)
        assert e == 0
        return dst, list(d)

    def mvm_tmp_bytes(self, wfmt, N, K, wdt=DT_I8):
        b = u32(0)
        e = self.lib.ref_mvm_tmp_bytes(wfmt, wdt, u32(N), u32(K), C.byref(b))
        assert e == 0
        return b.value

    def mvm(self, W, x, wfmt, N, K, offsetC, y_in, ydt, scale=None, wdt=DT_I8):
        W = np.ascontiguousarray(W)
        x = np.ascontiguousarray(x)
        tmpBytes = self.mvm_tmp_bytes(wfmt, N, K, wdt) + 2 * N * 4 + N * K + 64
        tmp = np.zeros(tmpBytes, np.uint8)
        if offsetC is not None:
            tmp[:N * 4] = np.ascontiguousarray(offsetC, dtype=np.int32).view(np.uint8)
        out = np.array(y_in, dtype=NP_OF[ydt]).reshape(N).copy()
        keep, sp = _scale_arg(scale)
        e = self.lib.ref_mvm(wfmt, wdt, u32(N), u32(K), _p(W), _p(x), u32(tmpBytes), _p(tmp), ydt,
                             _p(out), sp)
        assert e == 0, e
        return out

    def quantize(self, x, ddt, qdt, scale, mode=0, check_overrun=True):
        x = np.ascontiguousarray(x, dtype=NP_OF[ddt])
        q = np.zeros(x.size + 64, NP_OF[qdt])  # slack: detect writes past n
        s = np.array(scale, np.float32).reshape(-1).copy()
        e = self.lib.ref_quantize(ddt, _p(x), u32(x.size), qdt, _p(q), _p(s), int(mode))
        assert e == 0, e
        assert not (check_overrun and q[x.size:].any())
        return q[:x.size].reshape(x.shape), s

    def dequantize(self, q, qdt, scale):
        q = np.ascontiguousarray(q, dtype=NP_OF[qdt])
        out = np.zeros(q.size + 64, np.float32)
        s = np.array([scale], np.float32)
        e = self.lib.ref_dequantize(qdt, _p(q), u32(q.size), _p(s), _p(out))
        assert e == 0, e
        return out[:q.size].reshape(q.shape)

    def bias_offsetC(self, bias, offsetC, scale, packed_filter=True):
        b = None if bias is None else np.ascontiguousarray(bias, dtype=np.float32)
        o = None if offsetC is None else np.ascontiguousarray(offsetC, dtype=np.int32)
        N = b.size if b is not None else o.size
        out = np.zeros(N, np.int32)
        s = np.array([scale], np.float32)
        e = self.lib.ref_quantize_bias_offsetC(_p(b), u32(N), _p(o), int(packed_filter), _p(s), _p(out))
        assert e == 0, e
        return out

    def requantize(self, x, inScale, outScale):
        x = np.ascontiguousarray(x, dtype=np.int8)
        out = np.zeros(x.shape, np.int8)
        e = self.lib.ref_requantize(_p(x), u32(x.size), C.c_float(inScale), _p(out), C.c_float(outScale))
        assert e == 0, e
        return out
