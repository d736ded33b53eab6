"""Python host-side mirror of Bolt's blas_enhance / tensor_computing call sequences over the C-ABI.

Buffers are numpy arrays (Arch AMD_GFX950: host pointers, synchronous) or torch CUDA tensors
(Arch AMD_GFX950_DEVICE: device pointers, asynchronous on the library stream). The functions keep
the reference's calling order: size query -> transform -> copy offsetC to the head of tmp -> multiply
(compute/blas_enhance/tests/test_mmm.cpp:64-100, compute/tensor/src/fully_connected.cpp:396-475).
All arithmetic happens in libbolt_gfx950.so.
"""
import ctypes as C

import numpy as np

from . import capi
from .capi import (AMD_GFX950, AMD_GFX950_DEVICE, DF_NKN32K4, DF_NKNxKx, DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I8,
                   DT_I32, DT_U8_Q, TensorDesc, check, lib, tensor1d, tensor2df)

NP_OF = {DT_I8: np.int8, DT_I32: np.int32, DT_F32: np.float32, DT_U8_Q: np.uint8}


def _is_torch(t):
    return hasattr(t, "data_ptr")


def ptr(t):
    if t is None:
        return None
    if _is_torch(t):
        return C.c_void_p(t.data_ptr())
    return t.ctypes.data_as(C.c_void_p)


def arch_of(t):
    return AMD_GFX950_DEVICE if _is_torch(t) else AMD_GFX950


def _empty_like_mode(like, nbytes):
    """uint8 buffer of nbytes in the same memory space as `like`."""
    if _is_torch(like):
        import torch
        return torch.zeros(nbytes, dtype=torch.uint8, device=like.device)
    return np.zeros(nbytes, np.uint8)


def _scale_ptr(scale):
    if scale is None:
        return None, None
    arr = (C.c_float * len(scale))(*[float(np.float32(s)) for s in scale])
    return arr, C.cast(arr, C.c_void_p)


def _u32():
    return C.c_uint32(0)


# ---- GEMM -------------------------------------------------------------------------------------------
def rhs_desc(df, K, N):
    if df == DF_TRANSPOSE:
        return tensor2df(DT_I8, DF_TRANSPOSE, N, K)
    return tensor2df(DT_I8, df, K, N)


def mmm_transform_rhs_bytes(desc, arch=AMD_GFX950):
    b, r = _u32(), _u32()
    check(lib().matrix_matrix_multiply_transform_rhs_bytes_gfx950(desc, C.byref(b), C.byref(r), arch), "rhs_bytes")
    return b.value, r.value


def mmm_transform_rhs(W, df, K, N):
    """W: s8 [K,N] (DF_NORMAL) or [N,K] (DF_TRANSPOSE). Returns (blob, descTran, offset of offsetC)."""
    arch = arch_of(W)
    desc = rhs_desc(df, K, N)
    total, rhs = mmm_transform_rhs_bytes(desc, arch)
    blob = _empty_like_mode(W, total)
    dt = TensorDesc()
    check(lib().matrix_matrix_multiply_transform_rhs_gfx950(desc, ptr(W), C.byref(dt), ptr(blob), arch), "transform_rhs")
    return blob, dt, rhs


def mmm_tmp_bytes(adesc, bdesc, arch=AMD_GFX950):
    b = _u32()
    check(lib().matrix_matrix_multiply_tmp_bytes_gfx950(adesc, bdesc, C.byref(b), arch), "mmm_tmp_bytes")
    return b.value


def matrix_matrix_multiply(A, adesc, B, bdesc, tmp, Cbuf, cdesc, scale=None):
    arch = arch_of(A)
    keep, sp = _scale_ptr(scale)
    nbytes = tmp.numel() if _is_torch(tmp) else tmp.nbytes
    return lib().matrix_matrix_multiply_gfx950(adesc, ptr(A), bdesc, ptr(B), nbytes, ptr(tmp), cdesc, ptr(Cbuf), sp,
                                               arch)


# ---- GEMV -------------------------------------------------------------------------------------------
def mvm_desc(df, N, K, dt=DT_I8):
    if df == DF_TRANSPOSE:
        return tensor2df(dt, DF_TRANSPOSE, K, N)
    return tensor2df(dt, df, N, K)


def mvm_transform_weight_bytes(desc, arch=AMD_GFX950):
    b = _u32()
    check(lib().matrix_vector_multiply_transform_weight_bytes_gfx950(desc, C.byref(b), arch), "weight_bytes")
    return b.value


def mvm_transform_weight(W, df, N, K):
    arch = arch_of(W)
    desc = mvm_desc(df, N, K)
    total = mvm_transform_weight_bytes(desc, arch)
    blob = _empty_like_mode(W, total)
    dt = TensorDesc()
    check(lib().matrix_vector_multiply_transform_weight_gfx950(desc, ptr(W), C.byref(dt), ptr(blob), arch),
          "transform_weight")
    return blob, dt


def mvm_tmp_bytes(mdesc, vdesc, arch=AMD_GFX950):
    b = _u32()
    check(lib().matrix_vector_multiply_tmp_bytes_gfx950(mdesc, vdesc, C.byref(b), arch), "mvm_tmp_bytes")
    return b.value


def matrix_vector_multiply(W, mdesc, x, vdesc, tmp, y, rdesc, scale=None):
    arch = arch_of(x)
    keep, sp = _scale_ptr(scale)
    nbytes = 0 if tmp is None else (tmp.numel() if _is_torch(tmp) else tmp.nbytes)
    return lib().matrix_vector_multiply_gfx950(mdesc, ptr(W), vdesc, ptr(x), nbytes, ptr(tmp), rdesc, ptr(y), sp, arch)


# ---- quantize family ----------------------------------------------------------------------------------
def quantize(x, ddt, qdt, scale, mode=0, out=None):
    """scale: list of 1 (F32 input) or 2 (I32 input) floats, updated in place like the reference's F32*."""
    arch = arch_of(x)
    n = x.numel() if _is_torch(x) else x.size
    if out is None:
        if _is_torch(x):
            import torch
            out = torch.empty(n, dtype=torch.int8 if qdt == DT_I8 else torch.uint8, device=x.device)
        else:
            out = np.empty(n, NP_OF[qdt])
    sarr = (C.c_float * max(2, len(scale)))(*[float(np.float32(s)) for s in scale])
    qd = tensor1d(qdt, n)
    e = lib().quantize_gfx950(tensor1d(ddt, n), ptr(x), C.byref(qd), ptr(out), C.cast(sarr, C.c_void_p), mode, arch)
    check(e, "quantize")
    for i in range(len(scale)):
        scale[i] = np.float32(sarr[i])
    return out


def dequantize(q, qdt, scale, out=None):
    arch = arch_of(q)
    n = q.numel() if _is_torch(q) else q.size
    if out is None:
        if _is_torch(q):
            import torch
            out = torch.empty(n, dtype=torch.float32, device=q.device)
        else:
            out = np.empty(n, np.float32)
    s = (C.c_float * 1)(float(np.float32(scale)))
    e = lib().dequantize_gfx950(tensor1d(qdt, n), ptr(q), C.cast(s, C.c_void_p), tensor1d(DT_F32, 0), None,
                                tensor1d(DT_F32, n), ptr(out), arch)
    check(e, "dequantize")
    return out


def quantize_bias_offsetC(bias, offsetC, scale, N, packed_filter=True, like=None):
    like = bias if bias is not None else offsetC
    arch = arch_of(like)
    if _is_torch(like):
        import torch
        out = torch.empty(N, dtype=torch.int32, device=like.device)
    else:
        out = np.empty(N, np.int32)
    s = (C.c_float * 1)(float(np.float32(scale)))
    fdesc = tensor2df(DT_I8, DF_NKNxKx if packed_filter else DF_NORMAL, N, N)
    e = lib().quantize_bias_offsetC_gfx950(ptr(bias), tensor1d(DT_F32, N if bias is not None else 0), DT_I32,
                                           ptr(offsetC), fdesc, C.cast(s, C.c_void_p), ptr(out), arch)
    check(e, "quantize_bias_offsetC")
    return out


def requantize(x, inScale, outScale):
    arch = arch_of(x)
    n = x.numel() if _is_torch(x) else x.size
    if _is_torch(x):
        import torch
        out = torch.empty_like(x)
    else:
        out = np.empty_like(x)
    d = tensor1d(DT_I8, n)
    check(lib().requantize_gfx950(d, ptr(x), float(np.float32(inScale)), d, ptr(out), float(np.float32(outScale)), arch),
          "requantize")
    return out


# ---- int8 FullyConnected ------------------------------------------------------------------------------
def fully_connected_tmp_bytes(M, K, N, fdf, odt, arch=AMD_GFX950):
    b = _u32()
    idesc = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
    fdesc = tensor2df(DT_I8, fdf, K, N) if fdf == DF_NKNxKx else tensor2df(DT_I8, fdf, N, K)
    check(lib().fully_connected_infer_forward_tmp_bytes_gfx950(idesc, fdesc, tensor2df(odt, DF_NORMAL, M, N),
                                                               C.byref(b), arch), "fc_tmp_bytes")
    return b.value


def fully_connected(x, scaleI, filt, fdf, scaleW, bias, M, K, N, odt, scaleO=-1.0):
    """x: u8 [M,K]; filt: packed blob from mmm_transform_rhs (fdf DF_NKNxKx) or mvm_transform_weight
    (fdf DF_NKN32K4). Returns (output, output scale) like the reference's outputTensor / get_scale()."""
    arch = arch_of(x)
    nbytes = fully_connected_tmp_bytes(M, K, N, fdf, odt, arch)
    tmp = _empty_like_mode(x, nbytes)
    if _is_torch(x):
        import torch
        tdt = {DT_F32: torch.float32, DT_I32: torch.int32, DT_U8_Q: torch.uint8}[odt]
        out = torch.zeros((M, N), dtype=tdt, device=x.device)
    else:
        out = np.zeros((M, N), NP_OF[odt])
    so = C.c_float(float(np.float32(scaleO)))
    idesc = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
    fdesc = tensor2df(DT_I8, fdf, K, N) if fdf == DF_NKNxKx else tensor2df(DT_I8, fdf, N, K)
    e = lib().fully_connected_gfx950(idesc, ptr(x), float(np.float32(scaleI)), fdesc, ptr(filt),
                                     float(np.float32(scaleW)), tensor1d(DT_F32, N), ptr(bias), nbytes, ptr(tmp),
                                     tensor2df(odt, DF_NORMAL, M, N), ptr(out), C.byref(so), arch)
    check(e, "fully_connected")
    return out, np.float32(so.value)


# ---- int8 matmul ------------------------------------------------------------------------------------------
def tensor_nd(dt, shape):
    """TensorDesc for a row-major array of `shape` (outermost first), DF_NCHW like the reference's matmul operands."""
    d = TensorDesc()
    d.dt, d.df, d.nDims = dt, 0, len(shape)
    for i, v in enumerate(reversed(shape)):
        d.dims[i] = v
    return d


def matmul(A, adt, a_shape, transposeA, scaleA, B, bdt, b_shape, transposeB, scaleB, c_shape, cdt=DT_F32):
    """Mirrors matmul (compute/tensor/src/matmul.cpp:302-576, x86 int8 branch). Shapes are the stored ones."""
    arch = arch_of(A)
    ad, bd, cd = tensor_nd(adt, a_shape), tensor_nd(bdt, b_shape), tensor_nd(cdt, c_shape)
    nb = _u32()
    check(lib().matmul_infer_forward_tmp_bytes_gfx950(ad, bool(transposeA), bd, bool(transposeB), cd, C.byref(nb), arch),
          "matmul_tmp_bytes")
    tmp = _empty_like_mode(A, nb.value)
    count = int(np.prod(c_shape))
    if _is_torch(A):
        import torch
        out = torch.zeros(count, dtype=torch.float32 if cdt == DT_F32 else torch.int32, device=A.device)
    else:
        out = np.zeros(count, NP_OF[cdt])
    check(lib().matmul_gfx950(ad, bool(transposeA), ptr(A), float(np.float32(scaleA)), bd, bool(transposeB), ptr(B),
                              float(np.float32(scaleB)), nb.value, ptr(tmp), cd, ptr(out), arch), "matmul")
    return out
