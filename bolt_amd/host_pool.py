"""Host-side mirror of Bolt's quantised pooling and concatenation calls over the C-ABI
(compute/tensor/src/pooling.cpp:150-200, compute/tensor/src/concat.cpp:160-205). Buffers are numpy arrays
(host pointers, synchronous) or torch CUDA tensors (device pointers, asynchronous on the library stream).
All arithmetic happens in libbolt_gfx950.so."""
import ctypes as C

import numpy as np

from . import capi
from .capi import DF_NCHWC16, DT_I8, DT_U8_Q, TensorDesc, check, lib, tensor4df
from .host import _empty_like_mode, _is_torch, arch_of, ptr


def pooling_out_hw(ih, iw, p, ceil=True):
    """pooling_infer_output_size for ROUND_CEIL / ROUND_FLOOR (compute/tensor/src/pooling.cpp:37-85)."""
    def one(i, k, s, a, b):
        v = (i + a + b - k) / s
        return int(np.ceil(v) if ceil else np.floor(v)) + 1
    return (one(ih, p.kernel_h, p.stride_h, p.pad_top, p.pad_bottom),
            one(iw, p.kernel_w, p.stride_w, p.pad_left, p.pad_right))


def pooling_u8(x, n, c, ih, iw, p, in_scale, oh, ow, out=None):
    """x: u8 NCHWC16. Returns (u8 NCHWC16 output, output scale)."""
    idesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, ih, iw)
    odesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, oh, ow)
    if out is None:
        out = _empty_like_mode(x, n * c * oh * ow)
    sc = (C.c_float * 2)(float(np.float32(in_scale)), 0.0)
    check(lib().pooling_gfx950(idesc, ptr(x), p, C.cast(sc, C.c_void_p), odesc, ptr(out), None, arch_of(x)), "pooling")
    return out, np.float32(sc[1])


def concat(inputs, descs, axis, out_desc, scales=None, out=None):
    """inputs: buffers all in host or all in device memory; descs: their TensorDesc. Returns (output, output scale
    or None)."""
    num = len(inputs)
    like = next(t for t in inputs if t is not None)
    if out is None:
        out = _empty_like_mode(like, capi.tensor_num_bytes(out_desc))
    darr = (TensorDesc * max(num, 1))(*descs)
    parr = (C.c_void_p * max(num, 1))(*[None if t is None else ptr(t).value for t in inputs])
    sarr = osc = None
    if scales is not None:
        sarr = (C.c_float * max(num, 1))(*[float(np.float32(s)) for s in scales])
        osc = C.c_float(0.0)
    p = capi.ConcatParamSpec(axis, num)
    check(lib().concat_gfx950(num, darr, parr, sarr, p, None, out_desc, ptr(out),
                              None if osc is None else C.byref(osc), arch_of(like)), "concat")
    return out, (None if osc is None else np.float32(osc.value))
