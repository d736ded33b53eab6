"""Python host-side mirror of the reference's convolution call sequence
(compute/tensor/tests/test_convolution_int8.cpp:59-161, inference/engine/include/cpu/convolution_cpu.hpp:454-523):
transform_filter_bytes -> transform_filter -> infer_forward_tmp_bytes -> convolution. numpy buffers use
the host-pointer convention, torch CUDA tensors the device-pointer one. All arithmetic is in
libbolt_gfx950.so."""
import ctypes as C

import numpy as np

from . import capi
from .capi import (ACTIVATION_NULL, ACTIVATION_RELU, CONVOLUTION_ALGORITHM_DIRECT, DF_NCHW, DF_NCHWC8, DF_NCHWC16,
                   DF_NCHWC2NxC4, DT_F32, DT_I8, DT_I32, DT_U8_Q, ActivationParamSpec, TensorDesc, check, conv_param_spec,
                   lib, tensor1d, tensor4df)
from .host import NP_OF, _empty_like_mode, _is_torch, arch_of, ptr


def conv_out_hw(ih, iw, fh, fw, stride, pad, dilation=1):
    oh = (ih + 2 * pad - ((fh - 1) * dilation + 1)) // stride + 1
    ow = (iw + 2 * pad - ((fw - 1) * dilation + 1)) // stride + 1
    return oh, ow


def transform_filter(filt_nchw, oc, ic, fh, fw, p):
    arch = arch_of(filt_nchw)
    fdesc = tensor4df(DT_I8, DF_NCHW, oc, ic, fh, fw)
    b = C.c_uint32(0)
    check(lib().convolution_transform_filter_bytes_gfx950(fdesc, p, CONVOLUTION_ALGORITHM_DIRECT, C.byref(b), arch),
          "conv_filter_bytes")
    blob = _empty_like_mode(filt_nchw, b.value)
    ftm = TensorDesc()
    check(lib().convolution_transform_filter_gfx950(fdesc, ptr(filt_nchw), p, CONVOLUTION_ALGORITHM_DIRECT, C.byref(ftm),
                                                    ptr(blob), arch), "conv_transform_filter")
    return blob, ftm


def convolution(x, idf, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, bias, scale, relu, odt, odf=DF_NCHWC16,
                eltwise=None, dilation=1, tmp=None, out=None):
    """x: u8 activations in `idf`; blob / ftm from transform_filter; scale = [sI, sO, sF] (list, sO updated).
    Returns the output buffer in `odf` order. `tmp` / `out` may be handed in to reuse buffers across calls."""
    arch = arch_of(x)
    p = conv_param_spec(oc, fh, fw, stride, pad, dilation)
    oh, ow = conv_out_hw(ih, iw, fh, fw, stride, pad, dilation)
    idesc = tensor4df(DT_U8_Q, idf, n, ic, ih, iw)
    odesc = tensor4df(odt, odf, n, oc, oh, ow)
    b = C.c_uint32(0)
    check(lib().convolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, CONVOLUTION_ALGORITHM_DIRECT, C.byref(b),
                                                           arch), "conv_tmp_bytes")
    if tmp is None:
        tmp = _empty_like_mode(x, b.value)
    elif (tmp.numel() if _is_torch(tmp) else tmp.nbytes) < b.value:
        raise ValueError("tmp holds %d bytes, the convolution needs %d" % (tmp.numel() if _is_torch(tmp) else tmp.nbytes, b.value))
    count = n * oc * oh * ow
    if out is not None:
        pass
    elif _is_torch(x):
        import torch
        tdt = {DT_F32: torch.float32, DT_I32: torch.int32, DT_U8_Q: torch.uint8}[odt]
        out = torch.zeros(count, dtype=tdt, device=x.device)
    else:
        out = np.zeros(count, NP_OF[odt])
    sarr = (C.c_float * 3)(*[float(np.float32(v)) for v in scale])
    act = ActivationParamSpec()
    act.mode = ACTIVATION_RELU if relu else ACTIVATION_NULL
    e = lib().convolution_gfx950(idesc, ptr(x), ptr(eltwise), ftm, ptr(blob), p, CONVOLUTION_ALGORITHM_DIRECT,
                                 tensor1d(DT_F32, oc), ptr(bias), b.value, ptr(tmp), odesc, ptr(out), sarr, act, arch)
    check(e, "convolution")
    for i in range(3):
        scale[i] = np.float32(sarr[i])
    return out


def _conv_call_setup(x, idf, n, ic, ih, iw, ftm, oc, fh, fw, stride, pad, odt, odf, dilation, tmp, out):
    arch = arch_of(x)
    p = conv_param_spec(oc, fh, fw, stride, pad, dilation)
    oh, ow = conv_out_hw(ih, iw, fh, fw, stride, pad, dilation)
    idesc = tensor4df(DT_U8_Q, idf, n, ic, ih, iw)
    odesc = tensor4df(odt, odf, n, oc, oh, ow)
    b = C.c_uint32(0)
    check(lib().convolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, CONVOLUTION_ALGORITHM_DIRECT, C.byref(b),
                                                           arch), "conv_tmp_bytes")
    if tmp is None:
        tmp = _empty_like_mode(x, b.value)
    elif (tmp.numel() if _is_torch(tmp) else tmp.nbytes) < b.value:
        raise ValueError("tmp holds %d bytes, the convolution needs %d" % (tmp.numel() if _is_torch(tmp) else tmp.nbytes, b.value))
    count = n * oc * oh * ow
    if out is not None:
        pass
    elif _is_torch(x):
        import torch
        tdt = {DT_F32: torch.float32, DT_I32: torch.int32, DT_U8_Q: torch.uint8}[odt]
        out = torch.zeros(count, dtype=tdt, device=x.device)
    else:
        out = np.zeros(count, NP_OF[odt])
    return arch, p, idesc, odesc, b.value, tmp, out


def convolution_perchannel(x, idf, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, scale_w, bias, scale, relu, odt,
                           odf=DF_NCHWC16, eltwise=None, dilation=1, tmp=None, out=None):
    """The int8 convolution with one filter scale per output channel (bolt_gfx950_convolution_int8_perchannel; not in
    the reference). scale_w: fp32 [oc]; bias: fp32 [oc] or None; scale = [sI, sO] (list): sO > 0 on entry = static u8
    output scale, else dynamic and updated. odt: DT_F32 or DT_U8_Q."""
    arch, p, idesc, odesc, nbytes, tmp, out = _conv_call_setup(x, idf, n, ic, ih, iw, ftm, oc, fh, fw, stride, pad, odt, odf,
                                                               dilation, tmp, out)
    sarr = (C.c_float * 2)(*[float(np.float32(v)) for v in scale])
    act = ActivationParamSpec()
    act.mode = ACTIVATION_RELU if relu else ACTIVATION_NULL
    e = lib().bolt_gfx950_convolution_int8_perchannel(idesc, ptr(x), ptr(eltwise), ftm, ptr(blob), p, ptr(scale_w),
                                                      tensor1d(DT_F32, oc), ptr(bias), nbytes, ptr(tmp), odesc, ptr(out),
                                                      sarr, act, arch)
    check(e, "convolution_perchannel")
    for i in range(2):
        scale[i] = np.float32(sarr[i])
    return out


def convolution_async(x, idf, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, bias, dscale_in, filter_scale, scale_w,
                      dscale_out, relu, odt, odf=DF_NCHWC16, static_out=0.0, eltwise=None, dilation=1, tmp=None, out=None,
                      one_pass_room=True):
    """bolt_gfx950_convolution_async: device tensors only; dscale_in / dscale_out are one-element fp32 device tensors
    (input scale read, output scale left there); scale_w None = one filter scale `filter_scale`, else fp32 [oc] device.
    one_pass_room: hand over a tmp of bolt_gfx950_convolution_async_tmp_bytes (a dynamic u8 result may then run in one
    pass) instead of the synchronous call's size (always two passes)."""
    arch, p, idesc, odesc, nbytes, tmp, out = _conv_call_setup(x, idf, n, ic, ih, iw, ftm, oc, fh, fw, stride, pad, odt, odf,
                                                               dilation, tmp, out)
    if one_pass_room:
        b = C.c_uint32(0)
        check(lib().bolt_gfx950_convolution_async_tmp_bytes(idesc, ftm, odesc, p, C.byref(b)), "conv_async_tmp_bytes")
        if tmp.numel() < b.value:
            tmp = _empty_like_mode(x, b.value)
        nbytes = b.value
    act = ActivationParamSpec()
    act.mode = ACTIVATION_RELU if relu else ACTIVATION_NULL
    e = lib().bolt_gfx950_convolution_async(idesc, ptr(x), ptr(eltwise), ftm, ptr(blob), p, tensor1d(DT_F32, oc), ptr(bias),
                                            nbytes, ptr(tmp), odesc, ptr(out), ptr(dscale_in), float(filter_scale),
                                            ptr(scale_w), ptr(dscale_out), float(static_out), act)
    check(e, "convolution_async")
    return out


def bnn_transform_filter(filt_bits, fdt, fdf, oc, ic, fh, fw):
    """1-bit filter (DF_NCHW bit string or DF_NCHWN16C8 bytes) -> this library's blob
    (compute/tensor/src/cpu/arm/bnn/convolution_transform_bnn.h:32-86)."""
    arch = arch_of(filt_bits)
    fdesc = tensor4df(fdt, fdf, oc, ic, fh, fw)
    b = C.c_uint32(0)
    check(lib().convolution_transform_filter_bytes_bnn_gfx950(fdesc, C.byref(b), arch), "bnn_filter_bytes")
    blob = _empty_like_mode(filt_bits, b.value)
    ftm = TensorDesc()
    check(lib().convolution_transform_filter_bnn_gfx950(fdesc, ptr(filt_bits), C.byref(ftm), ptr(blob), arch),
          "bnn_transform_filter")
    return blob, ftm


def bnn_tmp_bytes(idt, n, ic, ih, iw, oc, fh, fw, stride, pad, like):
    """Bytes of tmp convolution_bnn needs for this shape (`like` selects host or device pointers)."""
    b = C.c_uint32(0)
    check(lib().convolution_infer_forward_tmp_bytes_bnn_gfx950(tensor4df(idt, DF_NCHWC8, n, ic, ih, iw),
                                                               conv_param_spec(oc, fh, fw, stride, pad), C.byref(b),
                                                               arch_of(like)), "bnn_tmp_bytes")
    return b.value


def convolution_bnn(x, idt, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, scale, bias, odt=DT_F32, tmp=None,
                    out=None):
    """x: fp32 NCHWC8 activations (idt = DT_F32) or packed bits (idt = the filter's type); scale / bias fp32 [oc].
    Mirrors convolution_bnn (compute/tensor/src/cpu/arm/bnn/convolution.cpp:16-72). Output NCHWC8."""
    arch = arch_of(x)
    p = conv_param_spec(oc, fh, fw, stride, pad)
    oh, ow = conv_out_hw(ih, iw, fh, fw, stride, pad)
    idesc = tensor4df(idt, DF_NCHWC8, n, ic, ih, iw)
    odesc = tensor4df(odt, DF_NCHWC8, n, oc, oh, ow)
    b = C.c_uint32(0)
    check(lib().convolution_infer_forward_tmp_bytes_bnn_gfx950(idesc, p, C.byref(b), arch), "bnn_tmp_bytes")
    if tmp is None:
        tmp = _empty_like_mode(x, b.value)
    elif (tmp.numel() if _is_torch(tmp) else tmp.nbytes) < b.value:
        raise ValueError("tmp holds %d bytes, the convolution needs %d" % (tmp.numel() if _is_torch(tmp) else tmp.nbytes, b.value))
    count = n * oc * oh * ow
    if out is not None:
        pass
    elif _is_torch(x):
        import torch
        out = torch.zeros(count, dtype={DT_F32: torch.float32, DT_I32: torch.int32}[odt], device=x.device)
    else:
        out = np.zeros(count, NP_OF[odt])
    act = ActivationParamSpec()
    act.mode = ACTIVATION_NULL
    e = lib().convolution_bnn_gfx950(idesc, ptr(x), ftm, ptr(blob), p, tensor1d(DT_F32, oc), ptr(scale),
                                     tensor1d(DT_F32, oc), ptr(bias), b.value, ptr(tmp), odesc, ptr(out), act, arch)
    check(e, "convolution_bnn")
    return out


def depthwise_transform_filter(filt_chw, c, fh, fw):
    """filt_chw: s8 [c][fh][fw] (the reference's [1, c, fh, fw] DF_NCHW). Returns (blob, ftm desc)."""
    arch = arch_of(filt_chw)
    fdesc = tensor4df(DT_I8, DF_NCHW, 1, c, fh, fw)
    b = C.c_uint32(0)
    check(lib().depthwise_convolution_transform_filter_bytes_int8_gfx950(fdesc, C.byref(b), arch), "dw_filter_bytes")
    blob = _empty_like_mode(filt_chw, b.value)
    ftm = TensorDesc()
    check(lib().depthwise_convolution_transform_filter_int8_gfx950(fdesc, ptr(filt_chw), C.byref(ftm), ptr(blob), arch),
          "dw_transform_filter")
    return blob, ftm


def depthwise_convolution_i32(x, n, c, ih, iw, blob, ftm, fh, fw, stride, bias, scale, relu, pad=0, out=None):
    """x: u8 NCHWC16. Returns int32 NCHWC16; scale = [sI, sO, sF] (sO written)."""
    arch = arch_of(x)
    p = conv_param_spec(c, fh, fw, stride, pad, 1, group=c)
    oh, ow = conv_out_hw(ih, iw, fh, fw, stride, pad)
    idesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, c, ih, iw)
    odesc = tensor4df(DT_I32, DF_NCHWC16, n, c, oh, ow)
    count = n * c * oh * ow
    if out is not None:
        pass
    elif _is_torch(x):
        import torch
        out = torch.zeros(count, dtype=torch.int32, device=x.device)
    else:
        out = np.zeros(count, np.int32)
    sarr = (C.c_float * 3)(*[float(np.float32(v)) for v in scale])
    act, none = ActivationParamSpec(), ActivationParamSpec()
    act.mode = ACTIVATION_RELU if relu else ACTIVATION_NULL
    none.mode = ACTIVATION_NULL
    blank = TensorDesc()
    e = lib().depthwise_pointwise_convolution_int8_gfx950(idesc, ptr(x), None, ftm, ptr(blob), blank, None, p,
                                                          tensor1d(DT_F32, c), ptr(bias), blank, None, 0, None, odesc,
                                                          ptr(out), sarr, act, none, arch)
    check(e, "depthwise_convolution")
    for i in range(3):
        scale[i] = np.float32(sarr[i])
    return out
