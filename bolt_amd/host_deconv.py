"""Python host-side mirror of the reference's deconvolution call sequence
(inference/engine/include/cpu/deconvolution_cpu.hpp:56-100,139-213): infer_output_size -> infer_forward_algorithm ->
transform_filter_bytes -> transform_filter -> infer_forward_tmp_bytes -> deconvolution. numpy buffers use the
host-pointer convention, torch CUDA tensors the device-pointer one. All arithmetic is in libbolt_gfx950.so."""
import ctypes as C

import numpy as np

from . import capi
from .capi import (ACTIVATION_NULL, ACTIVATION_RELU, CONVOLUTION_ALGORITHM_NULL, DF_NCHW, DT_F32, DT_I8, DT_U8_Q,
                   ActivationParamSpec, ConvolutionParamSpec, TensorDesc, check, lib, tensor1d, tensor4df)
from .host import NP_OF, _empty_like_mode, _is_torch, arch_of, ptr


def deconv_param_spec(oc, fh, fw, sh, sw, pt, pb, pl, pr):
    """createConvolutionParamSpec (parameter_spec.h:878-920) for a 2-D deconvolution."""
    p = ConvolutionParamSpec()
    p.num_outputs, p.kernel_t, p.kernel_h, p.kernel_w = oc, 1, fh, fw
    p.stride_t, p.stride_h, p.stride_w = 1, sh, sw
    p.pad_top, p.pad_bottom, p.pad_left, p.pad_right = pt, pb, pl, pr
    p.group, p.dilatedRate_t, p.dilatedRate_h, p.dilatedRate_w = 1, 1, 1, 1
    p.num_outputs_origin = oc
    p.convolution_type = 4  # CONVOLUTION_DECONVOLUTION
    return p


def plan(x, idf, n, ic, ih, iw, oc, fh, fw, p, odt):
    """Output desc and forward algorithm for a u8 input in `idf`."""
    arch = arch_of(x)
    idesc = tensor4df(DT_U8_Q, idf, n, ic, ih, iw)
    fdesc = tensor4df(DT_I8, DF_NCHW, ic, oc, fh, fw)
    odesc = TensorDesc()
    check(lib().deconvolution_infer_output_size_gfx950(idesc, fdesc, p, C.byref(odesc), odt, arch), "deconv_output_size")
    alg = C.c_int(CONVOLUTION_ALGORITHM_NULL)
    check(lib().deconvolution_infer_forward_algorithm_gfx950(idesc, fdesc, odesc, p, 0, C.byref(alg), odt, arch),
          "deconv_algorithm")
    return idesc, fdesc, odesc, alg.value


def transform_filter(filt, fdesc, p, alg):
    """filt: s8 [ic][oc][fh][fw]. Returns (blob, ftm desc, bytes the query asked for)."""
    arch = arch_of(filt)
    b = C.c_uint32(0)
    check(lib().deconvolution_transform_filter_bytes_gfx950(fdesc, p, alg, C.byref(b), arch), "deconv_filter_bytes")
    blob = _empty_like_mode(filt, b.value)
    ftm = TensorDesc()
    check(lib().deconvolution_transform_filter_gfx950(fdesc, ptr(filt), p, alg, C.byref(ftm), ptr(blob), arch),
          "deconv_transform_filter")
    return blob, ftm, b.value


def deconvolution(x, idesc, blob, ftm, p, alg, bias, scale, relu, odesc, tmp=None, out=None):
    """scale = [sI, sO, sF] (list, left as the call leaves the caller's array). Returns the output buffer (NCHWC16)."""
    arch = arch_of(x)
    b = C.c_uint32(0)
    check(lib().deconvolution_infer_forward_tmp_bytes_gfx950(idesc, ftm, odesc, p, alg, C.byref(b), arch), "deconv_tmp_bytes")
    if tmp is None:
        tmp = _empty_like_mode(x, b.value)
    count = 1
    for i in range(odesc.nDims):
        count *= odesc.dims[i]
    odt = odesc.dt
    if out is not None:
        pass
    elif _is_torch(x):
        import torch
        out = torch.zeros(count, dtype={DT_F32: torch.float32, DT_U8_Q: torch.uint8}[odt], device=x.device)
    else:
        out = np.zeros(count, NP_OF[odt])
    sarr = (C.c_float * 3)(*[float(np.float32(v)) for v in scale])
    act = ActivationParamSpec()
    act.mode = ACTIVATION_RELU if relu else ACTIVATION_NULL
    e = lib().deconvolution_gfx950(idesc, ptr(x), ftm, ptr(blob), p, alg, ftm, C.cast(sarr, C.c_void_p), tensor1d(DT_F32, p.num_outputs),
                                   ptr(bias), b.value, ptr(tmp), odesc, ptr(out), act, arch)
    check(e, "deconvolution")
    for i in range(3):
        scale[i] = np.float32(sarr[i])
    return out
