"""Host-side mirror of Bolt's int8 LSTM cell call (compute/tensor/src/rnn.cpp -> rnncell_int8,
compute/tensor/src/cpu/x86/int8/rnn.cpp:16-44) over the C-ABI. Buffers are numpy arrays (host pointers) or torch
CUDA tensors (device pointers, asynchronous). All arithmetic happens in libbolt_gfx950.so."""
import ctypes as C

import numpy as np

from . import capi, host
from .capi import (ACTIVATION_TANH, DF_NKN32, DF_NKNx_NKN32, DF_NORMAL, DT_F32, DT_I8, RNN_LSTM, RNNParamSpec, TensorDesc, check, lib,
                   tensor1d, tensor2df)
from .host import _empty_like_mode, arch_of, ptr


def lstm_param_spec(hdim, forget_bias=1.0, zoneout_cell=0.0, zoneout_output=0.0, bi_direction=False, num_projection=0):
    p = RNNParamSpec()
    p.mode, p.num_outputs, p.steps, p.num_projection = RNN_LSTM, hdim, -1, num_projection
    p.zoneout_cell, p.zoneout_output, p.bi_direction = zoneout_cell, zoneout_output, bool(bi_direction)
    p.forget_bias, p.activation_type = forget_bias, ACTIVATION_TANH
    return p


def transform_weight(W, N, K):
    """s8 [N][K] -> this library's matrix-vector blob (packed rows + compensation vector)."""
    blob, _ = host.mvm_transform_weight(W, DF_NORMAL, N, K)
    return blob


def rnn_transform_filter(W, N, K, p):
    """s8 [N][K] -> blob tagged DF_NKNx_NKN32: the matrix-vector blob followed by the GEMM packing."""
    arch = arch_of(W)
    desc = tensor2df(DT_I8, DF_NORMAL, N, K)
    nbytes = C.c_uint32(0)
    check(lib().rnn_transform_filter_bytes_gfx950(desc, p, C.byref(nbytes), arch), "rnn_transform_filter_bytes")
    blob = _empty_like_mode(W, nbytes.value)
    ftm = TensorDesc()
    check(lib().rnn_transform_filter_gfx950(desc, ptr(W), p, C.byref(ftm), ptr(blob), arch), "rnn_transform_filter")
    assert ftm.df == DF_NKNx_NKN32
    return blob


def lstmcell(x, blob, bias, scale, state, p, batch, xdim, out, x_stride=None, out_stride=None, tmp=None, fshape=None, both_packings=False,
             proj=None):
    """One step for `batch` rows; `state` ([batch][C | H]) and `out` are updated in place. fshape: (rows, cols) the
    filter descriptor declares, by default what `p` and xdim imply; both_packings: `blob` comes from
    rnn_transform_filter; proj: with p.num_projection > 0 the fp32 projection matrix in the DF_NKN32 layout
    [num_outputs / 32][num_projection][32] (lstm.cpp:170-173)."""
    hdim = p.num_outputs
    column = p.num_projection if p.num_projection > 0 else hdim
    x_stride = xdim if x_stride is None else x_stride
    out_stride = hdim if out_stride is None else out_stride
    xdesc = tensor2df(DT_F32, DF_NORMAL, batch, xdim)
    hdesc = tensor2df(DT_F32, DF_NORMAL, batch, hdim)
    frows, fcols = fshape or (4 * column, xdim + hdim)
    fdesc = (TensorDesc * 2)(tensor2df(DT_I8, DF_NKNx_NKN32 if both_packings else DF_NKN32, frows, fcols),
                             tensor2df(DT_F32, DF_NKN32, hdim, column))
    bdesc = (TensorDesc * 1)(tensor1d(DT_F32, 4 * column))
    arch = arch_of(state)
    nbytes = C.c_uint32(0)
    check(lib().rnncell_infer_forward_tmp_bytes_gfx950(xdesc, fdesc[0], hdesc, p, C.byref(nbytes), arch), "rnncell tmp")
    if tmp is None:
        tmp = _empty_like_mode(state, nbytes.value)
    filt = (C.c_void_p * 2)(ptr(blob).value, ptr(proj).value if proj is not None else None)
    biases = (C.c_void_p * 2)(ptr(bias).value, None)
    sc = (C.c_float * 2)(float(np.float32(scale[0])), float(np.float32(scale[1])))
    check(lib().rnncell_gfx950(xdesc, ptr(x), fdesc, filt, bdesc, biases, sc, ptr(state), nbytes.value, ptr(tmp), p,
                               x_stride, out_stride, hdesc, ptr(out), arch), "rnncell")
    return out
