"""ctypes bindings for the LSTM-cell parts of the CPU checkers (test infrastructure only)."""
import ctypes as C

import numpy as np

from checkers import _p, u32, vp

f32 = C.c_float


def orc_lstmcell(oracle, x, W, bias, scale, state, hdim, forget_bias=1.0, zc=0.0, zo=0.0, x_stride=None, bias_stride=None,
                 out_stride=None):
    """x [batch][x_stride], W s8 [4h][xdim+h], state [batch][2h] (copied). Returns (out, new state)."""
    batch = state.shape[0]
    xdim = W.shape[1] - hdim
    x_stride = xdim if x_stride is None else x_stride
    bias_stride = 4 * hdim if bias_stride is None else bias_stride
    out_stride = hdim if out_stride is None else out_stride
    L = oracle.lib
    L.orc_lstmcell_int8.argtypes = [u32, u32, u32, vp, u32, vp, vp, u32, vp, vp, f32, f32, f32, vp, u32]
    L.orc_lstmcell_int8.restype = None
    st = np.array(state, np.float32, copy=True)
    out = np.zeros((batch, out_stride), np.float32)
    sc = np.array(scale, np.float32)
    L.orc_lstmcell_int8(batch, xdim, hdim, _p(x), x_stride, _p(W), _p(bias), bias_stride, _p(sc), _p(st), forget_bias, zc,
                        zo, _p(out), out_stride)
    return out, st


def ref_lstmcell(ref, x, W, bias, scale, state, hdim, forget_bias=1.0, zc=0.0, zo=0.0, x_stride=None, out_stride=None):
    batch = state.shape[0]
    xdim = W.shape[1] - hdim
    x_stride = xdim if x_stride is None else x_stride
    out_stride = hdim if out_stride is None else out_stride
    L = ref.lib
    L.ref_lstmcell_int8.argtypes = [u32, u32, u32, vp, u32, vp, vp, vp, vp, f32, f32, f32, vp, u32]
    st = np.array(state, np.float32, copy=True)
    out = np.zeros((batch, out_stride), np.float32)
    sc = np.array(scale, np.float32)
    e = L.ref_lstmcell_int8(batch, xdim, hdim, _p(x), x_stride, _p(W), _p(bias), _p(sc), _p(st), forget_bias, zc, zo,
                            _p(out), out_stride)
    assert e == 0, e
    return out, st


def lstm_case(batch, xdim, hdim, seed, x_stride=None, bias_rows=None, bias_stride=None):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((batch, x_stride or xdim)).astype(np.float32)
    W = rng.integers(-127, 128, size=(4 * hdim, xdim + hdim), dtype=np.int8)
    rows = batch if bias_rows is None else bias_rows
    bias = (rng.standard_normal((rows, bias_stride or 4 * hdim)) * 0.5).astype(np.float32)
    state = (rng.standard_normal((batch, 2 * hdim)) * 0.7).astype(np.float32)
    return x, W, bias, state


def nkn32(Wp):
    """fp32 projection matrix [hdim][column] -> the DF_NKN32 layout the cell reads, [hdim / 32][column][32]"""
    hdim, column = Wp.shape
    return np.ascontiguousarray(Wp.reshape(hdim // 32, 32, column).transpose(0, 2, 1)).reshape(-1)


def orc_lstmcell_proj(oracle, x, W, Wp, bias, scale, state, hdim, column, forget_bias=1.0, zc=0.0, zo=0.0):
    """With a projection: W s8 [4 * column][xdim + hdim], Wp fp32 [hdim][column], state [batch][column + hdim]."""
    batch = state.shape[0]
    xdim = W.shape[1] - hdim
    L = oracle.lib
    L.orc_lstmcell_int8_proj.argtypes = [u32, u32, u32, u32, vp, u32, vp, vp, vp, u32, vp, vp, f32, f32, f32, vp, u32]
    L.orc_lstmcell_int8_proj.restype = None
    st = np.array(state, np.float32, copy=True)
    out = np.zeros((batch, hdim), np.float32)
    sc = np.array(scale, np.float32)
    wp = nkn32(Wp)
    L.orc_lstmcell_int8_proj(batch, xdim, hdim, column, _p(x), xdim, _p(W), _p(wp), _p(bias), 4 * column, _p(sc), _p(st),
                             forget_bias, zc, zo, _p(out), hdim)
    return out, st


def ref_lstmcell_proj(ref, x, W, Wp, bias, scale, state, hdim, column, forget_bias=1.0, zc=0.0, zo=0.0):
    batch = state.shape[0]
    xdim = W.shape[1] - hdim
    L = ref.lib
    L.ref_lstmcell_int8_proj.argtypes = [u32, u32, u32, u32, vp, u32, vp, vp, vp, vp, vp, f32, f32, f32, vp, u32]
    st = np.array(state, np.float32, copy=True)
    out = np.zeros((batch, hdim), np.float32)
    sc = np.array(scale, np.float32)
    wp = nkn32(Wp)
    e = L.ref_lstmcell_int8_proj(batch, xdim, hdim, column, _p(x), xdim, _p(W), _p(wp), _p(bias), _p(sc), _p(st), forget_bias,
                                 zc, zo, _p(out), hdim)
    assert e == 0, e
    return out, st


def lstm_proj_case(batch, xdim, hdim, column, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((batch, xdim)).astype(np.float32)
    W = rng.integers(-127, 128, size=(4 * column, xdim + hdim), dtype=np.int8)
    Wp = (rng.standard_normal((hdim, column)) / np.sqrt(column)).astype(np.float32)
    bias = (rng.standard_normal((batch, 4 * column)) * 0.5).astype(np.float32)
    state = (rng.standard_normal((batch, column + hdim)) * 0.7).astype(np.float32)
    return x, W, Wp, bias, state
