"""Pins the int8 LSTM-cell oracle.

Against the reference's own compiled lstmcell_int8 (oracle/_ref): outputs and both states to 6e-4 absolute.
That is as close as the reference is to itself: its 8-wide gate loop takes the sigmoid's reciprocal with
_mm256_rcp_ps (relative error up to 1.5 * 2^-12, and not the same bits on every x86 vendor) and exp from a
degree-5 polynomial (common/uni/include/x86_avx2_expand.h:60-111), while its scalar tail (lstm.cpp:151-161)
uses double-precision libm; the oracle follows the tail. Valid shapes have 4 * hdim % 32 == 0, so the tail
never runs in the reference and no tighter comparison with it exists; a wrong gate order, sign, bias row or
zoneout term shows as an error of 1e-2 or more. Cases: dynamic and static activation scales, zoneout on the
cell and on the output, x_dim = 0, row strides, several batch rows each with its own bias row.
The formula itself is pinned to 3e-6 by an independent float64 numpy cell fed exact integer products."""
import numpy as np
import pytest

from checkers import DT_U8_Q
from checkers_lstm import (lstm_case, lstm_proj_case, orc_lstmcell, orc_lstmcell_proj, ref_lstmcell, ref_lstmcell_proj)

W_SCALE = np.float32(1.0) / np.float32(0.004)

CASES = [  # batch, xdim, hdim, activation scale, forget_bias, zoneout_cell, zoneout_output
    (1, 48, 32, -1.0, 1.0, 0.0, 0.0),
    (3, 40, 64, -1.0, 0.0, 0.0, 0.0),
    (2, 24, 40, -1.0, 1.0, 0.1, 0.0),     # hdim % 8 == 0 but xdim + hdim not a multiple of 16
    (2, 24, 40, -1.0, 1.0, 0.0, 0.25),
    (2, 33, 48, -1.0, 0.5, 0.2, 0.3),
    (2, 16, 32, 20.0, 1.0, 0.0, 0.0),     # static activation scale
    (2, 0, 64, -1.0, 1.0, 0.0, 0.0),      # no x: the state alone drives the cell
]


@pytest.mark.parametrize("case", CASES)
def test_lstmcell_oracle_vs_reference(oracle, ref, case):
    batch, xdim, hdim, sA, fb, zc, zo = case
    x, W, bias, state = lstm_case(batch, xdim, hdim, 17)
    want, wst = ref_lstmcell(ref, x, W, bias, [sA, W_SCALE], state, hdim, fb, zc, zo)
    got, gst = orc_lstmcell(oracle, x, W, bias, [sA, W_SCALE], state, hdim, fb, zc, zo)
    assert np.abs(got - want).max() <= 6e-4
    assert np.abs(gst - wst).max() <= 6e-4


def test_lstmcell_oracle_strides_vs_reference(oracle, ref):
    """Rows of x 8 floats apart from dense, outputs 2 * hdim apart: the reference then reads bias row m at
    m * 2 * 4 * hdim (lstm.cpp:64,91)."""
    batch, xdim, hdim = 3, 24, 32
    x, W, bias, state = lstm_case(batch, xdim, hdim, 5, x_stride=xdim + 8, bias_stride=8 * hdim)
    want, wst = ref_lstmcell(ref, x, W, bias, [-1.0, W_SCALE], state, hdim, x_stride=xdim + 8, out_stride=2 * hdim)
    got, gst = orc_lstmcell(oracle, x, W, bias, [-1.0, W_SCALE], state, hdim, x_stride=xdim + 8, bias_stride=8 * hdim,
                            out_stride=2 * hdim)
    assert np.abs(got - want).max() <= 6e-4 and np.abs(gst - wst).max() <= 6e-4
    assert not got[:, hdim:].any()


def test_lstmcell_oracle_vs_float64_numpy(oracle):
    batch, xdim, hdim = 2, 20, 24
    x, W, bias, state = lstm_case(batch, xdim, hdim, 3)
    got, gst = orc_lstmcell(oracle, x, W, bias, [-1.0, W_SCALE], state, hdim, 1.0, 0.15, 0.35)
    for m in range(batch):
        xh = np.concatenate([x[m], state[m, hdim:]])
        q, s = oracle.quantize_f32(xh, DT_U8_Q)
        acc = W.astype(np.int64) @ (q.astype(np.int64) - 128)
        g = acc / (np.float64(s) * np.float64(W_SCALE)) + bias[m]
        i, gg, f, o = (g[k * hdim:(k + 1) * hdim] for k in range(4))
        sig = lambda v: 1 / (1 + np.exp(-v))  # noqa: E731
        c0 = state[m, :hdim].astype(np.float64)
        c1 = c0 * sig(f + 1.0) + sig(i) * np.tanh(gg)
        hid = sig(o) * np.tanh(c1)
        assert np.abs(got[m] - hid).max() <= 3e-6
        assert np.abs(gst[m, :hdim] - (c1 * 0.85 + c0 * 0.15)).max() <= 3e-6
        assert np.abs(gst[m, hdim:] - (hid * 0.65 + state[m, hdim:] * 0.35)).max() <= 3e-6


PROJ_CASES = [  # batch, xdim, hdim (num_outputs), column (num_projection), forget_bias, zoneout_cell, zoneout_output
    (2, 24, 32, 64, 1.0, 0.0, 0.0),
    (3, 40, 64, 32, 0.0, 0.0, 0.0),
    (2, 16, 32, 96, 1.0, 0.2, 0.0),
    (2, 16, 64, 48, 0.5, 0.1, 0.3),
]


@pytest.mark.parametrize("case", PROJ_CASES)
def test_lstmcell_projection_oracle_vs_reference(oracle, ref, case):
    """num_projection > 0 (lstm.cpp:60-62, 128, 165-173): the gates give `column` values per row, the hidden state and
    the output are the fp32 projection of those, and the zoneout of the output acts on the projected values. Against the
    reference's compiled cell to 6e-4 (the gates' own tolerance; the projection adds sums of at most 96 products of
    values below 1): a wrong layout of the projection matrix, state offset or order of projection and zoneout shows as
    an error of 1e-1."""
    batch, xdim, hdim, column, fb, zc, zo = case
    x, W, Wp, bias, state = lstm_proj_case(batch, xdim, hdim, column, 23)
    want, wst = ref_lstmcell_proj(ref, x, W, Wp, bias, [-1.0, W_SCALE], state, hdim, column, fb, zc, zo)
    got, gst = orc_lstmcell_proj(oracle, x, W, Wp, bias, [-1.0, W_SCALE], state, hdim, column, fb, zc, zo)
    assert np.abs(got - want).max() <= 6e-4 and np.abs(gst - wst).max() <= 6e-4
    assert np.abs(want).max() > 0.05


def test_lstmcell_projection_oracle_vs_float64_numpy(oracle):
    batch, xdim, hdim, column = 2, 20, 32, 40
    x, W, Wp, bias, state = lstm_proj_case(batch, xdim, hdim, column, 3)
    got, gst = orc_lstmcell_proj(oracle, x, W, Wp, bias, [-1.0, W_SCALE], state, hdim, column, 1.0, 0.15, 0.35)
    for m in range(batch):
        xh = np.concatenate([x[m], state[m, column:]])
        q, s = oracle.quantize_f32(xh, DT_U8_Q)
        acc = W.astype(np.int64) @ (q.astype(np.int64) - 128)
        g = acc / (np.float64(s) * np.float64(W_SCALE)) + bias[m]
        i, gg, f, o = (g[k * column:(k + 1) * column] for k in range(4))
        sig = lambda v: 1 / (1 + np.exp(-v))  # noqa: E731
        c0 = state[m, :column].astype(np.float64)
        c1 = c0 * sig(f + 1.0) + sig(i) * np.tanh(gg)
        hid = Wp.astype(np.float64) @ (sig(o) * np.tanh(c1))
        assert np.abs(got[m] - hid).max() <= 5e-6
        assert np.abs(gst[m, :column] - (c1 * 0.85 + c0 * 0.15)).max() <= 3e-6
        assert np.abs(gst[m, column:] - (hid * 0.65 + state[m, column:] * 0.35)).max() <= 5e-6
