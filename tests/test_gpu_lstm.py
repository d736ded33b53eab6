"""GPU parity of the int8 LSTM cell against the CPU oracle (pinned in test_oracle_lstm.py), through the C-ABI in
host-pointer and device-pointer mode. The quantised activations and the integer products are exact; outputs and
states are compared to 2e-6 absolute (expf / tanhf on the GPU against double-precision libm in the oracle; all
values are bounded by 1 for outputs and by a few units for the cell state)."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_lstm  # noqa: E402
from checkers_lstm import lstm_case, lstm_proj_case, nkn32, orc_lstmcell, orc_lstmcell_proj  # noqa: E402
from test_oracle_lstm import CASES, PROJ_CASES, W_SCALE  # noqa: E402

TOL = 2e-6


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def run_cell(torch, device_mode, x, W, bias, scale, state, hdim, fb, zc, zo, x_stride=None, out_stride=None):
    batch, xdim = state.shape[0], W.shape[1] - hdim
    put = (lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()) if device_mode else np.ascontiguousarray
    st = put(np.array(state, copy=True))
    out = put(np.zeros((batch, out_stride or hdim), np.float32))
    blob = host_lstm.transform_weight(put(W), 4 * hdim, xdim + hdim)
    p = host_lstm.lstm_param_spec(hdim, fb, zc, zo)
    host_lstm.lstmcell(put(x), blob, put(bias), scale, st, p, batch, xdim, out, x_stride, out_stride)
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return out.cpu().numpy(), st.cpu().numpy()
    return out, st


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CASES + [(2, 33, 36, -1.0, 0.5, 0.2, 0.3), (5, 100, 20, -1.0, 1.0, 0.0, 0.0)])
def test_lstmcell_vs_oracle(torch_mod, oracle, case, device_mode):
    print("lstm", case, device_mode, flush=True)
    batch, xdim, hdim, sA, fb, zc, zo = case
    x, W, bias, state = lstm_case(batch, xdim, hdim, 29)
    want, wst = orc_lstmcell(oracle, x, W, bias, [sA, W_SCALE], state, hdim, fb, zc, zo)
    got, gst = run_cell(torch_mod, device_mode, x, W, bias, [sA, W_SCALE], state, hdim, fb, zc, zo)
    assert np.abs(got - want).max() <= TOL and np.abs(gst - wst).max() <= TOL


@pytest.mark.parametrize("device_mode", [False, True])
def test_lstmcell_strides(torch_mod, oracle, device_mode):
    batch, xdim, hdim = 3, 24, 32
    x, W, bias, state = lstm_case(batch, xdim, hdim, 5, x_stride=xdim + 8, bias_stride=8 * hdim)
    want, wst = orc_lstmcell(oracle, x, W, bias, [-1.0, W_SCALE], state, hdim, x_stride=xdim + 8, bias_stride=8 * hdim,
                             out_stride=2 * hdim)
    got, gst = run_cell(torch_mod, device_mode, x, W, bias, [-1.0, W_SCALE], state, hdim, 1.0, 0.0, 0.0, xdim + 8, 2 * hdim)
    assert np.abs(got - want).max() <= TOL and np.abs(gst - wst).max() <= TOL
    assert not got[:, hdim:].any()


def test_lstmcell_steps_feed_back(torch_mod, oracle):
    """Four steps on the device with the state carried in place, against four oracle steps."""
    torch = torch_mod
    batch, xdim, hdim = 4, 64, 128
    x, W, bias, state = lstm_case(batch, xdim, hdim, 41)
    rng = np.random.default_rng(2)
    xs = [rng.standard_normal((batch, xdim)).astype(np.float32) for _ in range(4)]
    st_d = torch.from_numpy(state.copy()).cuda()
    out_d = torch.zeros((batch, hdim), device="cuda")
    blob = host_lstm.transform_weight(torch.from_numpy(W).cuda(), 4 * hdim, xdim + hdim)
    bias_d = torch.from_numpy(bias).cuda()
    p = host_lstm.lstm_param_spec(hdim)
    st_o = state
    for t in range(4):
        host_lstm.lstmcell(torch.from_numpy(xs[t]).cuda(), blob, bias_d, [-1.0, W_SCALE], st_d, p, batch, xdim, out_d)
        want, st_o = orc_lstmcell(oracle, xs[t], W, bias, [-1.0, W_SCALE], st_o, hdim)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    # an fp32 difference of 1e-7 ahead of a quantiser can move one activation by one step, so later steps are
    # held to a looser bound than a single one
    assert np.abs(out_d.cpu().numpy() - want).max() <= 5e-4
    assert np.abs(st_d.cpu().numpy() - st_o).max() <= 5e-4


def test_lstmcell_rejects_what_the_reference_rejects(torch_mod):
    hdim, xdim, batch = 32, 16, 1
    x, W, bias, state = lstm_case(batch, xdim, hdim, 1)
    blob = host_lstm.transform_weight(W, 4 * hdim, xdim + hdim)
    out = np.zeros((batch, hdim), np.float32)
    p = host_lstm.lstm_param_spec(hdim)
    p.num_projection = 16
    with pytest.raises(capi.BoltError):
        host_lstm.lstmcell(x, blob, bias, [-1.0, 1.0], state.copy(), p, batch, xdim, out)
    p = host_lstm.lstm_param_spec(hdim)
    p.activation_type = capi.ACTIVATION_RELU
    with pytest.raises(capi.BoltError):
        host_lstm.lstmcell(x, blob, bias, [-1.0, 1.0], state.copy(), p, batch, xdim, out)
    p = host_lstm.lstm_param_spec(hdim)    # a filter descriptor that does not match the cell (lstm.cpp:68-70)
    with pytest.raises(capi.BoltError):
        host_lstm.lstmcell(x, blob, bias, [-1.0, 1.0], state.copy(), p, batch, xdim, out, fshape=(4 * hdim, xdim + hdim + 8))
    with pytest.raises(capi.BoltError):
        host_lstm.lstmcell(x, blob, bias, [-1.0, 1.0], state.copy(), p, batch, xdim, out, fshape=(4 * hdim + 32, xdim + hdim))


def test_lstmcell_decode_shape_properties(torch_mod, oracle):
    """256 rows x (x 2048 + h 2048) -> 4 x 2048 gates: the GEMV shape of the headline workload inside its real
    caller. Row 0 and the last row against the oracle; every row must equal the same row computed alone."""
    torch = torch_mod
    batch, xdim, hdim = 256, 2048, 2048
    x, W, bias, state = lstm_case(batch, xdim, hdim, 77)
    put = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    blob = host_lstm.transform_weight(put(W), 4 * hdim, xdim + hdim)
    p = host_lstm.lstm_param_spec(hdim)
    st = put(state.copy())
    out = torch.zeros((batch, hdim), device="cuda")
    host_lstm.lstmcell(put(x), blob, put(bias), [-1.0, W_SCALE], st, p, batch, xdim, out)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    for m in (0, batch - 1):
        want, wst = orc_lstmcell(oracle, x[m:m + 1], W, bias[m:m + 1], [-1.0, W_SCALE], state[m:m + 1], hdim)
        assert np.abs(out[m].cpu().numpy() - want[0]).max() <= TOL
        assert np.abs(st[m].cpu().numpy() - wst[0]).max() <= TOL
    for m in (3, 100):
        st1 = put(state[m:m + 1].copy())
        out1 = torch.zeros((1, hdim), device="cuda")
        host_lstm.lstmcell(put(x[m:m + 1].copy()), blob, put(bias[m:m + 1].copy()), [-1.0, W_SCALE], st1, p, 1, xdim, out1)
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        assert torch.equal(out1[0], out[m]) and torch.equal(st1[0], st[m])


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("shape", [(1, 48, 32), (4, 64, 64), (5, 100, 20), (9, 33, 36), (70, 40, 88), (300, 64, 64)])
def test_lstmcell_gemm_route_returns_the_same_bits(torch_mod, oracle, shape, device_mode):
    """A weight that carries the GEMM packing sends calls of 4+ rows through the matrix cores; outputs and states
    must be the bytes of the matrix-vector route, and both within tolerance of the oracle."""
    torch = torch_mod
    batch, xdim, hdim = shape
    print("lstm gemm route", shape, device_mode, flush=True)
    x, W, bias, state = lstm_case(batch, xdim, hdim, 61)
    put = (lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()) if device_mode else np.ascontiguousarray
    p = host_lstm.lstm_param_spec(hdim, 1.0, 0.1, 0.2)
    res = []
    for both in (False, True):
        blob = (host_lstm.rnn_transform_filter(put(W), 4 * hdim, xdim + hdim, p) if both
                else host_lstm.transform_weight(put(W), 4 * hdim, xdim + hdim))
        st, out = put(state.copy()), put(np.zeros((batch, hdim), np.float32))
        host_lstm.lstmcell(put(x), blob, put(bias), [-1.0, W_SCALE], st, p, batch, xdim, out, both_packings=both)
        if device_mode:
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            st, out = st.cpu().numpy(), out.cpu().numpy()
        res.append((out, st))
    assert res[0][0].tobytes() == res[1][0].tobytes() and res[0][1].tobytes() == res[1][1].tobytes()
    want, wst = orc_lstmcell(oracle, x, W, bias, [-1.0, W_SCALE], state, hdim, 1.0, 0.1, 0.2)
    assert np.abs(res[1][0] - want).max() <= TOL and np.abs(res[1][1] - wst).max() <= TOL


def test_lstmcell_gemm_route_decode_shape(torch_mod):
    """256 rows x 8192 x 4096 through both routes: identical bytes."""
    torch = torch_mod
    batch, xdim, hdim = 256, 2048, 2048
    x, W, bias, state = lstm_case(batch, xdim, hdim, 78)
    put = lambda a: torch.from_numpy(a).cuda()  # noqa: E731
    p = host_lstm.lstm_param_spec(hdim)
    outs = []
    for both in (False, True):
        blob = (host_lstm.rnn_transform_filter(put(W), 4 * hdim, xdim + hdim, p) if both
                else host_lstm.transform_weight(put(W), 4 * hdim, xdim + hdim))
        st, out = put(state.copy()), torch.zeros((batch, hdim), device="cuda")
        host_lstm.lstmcell(put(x), blob, put(bias), [-1.0, W_SCALE], st, p, batch, xdim, out, both_packings=both)
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        outs.append((out, st))
    assert torch.equal(outs[0][0], outs[1][0]) and torch.equal(outs[0][1], outs[1][1])


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("both_packings", [False, True])
@pytest.mark.parametrize("case", PROJ_CASES + [(6, 64, 128, 256, 1.0, 0.0, 0.1)])
def test_lstmcell_projection_vs_oracle(torch_mod, oracle, case, device_mode, both_packings):
    """num_projection > 0 (lstm.cpp:60-62, 128, 165-178): the cell's `column` activated values per row go through the
    fp32 projection matrix (DF_NKN32) to give the output and the hidden state. The projection is one chain of fused
    multiply-adds per element in the reference's order, so it adds nothing to the gates' tolerance. Both weight routes
    (batched GEMV, and the GEMM packing from 4 rows on)."""
    print("lstm projection", case, device_mode, both_packings, flush=True)
    torch = torch_mod
    batch, xdim, hdim, column, fb, zc, zo = case
    x, W, Wp, bias, state = lstm_proj_case(batch, xdim, hdim, column, 31)
    want, wst = orc_lstmcell_proj(oracle, x, W, Wp, bias, [-1.0, W_SCALE], state, hdim, column, fb, zc, zo)
    put = (lambda a: torch.from_numpy(np.ascontiguousarray(a)).cuda()) if device_mode else np.ascontiguousarray
    st = put(np.array(state, copy=True))
    out = put(np.zeros((batch, hdim), np.float32))
    p = host_lstm.lstm_param_spec(hdim, fb, zc, zo, num_projection=column)
    if both_packings:
        blob = host_lstm.rnn_transform_filter(put(W), 4 * column, xdim + hdim, p)
    else:
        blob = host_lstm.transform_weight(put(W), 4 * column, xdim + hdim)
    host_lstm.lstmcell(put(x), blob, put(bias), [-1.0, W_SCALE], st, p, batch, xdim, out, both_packings=both_packings, proj=put(nkn32(Wp)))
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        out, st = out.cpu().numpy(), st.cpu().numpy()
    assert np.abs(out - want).max() <= TOL and np.abs(st - wst).max() <= TOL
    assert np.abs(want).max() > 0.05
