"""bolt_gfx950_set_stream: device-pointer calls are enqueued on the caller's stream (default priority),
bolt_gfx950_synchronize waits for that stream, and results equal the default-stream results."""
import ctypes as C

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I32, DT_U8_Q, tensor2df  # noqa: E402


def test_calls_follow_the_callers_stream(oracle):
    import torch
    assert torch.cuda.is_available()
    L = capi.lib()
    capi.check(L.bolt_gfx950_init(), "init")
    M, K, N = 300, 256, 200
    rng = np.random.default_rng(11)
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    x = rng.standard_normal(M * N).astype(np.float32)
    Ad, Wd, xd = torch.from_numpy(A).cuda(), torch.from_numpy(W).cuda(), torch.from_numpy(x).cuda()
    blob, bd, rhs = host.mmm_transform_rhs(Wd, DF_TRANSPOSE, K, N)
    off = blob[rhs:rhs + 4 * N].clone()
    Cd = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    q = torch.empty(M * N, dtype=torch.uint8, device="cuda")
    ds = torch.full((1,), -1.0, device="cuda")
    torch.cuda.synchronize()
    side = torch.cuda.Stream()          # default priority
    try:
        capi.check(L.bolt_gfx950_set_stream(C.c_void_p(side.cuda_stream)), "set_stream")
        print("GEMM + dynamic quantisation on a side stream", flush=True)
        capi.check(host.matrix_matrix_multiply(Ad, tensor2df(DT_U8_Q, DF_NORMAL, M, K), blob, bd, off, Cd,
                                               tensor2df(DT_I32, DF_NORMAL, M, N), None), "mmm")
        capi.check(L.bolt_gfx950_quantize_f32_async(xd.data_ptr(), M * N, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
        ms = C.c_float(-1.0)
        capi.check(L.bolt_gfx950_timer_start(), "timer")
        capi.check(L.bolt_gfx950_quantize_f32_async(xd.data_ptr(), M * N, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
        capi.check(L.bolt_gfx950_timer_stop(C.byref(ms)), "timer")
        assert ms.value > 0.0
        capi.check(L.bolt_gfx950_synchronize(), "sync")   # waits for the side stream
        assert side.query()
    finally:
        capi.check(L.bolt_gfx950_set_stream(None), "set_stream")
    offh = off.cpu().numpy().view(np.int32)
    assert np.array_equal(Cd.cpu().numpy(), oracle.mmm(A, W, offh, np.zeros((M, N), np.int32), DT_I32))
    wq, ws = oracle.quantize_f32(x, DT_U8_Q)
    assert np.array_equal(q.cpu().numpy(), wq)
    assert np.float32(ds.item()) == np.float32(ws)
    # back on the default stream: same bytes
    Cd2 = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    capi.check(host.matrix_matrix_multiply(Ad, tensor2df(DT_U8_Q, DF_NORMAL, M, K), blob, bd, off, Cd2,
                                           tensor2df(DT_I32, DF_NORMAL, M, N), None), "mmm")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert torch.equal(Cd, Cd2)
