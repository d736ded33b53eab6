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


def test_grid_wide_agreements_while_another_stream_holds_the_cus():
    """The one-pass u8 convolution and the one-launch quantiser keep values in registers while all workgroups of a
    launch agree on a maximum, which needs the whole grid resident. Here another stream keeps every CU busy with large
    bf16 products the whole time (a serving process sharing the device): the calls must return the bytes and scales
    they return on an idle device, whether their agreement completes once the other stream's workgroups drain or is
    abandoned after its bounded wait and redone in two passes."""
    import time

    import torch
    from bolt_amd import host_conv
    from bolt_amd.capi import DF_NCHWC8, DF_NCHWC16
    L = capi.lib()
    capi.check(L.bolt_gfx950_init(), "init")
    g = torch.Generator(device="cuda")
    g.manual_seed(1)
    n, ic, ih, iw, oc = 32, 64, 56, 56, 64
    xq = torch.randint(128, 256, (n * ic * ih * iw,), dtype=torch.uint8, device="cuda", generator=g)
    Wc = torch.randint(-127, 128, (oc, ic, 3, 3), dtype=torch.int8, device="cuda", generator=g)
    p = capi.conv_param_spec(oc, 3, 3, 1, 1)
    cblob, ftm = host_conv.transform_filter(Wc, oc, ic, 3, 3, p)
    cb = torch.randn(oc, device="cuda", generator=g) * 0.1
    xf = torch.randn(1 << 18, device="cuda", generator=g)

    def conv():
        sc = [30.0, -1.0, 80.0]
        out = host_conv.convolution(xq, DF_NCHWC8, n, ic, ih, iw, cblob, ftm, oc, 3, 3, 1, 1, cb, sc, True, DT_U8_Q, DF_NCHWC16)
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        return out.clone(), sc[1]

    def quant():
        s = [-1.0]
        q = host.quantize(xf, DT_F32, DT_U8_Q, s)
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        return q.clone(), s[0]
    ref_c, ref_cs = conv()
    ref_q, ref_qs = quant()
    side = torch.cuda.Stream()          # default priority
    A = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    B = torch.randn(8192, 8192, device="cuda", dtype=torch.bfloat16)
    worst = 0.0
    for it in range(40):
        with torch.cuda.stream(side):
            for _ in range(6):
                A @ B                   # half a millisecond each on every CU
        t1 = time.time()
        got_c, got_cs = conv()
        got_q, got_qs = quant()
        worst = max(worst, time.time() - t1)
        assert torch.equal(got_c, ref_c) and got_cs == ref_cs, it
        assert torch.equal(got_q, ref_q) and got_qs == ref_qs, it
    side.synchronize()
    print("worst pair of calls under contention: %.1f ms" % (worst * 1e3), flush=True)
    assert worst < 5.0                  # seconds: the bounded waits end (2^19 polls each) and nothing hangs


def test_async_entry_points_replay_from_a_captured_graph():
    """The device-scale forms depend on their arguments only, so a chain of them can be captured in a HIP graph: the
    dynamic quantiser that leaves its scale on the device (two passes, its slots cleared by a fill kernel, no memset
    node) feeding the per-channel product that reads that scale from the device. The graph is replayed four times with
    new activations, eager work and synchronisations in between; every replay must equal the eager chain."""
    import torch
    L = capi.lib()
    capi.check(L.bolt_gfx950_init(), "init")
    g = torch.Generator(device="cuda")
    g.manual_seed(4)
    M, K, N = 256, 1024, 768
    x = torch.randn(M * K, device="cuda", generator=g)
    W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
    off = blob[rhs:rhs + 4 * N].view(torch.int32).clone()
    sw = torch.rand(N, device="cuda", generator=g) * 150 + 50
    bias = torch.randn(N, device="cuda", generator=g) * 0.1
    q = torch.empty(M * K, dtype=torch.uint8, device="cuda")
    ds = torch.full((1,), -1.0, device="cuda")
    out = torch.empty((M, N), dtype=torch.float32, device="cuda")
    L.bolt_gfx950_mmm_int8_perchannel.argtypes = [C.c_uint32, C.c_uint32, C.c_uint32] + [C.c_void_p] * 7

    def chain():
        ds.fill_(-1.0)               # a fill kernel on the current stream (the library's stream below): dynamic scale asked for
        capi.check(L.bolt_gfx950_quantize_f32_async(x.data_ptr(), M * K, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
        capi.check(L.bolt_gfx950_mmm_int8_perchannel(M, N, K, q.data_ptr(), blob.data_ptr(), off.data_ptr(), out.data_ptr(),
                                                     ds.data_ptr(), sw.data_ptr(), bias.data_ptr()), "mmm_int8_perchannel")
    side = torch.cuda.Stream()       # default priority
    torch.cuda.synchronize()
    try:
        capi.check(L.bolt_gfx950_set_stream(C.c_void_p(side.cuda_stream)), "set_stream")
        with torch.cuda.stream(side):
            chain()
            chain()                  # nothing left to initialise inside the capture
        side.synchronize()
        graph = torch.cuda.CUDAGraph()
        with torch.cuda.graph(graph, stream=side):
            chain()
        side.synchronize()
        for rep in range(4):
            x.copy_(torch.randn(M * K, device="cuda", generator=g) * (rep + 1))
            torch.cuda.synchronize()
            graph.replay()
            torch.cuda.synchronize()
            got, got_scale = out.clone(), ds.clone()
            with torch.cuda.stream(side):
                chain()
            side.synchronize()
            print("graph replay", rep, float(got_scale.item()), flush=True)
            assert torch.equal(got_scale, ds) and torch.equal(got, out), rep
    finally:
        capi.check(L.bolt_gfx950_set_stream(None), "set_stream")
