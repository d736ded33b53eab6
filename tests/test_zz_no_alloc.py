"""bolt_gfx950_quantize_f32_noalloc (the entry point that allocates nothing: its partial-maximum slots live in a static
device array) against bolt_gfx950_quantize_f32_async, the entry point it is a variant of: same bytes, same device-side
scale, bit for bit, on two calls in a row -- the second on a smaller input, so that maxima left in the array by the
first call would show -- and for every scale mode and both output types."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi  # noqa: E402
from bolt_amd.capi import DT_I8, DT_U8_Q  # noqa: E402


def run(L, torch, fn, x, qdt, scale, mode):
    q = torch.full((x.numel(),), 77, dtype=torch.uint8 if qdt == DT_U8_Q else torch.int8, device="cuda")
    ds = torch.tensor([scale], dtype=torch.float32, device="cuda")
    capi.check(fn(x.data_ptr(), x.numel(), qdt, q.data_ptr(), ds.data_ptr(), mode), "quantize")
    return q, ds


def test_no_alloc_matches_async_two_calls_in_a_row():
    import torch
    assert torch.cuda.is_available()
    L = capi.lib()
    g = torch.Generator(device="cuda").manual_seed(20240701)
    big = torch.randn(4096 * 768 + 5, device="cuda", generator=g) * 9.0      # first call: large values
    small = torch.randn(1000, device="cuda", generator=g) * 0.01             # second call: smaller input, tiny values
    small[17] = -0.0425
    for qdt in (DT_U8_Q, DT_I8):
        for scale, mode in ((-1.0, 0), (1000.0, 0), (20.0, 1), (0.0, 1)):
            print("no_alloc", qdt, scale, mode, flush=True)
            got = [run(L, torch, L.bolt_gfx950_quantize_f32_noalloc, x, qdt, scale, mode) for x in (big, small)]
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            want = [run(L, torch, L.bolt_gfx950_quantize_f32_async, x, qdt, scale, mode) for x in (big, small)]
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            for (gq, gs), (wq, ws) in zip(got, want):
                assert torch.equal(gs, ws), (qdt, scale, mode, gs.item(), ws.item())
                assert torch.equal(gq, wq), (qdt, scale, mode)
            if scale < 0:
                assert np.float32(got[1][1].item()) == np.float32(127.0) / np.float32(0.0425)


def test_no_alloc_leaves_device_memory_alone():
    """After the one-time set-up (bolt_gfx950_init or a first call), a run of calls changes neither the free device
    memory the driver reports nor torch's own allocator's reservation."""
    import torch
    L = capi.lib()
    capi.check(L.bolt_gfx950_init(), "init")
    x = torch.randn(1 << 20, device="cuda")
    q = torch.zeros(1 << 20, dtype=torch.uint8, device="cuda")
    ds = torch.tensor([-1.0], device="cuda")
    capi.check(L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), x.numel(), DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "warm-up")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    torch.cuda.synchronize()
    free0, _ = torch.cuda.mem_get_info()
    reserved0 = torch.cuda.memory_reserved()
    for n in (1 << 20, 1000, 1 << 18, 64):
        for _ in range(8):
            capi.check(L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), n, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    torch.cuda.synchronize()
    free1, _ = torch.cuda.mem_get_info()
    assert free1 == free0, (free0, free1)
    assert torch.cuda.memory_reserved() == reserved0


def test_no_alloc_rejects_and_edges():
    import torch
    L = capi.lib()
    x = torch.zeros(64, device="cuda")
    q = torch.zeros(64, dtype=torch.uint8, device="cuda")
    ds = torch.tensor([-1.0], device="cuda")
    too_many = (1 << 30) + 1
    assert L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), too_many, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0) == capi.NOT_SUPPORTED
    assert b"2^30" in L.bolt_gfx950_last_error()
    assert L.bolt_gfx950_quantize_f32_noalloc(None, 64, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0) == capi.NULL_POINTER
    assert L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), 64, 6, q.data_ptr(), ds.data_ptr(), 0) == capi.NOT_SUPPORTED
    # all zeros: scale 1, every byte the zero point; n = 0: nothing is written
    capi.check(L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), 64, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
    capi.check(L.bolt_gfx950_quantize_f32_noalloc(x.data_ptr(), 0, DT_U8_Q, q.data_ptr(), ds.data_ptr(), 0), "quantize")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    assert ds.item() == 1.0 and bool((q == 128).all())
