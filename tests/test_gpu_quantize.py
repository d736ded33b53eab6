"""GPU parity tests for quantize / dequantize / requantize / bias fold against the CPU oracle.
u8 / s8 / int32 outputs and the returned scales are compared bit for bit; so are the fp32 outputs
(one reciprocal and one multiply, same order as the reference)."""
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import DT_F32, DT_I8, DT_I32, DT_U8_Q  # noqa: E402
from test_oracle_vs_ref import tie_table  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.fixture(params=[1, 0], ids=["one_launch", "two_pass"])
def fused(request, torch_mod):
    """Dynamic quantisation has two implementations: one cooperative launch that reads the tensor once (default
    where the tensor fits) and the two-pass form. The tests that use this fixture run under both."""
    L = capi.lib()
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused", request.param), "set_option")
    yield request.param
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused", 1), "set_option")


def both_modes(torch, x):
    yield "host", np.ascontiguousarray(x), (lambda t: np.asarray(t))
    yield "device", torch.from_numpy(np.ascontiguousarray(x)).cuda(), (lambda t: t.cpu().numpy())


@pytest.mark.parametrize("n", [1, 15, 16, 17, 1000, 65536, 4096 * 768 + 5])
@pytest.mark.parametrize("qdt", [DT_U8_Q, DT_I8])
def test_quantize_f32(torch_mod, oracle, fused, n, qdt):
    print("quantize_f32", n, qdt, flush=True)
    rng = np.random.default_rng(n)
    x = rng.standard_normal(n).astype(np.float32)
    for scale, mode in [(-1.0, 0), (20.0, 0), (1000.0, 0), (20.0, 1), (-1.0, 1), (0.0, 1)]:
        want, ws = oracle.quantize_f32(x, qdt, scale, mode)
        for name, buf, back in both_modes(torch_mod, x):
            s = [scale]
            got = back(host.quantize(buf, DT_F32, qdt, s, mode))
            assert s[0] == ws and np.array_equal(got, want), (name, scale, mode)


@pytest.mark.parametrize("qdt", [DT_U8_Q, DT_I8])
def test_quantize_f32_special_inputs(torch_mod, oracle, fused, qdt):
    cases = [np.zeros(33, np.float32),
             np.concatenate([np.full(40, 1e-3, np.float32), [1e6]]).astype(np.float32),
             tie_table(1.0), tie_table(0.5), np.array([-3.0, 3.0, -0.0, 1e-30, -1e30], np.float32)]
    for x in cases:
        for scale, mode in [(-1.0, 0), (1.0, 1), (0.5, 1), (2.0, 0)]:
            want, ws = oracle.quantize_f32(x, qdt, scale, mode)
            for name, buf, back in both_modes(torch_mod, x):
                s = [scale]
                got = back(host.quantize(buf, DT_F32, qdt, s, mode))
                assert s[0] == ws and np.array_equal(got, want), (name, scale, mode)


def test_quantize_f32_async_device_scale(torch_mod, oracle):
    torch = torch_mod
    L = capi.lib()
    rng = np.random.default_rng(1)
    x = rng.standard_normal(4096 * 64).astype(np.float32)
    dx = torch.from_numpy(x).cuda()
    for qdt, tdt in ((DT_U8_Q, torch.uint8), (DT_I8, torch.int8)):
        for scale, mode in [(-1.0, 0), (1000.0, 0), (20.0, 1)]:
            ds = torch.tensor([scale], dtype=torch.float32, device="cuda")
            q = torch.empty(x.size, dtype=tdt, device="cuda")
            capi.check(L.bolt_gfx950_quantize_f32_async(dx.data_ptr(), x.size, qdt, q.data_ptr(), ds.data_ptr(), mode),
                       "quantize_async")
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            want, ws = oracle.quantize_f32(x, qdt, scale, mode)
            assert np.float32(ds.item()) == ws and np.array_equal(q.cpu().numpy(), want)


@pytest.mark.parametrize("qdt", [DT_U8_Q, DT_I8])
def test_quantize_i32(torch_mod, oracle, fused, qdt):
    rng = np.random.default_rng(5)
    cases = [rng.integers(-200000, 200000, size=n, dtype=np.int32) for n in (1, 15, 16, 17, 4099, 32 * 64 * 56 * 56)]
    cases.append(np.zeros(20, np.int32))
    cases.append(np.array([524289, 524288, -(140 << 20), 300 << 20, -(128 << 20) - (1 << 19), -(1 << 31), (1 << 31) - 1,
                           (1 << 19), 3 << 19, -(1 << 19), -(3 << 19)], np.int64).astype(np.int32))
    for x in cases:
        for sc in ([-1.0, 0.37], [0.05, 0.37], [400.0, 0.37], [-1.0, -1.0], [2.0 ** -20, 1.0]):
            want, ws = oracle.quantize_i32(x, qdt, sc)
            for name, buf, back in both_modes(torch_mod, x):
                s = [np.float32(sc[0]), np.float32(sc[1])]
                got = back(host.quantize(buf, DT_I32, qdt, s))
                assert np.array_equal(np.array(s, np.float32), ws), (name, sc, s, ws)
                assert np.array_equal(got, want), (name, sc, x.size)


@pytest.mark.parametrize("n", [262144 + 3, 1 << 19, (1 << 19) + 16])
def test_quantize_one_launch_matches_two_pass(torch_mod, n):
    """Around the size limit of the one-launch form (512 K elements; above it both settings run the two-pass form):
    fp32 with a NaN and a known extreme, and int32 with INT32_MIN, each to u8 and s8; bytes and returned scales
    must be identical under both settings."""
    torch = torch_mod
    L = capi.lib()
    g = torch.Generator(device="cuda").manual_seed(n)
    x = torch.randn(n, device="cuda", generator=g) * 3.0
    x[n // 3] = float("nan")
    x[n // 2] = -77.25
    acc = torch.randint(-2000000, 2000000, (n,), dtype=torch.int32, device="cuda", generator=g)
    acc[n // 5] = -(1 << 31)
    out = {}
    try:
        for fused in (1, 0):
            capi.check(L.bolt_gfx950_set_option(b"quantize_fused", fused), "set_option")
            for qdt in (DT_U8_Q, DT_I8):
                s = [-1.0]
                q = host.quantize(x, DT_F32, qdt, s)
                s2 = [np.float32(-1.0), np.float32(0.37)]
                q2 = host.quantize(acc, DT_I32, qdt, s2)
                capi.check(L.bolt_gfx950_synchronize(), "sync")
                out[(fused, qdt)] = (q.clone(), s[0], q2.clone(), tuple(s2))
    finally:
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused", 1), "set_option")
    for qdt in (DT_U8_Q, DT_I8):
        a, b = out[(1, qdt)], out[(0, qdt)]
        assert a[1] == b[1] == np.float32(127.0) / np.float32(77.25) and a[3] == b[3]
        assert torch.equal(a[0], b[0]) and torch.equal(a[2], b[2])


def test_u8_to_i8(torch_mod, oracle):
    for n in [1, 63, 64, 65, 1000]:
        x = (np.arange(n) * 37 % 256).astype(np.uint8)
        for name, buf, back in both_modes(torch_mod, x):
            assert np.array_equal(back(host.quantize(buf, DT_U8_Q, DT_I8, [1.0])), oracle.u8_to_i8(x))


def test_bias_fold(torch_mod, oracle):
    s = np.float32(8.0)
    bias = np.concatenate([(np.arange(-20, 21) + 0.5) / 8.0, [0.3, -0.3, 1e3, -1e3, 0.0]]).astype(np.float32)
    off = (np.arange(bias.size, dtype=np.int32) - 7) * 1000
    N = bias.size
    for name, b, back in both_modes(torch_mod, bias):
        o = off if name == "host" else torch_mod.from_numpy(off).cuda()
        assert np.array_equal(back(host.quantize_bias_offsetC(b, o, s, N)), oracle.bias_offsetC(bias, off, s))
        assert np.array_equal(back(host.quantize_bias_offsetC(b, o, s, N, packed_filter=False)),
                              oracle.bias_offsetC(bias, None, s))
        assert np.array_equal(back(host.quantize_bias_offsetC(None, o, s, N)), off)
    rng = np.random.default_rng(3)
    b = rng.standard_normal(1024).astype(np.float32) * 0.1
    sc = np.float32(41.7) * np.float32(100.0)
    o = rng.integers(-10 ** 6, 10 ** 6, size=1024, dtype=np.int32)
    assert np.array_equal(host.quantize_bias_offsetC(b, o, sc, 1024), oracle.bias_offsetC(b, o, sc))


def test_dequantize(torch_mod, oracle):
    rng = np.random.default_rng(11)
    for n in [1, 16, 17, 100, 4096, 4096 * 768]:
        q = rng.integers(-2 ** 31, 2 ** 31 - 1, size=n, dtype=np.int64).astype(np.int32)
        for s in [0.37, 3.0, 4170.0, 1e-3]:
            want = oracle.dequantize(q, DT_I32, s)
            for name, buf, back in both_modes(torch_mod, q):
                assert np.array_equal(back(host.dequantize(buf, DT_I32, s)).view(np.int32), want.view(np.int32))
    for n in [1, 16, 17, 300]:
        q = rng.integers(0, 256, size=n, dtype=np.uint8)
        for s in [0.37, 3.0, 63.5]:
            want = oracle.dequantize(q, DT_U8_Q, s)
            for name, buf, back in both_modes(torch_mod, q):
                assert np.array_equal(back(host.dequantize(buf, DT_U8_Q, s)).view(np.int32), want.view(np.int32))


def test_requantize(torch_mod, oracle):
    x = np.arange(-128, 128, dtype=np.int8)
    for si, so in [(1.0, 1.0), (2.0, 1.0), (1.0, 0.9), (3.0, 2.0), (7.0, 6.99)]:
        for name, buf, back in both_modes(torch_mod, x):
            assert np.array_equal(back(host.requantize(buf, si, so)), oracle.requantize(x, si, so)), (si, so)


def test_requantize_ragged_and_unaligned(torch_mod, oracle):
    """Lengths that leave a tail behind the 16-byte body, and a device pointer that is not 16-byte aligned."""
    torch = torch_mod
    rng = np.random.default_rng(12)
    for n in (1, 15, 16, 17, 4099, 65536 + 3):
        x = rng.integers(-128, 128, size=n, dtype=np.int8)
        want = oracle.requantize(x, 5.0, 3.5)
        assert np.array_equal(host.requantize(x, 5.0, 3.5), want)
        big = torch.from_numpy(np.concatenate([np.zeros(3, np.int8), x])).cuda()
        got = host.requantize(big[3:], 5.0, 3.5)
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        assert np.array_equal(got.cpu().numpy(), want)


def test_roundtrip_properties_at_full_size(torch_mod):
    """Size-independent properties at the BERT FFN activation size (4096 x 3072): the extreme value
    maps to 1 / 255, zero maps to 128, quantize is monotone, and dequantize(quantize(x)) is within
    half a quantisation step."""
    torch = torch_mod
    n = 4096 * 3072
    g = torch.Generator(device="cuda").manual_seed(3)
    x = torch.randn(n, device="cuda", generator=g)
    x[123] = 0.0
    s = [-1.0]
    q = host.quantize(x, DT_F32, DT_U8_Q, s)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    amax = x.abs().max().item()
    assert s[0] == np.float32(127.0) / np.float32(amax)
    i = int(x.abs().argmax().item())
    assert int(q[i].item()) in (1, 255) and int(q[123].item()) == 128
    order = torch.argsort(x)
    assert bool((q[order][1:].to(torch.int16) >= q[order][:-1].to(torch.int16)).all())
    back = host.dequantize(q, DT_U8_Q, s[0])
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert float((back - x).abs().max().item()) <= 0.5 / float(s[0]) * 1.0001


def test_static_then_dynamic_without_sync(torch_mod, oracle):
    """Device-pointer mode: calls with a caller-given (static) scale return without waiting for their kernels. A
    dynamic call issued right behind them must return ITS scale, not a value that one of the earlier kernels
    left in the word the host reads the scale from. Large static tensors first, so that their kernels are still
    running when the dynamic calls are issued; no synchronisation anywhere in between."""
    torch = torch_mod
    L = capi.lib()
    rng = np.random.default_rng(77)
    big_f = torch.from_numpy(rng.standard_normal(4096 * 3072).astype(np.float32)).cuda()
    big_i = torch.from_numpy(rng.integers(-300000, 300000, size=4096 * 3072, dtype=np.int32)).cuda()
    small = rng.standard_normal(3000).astype(np.float32) * 5.0
    dsmall = torch.from_numpy(small).cuda()
    M, K, N = 8, 256, 64
    xq = rng.integers(1, 256, size=(M, K), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    bias = rng.standard_normal(N).astype(np.float32)
    blob, bdesc, rhs = host.mmm_transform_rhs(torch.from_numpy(W).cuda(), capi.DF_TRANSPOSE, K, N)
    dxq, dbias = torch.from_numpy(xq).cuda(), torch.from_numpy(bias).cuda()
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    want_q, want_s = oracle.quantize_f32(small, DT_U8_Q, -1.0, 0)
    want_fc, want_fs = oracle.fully_connected(xq, np.float32(21.0), W, np.float32(33.0), bias, DT_U8_Q)
    for fused in (1, 0):
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused", fused), "set_option")
        try:
            for rep in range(4):
                print("static_then_dynamic", fused, rep, flush=True)
                s_static = [np.float32(17.5)]
                host.quantize(big_f, DT_F32, DT_U8_Q, s_static, 1)        # static fp32 -> u8
                s_req = [np.float32(0.011), np.float32(0.37)]
                host.quantize(big_i, DT_I32, DT_U8_Q, s_req)               # static int32 -> u8
                s = [-1.0]
                q = host.quantize(dsmall, DT_F32, DT_U8_Q, s)              # dynamic, straight behind them
                assert s[0] == want_s, (fused, rep, s[0], want_s)
                host.quantize(big_f, DT_F32, DT_I8, [np.float32(3.25)], 1)
                host.quantize(big_i, DT_I32, DT_I8, [np.float32(0.02), np.float32(0.37)])
                out, so = host.fully_connected(dxq, 21.0, blob, capi.DF_NKNxKx, 33.0, dbias, M, K, N, DT_U8_Q, -1.0)
                assert so == want_fs, (fused, rep, so, want_fs)
                capi.check(L.bolt_gfx950_synchronize(), "sync")
                assert np.array_equal(q.cpu().numpy(), want_q)
                assert np.array_equal(out.cpu().numpy(), want_fc)
                assert s_static[0] == np.float32(17.5) and s_req[0] == np.float32(0.011)
        finally:
            capi.check(L.bolt_gfx950_set_option(b"quantize_fused", 1), "set_option")


def test_one_launch_quantiser_falls_back_when_its_wait_gives_up(torch_mod, oracle):
    """The one-launch dynamic quantiser waits for its whole grid a bounded number of polls. With the bound forced to
    one poll from the host, launches of more than a few workgroups give up: every workgroup then skips its stores,
    the kernel publishes a NaN scale and exits normally, and the call is redone in two passes. Bytes and scale must be
    the oracle's either way, and the fallback counter must have moved."""
    torch = torch_mod
    L = capi.lib()
    import ctypes as C
    before = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(before)), "counter")
    capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 1), "set_option")
    try:
        rng = np.random.default_rng(31)
        for n in (1000, 65536, 262144 + 16, 1 << 19):
            x = (rng.standard_normal(n) * 2.5).astype(np.float32)
            acc = rng.integers(-900000, 900000, size=n, dtype=np.int32)
            dx, dacc = torch.from_numpy(x).cuda(), torch.from_numpy(acc).cuda()
            for rep in range(3):
                print("fused fallback", n, rep, flush=True)
                for qdt in (DT_U8_Q, DT_I8):
                    want, ws = oracle.quantize_f32(x, qdt)
                    s = [-1.0]
                    q = host.quantize(dx, DT_F32, qdt, s)
                    capi.check(L.bolt_gfx950_synchronize(), "sync")
                    assert s[0] == ws and np.array_equal(q.cpu().numpy(), want), (n, rep, qdt)
                    want2, ws2 = oracle.quantize_i32(acc, qdt, [-1.0, 0.37])
                    s2 = [np.float32(-1.0), np.float32(0.37)]
                    q2 = host.quantize(dacc, DT_I32, qdt, s2)
                    capi.check(L.bolt_gfx950_synchronize(), "sync")
                    assert np.array_equal(np.array(s2, np.float32), ws2) and np.array_equal(q2.cpu().numpy(), want2), (n, rep, qdt)
                    assert np.array_equal(host.quantize(x, DT_F32, qdt, [-1.0]), want)     # host-pointer mode too
    finally:
        capi.check(L.bolt_gfx950_set_option(b"quantize_fused_spin", 0), "set_option")
    after = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(after)), "counter")
    assert after.value > before.value, "no launch gave up: the test did not exercise the fallback"
    # and with the default bound the one-launch form completes again
    s = [-1.0]
    q = host.quantize(dx, DT_F32, DT_U8_Q, s)
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    want, ws = oracle.quantize_f32(x, DT_U8_Q)
    assert s[0] == ws and np.array_equal(q.cpu().numpy(), want)
    final = C.c_ulonglong(0)
    capi.check(L.bolt_gfx950_get_counter(b"quantize_fused_fallbacks", C.byref(final)), "counter")
    assert final.value == after.value


def test_quantize_beyond_two_to_the_31_elements(torch_mod):
    """2^31 + 12 345 fp32 values (8.6 GB): element indices above 2^31 and byte offsets above 2^33. The tensor-wide dynamic
    scale must be 127 / max|x| with the maximum placed near the far end, and the bytes must equal those of chunk-wise
    calls with that scale given (static mode), which run at sizes the other tests hold against the CPU checker; the
    dequantised tensor is within half a step everywhere."""
    torch = torch_mod
    n = (1 << 31) + 12345
    g = torch.Generator(device="cuda").manual_seed(9)
    x = torch.empty(n, dtype=torch.float32, device="cuda")
    step = 1 << 28
    for lo in range(0, n, step):
        x[lo:lo + step].normal_(generator=g)
    x[n - 7] = 9.5                       # the maximum sits where only 64-bit addressing reaches
    print("quantize", n, "elements", flush=True)
    for qdt in (DT_U8_Q, DT_I8):
        s = [-1.0]
        q = host.quantize(x, DT_F32, qdt, s)
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        assert s[0] == np.float32(127.0) / np.float32(9.5), s
        for lo in (0, (1 << 31) - (1 << 20), n - (1 << 24) - 5):          # head, across 2^31, the ragged tail
            hi = min(n, lo + (1 << 24) + 5)
            sc = [float(s[0])]
            part = host.quantize(x[lo:hi].clone(), DT_F32, qdt, sc, 1)
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            assert sc[0] == s[0] and torch.equal(part, q[lo:hi]), (qdt, lo)
        if qdt == DT_U8_Q:
            back = host.dequantize(q, DT_U8_Q, s[0])
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            worst = 0.0
            for lo in range(0, n, step):
                worst = max(worst, float((back[lo:lo + step] - x[lo:lo + step]).abs().max().item()))
            assert worst <= 0.5 / float(s[0]) * 1.0001, worst
            del back
        del q
    del x
    torch.cuda.empty_cache()
