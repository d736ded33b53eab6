"""GPU parity of the quantised pooling and concatenation against the CPU oracle (itself pinned bit for bit
against the reference's compiled pooling_uint8 / concat_cpu in test_oracle_pool.py) and against the committed
golden vectors, through the C-ABI, in host-pointer and device-pointer mode. Everything is compared bit for
bit, the returned scales included. Full-size cases go through size-independent properties."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_pool  # noqa: E402
from bolt_amd.capi import DF_NCHWC16, DT_F32, DT_I8, POOLING_MAX, POOLING_MEAN, tensor4df  # noqa: E402
from checkers_pool import orc_concat, orc_pooling, pool_desc  # noqa: E402
from test_golden import load, same  # noqa: E402
from test_oracle_pool import CONCAT_CASES, POOL_CASES, concat_inputs, concat_layout, pool_input  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def put(torch, device_mode, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda() if device_mode else np.ascontiguousarray(a)


def get(t):
    if hasattr(t, "cpu"):
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return t.cpu().numpy()
    return t


def run_pool(torch, device_mode, case, x, in_scale):
    n, c, ih, iw, kh, kw, sh, sw, pt, pb, pl, pr, mean, cip, _ = case
    d = pool_desc(case)
    p = capi.pooling_param_spec(POOLING_MEAN if mean else POOLING_MAX, kh, kw, sh, sw, pt, pb, pl, pr, cip)
    out, s = host_pool.pooling_u8(put(torch, device_mode, x), n, c, ih, iw, p, in_scale, d.oh, d.ow)
    return get(out), s


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("relu", [True, False])
@pytest.mark.parametrize("case", POOL_CASES)
def test_pooling_vs_oracle(torch_mod, oracle, case, relu, device_mode):
    print("pool", case, relu, device_mode, flush=True)
    x = pool_input(case, 21, relu)
    want, ws = orc_pooling(oracle, pool_desc(case), x, 5.5)
    got, gs = run_pool(torch_mod, device_mode, case, x, 5.5)
    assert same(got, want) and same(np.float32(gs), np.float32(ws))


@pytest.mark.parametrize("case", [
    (2, 32, 20, 20, 20, 20, 1, 1, 0, 0, 0, 0, 1, 0, 0),     # 400 taps: 32-bit sums
    (1, 16, 40, 33, 17, 16, 3, 2, 5, 5, 4, 4, 1, 0, 0),     # 272 taps, clipped windows of fewer
    (1, 16, 40, 33, 17, 16, 3, 2, 5, 5, 4, 4, 1, 1, 0),
    (1, 16, 16, 16, 16, 16, 1, 1, 0, 0, 0, 0, 1, 0, 0),     # exactly 256 taps: the largest 16-bit case
])
def test_pooling_large_windows(torch_mod, oracle, case):
    print("pool large", case, flush=True)
    for relu in (True, False):
        x = pool_input(case, 33, relu)
        if relu:
            x[:] = np.maximum(x, 250)   # sums as large as they get
        want, ws = orc_pooling(oracle, pool_desc(case), x, 1.0)
        got, gs = run_pool(torch_mod, True, case, x, 1.0)
        assert same(got, want) and same(np.float32(gs), np.float32(ws))


def test_pooling_global_by_zero_kernel(torch_mod, oracle):
    """kernel_h = kernel_w = 0 means the whole image (compute/tensor/src/pooling.cpp:107-131)."""
    case = (2, 32, 7, 7, 7, 7, 1, 1, 0, 0, 0, 0, 1, 0, 0)
    x = pool_input(case, 2, True)
    want, ws = orc_pooling(oracle, pool_desc(case), x, 3.0)
    p = capi.pooling_param_spec(POOLING_MEAN, 0, 0, 1, 1, 0, 0, 0, 0)
    out, gs = host_pool.pooling_u8(put(torch_mod, True, x), 2, 32, 7, 7, p, 3.0, 1, 1)
    assert same(get(out), want) and same(np.float32(gs), np.float32(ws))


def test_pooling_rejects_what_the_reference_rejects(torch_mod):
    L = capi.lib()
    x = np.zeros(16 * 8 * 8, np.uint8)
    out = np.zeros(16 * 8 * 8, np.uint8)
    sc = np.zeros(2, np.float32)
    vp = lambda a: a.ctypes.data  # noqa: E731
    good = capi.pooling_param_spec(POOLING_MAX, 2, 2, 2, 2, 0, 0, 0, 0)
    d16 = tensor4df(capi.DT_U8_Q, DF_NCHWC16, 1, 16, 8, 8)
    o16 = tensor4df(capi.DT_U8_Q, DF_NCHWC16, 1, 16, 4, 4)
    assert L.pooling_gfx950(d16, vp(x), good, vp(sc), o16, vp(out), None, capi.AMD_GFX950) == capi.SUCCESS
    # pad >= kernel: NOT_SUPPORTED (pooling_int8.cpp:352-354)
    bad = capi.pooling_param_spec(POOLING_MAX, 2, 2, 2, 2, 2, 0, 0, 0)
    assert L.pooling_gfx950(d16, vp(x), bad, vp(sc), o16, vp(out), None, capi.AMD_GFX950) == capi.NOT_SUPPORTED
    # NCHWC8 input: NOT_MATCH (pooling_int8.cpp:337-339)
    d8 = tensor4df(capi.DT_U8_Q, capi.DF_NCHWC8, 1, 16, 8, 8)
    assert L.pooling_gfx950(d8, vp(x), good, vp(sc), o16, vp(out), None, capi.AMD_GFX950) == capi.NOT_MATCH
    # fp32 data is not this library's: NOT_SUPPORTED
    df = tensor4df(DT_F32, DF_NCHWC16, 1, 16, 8, 8)
    assert L.pooling_gfx950(df, vp(x), good, vp(sc), o16, vp(out), None, capi.AMD_GFX950) == capi.NOT_SUPPORTED
    assert L.pooling_gfx950(d16, None, good, vp(sc), o16, vp(out), None, capi.AMD_GFX950) == capi.NULL_POINTER


def run_concat(torch, device_mode, case, parts, scales):
    df, axis, dims, _ = case
    _, _, odims = concat_layout(case)
    descs = [tensor4df(DT_I8, df, *d) for d in dims]
    out, s = host_pool.concat([put(torch, device_mode, p) for p in parts], descs, axis, tensor4df(DT_I8, df, *odims),
                              scales)
    return get(out).view(np.int8), s


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CONCAT_CASES)
def test_concat_vs_oracle(torch_mod, oracle, case, device_mode):
    print("concat", case, device_mode, flush=True)
    parts = concat_inputs(case, 8)
    lens, loops, _ = concat_layout(case)
    want, ws = orc_concat(oracle, parts, lens, loops, case[3])
    got, gs = run_concat(torch_mod, device_mode, case, parts, case[3])
    assert same(got, want) and same(np.float32(gs), np.float32(ws))
    # without scales: a plain join, inputs untouched
    want2, _ = orc_concat(oracle, parts, lens, loops, None)
    got2, gs2 = run_concat(torch_mod, device_mode, case, parts, None)
    assert same(got2, want2) and gs2 is None


def test_concat_skips_empty_inputs_and_keeps_their_scales(torch_mod, oracle):
    case = (0, 1, [(2, 3, 5, 7), (2, 5, 5, 7)], [20.0, 31.0])
    parts = concat_inputs(case, 5)
    lens, loops, odims = concat_layout(case)
    want, _ = orc_concat(oracle, parts, lens, loops, [20.0, 31.0])   # minimum 20 either way
    descs = [tensor4df(DT_I8, 0, *case[2][0]), tensor4df(DT_I8, 0, 2, 0, 5, 7), tensor4df(DT_I8, 0, *case[2][1])]
    out, s = host_pool.concat([parts[0], None, parts[1]], descs, 1, tensor4df(DT_I8, 0, *odims), [20.0, 25.0, 31.0])
    assert same(out.view(np.int8), want) and s == np.float32(20.0)
    # an empty input with the smallest scale still sets the output scale (concat.cpp:175-177)
    out, s = host_pool.concat([parts[0], None, parts[1]], descs, 1, tensor4df(DT_I8, 0, *odims), [20.0, 5.0, 31.0])
    want, _ = orc_concat(oracle, [parts[0], np.zeros(0, np.int8), parts[1]], [lens[0], 0, lens[1]], loops,
                         [20.0, 5.0, 31.0])
    assert same(out.view(np.int8), want) and s == np.float32(5.0)


def test_concat_shape_errors(torch_mod):
    parts = [np.zeros(2 * 3 * 5 * 7, np.int8), np.zeros(2 * 5 * 5 * 7, np.int8)]
    descs = [tensor4df(DT_I8, 0, 2, 3, 5, 7), tensor4df(DT_I8, 0, 2, 5, 5, 7)]
    with pytest.raises(capi.BoltError):
        host_pool.concat(parts, descs, 1, tensor4df(DT_I8, 0, 2, 9, 5, 7), [1.0, 2.0])    # extents do not add up
    with pytest.raises(capi.BoltError):
        host_pool.concat(parts, descs, 2, tensor4df(DT_I8, 0, 2, 3, 10, 7), [1.0, 2.0])   # differ off the axis


def test_pool_and_concat_golden(torch_mod):
    g = load("pool_concat")
    for i, case in enumerate(g["pool_cases"]):
        case = tuple(int(v) for v in case)
        for device_mode in (False, True):
            y, s = run_pool(torch_mod, device_mode, case, g[f"pool_x{i}"], 12.75)
            assert same(y, g[f"pool_y{i}"]) and same(np.float32(s), g[f"pool_s{i}"])
    for i in range(int(g["concat_n"])):
        dims = [tuple(int(v) for v in d) for d in g[f"cat_dims{i}"]]
        case = (int(g[f"cat_meta{i}"][0]), int(g[f"cat_meta{i}"][1]), dims, list(g[f"cat_scales{i}"]))
        parts = [g[f"cat_in{i}_{j}"] for j in range(len(dims))]
        for device_mode in (False, True):
            y, s = run_concat(torch_mod, device_mode, case, parts, case[3])
            assert same(y, g[f"cat_y{i}"]) and same(np.float32(s), g[f"cat_s{i}"])


def test_pooling_full_size_properties(torch_mod):
    """32 x 64 x 112 x 112 (a ResNet stem's pooling input), 3 x 3 stride 2 pad 1. Max pooling commutes with any
    monotone byte map (here x -> 255 - (255 - x) // 2); a 1 x 1 mean window is the identity at or above the zero point 128; the mean of a constant image
    is that constant wherever 65536 / taps is exact."""
    torch = torch_mod
    n, c, ih, iw = 32, 64, 112, 112
    g = torch.Generator(device="cuda").manual_seed(7)
    x = torch.randint(0, 256, (n * c * ih * iw,), dtype=torch.uint8, device="cuda", generator=g)
    p = capi.pooling_param_spec(POOLING_MAX, 3, 3, 2, 2, 1, 1, 1, 1)
    y, s = host_pool.pooling_u8(x, n, c, ih, iw, p, 4.0, 56, 56)
    fx = (255 - (255 - x.to(torch.int32)) // 2).to(torch.uint8)
    fy, _ = host_pool.pooling_u8(fx, n, c, ih, iw, p, 4.0, 56, 56)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(fy, (255 - (255 - y.to(torch.int32)) // 2).to(torch.uint8)) and s == np.float32(4.0)
    # against torch's own max pooling on the same bytes
    xs = x.view(n, c // 16, ih, iw, 16).permute(0, 1, 4, 2, 3).reshape(n, c, ih, iw).float()
    ty = torch.nn.functional.max_pool2d(xs, 3, 2, 1).to(torch.uint8)
    ty = ty.view(n, c // 16, 16, 56, 56).permute(0, 1, 3, 4, 2).reshape(-1)
    assert torch.equal(y, ty)
    one = capi.pooling_param_spec(POOLING_MEAN, 1, 1, 1, 1, 0, 0, 0, 0)
    xr = x | 128   # at or above the zero point, as after a ReLU: below it the reference's mean saturates to 255
    z, _ = host_pool.pooling_u8(xr, n, c, ih, iw, one, 4.0, ih, iw)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(z, xr)
    z, _ = host_pool.pooling_u8(x, n, c, ih, iw, one, 4.0, ih, iw)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(z, torch.where(x >= 128, x, torch.full_like(x, 255)))
    k = torch.full_like(x, 201)
    m = capi.pooling_param_spec(POOLING_MEAN, 2, 2, 2, 2, 0, 0, 0, 0)
    z, _ = host_pool.pooling_u8(k, n, c, ih, iw, m, 4.0, 56, 56)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert bool((z == 201).all())


def test_concat_full_size_properties(torch_mod):
    """Two 32 x 256 x 56 x 56 NCHWC16 tensors joined along the channels: each half of the result is the
    stand-alone requantisation of that input to the smaller scale (requantize_gfx950, pinned elsewhere)."""
    torch = torch_mod
    from bolt_amd import host
    n, c, h, w = 32, 256, 56, 56
    g = torch.Generator(device="cuda").manual_seed(9)
    a = torch.randint(-128, 128, (n * c * h * w,), dtype=torch.int8, device="cuda", generator=g)
    b = torch.randint(-128, 128, (n * c * h * w,), dtype=torch.int8, device="cuda", generator=g)
    d = tensor4df(DT_I8, DF_NCHWC16, n, c, h, w)
    out, s = host_pool.concat([a, b], [d, d], 1, tensor4df(DT_I8, DF_NCHWC16, n, 2 * c, h, w), [9.0, 6.5])
    ra = host.requantize(a, 9.0, 6.5)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    o = out.view(torch.int8).view(n, 2, c * h * w)
    assert s == np.float32(6.5)
    assert torch.equal(o[:, 0].reshape(-1), ra.view(torch.int8).reshape(-1)) and torch.equal(o[:, 1].reshape(-1), b)
