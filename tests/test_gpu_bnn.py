"""GPU parity of the 1-bit (XNOR / DoReFa) convolution against the CPU oracle, whose sums are pinned
against a brute-force +-1 / {0,1} convolution in test_oracle_conv.py (the reference's kernels for this
path are ARMv8.2 assembly and do not build on x86). Integer sums and the fp32 fma(S, scale, bias)
outputs are compared bit for bit. Includes BASELINE configs[4] (256 -> 256 channels, 28 x 28, 3 x 3,
batch 64): one image against the oracle, the whole batch through size-independent properties."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host_conv  # noqa: E402
from bolt_amd.capi import DF_NCHW, DF_NCHWN16C8, DT_BIN01, DT_BIN11, DT_F32, DT_I32  # noqa: E402
from checkers_conv import ConvOracle, bnn_pack_filter_nchwn16c8, to_nchwc  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.fixture(scope="module")
def co(oracle):
    return ConvOracle(oracle)


def make_case(shape, xnor, seed):
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    rng = np.random.default_rng(seed)
    if xnor:
        x = rng.standard_normal((n, ic, ih, iw)).astype(np.float32)
        w = rng.choice(np.array([-1.0, 1.0], np.float32), size=(oc, ic, fh, fw))
    else:
        x = rng.random((n, ic, ih, iw)).astype(np.float32)
        w = rng.integers(0, 2, size=(oc, ic, fh, fw)).astype(np.float32)
    scale = (rng.random(oc) * 0.1 + 0.01).astype(np.float32)
    bias = rng.standard_normal(oc).astype(np.float32)
    return x, w, scale, bias


def put(torch, device_mode, a):
    a = np.ascontiguousarray(a)
    return torch.from_numpy(a).cuda() if device_mode else a


def get(device_mode, t):
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return t.cpu().numpy()
    return t


def nchw_bitstring(w, xnor):
    bits = (w >= (0.0 if xnor else 0.5)).astype(np.uint8).reshape(-1)
    return np.packbits(bits)          # MSB first


SHAPES = [
    (1, 32, 5, 5, 32, 3, 3, 1, 1),
    (2, 64, 7, 6, 32, 3, 3, 1, 1),
    (1, 32, 9, 9, 64, 1, 1, 1, 0),
    (2, 96, 8, 8, 160, 3, 3, 2, 1),
    (1, 64, 11, 10, 96, 5, 5, 2, 2),
    (3, 128, 14, 14, 64, 3, 3, 1, 1),
]


@pytest.fixture(params=[2, 1, 0], ids=["matrix_cores_fp4", "matrix_cores_int8", "vector_alu"])
def route(request):
    """Every route of the 1-bit convolution: matrix cores on operands expanded to E2M1 pairs (default where
    the shape has that kernel, as configs[4] does; otherwise it is the int8 form), matrix cores on int8
    operands, and xor / popcount on the vector ALU."""
    L = capi.lib()
    capi.check(L.bolt_gfx950_set_option(b"bnn_mfma", request.param), "set_option")
    yield request.param
    capi.check(L.bolt_gfx950_set_option(b"bnn_mfma", 1), "set_option")


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("xnor", [True, False])
@pytest.mark.parametrize("shape", SHAPES)
def test_bnn_conv(torch_mod, co, route, device_mode, xnor, shape):
    print("bnn", route, device_mode, xnor, shape, flush=True)
    torch = torch_mod
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    fdt = DT_BIN11 if xnor else DT_BIN01
    x, w, scale, bias = make_case(shape, xnor, sum(shape) + int(xnor))
    d = co.bnn_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, xnor)
    x8 = to_nchwc(x, 8)
    bits = co.bnn_pack_input(d, x8)
    wb = bnn_pack_filter_nchwn16c8(w, xnor)
    want_s, want_f = co.bnn_conv(d, bits, wb, scale, bias)

    blob, ftm = host_conv.bnn_transform_filter(put(torch, device_mode, wb), fdt, DF_NCHWN16C8, oc, ic, fh, fw)
    blob2, _ = host_conv.bnn_transform_filter(put(torch, device_mode, nchw_bitstring(w, xnor)), fdt, DF_NCHW, oc, ic, fh, fw)
    assert np.array_equal(get(device_mode, blob), get(device_mode, blob2))
    sc, bs = put(torch, device_mode, scale), put(torch, device_mode, bias)
    # fp32 activations, binarised by the library
    got_f = get(device_mode, host_conv.convolution_bnn(put(torch, device_mode, x8.reshape(-1)), DT_F32, n, ic, ih, iw,
                                                       blob, ftm, oc, fh, fw, stride, pad, sc, bs, DT_F32))
    assert np.array_equal(got_f.view(np.int32), want_f.view(np.int32))
    # packed activations, integer sums out
    got_s = get(device_mode, host_conv.convolution_bnn(put(torch, device_mode, bits), fdt, n, ic, ih, iw, blob, ftm, oc,
                                                       fh, fw, stride, pad, sc, bs, DT_I32))
    assert np.array_equal(got_s, want_s)


def test_bnn_errors(torch_mod):
    lib = capi.lib()
    b = capi.C.c_uint32(0)
    fd = capi.tensor4df(DT_BIN11, DF_NCHW, 32, 32, 3, 3)
    assert lib.convolution_transform_filter_bytes_bnn_gfx950(fd, capi.C.byref(b), 0) == capi.NOT_SUPPORTED
    assert lib.convolution_transform_filter_bytes_bnn_gfx950(fd, None, capi.AMD_GFX950) == capi.NULL_POINTER
    assert lib.convolution_transform_filter_bytes_bnn_gfx950(fd, capi.C.byref(b), capi.AMD_GFX950) == 0
    # the bit-packed filter (the reference's size, rounded up to 256) + its int8 expansion (K = 288 -> 320, N = 32)
    # + its E2M1 expansion (K bytes = 144 -> 192)
    assert b.value == (32 * 32 * 9 // 8 + 255) // 256 * 256 + 320 * 32 + 192 * 32
    bad = capi.tensor4df(capi.DT_I8, DF_NCHW, 32, 32, 3, 3)
    assert lib.convolution_transform_filter_bytes_bnn_gfx950(bad, capi.C.byref(b), capi.AMD_GFX950) == capi.NOT_SUPPORTED
    w = np.zeros(48 * 32 * 9 // 8, np.uint8)
    out = np.zeros_like(w)
    ftm = capi.TensorDesc()
    fd48 = capi.tensor4df(DT_BIN11, DF_NCHW, 48, 32, 3, 3)   # oc not a multiple of 32
    assert lib.convolution_transform_filter_bnn_gfx950(fd48, w.ctypes.data, capi.C.byref(ftm), out.ctypes.data,
                                                       capi.AMD_GFX950) == capi.NOT_SUPPORTED


@pytest.mark.parametrize("xnor", [True, False])
def test_bnn_many_pixels_every_route(torch_mod, co, route, xnor):
    """44 x 28 x 28 pixels x 256 channels is 135 tiles of 256 pixels: enough for the E2M1 kernel to be
    chosen, which the small shapes above never reach. Whole result against the oracle, fp32 and sums,
    XNOR and DoReFa, fp32 and bit-packed input."""
    torch = torch_mod
    shape = (44, 32, 28, 28, 256, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    print("bnn many pixels", route, xnor, shape, flush=True)
    fdt = DT_BIN11 if xnor else DT_BIN01
    x, w, scale, bias = make_case(shape, xnor, 5 + int(xnor))
    d = co.bnn_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, xnor)
    x8 = to_nchwc(x, 8)
    bits = co.bnn_pack_input(d, x8)
    wb = bnn_pack_filter_nchwn16c8(w, xnor)
    want_s, want_f = co.bnn_conv(d, bits, wb, scale, bias)
    blob, ftm = host_conv.bnn_transform_filter(put(torch, True, wb), fdt, DF_NCHWN16C8, oc, ic, fh, fw)
    sc, bs = put(torch, True, scale), put(torch, True, bias)
    got_f = get(True, host_conv.convolution_bnn(put(torch, True, x8.reshape(-1)), DT_F32, n, ic, ih, iw, blob, ftm, oc,
                                                fh, fw, stride, pad, sc, bs, DT_F32))
    assert np.array_equal(got_f.view(np.int32), want_f.view(np.int32))
    got_s = get(True, host_conv.convolution_bnn(put(torch, True, bits), fdt, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride,
                                                pad, sc, bs, DT_I32))
    assert np.array_equal(got_s, want_s)


def test_bnn_config5_single_image(torch_mod, co, route):
    shape = (1, 256, 28, 28, 256, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    x, w, scale, bias = make_case(shape, True, 55)
    d = co.bnn_desc(n, ic, ih, iw, oc, fh, fw, stride, pad, True)
    x8 = to_nchwc(x, 8)
    wb = bnn_pack_filter_nchwn16c8(w, True)
    want_s, want_f = co.bnn_conv(d, co.bnn_pack_input(d, x8), wb, scale, bias)
    torch = torch_mod
    blob, ftm = host_conv.bnn_transform_filter(put(torch, True, wb), DT_BIN11, DF_NCHWN16C8, oc, ic, fh, fw)
    got = get(True, host_conv.convolution_bnn(put(torch, True, x8.reshape(-1)), DT_F32, n, ic, ih, iw, blob, ftm, oc, fh,
                                              fw, stride, pad, put(torch, True, scale), put(torch, True, bias), DT_F32))
    assert np.array_equal(got.view(np.int32), want_f.view(np.int32))


def test_bnn_config5_full_batch_properties(torch_mod, co, route):
    """Batch 64 at the full shape: (1) image 9 of the batch equals the same image run alone and the
    oracle; (2) flipping every activation bit negates every XNOR sum whose window has no padding, and
    the sum of a window over an all-(+1) filter equals 2 * popcount(window) - taps * ic; (3) every sum
    has the parity of taps * ic and lies in [-taps*ic, taps*ic]."""
    torch = torch_mod
    shape = (64, 256, 28, 28, 256, 3, 3, 1, 1)
    n, ic, ih, iw, oc, fh, fw, stride, pad = shape
    x, w, scale, bias = make_case(shape, True, 77)
    w[0] = 1.0                       # output channel 0: all +1
    x8 = to_nchwc(x, 8)
    wb = bnn_pack_filter_nchwn16c8(w, True)
    blob, ftm = host_conv.bnn_transform_filter(put(torch, True, wb), DT_BIN11, DF_NCHWN16C8, oc, ic, fh, fw)
    sc, bs = put(torch, True, scale), put(torch, True, bias)
    xd = put(torch, True, x8.reshape(-1))
    s = get(True, host_conv.convolution_bnn(xd, DT_F32, n, ic, ih, iw, blob, ftm, oc, fh, fw, stride, pad, sc, bs, DT_I32))
    s = s.reshape(n, oc // 8, ih, iw, 8)
    per = ic * ih * iw
    one = get(True, host_conv.convolution_bnn(xd[9 * per:10 * per], DT_F32, 1, ic, ih, iw, blob, ftm, oc, fh, fw, stride,
                                              pad, sc, bs, DT_I32))
    assert np.array_equal(s[9].reshape(-1), one)
    d1 = co.bnn_desc(1, ic, ih, iw, oc, fh, fw, stride, pad, True)
    want1, _ = co.bnn_conv(d1, co.bnn_pack_input(d1, x8[9:10]), wb, scale, bias)
    assert np.array_equal(one, want1)
    taps = fh * fw * ic
    assert s.max() <= taps and s.min() >= -taps and np.all((s - taps) % 2 == 0)
    neg = get(True, host_conv.convolution_bnn(put(torch, True, (-x8).reshape(-1) - np.float32(1e-30)), DT_F32, n, ic, ih,
                                              iw, blob, ftm, oc, fh, fw, stride, pad, sc, bs, DT_I32))
    neg = neg.reshape(s.shape)
    assert np.array_equal(neg[:, :, 1:-1, 1:-1], -s[:, :, 1:-1, 1:-1])
    # all-(+1) filter: sum over the window of (+1 / -1) activations
    pm = np.where(x >= 0, 1, -1).astype(np.int32).sum(1)        # [n][ih][iw]
    box = sum(pm[:, 1 + dy:ih - 1 + dy, 1 + dx:iw - 1 + dx] for dy in (-1, 0, 1) for dx in (-1, 0, 1))
    assert np.array_equal(s[:, 0, 1:-1, 1:-1, 0], box)
