"""GPU parity of the int8 FullyConnected operator (x86 branch of the reference's fully_connected())
against the CPU oracle, whose composition was itself checked bit for bit against the reference's
compiled functions. Includes BASELINE configs[0]: M=64, K=1024, N=1024, fp32 bias, fp32 output."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import DF_NKN32K4, DF_NKNxKx, DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I32, DT_U8_Q  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def make_case(oracle, M, K, N, seed):
    rng = np.random.default_rng(seed)
    x = rng.standard_normal((M, K)).astype(np.float32)
    xq, sI = oracle.quantize_f32(x, DT_U8_Q)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
    sW = np.float32(1.0) / np.float32(0.01)
    return xq, sI, W, sW, bias


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("M,K,N", [(64, 1024, 1024), (1, 1024, 1024), (1, 77, 100), (5, 40, 33), (128, 768, 768),
                                   (16, 2048, 1024), (256, 3072, 768), (320, 1024, 512)])  # the last three: few rows, K deep enough for the column-panel kernel to be chosen over tiles
def test_fully_connected(torch_mod, oracle, device_mode, M, K, N):
    torch = torch_mod
    xq, sI, W, sW, bias = make_case(oracle, M, K, N, 20240601 + M)
    if M == 1:
        blob, _ = host.mvm_transform_weight(W, DF_NORMAL, N, K)
        fdf = DF_NKN32K4
    else:
        blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
        fdf = DF_NKNxKx

    def put(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda() if device_mode else np.ascontiguousarray(a)

    def get(t):
        if device_mode:
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            return t.cpu().numpy()
        return t
    dx, dblob, dbias = put(xq), put(blob), put(bias)
    for b, db in ((bias, dbias), (None, None)):
        out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_F32)
        want, wso = oracle.fully_connected(xq, sI, W, sW, b, DT_F32)
        assert so == wso and np.array_equal(get(out).view(np.int32), want.view(np.int32))
        out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_I32)
        want, _ = oracle.fully_connected(xq, sI, W, sW, b, DT_I32)
        assert np.array_equal(get(out), want)
        # u8 output, dynamic scale (int32 result -> stand-alone requantisation)
        out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_U8_Q, -1.0)
        want, wso = oracle.fully_connected(xq, sI, W, sW, b, DT_U8_Q, -1.0)
        assert so == wso and np.array_equal(get(out), want)
        # u8 output, known output scale (requantisation fused into the product's epilogue)
        out, so2 = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_U8_Q, float(wso))
        want, _ = oracle.fully_connected(xq, sI, W, sW, b, DT_U8_Q, float(wso))
        assert np.array_equal(get(out), want)


def test_fully_connected_rejects_unquantised_input(torch_mod):
    import ctypes as C
    L = capi.lib()
    x = np.zeros((2, 8), np.float32)
    blob, _, _ = host.mmm_transform_rhs(np.zeros((4, 8), np.int8), DF_TRANSPOSE, 8, 4)
    out = np.zeros((2, 4), np.float32)
    tmp = np.zeros(4096, np.uint8)
    so = C.c_float(-1)
    e = L.fully_connected_gfx950(capi.tensor2df(DT_F32, DF_NORMAL, 2, 8), host.ptr(x), 1.0,
                                 capi.tensor2df(capi.DT_I8, DF_NKNxKx, 8, 4), host.ptr(blob), 1.0,
                                 capi.tensor1d(DT_F32, 4), None, 4096, host.ptr(tmp),
                                 capi.tensor2df(DT_F32, DF_NORMAL, 2, 4), host.ptr(out), C.byref(so), capi.AMD_GFX950)
    assert e == capi.NOT_MATCH   # x86 requires DT_U8_Q activations (fully_connected.cpp:395)


def test_fully_connected_random_shapes(torch_mod, oracle):
    """Forty seeded random shapes (one row = the matrix-vector route, a few rows, a few hundred; K and N ragged, multiples
    of 8 and of 64) through every result type with and without a bias, against the CPU checker bit for bit."""
    torch = torch_mod
    rng = np.random.default_rng(20240608)

    def put(a):
        return torch.from_numpy(np.ascontiguousarray(a)).cuda()

    def get(t):
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return t.cpu().numpy()
    for it in range(40):
        M = int(rng.choice([1, 1, rng.integers(2, 20), rng.integers(20, 300), rng.choice([64, 128, 256, 320, 512])]))
        K = int(rng.choice([rng.integers(1, 100), 8 * rng.integers(1, 200), 64 * rng.integers(1, 40), rng.choice([768, 1024, 2048])]))
        N = int(rng.choice([rng.integers(1, 100), 8 * rng.integers(1, 150), rng.choice([256, 512, 768, 1024])]))
        print("fc random", it, M, K, N, flush=True)
        xq, sI, W, sW, bias = make_case(oracle, M, K, N, 7919 * it + 3)
        if M == 1:
            blob, _ = host.mvm_transform_weight(W, DF_NORMAL, N, K)
            fdf = DF_NKN32K4
        else:
            blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            fdf = DF_NKNxKx
        dx, dblob, dbias = put(xq), put(blob), put(bias)
        for b, db in ((bias, dbias), (None, None)):
            out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_F32)
            want, wso = oracle.fully_connected(xq, sI, W, sW, b, DT_F32)
            assert so == wso and np.array_equal(get(out).view(np.int32), want.view(np.int32)), (M, K, N, "f32")
            out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_I32)
            want, _ = oracle.fully_connected(xq, sI, W, sW, b, DT_I32)
            assert np.array_equal(get(out), want), (M, K, N, "i32")
            out, so = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_U8_Q, -1.0)
            want, wso = oracle.fully_connected(xq, sI, W, sW, b, DT_U8_Q, -1.0)
            assert so == wso and np.array_equal(get(out), want), (M, K, N, "u8 dynamic")
            out, _ = host.fully_connected(dx, sI, dblob, fdf, sW, db, M, K, N, DT_U8_Q, float(wso))
            want, _ = oracle.fully_connected(xq, sI, W, sW, b, DT_U8_Q, float(wso))
            assert np.array_equal(get(out), want), (M, K, N, "u8 static")
