"""GPU parity tests for the int8 GEMM / GEMV C-ABI against the CPU oracle: bit-exact int32, u8 and
fp32 outputs (fp32 is a single multiply of an exact int32 conversion, so it is compared bit for bit,
stricter than the 1e-6 relative the path asks for). Both pointer conventions are exercised:
numpy buffers (host pointers, AMD_GFX950) and torch CUDA tensors (device pointers,
AMD_GFX950_DEVICE)."""
import itertools
import sys

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import (DF_NKN32K4, DF_NKNxKx, DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I8, DT_I32, DT_U8_Q, tensor1d,
                           tensor2df)  # noqa: E402

EDGE = [1, 2, 7, 8, 9, 15, 16, 17, 31, 32, 33, 47, 48, 49, 63, 64, 65]
NP_OF = {DT_I32: np.int32, DT_F32: np.float32, DT_U8_Q: np.uint8}


def say(*a):
    print(*a, flush=True)
    sys.stdout.flush()


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def dev(torch, a):
    return torch.from_numpy(np.ascontiguousarray(a)).cuda()


def run_mmm(torch, device_mode, A, adf, B, bdf, M, K, N, offsetC, Cin, cdt, scale):
    """Reference call order: tmp bytes -> offsetC at the head of tmp -> multiply."""
    ad = tensor2df(DT_U8_Q, DF_TRANSPOSE, K, M) if adf == DF_TRANSPOSE else tensor2df(DT_U8_Q, DF_NORMAL, M, K)
    bd = host.rhs_desc(bdf, K, N)
    tmpBytes = host.mmm_tmp_bytes(ad, bd) + M * N * 4
    tmp = np.zeros(tmpBytes, np.uint8)
    if offsetC is not None:
        tmp[:4 * N] = np.ascontiguousarray(offsetC, dtype=np.int32).view(np.uint8)
    Cbuf = np.array(Cin, dtype=NP_OF[cdt]).reshape(M, N).copy()
    cd = tensor2df(cdt, DF_NORMAL, M, N)
    if device_mode:
        dA, dB, dT, dC = dev(torch, A), B if hasattr(B, "data_ptr") else dev(torch, B), dev(torch, tmp), dev(torch, Cbuf)
        e = host.matrix_matrix_multiply(dA, ad, dB, bd, dT, dC, cd, scale)
        capi.check(e, "mmm")
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return dC.cpu().numpy()
    Bh = B.cpu().numpy() if hasattr(B, "data_ptr") else B
    e = host.matrix_matrix_multiply(np.ascontiguousarray(A), ad, np.ascontiguousarray(Bh), bd, tmp, Cbuf, cd, scale)
    capi.check(e, "mmm")
    return Cbuf


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("bfmt", ["packed", "normal", "transpose"])
@pytest.mark.parametrize("transA", [False, True])
def test_mmm_i32_edges(torch_mod, oracle, device_mode, bfmt, transA):
    rng = np.random.default_rng(17 + device_mode + 2 * transA)
    shapes = list(itertools.product(EDGE, [1, 7, 8, 9, 16, 33, 64, 65, 130], EDGE))
    step = 23 if not device_mode else 7
    say("mmm i32 edges", device_mode, bfmt, transA, len(shapes[::step]))
    for M, K, N in shapes[::step]:
        A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        Cin = rng.integers(-1000, 1000, size=(M, N), dtype=np.int32)
        off = oracle.offsetC(W, True)
        Aarg = np.ascontiguousarray(A.T) if transA else A
        adf = DF_TRANSPOSE if transA else DF_NORMAL
        if bfmt == "packed":
            blob, dt, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            offb = off + rng.integers(-9999, 9999, size=N, dtype=np.int32)   # caller-folded bias
            got = run_mmm(torch_mod, device_mode, Aarg, adf, blob, DF_NKNxKx, M, K, N, offb, Cin, DT_I32, None)
            want = oracle.mmm(Aarg, W, offb, Cin, DT_I32, transA=transA)
        elif bfmt == "transpose":
            got = run_mmm(torch_mod, device_mode, Aarg, adf, W, DF_TRANSPOSE, M, K, N, None, Cin, DT_I32, None)
            want = oracle.mmm(Aarg, W, off, Cin, DT_I32, transA=transA)
        else:
            got = run_mmm(torch_mod, device_mode, Aarg, adf, np.ascontiguousarray(W.T), DF_NORMAL, M, K, N, None, Cin,
                          DT_I32, None)
            want = oracle.mmm(Aarg, W, off, Cin, DT_I32, transA=transA)
        assert np.array_equal(got, want), (M, K, N)


@pytest.mark.parametrize("M,K,N", [(3, 4095, 48), (5, 4097, 50), (2, 8200, 17), (385, 9, 49), (64, 1024, 1024),
                                   (128, 768, 768), (200, 136, 264)])
def test_mmm_all_outputs_device(torch_mod, oracle, M, K, N):
    say("mmm outputs", M, K, N)
    rng = np.random.default_rng(M * 7 + K)
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    off = oracle.offsetC(W, True) + rng.integers(-5000, 5000, size=N, dtype=np.int32)
    blob, dt, rhs = host.mmm_transform_rhs(dev(torch_mod, W), DF_TRANSPOSE, K, N)   # device-side pack kernel
    hblob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)                     # host-side pack
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert np.array_equal(blob.cpu().numpy()[:rhs + 4 * N], hblob[:rhs + 4 * N])
    Cin = rng.integers(-99, 99, size=(M, N), dtype=np.int32)
    got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, Cin, DT_I32, None)
    assert np.array_equal(got, oracle.mmm(A, W, off, Cin, DT_I32))
    s = np.float32(37.25)
    z = np.zeros((M, N), np.float32)
    got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, z, DT_F32, [s])
    want = oracle.mmm(A, W, off, z, DT_F32, scale=[s])
    assert np.array_equal(got.view(np.int32), want.view(np.int32))
    acc = oracle.mmm(A, W, off, np.zeros((M, N), np.int32), DT_I32)
    r = np.float32(127.0 / max(1, np.abs(acc).max()))
    zu = np.zeros((M, N), np.uint8)
    got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, zu, DT_U8_Q, [-1, r])
    assert np.array_equal(got, oracle.mmm(A, W, off, zu, DT_U8_Q, scale=[-1, r]))
    # DT_I32 output ignores a scale pointer (mmm.cpp:222-224)
    got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, Cin, DT_I32, [s])
    assert np.array_equal(got, oracle.mmm(A, W, off, Cin, DT_I32))


@pytest.mark.parametrize("tile", [0, 2, 7, 10, 11, 12, 13, 14, 15, 16])
def test_mmm_every_kernel_variant(torch_mod, oracle, tile):
    """Each GEMM kernel (general, register-staged tiles, LDS-DMA pipelines) is forced in turn on
    shapes with ragged M / N edges, one and many K tiles, and all four epilogues."""
    L = capi.lib()
    rng = np.random.default_rng(tile)
    try:
        capi.check(L.bolt_gfx950_set_option(b"gemm_tile", tile), "set_option")
        for M, K, N in [(1, 64, 16), (130, 128, 70), (256, 64, 256), (300, 256, 200), (257, 192, 513),
                        (512, 1024, 384), (100, 1040, 48), (260, 384, 300), (40, 896, 272), (512, 1536, 512),
                        (300, 768, 600), (128, 576, 128), (200, 448, 130), (129, 832, 257)]:
            say("variant", tile, M, K, N)
            A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
            W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
            off = oracle.offsetC(W, True) + rng.integers(-5000, 5000, size=N, dtype=np.int32)
            blob, dt, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            Cin = rng.integers(-99, 99, size=(M, N), dtype=np.int32)
            got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, Cin, DT_I32, None)
            assert np.array_equal(got, oracle.mmm(A, W, off, Cin, DT_I32)), (M, K, N)
            s = np.float32(3.5)
            z = np.zeros((M, N), np.float32)
            got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, z, DT_F32, [s])
            assert np.array_equal(got.view(np.int32), oracle.mmm(A, W, off, z, DT_F32, scale=[s]).view(np.int32))
            acc = oracle.mmm(A, W, off, np.zeros((M, N), np.int32), DT_I32)
            r = np.float32(127.0 / max(1, np.abs(acc).max()))
            zu = np.zeros((M, N), np.uint8)
            got = run_mmm(torch_mod, True, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, off, zu, DT_U8_Q, [-1, r])
            assert np.array_equal(got, oracle.mmm(A, W, off, zu, DT_U8_Q, scale=[-1, r])), (M, K, N)
    finally:
        L.bolt_gfx950_set_option(b"gemm_tile", -1)


@pytest.mark.parametrize("shape", [(4096, 3072, 768), (4096, 768, 768), (2048, 4096, 4096), (8192, 1024, 1024),
                                   (256, 3072, 768), (16, 4096, 4096)])
def test_mmm_variants_agree_at_full_size(torch_mod, oracle, shape):
    """The shapes whose kernel the launcher picks by measurement (128 x 128 tiles in pinned order, the two-group form,
    256 x 256 tiles, the few-rows kernel): at full size every variant and the launcher's own choice must give the same
    int32 and the same u8 bytes, and a sample of rows must equal the oracle."""
    torch = torch_mod
    M, K, N = shape
    L = capi.lib()
    g = torch.Generator(device="cuda").manual_seed(M + K + N)
    A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device="cuda", generator=g)
    W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
    off = blob[rhs:rhs + 4 * N].clone()
    ad = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
    r = np.float32(1.0 / (64.0 * np.sqrt(K)))
    outs = {}
    try:
        for tile in (-1, 12, 13, 14, 15, 16):
            say("full-size variant", tile, M, K, N)
            capi.check(L.bolt_gfx950_set_option(b"gemm_tile", tile), "set_option")
            Ci = torch.zeros((M, N), dtype=torch.int32, device="cuda")
            capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Ci, tensor2df(DT_I32, DF_NORMAL, M, N), None), "mmm i32")
            Cu = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
            capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Cu, tensor2df(DT_U8_Q, DF_NORMAL, M, N), [-1, r]), "mmm u8")
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            outs[tile] = (Ci, Cu)
    finally:
        L.bolt_gfx950_set_option(b"gemm_tile", -1)
    for tile, (Ci, Cu) in outs.items():
        assert torch.equal(Ci, outs[13][0]), tile
        assert torch.equal(Cu, outs[13][1]), tile
    rows = np.unique(np.concatenate([[0, M - 1], np.random.default_rng(1).integers(0, M, 6)]))
    Ah, Wh, offh = A[torch.from_numpy(rows).cuda()].cpu().numpy(), W.cpu().numpy(), off.cpu().numpy().view(np.int32)
    want = oracle.mmm(Ah, Wh, offh, np.zeros((len(rows), N), np.int32), DT_I32)
    assert np.array_equal(outs[-1][0].cpu().numpy()[rows], want)
    wantu = oracle.mmm(Ah, Wh, offh, np.zeros((len(rows), N), np.uint8), DT_U8_Q, scale=[-1, r])
    assert np.array_equal(outs[-1][1].cpu().numpy()[rows], wantu)


def test_mmm_launcher_choice_equals_general_kernel(torch_mod):
    """Sixty random shapes (few rows to 2 048, 1 to 4 096 columns, K a multiple of 16 or 64 up to 4 480) through whatever
    kernel the launcher picks -- few-rows kernel, 128 x 128 tiles, two-group form, 256 x 256 tiles, register-staged tiles
    -- against the plain general kernel: the same int32 (accumulating into C), fp32 and u8 bits."""
    torch = torch_mod
    L = capi.lib()
    rng = np.random.default_rng(11)
    g = torch.Generator(device="cuda").manual_seed(5)
    try:
        for it in range(60):
            M = int(rng.choice([rng.integers(1, 20), rng.integers(20, 300), rng.integers(300, 1200), rng.choice([128, 256, 512, 1024, 2048])]))
            N = int(rng.choice([rng.integers(1, 80), rng.integers(80, 600), rng.integers(600, 1500), rng.choice([256, 512, 768, 1024, 2304, 3072, 4096])]))
            K = int(rng.choice([64 * rng.integers(1, 12), 64 * rng.integers(12, 70), rng.choice([768, 1024, 2048, 3072, 4096]), 16 * rng.integers(4, 100)]))
            say("launcher choice", it, M, K, N)
            A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device="cuda", generator=g)
            W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
            blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            off = blob[rhs:rhs + 4 * N].clone()
            ad = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
            r = np.float32(1.0 / (64.0 * np.sqrt(K)))
            outs = []
            for tile in (-1, 0):
                capi.check(L.bolt_gfx950_set_option(b"gemm_tile", tile), "set_option")
                Ci = torch.full((M, N), 7, dtype=torch.int32, device="cuda")
                capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Ci, tensor2df(DT_I32, DF_NORMAL, M, N), None), "i32")
                Cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
                capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Cf, tensor2df(DT_F32, DF_NORMAL, M, N), [3.5]), "f32")
                Cu = torch.zeros((M, N), dtype=torch.uint8, device="cuda")
                capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Cu, tensor2df(DT_U8_Q, DF_NORMAL, M, N), [-1, r]), "u8")
                capi.check(L.bolt_gfx950_synchronize(), "sync")
                outs.append((Ci, Cf.view(torch.int32), Cu))
            for a_, b_ in zip(outs[0], outs[1]):
                assert torch.equal(a_, b_), (M, K, N)
    finally:
        L.bolt_gfx950_set_option(b"gemm_tile", -1)


def test_mmm_full_size_properties(torch_mod, oracle):
    """At the square-sweep size (4096^3) the oracle would take minutes, so the result is pinned by
    size-independent properties: linearity in A (A1 + A2 in the signed domain), rows reproduced by
    the GEMV kernel, and exact agreement on a random sample of outputs."""
    torch = torch_mod
    M = K = N = 4096
    g = torch.Generator(device="cuda").manual_seed(7)
    A1 = torch.randint(0, 128, (M, K), dtype=torch.uint8, device="cuda", generator=g)
    A2 = torch.randint(0, 128, (M, K), dtype=torch.uint8, device="cuda", generator=g)
    W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
    off = blob[rhs:rhs + 4 * N].clone()
    ad, cd = tensor2df(DT_U8_Q, DF_NORMAL, M, K), tensor2df(DT_I32, DF_NORMAL, M, N)

    def mm(A):
        C = torch.zeros((M, N), dtype=torch.int32, device="cuda")
        capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, C, cd, None), "mmm")
        return C
    C1, C2, C12 = mm(A1), mm(A2), mm(A1 + A2)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    # sum (a-128) w is affine in a: C(A1+A2) = C(A1) + C(A2) + 128 * colsum(W) = C1 + C2 - offsetC
    assert torch.equal(C12, C1 + C2 - off.view(torch.int32)[None, :])
    Wh, offh = W.cpu().numpy(), off.cpu().numpy().view(np.int32)
    rows = [0, 1, 255, 256, 2047, 4095]
    want = oracle.mmm(A1[rows].cpu().numpy(), Wh, offh, np.zeros((len(rows), N), np.int32), DT_I32)
    assert np.array_equal(C1[rows].cpu().numpy(), want)


@pytest.mark.parametrize("cdt,scale", [(DT_I32, None), (DT_F32, [37.25])])
def test_mmm_large_result_streamed(torch_mod, oracle, cdt, scale):
    """A result above 96 MiB is written with streaming stores (a different epilogue instantiation):
    5184 x 5184 x 4 bytes, K = 64 so that the oracle still finishes in seconds; C_in non-zero."""
    torch = torch_mod
    M = N = 5184
    K = 64
    rng = np.random.default_rng(5184)
    A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    off = oracle.offsetC(W, True) + rng.integers(-5000, 5000, size=N, dtype=np.int32)
    Cin = rng.integers(-100000, 100000, size=(M, N), dtype=np.int32)
    blob, bd, rhs = host.mmm_transform_rhs(torch.from_numpy(W).cuda(), DF_TRANSPOSE, K, N)
    Cd = torch.from_numpy(Cin.copy()).cuda()
    if cdt == DT_F32:
        Cd = Cd.view(torch.float32)
    say("streamed result", M, K, N, cdt)
    capi.check(host.matrix_matrix_multiply(torch.from_numpy(A).cuda(), tensor2df(DT_U8_Q, DF_NORMAL, M, K), blob, bd,
                                           torch.from_numpy(off).cuda().view(torch.uint8), Cd,
                                           tensor2df(cdt, DF_NORMAL, M, N), scale), "mmm")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    want = oracle.mmm(A, W, off, Cin.view(np.float32) if cdt == DT_F32 else Cin, cdt, scale=scale)
    assert np.array_equal(Cd.cpu().numpy().view(np.int32), want.view(np.int32))


def test_mmm_u8_epilogue_ties_and_saturation(torch_mod, oracle):
    M, K, N = 16, 8, 16
    A = np.full((M, K), 128, np.uint8)
    W = np.zeros((N, K), np.int8)
    blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
    accs = np.array([524289, 524288, 1572864, -524288, 1, -1, 0, 300 << 20, -(140 << 20), -(129 << 20),
                     -(128 << 20) - (1 << 19), 127 << 20, (127 << 20) + (1 << 19), 255 << 20, -(1 << 31),
                     (1 << 31) - 1], np.int64).astype(np.int32)
    r = np.float32(2.0 ** -20)
    zu = np.zeros((M, N), np.uint8)
    for mode in (False, True):
        got = run_mmm(torch_mod, mode, A, DF_NORMAL, blob, DF_NKNxKx, M, K, N, accs, zu, DT_U8_Q, [-1, r])
        assert np.array_equal(got, oracle.mmm(A, W, accs, zu, DT_U8_Q, scale=[-1, r]))
        assert got[0, 0] == 129 and got[0, 8] == 255 and got[0, 7] == 255


def run_mvm(torch, device_mode, W, mdesc, x, N, K, offsetC, yin, scale, vdt=DT_U8_Q, ydt=DT_I32):
    tmpBytes = host.mvm_tmp_bytes(mdesc, tensor1d(vdt, K)) + 2 * N * 4 + N * K + 64
    tmp = np.zeros(tmpBytes, np.uint8)
    if offsetC is not None:
        tmp[:4 * N] = np.ascontiguousarray(offsetC, dtype=np.int32).view(np.uint8)
    y = np.array(yin, dtype=NP_OF[ydt]).reshape(N).copy()
    vd, rd = tensor1d(vdt, K), tensor1d(ydt, N)
    if device_mode:
        dW = W if hasattr(W, "data_ptr") else dev(torch, W)
        dx, dT, dy = dev(torch, x), dev(torch, tmp), dev(torch, y)
        capi.check(host.matrix_vector_multiply(dW, mdesc, dx, vd, dT, dy, rd, scale), "mvm")
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        return dy.cpu().numpy()
    Wh = W.cpu().numpy() if hasattr(W, "data_ptr") else np.ascontiguousarray(W)
    capi.check(host.matrix_vector_multiply(Wh, mdesc, np.ascontiguousarray(x), vd, tmp, y, rd, scale), "mvm")
    return y


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("wfmt", ["packed", "normal", "transpose"])
def test_mvm_edges(torch_mod, oracle, device_mode, wfmt):
    rng = np.random.default_rng(7 + device_mode)
    Ns = [1, 2, 3, 7, 8, 9, 15, 16, 17, 31, 33, 63, 64, 65, 100, 200]
    Ks = [1, 2, 3, 4, 7, 8, 9, 15, 16, 17, 77, 1023, 1024, 1025, 2049, 4100]
    combos = list(itertools.product(Ns, Ks))[::(1 if device_mode else 3)]
    say("mvm edges", device_mode, wfmt, len(combos))
    for N, K in combos:
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        x = rng.integers(0, 256, size=K, dtype=np.uint8)
        yin = rng.integers(-500, 500, size=N, dtype=np.int32)
        if wfmt == "packed":
            blob, dt = host.mvm_transform_weight(W, DF_NORMAL, N, K)
            off = oracle.offsetC(W, True) + rng.integers(-3000, 3000, size=N, dtype=np.int32)
            args = (blob, host.mvm_desc(DF_NKN32K4, N, K), x, N, K, off)
        elif wfmt == "normal":
            off = oracle.offsetC(W, True)
            args = (W, host.mvm_desc(DF_NORMAL, N, K), x, N, K, None)
        else:
            off = oracle.offsetC(W, True)
            args = (np.ascontiguousarray(W.T), host.mvm_desc(DF_TRANSPOSE, N, K), x, N, K, None)
        got = run_mvm(torch_mod, device_mode, *args, yin, None)
        assert np.array_equal(got, oracle.mvm(W, x, off, yin, DT_I32)), (N, K)
        s = np.float32(11.5)
        z = np.zeros(N, np.float32)
        got = run_mvm(torch_mod, device_mode, *args, z, [s], ydt=DT_F32)
        assert np.array_equal(got.view(np.int32), oracle.mvm(W, x, off, z, DT_F32, scale=[s]).view(np.int32)), (N, K)
        if wfmt == "packed":   # u8 output is defined on the pre-packed route only (see test_oracle_vs_ref)
            r = np.float32(0.004)
            zu = np.zeros(N, np.uint8)
            got = run_mvm(torch_mod, device_mode, *args, zu, [-1, r], ydt=DT_U8_Q)
            assert np.array_equal(got, oracle.mvm(W, x, off, zu, DT_U8_Q, scale=[-1, r])), (N, K)


def test_mvm_decode_shape_and_device_pack(torch_mod, oracle):
    rng = np.random.default_rng(4096)
    N = K = 4096
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    blob, dt = host.mvm_transform_weight(dev(torch_mod, W), DF_NORMAL, N, K)
    off = oracle.offsetC(W, True)
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert np.array_equal(blob.cpu().numpy()[N * K:N * K + 4 * N].view(np.int32), off)
    for seed in range(4):
        x = np.random.default_rng(seed).integers(0, 256, size=K, dtype=np.uint8)
        z = np.zeros(N, np.int32)
        got = run_mvm(torch_mod, True, blob, host.mvm_desc(DF_NKN32K4, N, K), x, N, K, off, z, None)
        assert np.array_equal(got, oracle.mvm(W, x, off, z, DT_I32))
        # misaligned activation vector (byte-granular path)
        xx = dev(torch_mod, np.concatenate([[0], x]).astype(np.uint8))[1:]
        tmp = dev(torch_mod, off)
        y = torch_mod.zeros(N, dtype=torch_mod.int32, device="cuda")
        capi.check(host.matrix_vector_multiply(blob, host.mvm_desc(DF_NKN32K4, N, K), xx, tensor1d(DT_U8_Q, K),
                                               tmp.view(torch_mod.uint8), y, tensor1d(DT_I32, N), None), "mvm")
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        assert np.array_equal(y.cpu().numpy(), got)


@pytest.mark.parametrize("device_mode", [False, True])
def test_mvm_u8_matrix_s8_vector(torch_mod, oracle, device_mode):
    rng = np.random.default_rng(9)
    # includes shapes that take the vectorised kernels (rows: K % 16 == 0 rows, 16-byte aligned; K-major: M % 4 == 0)
    for M, K in list(itertools.product([1, 3, 4, 5, 8, 9, 17, 40], [1, 15, 16, 17, 63, 64, 65, 300])) + [
            (300, 512), (260, 1040), (1028, 96), (2048, 2048), (257, 4096)]:
        A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
        x = rng.integers(-127, 128, size=K, dtype=np.int8)
        yin = rng.integers(-500, 500, size=M, dtype=np.int32)
        got = run_mvm(torch_mod, device_mode, A, host.mvm_desc(DF_NORMAL, M, K, DT_U8_Q), x, M, K, None, yin, None,
                      vdt=DT_I8)
        assert np.array_equal(got, oracle.mvm_u8mat(A, x, yin, DT_I32)), (M, K)
        At = np.ascontiguousarray(A.T)
        got = run_mvm(torch_mod, device_mode, At, host.mvm_desc(DF_TRANSPOSE, M, K, DT_U8_Q), x, M, K, None, yin, None,
                      vdt=DT_I8)
        assert np.array_equal(got, oracle.mvm_u8mat(At, x, yin, DT_I32, a_is_KM=True)), (M, K)
        s = np.float32(3.0)
        z = np.zeros(M, np.float32)
        got = run_mvm(torch_mod, device_mode, A, host.mvm_desc(DF_NORMAL, M, K, DT_U8_Q), x, M, K, None, z, [s],
                      vdt=DT_I8, ydt=DT_F32)
        assert np.array_equal(got.view(np.int32), oracle.mvm_u8mat(A, x, z, DT_F32, scale=[s]).view(np.int32))


def test_per_channel_epilogue(torch_mod, oracle):
    """Per-output-channel weight scales + fp32 bias (not in the reference): closed form, and reduction
    to the reference's per-tensor result when all channel scales are equal."""
    torch = torch_mod
    rng = np.random.default_rng(5)
    L = capi.lib()
    for M, K, N in [(1, 256, 96), (7, 100, 33), (64, 1024, 1024)]:
        A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        off = oracle.offsetC(W, True)
        acc = oracle.mmm(A, W, off, np.zeros((M, N), np.int32), DT_I32)
        sI = np.float32(31.75)
        sW = (1.0 / rng.uniform(0.005, 0.02, size=N)).astype(np.float32)
        bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
        want = oracle.dequant_per_channel(acc, sI, sW, bias)
        blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
        dA, dB, dOff = dev(torch, A), dev(torch, blob), dev(torch, off)
        dsI, dsW, dbias = dev(torch, np.array([sI])), dev(torch, sW), dev(torch, bias)
        out = torch.zeros((M, N), dtype=torch.float32, device="cuda")
        capi.check(L.bolt_gfx950_mmm_int8_perchannel(M, N, K, dA.data_ptr(), dB.data_ptr(), dOff.data_ptr(),
                                                     out.data_ptr(), dsI.data_ptr(), dsW.data_ptr(), dbias.data_ptr()),
                   "mmm_perchannel")
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        assert np.array_equal(out.cpu().numpy().view(np.int32), want.view(np.int32))
        # all channels equal, no bias == reference per-tensor fp32 epilogue with scale = sI * sW
        sW1 = np.full(N, np.float32(100.0), np.float32)
        dsW1 = dev(torch, sW1)
        capi.check(L.bolt_gfx950_mmm_int8_perchannel(M, N, K, dA.data_ptr(), dB.data_ptr(), dOff.data_ptr(),
                                                     out.data_ptr(), dsI.data_ptr(), dsW1.data_ptr(), None), "mmm_pc")
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        ref = oracle.mmm(A, W, off, np.zeros((M, N), np.float32), DT_F32, scale=[sI * np.float32(100.0)])
        assert np.array_equal(out.cpu().numpy().view(np.int32), ref.view(np.int32))
        if M == 1:
            vblob, _ = host.mvm_transform_weight(W, DF_NORMAL, N, K)
            dV = dev(torch, vblob)
            y = torch.zeros(N, dtype=torch.float32, device="cuda")
            capi.check(L.bolt_gfx950_mvm_int8_perchannel(N, K, dV.data_ptr(), dA.data_ptr(), dOff.data_ptr(),
                                                         y.data_ptr(), dsI.data_ptr(), dsW.data_ptr(), dbias.data_ptr()),
                       "mvm_perchannel")
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            assert np.array_equal(y.cpu().numpy().view(np.int32), want[0].view(np.int32))


@pytest.mark.parametrize("tile", [-1, 0, 2, 7, 10, 11, 12, 13, 14, 15, 16])
def test_per_channel_u8_epilogue_every_kernel_variant(torch_mod, oracle, tile):
    """bolt_gfx950_mmm_int8_perchannel_u8 (not in the reference): the per-channel fp32 value -- the closed form that
    test_per_channel_epilogue holds against the reference's per-tensor epilogue -- put through the reference-pinned
    fp32 -> u8 quantiser with a static scale. Every kernel forced in turn, ragged and full tiles, with and without
    bias; equal to quantising the fp32 entry point's own output."""
    torch = torch_mod
    rng = np.random.default_rng(50 + tile)
    L = capi.lib()
    try:
        capi.check(L.bolt_gfx950_set_option(b"gemm_tile", tile), "set_option")
        for M, K, N in [(1, 64, 16), (130, 128, 70), (256, 64, 256), (257, 192, 513), (512, 1024, 384), (300, 768, 600),
                        (128, 576, 128), (512, 256, 512)]:
            say("per-channel u8", tile, M, K, N)
            A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
            W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
            off = oracle.offsetC(W, True)
            acc = oracle.mmm(A, W, off, np.zeros((M, N), np.int32), DT_I32)
            sI = np.float32(31.75)
            sW = (1.0 / rng.uniform(0.005, 0.02, size=N)).astype(np.float32)
            bias = (rng.standard_normal(N) * 0.1).astype(np.float32)
            blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            dA, dB, dOff = dev(torch, A), dev(torch, blob), dev(torch, off)
            dsI, dsW, dbias = dev(torch, np.array([sI])), dev(torch, sW), dev(torch, bias)
            for b, db in ((bias, dbias), (None, None)):
                f = oracle.dequant_per_channel(acc, sI, sW, b)
                so = np.float32(100.0 / max(1e-6, np.abs(f).max()))     # some values saturate at 1 / 255
                want, _ = oracle.quantize_f32(f, DT_U8_Q, so, 1)
                out = torch.full((M, N), 7, dtype=torch.uint8, device="cuda")
                capi.check(L.bolt_gfx950_mmm_int8_perchannel_u8(M, N, K, dA.data_ptr(), dB.data_ptr(), dOff.data_ptr(), out.data_ptr(),
                                                                dsI.data_ptr(), dsW.data_ptr(), db.data_ptr() if db is not None else None,
                                                                float(so)), "mmm_perchannel_u8")
                capi.check(L.bolt_gfx950_synchronize(), "sync")
                assert np.array_equal(out.cpu().numpy(), want), (tile, M, K, N, b is not None)
        assert L.bolt_gfx950_mmm_int8_perchannel_u8(1, 16, 64, dA.data_ptr(), dB.data_ptr(), dOff.data_ptr(), out.data_ptr(),
                                                    dsI.data_ptr(), dsW.data_ptr(), None, 0.0) == capi.NOT_MATCH
    finally:
        L.bolt_gfx950_set_option(b"gemm_tile", -1)


def _strided_batch_case(torch, oracle, N, K, batch, copies, with_bias, seed, pad=0):
    """One call of bolt_gfx950_mvm_int8_strided_batch checked row by row: slice b multiplies weight copy
    b % copies (every copy holds DIFFERENT weights, so a wrong copy index shows), has its own activation scale,
    shares the per-channel weight scales and the optional fp32 bias. Integer part: the reference's GEMV
    (mvm_avx512_vnni.cpp:703-759) on that copy; fp32 part: the per-channel closed form."""
    L = capi.lib()
    rng = np.random.default_rng(seed)
    Ws = rng.integers(-127, 128, size=(copies, N, K), dtype=np.int8)
    X = rng.integers(0, 256, size=(batch, K), dtype=np.uint8)
    sI = rng.uniform(5.0, 60.0, size=batch).astype(np.float32)
    sW = (1.0 / rng.uniform(0.005, 0.02, size=N)).astype(np.float32)
    bias = (rng.standard_normal(N) * 0.1).astype(np.float32) if with_bias else None
    blobs = [host.mvm_transform_weight(dev(torch, Ws[c]), DF_NORMAL, N, K)[0] for c in range(copies)]
    blob_bytes = (N + 15) // 16 * 16 * ((K + 7) // 8 * 8) + 4 * N
    stride = (blob_bytes + 255) // 256 * 256 + pad
    wbuf = torch.zeros(copies * stride, dtype=torch.uint8, device="cuda")
    for c in range(copies):
        wbuf[c * stride:c * stride + blob_bytes] = blobs[c][:blob_bytes]
    dX, dsI, dsW = dev(torch, X), dev(torch, sI), dev(torch, sW)
    dbias = dev(torch, bias) if with_bias else None
    y = torch.full((batch, N), float("nan"), dtype=torch.float32, device="cuda")
    capi.check(L.bolt_gfx950_mvm_int8_strided_batch(batch, N, K, wbuf.data_ptr(), stride, copies, dX.data_ptr(),
                                                    y.data_ptr(), dsI.data_ptr(), dsW.data_ptr(),
                                                    dbias.data_ptr() if with_bias else None), "mvm_strided_batch")
    capi.check(L.bolt_gfx950_synchronize(), "sync")
    got = y.cpu().numpy()
    offs = [oracle.offsetC(Ws[c], True) for c in range(copies)]
    zero = np.zeros(N, np.int32)
    for b in range(batch):
        c = b % copies
        acc = oracle.mvm(Ws[c], X[b], offs[c], zero, DT_I32)
        want = oracle.dequant_per_channel(acc.reshape(1, N), sI[b], sW, bias).reshape(-1)
        assert np.array_equal(got[b].view(np.int32), want.view(np.int32)), (N, K, batch, copies, with_bias, b)


@pytest.mark.parametrize("copies", [1, 3, 64])
@pytest.mark.parametrize("with_bias", [False, True], ids=["nobias", "bias"])
def test_mvm_strided_batch_decode_shape(torch_mod, oracle, copies, with_bias):
    """The benchmark's launch at its full shape: N = K = 4096, 256 vectors, rotating over `copies` weight blobs."""
    say("mvm_strided_batch", 4096, 4096, 256, copies, with_bias)
    _strided_batch_case(torch_mod, oracle, 4096, 4096, 256, copies, with_bias, seed=100 + copies)


@pytest.mark.parametrize("N,K,batch,copies", [(100, 77, 5, 2), (100, 77, 5, 1), (9, 1, 3, 3), (33, 4100, 7, 4),
                                               (16, 16, 1, 1), (257, 520, 300, 5)])
def test_mvm_strided_batch_ragged(torch_mod, oracle, N, K, batch, copies):
    """N % 16, K % 8 and K % 16 tails, fewer vectors than copies, more than 256 vectors, a stride with slack."""
    say("mvm_strided_batch ragged", N, K, batch, copies)
    _strided_batch_case(torch_mod, oracle, N, K, batch, copies, True, seed=N * 7 + K, pad=256)
    _strided_batch_case(torch_mod, oracle, N, K, batch, copies, False, seed=N * 7 + K + 1)


def test_mvm_strided_batch_arguments(torch_mod):
    L = capi.lib()
    torch = torch_mod
    t = torch.zeros(4096, dtype=torch.uint8, device="cuda")
    f = torch.zeros(64, dtype=torch.float32, device="cuda")
    p, q = t.data_ptr(), f.data_ptr()
    assert L.bolt_gfx950_mvm_int8_strided_batch(1, 16, 16, None, 0, 1, p, q, q, q, None) == capi.NULL_POINTER
    assert L.bolt_gfx950_mvm_int8_strided_batch(1, 16, 16, p, 0, 0, p, q, q, q, None) == capi.NOT_MATCH
    assert L.bolt_gfx950_mvm_int8_strided_batch(2, 16, 16, p, 16, 2, p, q, q, q, None) == capi.NOT_MATCH   # stride < blob
    assert L.bolt_gfx950_mvm_int8_strided_batch(2, 16, 16, p, 322, 2, p, q, q, q, None) == capi.NOT_MATCH  # stride % 4
    assert L.bolt_gfx950_mvm_int8_strided_batch(0, 16, 16, p, 0, 1, p, q, q, q, None) == capi.SUCCESS


def test_mmm_operand_of_four_gib_and_more(torch_mod):
    """A left-hand side of 4 GiB + 4 KiB (2^26 + 64 rows of 64 bytes): beyond what the tiled kernels address with their
    32-bit byte offsets, so the launcher must send it to the kernel that indexes with 64 bits -- through
    matrix_matrix_multiply with int32 and fp32 results, every row checked against an fp32 product of
    the same small integers (exact: every sum is below 2^24) taken in chunks."""
    torch = torch_mod
    M, K, N = (1 << 26) + 64, 64, 16
    g = torch.Generator(device="cuda")
    g.manual_seed(77)
    A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device="cuda", generator=g)
    W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device="cuda", generator=g)
    blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
    off = blob[rhs:rhs + 4 * N].clone()
    Ci = torch.zeros((M, N), dtype=torch.int32, device="cuda")
    print("mmm 4 GiB operand", M, K, N, flush=True)
    capi.check(host.matrix_matrix_multiply(A, tensor2df(DT_U8_Q, DF_NORMAL, M, K), blob, bd, off, Ci,
                                           tensor2df(DT_I32, DF_NORMAL, M, N), None), "mmm i32")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    Wf = W.to(torch.float32).t().contiguous()
    step = 1 << 22
    for lo in range(0, M, step):
        hi = min(M, lo + step)
        want = (A[lo:hi].to(torch.float32) - 128.0) @ Wf
        assert torch.equal(Ci[lo:hi], want.to(torch.int32)), (lo, hi)
    # an fp32 result of the same product (C += A.B on zeros, cvt(acc) * (1 / scale)) at the far end of the operand
    tail = slice(M - 4096, M)
    Cf = torch.zeros((M, N), dtype=torch.float32, device="cuda")
    capi.check(host.matrix_matrix_multiply(A, tensor2df(DT_U8_Q, DF_NORMAL, M, K), blob, bd, off, Cf,
                                           tensor2df(DT_F32, DF_NORMAL, M, N), [8.0]), "mmm f32")
    capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
    assert torch.equal(Cf[tail], Ci[tail].to(torch.float32) * (torch.tensor(1.0, device="cuda") / 8.0))
    del A, Ci, Cf
    torch.cuda.empty_cache()
