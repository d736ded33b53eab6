"""Degenerate shapes through the C-ABI: empty operands return SUCCESS and touch nothing, K = 0 leaves
offsetC + C_in (an empty sum), single-element tensors quantise like any other. Device and host pointers."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import (DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I8, DT_I32, DT_U8_Q, tensor1d, tensor2df)  # noqa: E402
from test_gpu_blas import run_mmm, run_mvm  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


@pytest.mark.parametrize("device_mode", [False, True])
def test_mmm_degenerate_shapes(torch_mod, oracle, device_mode):
    rng = np.random.default_rng(3)
    for M, K, N in [(0, 16, 8), (5, 16, 0), (0, 0, 0), (3, 0, 5), (1, 1, 1), (2, 3, 1), (1, 7, 33)]:
        if device_mode and 0 in (M, K, N):
            continue  # torch hands out null pointers for empty tensors and a null operand is NULL_POINTER, as in the reference
        print("mmm edge", device_mode, M, K, N, flush=True)
        A = rng.integers(0, 256, size=(M, K), dtype=np.uint8)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        off = (oracle.offsetC(W, True) if N and K else np.zeros(N, np.int32)) + rng.integers(-50, 50, size=N, dtype=np.int32)
        Cin = rng.integers(-1000, 1000, size=(M, N), dtype=np.int32)
        # unpacked right-hand side: tmp receives the compensation the transform computes, so C = C_in + sum (a - 128) w
        got = run_mmm(torch_mod, device_mode, A, DF_NORMAL, W, DF_TRANSPOSE, M, K, N, None, Cin, DT_I32, None)
        comp = oracle.offsetC(W, True) if N and K else np.zeros(N, np.int32)
        want = oracle.mmm(A, W, comp, Cin, DT_I32) if M and N else Cin
        assert np.array_equal(got, want), (M, K, N)
        if K:
            blob, dt, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            got = run_mmm(torch_mod, device_mode, A, DF_NORMAL, blob, capi.DF_NKNxKx, M, K, N, off, Cin, DT_I32, None)
            want = oracle.mmm(A, W, off, Cin, DT_I32) if M and N else Cin
            assert np.array_equal(got, want), (M, K, N)


@pytest.mark.parametrize("device_mode", [False, True])
def test_quantize_degenerate_sizes(torch_mod, oracle, device_mode):
    for n in (0, 1, 2, 15, 16, 17):
        if device_mode and n == 0:
            continue
        print("quantize edge", device_mode, n, flush=True)
        x = (np.arange(n, dtype=np.float32) - 3.5) * 0.37
        for qdt in (DT_U8_Q, DT_I8):
            xin = torch_mod.from_numpy(x).cuda() if device_mode else x
            s = [-1.0]
            q = host.quantize(xin, DT_F32, qdt, s)
            if device_mode:
                capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
                q = q.cpu().numpy()
            if n:
                wq, ws = oracle.quantize_f32(x, qdt)
                assert np.array_equal(np.asarray(q).view(np.uint8), wq.view(np.uint8)) and np.float32(s[0]) == np.float32(ws)
            else:
                assert np.asarray(q).size == 0
