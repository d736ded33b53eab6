"""int8 matmul (batched) on the GPU against the oracle composed the way the reference composes it
(compute/tensor/src/matmul.cpp:401-431,495-554): whole-tensor quantisation of A (u8) and B (s8), then one
u8 x s8 product per 2-D slice with cvt(acc) * (1 / (sA * sB)). Bit-exact."""
import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import DT_F32, DT_I8, DT_I32, DT_U8_Q  # noqa: E402


@pytest.fixture(scope="module")
def torch_mod():
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    return torch


def oracle_matmul(oracle, A, tA, B, tB, cdt):
    """The oracle's composition (checkers.Oracle.matmul), itself pinned against the reference's matmul() in
    tests/test_oracle_orchestration.py and tests/golden/orchestration.npz."""
    return oracle.matmul(A, tA, B, tB, cdt)


CASES = [  # (A shape, transposeA, B shape, transposeB)
    ((5, 9), False, (9, 7), False),
    ((2, 3, 16, 64), False, (2, 3, 64, 16), False),          # attention-like: per-head Q x K^T with K stored [d, S]
    ((2, 3, 16, 64), False, (2, 3, 24, 64), True),           # B stored transposed [N, K]
    ((4, 33, 20), True, (4, 33, 17), False),                 # A stored [K, M]
    ((3, 128, 64), False, (64, 48), False),                  # B shared by all slices
    ((12, 128, 64), False, (12, 128, 64), True),             # BERT head: [128, 64] x [128, 64]^T
    ((2, 256, 128), False, (2, 128, 256), False),
]


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", CASES)
def test_matmul_int8(torch_mod, oracle, device_mode, case):
    torch = torch_mod
    a_shape, tA, b_shape, tB = case
    print("matmul", device_mode, case, flush=True)
    rng = np.random.default_rng(sum(a_shape) + sum(b_shape))
    A = rng.standard_normal(a_shape).astype(np.float32)
    B = rng.standard_normal(b_shape).astype(np.float32)
    M = a_shape[-1] if tA else a_shape[-2]
    N = b_shape[-2] if tB else b_shape[-1]
    lead = a_shape[:-2] if len(a_shape) >= len(b_shape) else b_shape[:-2]
    c_shape = tuple(lead) + (M, N)

    def put(x):
        return torch.from_numpy(np.ascontiguousarray(x)).cuda() if device_mode else np.ascontiguousarray(x)
    for cdt in (DT_F32, DT_I32):
        want, sa, sb = oracle_matmul(oracle, A, tA, B, tB, cdt)
        got = host.matmul(put(A), DT_F32, a_shape, tA, -1.0, put(B), DT_F32, b_shape, tB, -1.0, c_shape, cdt)
        if device_mode:
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            got = got.cpu().numpy()
        assert np.array_equal(got.reshape(want.shape).view(np.int32), want.view(np.int32)), (case, cdt)
    # operands handed over already quantised, with their scales
    qa, sa = oracle.quantize_f32(A.reshape(-1), DT_U8_Q)
    qb, sb = oracle.quantize_f32(B.reshape(-1), DT_I8)
    got = host.matmul(put(qa), DT_U8_Q, a_shape, tA, sa, put(qb), DT_I8, b_shape, tB, sb, c_shape, DT_F32)
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        got = got.cpu().numpy()
    want, _, _ = oracle_matmul(oracle, A, tA, B, tB, DT_F32)
    assert np.array_equal(got.reshape(want.shape).view(np.int32), want.view(np.int32))


def test_matmul_errors(torch_mod):
    L = capi.lib()
    nb = capi.C.c_uint32(0)
    a, b, c = host.tensor_nd(DT_F32, (4, 8)), host.tensor_nd(DT_F32, (9, 4)), host.tensor_nd(DT_F32, (4, 4))
    assert L.matmul_infer_forward_tmp_bytes_gfx950(a, False, b, False, c, capi.C.byref(nb), capi.AMD_GFX950) == capi.NOT_MATCH
    b = host.tensor_nd(DT_F32, (8, 4))
    assert L.matmul_infer_forward_tmp_bytes_gfx950(a, False, b, False, c, None, capi.AMD_GFX950) == capi.NULL_POINTER
    assert L.matmul_infer_forward_tmp_bytes_gfx950(a, False, b, False, c, capi.C.byref(nb), 0) == capi.NOT_SUPPORTED
    assert L.matmul_infer_forward_tmp_bytes_gfx950(a, False, b, False, c, capi.C.byref(nb), capi.AMD_GFX950) == 0
    x = np.zeros(32, np.float32)
    v = host.tensor_nd(DT_U8_Q, (8, 1))   # a vector result wants B as U8_Q (or fp32), not I8
    cv = host.tensor_nd(DT_F32, (4, 1))
    vi = host.tensor_nd(DT_I8, (8, 1))
    assert L.matmul_gfx950(a, False, x.ctypes.data, -1.0, vi, False, x.ctypes.data, 1.0, 1 << 20, x.ctypes.data, cv,
                           x.ctypes.data, capi.AMD_GFX950) == capi.NOT_SUPPORTED


def oracle_matmul_vector(oracle, A, tA, B, tB, cdt):
    return oracle.matmul_vector(A, tA, B, tB, cdt)


VECTOR_CASES = [  # (A shape, transposeA, B shape, transposeB): one of M, N is 1
    ((1, 64), False, (64, 48), False),                       # row vector x matrix
    ((1, 100), False, (37, 100), True),                      # ... with B stored [N, K]
    ((2, 3, 1, 64), False, (2, 3, 64, 128), False),          # decode-step attention scores: q [1, d] x K^T
    ((50, 72), False, (72, 1), False),                       # matrix x column vector
    ((72, 50), True, (72, 1), False),                        # ... with A stored [K, M]
    ((4, 130, 96), False, (4, 96, 1), False),
    ((3, 1, 40), False, (40, 1), False),                     # both: treated as the row-vector case
    ((2100, 256), False, (256, 1), False),                   # enough rows for the two-rows-per-wave kernel
]


@pytest.mark.parametrize("device_mode", [False, True])
@pytest.mark.parametrize("case", VECTOR_CASES)
def test_matmul_int8_vector_result(torch_mod, oracle, device_mode, case):
    torch = torch_mod
    a_shape, tA, b_shape, tB = case
    print("matmul vector", device_mode, case, flush=True)
    rng = np.random.default_rng(sum(a_shape) + 7 * sum(b_shape))
    A = rng.standard_normal(a_shape).astype(np.float32)
    B = rng.standard_normal(b_shape).astype(np.float32)
    M = a_shape[-1] if tA else a_shape[-2]
    N = b_shape[-2] if tB else b_shape[-1]
    lead = a_shape[:-2] if len(a_shape) >= len(b_shape) else b_shape[:-2]
    c_shape = tuple(lead) + (M, N)

    def put(x):
        return torch.from_numpy(np.ascontiguousarray(x)).cuda() if device_mode else np.ascontiguousarray(x)
    for cdt in (DT_F32, DT_I32):
        want, sa, sb = oracle_matmul_vector(oracle, A, tA, B, tB, cdt)
        got = host.matmul(put(A), DT_F32, a_shape, tA, -1.0, put(B), DT_F32, b_shape, tB, -1.0, c_shape, cdt)
        if device_mode:
            capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
            got = got.cpu().numpy()
        assert np.array_equal(got.reshape(want.shape).view(np.int32), want.reshape(want.shape).view(np.int32)), (case, cdt)
    qa, sa = oracle.quantize_f32(A.reshape(-1), DT_I8)
    qb, sb = oracle.quantize_f32(B.reshape(-1), DT_U8_Q)
    got = host.matmul(put(qa), DT_I8, a_shape, tA, sa, put(qb), DT_U8_Q, b_shape, tB, sb, c_shape, DT_F32)
    if device_mode:
        capi.check(capi.lib().bolt_gfx950_synchronize(), "sync")
        got = got.cpu().numpy()
    want, _, _ = oracle_matmul_vector(oracle, A, tA, B, tB, DT_F32)
    assert np.array_equal(got.reshape(want.shape).view(np.int32), want.view(np.int32))
