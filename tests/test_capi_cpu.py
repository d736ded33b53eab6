"""Host-side checks that need no GPU: the C-ABI library loads and exports every declared symbol, the
size queries reproduce the reference's formulas, the host-pointer weight transform produces the
observable contract (blob size, offsetC position and value, transformed descriptor), and argument
validation returns the reference's EE codes."""
import ctypes as C
import itertools
import os
import re

import numpy as np
import pytest

from bolt_amd import capi, host
from bolt_amd.capi import (AMD_GFX950, DF_NKN32K4, DF_NKNxKx, DF_NORMAL, DF_TRANSPOSE, DT_F32, DT_I8, DT_I32, DT_U8_Q,
                           tensor1d, tensor2df)

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def test_library_exports_every_declared_symbol():
    L = capi.lib()
    header = open(os.path.join(ROOT, "include", "bolt_gfx950.h")).read()
    header = re.sub(r"/\*.*?\*/", "", header, flags=re.S)
    declared = set(re.findall(r"\b([A-Za-z_][A-Za-z0-9_]*_gfx950|bolt_gfx950_[a-z0-9_]+)\s*\(", header))
    assert len(declared) >= 20
    for name in declared:
        assert hasattr(L, name), name
    assert declared == set(capi.SIGNATURES), declared ^ set(capi.SIGNATURES)


def test_tensor_desc_layout():
    d = tensor2df(DT_I8, DF_TRANSPOSE, 3, 5)
    assert C.sizeof(d) == 92 and d.nDims == 2 and d.dims[0] == 5 and d.dims[1] == 3
    raw = bytes(d)
    assert raw[:12] == np.array([1, 13, 2], np.uint32).tobytes()


def test_size_queries_match_oracle(oracle):
    for N, K in itertools.product([1, 7, 16, 17, 48, 100, 1024, 3072], [1, 7, 8, 9, 77, 768, 4097]):
        for df in (DF_NORMAL, DF_TRANSPOSE):
            assert host.mmm_transform_rhs_bytes(host.rhs_desc(df, K, N)) == oracle.mmm_transform_rhs_bytes(N, K)
            assert host.mvm_transform_weight_bytes(host.mvm_desc(df, N, K)) == oracle.mvm_transform_weight_bytes(N, K)
        assert host.mmm_transform_rhs_bytes(host.rhs_desc(DF_NKNxKx, K, N)) == (0, 0)
        assert host.mvm_transform_weight_bytes(host.mvm_desc(DF_NKN32K4, N, K)) == N * 4
        assert host.mvm_tmp_bytes(host.mvm_desc(DF_NKN32K4, N, K), tensor1d(DT_U8_Q, K)) == N * 4
        assert host.mvm_transform_weight_bytes(host.mvm_desc(DF_NORMAL, N, K, DT_U8_Q)) == \
            oracle.mvm_transform_weight_bytes(N, K, DT_U8_Q)
        for M, tA, pk in itertools.product([1, 5, 24, 25, 64, 385], [False, True], [False, True]):
            ad = tensor2df(DT_U8_Q, DF_TRANSPOSE, K, M) if tA else tensor2df(DT_U8_Q, DF_NORMAL, M, K)
            bd = host.rhs_desc(DF_NKNxKx if pk else DF_TRANSPOSE, K, N)
            assert host.mmm_tmp_bytes(ad, bd) == oracle.mmm_tmp_bytes(N, M, K, tA, pk)
    assert host.mmm_transform_rhs_bytes(host.rhs_desc(DF_TRANSPOSE, 1024, 1024)) == (1052736, 1048576)
    assert host.mvm_transform_weight_bytes(host.mvm_desc(DF_NORMAL, 4096, 4096)) == 16793632


def mmm_unpack(blob, N, K):
    """Independent restatement of the fragment layout: 16-column blocks of 16*Kp bytes, each holding
    Kp//16 fragments [n16][k16] and, when Kp % 16 == 8, one [n16][k8] fragment."""
    Kp, N16 = (K + 7) // 8 * 8, (N + 15) // 16 * 16
    out = np.zeros((N16, Kp), np.int8)
    b = blob[:N16 * Kp].view(np.int8).reshape(N16 // 16, 16 * Kp)
    full = Kp // 16
    for nb in range(N16 // 16):
        if full:
            frag = b[nb, :full * 256].reshape(full, 16, 16)          # [kb][n][k]
            out[nb * 16:(nb + 1) * 16, :full * 16] = frag.transpose(1, 0, 2).reshape(16, full * 16)
        if Kp % 16:
            out[nb * 16:(nb + 1) * 16, full * 16:] = b[nb, full * 256:].reshape(16, 8)
    return out


@pytest.mark.parametrize("N,K", [(1, 1), (16, 16), (17, 9), (48, 64), (100, 77), (33, 24), (64, 4104)])
def test_host_weight_transform_contract(oracle, N, K):
    rng = np.random.default_rng(N * 131 + K)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    want_off = oracle.offsetC(W, True)
    Kp, N16 = (K + 7) // 8 * 8, (N + 15) // 16 * 16
    for df, src in ((DF_TRANSPOSE, W), (DF_NORMAL, np.ascontiguousarray(W.T))):
        blob, dt, rhs = host.mmm_transform_rhs(src, df, K, N)
        assert rhs == N16 * Kp and blob.size == rhs + 4 * N + 64
        assert (dt.dt, dt.df, dt.nDims, dt.dims[0], dt.dims[1]) == (DT_I8, DF_NKNxKx, 2, N, K)
        assert np.array_equal(blob[rhs:rhs + 4 * N].view(np.int32), want_off)
        full = mmm_unpack(blob, N, K)
        assert np.array_equal(full[:N, :K], W) and not full[N:].any() and not full[:, K:].any()
    for df, src in ((DF_NORMAL, W), (DF_TRANSPOSE, np.ascontiguousarray(W.T))):
        blob, dt = host.mvm_transform_weight(src, df, N, K)
        assert blob.size == 4 * N + N16 * Kp + 32
        assert (dt.dt, dt.df, dt.nDims, dt.dims[0], dt.dims[1]) == (DT_I8, DF_NKN32K4, 2, K, N)
        assert np.array_equal(blob[N16 * Kp:N16 * Kp + 4 * N].view(np.int32), want_off)
        full = blob[:N16 * Kp].view(np.int8).reshape(N16, Kp)
        assert np.array_equal(full[:N, :K], W) and not full[N:].any() and not full[:, K:].any()


def test_transform_of_packed_input_is_a_no_op():
    L = capi.lib()
    dt = capi.TensorDesc()
    dt.df = 1234
    dst = np.full(8, 7, np.uint8)
    src = np.zeros(8, np.int8)
    assert L.matrix_matrix_multiply_transform_rhs_gfx950(host.rhs_desc(DF_NKNxKx, 2, 2), host.ptr(src), C.byref(dt),
                                                        host.ptr(dst), AMD_GFX950) == capi.SUCCESS
    assert L.matrix_vector_multiply_transform_weight_gfx950(host.mvm_desc(DF_NKN32K4, 2, 2), host.ptr(src), C.byref(dt),
                                                           host.ptr(dst), AMD_GFX950) == capi.SUCCESS
    assert dt.df == 1234 and (dst == 7).all()


def test_error_codes_follow_the_reference():
    L = capi.lib()
    a = np.zeros((4, 8), np.uint8)
    b = np.zeros(16 * 8 + 64 + 4 * 4, np.int8)
    c = np.zeros((4, 4), np.int32)
    tmp = np.zeros(1024, np.uint8)
    ad, bd, cd = tensor2df(DT_U8_Q, DF_NORMAL, 4, 8), host.rhs_desc(DF_NKNxKx, 8, 4), tensor2df(DT_I32, DF_NORMAL, 4, 4)
    mm = L.matrix_matrix_multiply_gfx950
    # unknown arch -> NOT_SUPPORTED without touching anything (mmm.cpp:199,237)
    assert mm(ad, host.ptr(a), bd, host.ptr(b), 1024, host.ptr(tmp), cd, host.ptr(c), None, capi.X86_AVX512) == \
        capi.NOT_SUPPORTED
    # null operands / tmp missing while bytes != 0 -> NULL_POINTER (mmm.cpp:161-166)
    assert mm(ad, None, bd, host.ptr(b), 1024, host.ptr(tmp), cd, host.ptr(c), None, AMD_GFX950) == capi.NULL_POINTER
    assert mm(ad, host.ptr(a), bd, host.ptr(b), 1024, None, cd, host.ptr(c), None, AMD_GFX950) == capi.NULL_POINTER
    # empty C -> SUCCESS early (mmm.cpp:167-169)
    assert mm(ad, host.ptr(a), bd, host.ptr(b), 1024, host.ptr(tmp), tensor2df(DT_I32, DF_NORMAL, 0, 4), host.ptr(c),
              None, AMD_GFX950) == capi.SUCCESS
    # shape / dtype mismatch -> NOT_MATCH (mmm.cpp:181-197)
    assert mm(ad, host.ptr(a), bd, host.ptr(b), 1024, host.ptr(tmp), tensor2df(DT_I32, DF_NORMAL, 4, 5), host.ptr(c),
              None, AMD_GFX950) == capi.NOT_MATCH
    assert mm(tensor2df(DT_F32, DF_NORMAL, 4, 8), host.ptr(a), bd, host.ptr(b), 1024, host.ptr(tmp), cd, host.ptr(c),
              None, AMD_GFX950) == capi.NOT_MATCH
    assert mm(tensor1d(DT_U8_Q, 8), host.ptr(a), bd, host.ptr(b), 1024, host.ptr(tmp), cd, host.ptr(c), None,
              AMD_GFX950) == capi.NOT_MATCH
    mv = L.matrix_vector_multiply_gfx950
    x = np.zeros(8, np.uint8)
    y = np.zeros(4, np.int32)
    md = host.mvm_desc(DF_NKN32K4, 4, 8)
    assert mv(md, host.ptr(b), tensor1d(DT_U8_Q, 8), None, 1024, host.ptr(tmp), tensor1d(DT_I32, 4), host.ptr(y), None,
              AMD_GFX950) == capi.NULL_POINTER
    assert mv(md, host.ptr(b), tensor1d(DT_U8_Q, 9), host.ptr(x), 1024, host.ptr(tmp), tensor1d(DT_I32, 4), host.ptr(y),
              None, AMD_GFX950) == capi.NOT_MATCH
    # u8 matrix tagged DF_NK is refused (mvm.cpp:172-175)
    assert mv(tensor2df(DT_U8_Q, capi.DF_NK, 4, 8), host.ptr(b), tensor1d(DT_I8, 8), host.ptr(x), 1024, host.ptr(tmp),
              tensor1d(DT_I32, 4), host.ptr(y), None, AMD_GFX950) == capi.NOT_SUPPORTED
    # quantize without a scale pointer -> NOT_MATCH (avx512/quantize.cpp:123-125)
    qd = tensor1d(DT_U8_Q, 8)
    f = np.zeros(8, np.float32)
    assert L.quantize_gfx950(tensor1d(DT_F32, 8), host.ptr(f), C.byref(qd), host.ptr(x), None, 0, AMD_GFX950) == \
        capi.NOT_MATCH
    qd2 = tensor1d(DT_I32, 8)
    s = (C.c_float * 2)(1, 1)
    assert L.quantize_gfx950(tensor1d(DT_F32, 8), host.ptr(f), C.byref(qd2), host.ptr(x), C.cast(s, C.c_void_p), 0,
                             AMD_GFX950) == capi.NOT_SUPPORTED


def test_sizes_beyond_32_bits_are_refused_not_wrapped():
    """The reference's tmp sizes are 32-bit byte counts and its sums wrap silently; a tmp of a wrapped size would be
    overrun. Shapes whose tmp (FullyConnected: input copy + bias + an int32 result) or whose image (convolution: the
    kernels address it with 32-bit byte offsets) does not fit 32 bits are refused before anything is launched."""
    from bolt_amd.capi import DF_NCHWC8, DF_NCHWC16, DT_I8, tensor4df
    L = capi.lib()
    nb = C.c_uint32(0)
    M, K, N = (1 << 26) + 64, 64, 16                      # an int32 result of 4 GiB and a bit
    idesc, fdesc = tensor2df(DT_U8_Q, DF_NORMAL, M, K), tensor2df(DT_I8, DF_NKNxKx, K, N)
    assert L.fully_connected_infer_forward_tmp_bytes_gfx950(idesc, fdesc, tensor2df(DT_U8_Q, DF_NORMAL, M, N), C.byref(nb),
                                                            AMD_GFX950) == capi.NOT_SUPPORTED
    M = 1 << 20                                           # the same query at a size that fits
    idesc = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
    assert L.fully_connected_infer_forward_tmp_bytes_gfx950(idesc, fdesc, tensor2df(DT_U8_Q, DF_NORMAL, M, N), C.byref(nb),
                                                            AMD_GFX950) == capi.SUCCESS
    assert nb.value >= M * K + 4 * N + 4 * M * N
    # weight blobs of 4 GiB and more do not fit the 32-bit byte counts of the transform queries
    rb = C.c_uint32(0)
    wide = tensor2df(DT_I8, DF_NORMAL, 65536, 65536)
    assert L.matrix_matrix_multiply_transform_rhs_bytes_gfx950(wide, C.byref(nb), C.byref(rb), AMD_GFX950) == capi.NOT_SUPPORTED
    assert L.matrix_vector_multiply_transform_weight_bytes_gfx950(wide, C.byref(nb), AMD_GFX950) == capi.NOT_SUPPORTED
    # element-wise operators walk a tensor with 32-bit indices in grid strides: counts near 2^32 (and descs whose 32-bit
    # product wraps to something small) are refused before any pointer is looked at
    f = np.zeros(8, np.float32)
    x = np.zeros(8, np.uint8)
    qd = tensor1d(DT_U8_Q, 8)
    s1 = (C.c_float * 2)(-1, 0)
    for huge in (tensor1d(capi.DT_F32, 0xfffffff0), tensor4df(capi.DT_F32, capi.DF_NCHW, 65536, 65536, 1, 2)):
        assert L.quantize_gfx950(huge, host.ptr(f), C.byref(qd), host.ptr(x), C.cast(s1, C.c_void_p), 0, AMD_GFX950) == \
            capi.NOT_SUPPORTED
    p = capi.conv_param_spec(64, 3, 3, 1, 1)
    big = tensor4df(DT_U8_Q, DF_NCHWC8, 64, 64, 1024, 1024)          # 4 GiB of input
    assert L.convolution_infer_forward_tmp_bytes_gfx950(big, tensor4df(DT_I8, capi.DF_NCHWC2NxC4, 64, 64, 3, 3),
                                                        tensor4df(DT_U8_Q, DF_NCHWC16, 64, 64, 1024, 1024), p,
                                                        capi.CONVOLUTION_ALGORITHM_DIRECT, C.byref(nb), AMD_GFX950) \
        == capi.NOT_SUPPORTED


def test_pool_concat_lstm_argument_checks_and_size_queries():
    """Shape validation and size queries of the pooling / concatenation / LSTM-cell entry points answer before
    anything touches a GPU."""
    from bolt_amd.capi import (AMD_GFX950, DF_NCHWC8, DF_NCHWC16, DF_NKNx_NKN32, DT_F32, POOLING_MAX, RNNParamSpec,
                               pooling_param_spec, tensor4df)
    from bolt_amd.host_lstm import lstm_param_spec
    L = capi.lib()
    buf = np.zeros(16 * 8 * 8, np.uint8)
    vp = buf.ctypes.data
    good = pooling_param_spec(POOLING_MAX, 2, 2, 2, 2, 0, 0, 0, 0)
    d16, o16 = tensor4df(DT_U8_Q, DF_NCHWC16, 1, 16, 8, 8), tensor4df(DT_U8_Q, DF_NCHWC16, 1, 16, 4, 4)
    assert L.pooling_gfx950(d16, vp, good, None, o16, vp, None, capi.X86_AVX512) == capi.NOT_SUPPORTED
    assert L.pooling_gfx950(d16, None, good, None, o16, vp, None, AMD_GFX950) == capi.NULL_POINTER
    assert L.pooling_gfx950(tensor4df(DT_U8_Q, DF_NCHWC8, 1, 16, 8, 8), vp, good, None, o16, vp, None,
                            AMD_GFX950) == capi.NOT_MATCH
    assert L.pooling_gfx950(tensor4df(DT_F32, DF_NCHWC16, 1, 16, 8, 8), vp, good, None, o16, vp, None,
                            AMD_GFX950) == capi.NOT_SUPPORTED
    pad = pooling_param_spec(POOLING_MAX, 2, 2, 2, 2, 2, 0, 0, 0)       # pad >= kernel (pooling_int8.cpp:352-354)
    assert L.pooling_gfx950(d16, vp, pad, None, o16, vp, None, AMD_GFX950) == capi.NOT_SUPPORTED
    far = tensor4df(DT_U8_Q, DF_NCHWC16, 1, 16, 9, 4)                    # a window that starts below the image
    assert L.pooling_gfx950(d16, vp, good, None, far, vp, None, AMD_GFX950) == capi.NOT_SUPPORTED
    # concat: tmp bytes are zero; extents that do not add up are refused before any launch
    nb = C.c_uint32(7)
    descs = (capi.TensorDesc * 2)(tensor4df(DT_I8, 0, 2, 3, 5, 7), tensor4df(DT_I8, 0, 2, 5, 5, 7))
    assert L.concat_infer_forward_tmp_bytes_gfx950(2, descs, tensor4df(DT_I8, 0, 2, 8, 5, 7), C.byref(nb),
                                                   AMD_GFX950) == capi.SUCCESS and nb.value == 0
    ptrs = (C.c_void_p * 2)(vp, vp)
    sc = (C.c_float * 2)(2.0, 3.0)
    osc = C.c_float(0)
    assert L.concat_gfx950(2, descs, ptrs, sc, capi.ConcatParamSpec(1, 2), None, tensor4df(DT_I8, 0, 2, 9, 5, 7), vp,
                           C.byref(osc), AMD_GFX950) == capi.NOT_MATCH
    assert osc.value == 2.0   # the common scale is the smallest input scale (concat.cpp:175-177)
    # LSTM weight: matrix-vector blob + GEMM packing; a transformed descriptor needs no further bytes
    p = lstm_param_spec(64)
    N, K = 256, 96
    assert L.rnn_transform_filter_bytes_gfx950(tensor2df(DT_I8, DF_NORMAL, N, K), p, C.byref(nb), AMD_GFX950) == capi.SUCCESS
    assert nb.value == 2 * N * K + 4 * N
    assert L.rnn_transform_filter_bytes_gfx950(tensor2df(DT_I8, DF_NKNx_NKN32, N, K), p, C.byref(nb),
                                               AMD_GFX950) == capi.SUCCESS and nb.value == 0
    xd, hd = tensor2df(DT_F32, DF_NORMAL, 3, 32), tensor2df(DT_F32, DF_NORMAL, 3, 64)
    assert L.rnncell_infer_forward_tmp_bytes_gfx950(xd, tensor2df(DT_I8, DF_NORMAL, N, K), hd, p, C.byref(nb),
                                                    AMD_GFX950) == capi.SUCCESS and nb.value >= 3 * (K + 4 + 4 * N)
    proj = lstm_param_spec(64)
    proj.num_projection = 32
    plain = nb.value
    # with a projection the gates give num_projection values per row: the weight is [4 * 32][32 + 64], and tmp also
    # holds those values ahead of the fp32 projection
    assert L.rnncell_infer_forward_tmp_bytes_gfx950(xd, tensor2df(DT_I8, DF_NORMAL, 128, K), hd, proj, C.byref(nb),
                                                    AMD_GFX950) == capi.SUCCESS and nb.value >= 3 * (K + 4 + 4 * 128 + 4 * 32)
    assert nb.value != plain
    odd = lstm_param_spec(48)                 # the projection matrix comes in blocks of 32 rows (DF_NKN32)
    odd.num_projection = 32
    assert L.rnncell_infer_forward_tmp_bytes_gfx950(xd, tensor2df(DT_I8, DF_NORMAL, 128, 80), tensor2df(DT_F32, DF_NORMAL, 3, 48),
                                                    odd, C.byref(nb), AMD_GFX950) == capi.NOT_SUPPORTED
    assert C.sizeof(RNNParamSpec) == 36


def test_encoder_workspace_queries():
    """Size queries of the encoder layer and of a stack of layers (no GPU involved): argument checks, and the stack's
    workspace = the largest layer's + two [tokens, hidden] fp32 buffers that carry activations between layers."""
    L = capi.lib()
    C = capi.C
    one = C.c_float(0)
    ptr = C.cast(C.pointer(one), C.POINTER(C.c_float))

    def spec(ffn, hidden=256, heads=4):
        s = capi.BoltEncoderLayerInt8()
        s.batch, s.seq, s.hidden, s.heads, s.ffn = 4, 32, hidden, heads, ffn
        for name in ("wqkv", "wo", "w1", "w2"):
            setattr(s, name, C.addressof(one))   # never dereferenced by the queries
        for name in ("sqkv", "so", "s1", "s2", "ln1_gamma", "ln1_beta", "ln2_gamma", "ln2_beta"):
            setattr(s, name, ptr)
        return s

    n = C.c_size_t(0)
    a, b = spec(1024), spec(512)
    capi.check(L.bolt_gfx950_encoder_layer_int8_workspace_bytes(C.byref(a), C.byref(n)), "layer a")
    na = n.value
    capi.check(L.bolt_gfx950_encoder_layer_int8_workspace_bytes(C.byref(b), C.byref(n)), "layer b")
    nb = n.value
    assert na > nb > 0
    stack = (capi.BoltEncoderLayerInt8 * 3)(b, a, b)
    capi.check(L.bolt_gfx950_encoder_stack_int8_workspace_bytes(stack, 3, C.byref(n)), "stack")
    act = (4 * 32 * 256 * 4 + 255) // 256 * 256
    assert n.value == na + 2 * act
    assert L.bolt_gfx950_encoder_stack_int8_workspace_bytes(None, 3, C.byref(n)) == capi.NULL_POINTER
    assert L.bolt_gfx950_encoder_stack_int8_workspace_bytes(stack, 3, None) == capi.NULL_POINTER
    assert L.bolt_gfx950_encoder_stack_int8_workspace_bytes(stack, 0, C.byref(n)) == capi.NOT_SUPPORTED
    mixed = (capi.BoltEncoderLayerInt8 * 2)(a, spec(1024, hidden=128, heads=2))
    assert L.bolt_gfx950_encoder_stack_int8_workspace_bytes(mixed, 2, C.byref(n)) == capi.NOT_MATCH
    bad = (capi.BoltEncoderLayerInt8 * 1)(spec(1024, hidden=256, heads=3))   # hidden != heads * 64
    assert L.bolt_gfx950_encoder_stack_int8_workspace_bytes(bad, 1, C.byref(n)) == capi.NOT_SUPPORTED
