"""Two host threads calling the library at the same time, each on its own HIP stream with its own tensors -- what
CNN::clone() gives each user thread of the reference. Every thread has its own context inside the library (scratch
words, pinned scale word, quantiser sync area), so dynamic scales and results must come out as if it ran alone."""
import threading

import numpy as np
import pytest

pytestmark = pytest.mark.gpu

from bolt_amd import capi, host  # noqa: E402
from bolt_amd.capi import DF_NKNxKx, DF_TRANSPOSE, DT_F32, DT_I8, DT_I32, DT_U8_Q  # noqa: E402


def worker(idx, torch, oracle_results, errors, rounds):
    try:
        L = capi.lib()
        stream = torch.cuda.Stream()
        capi.check(L.bolt_gfx950_set_stream(stream.cuda_stream), "set_stream")
        rng = np.random.default_rng(500 + idx)
        M, K, N = 32 + 8 * idx, 256, 192
        x = (rng.standard_normal((M, K)) * (1.0 + idx)).astype(np.float32)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        bias = rng.standard_normal(N).astype(np.float32)
        big = (rng.standard_normal(700000 + 1000 * idx) * (3.0 + idx)).astype(np.float32)
        with torch.cuda.stream(stream):
            dx, dW, db, dbig = (torch.from_numpy(a).cuda() for a in (x, W, bias, big))
        stream.synchronize()
        blob, _, _ = host.mmm_transform_rhs(dW, DF_TRANSPOSE, K, N)
        want = oracle_results[idx]
        for r in range(rounds):
            s = [-1.0]
            xq = host.quantize(dx.view(-1), DT_F32, DT_U8_Q, s)                 # one-launch dynamic quantiser
            assert s[0] == want["sx"], (idx, r, "sx", s[0], want["sx"])
            sb = [-1.0]
            bq = host.quantize(dbig, DT_F32, DT_I8, sb)                          # two-pass dynamic quantiser
            assert sb[0] == want["sbig"], (idx, r, "sbig")
            out, so = host.fully_connected(xq.view(M, K), s[0], blob, DF_NKNxKx, 50.0, db, M, K, N, DT_U8_Q, -1.0)
            assert so == want["so"], (idx, r, "so", so, want["so"])
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            assert np.array_equal(xq.cpu().numpy().reshape(M, K), want["xq"]), (idx, r, "xq")
            assert np.array_equal(bq.cpu().numpy(), want["bq"]), (idx, r, "bq")
            assert np.array_equal(out.cpu().numpy(), want["out"]), (idx, r, "out")
        capi.check(L.bolt_gfx950_set_stream(None), "set_stream")
    except BaseException as e:  # noqa: BLE001 -- reported by the main thread
        errors.append((idx, repr(e)))


def test_two_threads_two_streams(oracle):
    import torch
    assert torch.cuda.is_available()
    capi.check(capi.lib().bolt_gfx950_init(), "init")
    expected = []
    for idx in range(2):
        rng = np.random.default_rng(500 + idx)
        M, K, N = 32 + 8 * idx, 256, 192
        x = (rng.standard_normal((M, K)) * (1.0 + idx)).astype(np.float32)
        W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
        bias = rng.standard_normal(N).astype(np.float32)
        big = (rng.standard_normal(700000 + 1000 * idx) * (3.0 + idx)).astype(np.float32)
        xq, sx = oracle.quantize_f32(x, DT_U8_Q)
        bq, sbig = oracle.quantize_f32(big, DT_I8)
        out, so = oracle.fully_connected(xq, sx, W, np.float32(50.0), bias, DT_U8_Q)
        expected.append({"xq": xq, "sx": sx, "bq": bq, "sbig": sbig, "out": out, "so": so})
    errors = []
    threads = [threading.Thread(target=worker, args=(i, torch, expected, errors, 40)) for i in range(2)]
    print("two threads start", flush=True)
    for t in threads:
        t.start()
    for t in threads:
        t.join(timeout=100)
    assert not any(t.is_alive() for t in threads), "a worker thread did not finish"
    assert not errors, errors
