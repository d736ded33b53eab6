#!/usr/bin/env python3
"""Benchmark of the quantized matrix-product hot path on one MI355X.

Headline workload (BASELINE.json configs[1]): int8 GEMV decode shape, N = K = 4096, 256 independent
activation vectors, per-output-channel weight scales, fp32 output. One "step" is one pass over the
256 vectors = ONE launch of the strided-batch GEMV kernel (bolt_gfx950_mvm_int8_strided_batch).
Every product streams a full 16 MiB weight blob; the blobs are `--copies` replicas of the same
packed matrix at different addresses (default 64 = 1 GiB, 4x the 256 MiB Infinity Cache), so each
product's weights come from HBM rather than from a cache warmed by the previous product.

Prints ONE JSON line. `value` is whole-job GB/s of ALGORITHMIC bytes (16 830 464 B per vector: the
weight matrix + activation vector + compensation vector + channel scales + fp32 result).
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
for p in (ROOT, os.path.join(ROOT, "tests")):
    if p not in sys.path:
        sys.path.insert(0, p)

N = K = 4096
BATCH = 256
BYTES_PER_VECTOR = N * K + K + 4 * N + 4 * N + 4 * N   # W + x + offsetC + scales + out = 16 830 464
OPS_PER_VECTOR = 2 * N * K
HBM_PEAK_GBS = 8000.0


def parse():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=50)
    ap.add_argument("--warmup", type=int, default=10)
    ap.add_argument("--copies", type=int, default=64, help="replicas of the weight blob the batch rotates over")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--cpu-seconds", type=float, default=10.0)
    ap.add_argument("--extras", action="store_true", help="also time the other hot-path kernels (stderr)")
    return ap.parse_args()


def cpu_baseline(W, xq, sI, sW0, seconds):
    """Reference's own x86 path (oracle/_ref) when this host can run it, else the C port; rank 0 only.
    Sample: the same 4096x4096 GEMV over the 256 vectors, repeated for about `seconds` of CPU time."""
    import numpy as np
    from checkers import DT_F32, Oracle, Ref
    n_done = 0
    if Ref.available():
        ref = Ref(threads=1)
        blob, _ = ref.mvm_transform_weight(0, N, K, W)
        off = blob[N * K:N * K + 4 * N].view(np.int32).copy()
        import ctypes as C
        tmp = np.zeros(2 * N * 4 + 64, np.uint8)      # offsetC at the head, as the reference's callers lay it out
        tmp[:4 * N] = off.view(np.uint8)
        yb = np.zeros(N, np.float32)
        sc = (C.c_float * 1)()
        xs = np.ascontiguousarray(xq)
        vp = C.c_void_p
        t0 = time.perf_counter()
        stop = False
        while not stop:
            for b in range(BATCH):
                yb.fill(0)                              # the product accumulates into its result
                sc[0] = float(sI[b] * sW0)
                e = ref.lib.ref_mvm(2, 1, C.c_uint32(N), C.c_uint32(K), blob.ctypes.data_as(vp),
                                    vp(xs.ctypes.data + b * K), C.c_uint32(tmp.size), tmp.ctypes.data_as(vp), 6,
                                    yb.ctypes.data_as(vp), sc)
                assert e == 0
                n_done += 1
                if time.perf_counter() - t0 >= seconds:
                    stop = True
                    break
        dt = time.perf_counter() - t0
        kind = "reference"
        what = "Bolt x86 AVX512-VNNI matrix_vector_multiply (pre-packed, fp32 out), 1 thread (the reference GEMV has no OpenMP)"
    else:
        orc = Oracle()
        off = orc.offsetC(W, True)
        z = np.zeros(N, np.float32)
        t0 = time.perf_counter()
        while n_done < 8 or time.perf_counter() - t0 < min(seconds, 5.0):
            orc.mvm(W, xq[n_done % BATCH], off, z, DT_F32, scale=[float(sI[n_done % BATCH] * sW0)])
            n_done += 1
        dt = time.perf_counter() - t0
        kind = "port"
        what = "scalar C port of the reference GEMV (host lacks avx512_vnni or oracle/_ref not built)"
    return {"value": n_done * BYTES_PER_VECTOR / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": kind,
            "sample": "%d GEMV calls N=K=4096 over the workload's vectors in %.1f s; %s" % (n_done, dt, what)}


def main():
    a = parse()
    if a.gpus != 1:
        print("bench.py: this path is built and measured on ONE GPU; --gpus %d is not supported "
              "(no collectives or sharding in this build)" % a.gpus, file=sys.stderr)
        sys.exit(2)
    import ctypes as C
    import numpy as np
    import torch
    from bolt_amd import capi, host
    from bolt_amd.capi import DF_NORMAL, DT_U8_Q
    from checkers import DT_I32, Oracle

    L = capi.lib()
    capi.check(L.bolt_gfx950_init(), "init")
    dev = torch.device("cuda:0")
    rng = np.random.default_rng(20240601)
    W = rng.integers(-127, 128, size=(N, K), dtype=np.int8)
    sW = (1.0 / rng.uniform(0.005, 0.02, size=N)).astype(np.float32)      # Bolt scale = 1 / step
    X = rng.standard_normal((BATCH, K)).astype(np.float32)

    # load time: pack once on the GPU, replicate the blob
    blob, _ = host.mvm_transform_weight(torch.from_numpy(W).to(dev), DF_NORMAL, N, K)
    blob_bytes = N * K + 4 * N
    stride = (blob_bytes + 255) // 256 * 256
    wbuf = torch.zeros(a.copies * stride, dtype=torch.uint8, device=dev)
    for c in range(a.copies):
        wbuf[c * stride:c * stride + blob_bytes] = blob[:blob_bytes]
    dX = torch.from_numpy(X).to(dev)
    xq = torch.empty((BATCH, K), dtype=torch.uint8, device=dev)
    dsI = torch.full((BATCH,), -1.0, dtype=torch.float32, device=dev)
    for b in range(BATCH):   # per-vector dynamic symmetric quantisation, scales stay on the GPU
        capi.check(L.bolt_gfx950_quantize_f32_async(dX[b].data_ptr(), K, DT_U8_Q, xq[b].data_ptr(),
                                                    dsI[b:b + 1].data_ptr(), 0), "quantize")
    dsW = torch.from_numpy(sW).to(dev)
    y = torch.zeros((BATCH, N), dtype=torch.float32, device=dev)
    capi.check(L.bolt_gfx950_synchronize(), "sync")

    def step():
        capi.check(L.bolt_gfx950_mvm_int8_strided_batch(BATCH, N, K, wbuf.data_ptr(), stride, a.copies, xq.data_ptr(),
                                                        y.data_ptr(), dsI.data_ptr(), dsW.data_ptr(), None), "mvm_batch")

    for _ in range(a.warmup):
        step()
    torch.cuda.synchronize()
    ms = C.c_float(0)
    t0 = time.perf_counter()
    capi.check(L.bolt_gfx950_timer_start(), "timer")
    for _ in range(a.steps):
        step()
    capi.check(L.bolt_gfx950_timer_stop(C.byref(ms)), "timer")   # HIP events on the launch stream
    torch.cuda.synchronize()
    wall = time.perf_counter() - t0
    ms_per_step = wall * 1e3 / a.steps
    launch_ms = ms.value / a.steps                               # one kernel launch per step
    value = BATCH * BYTES_PER_VECTOR / (ms_per_step * 1e-3) / 1e9
    achieved = BATCH * BYTES_PER_VECTOR / (launch_ms * 1e-3) / 1e9

    # parity spot check against the oracle (checker only; not timed)
    orc = Oracle()
    xq_h, sI_h, y_h = xq.cpu().numpy(), dsI.cpu().numpy(), y.cpu().numpy()
    off = orc.offsetC(W, True)
    ok = True
    for b in (0, 131, 255):
        acc = orc.mvm(W, xq_h[b], off, np.zeros(N, np.int32), DT_I32)
        want = orc.dequant_per_channel(acc.reshape(1, N), sI_h[b], sW)
        ok &= bool(np.array_equal(want.view(np.int32).reshape(-1), y_h[b].view(np.int32)))
    if not ok:
        print("bench.py: GPU result differs from the oracle", file=sys.stderr)
        sys.exit(1)

    traffic = None
    tpath = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(tpath):
        traffic = json.load(open(tpath)).get("gemv_s8u8_strided_batch_c2")

    out = {
        "metric": "int8 GEMV GB/s (N=K=4096, 256 independent vectors)", "value": value, "unit": "GB/s",
        "n_gpus": 1, "steps": a.steps, "warmup": a.warmup, "ms_per_step": ms_per_step, "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8 x u8 -> int32 accumulate -> f32",
        "data": "synthetic (seed 20240601): W int8 U[-127,127], per-channel scales 1/U(0.005,0.02), x ~ N(0,1) "
                "quantised per vector",
        "config": {"workload": "BASELINE configs[1]: int8 GEMV M=1 K=4096 N=4096 x 256 independent vectors, "
                               "per-output-channel scales, fp32 out; one strided-batch launch per step",
                   "weight_copies": a.copies, "vectors": BATCH},
        "roofline": {"bound": "hbm", "achieved": achieved, "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": achieved / HBM_PEAK_GBS, "traffic": traffic,
                     "kernel": "gemv_s8u8_kernel (strided batch)", "launch_ms": launch_ms,
                     "algorithmic_bytes_per_launch": BATCH * BYTES_PER_VECTOR},
        "tops": BATCH * OPS_PER_VECTOR / (ms_per_step * 1e-3) / 1e12,
        "parity_checked": True,
    }
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(W, xq_h, sI_h, float(sW[0]), a.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
