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
    ap.add_argument("--only", choices=["gemm", "gemm_data", "fc", "conv", "bnn", "encoder", "encoder_stack", "quantize", "pool", "lstm", "deconv", "depthwise", "ptq"],
                    help="run just this secondary workload and print its figures (profiling aid; not the bench line)")
    ap.add_argument("--no-extras", action="store_true",
                    help="skip the secondary measurements (GEMM sweep, FC, conv, BNN, quantize) in `other_kernels`")
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
    out = {"value": n_done * BYTES_PER_VECTOR / dt / 1e9, "unit": "GB/s", "cores": 1, "kind": kind,
           "sample": "%d GEMV calls N=K=4096 over the workload's vectors in %.1f s; %s; ONE 16 MiB weight blob re-read by "
                     "every call, so it is served from the host's last-level cache where that holds it" % (n_done, dt, what),
           "host_cpu": host_cpu_model(), "host_logical_cpus": os.cpu_count()}
    if kind == "reference":
        out.update(cpu_baseline_extras(ref, blob, tmp, xs, sI, sW0, max(2.0, seconds / 3)))
    return out


def host_cpu_model():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline_extras(ref, blob, tmp, xs, sI, sW0, seconds):
    """More of the reference's own x86 path on the host cores, each for about `seconds`: the same GEMV rotating over 16
    copies of the weight blob (256 MiB: from DRAM rather than the last-level cache), and the int8 GEMM
    (matrix_matrix_multiply, the only part of the path the reference runs on more than one thread) at BASELINE
    configs[0] (64 x 1024 x 1024) and at the BERT FFN shape 4096 x 768 x 3072, with 1 thread and with all."""
    import ctypes as C
    import numpy as np
    vp, u32 = C.c_void_p, C.c_uint32
    res = {}
    copies = [blob.copy() for _ in range(16)]
    yb = np.zeros(N, np.float32)
    sc = (C.c_float * 1)()
    n_done, t0 = 0, time.perf_counter()
    while time.perf_counter() - t0 < seconds:
        b = n_done % BATCH
        yb.fill(0)
        sc[0] = float(sI[b] * sW0)
        assert ref.lib.ref_mvm(2, 1, u32(N), u32(K), copies[n_done % 16].ctypes.data_as(vp), vp(xs.ctypes.data + b * K),
                               u32(tmp.size), tmp.ctypes.data_as(vp), 6, yb.ctypes.data_as(vp), sc) == 0
        n_done += 1
    dt = time.perf_counter() - t0
    res["gemv_rotating_16_weight_copies"] = {"value": n_done * BYTES_PER_VECTOR / dt / 1e9, "unit": "GB/s", "cores": 1,
                                             "sample": "%d calls in %.1f s over 256 MiB of weight blobs" % (n_done, dt)}
    del copies
    rng = np.random.default_rng(7)
    gem = []
    nproc = len(os.sched_getaffinity(0)) if hasattr(os, "sched_getaffinity") else (os.cpu_count() or 1)
    for (M, Kk, Nn) in ((64, 1024, 1024), (4096, 768, 3072)):
        A = rng.integers(0, 256, size=(M, Kk), dtype=np.uint8)
        Wn = rng.integers(-127, 128, size=(Nn, Kk), dtype=np.int8)
        pb, rhs, _ = ref.mmm_transform_rhs(1, Kk, Nn, Wn)
        tb = ref.mmm_tmp_bytes(False, 2, M, Kk, Nn) + 64
        t = np.zeros(tb, np.uint8)
        t[:4 * Nn] = pb[rhs:rhs + 4 * Nn]
        Cb = np.zeros((M, Nn), np.float32)
        s1 = (C.c_float * 1)(3000.0)
        for threads in sorted({1, nproc}):
            ref.lib.ref_set_threads(int(threads))
            n_done, t0 = 0, time.perf_counter()
            while n_done < 2 or time.perf_counter() - t0 < seconds / 2:
                Cb.fill(0)
                assert ref.lib.ref_mmm(0, 2, u32(M), u32(Kk), u32(Nn), A.ctypes.data_as(vp), pb.ctypes.data_as(vp), u32(tb),
                                       t.ctypes.data_as(vp), 6, Cb.ctypes.data_as(vp), s1) == 0
                n_done += 1
            dt = time.perf_counter() - t0
            gem.append({"M": M, "K": Kk, "N": Nn, "threads": int(threads), "tops": 2.0 * M * Kk * Nn * n_done / dt / 1e12,
                        "ms": dt / n_done * 1e3, "sample": "%d calls in %.1f s" % (n_done, dt)})
        ref.lib.ref_set_threads(1)
    res["gemm_int8_matrix_matrix_multiply"] = gem
    # the reference's int8 convolution at BASELINE configs[2] (32 x 64 x 56 x 56, 3 x 3, 64 -> 64, ReLU, u8 result with the
    # dynamic output scale) -- convolution_int8 has no OpenMP: one thread -- and its fp32 -> u8 quantiser at 4096 x 3072
    n, ic, ih, iw, oc = 32, 64, 56, 56, 64
    xq = rng.integers(128, 256, size=n * ic * ih * iw, dtype=np.uint8)
    Wc = rng.integers(-127, 128, size=(oc, ic, 3, 3), dtype=np.int8)
    cb = (rng.standard_normal(oc) * 0.1).astype(np.float32)
    cout = np.zeros(n * oc * ih * iw + 64, np.uint8)
    cs = (C.c_float * 3)(40.0, -1.0, 80.0)
    secs = C.c_double(0)
    ref.lib.ref_conv_int8_loop.argtypes = [u32] * 4 + [C.c_int] + [u32] * 11 + [C.c_int] + [vp] * 4 + [C.c_int, C.c_int, vp, C.c_int,
                                                                                                  C.POINTER(C.c_double)]
    reps, total, calls = 2, 0.0, 0
    while total < seconds / 2:
        assert ref.lib.ref_conv_int8_loop(n, ic, ih, iw, 2, oc, 3, 3, 1, 1, 1, 1, 1, 1, ih, iw, 1, xq.ctypes.data_as(vp),
                                          Wc.ctypes.data_as(vp), cb.ctypes.data_as(vp), C.cast(cs, vp), 1, 10, cout.ctypes.data_as(vp),
                                          reps, C.byref(secs)) == 0
        total += secs.value
        calls += reps
    ops = 2.0 * n * ih * iw * oc * ic * 9
    res["conv_c3_u8_dynamic_scale"] = {"ms": total / calls * 1e3, "tops": ops * calls / total / 1e12, "threads": 1,
                                       "sample": "%d calls of convolution_int8 in %.1f s (filter transformed once, outside the clock)" % (calls, total)}
    nq = 4096 * 3072
    xf = rng.standard_normal(nq).astype(np.float32)
    qo = np.zeros(nq + 64, np.uint8)
    qs = (C.c_float * 1)(-1.0)
    n_done, t0 = 0, time.perf_counter()
    while n_done < 2 or time.perf_counter() - t0 < seconds / 3:
        qs[0] = -1.0
        assert ref.lib.ref_quantize(6, xf.ctypes.data_as(vp), u32(nq), 10, qo.ctypes.data_as(vp), qs, 0) == 0
        n_done += 1
    dt = time.perf_counter() - t0
    res["quantize_f32_u8_dynamic"] = {"ms": dt / n_done * 1e3, "gbps": nq * 9 * n_done / dt / 1e9, "threads": 1,
                                      "algorithmic_bytes": nq * 9, "sample": "%d calls of quantize_x86 on 4096 x 3072 fp32 in %.1f s" % (n_done, dt)}
    return res


MFMA_PEAK_TOPS = 5000.0


def other_kernels(L, capi, host, torch, dev, only=None):
    """Secondary measurements of the same hot path, each timed with HIP events on the library stream
    over `reps` back-to-back calls with operands resident in HBM. Python issues every call, so shapes
    whose kernel runs under ~15 us (C1) are bound by call overhead, which is what a caller sees."""
    import ctypes as C
    import numpy as np
    from bolt_amd import host_conv
    from bolt_amd.capi import (DF_NCHWC8, DF_NCHWC16, DF_NCHWN16C8, DF_NKNxKx, DF_NORMAL, DF_TRANSPOSE, DT_BIN11, DT_F32,
                               DT_I32, DT_U8_Q, tensor2df)
    g = torch.Generator(device=dev).manual_seed(20240601)
    res = {}

    def want(name):
        return only is None or only == name

    def timed(fn, reps, warm=3):
        """Milliseconds per call: `reps` calls in up to five equal batches, each batch between HIP events on the
        library stream; the median batch is reported, so that one stall of the box does not set the figure."""
        for _ in range(warm):
            fn()
        capi.check(L.bolt_gfx950_synchronize(), "sync")
        batches = 5 if reps >= 10 else 1
        per = max(1, reps // batches)
        out = []
        for _ in range(batches):
            ms = C.c_float(0)
            capi.check(L.bolt_gfx950_timer_start(), "timer")
            for _ in range(per):
                fn()
            capi.check(L.bolt_gfx950_timer_stop(C.byref(ms)), "timer")
            out.append(ms.value / per)
        return sorted(out)[len(out) // 2]

    # -- int8 GEMM: square sweep + the BERT-base layer shapes, through both callers of the kernel:
    #    matrix_matrix_multiply (C += A.B: the int32 bits already in C are read and added, as the reference
    #    does, for int32 and fp32 results; u8 results start from zero) and FullyConnected (starts from the
    #    folded bias, never reads C; this is what a model's layers run)
    if want("gemm"):
        from bolt_amd.capi import AMD_GFX950_DEVICE, DT_I8, tensor1d
        gemm = []
        # 8192^3: 30 untimed calls first and 20 timed ones -- the clock the device holds under this load takes ~10 ms to
        # settle, and a figure taken from a cold start reads up to 20 % off in either direction
        for (M, K, N, reps, warm) in ((2048, 2048, 2048, 50, 3), (4096, 4096, 4096, 30, 10), (8192, 8192, 8192, 20, 30),
                                      (4096, 768, 768, 50, 3), (4096, 768, 3072, 50, 3), (4096, 3072, 768, 50, 3)):
            A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=g)
            W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)
            blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            off = blob[rhs:rhs + 4 * N].clone()
            bias = torch.randn(N, device=dev, generator=g) * 0.1
            ad = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
            fdesc = tensor2df(DT_I8, DF_NKNxKx, K, N)

            def add(path, nm, t):
                tops = 2.0 * M * N * K / t / 1e9
                gemm.append({"M": M, "K": K, "N": N, "path": path, "out": nm, "operands": "uniform u8 x uniform s8",
                             "ms": t, "tops": tops, "frac_mfma_peak": tops / MFMA_PEAK_TOPS})
            for cdt, tdt, sc, nm in ((DT_F32, torch.float32, [37.25], "f32"), (DT_I32, torch.int32, None, "i32_accumulate"),
                                     (DT_U8_Q, torch.uint8, [-1.0, 1e-5], "u8")):
                Cb = torch.zeros((M, N), dtype=tdt, device=dev)
                cd = tensor2df(cdt, DF_NORMAL, M, N)
                add("matrix_matrix_multiply", nm,
                    timed(lambda: capi.check(host.matrix_matrix_multiply(A, ad, blob, bd, off, Cb, cd, sc), "mmm"), reps, warm))
                del Cb
            for odt, tdt, so0, nm in ((DT_F32, torch.float32, -1.0, "f32"), (DT_U8_Q, torch.uint8, 0.05, "u8_static_scale")):
                nbytes = host.fully_connected_tmp_bytes(M, K, N, DF_NKNxKx, odt, AMD_GFX950_DEVICE)
                tmp = torch.empty(nbytes, dtype=torch.uint8, device=dev)
                out = torch.empty((M, N), dtype=tdt, device=dev)
                so = C.c_float(so0)
                od = tensor2df(odt, DF_NORMAL, M, N)
                add("fully_connected", nm,
                    timed(lambda: capi.check(L.fully_connected_gfx950(ad, host.ptr(A), 30.0, fdesc, host.ptr(blob), 100.0,
                                                                      tensor1d(DT_F32, N), host.ptr(bias), nbytes, host.ptr(tmp),
                                                                      od, host.ptr(out), C.byref(so), AMD_GFX950_DEVICE),
                                             "fully_connected"), reps, warm))
                del tmp, out
            del A, W, blob
        res["gemm_int8"] = gemm
        # -- few rows (a serving batch of 16-256 tokens against a layer's weights): these go to the kernel that hands every
        #    workgroup a 16-column weight panel and splits K over its waves, where it prices below the 128 x 128 tiles
        few = []
        for (M, K, N) in ((16, 4096, 4096), (64, 4096, 4096), (256, 3072, 768), (256, 4096, 1024), (256, 4096, 4096)):
            A = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=g)
            W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)
            blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            bias = torch.randn(N, device=dev, generator=g) * 0.1
            ad = tensor2df(DT_U8_Q, DF_NORMAL, M, K)
            fdesc = tensor2df(DT_I8, DF_NKNxKx, K, N)
            nbytes = host.fully_connected_tmp_bytes(M, K, N, DF_NKNxKx, DT_F32, AMD_GFX950_DEVICE)
            tmp = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            out = torch.empty((M, N), dtype=torch.float32, device=dev)
            so = C.c_float(-1.0)
            od = tensor2df(DT_F32, DF_NORMAL, M, N)
            t = timed(lambda: capi.check(L.fully_connected_gfx950(ad, host.ptr(A), 30.0, fdesc, host.ptr(blob), 100.0,
                                                                  tensor1d(DT_F32, N), host.ptr(bias), nbytes, host.ptr(tmp),
                                                                  od, host.ptr(out), C.byref(so), AMD_GFX950_DEVICE),
                                         "fully_connected"), 50)
            few.append({"M": M, "K": K, "N": N, "path": "fully_connected", "out": "f32", "ms": t,
                        "weight_gbps": N * K / t / 1e6, "tops": 2.0 * M * N * K / t / 1e9})
            del A, W, blob, tmp, out
        res["gemm_int8_few_rows"] = few
    if want("gemm_data"):
        from bolt_amd.capi import AMD_GFX950_DEVICE, DT_I8, tensor1d
        # -- the same kernel against what the device sustains: the clock it holds depends on how many operand
        #    bits toggle, so 8192^3 is also timed on operands as a network produces them and on constant ones,
        #    next to a register-resident MFMA loop with random and with all-zero operands
        M = K = N = 8192

        def quantised(x, per_row, lo, hi, zero_point):
            s = 127.0 / (x.abs().amax(dim=1, keepdim=True) if per_row else x.abs().max())
            return (torch.round(x * s) + zero_point).clamp(lo, hi)
        dists = (("uniform u8 x uniform s8",
                  lambda: torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=g),
                  lambda: torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)),
                 ("u8 of relu(N(0,1)), per-tensor scale x s8 of N(0,0.02), per-channel scale",
                  lambda: quantised(torch.relu(torch.randn((M, K), device=dev, generator=g)), False, 1, 255, 128).to(torch.uint8),
                  lambda: quantised(torch.randn((N, K), device=dev, generator=g) * 0.02, True, -127, 127, 0).to(torch.int8)),
                 ("constant: u8 128 x s8 0",
                  lambda: torch.full((M, K), 128, dtype=torch.uint8, device=dev),
                  lambda: torch.zeros((N, K), dtype=torch.int8, device=dev)))
        by_data = []
        for name, fa, fw in dists:
            A, W = fa(), fw()
            blob, bd, rhs = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
            bias = torch.randn(N, device=dev, generator=g) * 0.1
            nbytes = host.fully_connected_tmp_bytes(M, K, N, DF_NKNxKx, DT_U8_Q, AMD_GFX950_DEVICE)
            tmp = torch.empty(nbytes, dtype=torch.uint8, device=dev)
            out = torch.empty((M, N), dtype=torch.uint8, device=dev)
            so = C.c_float(0.05)
            t = timed(lambda: capi.check(L.fully_connected_gfx950(
                tensor2df(DT_U8_Q, DF_NORMAL, M, K), host.ptr(A), 30.0, tensor2df(DT_I8, DF_NKNxKx, K, N), host.ptr(blob), 100.0,
                tensor1d(DT_F32, N), host.ptr(bias), nbytes, host.ptr(tmp), tensor2df(DT_U8_Q, DF_NORMAL, M, N), host.ptr(out),
                C.byref(so), AMD_GFX950_DEVICE), "fully_connected"), 20, warm=30)  # long warm-up: the clock settles over ~10 ms
            tops = 2.0 * M * N * K / t / 1e9
            by_data.append({"M": M, "K": K, "N": N, "path": "fully_connected", "out": "u8_static_scale", "operands": name,
                            "ms": t, "tops": tops, "frac_mfma_peak": tops / MFMA_PEAK_TOPS})
            del A, W, blob, tmp, out
        rate = {}
        probe_so = os.path.join(ROOT, "bench_probe", "libbench_probe.so")   # bench-only library, not the product
        if os.path.exists(probe_so):
            P = C.CDLL(probe_so)
            P.bench_probe_mfma_int8_rate.argtypes = [C.c_int, C.POINTER(C.c_float)]
            torch.cuda.synchronize()
            for key, zero in (("random_operands_tops", 0), ("zero_operands_tops", 1)):
                v = C.c_float(0)
                if P.bench_probe_mfma_int8_rate(zero, C.byref(v)) != 0:
                    raise RuntimeError("bench_probe_mfma_int8_rate failed")
                rate[key] = v.value
        rate["note"] = ("v_mfma_i32_16x16x64_i8 back to back from registers, 8 waves per CU, no memory traffic: the device "
                        "lowers its clock when the operand bits are random")
        res["gemm_int8_8192_by_operand_data"] = by_data
        # the vendor library's int8 product on the same box and operand bits, as a yardstick only (int32 result, no
        # epilogue; torch routes _int_mm to the ROCm BLAS libraries): not a kernel of this library
        try:
            M = K = N = 8192
            va = torch.randint(-128, 128, (M, K), dtype=torch.int8, device=dev, generator=g)
            vb = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)
            for _ in range(30):
                torch._int_mm(va, vb.t())
            torch.cuda.synchronize()
            e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
            e0.record()
            for _ in range(20):
                torch._int_mm(va, vb.t())
            e1.record()
            torch.cuda.synchronize()
            tv = e0.elapsed_time(e1) / 20
            res["vendor_int8_gemm_8192"] = {"ms": tv, "tops": 2.0 * M * N * K / tv / 1e9,
                                            "frac_mfma_peak": 2.0 * M * N * K / tv / 1e9 / MFMA_PEAK_TOPS,
                                            "note": "torch._int_mm(A, B.t()) s8 x s8 -> int32, uniform random bytes, 30 untimed "
                                                    "calls first: the ROCm BLAS library's kernel, for comparison only"}
            del va, vb
        except Exception as ex:                                   # a build of torch without the int8 product
            res["vendor_int8_gemm_8192"] = {"error": repr(ex)[:200]}
        res["mfma_int8_sustained"] = rate
    # -- C1: FullyConnected M=64 K=1024 N=1024, fp32 out
    if want("fc"):
        M, K, N = 64, 1024, 1024
        x = torch.randint(0, 256, (M, K), dtype=torch.uint8, device=dev, generator=g)
        W = torch.randint(-127, 128, (N, K), dtype=torch.int8, device=dev, generator=g)
        blob, _, _ = host.mmm_transform_rhs(W, DF_TRANSPOSE, K, N)
        bias = torch.randn(N, device=dev, generator=g) * 0.1
        from bolt_amd.capi import AMD_GFX950_DEVICE, DT_I8, tensor1d
        nbytes = host.fully_connected_tmp_bytes(M, K, N, DF_NKNxKx, DT_F32, AMD_GFX950_DEVICE)
        tmp = torch.empty(nbytes, dtype=torch.uint8, device=dev)     # reused across calls, as an engine's shared tmp is
        out = torch.empty((M, N), dtype=torch.float32, device=dev)
        so = C.c_float(-1.0)
        idesc, fdesc, odesc = tensor2df(DT_U8_Q, DF_NORMAL, M, K), tensor2df(DT_I8, DF_NKNxKx, K, N), tensor2df(DT_F32, DF_NORMAL, M, N)
        t = timed(lambda: capi.check(L.fully_connected_gfx950(idesc, host.ptr(x), 30.0, fdesc, host.ptr(blob), 100.0,
                                                              tensor1d(DT_F32, N), host.ptr(bias), nbytes, host.ptr(tmp), odesc,
                                                              host.ptr(out), C.byref(so), AMD_GFX950_DEVICE), "fully_connected"), 200)
        res["fc_c1"] = {"ms": t, "tops": 2.0 * M * N * K / t / 1e9, "algorithmic_bytes": 1380352,
                        "gbps": 1380352 / t / 1e6, "note": "one launch (bias fold inside the GEMM kernel) issued from Python through ctypes"}
    # -- C3: int8 3x3 convolution 32x64x56x56 -> 64, ReLU, u8 out with dynamic output scale
    if want("conv"):
        n, ic, ih, iw, oc = 32, 64, 56, 56, 64
        xq = torch.randint(128, 256, (n * ic * ih * iw,), dtype=torch.uint8, device=dev, generator=g)
        Wc = torch.randint(-127, 128, (oc, ic, 3, 3), dtype=torch.int8, device=dev, generator=g)
        p = capi.conv_param_spec(oc, 3, 3, 1, 1)
        cblob, ftm = host_conv.transform_filter(Wc, oc, ic, 3, 3, p)
        cb = torch.randn(oc, device=dev, generator=g) * 0.1
        ops = 2.0 * n * ih * iw * oc * ic * 9
        ctmp = torch.empty(64 << 20, dtype=torch.uint8, device=dev)      # reused across calls, as an engine's shared tmp is
        # Every form is called through the C-ABI with arguments marshalled once, as a C++ caller's are: the synchronous
        # forms return the new output scale through a host pointer, so whatever the caller spends between two calls
        # adds to the time per call (the Python wrapper of the tests would add ~15 us of its own).
        from bolt_amd.capi import (ACTIVATION_RELU, AMD_GFX950_DEVICE, CONVOLUTION_ALGORITHM_DIRECT, ActivationParamSpec,
                                   tensor1d, tensor4df)
        act = ActivationParamSpec()
        act.mode = ACTIVATION_RELU
        idesc = tensor4df(DT_U8_Q, DF_NCHWC8, n, ic, ih, iw)
        bdesc = tensor1d(DT_F32, oc)
        sw = 1.0 / (torch.rand(oc, device=dev, generator=g) * 0.015 + 0.005)       # 1 / U(0.005, 0.02)
        dsi = torch.tensor([40.0], dtype=torch.float32, device=dev)
        dso = torch.zeros(1, dtype=torch.float32, device=dev)
        alg_bytes_u8 = 12882432
        alg_bytes_i32 = 6422528 * 5 + 36864 + 512

        def entry(nm, t, nbytes, note):
            res[nm] = {"ms": t, "tops": ops / t / 1e9, "frac_mfma_peak": ops / t / 1e9 / MFMA_PEAK_TOPS,
                       "algorithmic_bytes": nbytes, "note": note}
        for odt, nm, tdt in ((DT_U8_Q, "u8_dynamic_scale", torch.uint8), (DT_I32, "i32", torch.int32)):
            cout = torch.empty(n * oc * ih * iw, dtype=tdt, device=dev)
            odesc = tensor4df(odt, DF_NCHWC16, n, oc, ih, iw)
            sc = (C.c_float * 3)(40.0, -1.0, 80.0)
            args = (idesc, host.ptr(xq), None, ftm, host.ptr(cblob), p, CONVOLUTION_ALGORITHM_DIRECT, bdesc, host.ptr(cb),
                    ctmp.numel(), host.ptr(ctmp), odesc, host.ptr(cout), sc, act, AMD_GFX950_DEVICE)
            t = timed(lambda: capi.check(L.convolution_gfx950(*args), "convolution"), 50)
            entry("conv_c3_" + nm, t, alg_bytes_u8 if odt == DT_U8_Q else alg_bytes_i32,
                  "convolution_gfx950, one filter scale (the reference's contract: the u8 form returns its output scale "
                  "through the host pointer, so every call waits for the device once)")
        cout = torch.empty(n * oc * ih * iw, dtype=torch.uint8, device=dev)
        odesc = tensor4df(DT_U8_Q, DF_NCHWC16, n, oc, ih, iw)
        # BASELINE configs[2] as worded: per-output-channel filter scales, fp32 bias, ReLU, one output scale for the tensor
        sc2 = (C.c_float * 2)(40.0, -1.0)

        def perchannel_dynamic():
            sc2[1] = -1.0
            capi.check(L.bolt_gfx950_convolution_int8_perchannel(idesc, host.ptr(xq), None, ftm, host.ptr(cblob), p, host.ptr(sw), bdesc,
                                                                 host.ptr(cb), ctmp.numel(), host.ptr(ctmp), odesc, host.ptr(cout), sc2, act,
                                                                 AMD_GFX950_DEVICE), "conv perchannel")
        entry("conv_c3_u8_perchannel", timed(perchannel_dynamic, 50), alg_bytes_u8 + 512,
              "per-output-channel filter scales, dynamic output scale returned to the host (one pass; two when the grid-wide agreement is abandoned)")
        sc3 = (C.c_float * 2)(40.0, 2.5)
        t = timed(lambda: capi.check(L.bolt_gfx950_convolution_int8_perchannel(
            idesc, host.ptr(xq), None, ftm, host.ptr(cblob), p, host.ptr(sw), bdesc, host.ptr(cb), ctmp.numel(), host.ptr(ctmp), odesc,
            host.ptr(cout), sc3, act, AMD_GFX950_DEVICE), "conv perchannel static"), 50)
        entry("conv_c3_u8_perchannel_static_scale", t, alg_bytes_u8 + 512,
              "per-output-channel filter scales, calibrated (static) output scale: one pass, nothing returned")
        for nm, swp, fs, so, note in (
                ("conv_c3_u8_async", None, 80.0, 0.0, "one filter scale, dynamic output scale left in device memory: no wait for the host"),
                ("conv_c3_u8_perchannel_async", host.ptr(sw), 0.0, 0.0, "per-output-channel scales, dynamic output scale left in device memory"),
                ("conv_c3_u8_perchannel_static_async", host.ptr(sw), 0.0, 2.5, "per-output-channel scales, static output scale, asynchronous")):
            t = timed(lambda: capi.check(L.bolt_gfx950_convolution_async(
                idesc, host.ptr(xq), None, ftm, host.ptr(cblob), p, bdesc, host.ptr(cb), ctmp.numel(), host.ptr(ctmp), odesc, host.ptr(cout),
                host.ptr(dsi), fs, swp, host.ptr(dso), so, act), "conv async"), 50)
            entry(nm, t, alg_bytes_u8 + (512 if swp else 0), note)
    # -- C5: XNOR convolution 64x256x28x28 -> 256, fp32 out
    if want("bnn"):
        n, ic, ih, iw, oc = 64, 256, 28, 28, 256
        xb = torch.randint(0, 256, (n * ic // 8 * ih * iw,), dtype=torch.uint8, device=dev, generator=g)
        wb = torch.randint(0, 256, (oc * ic * 9 // 8,), dtype=torch.uint8, device=dev, generator=g)
        bblob, bftm = host_conv.bnn_transform_filter(wb, DT_BIN11, DF_NCHWN16C8, oc, ic, 3, 3)
        bs, bb = torch.rand(oc, device=dev, generator=g) + 0.5, torch.randn(oc, device=dev, generator=g) * 0.1
        btmp = torch.empty(host_conv.bnn_tmp_bytes(DT_BIN11, n, ic, ih, iw, oc, 3, 3, 1, 1, xb), dtype=torch.uint8, device=dev)
        bout = torch.empty(n * oc * ih * iw, dtype=torch.float32, device=dev)
        macs = float(n) * ih * iw * oc * ic * 9
        # default route: operands expanded to E2M1 pairs, fp4 matrix cores; then int8 matrix cores; then xor + popcount
        # on the vector ALU
        for route, key in ((2, "bnn_c5_xnor"), (1, "bnn_c5_xnor_int8_matrix_cores"), (0, "bnn_c5_xnor_vector_alu")):
            capi.check(L.bolt_gfx950_set_option(b"bnn_mfma", route), "set_option")
            t = timed(lambda: host_conv.convolution_bnn(xb, DT_BIN11, n, ic, ih, iw, bblob, bftm, oc, 3, 3, 1, 1, bs, bb,
                                                        DT_F32, tmp=btmp, out=bout), 20)
            res[key] = {"ms": t, "binary_tops": 2 * macs / t / 1e9, "algorithmic_bytes": 53061632,
                        "gbps": 53061632 / t / 1e6}
        capi.check(L.bolt_gfx950_set_option(b"bnn_mfma", 2), "set_option")
        res["bnn_c5_xnor"]["route"] = ("default route: operands expanded to E2M1 pairs, v_mfma_scale_f32_16x16x128_f8f6f4 "
                                       "(fp4 matrix cores); integer sums bit-exact on every route")
        res["bnn_c5_xnor_int8_matrix_cores"]["route"] = "operands expanded to int8, v_mfma_i32_16x16x64_i8"
        res["bnn_c5_xnor_vector_alu"]["route"] = "bit-packed operands, v_xor_b32 + v_bcnt_u32_b32 on the vector ALU"
        res["bnn_c5_xnor"]["frac_fp4_mfma_peak"] = res["bnn_c5_xnor"]["binary_tops"] / 10100.0
        res["bnn_c5_xnor_int8_matrix_cores"]["frac_mfma_peak"] = res["bnn_c5_xnor_int8_matrix_cores"]["binary_tops"] / MFMA_PEAK_TOPS
    # -- C4: BERT-base int8 encoder layer, batch 32 x seq 128 (4096 tokens), one C call per layer
    if want("encoder") or want("encoder_stack"):
        from bolt_amd.capi import DT_I8
        from bolt_amd.host_encoder import EncoderLayer
        rs = np.random.default_rng(20240604)
        batch, seq, hidden, heads, ffn = 32, 128, 768, 12, 3072
        P = {}
        for name, Nn, Kk in (("qkv", 3 * hidden, hidden), ("o", hidden, hidden), ("1", ffn, hidden), ("2", hidden, ffn)):
            # load-time weight quantisation, per output channel, through the library's own quantiser (one row at a time)
            Wf = torch.from_numpy((rs.standard_normal((Nn, Kk)) * 0.02).astype(np.float32)).to(dev)
            Wq = torch.empty((Nn, Kk), dtype=torch.int8, device=dev)
            sw = np.empty(Nn, np.float32)
            for r in range(Nn):
                sr = [-1.0]
                host.quantize(Wf[r], DT_F32, DT_I8, sr, out=Wq[r])
                sw[r] = sr[0]
            capi.check(L.bolt_gfx950_synchronize(), "sync")
            P["w" + name], P["s" + name] = Wq.cpu().numpy(), sw
            P["b" + name] = np.zeros(Nn, np.float32)
        for k in ("ln1", "ln2"):
            P[k + "_g"], P[k + "_b"] = np.ones(hidden, np.float32), np.zeros(hidden, np.float32)
        layer = EncoderLayer(torch, batch, seq, hidden, heads, ffn, P)
        hx = torch.randn((batch * seq, hidden), device=dev, generator=g)
        hy = torch.empty_like(hx)
        t = timed(lambda: layer(hx, hy), 50) if want("encoder") else None
        gemm_ops = 2.0 * batch * seq * hidden * (3 * hidden + hidden + 2 * ffn)
        if want("encoder"):
            res["bert_base_layer_c4"] = {"ms": t, "tokens_per_s": batch * seq / (t * 1e-3), "int8_gemm_tops": gemm_ops / t / 1e9,
                                     "config": "hidden 768, 12 heads, FFN 3072, seq 128, batch 32; int8 GEMMs with per-channel "
                                               "weight scales, dynamic per-tensor activation quantisation, fp32 attention / "
                                               "LayerNorm / GELU",
                                     "parity": "against the CPU oracle (tests/test_gpu_encoder.py): every int8 FullyConnected "
                                               "stage bit-exact and every fp32 stage within 2e-5 given the same stage input; "
                                               "whole-layer output 1.3e-4 relative in the L2 NORM -- the 1e-3 bar is read on "
                                               "that norm: single elements differ by up to 2.6e-3 of max|out| (0.02 % of them "
                                               "by more than 1e-3) where a 1-ulp fp32 difference ahead of a quantiser moves "
                                               "one activation by one int8 step"}
        # twelve such layers back to back (a BERT-base encoder; the same weights twelve times, which changes nothing
        # for the timing: 85 MB of packed weights per layer against 4 MiB of L2 per XCD), one C call for the stack:
        # every layer but the first takes its input's maximum from the LayerNorm that closed the layer before it
        if want("encoder_stack"):
            from bolt_amd.host_encoder import EncoderStack
            stack = EncoderStack(torch, [layer] * 12)
            ts = timed(lambda: stack(hx, hy), 10, warm=3)
            res["bert_base_12_layer_stack"] = {"ms": ts, "ms_per_layer": ts / 12, "tokens_per_s": batch * seq / (ts * 1e-3),
                                               "note": "bolt_gfx950_encoder_stack_int8: bit-identical to twelve single-layer calls "
                                                       "(tests/test_gpu_encoder.py); 11 launches for the first layer, 10 for the others"}
    # -- quantize family at the BERT FFN size (4096 x 3072). Two regimes: "hbm" rotates over 8 tensors (400 MB of
    #    fp32 / int32 input, more than the 256 MB Infinity Cache holds), "cache_resident" reuses one tensor, which is
    #    what a layer sees when the producer's output is still in the Infinity Cache
    if want("quantize"):
        cnt = 4096 * 3072
        R = 8
        xs = [torch.randn(cnt, device=dev, generator=g) for _ in range(R)]
        accs = [torch.randint(-200000, 200000, (cnt,), dtype=torch.int32, device=dev, generator=g) for _ in range(R)]
        q8 = [torch.empty(cnt, dtype=torch.uint8, device=dev) for _ in range(R)]
        fo = [torch.empty(cnt, dtype=torch.float32, device=dev) for _ in range(R)]
        dsc = torch.full((1,), -1.0, device=dev)
        it = [0]

        def rot(fn):
            def call():
                it[0] += 1
                fn(it[0] % R)
            return call

        def both(name, nbytes, fn):
            t_h = timed(rot(fn), 48, warm=8)
            t_c = timed(lambda: fn(0), 50)
            res[name] = {"n": cnt, "ms": t_h, "algorithmic_bytes": nbytes, "gbps": nbytes / t_h / 1e6,
                         "frac_hbm_peak": nbytes / t_h / 1e6 / HBM_PEAK_GBS, "ms_cache_resident": t_c,
                         "gbps_cache_resident": nbytes / t_c / 1e6}
        # the practical ceiling for this kind of kernel: a plain device-to-device copy of the same tensors (50 MB read,
        # 50 MB written per call, rotating like the others), done by the runtime's own copy
        both("device_copy_f32_reference", 8 * cnt, lambda i: fo[i].copy_(xs[i]))
        res["device_copy_f32_reference"]["note"] = ("torch's tensor copy of 4096 x 3072 fp32 (hipMemcpy-class kernel), not a kernel of "
                                                    "this library: what HBM delivers to a read-and-write stream of this size")
        both("quantize_f32_u8_dynamic", 9 * cnt,
             lambda i: capi.check(L.bolt_gfx950_quantize_f32_async(xs[i].data_ptr(), cnt, DT_U8_Q, q8[i].data_ptr(),
                                                                   dsc.data_ptr(), 0), "q"))
        both("dequantize_i32_f32", 8 * cnt, lambda i: host.dequantize(accs[i], DT_I32, 37.5, out=fo[i]))
        both("requantize_i32_u8_static", 5 * cnt, lambda i: host.quantize(accs[i], DT_I32, DT_U8_Q, [0.02, 37.5], out=q8[i]))
    # -- u8 pooling (NCHWC16) and s8 concatenation with a common scale: byte work, rotating over 16 inputs (more than
    #    the Infinity Cache holds) and on one input reused call after call
    if want("pool"):
        from bolt_amd import host_pool
        from bolt_amd.capi import DT_I8, POOLING_MAX, POOLING_MEAN, pooling_param_spec, tensor4df
        R = 16
        it = [0]

        def rot(fn):
            def call():
                it[0] += 1
                fn(it[0] % R)
            return call

        def both(name, nbytes, fn, cfg):
            t_h = timed(rot(fn), 80, warm=16)
            t_c = timed(lambda: fn(0), 50)
            res[name] = {"config": cfg, "ms": t_h, "algorithmic_bytes": nbytes, "gbps": nbytes / t_h / 1e6,
                         "frac_hbm_peak": nbytes / t_h / 1e6 / HBM_PEAK_GBS, "ms_cache_resident": t_c,
                         "gbps_cache_resident": nbytes / t_c / 1e6}
        n, c, ih, iw = 32, 64, 112, 112
        xs = [torch.randint(0, 256, (n * c * ih * iw,), dtype=torch.uint8, device=dev, generator=g) for _ in range(R)]
        ys = [torch.empty(n * c * 56 * 56, dtype=torch.uint8, device=dev) for _ in range(R)]
        pmax = pooling_param_spec(POOLING_MAX, 3, 3, 2, 2, 1, 1, 1, 1)
        pmean = pooling_param_spec(POOLING_MEAN, 2, 2, 2, 2, 0, 0, 0, 0)
        nb = n * c * (ih * iw + 56 * 56)
        both("pooling_u8_max_3x3_s2", nb, lambda i: host_pool.pooling_u8(xs[i], n, c, ih, iw, pmax, 4.0, 56, 56, out=ys[i]),
             "32 x 64 x 112 x 112 -> 56 x 56, pad 1")
        both("pooling_u8_mean_2x2_s2", nb, lambda i: host_pool.pooling_u8(xs[i], n, c, ih, iw, pmean, 4.0, 56, 56, out=ys[i]),
             "32 x 64 x 112 x 112 -> 56 x 56")
        half = n * c * ih * iw // 2
        d_in = tensor4df(DT_I8, DF_NCHWC16, n, 128, 56, 56)
        d_out = tensor4df(DT_I8, DF_NCHWC16, n, 256, 56, 56)
        cat = [torch.empty(2 * half, dtype=torch.uint8, device=dev) for _ in range(R)]
        both("concat_i8_rescale_channels", 4 * half,
             lambda i: host_pool.concat([xs[i][:half], xs[i][half:]], [d_in, d_in], 1, d_out, [9.0, 6.5], out=cat[i]),
             "2 x (32 x 128 x 56 x 56) -> 32 x 256 x 56 x 56, one input rescaled by 6.5 / 9, the other copied")
    # -- int8 deconvolution (decoder-style upsampling layer), depthwise convolution, weight-storage converters
    if want("deconv"):
        from bolt_amd import host_deconv
        n, ic, ih, iw, oc, fh, st_, pd = 16, 64, 28, 28, 64, 4, 2, 1
        xq = torch.randint(1, 256, (n * ic * ih * iw,), dtype=torch.uint8, device=dev, generator=g)
        Wd = torch.randint(-127, 128, (ic, oc, fh, fh), dtype=torch.int8, device=dev, generator=g)
        bd_ = torch.randn(oc, device=dev, generator=g) * 0.1
        pd_ = host_deconv.deconv_param_spec(oc, fh, fh, st_, st_, pd, pd, pd, pd)
        dtmp = torch.empty(256 << 20, dtype=torch.uint8, device=dev)
        for odt, nm, tdt in ((DT_U8_Q, "u8_dynamic_scale", torch.uint8), (DT_F32, "f32", torch.float32)):
            idesc, fdesc, odesc, alg = host_deconv.plan(xq, DF_NCHWC16, n, ic, ih, iw, oc, fh, fh, pd_, odt)
            dblob, dftm, _ = host_deconv.transform_filter(Wd, fdesc, pd_, alg)
            oh = fh + st_ * (ih - 1) - 2 * pd
            dout = torch.empty(n * oc * oh * oh, dtype=tdt, device=dev)
            t = timed(lambda: host_deconv.deconvolution(xq, idesc, dblob, dftm, pd_, alg, bd_, [40.0, -1.0, 80.0], True, odesc,
                                                        tmp=dtmp, out=dout), 20)
            ops = 2.0 * n * ih * iw * ic * oc * fh * fh
            res["deconv_4x4_s2_" + nm] = {"config": "16 x 64 x 28 x 28 -> 64 channels, 56 x 56, 4 x 4 kernel, stride 2, pad 1, ReLU (POINTWISE route)",
                                           "ms": t, "tops": ops / t / 1e9,
                                           "algorithmic_bytes": n * ic * ih * iw + ic * oc * fh * fh + n * oc * oh * oh * (1 if odt == DT_U8_Q else 4)}
    if want("depthwise"):
        n, c, ih, iw = 32, 256, 58, 58
        xq = torch.randint(1, 256, (n * c * ih * iw,), dtype=torch.uint8, device=dev, generator=g)
        Ww = torch.randint(-127, 128, (c, 3, 3), dtype=torch.int8, device=dev, generator=g)
        bw = torch.randn(c, device=dev, generator=g) * 0.1
        wblob, wftm = host_conv.depthwise_transform_filter(Ww, c, 3, 3)
        wout = torch.empty(n * c * 56 * 56, dtype=torch.int32, device=dev)
        t = timed(lambda: host_conv.depthwise_convolution_i32(xq, n, c, ih, iw, wblob, wftm, 3, 3, 1, bw, [40.0, -1.0, 80.0], True,
                                                              out=wout), 20)
        byt = n * c * (ih * iw + 4 * 56 * 56)
        res["depthwise_3x3_i32"] = {"config": "32 x 256 x 58 x 58 -> 56 x 56, 3 x 3, stride 1, no padding, ReLU, int32 result",
                                    "ms": t, "algorithmic_bytes": byt, "gbps": byt / t / 1e6, "frac_hbm_peak": byt / t / 1e6 / 8000.0}
    if want("ptq"):
        nW = 3072 * 768
        Wf = torch.randn(nW, device=dev, generator=g) * 0.02
        q8 = torch.empty(nW, dtype=torch.int8, device=dev)
        back = torch.empty(nW, dtype=torch.float32, device=dev)
        sc = (C.c_float * 1)(-1.0)

        def conv8():
            sc[0] = -1.0
            capi.check(L.ws_datatype_converter_int8_gfx950(Wf.data_ptr(), q8.data_ptr(), nW, sc, capi.AMD_GFX950_DEVICE), "ws8")
        t = timed(conv8, 20)
        t2 = timed(lambda: capi.check(L.dequantize_int8_weight_gfx950(nW, sc[0], q8.data_ptr(), back.data_ptr(),
                                                                      capi.AMD_GFX950_DEVICE), "dq8"), 20)
        res["ws_convert_int8_3072x768"] = {"ms": t, "algorithmic_bytes": nW * 9, "gbps": nW * 9 / t / 1e6,
                                           "note": "fp32 -> s8 weight storage with the tensor's own scale returned to the host (two reads, one write)"}
        res["dequantize_int8_weight_3072x768"] = {"ms": t2, "algorithmic_bytes": nW * 5, "gbps": nW * 5 / t2 / 1e6}
    # -- int8 LSTM cell at the decode shape: 256 rows, x 2048 + h 2048 -> 4 x 2048 gates (the headline GEMV, N = 8192,
    #    K = 4096, inside its caller: per-row quantisation, one batched GEMV launch, gates and state update)
    if want("lstm"):
        from bolt_amd import host_lstm
        batch, xdim, hdim = 256, 2048, 2048
        Wl = torch.randint(-127, 128, (4 * hdim, xdim + hdim), dtype=torch.int8, device=dev, generator=g)
        blob = host_lstm.transform_weight(Wl, 4 * hdim, xdim + hdim)
        xl = torch.randn((batch, xdim), device=dev, generator=g)
        bl = torch.randn((batch, 4 * hdim), device=dev, generator=g) * 0.5
        stl = torch.randn((batch, 2 * hdim), device=dev, generator=g) * 0.7
        ol = torch.empty((batch, hdim), device=dev)
        pl = host_lstm.lstm_param_spec(hdim)
        tmp = torch.empty(64 << 20, dtype=torch.uint8, device=dev)
        t = timed(lambda: host_lstm.lstmcell(xl, blob, bl, [-1.0, 250.0], stl, pl, batch, xdim, ol, tmp=tmp), 30)
        per_row = 4 * hdim * (xdim + hdim) + 4 * (xdim + 2 * hdim + 4 * hdim + 2 * hdim + hdim)
        blob2 = host_lstm.rnn_transform_filter(Wl, 4 * hdim, xdim + hdim, pl)
        t2 = timed(lambda: host_lstm.lstmcell(xl, blob2, bl, [-1.0, 250.0], stl, pl, batch, xdim, ol, tmp=tmp,
                                              both_packings=True), 50)
        res["lstmcell_int8_decode_matrix_cores"] = {
            "config": "same call with a weight that also carries the GEMM packing: the 256 rows go through the matrix "
                      "cores as one product that reads the weight once (same bytes out)",
            "ms": t2, "rows_per_s": batch / (t2 * 1e-3), "int8_tops": 2.0 * batch * 4 * hdim * (xdim + hdim) / t2 / 1e9}
        res["lstmcell_int8_decode"] = {"config": "256 rows, x 2048, h 2048 (weight 8192 x 4096 s8, read once per row)",
                                       "ms": t, "rows_per_s": batch / (t * 1e-3), "algorithmic_bytes": batch * per_row,
                                       "gbps": batch * per_row / t / 1e6,
                                       "note": "bytes counted per row: the ONE 33.5 MB weight stays in the 256 MB Infinity "
                                               "Cache between rows, so this is a cache figure, not an HBM fraction"}
    return res


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
    if a.only:
        print(json.dumps({"only": a.only, "other_kernels": other_kernels(L, capi, host, torch, dev, a.only)}), flush=True)
        return
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
    if not a.no_extras:
        out["other_kernels"] = other_kernels(L, capi, host, torch, dev)
        # the GEMM half of the metric next to the GEMV half: the int8 GEMM kernel at 8192^3 through FullyConnected
        # (fp32 result), one launch per call, timed with HIP events on the launch stream
        for ge in out["other_kernels"].get("gemm_int8", []):
            if ge["M"] == 8192 and ge["path"] == "fully_connected" and ge["out"] == "f32":
                tr = json.load(open(tpath)) if os.path.exists(tpath) else {}
                out["roofline_gemm"] = {"bound": "mfma", "achieved": ge["tops"], "peak": MFMA_PEAK_TOPS, "unit": "TOP/s",
                                        "frac": ge["tops"] / MFMA_PEAK_TOPS, "traffic": tr.get("gemm_u8s8_dma_8192"),
                                        "kernel": "gemm_u8s8_dma_kernel<2,4,8,4,5,3> (256 x 256 tiles, ping-pong K loop)",
                                        "launch_ms": ge["ms"], "ops_per_launch": 2 * 8192 ** 3,
                                        "workload": "int8 GEMM M = N = K = 8192 through fully_connected_gfx950, fp32 "
                                                    "result, uniform random operands"}
    if not a.no_cpu_baseline:
        out["cpu_baseline"] = cpu_baseline(W, xq_h, sI_h, float(sW[0]), a.cpu_seconds)
    print(json.dumps(out), flush=True)


if __name__ == "__main__":
    main()
