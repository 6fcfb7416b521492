#!/usr/bin/env python3
"""Benchmark of the quantized dequant-dot hot path on one MI355X.

A step is one pass of the hot path over one batch of synthetic input: one
Q4_K x Q8_K GEMV, N=11008 output rows, K=4096, M=1 token (a 7B model's
gate/up projection at decode), device-resident inputs, launched
back-to-back on one stream.  Consecutive steps read different copies of the
weight matrix, enough of them to exceed the 256 MB Infinity Cache, so the
figure is an HBM figure; the cache-resident rate is reported beside it.

Timing: whatever --steps says, the headline is the MEDIAN over 10 repetitions
of max(256, steps) back-to-back launches each, every repetition bracketed by
HIP events on the launch stream, after one untimed repetition (min and max are
reported beside it).  The prefill GEMM is timed the same way, 5 repetitions of
20 launches.

Prints ONE JSON line:  python bench.py [--gpus 1] [--steps K] [--warmup W]
"""
import argparse
import ctypes
import importlib
import json
import os
import re
import statistics
import subprocess
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)
sys.path.insert(0, os.path.join(ROOT, "tests"))

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
# HBM bytes per headline launch from rocprofv3 FETCH_SIZE + WRITE_SIZE, scaled by the
# same counters on the plain copy kernel: read from the committed counter summary
# (its "traffic_bytes_per_launch:" and "kernel:" lines), so the figure and the kernel
# it was taken on travel together; null when the summary is missing.
TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "gemv_q4_k_11008x4096_hbm_traffic_pmc.txt")
REPS, LAUNCHES_PER_REP = 10, 256
GEMM_LAUNCHES_PER_REP = 20


def traffic_from_profile():
    try:
        text = open(TRAFFIC_PROFILE).read()
    except OSError:
        return None, None
    m = re.search(r"^traffic_bytes_per_launch:\s*(\d+)", text, re.M)
    k = re.search(r"^kernel:\s*(.+)$", text, re.M)
    return (int(m.group(1)) if m else None), (k.group(1).strip() if k else None)


def summarize(per_launch_seconds):
    """median / min / max of the repetitions, in seconds per launch."""
    v = sorted(per_launch_seconds)
    return statistics.median(v), v[0], v[-1]
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published
MALL_BYTES = 256 << 20

FMT_BYTES = {"q4_k": 144, "q5_k": 176, "q6_k": 210, "q8_0": 34}


def gemv_bytes(fmt, rows, K, M=1):
    """Algorithmic bytes of one call: weights + activations + outputs
    (the reference's W + x + y accounting, unittest/test_gemv_q_benchmark.py:397-400)."""
    if fmt == "q8_0":
        w = rows * (K // 32) * 34
        x = M * (K // 32) * 34
    else:
        w = rows * (K // 256) * FMT_BYTES[fmt]
        x = M * (K // 256) * 292
    return w + x + 4 * M * rows


class Harness:
    def __init__(self):
        import torch
        self.torch = torch
        self.ckq = importlib.import_module("c-kernel-engine_amd")
        self.P = self.ckq.parity
        self.L = self.ckq.lib()
        assert self.L.ckq_init() == 0
        import ckq_testlib as T
        self.T = T

    def weight_copies(self, fmt, rows, K, seed, min_total=3 * MALL_BYTES // 2):
        """Distinct device buffers holding the same-shaped matrix (rows rolled
        so the contents differ), enough of them to defeat the Infinity Cache."""
        torch = self.torch
        W = self.T.synth_weights(fmt, rows, K, seed)
        rb = len(W) // rows
        base = torch.from_numpy(W).cuda().view(rows, rb)
        n = max(2, -(-min_total // len(W)))
        copies = [base.reshape(-1)]
        for i in range(1, n):
            copies.append(torch.roll(base, shifts=i * 17, dims=0).contiguous().reshape(-1))
        return W, copies

    def timed_reps(self, run, launches, reps):
        """`reps` repetitions of run(launches), each bracketed by events on the
        launch stream (torch's current stream, the one every *_dev call here is
        given), after one untimed repetition.  Returns seconds per launch of
        every repetition."""
        torch = self.torch
        run(launches)
        torch.cuda.synchronize()
        ev = [(torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)) for _ in range(reps)]
        for e0, e1 in ev:
            e0.record()
            run(launches)
            e1.record()
        torch.cuda.synchronize()
        return [e0.elapsed_time(e1) * 1e-3 / launches for e0, e1 in ev]

    def time_gemm_settled(self, fmt, rows, K, M, copies, xq_d, launches=20, settle_s=0.08):
        """The prefill GEMMs run against the chip's power limit, and the clock the
        power management holds under them settles over tens of milliseconds of
        continuous load (M = 512, 11008x4096: 75-80 us per launch in the first
        milliseconds after idle, 62-64 us from about 50 ms on).  Returns
        (settled, burst): `burst` = summary of the first 5 repetitions of
        `launches` launches after an idle, synchronised GPU (what a short burst
        of calls sees); `settled` = summary of the last third of the repetitions
        of a run that keeps launching, without a gap, for `settle_s` seconds or
        more (what a prefill of many layers sees)."""
        torch, P = self.torch, self.P
        out = torch.empty(M * rows, dtype=torch.float32, device="cuda")
        n = len(copies)
        ops = [(fmt, xq_d, c, None, out, M, rows, K) for c in copies]

        def run(count):
            full, rest = divmod(count, n)
            if full:
                P.dev_matmul_sequence(ops, repeat=full)
            if rest:
                P.dev_matmul_sequence(ops[:rest], repeat=1)

        burst = self.timed_reps(run, launches, 5)
        est = max(summarize(burst)[0], 1e-6)
        reps = max(15, int(settle_s * 1.5 / (est * launches)))
        torch.cuda.synchronize()
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        ev[0].record()
        for i in range(reps):
            run(launches)
            ev[i + 1].record()
        torch.cuda.synchronize()
        t = [ev[i].elapsed_time(ev[i + 1]) * 1e-3 / launches for i in range(reps)]
        return summarize(t[-(reps // 3):]), summarize(burst)

    def time_sequence_settled(self, ops, settle_s=0.1):
        """Median seconds per pass over `ops` (one ckq_matmul_sequence_dev call) in the last third of at
        least `settle_s` seconds of calls without a gap (see time_gemm_settled)."""
        torch, P = self.torch, self.P
        P.dev_matmul_sequence(ops)
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        P.dev_matmul_sequence(ops, repeat=2)
        e1.record()
        torch.cuda.synchronize()
        est = max(e0.elapsed_time(e1) * 0.5e-3, 1e-6)
        per = 4
        reps = max(15, int(settle_s * 1.5 / (est * per)))
        ev = [torch.cuda.Event(enable_timing=True) for _ in range(reps + 1)]
        ev[0].record()
        for i in range(reps):
            P.dev_matmul_sequence(ops, repeat=per)
            ev[i + 1].record()
        torch.cuda.synchronize()
        t = [ev[i].elapsed_time(ev[i + 1]) * 1e-3 / per for i in range(reps)]
        return statistics.median(t[-(reps // 3):])

    def time_gemv(self, fmt, rows, K, M, copies, xq_d, launches=LAUNCHES_PER_REP, reps=REPS, warmup=0):
        """Seconds per launch (median, min, max over the repetitions) of
        back-to-back launches rotating through the weight copies; one C call
        enqueues a whole repetition, so no Python runs between launches."""
        torch, P = self.torch, self.P
        out = torch.empty(M * rows, dtype=torch.float32, device="cuda")
        n = len(copies)
        ops = [(fmt, xq_d, c, None, out, M, rows, K) for c in copies]

        def run(count):
            full, rest = divmod(count, n)
            if full:
                P.dev_matmul_sequence(ops, repeat=full)
            if rest:
                P.dev_matmul_sequence(ops[:rest], repeat=1)

        if warmup:
            run(warmup)
        return summarize(self.timed_reps(run, launches, reps))

    def time_read_floor(self, copies, nbytes, launches=LAUNCHES_PER_REP, reps=5, tuned_search=True):
        """Seconds per launch of kernels that only pull `nbytes` out of the same
        rotated weight buffers: the one-load-per-lane read, and the fastest of a
        small search over the tuned streaming read (grid = what the chip holds,
        several loads in flight per lane)."""
        torch, L = self.torch, self.L
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        stream = ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)
        n = len(copies)
        ptrs = [ctypes.c_void_p(c.data_ptr()) for c in copies]
        sp = ctypes.c_void_p(sink.data_ptr())

        def plain(count):
            for i in range(count):
                L.ckq_read_dev(ptrs[i % n], nbytes, sp, stream)

        res = {"plain": summarize(self.timed_reps(plain, launches, reps))[0]}
        if not tuned_search:
            return res
        cus = torch.cuda.get_device_properties(0).multi_processor_count
        best = None
        for bpc in (2, 4, 8):
            for unroll in (1, 2, 4, 8):
                def tuned(count, b=bpc * cus, u=unroll):
                    for i in range(count):
                        L.ckq_read_tuned_dev(ptrs[i % n], nbytes, sp, b, u, stream)
                t = summarize(self.timed_reps(tuned, launches, 3))[0]
                if best is None or t < best[0]:
                    best = (t, bpc * cus, unroll)
        res["tuned"], res["tuned_blocks"], res["tuned_unroll"] = best
        return res

    def time_sequence(self, layers, launches, reps=5):
        """layers: list of op lists (one per rotated weight set); a step is one
        pass over one layer's ops.  Returns median seconds per step."""
        P = self.P
        flat = [op for layer in layers for op in layer]
        n = len(layers)

        def run(count):
            full, rest = divmod(count, n)
            if full:
                P.dev_matmul_sequence(flat, repeat=full)
            for layer in layers[:rest]:
                P.dev_matmul_sequence(layer, repeat=1)

        return summarize(self.timed_reps(run, launches, reps))[0]


def drop_in_latency(H, W, xq, rows, K):
    """Wall-clock microseconds per synchronous host-pointer call (PCIe copies of
    x and y and a stream synchronisation included): what a generated model pays
    per call when it links this library in place of the CPU kernels.  Never the
    roofline figure."""
    import numpy as np
    T, L = H.T, H.L
    p = T.ptr
    y = np.zeros(rows, np.float32)

    def med(fn, n):
        fn(); fn()
        ts = []
        for _ in range(n):
            t0 = time.perf_counter()
            fn()
            ts.append(time.perf_counter() - t0)
        return round(statistics.median(ts) * 1e6, 1)

    out = {"shape": "Q4_K %dx%d, weights resident, x_q8 %d B up and y %d B down per call" % (rows, K, len(xq), 4 * rows)}
    out["gemv_q4_k_q8_k"] = med(lambda: L.gemv_q4_k_q8_k(p(y), p(W), p(xq), rows, K), 200)
    xf = T.normal(K, 0.0, 1.0, seed=5)
    q = np.zeros(len(xq), np.uint8)
    out["quantize_row_q8_k_K%d" % K] = med(lambda: L.quantize_row_q8_k(p(xf), p(q), K), 200)
    pool = T.ref_pool(H.ckq.lib_path())
    if pool is None:
        out["pool_16_threads"] = None
    else:
        # the reference's own caller: ck_threadpool dispatching gemv_q4_k_q8_k_parallel_simd(ith, nth)
        for threads in (8, 16):
            T.ref_pool_set_threads(pool, threads)
            for whole, tag in ((0, "rows"), (1, "whole")):
                L.ckq_set_parallel_whole(whole)
                out["parallel_dispatch_%d_threads_%s" % (threads, tag)] = med(
                    lambda: pool.gemv_q4_k_q8_k_parallel_dispatch(p(y), p(W), p(xq), rows, K), 100)
        L.ckq_set_parallel_whole(-1)          # back to the library's default
        pool.ck_threadpool_global_destroy()
    # cold start in a fresh process: loading the shared object (dlopen), ckq_init() (HIP start-up, stream, the
    # scratch symbol, which loads the code object) and the first kernel
    code = ("import ctypes, time, numpy as np\n"
            "t0 = time.perf_counter(); L = ctypes.CDLL(%r); t1 = time.perf_counter()\n"
            "rc = L.ckq_init(); t2 = time.perf_counter()\n"
            "x = np.ones(256, np.float32); y = np.zeros(292, np.uint8)\n"
            "L.quantize_row_q8_k(x.ctypes.data_as(ctypes.c_void_p), y.ctypes.data_as(ctypes.c_void_p), 256); t3 = time.perf_counter()\n"
            "print(rc, (t1 - t0) * 1e3, (t2 - t1) * 1e3, (t3 - t2) * 1e3)\n" % H.ckq.lib_path())
    try:
        r = subprocess.run([sys.executable, "-c", code], capture_output=True, text=True, timeout=120)
        rc, load_ms, init_ms, first_ms = r.stdout.split()[-4:]
        out["cold_start_ms"] = {"dlopen": round(float(load_ms), 1), "ckq_init": round(float(init_ms), 1),
                                "first_call": round(float(first_ms), 1), "library_bytes": os.path.getsize(H.ckq.lib_path())}
    except Exception as e:                              # the timing is informative only
        out["cold_start_ms"] = {"error": str(e)[:200]}
    return out


def cpu_baseline(rows, K, seconds_budget=12.0):
    """Q4_K x Q8_K GEMV on the host cores, same shape.  Uses the reference's
    own kernels (oracle/_ref, built from the reference checkout) when that
    library loads, else this repository's restatement."""
    import numpy as np
    import ckq_testlib as T
    W = T.synth_weights("q4_k", rows, K, seed=1)
    xq = T.oracle_quantize(T.normal(K, seed=2), "q8_k")
    y = np.zeros(rows, np.float32)
    kind, lib, fn_name = "port", None, None
    ref = os.path.join(ROOT, "oracle", "_ref", "libckref_avx2.so")
    try:
        lib = ctypes.CDLL(ref)
        fn_name = "gemv_q4_k_q8_k_parallel_simd"
        kind = "reference"
    except OSError:
        lib = T.oracle()
        fn_name = "orc_gemv_q4_k_q8_k_parallel"
    fn = getattr(lib, fn_name)
    nth = max(1, min(os.cpu_count() or 1, 16))
    p = T.ptr

    # persistent threads with one barrier-bracketed round per call (the oracle library's
    # timing harness), as the reference's own pool runs a split GEMV
    orc = T.oracle()
    orc.orc_time_split_gemv.restype = ctypes.c_int
    orc.orc_time_split_gemv.argtypes = [ctypes.c_void_p] * 4 + [ctypes.c_int] * 4 + [ctypes.c_void_p]
    fn_addr = ctypes.cast(fn, ctypes.c_void_p)

    def timed(threads, iters):
        sec = np.zeros(iters, np.float64)
        rc = orc.orc_time_split_gemv(fn_addr, p(y), p(W), p(xq), rows, K, threads, iters, p(sec))
        if rc:
            raise RuntimeError("orc_time_split_gemv failed")
        return sec

    res = {}
    for threads in (1, nth):
        per = max(float(np.median(timed(threads, 5))), 1e-6)
        iters = int(max(20, min(20000, (seconds_budget / 3) / per)))
        ts = timed(threads, iters)
        res[threads] = (float(np.median(ts)), float(ts.mean()), iters)
    bytes_ = gemv_bytes("q4_k", rows, K)
    # the same call rotating over 22 copies of the weights (558 MB): every round reads its weights from DRAM,
    # like the GPU figure, which rotates over more weight bytes than the Infinity Cache holds
    ncopies = 22
    Wrot = np.tile(W, ncopies)
    orc.orc_time_split_gemv_rotating.restype = ctypes.c_int
    orc.orc_time_split_gemv_rotating.argtypes = ([ctypes.c_void_p] * 3 + [ctypes.c_size_t, ctypes.c_int, ctypes.c_void_p] +
                                                 [ctypes.c_int] * 4 + [ctypes.c_void_p])
    it_rot = int(max(2 * ncopies, min(4000, (seconds_budget / 3) / max(res[nth][0], 1e-6))))
    sec = np.zeros(it_rot, np.float64)
    if orc.orc_time_split_gemv_rotating(fn_addr, p(y), p(Wrot), len(W), ncopies, p(xq), rows, K, nth, it_rot, p(sec)):
        raise RuntimeError("orc_time_split_gemv_rotating failed")
    rot_med = float(np.median(sec[ncopies:]))
    del Wrot
    med, mean, iters = res[nth]
    model = "unknown"
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                model = line.split(":", 1)[1].strip()
                break
    except OSError:
        pass
    return {
        "value": round(bytes_ / med / 1e9, 3), "unit": "GB/s", "cores": nth, "kind": kind,
        "host_cores": os.cpu_count(), "cpu_model": model,
        "median_ms": round(med * 1e3, 4), "mean_ms": round(mean * 1e3, 4),
        "single_thread_gbs": round(bytes_ / res[1][0] / 1e9, 3),
        "rotated_gbs": round(bytes_ / rot_med / 1e9, 3), "rotated_median_ms": round(rot_med * 1e3, 4),
        "rotated_sample": "%d calls rotating over %d copies of the weights (%d MB, from DRAM), same threads" % (it_rot, ncopies, ncopies * len(W) >> 20),
        "sample": "%d calls of %s %dx%d M=1 row-split over %d persistent threads, one barrier-bracketed round per call, the same "
                  "25 MB of weights every call (they stay in the host's last-level cache) (median %.2f ms/call, mean %.2f); "
                  "single thread median %.2f ms/call" % (iters, fn_name, rows, K, nth, med * 1e3, mean * 1e3, res[1][0] * 1e3),
    }


# name -> (format, output rows, K, tokens): single workloads a profiler run can ask for with --only
PROFILE_WORKLOADS = {
    "gemv_q4_k_11008x4096": ("q4_k", 11008, 4096, 1),
    "gemm_q4_k_M512_11008x4096": ("q4_k", 11008, 4096, 512),
    "gemv_q6_k_32000x4096": ("q6_k", 32000, 4096, 1),
    "gemv_q6_k_4096x11008": ("q6_k", 4096, 11008, 1),
    "gemm_q6_k_M512_4096x11008": ("q6_k", 4096, 11008, 512),
    "gemm_q4_k_M2048_11008x4096": ("q4_k", 11008, 4096, 2048),
    "gemv_q4_k_4096x4096": ("q4_k", 4096, 4096, 1),
    "layer_7b_decode_chain_M1": None,        # eight launches per layer: four producers, four (grouped) matmuls
}


def build_7b_layer_steps(H):
    """Four rotated 7B decoder layers (502 MB of weights): the projection set as matmul
    entries (`layers`) and the real chain with its activation producers (`chains`)."""
    torch, P, T = H.torch, H.P, H.T
    # a 7B decoder layer's projection set at M=1: Q,K,V,O (4096x4096 Q4_K), gate, up
    # (11008x4096 Q4_K), down (4096x11008 Q6_K), one C call per layer, weights of
    # successive steps distinct (4 rotated layers = 502 MB).  The sequence call issues
    # independent same-shape entries as one launch; to keep the dependencies of a real
    # layer, O reads its activations from V's output buffer, gate/up from O's and down
    # from up's (the bytes are not meaningful activations; the timing does not care),
    # so the launches are Q+K+V | O | gate+up | down.
    x4k = P.dev_quantize(P.to_device(T.normal(4096, seed=31)), "q8_k")
    layers, keep, lbytes = [], [], 0
    for li in range(4):
        ops = []
        for j, (fmt, r, k) in enumerate([("q4_k", 4096, 4096)] * 4 + [("q4_k", 11008, 4096)] * 2 + [("q6_k", 4096, 11008)]):
            Wj = torch.from_numpy(T.synth_weights(fmt, r, k, seed=1000 + j)).cuda()
            if li:
                Wj = torch.roll(Wj.view(r, -1), shifts=li * 13 + j, dims=0).contiguous().reshape(-1)
            o = torch.zeros(r, dtype=torch.float32, device="cuda")
            keep += [Wj, o]
            src = x4k if j < 3 else ops[2][4] if j == 3 else ops[3][4] if j < 6 else ops[5][4]
            ops.append((fmt, src, Wj, None, o, 1, r, k))
            if li == 0:
                lbytes += gemv_bytes(fmt, r, k)
        layers.append(ops)
    # the same layer as the REAL chain, activation quantizers included, one C call per layer:
    # RMSNorm->Q8_K | Q+K+V | Q8_K(attention output; V's output stands in) | O | RMSNorm->Q8_K |
    # gate+up | SiLU(gate)*up->Q8_K | down: four matmul launches and four producer launches
    f32z = lambda n: torch.zeros(n, dtype=torch.float32, device="cuda")
    u8z = lambda n: torch.zeros(n, dtype=torch.uint8, device="cuda")
    xres = P.to_device(T.normal(4096, 0.0, 1.0, seed=32))
    gam = P.to_device(T.normal(4096, 1.0, 0.2, seed=33))
    chains = []
    for ops in layers:
        (q_, k_, v_, o_, g_, u_, d_) = ops
        xq_, aq_, fq_ = u8z(4672), u8z(4672), u8z(4672)
        hq_ = u8z(43 * 292)
        keep += [xq_, aq_, fq_, hq_]
        chains.append([
            ("rmsnorm_q8_k", xres, gam, xq_, 1, 4096, 4096, 1e-5),
            ("q4_k", xq_, q_[2], None, q_[4], 1, 4096, 4096), ("q4_k", xq_, k_[2], None, k_[4], 1, 4096, 4096),
            ("q4_k", xq_, v_[2], None, v_[4], 1, 4096, 4096),
            ("quantize_q8_k", v_[4], None, aq_, 1, 4096),
            ("q4_k", aq_, o_[2], None, o_[4], 1, 4096, 4096),
            ("rmsnorm_q8_k", o_[4], gam, fq_, 1, 4096, 4096, 1e-5),
            ("q4_k", fq_, g_[2], None, g_[4], 1, 11008, 4096), ("q4_k", fq_, u_[2], None, u_[4], 1, 11008, 4096),
            ("swiglu_q8_k", g_[4], u_[4], hq_, 1, 11008, 11008),
            ("q6_k", hq_, d_[2], None, d_[4], 1, 4096, 11008)])
    return layers, chains, keep, lbytes


def copy_calibration(H):
    """The plain copy kernel on 256 MiB, eight launches: known traffic for
    scaling rocprofv3 FETCH_SIZE / WRITE_SIZE readings."""
    torch = H.torch
    n = 256 << 20
    src = torch.empty(n, dtype=torch.uint8, device="cuda").random_(0, 255)
    dst = torch.empty_like(src)
    for _ in range(8):
        H.ckq.api.check(H.L.ckq_copy_dev(ctypes.c_void_p(dst.data_ptr()), ctypes.c_void_p(src.data_ptr()), n,
                                         ctypes.c_void_p(torch.cuda.current_stream().cuda_stream)), "ckq_copy_dev")
    torch.cuda.synchronize()


def clock_trace(H, name, launches, seconds=1.6):
    """Per-repetition launch times of one workload from an idle GPU through
    `seconds` of launches without a gap, with the shader clock rocm-smi reports
    sampled three times during the second half: how long the clock takes to
    settle under the kernel and where it settles."""
    import threading
    fmt, rows, K, M = PROFILE_WORKLOADS[name]
    P, T, torch = H.P, H.T, H.torch
    _, copies = H.weight_copies(fmt, rows, K, seed=rows + K, min_total=(3 * MALL_BYTES // 2) if M == 1 else 1)
    if M > 1:
        copies = copies[:2]
    x = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=K + M)), T.act_fmt(fmt), rows=M)
    out = torch.empty(M * rows, dtype=torch.float32, device="cuda")
    ops = [(fmt, x, c, None, out, M, rows, K) for c in copies]
    n = len(copies)
    launches = max(n, launches // n * n)
    P.dev_matmul_sequence(ops, repeat=1)
    torch.cuda.synchronize()
    time.sleep(0.5)

    sclk = []

    def sample():
        time.sleep(seconds * 0.5)
        for _ in range(3):
            try:
                o = subprocess.run(["rocm-smi", "--showclocks"], capture_output=True, text=True, timeout=20).stdout
                sclk.extend(line.split("(")[-1].split(")")[0] for line in o.splitlines() if "sclk" in line)
            except (OSError, subprocess.SubprocessError) as e:
                sclk.append("rocm-smi failed: %s" % e)
            time.sleep(0.1)

    th = threading.Thread(target=sample)
    th.start()
    t0 = time.perf_counter()
    ev = [torch.cuda.Event(enable_timing=True)]
    ev[0].record()
    while time.perf_counter() - t0 < seconds:
        for _ in range(8):
            P.dev_matmul_sequence(ops, repeat=launches // n)
            e = torch.cuda.Event(enable_timing=True)
            e.record()
            ev.append(e)
        if len(ev) > 17:
            ev[-17].synchronize()        # keep two batches queued: the GPU never waits for Python
    th.join()
    torch.cuda.synchronize()
    us = [ev[i].elapsed_time(ev[i + 1]) * 1e3 / launches for i in range(len(ev) - 1)]
    ms_at = [ev[0].elapsed_time(ev[i + 1]) for i in range(len(us))]
    marks = [0, 1, 2, 3, 5, 8, 12, 17, 25, 35, 50, 70, 100, 140, 200, 300, 500, 800]
    pts = []
    for m in marks:                      # the repetition under way m milliseconds after the first launch
        i = next((k for k, t in enumerate(ms_at) if t >= m), None)
        if i is not None:
            pts.append([m, round(us[i], 2)])
    tail = us[-(len(us) // 3):]
    probes = {}
    if M > 8:
        # what the first launches cost after other work or a short pause instead of a long idle: 12 repetitions of
        # 10 launches right after (a) 150 ms of single-token launches of the same matrix, (b-d) 100 ms of this
        # workload followed by a host sleep of 3 / 30 / 300 ms
        x1 = P.dev_quantize(P.to_device(T.normal(K, 0.0, 1.0, seed=K)), T.act_fmt(fmt))
        o1 = torch.empty(rows, dtype=torch.float32, device="cuda")
        gemv = [(fmt, x1, c, None, o1, 1, rows, K) for c in copies]
        est = max(statistics.median(tail), 1.0) * 1e-6

        def first_reps():
            e = [torch.cuda.Event(enable_timing=True) for _ in range(13)]
            e[0].record()
            for i in range(12):
                P.dev_matmul_sequence(ops, repeat=max(1, 10 // n))
                e[i + 1].record()
            torch.cuda.synchronize()
            per = max(1, 10 // n) * n
            return [round(e[i].elapsed_time(e[i + 1]) * 1e3 / per, 1) for i in range(12)]

        time.sleep(0.5)
        P.dev_matmul_sequence(gemv, repeat=max(1, int(0.15 / 8e-6) // n))
        probes["after_150ms_of_single_token_launches"] = first_reps()
        for pause in (0.003, 0.03, 0.3):
            P.dev_matmul_sequence(ops, repeat=max(1, int(0.1 / est) // n))
            torch.cuda.synchronize()
            time.sleep(pause)
            probes["after_100ms_of_this_workload_then_%gms_idle" % (pause * 1e3)] = first_reps()
    print(json.dumps({"only": name, "clock_trace": True, "launches_per_repetition": launches, "repetitions": len(us),
                      "us_per_launch_at_ms_after_idle": pts,
                      "settled_median_us": round(statistics.median(tail), 3), "sclk_during_second_half": sclk,
                      "first_120_launches_us": probes}))


def run_only(H, name, steps, warmup, calibrate, trace=False):
    if trace and PROFILE_WORKLOADS.get(name):
        clock_trace(H, name, max(1, steps))
        return
    if name == "layer_7b_decode_chain_M1":
        _, chains, keep, _ = build_7b_layer_steps(H)
        sc = H.time_sequence(chains, max(4, steps), 3)
        print(json.dumps({"only": name, "layers_per_repetition": max(4, steps), "repetitions": 4, "median_us_per_layer": round(sc * 1e6, 3)}))
        return
    fmt, rows, K, M = PROFILE_WORKLOADS[name]
    P, T = H.P, H.T
    _, copies = H.weight_copies(fmt, rows, K, seed=rows + K, min_total=(3 * MALL_BYTES // 2) if M == 1 else 1)
    if M > 1:
        copies = copies[:2]
    x = P.dev_quantize(P.to_device(T.normal(M * K, 0.0, 1.0, seed=K + M)), T.act_fmt(fmt), rows=M)
    if calibrate:
        copy_calibration(H)
    if M > 8:
        (med, lo, hi), _ = H.time_gemm_settled(fmt, rows, K, M, copies, x, max(1, steps))
    else:
        med, lo, hi = H.time_gemv(fmt, rows, K, M, copies, x, max(1, steps), 3, warmup=warmup)
    print(json.dumps({"only": name, "launches_per_repetition": max(1, steps), "repetitions": 4,
                      "median_us": round(med * 1e6, 3), "min_us": round(lo * 1e6, 3), "max_us": round(hi * 1e6, 3)}))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-extras", action="store_true", help="only the headline workload and the prefill GEMM")
    ap.add_argument("--no-latency", action="store_true", help="skip the host-pointer (drop-in) latency leg")
    ap.add_argument("--only", choices=sorted(PROFILE_WORKLOADS),
                    help="launch just this workload --steps times and exit (for rocprofv3 runs): no parity guard, "
                         "no CPU leg, a short JSON line")
    ap.add_argument("--clock-trace", action="store_true",
                    help="with --only: launch times from an idle GPU through 1.6 s of continuous launches, and the shader "
                         "clock rocm-smi reports meanwhile")
    ap.add_argument("--calibrate-copy", action="store_true",
                    help="also launch the plain copy kernel on a 256 MiB buffer (known traffic), for scaling "
                         "rocprofv3 FETCH_SIZE / WRITE_SIZE readings")
    a = ap.parse_args()
    if a.gpus != 1:
        sys.exit("bench.py: this build runs on one GPU; --gpus %d is not supported (the path shards by output "
                 "rows, one all-gather per matmul; nothing here uses a second GPU)" % a.gpus)

    H = Harness()
    if a.only:
        run_only(H, a.only, a.steps, a.warmup, a.calibrate_copy, a.clock_trace)
        return
    torch, P, T = H.torch, H.P, H.T
    rows, K, M = 11008, 4096, 1
    xf = T.normal(K, 0.0, 1.0, seed=4242)
    xq_d = P.dev_quantize(P.to_device(xf), "q8_k")
    W, copies = H.weight_copies("q4_k", rows, K, seed=4243)

    if a.calibrate_copy:
        copy_calibration(H)

    # parity guard on the exact buffers being timed
    import numpy as np
    y = P.dev_gemm_nt("q4_k", xq_d, copies[0], None, 1, rows, K).cpu().numpy().reshape(-1)
    err = T.norm_err(y, T.oracle_gemv("q4_k", W, xq_d.cpu().numpy(), rows, K))
    assert err <= 1e-4, "parity check failed before timing: %g" % err

    launches = max(LAUNCHES_PER_REP, a.steps)
    sec, sec_min, sec_max = H.time_gemv("q4_k", rows, K, M, copies, xq_d, launches, REPS, warmup=a.warmup)
    bytes_ = gemv_bytes("q4_k", rows, K, M)
    gbs = bytes_ / sec / 1e9
    sec_hot, _, _ = H.time_gemv("q4_k", rows, K, M, copies[:1], xq_d, launches, 5)
    read = H.time_read_floor(copies, len(W))
    traffic, traffic_kernel = traffic_from_profile()

    out = {
        "metric": "Q4_K GEMV GB/s (% HBM peak) at M=1; Q4_K x Q8_K GEMM TOPS at M=512",
        "value": round(gbs, 2), "unit": "GB/s", "n_gpus": 1, "steps": a.steps, "warmup": a.warmup,
        "ms_per_step": round(sec * 1e3, 6), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "int8 dot (Q4_K x Q8_K), fp32 accumulate", "data": "synthetic",
        "config": {"workload": "Q4_K x Q8_K GEMV N=11008 K=4096 M=1", "weights": "seeded N(0,0.02) -> Q4_K",
                   "activations": "seeded N(0,1) -> Q8_K (quantized on the GPU)",
                   "weight_copies_rotated": len(copies), "bytes_per_step": bytes_},
        "timing": {"method": "median of %d repetitions of %d back-to-back launches, HIP events on the launch stream, "
                             "after one untimed repetition" % (REPS, launches),
                   "median_us": round(sec * 1e6, 3), "min_us": round(sec_min * 1e6, 3), "max_us": round(sec_max * 1e6, 3)},
        "roofline": {"bound": "hbm", "achieved": round(gbs, 2), "peak": HBM_PEAK_GBS, "unit": "GB/s",
                     "frac": round(gbs / HBM_PEAK_GBS, 4), "traffic": traffic, "traffic_kernel": traffic_kernel},
        "pct_hbm_peak": round(100.0 * gbs / HBM_PEAK_GBS, 2),
        "cache_resident_gbs": round(bytes_ / sec_hot / 1e9, 2),
        # launches that only read the same weight bytes from the same rotated buffers: one 16-byte load per
        # lane, and the fastest tuned streaming read (grid = resident blocks, several loads in flight per lane)
        "plain_read_same_bytes": {"us": round(read["plain"] * 1e6, 3), "gbs": round(len(W) / read["plain"] / 1e9, 1),
                                  "gemv_over_read": round(sec / read["plain"], 3)},
        "tuned_read_same_bytes": {"us": round(read["tuned"] * 1e6, 3), "gbs": round(len(W) / read["tuned"] / 1e9, 1),
                                  "blocks": read["tuned_blocks"], "loads_in_flight_per_lane": read["tuned_unroll"],
                                  "gemv_over_read": round(sec / read["tuned"], 3)},
        "parity_norm_err": err,
    }

    # the GEMM half of the metric: prefill, M=512 x N=11008 x K=4096
    Mg = 512
    xg = P.dev_quantize(P.to_device(T.normal(Mg * K, seed=99)), "q8_k", rows=Mg)
    (sg, sg_min, sg_max), (sb, sb_min, sb_max) = H.time_gemm_settled("q4_k", rows, K, Mg, copies[:2], xg, GEMM_LAUNCHES_PER_REP)
    ops = 2.0 * Mg * rows * K
    out["roofline_gemm"] = {"bound": "mfma", "achieved": round(ops / sg / 1e12, 2), "peak": INT8_PEAK_TOPS, "unit": "TOP/s",
                            "frac": round(ops / sg / 1e12 / INT8_PEAK_TOPS, 4),
                            "workload": "Q4_K x Q8_K GEMM M=512 N=11008 K=4096", "ops_per_launch": ops,
                            "median_us": round(sg * 1e6, 2), "min_us": round(sg_min * 1e6, 2), "max_us": round(sg_max * 1e6, 2),
                            "method": "launches without a gap for >= 80 ms, HIP events around every %d; median of the last third of "
                                      "the repetitions (the clock under this kernel settles over ~50 ms of load)" % GEMM_LAUNCHES_PER_REP,
                            "after_idle": {"median_us": round(sb * 1e6, 2), "min_us": round(sb_min * 1e6, 2), "max_us": round(sb_max * 1e6, 2),
                                           "frac": round(ops / sb / 1e12 / INT8_PEAK_TOPS, 4),
                                           "method": "first 5 repetitions of %d launches on a GPU that was idle "
                                                     "(one untimed repetition and a synchronisation before)" % GEMM_LAUNCHES_PER_REP}}

    if not a.no_extras:
        extras = {}
        extras["gemm_q4_k_q8_k_M512"] = {"tops": round(ops / sg / 1e12, 2), "ms": round(sg * 1e3, 4),
                                         "frac_int8_peak": round(ops / sg / 1e12 / INT8_PEAK_TOPS, 4),
                                         "ops_per_call": ops, "kernel": "two-plane int8 MFMA (v_mfma_i32_32x32x32_i8) + bf16 MFMA min term"}
        # a longer prompt: four times the tokens against the same weights
        xg2 = P.dev_quantize(P.to_device(T.normal(2048 * K, seed=98)), "q8_k", rows=2048)
        (sg2, _, _), _ = H.time_gemm_settled("q4_k", rows, K, 2048, copies[:2], xg2, 8)
        extras["gemm_q4_k_q8_k_M2048"] = {"tops": round(2.0 * 2048 * rows * K / sg2 / 1e12, 2), "ms": round(sg2 * 1e3, 4),
                                          "frac_int8_peak": round(2.0 * 2048 * rows * K / sg2 / 1e12 / INT8_PEAK_TOPS, 4),
                                          "ops_per_call": 2.0 * 2048 * rows * K}
        del xg2
        # the same prefill step for the down projection of a Q4_K_M model: Q6_K weights, K = 11008
        r6, k6 = 4096, 11008
        _, cps6 = H.weight_copies("q6_k", r6, k6, seed=66, min_total=1)
        x6 = P.dev_quantize(P.to_device(T.normal(Mg * k6, seed=67)), "q8_k", rows=Mg)
        (s6, _, _), _ = H.time_gemm_settled("q6_k", r6, k6, Mg, cps6[:2] if len(cps6) > 1 else cps6, x6, GEMM_LAUNCHES_PER_REP)
        ops6 = 2.0 * Mg * r6 * k6
        extras["gemm_q6_k_q8_k_M512_4096x11008"] = {"tops": round(ops6 / s6 / 1e12, 2), "ms": round(s6 * 1e3, 4),
                                                    "frac_int8_peak": round(ops6 / s6 / 1e12 / INT8_PEAK_TOPS, 4),
                                                    "ops_per_call": ops6,
                                                    "kernel": "two-plane int8 MFMA on sc*(q-32) split by byte, three LDS stages"}
        del cps6, x6
        torch.cuda.empty_cache()
        # the gate / up shape in the other two K-quant formats (Q5_K_M and Q6_K models): the paired kernels
        for fq, kern in (("q5_k", "two-plane int8 MFMA on sc*q5 split by byte, min term as two more int8 MFMAs; two blocks per CU"),
                         ("q6_k", "two-plane int8 MFMA on sc*(q-32) split by byte; two blocks per CU on 64-token tiles")):
            _, cpsq = H.weight_copies(fq, rows, K, seed=70, min_total=1)
            (sq, _, _), _ = H.time_gemm_settled(fq, rows, K, Mg, cpsq[:2], xg, GEMM_LAUNCHES_PER_REP)
            extras["gemm_%s_q8_k_M512_11008x4096" % fq] = {"tops": round(ops / sq / 1e12, 2), "ms": round(sq * 1e3, 4),
                                                          "frac_int8_peak": round(ops / sq / 1e12 / INT8_PEAK_TOPS, 4),
                                                          "ops_per_call": ops, "kernel": kern}
            del cpsq
        torch.cuda.empty_cache()
        # and for a Q8_0 model's gate/up projection (small model: K = 896) and a 7B-sized one
        for name8, r8, k8 in (("gemm_q8_0_q8_0_M512_9728x896", 9728, 896), ("gemm_q8_0_q8_0_M512_11008x4096", 11008, 4096)):
            _, cps8 = H.weight_copies("q8_0", r8, k8, seed=88, min_total=1)
            x8 = P.dev_quantize(P.to_device(T.normal(Mg * k8, seed=89)), "q8_0", rows=Mg)
            (s8, _, _), _ = H.time_gemm_settled("q8_0", r8, k8, Mg, cps8[:2], x8, GEMM_LAUNCHES_PER_REP)
            ops8 = 2.0 * Mg * r8 * k8
            extras[name8] = {"tops": round(ops8 / s8 / 1e12, 2), "ms": round(s8 * 1e3, 4),
                             "frac_int8_peak": round(ops8 / s8 / 1e12 / INT8_PEAK_TOPS, 4), "ops_per_call": ops8,
                             "kernel": "one int8 MFMA per 32-block, fp16 scale products on the VALU"}
            del cps8, x8
            torch.cuda.empty_cache()
        # the fused prefill MLP of a small model (E = 896, I = 4864): Q8_0 gate/up, Q4_K down, device pointers
        Em, Im = 896, 4864
        xm = P.to_device(T.normal(Mg * Em, seed=90))
        w1m = P.to_device(T.synth_weights("q8_0", 2 * Im, Em, seed=91, std=0.25))
        w2m = P.to_device(T.synth_weights("q4_k", Em, Im, seed=92))
        outm = torch.empty(Mg * Em, dtype=torch.float32, device="cuda")
        scr = torch.zeros(16, dtype=torch.uint8, device="cuda")
        def mlp():
            H.L.fused_mlp_swiglu_prefill_w1w2_quant(P._dp(xm), P._dp(w1m), None, P.CK_DT["q8_0"], P._dp(w2m), None,
                                                    P.CK_DT["q4_k"], P._dp(outm), Mg, Em, Em, Im, Im, P._dp(scr))
        mlp(); mlp()
        import time as _t
        t0 = _t.perf_counter()
        for _ in range(10):
            mlp()                                   # synchronous entry point
        tm = (_t.perf_counter() - t0) / 10
        opsm = 2.0 * Mg * (2 * Im * Em + Em * Im)
        extras["fused_mlp_prefill_M512_E896_I4864"] = {"ms": round(tm * 1e3, 4), "tops": round(opsm / tm / 1e12, 2),
                                                       "note": "synchronous call: four kernels and a stream sync"}
        del xm, w1m, w2m, outm
        torch.cuda.empty_cache()
        for name, fmt, r, k in (("gemv_q4_k_4096x4096", "q4_k", 4096, 4096),
                                ("lm_head_q6_k_32000x4096", "q6_k", 32000, 4096),
                                ("down_q6_k_4096x11008", "q6_k", 4096, 11008),
                                ("lm_head_q8_0_151936x896", "q8_0", 151936, 896)):
            _, cps = H.weight_copies(fmt, r, k, seed=r + k)
            xq = P.dev_quantize(P.to_device(T.normal(k, seed=k)), T.act_fmt(fmt))
            s, _, _ = H.time_gemv(fmt, r, k, 1, cps, xq, 128, 5)
            b = gemv_bytes(fmt, r, k)
            rd = H.time_read_floor(cps, r * T.row_bytes(fmt, k), 128, 5, tuned_search=False)["plain"]
            extras[name] = {"gbs": round(b / s / 1e9, 1), "us": round(s * 1e6, 2), "frac_hbm": round(b / s / 1e9 / HBM_PEAK_GBS, 4),
                            "read_same_bytes_us": round(rd * 1e6, 2), "gemv_over_read": round(s / rd, 3)}
            del cps
            torch.cuda.empty_cache()
        # fp32-activation entry point (gemv_q4_k: weights dequantized on the fly, nothing quantized)
        xf_d = P.to_device(xf)
        outf = torch.empty(rows, dtype=torch.float32, device="cuda")
        sf = H.time_sequence([[("q4_k+f32", xf_d, c, None, outf, 1, rows, K)] for c in copies], 128, 5)
        bf = len(W) + 4 * K + 4 * rows
        extras["gemv_q4_k_f32act_11008x4096"] = {"gbs": round(bf / sf / 1e9, 1), "us": round(sf * 1e6, 2),
                                                 "frac_hbm": round(bf / sf / 1e9 / HBM_PEAK_GBS, 4),
                                                 "note": "fp32 activations, weights dequantized on the fly; back-to-back launches of one C call"}

        # fused producer rmsnorm -> Q8_K next to the plain quantizer (launch-bound at one token)
        gam_d = P.to_device(T.normal(K, 1.0, 0.2, seed=55))
        prod = {}
        for tk in (1, 512):
            xin = P.to_device(T.normal(tk * K, 0.0, 1.0, seed=56))
            for name, fn in (("rmsnorm_q8_k_fused", lambda: P.dev_rmsnorm_q8_k_fused(xin, gam_d, tk, K)),
                             ("quantize_q8_k", lambda: P.dev_quantize(xin, "q8_k", rows=tk))):
                for _ in range(5):
                    fn()
                torch.cuda.synchronize()
                e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
                e0.record()
                for _ in range(100):
                    fn()
                e1.record()
                torch.cuda.synchronize()
                prod["%s_T%d_us" % (name, tk)] = round(e0.elapsed_time(e1) * 10.0, 2)
        extras["producer_d4096"] = prod

        layers, chains, keep, lbytes = build_7b_layer_steps(H)
        s = H.time_sequence(layers, 64, 5)
        extras["layer_7b_projection_set_M1"] = {"us": round(s * 1e6, 2), "gbs": round(lbytes / s / 1e9, 1), "bytes": lbytes,
                                                "frac_hbm": round(lbytes / s / 1e9 / HBM_PEAK_GBS, 4), "launches": 4,
                                                "note": "Q+K+V and gate+up each as one grouped launch"}
        sc = H.time_sequence(chains, 64, 5)
        extras["layer_7b_decode_chain_M1"] = {"us": round(sc * 1e6, 2), "matmul_only_us": round(s * 1e6, 2),
                                              "producers_us": round((sc - s) * 1e6, 2), "launches": 8,
                                              "gbs_of_weight_bytes": round(lbytes / sc / 1e9, 1),
                                              "note": "norm->Q8_K, Q+K+V, Q8_K, O, norm->Q8_K, gate+up, SwiGLU->Q8_K, down in one C call"}
        del layers, keep, chains
        torch.cuda.empty_cache()

        # the same layer's projection set at prefill size (512 tokens, grouped-query attention: K and V
        # 1024 rows): Q,K,V | O | gate,up | down.  The sequence call issues Q+K+V and gate+up as one
        # matrix-core launch each; the same entries one launch each are timed beside it.
        Mp = 512
        xp = P.dev_quantize(P.to_device(T.normal(Mp * 4096, seed=34)), "q8_k", rows=Mp)
        hp = P.dev_quantize(P.to_device(T.normal(Mp * 11008, seed=35)), "q8_k", rows=Mp)
        pops, pkeep, pflop = [], [], 0.0
        for j, (fmt, r, k) in enumerate([("q4_k", 4096, 4096), ("q4_k", 1024, 4096), ("q4_k", 1024, 4096), ("q4_k", 4096, 4096),
                                         ("q4_k", 11008, 4096), ("q4_k", 11008, 4096), ("q6_k", 4096, 11008)]):
            Wj = torch.from_numpy(T.synth_weights(fmt, r, k, seed=1100 + j)).cuda()
            o = torch.zeros(Mp * r, dtype=torch.float32, device="cuda")
            pkeep += [Wj, o]
            pops.append((fmt, hp if k == 11008 else xp, Wj, None, o, Mp, r, k))
            pflop += 2.0 * Mp * r * k
        # O must not join the Q/K/V group, nor gate/up the one before: give them their own activations
        xp2 = xp.clone()
        pops[3] = pops[3][:1] + (xp2,) + pops[3][2:]
        xp3 = xp.clone()
        pops[4] = pops[4][:1] + (xp3,) + pops[4][2:]
        pops[5] = pops[5][:1] + (xp3,) + pops[5][2:]
        pre = {}
        for label, on in (("grouped", 1), ("one_launch_per_matrix", 0)):
            H.L.ckq_set_prefill_grouping(on)
            sp_ = H.time_sequence_settled(pops)
            pre[label + "_us"] = round(sp_ * 1e6, 2)
        H.L.ckq_set_prefill_grouping(1)
        pre.update({"tops": round(pflop / (pre["grouped_us"] * 1e-6) / 1e12, 1), "ops": pflop,
                    "launches_grouped": 4, "launches_ungrouped": "7 (K and V each with a K split and its reduction)",
                    "note": "Q 4096, K and V 1024, O 4096 (Q4_K, K = 4096), gate and up 11008 (Q4_K), down 4096x11008 (Q6_K); "
                            "clock settled"})
        extras["layer_7b_prefill_set_M512"] = pre
        del pops, pkeep, xp, xp2, xp3, hp
        torch.cuda.empty_cache()

        # small-model batched decode (Qwen2-0.5B-like: hidden 896 padded to K=1024, Q5_K
        # projections, Q8_0 LM head 151936x896), M tokens per step
        proj = [(896, 1024), (128, 1024), (128, 1024), (896, 1024), (4864, 1024), (4864, 1024), (896, 4864)]
        Wp = [torch.from_numpy(T.synth_weights("q5_k", r, k, seed=2000 + i)).cuda() for i, (r, k) in enumerate(proj)]
        _, heads = H.weight_copies("q8_0", 151936, 896, seed=2100, min_total=2 * MALL_BYTES)
        small = {}
        for Mb in (1, 2, 4, 8):
            xa = P.dev_quantize(P.to_device(T.normal(Mb * 1024, seed=41)), "q8_k", rows=Mb)
            xh = P.dev_quantize(P.to_device(T.normal(Mb * 896, seed=43)), "q8_0", rows=Mb)
            layers, nbytes = [], 0
            for hi, head in enumerate(heads):
                ops = []
                for j, ((r, k), Wj) in enumerate(zip(proj, Wp)):
                    # dependencies of a real layer, as in the 7B list: O reads Q's output buffer,
                    # gate/up read O's, down reads up's; Q, K, V (one input, K and V narrower) and
                    # gate, up are independent and share a launch at one token
                    src = xa if j < 3 else ops[0][4] if j == 3 else ops[3][4] if j < 6 else ops[5][4]
                    ops.append(("q5_k", src, Wj, None, torch.zeros(Mb * r, dtype=torch.float32, device="cuda"), Mb, r, k))
                    if hi == 0:
                        nbytes += gemv_bytes("q5_k", r, k, Mb)
                ops.append(("q8_0", xh, head, None, torch.empty(Mb * 151936, dtype=torch.float32, device="cuda"), Mb, 151936, 896))
                if hi == 0:
                    nbytes += gemv_bytes("q8_0", 151936, 896, Mb)
                layers.append(ops)
            s = H.time_sequence(layers, 32, 5)
            small["M%d" % Mb] = {"us": round(s * 1e6, 2), "gbs": round(nbytes / s / 1e9, 1), "tokens_per_s": round(Mb / s, 1)}
            del layers
        extras["small_model_decode_q5_k_layer_plus_q8_0_head"] = small
        del heads, Wp
        torch.cuda.empty_cache()
        out["extras"] = extras

    if not a.no_latency:
        out["drop_in_latency_us"] = drop_in_latency(H, W, xq_d.cpu().numpy(), rows, K)
    if not a.no_cpu:
        out["cpu_baseline"] = cpu_baseline(rows, K)
    print(json.dumps(out))


if __name__ == "__main__":
    main()
