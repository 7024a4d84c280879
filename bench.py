#!/usr/bin/env python3
"""Benchmark of the matmul hot path on one MI355X.

Headline workload (BASELINE.json configs[2], the one the north-star target is quoted on):
  uint8 [4096,4096] (zero-point 128) x int8 [4096,4096] (symmetric) -> int32 accumulate ->
  requantize to uint8 with scale 1/(K*64), zero-point 128, through the fused kernel
  (tfcc_rocm_gemm_u8s8s32_requant_u8, int32 accumulators not written).
One step = one such product with inputs resident in HBM.  value = 2*M*N*K / time, in TOP/s.

The same JSON line carries
  roofline      the dominant kernel against the int8 MFMA peak (5.0 POP/s dense); the same kernel after a long
                warm-up ("settled", with the shader clock and socket power the driver reports meanwhile: sclk_mhz,
                power_w) and as a short burst after idle ("burst"); what the matrix cores sustain alone on this box
                (matrix_cores_alone: register-resident loops with constant and with changing operands, in the
                kernel's own issue order with 32x32x32 and 16x16x64 instructions, and with the matrix cores busy only
                part of the time), each with its clock and power
  cpu_baseline  the reference's own AVX2 quantized matmul + requantize (oracle/_ref, kind
                "reference") or, where that library is absent, the scalar C oracle (kind "port"),
                timed on this host's cores on a bounded sample, with all threads and with the four the
                reference's test harness uses; an fp32 leg (C1 and the GEMMs of C4) through a plain
                OpenMP port and through the CPU BLAS torch ships; the CPU model
  other         the remaining BASELINE configs (fp32 GEMM + bias, attention-shaped batched fp32,
                skinny int8 decode GEMV, int32-writing variant), each with its own roofline figure

usage: python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-cpu] [--no-other] [--no-sampler]
"""
import argparse
import ctypes as C
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, ROOT)

PEAK_INT8_TOPS = 5000.0   # MI355X dense int8 MFMA
PEAK_FP32_TFLOPS = 157.3  # MI355X fp32 MFMA
PEAK_HBM_GBS = 8000.0     # MI355X HBM3E


_bench_lib = None


def bench_lib():
    """The benchmark's own measuring aids (wechat-tfcc_amd/csrc/probe.h): not part of the product library."""
    global _bench_lib
    if _bench_lib is None:
        path = os.path.join(ROOT, "wechat-tfcc_amd", "libtfcc_bench.so")
        if not os.path.exists(path):
            sys.exit("libtfcc_bench.so is missing: run __graft_entry__.build() first")
        lib = C.CDLL(path)
        lib.tfcc_bench_probe_mfma.argtypes = [C.c_void_p, C.c_int, C.c_int, C.c_uint, C.c_uint, C.c_void_p]
        lib.tfcc_bench_probe_mfma_duty.argtypes = [C.c_void_p, C.c_int, C.c_uint, C.c_uint, C.c_void_p]
        lib.tfcc_bench_probe_read.argtypes = [C.c_void_p, C.c_void_p, C.c_uint64, C.c_uint, C.c_void_p]
        lib.tfcc_bench_probe_launch.argtypes = [C.c_void_p, C.c_void_p]
        _bench_lib = lib
    return _bench_lib


def probe_check(status):
    if status != 0:
        sys.exit("measuring probe failed with status %d" % status)


# ---- clock and power of the GPU while a leg runs ---------------------------------------------------------------
# A child process, started before this process makes its first GPU call, samples what the driver publishes in
# sysfs - the shader clock (the level marked current in pp_dpm_sclk, what rocm-smi --showclocks prints) and the
# socket power (hwmon power1_input, what rocm-smi --showpower / amd-smi metric --power print) - every few
# milliseconds, with CLOCK_MONOTONIC stamps; the parent brackets a leg with the same clock and reads the samples
# that fall inside it.  The child only reads files: it never touches the GPU runtime.
_SAMPLER_CODE = r"""
import glob, os, sys, time
out, period = sys.argv[1], float(sys.argv[2])
dev = None
for d in sorted(glob.glob('/sys/class/drm/card*/device')):
    if os.path.exists(os.path.join(d, 'pp_dpm_sclk')):
        dev = d
        break
power = None
cap = None
if dev:
    for h in sorted(glob.glob(os.path.join(dev, 'hwmon', 'hwmon*'))):
        for name in ('power1_input', 'power1_average'):
            if os.path.exists(os.path.join(h, name)):
                power = os.path.join(h, name)
                break
        if power:
            if os.path.exists(os.path.join(h, 'power1_cap')):
                cap = open(os.path.join(h, 'power1_cap')).read().strip()
            break
f = open(out, 'w')
f.write('# source %s power %s cap_uW %s\n' % (dev, power, cap))
f.flush()
if not dev:
    sys.exit(0)
sclk = os.path.join(dev, 'pp_dpm_sclk')
while not os.path.exists(out + '.stop'):
    t = time.monotonic()
    mhz = -1
    try:
        for line in open(sclk):
            if '*' in line:
                mhz = int(''.join(ch for ch in line.split(':')[1] if ch.isdigit()))
    except (OSError, ValueError, IndexError):
        pass
    uw = -1
    if power:
        try:
            uw = int(open(power).read())
        except (OSError, ValueError):
            pass
    f.write('%.6f %d %d\n' % (t, mhz, uw))
    f.flush()
    rest = period - (time.monotonic() - t)
    if rest > 0:
        time.sleep(rest)
"""


class GpuSampler:
    def __init__(self, period_s=0.002):
        import subprocess
        import tempfile
        self.path = os.path.join(tempfile.mkdtemp(prefix="tfcc_bench_"), "samples.txt")
        self.proc = None
        self.error = None
        try:
            self.proc = subprocess.Popen([sys.executable, "-c", _SAMPLER_CODE, self.path, str(period_s)],
                                         stdin=subprocess.DEVNULL, stdout=subprocess.DEVNULL, stderr=subprocess.DEVNULL)
        except OSError as e:
            self.error = "sampler did not start: %s" % e

    def window(self, t0, t1):
        """Clock and power over the samples stamped inside [t0, t1] (time.monotonic() of this process)."""
        if self.proc is None:
            return {"available": False, "why": self.error}
        header, rows = "", []
        try:
            for line in open(self.path):
                if line.startswith("#"):
                    header = line[1:].strip()
                    continue
                parts = line.split()
                if len(parts) == 3 and t0 <= float(parts[0]) <= t1:
                    rows.append((int(parts[1]), int(parts[2])))
        except OSError as e:
            return {"available": False, "why": "no samples: %s" % e}
        mhz = [r[0] for r in rows if r[0] > 0]
        watts = [r[1] / 1e6 for r in rows if r[1] > 0]
        if not mhz and not watts:
            return {"available": False, "why": "neither pp_dpm_sclk nor hwmon power answered on this box (%s)" % header,
                    "samples": len(rows)}
        med = lambda v: round(sorted(v)[len(v) // 2], 1) if v else None  # noqa: E731
        res = {"available": True, "samples": len(rows), "sclk_mhz": med(mhz), "sclk_mhz_min": min(mhz) if mhz else None,
               "sclk_mhz_max": max(mhz) if mhz else None, "power_w": med(watts),
               "power_w_max": round(max(watts), 1) if watts else None, "source": header}
        cap = header.split("cap_uW")[-1].strip() if "cap_uW" in header else ""
        if cap.isdigit():
            res["power_cap_w"] = int(cap) / 1e6
        return res

    def close(self):
        if self.proc is not None:
            try:
                open(self.path + ".stop", "w").close()
                self.proc.wait(timeout=5)
            except Exception:
                self.proc.kill()
            self.proc = None


def time_launches(torch, fn, steps, warmup, pkg=None, stream=0):
    """Average duration of one call in ms, measured with HIP events on the stream fn launches on.
    With pkg and a (non-default) stream the timed launches are recorded once into a HIP graph and the graph
    is replayed: kernels of a few microseconds are otherwise limited by the Python launch loop, not the GPU."""
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    if pkg is not None and stream:
        import ctypes
        lib = pkg.lib()
        graph = ctypes.c_void_p()
        pkg.check(lib.tfcc_rocm_stream_begin_capture(stream))
        for _ in range(steps):
            fn()
        pkg.check(lib.tfcc_rocm_stream_end_capture(stream, ctypes.byref(graph)))
        pkg.check(lib.tfcc_rocm_graph_launch(graph, stream))  # first replay untimed
        torch.cuda.synchronize()
        start.record()
        pkg.check(lib.tfcc_rocm_graph_launch(graph, stream))
        stop.record()
        torch.cuda.synchronize()
        pkg.check(lib.tfcc_rocm_graph_destroy(graph))
        return start.elapsed_time(stop) / steps
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) / steps


def c3_setup(torch, pkg, dev, seed=0, size=4096):
    rng = np.random.default_rng(seed)
    a = rng.integers(0, 256, (size, size), dtype=np.uint8)
    b = rng.integers(-127, 128, (size, size), dtype=np.int8)
    ta, tb = torch.from_numpy(a).to(dev), torch.from_numpy(b).to(dev)
    rs, cs = pkg.reduce_sum(ta, True), pkg.reduce_sum(tb, False)
    f1 = lambda v: torch.tensor([v], dtype=torch.float32, device=dev)
    ranges = [f1(-128.0), f1(127.0), f1(-128.0), f1(127.0)]
    out_range = [f1(-128.0 * size * 64.0), f1(127.0 * size * 64.0)]
    return a, b, ta, tb, rs, cs, ranges, out_range


def make_c3_step(torch, pkg, ta, tb, rs, cs, ranges, out_range, want_acc, colsum_exact=False):
    """A closure that launches exactly one fused product into preallocated outputs."""
    m, k = ta.shape
    n = tb.shape[1]
    d = pkg.QGemmDesc()
    d.a, d.b, d.rowsum_a, d.colsum_b = ta.data_ptr(), tb.data_ptr(), rs.data_ptr(), cs.data_ptr()
    d.m, d.n, d.k, d.batch, d.stride_c = m, n, k, 1, m * n
    d.min_a, d.max_a, d.min_b, d.max_b = [r.data_ptr() for r in ranges]
    mn_c = torch.empty(1, dtype=torch.float32, device=ta.device)
    mx_c = torch.empty(1, dtype=torch.float32, device=ta.device)
    d.min_c, d.max_c = mn_c.data_ptr(), mx_c.data_ptr()
    d.colsum_b_is_exact = 1 if colsum_exact else 0
    q = torch.empty((m, n), dtype=torch.uint8, device=ta.device)
    acc = torch.empty((m, n), dtype=torch.int32, device=ta.device) if want_acc else None
    lib = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream
    acc_ptr = None if acc is None else acc.data_ptr()
    keep = (d, mn_c, mx_c, q, acc)

    def step():
        st = lib.tfcc_rocm_gemm_u8s8s32_requant_u8(stream, C.byref(d), acc_ptr, q.data_ptr(), 0.0, 0.0, 0.0, 0,
                                                   out_range[0].data_ptr(), out_range[1].data_ptr())
        if st != 0:
            pkg.check(st)
    step.keep = keep
    step.q = q
    step.acc = acc
    return step


def cpu_model_name():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_baseline(a, b, size):
    """The reference's CPU path on this host's cores, on bounded samples (about 25 s in all).
    int8 (the headline's workload): the reference's own AVX2 quantized matmul (offset matrix + kernel) followed by its
    AVX2 requantize, both from oracle/_ref, with every thread the process may use and with the four threads the
    reference's test harness runs on (tfcc/test/environment.cpp:40); the scalar C oracle on a smaller sample where
    oracle/_ref has not been built.
    fp32 (C1 and the six GEMMs of C4's layer): the reference's arithmetic lives in oneDNN 1.8.1, which is not in this
    image, so two stand-ins are timed: a plain OpenMP port in the oracle library (kind "port") and torch's CPU matmul
    (the BLAS torch ships: a vendor library, not oneDNN 1.8.1)."""
    sys.path.insert(0, os.path.join(ROOT, "tests"))
    import oracle_lib as O
    cores = len(os.sched_getaffinity(0))
    threads = min(int(os.environ.get("OMP_NUM_THREADS", cores)), cores)
    orc = O.oracle()
    orc.oracle_set_num_threads.argtypes = [C.c_int]
    orc.oracle_sgemm_f32_timing.argtypes = [C.c_void_p] * 4 + [C.c_uint] * 3
    orc.oracle_sgemm_f32_timing.restype = None
    ref = O.ref()
    ranges = (-128.0, 127.0, -128.0, 127.0)
    result = {}

    def int8_leg(nthreads, budget):
        orc.oracle_set_num_threads(nthreads)  # one OpenMP runtime in the process: the reference's kernels follow it
        rs, cs = O.reduce_sum(a, True), O.reduce_sum(b, False)
        oa, ob = O.qmatmul_offsets(*ranges, lib=ref)
        mn_c, mx_c = O.qmatmul_range(*ranges, lib=ref)
        q = np.empty((size, size), np.uint8)
        O.qgemm(a[:256], b, oa, ob, rs[:256], cs, lib=ref)  # warm the thread pool
        reps, t0 = 0, time.perf_counter()
        while True:
            c = O.qgemm(a, b, oa, ob, rs, cs, lib=ref)
            ref.ref_requantize_s32_u8(c.reshape(-1), c.size, mn_c, mx_c, -128.0 * size * 64.0, 127.0 * size * 64.0, 1,
                                      q.reshape(-1))
            reps += 1
            dt = time.perf_counter() - t0
            if dt > budget or reps >= 400:
                break
        return 2.0 * size ** 3 * reps / dt / 1e12, reps, dt

    if ref is not None:
        tops, reps, dt = int8_leg(threads, 8.0)
        result = {"value": round(tops, 4), "unit": "TOP/s", "cores": threads, "kind": "reference",
                  "sample": "%d full %d^3 products + requantize through the reference's AVX2 kernels (oracle/_ref), "
                            "%.1f s, %d OpenMP threads" % (reps, size, dt, threads)}
        tops4, reps4, dt4 = int8_leg(min(4, threads), 5.0)
        result["threads_4"] = {"value": round(tops4, 4), "unit": "TOP/s", "cores": min(4, threads),
                               "sample": "%d products, %.1f s (the thread count of the reference's test harness)" % (reps4, dt4)}
    else:
        sub = 1024
        sa, sb = np.ascontiguousarray(a[:sub, :sub]), np.ascontiguousarray(b[:sub, :sub])
        t0 = time.perf_counter()
        c = O.qgemm(sa, sb, -128, 0)
        O.requantize_s32_u8(c, -2147483648.0, 2147483648.0, -128.0 * sub * 64.0, 127.0 * sub * 64.0)
        dt = time.perf_counter() - t0
        result = {"value": round(2.0 * sub ** 3 / dt / 1e12, 5), "unit": "TOP/s", "cores": 1, "kind": "port",
                  "sample": "one %d^3 product + requantize through the scalar C oracle, %.1f s" % (sub, dt)}
    result["cpu_model"] = cpu_model_name()
    result["host_cores"] = cores

    # ---- fp32
    rng = np.random.default_rng(3)
    shapes = {"c1_128x768x3072_bias": [(128, 768, 3072)],
              "c4_layer_gemms_b8_s128": [(1024, 768, 768)] * 4 + [(1024, 768, 3072), (1024, 3072, 768)] +
                                        [(128, 64, 128)] * 96 + [(128, 128, 64)] * 96}
    fp32 = {}
    try:
        import torch
    except ImportError:
        torch = None
    for name, products in shapes.items():
        flop = sum(2.0 * m * n * k for m, k, n in products)
        distinct = sorted(set(products))
        ops = {sh: (rng.uniform(-1, 1, (sh[0], sh[1])).astype(np.float32), rng.uniform(-1, 1, (sh[1], sh[2])).astype(np.float32),
                    rng.uniform(-0.1, 0.1, sh[2]).astype(np.float32), np.empty((sh[0], sh[2]), np.float32)) for sh in distinct}
        entry = {"gflop_per_pass": round(flop / 1e9, 3)}
        for label, nthreads in (("all_threads", threads), ("threads_4", min(4, threads))):
            orc.oracle_set_num_threads(nthreads)

            def port_pass():
                for sh in products:
                    x, w, bias, out = ops[sh]
                    orc.oracle_sgemm_f32_timing(x.ctypes.data, w.ctypes.data, bias.ctypes.data, out.ctypes.data, sh[0], sh[2], sh[1])
            port_pass()
            reps, t0 = 0, time.perf_counter()
            while True:
                port_pass()
                reps += 1
                dt = time.perf_counter() - t0
                if dt > 1.5 or reps >= 200:
                    break
            entry["port_%s" % label] = {"gflops": round(flop * reps / dt / 1e9, 1), "cores": nthreads, "kind": "port",
                                        "sample": "%d passes, %.1f s, OpenMP rows x vectorised inner loop" % (reps, dt)}
            if torch is not None:
                torch.set_num_threads(nthreads)
                tops_ = {sh: (torch.from_numpy(v[0]), torch.from_numpy(v[1]), torch.from_numpy(v[2])) for sh, v in ops.items()}

                def torch_pass():
                    for sh in products:
                        x, w, bias = tops_[sh]
                        torch.addmm(bias, x, w)
                torch_pass()
                reps, t0 = 0, time.perf_counter()
                while True:
                    torch_pass()
                    reps += 1
                    dt = time.perf_counter() - t0
                    if dt > 1.5 or reps >= 500:
                        break
                entry["vendor_blas_%s" % label] = {
                    "gflops": round(flop * reps / dt / 1e9, 1), "cores": nthreads,
                    "kind": "torch %s CPU addmm: vendor BLAS, not the reference's oneDNN 1.8.1" % torch.__version__,
                    "sample": "%d passes, %.1f s" % (reps, dt)}
        fp32[name] = entry
    result["fp32"] = fp32
    return result


def bench_other(torch, pkg, dev, steps, warmup, c3, short_legs=False):
    """Remaining BASELINE configs; each entry: ms, achieved rate, bound, fraction of the bounding peak."""
    out = {}
    # These launches take microseconds: a handful of them after the host-side set-up of a case measures the clock
    # ramp and the first touch of the rotated buffers, not the kernel.  Whatever --steps / --warmup say, every case
    # here runs at least 300 untimed and 500 timed launches (the counts used are part of the output), unless
    # --short-legs asks for the given counts (counter collection, where every launch is slow).
    if not short_legs:
        steps, warmup = max(steps, 500), max(warmup, 300)
    out["launch_counts"] = {"timed": steps, "warmup": warmup}
    rng = np.random.default_rng(1)
    t = lambda x: torch.from_numpy(np.ascontiguousarray(x)).to(dev)
    lib = pkg.lib()
    stream = torch.cuda.current_stream().cuda_stream

    LLC_BYTES = 256 << 20  # last-level cache: a rotation of operand sets must exceed it to measure HBM

    def sets_beyond_llc(bytes_per_set):
        return max(2, int(1.25 * LLC_BYTES / bytes_per_set) + 1)

    def sgemm_case(name, shape_a, shape_b, bias, sets=None, step_by_step=False):
        p = pkg.matmul_plan(shape_a, shape_b, None if not bias else (shape_b[-1],))
        # operand sets rotated over more bytes than the last-level cache holds (sets=1: compute-bound, no rotation)
        per_set = 4 * (int(np.prod(shape_a)) + int(np.prod(shape_b)) + int(np.prod(p["shape"])))
        sets = sets or sets_beyond_llc(per_set)
        bufs = []
        for _ in range(sets):
            a = torch.randn(shape_a, device=dev, dtype=torch.float32)
            b = torch.randn(shape_b, device=dev, dtype=torch.float32)
            bi = torch.randn(shape_b[-1], device=dev, dtype=torch.float32) if bias else None
            c = torch.empty(p["shape"], device=dev, dtype=torch.float32)
            bufs.append((a, b, bi, c))
        idx = [0]

        def step():
            a, b, bi, c = bufs[idx[0] % sets]
            idx[0] += 1
            st = lib.tfcc_rocm_sgemm_strided_batched(stream, a.data_ptr(), p["stride_a"], b.data_ptr(), p["stride_b"],
                                                     None if bi is None else bi.data_ptr(), c.data_ptr(), p["stride_c"],
                                                     p["m"], p["n"], p["k"], p["batch"])
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, steps, warmup, pkg, stream)
        flop = 2.0 * p["m"] * p["n"] * p["k"] * p["batch"] + (p["m"] * p["n"] * p["batch"] if bias else 0)
        nbytes = 4.0 * (int(np.prod(shape_a)) + int(np.prod(shape_b)) + int(np.prod(p["shape"])) + (shape_b[-1] if bias else 0))
        tflops, gbs = flop / ms / 1e9, nbytes / ms / 1e6
        out[name] = {"ms": round(ms, 5), "tflops": round(tflops, 3), "frac_fp32_mfma": round(tflops / PEAK_FP32_TFLOPS, 4),
                     "gbs": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
        if step_by_step:
            # The same launches issued one by one instead of replayed from a recorded graph: the difference is what a
            # graph node costs over a plain launch on this runtime (the kernel is long enough to hide the host's launch cost).
            out[name]["ms_step_by_step"] = round(time_launches(torch, step, max(steps, 300), warmup), 5)

    sgemm_case("c1_fp32_128x768x3072_bias", (128, 768), (768, 3072), True)
    sgemm_case("c2_fp32_qk_16x12x128x64x128", (16, 12, 128, 64), (16, 12, 64, 128), False)
    sgemm_case("c2_fp32_pv_16x12x128x128x64", (16, 12, 128, 128), (16, 12, 128, 64), False)
    sgemm_case("c4_fp32_ffn_up_1024x768x3072_bias", (8, 128, 768), (768, 3072), True, sets=4, step_by_step=True)

    # C2, second case: a [1, 12, 64, 64] weight broadcast over the batch of a [16, 12, 128, 64] input
    def broadcast_case(name, shape_a, shape_b):
        p = pkg.matmul_plan(shape_a, shape_b)
        g = p["grid"]
        sets = sets_beyond_llc(4 * (int(np.prod(shape_a)) + int(np.prod(shape_b)) + int(np.prod(p["shape"]))))
        bufs = []
        for _ in range(sets):
            a = torch.randn(shape_a, device=dev, dtype=torch.float32)
            b = torch.randn(shape_b, device=dev, dtype=torch.float32)
            c = torch.empty(p["shape"], device=dev, dtype=torch.float32)
            d = pkg.SgemmDesc()
            d.a, d.b, d.c = a.data_ptr(), b.data_ptr(), c.data_ptr()
            d.m, d.n, d.k, d.lda, d.ldb, d.ldc = p["m"], p["n"], p["k"], p["k"], p["n"], p["n"]
            d.batch_outer, d.batch_inner = g["outer"], g["inner"]
            d.stride_a, d.stride_b, d.stride_c = g["strides"]
            d.inner_stride_a, d.inner_stride_b, d.inner_stride_c = g["inner_strides"]
            bufs.append((d, (a, b, c)))
        idx = [0]

        def step():
            d = bufs[idx[0] % sets][0]
            idx[0] += 1
            st = lib.tfcc_rocm_sgemm_general(stream, C.byref(d))
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, steps, warmup, pkg, stream)
        flop = 2.0 * p["m"] * p["n"] * p["k"] * p["batch"]
        nbytes = 4.0 * (int(np.prod(shape_a)) + int(np.prod(shape_b)) + int(np.prod(p["shape"])))
        out[name] = {"ms": round(ms, 5), "tflops": round(flop / ms / 1e9, 3),
                     "frac_fp32_mfma": round(flop / ms / 1e9 / PEAK_FP32_TFLOPS, 4), "gbs": round(nbytes / ms / 1e6, 1),
                     "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}

    broadcast_case("c2_fp32_broadcast_16x12x128x64_by_1x12x64x64", (16, 12, 128, 64), (1, 12, 64, 64))

    # C2, first product with K used as stored: scores = Q K^T from K [16, 12, 128, 64] (B given transposed)
    def qkt_case(name, B, H, S, D):
        sets = sets_beyond_llc(4 * (2 * B * H * S * D + B * H * S * S))
        bufs = []
        for _ in range(sets):
            q = torch.randn((B, H, S, D), device=dev, dtype=torch.float32)
            k = torch.randn((B, H, S, D), device=dev, dtype=torch.float32)
            c = torch.empty((B, H, S, S), device=dev, dtype=torch.float32)
            d = pkg.SgemmDesc()
            d.a, d.b, d.c = q.data_ptr(), k.data_ptr(), c.data_ptr()
            d.m, d.n, d.k, d.lda, d.ldb, d.ldc = S, S, D, D, D, S
            d.trans_b = 1
            d.batch_outer, d.batch_inner = B * H, 1
            d.stride_a, d.stride_b, d.stride_c = S * D, S * D, S * S
            bufs.append((d, (q, k, c)))
        idx = [0]

        def step():
            d = bufs[idx[0] % sets][0]
            idx[0] += 1
            st = lib.tfcc_rocm_sgemm_general(stream, C.byref(d))
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, steps, warmup, pkg, stream)
        flop = 2.0 * B * H * S * S * D
        nbytes = 4.0 * (2 * B * H * S * D + B * H * S * S)
        out[name] = {"ms": round(ms, 5), "tflops": round(flop / ms / 1e9, 3),
                     "frac_fp32_mfma": round(flop / ms / 1e9 / PEAK_FP32_TFLOPS, 4), "gbs": round(nbytes / ms / 1e6, 1),
                     "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}

    qkt_case("c2_fp32_qkt_k_as_stored_16x12x128x64", 16, 12, 128, 64)

    # C2 as one launch: softmax(q k^T / 8) v on [batch, seq, heads, size] tensors, 16 x 12 heads of 128 x 64
    def attention_case(name, B, H, S, D):
        sets = sets_beyond_llc(4 * 4 * B * S * H * D)
        bufs = []
        for _ in range(sets):
            q, k, v = (torch.randn((B, S, H, D), device=dev, dtype=torch.float32) for _ in range(3))
            o = torch.empty((B, S, H, D), device=dev, dtype=torch.float32)
            bufs.append((pkg.attention_desc(q, k, v, o, S, S, D, (H * D,) * 4, batch_outer=B, batch_inner=H,
                                            strides=(S * H * D,) * 4, inner_strides=(D,) * 4, divisor=8.0), (q, k, v, o)))
        idx = [0]

        def step():
            desc = bufs[idx[0] % sets][0]
            idx[0] += 1
            st = lib.tfcc_rocm_attention_f32(stream, desc)
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, steps, warmup, pkg, stream)
        flop = 4.0 * B * H * S * S * D
        nbytes = 4.0 * 4 * B * S * H * D
        out[name] = {"ms": round(ms, 5), "tflops": round(flop / ms / 1e9, 3),
                     "frac_fp32_mfma": round(flop / ms / 1e9 / PEAK_FP32_TFLOPS, 4), "gbs": round(nbytes / ms / 1e6, 1),
                     "frac_hbm": round(nbytes / ms / 1e6 / PEAK_HBM_GBS, 4)}

    attention_case("c2_fp32_attention_one_launch_16x12x128x64", 16, 12, 128, 64)
    sgemm_case("fp32_4096x4096x4096", (4096, 4096), (4096, 4096), False, sets=1)
    # one LSTM time step (tfcc::rnn::lstm_forward's inner loop): state product and cell in one launch
    for batch, hidden in ((1, 512), (4, 512), (8, 1024)):
        wh = torch.randn(hidden, 4 * hidden, device=dev) * 0.05
        inter = pkg.transpose(wh.reshape(hidden, 4, hidden), (0, 2, 1)).reshape(hidden, 4 * hidden)
        xw, bias_l = torch.randn(batch, 4 * hidden, device=dev), torch.randn(4 * hidden, device=dev)
        h0, c0 = torch.zeros(batch, hidden, device=dev), torch.zeros(batch, hidden, device=dev)
        h1 = torch.empty_like(h0)

        def step():
            st = lib.tfcc_rocm_lstm_step_f32(stream, batch, hidden, h0.data_ptr(), inter.data_ptr(), xw.data_ptr(),
                                             bias_l.data_ptr(), 0.0, c0.data_ptr(), h1.data_ptr(), c0.data_ptr())
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, max(steps, 50), warmup, pkg, stream)
        out["lstm_step_one_launch_batch%d_hidden%d" % (batch, hidden)] = {
            "ms": round(ms, 5), "gbs": round(16.0 * hidden * hidden / ms / 1e6, 1)}
    # up to eight rows of A in fp32 (C5's shape and a square weight): one streaming pass over B
    sgemm_case("fp32_few_rows_m1_4096x11008", (1, 4096), (4096, 11008), False, sets=2)
    sgemm_case("fp32_few_rows_m8_4096x11008", (8, 4096), (4096, 11008), False, sets=2)
    sgemm_case("fp32_few_rows_m8_4096x4096", (8, 4096), (4096, 4096), False)
    # what the fp32 matrix cores sustain alone (register-resident loop of the 4096^3 instruction count)
    probe_out = torch.empty(1024 * 256, dtype=torch.int32, device=dev)
    for label, changing in (("changing", 1),):
        def step():
            probe_check(bench_lib().tfcc_bench_probe_mfma(stream, 1, changing, 1024, 2048, probe_out.data_ptr()))
        ms = time_launches(torch, step, max(10, steps // 10), max(3, warmup // 10), pkg, stream)
        out["probe_fp32_matrix_cores_alone_%s_operands" % label] = {
            "ms": round(ms, 5), "tflops": round(1024 * 4 * 4 * 2048 * 4096.0 / ms / 1e9, 2)}

    # C3 as the reference's quantization::matmul returns it (tfcc/mkl/operations/tfcc_mklquantization.cpp:71-203): the
    # int32 tensor alone (67 MB written), no requantize
    a, b, ta, tb, rs, cs, ranges, out_range = c3
    d32 = pkg.QGemmDesc()
    d32.a, d32.b, d32.rowsum_a, d32.colsum_b = ta.data_ptr(), tb.data_ptr(), rs.data_ptr(), cs.data_ptr()
    d32.m, d32.n, d32.k, d32.batch, d32.stride_c = 4096, 4096, 4096, 1, 4096 * 4096
    d32.min_a, d32.max_a, d32.min_b, d32.max_b = [r.data_ptr() for r in ranges]
    range_c = torch.empty(2, dtype=torch.float32, device=dev)
    d32.min_c, d32.max_c = range_c.data_ptr(), range_c.data_ptr() + 4
    acc32 = torch.empty((4096, 4096), dtype=torch.int32, device=dev)

    def step32():
        st = lib.tfcc_rocm_gemm_u8s8s32(stream, C.byref(d32), acc32.data_ptr())
        if st != 0:
            pkg.check(st)
    ms = time_launches(torch, step32, steps, warmup)
    tops = 2.0 * 4096 ** 3 / ms / 1e9
    out["c3_int8_4096_int32_only"] = {"ms": round(ms, 5), "tops": round(tops, 2), "frac_int8_mfma": round(tops / PEAK_INT8_TOPS, 4)}
    del acc32
    # C3 with the int32 accumulators also written (67 MB more traffic)
    step = make_c3_step(torch, pkg, ta, tb, rs, cs, ranges, out_range, want_acc=True)
    ms = time_launches(torch, step, steps, warmup)
    tops = 2.0 * 4096 ** 3 / ms / 1e9
    out["c3_int8_4096_requant_plus_int32_out"] = {"ms": round(ms, 5), "tops": round(tops, 2),
                                                  "frac_int8_mfma": round(tops / PEAK_INT8_TOPS, 4)}
    # C3 with the caller's promise that colsum_b holds the true column sums of B (it does: reduce_sum made it),
    # as a weight matrix prepared once declares: the kernel then does not accumulate them itself
    step = make_c3_step(torch, pkg, ta, tb, rs, cs, ranges, out_range, want_acc=False, colsum_exact=True)
    ms = time_launches(torch, step, steps, warmup)
    tops = 2.0 * 4096 ** 3 / ms / 1e9
    out["c3_int8_4096_requant_colsum_declared_exact"] = {"ms": round(ms, 5), "tops": round(tops, 2),
                                                        "frac_int8_mfma": round(tops / PEAK_INT8_TOPS, 4)}

    # C3 the way the reference's callers run it (tfcc/test/quantization.cpp:112-118): row sums of A and column
    # sums of B are recomputed for every product, then the product itself (here with the fused requantize)
    gemm_step = make_c3_step(torch, pkg, ta, tb, rs, cs, ranges, out_range, want_acc=False)

    def call_sequence():
        for st in (lib.tfcc_rocm_reduce_sum_rows(stream, ta.data_ptr(), pkg.U8, 1, 4096, 4096, rs.data_ptr()),
                   lib.tfcc_rocm_reduce_sum_cols(stream, tb.data_ptr(), pkg.S8, 1, 4096, 4096, cs.data_ptr())):
            if st != 0:
                pkg.check(st)
        gemm_step()
    ms = time_launches(torch, call_sequence, steps, warmup)
    tops = 2.0 * 4096 ** 3 / ms / 1e9
    out["c3_int8_4096_with_row_and_column_sums_per_call"] = {"ms": round(ms, 5), "tops": round(tops, 2),
                                                            "frac_int8_mfma": round(tops / PEAK_INT8_TOPS, 4)}

    # C5: skinny decode shapes, B streamed once; rotate B buffers larger than the last-level cache
    n, k = 11008, 4096
    sets = 8
    bs = [t(rng.integers(-127, 128, (k, n), dtype=np.int8)) for _ in range(sets)]
    css = [pkg.reduce_sum(x, False) for x in bs]
    scale_b = t(rng.uniform(0.001, 0.01, n).astype(np.float32))
    # (flags 1: the caller's promise that colsum_b holds the true column sums of b - reduce_sum made them here -, as a
    # weight matrix prepared once declares; the kernel then forms no column sums of its own)
    for m, flags in ((1, 0), (4, 0), (8, 0), (1, 1), (4, 1), (8, 1)):
        am = t(rng.integers(0, 256, (m, k), dtype=np.uint8))
        rsm = pkg.reduce_sum(am, True)
        acc = torch.empty((m, n), dtype=torch.int32, device=dev)
        f32 = torch.empty((m, n), dtype=torch.float32, device=dev)
        idx = [0]

        def step():
            i = idx[0] % sets
            idx[0] += 1
            st = lib.tfcc_rocm_gemv_u8s8s32_flags(stream, am.data_ptr(), bs[i].data_ptr(), rsm.data_ptr(), css[i].data_ptr(),
                                                  -128, 0, m, n, k, acc.data_ptr(), 0.02, scale_b.data_ptr(), f32.data_ptr(),
                                                  flags)
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, max(steps, 50), warmup, pkg, stream)
        nbytes = k * n + m * k + 4 * n + 4 * m * n  # B + A + scales + fp32 out (algorithmic)
        gbs = nbytes / ms / 1e6
        name = "c5_int8_gemv_m%d_4096x11008" % m + ("_colsum_declared_exact" if flags else "")
        out[name] = {"ms": round(ms, 5), "gbs": round(gbs, 1), "frac_hbm": round(gbs / PEAK_HBM_GBS, 4),
                     "gops": round(2.0 * m * n * k / ms / 1e6, 1)}
    # what bounds those launches on this part: a launch that only reads the same 45 MB (same rotation of
    # buffers), and a launch of workgroups that do nothing
    probe_word = torch.zeros(16, dtype=torch.int32, device=dev)
    for blocks in (512, 1024, 2048):
        idx = [0]

        def step():
            i = idx[0] % sets
            idx[0] += 1
            probe_check(bench_lib().tfcc_bench_probe_read(stream, bs[i].data_ptr(), k * n, blocks, probe_word.data_ptr()))
        ms = time_launches(torch, step, max(steps, 50), warmup, pkg, stream)
        out["probe_read_only_45mb_%d_workgroups" % blocks] = {"ms": round(ms, 5), "gbs": round(k * n / ms / 1e6, 1),
                                                               "frac_hbm": round(k * n / ms / 1e6 / PEAK_HBM_GBS, 4)}

    def step():
        probe_check(bench_lib().tfcc_bench_probe_launch(stream, probe_word.data_ptr()))
    out["probe_empty_launch"] = {"ms": round(time_launches(torch, step, max(steps, 50), warmup, pkg, stream), 5)}

    # the same decode shapes on weights packed once (column slabs in matrix-core operand order)
    packs = [pkg.gemv_pack(x) for x in bs]
    for m in (1, 4, 8):
        am = t(rng.integers(0, 256, (m, k), dtype=np.uint8))
        rsm = pkg.reduce_sum(am, True)
        acc = torch.empty((m, n), dtype=torch.int32, device=dev)
        f32 = torch.empty((m, n), dtype=torch.float32, device=dev)
        idx = [0]

        def step():
            i = idx[0] % sets
            idx[0] += 1
            st = lib.tfcc_rocm_gemv_u8s8s32_packed(stream, am.data_ptr(), packs[i].data_ptr(), rsm.data_ptr(),
                                                   css[i].data_ptr(), -128, 0, m, n, k, acc.data_ptr(), 0.02,
                                                   scale_b.data_ptr(), f32.data_ptr())
            if st != 0:
                pkg.check(st)
        ms = time_launches(torch, step, max(steps, 50), warmup, pkg, stream)
        nbytes = k * n + m * k + 4 * n + 4 * m * n
        gbs = nbytes / ms / 1e6
        out["c5_int8_gemv_packed_m%d_4096x11008" % m] = {"ms": round(ms, 5), "gbs": round(gbs, 1),
                                                          "frac_hbm": round(gbs / PEAK_HBM_GBS, 4)}
    del packs

    # C4: one BERT-base encoder layer through the model runtime (fp32, batch 8, seq 128); the entrance
    # graph alone is timed with events on the runtime's stream, tensors resident in HBM
    import importlib
    mf = importlib.import_module("wechat_tfcc_amd.modelfile")
    rt = importlib.import_module("wechat_tfcc_amd.runtime_api")
    hidden, heads, ffn = 768, 12, 3072
    w = mf.bert_layer_weights(rng, hidden, ffn)
    # batch 8 x 128 positions (BASELINE configs[3]), and one sequence of 384 positions: the length of the
    # question-answering model the reference documents (samples/ConvertONNXModel.md:16), whose attention walks the
    # keys in three blocks of 128
    for name, batch, seq in (("c4_bert_base_layer_b8_s128_runtime", 8, 128), ("bert_base_layer_b1_s384_runtime", 1, 384)):
        graph = mf.bert_encoder_layer(w, batch, seq, heads)
        model = rt.Model(mf.write_model([graph], graph.name))
        x = {"hidden_states": rng.normal(size=(batch, seq, hidden)).astype(np.float32)}
        rows = batch * seq
        gemm_flop = 2.0 * rows * hidden * (4 * hidden + 2 * ffn) + 2 * 2.0 * batch * heads * seq * seq * (hidden // heads)
        entry = {"gemm_flop": gemm_flop, "nodes": len(graph.nodes)}
        for label, replay in (("step_by_step", False), ("graph_replay", True)):
            model.set_replay(replay)
            us = model.time(x, warmup=warmup, iters=steps)
            entry[label + "_us"] = round(us, 2)
            entry[label + "_tflops"] = round(gemm_flop / us / 1e6, 2)
            entry[label + "_frac_fp32_mfma"] = round(gemm_flop / us / 1e6 / PEAK_FP32_TFLOPS, 4)
        model.set_replay(False)
        model.close()
        out[name] = entry
    return out


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=2000,
                    help="timed launches; the default is long enough (about 0.15 s) for the clocks to settle")
    ap.add_argument("--warmup", type=int, default=500)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--no-other", action="store_true", help="skip the secondary configs")
    ap.add_argument("--short-legs", action="store_true",
                    help="secondary configs with the --steps / --warmup given instead of at least 500 / 300 launches, the "
                         "headline's settled and matrix-core legs cut to 40 launches, no operand-statistics legs "
                         "(for counter collection; the figures then include the clock ramp)")
    ap.add_argument("--headline-only", action="store_true",
                    help="only the timed launches of the headline kernel (for counter runs): no probes, no settled / "
                         "burst repeats, no secondary configs, no CPU leg")
    ap.add_argument("--no-sampler", action="store_true",
                    help="do not start the child process that samples clock and power (for runs under a profiler, whose "
                         "preloaded library has initialised the GPU before this program starts: nothing may be spawned then)")
    ap.add_argument("--copy-calibration", action="store_true",
                    help="instead of the benchmark, run a plain streaming kernel of known size (reads and writes "
                         "256 MiB each per launch) to calibrate the FETCH_SIZE / WRITE_SIZE counters against")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU: the matmul path has no multi-GPU part (run with --gpus 1)")

    # the clock / power sampler is a child process and starts before this process makes its first GPU call
    sampler = None if (args.headline_only or args.copy_calibration or args.no_sampler) else GpuSampler()
    import torch
    from __graft_entry__ import load_package
    pkg = load_package()
    pkg.lib()
    if not torch.cuda.is_available():
        sys.exit("bench.py needs a GPU")
    dev = torch.device("cuda:0")
    torch.cuda.set_device(dev)

    if args.copy_calibration:
        n = 64 * 1024 * 1024  # floats: 256 MiB in, 256 MiB out
        src = torch.ones(n, dtype=torch.float32, device=dev)
        dst = torch.empty_like(src)
        stream = torch.cuda.current_stream().cuda_stream
        for _ in range(args.warmup + args.steps):
            pkg.check(pkg.lib().tfcc_rocm_transform_f32(stream, src.data_ptr(), n, 1.0, 0.0, dst.data_ptr()))
        torch.cuda.synchronize()
        print(json.dumps({"calibration_kernel": "transform_kernel", "read_bytes_per_launch": 4 * n,
                          "write_bytes_per_launch": 4 * n, "launches": args.warmup + args.steps}))
        return

    size = 4096
    c3 = c3_setup(torch, pkg, dev, seed=0, size=size)
    a, b, ta, tb, rs, cs, ranges, out_range = c3
    step = make_c3_step(torch, pkg, ta, tb, rs, cs, ranges, out_range, want_acc=False)

    # warmup, then exactly K timed steps between synchronisation points
    for _ in range(args.warmup):
        step()
    torch.cuda.synchronize()
    start, stop = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    t0 = time.perf_counter()
    start.record()
    for _ in range(args.steps):
        step()
    stop.record()
    torch.cuda.synchronize()
    wall_ms = (time.perf_counter() - t0) * 1e3 / args.steps
    kernel_ms = start.elapsed_time(stop) / args.steps  # HIP events on the launch stream
    ops = 2.0 * size ** 3
    tops = ops / wall_ms / 1e9
    kernel_tops = ops / kernel_ms / 1e9

    result = {
        "metric": "int8 matmul TOPS (u8 x s8 -> s32 -> requantized u8, M=N=K=4096)",
        "value": round(tops, 2),
        "unit": "TOP/s",
        "n_gpus": 1,
        "steps": args.steps,
        "warmup": args.warmup,
        "ms_per_step": round(wall_ms, 5),
        "higher_is_better": True,
        "scaling": "weak",
        "vs_baseline": None,
        "dtype": "int8 (int32 accumulate, fp64 requantize)",
        "data": "synthetic (seeded uniform uint8 / int8, resident in HBM)",
        "config": {"workload": "BASELINE configs[2]: A u8[4096,4096] zp 128 x B s8[4096,4096] symmetric -> "
                               "int32 -> requantize u8, scale 1/(K*64), zp 128; fused kernel, uint8 output only",
                   "m": size, "n": size, "k": size},
        "roofline": {"bound": "mfma", "achieved": round(kernel_tops, 2), "peak": PEAK_INT8_TOPS, "unit": "TOP/s",
                     "frac": round(kernel_tops / PEAK_INT8_TOPS, 4), "traffic": None,
                     "kernel": "qgemm_w4_kernel<64,4,true,false,true>", "kernel_ms": round(kernel_ms, 5),
                     "algorithmic_ops_per_launch": ops,
                     "kernel_ms_is": "HIP events around the K timed launches / K: launch to launch, i.e. the kernel's own "
                                     "duration (what a kernel trace reports) plus the gap between dependent launches"},
    }
    traffic_file = os.path.join(ROOT, "profiles", "traffic.json")
    if os.path.exists(traffic_file):
        result["roofline"]["traffic"] = json.load(open(traffic_file)).get("qgemm_c3_bytes_per_launch")
        result["roofline"]["traffic_is"] = ("from profiles/traffic.json (FETCH_SIZE + WRITE_SIZE counter runs of this "
                                            "command with --headline-only, scaled by a copy kernel of known size), "
                                            "not measured in this run")
    if args.headline_only:
        print(json.dumps(result), flush=True)
        return

    def timed_with_power(fn, launches, warm):
        """ms per launch (HIP events) and the sampler's clock / power over the timed launches (first 30 ms left out)."""
        for _ in range(warm):
            fn()
        torch.cuda.synchronize()
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        m0 = time.monotonic()
        e0.record()
        for _ in range(launches):
            fn()
        e1.record()
        torch.cuda.synchronize()
        m1 = time.monotonic()
        w = sampler.window(m0 + 0.03, m1) if sampler is not None else {"available": False, "why": "--no-sampler"}
        keep = {k: w[k] for k in ("sclk_mhz", "power_w", "power_w_max", "samples") if k in w} if w.get("available") else w
        return e0.elapsed_time(e1) / launches, keep

    # The two regimes of the same launch: after a long warm-up, when the clocks have settled under the power limit
    # (with the shader clock and the socket power the driver reports meanwhile), and as a burst of a few launches
    # right after the GPU sat idle (the first launches run at the idle clocks).
    # (--short-legs: counter collection, where every launch is slow and only the dispatches' counters matter)
    long_n, long_w = (4000, 500) if not args.short_legs else (40, 10)
    ms, watt = timed_with_power(step, long_n, long_w)
    result["roofline"]["settled"] = {"steps": long_n, "warmup": long_w, "idle_before_s": 0.0, "kernel_ms": round(ms, 5),
                                     "achieved": round(ops / ms / 1e9, 2), "frac": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4)}
    settled_tops = ops / ms / 1e9
    if watt.get("available") is False:
        result["roofline"]["sclk_mhz"] = result["roofline"]["power_w"] = None
        result["roofline"]["clock_power_unavailable"] = watt.get("why")
    else:
        result["roofline"]["sclk_mhz"], result["roofline"]["power_w"] = watt.get("sclk_mhz"), watt.get("power_w")
        result["roofline"]["clock_power_is"] = (
            "median over the settled leg of the shader clock (pp_dpm_sclk, what rocm-smi --showclocks prints) and the "
            "socket power (hwmon power1_input), sampled every 2 ms by a child process; nominal peak is quoted at 2400 MHz")
        result["roofline"]["clock_power_detail"] = watt
        full = sampler.window(0, time.monotonic()) if sampler is not None else {}
        if "power_cap_w" in full:
            result["roofline"]["power_cap_w"] = full["power_cap_w"]
    torch.cuda.synchronize()
    time.sleep(0.5)
    ms = time_launches(torch, step, 20, 5)
    result["roofline"]["burst"] = {"steps": 20, "warmup": 5, "idle_before_s": 0.5, "kernel_ms": round(ms, 5),
                                   "achieved": round(ops / ms / 1e9, 2), "frac": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4)}

    # The same kernel, the same launch and the same instruction stream on operands of other statistics: what it does
    # per second depends on how many operand bits change from one matrix op to the next, i.e. on power.  The
    # headline keeps the uniform operands its configuration prescribes; these legs are evidence, not results.
    rng_alt = np.random.default_rng(7)
    # (Left out with --short-legs and with --no-sampler: without clock and power they say little, and a kernel trace of
    # the run then averages the headline kernel over its prescribed operands only.)
    alt_sets = {} if (args.short_legs or sampler is None) else {
        # a quantized bell curve: activations around the zero point 128, weights around 0 (sigma 12 codes each)
        "quantized_normal_sigma12": (np.clip(np.rint(rng_alt.normal(128.0, 12.0, (size, size))), 0, 255).astype(np.uint8),
                                     np.clip(np.rint(rng_alt.normal(0.0, 12.0, (size, size))), -127, 127).astype(np.int8)),
        # every element the same: no operand bit ever changes
        "constant": (np.full((size, size), 131, dtype=np.uint8), np.full((size, size), 3, dtype=np.int8)),
    }
    alt_out = {}
    for label, (a_alt, b_alt) in alt_sets.items():
        ta_alt, tb_alt = torch.from_numpy(a_alt).to(dev), torch.from_numpy(b_alt).to(dev)
        rs_alt, cs_alt = pkg.reduce_sum(ta_alt, True), pkg.reduce_sum(tb_alt, False)
        step_alt = make_c3_step(torch, pkg, ta_alt, tb_alt, rs_alt, cs_alt, ranges, out_range, want_acc=False)
        ms, watt = timed_with_power(step_alt, 3000, 500)
        alt_out[label] = {"kernel_ms": round(ms, 5), "tops": round(ops / ms / 1e9, 2),
                          "frac_of_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4), **watt}
        del step_alt, ta_alt, tb_alt
    result["roofline"]["same_kernel_other_operands"] = alt_out

    # What the matrix cores sustain with nothing else in the way: register-resident instruction loops of the
    # headline's op count, each with the clock and power read while it runs.
    #   constant / changing operands   four accumulators per wavefront, 2 x 4 wavefronts per CU
    #   gemm_order                     the product kernel's issue order (a wavefront owns 128 x 128 outputs in all 256
    #                                  accumulation registers, one operand stays for a row of blocks, half of every
    #                                  operand's bits flip per k step), with 32x32x32 and with 16x16x64 instructions
    #   busy_share                     the same with the wavefronts asleep part of the time: what a kernel whose
    #                                  matrix cores are busy that share of its cycles could reach under the power limit
    probe_out = torch.empty(512 * 256, dtype=torch.int32, device=dev)
    stream0 = torch.cuda.current_stream().cuda_stream
    probes = {}
    for label, kind, pattern, blocks, iters in (
            ("int8_32x32x32_constant_operands", 0, 0, 512, 256), ("int8_32x32x32_changing_operands", 0, 1, 512, 256),
            ("int8_32x32x32_gemm_order", 0, 2, 256, 128), ("int8_16x16x64_changing_operands", 2, 1, 512, 512),
            ("int8_16x16x64_gemm_order", 2, 2, 256, 64)):
        def probe():
            probe_check(bench_lib().tfcc_bench_probe_mfma(stream0, kind, pattern, blocks, iters, probe_out.data_ptr()))
        ms, watt = timed_with_power(probe, long_n, 300 if not args.short_legs else 10)
        probes[label] = {"tops": round(ops / ms / 1e9, 2), "frac_of_peak": round(ops / ms / 1e9 / PEAK_INT8_TOPS, 4), **watt}
    for sleep, share in ((1, 0.89), (2, 0.80), (4, 0.67), (8, 0.50)):
        def probe():
            probe_check(bench_lib().tfcc_bench_probe_mfma_duty(stream0, sleep, 256, 128, probe_out.data_ptr()))
        ms, watt = timed_with_power(probe, 3000 if not args.short_legs else 40, 300 if not args.short_legs else 10)
        probes["int8_32x32x32_gemm_order_busy_share_%.2f" % share] = {"tops": round(ops / ms / 1e9, 2), **watt}
    result["roofline"]["matrix_cores_alone"] = probes
    result["roofline"]["matrix_cores_alone_constant_operands"] = probes["int8_32x32x32_constant_operands"]["tops"]
    result["roofline"]["matrix_cores_alone_changing_operands"] = probes["int8_32x32x32_changing_operands"]["tops"]
    result["roofline"]["frac_of_matrix_cores_alone_changing_operands"] = round(
        settled_tops / probes["int8_32x32x32_changing_operands"]["tops"], 4)
    result["roofline"]["frac_of_matrix_cores_alone_gemm_order"] = round(settled_tops / probes["int8_32x32x32_gemm_order"]["tops"], 4)
    if not args.no_other:
        # on a stream of its own (not the default stream) so that short kernels can be timed as graph replays
        side = torch.cuda.Stream()
        torch.cuda.synchronize()
        with torch.cuda.stream(side):
            result["other"] = bench_other(torch, pkg, dev, max(10, args.steps // 2), args.warmup, c3, args.short_legs)
        torch.cuda.synchronize()
    if sampler is not None:
        sampler.close()
    if not args.no_cpu:
        result["cpu_baseline"] = cpu_baseline(a, b, size)
    print(json.dumps(result), flush=True)


if __name__ == "__main__":
    main()
