#!/usr/bin/env python3
"""Benchmark of the int8 affine path (Marian intgemm8 semantics) on one MI355X.

    python bench.py [--gpus 1] [--steps K] [--warmup W]

Prints ONE JSON line.  The headline workload is the transformer-base decode GEMM sweep: one
"step" is one pass over its 20 affine calls (abs-max quantize of the fp32 activations + int8 GEMM
with fused dequantize and bias), inputs and int8 weights resident in HBM.  The K steps are timed
three ways - launched eagerly from this process (the twenty C-ABI calls of a pass issued back to
back, the way Marian's forward tape launches), eagerly from a C++ host thread through the C++
wrappers (a child process), and replayed as HIP graphs - and the headline is the fastest of the
three (config.launch says which; all three are in the line).
Every step uses a different copy of the weights, rotating over more than 512 MB, so weights come
from HBM and not from the 256 MB Infinity Cache.

Also in the line: the roofline of the dominant kernel (per-launch duration from HIP events), the
CPU restatement of the reference path timed on this host, and the other workloads (encoder-size
GEMMs with their MFMA fraction, the shortlisted output layer, transformer-big decode tokens/s).
"""
import argparse
import importlib
import json
import os
import sys
import time

import numpy as np

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
    sys.path.insert(0, ROOT)
PKG = "marian-dev_amd"

HBM_PEAK_GBS = 8000.0        # MI355X HBM3E, published
INT8_PEAK_TOPS = 5000.0      # MI355X dense int8 MFMA, published (5.0 POP/s)

TRAFFIC_FILE = os.path.join(ROOT, "profiles", "hbm_traffic_pmc.txt")


def measured_traffic():
    """HBM bytes per launch of the kernels named in profiles/hbm_traffic_pmc.txt: the summary of two
    rocprofv3 --pmc runs (FETCH_SIZE, WRITE_SIZE) of `bench.py --pmc-probe`, written by
    `bench.py --pmc-summary`.  Lines `traffic_bytes_per_launch <key> = <bytes>`; `build_commit =`
    names the commit of the sources the counters were taken from.  ({} when the file is absent.)"""
    out = {"_commit": None}
    if not os.path.exists(TRAFFIC_FILE):
        return out
    for line in open(TRAFFIC_FILE):
        parts = line.split()
        if len(parts) >= 4 and parts[0] == "traffic_bytes_per_launch" and parts[2] == "=":
            out[parts[1]] = int(parts[3])
        if len(parts) >= 3 and parts[0] == "build_commit" and parts[1] == "=":
            out["_commit"] = parts[2]
    return out


DECODE_SHAPES = [(512, 1536), (512, 512), (512, 2048), (2048, 512), (512, 32000)]
DECODE_M = [1, 4, 16, 64]


def algorithmic_bytes(M, K, n_out, with_idx=False):
    """fp32 A read once + int8 W + fp32 bias + fp32 out (+ shortlist ids)."""
    return 4 * M * K + K * n_out + 4 * n_out + 4 * M * n_out + (4 * n_out if with_idx else 0)


def gemm_kernel_bytes(M, K, n_out, with_idx=False):
    """What the GEMM kernel itself has to move: int8 A, int8 W, bias, fp32 out."""
    return M * K + K * n_out + 4 * n_out + 4 * M * n_out + (4 * n_out if with_idx else 0)


class Op:
    """One affine call with all buffers preallocated; `copies` distinct weight copies."""

    def __init__(self, torch, integer, M, K, N, relu=False, copies=1, idx=None, seed=0):
        g = torch.Generator(device="cuda")
        g.manual_seed(1000 + seed)
        self.M, self.K, self.N, self.relu = M, K, N, int(relu)
        self.A = torch.randn(M, K, device="cuda", generator=g)
        self.bias = torch.randn(N, device="cuda", generator=g) * 0.01
        self.Aq = integer.QTensor.empty((M, K), integer.Type.intgemm8, "cuda")
        W = torch.randn(K, N, device="cuda", generator=g) * 0.02
        first = integer.prepareB(W)
        self.Bq = [first] + [integer.QTensor(first.data.clone(), first.shape, first.type, first.prepared)
                             for _ in range(copies - 1)]
        self.idx = idx
        self.n_out = N if idx is None else int(idx.numel())
        self.out = torch.empty(M, self.n_out, device="cuda")
        self.ops = 2 * M * K * self.n_out

    def launch_fused(self, lib, be, copy=0):
        """prepareA + affine through the single entry point (one kernel for small activations)."""
        b = self.Bq[copy % len(self.Bq)]
        r = lib.marian_hip_int8_affine_f32(
            self.A.data_ptr(), self.Aq.data_ptr(), b.data_ptr(), self.bias.data_ptr(),
            None if self.idx is None else self.idx.data_ptr(), 0 if self.idx is None else self.n_out,
            self.out.data_ptr(), self.M, self.K, self.N, 1.0, self.relu,
            be.workspace.data_ptr(), be.workspace_bytes, be.stream())
        assert r == 0, r

    def launch(self, lib, be, copy=0, prepare=True, gemm=True):
        st = be.stream()
        if prepare:
            r = lib.marian_hip_int8_prepare_a(self.A.data_ptr(), self.Aq.data_ptr(), self.M, self.K,
                                              be.workspace.data_ptr(), be.workspace_bytes, st)
            assert r == 0, r
        if gemm:
            b = self.Bq[copy % len(self.Bq)]
            if self.idx is None:
                r = lib.marian_hip_int8_affine(self.Aq.data_ptr(), b.data_ptr(), self.bias.data_ptr(),
                                               self.out.data_ptr(), self.M, self.K, self.N, 1.0,
                                               self.relu, st)
            else:
                r = lib.marian_hip_int8_affine_shortlist(self.Aq.data_ptr(), b.data_ptr(),
                                                         self.bias.data_ptr(), self.idx.data_ptr(),
                                                         self.n_out, self.out.data_ptr(), self.M,
                                                         self.K, self.N, 1.0, self.relu, st)
            assert r == 0, r


def BigDecoder(torch, integer, ops, sets):
    """Transformer-big decoder step of the benchmark (configuration 3): 6 layers, d = 1024,
    ffn = 4096, 16 heads, tied 32000-word output layer, beam 4 x batch 32, 20 cached target positions,
    source lengths uniform 20..60."""
    step_mod = importlib.import_module(PKG + ".decoder_step")
    return step_mod.DecoderStep(sets=sets)


def capture(torch, fn):
    """Record fn's launches into a HIP graph (no memset nodes: the path has none)."""
    s = torch.cuda.Stream()
    s.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(s):
        fn()  # warm every kernel (module load, LDS attribute) before capture
    torch.cuda.current_stream().wait_stream(s)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        fn()
    return g


def time_graphs(torch, graphs, steps, warmup):
    """Replays graphs round-robin; returns seconds for exactly `steps` replays."""
    for i in range(warmup):
        graphs[i % len(graphs)].replay()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(steps):
        graphs[i % len(graphs)].replay()
    torch.cuda.synchronize()
    return time.perf_counter() - t0


def per_launch_ms(torch, launches, repeat):
    """Average duration of one launch from HIP events recorded on the launch stream: each event
    pair brackets one pass over `launches` (distinct weight copies) issued back to back, and the
    passes are queued behind a spinning kernel so the host never starves the stream.  Returns
    (mean, median) over the passes, per launch, in ms."""
    stream = torch.cuda.current_stream()
    n = len(launches)
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(repeat)]
    for f in launches:
        f()
    torch.cuda.synchronize()
    torch.cuda._sleep(int(2.0e9 * 0.02 * max(1, n * repeat // 100)))  # ~20 ms per 100 launches
    for r in range(repeat):
        starts[r].record(stream)
        for f in launches:
            f()
        ends[r].record(stream)
    torch.cuda.synchronize()
    d = np.array([starts[r].elapsed_time(ends[r]) / n for r in range(repeat)])
    return float(d.mean()), float(np.median(d))


def cpu_model():
    try:
        for line in open("/proc/cpuinfo"):
            if line.startswith("model name"):
                return line.split(":", 1)[1].strip()
    except OSError:
        pass
    return "unknown"


def cpu_sweep_work():
    from oracle import oracle as orc
    synth = importlib.import_module(PKG + ".synth")
    work = []
    for (K, N) in DECODE_SHAPES:
        W = synth.normal(1002, synth.STREAM_W, (K, N), 0.02)
        Bq = orc.prepare_b(W)
        bias = synth.normal(1002, synth.STREAM_BIAS, (N,), 0.01)
        for M in DECODE_M:
            A = synth.normal(1002, synth.STREAM_A, (M, K), 1.0)
            work.append((orc.AffineF32(M, K, N), A, Bq, bias, 2 * M * K * N))
    for f, A, Bq, bias, _ in work:
        f(A, Bq, bias)
    return work


def cpu_sweep_passes(work, seconds):
    passes = 0
    t0 = time.perf_counter()
    while True:
        for f, A, Bq, bias, _ in work:
            f(A, Bq, bias)
        passes += 1
        dt = time.perf_counter() - t0
        if dt > seconds:
            return passes, dt


def cpu_worker(seconds):
    """One of the independent instances of the aggregate CPU figure (no GPU, no torch)."""
    work = cpu_sweep_work()
    passes, dt = cpu_sweep_passes(work, seconds)
    print(json.dumps({"passes": passes, "seconds": dt, "ops_per_pass": sum(w[4] for w in work)}))


def cpp_host_figure(program, key, args=("300", "30")):
    """A figure measured by one of the C++ host programs of marian-dev_amd/host (built by build()),
    which launch call after call from a C++ thread through the C++ wrappers, no recorded graph: the
    value of `key` in the line of JSON the program prints, or None when the program is not there.
    It runs as a child process while this one is idle."""
    import subprocess
    exe = os.path.join(ROOT, PKG, "host", program)
    if not os.path.exists(exe):
        return None
    try:
        out = subprocess.run([exe] + list(args), capture_output=True, text=True, timeout=180)
        return round(json.loads(out.stdout.strip().splitlines()[-1])[key], 4)
    except Exception as e:   # noqa: BLE001 - a measurement that is reported as absent, not a failure of the run
        print("%s failed: %r" % (program, e), file=sys.stderr)
        return None


def eager_sweep_cpp_host(steps=300, warmup=30):
    """The twenty calls of the decode sweep, ms per pass over `steps` passes (host/eager_sweep.cpp)."""
    return cpp_host_figure("eager_sweep", "eager_ms_per_pass_cpp_host", (str(int(steps)), str(int(warmup))))


def cpu_baseline(seconds=10.0, aggregate_seconds=6.0, big_seconds=6.0):
    """The CPU restatement of the reference path (prepareA + VNNI multiply + unquantize/bias, one
    thread per GEMM like one Marian CPU worker, reference src/common/config.cpp:245-247) timed on
    this host, bounded in time: the decode sweep on one core (whole and per shape), the same sweep
    in one independent process per core of this job's share, and the 49 GEMMs of the
    transformer-big decoding step at M = 128 on one core."""
    import subprocess
    from oracle import oracle as orc
    work = cpu_sweep_work()
    ops_per_pass = sum(w[4] for w in work)
    passes, dt = cpu_sweep_passes(work, seconds)
    per_shape = {}
    for f, A, Bq, bias, ops in work:
        n, t0 = 0, time.perf_counter()
        while n < 3 or time.perf_counter() - t0 < 0.05:
            f(A, Bq, bias)
            n += 1
        per_shape["M%d_%dx%d" % (f.M, f.K, f.N)] = round((time.perf_counter() - t0) / n * 1e6, 1)
    # one instance per core of this job's share (at most 16: what a one-GPU job is given)
    try:
        share = len(os.sched_getaffinity(0))
    except AttributeError:
        share = os.cpu_count() or 1
    instances = max(1, min(share, 16))
    procs = []
    agg_ops_per_s = 0.0
    try:
        for _ in range(instances):
            procs.append(subprocess.Popen([sys.executable, os.path.abspath(__file__), "--cpu-worker", str(aggregate_seconds)],
                                          stdout=subprocess.PIPE, stdin=subprocess.DEVNULL, text=True))
        for pr in procs:
            out, _ = pr.communicate(timeout=aggregate_seconds * 10 + 120)
            r = json.loads(out.strip().splitlines()[-1])
            agg_ops_per_s += r["passes"] * r["ops_per_pass"] / r["seconds"]
    finally:
        # every child is reaped on every path (an exception above, a worker that hangs)
        for pr in procs:
            if pr.poll() is None:
                pr.kill()
            try:
                pr.wait(timeout=10)
            except subprocess.TimeoutExpired:
                pass
            if pr.stdout:
                pr.stdout.close()
    # transformer-big decoding step: 48 layer GEMMs + the vocabulary GEMM at M = 128, random int8
    # weights (121 MB, every matrix its own memory), fp32 activations quantized per call
    rng = np.random.default_rng(77)
    d, ffn, V, M = 1024, 4096, 32000, 128
    layer = [(d, d)] * 6 + [(d, ffn), (ffn, d)]
    big = []
    for (K, N) in layer * 6 + [(d, V)]:
        Bq = rng.integers(-127, 128, size=K * N + 4, dtype=np.int8)
        Bq[-4:] = np.frombuffer(np.float32(6000.0).tobytes(), np.int8)
        big.append((orc.AffineF32(M, K, N), rng.standard_normal((M, K)).astype(np.float32), Bq,
                    np.zeros(N, np.float32)))
    for f, A, Bq, bias in big[:2]:
        f(A, Bq, bias)
    steps, t0 = 0, time.perf_counter()
    while steps < 1 or time.perf_counter() - t0 < big_seconds:
        for f, A, Bq, bias in big:
            f(A, Bq, bias)
        steps += 1
    big_dt = (time.perf_counter() - t0) / steps
    return {"value": round(ops_per_pass * passes / dt / 1e12, 5), "unit": "TOPS", "cores": 1,
            "kind": "port",
            "isa": "avx512-vnni" if orc.has_vnni() else "scalar",
            "cpu_model": cpu_model(), "host_cpus": os.cpu_count(), "cpus_in_share": share,
            "sample": "%d passes of the same 20-shape decode sweep in %.1f s on one core" % (passes, dt),
            "per_shape_single_core_us": per_shape,
            "aggregate": {"value": round(agg_ops_per_s / 1e12, 4), "unit": "TOPS", "cores": instances,
                          "sample": "%d independent single-threaded processes, %.0f s of the same sweep each"
                                    % (instances, aggregate_seconds)},
            "transformer_big_decode": {
                "what": "GEMM-only decode step at M=128 (48 layer GEMMs + 32000-vocab GEMM, each with its "
                        "prepareA) on one core",
                "ms_per_step": round(big_dt * 1e3, 2), "hyp_tokens_per_s": round(M / big_dt, 1),
                "output_tokens_per_s": round(32 / big_dt, 1), "cores": 1,
                "sample": "%d steps in %.1f s" % (steps, big_dt * steps)}}


def pmc_probe(torch, integer, lib, be):
    """A few launches each of: a plain elementwise copy of 64 MiB (reads 64 MiB, writes 64 MiB:
    the yardstick the counters are scaled by), the fused decode kernel on the vocabulary
    projection at M = 64, and the two encoder-size GEMMs.  Each launch uses a fresh weight copy."""
    src = torch.randn(16 * 1024 * 1024, device="cuda")
    dst = torch.empty_like(src)
    for _ in range(3):
        torch.add(src, 1.0, out=dst)
    torch.cuda.synchronize()
    o = Op(torch, integer, 64, 512, 32000, copies=6, seed=43)
    for c in range(6):
        o.launch_fused(lib, be, c)
    torch.cuda.synchronize()
    for (M, K, N) in [(4096, 1024, 4096), (4096, 4096, 1024)]:
        e = Op(torch, integer, M, K, N, relu=True, copies=4, seed=77)
        e.launch(lib, be, 0, prepare=True, gemm=False)
        for c in range(4):
            e.launch(lib, be, c, prepare=False)
        torch.cuda.synchronize()
        del e


def probe_ceilings(torch):
    """Machine ceilings behind the roofline discussion, measured with the probe kernels of the tuning
    build (include/marian_hip_int8_tuning.h) and HIP events; prints a text table.  Nothing here
    touches the shipped library's kernels."""
    import ctypes
    T = importlib.import_module(PKG + "._lib").tuning_lib()
    st = torch.cuda.current_stream().cuda_stream
    pool_bytes = 1 << 30
    pool = torch.randint(-128, 128, (pool_bytes,), dtype=torch.int8, device="cuda")
    dst = torch.empty(1 << 28, dtype=torch.int8, device="cuda")
    print("machine ceilings on %s (%d compute units)" % (torch.cuda.get_device_name(0),
                                                          torch.cuda.get_device_properties(0).multi_processor_count))

    def stream(read_bytes, write_bytes, wgs, threads, u=8, nt=0, rotate=True):
        n = max(1, pool_bytes // max(read_bytes, 16)) if rotate else 1
        n = min(n, 64)
        launches = [(lambda i=i: T.marian_hip_probe_stream(pool.data_ptr() + i * read_bytes, read_bytes, dst.data_ptr(),
                                                            write_bytes, wgs, threads, u, nt, st)) for i in range(n)]
        reps = max(3, 60 // n)
        mean, med = per_launch_ms(torch, launches, reps)
        return med * 1e3   # us

    print("\n-- back-to-back launch floor (a kernel that moves 16 bytes, 100 launches per timed pass) --")
    tiny = [(lambda: T.marian_hip_probe_stream(pool.data_ptr(), 16, dst.data_ptr(), 16, 1, 64, 1, 0, st))] * 100
    print("  %.2f us per launch" % (per_launch_ms(torch, tiny, 5)[1] * 1e3))
    print("\n-- read-only pass (1024 workgroups x 256 threads, 8 loads in flight), rotating over 1 GiB --")
    for mb in (16, 32, 64, 256, 1024):
        us = stream(mb << 20, 16, 1024, 256)
        print("  %5d MiB  %8.2f us  %6.2f TB/s" % (mb, us, (mb << 20) / us / 1e6))
    print("\n-- read-only pass over the same 64 MiB every launch (Infinity-Cache resident) --")
    us = stream(64 << 20, 16, 1024, 256, rotate=False)
    print("  %5d MiB  %8.2f us  %6.2f TB/s" % (64, us, (64 << 20) / us / 1e6))
    print("\n-- write-only pass (1024 x 256), plain and non-temporal stores --")
    for mb in (16, 64, 256):
        for nt in (0, 1):
            us = stream(16, mb << 20, 1024, 256, 8, nt)
            print("  %5d MiB  %s  %8.2f us  %6.2f TB/s" % (mb, "nt   " if nt else "plain", us, (mb << 20) / us / 1e6))
    print("\n-- copy of 64 MiB (read 64 MiB, then write 64 MiB) --")
    us = stream(64 << 20, 64 << 20, 2048, 256)
    print("  %8.2f us  %6.2f TB/s (read + written bytes)" % (us, 2 * (64 << 20) / us / 1e6))
    print("\n-- data movement of the dominant decode call (M=64, K=512, N=32000: 16.4 MB of weights + 128 KB of"
          " activations read, 8.2 MB written), the grid of its kernel (250 workgroups x 512 threads) --")
    rb, wb = 512 * 32000 + 64 * 512 * 4, 64 * 32000 * 4
    us_w = stream(rb, 16, 250, 512)
    us_c = stream(rb, wb, 250, 512, 8, 1)
    print("  weight stream alone     %8.2f us  %6.2f TB/s" % (us_w, rb / us_w / 1e6))
    print("  reads + output stores   %8.2f us  %6.2f TB/s of the %d algorithmic bytes" % (us_c, (rb + wb) / us_c / 1e6, rb + wb))
    print("  (HBM roofline of those bytes at 8 TB/s: %.2f us)" % ((rb + wb) / 8e6))
    print("\n-- encoder-size operand and output sizes --")
    for name, r_, w_ in (("read 4096x4096 fp32 (67 MB), as the abs-max pass", 4096 * 4096 * 4, 16),
                         ("read 67 MB fp32 + write 16.8 MB int8, as the quantize pass", 4096 * 4096 * 4, 4096 * 4096),
                         ("write 4096x4096 fp32 (67 MB), as the GEMM's output", 16, 4096 * 4096 * 4)):
        us = stream(r_, w_, 2048, 256, 8, 0)
        print("  %-62s %8.2f us  %6.2f TB/s" % (name, us, (max(r_, 16) + max(w_, 16)) / us / 1e6))
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    print("\n-- one compute unit's LDS, vector L1 and matrix cores under instruction mixes (marian_hip_probe_mix: every "
          "wave repeats a body of 16 slots with R ds_read_b128, M v_mfma_i32_32x32x32_i8, D global_load_lds_dwordx4 and "
          "G global_load_dwordx4, 1 KB per wave and memory instruction; one workgroup per CU on all CUs; bytes per shader "
          "clock and CU, median over the workgroups) --")
    print("  %-5s %-3s %-3s %-3s %-3s %-8s | %9s %9s %9s %9s | %6s %8s" %
          ("waves", "R", "M", "D", "G", "span", "LDS rd", "DMA", "to regs", "LDS total", "MFMA", "clock"))
    print("  %-5s %-3s %-3s %-3s %-3s %-8s | %9s %9s %9s %9s | %6s %8s" %
          ("", "", "", "", "", "", "B/clk/CU", "B/clk/CU", "B/clk/CU", "B/clk/CU", "issue", "MHz"))

    def mix(waves, R, M, D, G, span, iters=400, split=0, stagger=65536, wgs=None):
        wgs = wgs or cus
        clocks = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        for _ in range(2):
            r = T.marian_hip_probe_mix(pool.data_ptr(), span, stagger, waves, R, M, D, G, split, iters, wgs, clocks.data_ptr(),
                                       sink.data_ptr(), st)
            assert r == 0, r
        torch.cuda.synchronize()
        c = clocks.cpu().numpy().reshape(-1, 2).astype(np.float64)
        clk = float(np.median(c[:, 0]))
        mhz = float(np.median(c[:, 0] / c[:, 1]) * 100.0)
        per = waves * 1024.0 * iters / clk
        cw = lw = waves
        if split:
            cw = lw = 4
        name = "%d KB" % (span >> 10) if span < (1 << 20) else "%d MB" % (span >> 20)
        rd, dma, gl = R * per * cw / waves, D * per * lw / waves, G * per * lw / waves
        print("  %-5s %-3d %-3d %-3d %-3d %-8s | %9.1f %9.1f %9.1f %9.1f | %5.0f%% %8.0f" %
              ("4+4" if split else str(waves), R, M, D, G, name, rd, dma, gl, rd + dma,
               100.0 * (cw / 4.0) * M * 32.0 * iters / clk, mhz))

    KB, MB = 1 << 10, 1 << 20
    for waves in (4, 8, 16):
        mix(waves, 16, 0, 0, 0, 64 * KB)                 # LDS reads alone
    for waves in (4, 8):
        mix(waves, 16, 0, 8, 0, 2 * MB)                  # with operand blocks arriving, 2 : 1 and 4 : 1
        mix(waves, 16, 0, 4, 0, 2 * MB)
    for span in (64 * KB, 2 * MB):                        # global -> LDS alone: vector L1 hits, L2 hits
        for waves in (4, 8, 16):
            mix(waves, 0, 0, 16, 0, span)
    for span in (64 * KB, 2 * MB):                        # global -> registers alone
        for waves in (4, 8, 16):
            mix(waves, 0, 0, 0, 16, span)
    mix(8, 0, 0, 8, 8, 2 * MB)
    for waves in (4, 8):                                  # matrix instructions with 0 / 0.5 / 0.75 / 1 / 1.5 / 2 KB of fragments each
        for R in (0, 4, 6, 8, 12, 16):
            mix(waves, R, 8, 0, 0, 64 * KB)
    for waves in (4, 8):                                  # matrix instructions with operand blocks arriving only
        mix(waves, 0, 8, 4, 0, 2 * MB)
        mix(waves, 0, 8, 0, 4, 2 * MB)
    print("  -- the large-M kernels' own mixes --")
    mix(4, 8, 8, 4, 0, 2 * MB)     # the 128x128 tile, four waves of 64x64
    mix(8, 12, 8, 4, 0, 2 * MB)    # the same tile by eight waves of 64x32 (two per SIMD)
    mix(8, 8, 8, 4, 0, 2 * MB, split=1)   # four waves multiply, four waves load
    mix(8, 8, 8, 3, 0, 2 * MB, split=1)   # the same at 48 bytes per clock of operand blocks
    mix(8, 8, 8, 2, 0, 2 * MB, split=1)   # and at 32
    mix(4, 8, 8, 3, 0, 2 * MB)
    mix(4, 8, 8, 2, 0, 2 * MB)
    mix(4, 6, 8, 3, 0, 2 * MB)     # two 256x128 tiles, four waves of 128x64
    mix(8, 6, 8, 3, 0, 2 * MB, split=1)
    mix(8, 6, 8, 2, 0, 2 * MB)     # the 256x256 tile, eight waves of 128x64
    mix(8, 4, 8, 1, 2, 2 * MB)     # the same with the weights from global memory straight into registers
    mix(8, 4, 8, 2, 2, 2 * MB)
    mix(4, 4, 8, 2, 4, 2 * MB)     # 128x128, four waves, weights straight into registers

    print("\n-- read-only streaming from HBM by instruction form and bytes in flight (marian_hip_probe_mix over 1 GiB, every "
          "workgroup its own 4 MiB-apart region; 16 KB per wave and round; chip-wide rate from the 100 MHz clock) --")

    def hbm(waves, D, G, wgs, iters=48):
        clocks = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        span = 1024 * MB
        for _ in range(2):
            r = T.marian_hip_probe_mix(pool.data_ptr(), span, span // wgs, waves, 0, 0, D, G, 0, iters, wgs,
                                       clocks.data_ptr(), sink.data_ptr(), st)
            assert r == 0, r
        torch.cuda.synchronize()
        c = clocks.cpu().numpy().reshape(-1, 2).astype(np.float64)
        secs = float(np.median(c[:, 1])) * 1e-8
        total = wgs * waves * 1024.0 * (D + G) * iters
        print("  %3d workgroups x %2d waves, %-34s %7.1f MB in %7.1f us  %5.2f TB/s" %
              (wgs, waves, "global_load_lds_dwordx4 (no VGPRs)" if D else "global_load_dwordx4 into registers", total / 1e6,
               secs * 1e6, total / secs / 1e12))

    for waves in (4, 8, 16):
        hbm(waves, 16, 0, cus)
        hbm(waves, 0, 16, cus)

    print("\n-- the same access pattern as whole launches (HIP events, back-to-back launches, each over fresh bytes): one "
          "workgroup of 16 waves per CU reads its own contiguous share of the buffer, 16 KB per workgroup and step --")
    for mb in (64, 256, 1024):
        span = mb * MB
        iters = span // (cus * 16 * 16 * KB)
        n = max(1, min(16, pool_bytes // span))
        clocks = torch.zeros(2 * cus, dtype=torch.int64, device="cuda")
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        for form, (D, G) in (("global_load_lds_dwordx4", (16, 0)), ("global_load_dwordx4", (0, 16))):
            launches = [(lambda i=i, D=D, G=G: T.marian_hip_probe_mix(pool.data_ptr() + i * span, span, span // cus, 16, 0, 0, D, G, 0,
                                                                  iters, cus, clocks.data_ptr(), sink.data_ptr(), st))
                        for i in range(n)]
            mean, med = per_launch_ms(torch, launches, max(3, 48 // n))
            print("  %5d MiB  %-24s %8.2f us  %6.2f TB/s" % (mb, form, med * 1e3, span / (med * 1e-3) / 1e12))
    print("\n-- sustained v_mfma_i32_32x32x32_i8 rate on random operand bits --")
    for per_cu in (1, 2):
        wgs, iters = cus * per_cu, 4000
        clocks = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
        sink = torch.zeros(4, dtype=torch.int32, device="cuda")
        f = lambda: T.marian_hip_probe_mfma(pool.data_ptr(), iters, wgs, clocks.data_ptr(), sink.data_ptr(), st)
        mean, med = per_launch_ms(torch, [f], 6)
        c = clocks.cpu().numpy().reshape(-1, 2).astype(np.float64)
        mhz = float(np.median(c[:, 0] / c[:, 1]) * 100.0)
        ops = 2.0 * 32 ** 3 * 8 * iters * 4 * wgs
        print("  %d workgroup(s) of 4 waves per CU: %7.1f TOPS over the launch (%.1f us), "
              "shader clock %.0f MHz -> %d CUs x 8192 op/clk x clock = %.0f TOPS"
              % (per_cu, ops / (med * 1e-3) / 1e12, med * 1e3, mhz, cus, cus * 8192 * mhz * 1e6 / 1e12))


def measured_int8_peak(torch):
    """Sustained int8 matrix rate of this device from the tuning build's MFMA probe (HIP events around
    the launches), with the shader clock it holds meanwhile and CUs x 8192 op/clk x that clock.  None
    when the tuning build is absent."""
    try:
        T = importlib.import_module(PKG + "._lib").tuning_lib()
    except Exception:
        return None
    st = torch.cuda.current_stream().cuda_stream
    cus = torch.cuda.get_device_properties(0).multi_processor_count
    data = torch.randint(-128, 128, (4096,), dtype=torch.int8, device="cuda")
    wgs, iters = cus, 4000
    clocks = torch.zeros(2 * wgs, dtype=torch.int64, device="cuda")
    sink = torch.zeros(4, dtype=torch.int32, device="cuda")
    f = lambda: T.marian_hip_probe_mfma(data.data_ptr(), iters, wgs, clocks.data_ptr(), sink.data_ptr(), st)
    mean, med = per_launch_ms(torch, [f, f, f], 4)
    c = clocks.cpu().numpy().reshape(-1, 2).astype(np.float64)
    mhz = float(np.median(c[:, 0] / c[:, 1]) * 100.0)
    ops = 2.0 * 32 ** 3 * 8 * iters * 4 * wgs
    return {"sustained_tops": round(ops / (med * 1e-3) / 1e12, 1),
            "shader_clock_mhz": round(mhz, 0),
            "cus_x_8192_x_clock_tops": round(cus * 8192 * mhz * 1e6 / 1e12, 1),
            "how": "tuning build's MFMA probe: %d workgroups of 4 waves (one wave per SIMD), %d x 8 "
                   "v_mfma_i32_32x32x32_i8 per wave on random operand bits, %.0f us per launch; clock = shader "
                   "clocks / 100 MHz reference clocks inside the loop" % (wgs, iters, med * 1e3)}


def measured_read_bw(torch):
    """What a read-only pass over 256 MiB (rotating over 1 GiB, so from HBM) reaches on this device,
    with the tuning build's streaming probe (1024 workgroups x 256 threads, 8 loads of 16 bytes in
    flight per thread; HIP events around the launches).  None when the tuning build is absent."""
    try:
        T = importlib.import_module(PKG + "._lib").tuning_lib()
    except Exception:
        return None
    st = torch.cuda.current_stream().cuda_stream
    pool = torch.empty(1 << 30, dtype=torch.int8, device="cuda").random_(-128, 127)
    dst = torch.empty(4096, dtype=torch.int8, device="cuda")
    rb = 256 << 20
    launches = [(lambda i=i: T.marian_hip_probe_stream(pool.data_ptr() + i * rb, rb, dst.data_ptr(), 16, 1024, 256, 8, 0, st))
                for i in range(4)]
    mean, med = per_launch_ms(torch, launches, 6)
    del pool
    return {"gbs": round(rb / (med * 1e-3) / 1e9, 1),
            "how": "tuning build's streaming probe: read-only pass over 256 MiB, four regions of a 1 GiB pool in turn, "
                   "1024 workgroups x 256 threads, 8 x 16 bytes in flight per thread, %.1f us per launch" % (med * 1e3)}


def pmc_summary(fetch_csv, write_csv):
    """Summarises the two rocprofv3 --pmc runs of `bench.py --pmc-probe` (FETCH_SIZE, WRITE_SIZE; KiB
    per dispatch) as the text of profiles/hbm_traffic_pmc.txt."""
    import csv
    import subprocess

    def short(name):
        for key, pat in (("copy64", "vectorized_elementwise_kernel<4, at::native::CUDAFunctorOnSelf_add<float>"),
                         ("stream32_fused_M64_K512_N32000", "gemm_stream32_kernel<2, 4, 2, 8, 1, 4, 64"),
                         ("gemm_pair", "gemm_pair_kernel"), ("gemm_mfma32", "gemm_mfma32_kernel"),
                         ("gemm_mfma32_split", "gemm_mfma32_split_kernel"),
                         ("absmax", "absmax_partial_kernel"), ("quantize_a", "quantize_a_kernel"),
                         ("prepare_a_onepass", "prepare_a_onepass_kernel")):
            if pat in name:
                if key in ("gemm_mfma32", "gemm_mfma32_split", "prepare_a_onepass"):   # keep the template arguments apart
                    return key + "|" + name.split(pat)[1].split("(")[0]
                return key
        return None

    def load(path, counter):
        acc = {}
        for row in csv.DictReader(open(path)):
            if row["Counter_Name"] != counter:
                continue
            k = short(row["Kernel_Name"])
            if k is None:
                continue
            k = (k, int(row["Grid_Size"]))
            acc.setdefault(k, []).append(float(row["Counter_Value"]))
        return {k: sum(v) / len(v) for k, v in acc.items()}

    fetch, write = load(fetch_csv, "FETCH_SIZE"), load(write_csv, "WRITE_SIZE")
    copy_key = [k for k in fetch if k[0] == "copy64"][0]
    f_scale, w_scale = 65536.0 / fetch[copy_key], 65536.0 / write[copy_key]
    try:
        commit = subprocess.run(["git", "-C", ROOT, "rev-parse", "--short", "HEAD"], capture_output=True, text=True).stdout.strip()
    except OSError:
        commit = ""
    print("yardstick: plain elementwise copy of 64 MiB fp32 (torch.add(src, 1.0, out=dst): reads 65536 KiB, writes 65536 KiB)")
    print("  FETCH_SIZE %9.1f KiB -> scale factor %.4f" % (fetch[copy_key], f_scale))
    print("  WRITE_SIZE %9.1f KiB -> scale factor %.4f" % (write[copy_key], w_scale))
    print("")
    print("%-58s %10s %12s %10s %12s" % ("kernel | grid size (threads)", "FETCH raw", "FETCH scaled", "WRITE", "total KiB"))
    lines = []
    for k in sorted(fetch):
        if k[0] == "copy64":
            continue
        fs, w = fetch[k] * f_scale, write.get(k, 0.0) * w_scale
        print("%-58s %10.1f %12.1f %10.1f %12.1f" % ("%s | %d" % k, fetch[k], fs, w, fs + w))
        lines.append((k, int((fs + w) * 1024)))
    print("")
    for (name, grid), b in lines:
        key = name if name.startswith("stream32") else "%s_grid%d" % (name.replace("|", "").replace(" ", "").replace(",", "_"), grid)
        print("traffic_bytes_per_launch %s = %d" % (key, b))
    print("build_commit = %s" % (commit or "unknown"))


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=200)
    ap.add_argument("--warmup", type=int, default=20)
    ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
    ap.add_argument("--pmc-probe", action="store_true",
                    help="launch the dominant kernels and a plain copy a few times and exit "
                         "(for rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE)")
    ap.add_argument("--only", default="", help="comma list of extra workloads: encoder,shortlist,big")
    ap.add_argument("--cpu-worker", type=float, default=0.0, metavar="SECONDS",
                    help="(internal) one instance of the aggregate CPU baseline; no GPU")
    ap.add_argument("--probe-ceilings", action="store_true",
                    help="measure the machine ceilings (read / write / copy bandwidth by footprint, launch "
                         "floor, data movement of the dominant call, sustained int8 MFMA rate and clock) "
                         "with the tuning build's probe kernels, print a text table and exit")
    ap.add_argument("--pmc-summary", nargs=2, metavar=("FETCH_CSV", "WRITE_CSV"),
                    help="summarise two rocprofv3 --pmc counter_collection.csv files of --pmc-probe runs "
                         "(the text of profiles/hbm_traffic_pmc.txt) and exit; no GPU")
    args = ap.parse_args()
    if args.cpu_worker > 0:
        cpu_worker(args.cpu_worker)
        return
    if args.pmc_summary:
        pmc_summary(*args.pmc_summary)
        return
    if args.gpus != 1:
        sys.exit("bench.py: this path runs on one GPU (no collectives are part of it); use --gpus 1")

    import torch
    assert torch.cuda.is_available(), "bench.py needs a GPU"
    integer = importlib.import_module(PKG + ".integer")
    integer.Type = importlib.import_module(PKG + ".types").Type
    lib = importlib.import_module(PKG + "._lib").lib()
    torch.cuda.set_device(0)
    be = integer.Backend.get("cuda:0")
    extras = set(x for x in args.only.split(",") if x) or {"encoder", "shortlist", "big"}

    if args.pmc_probe:
        pmc_probe(torch, integer, lib, be)
        return
    if args.probe_ceilings:
        probe_ceilings(torch)
        return

    # ---------------- headline: transformer-base decode sweep -------------------------------
    sweep_bytes = sum(K * N for K, N in DECODE_SHAPES) * len(DECODE_M)
    sets = max(2, int(np.ceil(512e6 / sweep_bytes)) + 1)       # rotate > 512 MB of weights
    ops_list = [Op(torch, integer, M, K, N, copies=sets, seed=i * 10 + j)
                for i, (K, N) in enumerate(DECODE_SHAPES) for j, M in enumerate(DECODE_M)]
    step_ops = sum(o.ops for o in ops_list)
    step_bytes = sum(algorithmic_bytes(o.M, o.K, o.N) for o in ops_list)

    def step(copy):
        for o in ops_list:
            o.launch_fused(lib, be, copy)

    graphs = [capture(torch, (lambda c=c: step(c))) for c in range(sets)]
    dt = time_graphs(torch, graphs, args.steps, args.warmup)
    ms_per_step = dt / args.steps * 1e3
    tops = step_ops / (dt / args.steps) / 1e12
    # same with one weight set (Infinity-Cache resident), and eager launches from the host
    dt_res = time_graphs(torch, graphs[:1], args.steps, args.warmup)
    # The same passes launched eagerly, call after call on the stream, as Marian's forward tape
    # launches (reference src/graph/expression_graph.cpp:141-175): the twenty C-ABI calls of a pass
    # with their arguments bound beforehand, so that the host loop is the calls and nothing else.
    fn = lib.marian_hip_int8_affine_f32
    ws_ptr, ws_bytes, st_ptr = be.workspace.data_ptr(), be.workspace_bytes, be.stream()
    bound = [[(o.A.data_ptr(), o.Aq.data_ptr(), o.Bq[c].data_ptr(), o.bias.data_ptr(), None, 0, o.out.data_ptr(),
               o.M, o.K, o.N, 1.0, o.relu, ws_ptr, ws_bytes, st_ptr) for o in ops_list] for c in range(sets)]

    def eager_passes(n):
        for p in range(n):
            for a in bound[p % sets]:
                if fn(*a) != 0:
                    raise RuntimeError("marian_hip_int8_affine_f32 failed")
    eager_passes(args.warmup)
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    eager_passes(args.steps)
    t_issued = time.perf_counter()
    torch.cuda.synchronize()
    eager_dt = time.perf_counter() - t0
    eager_ms = eager_dt / args.steps * 1e3
    eager_host_ms = (t_issued - t0) / args.steps * 1e3   # what the host loop alone takes per pass
    # ... and the same K passes from a C++ host thread through the C++ wrappers (a child process)
    eager_cpp = eager_sweep_cpp_host(args.steps, args.warmup)
    # the headline is the fastest of the three ways to launch the same twenty calls per pass
    graph_ms, graph_tops = ms_per_step, tops
    eager_tops = step_ops / (eager_dt / args.steps) / 1e12
    launch = "HIP graph replay"
    if eager_tops > tops:
        ms_per_step, tops, dt = eager_ms, eager_tops, eager_dt
        launch = "eager: the twenty C-ABI calls of a pass issued back to back from this process, no recorded graph"
    if eager_cpp and step_ops / (eager_cpp * 1e-3) / 1e12 > tops:
        ms_per_step, tops, dt = eager_cpp, step_ops / (eager_cpp * 1e-3) / 1e12, eager_cpp * 1e-3 * args.steps
        launch = ("eager: the twenty calls of a pass issued back to back from a C++ host thread through the C++ "
                  "wrappers (marian-dev_amd/host/eager_sweep, a child process), no recorded graph")

    # ---------------- roofline of the dominant kernel ----------------------------------------
    # vocabulary projection of the sweep at M = 64 (16.4 MB of int8 weights, 8.2 MB of output):
    # the fused quantize + GEMM kernel, which moves exactly the algorithmic bytes of the call
    dom = [o for o in ops_list if o.N == 32000 and o.M == 64][0]
    mean_ms, med_ms = per_launch_ms(
        torch, [(lambda c=c: dom.launch_fused(lib, be, c)) for c in range(sets)], 12)
    dom_bytes = algorithmic_bytes(dom.M, dom.K, dom.N)
    traffic = measured_traffic()
    achieved = dom_bytes / (mean_ms * 1e-3) / 1e9
    read_bw = measured_read_bw(torch)
    roofline = {"bound": "hbm", "achieved": round(achieved, 1), "peak": HBM_PEAK_GBS,
                "unit": "GB/s", "frac": round(achieved / HBM_PEAK_GBS, 4),
                "frac_of_measured_read_bw": None if not read_bw else round(achieved / read_bw["gbs"], 4),
                "measured_read_bw": read_bw,
                "traffic": traffic.get("stream32_fused_M64_K512_N32000"),
                "traffic_source": "profiles/hbm_traffic_pmc.txt (rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE, scaled by a "
                                  "64 MiB copy), sources at commit %s" % traffic["_commit"]
                                  if traffic.get("stream32_fused_M64_K512_N32000") else None,
                "kernel": "gemm_stream32_kernel<MT32=2,WN=4,KW=2,PW=8,fused> M=64 K=512 N=32000",
                "bytes_per_launch": dom_bytes, "avg_launch_us": round(mean_ms * 1e3, 3),
                "median_launch_us": round(med_ms * 1e3, 3),
                "launches_timed": 12 * sets}

    per_shape = {}
    for (K, N) in DECODE_SHAPES:
        for M in DECODE_M:
            o = [x for x in ops_list if (x.M, x.K, x.N) == (M, K, N)][0]
            o.launch(lib, be, 0, prepare=True, gemm=False)
            g_ms, _ = per_launch_ms(
                torch, [(lambda c=c, o=o: o.launch(lib, be, c, prepare=False)) for c in range(sets)], 3)
            f_ms, _ = per_launch_ms(
                torch, [(lambda c=c, o=o: o.launch_fused(lib, be, c)) for c in range(sets)], 3)
            per_shape["M%d_%dx%d" % (M, K, N)] = {
                "affine_f32_us": round(f_ms * 1e3, 2), "gemm_only_us": round(g_ms * 1e3, 2),
                "affine_hbm_frac": round(algorithmic_bytes(M, K, N) / (f_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}

    out = {
        "metric": "int8 affine TOPS & % roofline; transformer-big int8 decode tokens/sec",
        "value": round(tops, 4), "unit": "TOPS", "n_gpus": 1, "steps": args.steps,
        "warmup": args.warmup, "ms_per_step": round(ms_per_step, 5), "higher_is_better": True,
        "scaling": "weak", "vs_baseline": None, "dtype": "int8",
        "dtype_detail": "int8 x int8 -> int32 accumulate, fp32 quantize and epilogue",
        "data": "synthetic",
        "config": {"workload": "transformer-base decode GEMM sweep: M in {1,4,16,64} x "
                               "{512x1536, 512x512, 512x2048, 2048x512, 512x32000}, "
                               "prepareA + int8 affine with bias per shape",
                   "launch": "%s; %d rotating weight sets (%.0f MB)" % (launch, sets, sets * sweep_bytes / 1e6),
                   "step_ops": step_ops, "step_algorithmic_bytes": step_bytes},
        "step_hbm_frac": round(step_bytes / (dt / args.steps) / 1e9 / HBM_PEAK_GBS, 4),
        "value_cache_resident_tops": round(step_ops / (dt_res / args.steps) / 1e12, 4),
        "eager_ms_per_step": round(eager_ms, 5), "eager_tops": round(eager_tops, 4),
        "eager_host_issue_ms_per_step": round(eager_host_ms, 5),
        "graph_replay_ms_per_step": round(graph_ms, 5), "graph_replay_tops": round(graph_tops, 4),
        "eager_ms_per_step_cpp_host": eager_cpp,
        "eager_tops_cpp_host": round(step_ops / (eager_cpp * 1e-3) / 1e12, 4) if eager_cpp else None,
        "roofline": roofline,
        "per_shape": per_shape,
    }
    del graphs
    del ops_list

    # ---------------- encoder-size GEMMs (MFMA-bound case) ------------------------------------
    if "encoder" in extras:
        enc = {}
        sustained = measured_int8_peak(torch)
        for (M, K, N) in [(4096, 1024, 4096), (4096, 4096, 1024)]:
            o = Op(torch, integer, M, K, N, relu=True, copies=4, seed=77)
            o.launch(lib, be, 0, prepare=True, gemm=False)
            g_ms, g_med = per_launch_ms(
                torch, [(lambda c=c: o.launch(lib, be, c, prepare=False)) for c in range(4)], 10)
            p_ms, _ = per_launch_ms(torch, [(lambda: o.launch(lib, be, 0, gemm=False))], 10)
            # the call BASELINE defines (fp32 A in, fp32 out) through the single entry point, timed as one
            f_ms, _ = per_launch_ms(torch, [(lambda c=c: o.launch_fused(lib, be, c)) for c in range(4)], 10)
            # the same call when the producer of A left its abs-max (no abs-max pass) and this call leaves
            # the abs-max of its own output for the next one
            amax_in = torch.zeros(2048, device="cuda")
            amax_in[0] = o.A.abs().max()
            amax_out = torch.empty(2048, device="cuda")

            def chained(c, o=o, amax_in=amax_in, amax_out=amax_out):
                b = o.Bq[c % len(o.Bq)]
                r = lib.marian_hip_int8_affine_f32_chained(
                    o.A.data_ptr(), o.Aq.data_ptr(), b.data_ptr(), o.bias.data_ptr(), None, 0, o.out.data_ptr(),
                    o.M, o.K, o.N, 1.0, o.relu, amax_in.data_ptr(), amax_out.data_ptr(),
                    be.workspace.data_ptr(), be.workspace_bytes, be.stream())
                assert r == 0, r
            c_ms, _ = per_launch_ms(torch, [(lambda c=c: chained(c)) for c in range(4)], 10)
            chained(0)
            torch.cuda.synchronize()
            slots_ok = bool(float(amax_out.max()) == float(o.out.abs().max()))
            t_all = f_ms * 1e-3
            enc["M%d_K%d_N%d" % (M, K, N)] = {
                "gemm_us": round(g_ms * 1e3, 2), "gemm_median_us": round(g_med * 1e3, 2),
                "prepare_a_us": round(p_ms * 1e3, 2),
                "affine_f32_us": round(f_ms * 1e3, 2),
                "affine_f32_chained_us": round(c_ms * 1e3, 2),
                "chained_leaves_exact_absmax": slots_ok,
                "gemm_tops": round(o.ops / (g_ms * 1e-3) / 1e12, 1),
                "gemm_mfma_frac": round(o.ops / (g_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4),
                "gemm_frac_of_sustained": None if not sustained else
                    round(o.ops / (g_ms * 1e-3) / 1e12 / sustained["sustained_tops"], 4),
                "gemm_hbm_frac": round(gemm_kernel_bytes(M, K, N) / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
                "affine_tops": round(o.ops / t_all / 1e12, 1),
                "affine_hbm_frac": round(algorithmic_bytes(M, K, N) / t_all / 1e9 / HBM_PEAK_GBS, 4),
                "affine_chained_hbm_frac": round(algorithmic_bytes(M, K, N) / (c_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
            del o
        # a few rows or columns past a whole number of tiles (encoder M is a sum of sentence lengths)
        for (M, K, N) in [(4100, 1024, 4096), (2050, 1024, 2056), (4100, 4096, 1024)]:
            o = Op(torch, integer, M, K, N, relu=True, copies=4, seed=78)
            o.launch(lib, be, 0, prepare=True, gemm=False)
            g_ms, g_med = per_launch_ms(
                torch, [(lambda c=c: o.launch(lib, be, c, prepare=False)) for c in range(4)], 10)
            enc["M%d_K%d_N%d" % (M, K, N)] = {
                "gemm_us": round(g_ms * 1e3, 2), "gemm_median_us": round(g_med * 1e3, 2),
                "gemm_tops": round(o.ops / (g_ms * 1e-3) / 1e12, 1),
                "gemm_mfma_frac": round(o.ops / (g_ms * 1e-3) / 1e12 / INT8_PEAK_TOPS, 4)}
            del o
        out["encoder"] = enc
        out["int8_peak_tops_used"] = INT8_PEAK_TOPS
        out["int8_peak_measured"] = sustained

    # ---------------- shortlisted output layer -------------------------------------------------
    if "shortlist" in extras:
        synth = importlib.import_module(PKG + ".synth")
        sl = {}
        M, K, N = 256, 1024, 32000
        for name, ids in [("full", None), ("n504", synth.shortlist(11, N, 504, 504)),
                          ("n1000", synth.shortlist(12, N, 1000, 1000)),
                          ("n2000", synth.shortlist(13, N, 2000, 2000))]:
            idx = None if ids is None else torch.from_numpy(ids.view(np.int32)).cuda()
            o = Op(torch, integer, M, K, N, copies=8 if ids is None else 2, idx=idx, seed=5)
            o.launch(lib, be, 0, prepare=True, gemm=False)
            g_ms, _ = per_launch_ms(
                torch, [(lambda c=c: o.launch(lib, be, c, prepare=False)) for c in range(len(o.Bq))], 6)
            sl[name] = {"n_out": o.n_out, "gemm_us": round(g_ms * 1e3, 2),
                        "gemm_tops": round(o.ops / (g_ms * 1e-3) / 1e12, 2),
                        "gemm_hbm_frac": round(gemm_kernel_bytes(M, K, o.n_out, ids is not None)
                                               / (g_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4)}
            del o
        out["shortlist"] = sl

    # ---------------- transformer-big decode step (GEMMs only) ----------------------------------
    if "big" in extras:
        d, ffn, V, M = 1024, 4096, 32000, 128
        layer = [(d, d, 0)] * 6 + [(d, ffn, 1), (ffn, d, 0)]     # self q,k,v,o; ctx q,o; ffn1, ffn2
        shapes = layer * 6 + [(d, V, 0)]
        wbytes = sum(K * N for K, N, _ in shapes)
        bsets = max(2, int(np.ceil(512e6 / wbytes)) + 1)
        ops_big = [Op(torch, integer, M, K, N, relu=r, copies=bsets, seed=200 + i)
                   for i, (K, N, r) in enumerate(shapes)]

        def big_step(copy):
            for o in ops_big:
                o.launch_fused(lib, be, copy)

        bgraphs = [capture(torch, (lambda c=c: big_step(c))) for c in range(bsets)]
        n = max(20, args.steps // 2)
        bdt = time_graphs(torch, bgraphs, n, max(4, args.warmup // 2))
        out["transformer_big_decode"] = {
            "what": "GEMM-only decode step at beam 4 x batch 32 (M=128): 48 layer GEMMs + "
                    "32000-vocab output GEMM, each with its prepareA; self-attention K/V "
                    "projections taken at M=128",
            "ms_per_step": round(bdt / n * 1e3, 4),
            "hyp_tokens_per_s": round(M * n / bdt, 1),
            "output_tokens_per_s": round(32 * n / bdt, 1),
            "tops": round(sum(o.ops for o in ops_big) * n / bdt / 1e12, 2),
            "weight_hbm_frac": round(wbytes * n / bdt / 1e9 / HBM_PEAK_GBS, 4),
            "weight_sets": bsets}
        del bgraphs
        del ops_big

        # the same step with everything between the GEMMs (N3 operators) through the host mirrors
        ops_mod = importlib.import_module(PKG + ".ops")
        dec = BigDecoder(torch, integer, ops_mod, bsets)
        # chained and unchained steps give the same bits
        same = bool(torch.equal(dec.step(0, chained=True), dec.step(0, chained=False)))
        unch = [capture(torch, (lambda c=c: dec.step(c, chained=False))) for c in range(bsets)]
        udt = time_graphs(torch, unch, n, max(4, args.warmup // 2))
        del unch
        # the same n-best whether log-softmax and n-best are two launches (the log-probabilities
        # written out, as the reference's graph does) or one
        lp0 = dec.step(0)
        v_sep, k_sep = ops_mod.getNBestListOfBeams(lp0.view(dec.beam, 1, dec.batch, dec.V), dec.beam)
        v_one, k_one = dec.step(0, fused_tail=True)
        same_tail = bool(torch.equal(v_sep, v_one) and torch.equal(k_sep, k_one))
        sep = [capture(torch, (lambda c=c: dec.step(c))) for c in range(bsets)]
        sdt = time_graphs(torch, sep, n, max(4, args.warmup // 2))
        del sep
        full = [capture(torch, (lambda c=c: dec.step(c, fused_tail=True))) for c in range(bsets)]
        fdt = time_graphs(torch, full, n, max(4, args.warmup // 2))
        # the same bits whether projections and attention are one launch or two
        o_f = dec.step(0, fused_tail=True)
        o_s = dec.step(0, fused_tail=True, fused_attention=False)
        same_att = bool(torch.equal(o_f[0], o_s[0]) and torch.equal(o_f[1], o_s[1]))
        sepatt = [capture(torch, (lambda c=c: dec.step(c, fused_tail=True, fused_attention=False))) for c in range(bsets)]
        sadt = time_graphs(torch, sepatt, n, max(4, args.warmup // 2))
        del sepatt
        gonly = [capture(torch, (lambda c=c: dec.step(c, gemm_only=True))) for c in range(bsets)]
        gdt = time_graphs(torch, gonly, n, max(4, args.warmup // 2))
        # the same step launched eagerly, call by call, from this Python host (Marian launches its
        # forward tape eagerly too, from C++): the host's own time per call - ctypes, torch's
        # allocator for every output - is part of this figure
        for c in range(3):
            dec.step(c, fused_tail=True)
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for c in range(10):
            dec.step(c, fused_tail=True)
        torch.cuda.synchronize()
        eager_full_ms = (time.perf_counter() - t0) / 10 * 1e3
        dk = dec.d // dec.H
        cache_bytes = 2 * dec.layers * 4 * dk * dec.H * (dec.M * dec.T + dec.batch * dec.L)
        step_bytes_big = dec.weight_bytes + cache_bytes + 4 * dec.M * dec.V
        sel = [capture(torch, (lambda c=c: dec.step(c, fused_tail=True, select=True))) for c in range(bsets)]
        seldt = time_graphs(torch, sel, n, max(4, args.warmup // 2))
        del sel
        dec.by_ancestors = True    # the same step on caches that are never moved
        dec.anc = torch.randint(0, dec.M, (dec.M, dec.cap), device="cuda", dtype=torch.int32)
        dec.anc = (dec.anc // dec.batch * dec.batch + torch.arange(dec.M, device="cuda", dtype=torch.int32)[:, None] % dec.batch).contiguous()
        dec.anc_next = torch.empty_like(dec.anc)
        sel = [capture(torch, (lambda c=c: dec.step(c, fused_tail=True, select=True))) for c in range(bsets)]
        ancdt = time_graphs(torch, sel, n, max(4, args.warmup // 2))
        del sel
        dec.by_ancestors = False
        eager_step_ms = cpp_host_figure("eager_step", "eager_ms_per_step_cpp_host", ("200", "20"))
        graph_step_ms = fdt / n * 1e3
        # the figure of the step: the faster of the two ways to launch the same 58 kernels
        step_ms = min(graph_step_ms, eager_step_ms) if eager_step_ms else graph_step_ms
        out["transformer_big_decode_full"] = {
            "what": "full decoder step through the host mirrors, from the previous step's word indices: embedding rows x "
                    "sqrt(d) + position signal (one launch), 49 int8 affine products + per layer "
                    "2 attentions (20 cached positions + the new one, appended by the call; "
                    "source lengths uniform 20..60, padded to 60 positions with mask), 3 skip-add+layer-norm; the self-attention "
                    "projections Wq, Wk, Wv and the self-attention are one launch, the context attention's Wq and the context "
                    "attention another (58 launches per step); log-softmax over 32000, beam/batch transposition + n-best per "
                    "sentence in one launch (the log-probabilities are not written out); no hypothesis bookkeeping; the "
                    "abs-max of every GEMM input is left by the kernel that produced it",
            "ms_per_step": round(step_ms, 4),
            "launch": ("eager: the 58 launches of a step call by call from a C++ host thread (host/eager_step.cpp), no graph"
                       if step_ms < graph_step_ms else "the step as a replayed HIP graph"),
            "graph_replay_ms_per_step": round(graph_step_ms, 4),
            "variants": "the ms_per_step_* figures below are replayed graphs of the Python mirror's step: compare them with "
                        "graph_replay_ms_per_step",
            "ms_per_step_with_state_selection": round(seldt / n * 1e3, 4),
            "ms_per_step_with_state_selection_by_ancestors": round(ancdt / n * 1e3, 4),
            "state_selection_by_ancestors": "the caches stay where they were written; a table [hypotheses, positions] says in "
                                            "whose cache entry a position of a hypothesis's history lies (here: a random "
                                            "hypothesis of the same sentence per position), the selection rewrites the table "
                                            "and the self-attention follows it",
            "state_selection": "the step preceded by the beam search's selection of the surviving hypotheses' cached keys "
                               "and values (rows(state, hypIndices) over all layers as one gather of the positions in use, %d MB read and written); "
                               "hypothesis indices resident on the device" % round(dec.state.numel() * 4 / 1e6 * (dec.T - 1) / dec.cap),
            "ms_per_step_projections_and_attention_as_separate_launches": round(sadt / n * 1e3, 4),
            "one_launch_attention_equals_separate_launches": same_att,
            "ms_per_step_logsoftmax_and_nbest_as_two_launches": round(sdt / n * 1e3, 4),
            "one_launch_tail_equals_two_launches": same_tail,
            "ms_per_step_unchained": round(udt / n * 1e3, 4),
            "chained_equals_unchained": same,
            "eager_ms_per_step_python_host": round(eager_full_ms, 4),
            "eager_ms_per_step_cpp_host": eager_step_ms,
            "eager_hyp_tokens_per_s_cpp_host": round(dec.M / (eager_step_ms * 1e-3), 1) if eager_step_ms else None,
            "step_hbm_frac": round(step_bytes_big / (step_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "weight_hbm_frac": round(dec.weight_bytes / (step_ms * 1e-3) / 1e9 / HBM_PEAK_GBS, 4),
            "step_algorithmic_bytes": {"int8_weights": dec.weight_bytes, "cached_keys_and_values_read": cache_bytes,
                                       "logits_written": 4 * dec.M * dec.V},
            "hyp_tokens_per_s": round(dec.M / (step_ms * 1e-3), 1),
            "output_tokens_per_s": round(dec.batch / (step_ms * 1e-3), 1),
            "gemm_only_ms_per_step_same_harness": round(gdt / n * 1e3, 4),
            "non_gemm_share": round(1.0 - gdt / fdt, 3)}
        del full, gonly, dec

    if not args.no_cpu:
        cpu = cpu_baseline()
        big_cpu = cpu.pop("transformer_big_decode")
        out["cpu_baseline"] = cpu
        if "transformer_big_decode" in out:   # the CPU figure beside the tokens/s it belongs to
            out["transformer_big_decode"]["cpu_baseline"] = big_cpu
            out["transformer_big_decode_full"]["cpu_baseline_gemm_only"] = big_cpu
    else:
        out["cpu_baseline"] = None
    print(json.dumps(out))


if __name__ == "__main__":
    main()
