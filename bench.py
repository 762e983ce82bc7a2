#!/usr/bin/env python3
"""Benchmark of the quantized-linear hot path on one MI355X.

Workload (BASELINE.json configs[1] at M = 1): the four W4A16 g128 asymmetric quantized linears of a
Llama-2-7B decoder layer -- fused QKV (12288x4096), O-proj (4096x4096), gate+up (22016x4096) and
down (4096x11008) -- applied to one fp16 activation row.  One *step* is one pass over those four
linears for one layer.  Consecutive steps use different layers' weights (NL resident copies, more
than the 256 MB Infinity Cache in total), so every step streams its weights from HBM as a decode
pass over a real model does.  All K timed steps are captured in one HIP graph (the launch-bound
inner loop of a decode step) and replayed once between synchronisations.

Output.  stdout carries ONE compact JSON line (under 4 kB, `compact_line`): the headline keys (`metric`, `value` =
algorithmic bytes moved per second over the timed region by the reference's own footprint formula,
reproduce/fig9/plot_bandwidth_size.py:37-44, `ms_per_step`, ...), `roofline` = the dominant kernel (gate+up)
against the 8 TB/s HBM peak, its duration measured here with HIP events on the launch stream, beside two
ceilings measured in the same run (`roofline.empirical`: a pure streaming read of the same number of bytes, and a
large dense fp16 GEMM of the vendor library), `cpu_baseline` = the torch CPU port of the reference's test path on
the same four shapes on this machine's host cores (dequant + matmul, and matmul alone), and one short row per
shape of the further sections.  The full report -- every section below with every field -- goes to stderr and to
the side file `bench_report.json` (`write_report`).  Further sections, none of them part of `value`: `small_m` (configs[1] at
M = 4 / 16, configs[2]: the bit-width sweep at N = K = 8192, the Llama-3-70B shapes at M = 1 and 16),
`gemm_m256` and `gemm_m32_m64_m128` (configs[3]), `gemm_prefill_m8192` (the Llama-2-7B layers at configs[4]'s
prefill row count) and `decode` (configs[4]: the Llama-2-7B-shaped decode loop at batch 1 / 16 / 64).

Other modes (each prints its own JSON and exits): `--counter-pass` and `--counter-pass-matrix` (a few eager
launches of the GEMV kernels / of the matrix-core kernels beside a copy of known size, for `rocprofv3 --pmc`),
`--shape-sets` (the reference's figure 6 / 9 / 10 and table 3 shape sets: achieved bandwidth and speed-up over the
dense fp16 GEMM), `--launch-floor` (an empty kernel and a pure streaming read), `--ablation` (each kernel family
beside timing builds of itself that leave one part out).

Every per-kernel timing rotates over at least 512 MB of distinct packed weights (twice the 256 MB
Infinity Cache), so each launch streams its weights from HBM.
"""
import argparse
import json
import os
import sys
import time

ROOT = os.path.dirname(os.path.abspath(__file__))
PKG_PARENT = os.path.join(ROOT, "qfactory-ae_amd")
for _p in (ROOT, PKG_PARENT):
    if _p not in sys.path:
        sys.path.insert(0, _p)
os.environ.setdefault("QFACTORY_CACHE_DIR", os.path.join(PKG_PARENT, "jit_cache"))
os.environ.setdefault("QFACTORY_LOG_LEVEL", "WARNING")

HBM_PEAK_GBPS = 8000.0
MFMA_F16_PEAK_TFLOPS = 2516.6          # 256 CUs x 4096 FLOP/clk x 2.4 GHz, dense fp16
GEMM_SHAPES = [("qkv70b", 10240, 8192), ("o70b", 8192, 8192), ("gate_up70b", 57344, 8192), ("down70b", 8192, 28672)]
SHAPES = [("qkv", 12288, 4096), ("o", 4096, 4096), ("gate_up", 22016, 4096), ("down", 4096, 11008)]  # (name, N, K)
NBITS, GS = 4, 128
DOMINANT = "gate_up"


def algorithmic_bytes(M, N, K, nbits=NBITS, gs=GS, sym=False):
    b = (M * K + M * N) * 2 + N * K * nbits / 8 + N * (K // gs) * 2
    if not sym:
        b += N * (K // gs) * nbits / 8
    return b


def log(*a):
    print(*a, file=sys.stderr, flush=True)


def build_layers(n_layers, M):
    import torch
    from qfactory import QLinear
    flags = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
    g = torch.Generator(device="cuda").manual_seed(0)
    layers = []
    for _ in range(n_layers):
        layer = {}
        for name, N, K in SHAPES:
            lin = QLinear.empty(M, K, N, NBITS, GS, sym=False, compile_flags=flags)
            lin.w.copy_(torch.randint(-128, 128, lin.w.shape, dtype=torch.int8, device="cuda", generator=g))
            lin.s.copy_((torch.rand(lin.s.shape, device="cuda", generator=g) * 0.019 + 0.001).to(torch.float16))
            lin.z.copy_(torch.randint(-128, 128, lin.z.shape, dtype=torch.int8, device="cuda", generator=g))
            layer[name] = lin
        layers.append(layer)
    acts = {K: torch.randn(M, K, device="cuda", generator=g).to(torch.float16) for K in {k for _, _, k in SHAPES}}
    return layers, acts


def run_step(layer, acts):
    outs = []
    for name, N, K in SHAPES:
        outs.append(layer[name](acts[K]))
    return outs


def check_against_oracle(layer, acts):
    """One linear of the benchmark data against the CPU oracle (the checker, not the thing timed)."""
    import numpy as np
    from oracle import qf_oracle
    lin = layer["o"]
    out = lin(acts[4096]).cpu().numpy()
    rows = np.arange(0, 4096, 8)
    ref = qf_oracle.qlinear_np(acts[4096].cpu().numpy(), lin.w.cpu().numpy()[rows], lin.s.cpu().numpy()[rows],
                               lin.z.cpu().numpy()[rows], NBITS, GS)
    m = qf_oracle.error_metrics(out[:, rows], ref)
    assert m["max_rel"] <= 1e-2 and m["nrms"] <= 1e-3, f"benchmark data fails parity: {m}"
    return m


COLD_BYTES = 512 << 20          # distinct packed bytes a per-kernel timing rotates over: 2 x the 256 MB Infinity Cache


def cold_copies(bytes_per_copy, minimum=2):
    """Number of distinct weight copies a timing needs so that a launch never finds its weights in a cache."""
    return max(minimum, -(-COLD_BYTES // int(bytes_per_copy)))


def weight_sets(lin, n, gen):
    """`n` independent sets of packed tensors (w, s, z) shaped like the layer's, random bytes / scales in range."""
    import torch
    sets = []
    for _ in range(n):
        w = torch.randint(-128, 128, lin.w.shape, dtype=torch.int8, device="cuda", generator=gen)
        s = (torch.rand(lin.s.shape, device="cuda", generator=gen) * 0.019 + 0.001).to(torch.float16)
        z = None if lin.z is None else torch.randint(-128, 128, lin.z.shape, dtype=torch.int8, device="cuda", generator=gen)
        sets.append((w, s, z))
    return sets


WARM_MS = 30.0                  # untimed replays in front of a timing: at least two, and at least this long


def warm_replays(graph):
    """Replay `graph` untimed until the GPU has worked for WARM_MS without a pause (at least twice).  After the
    allocations and host work in front of a timing the first replays read slow -- the 22016 x 4096 GEMV 9.6 us
    per launch in the first 5 ms against 9.1 - 9.2 from the third measurement of the same graph on -- so every
    timing starts from the same sustained state."""
    import torch
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    graph.replay()
    end.record()
    torch.cuda.synchronize()
    once = max(start.elapsed_time(end), 1e-3)
    for _ in range(max(1, min(200, int(WARM_MS / once)))):
        graph.replay()
    torch.cuda.synchronize()
    # One more replay on its own: the first replay behind a burst of queued ones takes about 40 us longer than
    # every later one (2 us per step of a 20-step graph: 27.5 against 25.7 us per step measured), whatever its length.
    graph.replay()
    torch.cuda.synchronize()


def kernel_event_time_us(func, sets, x, n_out, reps=None):
    """Average duration of one launch of a compiled closure with cold weights.

    `reps` back-to-back launches (rotating over the distinct weight sets, at least 512 MB of them) are
    captured in a HIP graph on a side stream; the replay is bracketed by HIP events recorded on the stream
    it is launched on, and the elapsed time is divided by `reps`.  Back-to-back launches on one stream
    serialise on this GPU, so this is the per-launch duration a kernel trace reports -- once the replay's own
    fixed cost (about 9 us between the first event and the first kernel, measured) is spread over enough
    launches: at least 64 and two passes over the weight sets; 16 launches read 0.5 us per launch high.  The timed
    replays follow WARM_MS of untimed ones (`warm_replays`).
    """
    import torch
    reps = reps or max(64, 2 * len(sets))
    out = torch.empty(x.shape[0], n_out, dtype=torch.float16, device="cuda")

    def launches():
        for i in range(reps):
            w, s, z = sets[i % len(sets)]
            rc = func(x, w, out, s, z) if z is not None else func(x, w, out, s)
            assert rc == 0

    launches()
    torch.cuda.synchronize()
    graph = torch.cuda.CUDAGraph()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        with torch.cuda.graph(graph, stream=side):
            launches()
    torch.cuda.current_stream().wait_stream(side)
    warm_replays(graph)
    best = []
    for _ in range(5):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        end.record()
        torch.cuda.synchronize()
        best.append(start.elapsed_time(end) * 1e3 / reps)
    best.sort()
    return best[len(best) // 2]


def stream_read_time_us(nbytes):
    """A pure 128-bit streaming read (qf_stream_read of libqfactory_hip.so) of `nbytes` cold bytes, timed like a
    kernel above: the ceiling this machine gives a launch that only has to read that many bytes."""
    import torch
    from qfactory import native
    nbytes = int(nbytes) // 4096 * 4096
    n = cold_copies(nbytes)
    bufs = [torch.randint(-128, 128, (nbytes,), dtype=torch.int8, device="cuda") for _ in range(n)]
    sink = torch.zeros(4096, dtype=torch.int32, device="cuda")          # qf_stream_read writes one word per block, index modulo 4096
    reps = max(64, 2 * n)

    def launches():
        for i in range(reps):
            native.stream_read(bufs[i % n], sink)

    launches()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        launches()
    torch.cuda.current_stream().wait_stream(side)
    warm_replays(graph)
    times = []
    for _ in range(5):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) * 1e3 / reps)
    times.sort()
    return times[len(times) // 2]


def _graph_time_us(launches, reps):
    """`launches()` enqueues `reps` back-to-back launches; they are captured in a HIP graph, the replay is timed with
    HIP events on the launch stream (median of five), and the time per launch is returned."""
    import torch
    launches()
    torch.cuda.synchronize()
    graph, side = torch.cuda.CUDAGraph(), torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side), torch.cuda.graph(graph, stream=side):
        launches()
    torch.cuda.current_stream().wait_stream(side)
    warm_replays(graph)
    times = []
    for _ in range(5):
        start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        start.record()
        graph.replay()
        end.record()
        torch.cuda.synchronize()
        times.append(start.elapsed_time(end) * 1e3 / reps)
    times.sort()
    return times[len(times) // 2]


def launch_floor_report():
    """What a launch costs before it does any work, and what a pure streaming read of a given size reaches, both timed
    like the kernels (back-to-back launches in a HIP graph): a kernel that does nothing at several grid sizes, and
    qf_stream_read at the footprints of the benchmark shapes.  The gap between a GEMV and 8 TB/s that is not the
    kernel's own is read off these."""
    from qfactory import native
    report = {"empty_kernel_us": [], "stream_read": []}
    for blocks, threads in ((1, 64), (256, 64), (256, 256), (1024, 256), (2752, 256), (4096, 256), (11008, 64), (16384, 256)):
        us = _graph_time_us(lambda: [native.empty_launch(blocks, threads) for _ in range(64)], 64)
        report["empty_kernel_us"].append({"blocks": blocks, "threads": threads, "us": round(us, 3)})
        log(f"[bench] empty kernel {blocks:6d} x {threads:4d}: {us:6.2f} us per launch")
    sizes = [(f"{name} M=1", algorithmic_bytes(1, N, K)) for name, N, K in SHAPES + GEMM_SHAPES]
    sizes += [("1 MiB", 1 << 20), ("4 MiB", 4 << 20), ("512 MiB", 512 << 20)]
    for what, nbytes in sizes:
        us = stream_read_time_us(nbytes)
        report["stream_read"].append({"what": what, "bytes": int(nbytes), "us": round(us, 3),
                                      "GB/s": round(nbytes / us / 1e3, 1), "frac_of_8TB/s": round(nbytes / us / 1e3 / HBM_PEAK_GBPS, 4)})
        log(f"[bench] stream read {what:18s} {int(nbytes):10d} B: {us:8.2f} us  {nbytes / us / 1e3:7.1f} GB/s")
    return report


def dense_square_tflops(n=8192, reps=10):
    """A large square dense fp16 GEMM of the vendor library (torch.matmul): the matrix-core ceiling this machine
    gives a well-shaped problem.  Same timing protocol as the kernels (graph, warm replays, HIP events)."""
    import torch
    a = torch.randn(n, n, device="cuda", dtype=torch.float16)
    b = torch.randn(n, n, device="cuda", dtype=torch.float16)
    out = torch.empty(n, n, device="cuda", dtype=torch.float16)
    us = _graph_time_us(lambda: [torch.matmul(a, b, out=out) for _ in range(reps)], reps)
    return 2.0 * n ** 3 / us / 1e6


def module_time_us(lins, x, reps=256, out=None):
    """Average time of one eager ``layer(x)`` call -- output allocation, Python checks, ctypes and the launch, as the
    reference's latency harness times it (qfactory/testing.py:31-35) -- rotating over the layers' weight copies;
    wall clock around `reps` calls with a synchronisation on both sides.  At small M this is bound by the host
    (the kernel is shorter than its enqueue), which is why the decode loop replays HIP graphs.  With ``out``: the
    same through ``layer.forward(x, out=out)``, i.e. without the allocator."""
    import torch
    call = (lambda lin: lin(x)) if out is None else (lambda lin: lin.forward(x, out=out))
    for i in range(16):
        call(lins[i % len(lins)])
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    for i in range(reps):
        call(lins[i % len(lins)])
    torch.cuda.synchronize()
    return (time.perf_counter() - t0) / reps * 1e6


def dense_fp16_time_us(M, N, K, total_bytes=COLD_BYTES, reps=None):
    """The vendor library's dense fp16 GEMM of the same shape (torch.matmul on hipBLASLt / rocBLAS), cold
    weights: the comparison the reference's own evaluation makes against cuBLAS
    (qfactory/testing.py:36-41).  A reported yardstick, not part of the path.  Timed exactly like the project's
    kernels: back-to-back launches in one HIP graph, WARM_MS of untimed replays first, HIP events on the launch
    stream, median of five."""
    import torch
    n = max(2, -(-int(total_bytes) // (N * K * 2)))
    ws = [torch.randn(N, K, device="cuda", dtype=torch.float16) for _ in range(n)]
    x = torch.randn(M, K, device="cuda", dtype=torch.float16)
    out = torch.empty(M, N, device="cuda", dtype=torch.float16)
    reps = reps or max(64, 2 * n)

    def launches():
        for i in range(reps):
            torch.matmul(x, ws[i % n].T, out=out)

    return _graph_time_us(launches, reps)


def gemm_report(M=256, shapes=None, reps=None):
    """BASELINE.json configs[3]: W4A16 g128 GEMM on Llama-3-70B-style shapes, per shape microseconds, TFLOP/s,
    the fraction of the dense fp16 MFMA peak and of the HBM peak (M <= 64 is HBM-bound by arithmetic intensity).
    With ``shapes`` / ``reps``: the same report on other layers (the prefill section: launches of a millisecond
    need no 64 per graph to reach the sustained clock)."""
    import torch
    from qfactory import QLinear
    flags = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
    g = torch.Generator(device="cuda").manual_seed(1)
    report = []
    for name, N, K in (shapes or GEMM_SHAPES):
        lin = QLinear.empty(M, K, N, NBITS, GS, sym=False, compile_flags=flags)
        sets = weight_sets(lin, cold_copies(N * K // 2), g)
        x = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
        us = kernel_event_time_us(lin.func, sets, x, N, reps=reps)
        description = lin.func.runtime.description
        del lin, sets
        torch.cuda.empty_cache()
        dense_us = dense_fp16_time_us(M, N, K, reps=reps)
        flops = 2.0 * M * N * K
        rec = {"name": name, "N": N, "K": K, "M": M, "us": round(us, 2), "TFLOP/s": round(flops / us / 1e6, 1),
               "mfma_frac": round(flops / us / 1e6 / MFMA_F16_PEAK_TFLOPS, 4),
               "GB/s": round(algorithmic_bytes(M, N, K) / us / 1e3, 1),
               "hbm_frac": round(algorithmic_bytes(M, N, K) / us / 1e3 / HBM_PEAK_GBPS, 4),
               "dense_fp16_us": round(dense_us, 2), "speedup_over_dense_fp16": round(dense_us / us, 3),
               "kernel": description}
        report.append(rec)
        log(f"[bench] GEMM M={M} {name:11s} N={N:6d} K={K:6d} {us:8.2f} us {rec['TFLOP/s']:7.1f} TFLOP/s "
            f"{100 * rec['mfma_frac']:5.1f}% of fp16 MFMA peak, {100 * rec['hbm_frac']:5.1f}% of HBM peak; "
            f"dense fp16 torch.matmul {dense_us:8.2f} us (x{rec['speedup_over_dense_fp16']:.2f})")
    return report


COPY_BYTES = 64 << 20

# HBM traffic per launch of the dominant kernel, from hardware counters: rocprofv3 --pmc FETCH_SIZE
# and --pmc WRITE_SIZE over `bench.py --counter-pass`, each scaled by what the same counter reads
# for the 64 MiB stream copy of that run (which moves COPY_BYTES each way).  A stored measurement:
# keyed by the description of the specialisation it was taken on, reported with that key, and null
# for any other specialisation (profiles/gemv_w4g128_llama2_7b_m1_hbm_traffic_pmc.md holds the run).
MEASURED_TRAFFIC = {
    "regime=gemv M=1 N=22016 K=4096 NBITS=4 GS=128 SYM=0 decode=deferred nt_b=1 MT=1 STEPS=1 U=4 VB=16 WK=2 WN=2 "
    "QF_FUSED_AND_OR=2 QF_GEMV_QUANT_DEDUP=1": 47041000,
}


def counter_pass(layers, acts, reps=5):
    import torch
    from qfactory import native
    src = torch.randint(-128, 128, (COPY_BYTES,), dtype=torch.int8, device="cuda")
    dst = torch.empty_like(src)
    torch.cuda.synchronize()
    for r in range(reps):
        for name, N, K in SHAPES:
            layers[r % len(layers)][name](acts[K])
        native.stream_copy(dst, src)
    torch.cuda.synchronize()
    assert torch.equal(dst, src)
    log(f"[bench] counter pass: {reps} launches of each kernel and of a {COPY_BYTES} byte stream copy")


def counter_pass_matrix(reps=3):
    """The launches of the matrix-core kernels to put under `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`: the
    A-stationary kernel (gate_up at M = 16; down at M = 16 and the 8192 x 8192 projection at M = 16 with their rows
    split over four and two blocks), the GEMM kernel on the four Llama-3-70B shapes at M = 256 and on the Llama-2-7B
    qkv and gate_up layers at 8192 rows, each `reps` times over two weight copies, and the 64 MiB stream copy that
    scales the counters."""
    import torch
    from qfactory import native
    src = torch.randint(-128, 128, (COPY_BYTES,), dtype=torch.int8, device="cuda")
    dst = torch.empty_like(src)
    problems = [(16, 22016, 4096), (16, 4096, 11008), (16, 8192, 8192)] + [(256, N, K) for _, N, K in GEMM_SHAPES] + [(8192, 12288, 4096), (8192, 22016, 4096)]
    for M, N, K in problems:
        lin, sets, x = _timed_problem(M, N, K, NBITS, False, copies=2)
        out = torch.empty(M, N, dtype=torch.float16, device="cuda")
        torch.cuda.synchronize()
        for r in range(reps):
            w, s_, z = sets[r % len(sets)]
            assert lin.func(x, w, out, s_, z) == 0
            native.stream_copy(dst, src)
        torch.cuda.synchronize()
        log(f"[bench] counter pass: {reps} launches of {lin.func.runtime.description}")
        del lin, sets, x, out
        torch.cuda.empty_cache()
    assert torch.equal(dst, src)


def _timed_problem(M, N, K, nbits, sym, copies=None):
    """One QLinear of the problem plus enough random packed-tensor sets to defeat the caches (>= 512 MB)."""
    import torch
    from qfactory import QLinear
    flags = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
    g = torch.Generator(device="cuda").manual_seed(2)
    lin = QLinear.empty(M, K, N, nbits, GS, sym=sym, compile_flags=flags)
    sets = weight_sets(lin, copies or cold_copies(N * K * nbits // 8), g)
    x = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
    return lin, sets, x


def small_m_report():
    """BASELINE.json configs[1] at M in {4, 16}, configs[2] (N = K = 8192, M in {1, 16}, 2/3/4/8-bit,
    symmetric and asymmetric) and the Llama-3-70B shapes at M = 1: per shape microseconds and the fraction
    of the 8 TB/s HBM roofline."""
    import torch
    report = []

    def one(tag, M, N, K, nbits, sym):
        lin, sets, x = _timed_problem(M, N, K, nbits, sym)
        us = kernel_event_time_us(lin.func, sets, x, N)
        b = algorithmic_bytes(M, N, K, nbits, GS, sym)
        rec = {"config": tag, "M": M, "N": N, "K": K, "bits": nbits, "sym": sym, "us": round(us, 3),
               "GB/s": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 4),
               "TFLOP/s": round(2.0 * M * N * K / us / 1e6, 2), "kernel": lin.func.runtime.description}
        report.append(rec)
        log(f"[bench] {tag} M={M:3d} N={N:6d} K={K:6d} b={nbits} {'sym ' if sym else 'asym'} {us:8.2f} us "
            f"{rec['GB/s']:7.1f} GB/s {100 * rec['hbm_frac']:5.1f}% of HBM peak")
        del lin, sets
        torch.cuda.empty_cache()

    for M in (4, 16):
        for name, N, K in SHAPES:
            one("configs[1]", M, N, K, NBITS, False)
    for M in (1, 16):
        for nbits in (2, 3, 4, 8):
            for sym in (False, True):
                one("configs[2]", M, 8192, 8192, nbits, sym)
    # the 28672-wide end of the "4096 - 28672-wide LLM shapes" the GEMV target names: Llama-3-70B at M = 1
    for name, N, K in GEMM_SHAPES:
        one("70b-gemv", 1, N, K, NBITS, False)
    for name, N, K in GEMM_SHAPES:                         # ... and at sixteen rows: K = 8192 and 28672 split over blocks
        one("70b-m16", 16, N, K, NBITS, False)
    return report


def ablation_report():
    """Where the time of a launch goes: per kernel family, the product's object beside timing builds of the same
    tiling that leave one part out (`prebuild.ABLATIONS`: the headers' `QF_*_EXPERIMENT` knobs; their results are wrong
    by design and nothing but this mode compiles them), and a pure streaming read of the same bytes.  Cold weights,
    timed like every other kernel here."""
    import torch
    import prebuild
    from qfactory.jit import jit
    report = []
    for M, N, K in prebuild.ABLATION_PROBLEMS:
        op, regime, builds = prebuild.ablation_builds(M, N, K)
        lin, sets, x = _timed_problem(M, N, K, NBITS, False)
        rows = []
        for bits, label, obj in builds:
            func = op._wrap(jit.compile(obj), builds[0][2])
            us = kernel_event_time_us(func, sets, x, N)
            rows.append({"knob": bits, "what": label, "us": round(us, 3)})
            log(f"[bench] ablation M={M:4d} N={N:6d} K={K:6d} {regime:6s} knob {bits:3d} {us:9.2f} us  {label}")
        read_us = stream_read_time_us(algorithmic_bytes(M, N, K) - 2 * M * (N + K))
        log(f"[bench] ablation M={M:4d} N={N:6d} K={K:6d} read of the packed tensors {read_us:9.2f} us")
        report.append({"M": M, "N": N, "K": K, "regime": regime, "kernel": lin.func.runtime.description,
                       "builds": rows, "read_of_the_packed_tensors_us": round(read_us, 3)})
        del lin, sets, x
        torch.cuda.empty_cache()
    return report


def shape_set_problems():
    """The reference's bandwidth and speed-up experiments as (figure, M, N, K, bits, group size) problems:
    fig 9 (reproduce/fig9/plot_bandwidth_size.py:12,32-33: `squares-pure`, M = 1, W4 with and without groups),
    fig 10 (reproduce/fig10/plot_bandwidth_bits.py:28-30: `squares-pure`, M = 1, 8 / 4 / 2 bits g128),
    fig 6 (reproduce/fig6/bench_kernels.py:24-30: `operator`, M = 1, 8 / 4 / 2 bits g128) and
    table 3 (reproduce/tab3/bench_kernels.py:25-33: `operator`, W4 g128 at M = 1 / 2 / 4)."""
    with open(os.path.join(ROOT, "tests", "golden", "nkg_shapes.json")) as f:
        sets = json.load(f)
    problems, seen = [], set()

    def add(fig, M, N, K, bits, gs):
        key = (M, N, K, bits, gs)
        entry = next((p for p in problems if p["key"] == key), None)
        if entry is None:
            entry = {"key": key, "figures": [], "M": M, "N": N, "K": K, "bits": bits, "GS": gs}
            problems.append(entry)
        if fig not in entry["figures"]:
            entry["figures"].append(fig)

    for N, K, _ in sets["squares-pure"]:
        add("fig9", 1, N, K, 4, 128)
        add("fig9", 1, N, K, 4, -1)
        for bits in (8, 4, 2):
            add("fig10", 1, N, K, bits, 128)
    for N, K, _ in sets["operator"]:
        for bits in (8, 4, 2):
            add("fig6", 1, N, K, bits, 128)
        for M in (1, 2, 4):
            add("tab3", M, N, K, 4, 128)
    return problems


def footprint(M, N, K, bits, gs):
    """reproduce/fig9/plot_bandwidth_size.py:37-44 (`get_memory_footprint`); bits == 16: the dense fp16 GEMM."""
    if bits == 16:
        return (M * K + K * N + M * N) * 2
    if gs == -1:
        return (M * K + M * N) * 2 + K * N * bits / 8
    return (M * K + M * N) * 2 + K * N * (bits / 8 + (2 + bits / 8) / gs)


def shape_sets_report():
    """Kernel time, achieved bandwidth by the reference's footprint formula and speed-up over the vendor's dense fp16
    GEMM for every problem of `shape_set_problems`, cold weights, timed like every other section."""
    import torch
    from qfactory import QLinear
    flags = {"enable_transform": False, "enable_schedule": False, "enable_lower": False}
    g = torch.Generator(device="cuda").manual_seed(4)
    rows, dense = [], {}
    for prob in shape_set_problems():
        M, N, K, bits, gs = prob["key"]
        if (M, N, K) not in dense:
            dense[(M, N, K)] = dense_fp16_time_us(M, N, K)
            torch.cuda.empty_cache()
        try:
            lin = QLinear.empty(M, K, N, bits, gs, sym=False, compile_flags=flags)
        except Exception as exc:                        # a shape a kernel family rejects is reported, not hidden
            rows.append({**{k: prob[k] for k in ("figures", "M", "N", "K", "bits", "GS")}, "error": str(exc)[:200]})
            log(f"[bench] shape sets: M={M} N={N} K={K} b={bits} GS={gs}: {exc}")
            continue
        x = torch.randn(M, K, device="cuda", generator=g).to(torch.float16)
        if gs == -1:
            n_copies = cold_copies(N * K * bits // 8)
            ws = [torch.randint(-128, 128, lin.w.shape, dtype=torch.int8, device="cuda", generator=g) for _ in range(n_copies)]
            func = lin.func_for(torch.float16)
            us = kernel_event_time_us(lambda a, w, out, s, z=None: func(a, w, out), [(w, None, None) for w in ws], x, N)
            del ws
        else:
            sets = weight_sets(lin, cold_copies(N * K * bits // 8), g)
            us = kernel_event_time_us(lin.func, sets, x, N)
            del sets
        b = footprint(M, N, K, bits, gs)
        d_us = dense[(M, N, K)]
        rows.append({"figures": prob["figures"], "M": M, "N": N, "K": K, "bits": bits, "GS": gs, "us": round(us, 3),
                     "GB/s": round(b / us / 1e3, 1), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 4),
                     "dense_fp16_us": round(d_us, 3), "dense_fp16_GB/s": round(footprint(M, N, K, 16, -1) / d_us / 1e3, 1),
                     "speedup_over_dense_fp16": round(d_us / us, 3)})
        log(f"[bench] shape sets {'/'.join(prob['figures']):12s} M={M} N={N:6d} K={K:6d} b={bits} GS={gs:4d} {us:9.2f} us "
            f"{rows[-1]['GB/s']:8.1f} GB/s  dense fp16 {d_us:9.2f} us (x{rows[-1]['speedup_over_dense_fp16']:.2f})")
        del lin
        torch.cuda.empty_cache()

    def geomean(values):
        values = [v for v in values if v > 0]
        prod = 1.0
        for v in values:
            prod *= v
        return round(prod ** (1.0 / len(values)), 3) if values else None

    ok = [r for r in rows if "us" in r]
    summary = {
        "what": "speed-up over the vendor's dense fp16 GEMM (geometric mean, as reproduce/tab3/bench_kernels.py:36-47 and "
                "reproduce/fig6/bench_kernels.py:54-59 form it) and achieved bandwidth by the reference's footprint formula",
        "tab3_geomean_speedup_by_M": {str(M): geomean([r["speedup_over_dense_fp16"] for r in ok if "tab3" in r["figures"] and r["M"] == M])
                                      for M in (1, 2, 4)},
        "fig6_geomean_speedup_by_bits": {str(b): geomean([r["speedup_over_dense_fp16"] for r in ok if "fig6" in r["figures"] and r["bits"] == b])
                                         for b in (8, 4, 2)},
        "fig9_GB/s_by_size": [{"N": r["N"], "K": r["K"], "GS": r["GS"], "GB/s": r["GB/s"]} for r in ok if "fig9" in r["figures"]],
        "fig10_GB/s_by_bits": [{"N": r["N"], "bits": r["bits"], "GB/s": r["GB/s"]} for r in ok if "fig10" in r["figures"]],
        "problems": len(rows), "rejected": len(rows) - len(ok),
    }
    return {"summary": summary, "rows": rows}


def decode_report(batches=(1, 16, 64), prompt_len=128, new_tokens=128):
    """BASELINE.json configs[4]: the Llama-2-7B-shaped greedy decode loop (32 layers, every linear a W4A16 g128
    QLinear, random weights and prompt ids): tokens/s and the share of a decode step spent in the quantized
    linears, per batch size (qfactory-ae_amd/decode_llama.py)."""
    import torch
    import decode_llama
    shape = decode_llama.LlamaShape(max_len=prompt_len + new_tokens)
    report = []
    for batch in batches:
        rec = decode_llama.run(shape, batch, prompt_len, new_tokens)
        report.append(rec)
        log(f"[bench] decode batch={batch:3d}: {rec['value']:9.1f} tokens/s, step {rec['decode_step_us']:8.1f} us, "
            f"quantized linears {rec['quantized_linears_us_per_step']:8.1f} us ({100 * rec['quantized_linear_share']:.0f}%), "
            f"prefill {rec['prefill_tokens_per_s']:9.1f} tokens/s")
        torch.cuda.empty_cache()
    return report


def cpu_model_string():
    try:
        with open("/proc/cpuinfo") as f:
            for line in f:
                if line.lower().startswith("model name"):
                    return line.split(":", 1)[1].strip()
    except OSError:
        pass
    import platform
    return platform.processor() or platform.machine()


def cpu_baseline(budget_s=16.0, gpu_us=None):
    """The reference's test path (tests/acc_gptq.py:31-38,52; tests/acc_gemv.py:12-14) as a torch-CPU port on this
    machine's host cores, over the same four shapes at M = 1, bounded to about `budget_s`: per shape two timings,
    "dequant + matmul" (unpack the packed tensors, dequantise to fp16, fp32 matmul) and "matmul only" (the fp32
    matmul on weights dequantised beforehand), median of the timed iterations after one warm-up.  `value` is the
    algorithmic bytes of one pass over the four shapes divided by the dequant + matmul time of that pass."""
    import torch
    from oracle import qf_oracle
    g = torch.Generator().manual_seed(0)
    rows = []
    per_shape_budget = budget_s / len(SHAPES)
    for name, N, K in SHAPES:
        w = torch.randint(-128, 128, (N, K * NBITS // 8), dtype=torch.int8, generator=g)
        s = (torch.rand(N, K // GS, generator=g) * 0.019 + 0.001).to(torch.float16)
        z = torch.randint(-128, 128, (N, K // GS * NBITS // 8), dtype=torch.int8, generator=g)
        A = torch.randn(1, K, generator=g).to(torch.float16)

        def full():
            return qf_oracle.torch_cpu_forward(A, w, s, z, NBITS, GS)

        dq32 = qf_oracle.torch_cpu_dequant(w, s, z, NBITS, GS).to(torch.float32)
        a32 = A.to(torch.float32)

        def matmul_only():
            return (a32 @ dq32.T).to(torch.float16)

        def median_time(fn, budget):
            fn()                                        # warm-up
            times = []
            t_end = time.perf_counter() + budget
            while len(times) < 5 or (time.perf_counter() < t_end and len(times) < 50):
                t0 = time.perf_counter()
                fn()
                times.append(time.perf_counter() - t0)
            times.sort()
            return times[len(times) // 2], times[0], len(times)

        full_med, full_min, n_full = median_time(full, 0.8 * per_shape_budget)
        mm_med, mm_min, n_mm = median_time(matmul_only, 0.2 * per_shape_budget)
        row = {"name": name, "N": N, "K": K, "M": 1, "dequant_matmul_us": round(full_med * 1e6, 1),
               "dequant_matmul_min_us": round(full_min * 1e6, 1), "matmul_only_us": round(mm_med * 1e6, 1),
               "matmul_only_min_us": round(mm_min * 1e6, 1), "iterations": [n_full, n_mm],
               "GB/s": round(algorithmic_bytes(1, N, K) / full_med / 1e9, 3)}
        if gpu_us and name in gpu_us:
            row["gpu_kernel_us"] = gpu_us[name]
            row["gpu_over_cpu"] = round(full_med * 1e6 / gpu_us[name], 1)
        rows.append(row)
        log(f"[bench] cpu {name:8s} dequant + matmul {full_med * 1e3:8.2f} ms (min {full_min * 1e3:.2f}, {n_full} iterations), "
            f"matmul only {mm_med * 1e3:8.2f} ms (min {mm_min * 1e3:.2f}, {n_mm} iterations)")
        del dq32
    total_bytes = sum(algorithmic_bytes(1, N, K) for _, N, K in SHAPES)
    full_s = sum(r["dequant_matmul_us"] for r in rows) * 1e-6
    mm_s = sum(r["matmul_only_us"] for r in rows) * 1e-6
    return {"value": round(total_bytes / full_s / 1e9, 4), "unit": "GB/s", "cores": torch.get_num_threads(), "kind": "port",
            "sample": f"the 4 Llama-2-7B W4A16 g128 shapes at M=1, {rows[0]['iterations'][0]}+ iterations each after a warm-up, "
                      "torch CPU unpack + fp16 dequant + fp32 matmul (median)",
            "dequant_matmul_ms": round(full_s * 1e3, 2), "matmul_only_ms": round(mm_s * 1e3, 2),
            "matmul_only_GB/s": round(total_bytes / mm_s / 1e9, 3),
            "cpu_model": cpu_model_string(), "host_cpus": os.cpu_count(), "shapes": rows}


def compact_line(full):
    """The one JSON object printed on stdout: the headline, the roofline of the dominant kernel, a few numbers per
    section and the CPU baseline -- small enough to survive any log tail (under 4 kB).  Everything else (per-shape
    records, kernel descriptions, the small-M / GEMM / prefill tables) is in the full report, which goes to stderr
    and to a side file."""
    line = {k: full[k] for k in ("metric", "value", "unit", "n_gpus", "steps", "warmup", "ms_per_step", "higher_is_better",
                                 "scaling", "vs_baseline", "dtype", "data", "config", "hbm_frac_whole_step")}
    roof = full["roofline"]
    line["roofline"] = {k: roof[k] for k in ("bound", "achieved", "peak", "unit", "frac", "traffic", "kernel", "avg_launch_us",
                                             "algorithmic_bytes_per_launch")}
    line["roofline"]["empirical"] = {k: roof["empirical"][k] for k in ("stream_read_GB/s", "stream_read_us", "frac_of_stream_read",
                                                                       "dense_fp16_TFLOP/s")}
    line["shapes"] = [{"name": r["name"], "us": r["us"], "hbm_frac": r["hbm_frac"], "stream_read_us": r["stream_read_us"]}
                      for r in full["shapes"]]
    line["parity"] = {k: float(f"{v:.3g}") for k, v in full["parity"].items()}
    if "gemm_m256" in full:
        line["gemm_m256"] = [{"name": r["name"], "us": r["us"], "mfma_frac": r["mfma_frac"], "dense_fp16_us": r["dense_fp16_us"]}
                             for r in full["gemm_m256"]["shapes"]]
    if "small_m" in full:
        line["small_m16"] = [{"N": r["N"], "K": r["K"], "bits": r["bits"], "us": r["us"], "hbm_frac": r["hbm_frac"]}
                             for r in full["small_m"] if r["M"] == 16 and not r["sym"]]
    if "decode" in full:
        line["decode"] = [{"batch": r["batch"], "tokens_per_s": round(r["value"], 1), "step_us": round(r["decode_step_us"], 1),
                           "linear_share": round(r["quantized_linear_share"], 3)} for r in full["decode"]]
    if "cpu_baseline" in full:
        cb = full["cpu_baseline"]
        line["cpu_baseline"] = {k: cb[k] for k in ("value", "unit", "cores", "kind", "sample", "dequant_matmul_ms",
                                                   "matmul_only_ms", "cpu_model", "host_cpus")}
    if "report_file" in full:
        line["report_file"] = full["report_file"]
    return line


def write_report(full):
    """The full report as a side file (gpurun_out/bench_report.json when that directory can be made) and on stderr."""
    text = json.dumps(full, indent=1)
    log("[bench] full report:")
    log(text)
    try:
        out_dir = os.path.join(ROOT, "gpurun_out")
        os.makedirs(out_dir, exist_ok=True)
        path = os.path.join(out_dir, "bench_report.json")
        with open(path, "w") as f:
            f.write(text + "\n")
        return os.path.relpath(path, ROOT)
    except OSError as exc:
        log(f"[bench] could not write the side file: {exc}")
        return None


def main():
    ap = argparse.ArgumentParser()
    ap.add_argument("--gpus", type=int, default=1)
    ap.add_argument("--steps", type=int, default=256)
    ap.add_argument("--warmup", type=int, default=32)
    ap.add_argument("--layers", type=int, default=8, help="distinct resident weight copies cycled through")
    ap.add_argument("--no-cpu-baseline", action="store_true")
    ap.add_argument("--no-gemm", action="store_true", help="skip the M=256 GEMM report")
    ap.add_argument("--no-module-time", action="store_true",
                    help="skip the eager layer(x) timing (its launches would mix into a kernel trace's averages)")
    ap.add_argument("--small-m", action="store_true", help="accepted for compatibility: the small-M report is on by default")
    ap.add_argument("--no-small-m", action="store_true",
                    help="skip configs[1] at M = 4, 16, the configs[2] bit-width sweep and the 70B shapes at M = 1")
    ap.add_argument("--no-decode", action="store_true", help="skip the configs[4] decode loop")
    ap.add_argument("--no-graph", action="store_true", help="enqueue the timed steps eagerly from Python")
    ap.add_argument("--launch-floor", action="store_true",
                    help="only measure the launch floor (a kernel that does nothing, several grids) and the streaming-read "
                         "ceiling at the benchmark footprints; prints one JSON object")
    ap.add_argument("--counter-pass", action="store_true",
                    help="only launch each of the four kernels (cold weights) and a 64 MiB stream copy a few times, "
                         "eagerly: the run to put under `rocprofv3 --pmc FETCH_SIZE` / `--pmc WRITE_SIZE`")
    ap.add_argument("--counter-pass-matrix", action="store_true",
                    help="the same for the matrix-core kernels: gate_up and down at M = 16, the four GEMMs at M = 256, qkv and "
                         "gate_up at 8192 rows")
    ap.add_argument("--ablation", action="store_true",
                    help="only the phase ablation: each kernel family's object beside timing builds that leave one part "
                         "out, on the 7B layers at M = 1 and 16 and three GEMM problems; prints one JSON object")
    ap.add_argument("--shape-sets", action="store_true",
                    help="only the reference's bandwidth tables: its `squares` and `operator` shape sets at M in {1, 2, 4}, "
                         "8 / 4 / 2 bits, with and without groups; prints one JSON object, writes gpurun_out/shape_sets.json")
    args = ap.parse_args()
    if args.gpus != 1:
        sys.exit("bench.py measures one GPU's share of the path; this build runs on exactly one GPU (--gpus 1)")

    import torch
    assert torch.cuda.is_available(), "bench.py needs the MI355X"
    torch.cuda.set_device(0)
    if args.launch_floor:
        print(json.dumps({"launch_floor": launch_floor_report()}), flush=True)
        return
    if args.counter_pass_matrix:
        counter_pass_matrix()
        return
    if args.ablation:
        print(json.dumps({"ablation": ablation_report()}), flush=True)
        return
    if args.shape_sets:
        report = shape_sets_report()
        try:
            os.makedirs(os.path.join(ROOT, "gpurun_out"), exist_ok=True)
            with open(os.path.join(ROOT, "gpurun_out", "shape_sets.json"), "w") as f:
                json.dump(report, f, indent=1)
        except OSError as exc:
            log(f"[bench] could not write the side file: {exc}")
        print(json.dumps(report["summary"]), flush=True)
        return
    M = 1
    layers, acts = build_layers(args.layers, M)
    parity = check_against_oracle(layers[0], acts)
    log(f"[bench] parity of benchmark data vs oracle: {parity}")

    step_bytes = sum(algorithmic_bytes(M, N, K) for _, N, K in SHAPES)

    if args.counter_pass:
        counter_pass(layers, acts)
        return
    dominant_kernel = layers[0][DOMINANT].func.runtime.description
    if dominant_kernel not in MEASURED_TRAFFIC:
        sys.exit(f"bench.py: MEASURED_TRAFFIC holds no counter measurement for the dominant kernel as it is built now "
                 f"({dominant_kernel!r}): rerun the two rocprofv3 --pmc passes over `bench.py --counter-pass` and store "
                 "the scaled FETCH_SIZE + WRITE_SIZE figure under this description")

    for i in range(args.warmup):
        run_step(layers[i % len(layers)], acts)
    torch.cuda.synchronize()

    if args.no_graph:
        torch.cuda.synchronize()
        t0 = time.perf_counter()
        for i in range(args.steps):
            run_step(layers[i % len(layers)], acts)
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    else:
        graph = torch.cuda.CUDAGraph()
        side = torch.cuda.Stream()
        side.wait_stream(torch.cuda.current_stream())
        with torch.cuda.stream(side):
            with torch.cuda.graph(graph, stream=side):
                for i in range(args.steps):
                    run_step(layers[i % len(layers)], acts)
        torch.cuda.current_stream().wait_stream(side)
        torch.cuda.synchronize()
        warm_replays(graph)                              # untimed: uploads the graph, brings the GPU to its sustained state
        t0 = time.perf_counter()
        graph.replay()
        torch.cuda.synchronize()
        elapsed = time.perf_counter() - t0
    ms_per_step = elapsed / args.steps * 1e3
    value = step_bytes / (elapsed / args.steps) / 1e9

    # per-kernel durations (HIP events on the launch stream), cold weights: >= 512 MB of distinct packed tensors each
    shapes_report = []
    dominant = None
    g = torch.Generator(device="cuda").manual_seed(3)
    for name, N, K in SHAPES:
        lin = layers[0][name]
        sets = weight_sets(lin, cold_copies(N * K // 2), g)
        us = kernel_event_time_us(lin.func, sets, acts[K], N)
        del sets
        torch.cuda.empty_cache()
        b = algorithmic_bytes(M, N, K)
        rec = {"name": name, "N": N, "K": K, "M": M, "us": round(us, 3), "GB/s": round(b / us / 1e3, 1),
               "TFLOP/s": round(2 * M * N * K / us / 1e6, 3), "hbm_frac": round(b / us / 1e3 / HBM_PEAK_GBPS, 4),
               "bytes": int(b), "kernel": lin.func.runtime.description}
        stream_us = stream_read_time_us(b)
        rec["stream_read_us"] = round(stream_us, 3)
        rec["frac_of_stream_read"] = round(stream_us / us, 4)
        if not args.no_module_time:
            rec["module_us"] = round(module_time_us([layer[name] for layer in layers], acts[K]), 2)
            rec["module_out_us"] = round(module_time_us([layer[name] for layer in layers], acts[K],
                                                        out=torch.empty(M, N, dtype=torch.float16, device="cuda")), 2)
        shapes_report.append(rec)
        log(f"[bench] {name:8s} N={N:6d} K={K:6d}  {us:7.2f} us  {rec['GB/s']:7.1f} GB/s  {100 * rec['hbm_frac']:5.1f}% of HBM peak"
            f"  (a pure streaming read of the same bytes: {stream_us:.2f} us)"
            + (f"  (eager layer(x): {rec['module_us']:.2f} us per call, forward(x, out=...): {rec['module_out_us']:.2f})" if "module_us" in rec else ""))
        if name == DOMINANT:
            dominant = rec
    dense_tflops = dense_square_tflops()
    log(f"[bench] ceilings measured here: streaming read of {dominant['bytes']} bytes {dominant['bytes'] / dominant['stream_read_us'] / 1e3:.1f} GB/s, "
        f"dense fp16 8192^3 torch.matmul {dense_tflops:.1f} TFLOP/s")

    result = {
        "metric": "W4A16 g128 GEMV (M=1) algorithmic HBM throughput over the Llama-2-7B linear shapes",
        "value": round(value, 1), "unit": "GB/s", "n_gpus": 1, "steps": args.steps, "warmup": args.warmup,
        "ms_per_step": round(ms_per_step, 5), "higher_is_better": True, "scaling": "weak", "vs_baseline": None,
        "dtype": "f16", "data": "synthetic",
        "config": {"workload": "configs[1] at M=1: W4A16 g128 asymmetric GEMV over Llama-2-7B shapes "
                               "(12288x4096, 4096x4096, 22016x4096, 4096x11008), one step = the four linears of one layer",
                   "bits": NBITS, "group_size": GS, "M": M, "weight_copies": args.layers,
                   "bytes_per_step": int(step_bytes), "timed_with": "eager" if args.no_graph else "one HIP graph of all steps"},
        "hbm_frac_whole_step": round(value / HBM_PEAK_GBPS, 4),
        "roofline": {"bound": "hbm", "achieved": dominant["GB/s"], "peak": HBM_PEAK_GBPS, "unit": "GB/s",
                     "frac": round(dominant["GB/s"] / HBM_PEAK_GBPS, 4),
                     "traffic": MEASURED_TRAFFIC[dominant["kernel"]],
                     "traffic_source": "stored rocprofv3 --pmc FETCH_SIZE + WRITE_SIZE measurement of this specialisation",
                     "kernel": f"qf::gemv_kernel {DOMINANT} N=22016 K=4096 M=1", "avg_launch_us": dominant["us"],
                     "algorithmic_bytes_per_launch": dominant["bytes"],
                     "empirical": {"stream_read_GB/s": round(dominant["bytes"] / dominant["stream_read_us"] / 1e3, 1),
                                   "stream_read_us": dominant["stream_read_us"],
                                   "frac_of_stream_read": dominant["frac_of_stream_read"],
                                   "what": "qf_stream_read of the same number of cold bytes, timed like the kernel",
                                   "dense_fp16_TFLOP/s": round(dense_tflops, 1),
                                   "dense_fp16_what": "torch.matmul 8192 x 8192 x 8192 (vendor library), hot operands"}},
        "shapes": shapes_report,
        "parity": parity,
    }
    if not args.no_gemm:
        result["gemm_m256"] = {"peak_TFLOP/s": MFMA_F16_PEAK_TFLOPS, "dense_fp16_TFLOP/s_measured": round(dense_tflops, 1),
                               "shapes": gemm_report(256)}
        result["gemm_m32_m64_m128"] = [rec for m_rows in (32, 64, 128) for rec in gemm_report(m_rows)]
        # configs[4]'s prefill: 64 sequences x 128 prompt tokens through the Llama-2-7B layers
        result["gemm_prefill_m8192"] = gemm_report(8192, shapes=SHAPES, reps=16)
    if not args.no_small_m:
        result["small_m"] = small_m_report()
    if not args.no_decode:
        del layers
        torch.cuda.empty_cache()
        result["decode"] = decode_report()
    if not args.no_cpu_baseline:
        result["cpu_baseline"] = cpu_baseline(gpu_us={r["name"]: r["us"] for r in shapes_report})
    path = write_report(result)
    if path:
        result["report_file"] = path
    print(json.dumps(compact_line(result), separators=(",", ":")), flush=True)


if __name__ == "__main__":
    main()
