"""Device-side timing of a callable that enqueues work on the current HIP stream.

Counterpart of the reference's ``qfactory/profile.py:5-10`` (two ``triton.testing.do_bench`` passes,
the second with a 50 ms warm-up, then a one-second cool-down).  Here the timer is built on HIP
events recorded on the stream the work is enqueued on; between timed calls a buffer larger than the
L2 and Infinity caches is overwritten so that every call starts cold, like do_bench does.
"""
import os
import time

import torch

_FLUSH_BYTES = 512 * 1024 * 1024
_flush_buffer = None


def _flush():
    global _flush_buffer
    if _flush_buffer is None:
        _flush_buffer = torch.empty(_FLUSH_BYTES // 4, dtype=torch.int32, device="cuda")
    _flush_buffer.zero_()


def do_bench(func, warmup=25, rep=100, flush=True, max_calls=2000):
    """Mean milliseconds per call of ``func``; ``warmup`` / ``rep`` are time budgets in ms."""
    func()
    torch.cuda.synchronize()
    start, end = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(5):
        func()
    end.record()
    torch.cuda.synchronize()
    estimate = max(start.elapsed_time(end) / 5, 1e-4)
    n_warmup = max(1, min(max_calls, int(warmup / estimate)))
    n_repeat = max(1, min(max_calls, int(rep / estimate)))
    for _ in range(n_warmup):
        func()
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_repeat)]
    for i in range(n_repeat):
        if flush:
            _flush()
        starts[i].record()
        func()
        ends[i].record()
    torch.cuda.synchronize()
    times = [s.elapsed_time(e) for s, e in zip(starts, ends)]
    return sum(times) / len(times)


def benchmark(func):
    """Seconds per call (reference signature).  ``QFACTORY_BENCH_COOLDOWN`` (seconds, default 0)
    restores the reference's sleep between candidates."""
    do_bench(func)  # warm-up pass
    t = do_bench(func, warmup=50) / 1e3
    torch.cuda.synchronize()
    cooldown = float(os.environ.get("QFACTORY_BENCH_COOLDOWN", "0"))
    if cooldown > 0:
        time.sleep(cooldown)
    return t
