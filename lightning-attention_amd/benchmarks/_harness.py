"""Timing / memory harness for the benchmark tables (no Triton): same protocol as the
``triton.testing.do_bench`` calls in the reference's benchmarks (warm-up by time, then
repetitions for >= 100 ms, gradients cleared between repetitions, median of per-call times
taken with device events).  The warm-up is 60 ms instead of the reference's 25: coming out of idle,
or after a change of shape, the chip's clocks take 20-30 ms under load to settle, and short calls
measured inside that window read up to twice their steady time."""
import statistics

import torch

from lightning_attn.utils import get_memory


def do_bench(fn, warmup_ms=60.0, rep_ms=100.0, grads=()):
    fn()
    torch.cuda.synchronize()
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(3):
        fn()
    e1.record()
    torch.cuda.synchronize()
    est = max(e0.elapsed_time(e1) / 3, 1e-3)
    for _ in range(max(1, int(warmup_ms / est))):
        fn()
    reps = max(5, int(rep_ms / est))
    starts = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    ends = [torch.cuda.Event(enable_timing=True) for _ in range(reps)]
    for i in range(reps):
        for t in grads:
            t.grad = None
        starts[i].record()
        fn()
        ends[i].record()
    torch.cuda.synchronize()
    return statistics.median(s.elapsed_time(e) for s, e in zip(starts, ends))


def peak_memory_mb(fn, device, rep=20):
    torch.cuda.synchronize()
    get_memory(device)
    vals = []
    for _ in range(rep):
        fn()
        torch.cuda.synchronize()
        vals.append(get_memory(device))
    return sum(vals) / len(vals)


def print_table(title, xs, columns):
    """columns: list of (name, values); same text layout as the reference's tables."""
    print("%s:" % title)
    print("   %8s" % "n" + "".join("  %18s" % name for name, _ in columns))
    for i, x in enumerate(xs):
        print("%-2d %8.1f" % (i, float(x)) + "".join("  %18.6f" % vals[i] for _, vals in columns))
