"""Timing helpers shared by bench.py and bench_experiments.py."""
import sys

MiB = 1 << 20
GiB = 1 << 30
HBM_PEAK_GBPS = 8000.0

def log(*a):
    print(*a, file=sys.stderr, flush=True)


# ------------------------------------------------------------------------------------- timing

def time_region(fn, steps, warmup):
    """Average seconds per call of fn over `steps` back-to-back launches on the current stream,
    bracketed by HIP events on that stream."""
    import torch
    for _ in range(warmup):
        fn()
    torch.cuda.synchronize()
    start = torch.cuda.Event(enable_timing=True)
    stop = torch.cuda.Event(enable_timing=True)
    start.record()
    for _ in range(steps):
        fn()
    stop.record()
    torch.cuda.synchronize()
    return start.elapsed_time(stop) * 1e-3 / steps


def time_each(fn, steps, warmup, before=None):
    """Per-launch times (seconds), each launch bracketed by its own event pair; `before` runs
    untimed ahead of every launch (e.g. a cache flush)."""
    import torch
    for _ in range(warmup):
        fn()
    out = []
    for _ in range(steps):
        if before:
            before()
        start = torch.cuda.Event(enable_timing=True)
        stop = torch.cuda.Event(enable_timing=True)
        start.record()
        fn()
        stop.record()
        torch.cuda.synchronize()
        out.append(start.elapsed_time(stop) * 1e-3)
    return out


def gbps(nbytes, seconds):
    return nbytes / seconds / 1e9


def _abi():
    """The bound library and torch's current stream handle (the stream the HIP events are on)."""
    import torch
    from l2_torch_alloc_amd import wrapper
    return wrapper.library(), torch.cuda.current_stream().cuda_stream
