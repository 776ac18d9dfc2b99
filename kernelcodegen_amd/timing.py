"""HIP-event timing shared by the perf_*.py harnesses."""
import time


def time_launches(fn, iters, settle_ms=30.0):
    """Average milliseconds per call of `fn` over `iters` calls, bracketed by HIP events on
    the current stream.  Before the timed region `fn` runs for at least `settle_ms`: the
    shader clock drops within a millisecond of idle time (allocations, host work between
    shapes) and takes tens of milliseconds of load to come back."""
    import torch
    for _ in range(3):
        fn()
    torch.cuda.synchronize()
    t0 = time.perf_counter()
    fn()
    torch.cuda.synchronize()
    one_ms = max((time.perf_counter() - t0) * 1e3, 1e-3)
    for _ in range(min(5000, int(settle_ms / one_ms) + 1)):
        fn()
    e0 = torch.cuda.Event(enable_timing=True)
    e1 = torch.cuda.Event(enable_timing=True)
    e0.record()
    for _ in range(iters):
        fn()
    e1.record()
    torch.cuda.synchronize()
    return e0.elapsed_time(e1) / iters
