"""Timing of GPU work with HIP events (the role of ``daceml/testing/profiling/event_profiler.py:22-143``
on a ROCm device; torch's ``cuda`` events are HIP events there).

Two ways of measuring:

* :func:`time_funcs` records an event after every function of every iteration on torch's current stream, as
  the reference's ``CudaTimer`` / ``time_funcs`` do, and :func:`print_time_statistics` prints the same table;
* :func:`graph_time_us` records ``reps`` launches into one HIP graph and times whole replays, which removes the
  host's launch gaps: the figure to compare with a profiler's kernel durations.

The core clock of the part drops while it runs memory-bound or idle and needs tens of milliseconds of work
to come back up, so both take ``warm_ms``: untimed repetitions for at least that long before measuring.
"""
import statistics
import time
import typing


def _require_gpu():
    import torch
    if not torch.cuda.is_available():
        raise RuntimeError("timing with HIP events needs a GPU")
    return torch


def warm_up(fn: typing.Callable[[], None], warm_ms: float) -> int:
    """Call ``fn`` and wait for it, again and again, for at least ``warm_ms`` milliseconds; returns the count."""
    torch = _require_gpu()
    n, t_end = 0, time.perf_counter() + warm_ms * 1e-3
    while True:
        fn()
        torch.cuda.synchronize()
        n += 1
        if time.perf_counter() >= t_end:
            return n


class EventTimer:
    """Times ``n`` consecutive regions on the current stream with ``n + 1`` events."""

    def __init__(self, n: int):
        torch = _require_gpu()
        self.events = [torch.cuda.Event(enable_timing=True) for _ in range(n + 1)]
        self.recorded = 0

    def start(self):
        self.events[0].record()
        self.recorded = 1

    def next(self):
        if self.recorded == 0:
            raise RuntimeError("EventTimer.next() before start()")
        if self.recorded >= len(self.events):
            raise RuntimeError("more regions than the timer was made for")
        self.events[self.recorded].record()
        self.recorded += 1

    def end(self):
        if self.recorded != len(self.events):
            raise RuntimeError(f"{self.recorded - 1} of {len(self.events) - 1} regions were recorded")
        self.events[-1].synchronize()

    def get_times(self) -> typing.List[float]:
        """Milliseconds of each region."""
        return [a.elapsed_time(b) for a, b in zip(self.events[:-1], self.events[1:])]


def time_funcs(funcs, func_names=None, num_iters=100, warmups=5, warm_ms=0.0) -> typing.List[typing.List[float]]:
    """Run ``funcs`` one after the other ``num_iters`` times; milliseconds of each function on each iteration
    (``times[i][it]``), after ``warmups`` untimed iterations and ``warm_ms`` milliseconds of them."""
    torch = _require_gpu()
    del func_names  # kept for the reference's signature; there are no profiler ranges to name here

    def once():
        for f in funcs:
            f()

    for _ in range(warmups):
        once()
    torch.cuda.synchronize()
    if warm_ms > 0:
        warm_up(once, warm_ms)
    timer = EventTimer(len(funcs))
    times = [[] for _ in funcs]
    for _ in range(num_iters):
        timer.start()
        for f in funcs:
            f()
            timer.next()
        timer.end()
        for i, t in enumerate(timer.get_times()):
            times[i].append(t)
    return times


def time_statistics(times, func_names) -> typing.List[typing.List[typing.Any]]:
    """Rows ``[name, min, mean, median, stdev, max]`` of the result of :func:`time_funcs`."""
    return [[name, min(t), statistics.mean(t), statistics.median(t), statistics.stdev(t) if len(t) > 1 else 0.0, max(t)]
            for name, t in zip(func_names, times)]


def print_time_statistics(times, func_names):
    headers = ["Name", "Min", "Mean", "Median", "Stdev", "Max"]
    rows = time_statistics(times, func_names)
    try:
        import tabulate
        print(tabulate.tabulate(rows, headers=headers, floatfmt=".4f", tablefmt="github"))
    except ImportError:
        print(" | ".join(headers))
        for r in rows:
            print(" | ".join([str(r[0])] + [f"{v:.4f}" for v in r[1:]]))


def graph_time_us(launch: typing.Callable[[], None], reps=50, replays=5, warm_ms=40.0) -> float:
    """Microseconds of one ``launch``: ``reps`` launches recorded back to back in a HIP graph, the best of
    ``replays`` replays timed between two events on the stream the graph runs on, after ``warm_ms`` of replays."""
    torch = _require_gpu()
    launch()  # loads the code object
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(reps):
            launch()
    warm_up(g.replay, warm_ms)
    best = float("inf")
    for _ in range(replays):
        e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
        e0.record()
        g.replay()
        e1.record()
        torch.cuda.synchronize()
        best = min(best, e0.elapsed_time(e1) * 1e3 / reps)
    return best
