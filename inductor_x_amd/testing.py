"""Timing helper for compiled-versus-eager comparisons.

Counterpart of the harness the reference's test scripts share (reference
test/npu_indexing/utils.py:26-65: wall clock around `times * repeat` calls with a stream
synchronisation on both sides, microseconds per call and the gain over eager printed).  Two
things differ: the clock is a pair of HIP events on the stream the calls go to, and with
`graph=True` the calls are replayed from a HIP graph, so kernels of a few microseconds are not
hidden behind the host's per-launch cost."""
from __future__ import annotations

from typing import Callable, Sequence

import torch


def _event_us(fn: Callable[[], object], calls: int) -> float:
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    torch.cuda.synchronize()
    start.record()
    for _ in range(calls):
        fn()
    end.record()
    end.synchronize()
    return start.elapsed_time(end) * 1e3 / calls


def _graph_us(fn: Callable[[], object], calls: int, per_graph: int = 20) -> float:
    fn()
    side = torch.cuda.Stream()
    side.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(side):
        fn()
    torch.cuda.current_stream().wait_stream(side)
    torch.cuda.synchronize()
    g = torch.cuda.CUDAGraph()
    with torch.cuda.graph(g):
        for _ in range(per_graph):
            fn()
    g.replay()
    replays = max(calls // per_graph, 1)
    return _event_us(g.replay, replays) / per_graph


def benchmark_test(fn: Callable, fn_compiled: Callable, args: Sequence = (), name: str = "gen_fn", times: int = 10,
                   repeat: int = 10, graph: bool = False, verbose: bool = True) -> tuple[float, float]:
    """Microseconds per call of the eager and of the compiled function, `times * repeat` calls each
    after two warm-up calls.  Returns (time_eager, time_compiled) like the reference's helper."""
    calls = max(times * repeat, 1)
    for f in (fn_compiled, fn):
        for _ in range(2):
            f(*args)
    timer = _graph_us if graph else _event_us
    time_compiled = timer(lambda: fn_compiled(*args), calls)
    time_eager = timer(lambda: fn(*args), calls)
    if verbose:
        gain = (time_eager - time_compiled) / time_compiled * 100
        print(f"benchmark_{name}: eager {time_eager:.3f} us, compiled {time_compiled:.3f} us ({gain:+.1f} %)")
    return time_eager, time_compiled
