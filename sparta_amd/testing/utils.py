"""Latency measurement and result checking (API of sparta/testing/utils.py:9-73)."""
from typing import Callable, List, Optional

import torch


def check(func: Callable, inputs: List, target_outputs: List, atol: Optional[float] = None,
          rtol: Optional[float] = None):
    """Run `func(*inputs)` and compare with the targets.

    Tolerances default to the reference's atol 1e-4 / rtol 1e-8 for float32 and
    to atol = rtol = 1e-2 for 16-bit types.
    """
    outputs = func(*inputs)
    if len(target_outputs) == 1:
        outputs = [outputs]
    assert len(outputs) == len(target_outputs), \
        f'expected {len(target_outputs)} outputs, got {len(outputs)}'
    for got, want in zip(outputs, target_outputs):
        half = got.dtype in (torch.float16, torch.bfloat16)
        a = atol if atol is not None else (1e-2 if half else 1e-4)
        r = rtol if rtol is not None else (1e-2 if half else 1e-8)
        torch.testing.assert_close(got, want.to(got.dtype), atol=a, rtol=r)


def _device_time_ms(func: Callable, inputs: List, num_iters: int, min_device_ms: float = 5.0,
                    max_replays: int = 200) -> float:
    """Mean device time of one `func(*inputs)` call in milliseconds: `num_iters` calls are
    captured into one graph on a side stream and the graph is replayed, bracketed by events on
    that stream, until at least `min_device_ms` of device time has been measured.  The host
    cost of a call (argument marshalling, the allocator, the launch itself: 10 us and more) is
    paid once, at capture, and is not part of the result."""
    stream = torch.cuda.Stream()
    graph = torch.cuda.CUDAGraph()
    stream.wait_stream(torch.cuda.current_stream())
    with torch.cuda.stream(stream):
        with torch.cuda.graph(graph, stream=stream):
            for _ in range(num_iters):
                func(*inputs)
        graph.replay()   # untimed: the first replay pages the graph in
        stream.synchronize()
        total_ms, replays = 0.0, 0
        while replays < max_replays and (replays == 0 or total_ms < min_device_ms):
            begin = torch.cuda.Event(enable_timing=True)
            end = torch.cuda.Event(enable_timing=True)
            begin.record(stream)
            graph.replay()
            end.record(stream)
            stream.synchronize()
            total_ms += begin.elapsed_time(end)
            replays += 1
    torch.cuda.current_stream().wait_stream(stream)
    return total_ms / (replays * num_iters)


def profile(func: Callable, inputs: List, target_outputs: Optional[List] = None,
            num_warmups: int = 10, num_iters: int = 10, cuda: bool = False) -> float:
    """Mean latency of `func(*inputs)` in milliseconds.

    cuda=False: wall time of the calls as issued from Python, measured with device events
    on the current stream (utils.py:46-54) - it includes whatever the host adds between
    launches.  cuda=True: time spent on the device only, the semantics of the reference's
    profiler branch that sums the kernel times of a trace (utils.py:37-45); here the calls
    are replayed from a captured graph (see _device_time_ms), and a function that cannot be
    captured (one that synchronises with the host) is timed as with cuda=False.
    A failing check raises AssertionError; any failure while timing yields inf (utils.py:55-56)."""
    if target_outputs is not None:
        check(func, inputs, target_outputs)
    try:
        for _ in range(num_warmups):
            func(*inputs)
        torch.cuda.synchronize()
        if cuda:
            try:
                return _device_time_ms(func, inputs, max(num_iters, 1))
            except Exception:
                torch.cuda.synchronize()   # not capturable: fall through to event timing
        begin = torch.cuda.Event(enable_timing=True)
        end = torch.cuda.Event(enable_timing=True)
        begin.record()
        for _ in range(num_iters):
            func(*inputs)
        end.record()
        torch.cuda.synchronize()
        return begin.elapsed_time(end) / num_iters
    except Exception:
        return float('inf')
