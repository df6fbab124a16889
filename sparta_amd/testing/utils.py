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


def profile(func: Callable, inputs: List, target_outputs: Optional[List] = None,
            num_warmups: int = 10, num_iters: int = 10, cuda: bool = False) -> float:
    """Mean latency of `func(*inputs)` in milliseconds, measured with device
    events on the current stream.  `cuda` is accepted for call compatibility;
    event timing is used either way.  A failing check raises AssertionError;
    any failure while timing yields inf (utils.py:55-56)."""
    if target_outputs is not None:
        check(func, inputs, target_outputs)
    try:
        for _ in range(num_warmups):
            func(*inputs)
        torch.cuda.synchronize()
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
