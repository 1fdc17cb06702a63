"""How one function is timed (reference: src/kernl/benchmark/benchmark_fixture.py:51-121).

The run count comes from a 5-run estimate and two time budgets (warm-up and measurement, in milliseconds of estimated
run time).  Each measured run starts on cold caches: a 256 MB buffer is rewritten first, which evicts the 4 MB L2 of
every XCD and the 256 MB memory-side cache of the MI355X.  Two series are taken: device time between two HIP events
recorded on the current stream around the run, and host wall-clock time around the run plus a synchronisation.  On a
machine without a GPU only the wall-clock series exists (and is reported for both).
"""
import gc
from dataclasses import dataclass
from time import perf_counter_ns
from typing import Any, Callable, Iterable, Optional

import torch

from kernl_amd.benchmark.stats import Samples

FLUSH_BYTES = 256 * 1000 * 1000


@dataclass
class Measurement:
    device: Samples   # HIP-event time per run, ms
    wall: Samples     # host wall-clock time per run including the synchronisation, ms
    return_value: Any


def _sync(on_gpu: bool) -> None:
    if on_gpu:
        torch.cuda.synchronize()


def measure(fn: Callable, *args, warmup_ms: float = 25.0, rep_ms: float = 100.0,
            grad_to_none: Optional[Iterable[torch.Tensor]] = None, max_runs: int = 10000, **kwargs) -> Measurement:
    on_gpu = torch.cuda.is_available()
    # run-time estimate: one untimed run, then five timed ones
    fn(*args, **kwargs)
    _sync(on_gpu)
    t0 = perf_counter_ns()
    for _ in range(5):
        fn(*args, **kwargs)
    _sync(on_gpu)
    estimate_ms = max((perf_counter_ns() - t0) * 1e-6 / 5, 1e-3)
    n_warmup = min(max_runs, max(1, int(warmup_ms / estimate_ms)))
    n_runs = min(max_runs, max(1, int(rep_ms / estimate_ms)))

    flush = torch.empty(FLUSH_BYTES, dtype=torch.int8, device="cuda") if on_gpu else None

    def prepare():
        if grad_to_none is not None:
            for t in grad_to_none:
                t.grad = None
        if flush is not None:
            flush.zero_()

    value = None
    for _ in range(n_warmup):
        value = fn(*args, **kwargs)

    device_ms = None
    if on_gpu:
        starts = [torch.cuda.Event(enable_timing=True) for _ in range(n_runs)]
        ends = [torch.cuda.Event(enable_timing=True) for _ in range(n_runs)]
        for i in range(n_runs):
            prepare()
            starts[i].record()
            fn(*args, **kwargs)
            ends[i].record()
        torch.cuda.synchronize()
        device_ms = [s.elapsed_time(e) for s, e in zip(starts, ends)]
        gc.collect()
        torch.cuda.empty_cache()

    wall_ms = []
    for _ in range(n_runs):
        prepare()
        _sync(on_gpu)
        t0 = perf_counter_ns()
        fn(*args, **kwargs)
        _sync(on_gpu)
        wall_ms.append((perf_counter_ns() - t0) * 1e-6)
    if on_gpu:
        gc.collect()
        torch.cuda.empty_cache()
    wall = Samples(wall_ms)
    return Measurement(device=Samples(device_ms) if device_ms is not None else wall, wall=wall, return_value=value)
