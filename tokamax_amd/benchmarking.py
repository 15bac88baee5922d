"""Timing of device work with HIP events, and the record the autotuner stores.

Counterpart of tokamax/_src/benchmarking.py: `BenchmarkData` keeps the reference's fields
(:76-95) so that cache files have the same schema; the timer replaces CUPTI/xprof
(:432-471) with HIP events recorded on the stream the kernels are launched on.
"""

from __future__ import annotations

import dataclasses
import statistics
import time
from typing import Any, Callable

import torch


@dataclasses.dataclass(frozen=True)
class BenchmarkData:
  """Timings of one (op, arguments, config)."""

  compile_time_ms: float
  lower_time_ms: float
  evaluation_times_ms: tuple[float, ...]
  metadata: dict = dataclasses.field(default_factory=dict)
  peak_memory_mb: float | None = None

  @property
  def median_evaluation_time_ms(self) -> float:
    return float(statistics.median(self.evaluation_times_ms))

  def to_json_dict(self) -> dict:
    d = dict(
        compile_time_ms=self.compile_time_ms,
        lower_time_ms=self.lower_time_ms,
        evaluation_times_ms=list(self.evaluation_times_ms),
        metadata=dict(self.metadata),
    )
    if self.peak_memory_mb is not None:
      d["peak_memory_mb"] = self.peak_memory_mb
    return d

  @classmethod
  def from_json_dict(cls, d: dict) -> "BenchmarkData":
    return cls(
        compile_time_ms=float(d.get("compile_time_ms", 0.0)),
        lower_time_ms=float(d.get("lower_time_ms", 0.0)),
        evaluation_times_ms=tuple(float(x) for x in d["evaluation_times_ms"]),
        metadata=dict(d.get("metadata", {})),
        peak_memory_mb=d.get("peak_memory_mb"),
    )


def time_on_stream(fn: Callable[[], Any], *, iterations: int = 5, warmup: int = 1, device=None) -> tuple[float, ...]:
  """Device time of each of `iterations` calls of `fn`, in ms, from HIP events on the current stream."""
  stream = torch.cuda.current_stream(device)
  for _ in range(warmup):
    fn()
  stream.synchronize()
  times = []
  for _ in range(iterations):
    start = torch.cuda.Event(enable_timing=True)
    end = torch.cuda.Event(enable_timing=True)
    start.record(stream)
    fn()
    end.record(stream)
    end.synchronize()
    times.append(start.elapsed_time(end))
  return tuple(times)


# Calls shorter than this are timed inside a captured graph: the host needs tens of microseconds to issue one
# call, so events around eager calls of a shorter kernel measure the host, not the kernel.
GRAPH_TIMING_BELOW_MS = 0.25


def time_in_graph(fn: Callable[[], Any], *, iterations: int = 5, launches: int = 16, device=None) -> tuple[float, ...]:
  """Device time per call of `fn`, in ms, from `iterations` replays of a HIP graph that holds `launches` back-to-back
  calls (events around each replay; the reference's timer, CUPTI kernel times, likewise leaves the host out,
  benchmarking.py:432-471). `fn` must be capturable: device work on the current stream only, no synchronisation."""
  side = torch.cuda.Stream(device=device)
  side.wait_stream(torch.cuda.current_stream(device))
  with torch.cuda.stream(side):
    fn()  # once outside capture on this stream: whatever the call sets up per stream exists before capture
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
      for _ in range(launches):
        fn()
    graph.replay()
    side.synchronize()
    times = []
    for _ in range(iterations):
      start = torch.cuda.Event(enable_timing=True)
      end = torch.cuda.Event(enable_timing=True)
      start.record(side)
      graph.replay()
      end.record(side)
      end.synchronize()
      times.append(start.elapsed_time(end) / launches)
  torch.cuda.current_stream(device).wait_stream(side)
  del graph
  return tuple(times)


def benchmark(fn: Callable[[], Any], *, iterations: int = 5, warmup: int = 1, device=None) -> BenchmarkData:
  """Runs `fn` once untimed (the "compile"/first-launch cost), then times it: eagerly, and calls that turn out
  shorter than GRAPH_TIMING_BELOW_MS again inside a captured graph (`metadata["timing"]` says which)."""
  t0 = time.perf_counter()
  fn()
  torch.cuda.current_stream(device).synchronize()
  first_ms = (time.perf_counter() - t0) * 1e3
  times = time_on_stream(fn, iterations=iterations, warmup=warmup, device=device)
  metadata = {"timing": "eager"}
  if statistics.median(times) < GRAPH_TIMING_BELOW_MS:
    try:
      times = time_in_graph(fn, iterations=iterations, device=device)
      metadata = {"timing": "graph"}
    except RuntimeError:  # not capturable: the eager times stand
      torch.cuda.synchronize(device)
  return BenchmarkData(compile_time_ms=first_ms, lower_time_ms=0.0, evaluation_times_ms=times, metadata=metadata)
