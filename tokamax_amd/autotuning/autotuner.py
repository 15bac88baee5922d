"""Autotuner: time every candidate config, keep failures as data.

Follows tokamax/_src/autotuning/autotuner.py: `AutotuningData.fastest_config` (:47-59) picks the
minimum median time and raises an `ExceptionGroup` when every config failed; `Autotuner.autotune`
(:125-217) never raises for a failing config, it records the exception under that config. The
kernels are precompiled, so there is no compile pool; configs are timed one after another.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Callable, Generic, Iterable, TypeVar

from exceptiongroup import ExceptionGroup

from tokamax_amd import benchmarking

BenchmarkData = benchmarking.BenchmarkData
K = TypeVar("K")


class AutotuningData(dict, Generic[K]):
  """Mapping config -> BenchmarkData | Exception."""

  @property
  def fastest_config(self) -> K:
    valid = [(c, d) for c, d in self.items() if isinstance(d, BenchmarkData)]
    if not valid:
      if self:
        raise ExceptionGroup("All configs failed", [e for e in self.values() if isinstance(e, Exception)])
      raise ValueError("Autotuning data is empty")
    return min(valid, key=lambda x: x[1].median_evaluation_time_ms)[0]

  def prune(self) -> "AutotuningData[K]":
    if not self:
      return self
    config = self.fastest_config
    return AutotuningData({config: self[config]})

  def prune_errors(self) -> dict:
    return {k: v for k, v in self.items() if isinstance(v, BenchmarkData)}

  def __or__(self, other):
    return AutotuningData(dict.__or__(self, other))

  def __hash__(self):  # immutable by convention, like the reference's immutabledict
    return hash(tuple(self.keys()))


@dataclasses.dataclass(frozen=True)
class Autotuner:
  """Times `fn_factory(config)(*args, **kwargs)` for every config."""

  iterations: int = 5
  warmup: int = 1
  # Passes over the config list, the second in reverse order; a config keeps the pass with the lower median. The
  # clock a kernel runs at depends on what ran just before it (the first config after an idle device measured up to
  # 8 % slow, enough to hide a 10 % faster tile), so one pass in one order ranks neighbours unfairly.
  passes: int = 2

  def autotune(self, fn_factory: Callable[[Any], Callable[..., Any]], configs: Iterable[Any], *args,
               timeout: float | None = 600.0, **kwargs) -> AutotuningData:
    del timeout  # precompiled kernels: nothing here can block on a compiler
    configs = list(configs)
    results = {}
    for sweep in range(max(self.passes, 1)):
      for config in (configs if sweep % 2 == 0 else reversed(configs)):
        if isinstance(results.get(config), Exception):
          continue
        try:
          fn = fn_factory(config)
          data = benchmarking.benchmark(lambda: fn(*args, **kwargs), iterations=self.iterations, warmup=self.warmup)
        except Exception as e:  # pylint: disable=broad-exception-caught
          results[config] = e
          continue
        seen = results.get(config)
        if seen is None or data.median_evaluation_time_ms < seen.median_evaluation_time_ms:
          results[config] = data
    return AutotuningData(results)
