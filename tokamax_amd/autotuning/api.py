"""`autotune` and `AutotuningResult`.

Counterpart of tokamax/_src/autotuning/api.py: `AutotuningResult` (:70-199) is a serialisable set
of (bound arguments -> timings) that can be pushed as an overlay over the shipped cache with a
`with` block (:151-167); `autotune` (:322-418) tunes a list of bound arguments. The reference can
also discover the ops inside a jitted function from its HLO; without a tracing compiler there is
nothing to walk, so this `autotune` takes the bound arguments directly.
"""

from __future__ import annotations

import dataclasses
import json
from typing import Iterable, Sequence

from tokamax_amd import benchmarking
from tokamax_amd import op as op_lib
from tokamax_amd.autotuning import autotuner as autotuner_lib
from tokamax_amd.autotuning import cache as cache_lib

AutotuningData = autotuner_lib.AutotuningData


@dataclasses.dataclass(frozen=True)
class AutotuningResult:
  """Autotuning results for a device kind: ((BoundArguments, AutotuningData), ...)."""

  device_kind: str
  data: tuple

  def __enter__(self):
    overlay: dict = {}
    for ba, tuning in self.data:
      key = ba.autotuning_cache_key
      overlay.setdefault(ba.op.replace(vjp=None), {}).setdefault(self.device_kind, {})[key] = tuning
    stack = op_lib.AUTOTUNING_CACHE_OVERLAY_STACK
    object.__setattr__(self, "_token", stack.set(stack.get() + (overlay,)))
    return self

  def __exit__(self, *exc):
    op_lib.AUTOTUNING_CACHE_OVERLAY_STACK.reset(self._token)  # pylint: disable=no-member
    return False

  def dumps(self) -> str:
    items = []
    for ba, tuning in self.data:
      entry = {
          cache_lib.config_to_json(c): d.to_json_dict()
          for c, d in tuning.items() if isinstance(d, benchmarking.BenchmarkData)
      }
      items.append(dict(bound_args=ba.to_json_dict(), data=entry))
    return json.dumps(dict(device_kind=self.device_kind, data=items), indent=2)

  @classmethod
  def loads(cls, s: str, ops: dict) -> "AutotuningResult":
    """`ops` maps op class names to op instances (to rebuild the bound arguments)."""
    raw = json.loads(s)
    data = []
    for item in raw["data"]:
      op_json = item["bound_args"]["op"]
      op = ops[op_json["__class__"]]
      spec = op.arg_spec_from_json(item["bound_args"]["arguments"])
      ba = op.bind(**spec)
      tuning = AutotuningData({
          op.config_cls(**json.loads(c)): benchmarking.BenchmarkData.from_json_dict(d)
          for c, d in item["data"].items()
      })
      data.append((ba, tuning))
    return cls(raw["device_kind"], tuple(data))


def autotune(bound_args: Iterable[op_lib.BoundArguments], *, ignore_cache: bool = False,
             all_implementations: bool = False,
             autotuner: autotuner_lib.Autotuner = autotuner_lib.Autotuner()) -> AutotuningResult:
  """Autotunes each of `bound_args`; already cached ones are skipped unless `ignore_cache`."""
  del all_implementations  # one implementation per op in this package
  results = []
  seen = set()
  for ba in bound_args:
    if ba in seen:
      continue
    seen.add(ba)
    if not ignore_cache and ba.cached_autotuning_data is not None:
      continue
    results.append((ba, ba.autotune(autotuner=autotuner, cache_results=False)))
  return AutotuningResult(op_lib.device_kind(), tuple(results))


def save_cache_file(ops_results: Sequence[tuple], path: str) -> None:
  """Writes {(ba -> data)} of ONE op class as a shipped-cache JSON file (key -> {config -> timings})."""
  data = {ba.autotuning_cache_key: tuning for ba, tuning in ops_results}
  op = ops_results[0][0].op if ops_results else None
  with open(path, "w", encoding="utf-8") as f:
    f.write(cache_lib.dumps(op, data))
