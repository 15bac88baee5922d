"""`autotune`, `get_bound_args` and `AutotuningResult`.

Counterpart of tokamax/_src/autotuning/api.py: `AutotuningResult` (:70-199) is a serialisable set
of (bound arguments -> timings) that can be pushed as an overlay over the shipped cache with a
`with` block (:151-167); `get_bound_args(f, *args, **kwargs)` (:202-239) lists the unique op calls a
function makes; `autotune(f, *args)` (:322-418) tunes them, or a list of bound arguments. The
reference finds the calls by lowering `f` and walking its HLO for the payload every op leaves there
(hlo_utils.py:263-286); here `f` is run once, eagerly, while every `Op.__call__` records its bound
arguments.
"""

from __future__ import annotations

import dataclasses
import json
import logging
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


def get_bound_args(f, *args, **kwargs) -> tuple:
  """The unique `BoundArguments` of all ops `f(*args, **kwargs)` calls (api.py:202-239).

  `f` is run once; ops are unique by (op class, autotuning cache key), in call order, and carry no config (the
  one a call was made with is not part of what gets tuned). A sequence of `BoundArguments` is returned as it is."""
  if isinstance(f, (list, tuple)) and all(isinstance(b, op_lib.BoundArguments) for b in f):
    if args or kwargs:
      raise ValueError("`args` / `kwargs` are only supported if `f` is callable.")
    return tuple(f)
  if not callable(f):
    raise TypeError(f"expected a callable or a sequence of BoundArguments, got {type(f).__name__}")
  calls: list = []
  token = op_lib.OP_CALL_RECORDER.set(calls)
  try:
    f(*args, **kwargs)
  finally:
    op_lib.OP_CALL_RECORDER.reset(token)
  seen, unique = set(), []
  for ba in calls:
    ba = op_lib.BoundArguments(ba.op.replace(config=None), ba.arguments)
    key = (type(ba.op).__name__, ba.autotuning_cache_key)
    if key not in seen:
      seen.add(key)
      unique.append(ba)
  return tuple(unique)


def autotune(f, *args, ignore_cache: bool = False, all_implementations: bool = False, progress_bar: bool = False,
             timeout: float | None = 600.0, max_workers: int | None = None,
             autotuner: autotuner_lib.Autotuner | None = None) -> AutotuningResult:
  """Autotunes all ops `f(*args)` calls (api.py:322-418).

  `f` is a callable or a sequence of `BoundArguments`; to tune a callable with keyword arguments pass
  `get_bound_args(f, *args, **kwargs)`. Ops already in the autotuning cache are skipped unless `ignore_cache`. A
  failure to tune one op is logged and leaves that op out of the result. `all_implementations` and `max_workers`
  are accepted for the reference's signature: each op here has one implementation, and its kernel variants are
  precompiled, so there is no compilation to spread over workers."""
  del all_implementations, max_workers, progress_bar
  bound_args = get_bound_args(f, *args)
  if not ignore_cache:
    bound_args = [ba for ba in bound_args if ba.cached_autotuning_data is None]
  kinds = {k for k in map(op_lib.infer_device_kind, bound_args) if k is not None and k != "cpu"}
  if len(kinds) > 1:
    raise ValueError(f"Multiple device kinds found: {kinds}")
  device_kind = kinds.pop() if kinds else op_lib.device_kind()
  autotuner = autotuner if autotuner is not None else autotuner_lib.Autotuner()
  results = []
  for ba in bound_args:
    try:
      results.append((ba, ba.autotune(autotuner=autotuner, cache_results=False, timeout=timeout)))
    except Exception:  # pylint: disable=broad-exception-caught
      logging.getLogger(__name__).exception("Failed to autotune for op %s", ba.op)
  return AutotuningResult(device_kind, tuple(results))


def save_cache_file(ops_results: Sequence[tuple], path: str) -> None:
  """Writes {(ba -> data)} of ONE op class as a shipped-cache JSON file (key -> {config -> timings})."""
  data = {ba.autotuning_cache_key: tuning for ba, tuning in ops_results}
  op = ops_results[0][0].op if ops_results else None
  with open(path, "w", encoding="utf-8") as f:
    f.write(cache_lib.dumps(op, data))
