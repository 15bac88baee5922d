"""Base class for ops: bind -> pick a config -> run `_fwd`, with a custom VJP.

Restates tokamax/_src/ops/op.py for torch tensors. Kept identical in behaviour:
  * `Op.__call__` (op.py:196-307): bind, device check (`NotImplementedError("Not supported on ...")`,
    :209-211), config selection through `BoundArguments.default_config`, `_fwd`, and the op's own
    `vjp` for gradients (here via `torch.autograd.Function` instead of `jax.custom_vjp`).
  * `BoundArguments.get_config` (op.py:477-516): `op.config` -> NullConfig shortcut -> overlay stack
    (innermost first) -> shipped JSON cache (fastest config by median) -> autotune -> heuristics ->
    `ValueError("No config found ...")`.
  * `autotuning_configs = {heuristics_config} | op._get_autotuning_configs(ba)` (op.py:558-561).
Not restated: the vmap capture and the HLO metadata payload, which only exist under JAX tracing.
"""

from __future__ import annotations

import abc
import collections
import contextvars
import dataclasses
import functools
import inspect
import json
import logging
from typing import Any, Callable, ClassVar, Mapping

import torch

from tokamax_amd import benchmarking
from tokamax_amd import config as config_lib
from tokamax_amd import serialization
from tokamax_amd.autotuning import autotuner as autotuner_lib
from tokamax_amd.autotuning import cache as autotuning_cache

AutotuningData = autotuner_lib.AutotuningData
DeviceKind = str
logger = logging.getLogger("tokamax_amd")


@dataclasses.dataclass(frozen=True)
class NullConfig:
  ...


_NULL_CONFIG = NullConfig()


class AUTO:
  """Sentinel: autotune over `BoundArguments.autotuning_configs`."""


# Names of GPUs whose marketing name the runtime may not report (it needs a PCI-id table that
# is not always installed): fall back to the architecture.
_ARCH_DEVICE_KINDS = {"gfx950": "AMD Instinct MI355X", "gfx942": "AMD Instinct MI300X", "gfx90a": "AMD Instinct MI250X"}


def device_kind(device=None) -> DeviceKind:
  """The key autotuning caches are filed under (the role of `jax.Device.device_kind`)."""
  if not torch.cuda.is_available():
    return "cpu"
  index = device.index if isinstance(device, torch.device) else device
  return _device_kind_of(torch.cuda.current_device() if index is None else int(index))


@functools.lru_cache(maxsize=None)
def _device_kind_of(index: int) -> DeviceKind:
  props = torch.cuda.get_device_properties(index)
  arch = getattr(props, "gcnArchName", "").split(":")[0]
  if arch in _ARCH_DEVICE_KINDS:
    return _ARCH_DEVICE_KINDS[arch]
  return props.name


def default_device() -> torch.device:
  if torch.cuda.is_available():
    return torch.device("cuda", torch.cuda.current_device())
  return torch.device("cpu")


@dataclasses.dataclass(frozen=True)
class Op(abc.ABC):
  """Base class for operations (see module docstring)."""

  config_cls: ClassVar[type] = NullConfig
  supports_symbolic_shapes: ClassVar[bool] = True

  config: Any = None
  _: dataclasses.KW_ONLY
  # `vjp(residuals, out, dout, *args, **kwargs)` returns gradients for the positional arguments,
  # as a tuple, or as a dict {"argname": gradient}.
  vjp: Callable[..., Any] | None = None

  def __call__(self, *args, return_residuals: bool = False, **kwargs):
    ba = self.bind(*args, return_residuals=return_residuals, **kwargs)
    recorder = OP_CALL_RECORDER.get()
    if recorder is not None:
      recorder.append(ba)
    tensors = ba.tensors
    for device in {t.device for t in tensors} or {default_device()}:
      if not self.supported_on(device):
        raise NotImplementedError(f"Not supported on {device_kind(device) if device.type == 'cuda' else device}.")
    config = ba.default_config

    needs_grad = self.vjp is not None and torch.is_grad_enabled() and any(t.requires_grad for t in tensors)
    if not needs_grad:
      # (Every parameter of `_fwd` can be passed by name; that spares splitting the arguments by parameter kind.)
      out, residuals = self._fwd(config=config, **ba.arguments)
      return (out, residuals) if return_residuals else out
    return _call_with_vjp(self, ba, config, return_residuals)

  def bind(self, *args, return_residuals: bool = False, **kwargs) -> "BoundArguments":
    """Binds the op to the given arguments."""
    ba = self._fwd_signature.bind(*args, return_residuals=return_residuals, **kwargs)
    ba.apply_defaults()
    return BoundArguments(self, ba.arguments)

  def _bind_all(self, **arguments) -> "BoundArguments":
    """`bind` for a caller that names every parameter of `_fwd` (a subclass's own `bind`, which has the defaults in its
    signature): the arguments are put in signature order without going through `inspect`, which costs about 10 us
    per call."""
    names = _FWD_PARAMETER_NAMES.get(type(self))
    if names is None:
      names = tuple(self._fwd_signature.parameters)
      _FWD_PARAMETER_NAMES[type(self)] = names
    if len(arguments) != len(names):
      return self.bind(**arguments)  # (something is missing or unknown: the slow path reports it)
    try:
      return BoundArguments(self, {n: arguments[n] for n in names})
    except KeyError:
      return self.bind(**arguments)

  def replace(self, **kwargs) -> "Op":
    new_op = dataclasses.replace(self, **kwargs)
    # Ops may install a default VJP in `__post_init__`; an explicit `vjp=None` must win.
    if "vjp" in kwargs:
      object.__setattr__(new_op, "vjp", kwargs["vjp"])
    return new_op

  def get_autotuning_cache(self, device_kind_: DeviceKind | None = None) -> dict:
    self_no_vjp = self.replace(vjp=None)
    if device_kind_ is None:
      device_kind_ = device_kind()
    if config_lib.ignore_autotuning_cache.value:
      logger.warning("Ignoring autotuning cache for %s", self_no_vjp)
      return {}
    cache = _AUTOTUNING_CACHE.get(self_no_vjp)
    if cache is None:
      cache = autotuning_cache.AutotuningCache(self_no_vjp)
      _AUTOTUNING_CACHE[self_no_vjp] = cache
    return cache[device_kind_]

  @abc.abstractmethod
  def _fwd(self, *args, **kwargs):
    ...

  def _get_heuristics_config(self, ba: "BoundArguments"):
    del ba
    if type(self).config_cls is NullConfig:
      return _NULL_CONFIG
    raise NotImplementedError("`_get_heuristics_config` not implemented.")

  def _get_autotuning_cache_key(self, ba: "BoundArguments"):
    return CacheKey(tuple((k, serialization.abstractify(v)) for k, v in ba.arguments.items()))

  def _get_autotuning_configs(self, ba: "BoundArguments") -> set:
    del ba
    return set()

  @property
  def signature(self) -> inspect.Signature:
    if type(self).bind is not Op.bind:
      return inspect.signature(self.bind)
    return self._fwd_signature

  @property
  def _fwd_signature(self) -> inspect.Signature:
    # Per class, not per call: building a Signature costs tens of microseconds and an op call binds
    # its arguments several times.
    sig = _FWD_SIGNATURES.get(type(self))
    if sig is None:
      full = inspect.signature(type(self)._fwd)
      params = [p for name, p in full.parameters.items() if name not in ("self", "config")]
      sig = full.replace(parameters=tuple(params))
      _FWD_SIGNATURES[type(self)] = sig
    return sig

  def supported_on(self, device: torch.device) -> bool:
    del device
    return True


_FWD_SIGNATURES: dict = {}


class CacheKey(tuple):
  """Hashable (name, abstract value) pairs in signature order; JSON form = the cache-file key."""

  def to_json(self) -> str:
    return json.dumps({k: serialization.to_jsonable(v) for k, v in self}, separators=(",", ":"))

  def __repr__(self):
    return f"CacheKey({self.to_json()})"


_AUTOTUNING_CACHE: dict = {}

# Config memo. Resolving a config walks the overlay stack and the JSON cache with a key built from
# every argument; an eager caller repeats that for identical shapes on every call. The result is
# kept per op instance under a cheap structural signature of the arguments plus everything else the
# answer depends on: this counter (bumped whenever cached autotuning data changes), the two config
# options, and the identity of the overlay stack.
_CONFIG_EPOCH = [0]


_FWD_PARAMETER_NAMES: dict = {}


def config_epoch() -> int:
  """The counter that `bump_config_epoch` advances (for callers that memoise on top of the resolved config)."""
  return _CONFIG_EPOCH[0]


def bump_config_epoch() -> None:
  _CONFIG_EPOCH[0] += 1


class _Unhashable(Exception):
  pass


def _fast_signature(v):
  """A cheap hashable stand-in for one argument: shapes, dtypes and devices of arrays, values of the rest."""
  if isinstance(v, torch.Tensor):
    return (v.shape, v.dtype, v.device)
  if v is None or isinstance(v, (bool, int, float, str, torch.dtype)):
    return v
  sig = getattr(v, "_fast_signature", None)
  if sig is not None:
    return sig()
  if isinstance(v, (tuple, list)):
    return tuple(_fast_signature(x) for x in v)
  if callable(v) and not dataclasses.is_dataclass(v):
    return ("callable", id(v))
  try:
    hash(v)
  except TypeError:
    raise _Unhashable from None
  return v
# Stack of {op: {device_kind: {key: AutotuningData}}} overlays pushed by `AutotuningResult`.
# While a list is installed here, every `Op.__call__` appends its bound arguments to it: how `autotune(f, *args)`
# finds the ops a function runs. (The reference walks the function's lowered HLO for the payloads its ops leave
# there, tokamax/_src/hlo_utils.py:263-286; eager calls leave the same record here.)
OP_CALL_RECORDER: contextvars.ContextVar[list | None] = contextvars.ContextVar("OP_CALL_RECORDER", default=None)

AUTOTUNING_CACHE_OVERLAY_STACK: contextvars.ContextVar[tuple] = contextvars.ContextVar(
    "AUTOTUNING_CACHE_OVERLAY_STACK", default=()
)


@dataclasses.dataclass(frozen=True)
class BoundArguments:
  """Bound arguments for an op's `__call__` method."""

  op: Op
  arguments: Mapping[str, Any]

  def __post_init__(self):
    object.__setattr__(self, "arguments", collections.OrderedDict(self.arguments))

  def __hash__(self):
    return hash((self.op.replace(vjp=None), self.autotuning_cache_key))

  def __eq__(self, other):
    return (isinstance(other, BoundArguments) and self.op.replace(vjp=None) == other.op.replace(vjp=None)
            and self.autotuning_cache_key == other.autotuning_cache_key)

  @property
  def signature(self) -> inspect.Signature:
    return self.op._fwd_signature  # pylint: disable=protected-access

  @functools.cached_property
  def tensors(self) -> tuple:
    """Every tensor among the arguments (inside containers and quantised arrays too)."""
    out: list = []
    for v in self.arguments.values():
      if v is not None and v is not False and v is not True:  # (most arguments of a call are defaults)
        _collect_tensors(v, out)
    return tuple(out)

  @functools.cached_property
  def _bound_args(self) -> inspect.BoundArguments:
    return inspect.BoundArguments(self.signature, collections.OrderedDict(self.arguments))

  @property
  def args(self) -> tuple:
    return self._bound_args.args

  @property
  def kwargs(self) -> dict:
    return self._bound_args.kwargs

  @property
  def default_config(self):
    """`op.config`, else cache, else autotune / heuristics / error by the cache-miss option."""
    fallback = config_lib.autotuning_cache_miss_fallback.value
    memo_key = None
    if fallback != "autotune":  # (autotuning has side effects: never answered from the memo)
      try:
        memo_key = (tuple((k, v if v is None or v is False or v is True else _fast_signature(v))
                          for k, v in self.arguments.items()), _CONFIG_EPOCH[0], fallback,
                    config_lib.ignore_autotuning_cache.value, id(AUTOTUNING_CACHE_OVERLAY_STACK.get()))
      except _Unhashable:
        memo_key = None
    memo = self.op.__dict__.get("_config_memo")
    if memo_key is not None and memo is not None and memo_key in memo:
      return memo[memo_key]
    config = self.get_config(
        autotune_configs=AUTO if fallback == "autotune" else None,
        allow_heuristics=fallback != "error",
    )
    if memo_key is not None:
      if memo is None or len(memo) > 256:
        memo = {}
        object.__setattr__(self.op, "_config_memo", memo)
      # The overlay stack tuple is kept alive with the entry, so its id cannot be reused meanwhile.
      memo[memo_key] = config
      memo.setdefault("_keepalive", []).append(AUTOTUNING_CACHE_OVERLAY_STACK.get())
    return config

  def get_config(self, check_autotuning_cache: bool = True, autotune_configs=None,
                 cache_autotuning_results: bool = True, allow_heuristics: bool = True):
    if (config := self.op.config) is not None:
      return config
    if (heuristics_config := self.heuristics_config) is _NULL_CONFIG:
      return heuristics_config
    if check_autotuning_cache:
      data = self.cached_autotuning_data
      if data is not None and len(data):
        return data.fastest_config
    if autotune_configs is not None:
      return self.autotune(autotune_configs, cache_results=cache_autotuning_results).fastest_config
    if allow_heuristics:
      return heuristics_config
    raise ValueError(f"No config found for {self}.")

  @property
  def heuristics_config(self):
    return self.op._get_heuristics_config(self)  # pylint: disable=protected-access

  @functools.cached_property
  def autotuning_cache_key(self):
    return self.op._get_autotuning_cache_key(self)  # pylint: disable=protected-access

  @property
  def cached_autotuning_data(self) -> AutotuningData | None:
    if config_lib.ignore_autotuning_cache.value:
      return None
    kind = infer_device_kind(self) or device_kind()
    key = self.autotuning_cache_key
    op_no_vjp = self.op.replace(vjp=None)
    for overlay in reversed(AUTOTUNING_CACHE_OVERLAY_STACK.get()):
      data = overlay.get(op_no_vjp, {}).get(kind, {}).get(key)
      if data is not None:
        return data
    try:
      return self.op.get_autotuning_cache(kind)[key]
    except KeyError:
      logger.info("Autotuning cache miss for %s on %s with key %s", self.op, kind, key)
      return None

  @property
  def autotuning_configs(self) -> set:
    return {self.heuristics_config} | self.op._get_autotuning_configs(self)  # pylint: disable=protected-access

  def benchmark(self, iterations: int = 5) -> benchmarking.BenchmarkData:
    args, kwargs = self.args, self.kwargs
    return benchmarking.benchmark(lambda: self.op(*args, **kwargs), iterations=iterations)

  def autotune(self, configs=AUTO, autotuner: autotuner_lib.Autotuner = autotuner_lib.Autotuner(),
               cache_results: bool = True, timeout: float | None = None) -> AutotuningData:
    if configs is AUTO:
      configs = self.autotuning_configs
    op_fn = lambda config: self.op.replace(config=config)
    data = autotuner.autotune(op_fn, configs, *self.args, timeout=timeout, **self.kwargs)
    if cache_results:
      self.op.get_autotuning_cache()[self.autotuning_cache_key] = data
      bump_config_epoch()
    return data

  def to_json_dict(self) -> dict:
    """`{"op": ..., "arguments": ...}` with abstract arguments (the reference's BOUND_ARGS_ADAPTER form)."""
    op = self.op.replace(vjp=None)
    op_json = {"__class__": type(op).__name__}
    for f in dataclasses.fields(op):
      if f.name not in ("_", "vjp"):
        op_json[f.name] = serialization.to_jsonable(getattr(op, f.name))
    return dict(op=op_json, arguments=json.loads(self.autotuning_cache_key.to_json()))

  def replace(self, **kwargs) -> "BoundArguments":
    return dataclasses.replace(self, **kwargs)


_SCALARS = (str, int, float, bool, torch.dtype)


def _collect_tensors(x, out: list) -> None:
  """Appends every tensor inside `x` to `out` (through containers, dataclasses and objects with a `_leaves()` method; common cases first)."""
  if isinstance(x, torch.Tensor):
    out.append(x)
  elif x is None or isinstance(x, _SCALARS):
    return
  elif isinstance(x, dict):
    for v in x.values():
      _collect_tensors(v, out)
  elif isinstance(x, (tuple, list)):
    for v in x:
      _collect_tensors(v, out)
  elif hasattr(x, "_leaves"):
    for v in x._leaves():  # pylint: disable=protected-access
      _collect_tensors(v, out)
  elif dataclasses.is_dataclass(x) and not isinstance(x, type):
    for f in dataclasses.fields(x):
      _collect_tensors(getattr(x, f.name), out)


def infer_devices(ba: BoundArguments) -> set:
  return {x.device for x in ba.tensors}


def infer_device_kind(ba: BoundArguments) -> DeviceKind | None:
  kinds = {device_kind(d) if d.type == "cuda" else "cpu" for d in infer_devices(ba)}
  if not kinds:
    return None
  if len(kinds) == 1:
    return kinds.pop()
  raise ValueError(f"Multiple device kinds found: {kinds}")


def _call_with_vjp(op: Op, ba: BoundArguments, config, return_residuals: bool):
  """Runs `_fwd` under a torch.autograd.Function whose backward is `op.vjp` (op.py:276-307)."""
  arguments = dict(ba.arguments)
  names = [k for k, v in arguments.items() if isinstance(v, torch.Tensor) and v.is_floating_point()]
  tensors = [arguments[k] for k in names]
  pos_names = [
      n for n, p in ba.signature.parameters.items()
      if p.kind in (p.POSITIONAL_ONLY, p.POSITIONAL_OR_KEYWORD)
  ]

  class _Fn(torch.autograd.Function):

    @staticmethod
    def forward(ctx, *ts):
      full = dict(arguments)
      full.update(zip(names, ts))
      bound = BoundArguments(op, full)
      kwargs = dict(bound.kwargs)
      kwargs["return_residuals"] = True
      out, residuals = op._fwd(*bound.args, config=config, **kwargs)  # pylint: disable=protected-access
      # Inputs and residuals go through save_for_backward, and the output is not kept at all (`vjp` does not use
      # it): a tensor this function returns, held as a plain attribute of ctx, would close the cycle
      # out -> grad_fn -> ctx -> out, and the activations would live until the cyclic collector runs.
      ctx.has_residuals = residuals is not None
      ctx.save_for_backward(*ts, *([residuals] if residuals is not None else []))
      if return_residuals:
        ctx.mark_non_differentiable(residuals)
        return out, residuals
      return out

    @staticmethod
    def backward(ctx, dout, *unused):
      saved = ctx.saved_tensors
      ts, residuals = (saved[:-1], saved[-1]) if ctx.has_residuals else (saved, None)
      full = dict(arguments)
      full.update(zip(names, ts))
      bound = BoundArguments(op, full)
      kwargs = dict(bound.kwargs)
      kwargs.pop("return_residuals")
      with torch.no_grad():
        grads = op.vjp(residuals, None, dout, *bound.args, **kwargs)
      by_name = dict(grads) if isinstance(grads, dict) else dict(zip(pos_names, grads))
      return tuple(by_name.get(n) for n in names)

  return _Fn.apply(*tensors)
