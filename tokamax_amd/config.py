"""Configuration options, usable as context managers.

Mirrors the three options of the reference (tokamax/_src/config.py:62-95) with the same names and
meaning. The reference backs them with absl flags + a JAX user context; here the value comes from
a `contextvars` override if one is active, else from the environment variable of the same name
in upper case (e.g. TOKAMAX_AUTOTUNING_CACHE_MISS_FALLBACK), else from the default.
"""

from __future__ import annotations

import contextlib
import contextvars
import os
from typing import Any, Callable, Generic, Sequence, TypeVar

T = TypeVar("T")
_UNSET = object()


def _parse_bool(s: str) -> bool:
  v = s.strip().lower()
  if v in ("1", "true", "t", "yes", "y"):
    return True
  if v in ("0", "false", "f", "no", "n"):
    return False
  raise ValueError(s)


class _ConfigOption(Generic[T]):
  """One option: `opt.value` reads it, `with opt(v):` overrides it in the current context."""

  def __init__(self, name: str, default: T, parser: Callable[[str], T], choices: Sequence[T] | None = None, doc: str = ""):
    self.name = name
    self.default = default
    self._parser = parser
    self._choices = choices
    self.__doc__ = doc
    self._var: contextvars.ContextVar[Any] = contextvars.ContextVar(name, default=_UNSET)

  def _validate(self, value):
    if isinstance(value, str) and self._parser is not str:
      try:
        value = self._parser(value)
      except ValueError as e:
        raise ValueError(f"Invalid value for config `{self.name}`: {value}") from e
    if self._choices is not None and value not in self._choices:
      raise ValueError(f"Invalid value for config `{self.name}`: {value}")
    return value

  @contextlib.contextmanager
  def __call__(self, value: T | str):
    token = self._var.set(self._validate(value))
    try:
      yield
    finally:
      self._var.reset(token)

  @property
  def value(self) -> T:
    v = self._var.get()
    if v is not _UNSET:
      return v
    env = os.environ.get(self.name.upper())
    if env is not None:
      return self._validate(env)
    return self.default


autotuning_cache_miss_fallback: _ConfigOption[str] = _ConfigOption(
    "tokamax_autotuning_cache_miss_fallback",
    "heuristics",
    str,
    choices=("heuristics", "autotune", "error"),
    doc=(
        "Fallback when no config is found in the autotuning cache by `BoundArguments.default_config`"
        " ('heuristics' - use heuristics to create a config; 'autotune' - autotune over the default"
        " autotuning configs and use the fastest; 'error' - raise an error)"
    ),
)

cross_compile: _ConfigOption[bool] = _ConfigOption(
    "tokamax_cross_compile",
    False,
    _parse_bool,
    doc="Disables the checks that the right hardware (a gfx950 GPU) is present.",
)

ignore_autotuning_cache: _ConfigOption[bool] = _ConfigOption(
    "tokamax_ignore_autotuning_cache",
    False,
    _parse_bool,
    doc="If true, ignore the autotuning cache when looking for configs and autotuning.",
)
