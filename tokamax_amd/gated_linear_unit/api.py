"""Gated linear unit API (tokamax/_src/ops/gated_linear_unit/api.py:28-110): registry and fallback."""

from __future__ import annotations

import types
from typing import Any, Callable, Sequence

from exceptiongroup import ExceptionGroup

from tokamax_amd.gated_linear_unit import hip

_IMPLEMENTATIONS: dict[str, Callable[..., Any]] = dict(hip=hip.HipGatedLinearUnit())
_DEFAULT_IMPLEMENTATIONS: tuple[str, ...] = ("hip",)
IMPLEMENTATIONS = types.MappingProxyType(_IMPLEMENTATIONS)


def gated_linear_unit(x, weights, *, activation=None, precision=None,
                      implementation: str | Sequence[str | Callable[..., Any]] | None = None):
  """`activation(x @ w_gate) * (x @ w_up)` for `x [*B, M, K]` and fused weights `[K, 2, N]` or a
  `(w_gate, w_up)` pair of `[K, N]` arrays. SwiGLU with `activation=torch.nn.functional.silu`, GEGLU with
  a tanh gelu, ReGLU with `torch.relu`, GLU with `torch.sigmoid`, bilinear with `None`."""
  if implementation is None:
    implementation = _DEFAULT_IMPLEMENTATIONS
  if isinstance(implementation, str) or callable(implementation):
    implementation = (implementation,)
  errors = []
  for impl in implementation:
    if isinstance(impl, str):
      if impl not in IMPLEMENTATIONS:
        raise ValueError(f"Unknown implementation: {impl}")
      impl = IMPLEMENTATIONS[impl]
    try:
      return impl(x, weights, activation=activation, precision=precision)
    except NotImplementedError as e:
      if len(implementation) == 1:
        raise
      errors.append(e)
  raise ExceptionGroup("all implementations failed", errors)
