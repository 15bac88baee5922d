"""Ragged dot API: implementation registry and ordered fallback.

Restates tokamax/_src/ops/ragged_dot/api.py (:29-73 registry, :77-134 `ragged_dot`, :137-240
`ragged_dot_general`). This package registers a single implementation, "hip"; the reference's own
"xla"/"triton"/"mosaic" backends live in the reference and are not re-created here, so the default
chain is `("hip",)`. Callables may be passed in the `implementation` sequence exactly as in the
reference, which is how a caller chains a fallback of their own.
"""

from __future__ import annotations

import types
from typing import Any, Callable, Sequence

from exceptiongroup import ExceptionGroup

from tokamax_amd.ragged_dot import base
from tokamax_amd.ragged_dot import hip

_IMPLEMENTATIONS: dict[str, Callable[..., Any]] = dict(hip=hip.HipRaggedDot())
_DEFAULT_IMPLEMENTATIONS: tuple[str, ...] = ("hip",)

IMPLEMENTATIONS = types.MappingProxyType(_IMPLEMENTATIONS)


def ragged_dot(
    lhs,
    rhs,
    group_sizes,
    precision=None,
    preferred_element_type=None,
    group_offset=None,
    activation=None,
    manual_axis_type=None,
    *,
    implementation: str | Sequence[str | Callable[..., Any]] | None = None,
):
  """Ragged matrix multiplication: lhs [m,k], rhs [g,k,n], group_sizes [g] -> [m,n].

  Same arguments as the reference's `tokamax.ragged_dot` (api.py:77-134). `activation`, when given,
  is applied in the accumulator dtype before the cast to the output dtype. If a sequence of
  implementations is passed, the first that does not raise `NotImplementedError` is used.
  """
  return ragged_dot_general(
      lhs,
      rhs,
      group_sizes=group_sizes,
      ragged_dot_dimension_numbers=base.DEFAULT_RAGGED_DOT_DIM_NUMS,
      precision=precision,
      preferred_element_type=preferred_element_type,
      group_offset=group_offset,
      activation=activation,
      manual_axis_type=manual_axis_type,
      implementation=implementation,
  )


def ragged_dot_general(
    lhs,
    rhs,
    group_sizes,
    ragged_dot_dimension_numbers: base.RaggedDotDimensionNumbers,
    precision=None,
    preferred_element_type=None,
    group_offset=None,
    activation=None,
    manual_axis_type=None,
    *,
    implementation: str | Sequence[str | Callable[..., Any]] | None = None,
):
  """Ragged matrix multiplication with explicit dimension numbers (api.py:137-240)."""
  if group_offset is not None:
    raise NotImplementedError("`group_offset` is not yet supported.")

  if implementation is None:
    implementation = _DEFAULT_IMPLEMENTATIONS
  elif isinstance(implementation, str):
    implementation = (implementation,)
  elif not implementation:
    raise ValueError("`implementation` must not be an empty sequence.")

  # check that reduction dimensions sizes match
  lhs_contract, rhs_contract = ragged_dot_dimension_numbers.dot_dimension_numbers[0]
  if len(lhs_contract) != len(rhs_contract):
    raise ValueError("contracting dimension lists differ in length")
  for dim1, dim2 in zip(lhs_contract, rhs_contract):
    if lhs.shape[dim1] != rhs.shape[dim2]:
      raise ValueError(
          f"The reduction dimension {dim1} of lhs={tuple(lhs.shape)} equal to {lhs.shape[dim1]} does not match"
          f" the reduction dimension {dim2} of rhs={tuple(rhs.shape)} equal to {rhs.shape[dim2]} for"
          f" ragged_dot_dimension_numbers={ragged_dot_dimension_numbers}."
      )

  errors = []
  for impl in implementation:
    if isinstance(impl, str):
      if impl not in IMPLEMENTATIONS:
        raise ValueError(f"Unknown implementation: {impl}")
      impl = IMPLEMENTATIONS[impl]

    try:
      kwargs = {}
      if manual_axis_type is not None:
        kwargs["manual_axis_type"] = manual_axis_type
      return impl(
          lhs,
          rhs,
          group_sizes=group_sizes,
          ragged_dot_dimension_numbers=ragged_dot_dimension_numbers,
          precision=precision,
          preferred_element_type=preferred_element_type,
          activation=activation,
          **kwargs,
      )
    except NotImplementedError as e:
      if len(implementation) == 1:
        raise
      errors.append(e)

  raise ExceptionGroup("all implementations failed", errors)
