"""Ragged dot base class: argument binding, group sizes, VJP wiring.

Restates tokamax/_src/ops/ragged_dot/base.py for torch tensors:
  * the three dimension-number sets (:40-54),
  * `GroupSizes` (:60-168) and `generate_group_sizes` (:171-196),
  * `RaggedDot.bind` (:226-288),
  * `vjp` (:363-462): dlhs = dout . rhs[g]^T, drhs[g] = lhs[rows_g]^T . dout[rows_g].
In the reference, `RaggedDot._fwd` is the XLA implementation (`jax.lax.ragged_dot_general`). That
implementation belongs to JAX and is not part of this package: here the base class has no compute
path of its own, so its `_fwd` raises `NotImplementedError` and `HipRaggedDot` is the only backend.
"""

from __future__ import annotations

import dataclasses
import functools
from typing import Any, Callable, Sequence

import numpy as np
import torch

from tokamax_amd import op
from tokamax_amd import precision as precision_lib
from tokamax_amd import quantization
from tokamax_amd import serialization

QArray = quantization.QArray
AsQArray = quantization.AsQArray
ShapeDtype = serialization.ShapeDtype
CanonicalPrecision = precision_lib.CanonicalPrecision
Residuals = Any
ActivationFunction = Callable[[torch.Tensor], torch.Tensor]


def _tuple2(x):
  return tuple(tuple(int(i) for i in d) for d in x)


@dataclasses.dataclass(frozen=True)
class RaggedDotDimensionNumbers:
  """Same fields as `jax.lax.RaggedDotDimensionNumbers`."""

  dot_dimension_numbers: Any  # ((lhs_contract, rhs_contract), (lhs_batch, rhs_batch))
  lhs_ragged_dimensions: Sequence[int]
  rhs_group_dimensions: Sequence[int]

  def __post_init__(self):
    (lc, rc), (lb, rb) = self.dot_dimension_numbers
    object.__setattr__(self, "dot_dimension_numbers", (_tuple2((lc, rc)), _tuple2((lb, rb))))
    object.__setattr__(self, "lhs_ragged_dimensions", tuple(int(i) for i in self.lhs_ragged_dimensions))
    object.__setattr__(self, "rhs_group_dimensions", tuple(int(i) for i in self.rhs_group_dimensions))

  def _to_jsonable(self):
    return dict(
        dot_dimension_numbers=[[list(d) for d in pair] for pair in self.dot_dimension_numbers],
        lhs_ragged_dimensions=list(self.lhs_ragged_dimensions),
        rhs_group_dimensions=list(self.rhs_group_dimensions),
    )

  @classmethod
  def from_json(cls, d) -> "RaggedDotDimensionNumbers":
    return cls(d["dot_dimension_numbers"], d["lhs_ragged_dimensions"], d["rhs_group_dimensions"])


DEFAULT_RAGGED_DOT_DIM_NUMS = RaggedDotDimensionNumbers((([1], [1]), ([], [])), [0], [0])
TRANS_RHS_RAGGED_DOT_DIM_NUMS = RaggedDotDimensionNumbers((([1], [2]), ([], [])), [0], [0])
RAGGED_CONTRACTING_DOT_DIM_NUMS = RaggedDotDimensionNumbers((([0], [0]), ([], [])), [0], [])


def generate_group_sizes(*, m: int, num_groups: int, p: Sequence[float] | None = None, seed: int = 0) -> tuple[int, ...]:
  """Random group sizes: `m` draws over `num_groups` groups, counted (base.py:171-196)."""
  if p is None:
    return _uniform_group_sizes(m, num_groups, seed)
  rng = np.random.default_rng(seed)
  group_ids = rng.choice(num_groups, (m,), p=p, replace=True)
  return tuple(map(int, np.bincount(group_ids, minlength=num_groups)))


@functools.lru_cache(maxsize=256)
def _uniform_group_sizes(m: int, num_groups: int, seed: int) -> tuple[int, ...]:
  # Memoised: the abstract form of a GroupSizes argument asks for this on every op call.
  rng = np.random.default_rng(seed)
  group_ids = rng.choice(num_groups, (m,), p=None, replace=True)
  return tuple(map(int, np.bincount(group_ids, minlength=num_groups)))


class GroupSizes:
  """A group sizes array with representative values (base.py:60-168).

  `value` is the real array (a tensor, or a NumPy array when built from an abstract spec);
  `repr_value_or_total_size` is either a representative sequence of sizes or the total number of
  rows, and is what equality, hashing and serialisation use: the real values change every step.
  """

  __slots__ = ("value", "repr_value_or_total_size")

  def __init__(self, value, repr_value_or_total_size: Sequence[int] | int):
    dtype = value.dtype
    if isinstance(dtype, torch.dtype):
      is_int = not dtype.is_floating_point and not dtype.is_complex and dtype != torch.bool
    else:
      is_int = np.issubdtype(dtype, np.integer)
    if not is_int:
      raise ValueError("Group sizes must be integers.")
    (num_groups,) = value.shape
    if not isinstance(repr_value_or_total_size, int):
      if len(repr_value_or_total_size) != num_groups:
        raise ValueError("Representative value must have same length as the group sizes.")
      repr_value_or_total_size = tuple(int(x) for x in repr_value_or_total_size)
    if isinstance(value, ShapeDtype):
      if isinstance(repr_value_or_total_size, int):
        representative = generate_group_sizes(m=repr_value_or_total_size, num_groups=num_groups)
      else:
        representative = repr_value_or_total_size
      value = np.asarray(representative, np.int32)
    object.__setattr__(self, "value", value)
    object.__setattr__(self, "repr_value_or_total_size", repr_value_or_total_size)

  def __setattr__(self, *a):
    raise dataclasses.FrozenInstanceError("GroupSizes is immutable")

  @property
  def representative_value(self) -> tuple[int, ...]:
    if isinstance(self.repr_value_or_total_size, int):
      assert isinstance(self.value, np.ndarray)
      return tuple(map(int, self.value))
    return self.repr_value_or_total_size

  @property
  def shape(self):
    return tuple(self.value.shape)

  def __eq__(self, other) -> bool:
    return (isinstance(other, GroupSizes) and tuple(self.value.shape) == tuple(other.value.shape)
            and self.repr_value_or_total_size == other.repr_value_or_total_size)

  def __hash__(self) -> int:
    return hash((tuple(self.value.shape), self.repr_value_or_total_size))

  def __repr__(self):
    return f"GroupSizes(num_groups={self.value.shape[0]}, repr={self.repr_value_or_total_size})"

  def _leaves(self):
    yield self.value

  def _abstractify(self):
    return GroupSizes(ShapeDtype(tuple(self.value.shape), torch.int32), self.repr_value_or_total_size)

  def _to_jsonable(self):
    if isinstance(self.repr_value_or_total_size, int):
      return dict(num_groups=int(self.value.shape[0]), total_size=self.repr_value_or_total_size)
    return list(self.representative_value)

  @classmethod
  def from_json(cls, x) -> "GroupSizes":
    if isinstance(x, dict):
      return cls(ShapeDtype((x["num_groups"],), torch.int32), int(x["total_size"]))
    return cls(ShapeDtype((len(x),), torch.int32), tuple(x))

  def to_tensor(self, device) -> torch.Tensor:
    v = self.value
    if isinstance(v, torch.Tensor):
      return v
    return torch.as_tensor(np.asarray(v, np.int32), device=device)


@dataclasses.dataclass(frozen=True)
class RaggedDot(op.Op):
  """Ragged dot base class (MegaBlocks-style grouped matmul)."""

  _: dataclasses.KW_ONLY
  checkify_group_sizes: bool = False

  def bind(  # pylint: disable=arguments-differ
      self,
      lhs,
      rhs,
      *,
      group_sizes,
      ragged_dot_dimension_numbers: RaggedDotDimensionNumbers | None = None,
      precision=None,
      preferred_element_type=None,
      return_residuals: bool = False,
      group_offset=None,
      activation: ActivationFunction | None = None,
      manual_axis_type=None,
      rhs_scale=None,
      rhs_bias=None,
      maybe_quantize_lhs: bool = False,
      zero_initialize: bool = True,
      fuse_gateup_activation: str | None = None,
      lhs_quantization_dtype=None,
      rhs_quantization_dtype=None,
  ) -> op.BoundArguments:
    if ragged_dot_dimension_numbers is None:
      ragged_dot_dimension_numbers = DEFAULT_RAGGED_DOT_DIM_NUMS

    if isinstance(group_sizes, (list, tuple)):
      group_sizes = tuple(int(g) for g in group_sizes)
      device = lhs.device if isinstance(lhs, torch.Tensor) else None
      group_sizes = GroupSizes(torch.tensor(group_sizes, dtype=torch.int32, device=device), group_sizes)

    if ragged_dot_dimension_numbers == DEFAULT_RAGGED_DOT_DIM_NUMS:
      if not isinstance(group_sizes, GroupSizes):
        group_sizes = GroupSizes(group_sizes, int(lhs.shape[0]))
      if self.checkify_group_sizes and isinstance(group_sizes.value, torch.Tensor):
        gs = group_sizes.value
        # The reference records these with checkify (base.py:262-266); eager mode can raise directly.
        if bool((gs.to(torch.int64) < 0).any()):
          raise ValueError("Negative group size.")
        if int(gs.to(torch.int64).sum()) > lhs.shape[0]:
          raise ValueError("Group size sum > num rows.")

    if preferred_element_type is not None:
      preferred_element_type = serialization.as_dtype(preferred_element_type)
    return self._bind_all(
        lhs=lhs,
        rhs=rhs,
        group_sizes=group_sizes,
        ragged_dot_dimension_numbers=ragged_dot_dimension_numbers,
        precision=precision_lib.canonicalize_precision(precision),
        preferred_element_type=preferred_element_type,
        return_residuals=return_residuals,
        group_offset=group_offset,
        activation=activation,
        manual_axis_type=manual_axis_type,
        rhs_scale=rhs_scale,
        rhs_bias=rhs_bias,
        maybe_quantize_lhs=maybe_quantize_lhs,
        zero_initialize=zero_initialize,
        fuse_gateup_activation=fuse_gateup_activation,
        lhs_quantization_dtype=lhs_quantization_dtype,
        rhs_quantization_dtype=rhs_quantization_dtype,
    )

  def _fwd(
      self,
      lhs,
      rhs,
      *,
      group_sizes,
      ragged_dot_dimension_numbers: RaggedDotDimensionNumbers,
      precision: CanonicalPrecision,
      preferred_element_type: torch.dtype | None,
      return_residuals: bool,
      config,
      activation: ActivationFunction | None = None,
      manual_axis_type=None,
      group_offset=None,
      rhs_scale=None,
      rhs_bias=None,
      maybe_quantize_lhs: bool = False,
      zero_initialize: bool = True,
      fuse_gateup_activation: str | None = None,
      lhs_quantization_dtype=None,
      rhs_quantization_dtype=None,
  ):
    raise NotImplementedError(
        "The base implementation of the reference is jax.lax.ragged_dot_general (XLA); it is not part of"
        " this package. Use implementation='hip'."
    )

  def arg_spec_from_json(self, spec: dict) -> dict:
    """Turns one parsed cache-file key back into `bind` keyword arguments (abstract arrays)."""
    out = dict(spec)
    for name in ("lhs", "rhs", "group_offset", "rhs_scale", "rhs_bias"):
      if name in out:
        out[name] = serialization.array_spec_from_json(out[name])
    if "group_sizes" in out:
      # Wrapped in `GroupSizes` only under the default dimension numbers (see `bind`); a plain array otherwise.
      gs = out["group_sizes"]
      out["group_sizes"] = serialization.array_spec_from_json(gs) if isinstance(gs, str) else GroupSizes.from_json(gs)
    if out.get("ragged_dot_dimension_numbers") is not None:
      out["ragged_dot_dimension_numbers"] = RaggedDotDimensionNumbers.from_json(out["ragged_dot_dimension_numbers"])
    if isinstance(out.get("precision"), list):
      out["precision"] = tuple(out["precision"])
    for name in ("preferred_element_type", "lhs_quantization_dtype", "rhs_quantization_dtype"):
      if out.get(name) is not None:
        out[name] = serialization.as_dtype(out[name])
    if isinstance(out.get("activation"), str):
      out["activation"] = _ACTIVATION_BY_NAME.get(out["activation"], out["activation"])
    return out


_ACTIVATION_BY_NAME: dict[str, Callable] = {}


def vjp(
    residuals,
    out,
    dout,
    lhs,
    rhs,
    *,
    group_sizes,
    ragged_dot_dimension_numbers: RaggedDotDimensionNumbers,
    precision: CanonicalPrecision,
    preferred_element_type: torch.dtype | None,
    activation: ActivationFunction | None = None,
    dlhs_ragged_dot: Callable[..., torch.Tensor],
    drhs_ragged_dot: Callable[..., torch.Tensor],
    manual_axis_type=None,
    group_offset=None,
    rhs_scale=None,
    rhs_bias=None,
    maybe_quantize_lhs: bool = False,
    zero_initialize: bool = True,
    fuse_gateup_activation: str | None = None,
    lhs_quantization_dtype=None,
    rhs_quantization_dtype=None,
):
  """Ragged dot VJP (base.py:363-462)."""
  del out, preferred_element_type, manual_axis_type

  if (group_offset is not None or rhs_scale is not None or rhs_bias is not None or maybe_quantize_lhs
      or not zero_initialize or fuse_gateup_activation is not None or lhs_quantization_dtype is not None
      or rhs_quantization_dtype is not None):
    raise NotImplementedError(
        "group_offset, rhs_scale, rhs_bias, maybe_quantize_lhs, zero_initialize, fuse_gateup_activation,"
        " lhs_quantization_dtype, rhs_quantization_dtype are not supported on the ragged_dot backward path"
        " for now."
    )
  if isinstance(lhs, (QArray, AsQArray)) or isinstance(rhs, (QArray, AsQArray)):
    raise NotImplementedError("Quantised inputs are not supported on the ragged_dot backward path.")

  if activation is not None:
    # d(activation)/d(residuals) applied to dout, as `jax.vjp(activation, residuals)` does (base.py:412-414).
    with torch.enable_grad():
      r = residuals.detach().requires_grad_(True)
      a = activation(r)
    (dout,) = torch.autograd.grad(a, r, dout.to(a.dtype))

  # The two cotangents are ragged dots again (base.py:416-461 derives their dimension numbers from the forward's
  # in general). The kernels here know three layouts, so the derivation is a table: for each forward layout, the
  # operands and the layout of the product that yields each cotangent.
  try:
    (dlhs_a, dlhs_b, dlhs_dims), (drhs_a, drhs_b, drhs_dims) = _COTANGENT_PRODUCTS[ragged_dot_dimension_numbers]
  except KeyError:
    raise NotImplementedError("Unsupported ragged dot dimension numbers on the backward path.") from None
  operands = {"lhs": lhs, "rhs": rhs, "dout": dout}
  dlhs = dlhs_ragged_dot(operands[dlhs_a], operands[dlhs_b], group_sizes=group_sizes,
                         ragged_dot_dimension_numbers=dlhs_dims, precision=precision, preferred_element_type=lhs.dtype)
  drhs = drhs_ragged_dot(operands[drhs_a], operands[drhs_b], group_sizes=group_sizes,
                         ragged_dot_dimension_numbers=drhs_dims, precision=precision, preferred_element_type=rhs.dtype)
  return dlhs, drhs


# forward layout -> ((first operand, second operand, layout) for d lhs, the same for d rhs)
_COTANGENT_PRODUCTS = {
    # out[m,n] = lhs[m,k] . rhs[g,k,n]:  dlhs[m,k] = dout[m,n] . rhs[g,k,n]^T,  drhs[g,k,n] = lhs[rows_g]^T . dout[rows_g]
    DEFAULT_RAGGED_DOT_DIM_NUMS: (("dout", "rhs", TRANS_RHS_RAGGED_DOT_DIM_NUMS),
                                  ("lhs", "dout", RAGGED_CONTRACTING_DOT_DIM_NUMS)),
    # out[m,k] = lhs[m,n] . rhs[g,k,n]^T:  dlhs[m,n] = dout[m,k] . rhs[g,k,n],  drhs[g,k,n] = dout[rows_g]^T . lhs[rows_g]
    TRANS_RHS_RAGGED_DOT_DIM_NUMS: (("dout", "rhs", DEFAULT_RAGGED_DOT_DIM_NUMS),
                                    ("dout", "lhs", RAGGED_CONTRACTING_DOT_DIM_NUMS)),
    # out[g,k,n] = lhs[rows_g,k]^T . rhs[rows_g,n]:  dlhs[m,k] = rhs[m,n] . dout[g,k,n]^T,  drhs[m,n] = lhs[m,k] . dout[g,k,n]
    RAGGED_CONTRACTING_DOT_DIM_NUMS: (("rhs", "dout", TRANS_RHS_RAGGED_DOT_DIM_NUMS),
                                      ("lhs", "dout", DEFAULT_RAGGED_DOT_DIM_NUMS)),
}
