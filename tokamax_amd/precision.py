"""Precision vocabulary of the operator API.

Restates the part of tokamax/_src/precision.py (:72-101 `canonicalize_precision`, `is_default`)
that `RaggedDot.bind` needs, without JAX: `Precision` and `DotAlgorithmPreset` are local enums
with the member names of `jax.lax.Precision` / `jax.lax.DotAlgorithmPreset`.
"""

from __future__ import annotations

import enum
from typing import Tuple, Union

import torch


class Precision(enum.Enum):
  DEFAULT = 0
  HIGH = 1
  HIGHEST = 2

  @classmethod
  def _missing_(cls, value):
    aliases = {"default": cls.DEFAULT, "fastest": cls.DEFAULT, "bfloat16": cls.DEFAULT, "high": cls.HIGH,
               "bfloat16_3x": cls.HIGH, "tensorfloat32": cls.HIGH, "highest": cls.HIGHEST, "float32": cls.HIGHEST}
    if isinstance(value, str) and value.lower() in aliases:
      return aliases[value.lower()]
    if isinstance(value, str) and value in cls.__members__:
      return cls[value]
    return None


class DotAlgorithmPreset(enum.Enum):
  DEFAULT = enum.auto()
  F16_F16_F16 = enum.auto()
  F16_F16_F32 = enum.auto()
  BF16_BF16_BF16 = enum.auto()
  BF16_BF16_F32 = enum.auto()
  BF16_BF16_F32_X3 = enum.auto()
  BF16_BF16_F32_X6 = enum.auto()
  BF16_BF16_F32_X9 = enum.auto()
  TF32_TF32_F32 = enum.auto()
  TF32_TF32_F32_X3 = enum.auto()
  F32_F32_F32 = enum.auto()
  F64_F64_F64 = enum.auto()
  ANY_F8_ANY_F8_F32 = enum.auto()


CanonicalPrecision = Union[Tuple[Precision, Precision], DotAlgorithmPreset]


def canonicalize_precision(precision) -> CanonicalPrecision:
  """Follows tokamax/_src/precision.py:72-101."""
  if precision is None:
    return Precision.DEFAULT, Precision.DEFAULT
  if isinstance(precision, str):
    if precision in DotAlgorithmPreset.__members__:
      return DotAlgorithmPreset[precision]
    try:
      return (Precision(precision),) * 2
    except ValueError:
      raise ValueError(
          f"Unsupported enum value: {precision}. Must be refer to either a `DotAlgorithmPreset` or a `Precision` enum."
      ) from None
  if isinstance(precision, Precision):
    return precision, precision
  if isinstance(precision, DotAlgorithmPreset):
    return precision
  if isinstance(precision, (list, tuple)) and len(precision) == 2:
    p0, p1 = precision
    if isinstance(p0, Precision) and isinstance(p1, Precision):
      return p0, p1
    if isinstance(p0, str) and isinstance(p1, str):
      return Precision(p0), Precision(p1)
  raise ValueError(f"Invalid precision: {precision}")


def is_default(a_dtype: torch.dtype, b_dtype: torch.dtype, precision: CanonicalPrecision) -> bool:
  """True if `precision` asks for nothing beyond what the native MFMA of these dtypes gives.

  On gfx950 the f32 kernel uses the true-f32 MFMA, so every `Precision` level is met for f32
  inputs; bf16/f16/fp8 inputs are multiplied exactly and accumulated in f32.
  """
  if isinstance(precision, tuple):
    return True
  if precision == DotAlgorithmPreset.DEFAULT:
    return True
  if a_dtype == b_dtype == torch.bfloat16:
    return precision == DotAlgorithmPreset.BF16_BF16_F32
  if a_dtype == b_dtype == torch.float16:
    return precision == DotAlgorithmPreset.F16_F16_F32
  if a_dtype == b_dtype == torch.float32:
    return precision == DotAlgorithmPreset.F32_F32_F32
  return False
