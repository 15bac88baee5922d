"""Quantised-array containers of the operator API.

`QArray` restates the fields of `qwix.QArray` that the reference's kernels read (`qvalue`,
`scale`, `zero_point`, `qtype`; tokamax/_src/quantization.py:25, and its use in
tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:45-75). `scale.shape[i]` divides
`qvalue.shape[i]`; each scale entry covers a tile of `qvalue.shape[i] // scale.shape[i]` entries.
`AsQArray` (quantization.py:39-78) asks for quantisation on the fly: `as_qarray` runs the absmax
quantisation kernel of the HIP library; `as_array_or_qarray_without_zero_point` (:85-93) dequantises
operands that carry a zero point, which no kernel takes.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Collection, Mapping

import torch


@dataclasses.dataclass(frozen=True)
class QArray:
  qvalue: Any  # torch.Tensor or ShapeDtype
  scale: Any
  zero_point: Any = None
  qtype: torch.dtype | None = None

  def __post_init__(self):
    if self.qtype is None:
      object.__setattr__(self, "qtype", self.qvalue.dtype)

  def _fast_signature(self):
    """Structural stand-in used by the op's config memo (shapes, dtypes, devices)."""
    sig = lambda t: None if t is None else (tuple(t.shape), t.dtype, getattr(t, "device", None))
    return ("QArray", sig(self.qvalue), sig(self.scale), sig(self.zero_point), self.qtype)

  shape = property(lambda self: tuple(self.qvalue.shape))
  dtype = property(lambda self: self.scale.dtype)  # the dtype it dequantises to
  ndim = property(lambda self: len(self.qvalue.shape))

  @property
  def scale_tile_shape(self) -> tuple[int, ...]:
    return tuple(q // s for q, s in zip(self.qvalue.shape, self.scale.shape))


@dataclasses.dataclass(frozen=True, eq=False)
class AsQArray:
  """An array to be quantised before the computation (quantization.py:39-78).

  `channelwise_axes` get one scale per index, `tiled_axes` ({axis: tile size, or a fraction of the axis}) one per
  tile, every other axis shares its scale: the arguments of `qwix.quantize`, whose "absmax" calibration
  `as_qarray` runs on the device (scale = absmax / qmax, values rounded to nearest even)."""

  value: Any
  qtype: torch.dtype
  channelwise_axes: Collection[int] = ()
  tiled_axes: Mapping[int, int | float] | None = None
  calibration_method: str = "absmax"

  shape = property(lambda self: tuple(self.value.shape))
  dtype = property(lambda self: self.value.dtype)
  ndim = property(lambda self: len(self.value.shape))

  def _key(self):
    tiled = None if self.tiled_axes is None else tuple(sorted(self.tiled_axes.items()))
    value = self.value if not isinstance(self.value, torch.Tensor) else id(self.value)  # (arrays compare by identity)
    return (value, self.qtype, tuple(self.channelwise_axes), tiled, self.calibration_method)

  def __eq__(self, other):
    return isinstance(other, AsQArray) and self._key() == other._key()

  def __hash__(self):
    return hash(self._key())

  @property
  def tile_shape(self) -> tuple[int, ...]:
    """Entries of `value` per scale along every axis."""
    shape = self.shape
    tile = list(shape)
    for ax in self.channelwise_axes:
      tile[ax % len(shape)] = 1
    for ax, t in (self.tiled_axes or {}).items():
      ax %= len(shape)
      size = int(round(shape[ax] * t)) if isinstance(t, float) and t < 1 else int(t)
      if size < 1 or shape[ax] % size:
        raise ValueError(f"tile size {t} does not divide axis {ax} of {shape}")
      tile[ax] = size
    return tuple(tile)

  @property
  def scale_shape(self) -> tuple[int, ...]:
    return tuple(d // t for d, t in zip(self.shape, self.tile_shape))

  def _fast_signature(self):
    return ("AsQArray", tuple(self.value.shape), self.value.dtype, getattr(self.value, "device", None), self.qtype,
            self.tile_shape, self.calibration_method)

  def abstract_qarray(self) -> QArray:
    """The shapes and types `as_qarray` returns, without running it."""
    from tokamax_amd.serialization import ShapeDtype  # pylint: disable=g-import-not-at-top
    storage = torch.float8_e4m3fn if self.qtype == torch.float8_e4m3fn else torch.int8
    return QArray(ShapeDtype(self.shape, storage), ShapeDtype(self.scale_shape, torch.float32), None, self.qtype)

  def as_qarray(self) -> QArray:
    """Quantises `value` on the device (the HIP kernel behind `tkx_quantize`)."""
    if self.calibration_method != "absmax":
      raise NotImplementedError(f"calibration method {self.calibration_method!r} is not supported (absmax only)")
    from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
    qvalue, scale = hip_ops.quantize(self.value, self.qtype, self.tile_shape)
    return QArray(qvalue, scale, None, self.qtype)


def as_array_or_qarray(x):
  """An `AsQArray` quantised, anything else as it is (quantization.py:80-83)."""
  return x.as_qarray() if isinstance(x, AsQArray) else x


def as_array_or_qarray_without_zero_point(x):
  """As above, and a quantised array with a zero point dequantised to bf16, `(qvalue - zero_point) * scale`
  (quantization.py:85-93: none of the kernels takes a zero point)."""
  y = as_array_or_qarray(x)
  if isinstance(y, QArray) and y.zero_point is not None:
    from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
    return hip_ops.dequantize(y.qvalue, y.scale, y.zero_point)
  return y
