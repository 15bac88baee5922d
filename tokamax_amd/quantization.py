"""Quantised-array containers of the operator API.

`QArray` restates the fields of `qwix.QArray` that the reference's kernels read (`qvalue`,
`scale`, `zero_point`, `qtype`; tokamax/_src/quantization.py:25, and its use in
tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:45-75). `scale.shape[i]` divides
`qvalue.shape[i]`; each scale entry covers a tile of `qvalue.shape[i] // scale.shape[i]` entries.
A `QArray` whose `qvalue` is uint8 with `qtype` int4 holds two values per byte along its second-to-last axis (entry
2 i in bits 0-3, entry 2 i + 1 in bits 4-7); its `shape` is the shape of the values, not of the bytes. `pack_int4`
makes one from int4 values in int8 storage. (The reference holds int4 as `jnp.int4` arrays and leaves the packing to
XLA; this is the layout the streaming small-m kernel reads.)
`AsQArray` (quantization.py:39-78) asks for quantisation on the fly: `as_qarray` runs the absmax
quantisation kernel of the HIP library; `as_array_or_qarray_without_zero_point` (:85-93) dequantises
operands that carry a zero point, which no kernel takes.
"""

from __future__ import annotations

import dataclasses
from typing import Any, Collection, Mapping

import torch


# torch builds without an int4 dtype cannot name the type: there `PACKED_INT4` marks a packed array.
PACKED_INT4 = getattr(torch, "int4", "int4x2")
_FOUR_BIT_TYPES = tuple({PACKED_INT4, "int4x2"})


@dataclasses.dataclass(frozen=True)
class QArray:
  qvalue: Any  # torch.Tensor or ShapeDtype
  scale: Any
  zero_point: Any = None
  qtype: torch.dtype | None = None

  def __post_init__(self):
    if self.qtype is None:
      object.__setattr__(self, "qtype", self.qvalue.dtype)
    if self.qvalue.dtype == torch.uint8 and self.qtype not in _FOUR_BIT_TYPES:
      # uint8 storage means one thing here: int4 packed two to a byte. Anything else in bytes would be unpacked as
      # nibbles and give wrong results without a word.
      raise NotImplementedError(f"a uint8 qvalue is packed int4 and needs qtype int4 (got {self.qtype}); other uint8"
                                " quantised types are not supported")

  def _leaves(self):
    return (self.qvalue, self.scale, self.zero_point)

  def _fast_signature(self):
    """Structural stand-in used by the op's config memo (shapes, dtypes, devices)."""
    sig = lambda t: None if t is None else (tuple(t.shape), t.dtype, getattr(t, "device", None))
    return ("QArray", sig(self.qvalue), sig(self.scale), sig(self.zero_point), self.qtype)

  @property
  def packed(self) -> bool:
    """Two int4 values per byte of `qvalue` along its second-to-last axis: uint8 storage under a 4-bit qtype."""
    return self.qvalue.dtype == torch.uint8 and self.qtype in _FOUR_BIT_TYPES

  @property
  def shape(self) -> tuple[int, ...]:
    """The shape of the values (for packed int4: twice the bytes along the second-to-last axis)."""
    shape = tuple(self.qvalue.shape)
    return shape[:-2] + (2 * shape[-2], shape[-1]) if self.packed else shape

  dtype = property(lambda self: self.scale.dtype)  # the dtype it dequantises to
  ndim = property(lambda self: len(self.qvalue.shape))

  @property
  def scale_tile_shape(self) -> tuple[int, ...]:
    return tuple(q // s for q, s in zip(self.shape, self.scale.shape))

  def unpacked(self) -> "QArray":
    """The same values in int8 storage (on arrays: the unpacking kernel; on shapes: the shape it returns)."""
    if not self.packed:
      return self
    if isinstance(self.qvalue, torch.Tensor):
      from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
      return QArray(hip_ops.unpack_int4(self.qvalue), self.scale, self.zero_point, self.qtype)
    return QArray(type(self.qvalue)(self.shape, torch.int8), self.scale, self.zero_point, self.qtype)


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


def pack_int4(q: QArray) -> QArray:
  """`q` (int4 values in int8 storage, an even number of entries along the second-to-last axis) with two values per
  byte along that axis."""
  if q.packed:
    return q
  if q.qvalue.dtype != torch.int8 or q.zero_point is not None:
    raise NotImplementedError("pack_int4 takes int4 values in int8 storage without a zero point")
  from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
  return QArray(hip_ops.pack_int4(q.qvalue), q.scale, None, PACKED_INT4)


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
