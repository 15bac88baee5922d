"""Quantised-array containers of the operator API.

`QArray` restates the fields of `qwix.QArray` that the reference's kernels read (`qvalue`,
`scale`, `zero_point`, `qtype`; tokamax/_src/quantization.py:25, and its use in
tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:45-75). `scale.shape[i]` divides
`qvalue.shape[i]`; each scale entry covers a tile of `qvalue.shape[i] // scale.shape[i]` entries.
`AsQArray` (quantization.py:39-78) asks for quantisation inside the kernel; the hip implementation
does not quantise on the fly and rejects it with `NotImplementedError`.
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


@dataclasses.dataclass(frozen=True)
class AsQArray:
  """An array to be quantised before the computation (unsupported by the hip kernels)."""

  value: Any
  qtype: torch.dtype
  channelwise_axes: Collection[int] = ()
  tiled_axes: Mapping[int, int | float] | None = None
  calibration_method: str = "absmax"

  shape = property(lambda self: tuple(self.value.shape))
  dtype = property(lambda self: self.value.dtype)
  ndim = property(lambda self: len(self.value.shape))
