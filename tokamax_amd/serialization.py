"""Abstract array specs and the JSON form of argument specs.

The JSON schema is the one the reference writes into its autotuning caches
(tokamax/_src/pydantic.py:266-376; e.g. tokamax/data/autotuning/nvidia_h100_80gb_hbm3/
pallas_mosaic_gpu_ragged_dot.json:1-18): arrays as `"bf16[131072,7168]"`, enums by name, dtypes by
name, group sizes as `{"num_groups": G, "total_size": m}` or a list of ints, quantised arrays as
`{"qvalue": ..., "scale": ..., "zero_point": ..., "qtype": "jax.numpy.<name>"}`.
"""

from __future__ import annotations

import dataclasses
import enum
import re
from typing import Any

import torch

from tokamax_amd import quantization

SHORT_DTYPE_NAMES = {
    "bool": torch.bool,
    "i8": torch.int8,
    "i16": torch.int16,
    "i32": torch.int32,
    "i64": torch.int64,
    "u8": torch.uint8,
    "u16": torch.uint16,
    "u32": torch.uint32,
    "u64": torch.uint64,
    "f16": torch.float16,
    "f32": torch.float32,
    "f64": torch.float64,
    "bf16": torch.bfloat16,
    "f8_e4m3fn": torch.float8_e4m3fn,
    "f8_e5m2": torch.float8_e5m2,
    "f8_e4m3fnuz": torch.float8_e4m3fnuz,
    "f8_e5m2fnuz": torch.float8_e5m2fnuz,
}
_SHORT_OF = {v: k for k, v in SHORT_DTYPE_NAMES.items()}
# numpy-style long names, as the reference prints dtypes (`preferred_element_type: "bfloat16"`).
LONG_DTYPE_NAMES = {
    "bool": torch.bool, "int8": torch.int8, "int16": torch.int16, "int32": torch.int32, "int64": torch.int64,
    "uint8": torch.uint8, "uint16": torch.uint16, "uint32": torch.uint32, "uint64": torch.uint64,
    "float16": torch.float16, "float32": torch.float32, "float64": torch.float64, "bfloat16": torch.bfloat16,
    "float8_e4m3fn": torch.float8_e4m3fn, "float8_e5m2": torch.float8_e5m2,
    "float8_e4m3fnuz": torch.float8_e4m3fnuz, "float8_e5m2fnuz": torch.float8_e5m2fnuz,
}
# (sub-byte integers, where this torch names them: the qtype of an int4 QArray, "int4" in the reference's keys too)
LONG_DTYPE_NAMES.update({f"{u}int{b}": getattr(torch, f"{u}int{b}") for u in ("", "u") for b in range(1, 8)
                         if hasattr(torch, f"{u}int{b}")})
_LONG_OF = {v: k for k, v in LONG_DTYPE_NAMES.items()}


def as_dtype(x) -> torch.dtype:
  """torch.dtype from a torch.dtype, a short name ('bf16') or a long name ('bfloat16')."""
  if isinstance(x, torch.dtype):
    return x
  if isinstance(x, str):
    name = x.rsplit(".", 1)[-1]
    if name in LONG_DTYPE_NAMES:
      return LONG_DTYPE_NAMES[name]
    if name in SHORT_DTYPE_NAMES:
      return SHORT_DTYPE_NAMES[name]
  raise ValueError(f"unknown dtype: {x!r}")


def dtype_name(dtype) -> str:
  return dtype if isinstance(dtype, str) else _LONG_OF[dtype]


@dataclasses.dataclass(frozen=True)
class ShapeDtype:
  """Shape and dtype of an array, without data (the role of jax.ShapeDtypeStruct)."""

  shape: tuple[int, ...]
  dtype: torch.dtype

  def __post_init__(self):
    object.__setattr__(self, "shape", tuple(int(d) for d in self.shape))
    object.__setattr__(self, "dtype", as_dtype(self.dtype))

  @property
  def ndim(self) -> int:
    return len(self.shape)

  def short_str(self) -> str:
    return f"{_SHORT_OF[self.dtype]}[{','.join(map(str, self.shape))}]"

  _PATTERN = re.compile(r"^(.*?)\[(.*?)\]$")

  @classmethod
  def parse(cls, s: str) -> "ShapeDtype":
    m = cls._PATTERN.match(s)
    if m is None or m.group(1) not in SHORT_DTYPE_NAMES:
      raise ValueError(f"Invalid ShapeDtype: {s}")
    dims = [int(d) for d in m.group(2).split(",") if d.strip()]
    return cls(tuple(dims), SHORT_DTYPE_NAMES[m.group(1)])


def is_array(x) -> bool:
  return isinstance(x, torch.Tensor)


def abstractify(x):
  """Replaces arrays by `ShapeDtype` (recursively through the containers used in arguments)."""
  if isinstance(x, torch.Tensor):
    return ShapeDtype(tuple(x.shape), x.dtype)
  if isinstance(x, quantization.QArray):
    return quantization.QArray(abstractify(x.qvalue), abstractify(x.scale), abstractify(x.zero_point), x.qtype)
  if isinstance(x, quantization.AsQArray):
    return dataclasses.replace(x, value=abstractify(x.value))
  if hasattr(x, "_abstractify"):
    return x._abstractify()  # pylint: disable=protected-access
  if isinstance(x, tuple):
    return tuple(abstractify(v) for v in x)
  if isinstance(x, list):
    return [abstractify(v) for v in x]
  if isinstance(x, dict):
    return {k: abstractify(v) for k, v in x.items()}
  return x


def to_jsonable(x) -> Any:
  """The JSON-ready form of one (abstract) argument value."""
  if x is None or isinstance(x, (bool, int, float, str)):
    return x
  if isinstance(x, torch.Tensor):
    return ShapeDtype(tuple(x.shape), x.dtype).short_str()
  if isinstance(x, ShapeDtype):
    return x.short_str()
  if isinstance(x, torch.dtype):
    return dtype_name(x)
  if isinstance(x, enum.Enum):
    return x.name
  if isinstance(x, quantization.QArray):
    return dict(qvalue=to_jsonable(x.qvalue), scale=to_jsonable(x.scale), zero_point=to_jsonable(x.zero_point),
                qtype=f"jax.numpy.{dtype_name(x.qtype)}")
  if hasattr(x, "_to_jsonable"):
    return x._to_jsonable()  # pylint: disable=protected-access
  if dataclasses.is_dataclass(x):
    return {f.name: to_jsonable(getattr(x, f.name)) for f in dataclasses.fields(x)}
  if isinstance(x, (tuple, list)):
    return [to_jsonable(v) for v in x]
  if isinstance(x, dict):
    return {k: to_jsonable(v) for k, v in x.items()}
  if callable(x):
    return f"{getattr(x, '__module__', '')}.{getattr(x, '__qualname__', repr(x))}"
  raise TypeError(f"cannot serialise {type(x).__name__}: {x!r}")


def array_spec_from_json(v):
  """Parses `"bf16[m,k]"` or a quantised-array dict; leaves anything else untouched."""
  if isinstance(v, str):
    try:
      return ShapeDtype.parse(v)
    except ValueError:
      return v
  if isinstance(v, dict) and set(v) >= {"qvalue", "scale"}:
    qtype = v.get("qtype")
    return quantization.QArray(
        array_spec_from_json(v["qvalue"]),
        array_spec_from_json(v["scale"]),
        array_spec_from_json(v.get("zero_point")),
        as_dtype(qtype) if qtype is not None else None,
    )
  return v
