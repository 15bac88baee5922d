"""Benchmark argument specifications for ragged dot.

The shapes of tokamax/_src/ops/ragged_dot/arg_specs.py:23-155 (DeepSeek-V3 / gpt-oss MaxText
shapes, `8x7b`, `compute_bound`, `memory_bound`) plus the five configurations this build is
measured on. FLOP convention: 2 * sum(group_sizes) * k * n (tokamax/_src/ops/ragged_dot/bench.py:52-56).
"""

from __future__ import annotations

import dataclasses
from typing import Any

import torch

from tokamax_amd.ragged_dot import base
from tokamax_amd.serialization import ShapeDtype


@dataclasses.dataclass(frozen=True)
class ArgSpec:
  name: str
  args: dict
  project: str = ""
  tags: tuple[str, ...] = ()

  @property
  def full_name(self) -> str:
    return f"{self.project}_{self.name}" if self.project else self.name


def _make_spec(name, num_groups, m, n, k, lhs_dtype, rhs_dtype, group_sizes=None, project="", tags=()) -> ArgSpec:
  lhs = ShapeDtype((m, k), lhs_dtype)
  rhs = ShapeDtype((num_groups, k, n), rhs_dtype)
  gs_spec = ShapeDtype((num_groups,), torch.int32)
  if group_sizes is None:
    group_sizes = base.GroupSizes(gs_spec, m)
  else:
    assert len(group_sizes) == num_groups
    group_sizes = base.GroupSizes(gs_spec, tuple(group_sizes))
  return ArgSpec(name=name, args=dict(lhs=lhs, rhs=rhs, group_sizes=group_sizes), project=project, tags=tuple(tags))


def _make_maxtext_spec(name_prefix, num_groups, *, m, n, k, tags=()) -> ArgSpec:
  return _make_spec(f"{name_prefix}-{m}x{k}_{num_groups}x{k}x{n}", num_groups, m, n, k, torch.bfloat16,
                    torch.bfloat16, project="maxtext", tags=tags)


_BF16 = torch.bfloat16
SPEC_SHAPES = {
    "compute_bound": (8, 4096, 4096, 4096, _BF16, _BF16, [4096] + [0] * 7, "", ("primary", "ci_tests")),
    "memory_bound": (8, 8, 4096, 4096, _BF16, _BF16, [1] * 8, "", ("primary", "ci_tests")),
    "8x7b": (8, 8192, 14336, 4096, _BF16, _BF16, None, "mixtral", ("primary", "ci_tests")),
}

# (project prefix, groups, m, n, k[, tags]) of the MaxText shapes, arg_specs.py:91-155.
_MAXTEXT_SHAPES = (
    ("deepseek-v3", 256, 131072, 1024, 7168, ("primary",)),
    ("deepseek-v3", 256, 131072, 7168, 1024, ("primary",)),
    ("deepseek-v3", 256, 131072, 512, 7168, ("primary",)),
    ("deepseek-v3", 256, 131072, 7168, 512, ("primary",)),
    ("deepseek-v3", 256, 262144, 512, 7168, ("primary",)),
    ("deepseek-v3", 256, 262144, 7168, 256, ("primary",)),
    ("deepseek-v3", 256, 262144, 7168, 1024, ("primary",)),
    ("deepseek-v3", 256, 262144, 1024, 7168, ("primary",)),
    ("deepseek-v3", 256, 262144, 2048, 7168, ("primary",)),
    ("gpt-oss", 128, 327680, 2880, 2880, ()),
    ("gpt-oss", 128, 393216, 768, 2048, ()),
    ("gpt-oss", 128, 393216, 2048, 768, ()),
    ("gpt-oss", 128, 524288, 1536, 4096, ()),
    ("gpt-oss", 128, 524288, 4096, 1536, ()),
    ("gpt-oss", 256, 524288, 2048, 7168, ()),
    ("gpt-oss", 128, 262144, 1536, 4096, ()),
    ("gpt-oss", 128, 262144, 4096, 1536, ()),
    ("gpt-oss", 128, 131072, 2048, 7168, ()),
    ("gpt-oss", 128, 131072, 768, 2048, ()),
    ("gpt-oss", 128, 131072, 1536, 4096, ()),
    ("gpt-oss", 128, 131072, 4096, 1536, ()),
    ("gpt-oss", 256, 131072, 2048, 7168, ()),
    ("gpt-oss", 256, 65536, 2048, 7168, ()),
    ("gpt-oss", 256, 131072, 512, 7168, ()),
    ("gpt-oss", 256, 131072, 7168, 512, ()),
    ("gpt-oss", 256, 262144, 7168, 512, ()),
    ("gpt-oss", 256, 262144, 512, 7168, ()),
    ("gpt-oss", 256, 262144, 7168, 256, ()),
    ("gpt-oss", 256, 262144, 7168, 1024, ()),
    ("gpt-oss", 256, 262144, 1024, 7168, ()),
)

ARG_SPECS = tuple(
    _make_maxtext_spec(prefix, groups, m=m, n=n, k=k, tags=tags) for prefix, groups, m, n, k, tags in _MAXTEXT_SHAPES
) + tuple(_make_spec(name, *args) for name, args in SPEC_SHAPES.items())


def flops(lhs, rhs, *, group_sizes) -> int:
  """2 * sum(group sizes) * k * n (bench.py:52-56)."""
  del lhs
  _, k, n = rhs.shape
  gs = group_sizes.representative_value if isinstance(group_sizes, base.GroupSizes) else group_sizes
  return 2 * int(sum(int(x) for x in gs)) * int(k) * int(n)


def random_initialize(spec_args: dict, device, seed: int = 0) -> dict:
  """Concrete arguments for an arg spec, as the reference's benchmarks and `test_bench` make them
  (tokamax/_src/numerics.py:179-264 and base.py:99-106): abstract arrays become standard-normal values cast to their
  type, drawn on the device; a `GroupSizes` spec becomes its representative sizes (an int32 device tensor)."""
  gen = torch.Generator(device=device)
  gen.manual_seed(seed)
  out = {}
  for name, x in spec_args.items():
    if isinstance(x, base.GroupSizes):
      out[name] = torch.tensor(x.representative_value, dtype=torch.int32, device=device)
    elif isinstance(x, ShapeDtype):
      t = torch.empty(tuple(x.shape), dtype=torch.float32 if x.dtype == torch.float32 else torch.bfloat16, device=device)
      t.normal_(0.0, 1.0, generator=gen)
      out[name] = t.to(x.dtype)
    else:
      out[name] = x
  return out
