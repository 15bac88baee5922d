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

ARG_SPECS = (
    _make_maxtext_spec("deepseek-v3", 256, m=131072, n=1024, k=7168, tags=("primary",)),
    _make_maxtext_spec("deepseek-v3", 256, m=131072, n=7168, k=1024, tags=("primary",)),
    _make_maxtext_spec("deepseek-v3", 256, m=131072, n=512, k=7168, tags=("primary",)),
    _make_maxtext_spec("deepseek-v3", 256, m=131072, n=7168, k=512, tags=("primary",)),
    _make_maxtext_spec("deepseek-v3", 256, m=262144, n=2048, k=7168, tags=("primary",)),
    _make_maxtext_spec("gpt-oss", 128, m=131072, n=768, k=2048),
    _make_maxtext_spec("gpt-oss", 128, m=131072, n=1536, k=4096),
    _make_maxtext_spec("gpt-oss", 256, m=65536, n=2048, k=7168),
    _make_maxtext_spec("gpt-oss", 256, m=131072, n=2048, k=7168),
) + tuple(_make_spec(name, *args) for name, args in SPEC_SHAPES.items())


def flops(lhs, rhs, *, group_sizes) -> int:
  """2 * sum(group sizes) * k * n (bench.py:52-56)."""
  del lhs
  _, k, n = rhs.shape
  gs = group_sizes.representative_value if isinstance(group_sizes, base.GroupSizes) else group_sizes
  return 2 * int(sum(int(x) for x in gs)) * int(k) * int(n)
