"""Seeded synthetic MoE workloads: the five configurations ragged dot is measured on.

Group sizes come from NumPy's `default_rng(seed)` (host, a few hundred integers); the large operands
are generated on the device with torch's generator, so nothing big crosses PCIe.
  fp32      lhs [1024,512], rhs [8,512,1024], uniform multinomial groups
  mixtral   m=16384, k=4096, n=14336, G=8, bf16, top-2 router over Gaussian logits (mild skew)
  deepseek  m=65536, k=7168, n=2048, G=256, bf16, Zipf(1.1)-skewed groups, ~5% of experts empty
  decode    m=256, k=2048, n=768, G=128, bf16 lhs x int8 rhs with f32 per-(group, column) scales
  fp8       the mixtral shape with e4m3fn operands, per-row and per-(group, column) f32 scales
  vjp       m=4096, k=4096, n=14336, G=8, bf16 (lhs, rhs, dout)
"""

from __future__ import annotations

import dataclasses

import numpy as np
import torch


@dataclasses.dataclass
class Workload:
  name: str
  m: int
  k: int
  n: int
  num_groups: int
  group_sizes: np.ndarray  # int32 [G], host copy
  lhs: torch.Tensor
  rhs: torch.Tensor
  lhs_scale: torch.Tensor | None = None
  rhs_scale: torch.Tensor | None = None
  dout: torch.Tensor | None = None
  out_dtype: torch.dtype = torch.bfloat16
  seed: int = 0

  @property
  def flops(self) -> int:
    """2 * sum(group_sizes) * k * n, the reference's convention."""
    return 2 * int(self.group_sizes.sum()) * self.k * self.n

  @property
  def nonempty_groups(self) -> int:
    return int((self.group_sizes > 0).sum())

  def algorithmic_bytes(self) -> int:
    """Each operand once; only the weights (and scales) of non-empty groups count."""
    rows = int(self.group_sizes.sum())
    b = rows * self.k * self.lhs.element_size()
    b += self.nonempty_groups * self.k * self.n * self.rhs.element_size()
    b += self.m * self.n * torch.empty((), dtype=self.out_dtype).element_size()
    if self.lhs_scale is not None:
      b += rows * 4
    if self.rhs_scale is not None:
      b += self.nonempty_groups * self.n * 4
    return b


def router_top2_group_sizes(tokens: int, num_groups: int, seed: int) -> np.ndarray:
  rng = np.random.default_rng(seed)
  logits = rng.normal(size=(tokens, num_groups))
  top2 = np.argsort(-logits, axis=1)[:, :2]
  return np.bincount(top2.ravel(), minlength=num_groups).astype(np.int32)


def zipf_group_sizes(m: int, num_groups: int, seed: int, s: float = 1.1, empty_fraction: float = 0.05) -> np.ndarray:
  rng = np.random.default_rng(seed)
  ranks = rng.permutation(num_groups) + 1
  p = ranks.astype(np.float64) ** (-s)
  empty = rng.choice(num_groups, int(round(empty_fraction * num_groups)), replace=False)
  p[empty] = 0.0
  p /= p.sum()
  return rng.multinomial(m, p).astype(np.int32)


def decode_group_sizes(tokens: int, top_k: int, num_groups: int, seed: int) -> np.ndarray:
  rng = np.random.default_rng(seed)
  picks = np.concatenate([rng.choice(num_groups, top_k, replace=False) for _ in range(tokens)])
  return np.bincount(picks, minlength=num_groups).astype(np.int32)


def _normal(shape, std, dtype, device, gen):
  x = torch.empty(shape, dtype=torch.float32 if dtype == torch.float32 else torch.bfloat16, device=device)
  x.normal_(0.0, std, generator=gen)
  return x.to(dtype)


def _fp8_quantize(x: torch.Tensor, dim: int):
  """absmax/448 scaling along `dim` -> (e4m3fn values, f32 scales with that dim kept as 1)."""
  amax = x.abs().amax(dim=dim, keepdim=True).float().clamp_min(1e-12)
  scale = amax / 448.0
  q = (x.float() / scale).to(torch.float8_e4m3fn)
  return q, scale


def make(name: str, device, seed: int = 0, *, m: int | None = None) -> Workload:
  """Builds one workload on `device`. `m` overrides the row count (for CPU-sized samples)."""
  gen = torch.Generator(device=device)
  gen.manual_seed(seed)
  bf16 = torch.bfloat16
  if name == "fp32":
    m_, k, n, G = m or 1024, 512, 1024, 8
    gs = np.random.default_rng(seed).multinomial(m_, [1.0 / G] * G).astype(np.int32)
    return Workload(name, m_, k, n, G, gs, _normal((m_, k), 1.0, torch.float32, device, gen),
                    _normal((G, k, n), k ** -0.5, torch.float32, device, gen), out_dtype=torch.float32, seed=seed)
  if name == "mixtral":
    m_, k, n, G = m or 16384, 4096, 14336, 8
    gs = router_top2_group_sizes(m_ // 2, G, seed)
    return Workload(name, m_, k, n, G, gs, _normal((m_, k), 1.0, bf16, device, gen),
                    _normal((G, k, n), k ** -0.5, bf16, device, gen), seed=seed)
  if name == "deepseek":
    m_, k, n, G = m or 65536, 7168, 2048, 256
    gs = zipf_group_sizes(m_, G, seed)
    return Workload(name, m_, k, n, G, gs, _normal((m_, k), 1.0, bf16, device, gen),
                    _normal((G, k, n), k ** -0.5, bf16, device, gen), seed=seed)
  if name == "decode":
    m_, k, n, G = m or 256, 2048, 768, 128
    gs = decode_group_sizes(m_ // 8, 8, G, seed)
    rhs = torch.randint(-127, 128, (G, k, n), dtype=torch.int8, device=device, generator=gen)
    scale = (torch.rand((G, 1, n), device=device, generator=gen) + 0.5) / 127.0
    return Workload(name, m_, k, n, G, gs, _normal((m_, k), 1.0, bf16, device, gen), rhs, rhs_scale=scale, seed=seed)
  if name == "fp8":
    m_, k, n, G = m or 16384, 4096, 14336, 8
    gs = router_top2_group_sizes(m_ // 2, G, seed)
    lhs_q, lhs_s = _fp8_quantize(_normal((m_, k), 1.0, bf16, device, gen), dim=1)
    rhs_q = torch.empty((G, k, n), dtype=torch.float8_e4m3fn, device=device)
    rhs_s = torch.empty((G, 1, n), dtype=torch.float32, device=device)
    for g in range(G):  # one expert at a time keeps the f32 temporaries small
      q, s = _fp8_quantize(_normal((k, n), k ** -0.5, bf16, device, gen), dim=0)
      rhs_q[g], rhs_s[g] = q, s
    return Workload(name, m_, k, n, G, gs, lhs_q, rhs_q, lhs_scale=lhs_s, rhs_scale=rhs_s, seed=seed)
  if name == "vjp":
    m_, k, n, G = m or 4096, 4096, 14336, 8
    gs = router_top2_group_sizes(m_ // 2, G, seed)
    return Workload(name, m_, k, n, G, gs, _normal((m_, k), 1.0, bf16, device, gen),
                    _normal((G, k, n), k ** -0.5, bf16, device, gen), dout=_normal((m_, n), 1.0, bf16, device, gen),
                    seed=seed)
  raise ValueError(f"unknown workload {name!r}")
