"""Gated linear unit on the gate-up fused forward kernel of the ragged dot.

`activation(x @ weights[:, 0]) * (x @ weights[:, 1])` (tokamax/_src/ops/gated_linear_unit/base.py:60-120).
Fused weights `[K, 2, N]` are, row by row, `[gate | up]`: exactly the `[1, K, 2N]` weight layout of the
ragged dot's gate-up mode with a single group that owns every row, so this op is that kernel with
`group_sizes = [M]`; the product is formed on the f32 accumulators and rounded once to `x.dtype`, as
the reference does (base.py:108-118).
"""

from __future__ import annotations

import dataclasses

import torch

from tokamax_amd import op
from tokamax_amd import precision as precision_lib
from tokamax_amd.ragged_dot import hip as ragged_hip
from tokamax_amd.ragged_dot import hip_ops


@dataclasses.dataclass(frozen=True)
class HipGatedLinearUnit(op.Op):
  """`gated_linear_unit` with `implementation="hip"`; its config is the ragged dot's `Config`."""

  config_cls = ragged_hip.Config

  def bind(self, x, weights, *, activation=None, precision=None, return_residuals: bool = False):  # pylint: disable=arguments-differ
    return super().bind(x=x, weights=weights, activation=activation,
                        precision=precision_lib.canonicalize_precision(precision), return_residuals=return_residuals)

  def _ragged_bound_args(self, x, weights):
    """The bound arguments of the equivalent one-group gate-up ragged dot (for its config machinery)."""
    k = x.shape[-1]
    rows = 1
    for d in x.shape[:-1]:
      rows *= int(d)
    w = weights if not isinstance(weights, (tuple, list)) else None
    n2 = 2 * int(weights[0].shape[-1]) if w is None else 2 * int(w.shape[-1])
    dev = x.device
    gs = torch.empty(1, dtype=torch.int32, device=dev)
    lhs = torch.empty((rows, k), dtype=x.dtype, device="meta")
    rhs = torch.empty((1, k, n2), dtype=x.dtype, device="meta")
    return ragged_hip.HipRaggedDot().bind(lhs, rhs, group_sizes=gs, fuse_gateup_activation="silu")

  def _get_heuristics_config(self, ba: op.BoundArguments):
    x, weights = ba.arguments["x"], ba.arguments["weights"]
    return ragged_hip.HipRaggedDot()._get_heuristics_config(self._ragged_bound_args(x, weights))  # pylint: disable=protected-access

  def _get_autotuning_configs(self, ba: op.BoundArguments):
    x, weights = ba.arguments["x"], ba.arguments["weights"]
    return ragged_hip.HipRaggedDot()._get_autotuning_configs(self._ragged_bound_args(x, weights))  # pylint: disable=protected-access

  def supported_on(self, device: torch.device) -> bool:
    return ragged_hip.HipRaggedDot().supported_on(device)

  def _fwd(self, x, weights, *, activation, precision, return_residuals, config):
    if return_residuals:
      raise NotImplementedError("The hip gated linear unit does not return residuals.")
    if isinstance(weights, (tuple, list)):
      gate_w, up_w = weights
      if gate_w.shape != up_w.shape or gate_w.dim() != 2:
        raise ValueError("unfused weights must be two [K, N] arrays")
      fused = torch.stack([gate_w, up_w], dim=1)  # [K, 2, N]
    else:
      fused = weights
    if fused.dim() != 3 or fused.shape[1] != 2 or fused.shape[0] != x.shape[-1]:
      raise ValueError(f"expected weights [K, 2, N] with K = {x.shape[-1]}, got {tuple(fused.shape)}")
    if fused.dtype != x.dtype or not precision_lib.is_default(x.dtype, fused.dtype, precision):
      raise NotImplementedError("x and weights must share a dtype, at the default precision.")
    k, _, n = fused.shape
    lead = x.shape[:-1]
    x2 = x.reshape(-1, k)
    rows = x2.shape[0]
    rhs = fused.reshape(1, k, 2 * n)
    gs = torch.full((1,), rows, dtype=torch.int32, device=x.device)
    name = None if activation is None else ragged_hip._fused_activation_name(activation)  # pylint: disable=protected-access
    kcfg = config.to_kernel_config()
    if activation is None or name is not None:
      out = hip_ops.ragged_dot_fwd(x2, rhs, gs, config=kcfg, out_dtype=x.dtype, activation=name, gateup=True)
    else:
      # A callable with no in-kernel twin: gate and up in one f32 GEMM, the rest in torch on f32.
      both = hip_ops.ragged_dot_fwd(x2, rhs, gs, config=self._plain_config(x2, rhs, gs), out_dtype=torch.float32)
      out = (activation(both[:, :n]) * both[:, n:]).to(x.dtype)
    return out.reshape(*lead, n), None

  @staticmethod
  def _plain_config(x2, rhs, gs):
    rd = ragged_hip.HipRaggedDot()
    return rd._get_heuristics_config(rd.bind(x2, rhs, group_sizes=gs)).to_kernel_config()  # pylint: disable=protected-access
