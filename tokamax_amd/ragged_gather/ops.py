"""The three row-movement ops of an MoE layer on one HIP kernel (`tkx_ragged_gather_rows`).

  ragged_gather(x, indices, start, end)          = x[indices]                      ragged_gather/base.py:25-32
  ragged_scatter(x, indices, start, end)         = where(start <= indices < end, x[indices], 0)
                                                                                   ragged_scatter/base.py:26-38
  ragged_gather_reduce(x, indices, w, valid, R)  = sum over groups of R rows of valid * w * x[indices], in f32
                                                                                   ragged_gather_reduce/base.py:26-40
"""

from __future__ import annotations

import ctypes
import dataclasses

import torch

from tokamax_amd import _lib
from tokamax_amd import op
from tokamax_amd.ragged_dot import hip as ragged_hip
from tokamax_amd.ragged_dot import hip_ops


def _scalar_i32(v, device) -> torch.Tensor:
  if isinstance(v, torch.Tensor):
    return v.reshape(-1)[:1].to(device=device, dtype=torch.int32).contiguous()
  return torch.tensor([int(v)], dtype=torch.int32, device=device)


def _gather_rows(x, indices, *, weights=None, valid=None, start=None, end=None, reduce: int = 1) -> torch.Tensor:
  if x.dim() != 2 or indices.dim() != 1:
    raise ValueError(f"expected x [rows, hidden] and indices [n], got {tuple(x.shape)} and {tuple(indices.shape)}")
  if not x.is_cuda:
    raise NotImplementedError("the hip implementation needs tensors on an AMD GPU (got a CPU tensor)")
  if x.dtype not in (torch.float32, torch.bfloat16, torch.float16):
    raise NotImplementedError(f"dtype {x.dtype} is not supported by the hip implementation")
  if indices.numel() % reduce:
    raise ValueError("the number of indices must be a multiple of reduce_group_size")
  lib = _lib.load()
  x = x.contiguous()
  idx = indices.to(torch.int32).contiguous()
  out_rows = idx.numel() // reduce
  if weights is not None:
    weights = weights.to(torch.float32).contiguous()
  if valid is not None:
    valid = valid.to(torch.uint8).contiguous()
  if start is not None:
    start, end = _scalar_i32(start, x.device), _scalar_i32(end, x.device)
  out = torch.empty((out_rows, x.shape[1]), dtype=x.dtype, device=x.device)
  p = lambda t: ctypes.c_void_p(0 if t is None else t.data_ptr())
  with torch.cuda.device(x.device):
    st = lib.tkx_ragged_gather_rows(p(x), p(idx), p(weights), p(valid), p(start), p(end), p(out), x.shape[0], out_rows,
                                    x.shape[1], reduce, hip_ops.dtype_code(x.dtype),
                                    ctypes.c_void_p(torch.cuda.current_stream(x.device).cuda_stream))
  _lib.check(st)
  return out


class _RowOp(op.Op):
  """Shared pieces: no tunables (`NullConfig`), gfx950 only."""

  def supported_on(self, device: torch.device) -> bool:
    return ragged_hip.HipRaggedDot().supported_on(device)


@dataclasses.dataclass(frozen=True)
class HipRaggedGather(_RowOp):
  def bind(self, x, indices, start, end, *, return_residuals: bool = False):  # pylint: disable=arguments-differ
    return super().bind(x=x, indices=indices, start=start, end=end, return_residuals=return_residuals)

  def _fwd(self, x, indices, start, end, *, return_residuals=False, config=None):
    del start, end, return_residuals, config  # the row range plays no part in the definition (base.py:25-32)
    return _gather_rows(x, indices), None


@dataclasses.dataclass(frozen=True)
class HipRaggedScatter(_RowOp):
  def bind(self, x, indices, start, end, *, return_residuals: bool = False):  # pylint: disable=arguments-differ
    return super().bind(x=x, indices=indices, start=start, end=end, return_residuals=return_residuals)

  def _fwd(self, x, indices, start, end, *, return_residuals=False, config=None):
    del return_residuals, config
    return _gather_rows(x, indices, start=start, end=end), None


@dataclasses.dataclass(frozen=True)
class HipRaggedGatherReduce(_RowOp):
  def bind(self, x, indices, topk_weights, valid_rows_mask, *, reduce_group_size: int, return_residuals: bool = False):  # pylint: disable=arguments-differ
    return super().bind(x=x, indices=indices, topk_weights=topk_weights, valid_rows_mask=valid_rows_mask,
                        reduce_group_size=reduce_group_size, return_residuals=return_residuals)

  def _fwd(self, x, indices, topk_weights, valid_rows_mask, *, reduce_group_size, return_residuals=False, config=None):
    del return_residuals, config
    return _gather_rows(x, indices, weights=topk_weights, valid=valid_rows_mask, reduce=int(reduce_group_size)), None


def ragged_gather(x, indices, start, end):
  """`x[indices]` ([in, hidden], int[out] -> [out, hidden])."""
  return HipRaggedGather()(x, indices, start, end)


def ragged_scatter(x, indices, start, end):
  """`x[indices]` with the rows whose index lies outside `[start, end)` set to zero."""
  return HipRaggedScatter()(x, indices, start, end)


def ragged_gather_reduce(x, indices, topk_weights, valid_rows_mask, reduce_group_size: int):
  """Sums, over consecutive groups of `reduce_group_size` gathered rows, `valid * weight * x[index]` in
  f32 and rounds to `x.dtype` ([n, hidden] -> [n / reduce_group_size, hidden])."""
  return HipRaggedGatherReduce()(x, indices, topk_weights, valid_rows_mask, reduce_group_size=reduce_group_size)
