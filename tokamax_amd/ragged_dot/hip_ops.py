"""Thin adapters from torch device tensors to the C ABI (pointers + sizes + stream).

PyTorch is used for device memory and streams only; all arithmetic happens in the HIP library.
"""

from __future__ import annotations

import contextlib
import ctypes
import dataclasses
import functools
import math
import threading

import torch

from tokamax_amd import _lib

_DTYPE_CODE = {
    torch.float32: _lib.TKX_F32,
    torch.bfloat16: _lib.TKX_BF16,
    torch.float16: _lib.TKX_F16,
    torch.float8_e4m3fn: _lib.TKX_F8E4M3FN,
    torch.int8: _lib.TKX_I8,
    torch.uint8: _lib.TKX_I4X2,  # uint8 storage = int4 packed two to a byte along the second-to-last axis
}

SCHEDULE_FIELDS = ("group_id", "block_start", "actual_start", "actual_end", "start_within_block", "actual_size")


class _LaunchLog(threading.local):
  """What the functions of this module launched while a caller was listening (`records` is a list then): a
  `ForwardLaunch` for a forward call, None for anything else (a pass over an operand, a quantisation, drhs). The
  operator's eager fast path reads it to learn whether a call came down to one forward launch on the caller's own
  tensors, which it can then repeat without the planning in front of it."""
  records = None


LAUNCH_LOG = _LaunchLog()


def _log_launch(entry) -> None:
  if LAUNCH_LOG.records is not None:
    LAUNCH_LOG.records.append(entry)


@dataclasses.dataclass
class ForwardLaunch:
  """One forward launch, repeatable on other buffers of the same shapes: `launch(pointers, out_ptr, ws_ptr, stream)`
  with `pointers` in the order of `POINTER_NAMES` (0 for an absent operand) returns the C status."""

  POINTER_NAMES = ("lhs", "rhs", "group_sizes", "group_offset", "lhs_scale", "rhs_scale", "rhs_bias")
  pointers: tuple          # the addresses this launch was made with, in that order
  launch: object
  out: torch.Tensor        # the result it returned (for the caller to recognise it)
  new_workspace: object    # () -> the int32 workspace tensor of a repeat


def dtype_code(dtype: torch.dtype) -> int:
  try:
    return _DTYPE_CODE[dtype]
  except KeyError:
    raise NotImplementedError(f"dtype {dtype} is not supported by the hip implementation") from None


@dataclasses.dataclass(frozen=True)
class KernelConfig:
  """Launch parameters handed to the C ABI (see TkxConfig in include/tkx_ragged_dot.h)."""

  block_m: int
  block_n: int
  block_k: int
  waves_m: int
  waves_n: int
  num_stages: int = 2
  grid_tile_width: int = 1
  align_tile: int = 8
  split_k: int = 1
  persistent: int = 0

  def to_c(self) -> _lib.TkxConfig:
    return _config_struct(self)


@functools.lru_cache(maxsize=256)
def _config_struct(c: "KernelConfig") -> _lib.TkxConfig:
  """The C struct of a config (built once per distinct config; the library only reads it)."""
  return _lib.TkxConfig(c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.grid_tile_width, c.align_tile,
                        c.num_stages, c.split_k, c.persistent)


@functools.lru_cache(maxsize=1024)
def _workspace_words(m: int, num_groups: int, block_m: int) -> int:
  nbytes = _lib.load().tkx_ragged_dot_workspace_bytes(m, num_groups, block_m)
  if nbytes < 0:
    raise ValueError(f"bad sizes m={m} G={num_groups} block_m={block_m}")
  return nbytes // 4


def _on_device(device):
  """Context that makes `device` current for the launch; free when it already is."""
  if device.index is None or torch.cuda.current_device() == device.index:
    return contextlib.nullcontext()
  return torch.cuda.device(device)


def _require_cuda(*tensors):
  for t in tensors:
    if t is not None and not t.is_cuda:
      raise NotImplementedError("the hip implementation needs tensors on an AMD GPU (got a CPU tensor)")


def _ptr(t):
  return ctypes.c_void_p(0 if t is None else t.data_ptr())


def _stream(device) -> ctypes.c_void_p:
  return ctypes.c_void_p(torch.cuda.current_stream(device).cuda_stream)


def _group_sizes_i32(group_sizes: torch.Tensor) -> torch.Tensor:
  if group_sizes.dtype != torch.int32:
    group_sizes = group_sizes.to(torch.int32)  # uint32 / int64 inputs are legal in the reference
  return group_sizes.contiguous()


def workspace(m: int, num_groups: int, block_m: int, device, block_n: int = 0, split_k: int = 1) -> torch.Tensor:
  """The schedule workspace of a tiled call; with split_k > 1 the partial tiles of the split last round behind it."""
  if split_k > 1:
    return torch.empty(_split_workspace_words(m, num_groups, block_m, block_n), dtype=torch.int32, device=device)
  return torch.empty(_workspace_words(m, num_groups, block_m), dtype=torch.int32, device=device)


@functools.lru_cache(maxsize=1024)
def _split_workspace_words(m: int, num_groups: int, block_m: int, block_n: int) -> int:
  nbytes = _lib.load().tkx_ragged_dot_split_workspace_bytes(m, num_groups, block_m, block_n)
  if nbytes < 0:
    raise ValueError(f"bad sizes m={m} G={num_groups} block_m={block_m} block_n={block_n}")
  return nbytes // 4


_SPLIT_WORKSPACES: dict = {}
_SUPERSEDED_WORKSPACES: list = []
_UNUSED_WORKSPACES: dict = {}


def split_workspace(m: int, n: int, split_k: int, device, persistent: int = 0) -> torch.Tensor:
  """The workspace of a streaming-kernel call that completes tiles across workgroups (a split contraction, or the
  persistent form): arrival counters, which the kernel needs zero on entry and leaves zero, then room for the partial
  sums. One buffer per (device, stream), zeroed when it is made and replaced by a larger one when a call needs more;
  calls on one stream are ordered, so they can share it.

  A buffer that was handed out is never released: a HIP graph captured earlier holds its address, and replays must
  keep finding counters that nobody else writes (superseded buffers stay referenced until the process ends). The
  buffer belongs to the stream the call was made (or captured) on: a captured graph must be replayed on a stream that
  no other split or persistent call uses at the same time, since they would share one set of counters."""
  device = torch.device(device)
  lib = _lib.load()
  nbytes = (lib.tkx_ragged_dot_decode_persistent_workspace_bytes() if persistent
            else lib.tkx_ragged_dot_decode_workspace_bytes(m, n, split_k))
  key = (device.index if device.index is not None else torch.cuda.current_device(),
         torch.cuda.current_stream(device).cuda_stream)
  ws = _SPLIT_WORKSPACES.get(key)
  if ws is None or ws.numel() * 4 < nbytes:
    if torch.cuda.is_current_stream_capturing():
      # (Memory allocated under capture belongs to the graph, and the counters must be zero before its first replay.)
      raise RuntimeError("the workspace of a split contraction has to exist before a HIP graph is captured: make one"
                         " call with these shapes on the capture stream first")
    if ws is not None:
      _SUPERSEDED_WORKSPACES.append(ws)
    ws = torch.zeros(max(nbytes // 4, 1 << 20), dtype=torch.int32, device=device)
    _SPLIT_WORKSPACES[key] = ws
  return ws


def schedule(group_sizes: torch.Tensor, m: int, block_m: int, align_tile: int = 8):
  """Runs the on-device scheduler; returns a dict of the six task arrays, the launch-order span
  arrays (`span_first`, `span_width`; spans are one task wide here), group_offsets and the counters."""
  _require_cuda(group_sizes)
  lib = _lib.load()
  gs = _group_sizes_i32(group_sizes)
  G = gs.numel()
  ws = workspace(m, G, block_m, gs.device)
  _lib.check(lib.tkx_ragged_dot_schedule(_ptr(gs), G, m, block_m, align_tile, _ptr(ws), _stream(gs.device)))
  tid_size = lib.tkx_ragged_dot_tid_size(m, G, block_m)
  out = {}
  for i, name in enumerate(SCHEDULE_FIELDS):
    off = lib.tkx_ragged_dot_workspace_offset(m, G, block_m, 3 + i)
    out[name] = ws[off:off + tid_size]
  for i, name in enumerate(("span_first", "span_width")):
    off = lib.tkx_ragged_dot_workspace_offset(m, G, block_m, 9 + i)
    out[name] = ws[off:off + tid_size]
  off = lib.tkx_ragged_dot_workspace_offset(m, G, block_m, 2)
  out["group_offsets"] = ws[off:off + G + 1]
  out["num_tasks"] = ws[0:1]
  out["total_rows"] = ws[1:2]
  return out


def ragged_dot_fwd(lhs, rhs, group_sizes, *, config: KernelConfig, out_dtype: torch.dtype, trans_rhs: bool = False,
                   lhs_scale=None, rhs_scale=None, activation: str | None = None, rhs_bias=None,
                   gateup: bool = False, group_offset=None, workspace_out: list | None = None) -> torch.Tensor:
  """out[m,n] = lhs[m,k] . rhs[g,k,n]   (trans_rhs: out[m,k] = lhs[m,n] . rhs[g,k,n]^T).

  `rhs_scale` is [g,n] / [g,1,n], or [g,blocks,n] with `blocks` scale blocks along k (streaming small-m
  kernel only). `rhs_bias` ([g,n] or [g,1,n]) is added to the scaled result before the activation. `gateup`: rhs
  columns are [gate | up] and out[m,n/2] = activation(gate part) * (up part) (base.py:211-217).
  `group_offset` (device int32 tensor of one element): `group_sizes` covers every group of the job, rhs holds the
  groups [offset, offset + g) of them, and the rows of all other groups come out zero (the call of one
  expert-parallel shard, experimental/gmm_v2/gmm_v2_test.py:44-101).
  `workspace_out`, if given, receives the int32 workspace the call filled (schedule arrays included)."""
  _require_cuda(lhs, rhs, group_sizes, lhs_scale, rhs_scale, rhs_bias, group_offset)
  lib = _lib.load()
  if lhs.dim() != 2 or rhs.dim() != 3:
    raise ValueError(f"expected lhs [m,k] and rhs [g,k,n], got {tuple(lhs.shape)} and {tuple(rhs.shape)}")
  lhs, rhs = lhs.contiguous(), rhs.contiguous()
  gs = _group_sizes_i32(group_sizes)
  G, k, n = rhs.shape
  if rhs.dtype == torch.uint8:
    k *= 2  # packed int4: a byte row holds two contraction rows
    if trans_rhs:
      raise NotImplementedError("packed int4 weights take the default dimension numbers; unpack_int4 them first")
  m = lhs.shape[0]
  if group_offset is None:
    if gs.numel() != G:
      raise ValueError(f"group_sizes has {gs.numel()} entries, rhs has {G} groups")
  else:
    if trans_rhs:
      raise NotImplementedError("group_offset needs the default dimension numbers")
    if group_offset.numel() != 1 or gs.numel() < 1:
      raise ValueError("group_offset must hold one element and group_sizes at least one")
    if group_offset.dtype != torch.int32:
      group_offset = group_offset.to(torch.int32)
    group_offset = group_offset.contiguous()
  if lhs.shape[1] != (n if trans_rhs else k):
    raise ValueError("contraction sizes of lhs and rhs differ")
  if (rhs_bias is not None or gateup) and trans_rhs:
    raise NotImplementedError("bias and gate-up fusion need the default dimension numbers")
  if gateup and n % 2:
    raise ValueError("gate-up fusion needs an even number of rhs columns")
  lhs_scale_blocks = 1
  if lhs.dtype == torch.float8_e4m3fn and rhs.dtype == torch.uint8:
    # The kernel takes the weights' +8 bias off with the row sums of the fp8 activations, which lie behind the row
    # scales: f32 [2, m]. A caller that holds both already passes them in that form.
    # With rhs scales per k-block: [blocks + k / 128, m], the lhs scales per k-block and the row sums per 128 columns.
    if lhs_scale is None:
      raise NotImplementedError("fp8 activations over packed int4 weights need one lhs scale per row")
    blocks = int(rhs_scale.shape[1]) if rhs_scale is not None and rhs_scale.dim() == 3 else 1
    sum_rows = 1 if blocks == 1 else k // 128
    if tuple(lhs_scale.shape) != (blocks + sum_rows, m):
      if lhs_scale.numel() == m:
        per_block = lhs_scale.reshape(1, m).expand(blocks, m)
      elif tuple(lhs_scale.shape) == (m, blocks):
        per_block = lhs_scale.t()
      else:
        raise NotImplementedError("fp8 activations over packed int4 weights: lhs scale [m] / [m, 1] / [m, k-blocks], or"
                                  " [k-blocks + sum rows, m] with the row sums")
      if blocks > 1 and k % 128:
        raise NotImplementedError("scale blocks along k need k % 128 == 0 here")
      both = torch.empty((blocks + sum_rows, m), dtype=torch.float32, device=lhs.device)
      both[:blocks].copy_(per_block)
      row_sums_fp8(lhs, out=both[blocks:], per_128_columns=blocks > 1)
      lhs_scale = both
    lhs_scale = lhs_scale.to(torch.float32).contiguous().view(-1)
    lhs_scale_blocks = blocks
  elif lhs_scale is not None:
    if lhs_scale.dim() == 2 and lhs_scale.shape[1] > 1:
      # One scale per (row, k-block): the kernels take them as [k-blocks, m].
      lhs_scale_blocks = int(lhs_scale.shape[1])
      lhs_scale = lhs_scale.to(torch.float32).t().contiguous().view(-1)
    else:
      lhs_scale = lhs_scale.to(torch.float32).contiguous().view(-1)
    if lhs_scale.numel() != m * lhs_scale_blocks:
      raise NotImplementedError("lhs scale must be one f32 per row (or per row and k-block)")
  scale_blocks = 1
  if rhs_scale is not None:
    if rhs_scale.dim() == 3 and rhs_scale.shape[1] > 1:
      scale_blocks = int(rhs_scale.shape[1])
    rhs_scale = rhs_scale.to(torch.float32).contiguous().view(-1)
    if rhs_scale.numel() != G * scale_blocks * n or k % scale_blocks:
      raise NotImplementedError("rhs scale must be one f32 per (group, column) or per (group, k-block, column)")
  if lhs_scale_blocks != 1 and lhs_scale_blocks != scale_blocks:
    raise NotImplementedError("lhs and rhs scales must have the same number of blocks along k")
  if (lhs_scale is not None and lhs_scale_blocks == 1 and scale_blocks > 1 and config.block_m != 16
      and lhs.dtype in (torch.int8, torch.float8_e4m3fn)):
    # The kernels that fold both operands' scales in per k-block read the lhs scales as [k-blocks, m].
    lhs_scale = lhs_scale.view(1, m).expand(scale_blocks, m).contiguous().view(-1)
  if rhs_bias is not None:
    rhs_bias = rhs_bias.to(torch.float32).contiguous().view(-1)
    if rhs_bias.numel() != G * n:
      raise NotImplementedError("rhs bias must be one value per (group, column)")
  out_cols = k if trans_rhs else n // 2 if gateup else n
  device = lhs.device
  out = torch.empty((m, out_cols), dtype=out_dtype, device=device)
  if config.block_m == 16 and (config.split_k > 1 or config.persistent > 0):
    new_workspace = lambda: split_workspace(m, n, config.split_k, device, config.persistent)
  elif config.block_m == 16:
    # The streaming kernel without a split touches no workspace (the entry point only wants a pointer): one
    # allocation per device, not one per call.
    unused = _UNUSED_WORKSPACES.get(device)
    if unused is None:
      unused = _UNUSED_WORKSPACES[device] = torch.empty(64, dtype=torch.int32, device=device)
    new_workspace = lambda: unused
  else:
    new_workspace = lambda: workspace(m, G, config.block_m, device, config.block_n, config.split_k)
  ws = new_workspace()
  cfg = ctypes.byref(config.to_c())
  a_code, b_code, o_code = dtype_code(lhs.dtype), dtype_code(rhs.dtype), dtype_code(out_dtype)
  act_code = _lib.ACTIVATIONS[activation]
  # (Addresses go to the C ABI as plain integers: the declared argument types convert them.)
  if rhs_bias is None and not gateup and scale_blocks == 1 and group_offset is None:
    mode = _lib.TKX_MODE_TRANS_RHS if trans_rhs else _lib.TKX_MODE_DEFAULT
    fwd = lib.tkx_ragged_dot_fwd

    def launch(p, out_ptr, ws_ptr, stream):
      return fwd(p[0], p[1], p[2], p[4], p[5], out_ptr, ws_ptr, m, k, n, G, a_code, b_code, o_code, mode, act_code, cfg, stream)
  else:
    num_sizes, glu = gs.numel(), 1 if gateup else 0
    fused = lib.tkx_ragged_dot_fwd_fused

    def launch(p, out_ptr, ws_ptr, stream):
      return fused(p[0], p[1], p[2], p[3], p[4], p[5], p[6], out_ptr, ws_ptr, m, k, n, G, num_sizes, scale_blocks, a_code,
                   b_code, o_code, act_code, glu, cfg, stream)
  pointers = tuple(0 if t is None else t.data_ptr() for t in (lhs, rhs, gs, group_offset, lhs_scale, rhs_scale, rhs_bias))
  with _on_device(device):
    st = launch(pointers, out.data_ptr(), ws.data_ptr(), torch.cuda.current_stream(device).cuda_stream)
  _lib.check(st)
  if workspace_out is not None:
    workspace_out.append(ws)
  _log_launch(ForwardLaunch(pointers, launch, out, new_workspace))
  return out


def dequantize_weights(qvalue: torch.Tensor, scale: torch.Tensor) -> torch.Tensor:
  """bf16 [g,k,n] = int8 qvalue [g,k,n] * scale [g, k/t_k, n] repeated t_k times along k (quantization.py:80-83)."""
  _log_launch(None)
  _require_cuda(qvalue, scale)
  lib = _lib.load()
  if qvalue.dim() != 3 or scale.dim() != 3 or qvalue.dtype != torch.int8:
    raise NotImplementedError("expected int8 qvalue [g,k,n] and scale [g, k/t_k, n]")
  G, k, n = qvalue.shape
  if scale.shape[0] != G or scale.shape[2] != n or scale.shape[1] < 1 or k % scale.shape[1] != 0:
    raise NotImplementedError(f"scale shape {tuple(scale.shape)} does not tile qvalue {tuple(qvalue.shape)} along k")
  qvalue = qvalue.contiguous()
  scale = scale.to(torch.float32).contiguous()
  out = torch.empty((G, k, n), dtype=torch.bfloat16, device=qvalue.device)
  with _on_device(qvalue.device):
    st = lib.tkx_dequantize_weights(_ptr(qvalue), _ptr(scale), _ptr(out), G, k, n, k // scale.shape[1],
                                    _lib.TKX_I8, _lib.TKX_BF16, _stream(qvalue.device))
  _lib.check(st)
  return out


_QMAX = {torch.int8: 127.0, torch.float8_e4m3fn: 448.0}
for _bits in range(2, 8):
  if hasattr(torch, f"int{_bits}"):
    _QMAX[getattr(torch, f"int{_bits}")] = float(2 ** (_bits - 1) - 1)  # sub-byte integers live in int8 storage


def quantize(x: torch.Tensor, qtype: torch.dtype, tile_shape, bound: float | None = None) -> tuple[torch.Tensor, torch.Tensor]:
  """(qvalue, scale) of the absmax quantisation of `x` with one scale per tile of `tile_shape`
  (`qwix.quantize(x, qtype, tiled_axes=dict(enumerate(tile_shape)))`, quantization.py:65-78):
  scale = absmax(tile) / bound (1 for an all-zero tile), qvalue = round_to_nearest_even(x / scale), saturated at qmax.
  `bound` defaults to qmax (127, 7, 448); qmax + 0.5 is the other convention in use for integers (then -qmax - 1 appears).

  x f32, bf16 or f16: [rows, cols] with tiles one row tall and a multiple of 8 columns wide, or several rows tall and
  1 column or a multiple of 8 columns wide; or weights [g, k, n] with a tile (1, t_k, t_n) (taken as g * k rows) or a
  tile (t_g, k, t_n) of whole groups (one scale per tensor: (g, k, n)). qtype int8, fp8 (e4m3fn) or a sub-byte integer
  (int4: values in [-7, 7], kept in int8 storage)."""
  _log_launch(None)
  _require_cuda(x)
  lib = _lib.load()
  if qtype not in _QMAX:
    raise NotImplementedError(f"quantisation to {qtype} is not supported by the hip implementation")
  if x.dim() not in (2, 3) or len(tile_shape) != x.dim():
    raise NotImplementedError("expected an array of 2 or 3 dimensions and a tile shape of as many")
  tile_shape = tuple(int(t) for t in tile_shape)
  if any(t < 1 or d % t for d, t in zip(x.shape, tile_shape)):
    raise NotImplementedError(f"tile shape {tile_shape} does not tile {tuple(x.shape)}")
  t_r, t_c = tile_shape[-2], tile_shape[-1]
  if x.dim() == 3:
    if tile_shape[0] != 1:
      # A tile over several groups is a run of consecutive rows of [g * k, n] only when it takes whole groups.
      if tile_shape[1] != x.shape[1]:
        raise NotImplementedError("a tile over several groups must span their whole contraction: (t_g, k, t_n)")
      t_r = tile_shape[0] * x.shape[1]
    rows, cols = x.shape[0] * x.shape[1], x.shape[2]
  else:
    rows, cols = x.shape
  x = x.contiguous()
  storage = torch.float8_e4m3fn if qtype == torch.float8_e4m3fn else torch.int8
  qvalue = torch.empty(x.shape, dtype=storage, device=x.device)
  scale = torch.empty(tuple(d // t for d, t in zip(x.shape, tile_shape)), dtype=torch.float32, device=x.device)
  with _on_device(x.device):
    st = lib.tkx_quantize(_ptr(x), _ptr(qvalue), _ptr(scale), rows, cols, t_r, t_c, dtype_code(x.dtype), dtype_code(storage),
                          ctypes.c_float(_QMAX[qtype]), ctypes.c_float(0.0 if bound is None else bound), _stream(x.device))
  _lib.check(st)
  return qvalue, scale


def ragged_dot_fwd_fp8_out(lhs, rhs, group_sizes, *, config: KernelConfig, lhs_scale=None, rhs_scale=None,
                           activation: str | None = None) -> tuple[torch.Tensor, torch.Tensor]:
  """(qvalue fp8 [m,n], scale f32 [m, n/128]) of lhs[m,k] . rhs[g,k,n], quantised per (row, 128 columns) in the
  kernel's epilogue (`tkx_ragged_dot_fwd_fp8_out`): bf16 x bf16 or fp8 x fp8 with one scale per row / per (group,
  column), n % 128 == 0, a tiled variant. NotImplementedError where the library has no such kernel."""
  _log_launch(None)
  _require_cuda(lhs, rhs, group_sizes, lhs_scale, rhs_scale)
  lib = _lib.load()
  if lhs.dim() != 2 or rhs.dim() != 3:
    raise ValueError(f"expected lhs [m,k] and rhs [g,k,n], got {tuple(lhs.shape)} and {tuple(rhs.shape)}")
  lhs, rhs = lhs.contiguous(), rhs.contiguous()
  gs = _group_sizes_i32(group_sizes)
  G, k, n = rhs.shape
  m = lhs.shape[0]
  if gs.numel() != G or lhs.shape[1] != k:
    raise ValueError("group_sizes / contraction sizes do not fit rhs")
  if n % 128:
    raise NotImplementedError("a quantised result needs n % 128 == 0")
  if lhs_scale is not None:
    lhs_scale = lhs_scale.to(torch.float32).contiguous().view(-1)
    if lhs_scale.numel() != m:
      raise NotImplementedError("lhs scale must be one f32 per row")
  if rhs_scale is not None:
    rhs_scale = rhs_scale.to(torch.float32).contiguous().view(-1)
    if rhs_scale.numel() != G * n:
      raise NotImplementedError("rhs scale must be one f32 per (group, column)")
  out = torch.empty((m, n), dtype=torch.float8_e4m3fn, device=lhs.device)
  out_scale = torch.empty((m, n // 128), dtype=torch.float32, device=lhs.device)
  ws = workspace(m, G, config.block_m, lhs.device)
  # (The quantising epilogue needs a row's 128 columns complete in one workgroup: no split last round here.)
  cfg = dataclasses.replace(config, split_k=1).to_c()
  with _on_device(lhs.device):
    st = lib.tkx_ragged_dot_fwd_fp8_out(_ptr(lhs), _ptr(rhs), _ptr(gs), _ptr(lhs_scale), _ptr(rhs_scale), _ptr(out),
                                        _ptr(out_scale), _ptr(ws), m, k, n, G, dtype_code(lhs.dtype), dtype_code(rhs.dtype),
                                        _lib.ACTIVATIONS[activation], ctypes.byref(cfg), _stream(lhs.device))
  _lib.check(st)
  return out, out_scale


def row_sums_fp8(x: torch.Tensor, out: torch.Tensor | None = None, per_128_columns: bool = False) -> torch.Tensor:
  """f32 [rows]: the sums of the rows of an fp8 (e4m3fn) matrix [rows, cols], cols % 16 == 0; `per_128_columns`
  (cols % 128 == 0): f32 [cols / 128, rows], one sum per run of 128 columns. What the fp8 x packed-int4 forward takes
  behind its row scales (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:436-470 packs the sum of an activation row, or of
  each of its subchannels, with its scales the same way)."""
  _log_launch(None)
  _require_cuda(x)
  if x.dtype != torch.float8_e4m3fn or x.dim() != 2:
    raise ValueError(f"expected an fp8 (e4m3fn) matrix, got {x.dtype} {tuple(x.shape)}")
  x = x.contiguous()
  if per_128_columns and x.shape[1] % 128:
    raise NotImplementedError("sums per 128 columns need cols % 128 == 0")
  shape = (x.shape[1] // 128, x.shape[0]) if per_128_columns else (x.shape[0],)
  if out is None:
    out = torch.empty(shape, dtype=torch.float32, device=x.device)
  if out.dtype != torch.float32 or out.numel() != math.prod(shape) or not out.is_contiguous() or out.device != x.device:
    raise ValueError("out must be a contiguous f32 tensor with one entry per sum, on x's device")
  if x.shape[0] and x.shape[1]:
    lib = _lib.load()
    with _on_device(x.device):
      _lib.check(lib.tkx_row_sums_fp8(_ptr(x), _ptr(out), x.shape[0], x.shape[1], 128 if per_128_columns else x.shape[1],
                                      _stream(x.device)))
  return out


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
  """int8 [.., 2 r, c] from uint8 [.., r, c] holding two int4 per byte along the second-to-last axis (entry 2 i in
  bits 0-3, entry 2 i + 1 in bits 4-7, two's complement)."""
  return _int4_repack(packed, True)


def pack_int4(values: torch.Tensor) -> torch.Tensor:
  """The inverse of `unpack_int4` for int8 values in [-8, 7] (the low four bits of anything else are kept)."""
  return _int4_repack(values, False)


def _int4_repack(x: torch.Tensor, unpack: bool) -> torch.Tensor:
  _log_launch(None)
  _require_cuda(x)
  want = torch.uint8 if unpack else torch.int8
  if x.dtype != want or x.dim() < 2 or x.shape[-1] % 16 or (not unpack and x.shape[-2] % 2):
    raise NotImplementedError(f"expected {want} [.., rows, cols] with cols % 16 == 0 (and an even number of rows to pack),"
                              f" got {x.dtype} {tuple(x.shape)}")
  x = x.contiguous()
  rows = x.shape[-2] * 2 if unpack else x.shape[-2] // 2
  out = torch.empty((*x.shape[:-2], rows, x.shape[-1]), dtype=torch.int8 if unpack else torch.uint8, device=x.device)
  packed_rows = (x.numel() if unpack else out.numel()) // x.shape[-1]
  if packed_rows:
    lib = _lib.load()
    with _on_device(x.device):
      fn = lib.tkx_unpack_int4 if unpack else lib.tkx_pack_int4
      _lib.check(fn(_ptr(x), _ptr(out), packed_rows, x.shape[-1], _stream(x.device)))
  return out


def dequantize(qvalue: torch.Tensor, scale: torch.Tensor, zero_point: torch.Tensor | None = None) -> torch.Tensor:
  """bf16 = (qvalue - zero_point) * scale with each scale (and zero point) entry repeated over its tile
  (quantization.py:80-93).

  qvalue int8 or fp8 (e4m3fn): [rows, cols] with scale [rows/t_r, cols/t_c], or weights [g,k,n] with scale
  [g, k/t_k, n/t_n]; t_c / t_n is 1 or a multiple of 16. `zero_point`, if given, has the scale's shape."""
  _log_launch(None)
  _require_cuda(qvalue, scale, zero_point)
  lib = _lib.load()
  if qvalue.dtype not in (torch.int8, torch.float8_e4m3fn) or qvalue.dim() not in (2, 3) or scale.dim() != qvalue.dim():
    raise NotImplementedError("expected an int8 or fp8 qvalue of 2 or 3 dimensions and a scale of as many")
  if any(s < 1 or q % s for q, s in zip(qvalue.shape, scale.shape)):
    raise NotImplementedError(f"scale shape {tuple(scale.shape)} does not tile qvalue {tuple(qvalue.shape)}")
  if qvalue.dim() == 3:
    if scale.shape[0] != qvalue.shape[0]:
      raise NotImplementedError("one scale set per group expected")
    rows, cols = qvalue.shape[0] * qvalue.shape[1], qvalue.shape[2]
  else:
    rows, cols = qvalue.shape
  t_r, t_c = qvalue.shape[-2] // scale.shape[-2], qvalue.shape[-1] // scale.shape[-1]
  qvalue = qvalue.contiguous()
  scale = scale.to(torch.float32).contiguous()
  out = torch.empty(qvalue.shape, dtype=torch.bfloat16, device=qvalue.device)
  with _on_device(qvalue.device):
    if zero_point is None:
      st = lib.tkx_dequantize(_ptr(qvalue), _ptr(scale), _ptr(out), rows, cols, t_r, t_c, dtype_code(qvalue.dtype),
                              _lib.TKX_BF16, _stream(qvalue.device))
    else:
      if tuple(zero_point.shape) != tuple(scale.shape):
        raise NotImplementedError("the zero point must have the scale's shape")
      zero_point = zero_point.to(torch.float32).contiguous()
      st = lib.tkx_dequantize_zero_point(_ptr(qvalue), _ptr(scale), _ptr(zero_point), _ptr(out), rows, cols, t_r, t_c,
                                         dtype_code(qvalue.dtype), _lib.TKX_BF16, _stream(qvalue.device))
  _lib.check(st)
  return out


def ragged_dot_drhs(lhs, dout, group_sizes, num_groups: int, *, config: KernelConfig,
                    out_dtype: torch.dtype) -> torch.Tensor:
  """out[g,k,n] = lhs[rows_g,k]^T . dout[rows_g,n]."""
  _log_launch(None)
  _require_cuda(lhs, dout, group_sizes)
  lib = _lib.load()
  if lhs.dim() != 2 or dout.dim() != 2 or lhs.shape[0] != dout.shape[0]:
    raise ValueError(f"expected lhs [m,k] and dout [m,n], got {tuple(lhs.shape)} and {tuple(dout.shape)}")
  if lhs.dtype != dout.dtype:
    raise NotImplementedError("lhs and dout must have the same dtype")
  lhs, dout = lhs.contiguous(), dout.contiguous()
  gs = _group_sizes_i32(group_sizes)
  if gs.numel() != num_groups:
    raise ValueError("group_sizes length differs from num_groups")
  m, k = lhs.shape
  n = dout.shape[1]
  out = torch.empty((num_groups, k, n), dtype=out_dtype, device=lhs.device)
  ws = workspace(m, num_groups, 128, lhs.device)
  cfg = config.to_c()
  with _on_device(lhs.device):
    st = lib.tkx_ragged_dot_drhs(_ptr(lhs), _ptr(dout), _ptr(gs), _ptr(out), _ptr(ws), m, k, n, num_groups,
                                 dtype_code(lhs.dtype), dtype_code(out_dtype), ctypes.byref(cfg), _stream(lhs.device))
  _lib.check(st)
  return out
