"""Ragged dot on gfx950 (MI355X): `implementation="hip"`.

Slots into the operator framework the way the reference's GPU backend does
(tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu.py:85-518): a `RaggedDot` subclass with its own
`Config`, `_fwd`, heuristics, autotuning search space and `supported_on`; anything it cannot run
raises `NotImplementedError` so that the dispatcher may try the next implementation. All three
dimension-number sets run natively: the transposed-rhs case (dlhs) reads rhs in place instead
of materialising `rhs.mT` as the reference does (pallas_mosaic_gpu.py:148-150).
"""

from __future__ import annotations

import dataclasses
import functools
from functools import partial
from typing import ClassVar

import torch

from tokamax_amd import _lib
from tokamax_amd import config as config_lib
from tokamax_amd import op
from tokamax_amd import precision as precision_lib
from tokamax_amd import quantization
from tokamax_amd.serialization import ShapeDtype
from tokamax_amd.ragged_dot import base
from tokamax_amd.ragged_dot import hip_ops

QArray = base.QArray
AsQArray = base.AsQArray
GroupSizes = base.GroupSizes


@dataclasses.dataclass(frozen=True)
class Config:
  """Tunables of the hip kernels; counterpart of pallas_mosaic_gpu_common.py:45-73.

  (block_m, block_n, block_k, waves_m, waves_n, num_stages) selects a precompiled kernel variant;
  `grid_tile_width` m-tasks share one n-panel of rhs in launch order (L2 reuse);
  `align_tile` is the row alignment of task starts (the reference's `align_tile`, default 8);
  `split_k` workgroups share the contraction of one output tile (the reference's field of that name): on the streaming
  small-m kernel (block_m == 16) every tile is split; on a tiled forward / dlhs kernel of at least 128 rows only the
  tiles of the launch's last, partial round of workgroups are, into at most that many parts;
  `persistent` (the reference's flag of that name, pallas_mosaic_gpu_common.py:55; here a count): above 0 the streaming
  small-m kernel runs as that many resident workgroups per compute unit, each with an equal share of the weight bytes
  of the non-empty tiles, instead of one workgroup per (group, column tile).
  """

  block_m: int
  block_n: int
  block_k: int
  waves_m: int = 2
  waves_n: int = 2
  num_stages: int = 2
  grid_tile_width: int = 8
  align_tile: int = 8
  split_k: int = 1
  persistent: int = 0

  def __post_init__(self):
    for f in dataclasses.fields(self):
      v = getattr(self, f.name)
      if not isinstance(v, int) or isinstance(v, bool) or v < (0 if f.name == "persistent" else 1):
        raise ValueError(f"Config.{f.name} must be a positive int, got {v!r}")
    if self.block_m % 8 != 0:
      raise ValueError(f"Config.block_m must be a multiple of 8, got {self.block_m}")

  def to_kernel_config(self) -> hip_ops.KernelConfig:
    return hip_ops.KernelConfig(self.block_m, self.block_n, self.block_k, self.waves_m, self.waves_n,
                                self.num_stages, self.grid_tile_width, self.align_tile, self.split_k, self.persistent)


_COMPUTE_UNITS = 256  # of an MI355X: a launch's tiles run in rounds of that many


def _tiled_split_pays(mode: int, block_m: int, block_n: int, rows: int, cols: int, num_groups: int) -> bool:
  """Whether a tiled forward / dlhs launch gets `split_k` (the tiles of its last, partial round of workgroups are cut
  along the contraction; the kernel itself decides into how many parts, and leaves a round that is more than half full
  alone). Measured on the backward product of the Mixtral shape (m = 4096: 2.4 rounds of 128 x 256 tiles): +23 %; on
  the forward pass at m = 16384 (14.4 rounds) the exchange of partial tiles costs what the shorter round saves, so
  launches of 8 rounds and more stay as they are. Tiles of at least 128 rows have the kernels for it."""
  if mode not in (0, 1) or block_m < 128:
    return False
  tiles = (-(-rows // block_m) + (num_groups - 1) // 2) * -(-cols // block_n)
  return tiles < 8 * _COMPUTE_UNITS


# Constants of `_tile_cost`, fitted by tokamax_amd/data/autotuning/tile_cost.py to the timings beside it.
_TILE_COST_FIT = dict(
    mfma_flop_per_us=6.142e6,    # a CU's MFMA rate on a full tile
    load_byte_per_us=59.31e3,    # a CU's rate of bringing operand slices into LDS
    partial_block=1.475,         # 32-row blocks' worth of rows that a task costs beyond the rows it has
    four_wave_factor=1.033,      # MFMA time of a 4-wave tile against an 8-wave one
    in_flight_full=64.97,        # contraction elements in flight from which loads run at their full rate
    in_flight_exponent=1.802,
    fixed_us=3.348,              # per tile: start-up and epilogue
    fixed_area_us=3.636,         # ... more per 256x256 of output
    shared_cu_mfma=1.396,        # two workgroups on a CU: each k-step takes 2x this (MFMA bound)
    shared_cu_load=0.9206,       # ... or 2x this (load bound)
    tail_floor=0.4117,           # a partial round behind full ones costs at least this share of a round
    exchange_us=26.43,           # price of splitting the last round along the contraction
    group_straddle=0.8914,       # extra tiles per group at an arbitrary row offset
    short_piece=1.526,           # time of loading 64-byte pieces of rows against 128-byte ones
)


def _tile_cost(variant, split_k: int, rows: int, cols: int, contraction: int, num_groups: int, mode: int = 0,
               fit=_TILE_COST_FIT, rhs_bytes: float = 2.0, shares_cu: bool | None = None) -> float:
  """Estimated time (us) of a tiled forward / dlhs launch of 16-bit operands: rounds of workgroups times the time of a
  tile. A tile's k-step costs the larger of its MFMA time (less where the task's rows do not fill the share of the
  wave that holds them) and the time to bring its operand slices into LDS, which a pipeline with less than about 65
  contraction elements in flight stretches; a tile also pays a fixed time (start-up and epilogue, growing with its
  area). Shapes whose LDS lets two 4-wave workgroups share a CU run two tiles at a time at less than half the pace
  each, so that their fixed times overlap. A group of r rows at an arbitrary offset touches about r / block_m + 0.89
  tiles. A partial round behind full ones overlaps with them in part; with `split_k` its tiles are cut into parts at
  the price of the exchange.
  The constants were fitted to the measured times of every compiled variant on 122 shapes (m = 256 .. 262144, k and
  n = 256 .. 14336, 2 .. 256 groups, forward and dlhs; 2852 timings): the variant this picks is within 4 % of the
  fastest one on average and 31 % at worst on those shapes. On 12 further shapes that no fit has seen it is within
  6 % on average and 24 % at worst (8 % and 48 % before the term for 64-byte pieces, which one of them prompted),
  against 21 % and 52 % for rules on rows per group alone; an earlier fit to 110 of the shapes was within 10 % and 47 %
  on the 12 others, against 30 % and 77 % for those rules."""
  bm, bn, bk, wm, wn, ns = variant
  tasks = min(rows / bm + fit["group_straddle"] * num_groups, -(-rows // bm) + num_groups - 1)
  tiles = tasks * -(-cols // bn)
  four_waves = wm * wn == 4
  two_per_cu = four_waves and 2 * ns * (bm * 2 + bn * rhs_bytes) * bk <= 160 * 1024
  if shares_cu is not None:
    two_per_cu = shares_cu  # (the caller knows: 8-wave tiles of converted weights on one row of waves can share too)
  # (the waves of a tile split its rows `wm` ways and the slowest one sets the pace: the rows count against a wave's share)
  active = min(1.0, (rows / tasks + fit["partial_block"] * 32) * wm / bm)
  mma_us = bm * bn * bk * 2 / fit["mfma_flop_per_us"] * active * (fit["four_wave_factor"] if four_waves else 1.0)
  in_flight = min(1.0, ((ns - 1) * bk / fit["in_flight_full"]) ** fit["in_flight_exponent"])
  # (a 32-element slice of an operand that is contiguous along the contraction, as the lhs is and in dlhs the weights
  # are too, is read in 64-byte pieces)
  short = fit["short_piece"] if bk < 64 else 1.0
  load_us = (bm * 2 * short + bn * rhs_bytes * (short if mode == 1 else 1.0)) * bk / fit["load_byte_per_us"] / in_flight
  steps = -(-contraction // bk)
  fixed_us = fit["fixed_us"] + fit["fixed_area_us"] * bm * bn / 65536
  alone_us = steps * max(mma_us, load_us) + fixed_us
  if two_per_cu:
    tile_us = steps * 2 * max(fit["shared_cu_mfma"] * mma_us, fit["shared_cu_load"] * load_us) + fixed_us
  else:
    tile_us = alone_us
  slots = _COMPUTE_UNITS * (2 if two_per_cu else 1)
  full_rounds = int(tiles // slots)
  rest = tiles - full_rounds * slots
  total = full_rounds * tile_us
  if rest > 0:
    last = alone_us if two_per_cu and rest <= _COMPUTE_UNITS else tile_us
    if full_rounds > 0 and not shares_cu:
      # (not behind a round of paired 8-wave workgroups: those start together and end together)
      last *= fit["tail_floor"] + (1 - fit["tail_floor"]) * rest / slots
    if split_k > 1:
      beyond = int(tiles) % _COMPUTE_UNITS
      parts = min(split_k, _COMPUTE_UNITS // beyond) if beyond > 0 else 1
      if parts > 1:
        last = last / parts + fit["exchange_us"]
    total += last
  return total


def _streaming_split(tiles: int, contraction: int, block_n: int, depth: int) -> int:
  """Workgroups per (group, column tile) of the streaming small-m kernel. Unsplit, a launch has `tiles` workgroups;
  with fewer than one per CU, splitting the contraction until there are 256 measured 1.3x (128 tiles) to 3.5x
  (16 tiles) faster, 8 splits at most (beyond that the reduction costs more than the parallelism gains); from
  about 190 tiles on it measured slower at every split (each workgroup's fixed costs outweigh the finer balance)."""
  if block_n != 128 or depth > 4 or tiles < 1:
    return 1
  split = 1
  while split < 8 and tiles * split * 2 <= 256 and contraction % (128 * split * 2 * min(depth, 4)) == 0:
    split *= 2
  return split


_ACTIVATION_NAMES = {
    torch.relu: "relu",
    torch.nn.functional.relu: "relu",
    torch.tanh: "tanh",
    torch.nn.functional.tanh: "tanh",
    torch.nn.functional.silu: "silu",
    torch.sigmoid: "sigmoid",
    torch.nn.functional.sigmoid: "sigmoid",
}


# `fuse_gateup_activation` names (experimental/gmm_v2/gmm_v2.py:96-107) -> in-kernel activation.
# "gelu" is `jax.nn.gelu(gate)`, whose default is the tanh form.
_GATEUP_ACTIVATIONS = {"silu": "silu", "gelu": "gelu_tanh", "gelu_tanh": "gelu_tanh", "swigluoai": "swigluoai",
                       "silu_and_mul_with_clamp": "silu_and_mul_with_clamp"}


def _fused_activation_name(activation) -> str | None:
  """Name of the in-kernel epilogue for a known activation callable, else None."""
  try:
    return _ACTIVATION_NAMES.get(activation)
  except TypeError:  # unhashable callable
    return None


def _scale_blocks_along_k(q: QArray) -> int | None:
  """Number of scale blocks along k of a quantised rhs [g,k,n] (scale [g, blocks, n]), or None if the
  scale has another form."""
  g, k, n = q.qvalue.shape
  shape = tuple(q.scale.shape)
  if len(shape) != 3 or shape[0] != g or shape[2] != n or shape[1] < 1 or k % shape[1] != 0:
    return None
  return shape[1]


def _rhs_scale_tiles(q: QArray) -> bool:
  """Scale [g, k/t_k, n/t_n] with t_n a multiple of 16 (block scales along both k and n)."""
  g, k, n = q.qvalue.shape
  shape = tuple(q.scale.shape)
  return (len(shape) == 3 and shape[0] == g and shape[1] >= 1 and shape[2] >= 1 and k % shape[1] == 0
          and n % shape[2] == 0 and (n // shape[2]) % 16 == 0)


def _per_column_rhs_scale(rhs):
  """A quantised rhs whose scale is tiled along n ([g, k/t_k, n/t_n], e.g. 128 x 128 blocks) with every scale
  repeated over its t_n columns ([g, k/t_k, n]): the form the kernels take. Works on tensors and on shapes."""
  if not isinstance(rhs, QArray) or len(rhs.scale.shape) != 3 or len(rhs.qvalue.shape) != 3:
    return rhs
  g, n = rhs.qvalue.shape[0], rhs.qvalue.shape[2]
  gs, nt = rhs.scale.shape[0], rhs.scale.shape[2]
  if (nt == n and gs == g) or nt < 1 or n % nt != 0 or gs < 1 or g % gs != 0:
    return rhs
  if isinstance(rhs.scale, torch.Tensor):
    # (a scale set shared by runs of g / gs consecutive groups, e.g. by all of them, is repeated for each)
    scale = rhs.scale.repeat_interleave(g // gs, dim=0) if gs != g else rhs.scale
    scale = scale.repeat_interleave(n // nt, dim=2) if nt != n else scale.contiguous()
  else:
    scale = ShapeDtype((g, rhs.scale.shape[1], n), rhs.scale.dtype)
  return QArray(rhs.qvalue, scale, rhs.zero_point, rhs.qtype)


def _per_row_lhs_scale(lhs):
  """A quantised lhs [m, k] whose scale rows are shared by runs of consecutive lhs rows ([m / t_m, blocks]: tiles
  several rows tall, one scale per tensor) with each scale row repeated for its lhs rows. Works on tensors and on shapes."""
  if not isinstance(lhs, QArray) or len(lhs.scale.shape) != 2 or len(lhs.qvalue.shape) != 2:
    return lhs
  m = lhs.qvalue.shape[0]
  rows, blocks = lhs.scale.shape
  k = lhs.qvalue.shape[1]
  if rows == m or rows < 1 or m % rows != 0 or blocks < 1 or k % blocks != 0 or (blocks != 1 and (k // blocks) % 16 != 0):
    return lhs  # (as it should be, or a form that is widened with its own tile shape)
  if isinstance(lhs.scale, torch.Tensor):
    scale = lhs.scale.repeat_interleave(m // rows, dim=0)  # (scale tiles several rows tall: (256, 1), one per tensor)
  else:
    scale = ShapeDtype((m, lhs.scale.shape[1]), lhs.scale.dtype)
  return QArray(lhs.qvalue, scale, lhs.zero_point, lhs.qtype)


def _lhs_scale_blocks(q: QArray) -> int | None:
  """Number of scale blocks along k of a quantised lhs [m,k] (scale [m, blocks], blocks of a multiple of 16
  columns), or None if the scale has another form."""
  m, k = q.qvalue.shape
  shape = tuple(q.scale.shape)
  if shape == (m, 1):
    return 1
  if len(shape) != 2 or shape[0] != m or shape[1] < 1 or k % shape[1] != 0 or (k // shape[1]) % 16 != 0:
    return None
  return shape[1]


def _widening_pass_takes(q: QArray) -> bool:
  """Whether `tkx_dequantize` takes this operand: the scale tiles the values, in blocks 1 or a multiple of 16 columns
  wide (the last axis), over row-major values whose rows are a multiple of 16 entries."""
  shape, sshape = tuple(q.qvalue.shape), tuple(q.scale.shape)
  if len(shape) != len(sshape) or len(shape) not in (2, 3) or shape[-1] % 16:
    return False
  if any(s < 1 or d % s for d, s in zip(shape, sshape)):
    return False
  if len(shape) == 3 and sshape[0] != shape[0]:
    return False
  t_c = shape[-1] // sshape[-1]
  return t_c == 1 or t_c % 16 == 0


def _widening_plan(lhs, rhs, allow_native: bool = True) -> tuple[bool, bool, bool]:
  """(widen lhs, widen rhs, native k-blocks): how a pair of (possibly quantised) operands reaches the kernels.

  * One scale per lhs row and one per (group, column): applied in the kernels' epilogue (bf16 x int8, fp8 x fp8,
    int8 x int8), nothing is widened.
  * "native k-blocks" (`allow_native`: no gate-up fusion): scales [g, k/t_k, n] go to the kernels as they are, to
    - fp8 x fp8 and int8 x int8 with the same k-blocks on both sides (xs[row, k_sub] ws[g, k_sub, n],
      pallas_mosaic_gpu_kernel_sm100_i8_quant.py:51-102): MFMA kernels that fold the scales in per k-block;
    - int8 or fp8 weights under a bf16 lhs (the scale tile (1, t_k, 1) of pallas_mosaic_gpu_kernel_sm90_quant.py:91-97;
      fp8 weights also with a single block): kernels that scale the weights while they widen them; a quantised lhs
      is widened to bf16 for them.
    t_k is a power of two that the kernels' k-step divides.
  * Everything else that is quantised is dequantised to bf16 by a widening pass first; an fp8 operand whose partner
    was widened is widened too (there is no bf16 x fp8 kernel outside the native ones)."""
  lhs_q, rhs_q = isinstance(lhs, QArray), isinstance(rhs, QArray)
  widen_lhs = widen_rhs = False
  blocks = lhs_blocks = None  # (scale blocks along k of a quantised rhs / lhs)
  if lhs_q:
    lhs_blocks = _lhs_scale_blocks(lhs)
    if lhs_blocks is None:
      # Any other tiling (row blocks, one scale per column, 2-d blocks) goes through the widening pass, as the
      # reference's sm90 path dequantises a quantised lhs first (pallas_mosaic_gpu.py:152-154).
      if not _widening_pass_takes(lhs):
        raise NotImplementedError("lhs scale must tile lhs [m,k] in blocks 1 or a multiple of 16 columns wide, got"
                                  f" {tuple(lhs.scale.shape)}")
      lhs_blocks = 0
    widen_lhs = lhs_blocks != 1 or _dtype_of(lhs) == torch.int8  # (unless int8 meets int8 below)
  if rhs_q:
    blocks = _scale_blocks_along_k(rhs)
    if blocks is None and not _rhs_scale_tiles(rhs) and not _widening_pass_takes(rhs):
      raise NotImplementedError("rhs scale must have shape [g,1,n], [g,k/t_k,n] or [g,k/t_k,n/t_n] with 16 | t_n, got"
                                f" {tuple(rhs.scale.shape)}")
    widen_rhs = blocks is None or blocks > 1
  eight_bit_float = lambda x: _dtype_of(x) == torch.float8_e4m3fn
  both_int8 = (lhs_q and rhs_q and _dtype_of(lhs) == torch.int8 and _dtype_of(rhs) == torch.int8
               and lhs.qvalue.dtype == torch.int8 and rhs.qvalue.dtype == torch.int8)
  both_fp8 = lhs_q and rhs_q and eight_bit_float(lhs) and eight_bit_float(rhs)
  if (allow_native and (both_fp8 or both_int8) and blocks is not None and (blocks > 1 or both_int8)
      and lhs_blocks == blocks):
    # The same k-blocks on both sides: the fp8 (int8) MFMA kernels that fold the scales in per k-block; int8 x int8
    # also with a single block (there is no other kernel that contracts int8 activations).
    m, k = lhs.qvalue.shape
    rows = k // blocks
    step = 128 if both_fp8 else 64
    shape_ok = k % step == 0 and (blocks == 1 or (rows % step == 0 and rows & (rows - 1) == 0))
    # (Groups of a few rows are better off with a widened lhs and the streaming small-m kernel, below.)
    if both_int8 and blocks == 1 and k % 16 == 0:
      return False, False, False  # one scale per row and per column: the plain int8 MFMA variants, scales in the epilogue
    if shape_ok and m % 4 == 0 and rhs.qvalue.shape[2] % 16 == 0 and m > 8 * rhs.qvalue.shape[0]:
      return False, False, True
  if rhs_q and allow_native and blocks is not None and rhs.qvalue.dtype in (torch.int8, torch.float8_e4m3fn):
    # Kernels of their own (bf16 lhs; 256-column tiles) for int8 weights with several scale blocks along k and
    # for fp8 weights with any number of them, unless fp8 meets fp8 with one scale each (the fp8 MFMA kernels).
    _, k, n = rhs.qvalue.shape
    rows = k // blocks
    shape_ok = n % 16 == 0 and k % 64 == 0 and (blocks == 1 or (rows % 64 == 0 and rows & (rows - 1) == 0))
    fp8_pair = lhs_q and eight_bit_float(lhs) and not widen_lhs and blocks == 1
    wanted = blocks > 1 or (eight_bit_float(rhs) and not fp8_pair)
    lhs_becomes_bf16 = lhs_q or lhs.dtype == torch.bfloat16  # (a quantised lhs is widened for it)
    if shape_ok and wanted and lhs_becomes_bf16:
      return lhs_q, False, True
  if widen_rhs and lhs_q and eight_bit_float(lhs):
    widen_lhs = True
  if widen_lhs and rhs_q and eight_bit_float(rhs):
    widen_rhs = True
  if lhs_q and eight_bit_float(lhs) and not widen_lhs and not eight_bit_float(rhs):
    # fp8 activations meet fp8 weights on the fp8 MFMAs (and packed int4 ones in kernels of their own, settled before
    # this plan); under any other partner (int8 or 16-bit weights) they are widened.
    widen_lhs = True
  if (widen_lhs and not rhs_q and eight_bit_float(rhs)) or (widen_rhs and not lhs_q and eight_bit_float(lhs)):
    raise NotImplementedError("A raw fp8 operand cannot meet a widened (bf16) one.")
  return widen_lhs, widen_rhs, False


_SUB_BYTE_INTS = tuple(getattr(torch, f"int{b}") for b in range(1, 8) if hasattr(torch, f"int{b}"))


def _dtype_of(x) -> torch.dtype:
  """The element type the kernels see. torch has no packed sub-byte tensors: a QArray whose qtype is int4
  (or another sub-byte integer) holds its values in int8 storage and runs as int8."""
  if isinstance(x, QArray) and x.qtype in _SUB_BYTE_INTS and x.qvalue.dtype == torch.int8:
    return torch.int8
  return x.qtype if isinstance(x, (QArray, AsQArray)) else x.dtype


@functools.lru_cache(maxsize=None)
def _variant_table():
  """{(mode, lhs dtype code, rhs dtype code): [(bm, bn, bk, wm, wn, stages), ...]} from the library."""
  table: dict = {}
  for kind in (0, 1):
    for v in _lib.variants(kind):
      key = (v["mode"], v["lhs_dtype"], v["rhs_dtype"])
      table.setdefault(key, []).append((v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"]))
  return table


_MODE_OF_DIMS = {
    base.DEFAULT_RAGGED_DOT_DIM_NUMS: 0,
    base.TRANS_RHS_RAGGED_DOT_DIM_NUMS: 1,
    base.RAGGED_CONTRACTING_DOT_DIM_NUMS: 2,
}


@functools.lru_cache(maxsize=None)
def _is_gfx950(device: torch.device) -> bool:
  arch = getattr(torch.cuda.get_device_properties(device), "gcnArchName", "")
  return arch.split(":")[0] == "gfx950"


@dataclasses.dataclass(frozen=True)
class _Route:
  """How one call reaches the kernels; computed from shapes and types only, so that the forward pass (on arrays) and
  the choice of a config (on abstract arguments) cannot disagree."""

  mode: int          # variant-table mode: 0 forward, 1 dlhs, 2 drhs, 3 forward with gate-up fusion, 4 k-block scales
  lhs: object        # operands in the form the plan was made for (shared scales repeated, raw rhs_scale folded in)
  rhs: object
  lhs_dtype: torch.dtype  # element types the kernel sees
  rhs_dtype: torch.dtype
  widen_lhs: bool    # the operand goes through the widening pass (tkx_dequantize) first
  widen_rhs: bool
  native_k_blocks: bool
  cast_bf16: bool    # the BF16_BF16_F32 preset: both (unquantised) operands are cast to bf16
  preferred_element_type: object

  @property
  def key(self):
    return (self.mode, hip_ops.dtype_code(self.lhs_dtype), hip_ops.dtype_code(self.rhs_dtype))


def _route(lhs, rhs, *, dims, precision, rhs_scale, fuse_gateup_activation, preferred_element_type) -> _Route:
  """Plans a call. `lhs` / `rhs` are arrays, `QArray`s or their abstract forms (an `AsQArray` has been turned into the
  `QArray` it quantises to, an operand with a zero point into the bf16 array it dequantises to)."""
  mode = _MODE_OF_DIMS.get(dims)
  if mode is None:
    raise NotImplementedError("Unsupported ragged dot dimension numbers.")
  if rhs_scale is not None:
    # The raw-array form of quantised weights (experimental/gmm_v2/gmm_v2.py:1193-1199): rhs holds the quantised values
    # and rhs_scale is [g, k-blocks, 1, n]; the result defaults to lhs.dtype (:1369-1370).
    if isinstance(lhs, QArray) or isinstance(rhs, QArray):
      raise NotImplementedError("rhs_scale comes with raw arrays, not QArrays.")
    g, k, n = rhs.shape
    if len(rhs_scale.shape) != 4 or tuple(rhs_scale.shape[::2]) != (g, 1) or rhs_scale.shape[3] != n:
      raise NotImplementedError(f"rhs_scale must have shape [g, k-blocks, 1, n], got {tuple(rhs_scale.shape)}")
    scale = (rhs_scale.reshape(g, rhs_scale.shape[1], n) if isinstance(rhs_scale, torch.Tensor)
             else ShapeDtype((g, rhs_scale.shape[1], n), rhs_scale.dtype))
    rhs = QArray(rhs, scale)
    if preferred_element_type is None:
      preferred_element_type = lhs.dtype
  gateup = fuse_gateup_activation is not None
  if (gateup or rhs_scale is not None) and mode != 0:
    raise NotImplementedError("rhs_scale and fuse_gateup_activation need the default dimension numbers.")
  if isinstance(rhs, QArray) and rhs.packed:
    # Packed int4 that `_settle_packed_int4` left packed: bf16 lhs x a kernel that reads the bytes, scales as they are
    # (blocks along k: the kernels' own form, as for int8 weights).
    if not precision_lib.is_default(lhs.dtype, rhs.dtype, precision):
      raise NotImplementedError(f"{precision=} not supported.")
    if preferred_element_type is None:
      preferred_element_type = torch.promote_types(lhs.dtype, rhs.dtype)
    k_blocks = rhs.scale.shape[1] > 1
    if isinstance(lhs, QArray):
      # fp8 or int8 activations with one scale per row: the kernels that feed the nibbles to the fp8 / int8 MFMAs.
      lhs_dt = torch.int8 if _dtype_of(lhs) == torch.int8 else torch.float8_e4m3fn
      return _Route(3 if gateup else 4 if k_blocks else 0, _per_row_lhs_scale(lhs), rhs, lhs_dt, torch.uint8,
                    False, False, k_blocks, False, preferred_element_type)
    return _Route(3 if gateup else 4 if k_blocks else 0, lhs, rhs, torch.bfloat16, torch.uint8, False, False, k_blocks,
                  False, preferred_element_type)
  lhs_dt, rhs_dt = _dtype_of(lhs), _dtype_of(rhs)
  widen_lhs = widen_rhs = native = False
  if mode == 0:
    lhs, rhs = _per_row_lhs_scale(lhs), _per_column_rhs_scale(rhs)
    widen_lhs, widen_rhs, native = _widening_plan(lhs, rhs, allow_native=not gateup)
    if (gateup and isinstance(rhs, QArray) and not widen_rhs and rhs.qvalue.dtype in (torch.int8, torch.float8_e4m3fn)
        and rhs.qvalue.shape[2] % 32):
      # Gate-up fusion reads the up half of a weight row n / 2 elements in, which is a whole 16-byte piece of one-byte
      # weights only if n % 32 == 0: otherwise the weights are widened first (and quantised activations with them).
      widen_rhs = True
      widen_lhs = widen_lhs or isinstance(lhs, QArray)
  else:
    # dlhs / drhs contract unquantised operands (base.py:395-410 rejects quantised ones on the backward path); a
    # quantised operand in a direct call is widened first, as pallas_mosaic_gpu.py:170 does for the drhs product.
    for x in (lhs, rhs):
      if isinstance(x, QArray) and not _widening_pass_takes(x):
        raise NotImplementedError(f"cannot dequantise an operand with scale {tuple(x.scale.shape)} for this product")
    widen_lhs, widen_rhs = isinstance(lhs, QArray), isinstance(rhs, QArray)
  lhs_dt = torch.bfloat16 if widen_lhs else lhs_dt
  rhs_dt = torch.bfloat16 if widen_rhs else rhs_dt
  in_dtype = lhs.dtype if isinstance(lhs, QArray) else lhs_dt   # (a QArray's dtype: what it dequantises to)
  w_dtype = rhs.dtype if isinstance(rhs, QArray) else rhs_dt
  cast_bf16 = False
  if not precision_lib.is_default(in_dtype, w_dtype, precision):
    if (precision == precision_lib.DotAlgorithmPreset.BF16_BF16_F32 and not isinstance(lhs, QArray)
        and not isinstance(rhs, QArray)):
      cast_bf16 = True
      lhs_dt = rhs_dt = torch.bfloat16
    else:
      raise NotImplementedError(f"{precision=} not supported.")
  if preferred_element_type is None:
    preferred_element_type = torch.promote_types(in_dtype, w_dtype)
  if mode == 0:
    mode = 3 if gateup else 4 if native else 0
  return _Route(mode, lhs, rhs, lhs_dt, rhs_dt, widen_lhs, widen_rhs, native, cast_bf16, preferred_element_type)


_PACKED_INT4_TILE_STEP = 64  # k-step of the tiled kernels that read packed int4 weights
_PACKED_INT4_FP8_TILE_STEP = 128  # ... under fp8 activations


def _settle_packed_int4(lhs, rhs, *, dims, plain: bool = True, gateup: bool = False):
  """An rhs of packed int4 (two values per byte along k) stays packed when a kernel reads it as it is: default
  dimension numbers, a plain bf16 lhs, n % 16 == 0, and either
  * the tiled kernels: k a multiple of their k-step (64); one scale per (group, column), or, without gate-up fusion, per
    (group, k-block, column) with blocks of a power of two >= 64 rows, or
  * the streaming small-m kernel: no bias and no gate-up fusion (`plain`), at most 8 rows per group on average,
    k % 1024 == 0, one scale per (group, column) or per (group, k-block, column) with blocks of a power of two >= 32 rows;
  or under an lhs quantised to fp8 (e4m3fn) with one scale per row (or shared by runs of rows) and k % 128 == 0: the
  tiled kernels that feed the nibbles to the fp8 MFMAs (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:258-300), with one
  scale per (group, column), or, without gate-up fusion and with m % 4 == 0, per (group, k-block, column) with blocks
  of a power of two >= 128 rows (the lhs scales then per row or per (row, same k-block));
  or under an lhs quantised to int8 in the same forms (blocks of a power of two >= 64 rows): the int8 MFMAs on the
  nibbles (pallas_mosaic_gpu_kernel_sm100_i8_quant.py:114-190). Gate-up fusion over packed weights needs n % 32 == 0.
  Every other call gets the values unpacked to int8 storage first (then the int8 paths).
  Works on arrays and on shapes, so the forward pass and the choice of a config settle it alike."""
  if not (isinstance(rhs, QArray) and rhs.packed):
    return rhs
  g, k, n = rhs.shape
  scale = tuple(rhs.scale.shape)
  blocks = scale[1] if len(scale) == 3 and scale[0] == g and scale[2] == n and scale[1] >= 1 and k % scale[1] == 0 else None
  rows = k // blocks if blocks else 0
  scale_ok = blocks == 1 or (blocks is not None and rows % 32 == 0 and rows & (rows - 1) == 0)
  reads_packed = (dims == base.DEFAULT_RAGGED_DOT_DIM_NUMS and not isinstance(lhs, (QArray, AsQArray))
                  and lhs.dtype == torch.bfloat16 and rhs.zero_point is None and n % 16 == 0)
  streams = (reads_packed and plain and scale_ok and lhs.shape[0] <= 8 * g and k % 1024 == 0 and (k // 8) * n < 2**31
             and lhs.shape[0] * k * 2 < 2**32)
  tiles = (reads_packed and k % _PACKED_INT4_TILE_STEP == 0
           and (blocks == 1 or (scale_ok and not gateup and rows % _PACKED_INT4_TILE_STEP == 0)))
  if gateup and n % 32:
    return rhs.unpacked()  # (the up half of a weight row must start on a 16-byte piece: 16 columns of one-byte storage)
  lhs_rows = _per_row_lhs_scale(lhs)
  fp8_tiles = (dims == base.DEFAULT_RAGGED_DOT_DIM_NUMS and isinstance(lhs_rows, QArray) and lhs_rows.zero_point is None
               and lhs_rows.qtype == torch.float8_e4m3fn and len(lhs_rows.qvalue.shape) == 2
               and rhs.zero_point is None and n % 16 == 0 and k % _PACKED_INT4_FP8_TILE_STEP == 0 and blocks is not None
               and tuple(lhs_rows.scale.shape) in ((lhs_rows.qvalue.shape[0], 1), (lhs_rows.qvalue.shape[0], blocks))
               and (blocks == 1 or (scale_ok and not gateup and rows % _PACKED_INT4_FP8_TILE_STEP == 0
                                    and lhs_rows.qvalue.shape[0] % 4 == 0)))
  # ... or quantised to int8 likewise: the int8 MFMAs on the nibbles (pallas_mosaic_gpu_kernel_sm100_i8_quant.py:
  # 114-190); scale blocks of a power of two >= 64 rows (not under gate-up fusion).
  int8_tiles = (dims == base.DEFAULT_RAGGED_DOT_DIM_NUMS and isinstance(lhs_rows, QArray) and lhs_rows.zero_point is None
                and _dtype_of(lhs_rows) == torch.int8 and lhs_rows.qvalue.dtype == torch.int8
                and len(lhs_rows.qvalue.shape) == 2 and rhs.zero_point is None and n % 16 == 0
                and k % _PACKED_INT4_FP8_TILE_STEP == 0 and blocks is not None
                and tuple(lhs_rows.scale.shape) in ((lhs_rows.qvalue.shape[0], 1), (lhs_rows.qvalue.shape[0], blocks))
                and (blocks == 1 or (scale_ok and not gateup and rows % _PACKED_INT4_TILE_STEP == 0
                                     and lhs_rows.qvalue.shape[0] % 4 == 0)))
  return rhs if streams or tiles or fp8_tiles or int8_tiles else rhs.unpacked()


def _abstract_operand(x):
  """The abstract form of what `_concrete_operand` returns."""
  if isinstance(x, AsQArray):
    return x.abstract_qarray()
  if isinstance(x, QArray) and x.zero_point is not None:
    return ShapeDtype(tuple(x.shape), torch.bfloat16)
  return x


def _concrete_operand(x):
  """An `AsQArray` quantised on the device; an operand with a zero point dequantised to bf16 (quantization.py:85-93:
  none of the kernels takes a zero point)."""
  return quantization.as_array_or_qarray_without_zero_point(x)


_PLAIN_ARGUMENT_TYPES = (bool, int, float, str, torch.dtype, base.RaggedDotDimensionNumbers)


def _make_plan(records, out, lhs, rhs, group_sizes):
  """The shortcut for calls like the one that left `records` and returned `out`, or None if that call was more than
  one forward launch on the caller's own buffers."""
  if len(records) != 1 or not isinstance(records[0], hip_ops.ForwardLaunch) or records[0].out is not out:
    return None
  record = records[0]
  if out.device.index != torch.cuda.current_device():
    return None  # (the launch ran under a device guard; the shortcut has none)

  def leaves(lhs, rhs, group_sizes):
    return ((lhs,) if type(lhs) is torch.Tensor else (lhs.qvalue, lhs.scale)) + \
           ((rhs,) if type(rhs) is torch.Tensor else (rhs.qvalue, rhs.scale)) + (group_sizes,)

  given = [t.data_ptr() for t in leaves(lhs, rhs, group_sizes)]
  if 0 in given or len(set(given)) != len(given):
    return None
  source = []  # for every pointer of the launch: which of the caller's tensors it was, -1 for an absent operand
  for p in record.pointers:
    if p == 0:
      source.append(-1)
    elif p in given:
      source.append(given.index(p))
    else:
      return None  # (a buffer this call made itself: a widened or repeated operand, converted group sizes)
  source = tuple(source)
  launch, new_workspace = record.launch, record.new_workspace
  shape, dtype, device = tuple(out.shape), out.dtype, out.device

  def plan(lhs, rhs, group_sizes):
    tensors = leaves(lhs, rhs, group_sizes)
    result = torch.empty(shape, dtype=dtype, device=device)
    ws = new_workspace()
    status = launch([0 if i < 0 else tensors[i].data_ptr() for i in source], result.data_ptr(), ws.data_ptr(),
                    torch.cuda.current_stream(device).cuda_stream)
    if status != 0:
      _lib.check(status)
    return result

  return plan


@dataclasses.dataclass(frozen=True)
class HipRaggedDot(base.RaggedDot):
  """Hand-written HIP ragged dot for gfx950. Physical layout `mk,gkn->mn`, rhs never transposed."""

  config_cls: ClassVar[type] = Config
  supports_symbolic_shapes: ClassVar[bool] = False
  # With `preferred_element_type` fp8 (e4m3fn): return the result quantised per (row, 128 columns) as a QArray instead
  # of widening it (pallas_mosaic_gpu.py:93, :316-318).
  enable_fused_epilogue_quant: bool = False

  def __post_init__(self):
    if self.vjp is None:
      # A fresh op per call avoids infinite recursion (pallas_mosaic_gpu.py:95-100).
      fn = lambda *a, **kw: HipRaggedDot()(*a, **kw)  # pylint: disable=unnecessary-lambda
      object.__setattr__(self, "vjp", partial(base.vjp, dlhs_ragged_dot=fn, drhs_ragged_dot=fn))

  # -- eager fast path -------------------------------------------------------------------------
  def __call__(self, lhs, rhs, *, return_residuals: bool = False, **kwargs):
    """The operator call (`Op.__call__`) with a shortcut for repeated eager calls: a call that came down to one
    forward launch on the caller's own tensors (no pass over an operand in front of it, nothing applied to the result
    behind it, no gradient wanted) is remembered under the shapes, types and arguments it was made with, and the next
    call of that kind goes straight to the C ABI: allocate the result, pass the addresses. Binding, the choice of a
    config and the routing cost about 45 us of Python per call, more than the small-m kernels take."""
    key = None if return_residuals else self._plan_key(lhs, rhs, kwargs)
    plans = self.__dict__.get("_plans")
    if key is not None and plans is not None:
      plan = plans.get(key)
      if plan is not None:
        return plan(lhs, rhs, kwargs["group_sizes"])
    if key is None:
      return super().__call__(lhs, rhs, return_residuals=return_residuals, **kwargs)
    log = hip_ops.LAUNCH_LOG
    outer, log.records = log.records, []
    try:
      out = super().__call__(lhs, rhs, **kwargs)
      records = log.records
    finally:
      log.records = outer
    if outer is not None:
      outer.extend(records)
    plan = _make_plan(records, out, lhs, rhs, kwargs["group_sizes"])
    if plan is not None:
      if plans is None or len(plans) > 64:
        plans = {}
        object.__setattr__(self, "_plans", plans)
      plans[key] = plan
    return out

  def _plan_key(self, lhs, rhs, kwargs):
    """What a remembered launch depends on, or None for a call that always takes the full path."""
    if self.checkify_group_sizes or op.OP_CALL_RECORDER.get() is not None:
      return None
    group_sizes = kwargs.get("group_sizes")
    if type(group_sizes) is not torch.Tensor or not group_sizes.is_cuda:
      return None
    grad = torch.is_grad_enabled()
    parts = []
    for x in (lhs, rhs):
      if type(x) is torch.Tensor:
        leaves = (x,)
      elif type(x) is QArray and x.zero_point is None:
        leaves = (x.qvalue, x.scale)
        parts.append(x.qtype)
      else:
        return None
      for t in leaves:
        if type(t) is not torch.Tensor or not t.is_cuda or (grad and t.requires_grad):
          return None
        parts.append((t.shape, t.dtype, t.is_contiguous()))
    parts.append((group_sizes.shape, group_sizes.dtype, group_sizes.is_contiguous(), lhs.device if type(lhs) is torch.Tensor
                  else lhs.qvalue.device))
    for name, v in kwargs.items():
      if name == "group_sizes":
        continue
      if not (v is None or type(v) in _PLAIN_ARGUMENT_TYPES):
        return None  # (tensors, callables: the full path)
      parts.append((name, v))
    parts.append((op.config_epoch(), config_lib.autotuning_cache_miss_fallback.value,
                  config_lib.ignore_autotuning_cache.value, id(op.AUTOTUNING_CACHE_OVERLAY_STACK.get()),
                  torch.cuda.current_device()))
    return tuple(parts)

  # -- forward ---------------------------------------------------------------------------------
  def _fwd(
      self,
      lhs,
      rhs,
      *,
      group_sizes,
      ragged_dot_dimension_numbers,
      precision,
      preferred_element_type,
      return_residuals,
      config: Config,
      activation=None,
      manual_axis_type=None,
      group_offset=None,
      rhs_scale=None,
      rhs_bias=None,
      maybe_quantize_lhs=False,
      zero_initialize=True,
      fuse_gateup_activation=None,
      lhs_quantization_dtype=None,
      rhs_quantization_dtype=None,
  ):
    del manual_axis_type  # sharding annotation only; no meaning on a single device
    # `maybe_quantize_lhs` permits quantising lhs when rhs is quantised (base.py:208); the lhs stays as it is
    # here (16-bit lhs x int8 weights, the more exact of the two choices). `zero_initialize=False` only
    # releases the rows of no group from being zero (base.py:209-210); they are zeroed all the same.
    del maybe_quantize_lhs, zero_initialize
    if lhs_quantization_dtype is not None or rhs_quantization_dtype is not None:
      # (gmm_v2's own arguments: quantise an operand to that type inside the TPU kernel. Callers here say the same
      # with an `AsQArray` operand.)
      raise NotImplementedError("lhs_quantization_dtype / rhs_quantization_dtype are not supported by the hip"
                                " implementation; pass an AsQArray operand instead.")
    gateup = None
    if fuse_gateup_activation is not None:
      gateup = _GATEUP_ACTIVATIONS.get(fuse_gateup_activation)
      if gateup is None:
        raise NotImplementedError(f"fuse_gateup_activation={fuse_gateup_activation!r} is not supported by the hip"
                                  f" implementation (supported: {sorted(_GATEUP_ACTIVATIONS)}).")
      if return_residuals:
        raise NotImplementedError("return_residuals is not supported with fuse_gateup_activation.")
    if group_offset is not None and ragged_dot_dimension_numbers != base.DEFAULT_RAGGED_DOT_DIM_NUMS:
      raise NotImplementedError("group_offset needs the default dimension numbers.")

    # Quantise / dequantise what the kernels cannot take as it is, then plan the call on shapes and types.
    lhs, rhs = _concrete_operand(lhs), _concrete_operand(rhs)
    rhs = _settle_packed_int4(lhs, rhs, dims=ragged_dot_dimension_numbers,
                              plain=rhs_bias is None and fuse_gateup_activation is None and rhs_scale is None,
                              gateup=fuse_gateup_activation is not None)
    route = _route(lhs, rhs, dims=ragged_dot_dimension_numbers, precision=precision,
                   rhs_scale=rhs_scale, fuse_gateup_activation=fuse_gateup_activation,
                   preferred_element_type=preferred_element_type)
    lhs, rhs, preferred_element_type = route.lhs, route.rhs, route.preferred_element_type
    mode = _MODE_OF_DIMS[ragged_dot_dimension_numbers]

    lhs_scale = rhs_scale_ = None
    if isinstance(lhs, QArray):
      if route.widen_lhs:
        lhs_v = hip_ops.dequantize(lhs.qvalue, lhs.scale)
      else:
        lhs_scale, lhs_v = lhs.scale, lhs.qvalue  # one scale per row (or the kernels' own k-blocks)
    else:
      lhs_v = lhs
    if isinstance(rhs, QArray):
      g, k, n = rhs.shape
      if not route.widen_rhs:
        # One scale per (group, column): applied in the epilogue. Native k-blocks: [g, k/t_k, n] goes as it is.
        rhs_scale_, rhs_v = rhs.scale, rhs.qvalue
      else:
        blocks = _scale_blocks_along_k(rhs) if mode == 0 else None
        rows = k // blocks if blocks else 0
        if (blocks and config.block_m == 16 and rhs.qvalue.dtype == torch.int8 and not isinstance(lhs, QArray)
            and rows % 32 == 0 and rows & (rows - 1) == 0 and rhs_bias is None and fuse_gateup_activation is None):
          # The streaming small-m kernel scales int8 weights per k-block while it widens them.
          rhs_scale_, rhs_v = rhs.scale, rhs.qvalue
        else:
          # Scales that change along k (or in blocks along n): widened to bf16 by a streaming pass, then the
          # bf16 kernels.
          rhs_v = hip_ops.dequantize(rhs.qvalue, rhs.scale)
    else:
      rhs_v = rhs
    if route.cast_bf16:
      lhs_v, rhs_v = lhs_v.to(torch.bfloat16), rhs_v.to(torch.bfloat16)

    # fp8 output: widened to the weights' type by default (pallas_mosaic_gpu.py:197-205); with
    # `enable_fused_epilogue_quant` the result is quantised to fp8 per (row, 128 columns) and returned as a QArray
    # (pallas_mosaic_gpu_common.py:63-68, pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:797-824).
    quantize_out = False
    if preferred_element_type == torch.float8_e4m3fn:
      if self.enable_fused_epilogue_quant and mode == 0 and gateup is None and not return_residuals:
        quantize_out = True
        preferred_element_type = torch.float32  # the accumulator's type is what gets quantised
      else:
        preferred_element_type = rhs.dtype if isinstance(rhs, QArray) else rhs_v.dtype
    if preferred_element_type not in (torch.float32, torch.bfloat16, torch.float16):
      raise NotImplementedError(f"Output dtype {preferred_element_type} not supported.")

    device = lhs_v.device
    gs = group_sizes.to_tensor(device) if isinstance(group_sizes, GroupSizes) else group_sizes
    if not isinstance(gs, torch.Tensor):
      gs = torch.as_tensor(gs, dtype=torch.int32, device=device)

    if group_offset is not None:
      # One int32 on the device: the kernels read it there, so nothing synchronises with the host.
      group_offset = torch.as_tensor(group_offset, device=device).to(torch.int32).reshape(-1)
      if group_offset.numel() != 1:
        raise ValueError("group_offset must hold one element")

    kcfg = config.to_kernel_config()
    fused = None
    if activation is not None and not return_residuals:
      fused = _fused_activation_name(activation)

    if (rhs_bias is not None or gateup is not None) and mode != 0:
      raise NotImplementedError("rhs_bias and fuse_gateup_activation need the default dimension numbers.")
    if rhs_bias is not None:
      g, _, n = rhs_v.shape
      if tuple(rhs_bias.shape) != (g, 1, n):
        raise NotImplementedError(f"rhs_bias must have shape [g,1,n], got {tuple(rhs_bias.shape)}")

    if gateup is not None:
      # act(gate) * up in the kernel; an `activation` on top of that is applied to the f32 result.
      kernel_out = torch.float32 if activation is not None else preferred_element_type
      dot_out = hip_ops.ragged_dot_fwd(lhs_v, rhs_v, gs, config=kcfg, out_dtype=kernel_out, lhs_scale=lhs_scale,
                                       rhs_scale=rhs_scale_, rhs_bias=rhs_bias, activation=gateup, gateup=True,
                                       group_offset=group_offset)
      if activation is not None:
        dot_out = activation(dot_out).to(preferred_element_type)
      return dot_out, None

    if (quantize_out and rhs_v.shape[2] % 128 == 0 and rhs_bias is None and group_offset is None
        and (activation is None or fused is not None) and lhs_v.dtype == rhs_v.dtype
        and lhs_v.dtype in (torch.bfloat16, torch.float8_e4m3fn)
        and (rhs_scale_ is None or rhs_scale_.numel() == rhs_v.shape[0] * rhs_v.shape[2])
        and (lhs_scale is None or lhs_scale.numel() == lhs_v.shape[0])):
      # Quantised in the GEMM's epilogue, where the kernel has one (bf16 x bf16, fp8 x fp8; tiled variants).
      try:
        qvalue, scale = hip_ops.ragged_dot_fwd_fp8_out(lhs_v, rhs_v, gs, config=kcfg, lhs_scale=lhs_scale,
                                                       rhs_scale=rhs_scale_, activation=fused)
        return QArray(qvalue, scale, None, torch.float8_e4m3fn), None
      except NotImplementedError:
        pass  # (this variant cannot: the pass over an f32 result below)
    if mode == 2:
      dot_out = hip_ops.ragged_dot_drhs(lhs_v, rhs_v, gs, gs.numel(), config=kcfg, out_dtype=preferred_element_type)
    else:
      # A callable with no in-kernel twin is applied to an f32 result, i.e. still in the accumulator
      # dtype, and cast afterwards.
      unfused = activation is not None and not return_residuals and fused is None
      kernel_out = torch.float32 if unfused else preferred_element_type
      dot_out = hip_ops.ragged_dot_fwd(lhs_v, rhs_v, gs, config=kcfg, out_dtype=kernel_out, trans_rhs=(mode == 1),
                                       lhs_scale=lhs_scale, rhs_scale=rhs_scale_, activation=fused, rhs_bias=rhs_bias,
                                       group_offset=group_offset)
      if unfused:
        dot_out = activation(dot_out).to(preferred_element_type)
    if quantize_out:
      # (a pass of its own over the f32 result, where the epilogue above could not do it)
      n_out = dot_out.shape[1]
      sub = 128 if n_out % 128 == 0 else n_out
      qvalue, scale = hip_ops.quantize(dot_out, torch.float8_e4m3fn, (1, sub))
      return QArray(qvalue, scale, None, torch.float8_e4m3fn), None

    residuals = dot_out
    if activation is not None and return_residuals:
      dot_out = activation(dot_out)
    elif activation is not None and mode == 2:
      dot_out = activation(dot_out)
    return dot_out, residuals if return_residuals else None

  # -- configs ---------------------------------------------------------------------------------
  def _problem(self, ba: op.BoundArguments):
    lhs, rhs = _abstract_operand(ba.args[0]), _abstract_operand(ba.args[1])
    rhs = _settle_packed_int4(lhs, rhs, dims=ba.kwargs["ragged_dot_dimension_numbers"],
                              plain=(ba.kwargs.get("rhs_bias") is None and ba.kwargs.get("fuse_gateup_activation") is None
                                     and ba.kwargs.get("rhs_scale") is None),
                              gateup=ba.kwargs.get("fuse_gateup_activation") is not None)
    route = _route(lhs, rhs, dims=ba.kwargs["ragged_dot_dimension_numbers"],
                   precision=ba.kwargs.get("precision"), rhs_scale=ba.kwargs.get("rhs_scale"),
                   fuse_gateup_activation=ba.kwargs.get("fuse_gateup_activation"),
                   preferred_element_type=ba.kwargs.get("preferred_element_type"))
    lhs_shape, rhs_shape = tuple(lhs.shape), tuple(rhs.shape)
    if route.mode == 2:
      num_groups = int(ba.kwargs["group_sizes"].shape[0])
      rows, cols, contraction = lhs_shape[1], rhs_shape[1], lhs_shape[0]
    elif route.mode == 1:
      num_groups = rhs_shape[0]
      rows, cols, contraction = lhs_shape[0], rhs_shape[1], rhs_shape[2]
    else:
      num_groups = rhs_shape[0]
      rows, cols, contraction = lhs_shape[0], rhs_shape[2], rhs_shape[1]
    return route.mode, route.key, num_groups, rows, cols, contraction, route

  def _get_heuristics_config(self, ba: op.BoundArguments) -> Config:
    mode, key, num_groups, rows, cols, contraction, route = self._problem(ba)
    variants = _variant_table().get(key)
    if not variants:
      raise NotImplementedError(f"No hip kernel for dtypes/mode {key}.")
    if mode == 4:
      # The streaming small-m kernel takes per-k-block scales in its 128-column form (listed with the
      # plain forward variants).
      variants = variants + [v for v in _variant_table().get((0, key[1], key[2]), []) if v[0] == 16 and v[1] == 128]
    # The streaming small-m kernel (listed with block_m == 16; forward only) needs k % 1024 == 0 and
    # n % 8 == 0, and a weight slice (k/4 rows of n) that a 32-bit buffer offset spans.
    wbytes = 1 if key[2] in (_lib.TKX_I8, _lib.TKX_I4X2) else 2
    streaming_ok = (mode in (0, 4) and ba.kwargs.get("rhs_bias") is None and contraction % 1024 == 0 and cols % 8 == 0
                    and (contraction // 4) * cols * wbytes < 2**31)
    usable = [v for v in variants if v[0] != 16 or streaming_ok]
    if key[2] == _lib.TKX_I4X2:
      # Packed int4 weights: the tiled kernels take whole k-steps, the streaming kernel a weight slice of whole
      # 16-byte pieces.
      usable = [v for v in usable if (cols % 16 == 0 if v[0] == 16 else contraction % v[2] == 0)]
      if not usable:
        raise NotImplementedError("No hip kernel reads these packed int4 weights as they are.")
    if mode == 4:
      # The k-step of a tiled variant has to divide the rows of a scale block (and the contraction).
      blocks = route.rhs.scale.shape[1]
      step = contraction // blocks if blocks > 1 else contraction
      usable = [v for v in usable if v[0] == 16 or step % v[2] == 0]
      if not usable:
        raise NotImplementedError(f"No hip kernel variant whose k-step divides {step} rows.")
    # Rows per group decide the m-tile: a tile much taller than a group wastes MFMA work on rows
    # that are masked out at the store; a short tile re-reads the weights more often.
    rows_per_group = rows / max(num_groups, 1) if mode != 2 else rows
    want_m = (256 if rows_per_group >= 1024 else 128 if rows_per_group >= 192 else 64 if rows_per_group >= 48
              else 32 if rows_per_group > 7 else 16)  # 16 = one pass of the streaming kernel; the mean must
    # leave room for the largest group, which re-reads its weights for every further 16 rows (measured: at 5 and 6 rows
    # per group the streaming kernel is ahead or within 10 %, at 8 the 32-row tiles are up to 40 % ahead)
    want_n = 256 if cols >= 2048 else 128
    # bf16 activations over int8 / packed int4 weights with one scale per (group, column): the 128 x 256 tile on one
    # row of waves is small enough for two workgroups to share a CU (64 KB of LDS with two stages of int8 weights, 72 KB
    # with three of int4; 128 registers) and was the fastest or within a few percent of it from 12 rows per group up to
    # 2048 (43 measured shapes per kind).
    # (int8 activations over packed int4 weights have such a tile too, 128 x 256 x 128 with two stages: the fastest on 22
    # of 26 shapes until the tile on four waves below, which is 1-2 % ahead of it on most)
    int8_int4 = key[1] == _lib.TKX_I8 and key[2] == _lib.TKX_I4X2
    f8_int4 = key[1] == _lib.TKX_F8E4M3FN and key[2] == _lib.TKX_I4X2
    # fp8 or int8 activations over packed int4 weights, plain or with gate-up fusion: 128 x 256 x 128 on one row of
    # four waves (128 accumulators per lane, one set of converted fragments) with two stages is 64 KB, so two 4-wave
    # workgroups share a CU behind barriers of their own: the fastest or within 2 % of it on 73 of the 87 measured shapes
    # with 12 rows per group or more (most of the others have too few tiles for it and take the rule below).
    pairs_of_four = (f8_int4 or int8_int4) and mode in (0, 3)
    converted_plain = mode == 0 and ((key[1] == _lib.TKX_BF16 and key[2] in (_lib.TKX_I8, _lib.TKX_I4X2)) or int8_int4
                                     or f8_int4)
    if mode in (0, 3, 4) and key[1] != _lib.TKX_F32 and rows_per_group >= (12 if converted_plain else 96):
      # The forward kernels other than f32 (16-bit operands without scales are re-ranked by the cost model below): the
      # taller and wider tile pays off earlier than the thresholds above say. Measured on 14 shapes per kind (int8 and
      # packed int4 weights, fp8 x fp8, gate-up fusion, scales per k-block): the 256-row tile wins from about 256
      # rows per group, the 128-row one from about 100, and 256 columns from a few tiles' worth of them.
      want_m = 256 if rows_per_group >= 224 else 128
      want_n = 256 if cols >= 512 else 128
      if (key[1] == _lib.TKX_BF16 and key[2] in (_lib.TKX_I8, _lib.TKX_I4X2, _lib.TKX_F8E4M3FN)) or int8_int4 or pairs_of_four:
        # (also with gate-up fusion, where the tile sits on one row of four waves, likewise two per CU: 6 % ahead of the
        # 256-row tile at the Mixtral shape and 16-31 % at 128 rows per group; and with scales per k-block: 8-13 %
        # ahead at 128-256 rows per group, even at the Mixtral shape)
        want_m = 128
      # ... unless so few tiles come of it that half the chip would idle: then the largest tile that gives every CU one.
      tiles = lambda bm, bn: (rows / bm + 0.88 * num_groups) * -(-cols // (bn // 2 if mode == 3 else bn))
      if tiles(want_m, want_n) < _COMPUTE_UNITS // 2:
        # (gate-up fusion and scales per k-block have 256-column tiles only: of the shapes there are)
        shapes = ((256, 256), (128, 256), (128, 128), (64, 128), (32, 128)) if mode == 0 else sorted(
            {(v[0], v[1]) for v in usable if v[0] > 16}, key=lambda t: (-t[0] * t[1], -t[1]))
        want_m, want_n = next((t for t in shapes[:-1] if t[0] <= want_m and tiles(*t) >= _COMPUTE_UNITS), shapes[-1])
    if mode == 0 and key[1] == _lib.TKX_F32:
      # f32 operands run on the f32 MFMAs at a sixteenth of the bf16 rate: loads never bound them, and the 32-row tile
      # (four of its workgroups share a CU) was the fastest of the three on every measured shape, 128 to 1400 rows
      # per group (9-47 % ahead of the taller ones).
      want_m, want_n = 32, 128
    # The streaming kernel on int8 weights has a wide form (256 columns per workgroup, two workgroups
    # per CU) that streams 7-9% faster when its workgroups fill the chip evenly, and slower than the
    # 128-column form when they do not (measured: 384 workgroups on 256 CUs lose 10%).
    wide_wgs = num_groups * -(-cols // 256)
    stream_n = 256 if mode == 0 and cols % 16 == 0 and wide_wgs / (-(-wide_wgs // 512) * 512) >= 0.9 else 128

    def score(v):
      bm, bn, bk, wm, wn, ns = v
      if bm == 16:
        return (abs(bm - want_m), abs(bn - stream_n), 0, 0, 0, ns)
      # drhs streams two row-contiguous operands: shallower k-steps with more stages in flight win there.
      if mode == 2:
        # A group's contraction (its rows) is short next to the tile it produces, so the store of a
        # tile weighs as much as its MFMAs: up to about 1500 rows per group two 4-wave workgroups
        # per CU (one stores while the other computes) beat one 8-wave workgroup with the larger tile.
        if contraction / max(num_groups, 1) < 1536:
          return (abs(bm - 256), abs(bn - 128), abs(wm * wn - 4), 0, bk, ns)
        return (abs(bm - want_m), abs(bn - want_n), -(wm * wn), 0, bk, ns)
      # One workgroup per CU (8 waves): what hides the latency of the weight stream is the depth of
      # contraction in flight, (stages - 1) * block_k; beyond 96 more depth buys nothing (it measured
      # 1.5% slower), and at equal depth the longer k-step has fewer barriers per flop.
      in_flight = min((ns - 1) * bk, 96) if wm * wn == 8 else 0
      # (With per-k-block scales the shorter k-step measured 3 % faster at equal depth: 991 against 961 TFLOP/s.)
      # Integer or fp8 MFMAs on both sides: the longer k-step again.
      short_k = mode == 4 and key[1] == _lib.TKX_BF16
      # Weights that are converted on the way from LDS to the MFMA (int8, packed int4, fp8 under a bf16 lhs): every
      # wave converts the fragments of its own columns, so one row of waves converts each weight once where two rows
      # convert it twice (measured 1.01-1.44 x, typically 1.1-1.2 x, over three shapes, both scale forms, both tile
      # heights; 16-bit operands lose 5 % with it: their LDS reads grow by half and nothing is saved).
      converted = key[1] == _lib.TKX_BF16 and key[2] in (_lib.TKX_I8, _lib.TKX_I4X2, _lib.TKX_F8E4M3FN)
      # (fp8 activations over packed int4 weights turn nibbles into fp8 bytes the same way: the 128-row tile runs at
      # 2070-2270 TFLOP/s on one row of waves against 1660-2050 on two at the Mixtral shape; their 256-row tile exists
      # on two rows only)
      two_wave_rows = wm - 1 if converted or int8_int4 or (key[1] == _lib.TKX_F8E4M3FN and key[2] == _lib.TKX_I4X2) else 0
      if mode == 4 and key[1] == _lib.TKX_F8E4M3FN and contraction < 1280:
        # (with scales per k-block and a contraction of a few k-steps the tile on two rows of waves was ahead on the
        # three such shapes measured: by 1-2 % at k = 896 and 1152, by 63 % at k = 768 with 12288 columns)
        two_wave_rows = 0
      # ... and among those, the variant whose LDS lets two of its workgroups share a CU (the library gives such a
      # kernel 128 registers: 8 waves on one row, at most 64 accumulators per lane)
      stage_bytes = ((bm * (1 if int8_int4 else 2) + bn * (0.5 if key[2] == _lib.TKX_I4X2 else 1.0)) * bk
                     + (bn * 4 if mode == 4 else 0))
      alone_on_cu = 0 if ((converted or (int8_int4 and mode == 0)) and wm == 1 and wn == 8 and bm * bn <= 128 * 256
                          and 2 * ns * stage_bytes <= 160 * 1024) else 1
      four_wave_pair = 0 if pairs_of_four and (wm, wn) == (1, 4) and 2 * ns * (bm + bn * 0.5) * bk <= 160 * 1024 else 1
      return (abs(bm - want_m), abs(bn - want_n), two_wave_rows, four_wave_pair, -(wm * wn),
              alone_on_cu if converted or int8_int4 else 0, -in_flight,
              bk if short_k else -bk, ns)

    bm, bn, bk, wm, wn, ns = min(usable, key=score)
    modelled_split = None
    if bm != 16 and mode in (0, 1) and key[1] == key[2] and key[1] in (_lib.TKX_BF16, _lib.TKX_F16):
      # 16-bit operands without scales: the tile that the cost model expects to finish first, with or without the
      # split of the last round (the rules above stay in charge of the choice for the streaming small-m kernel).
      best = None
      for v in usable:
        if v[0] == 16:
          continue
        for sk in (1, 4) if _tiled_split_pays(mode, v[0], v[1], rows, cols, num_groups) else (1,):
          # (ties: the longer k-step has fewer barriers per flop, then the deeper pipeline)
          cost = (round(_tile_cost(v, sk, rows, cols, contraction, num_groups, mode), 3), -v[2], -v[5], sk)
          if best is None or cost < best[0]:
            best = (cost, v, sk)
      if best is not None:
        (bm, bn, bk, wm, wn, ns), modelled_split = best[1], best[2]
    # grid_tile_width m-tasks of one group run side by side on an n-panel of its weights (a span never
    # crosses a group, so small groups simply get short spans). With the 32 tiles an XCD runs at a
    # time, 8 wide x 4 n-panels needs the fewest distinct operand panels in its L2; 16 wide measured
    # the same speed on the Mixtral shape with 50% more traffic past L2.
    width = 8
    split_k = 1
    if bm == 16:
      width = 1  # the streaming small-m kernel has no tile order to tune
      split_k = _streaming_split(num_groups * -(-cols // bn), contraction, bn, ns)
    elif modelled_split is not None:
      split_k = modelled_split
    elif _tiled_split_pays(mode, bm, bn, rows, cols, num_groups):
      # ... only where the estimate of the launch says that the shorter last round is worth the exchange, which a
      # short contraction is not. (One-byte activations: a k-step moves the bytes and takes the MFMA time of a
      # 16-bit k-step half as long.)
      narrow = 2 if key[1] in (_lib.TKX_F8E4M3FN, _lib.TKX_I8) else 1
      v, rb = (bm, bn, bk // narrow, wm, wn, ns), {_lib.TKX_I8: 1.0, _lib.TKX_I4X2: 0.5}.get(key[2], 2.0)
      shares = None
      if key[1] == _lib.TKX_BF16 and key[2] in (_lib.TKX_I8, _lib.TKX_I4X2, _lib.TKX_F8E4M3FN) and wm == 1 and wn == 8:
        stage = (bm * 2 + bn * rb) * bk + (bn * 4 if mode == 4 else 0)
        shares = bm * bn <= 128 * 256 and 2 * ns * stage <= 160 * 1024
      if int8_int4 and mode == 0 and wm == 1 and wn == 8:
        shares = bm * bn <= 128 * 256 and 2 * ns * (bm + bn * 0.5) * bk <= 160 * 1024
      if pairs_of_four and (wm, wn) == (1, 4):
        shares = 2 * ns * (bm + bn * 0.5) * bk <= 160 * 1024
      estimate = lambda sk: _tile_cost(v, sk, rows, cols, contraction // narrow, num_groups, mode,
                                       rhs_bytes=2.0 if narrow == 2 else rb, shares_cu=shares)
      if key[1] == _lib.TKX_F32 or estimate(4) < estimate(1):
        split_k = 4
    return Config(block_m=bm, block_n=bn, block_k=bk, waves_m=wm, waves_n=wn, num_stages=ns, grid_tile_width=width,
                  align_tile=8, split_k=split_k)

  def _get_autotuning_configs(self, ba: op.BoundArguments) -> set[Config]:
    mode, key = self._problem(ba)[:2]
    configs = set()
    problem = self._problem(ba)
    variants = list(_variant_table().get(key, []))
    if mode == 4:
      # (the streaming small-m kernel takes scales per k-block in its 128-column form, listed with the plain variants)
      variants += [v for v in _variant_table().get((0, key[1], key[2]), []) if v[0] == 16 and v[1] == 128]
    block_rows = 0
    if mode == 4 and problem[6].rhs.scale.shape[1] > 1:
      block_rows = problem[5] // problem[6].rhs.scale.shape[1]
    for bm, bn, bk, wm, wn, ns in variants:
      if key[2] == _lib.TKX_I4X2 and bm != 16 and problem[5] % bk:
        continue  # (packed int4 weights in a tiled kernel: whole k-steps)
      if bm != 16 and block_rows % bk:
        continue  # (the k-step of a tiled kernel divides the rows of a scale block)
      widths = (1,) if (mode == 2 or bm == 16) else (1, 2, 4, 8, 16)
      for w in widths:
        configs.add(Config(block_m=bm, block_n=bn, block_k=bk, waves_m=wm, waves_n=wn, num_stages=ns,
                           grid_tile_width=w))
        if _tiled_split_pays(mode, bm, bn, problem[3], problem[4], problem[2]):
          configs.add(Config(block_m=bm, block_n=bn, block_k=bk, waves_m=wm, waves_n=wn, num_stages=ns,
                             grid_tile_width=w, split_k=4))
      if bm == 16 and bn == 128 and ns <= 4:
        _, _, num_groups, _, cols, contraction, _ = self._problem(ba)
        for split_k in (2, 4, 8):
          if contraction % (128 * split_k * ns) == 0:
            configs.add(Config(block_m=bm, block_n=bn, block_k=bk, waves_m=wm, waves_n=wn, num_stages=ns,
                               grid_tile_width=1, split_k=split_k))
        # The persistent form (empty groups' workgroups help): one-byte weights with one scale per (group, column).
        if (mode == 0 and key[2] in (_lib.TKX_I8, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2) and num_groups <= 256
            and num_groups * -(-cols // 128) <= 1024):
          configs.add(Config(block_m=bm, block_n=bn, block_k=bk, waves_m=wm, waves_n=wn, num_stages=ns,
                             grid_tile_width=1, persistent=1))
    return configs

  def supported_on(self, device: torch.device) -> bool:
    if config_lib.cross_compile.value:
      return True
    if device.type != "cuda" or not torch.cuda.is_available() or torch.version.hip is None:
      return False
    return _is_gfx950(device)
