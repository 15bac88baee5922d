"""CPU oracle for tokamax.ragged_dot -- TEST INFRASTRUCTURE ONLY.

This file restates, in NumPy, the algorithm of the reference's
`implementation="xla"` ragged dot and of its GPU tile scheduler.  Nothing in the
shipped package imports it: only `tests/`, `__graft_entry__.smoke()` and the
`cpu_baseline` leg of `bench.py` do, and only as the checker / the timed CPU
baseline.

The arithmetic of the reference's XLA path lives in un-vendored third-party
packages (`jax>=0.11.0`: `jax.lax.ragged_dot_general`; `qwix>=0.1.2`:
`dequantize`), which are not installed here, and the reference's own tests hold
no stored floating-point outputs (they compare against JAX live).  Each function
below therefore cites the reference call site it follows, and says what pins it:

  function                     follows (reference file:line)                      pinned by
  ---------------------------  -------------------------------------------------  ------------------------------------
  group_offsets                pallas_mosaic_gpu_common.py:119-121                closed form (np.cumsum), brute force
  group_info_create_aligned    pallas_mosaic_gpu_common.py:87-151                 the 4 known-answer tests of
                                                                                  pallas_mosaic_gpu_common_test.py:27-84
  ragged_dot (3 dim-number     base.py:291-360 (+ :40-54 dim numbers); jax doc    brute-force loops on tiny inputs; G=1
    sets)                      of lax.ragged_dot_general                          -> plain GEMM; equal groups -> batched
                                                                                  GEMM (bench.py:43-49); all rows in
                                                                                  group 0 (bench.py:35-39); autograd of
                                                                                  the forward for dlhs/drhs
  dequantize                   quantization.py:80-83;                             the in-repo restatement
                               ..._sm100_fp8_quant_test.py:229-232                q.astype(f32)*repeat(scale, tile)
  round_to_bf16 / e4m3fn       base.py:342-354 (.astype(out_dtype))               torch's bf16 / float8_e4m3fn casts
                                                                                  (library routine), exhaustive for fp8
  generate_group_sizes         base.py:171-196                                    what the definition fixes: the three
                                                                                  cases of base_test.py:45-51 (incl.
                                                                                  G > m), a one-hot p, counts within 4
                                                                                  sigma of p*m at m = 1e6, m = 1 / G = 1,
                                                                                  seed selects the draw; the exact values
                                                                                  per seed are NumPy's (no stored vector
                                                                                  in the reference to compare with)

  ragged_dot_fused / gateup    base.py:205-217 (docstring of `rhs_bias` and       composition of `ragged_dot` with the
                               `fuse_gateup_activation`); the gate-up forms of    formulas of that docstring; the gate-up
                               experimental/gmm_v2/gmm_v2.py:29-50,96-107 (bias    forms against torch's silu / sigmoid /
                               joins the accumulator before them, :662-663)       gelu(approximate="tanh") / clamp
                                                                                  (library routines) and hand-computed
                                                                                  values at and past the clipping limits

  gated_linear_unit            gated_linear_unit/base.py:60-120                   torch matmul + torch activations on
                                                                                  f64 (library routines)

  ragged_gather / _scatter /   ragged_gather/base.py:25-32, ragged_scatter/        NumPy fancy indexing (library
    _gather_reduce             base.py:26-38, ragged_gather_reduce/base.py:26-40    routine) + loops on a tiny case

  quantize_absmax              quantization.py:65-78 (the call of qwix.quantize)  the reference's own statement of the
                               pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:802-   calibration (absmax / qmax, clip) for
                               822 (the same calibration, in the tree)            fp8; max |q| == qmax per tile; error
                                                                                  <= scale / 2; exact powers of two;
                                                                                  torch's float8_e4m3fn cast; zero tile
  dequantize_zero_point        quantization.py:85-93                              hand-computed values
  pack_int4 / unpack_int4      no counterpart (the reference holds int4 as        hand-computed bytes for all 16 values
                               jnp.int4 arrays; the layout is this library's)     on either side; round trip

Status of "parity unpinned": `qwix.quantize` itself (qwix>=0.1.2, pyproject.toml:27) is not in the tree.
`quantize_absmax` follows the form of its absmax calibration that the reference writes out for fp8; for the integer
types the bound qwix divides by (127 against 127.5 for int8) is NOT fixed by anything in the tree: parity unpinned.
The integer quantisers that ARE in the tree divide by iinfo.max, i.e. 127 (pallas_mosaic_tpu_kernel.py:267-277,
experimental/gmm_v2/util.py:28-50, gmm_v2.py:563): the default here; `bound` selects the other convention.
Quantising and dequantising with one and the same rule, as every test of the reference does
(test_base.py:36-62, :187-242), keeps that choice out of the results compared.
"gelu" in the gate-up forms is `jax.nn.gelu(gate)` (gmm_v2.py:99-100); JAX is not
in the tree, and its documented default (`approximate=True`, the tanh form) is
taken. Everything else above has a pin listed.
"""

from __future__ import annotations

import numpy as np

# Dimension-number sets of the reference (base.py:40-54), named by what they compute.
DEFAULT = "default"  # lhs[m,k] . rhs[g,k,n] -> [m,n]        (base.py:40-44)
TRANS_RHS = "trans_rhs"  # lhs[m,n'] . rhs[g,k',n'] -> [m,k']   (base.py:45-49)  (dlhs)
RAGGED_CONTRACTING = "ragged_contracting"  # lhs[m,k] , rhs[m,n] -> [g,k,n]  (base.py:50-54)  (drhs)


# ----------------------------------------------------------------------------
# Integer part: offsets and tile schedule (bit-exact contract)
# ----------------------------------------------------------------------------
def group_offsets(group_sizes) -> np.ndarray:
  """Exclusive prefix sum of clamped group sizes, length G+1.

  Follows pallas_mosaic_gpu_common.py:119-121: sizes are clamped at 0, cast to
  int32, `cumulative_sum(include_initial=True)`.
  """
  gs = np.maximum(np.asarray(group_sizes).astype(np.int64), 0).astype(np.int32)
  out = np.zeros(gs.shape[0] + 1, np.int32)
  np.cumsum(gs, out=out[1:])
  return out


def _cdiv(a, b):
  return -(-a // b)


def group_info_create_aligned(group_sizes, tile: int, tid_size: int, align_tile: int = 8):
  """Tile schedule; literal restatement of `GroupInfo.create_aligned`.

  Follows pallas_mosaic_gpu_common.py:119-151 line by line.  Returns a dict of six
  int32 arrays of length `tid_size`: group_id, block_start, actual_start,
  actual_end, start_within_block, actual_size -- plus `num_tasks` (the number of
  tasks that belong to some non-empty group = group_start_tasks[-1]).
  """
  gs = np.asarray(group_sizes)
  gs = np.maximum(np.zeros_like(gs), gs).astype(np.int32)  # :119-120
  G = gs.shape[0]
  group_starts = np.zeros(G + 1, np.int32)  # :121
  np.cumsum(gs, out=group_starts[1:])
  group_starts_aligned = (group_starts[:-1] // align_tile) * align_tile  # :122
  group_ends = group_starts[:-1] + gs  # :124
  group_num_blocks = np.where(gs == 0, 0, _cdiv(group_ends - group_starts_aligned, tile))  # :125-127
  group_start_tasks = np.zeros(G + 1, np.int32)  # :128-130
  np.cumsum(group_num_blocks, out=group_start_tasks[1:])
  group_end_tasks = group_start_tasks[:-1] + group_num_blocks  # :132
  task_idx = np.arange(tid_size, dtype=np.int32)  # :133
  task_group_idx = np.searchsorted(group_end_tasks[:-1], task_idx, side="right").astype(np.int32)  # :136-138
  task_block_idx = task_idx - group_start_tasks[task_group_idx]  # :139
  task_starts = group_starts_aligned[task_group_idx] + tile * task_block_idx  # :140
  task_valid_starts = np.maximum(task_starts, group_starts[task_group_idx])  # :141
  task_valid_ends = np.minimum(task_starts + tile, group_ends[task_group_idx])  # :142
  task_valid_size = np.maximum(0, task_valid_ends - task_valid_starts)  # :143
  i32 = lambda x: np.asarray(x, np.int32)
  return dict(
      group_id=i32(task_group_idx),
      block_start=i32(task_starts),
      actual_start=i32(task_valid_starts),
      actual_end=i32(task_valid_ends),
      start_within_block=i32(task_valid_starts - task_starts),
      actual_size=i32(task_valid_size),
      num_tasks=int(group_start_tasks[-1]),
  )


def generate_group_sizes(*, m: int, num_groups: int, p=None, seed: int = 0):
  """Restatement of base.py:171-196 (`generate_group_sizes`)."""
  rng = np.random.default_rng(seed)
  group_ids = rng.choice(num_groups, (m,), p=p, replace=True)
  return tuple(map(int, np.bincount(group_ids, minlength=num_groups)))


# ----------------------------------------------------------------------------
# Dtype helpers
# ----------------------------------------------------------------------------
def round_to_bf16(x) -> np.ndarray:
  """float32 -> nearest-even bfloat16, returned as float32 holding the bf16 value."""
  x = np.ascontiguousarray(x, np.float32)
  u = x.view(np.uint32).astype(np.uint64)
  rounded = ((u + 0x7FFF + ((u >> 16) & 1)) >> 16) << 16
  out = rounded.astype(np.uint32).view(np.float32)
  return np.where(np.isnan(x), x, out)


def bf16_bits(x) -> np.ndarray:
  """float32 -> uint16 bf16 bit patterns (round to nearest even)."""
  return (round_to_bf16(x).view(np.uint32) >> 16).astype(np.uint16)


def bf16_from_bits(bits) -> np.ndarray:
  return (np.asarray(bits, np.uint16).astype(np.uint32) << 16).view(np.float32)


def _e4m3fn_table() -> np.ndarray:
  """All 256 OCP float8_e4m3fn values (bias 7, no inf, 0x7f/0xff = NaN)."""
  t = np.zeros(256, np.float32)
  for b in range(256):
    s = -1.0 if b & 0x80 else 1.0
    e = (b >> 3) & 0xF
    m = b & 0x7
    if e == 0xF and m == 0x7:
      v = np.nan
    elif e == 0:
      v = s * (m / 8.0) * 2.0 ** (-6)
    else:
      v = s * (1.0 + m / 8.0) * 2.0 ** (e - 7)
    t[b] = v
  return t


E4M3FN_TABLE = _e4m3fn_table()


def e4m3fn_decode(bits) -> np.ndarray:
  return E4M3FN_TABLE[np.asarray(bits, np.uint8)]


def e4m3fn_encode(x) -> np.ndarray:
  """float32 -> uint8 e4m3fn bits, round to nearest even, saturating to +-448."""
  x = np.asarray(x, np.float32)
  pos = E4M3FN_TABLE[:0x7F].astype(np.float64)  # 0 .. 448, ascending
  a = np.minimum(np.abs(x).astype(np.float64), 448.0)
  hi = np.searchsorted(pos, a, side="left").clip(0, 0x7E)
  lo = (hi - 1).clip(0, 0x7E)
  dlo, dhi = np.abs(a - pos[lo]), np.abs(pos[hi] - a)
  pick_hi = (dhi < dlo) | ((dhi == dlo) & (hi % 2 == 0))
  code = np.where(pick_hi, hi, lo).astype(np.uint8)
  code = np.where(np.signbit(x), code | 0x80, code).astype(np.uint8)
  return np.where(np.isnan(x), np.uint8(0x7F), code)


def dequantize(qvalue, scale) -> np.ndarray:
  """`qvalue.astype(f32) * broadcast(scale)` with tile-repeat broadcasting.

  Follows quantization.py:80-83 (`qwix.dequantize`, zero_point=None) as restated in
  the reference's own test, pallas_mosaic_gpu_kernel_sm100_fp8_quant_test.py:229-232:
  `scale.shape[i]` divides `qvalue.shape[i]`; each scale entry covers a tile of
  `qvalue.shape[i] // scale.shape[i]` along axis i.
  """
  q = np.asarray(qvalue, np.float32)
  s = np.asarray(scale, np.float32)
  assert q.ndim == s.ndim, (q.shape, s.shape)
  for ax in range(q.ndim):
    assert q.shape[ax] % s.shape[ax] == 0, (q.shape, s.shape)
    s = np.repeat(s, q.shape[ax] // s.shape[ax], axis=ax)
  return q * s


def dequantize_zero_point(qvalue, scale, zero_point) -> np.ndarray:
  """`(qvalue - zero_point) * scale`, scale and zero point repeated over their tiles: the asymmetric form of
  `qwix.dequantize` that quantization.py:85-93 applies before any kernel sees the operand."""
  q = np.asarray(qvalue, np.float32)
  s, z = np.asarray(scale, np.float32), np.asarray(zero_point, np.float32)
  assert q.ndim == s.ndim and s.shape == z.shape, (q.shape, s.shape, z.shape)
  for ax in range(q.ndim):
    rep = q.shape[ax] // s.shape[ax]
    s, z = np.repeat(s, rep, axis=ax), np.repeat(z, rep, axis=ax)
  return (q - z) * s


def pack_int4(values) -> np.ndarray:
  """uint8 [.., r/2, c] from int values in [-8, 7] [.., r, c]: entry 2 i of the second-to-last axis in bits 0-3 of byte
  i, entry 2 i + 1 in bits 4-7 (two's complement). The packed layout of the HIP library (TKX_I4X2); the reference has no
  packed layout of its own."""
  v = np.asarray(values).astype(np.int64)
  lo, hi = v[..., 0::2, :] & 0xF, v[..., 1::2, :] & 0xF
  return (lo | (hi << 4)).astype(np.uint8)


def unpack_int4(packed) -> np.ndarray:
  """The inverse of `pack_int4`: int8 [.., 2 r, c]."""
  p = np.asarray(packed).astype(np.int64)
  nib = np.stack([p & 0xF, (p >> 4) & 0xF], axis=-2)  # [.., r, 2, c]
  nib = np.where(nib >= 8, nib - 16, nib)
  return nib.reshape(*p.shape[:-2], 2 * p.shape[-2], p.shape[-1]).astype(np.int8)


QMAX = {"int8": 127.0, "int4": 7.0, "fp8": 448.0}


def quantize_absmax(x, qtype: str, tile_shape, bound=None, reciprocal=False):
  """Symmetric absmax quantisation with one f32 scale per tile: what `AsQArray.as_qarray` asks of
  `qwix.quantize(x, qtype, tiled_axes=dict(enumerate(tile_shape)))` (quantization.py:65-78), stated the way the
  reference states the same calibration itself (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:802-822):
    scale = absmax(tile) / qmax, 1 where the tile is all zero;  q = x / scale, rounded to nearest even, clipped to +-qmax
  with qmax the largest finite value of the type (127, 7, 448). `bound` (default qmax) replaces qmax in the scale;
  with a bound above qmax (integers: qmax + 0.5) values are clipped to [-qmax - 1, qmax]. The reference's own integer
  quantisers divide by iinfo.max = qmax (pallas_mosaic_tpu_kernel.py:267-277, experimental/gmm_v2/util.py:28-50); what
  qwix divides by is PARITY UNPINNED (qwix is not in the reference tree). `reciprocal`: x * (1 / scale) instead of
  x / scale, the form of the reference's quantisation fused into a kernel's epilogue. Returns (q, scale): q int8 for the integer
  types, the uint8 e4m3fn codes for "fp8"; scale float32 of shape x.shape / tile_shape. All arithmetic in float32."""
  x = np.asarray(x, np.float32)
  qmax = np.float32(QMAX[qtype])
  bound = qmax if bound is None else np.float32(bound)
  lo = -qmax - np.float32(1) if bound > qmax else -qmax
  tile_shape = tuple(int(t) for t in tile_shape)
  assert x.ndim == len(tile_shape) and all(d % t == 0 for d, t in zip(x.shape, tile_shape)), (x.shape, tile_shape)
  split = []
  for d, t in zip(x.shape, tile_shape):
    split += [d // t, t]
  tiles = x.reshape(split)
  inner = tuple(range(1, 2 * x.ndim, 2))
  absmax = np.abs(tiles).max(axis=inner)
  scale = np.where(absmax == 0, np.float32(1), absmax / bound).astype(np.float32)
  full = scale
  for ax, t in enumerate(tile_shape):
    full = np.repeat(full, t, axis=ax)
  if reciprocal:
    # the reference's fused output quantisation multiplies by the reciprocal of the (rounded) scale
    # (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:813-822)
    q = np.clip((x * (np.float32(1) / full)).astype(np.float32), lo, qmax)
  else:
    q = np.clip((x / full).astype(np.float32), lo, qmax)
  if qtype == "fp8":
    return e4m3fn_encode(q), scale
  return np.rint(q).astype(np.int8), scale


# ----------------------------------------------------------------------------
# Floating-point part
# ----------------------------------------------------------------------------
def _round_out(x, out_dtype: str):
  if out_dtype in ("f32", "float32"):
    return x.astype(np.float32)
  if out_dtype in ("f64", "float64"):
    return x.astype(np.float64)
  if out_dtype in ("bf16", "bfloat16"):
    return round_to_bf16(x.astype(np.float32))
  if out_dtype in ("f16", "float16"):
    return x.astype(np.float16).astype(np.float32)
  raise ValueError(out_dtype)


def ragged_dot(lhs, rhs, group_sizes, mode: str = DEFAULT, *, acc_dtype=np.float32, out_dtype: str = "f32"):
  """Per-group GEMM restating `RaggedDot._fwd` (base.py:291-360).

  `lhs`/`rhs` are float arrays already holding the (de-quantised) input values.
  Accumulates in `acc_dtype` (f32 = the reference's accumulator, base.py:345-346;
  f64 = a tighter yardstick) and rounds once to `out_dtype` (base.py:354).  Rows
  `>= sum(group_sizes)` are zero for DEFAULT/TRANS_RHS, as in the XLA path; groups
  with no rows give a zero [k,n] block for RAGGED_CONTRACTING.
  """
  off = group_offsets(group_sizes)
  G = len(off) - 1
  lhs = np.asarray(lhs, acc_dtype)
  rhs = np.asarray(rhs, acc_dtype)
  if mode == DEFAULT:
    m, k = lhs.shape
    g2, k2, n = rhs.shape
    assert g2 == G and k2 == k
    out = np.zeros((m, n), acc_dtype)
    for g in range(G):
      s, e = int(off[g]), min(int(off[g + 1]), m)
      if e > s:
        out[s:e] = lhs[s:e] @ rhs[g]
  elif mode == TRANS_RHS:
    m, n = lhs.shape
    g2, k, n2 = rhs.shape
    assert g2 == G and n2 == n
    out = np.zeros((m, k), acc_dtype)
    for g in range(G):
      s, e = int(off[g]), min(int(off[g + 1]), m)
      if e > s:
        out[s:e] = lhs[s:e] @ rhs[g].T
  elif mode == RAGGED_CONTRACTING:
    m, k = lhs.shape
    m2, n = rhs.shape
    assert m2 == m
    out = np.zeros((G, k, n), acc_dtype)
    for g in range(G):
      s, e = int(off[g]), min(int(off[g + 1]), m)
      if e > s:
        out[g] = lhs[s:e].T @ rhs[s:e]
  else:
    raise ValueError(mode)
  return _round_out(out, out_dtype)


def silu(x):
  return x / (1.0 + np.exp(-x))


def gelu_tanh(x):
  return 0.5 * x * (1.0 + np.tanh(0.7978845608028654 * (x + 0.044715 * x ** 3)))


def gateup(gate, up, name: str):
  """The fused gate-up forms of experimental/gmm_v2/gmm_v2.py:96-107 on f64 arrays.

  "silu": silu(gate) * up; "gelu" (`jax.nn.gelu`, whose default is the tanh form) and "gelu_tanh":
  gelu_tanh(gate) * up; "swigluoai" (gmm_v2.py:29-38): gate clipped from above at 7, up clipped to
  [-7, 7], (up + 1) * gate * sigmoid(1.702 gate); "silu_and_mul_with_clamp" (gmm_v2.py:41-50): the
  same clipping at 10, silu(gate) * up.
  """
  gate, up = np.asarray(gate, np.float64), np.asarray(up, np.float64)
  if name == "silu":
    return silu(gate) * up
  if name in ("gelu", "gelu_tanh"):
    return gelu_tanh(gate) * up
  if name == "swigluoai":
    gate, up = np.minimum(gate, 7.0), np.clip(up, -7.0, 7.0)
    return (up + 1.0) * (gate / (1.0 + np.exp(-1.702 * gate)))
  if name == "silu_and_mul_with_clamp":
    gate, up = np.minimum(gate, 10.0), np.clip(up, -10.0, 10.0)
    return silu(gate) * up
  raise NotImplementedError(name)


def ragged_dot_fused(lhs, rhs, group_sizes, *, rhs_bias=None, gateup_activation=None, group_offset=None,
                     acc_dtype=np.float64, out_dtype: str = "f64"):
  """`ragged_dot(lhs, rhs) + rhs_bias`, then `act(tmp[:, :n]) * tmp[:, n:]` (base.py:205-217).

  `rhs_bias` is [G, 1, 2n] (or [G, 2n]): row i gets the bias of its group; rows past the last group
  stay zero. `gateup_activation` is a name `gateup` knows; None leaves `tmp` as it is.
  `group_offset` (experimental/gmm_v2/gmm_v2_test.py:44-101): `group_sizes` lists every group of the
  job, `rhs` and `rhs_bias` hold the groups [offset, offset + G) of them, and the rows of all other
  groups are zero (before the gate-up form, which maps zeros to zero).
  """
  lhs_, rhs_ = np.asarray(lhs), np.asarray(rhs)
  G = rhs_.shape[0]
  goff = 0 if group_offset is None else int(np.asarray(group_offset).reshape(-1)[0])
  off = group_offsets(group_sizes)
  if group_offset is None:
    tmp = np.asarray(ragged_dot(lhs_, rhs_, group_sizes, DEFAULT, acc_dtype=acc_dtype, out_dtype="f64"), np.float64)
  else:
    tmp = np.zeros((lhs_.shape[0], rhs_.shape[2]), np.float64)
    for j in range(len(off) - 1):
      s, e = int(off[j]), min(int(off[j + 1]), tmp.shape[0])
      if 0 <= j - goff < G and e > s:
        tmp[s:e] = ragged_dot(lhs_[s:e], rhs_[j - goff:j - goff + 1], [e - s], DEFAULT, acc_dtype=acc_dtype,
                              out_dtype="f64")
  if rhs_bias is not None:
    bias = np.asarray(rhs_bias, np.float64).reshape(G, -1)
    for j in range(len(off) - 1):
      s, e = int(off[j]), min(int(off[j + 1]), tmp.shape[0])
      if 0 <= j - goff < G and e > s:
        tmp[s:e] += bias[j - goff]
  if gateup_activation is not None:
    n = tmp.shape[1] // 2
    tmp = gateup(tmp[:, :n], tmp[:, n:], gateup_activation)
  return _round_out(tmp, out_dtype)


def gated_linear_unit(x, weights, activation=None):
  """`activation(x @ weights[:, 0]) * (x @ weights[:, 1])` in float64 (gated_linear_unit/base.py:60-120);
  `weights` is [K, 2, N], `activation` a NumPy callable or None."""
  x = np.asarray(x, np.float64)
  w = np.asarray(weights, np.float64)
  gate, up = x @ w[:, 0, :], x @ w[:, 1, :]
  return (gate if activation is None else activation(gate)) * up


def _jax_take_rows(x, indices):
  """Row lookup `x[indices]` with JAX's indexing rules, which differ from NumPy's for indices outside the array:
  a negative index counts from the end (i -> i + len(x)), and what is then still outside [0, len(x)) is clamped
  to the nearest row instead of raising (JAX documents gathers through indexing as clamped)."""
  x = np.asarray(x)
  idx = np.asarray(indices).astype(np.int64)
  idx = np.where(idx < 0, idx + len(x), idx)
  return x[np.clip(idx, 0, len(x) - 1)]


def ragged_gather(x, indices):
  """`x[indices]` (ragged_gather/base.py:25-32)."""
  return _jax_take_rows(x, indices)


def ragged_scatter(x, indices, start: int, end: int):
  """`where(start <= indices < end, x[indices], 0)` (ragged_scatter/base.py:26-38)."""
  idx = np.asarray(indices)
  out = _jax_take_rows(x, idx)
  return np.where(((idx >= start) & (idx < end))[:, None], out, 0).astype(out.dtype)


def ragged_gather_reduce(x, indices, topk_weights, valid_rows_mask, reduce_group_size: int):
  """f32 `sum over groups of R rows of valid * weight * x[index]` (ragged_gather_reduce/base.py:26-40),
  returned as float32 (the caller rounds to the input type)."""
  out = _jax_take_rows(np.asarray(x, np.float32), indices) * np.asarray(topk_weights, np.float32)[:, None]
  out = np.where(np.asarray(valid_rows_mask, bool)[:, None], out, np.float32(0))
  return out.reshape(-1, reduce_group_size, out.shape[-1]).sum(axis=1, dtype=np.float32)


def ragged_dot_bruteforce(lhs, rhs, group_sizes, mode: str = DEFAULT):
  """Element-by-element float64 loops (tiny inputs only): the pin for `ragged_dot`."""
  lhs = np.asarray(lhs, np.float64)
  rhs = np.asarray(rhs, np.float64)
  gs = [max(int(x), 0) for x in group_sizes]
  G = len(gs)
  row_group = []
  for g, s in enumerate(gs):
    row_group += [g] * s
  if mode == DEFAULT:
    m, k = lhs.shape
    n = rhs.shape[2]
    out = np.zeros((m, n))
    for i in range(min(m, len(row_group))):
      for j in range(n):
        acc = 0.0
        for kk in range(k):
          acc += lhs[i, kk] * rhs[row_group[i], kk, j]
        out[i, j] = acc
  elif mode == TRANS_RHS:
    m, n = lhs.shape
    k = rhs.shape[1]
    out = np.zeros((m, k))
    for i in range(min(m, len(row_group))):
      for kk in range(k):
        acc = 0.0
        for j in range(n):
          acc += lhs[i, j] * rhs[row_group[i], kk, j]
        out[i, kk] = acc
  elif mode == RAGGED_CONTRACTING:
    m, k = lhs.shape
    n = rhs.shape[1]
    out = np.zeros((G, k, n))
    for i in range(min(m, len(row_group))):
      g = row_group[i]
      for kk in range(k):
        for j in range(n):
          out[g, kk, j] += lhs[i, kk] * rhs[i, j]
  else:
    raise ValueError(mode)
  return out


def rel_l2(actual, expected) -> float:
  """Relative L2 error ||a-e|| / ||e|| in float64 (the tolerance metric of the spec)."""
  a = np.asarray(actual, np.float64).ravel()
  e = np.asarray(expected, np.float64).ravel()
  den = np.linalg.norm(e)
  return float(np.linalg.norm(a - e) / (den if den > 0 else 1.0))
