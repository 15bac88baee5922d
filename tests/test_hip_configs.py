"""The five measured configurations at full size, checked through size-independent properties.

The CPU oracle cannot run a 2 TFLOP problem in seconds, so at full size each configuration is checked
by (a) the oracle on a seeded sample with one row out of every 32-row block of every group, (b) exact linearity under a
power-of-two scaling of lhs, (c) zero rows past sum(group_sizes) and untouched-by-construction empty
groups, (d) run-twice bit equality. The fp32 configuration is small enough to compare in full.
"""

import numpy as np
import pytest
import torch

import tokamax_amd
from tokamax_amd import _lib
from oracle import ragged_dot_oracle as O
from tokamax_amd.ragged_dot import arg_specs, base, workloads

pytestmark = pytest.mark.gpu


def _np(x):
  return x.detach().float().cpu().numpy()


def _sample_rows(gs, per_group, seed):
  rng = np.random.default_rng(seed)
  off = O.group_offsets(gs)
  rows, groups = [], []
  for g in range(len(gs)):
    s, e = int(off[g]), int(off[g + 1])
    if e > s:
      # first and last row of the group (tile-straddling edges) plus random interior rows
      pick = {s, e - 1} | set(rng.integers(s, e, per_group).tolist())
      rows += sorted(pick)
      groups += [g] * len(pick)
  return np.array(rows), np.array(groups)


def _sample_every_block(gs, seed, block=32):
  """One random row out of every `block` consecutive rows of every group (counted from the group's first row), and
  each group's first and last row: every 32-row block of every m-tile of every task gets a row, so a tile, a wave's
  row block or a group boundary that is addressed wrongly cannot slip through."""
  rng = np.random.default_rng(seed)
  off = O.group_offsets(gs)
  rows, groups = [], []
  for g in range(len(gs)):
    s, e = int(off[g]), int(off[g + 1])
    if e <= s:
      continue
    pick = {s, e - 1}
    for b0 in range(s, e, block):
      pick.add(int(rng.integers(b0, min(b0 + block, e))))
    rows += sorted(pick)
    groups += [g] * len(pick)
  return np.array(rows), np.array(groups)


def _check_rows(out, lhs_f, rhs_of_group, rows, groups, tol):
  """The sampled rows of `out` against the oracle's definition, group by group: lhs rows of group g times rhs[g], one
  f32 BLAS product per group on the host (`rhs_of_group(g)` brings one group's weights over at a time)."""
  got = _np(out[torch.as_tensor(rows, device=out.device)])
  want = np.empty(got.shape, np.float32)
  for g in np.unique(groups):
    sel = np.nonzero(groups == g)[0]
    want[sel] = lhs_f[sel].astype(np.float32) @ rhs_of_group(int(g)).astype(np.float32)
  err = O.rel_l2(got, want)
  assert err <= tol, f"rel_l2 {err:.3e} > {tol}"
  # row by row as well: an error confined to a few rows must not hide in the norm of thousands
  per_row = np.linalg.norm(got - want, axis=1) / np.maximum(np.linalg.norm(want, axis=1), 1e-30)
  assert per_row.max() <= 4 * tol, f"row {rows[int(per_row.argmax())]}: rel_l2 {per_row.max():.3e}"


def test_fp32_config_in_full(device):
  w = workloads.make("fp32", device)
  gs = torch.tensor(w.group_sizes, device=device)
  out = tokamax_amd.ragged_dot(w.lhs, w.rhs, gs, precision="highest")
  assert out.dtype == torch.float32
  want = O.ragged_dot(_np(w.lhs), _np(w.rhs), w.group_sizes, acc_dtype=np.float32, out_dtype="f32")
  assert O.rel_l2(_np(out), want) <= 1e-5
  want64 = O.ragged_dot(_np(w.lhs), _np(w.rhs), w.group_sizes, acc_dtype=np.float64, out_dtype="f64")
  assert O.rel_l2(_np(out), want64) <= 1e-5


@pytest.mark.parametrize("name", ["mixtral", "deepseek"])
def test_bf16_prefill_configs(name, device):
  w = workloads.make(name, device)
  gs = torch.tensor(w.group_sizes, device=device)
  out = tokamax_amd.ragged_dot(w.lhs, w.rhs, gs)
  assert out.dtype == torch.bfloat16 and tuple(out.shape) == (w.m, w.n)
  rows, groups = _sample_every_block(w.group_sizes, 0)  # 512 rows and more (mixtral), 2048 and more (deepseek)
  assert len(rows) >= w.m // 32
  lhs_f = _np(w.lhs[torch.as_tensor(rows, device=device)])
  _check_rows(out, lhs_f, lambda g: _np(w.rhs[g]), rows, groups, 2e-3)
  # linearity: scaling lhs by 2 scales every output by exactly 2 (power of two: no rounding anywhere)
  out2 = tokamax_amd.ragged_dot(w.lhs * 2, w.rhs, gs)
  assert torch.equal(out2, out * 2)
  assert torch.equal(tokamax_amd.ragged_dot(w.lhs, w.rhs, gs), out)  # deterministic
  if name == "deepseek":
    assert (w.group_sizes == 0).sum() >= 8
  del out2
  # a shorter total leaves a zero tail
  short = w.group_sizes.copy()
  short[np.argmax(short)] -= 100
  out3 = tokamax_amd.ragged_dot(w.lhs, w.rhs, torch.tensor(short, device=device))
  assert torch.count_nonzero(out3[int(short.sum()):]) == 0


def test_decode_int8_config(device):
  w = workloads.make("decode", device)
  gs = torch.tensor(w.group_sizes, device=device)
  rhs = tokamax_amd.QArray(w.rhs, w.rhs_scale)
  out = tokamax_amd.ragged_dot(w.lhs, rhs, gs, preferred_element_type=torch.bfloat16)
  want = O.ragged_dot(_np(w.lhs), O.dequantize(w.rhs.cpu().numpy(), _np(w.rhs_scale)), w.group_sizes,
                      acc_dtype=np.float64, out_dtype="f64")
  assert O.rel_l2(_np(out), want) <= 3e-2
  assert O.rel_l2(_np(out), want) <= 3e-3  # in fact bf16-rounding accurate: int8 -> bf16 is exact
  out32 = tokamax_amd.ragged_dot(w.lhs, rhs, gs, preferred_element_type=torch.float32)
  assert O.rel_l2(_np(out32), want) <= 1e-5
  assert (w.group_sizes == 0).any() and w.group_sizes.sum() == w.m


def test_fp8_config(device):
  w = workloads.make("fp8", device)
  gs = torch.tensor(w.group_sizes, device=device)
  out = tokamax_amd.ragged_dot(tokamax_amd.QArray(w.lhs, w.lhs_scale), tokamax_amd.QArray(w.rhs, w.rhs_scale), gs,
                               preferred_element_type=torch.bfloat16)
  rows, groups = _sample_every_block(w.group_sizes, 1)
  assert len(rows) >= w.m // 32
  idx = torch.as_tensor(rows, device=device)
  lhs_f = _np(w.lhs[idx]) * _np(w.lhs_scale[idx])
  _check_rows(out, lhs_f, lambda g: _np(w.rhs[g]) * _np(w.rhs_scale[g]), rows, groups, 3e-3)
  assert torch.equal(tokamax_amd.ragged_dot(tokamax_amd.QArray(w.lhs, w.lhs_scale), tokamax_amd.QArray(w.rhs, w.rhs_scale),
                                            gs, preferred_element_type=torch.bfloat16), out)


@pytest.mark.parametrize("scales", ["per_column", "per_128_k_rows"])
def test_packed_int4_weights_at_the_prefill_size(scales, device):
  """The Mixtral prefill shape over int4 weights packed two to a byte, read by the tiled kernels as they are: one row
  out of every 32-row block of every group against the oracle's definition on the unpacked, dequantised values (with
  scales per k-block the kernel rounds weight x scale to bf16, like the reference's in-kernel dequantisation), exact
  linearity, determinism."""
  w = workloads.make("mixtral", device)
  gs = torch.tensor(w.group_sizes, device=device)
  gen = torch.Generator(device=device).manual_seed(3)
  q = torch.randint(-8, 8, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen)
  blocks = 1 if scales == "per_column" else w.k // 128
  scale = (torch.rand(w.num_groups, blocks, w.n, device=device, generator=gen) + 0.5) / (7 * w.k ** 0.5)
  packed = tokamax_amd.pack_int4(tokamax_amd.QArray(q, scale, None, getattr(torch, "int4", torch.int8)))
  assert packed.packed and tuple(packed.qvalue.shape) == (w.num_groups, w.k // 2, w.n)
  op = tokamax_amd.HipRaggedDot()
  bound = op.bind(w.lhs, packed, group_sizes=gs, preferred_element_type=torch.bfloat16)
  assert op._problem(bound)[1][2] == _lib.TKX_I4X2 and bound.default_config.block_m >= 128  # stays packed, tiled kernel
  out = tokamax_amd.ragged_dot(w.lhs, packed, gs, preferred_element_type=torch.bfloat16)
  assert out.dtype == torch.bfloat16 and tuple(out.shape) == (w.m, w.n)
  rows, groups = _sample_every_block(w.group_sizes, 2)
  assert len(rows) >= w.m // 32
  lhs_f = _np(w.lhs[torch.as_tensor(rows, device=device)])

  def weights(g):
    values = O.dequantize(q[g].cpu().numpy()[None], _np(scale[g])[None])[0]
    return O.round_to_bf16(values) if blocks > 1 else values

  _check_rows(out, lhs_f, weights, rows, groups, 3e-3)
  assert torch.equal(tokamax_amd.ragged_dot(w.lhs * 2, packed, gs, preferred_element_type=torch.bfloat16), out * 2)
  assert torch.equal(tokamax_amd.ragged_dot(w.lhs, packed, gs, preferred_element_type=torch.bfloat16), out)


def test_fp8_activations_over_packed_int4_weights_at_the_prefill_size(device):
  """The Mixtral prefill shape with activations quantised to fp8 per row over int4 weights packed two to a byte, on the
  fp8 MFMAs (the 128-row tile on one row of four waves): one row out of every 32-row block of every group against the oracle's definition on
  the dequantised operands; scaling the activations' scales by two doubles the result exactly (the affine correction
  with the row sums is applied before the scales); determinism."""
  w = workloads.make("fp8", device)
  gs = torch.tensor(w.group_sizes, device=device)
  gen = torch.Generator(device=device).manual_seed(5)
  q = torch.randint(-8, 8, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen)
  scale = (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen) + 0.5) / (7 * w.k ** 0.5)
  packed = tokamax_amd.pack_int4(tokamax_amd.QArray(q, scale, None, getattr(torch, "int4", torch.int8)))
  lhs = tokamax_amd.QArray(w.lhs, w.lhs_scale)
  op = tokamax_amd.HipRaggedDot()
  bound = op.bind(lhs, packed, group_sizes=gs, preferred_element_type=torch.bfloat16)
  assert op._problem(bound)[1] == (0, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2) and bound.default_config.block_m == 128
  out = tokamax_amd.ragged_dot(lhs, packed, gs, preferred_element_type=torch.bfloat16)
  assert out.dtype == torch.bfloat16 and tuple(out.shape) == (w.m, w.n)
  rows, groups = _sample_every_block(w.group_sizes, 2)
  assert len(rows) >= w.m // 32
  index = torch.as_tensor(rows, device=device)
  lhs_f = (O.e4m3fn_decode(w.lhs[index].view(torch.uint8).cpu().numpy()).astype(np.float64)
           * _np(w.lhs_scale.reshape(w.m, 1)[index]))
  _check_rows(out, lhs_f, lambda g: O.dequantize(q[g].cpu().numpy()[None], _np(scale[g])[None])[0], rows, groups, 3e-3)
  doubled = tokamax_amd.QArray(w.lhs, w.lhs_scale * 2)
  assert torch.equal(tokamax_amd.ragged_dot(doubled, packed, gs, preferred_element_type=torch.bfloat16), out * 2)
  assert torch.equal(tokamax_amd.ragged_dot(lhs, packed, gs, preferred_element_type=torch.bfloat16), out)


def test_vjp_config(device):
  w = workloads.make("vjp", device)
  gs = torch.tensor(w.group_sizes, device=device)
  dlhs = tokamax_amd.ragged_dot_general(w.dout, w.rhs, gs, base.TRANS_RHS_RAGGED_DOT_DIM_NUMS)
  assert dlhs.dtype == torch.bfloat16 and tuple(dlhs.shape) == (w.m, w.k)
  rows, groups = _sample_every_block(w.group_sizes, 2)
  assert len(rows) >= w.m // 32
  dout_f = _np(w.dout[torch.as_tensor(rows, device=device)])
  _check_rows(dlhs, dout_f, lambda g: _np(w.rhs[g]).T, rows, groups, 2e-3)
  drhs = tokamax_amd.ragged_dot_general(w.lhs, w.dout, gs, base.RAGGED_CONTRACTING_DOT_DIM_NUMS)
  assert drhs.dtype == torch.bfloat16 and tuple(drhs.shape) == (w.num_groups, w.k, w.n)
  # drhs[g][kk, :] = lhs[rows_g, kk]^T . dout[rows_g, :] for sampled (g, kk)
  off = O.group_offsets(w.group_sizes)
  # one k-row out of every 32 of every group's [k, n] result
  rng = np.random.default_rng(3)
  for g in range(w.num_groups):
    s, e = int(off[g]), int(off[g + 1])
    kks = torch.as_tensor(np.array([int(rng.integers(b0, b0 + 32)) for b0 in range(0, w.k, 32)]), device=device)
    got = _np(drhs[g][kks])
    want = _np(w.lhs[s:e][:, kks]).astype(np.float32).T @ _np(w.dout[s:e]).astype(np.float32)
    assert O.rel_l2(got, want) <= 2e-3, g
    per_row = np.linalg.norm(got - want, axis=1) / np.maximum(np.linalg.norm(want, axis=1), 1e-30)
    assert per_row.max() <= 8e-3, (g, int(kks[int(per_row.argmax())]))
  # the same gradients through autograd of the public API
  lhs = w.lhs[:512].clone().requires_grad_(True)
  rhs = w.rhs.clone().requires_grad_(True)
  small = np.array([64] * 8, np.int32)
  out = tokamax_amd.ragged_dot(lhs, rhs, torch.tensor(small, device=device))
  out.backward(w.dout[:512])
  want_dlhs = tokamax_amd.ragged_dot_general(w.dout[:512], w.rhs, torch.tensor(small, device=device), base.TRANS_RHS_RAGGED_DOT_DIM_NUMS)
  assert torch.equal(lhs.grad, want_dlhs)


@pytest.mark.parametrize("spec", [s for s in arg_specs.ARG_SPECS if "ci_tests" in s.tags], ids=lambda s: s.full_name)
def test_bench_arg_specs(spec, device):
  """The reference's `test_bench` (test_base.py:316-344) over its `ci_tests` arg specs (arg_specs.py:23-60:
  compute_bound, memory_bound, mixtral 8x7b): standard-normal inputs, representative group sizes, the first
  sum(group_sizes) rows against the reference definition within atol=0.01, rtol=0.005 (the 8x7b shape on sampled
  rows of every group, the other two in full)."""
  kwargs = arg_specs.random_initialize(spec.args, device)
  lhs, rhs, gs = kwargs["lhs"], kwargs["rhs"], kwargs["group_sizes"]
  sizes = np.array(spec.args["group_sizes"].representative_value, np.int32)
  count = int(sizes.sum())
  assert count <= lhs.shape[0] and tuple(gs.shape) == (rhs.shape[0],)
  out = tokamax_amd.ragged_dot(lhs, rhs, gs)
  assert out.dtype == torch.bfloat16 and tuple(out.shape) == (lhs.shape[0], rhs.shape[2])
  if lhs.shape[0] * rhs.shape[1] * rhs.shape[2] <= 2 ** 37:
    want = O.ragged_dot(_np(lhs), _np(rhs), sizes, acc_dtype=np.float32, out_dtype="f32")
    np.testing.assert_allclose(_np(out)[:count], want[:count], atol=0.01, rtol=0.005)
    assert O.rel_l2(_np(out)[:count], want[:count]) <= 2e-3
  else:
    rows, groups = _sample_rows(sizes, 24, 5)
    lhs_f = _np(lhs[torch.as_tensor(rows, device=device)])
    _check_rows(out, lhs_f, lambda g: _np(rhs[g]), rows, groups, 2e-3)
  assert arg_specs.flops(**spec.args) == 2 * count * rhs.shape[1] * rhs.shape[2]
