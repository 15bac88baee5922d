"""Pins the CPU oracle before anything is compared against it (no GPU needed).

Integer part: the literal known-answer vectors of the reference's own scheduler test
(tests/golden/scheduler_kat.json, from pallas_mosaic_gpu_common_test.py:27-84) plus invariants.
Floating-point part: the reference stores no outputs, so `ragged_dot` is pinned by what the
mathematics fixes -- brute-force loops, special cases that reduce to a library GEMM, autograd of the
forward for the two backward contractions -- each chosen so that a dropped term, a wrong index or a
transposed operand fails.
"""

import json
import os

import numpy as np
import pytest
import torch

from oracle import c_oracle
from oracle import ragged_dot_oracle as O

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
FIELDS = ("group_id", "block_start", "actual_start", "actual_end", "start_within_block", "actual_size")

with open(os.path.join(GOLDEN, "scheduler_kat.json")) as _f:
  KAT = json.load(_f)


@pytest.mark.parametrize("case", KAT, ids=[c["name"] for c in KAT])
@pytest.mark.parametrize("impl", ["numpy", "c"])
def test_scheduler_known_answers(case, impl):
  fn = O.group_info_create_aligned if impl == "numpy" else c_oracle.create_aligned
  got = fn(np.array(case["group_sizes"], np.int32), case["tile"], case["tid_size"], case["align_tile"])
  for f in FIELDS:
    np.testing.assert_array_equal(got[f], np.array(case[f], np.int32), err_msg=f)


@pytest.mark.parametrize("seed", range(6))
def test_scheduler_invariants_and_c_agrees(seed):
  rng = np.random.default_rng(seed)
  G = int(rng.integers(1, 40))
  gs = rng.integers(0, 70, G).astype(np.int32)
  gs[rng.random(G) < 0.3] = 0
  if seed == 0:
    gs[0] = -5  # negative sizes count as zero (pallas_mosaic_gpu_common.py:119)
  tile = int(rng.choice([8, 16, 32, 64]))
  total = int(np.maximum(gs, 0).sum())
  m = total + int(rng.integers(0, 20))
  tid = -(-m // tile) + G - 1
  a = O.group_info_create_aligned(gs, tile, tid, 8)
  b = c_oracle.create_aligned(gs, tile, tid, 8)
  for f in FIELDS:
    np.testing.assert_array_equal(a[f], b[f], err_msg=f)
  assert a["num_tasks"] == b["num_tasks"] <= tid
  nt = a["num_tasks"]
  off = O.group_offsets(gs)
  np.testing.assert_array_equal(off, c_oracle.group_offsets(gs))
  np.testing.assert_array_equal(off, np.concatenate([[0], np.cumsum(np.maximum(gs, 0))]))
  # store ranges of the real tasks partition [0, total) in order
  assert int(a["actual_size"][:nt].sum()) == total
  pos = 0
  for t in range(nt):
    assert a["actual_start"][t] == pos and a["actual_size"][t] > 0
    pos = a["actual_end"][t]
    assert a["block_start"][t] % 8 == 0
    assert 0 <= a["start_within_block"][t] < 8
    g = a["group_id"][t]
    assert off[g] <= a["actual_start"][t] and a["actual_end"][t] <= off[g + 1]
    assert a["actual_end"][t] <= a["block_start"][t] + tile
  assert pos == total
  assert np.all(np.diff(a["group_id"][:nt]) >= 0)  # tasks of a group are contiguous
  assert np.all(a["actual_size"][nt:] == 0)


# What the mathematics fixes of `generate_group_sizes` (base.py:171-196: `m` draws with replacement over the
# groups with probabilities `p`, counted per group). The reference stores no sizes for any seed, so the exact
# values are compared between the oracle and the product twin only; each property below fails for a plausible
# mistake (ignoring `p`, dropping `minlength`, a fixed generator, counting something other than the draws).
@pytest.mark.parametrize("m,num_groups,p", [(256, 4, None), (16, 64, None), (256, 4, (0.1, 0.2, 0.3, 0.4))])
def test_generate_group_sizes_reference_cases(m, num_groups, p):
  # The three parametrisations of base_test.py:45-51; (16, 64) has more groups than rows, so the trailing
  # groups nobody drew must still be listed (with 16 draws over 64 groups some always are empty).
  gs = O.generate_group_sizes(m=m, num_groups=num_groups, p=p)
  assert isinstance(gs, tuple) and all(isinstance(v, int) for v in gs)
  assert len(gs) == num_groups and sum(gs) == m and min(gs) >= 0
  from tokamax_amd.ragged_dot import base
  assert base.generate_group_sizes(m=m, num_groups=num_groups, p=p) == gs


def test_generate_group_sizes_one_hot_p_puts_every_row_in_that_group():
  for hot in (0, 2, 4):
    p = [0.0] * 5
    p[hot] = 1.0
    want = [0] * 5
    want[hot] = 1000
    assert O.generate_group_sizes(m=1000, num_groups=5, p=p) == tuple(want)


def test_generate_group_sizes_frequencies_follow_p():
  from tokamax_amd.ragged_dot import base
  m = 10 ** 6
  p = np.array((0.1, 0.2, 0.3, 0.4))
  for seed in (0, 7):
    gs = np.array(O.generate_group_sizes(m=m, num_groups=4, p=tuple(p), seed=seed))
    sigma = np.sqrt(m * p * (1 - p))  # each count is binomial(m, p_i)
    assert np.all(np.abs(gs - m * p) <= 4 * sigma), (gs, m * p, sigma)
    assert base.generate_group_sizes(m=m, num_groups=4, p=tuple(p), seed=seed) == tuple(gs)
  # p=None is the uniform distribution: the same test with p_i = 1/G, and no group anywhere near p's pattern.
  gs = np.array(O.generate_group_sizes(m=m, num_groups=8))
  assert np.all(np.abs(gs - m / 8) <= 4 * np.sqrt(m * (1 / 8) * (7 / 8)))


def test_generate_group_sizes_seed_selects_the_draw():
  from tokamax_amd.ragged_dot import base
  a = O.generate_group_sizes(m=4096, num_groups=16, seed=3)
  assert a == O.generate_group_sizes(m=4096, num_groups=16, seed=3)   # a function of its arguments only
  assert a != O.generate_group_sizes(m=4096, num_groups=16, seed=4)   # and the seed is used
  assert a != O.generate_group_sizes(m=4096, num_groups=16)           # default seed is 0, not 3
  assert O.generate_group_sizes(m=4096, num_groups=16) == O.generate_group_sizes(m=4096, num_groups=16, seed=0)
  for seed in (0, 3, 4):
    assert base.generate_group_sizes(m=4096, num_groups=16, seed=seed) == O.generate_group_sizes(m=4096, num_groups=16, seed=seed)


def test_generate_group_sizes_counts_the_draws():
  # With m = 1 exactly one group holds the row; with G = 1 every row lands in it.
  for seed in range(5):
    gs = O.generate_group_sizes(m=1, num_groups=7, seed=seed)
    assert sorted(gs) == [0] * 6 + [1]
  assert O.generate_group_sizes(m=123, num_groups=1) == (123,)
  assert O.generate_group_sizes(m=0, num_groups=3) == (0, 0, 0)


@pytest.mark.parametrize("mode", [O.DEFAULT, O.TRANS_RHS, O.RAGGED_CONTRACTING])
def test_ragged_dot_vs_bruteforce(mode):
  rng = np.random.default_rng(3)
  G, m, k, n = 3, 13, 5, 7
  gs = [4, 0, 6]  # 3 trailing rows belong to no group
  lhs = rng.normal(size=(m, n if mode == O.TRANS_RHS else k))
  rhs = rng.normal(size=(m, n)) if mode == O.RAGGED_CONTRACTING else rng.normal(size=(G, k, n))
  want = O.ragged_dot_bruteforce(lhs, rhs, gs, mode)
  got = O.ragged_dot(lhs, rhs, gs, mode, acc_dtype=np.float64, out_dtype="f64")
  np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
  got32 = c_oracle.ragged_dot_f32(lhs, rhs, np.array(gs, np.int32), {O.DEFAULT: 0, O.TRANS_RHS: 1, O.RAGGED_CONTRACTING: 2}[mode])
  np.testing.assert_allclose(got32, want, rtol=2e-5, atol=2e-5)
  if mode != O.RAGGED_CONTRACTING:
    assert np.all(got[10:] == 0)  # rows past sum(group_sizes) are zero
  else:
    assert np.all(got[1] == 0)  # empty group


def test_special_cases_reduce_to_library_gemm():
  rng = np.random.default_rng(4)
  G, m, k, n = 4, 32, 16, 24
  lhs, rhs = rng.normal(size=(m, k)), rng.normal(size=(G, k, n))
  # one group -> plain GEMM
  np.testing.assert_allclose(O.ragged_dot(lhs, rhs[:1], [m], acc_dtype=np.float64, out_dtype="f64"), lhs @ rhs[0], rtol=1e-12)
  # all rows in group 0 (bench.py:35-39)
  np.testing.assert_allclose(O.ragged_dot(lhs, rhs, [m, 0, 0, 0], acc_dtype=np.float64, out_dtype="f64"), lhs @ rhs[0], rtol=1e-12)
  # even groups -> batched GEMM (bench.py:43-49)
  want = np.einsum("gmk,gkn->gmn", lhs.reshape(G, m // G, k), rhs).reshape(m, n)
  np.testing.assert_allclose(O.ragged_dot(lhs, rhs, [m // G] * G, acc_dtype=np.float64, out_dtype="f64"), want, rtol=1e-12)
  # the group of each row matters: permuting the weights of two groups changes exactly their rows
  swapped = rhs[[1, 0, 2, 3]]
  a = O.ragged_dot(lhs, rhs, [8] * 4, acc_dtype=np.float64, out_dtype="f64")
  b = O.ragged_dot(lhs, swapped, [8] * 4, acc_dtype=np.float64, out_dtype="f64")
  np.testing.assert_allclose(a[:8], lhs[:8] @ rhs[0], rtol=1e-12)
  np.testing.assert_allclose(b[:8], lhs[:8] @ rhs[1], rtol=1e-12)
  np.testing.assert_array_equal(a[16:], b[16:])


def test_backward_contractions_match_autograd_of_forward():
  rng = np.random.default_rng(5)
  G, m, k, n = 3, 20, 6, 9
  gs = [7, 0, 9]
  lhs = torch.tensor(rng.normal(size=(m, k)), requires_grad=True)
  rhs = torch.tensor(rng.normal(size=(G, k, n)), requires_grad=True)
  dout = rng.normal(size=(m, n))
  off = O.group_offsets(gs)
  out = torch.zeros(m, n, dtype=torch.float64)
  pieces = []
  for g in range(G):
    s, e = int(off[g]), int(off[g + 1])
    pieces.append(lhs[s:e] @ rhs[g])
  out = torch.cat(pieces + [torch.zeros(m - int(off[-1]), n, dtype=torch.float64)])
  out.backward(torch.tensor(dout))
  np.testing.assert_allclose(O.ragged_dot(dout, rhs.detach().numpy(), gs, O.TRANS_RHS, acc_dtype=np.float64, out_dtype="f64"),
                             lhs.grad.numpy(), rtol=1e-12, atol=1e-12)
  np.testing.assert_allclose(
      O.ragged_dot(lhs.detach().numpy(), dout, gs, O.RAGGED_CONTRACTING, acc_dtype=np.float64, out_dtype="f64"),
      rhs.grad.numpy(), rtol=1e-12, atol=1e-12)


def test_f32_accumulation_and_single_rounding():
  rng = np.random.default_rng(6)
  lhs = O.round_to_bf16(rng.normal(size=(16, 64)).astype(np.float32))
  rhs = O.round_to_bf16(rng.normal(size=(2, 64, 8)).astype(np.float32))
  f64 = O.ragged_dot(lhs, rhs, [9, 7], acc_dtype=np.float64, out_dtype="f64")
  f32 = O.ragged_dot(lhs, rhs, [9, 7], acc_dtype=np.float32, out_dtype="f32")
  assert f32.dtype == np.float32 and O.rel_l2(f32, f64) < 1e-6
  bf = O.ragged_dot(lhs, rhs, [9, 7], acc_dtype=np.float32, out_dtype="bf16")
  np.testing.assert_array_equal(bf, torch.tensor(f32).to(torch.bfloat16).float().numpy())


def test_bf16_rounding_matches_torch():
  rng = np.random.default_rng(7)
  x = np.concatenate([rng.normal(size=4096).astype(np.float32) * 10.0 ** rng.integers(-20, 20, 4096),
                      np.array([0.0, -0.0, 1.0, 65504.0, 3.3895314e38, 1.0000001, 1.00390625, 1.01171875], np.float32)])
  want = torch.tensor(x).to(torch.bfloat16)
  np.testing.assert_array_equal(O.round_to_bf16(x), want.float().numpy())
  np.testing.assert_array_equal(O.bf16_bits(x), want.view(torch.int16).numpy().view(np.uint16))
  np.testing.assert_array_equal(O.bf16_from_bits(O.bf16_bits(x)), want.float().numpy())


def test_e4m3fn_matches_torch_exhaustively():
  bits = np.arange(256, dtype=np.uint8)
  want = torch.tensor(bits).view(torch.float8_e4m3fn).float().numpy()
  got = O.e4m3fn_decode(bits)
  np.testing.assert_array_equal(np.isnan(got), np.isnan(want))
  np.testing.assert_array_equal(got[~np.isnan(want)], want[~np.isnan(want)])
  rng = np.random.default_rng(8)
  x = np.concatenate([rng.normal(size=20000).astype(np.float32) * 10.0 ** rng.integers(-4, 3, 20000),
                      got[~np.isnan(got)], np.array([448.0, -448.0, 464.0, 0.0009765625, 0.0029296875], np.float32)])
  x = x[np.abs(x) <= 464]  # torch saturates differently above the last rounding boundary; stay in range
  enc = O.e4m3fn_encode(x)
  tw = torch.tensor(x).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
  np.testing.assert_array_equal(O.e4m3fn_decode(enc), O.e4m3fn_decode(tw))


def test_int4_weights_as_fp8_denormals_and_as_int8_times_16():
  """What the kernels that feed packed int4 weights to the fp8 and int8 matrix instructions rest on
  (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:258-300, ..._sm100_i8_quant.py:114-190): the byte 0000uuuu, u = nibble
  xor 8 = w + 8, decodes as the e4m3 value u / 512 for every int4 w, so sum(x w) = 512 sum(x (w + 8) / 512) - 8 sum(x)
  in exact arithmetic; and a nibble at the top of a byte is the int8 value 16 w. On a small product against the
  oracle's definition."""
  w = np.arange(-8, 8)
  nibbles = (w & 0xF).astype(np.uint8)
  np.testing.assert_array_equal(O.e4m3fn_decode(nibbles ^ 8), (w + 8) / 512.0)
  np.testing.assert_array_equal((nibbles << 4).astype(np.uint8).view(np.int8), 16 * w)
  rng = np.random.default_rng(4)
  k, n, rows = 256, 24, 5
  x = O.e4m3fn_decode(rng.integers(0, 256, (rows, k)).astype(np.uint8) & 0x77 | 0x08).astype(np.float64)  # finite fp8 values
  values = rng.integers(-8, 8, (1, k, n))
  want = O.ragged_dot(x, values.astype(np.float64), np.array([rows], np.int32), O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  packed = O.pack_int4(values)[0]
  as_fp8 = np.empty((k, n))
  as_fp8[0::2], as_fp8[1::2] = O.e4m3fn_decode((packed & 0xF) ^ 8), O.e4m3fn_decode((packed >> 4) ^ 8)
  np.testing.assert_allclose(512 * (x @ as_fp8) - 8 * x.sum(axis=1, keepdims=True), want, rtol=0, atol=1e-9)
  as_int8 = np.empty((k, n))
  as_int8[0::2], as_int8[1::2] = (packed << 4).astype(np.uint8).view(np.int8), (packed & 0xF0).astype(np.uint8).view(np.int8)
  np.testing.assert_array_equal((x @ as_int8) / 16, want)


def test_fused_epilogue_terms():
  """rhs_bias and gate-up fusion (base.py:205-217): the activations against torch's, the composition
  against brute force on a tiny case."""
  x = np.linspace(-6, 6, 97)
  np.testing.assert_allclose(O.silu(x), torch.nn.functional.silu(torch.tensor(x)).numpy(), rtol=1e-12, atol=1e-15)
  np.testing.assert_allclose(O.gelu_tanh(x), torch.nn.functional.gelu(torch.tensor(x), approximate="tanh").numpy(),
                             rtol=1e-12, atol=1e-15)
  rng = np.random.default_rng(5)
  gs = np.array([2, 0, 3], np.int32)
  lhs, rhs = rng.normal(size=(7, 5)), rng.normal(size=(3, 5, 8))
  bias = rng.normal(size=(3, 1, 8))
  tmp = O.ragged_dot_bruteforce(lhs, rhs, gs)
  for g, (s, e) in enumerate([(0, 2), (2, 2), (2, 5)]):
    tmp[s:e] += bias[g, 0]
  np.testing.assert_allclose(O.ragged_dot_fused(lhs, rhs, gs, rhs_bias=bias), tmp, rtol=1e-12, atol=1e-12)
  assert np.all(O.ragged_dot_fused(lhs, rhs, gs, rhs_bias=bias)[5:] == 0)  # rows of no group get no bias
  want = torch.nn.functional.silu(torch.tensor(tmp[:, :4])).numpy() * tmp[:, 4:]
  np.testing.assert_allclose(O.ragged_dot_fused(lhs, rhs, gs, rhs_bias=bias, gateup_activation="silu"), want,
                             rtol=1e-12, atol=1e-12)


def test_clamped_gateup_forms():
  """"swigluoai" and "silu_and_mul_with_clamp" (experimental/gmm_v2/gmm_v2.py:29-50): against torch's clamp /
  sigmoid / silu, and values worked by hand where the clipping acts: the gate is clipped from above
  only, the up part on both sides, and "swigluoai" multiplies by up + 1."""
  rng = np.random.default_rng(2)
  gate, up = rng.normal(0, 6, 400), rng.normal(0, 6, 400)
  g, u = torch.tensor(gate), torch.tensor(up)
  gc, uc = g.clamp(max=7.0), u.clamp(-7.0, 7.0)
  np.testing.assert_allclose(O.gateup(gate, up, "swigluoai"), ((uc + 1) * gc * torch.sigmoid(1.702 * gc)).numpy(),
                             rtol=1e-12, atol=1e-12)
  gc, uc = g.clamp(max=10.0), u.clamp(-10.0, 10.0)
  np.testing.assert_allclose(O.gateup(gate, up, "silu_and_mul_with_clamp"),
                             (torch.nn.functional.silu(gc) * uc).numpy(), rtol=1e-12, atol=1e-12)
  # gate 9 -> 7 and up 9 -> 7: 8 * 7 * sigmoid(11.914) = 56 / (1 + e^-11.914) = 56 / 1.0000066967 = 55.999625
  np.testing.assert_allclose(O.gateup([9.0], [9.0], "swigluoai"), [55.999625], rtol=2e-8)
  # up -9 -> -7: (-7 + 1) * 7 * sigmoid(11.914) = -41.999719; a zero gate gives zero; gate -> -inf gives 0 (not clipped below)
  np.testing.assert_allclose(O.gateup([7.0], [-9.0], "swigluoai"), [-41.999719], rtol=2e-8)
  assert O.gateup([0.0], [3.0], "swigluoai")[0] == 0.0
  assert abs(O.gateup([-40.0], [3.0], "swigluoai")[0]) < 1e-25
  # up = -1 cancels "swigluoai" and not the clamped silu; silu(1) = 1 / (1 + 1/e) = 0.7310585786
  assert O.gateup([1.0], [-1.0], "swigluoai")[0] == 0.0
  np.testing.assert_allclose(O.gateup([1.0], [-1.0], "silu_and_mul_with_clamp"), [-0.7310585786], rtol=1e-9)
  # gate 12 -> 10, up 12 -> 10: silu(10) * 10 = 100 / (1 + e^-10) = 99.995460
  np.testing.assert_allclose(O.gateup([12.0], [12.0], "silu_and_mul_with_clamp"), [99.995460], rtol=2e-8)
  np.testing.assert_allclose(O.gateup(gate, up, "gelu"), O.gateup(gate, up, "gelu_tanh"))
  with pytest.raises(NotImplementedError):
    O.gateup(gate, up, "relu")


def test_group_offset_shards():
  """`group_offset` (experimental/gmm_v2/gmm_v2_test.py:44-101): rhs holds the groups [offset, offset + G)
  of the job's group sizes and every other group's rows are zero. Pinned by explicit loops on a tiny
  case and by the identity it exists for: the shards' outputs add up to the unsharded result."""
  rng = np.random.default_rng(4)
  gs = np.array([2, 0, 3, 1, 4], np.int32)  # 10 rows, then 2 rows of no group
  lhs, rhs = rng.normal(size=(12, 5)), rng.normal(size=(5, 5, 6))
  bias = rng.normal(size=(5, 1, 6))
  full = O.ragged_dot_fused(lhs, rhs, gs, rhs_bias=bias)
  np.testing.assert_array_equal(O.ragged_dot_fused(lhs, rhs, gs, rhs_bias=bias, group_offset=[0]), full)
  # groups 2 and 3 (rows 2..5) as a shard of two groups
  want = np.zeros((12, 6))
  for i in range(2, 5):
    want[i] = lhs[i] @ rhs[2] + bias[2, 0]
  want[5] = lhs[5] @ rhs[3] + bias[3, 0]
  got = O.ragged_dot_fused(lhs, rhs[2:4], gs, rhs_bias=bias[2:4], group_offset=np.array([2]))
  np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
  parts = [O.ragged_dot_fused(lhs, rhs[o:o + c], gs, rhs_bias=bias[o:o + c], group_offset=[o]) for o, c in ((0, 2), (2, 2), (4, 1))]
  np.testing.assert_allclose(sum(parts), full, rtol=1e-12, atol=1e-12)
  # a shard past the last group, and one that starts before the first: entries outside the sizes are empty
  assert not O.ragged_dot_fused(lhs, rhs[:2], gs, group_offset=[5]).any()
  got = O.ragged_dot_fused(lhs, rhs[:3], gs, group_offset=[-2])  # local group 2 is global group 0
  want = np.zeros((12, 6))
  want[:2] = lhs[:2] @ rhs[2]
  np.testing.assert_allclose(got, want, rtol=1e-12, atol=1e-12)
  # the gate-up form keeps the other groups' rows at zero
  glu = O.ragged_dot_fused(lhs, rhs[2:4], gs, rhs_bias=bias[2:4], group_offset=[2], gateup_activation="swigluoai")
  assert glu.shape == (12, 3) and not glu[:2].any() and not glu[6:].any() and glu[2:6].all()


def test_gated_linear_unit_matches_torch():
  rng = np.random.default_rng(3)
  x, w = rng.normal(size=(2, 5, 7)), rng.normal(size=(7, 2, 4))
  xt, wt = torch.tensor(x), torch.tensor(w)
  want = torch.nn.functional.silu(xt @ wt[:, 0]) * (xt @ wt[:, 1])
  np.testing.assert_allclose(O.gated_linear_unit(x, w, O.silu), want.numpy(), rtol=1e-12, atol=1e-12)
  np.testing.assert_allclose(O.gated_linear_unit(x, w), ((xt @ wt[:, 0]) * (xt @ wt[:, 1])).numpy(), rtol=1e-12, atol=1e-12)
  # one group that owns every row of the fused gate-up ragged dot is the same thing
  np.testing.assert_allclose(O.ragged_dot_fused(x.reshape(10, 7), w.reshape(1, 7, 8), [10], gateup_activation="silu"),
                             want.numpy().reshape(10, 4), rtol=1e-12, atol=1e-12)


def test_row_movement_ops_against_loops():
  rng = np.random.default_rng(9)
  x = rng.normal(size=(6, 3)).astype(np.float32)
  idx = np.array([5, 0, 0, 3, 2, 4, 1, 1], np.int32)
  w = rng.normal(size=8).astype(np.float32)
  valid = np.array([1, 0, 1, 1, 1, 1, 0, 1], bool)
  assert np.array_equal(O.ragged_gather(x, idx), np.stack([x[i] for i in idx]))
  want = np.stack([x[i] if 1 <= i < 4 else np.zeros(3, np.float32) for i in idx])
  assert np.array_equal(O.ragged_scatter(x, idx, 1, 4), want)
  want = np.zeros((4, 3), np.float32)
  for g in range(8):
    if valid[g]:
      want[g // 2] += w[g] * x[idx[g]]
  np.testing.assert_allclose(O.ragged_gather_reduce(x, idx, w, valid, 2), want, rtol=1e-6, atol=1e-7)


def test_row_lookup_outside_the_array_wraps_then_clamps():
  """`x[indices]` in the reference is JAX indexing: -1 is the last row, and what is still outside is clamped."""
  x = np.arange(12, dtype=np.float32).reshape(4, 3)
  idx = np.array([-1, -4, -5, -100, 3, 4, 99, 0], np.int32)
  want = np.stack([x[3], x[0], x[0], x[0], x[3], x[3], x[3], x[0]])  # by hand
  assert np.array_equal(O.ragged_gather(x, idx), want)
  # the scatter mask tests the index as given: -1 lies outside [0, 4) although it reads the last row
  assert np.array_equal(O.ragged_scatter(x, idx, 0, 4), np.where(((idx >= 0) & (idx < 4))[:, None], want, 0))
  got = O.ragged_gather_reduce(x, idx, np.ones(8, np.float32), np.ones(8, bool), 2)
  assert np.array_equal(got, want.reshape(4, 2, 3).sum(1))


@pytest.mark.parametrize("gs,m,tile", [([300, 300, 300], 512, 128), ([5, 1000, 7], 256, 64), ([0, 2000], 130, 32),
                                        ([129, 129, 129, 129, 129, 129, 129, 129], 520, 128), ([4000], 8, 16)])
def test_group_sizes_beyond_m_keep_every_row_below_m_inside_the_task_slots(gs, m, tile):
  """Group sizes are unchecked device data (checkify is off by default, base.py:223): they may add up to more
  than m. The task arrays have tid_size = cdiv(m, tile) + G - 1 slots; the claim the kernels rely on is that
  every task that stores a row below m has an index below tid_size, so dropping the tasks past the slots and
  cutting the stored rows at m loses nothing below m and never indexes past the arrays."""
  G = len(gs)
  tid_size = -(-m // tile) + G - 1
  big = O.group_info_create_aligned(np.array(gs, np.int32), tile, 4 * (sum(gs) // tile + G + 1), 8)
  nt = big["num_tasks"]
  assert nt > tid_size or sum(gs) <= m + tile * G  # (the cases are meant to overflow the slots)
  covered = np.zeros(m, bool)
  for t in range(nt):
    lo, hi = int(big["actual_start"][t]), int(big["actual_end"][t])
    if lo < m:
      assert t < tid_size, (t, tid_size, lo)
      hi = min(hi, m)            # what the kernel stores after its clamp
      assert not covered[lo:hi].any()
      covered[lo:hi] = True
  assert covered[:min(m, sum(gs))].all()
  # the slots the kernel does read hold the same tasks as the unbounded schedule
  small = O.group_info_create_aligned(np.array(gs, np.int32), tile, tid_size, 8)
  for name in ("group_id", "block_start", "actual_start", "actual_end"):
    keep = min(nt, tid_size)
    assert np.array_equal(small[name][:keep], big[name][:keep])


def test_dequantize_is_tile_repeat():
  rng = np.random.default_rng(9)
  q = rng.integers(-127, 128, (2, 8, 6)).astype(np.int8)
  s = rng.uniform(0.5, 1.5, (2, 2, 6)).astype(np.float32)
  want = q.astype(np.float32) * np.repeat(s, 4, axis=1)  # ..._sm100_fp8_quant_test.py:229-232
  np.testing.assert_array_equal(O.dequantize(q, s), want)
  # scales constant along k commute with the contraction (the epilogue-scale identity)
  lhs = rng.normal(size=(5, 8))
  s1 = rng.uniform(0.5, 1.5, (2, 1, 6)).astype(np.float32)
  a = O.ragged_dot(lhs, O.dequantize(q, s1), [3, 2], acc_dtype=np.float64, out_dtype="f64")
  b = O.ragged_dot(lhs, q.astype(np.float64), [3, 2], acc_dtype=np.float64, out_dtype="f64")
  b[:3] *= s1[0, 0]
  b[3:] *= s1[1, 0]
  np.testing.assert_allclose(a, b, rtol=2e-6)  # dequantize rounds q*s to f32


def test_golden_fixtures_match_oracle():
  z = np.load(os.path.join(GOLDEN, "ragged_dot_small.npz"))
  gs = z["gs"]
  f = lambda *a, **kw: O.ragged_dot(*a, acc_dtype=np.float64, out_dtype="f64", **kw)
  np.testing.assert_allclose(f(z["lhs"], z["rhs"], gs), z["fwd"], rtol=1e-12, atol=1e-12)
  np.testing.assert_allclose(f(z["dout"], z["rhs"], gs, mode=O.TRANS_RHS), z["dlhs"], rtol=1e-12, atol=1e-12)
  np.testing.assert_allclose(f(z["lhs"], z["dout"], gs, mode=O.RAGGED_CONTRACTING), z["drhs"], rtol=1e-12, atol=1e-12)
  np.testing.assert_allclose(f(z["lhs"], O.dequantize(z["q8"], z["q8_scale"]), gs), z["fwd_q8"], rtol=1e-12, atol=1e-12)
  # the brute-force loops agree with the stored vectors too (small enough to run here)
  np.testing.assert_allclose(O.ragged_dot_bruteforce(z["lhs"][:40], z["rhs"], [23, 0, 17, 0]), z["fwd"][:40], rtol=1e-10, atol=1e-10)


# ---- absmax quantisation (AsQArray.as_qarray) -----------------------------------------------------
@pytest.mark.parametrize("qtype", ["int8", "int4", "fp8"])
@pytest.mark.parametrize("shape,tile", [((6, 32), (1, 8)), ((6, 32), (1, 32)), ((8, 16), (4, 1)), ((8, 16), (8, 8)),
                                        ((2, 8, 16), (1, 8, 1)), ((2, 8, 16), (1, 4, 8))])
def test_quantize_absmax_properties(qtype, shape, tile):
  """What the definition fixes: the largest entry of every tile maps to +-qmax, no entry lies further than half a
  quantisation step from its dequantised value, an all-zero tile gets scale 1, scale shapes are shape / tile."""
  rng = np.random.default_rng(sum(shape) + sum(tile))
  x = rng.normal(0, 3, shape).astype(np.float32)
  x[(0,) * len(shape)] = 0.0
  q, scale = O.quantize_absmax(x, qtype, tile)
  qmax = O.QMAX[qtype]
  assert scale.shape == tuple(d // t for d, t in zip(shape, tile)) and scale.dtype == np.float32
  qf = O.e4m3fn_decode(q) if qtype == "fp8" else q.astype(np.float32)
  split = []
  for d, t in zip(shape, tile):
    split += [d // t, t]
  inner = tuple(range(1, 2 * len(shape), 2))
  assert np.all(np.abs(qf).reshape(split).max(axis=inner) == qmax)
  absmax = np.abs(x).reshape(split).max(axis=inner)
  np.testing.assert_allclose(scale, absmax / np.float32(qmax), rtol=1e-6)
  back = O.dequantize(qf, scale)
  full = O.dequantize(np.ones(shape, np.float32), scale)
  if qtype == "fp8":  # e4m3: 3 mantissa bits -> relative step 2^-3, half of it plus the subnormal floor
    assert np.all(np.abs(back - x) <= np.maximum(np.abs(x) * 2.0 ** -4, full * 2.0 ** -10) * 1.0001)
  else:
    assert np.all(np.abs(back - x) <= full * 0.5 * 1.0001)
  z, zs = O.quantize_absmax(np.zeros(shape, np.float32), qtype, tile)
  assert np.all(zs == 1) and np.all(z == 0)


def test_quantize_absmax_exact_cases():
  # powers of two: absmax = 127 / 4 -> scale = 1/4 exactly, every multiple of 1/4 is its own code
  x = np.array([[31.75, -0.25, 0.5, 10.0, -31.75, 0.0, 1.25, -7.5]], np.float32)
  q, s = O.quantize_absmax(x, "int8", (1, 8))
  assert s[0, 0] == 0.25 and q.tolist() == [[127, -1, 2, 40, -127, 0, 5, -30]]
  # ties go to the even code: with scale 1, x.5 rounds to the even neighbour
  x = np.array([[127.0, 0.5, 1.5, 2.5, -0.5, -1.5, -2.5, 3.49]], np.float32)
  q, s = O.quantize_absmax(x, "int8", (1, 8))
  assert s[0, 0] == 1.0 and q.tolist() == [[127, 0, 2, 2, 0, -2, -2, 3]]
  # int4: qmax 7
  q, s = O.quantize_absmax(np.array([[3.5, -1.0, 0.24, 0.26]], np.float32), "int4", (1, 4))
  assert s[0, 0] == 0.5 and q.tolist() == [[7, -2, 0, 1]]
  # fp8: x / scale rounded the way torch casts to float8_e4m3fn (library routine), for every tile
  rng = np.random.default_rng(1)
  x = rng.normal(0, 1, (16, 64)).astype(np.float32)
  q, s = O.quantize_absmax(x, "fp8", (1, 16))
  want = (torch.tensor(x) / torch.tensor(np.repeat(s, 16, axis=1))).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
  assert np.array_equal(q, want)
  # the per-column form: a tile (k, 1) of weights [k, n] gives one scale per column
  w = rng.normal(0, 1, (8, 4)).astype(np.float32)
  q, s = O.quantize_absmax(w, "int8", (8, 1))
  assert s.shape == (1, 4) and np.allclose(s[0], np.abs(w).max(axis=0) / 127)
  for c in range(4):
    assert np.array_equal(q[:, c], np.rint(w[:, c] / s[0, c]).astype(np.int8))


def test_quantize_absmax_with_the_half_step_bound_by_hand():
  """bound = qmax + 0.5 (the convention of symmetric integer quantisers that use the type's whole range): the scale is
  absmax / 127.5, the extreme value rounds to an end of [-128, 127], everything else follows from the scale."""
  x = np.array([[-127.5, 127.5, 63.75, 0.4, -0.6, 1.5, 2.5, 0.0]], np.float32)
  q, s = O.quantize_absmax(x, "int8", (1, 8), bound=127.5)
  assert s[0, 0] == 1.0 and q.tolist() == [[-128, 127, 64, 0, -1, 2, 2, 0]]  # -127.5 -> -128 (even), +127.5 -> 128 -> clipped
  q, s = O.quantize_absmax(np.array([[3.75, -3.75, 0.25, -1.0]], np.float32), "int4", (1, 4), bound=7.5)
  assert s[0, 0] == 0.5 and q.tolist() == [[7, -8, 0, -2]]
  # the default bound is qmax: nothing below -qmax
  q, s = O.quantize_absmax(x, "int8", (1, 8))
  assert s[0, 0] == np.float32(127.5) / np.float32(127) and q.min() == -127


def test_quantize_absmax_reciprocal_form():
  """`reciprocal=True` (the reference's fused output quantisation, acc * (1.0 / out_scale)): the same scales, values
  equal to torch's own float8 cast of x * (1 / scale) in f32, and within one code of the dividing form."""
  rng = np.random.default_rng(5)
  x = rng.normal(0, 3, (32, 256)).astype(np.float32)
  q_div, s_div = O.quantize_absmax(x, "fp8", (1, 128))
  q_rcp, s_rcp = O.quantize_absmax(x, "fp8", (1, 128), reciprocal=True)
  assert np.array_equal(s_div, s_rcp)
  inv = (torch.tensor(1.0) / torch.tensor(np.repeat(s_rcp, 128, axis=1)))
  want = (torch.tensor(x) * inv).clamp(-448, 448).to(torch.float8_e4m3fn).view(torch.uint8).numpy()
  assert np.array_equal(q_rcp, want)
  diff = np.abs(q_div.astype(np.int16) - q_rcp.astype(np.int16))
  assert diff.max() <= 1 and (diff != 0).mean() < 0.01
  # 1 / 3 is not a float: 3 * fl(1 / 3) rounds to 1 here, but a quotient on a boundary can land on its other side
  one = O.quantize_absmax(np.array([[1344.0, 3.0] + [0.0] * 6], np.float32), "fp8", (1, 8), reciprocal=True)
  assert one[1][0, 0] == 3.0 and O.e4m3fn_decode(one[0])[0, :2].tolist() == [448.0, 1.0]


def test_dequantize_zero_point_by_hand():
  q = np.array([[10, -3, 0, 7]], np.int8)
  got = O.dequantize_zero_point(q, np.array([[0.5, 2.0]], np.float32), np.array([[2.0, -1.0]], np.float32))
  assert got.tolist() == [[4.0, -2.5, 2.0, 16.0]]  # (10 - 2) / 2, (-3 - 2) / 2, (0 + 1) * 2, (7 + 1) * 2


def test_int4_packing_by_hand():
  """All 16 values in the low and in the high half of a byte, written out by hand: -8..-1 are 0x8..0xF, 0..7 are 0x0..0x7;
  the even entry of a pair sits in bits 0-3."""
  values = np.arange(-8, 8)
  low = np.stack([values, np.zeros(16, int)], 0).T.reshape(32, 1)    # pairs (v, 0): byte = v's nibble
  high = np.stack([np.zeros(16, int), values], 0).T.reshape(32, 1)   # pairs (0, v): byte = v's nibble << 4
  nibbles = np.array([8, 9, 10, 11, 12, 13, 14, 15, 0, 1, 2, 3, 4, 5, 6, 7])
  assert O.pack_int4(low)[:, 0].tolist() == nibbles.tolist()
  assert O.pack_int4(high)[:, 0].tolist() == (nibbles * 16).tolist()
  assert O.pack_int4(np.array([[-8], [7]])).tolist() == [[0x78]]
  assert O.pack_int4(np.array([[1], [-1]])).tolist() == [[0xF1]]
  assert O.unpack_int4(np.array([[0x78, 0xF1]], np.uint8)).tolist() == [[-8, 1], [7, -1]]
  rng = np.random.default_rng(0)
  q = rng.integers(-8, 8, (3, 10, 16)).astype(np.int8)
  packed = O.pack_int4(q)
  assert packed.shape == (3, 5, 16) and packed.dtype == np.uint8
  assert np.array_equal(O.unpack_int4(packed), q)
