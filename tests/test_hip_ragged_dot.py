"""GPU parity tests: the HIP path (through the C ABI) against the CPU oracle.

Case list and tolerances follow the reference's shared suite
(tokamax/_src/ops/ragged_dot/test_base.py:97-344) and scheduler test
(pallas_mosaic_gpu_common_test.py:27-84). Bars: offsets and tile schedule bit-exact; relative L2
error vs an f32/f64-accumulated reference <= 1e-5 (f32), <= 2e-3 (bf16/f16), <= 3e-2 (fp8, int8-dequant).
"""

import dataclasses
import itertools
import json
import os

import numpy as np
import pytest
import torch

import tokamax_amd
from oracle import ragged_dot_oracle as O
from tokamax_amd import _lib
from tokamax_amd.ragged_dot import base, hip, hip_ops, workloads

pytestmark = pytest.mark.gpu

GOLDEN = os.path.join(os.path.dirname(__file__), "golden")
TOL = {torch.float32: 1e-5, torch.bfloat16: 2e-3, torch.float16: 2e-3, "fp8": 3e-2, "int8": 3e-2}
OP = hip.HipRaggedDot()


def _np(x):
  return x.detach().float().cpu().numpy()


def _inputs(name, G, m, k, n, dtype, device, random_groups=False, std=0.1):
  """Same recipe as test_base.py:108-150: rng seeded by the test name, N(0, std^2) cast to dtype."""
  rng = np.random.default_rng(sum(name.encode()))
  a = torch.tensor(rng.normal(0.0, std, (m, k)).astype(np.float32)).to(dtype).to(device)
  b = torch.tensor(rng.normal(0.0, std, (G, k, n)).astype(np.float32)).to(dtype).to(device)
  if random_groups:
    gs = rng.integers(0, m // G, (G,)).astype(np.int32)
  else:
    gs = np.array([m // G] * G, np.int32)
  return a, b, gs


def _ref(a, b, gs, mode=O.DEFAULT):
  return O.ragged_dot(_np(a), _np(b), gs, mode, acc_dtype=np.float64, out_dtype="f64")


def _check(actual, expected, tol, rows=None):
  a, e = _np(actual), np.asarray(expected)
  if rows is not None:
    a, e = a[:rows], e[:rows]
  err = O.rel_l2(a, e)
  assert err <= tol, f"rel_l2 {err:.3e} > {tol}"


def _check_spans(ws, m, G, block_m, width, gs):
  """Launch-order spans: consecutive tasks of one group, at most `width` wide, as even as possible."""
  lib = _lib.load()
  tid = lib.tkx_ragged_dot_tid_size(m, G, block_m)
  arr = lambda which: ws[lib.tkx_ragged_dot_workspace_offset(m, G, block_m, which):][:tid].cpu().numpy()
  num_tasks = int(ws[0].item())
  gid, first, wid = arr(3)[:num_tasks], arr(9)[:num_tasks], arr(10)[:num_tasks]
  assert num_tasks == O.group_info_create_aligned(gs, block_m, tid, 8)["num_tasks"]
  t = 0
  while t < num_tasks:
    w = int(wid[t])
    assert 1 <= w <= width and int(first[t]) == t and t + w <= num_tasks
    assert (first[t:t + w] == t).all() and (wid[t:t + w] == w).all() and (gid[t:t + w] == gid[t]).all()
    t += w
  for g in np.unique(gid):
    tasks = int((gid == g).sum())
    widths = wid[gid == g]
    assert len(np.unique(first[gid == g])) == -(-tasks // width) and widths.max() - widths.min() <= 1


# ---- part (1): offsets and tile schedule, bit exact ----------------------------------------------
with open(os.path.join(GOLDEN, "scheduler_kat.json")) as _f:
  KAT = json.load(_f)


@pytest.mark.parametrize("case", KAT, ids=[c["name"] for c in KAT])
def test_schedule_known_answers(case, device):
  gs = torch.tensor(case["group_sizes"], dtype=torch.int32, device=device)
  m = sum(case["group_sizes"])
  lib = _lib.load()
  # the C ABI derives tid_size = cdiv(m, tile) + G - 1; compare on the common prefix
  got = hip_ops.schedule(gs, m, case["tile"], case["align_tile"])
  tid = min(case["tid_size"], got["group_id"].numel())
  want = O.group_info_create_aligned(case["group_sizes"], case["tile"], got["group_id"].numel(), case["align_tile"])
  for f in hip_ops.SCHEDULE_FIELDS:
    np.testing.assert_array_equal(got[f].cpu().numpy()[:tid], np.array(case[f], np.int32)[:tid], err_msg=f)
    np.testing.assert_array_equal(got[f].cpu().numpy(), want[f], err_msg=f)
  assert lib.tkx_ragged_dot_tid_size(m, len(case["group_sizes"]), case["tile"]) == got["group_id"].numel()


@pytest.mark.parametrize("seed", range(8))
def test_schedule_random_bit_exact(seed, device):
  rng = np.random.default_rng(seed)
  G = int(rng.choice([1, 2, 7, 8, 64, 128, 256, 300, 1000]))
  gs = rng.integers(0, 400, G).astype(np.int32)
  gs[rng.random(G) < 0.3] = 0
  if seed % 2:
    gs[rng.integers(0, G)] = -3  # negative sizes are clamped to zero
  tile = int(rng.choice([8, 16, 32, 64, 128, 256]))
  m = int(np.maximum(gs, 0).sum()) + int(rng.integers(0, 300))
  got = hip_ops.schedule(torch.tensor(gs, device=device), max(m, 1), tile, 8)
  want = O.group_info_create_aligned(gs, tile, got["group_id"].numel(), 8)
  for f in hip_ops.SCHEDULE_FIELDS:
    np.testing.assert_array_equal(got[f].cpu().numpy(), want[f], err_msg=f)
  np.testing.assert_array_equal(got["group_offsets"].cpu().numpy(), O.group_offsets(gs))
  assert int(got["num_tasks"].item()) == want["num_tasks"]
  assert int(got["total_rows"].item()) == int(np.maximum(gs, 0).sum())


@pytest.mark.parametrize("name,block_m", [("mixtral", 256), ("deepseek", 128), ("decode", 32)])
def test_schedule_of_benchmark_group_sizes(name, block_m, device):
  gs = {"mixtral": lambda: workloads.router_top2_group_sizes(8192, 8, 0),
        "deepseek": lambda: workloads.zipf_group_sizes(65536, 256, 0),
        "decode": lambda: workloads.decode_group_sizes(32, 8, 128, 0)}[name]()
  m = int(gs.sum())
  got = hip_ops.schedule(torch.tensor(gs, device=device), m, block_m, 8)
  want = O.group_info_create_aligned(gs, block_m, got["group_id"].numel(), 8)
  for f in hip_ops.SCHEDULE_FIELDS:
    np.testing.assert_array_equal(got[f].cpu().numpy(), want[f], err_msg=f)
  if name == "deepseek":
    assert (gs == 0).sum() >= 10  # empty experts produce no task
    assert set(got["group_id"].cpu().numpy()[:want["num_tasks"]].tolist()) == set(np.nonzero(gs)[0].tolist())


# ---- the reference's shared suite -----------------------------------------------------------------
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_simple(dtype, device):
  a, b, gs = _inputs("test_simple", 8, 1024, 128, 256, dtype, device)
  # uint32 group sizes are legal input (test_base.py:137)
  out = tokamax_amd.ragged_dot(a, b, torch.tensor(gs.astype(np.uint32), device=device), preferred_element_type=torch.float32)
  assert out.dtype == torch.float32
  _check(out, _ref(a, b, gs), TOL[dtype])


@pytest.mark.parametrize("width", [1, 3, 8, 16])
def test_launch_order_spans(width, device):
  rng = np.random.default_rng(width)
  G, m, k, n = 9, 2048, 128, 256
  gs = np.array([300, 0, 129, 1, 640, 0, 7, 512, 130], np.int32)
  a = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  b = torch.tensor(rng.normal(0, 0.1, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
  for block_m, cfg in ((128, hip_ops.KernelConfig(128, 128, 64, 2, 2, 2, grid_tile_width=width)),
                       (32, hip_ops.KernelConfig(32, 128, 64, 1, 4, 4, grid_tile_width=width))):
    got_ws = []
    out = hip_ops.ragged_dot_fwd(a, b, torch.tensor(gs, device=device), config=cfg, out_dtype=torch.float32,
                                 workspace_out=got_ws)
    _check_spans(got_ws[0], m, G, block_m, width, gs)
    _check(out, _ref(a, b, gs), 1e-5)


def test_padded(device):
  a, b, gs = _inputs("test_padded", 8, 1024, 128, 256, torch.bfloat16, device, random_groups=True)
  out = tokamax_amd.ragged_dot(a, b, torch.tensor(gs, device=device), preferred_element_type=torch.float32)
  count = int(gs.sum())
  _check(out, _ref(a, b, gs), TOL[torch.bfloat16], rows=count)
  assert torch.count_nonzero(out[count:]) == 0  # rows past sum(group_sizes) are zero, as in the XLA path


def test_zero_group_sizes(device):
  a, b, gs = _inputs("test_zero_group_sizes", 8, 1024, 128, 256, torch.bfloat16, device, random_groups=True)
  for i in range(2 ** 8):  # every zero / non-zero pattern (test_base.py:172-185)
    mask = np.unpackbits(np.uint8(i)).astype(bool)
    gs_ = np.where(mask, gs, 0).astype(np.int32)
    out = tokamax_amd.ragged_dot(a, b, torch.tensor(gs_, device=device), preferred_element_type=torch.float32)
    count = int(gs_.sum())
    err = O.rel_l2(_np(out), _ref(a, b, gs_))
    assert err <= TOL[torch.bfloat16], (gs_.tolist(), err)
    assert torch.count_nonzero(out[count:]) == 0, gs_.tolist()


@pytest.mark.parametrize("out_type", [None, torch.bfloat16, torch.float32])
def test_preferred_element_type(out_type, device):
  a, b, gs = _inputs("test_preferred_element_type", 8, 1024, 128, 256, torch.bfloat16, device)
  out = tokamax_amd.ragged_dot(a, b, torch.tensor(gs, device=device), preferred_element_type=out_type)
  assert out.dtype == (out_type or torch.bfloat16)
  want = O.ragged_dot(_np(a), _np(b), gs, acc_dtype=np.float32, out_dtype="bf16" if out.dtype == torch.bfloat16 else "f32")
  _check(out, want, 2e-3)
  if out.dtype == torch.bfloat16:
    # one rounding of an f32 accumulator: at most 1 bf16 ulp from the oracle's rounding
    ulp = np.abs(_np(out) - want) / np.maximum(np.abs(want), 1e-30)
    assert float(np.quantile(ulp, 0.999)) <= 2 ** -7


def test_group_sizes_wrapper(device):
  a, b, gs = _inputs("test_group_sizes", 8, 1024, 128, 256, torch.bfloat16, device)
  wrapped = base.GroupSizes(torch.tensor(gs, device=device), (1,) * 8)
  out = tokamax_amd.ragged_dot(a, b, wrapped, preferred_element_type=torch.float32)
  _check(out, _ref(a, b, gs), TOL[torch.bfloat16])


@pytest.mark.parametrize("activation", [None, torch.relu, torch.tanh, torch.nn.functional.silu, torch.sigmoid])
def test_activation(activation, device):
  a, b, gs = _inputs("test_activation", 8, 512, 128, 256, torch.bfloat16, device, std=0.3)
  out = tokamax_amd.ragged_dot(a, b, torch.tensor(gs, device=device), preferred_element_type=torch.float32, activation=activation)
  want = torch.tensor(_ref(a, b, gs))
  if activation is not None:
    want = activation(want)
  _check(out, want.numpy(), 2e-3)


@pytest.mark.parametrize("m,k,n", list(itertools.product((1024, 128), (128, 64), (256, 128))))
@pytest.mark.parametrize("activation", [None, torch.relu, torch.tanh])
def test_vjp(m, k, n, activation, device):
  """test_base.py:259-293: bf16 inputs, f32 reference, grads within atol=0.02, rtol=0.005."""
  G = 8
  a, b, gs = _inputs("test_vjp", G, m, k, n, torch.bfloat16, device)
  gst = torch.tensor(gs, device=device)
  a_ref = a.detach().float().cpu().double().requires_grad_(True)
  b_ref = b.detach().float().cpu().double().requires_grad_(True)
  off = O.group_offsets(gs)
  ref_out = torch.cat([a_ref[int(off[g]):int(off[g + 1])] @ b_ref[g] for g in range(G)])
  if activation is not None:
    ref_out = activation(ref_out)
  a_t = a.clone().requires_grad_(True)
  b_t = b.clone().requires_grad_(True)
  out = tokamax_amd.ragged_dot(a_t, b_t, gst, precision="BF16_BF16_F32", preferred_element_type=torch.float32,
                               activation=activation)
  np.testing.assert_allclose(_np(out), ref_out.detach().numpy(), atol=1e-5 + 2e-3 * float(ref_out.detach().abs().max()))
  dout = (ref_out.detach() - ref_out.detach().mean()) / ref_out.detach().std()
  dout = dout.to(torch.bfloat16).double()  # bottleneck the precision as the reference's test does
  ref_out.backward(dout)
  out.backward(dout.float().to(device))
  assert a_t.grad.dtype == torch.bfloat16 and b_t.grad.dtype == torch.bfloat16
  np.testing.assert_allclose(_np(a_t.grad), a_ref.grad.numpy(), atol=0.02, rtol=0.005)
  np.testing.assert_allclose(_np(b_t.grad), b_ref.grad.numpy(), atol=0.02, rtol=0.005)
  assert O.rel_l2(_np(a_t.grad), a_ref.grad.numpy()) <= 4e-3  # bf16 dout . bf16 rhs, rounded to bf16
  assert O.rel_l2(_np(b_t.grad), b_ref.grad.numpy()) <= 4e-3


@pytest.mark.parametrize("b_tile_shape,supported", [((1, 256, 1), True), ((1, 16, 1), True), ((1, 1, 16), True),
                                                    ((1, 64, 32), True), ((1, 1, 8), True), ((2, 256, 1), True),
                                                    ((4, 64, 128), True), ((3, 1, 1), False)])
def test_quantized_int8_weights(b_tile_shape, supported, device):
  """bf16 x int8: per-(group, column) scales run in the kernels' epilogue, sub-channel scales along k and
  scale tiles along n are repeated over their columns first, scales shared by runs of groups over those groups; a
  tile that does not divide the array is declined."""
  G, m, k, n = 8, 512, 256, 512
  a, _, gs = _inputs("test_quantized", G, m, k, n, torch.bfloat16, device, random_groups=True)
  rng = np.random.default_rng(11)
  q = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
  sshape = tuple(-(-d // t) for d, t in zip((G, k, n), b_tile_shape))
  scale = torch.tensor((rng.uniform(0.5, 1.5, sshape) / 127 * 0.1).astype(np.float32), device=device)
  rhs = tokamax_amd.QArray(q, scale)
  gst = torch.tensor(gs, device=device)
  if not supported:
    with pytest.raises(NotImplementedError):
      tokamax_amd.ragged_dot(a, rhs, gst)
    return
  for act in (None, torch.relu, torch.tanh):
    out = tokamax_amd.ragged_dot(a, rhs, gst, activation=act, preferred_element_type=torch.float32)
    want = torch.tensor(O.ragged_dot(_np(a), O.dequantize(q.cpu().numpy(), _np(scale)), gs, acc_dtype=np.float64, out_dtype="f64"))
    want = act(want) if act is not None else want
    count = int(gs.sum())
    _check(out, want.numpy(), TOL["int8"], rows=count)
    np.testing.assert_allclose(_np(out)[:count], want.numpy()[:count], atol=0.01, rtol=0.005)  # test_base.py:240-242
  # An `AsQArray` without tiling: one scale for the whole tensor (quantised on the device, then repeated per column).
  w = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
  out = tokamax_amd.ragged_dot(a, tokamax_amd.AsQArray(w, torch.int8), gst, preferred_element_type=torch.float32)
  wq, ws = O.quantize_absmax(_np(w), "int8", (G, k, n))
  assert ws.shape == (1, 1, 1)
  want = O.ragged_dot(_np(a), O.dequantize(wq, ws), gs, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, TOL["int8"], rows=int(gs.sum()))
  with pytest.raises(NotImplementedError):  # a tile over several groups that does not span their contraction
    hip_ops.quantize(w, torch.int8, (2, 16, 1))


def test_fp8_with_row_and_column_scales(device):
  G, m, k, n = 8, 512, 256, 512
  rng = np.random.default_rng(12)
  x = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device)
  w = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device)
  xs, ws = x.abs().amax(1, keepdim=True) / 448, w.abs().amax(1, keepdim=True) / 448
  xq, wq = (x / xs).to(torch.float8_e4m3fn), (w / ws).to(torch.float8_e4m3fn)
  gs = np.array([33, 67, 50, 80, 70, 60, 90, 62], np.int32)
  out = tokamax_amd.ragged_dot(tokamax_amd.QArray(xq, xs), tokamax_amd.QArray(wq, ws), torch.tensor(gs, device=device),
                               preferred_element_type=torch.bfloat16)
  assert out.dtype == torch.bfloat16
  # against the same quantised values (kernel arithmetic) ...
  want_q = O.ragged_dot(O.dequantize(O.e4m3fn_decode(xq.view(torch.uint8).cpu().numpy()), _np(xs)),
                        O.dequantize(O.e4m3fn_decode(wq.view(torch.uint8).cpu().numpy()), _np(ws)), gs,
                        acc_dtype=np.float64, out_dtype="f64")
  _check(out, want_q, 2e-3)
  _check(out, want_q, TOL["fp8"])
  # ... and, for scale, against the unquantised problem: two e4m3 operands (3 mantissa bits each)
  # put about 2^-4.7 of relative noise on every product, which no kernel can remove
  _check(out, O.ragged_dot(_np(x), _np(w), gs, acc_dtype=np.float64, out_dtype="f64"), 6e-2)


@pytest.mark.parametrize("group_sizes", [(33, 67, 50, 80, 70, 60, 90, 62), (1, 7, 199, 1, 100, 50, 151, 3),
                                         (0, 130, 0, 200, 0, 98, 84, 0)])
@pytest.mark.parametrize("block_m", [32, 64, 128, 256])
def test_straddling_groups(group_sizes, block_m, device):
  """..._sm100_fp8_quant_test.py:313-331: tiles that straddle two groups; no write outside a task's rows."""
  G, m, k, n = 8, 512, 128, 256
  a, b, _ = _inputs("test_straddling", G, m, k, n, torch.bfloat16, device)
  gs = np.array(group_sizes, np.int32)
  table = hip._variant_table()[(0, _lib.TKX_BF16, _lib.TKX_BF16)]
  bm, bn, bk, wm, wn, ns = next(v for v in table if v[0] == block_m)
  op = hip.HipRaggedDot(config=hip.Config(bm, bn, bk, wm, wn, ns, grid_tile_width=2))
  out = op(a, b, group_sizes=torch.tensor(gs, device=device), preferred_element_type=torch.float32)
  _check(out, _ref(a, b, gs), TOL[torch.bfloat16])
  again = op(a, b, group_sizes=torch.tensor(gs, device=device), preferred_element_type=torch.float32)
  assert torch.equal(out, again)  # run-twice bit equality (..._fp8_quant_test.py:274-280)


def test_golden_fixtures(device):
  z = np.load(os.path.join(GOLDEN, "ragged_dot_small.npz"))
  gs = torch.tensor(z["gs"], device=device)
  bf = lambda x: torch.tensor(x).to(torch.bfloat16).to(device)
  lhs, rhs, dout = bf(z["lhs"]), bf(z["rhs"]), bf(z["dout"])
  f32 = torch.float32
  _check(tokamax_amd.ragged_dot(lhs, rhs, gs, preferred_element_type=f32), z["fwd"], 1e-5)
  _check(tokamax_amd.ragged_dot_general(dout, rhs, gs, base.TRANS_RHS_RAGGED_DOT_DIM_NUMS, preferred_element_type=f32), z["dlhs"], 1e-5)
  _check(tokamax_amd.ragged_dot_general(lhs, dout, gs, base.RAGGED_CONTRACTING_DOT_DIM_NUMS, preferred_element_type=f32), z["drhs"], 1e-5)
  q8 = tokamax_amd.QArray(torch.tensor(z["q8"], device=device), torch.tensor(z["q8_scale"], device=device))
  _check(tokamax_amd.ragged_dot(lhs, q8, gs, preferred_element_type=f32), z["fwd_q8"], 1e-5)
  x8 = tokamax_amd.QArray(torch.tensor(z["x8"], device=device).view(torch.float8_e4m3fn), torch.tensor(z["x8_scale"], device=device))
  w8 = tokamax_amd.QArray(torch.tensor(z["w8"], device=device).view(torch.float8_e4m3fn), torch.tensor(z["w8_scale"], device=device))
  _check(tokamax_amd.ragged_dot(x8, w8, gs, preferred_element_type=f32), z["fwd_f8"], 1e-4)


def _variant_cases():
  cases = []
  for kind in (0, 1):
    for v in _lib.variants(kind):
      cases.append(pytest.param(v, id="mode{mode}-d{lhs_dtype}x{rhs_dtype}-{block_m}x{block_n}x{block_k}-w{waves_m}x{waves_n}-s{num_stages}".format(**v)))
  return cases


_TORCH_DTYPE = {_lib.TKX_F32: torch.float32, _lib.TKX_BF16: torch.bfloat16, _lib.TKX_F16: torch.float16,
                _lib.TKX_F8E4M3FN: torch.float8_e4m3fn, _lib.TKX_I8: torch.int8, _lib.TKX_I4X2: torch.uint8}


@pytest.mark.parametrize("v", _variant_cases())
def test_every_kernel_variant_through_c_abi(v, device):
  """Each compiled tile shape, called through the C ABI, on ragged groups with an empty one and a tail."""
  rng = np.random.default_rng(v["block_m"] * 7 + v["block_n"] + v["mode"])
  G, m, k, n = 6, 640, 256, 384
  if v["block_m"] == 16:
    k = 1024  # the streaming small-m kernel splits k over 4 waves x 8 steps of 32
  gs = np.array([100, 0, 257, 9, 130, 80], np.int32)  # sum 576 < m
  gst = torch.tensor(gs, device=device)
  cfg = hip_ops.KernelConfig(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"],
                             grid_tile_width=3)
  lt, rt = _TORCH_DTYPE[v["lhs_dtype"]], _TORCH_DTYPE[v["rhs_dtype"]]
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device)
  if v["mode"] == 3:  # forward with gate-up fusion and a bias: rhs [g, k, 2 n'] -> out [m, n']
    lhs = mk((m, k), 1.0).to(lt)
    bias = mk((G, 1, n), 0.5)
    scale = lhs_scale = None
    lhs_f = _np(lhs)
    if lt == torch.float8_e4m3fn:  # (over packed int4 weights) one scale per row
      lhs_scale = mk((m, 1), 0.1).abs() + 0.05
      lhs_f = lhs_f * _np(lhs_scale)
    if lt == torch.int8:  # (likewise)
      lhs = torch.tensor(rng.integers(-127, 128, (m, k)).astype(np.int8), device=device)
      lhs_scale = mk((m, 1), 0.01).abs() + 0.005
      lhs_f = _np(lhs) * _np(lhs_scale)
    if rt == torch.int8:  # int8 weights with one scale per (group, column)
      rhs = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
      scale = mk((G, 1, n), 0.005).abs() + 1e-3
      rhs_f = O.dequantize(rhs.cpu().numpy(), _np(scale))
    elif rt == torch.uint8:  # int4 weights, two to a byte along k
      values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
      rhs = torch.tensor(O.pack_int4(values), device=device)
      scale = mk((G, 1, n), 0.05).abs() + 1e-2
      rhs_f = O.dequantize(values, _np(scale))
    else:
      rhs = mk((G, k, n), k ** -0.5).to(rt)
      rhs_f = _np(rhs)
    out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, rhs_bias=bias, activation="silu",
                                 gateup=True, rhs_scale=scale, lhs_scale=lhs_scale)
    want = O.ragged_dot_fused(lhs_f, rhs_f, gs, rhs_bias=_np(bias), gateup_activation="silu")
    _check(out, want, 1e-5 if lhs_scale is None else 1e-4)
    assert out.shape == (m, n // 2) and torch.count_nonzero(out[int(gs.sum()):]) == 0
    return
  if v["mode"] == 4 and lt == torch.float8_e4m3fn:  # fp8 x fp8, scales per block of 128 k rows on both sides, a bias
    lhs = mk((m, k), 1.0).to(lt)
    if rt == torch.uint8:  # ... or fp8 over int4 weights, two to a byte along k
      rhs_values = rng.integers(-8, 8, (G, k, n)).astype(np.float64)
      rhs = torch.tensor(O.pack_int4(rhs_values.astype(np.int8)), device=device)
    else:
      rhs = mk((G, k, n), 1.0).to(rt)
      rhs_values = O.e4m3fn_decode(rhs.view(torch.uint8).cpu().numpy()).astype(np.float64)
    xs, ws_ = mk((m, 2), 0.1).abs() + 0.05, mk((G, 2, n), 0.1).abs() + 0.05
    bias = mk((G, 1, n), 0.5)
    out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, lhs_scale=xs, rhs_scale=ws_, rhs_bias=bias)
    lhs_f = O.dequantize(O.e4m3fn_decode(lhs.view(torch.uint8).cpu().numpy()).astype(np.float64), _np(xs))
    rhs_f = O.dequantize(rhs_values, _np(ws_))
    _check(out, O.ragged_dot_fused(lhs_f, rhs_f, gs, rhs_bias=_np(bias)), 1e-4)
    assert torch.count_nonzero(out[int(gs.sum()):]) == 0
    return
  if v["mode"] == 4 and lt == torch.int8:  # int8 x int8 on the int8 MFMAs, scales per block of 64 k rows on both sides
    lhs = torch.tensor(rng.integers(-127, 128, (m, k)).astype(np.int8), device=device)
    rhs = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
    if rt == torch.uint8:  # ... or int8 over int4 weights, two to a byte along k
      rhs = torch.tensor(rng.integers(-8, 8, (G, k, n)).astype(np.int8), device=device)
    for blocks in (k // v["block_k"],):  # scale blocks of one k-step (128 or 64 rows); one block runs the mode-0 variants
      xs, ws_ = mk((m, blocks), 0.01).abs() + 0.005, mk((G, blocks, n), 0.01).abs() + 0.005
      bias = mk((G, 1, n), 0.5)
      stored = hip_ops.pack_int4(rhs) if rt == torch.uint8 else rhs
      out = hip_ops.ragged_dot_fwd(lhs, stored, gst, config=cfg, out_dtype=torch.float32, lhs_scale=xs, rhs_scale=ws_, rhs_bias=bias)
      lhs_f = O.dequantize(lhs.cpu().numpy().astype(np.float64), _np(xs))
      rhs_f = O.dequantize(rhs.cpu().numpy().astype(np.float64), _np(ws_))
      _check(out, O.ragged_dot_fused(lhs_f, rhs_f, gs, rhs_bias=_np(bias)), 1e-5)  # int32 sums are exact
      assert torch.count_nonzero(out[int(gs.sum()):]) == 0
    return
  if v["mode"] == 4:  # forward over int8 / fp8 weights with per-k-block scales (4 blocks of 64 rows) and a bias
    lhs = mk((m, k), 1.0).to(lt)
    if rt == torch.int8:
      rhs = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
      rhs_values = rhs.cpu().numpy()
    elif rt == torch.uint8:  # int4 weights, two to a byte along k
      rhs_values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
      rhs = torch.tensor(O.pack_int4(rhs_values), device=device)
    else:
      rhs = mk((G, k, n), 1.0).to(rt)
      rhs_values = O.e4m3fn_decode(rhs.view(torch.uint8).cpu().numpy())
    scale = mk((G, 4, n), 0.01).abs() + 1e-3
    bias = mk((G, 1, n), 0.5)
    out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale, rhs_bias=bias)
    # the kernel rounds weight x scale to bf16 (as the widening pass does): the oracle contracts those values
    rhs_f = O.round_to_bf16(O.dequantize(rhs_values, _np(scale)))
    want = O.ragged_dot_fused(_np(lhs), rhs_f, gs, rhs_bias=_np(bias))
    _check(out, want, 1e-5)
    assert torch.count_nonzero(out[int(gs.sum()):]) == 0
    return
  if v["mode"] == 2:
    lhs, dout = mk((m, k), 1.0).to(lt), mk((m, n), 1.0).to(lt)
    out = hip_ops.ragged_dot_drhs(lhs, dout, gst, G, config=cfg, out_dtype=torch.float32)
    _check(out, _ref(lhs, dout, gs, O.RAGGED_CONTRACTING), TOL[lt])
    return
  lhs_scale = rhs_scale = None
  if rt in (torch.int8, torch.uint8) and lt == torch.int8:  # int8 x int8 (or packed int4), one scale per row and per (group, column)
    lhs = torch.tensor(rng.integers(-127, 128, (m, k)).astype(np.int8), device=device)
    top = 127 if rt == torch.int8 else 7
    rhs = torch.tensor(rng.integers(-top - 1, top + 1, (G, k, n)).astype(np.int8), device=device)
    lhs_scale, rhs_scale = mk((m, 1), 0.01).abs() + 0.005, mk((G, 1, n), 0.01).abs() + 0.005
    lhs_f = O.dequantize(lhs.cpu().numpy().astype(np.float64), _np(lhs_scale))
    rhs_f = O.dequantize(rhs.cpu().numpy().astype(np.float64), _np(rhs_scale))
    if rt == torch.uint8:
      rhs = hip_ops.pack_int4(rhs)
    tol = 1e-5  # the int32 sums are exact
  elif rt == torch.int8:
    rhs = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
    rhs_scale = mk((G, 1, n), 0.01).abs() + 1e-3
    rhs_f = O.dequantize(rhs.cpu().numpy(), _np(rhs_scale))
    lhs = mk((m, k), 1.0).to(lt)
    lhs_f = _np(lhs)
    tol = 1e-5
  elif rt == torch.uint8 and lt == torch.float8_e4m3fn:  # fp8 activations x packed int4 weights on the fp8 MFMAs
    values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
    rhs = torch.tensor(O.pack_int4(values), device=device)
    lhs = mk((m, k), 1.0).to(lt)
    lhs_scale, rhs_scale = mk((m, 1), 0.1).abs() + 0.05, mk((G, 1, n), 0.1).abs() + 1e-2
    lhs_f, rhs_f = _np(lhs) * _np(lhs_scale), O.dequantize(values, _np(rhs_scale))
    tol = 1e-4
  elif rt == torch.uint8:  # int4 weights, two to a byte along k
    values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
    rhs = torch.tensor(O.pack_int4(values), device=device)
    rhs_scale = mk((G, 1, n), 0.1).abs() + 1e-2
    rhs_f = O.dequantize(values, _np(rhs_scale))
    lhs = mk((m, k), 1.0).to(lt)
    lhs_f = _np(lhs)
    tol = 1e-5
  elif rt == torch.float8_e4m3fn and lt == torch.bfloat16:  # the streaming small-m kernel on fp8 weights
    rhs = mk((G, k, n), 1.0).to(rt)
    rhs_scale = mk((G, 1, n), 0.01).abs() + 1e-3
    rhs_f = O.dequantize(O.e4m3fn_decode(rhs.view(torch.uint8).cpu().numpy()), _np(rhs_scale))
    lhs = mk((m, k), 1.0).to(lt)
    lhs_f = _np(lhs)
    tol = 1e-5
  elif lt == torch.float8_e4m3fn:
    lhs, rhs = mk((m, k), 1.0).to(lt), mk((G, k, n), 1.0).to(rt)
    lhs_scale, rhs_scale = mk((m, 1), 0.1).abs() + 0.05, mk((G, 1, n), 0.1).abs() + 0.05
    lhs_f, rhs_f = _np(lhs) * _np(lhs_scale), _np(rhs) * _np(rhs_scale)
    tol = 1e-4
  else:
    trans = v["mode"] == 1
    lhs, rhs = mk((m, n if trans else k), 1.0).to(lt), mk((G, k, n), k ** -0.5).to(rt)
    lhs_f, rhs_f = _np(lhs), _np(rhs)
    tol = TOL[lt] if lt == torch.float32 else 1e-5  # f32 output of exact bf16/f16 products
  out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, trans_rhs=(v["mode"] == 1),
                               lhs_scale=lhs_scale, rhs_scale=rhs_scale)
  want = O.ragged_dot(lhs_f, rhs_f, gs, O.TRANS_RHS if v["mode"] == 1 else O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, tol)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  if v["block_m"] >= 128:
    # The same call with its tiles cut along the contraction (a launch this small is one partial round of workgroups,
    # so every tile is split): 2 and 3 parts, and 12 = 256 CUs / 20 tiles, most of which get no k-step at all.
    for split_k in (2, 3, 16):
      split = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=dataclasses.replace(cfg, split_k=split_k), out_dtype=torch.float32,
                                     trans_rhs=(v["mode"] == 1), lhs_scale=lhs_scale, rhs_scale=rhs_scale)
      _check(split, want, tol)
      assert torch.count_nonzero(split[int(gs.sum()):]) == 0
      if lt == torch.int8:
        assert torch.equal(split, out)  # int32 sums do not depend on how they are grouped
      again = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=dataclasses.replace(cfg, split_k=split_k), out_dtype=torch.float32,
                                     trans_rhs=(v["mode"] == 1), lhs_scale=lhs_scale, rhs_scale=rhs_scale)
      assert torch.equal(again, split)  # parts are added in the order of their index, whoever arrives last


@pytest.mark.parametrize("trans", [False, True])
@pytest.mark.parametrize("m,split_k,parts", [(4096, 4, 4), (4096, 2, 2), (4608, 4, 2), (5632, 4, 1), (8192, 8, 1)])
def test_last_round_of_a_tiled_launch_split_along_the_contraction(m, split_k, parts, trans, device):
  """`split_k` on a tiled kernel: only the tiles beyond the last multiple of the CU count are cut, into
  min(split_k, CUs / their number) parts. 128 x 256 tiles on n = 2304: m = 4096 gives 33 m-tasks x 9 = 297 tiles, 41
  beyond 256 (6 parts would fit, split_k decides); 4608: 37 x 9 = 333, 77 beyond (3 fit: 2 when split_k is 2... here 4
  asks, 3 fit); 5632: 45 x 9 = 405, 149 beyond (no split: the round is more than half full); 8192: 65 x 9 = 585, 73
  beyond 512."""
  del parts  # (documentation of the case; the result must be the same whatever the kernel decides)
  rng = np.random.default_rng(m + split_k)
  G, contraction, other = 2, 520, 2304
  gs = np.array([m // 2 + 37, m // 2 - 37 - 5], np.int32)
  k, n = (other, contraction) if trans else (contraction, other)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device).to(torch.bfloat16)
  lhs, rhs = mk((m, contraction), 1.0), mk((G, k, n), contraction ** -0.5)
  gst = torch.tensor(gs, device=device)
  cfg = hip_ops.KernelConfig(128, 256, 64, 2, 4, 3, grid_tile_width=4)
  plain = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, trans_rhs=trans)
  split_cfg = dataclasses.replace(cfg, split_k=split_k)
  split = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=split_cfg, out_dtype=torch.float32, trans_rhs=trans)
  # f32 sums of exact products in another grouping: equal to rounding, and equal bits where nothing was split
  assert O.rel_l2(_np(split), _np(plain)) <= 1e-6
  assert torch.equal(split[:1024], plain[:1024])  # (the launch's first 256 tiles cover these rows)
  assert torch.count_nonzero(split[int(gs.sum()):]) == 0
  # the launch's last tiles, which are the split ones, hold the last rows: those against the oracle's definition
  first = int(gs.sum()) - 400
  assert first > gs[0]
  w1 = _np(rhs[1]).astype(np.float64)
  want = _np(lhs[first:int(gs.sum())]).astype(np.float64) @ (w1.T if trans else w1)
  _check(split[first:int(gs.sum())], want, 1e-5)
  for _ in range(3):
    assert torch.equal(hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=split_cfg, out_dtype=torch.float32, trans_rhs=trans), split)
  if not trans:
    # the fused entry point: bias, activation and a group offset ride on the split tiles' epilogue
    bias = torch.tensor(rng.normal(0, 0.5, (G, 1, n)).astype(np.float32), device=device)
    a = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.bfloat16, rhs_bias=bias, activation="silu")
    b = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=split_cfg, out_dtype=torch.bfloat16, rhs_bias=bias, activation="silu")
    assert O.rel_l2(_np(b), _np(a)) <= 3e-3 and (b != a).float().mean() < 0.01  # a bf16 rounding flips here and there
    off = torch.tensor([1], dtype=torch.int32, device=device)
    gs3 = torch.tensor(np.array([100, gs[0] - 100, gs[1]], np.int32), device=device)
    a = hip_ops.ragged_dot_fwd(lhs, rhs, gs3, config=cfg, out_dtype=torch.float32, group_offset=off)
    b = hip_ops.ragged_dot_fwd(lhs, rhs, gs3, config=split_cfg, out_dtype=torch.float32, group_offset=off)
    assert O.rel_l2(_np(b), _np(a)) <= 1e-6 and torch.count_nonzero(b[:100]) == 0


def test_tiled_split_is_declined_where_no_kernel_has_it(device):
  G, m, k, n = 2, 512, 256, 512
  a, b, gs = _inputs("split_declined", G, m, k, n, torch.bfloat16, device)
  gst = torch.tensor(gs, device=device)
  small = hip_ops.KernelConfig(64, 128, 64, 2, 2, 4, split_k=2)  # tiles of fewer than 128 rows
  with pytest.raises(NotImplementedError, match="split"):
    hip_ops.ragged_dot_fwd(a, b, gst, config=small, out_dtype=torch.float32)
  glu = dataclasses.replace(next(hip_ops.KernelConfig(*v[:6]) for v in hip._variant_table()[(3, _lib.TKX_BF16, _lib.TKX_BF16)]
                                 if v[0] >= 128), split_k=2)
  with pytest.raises(NotImplementedError, match="split"):
    hip_ops.ragged_dot_fwd(a, b, gst, config=glu, out_dtype=torch.float32, gateup=True, activation="silu")
  with pytest.raises(ValueError, match="split_k"):
    hip_ops.ragged_dot_fwd(a, b, gst, config=hip_ops.KernelConfig(128, 256, 64, 2, 4, 3, split_k=17), out_dtype=torch.float32)
  drhs = dataclasses.replace(next(hip_ops.KernelConfig(*v[:6]) for v in hip._variant_table()[(2, _lib.TKX_BF16, _lib.TKX_BF16)]),
                             split_k=2)
  # (drhs has no last-round split either: its entry point ignores the field, as it always has)
  out = hip_ops.ragged_dot_drhs(a, torch.randn(m, n, device=device).to(torch.bfloat16), gst, G, config=drhs, out_dtype=torch.float32)
  assert out.shape == (G, k, n)
  # the quantised-output entry point drops the split (its epilogue needs whole rows of 128 columns in one workgroup)
  q, s = hip_ops.ragged_dot_fwd_fp8_out(a, b, gst, config=hip_ops.KernelConfig(128, 256, 64, 2, 4, 3, split_k=4))
  q1, s1 = hip_ops.ragged_dot_fwd_fp8_out(a, b, gst, config=hip_ops.KernelConfig(128, 256, 64, 2, 4, 3))
  assert torch.equal(q.view(torch.uint8), q1.view(torch.uint8)) and torch.equal(s, s1)


def _plain_tiled_variants():
  """Forward and dlhs tile variants whose operands share one unquantised type."""
  return [v for v in _variant_cases() if v.values[0]["mode"] in (0, 1) and v.values[0]["block_m"] != 16
          and v.values[0]["lhs_dtype"] == v.values[0]["rhs_dtype"] and v.values[0]["lhs_dtype"] in (_lib.TKX_F32, _lib.TKX_BF16, _lib.TKX_F16)]


@pytest.mark.parametrize("contraction", [40, 104, 200])
@pytest.mark.parametrize("v", _plain_tiled_variants())
def test_contraction_lengths_that_are_not_whole_steps(v, contraction, device):
  """Any contraction length whose rows are 16-byte multiples is taken: what the pipelined k-steps leave over (a
  partial step; for the split-pipeline variants up to two) goes through a zero-filled masked path."""
  rng = np.random.default_rng(contraction + v["block_k"])
  G, m, other = 3, 200, 136
  gs = np.array([90, 0, 97], np.int32)
  dt = _TORCH_DTYPE[v["lhs_dtype"]]
  trans = v["mode"] == 1
  k, n = (other, contraction) if trans else (contraction, other)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device).to(dt)
  lhs, rhs = mk((m, contraction), 1.0), mk((G, k, n), contraction ** -0.5)
  cfg = hip_ops.KernelConfig(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"],
                             grid_tile_width=2)
  out = hip_ops.ragged_dot_fwd(lhs, rhs, torch.tensor(gs, device=device), config=cfg, out_dtype=torch.float32, trans_rhs=trans)
  want = O.ragged_dot(_np(lhs), _np(rhs), gs, O.TRANS_RHS if trans else O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0


@pytest.mark.parametrize("block_n,depth", [(128, 2), (128, 4), (128, 8), (256, 2), (256, 4)])
@pytest.mark.parametrize("case", ["ragged", "two_chunks", "all_empty", "one_big_group", "first_and_last_empty",
                                  "many_groups"])
def test_small_m_int8_kernel_edges(case, block_n, depth, device):
  """The streaming small-m kernel (128 columns per workgroup, and the wide one with 256): empty groups
  anywhere, more than 64 groups, groups taller than one 16-row pass, a column count that is not a
  multiple of its column tile, and a zero tail."""
  rng = np.random.default_rng(len(case) + depth)
  k, n = 1024, 208 if block_n == 128 else 464  # one partial tile; a whole and a partial tile
  if case == "ragged":
    gs = np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32)
  elif case == "two_chunks":
    gs = rng.integers(0, 4, 70).astype(np.int32)
    gs[[0, 63, 64, 69]] = [0, 2, 0, 5]
  elif case == "all_empty":
    gs = np.zeros(5, np.int32)
  elif case == "one_big_group":
    gs = np.array([0, 45, 0], np.int32)
  elif case == "many_groups":  # more groups than the workgroup has threads: the row-offset sum loops
    gs = rng.integers(0, 3, 600).astype(np.int32)
  else:
    gs = np.array([0, 4, 9, 0], np.int32)
  G, m = len(gs), int(gs.sum()) + 11
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  rhs = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((np.abs(rng.normal(0, 0.01, (G, 1, n))) + 1e-3).astype(np.float32), device=device)
  cfg = hip_ops.KernelConfig(16, block_n, 32, 1, 4, depth)
  out = hip_ops.ragged_dot_fwd(lhs, rhs, torch.tensor(gs, device=device), config=cfg, out_dtype=torch.float32,
                               rhs_scale=scale)
  want = O.ragged_dot(_np(lhs), O.dequantize(rhs.cpu().numpy(), _np(scale)), gs, O.DEFAULT, acc_dtype=np.float64,
                      out_dtype="f64")
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  # bf16 output, and the same bits on a second run (fixed reduction order)
  out16 = hip_ops.ragged_dot_fwd(lhs, rhs, torch.tensor(gs, device=device), config=cfg, out_dtype=torch.bfloat16,
                                 rhs_scale=scale)
  assert torch.equal(out16, out.to(torch.bfloat16))
  assert torch.equal(out, hip_ops.ragged_dot_fwd(lhs, rhs, torch.tensor(gs, device=device), config=cfg,
                                                 out_dtype=torch.float32, rhs_scale=scale))


@pytest.mark.parametrize("split_k,depth", [(2, 2), (2, 4), (4, 2), (8, 2), (4, 4)])
@pytest.mark.parametrize("case", ["ragged", "two_chunks", "all_empty", "one_big_group", "first_and_last_empty",
                                  "beyond_m"])
@pytest.mark.parametrize("weights", ["int8", "bf16", "int8_blocks"])
def test_small_m_kernel_with_the_contraction_split_over_workgroups(case, split_k, depth, weights, device):
  """split_k workgroups per (group, column tile): partial sums through the workspace, added by the last to arrive in
  the order of the split index. Same edges as the unsplit kernel, group sizes that add up to more than m, the same
  bits on a second run, and the arrival counters back at zero afterwards (the next call relies on it)."""
  rng = np.random.default_rng(len(case) + depth + split_k)
  k, n = 128 * split_k * depth * (2 if case == "ragged" else 1), 208
  if case == "ragged":
    gs = np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32)
  elif case == "two_chunks":
    gs = rng.integers(0, 4, 70).astype(np.int32)
    gs[[0, 63, 64, 69]] = [0, 2, 0, 5]
  elif case == "all_empty":
    gs = np.zeros(5, np.int32)
  elif case == "one_big_group":
    gs = np.array([0, 45, 0], np.int32)
  elif case == "beyond_m":
    gs = np.array([5, 9, 7, 4], np.int32)
  else:
    gs = np.array([0, 4, 9, 0], np.int32)
  G = len(gs)
  m = 17 if case == "beyond_m" else int(gs.sum()) + 11
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  scale = None
  if weights == "bf16":
    rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
    dense = _np(rhs)
  else:
    blocks = 1 if weights == "int8" else k // 64
    rhs = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
    scale = torch.tensor((np.abs(rng.normal(0, 0.01, (G, blocks, n))) + 1e-3).astype(np.float32), device=device)
    dense = O.dequantize(rhs.cpu().numpy(), _np(scale))
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth, split_k=split_k)
  gst = torch.tensor(gs, device=device)
  out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  clipped = np.diff(np.minimum(np.concatenate([[0], np.cumsum(gs)]), m)).astype(np.int32)
  want = O.ragged_dot(_np(lhs), dense, clipped, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 2e-3 if weights == "int8_blocks" else 1e-5)
  assert torch.count_nonzero(out[int(clipped.sum()):]) == 0
  ws = hip_ops.split_workspace(m, n, split_k, device)
  counter_words = _lib.load().tkx_ragged_dot_decode_counter_bytes(split_k) // 4
  assert counter_words >= G * 2 and torch.count_nonzero(ws[:counter_words]) == 0
  again = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  assert torch.equal(out, again)
  out16 = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.bfloat16, rhs_scale=scale)
  assert torch.equal(out16, out.to(torch.bfloat16))


@pytest.mark.parametrize("depth", [2, 4])
@pytest.mark.parametrize("case", ["sparse", "sparse_many_tiles", "mostly_empty", "ragged_tall", "two_chunks", "all_empty",
                                  "none_empty", "beyond_m", "one_row"])
@pytest.mark.parametrize("weights", ["int8", "fp8", "int4"])
def test_small_m_kernel_persistent_form(case, depth, weights, device):
  """`persistent = 1`: the workgroups of empty groups contract the tails of the other groups' tiles, whose parts meet
  through the workspace. Cases in which they help (no group above 16 rows, some groups empty: few or many helpers per
  tile, one or several column tiles, a partial last tile) and cases that run as the plain kernel does (a tall group, no
  empty group, nothing but empty groups); sizes that add up to more than m; lhs rows of no group that hold NaN (nothing
  of them may reach a result); the same bits on a second run; the arrival counters back at zero afterwards."""
  rng = np.random.default_rng(len(case) + depth)
  k, n = 1024, 208
  if case == "sparse":
    gs = np.array([3, 0, 0, 16, 1, 0, 7, 2, 0, 0, 4], np.int32)
  elif case == "sparse_many_tiles":
    gs, k, n = np.array([2, 0, 1, 0, 0, 5, 1, 0], np.int32), 512, 848
  elif case == "mostly_empty":  # several helper workgroups per tile: tails cut into pieces
    gs, k = np.zeros(40, np.int32), 2048
    gs[[3, 17, 38]] = [2, 16, 1]
  elif case == "ragged_tall":
    gs = np.array([3, 0, 0, 17, 1, 0, 45, 2], np.int32)
  elif case == "two_chunks":
    gs = rng.integers(0, 4, 70).astype(np.int32)
    gs[[0, 63, 64, 69]] = [0, 2, 0, 5]
  elif case == "all_empty":
    gs = np.zeros(5, np.int32)
  elif case == "none_empty":
    gs = np.array([1, 4, 16, 2], np.int32)
  elif case == "beyond_m":
    gs = np.array([5, 0, 9, 7, 0, 4], np.int32)
  else:
    gs, k = np.array([0, 0, 1, 0], np.int32), 128
  G = len(gs)
  m = 17 if case == "beyond_m" else int(gs.sum()) + 11
  clipped = np.diff(np.minimum(np.concatenate([[0], np.cumsum(gs)]), m)).astype(np.int32)
  lhs_np = rng.normal(0, 1, (m, k)).astype(np.float32)
  lhs = torch.tensor(lhs_np, device=device).to(torch.bfloat16)
  lhs[int(clipped.sum()):] = float("nan")
  scale = torch.tensor((np.abs(rng.normal(0, 0.01, (G, 1, n))) + 1e-3).astype(np.float32), device=device)
  if weights == "fp8":
    rhs = torch.tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
    dense = rhs.float().cpu().numpy() * _np(scale)
    call_rhs = rhs
  elif weights == "int4":
    q4 = torch.tensor(rng.integers(-8, 8, (G, k, n)).astype(np.int8), device=device)
    dense = O.dequantize(q4.cpu().numpy(), _np(scale))
    call_rhs = hip_ops.pack_int4(q4)
  else:
    rhs = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
    dense = O.dequantize(rhs.cpu().numpy(), _np(scale))
    call_rhs = rhs
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth, persistent=1)
  gst = torch.tensor(gs, device=device)
  out = hip_ops.ragged_dot_fwd(lhs, call_rhs, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  lhs_f = _np(lhs)
  lhs_f[int(clipped.sum()):] = 0
  want = O.ragged_dot(lhs_f, dense, clipped, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(clipped.sum()):]) == 0
  ws = hip_ops.split_workspace(m, n, 1, device, persistent=1)
  counter_words = _lib.load().tkx_ragged_dot_decode_counter_bytes(2) // 4
  assert ws.numel() * 4 >= _lib.load().tkx_ragged_dot_decode_persistent_workspace_bytes()
  assert torch.count_nonzero(ws[:counter_words]) == 0
  again = hip_ops.ragged_dot_fwd(lhs, call_rhs, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  assert torch.equal(out, again)
  out16 = hip_ops.ragged_dot_fwd(lhs, call_rhs, gst, config=cfg, out_dtype=torch.bfloat16, rhs_scale=scale)
  assert torch.equal(out16, out.to(torch.bfloat16))


def test_persistent_form_declines_what_it_does_not_take(device):
  """bf16 weights, scales per k-block, the wide tile, a split contraction on top and more than 256 groups are
  `NotImplementedError` with `persistent = 1`; the entry point without a workspace declines it too."""
  rng = np.random.default_rng(2)
  k, n = 1024, 256
  mk_lhs = lambda m: torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  gs = torch.tensor([1, 0, 2, 1], dtype=torch.int32, device=device)
  i8 = torch.tensor(rng.integers(-128, 128, (4, k, n)).astype(np.int8), device=device)
  one = torch.ones(4, 1, n, device=device)
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(mk_lhs(4), i8.to(torch.bfloat16), gs, config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, persistent=1),
                           out_dtype=torch.float32)
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(mk_lhs(4), i8, gs, config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, persistent=1),
                           out_dtype=torch.float32, rhs_scale=torch.ones(4, 4, n, device=device))
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(mk_lhs(4), i8, gs, config=hip_ops.KernelConfig(16, 256, 32, 1, 4, 2, persistent=1),
                           out_dtype=torch.float32, rhs_scale=one)
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(mk_lhs(4), i8, gs, config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, split_k=2, persistent=1),
                           out_dtype=torch.float32, rhs_scale=one)
  with pytest.raises(ValueError):
    hip_ops.ragged_dot_fwd(mk_lhs(4), i8, gs, config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, persistent=3),
                           out_dtype=torch.float32, rhs_scale=one)
  G = 300
  big = torch.zeros(G, 128, 128, dtype=torch.int8, device=device)
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(torch.zeros(8, 128, dtype=torch.bfloat16, device=device), big,
                           torch.zeros(G, dtype=torch.int32, device=device),
                           config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, persistent=1), out_dtype=torch.float32,
                           rhs_scale=torch.ones(G, 1, 128, device=device))


def test_public_op_splits_the_contraction_when_a_launch_has_few_tiles(device):
  """8 groups x 512 columns = 32 (group, column tile) pairs: the heuristics split the contraction 8 ways (256
  workgroups), the autotuning search space offers the splits that divide k, and the result matches the oracle."""
  rng = np.random.default_rng(11)
  G, k, n = 8, 4096, 512
  gs = np.array([2, 0, 1, 3, 0, 1, 2, 1], np.int32)
  m = int(gs.sum()) + 2
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, 1, n)) / 127 * 0.1).astype(np.float32), device=device)
  rhs = tokamax_amd.QArray(q, scale)
  gst = torch.tensor(gs, device=device)
  op = tokamax_amd.HipRaggedDot()
  ba = op.bind(lhs, rhs, group_sizes=gst)
  cfg = op._get_heuristics_config(ba)
  assert (cfg.block_m, cfg.block_n, cfg.split_k) == (16, 128, 8)
  splits = {c.split_k for c in op._get_autotuning_configs(ba) if c.block_m == 16}
  assert splits == {1, 2, 4, 8}
  out = op(lhs, rhs, group_sizes=gst, preferred_element_type=torch.float32)
  want = O.ragged_dot(_np(lhs), O.dequantize(q.cpu().numpy(), _np(scale)), gs, O.DEFAULT, acc_dtype=np.float64,
                      out_dtype="f64")
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0


def test_int4_pack_and_unpack_kernels(device):
  """tkx_pack_int4 / tkx_unpack_int4 against the oracle's bytes, bit for bit, and the round trip."""
  rng = np.random.default_rng(3)
  q = rng.integers(-8, 8, (3, 64, 48)).astype(np.int8)
  packed = hip_ops.pack_int4(torch.tensor(q, device=device))
  assert packed.dtype == torch.uint8 and tuple(packed.shape) == (3, 32, 48)
  assert np.array_equal(packed.cpu().numpy(), O.pack_int4(q))
  assert np.array_equal(hip_ops.unpack_int4(packed).cpu().numpy(), q)
  every_byte = torch.arange(256, dtype=torch.uint8, device=device).reshape(1, 16, 16)
  assert np.array_equal(hip_ops.unpack_int4(every_byte).cpu().numpy(), O.unpack_int4(every_byte.cpu().numpy()))


# (There is no 8-deep variant with scales per k-block.)
@pytest.mark.parametrize("scales,depth,split_k", [(s, d, k) for s in ("per_column", "k_blocks")
                                                  for d, k in ((2, 1), (4, 1), (8, 1), (2, 2), (4, 2))
                                                  if not (d == 8 and s == "k_blocks")])
@pytest.mark.parametrize("case", ["ragged", "one_big_group", "first_and_last_empty"])
def test_small_m_kernel_on_packed_int4_weights(case, scales, depth, split_k, device):
  """Two int4 per byte along k: the streaming kernel's result matches the oracle on the unpacked values, and is the
  int8 kernel's result on them bit for bit (same contraction order; only the loads and the widening differ)."""
  rng = np.random.default_rng(len(case) + depth)
  k, n = 2048, 208
  gs = {"ragged": np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32), "one_big_group": np.array([0, 45, 0], np.int32),
        "first_and_last_empty": np.array([0, 4, 9, 0], np.int32)}[case]
  G, m = len(gs), int(gs.sum()) + 5
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
  blocks = 1 if scales == "per_column" else k // 128
  scale = torch.tensor((np.abs(rng.normal(0, 0.05, (G, blocks, n))) + 1e-2).astype(np.float32), device=device)
  packed = torch.tensor(O.pack_int4(q), device=device)
  gst = torch.tensor(gs, device=device)
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth, split_k=split_k)
  out = hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  want = O.ragged_dot(_np(lhs), O.dequantize(q, _np(scale)), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 2e-3 if scales == "k_blocks" else 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  cfg8 = hip_ops.KernelConfig(16, 128, 32, 1, 4, min(depth, 4), split_k=split_k)
  same = hip_ops.ragged_dot_fwd(lhs, torch.tensor(q, device=device), gst, config=cfg8, out_dtype=torch.float32, rhs_scale=scale)
  assert torch.equal(out, same)


def _packed_int4_tile_cases():
  return [pytest.param(v, id="{block_m}x{block_n}x{block_k}-w{waves_m}x{waves_n}-s{num_stages}".format(**v))
          for v in _lib.variants(0) if v["rhs_dtype"] == _lib.TKX_I4X2 and v["lhs_dtype"] == _lib.TKX_BF16
          and v["block_m"] != 16 and v["mode"] == 0]


@pytest.mark.parametrize("v", _packed_int4_tile_cases())
def test_tiled_kernels_on_packed_int4_weights(v, device):
  """The tiled kernels read int4 weights two to a byte along k: an odd number of k-steps, a ragged last column tile,
  groups that start and end inside tiles, an empty group, rows after the last group. Against the oracle on the
  unpacked values, against the int8 kernel of the same tile on them (the same products, summed in another order
  inside a pair of MFMA atoms), and bit for bit against itself."""
  rng = np.random.default_rng(v["block_m"] + v["num_stages"])
  G, k, n = 5, 5 * v["block_k"], 272
  gs = np.array([3, 300, 0, 70, 129], np.int32)
  m = int(gs.sum()) + 9
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
  scale = torch.tensor((np.abs(rng.normal(0, 0.05, (G, 1, n))) + 1e-2).astype(np.float32), device=device)
  packed = torch.tensor(O.pack_int4(values), device=device)
  cfg = hip_ops.KernelConfig(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"], grid_tile_width=2)
  out = hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  want = O.ragged_dot(_np(lhs), O.dequantize(values, _np(scale)), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  assert torch.equal(out, hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale))
  int8_tiles = {(x["block_m"], x["block_n"], x["block_k"], x["waves_m"], x["waves_n"], x["num_stages"])
                for x in _lib.variants(0) if x["rhs_dtype"] == _lib.TKX_I8 and x["lhs_dtype"] == _lib.TKX_BF16 and x["mode"] == 0}
  if (cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages) in int8_tiles:
    same = hip_ops.ragged_dot_fwd(lhs, torch.tensor(values, device=device), gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
    torch.testing.assert_close(out, same, rtol=2e-6, atol=2e-5)
  # bf16 result and no scale at all; a contraction that is not whole k-steps is declined, not mis-read
  plain = hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.bfloat16)
  _check(plain, O.ragged_dot(_np(lhs), values.astype(np.float64), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 4e-3)
  with pytest.raises(NotImplementedError, match="block_k"):
    hip_ops.ragged_dot_fwd(lhs[:, :k - 32].contiguous(), packed[:, :k // 2 - 16].contiguous(), gst, config=cfg, out_dtype=torch.float32)
  # one expert-parallel shard: the sizes of every group of the job, the weights of groups 1..3 only, a bias
  offset = torch.tensor([1], dtype=torch.int32, device=device)
  bias = torch.tensor(rng.normal(0, 1, (3, 1, n)).astype(np.float32), device=device)
  shard = hip_ops.ragged_dot_fwd(lhs, packed[1:4].contiguous(), gst, config=cfg, out_dtype=torch.float32,
                                 rhs_scale=scale[1:4].contiguous(), rhs_bias=bias, group_offset=offset)
  lo, hi = int(gs[:1].sum()), int(gs[:4].sum())
  want_shard = np.zeros((m, n))
  want_shard[lo:hi] = want[lo:hi] + np.repeat(_np(bias)[:, 0], gs[1:4], axis=0)
  _check(shard, want_shard, 1e-5)
  assert torch.count_nonzero(shard[:lo]) == 0 and torch.count_nonzero(shard[hi:]) == 0


def _fp8_over_packed_int4_cases():
  return [pytest.param(v, id="{block_m}x{block_n}x{block_k}-w{waves_m}x{waves_n}-s{num_stages}".format(**v))
          for v in _lib.variants(0) if v["rhs_dtype"] == _lib.TKX_I4X2 and v["lhs_dtype"] == _lib.TKX_F8E4M3FN and v["mode"] == 0]


def test_row_sums_of_fp8_rows(device):
  """tkx_row_sums_fp8 against sums in float64 of the decoded bytes: every finite e4m3fn value occurs, rows shorter and
  longer than a wave's 1024-byte step, a row count that is not whole workgroups."""
  rng = np.random.default_rng(31)
  for rows, cols in ((7, 16), (33, 1040), (4, 4096), (9, 1408)):
    codes = rng.integers(0, 256, (rows, cols)).astype(np.uint8)
    codes[(codes & 0x7f) == 0x7f] = 0x08  # (no NaN)
    x = torch.tensor(codes, device=device).view(torch.float8_e4m3fn)
    sums = hip_ops.row_sums_fp8(x)
    want = O.e4m3fn_decode(codes).astype(np.float64).sum(axis=1)
    scale = np.abs(O.e4m3fn_decode(codes).astype(np.float64)).sum(axis=1)
    assert sums.dtype == torch.float32 and tuple(sums.shape) == (rows,)
    assert np.all(np.abs(_np(sums) - want) <= 1e-6 * scale)
    if cols % 128 == 0:
      chunks = hip_ops.row_sums_fp8(x, per_128_columns=True)
      values = O.e4m3fn_decode(codes).astype(np.float64).reshape(rows, cols // 128, 128)
      assert tuple(chunks.shape) == (cols // 128, rows)
      assert np.all(np.abs(_np(chunks).T - values.sum(axis=2)) <= 1e-6 * np.abs(values).sum(axis=2))
  with pytest.raises(ValueError):
    hip_ops.row_sums_fp8(torch.zeros(4, 16, device=device))
  with pytest.raises(NotImplementedError, match="multiple of 16"):
    hip_ops.row_sums_fp8(torch.zeros(4, 24, device=device).to(torch.float8_e4m3fn))


@pytest.mark.parametrize("v", _fp8_over_packed_int4_cases())
def test_tiled_kernels_on_fp8_activations_and_packed_int4_weights(v, device):
  """The fp8 MFMAs on int4 weights (weight w goes in as the e4m3 denormal (w + 8) / 512, the epilogue takes
  8 rowsum(x) off: pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:258-300): an odd number of k-steps, a ragged last column
  tile, groups that start and end inside tiles, an empty group, rows after the last group. Against the oracle on the
  dequantised operands, against the fp8 x fp8 kernels on the same values (int4 values are exact in fp8; another
  summation order), bit for bit against itself, with the row sums computed by the call and handed in, split along the
  contraction, and as one expert-parallel shard with a bias."""
  rng = np.random.default_rng(v["block_m"] + v["num_stages"] + v["waves_m"])
  G, k, n = 5, 5 * v["block_k"], 272
  gs = np.array([3, 300, 0, 70, 129], np.int32)
  m = int(gs.sum()) + 9
  gst = torch.tensor(gs, device=device)
  x = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32) * rng.uniform(0.1, 10, (m, 1)).astype(np.float32), device=device)
  xs = x.abs().amax(dim=1, keepdim=True) / 448
  xq = (x / xs).to(torch.float8_e4m3fn)
  values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
  values[0, :, 0], values[0, :, 1] = -8, 7  # (the two ends of the range in whole columns)
  scale = torch.tensor((np.abs(rng.normal(0, 0.05, (G, 1, n))) + 1e-2).astype(np.float32), device=device)
  packed = torch.tensor(O.pack_int4(values), device=device)
  cfg = hip_ops.KernelConfig(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"], grid_tile_width=2)
  call = lambda cfg=cfg, lhs_scale=xs, **kw: hip_ops.ragged_dot_fwd(xq, packed, gst, config=cfg, out_dtype=torch.float32,
                                                                    lhs_scale=lhs_scale, rhs_scale=scale, **kw)
  out = call()
  lhs_f = O.e4m3fn_decode(xq.view(torch.uint8).cpu().numpy()).astype(np.float64) * _np(xs)
  want = O.ragged_dot(lhs_f, O.dequantize(values, _np(scale)), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  # f32 sums of up to 640 products of size up to 448 * 15 / 512 each, 512 times that, less 8 times an f32 row sum
  _check(out, want, 5e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  assert torch.equal(out, call())
  both = torch.cat([xs.view(1, m), hip_ops.row_sums_fp8(xq).view(1, m)])
  assert torch.equal(out, call(lhs_scale=both))
  f8_tiles = [x_ for x_ in _lib.variants(0) if x_["rhs_dtype"] == x_["lhs_dtype"] == _lib.TKX_F8E4M3FN and x_["mode"] == 0
              and x_["block_m"] == 128]
  as_fp8 = torch.tensor(values, device=device).to(torch.float32).to(torch.float8_e4m3fn)
  t = f8_tiles[0]
  f8_cfg = hip_ops.KernelConfig(t["block_m"], t["block_n"], t["block_k"], t["waves_m"], t["waves_n"], t["num_stages"])
  same = hip_ops.ragged_dot_fwd(xq, as_fp8, gst, config=f8_cfg, out_dtype=torch.float32, lhs_scale=xs, rhs_scale=scale)
  assert O.rel_l2(_np(out), _np(same)) <= 2e-5
  if v["block_m"] >= 128:
    for split_k in (2, 3):
      split = call(dataclasses.replace(cfg, split_k=split_k))
      _check(split, want, 5e-5)
      assert torch.equal(split, call(dataclasses.replace(cfg, split_k=split_k)))
  # bf16 result without a weight scale; no lhs scale, scale blocks of another size than a power of two and a
  # contraction that is not whole k-steps are declined
  plain = hip_ops.ragged_dot_fwd(xq, packed, gst, config=cfg, out_dtype=torch.bfloat16, lhs_scale=xs)
  _check(plain, O.ragged_dot(lhs_f, values.astype(np.float64), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 4e-3)
  with pytest.raises(NotImplementedError, match="lhs scale"):
    hip_ops.ragged_dot_fwd(xq, packed, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(xq, packed, gst, config=cfg, out_dtype=torch.float32, lhs_scale=xs,
                           rhs_scale=scale.expand(G, 2, n).contiguous())  # (blocks of 320 rows: not a power of two)
  with pytest.raises(NotImplementedError, match="block_k"):
    hip_ops.ragged_dot_fwd(xq[:, :k - 32].contiguous(), packed[:, :k // 2 - 16].contiguous(), gst, config=cfg,
                           out_dtype=torch.float32, lhs_scale=xs)
  offset = torch.tensor([1], dtype=torch.int32, device=device)
  bias = torch.tensor(rng.normal(0, 1, (3, 1, n)).astype(np.float32), device=device)
  shard = hip_ops.ragged_dot_fwd(xq, packed[1:4].contiguous(), gst, config=cfg, out_dtype=torch.float32, lhs_scale=xs,
                                 rhs_scale=scale[1:4].contiguous(), rhs_bias=bias, group_offset=offset)
  lo, hi = int(gs[:1].sum()), int(gs[:4].sum())
  want_shard = np.zeros((m, n))
  want_shard[lo:hi] = want[lo:hi] + np.repeat(_np(bias)[:, 0], gs[1:4], axis=0)
  _check(shard, want_shard, 5e-5)
  assert torch.count_nonzero(shard[:lo]) == 0 and torch.count_nonzero(shard[hi:]) == 0


def test_gateup_over_one_byte_weights_whose_halves_are_not_whole_16_byte_pieces(device):
  """Gate-up fusion reads the up half of a weight row n / 2 elements in. With one-byte weights that is a whole 16-byte
  piece only if n % 32 == 0: the library declines other widths, and the op widens such weights to bf16 first (int8
  weights and packed int4 ones alike) instead of reading up columns from the wrong place."""
  rng = np.random.default_rng(77)
  G, k, n, rows = 3, 256, 272, 96
  m = G * rows
  gs = torch.full((G,), rows, dtype=torch.int32, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-8, 8, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, 1, n)) * 0.02).astype(np.float32), device=device)
  want = O.ragged_dot_fused(_np(lhs), O.dequantize(q.cpu().numpy(), _np(scale)), np.full(G, rows, np.int32), gateup_activation="silu")
  op = tokamax_amd.HipRaggedDot()
  int4 = getattr(torch, "int4", torch.int8)
  for rhs in (tokamax_amd.QArray(q, scale), tokamax_amd.pack_int4(tokamax_amd.QArray(q, scale, None, int4))):
    bound = op.bind(lhs, rhs, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    assert op._problem(bound)[1] == (3, _lib.TKX_BF16, _lib.TKX_BF16)
    out = op(lhs, rhs, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    assert tuple(out.shape) == (m, n // 2)
    _check(out, want, 5e-3)  # (weights times scales rounded to bf16)
  cfg = hip_ops.KernelConfig(128, 256, 64, 2, 4, 3)
  with pytest.raises(NotImplementedError, match="n % 32"):
    hip_ops.ragged_dot_fwd(lhs, q, gs, config=cfg, out_dtype=torch.float32, rhs_scale=scale, gateup=True, activation="silu")
  # 256 columns: the int8 weights are read as they are
  narrow = tokamax_amd.QArray(q[:, :, :256].contiguous(), scale[:, :, :256].contiguous())
  bound = op.bind(lhs, narrow, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
  assert op._problem(bound)[1] == (3, _lib.TKX_BF16, _lib.TKX_I8)
  out = op(lhs, narrow, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
  _check(out, O.ragged_dot_fused(_np(lhs), O.dequantize(q[:, :, :256].cpu().numpy(), _np(scale[:, :, :256])),
                                 np.full(G, rows, np.int32), gateup_activation="silu"), 1e-5)


def _int8_over_packed_int4_cases():
  return [pytest.param(v, id="mode{mode}-{block_m}x{block_n}x{block_k}-w{waves_m}x{waves_n}-s{num_stages}".format(**v))
          for v in _lib.variants(0) if v["rhs_dtype"] == _lib.TKX_I4X2 and v["lhs_dtype"] == _lib.TKX_I8 and v["mode"] in (0, 4)]


@pytest.mark.parametrize("v", _int8_over_packed_int4_cases())
def test_tiled_kernels_on_int8_activations_and_packed_int4_weights(v, device):
  """The int8 MFMAs on int4 weights read two to a byte (a nibble at the top of its byte is 16 w; the factor goes out
  where the exact int32 sums become floats; pallas_mosaic_gpu_kernel_sm100_i8_quant.py:114-190): against the oracle on
  the dequantised operands and bit for bit against the int8 x int8 kernels on the unpacked values, with one scale per
  row and per (group, column) or with scales per k-block on both sides; the two ends of the int4 range in whole
  columns, ragged groups, an empty one, rows of no group, a ragged last column tile; the split last round; the public
  op keeps the weights packed."""
  rng = np.random.default_rng(v["block_m"] + v["num_stages"] + v["mode"])
  G, k, n = 5, 5 * 128, 272
  gs = np.array([3, 300, 0, 70, 131], np.int32)
  m = int(gs.sum()) + 8
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.integers(-127, 128, (m, k)).astype(np.int8), device=device)
  values = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
  values[0, :, 0], values[0, :, 1] = -8, 7
  unpacked = torch.tensor(values, device=device)
  packed = hip_ops.pack_int4(unpacked)
  blocks = 1 if v["mode"] == 0 else 5
  mk = lambda shape, std: torch.tensor(np.abs(rng.normal(0, std, shape)).astype(np.float32) + std / 4, device=device)
  xs, ws_ = mk((m, blocks), 0.01), mk((G, blocks, n), 0.05)
  cfg = hip_ops.KernelConfig(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"], grid_tile_width=2)
  out = hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.float32, lhs_scale=xs, rhs_scale=ws_)
  lhs_f = O.dequantize(lhs.cpu().numpy().astype(np.float64), _np(xs))
  want = O.ragged_dot(lhs_f, O.dequantize(values.astype(np.float64), _np(ws_)), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5 if blocks > 1 else 1e-6)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  twin = next(x for x in _lib.variants(0) if x["lhs_dtype"] == x["rhs_dtype"] == _lib.TKX_I8 and x["mode"] == v["mode"]
              and k // blocks % x["block_k"] == 0)
  twin_cfg = hip_ops.KernelConfig(twin["block_m"], twin["block_n"], twin["block_k"], twin["waves_m"], twin["waves_n"], twin["num_stages"])
  same = hip_ops.ragged_dot_fwd(lhs, unpacked, gst, config=twin_cfg, out_dtype=torch.float32, lhs_scale=xs, rhs_scale=ws_)
  assert torch.equal(out, same)  # the same integers, and 16 s / 16 rounds like s
  if v["mode"] == 0 and v["block_m"] >= 128:
    split = hip_ops.ragged_dot_fwd(lhs, packed, gst, config=dataclasses.replace(cfg, split_k=3), out_dtype=torch.float32,
                                   lhs_scale=xs, rhs_scale=ws_)
    assert torch.equal(split, out)  # int32 sums do not depend on how they are grouped
  with pytest.raises(NotImplementedError):
    hip_ops.ragged_dot_fwd(lhs, packed, gst, config=cfg, out_dtype=torch.float32, rhs_scale=ws_)
  # the public op: a QArray of int8 activations over the packed weights names this kind of kernel
  int4 = getattr(torch, "int4", torch.int8)
  q_lhs = tokamax_amd.QArray(lhs, xs)
  q_rhs = tokamax_amd.pack_int4(tokamax_amd.QArray(unpacked, ws_, None, int4))
  op = tokamax_amd.HipRaggedDot()
  assert _lib_key(op, q_lhs, q_rhs, gst) == (v["mode"], _lib.TKX_I8, _lib.TKX_I4X2)
  _check(op(q_lhs, q_rhs, group_sizes=gst, preferred_element_type=torch.float32), want, 1e-5)
  if v["mode"] == 0 and v["block_m"] == 256:
    # gate-up fusion over the same weights read as [gate | up]: kernels of the same kind
    # (each half of a weight row must be whole 16-byte pieces, 16 columns of one-byte storage: with n = 272 the
    # operands are widened to bf16 instead, with n = 256 the weights stay packed)
    wide = op.bind(q_lhs, q_rhs, group_sizes=gst, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    assert op._problem(wide)[1] == (3, _lib.TKX_BF16, _lib.TKX_BF16)
    fused = op(q_lhs, q_rhs, group_sizes=gst, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    _check(fused, O.ragged_dot_fused(lhs_f, O.dequantize(values.astype(np.float64), _np(ws_)), gs, gateup_activation="silu"), 1e-2)
    with pytest.raises(NotImplementedError, match="n % 32"):
      hip_ops.ragged_dot_fwd(lhs, packed, gst, config=hip_ops.KernelConfig(256, 256, 128, 2, 4, 3), out_dtype=torch.float32,
                             lhs_scale=xs, rhs_scale=ws_, gateup=True, activation="silu")
    q_256 = tokamax_amd.pack_int4(tokamax_amd.QArray(unpacked[:, :, :256].contiguous(), ws_[:, :, :256].contiguous(), None, int4))
    bound = op.bind(q_lhs, q_256, group_sizes=gst, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    assert op._problem(bound)[1] == (3, _lib.TKX_I8, _lib.TKX_I4X2)
    fused = op(q_lhs, q_256, group_sizes=gst, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
    _check(fused, O.ragged_dot_fused(lhs_f, O.dequantize(values[:, :, :256].astype(np.float64), _np(ws_[:, :, :256])), gs,
                                     gateup_activation="silu"), 1e-5)


def test_public_op_on_fp8_activations_and_packed_int4_weights(device):
  """An lhs quantised to fp8 per row (a QArray, or an AsQArray the op quantises) over packed int4 weights: the op
  keeps the weights packed and the heuristics name a kernel of the fp8 x int4 kind; same result as on the unpacked
  weights (which are widened for bf16 kernels), to the rounding of those; the oracle on the dequantised operands.
  Scales per k-block fall back to the unpacked path."""
  rng = np.random.default_rng(12)
  G, k, n, rows = 4, 512, 256, 160
  m = G * rows
  q = torch.tensor(rng.integers(-8, 8, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, 1, n)) / 7 * 0.1).astype(np.float32), device=device)
  int4 = getattr(torch, "int4", torch.int8)
  plain = tokamax_amd.QArray(q, scale, None, int4)
  packed = tokamax_amd.pack_int4(plain)
  x = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device)
  xs = x.abs().amax(dim=1, keepdim=True) / 448
  lhs = tokamax_amd.QArray((x / xs).to(torch.float8_e4m3fn), xs)
  gs = torch.full((G,), rows, dtype=torch.int32, device=device)
  op = tokamax_amd.HipRaggedDot()
  key = _lib_key(op, lhs, packed, gs)
  assert key == (0, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  cfg = op._get_heuristics_config(op.bind(lhs, packed, group_sizes=gs))
  assert cfg.block_k == 128 and cfg.block_m >= 32
  out = op(lhs, packed, group_sizes=gs, preferred_element_type=torch.float32)
  lhs_f = O.e4m3fn_decode(lhs.qvalue.view(torch.uint8).cpu().numpy()).astype(np.float64) * _np(xs)
  want = O.ragged_dot(lhs_f, O.dequantize(q.cpu().numpy(), _np(scale)), np.full(G, rows, np.int32), O.DEFAULT,
                      acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 5e-5)
  ref = op(lhs, plain, group_sizes=gs, preferred_element_type=torch.float32)
  assert O.rel_l2(_np(out), _np(ref)) <= 1e-2  # (the unpacked path rounds scaled operands to bf16)
  # an AsQArray lhs is quantised by the op, then takes the same kernels
  as_q = tokamax_amd.AsQArray(x.to(torch.bfloat16), torch.float8_e4m3fn, channelwise_axes=(0,))
  assert _lib_key(op, as_q, packed, gs) == key
  quantised = as_q.as_qarray()
  out_q = op(as_q, packed, group_sizes=gs, preferred_element_type=torch.float32)
  lhs_q = O.e4m3fn_decode(quantised.qvalue.view(torch.uint8).cpu().numpy()).astype(np.float64) * _np(quantised.scale)
  _check(out_q, O.ragged_dot(lhs_q, O.dequantize(q.cpu().numpy(), _np(scale)), np.full(G, rows, np.int32), O.DEFAULT,
                             acc_dtype=np.float64, out_dtype="f64"), 5e-5)
  # gate-up fusion over the same weights read as [gate | up]: the kernels of the fp8 x int4 kind again
  bound = op.bind(lhs, packed, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
  assert op._problem(bound)[1] == (3, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2) and bound.default_config.block_k == 128
  fused = op(lhs, packed, group_sizes=gs, preferred_element_type=torch.float32, fuse_gateup_activation="silu")
  assert tuple(fused.shape) == (m, n // 2)
  _check(fused, O.ragged_dot_fused(lhs_f, O.dequantize(q.cpu().numpy(), _np(scale)), np.full(G, rows, np.int32),
                                   gateup_activation="silu"), 5e-5)
  # scales per block of 128 k rows on the weights, per row or per (row, same block) on the activations: kernels of
  # the same kind that fold every k-step in with its scales and its own row sums
  scale4 = torch.tensor((rng.uniform(0.5, 1.5, (G, 4, n)) / 7 * 0.1).astype(np.float32), device=device)
  blocks = tokamax_amd.pack_int4(tokamax_amd.QArray(q, scale4, None, int4))
  assert _lib_key(op, lhs, blocks, gs) == (4, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  rhs_f = O.dequantize(q.cpu().numpy(), _np(scale4))
  _check(op(lhs, blocks, group_sizes=gs, preferred_element_type=torch.float32),
         O.ragged_dot(lhs_f, rhs_f, np.full(G, rows, np.int32), O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 5e-5)
  xs4 = torch.tensor(rng.uniform(0.5, 1.5, (m, 4)).astype(np.float32), device=device) * xs
  lhs4 = tokamax_amd.QArray(lhs.qvalue, xs4)
  assert _lib_key(op, lhs4, blocks, gs) == (4, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  lhs4_f = O.dequantize(O.e4m3fn_decode(lhs.qvalue.view(torch.uint8).cpu().numpy()).astype(np.float64), _np(xs4))
  _check(op(lhs4, blocks, group_sizes=gs, preferred_element_type=torch.float32),
         O.ragged_dot(lhs4_f, rhs_f, np.full(G, rows, np.int32), O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 5e-5)
  # blocks of 32 rows: no kernel of this kind; the weights are unpacked and the widened path runs
  small = tokamax_amd.pack_int4(tokamax_amd.QArray(q, scale.expand(G, 16, n).contiguous(), None, int4))
  assert _lib_key(op, lhs, small, gs)[2] != _lib.TKX_I4X2
  _check(op(lhs, small, group_sizes=gs, preferred_element_type=torch.float32), want, 1e-2)


def _lib_key(op, lhs, rhs, gs):
  return op._problem(op.bind(lhs, rhs, group_sizes=gs))[1]


def test_public_op_on_packed_int4_weights(device):
  """`pack_int4` of a quantised rhs: the op keeps it packed, for the streaming kernel with a few rows per group and
  for the tiled kernels with many (the heuristics name them); with a bias or another lhs type it unpacks to int8
  first. Same results as the unpacked QArray: bit for bit where the same kernel contracts in the same order, else to
  the rounding of f32 sums in another order."""
  rng = np.random.default_rng(8)
  G, k, n = 16, 1024, 256
  q = torch.tensor(rng.integers(-7, 8, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, 1, n)) / 7 * 0.1).astype(np.float32), device=device)
  int4 = getattr(torch, "int4", torch.int8)
  plain = tokamax_amd.QArray(q, scale, None, int4)
  packed = tokamax_amd.pack_int4(plain)
  assert packed.packed and packed.shape == (G, k, n) and tuple(packed.qvalue.shape) == (G, k // 2, n)
  op = tokamax_amd.HipRaggedDot()
  for rows in (2, 40):
    gs = torch.full((G,), rows, dtype=torch.int32, device=device)
    lhs = torch.tensor(rng.normal(0, 1, (G * rows, k)).astype(np.float32), device=device).to(torch.bfloat16)
    cfg = op._get_heuristics_config(op.bind(lhs, packed, group_sizes=gs))
    assert (cfg.block_m == 16) == (rows == 2)
    out = op(lhs, packed, group_sizes=gs, preferred_element_type=torch.float32)
    ref = op(lhs, plain, group_sizes=gs, preferred_element_type=torch.float32)
    want = O.ragged_dot(_np(lhs), O.dequantize(q.cpu().numpy(), _np(scale)), np.full(G, rows, np.int32), O.DEFAULT,
                        acc_dtype=np.float64, out_dtype="f64")
    _check(out, want, 1e-5)
    if rows == 2:
      assert torch.equal(out, ref)
    else:
      assert cfg.block_m >= 32 and _lib_key(op, lhs, packed, gs)[2] == _lib.TKX_I4X2
      torch.testing.assert_close(out, ref, rtol=1e-5, atol=1e-5)
  bias = torch.tensor(rng.normal(0, 1, (G, 1, n)).astype(np.float32), device=device)
  gs = torch.full((G,), 2, dtype=torch.int32, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (G * 2, k)).astype(np.float32), device=device).to(torch.bfloat16)
  # (a bias: the tiled kernels still read the bytes)
  torch.testing.assert_close(op(lhs, packed, group_sizes=gs, rhs_bias=bias, preferred_element_type=torch.float32),
                             op(lhs, plain, group_sizes=gs, rhs_bias=bias, preferred_element_type=torch.float32), rtol=1e-5, atol=1e-5)
  # gate-up fusion and scales per block of 256 k rows, with many rows per group: the tiled kernels' forms for them
  gs = torch.full((G,), 40, dtype=torch.int32, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (G * 40, k)).astype(np.float32), device=device).to(torch.bfloat16)
  torch.testing.assert_close(op(lhs, packed, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.float32),
                             op(lhs, plain, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.float32),
                             rtol=1e-5, atol=1e-5)
  scale_k = torch.tensor((rng.uniform(0.5, 1.5, (G, k // 256, n)) / 7 * 0.1).astype(np.float32), device=device)
  plain_k = tokamax_amd.QArray(q, scale_k, None, int4)
  packed_k = tokamax_amd.pack_int4(plain_k)
  assert _lib_key(op, lhs, packed_k, gs)[::2] == (4, _lib.TKX_I4X2)
  out = op(lhs, packed_k, group_sizes=gs, preferred_element_type=torch.float32)
  want = O.ragged_dot(_np(lhs), O.round_to_bf16(O.dequantize(q.cpu().numpy(), _np(scale_k))), np.full(G, 40, np.int32), O.DEFAULT,
                      acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5)
  torch.testing.assert_close(out, op(lhs, plain_k, group_sizes=gs, preferred_element_type=torch.float32), rtol=1e-5, atol=1e-5)


@pytest.mark.parametrize("groups,n", [(128, 768), (8, 512)])
def test_small_m_call_replayed_from_a_captured_graph(groups, n, device):
  """The call path for serving loops: the public op captured into a HIP graph once (after one eager call on the
  capture stream, which creates whatever the op keeps per stream) and replayed with new activations and new group
  sizes written into the captured tensors. Every replay is checked against an eager call, with eager work and
  synchronisations in between. (8 groups x 512 columns takes the split contraction: its arrival counters must be
  back at zero after every replay.)"""
  rng = np.random.default_rng(groups)
  k = 2048
  m = 2 * groups
  q = torch.tensor(rng.integers(-127, 128, (groups, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (groups, 1, n)) / 127).astype(np.float32), device=device)
  rhs = tokamax_amd.QArray(q, scale)
  lhs = torch.zeros((m, k), dtype=torch.bfloat16, device=device)
  gs = torch.zeros((groups,), dtype=torch.int32, device=device)
  op = tokamax_amd.HipRaggedDot()

  def fill(seed):
    r = np.random.default_rng(seed)
    sizes = r.multinomial(m - 3, np.ones(groups) / groups).astype(np.int32)
    lhs.copy_(torch.tensor(r.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16))
    gs.copy_(torch.tensor(sizes, device=device))

  fill(0)
  side = torch.cuda.Stream(device=device)
  side.wait_stream(torch.cuda.current_stream(device))
  with torch.cuda.stream(side):
    op(lhs, rhs, group_sizes=gs, preferred_element_type=torch.bfloat16)
    side.synchronize()
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
      out = op(lhs, rhs, group_sizes=gs, preferred_element_type=torch.bfloat16)
  torch.cuda.current_stream(device).wait_stream(side)
  for seed in (1, 2, 3):
    fill(seed)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    eager = op(lhs, rhs, group_sizes=gs, preferred_element_type=torch.bfloat16)
    assert torch.equal(out, eager), f"replay {seed}"
    assert float(eager.float().abs().sum()) > 0


@pytest.mark.parametrize("dtype,cfg", [
    (torch.bfloat16, (256, 256, 64, 2, 4, 3)), (torch.bfloat16, (256, 256, 32, 2, 4, 4)), (torch.bfloat16, (128, 128, 64, 2, 2, 4)),
    (torch.bfloat16, (64, 128, 64, 2, 2, 4)), (torch.float8_e4m3fn, (128, 256, 128, 2, 4, 3)), (torch.float8_e4m3fn, (256, 256, 128, 2, 4, 2))])
def test_fp8_output_quantised_in_the_epilogue(dtype, cfg, device):
  """tkx_ragged_dot_fwd_fp8_out: values and scales are those of the absmax quantisation (oracle, in the reciprocal
  form of the reference's fused epilogue) of the f32 result of the same kernel, bit for bit; rows of no group are
  zeros with scale 1; ragged groups with an empty one, partial
  tiles at group boundaries and a column count that is not a multiple of the tile."""
  variants = {(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"])
              for v in _lib.variants(0) if v["lhs_dtype"] == hip_ops.dtype_code(dtype)}
  if cfg not in variants:
    pytest.skip("variant not compiled")
  rng = np.random.default_rng(sum(cfg))
  G, m, k, n = 5, 700, 256, 384
  gs = np.array([130, 0, 257, 9, 280], np.int32)  # 676 rows, 24 of no group
  gst = torch.tensor(gs, device=device)
  kc = hip_ops.KernelConfig(*cfg, grid_tile_width=2)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(dtype)
  rhs = torch.tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), device=device).to(dtype)
  ls = rs = None
  if dtype == torch.float8_e4m3fn:
    ls = torch.tensor(rng.uniform(0.5, 1.5, (m, 1)).astype(np.float32), device=device)
    rs = torch.tensor(rng.uniform(0.5, 1.5, (G, 1, n)).astype(np.float32), device=device)
  for act in (None, "silu"):
    q, s = hip_ops.ragged_dot_fwd_fp8_out(lhs, rhs, gst, config=kc, lhs_scale=ls, rhs_scale=rs, activation=act)
    dense = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=kc, out_dtype=torch.float32, lhs_scale=ls, rhs_scale=rs, activation=act)
    wq, wsc = O.quantize_absmax(_np(dense), "fp8", (1, 128), reciprocal=True)  # acc * (1 / scale), as the reference fuses it
    assert np.array_equal(_np(s), wsc), act
    assert np.array_equal(q.view(torch.uint8).cpu().numpy(), wq), act
    assert torch.count_nonzero(q[676:].view(torch.uint8)) == 0 and torch.all(s[676:] == 1)
    # The standalone pass divides: the same scales, and values that differ at most by one fp8 step in a few places
    # (quotients on a rounding boundary).
    q2, s2 = hip_ops.quantize(dense, torch.float8_e4m3fn, (1, 128))
    assert torch.equal(s2, s)
    a, b = q.view(torch.uint8).to(torch.int16), q2.view(torch.uint8).to(torch.int16)
    assert int((a - b).abs().max()) <= 1 and float((a != b).float().mean()) < 2e-3


def test_fp8_output_needs_a_kernel_that_has_it(device):
  lhs = torch.zeros((32, 1024), dtype=torch.bfloat16, device=device)
  rhs = torch.zeros((4, 1024, 128), dtype=torch.bfloat16, device=device)
  gs = torch.full((4,), 8, dtype=torch.int32, device=device)
  with pytest.raises(NotImplementedError, match="cannot quantise"):
    hip_ops.ragged_dot_fwd_fp8_out(lhs, rhs, gs, config=hip_ops.KernelConfig(16, 128, 32, 1, 4, 2))
  with pytest.raises(NotImplementedError, match="128"):
    hip_ops.ragged_dot_fwd_fp8_out(lhs, rhs[:, :, :64].contiguous(), gs, config=hip_ops.KernelConfig(128, 128, 64, 2, 2, 4))


@pytest.mark.parametrize("seed", range(48))
def test_random_shapes_through_the_public_op(seed, device):
  """Seeded random problems (any k and n that are multiples of 8, 1 to 9 groups, empty groups, a tail of rows of no
  group, 0 to ~300 rows per group) through the public entry points with the heuristics' configs: forward and both
  cotangent products against the oracle, rows of no group zero."""
  rng = np.random.default_rng(1000 + seed)
  dtype = (torch.bfloat16, torch.float16, torch.float32)[seed % 3]
  G = int(rng.integers(1, 10))
  k, n = 8 * int(rng.integers(1, 66)), 8 * int(rng.integers(1, 66))
  scale = (1, 8, 60, 300)[int(rng.integers(0, 4))]
  gs = rng.integers(0, scale + 1, G).astype(np.int32)
  gs[rng.random(G) < 0.2] = 0
  m = int(gs.sum()) + int(rng.integers(0, 20))
  if m == 0:
    m, gs[0] = 8, 5
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(dtype)
  rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(dtype)
  dout = torch.tensor(rng.normal(0, 1, (m, n)).astype(np.float32), device=device).to(dtype)
  gst = torch.tensor(gs, device=device)
  count, tol, f32 = int(gs.sum()), TOL[dtype], torch.float32
  out = tokamax_amd.ragged_dot(lhs, rhs, gst, preferred_element_type=f32)
  _check(out, _ref(lhs, rhs, gs), tol)
  assert torch.count_nonzero(out[count:]) == 0
  dlhs = tokamax_amd.ragged_dot_general(dout, rhs, gst, base.TRANS_RHS_RAGGED_DOT_DIM_NUMS, preferred_element_type=f32)
  _check(dlhs, _ref(dout, rhs, gs, O.TRANS_RHS), tol)
  assert torch.count_nonzero(dlhs[count:]) == 0
  drhs = tokamax_amd.ragged_dot_general(lhs, dout, gst, base.RAGGED_CONTRACTING_DOT_DIM_NUMS, preferred_element_type=f32)
  want = _ref(lhs, dout, gs, O.RAGGED_CONTRACTING)
  if np.abs(want).max() > 0:
    _check(drhs, want, tol)
  assert torch.count_nonzero(drhs[torch.tensor(gs == 0, device=device)]) == 0


@pytest.mark.parametrize("seed", range(42))
def test_random_quantised_problems_through_the_public_op(seed, device):
  """Seeded random problems with quantised operands: int8 weights with one scale per (group, column), per k-block or
  per (k-block, 16-column block); int8 x int8 and fp8 x fp8 with per-row / per-column scales; int4 weights packed two
  to a byte with one scale per (group, column) or per k-block. Whatever route the call takes (epilogue scales, scaled
  while widened, folded per k-block, widening pass, streaming kernel, packed bytes read as they are or unpacked first),
  the result is the oracle's contraction of the dequantised operands."""
  rng = np.random.default_rng(5000 + seed)
  kind = ("int8_column", "int8_k_blocks", "int8_tiles", "int8_int8", "fp8_fp8", "int4_column", "int4_k_blocks")[seed % 7]
  G = int(rng.integers(1, 8))
  k, n = 64 * int(rng.integers(1, 9)), 16 * int(rng.integers(1, 30))
  per_group = (2, 40, 200)[int(rng.integers(0, 3))]
  gs = rng.integers(0, per_group + 1, G).astype(np.int32)
  m = int(gs.sum()) + int(rng.integers(0, 9))
  if m == 0:
    m, gs[0] = 4, 3
  gst = torch.tensor(gs, device=device)
  f32 = torch.float32
  tensor = lambda x, dt=f32: torch.tensor(np.asarray(x), device=device).to(dt)
  w8 = rng.integers(-127, 128, (G, k, n)).astype(np.int8)
  if kind in ("int8_column", "int8_k_blocks", "int8_tiles"):
    lhs = tensor(rng.normal(0, 1, (m, k)).astype(np.float32), torch.bfloat16)
    blocks = 1 if kind == "int8_column" else k // 64
    cols = n // 16 if kind == "int8_tiles" else n
    scale = (rng.uniform(0.5, 1.5, (G, blocks, cols)) / 127 * k ** -0.5).astype(np.float32)
    rhs = tokamax_amd.QArray(tensor(w8, torch.int8), tensor(scale))
    lhs_f, rhs_f, tol = _np(lhs), O.dequantize(w8, scale), 2e-3
  elif kind in ("int4_column", "int4_k_blocks"):
    lhs = tensor(rng.normal(0, 1, (m, k)).astype(np.float32), torch.bfloat16)
    w4 = rng.integers(-8, 8, (G, k, n)).astype(np.int8)
    blocks = 1 if kind == "int4_column" else k // 64
    scale = (rng.uniform(0.5, 1.5, (G, blocks, n)) / 7 * k ** -0.5).astype(np.float32)
    rhs = tokamax_amd.pack_int4(tokamax_amd.QArray(tensor(w4, torch.int8), tensor(scale), None, getattr(torch, "int4", torch.int8)))
    assert rhs.packed
    lhs_f, rhs_f, tol = _np(lhs), O.dequantize(w4, scale), 2e-3
  elif kind == "int8_int8":
    a8 = rng.integers(-127, 128, (m, k)).astype(np.int8)
    sa = (rng.uniform(0.5, 1.5, (m, 1)) / 127).astype(np.float32)
    sb = (rng.uniform(0.5, 1.5, (G, 1, n)) / 127 * k ** -0.5).astype(np.float32)
    lhs = tokamax_amd.QArray(tensor(a8, torch.int8), tensor(sa))
    rhs = tokamax_amd.QArray(tensor(w8, torch.int8), tensor(sb))
    lhs_f, rhs_f, tol = O.dequantize(a8, sa), O.dequantize(w8, sb), 2e-3
  else:
    a = tensor(rng.normal(0, 1, (m, k)).astype(np.float32), torch.float8_e4m3fn)
    b = tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), torch.float8_e4m3fn)
    sa = rng.uniform(0.5, 1.5, (m, 1)).astype(np.float32)
    sb = (rng.uniform(0.5, 1.5, (G, 1, n)) * k ** -0.5).astype(np.float32)
    lhs, rhs = tokamax_amd.QArray(a, tensor(sa)), tokamax_amd.QArray(b, tensor(sb))
    lhs_f, rhs_f, tol = _np(a) * sa, _np(b) * sb, 2e-3
  out = tokamax_amd.ragged_dot(lhs, rhs, gst, preferred_element_type=f32)
  want = O.ragged_dot(lhs_f, rhs_f, gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, tol)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0


def test_public_op_picks_the_wide_small_m_kernel_when_it_fills_the_chip(device):
  """64 groups x 2048 columns = 512 workgroups of 256 columns (two per CU): the heuristics name the wide
  streaming kernel, and the public entry's result on it matches the oracle."""
  rng = np.random.default_rng(5)
  G, k, n = 64, 1024, 2048
  gs = rng.integers(0, 5, G).astype(np.int32)
  m = int(gs.sum()) + 3
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, 1, n)) / 127 * 0.1).astype(np.float32), device=device)
  rhs = tokamax_amd.QArray(q, scale)
  gst = torch.tensor(gs, device=device)
  op = tokamax_amd.HipRaggedDot()
  cfg = op._get_heuristics_config(op.bind(lhs, rhs, group_sizes=gst))
  assert (cfg.block_m, cfg.block_n) == (16, 256)
  out = op(lhs, rhs, group_sizes=gst, preferred_element_type=torch.float32)
  want = np.zeros((m, n))
  start = 0
  for g in range(G):  # group by group: the widened weights of all groups at once would take 1 GB
    w = O.dequantize(q[g:g + 1].cpu().numpy(), _np(scale[g:g + 1]))
    rows = slice(start, start + int(gs[g]))
    want[rows] = O.ragged_dot(_np(lhs[rows]), w, gs[g:g + 1], O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
    start += int(gs[g])
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0


@pytest.mark.parametrize("depth", [2, 4])
@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float16])
@pytest.mark.parametrize("case", ["ragged", "two_chunks", "all_empty", "one_big_group"])
def test_small_m_16bit_weight_kernel_edges(case, dtype, depth, device):
  """The streaming small-m kernel on 16-bit weights (no scales): same edge cases as with int8 weights,
  and the public entry picks it for groups of at most 16 rows."""
  rng = np.random.default_rng(len(case) + depth)
  k, n = 2048, 208
  if case == "ragged":
    gs = np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32)
  elif case == "two_chunks":
    gs = rng.integers(0, 4, 70).astype(np.int32)
    gs[[0, 63, 64, 69]] = [0, 2, 0, 5]
  elif case == "all_empty":
    gs = np.zeros(5, np.int32)
  else:
    gs = np.array([0, 45, 0], np.int32)
  G, m = len(gs), int(gs.sum()) + 11
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(dtype)
  rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(dtype)
  gst = torch.tensor(gs, device=device)
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth)
  out = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32)
  want = O.ragged_dot(_np(lhs), _np(rhs), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-5)  # f32 output of exact 16-bit products
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  out16 = hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=dtype)
  assert torch.equal(out16, out.to(dtype))
  assert torch.equal(out, hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=cfg, out_dtype=torch.float32))
  if case == "ragged" and depth == 2:
    op = tokamax_amd.HipRaggedDot()
    small = np.array([3, 0, 0, 7, 1, 0, 6, 2], np.int32)
    assert op._get_heuristics_config(op.bind(lhs[:19], rhs, group_sizes=torch.tensor(small, device=device))).block_m == 16
    _check(op(lhs[:19], rhs, group_sizes=torch.tensor(small, device=device), preferred_element_type=torch.float32),
           O.ragged_dot(_np(lhs[:19]), _np(rhs), small, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 1e-5)


@pytest.mark.parametrize("act", ["silu", "gelu"])
@pytest.mark.parametrize("m,k,n2,gs", [
    (300, 256, 512, [100, 0, 57, 120]),          # ragged groups, an empty one, a tail of 23 rows
    (64, 128, 144, [5, 7, 0, 40]),               # n' = 72: not a multiple of the tile's 128 output columns
    (1100, 512, 1024, [1024, 0, 76]),            # a group of several 256-row tasks
])
def test_rhs_bias_and_gateup_fusion(m, k, n2, gs, act, device):
  """`rhs_bias` and `fuse_gateup_activation` through the op (base.py:205-217) against the oracle's
  composition; bf16 inputs, f32 and bf16 outputs; the bias alone, with and without an activation."""
  rng = np.random.default_rng(m + n2)
  gs = np.array(gs, np.int32)
  G = len(gs)
  gst = torch.tensor(gs, device=device)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device)
  lhs, rhs = mk((m, k), 1.0).to(torch.bfloat16), mk((G, k, n2), k ** -0.5).to(torch.bfloat16)
  bias = mk((G, 1, n2), 0.7).to(torch.bfloat16)
  op = tokamax_amd.HipRaggedDot()
  out = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation=act, preferred_element_type=torch.float32)
  want = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, rhs_bias=_np(bias), gateup_activation=act)
  assert out.shape == (m, n2 // 2)
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  out16 = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation=act)
  assert out16.dtype == torch.bfloat16
  _check(out16, want, 2e-3)
  # without a bias
  _check(op(lhs, rhs, group_sizes=gst, fuse_gateup_activation=act, preferred_element_type=torch.float32),
         O.ragged_dot_fused(_np(lhs), _np(rhs), gs, gateup_activation=act), 1e-5)
  # the bias alone, and under a fused activation
  plain = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, rhs_bias=_np(bias))
  _check(op(lhs, rhs, group_sizes=gst, rhs_bias=bias, preferred_element_type=torch.float32), plain, 1e-5)
  got = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, activation=torch.nn.functional.silu,
           preferred_element_type=torch.float32)
  _check(got, O.silu(plain), 1e-5)
  with pytest.raises(NotImplementedError):
    op(lhs, rhs, group_sizes=gst, fuse_gateup_activation="relu")


@pytest.mark.parametrize("blocks", [1, 4])
def test_gateup_fusion_over_int8_weights(blocks, device):
  """Gate-up fusion with quantised weights (the reference's gmm_v2 test crosses `fuse_act` with `use_weight_scale`,
  experimental/gmm_v2/gmm_v2_test.py:1158-1166): one scale per (group, column) runs on gate-up variants of the
  int8-weight kernels; scales per k-block go through the widening pass and the bf16 gate-up kernels."""
  rng = np.random.default_rng(13 + blocks)
  m, k, n2 = 300, 256, 512
  gs = np.array([100, 0, 57, 120], np.int32)
  G = len(gs)
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-127, 128, (G, k, n2)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, blocks, n2)) * k ** -0.5 / 127 * 2).astype(np.float32), device=device)
  bias = torch.tensor(rng.normal(0, 0.7, (G, 1, n2)).astype(np.float32), device=device).to(torch.bfloat16)
  rhs = tokamax_amd.QArray(q, scale)
  op = tokamax_amd.HipRaggedDot()
  want = O.ragged_dot_fused(_np(lhs), O.dequantize(q.cpu().numpy(), _np(scale)), gs, rhs_bias=_np(bias),
                            gateup_activation="silu")
  out = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation="silu", preferred_element_type=torch.float32)
  assert out.shape == (m, n2 // 2)
  _check(out, want, 1e-5 if blocks == 1 else 4e-3)  # (widened weights are rounded to bf16)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  # the raw-array form of the same call
  out2 = op(lhs, q, group_sizes=gst, rhs_scale=scale.reshape(G, blocks, 1, n2), rhs_bias=bias, fuse_gateup_activation="silu",
            preferred_element_type=torch.float32)
  assert torch.equal(out, out2)


@pytest.mark.parametrize("act", ["swigluoai", "silu_and_mul_with_clamp", "gelu_tanh"])
def test_clamped_gateup_forms(act, device):
  """The clamped gate-up forms (experimental/gmm_v2/gmm_v2.py:29-50) through the op, on products wide
  enough (standard deviation 6) that a good part of the gates and ups lies past the limits of 7 and 10;
  the C ABI declines them outside gate-up fusion."""
  rng = np.random.default_rng(17)
  m, k, n2 = 300, 256, 512
  gs = np.array([100, 0, 57, 120], np.int32)
  G = len(gs)
  gst = torch.tensor(gs, device=device)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device)
  lhs, rhs = mk((m, k), 1.0).to(torch.bfloat16), mk((G, k, n2), 6.0 * k ** -0.5).to(torch.bfloat16)
  bias = mk((G, 1, n2), 2.0).to(torch.bfloat16)
  op = tokamax_amd.HipRaggedDot()
  tmp = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, rhs_bias=_np(bias))[:int(gs.sum())]
  assert (np.abs(tmp) > 10).mean() > 0.05 and (np.abs(tmp) < 7).mean() > 0.5  # both sides of the limits are hit
  want = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, rhs_bias=_np(bias), gateup_activation=act)
  out = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation=act, preferred_element_type=torch.float32)
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  _check(op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation=act), want, 2e-3)
  if act != "gelu_tanh":
    cfg = op._get_heuristics_config(op.bind(lhs, rhs, group_sizes=gst))
    kc = hip_ops.KernelConfig(cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages)
    with pytest.raises(ValueError, match="gate-up"):
      hip_ops.ragged_dot_fwd(lhs, rhs, gst, config=kc, out_dtype=torch.float32, activation=act, rhs_bias=bias.float())


@pytest.mark.parametrize("offset,local", [(0, 6), (2, 3), (4, 2), (5, 3), (-1, 3), (7, 2)])
def test_group_offset_tiled_kernels(offset, local, device):
  """`group_offset` (experimental/gmm_v2/gmm_v2_test.py:44-101) through the op on the tiled kernels: rhs and
  rhs_bias hold `local` of the 6 groups, starting at `offset` (also past either end of the sizes); the rows
  of the other groups and the rows of no group are zero; with and without gate-up fusion."""
  rng = np.random.default_rng(40 + offset)
  gs = np.array([100, 0, 57, 120, 3, 260], np.int32)
  m, k, n2 = int(gs.sum()) + 20, 256, 512
  gst = torch.tensor(gs, device=device)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device)
  lhs, rhs = mk((m, k), 1.0).to(torch.bfloat16), mk((local, k, n2), k ** -0.5).to(torch.bfloat16)
  bias = mk((local, 1, n2), 0.7).to(torch.bfloat16)
  goff = torch.tensor([offset], dtype=torch.int32, device=device)
  op = tokamax_amd.HipRaggedDot()
  for act in (None, "silu"):
    want = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, rhs_bias=_np(bias), gateup_activation=act, group_offset=[offset])
    out = op(lhs, rhs, group_sizes=gst, rhs_bias=bias, fuse_gateup_activation=act, group_offset=goff,
             preferred_element_type=torch.float32)
    if np.any(want):
      _check(out, want, 1e-5)
    assert torch.equal(out == 0, torch.tensor(want == 0, device=device))  # the same rows are exactly zero
  # without a bias, bf16 out, and the offset as a plain int
  want = O.ragged_dot_fused(_np(lhs), _np(rhs), gs, group_offset=[offset])
  out = op(lhs, rhs, group_sizes=gst, group_offset=offset)
  if np.any(want):
    _check(out, want, 2e-3)
  assert torch.count_nonzero(out[torch.tensor(~want.any(axis=1), device=device)]) == 0
  with pytest.raises(NotImplementedError):  # the public entry declines it, as api.py:183-184 does
    tokamax_amd.ragged_dot(lhs, rhs, gst, group_offset=goff)


def test_group_offset_shards_add_up_and_follow_the_device_value(device):
  """Four expert-parallel shards of 8 experts (2 each) of one job add up to the unsharded result: bit for bit in f32
  under one fixed tile configuration without a split last round (every row is computed by exactly one shard, by the
  same kernel), and to f32 rounding under the configurations the heuristics choose per call (a launch of few tiles
  has its last round split along the contraction, and the shards' launches are smaller than the whole job's); the
  offset is read on the device, so one tensor updated in place serves all four calls."""
  rng = np.random.default_rng(8)
  G, k, n = 8, 512, 1024
  gs = rng.multinomial(1500, [1 / G] * G).astype(np.int32)
  m = int(gs.sum()) + 36
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
  goff = torch.zeros(1, dtype=torch.int32, device=device)
  for op in (tokamax_amd.HipRaggedDot(config=hip.Config(128, 256, 64, 2, 4, 3)), tokamax_amd.HipRaggedDot()):
    full = op(lhs, rhs, group_sizes=gst, preferred_element_type=torch.float32)
    total = torch.zeros_like(full)
    for shard in range(4):
      goff.fill_(2 * shard)
      part = op(lhs, rhs[2 * shard:2 * shard + 2], group_sizes=gst, group_offset=goff, preferred_element_type=torch.float32)
      rows = slice(int(gs[:2 * shard].sum()), int(gs[:2 * shard + 2].sum()))
      assert torch.count_nonzero(part[:rows.start]) == 0 and torch.count_nonzero(part[rows.stop:]) == 0
      total += part
    if op.config is not None:
      assert torch.equal(total, full)
    else:
      assert O.rel_l2(_np(total), _np(full)) <= 1e-6


@pytest.mark.parametrize("block_n,split_k", [(128, 1), (256, 1), (128, 2), (128, 4), (128, -1), (128, -2)])
@pytest.mark.parametrize("offset,local", [(0, 9), (3, 4), (7, 4), (-2, 5)])
def test_group_offset_small_m_kernel(offset, local, block_n, split_k, device):
  """`group_offset` in the streaming small-m kernel (int8 weights), also with the contraction split over workgroups
  and in the persistent form (split_k -1 here; -2: with no group above 16 rows, so that empty groups' workgroups help):
  the kernel derives its row ranges from the job's sizes and the device-side offset; rows of other groups are zero."""
  rng = np.random.default_rng(60 + offset)
  gs = np.array([3, 0, 5, 17, 1, 0, 16, 2, 4], np.int32)
  if split_k == -2:
    gs[3] = 12
  k, n = 1024, 464
  m = int(gs.sum()) + 5
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  rhs = torch.tensor(rng.integers(-128, 128, (local, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((np.abs(rng.normal(0, 0.01, (local, 1, n))) + 1e-3).astype(np.float32), device=device)
  cfg = hip_ops.KernelConfig(16, block_n, 32, 1, 4, 2, split_k=max(split_k, 1), persistent=int(split_k < 0))
  goff = torch.tensor([offset], dtype=torch.int32, device=device)
  out = hip_ops.ragged_dot_fwd(lhs, rhs, torch.tensor(gs, device=device), config=cfg, out_dtype=torch.float32,
                               rhs_scale=scale, group_offset=goff)
  want = O.ragged_dot_fused(_np(lhs), O.dequantize(rhs.cpu().numpy(), _np(scale)), gs, group_offset=[offset])
  _check(out, want, 1e-5)
  assert torch.equal(out == 0, torch.tensor(want == 0, device=device))


def test_raw_rhs_scale_argument(device):
  """The `rhs_scale` argument of RaggedDot (base.py:208; shape [g, k-blocks, 1, n] with raw int8 weights,
  experimental/gmm_v2/gmm_v2.py:1193-1199) gives what the same weights give as a QArray; the result defaults
  to lhs.dtype."""
  rng = np.random.default_rng(12)
  G, m, k, n = 4, 300, 256, 512
  gs = np.array([100, 0, 80, 110], np.int32)
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
  op = tokamax_amd.HipRaggedDot()
  for blocks in (1, 4):
    scale = torch.tensor((rng.uniform(0.5, 1.5, (G, blocks, n)) / 127 * 0.1).astype(np.float32), device=device)
    out = op(lhs, q, group_sizes=gst, rhs_scale=scale.reshape(G, blocks, 1, n))
    assert out.dtype == torch.bfloat16
    assert torch.equal(out, op(lhs, tokamax_amd.QArray(q, scale), group_sizes=gst, preferred_element_type=torch.bfloat16))
    _check(out, O.ragged_dot(_np(lhs), O.dequantize(q.cpu().numpy(), _np(scale)), gs, acc_dtype=np.float64, out_dtype="f64"),
           3e-3)
  with pytest.raises(NotImplementedError):
    op(lhs, q, group_sizes=gst, rhs_scale=scale)  # not [g, blocks, 1, n]
  # permissions the kernels do not use: lhs stays unquantised, rows of no group are zeroed anyway
  again = op(lhs, q, group_sizes=gst, rhs_scale=scale.reshape(G, blocks, 1, n), maybe_quantize_lhs=True, zero_initialize=False)
  assert torch.equal(again, out)
  with pytest.raises(NotImplementedError):
    op(lhs, q, group_sizes=gst, rhs_scale=scale.reshape(G, blocks, 1, n), lhs_quantization_dtype=torch.int8)


@pytest.mark.parametrize("qdtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("rows,cols,t_r,t_c", [(96, 256, 1, 128), (96, 256, 1, 256), (512, 128, 64, 1), (512, 256, 128, 128),
                                               (40, 48, 8, 16)])
def test_dequantize_kernel_bit_exact(rows, cols, t_r, t_c, qdtype, device):
  """`tkx_dequantize`: int8 / fp8 values times block scales, rounded to bf16 -- bit for bit the oracle's
  dequantisation (quantization.py:80-83) rounded to bf16 (one f32 multiply, one rounding)."""
  rng = np.random.default_rng(rows + t_c)
  if qdtype == torch.int8:
    q = torch.tensor(rng.integers(-128, 128, (rows, cols)).astype(np.int8), device=device)
    qf = q.cpu().numpy()
  else:
    q = torch.tensor(rng.integers(0, 256, (rows, cols)).astype(np.uint8), device=device)
    q = torch.where((q & 0x7f) == 0x7f, torch.zeros_like(q), q).view(torch.float8_e4m3fn)  # no NaN codes
    qf = O.e4m3fn_decode(q.view(torch.uint8).cpu().numpy())
  scale = torch.tensor(rng.uniform(0.01, 2.0, (rows // t_r, cols // t_c)).astype(np.float32), device=device)
  got = hip_ops.dequantize(q, scale)
  want = O.round_to_bf16(O.dequantize(qf, _np(scale)))
  np.testing.assert_array_equal(_np(got), want)
  # weights [g, k, n] with scale [g, k/t_k, n/t_n] are the same pass over g * k rows
  if rows % (2 * t_r) == 0:
    got3 = hip_ops.dequantize(q.view(2, rows // 2, cols), scale.view(2, -1, cols // t_c))
    np.testing.assert_array_equal(_np(got3).reshape(rows, cols), want)


@pytest.mark.parametrize("case", ["fp8_blocks_128", "fp8_row_x_k_blocks", "fp8_k_sub", "int8_k_sub", "int8_row_col"])
def test_k_subchannel_scales_through_widening(case, device):
  """Scales that change along the contraction on both operands -- the fp8 recipe with [m, k/128] and
  [g, k/128, n/128] scales, and the int8 activation form acc += (x_q . w_q) xs[row, k_sub] ws[g, k_sub, n]
  (pallas_mosaic_gpu_kernel_sm100_i8_quant.py:51-102) -- go through the widening pass and the bf16 (or
  bf16 x int8) kernels; the oracle contracts the dequantised operands in f64."""
  rng = np.random.default_rng(len(case))
  G, m, k, n = 4, 300, 512, 256
  gs = np.array([100, 0, 80, 110], np.int32)
  gst = torch.tensor(gs, device=device)
  def quantised(shape, qdtype, scale_shape, spread):
    if qdtype == torch.int8:
      q = torch.tensor(rng.integers(-127, 128, shape).astype(np.int8), device=device)
      qf = q.cpu().numpy().astype(np.float64)
    else:
      q = torch.tensor(rng.normal(0, 1.0, shape).astype(np.float32), device=device).to(torch.float8_e4m3fn)
      qf = O.e4m3fn_decode(q.view(torch.uint8).cpu().numpy()).astype(np.float64)
    scale = torch.tensor((rng.uniform(0.5, 1.5, scale_shape) * spread).astype(np.float32), device=device)
    return tokamax_amd.QArray(q, scale), O.dequantize(qf, _np(scale))
  f8, i8 = torch.float8_e4m3fn, torch.int8
  lhs_spec, rhs_spec = {
      "fp8_blocks_128": (((m, k), f8, (m, k // 128), 1.0), ((G, k, n), f8, (G, k // 128, n // 128), k ** -0.5)),
      "fp8_row_x_k_blocks": (((m, k), f8, (m, 1), 1.0), ((G, k, n), f8, (G, k // 128, n), k ** -0.5)),
      # (the same k-blocks on both sides: the fp8 MFMA kernel that folds the scales in after every k-block)
      "fp8_k_sub": (((m, k), f8, (m, k // 128), 1.0), ((G, k, n), f8, (G, k // 128, n), k ** -0.5)),
      "int8_k_sub": (((m, k), i8, (m, k // 64), 1 / 127), ((G, k, n), i8, (G, k // 64, n), k ** -0.5 / 127)),
      "int8_row_col": (((m, k), i8, (m, 1), 1 / 127), ((G, k, n), i8, (G, 1, n), k ** -0.5 / 127)),
  }[case]
  lhs, lhs_f = quantised(*lhs_spec)
  rhs, rhs_f = quantised(*rhs_spec)
  out = tokamax_amd.ragged_dot(lhs, rhs, gst, preferred_element_type=torch.float32)
  want = O.ragged_dot(lhs_f, rhs_f, gs, acc_dtype=np.float64, out_dtype="f64")
  count = int(gs.sum())
  _check(out, want, TOL["fp8"], rows=count)
  assert O.rel_l2(_np(out)[:count], want[:count]) < 6e-3  # two operands rounded to bf16, f32 accumulation
  assert torch.count_nonzero(out[count:]) == 0


@pytest.mark.parametrize("blocks", [1, 4])
@pytest.mark.parametrize("depth", [2, 4])
def test_small_m_kernel_fp8_weights(blocks, depth, device):
  """The streaming small-m kernel on fp8 (e4m3fn) weights: one scale per (group, column) in the epilogue (an fp8
  value is a bf16 value exactly, so the f32 result is exact up to accumulation order), or per k-block while the
  weights are widened; the public entry picks it for groups of a few rows."""
  rng = np.random.default_rng(30 + blocks + depth)
  gs = np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32)
  G, k, n = len(gs), 1024, 208
  m = int(gs.sum()) + 11
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
  qf = O.e4m3fn_decode(q.view(torch.uint8).cpu().numpy()).astype(np.float64)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, blocks, n)) * k ** -0.5).astype(np.float32), device=device)
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth)
  out = hip_ops.ragged_dot_fwd(lhs, q, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  if blocks == 1:
    want = O.ragged_dot(_np(lhs), O.dequantize(qf, _np(scale)), gs, acc_dtype=np.float64, out_dtype="f64")
    _check(out, want, 1e-5)
  else:  # weight x scale rounded to bf16
    want = O.ragged_dot(_np(lhs), O.round_to_bf16(O.dequantize(qf, _np(scale))), gs, acc_dtype=np.float64, out_dtype="f64")
    _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  if depth == 2:
    op = tokamax_amd.HipRaggedDot()
    small = np.array([3, 0, 0, 7, 1, 0, 6, 2], np.int32)
    rhs = tokamax_amd.QArray(q, scale)
    sgt = torch.tensor(small, device=device)
    assert op._get_heuristics_config(op.bind(lhs[:19], rhs, group_sizes=sgt)).block_m == 16
    got = op(lhs[:19], rhs, group_sizes=sgt, preferred_element_type=torch.float32)
    _check(got, O.ragged_dot(_np(lhs[:19]), O.dequantize(qf, _np(scale)), small, acc_dtype=np.float64, out_dtype="f64"), 4e-3)
    # an fp8 lhs with scales per (row, k-block) is widened for the same kernel (20 rows: a multiple of 4)
    a8 = torch.tensor(rng.normal(0, 1, (20, k)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
    xs = torch.tensor(rng.uniform(0.5, 1.5, (20, blocks)).astype(np.float32), device=device)
    lq = tokamax_amd.QArray(a8, xs)
    # (with one scale per row and per column the pair stays on the fp8 MFMA kernels)
    assert (op._get_heuristics_config(op.bind(lq, rhs, group_sizes=sgt)).block_m == 16) == (blocks > 1)
    got = op(lq, rhs, group_sizes=sgt, preferred_element_type=torch.float32)
    lhs_f = O.dequantize(O.e4m3fn_decode(a8.view(torch.uint8).cpu().numpy()).astype(np.float64), _np(xs))
    _check(got, O.ragged_dot(lhs_f, O.dequantize(qf, _np(scale)), small, acc_dtype=np.float64, out_dtype="f64"), 6e-3,
           rows=int(small.sum()))


def test_bf16_activations_fp8_weights(device):
  """bf16 x fp8 (e4m3fn) weights with one scale per (group, column) or per (group, 128 k rows, column): the kernels
  that scale the weights while they widen them; an fp8 lhs with row scales is widened first for them."""
  rng = np.random.default_rng(21)
  G, m, k, n = 4, 300, 512, 256
  gs = np.array([100, 0, 80, 110], np.int32)
  gst = torch.tensor(gs, device=device)
  count = int(gs.sum())
  a16 = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
  qf = O.e4m3fn_decode(q.view(torch.uint8).cpu().numpy()).astype(np.float64)
  op = tokamax_amd.HipRaggedDot()
  for blocks in (1, k // 128):
    scale = torch.tensor((rng.uniform(0.5, 1.5, (G, blocks, n)) * k ** -0.5).astype(np.float32), device=device)
    rhs = tokamax_amd.QArray(q, scale)
    cfg = op._get_heuristics_config(op.bind(a16, rhs, group_sizes=gst))
    assert cfg.block_n == 256 and cfg.block_m != 16
    out = tokamax_amd.ragged_dot(a16, rhs, gst, preferred_element_type=torch.float32)
    want = O.ragged_dot(_np(a16), O.dequantize(qf, _np(scale)), gs, acc_dtype=np.float64, out_dtype="f64")
    _check(out, want, 4e-3, rows=count)  # weight x scale rounded to bf16
    assert torch.count_nonzero(out[count:]) == 0
  a8 = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
  a_scale = torch.tensor(rng.uniform(0.5, 1.5, (m, 1)).astype(np.float32), device=device)
  lhs_f = O.dequantize(O.e4m3fn_decode(a8.view(torch.uint8).cpu().numpy()).astype(np.float64), _np(a_scale))
  out = tokamax_amd.ragged_dot(tokamax_amd.QArray(a8, a_scale), rhs, gst, preferred_element_type=torch.float32)
  _check(out, O.ragged_dot(lhs_f, O.dequantize(qf, _np(scale)), gs, acc_dtype=np.float64, out_dtype="f64"), 6e-3, rows=count)


@pytest.mark.parametrize("qdtype", [torch.float8_e4m3fn, torch.int8])
def test_per_tensor_scales(qdtype, device):
  """One scale per tensor on both operands (scale shapes [1,1] and [1,1,1]), the plainest fp8 / int8 recipe: the
  scales are repeated per row and per (group, column) and the pair runs on the fp8 / int8 MFMA kernels."""
  rng = np.random.default_rng(31)
  G, m, k, n = 4, 300, 512, 256
  gs = np.array([100, 0, 80, 110], np.int32)
  gst = torch.tensor(gs, device=device)
  if qdtype == torch.int8:
    a = torch.tensor(rng.integers(-127, 128, (m, k)).astype(np.int8), device=device)
    b = torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device)
    af, bf = a.cpu().numpy().astype(np.float64), b.cpu().numpy().astype(np.float64)
  else:
    a = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(qdtype)
    b = torch.tensor(rng.normal(0, 1, (G, k, n)).astype(np.float32), device=device).to(qdtype)
    af = O.e4m3fn_decode(a.view(torch.uint8).cpu().numpy()).astype(np.float64)
    bf = O.e4m3fn_decode(b.view(torch.uint8).cpu().numpy()).astype(np.float64)
  sa, sb = torch.full((1, 1), 0.037, device=device), torch.full((1, 1, 1), 0.0021, device=device)
  op = tokamax_amd.HipRaggedDot()
  lhs, rhs = tokamax_amd.QArray(a, sa), tokamax_amd.QArray(b, sb)
  key = op._problem(op.bind(lhs, rhs, group_sizes=gst))[1]
  assert key[1] == key[2] == hip_ops.dtype_code(qdtype)  # nothing is widened
  out = op(lhs, rhs, group_sizes=gst, preferred_element_type=torch.float32)
  want = O.ragged_dot(af * 0.037, bf * 0.0021, gs, acc_dtype=np.float64, out_dtype="f64")
  _check(out, want, 1e-4, rows=int(gs.sum()))


def test_int4_values_in_int8_storage(device):
  """fp8 x int4 with scale tile (1, 128, 1) (pallas_mosaic_gpu_kernel_sm100_fp8_quant.py:266-350) and bf16 x int4:
  torch holds int4 values in int8 storage (qtype says int4); they run as int8."""
  rng = np.random.default_rng(3)
  G, m, k, n = 4, 300, 512, 256
  gs = np.array([100, 0, 80, 110], np.int32)
  gst = torch.tensor(gs, device=device)
  q = torch.tensor(rng.integers(-8, 8, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((rng.uniform(0.5, 1.5, (G, k // 128, n)) * k ** -0.5 / 7).astype(np.float32), device=device)
  rhs = tokamax_amd.QArray(q, scale, qtype=torch.int4)
  rhs_f = O.dequantize(q.cpu().numpy().astype(np.float64), _np(scale))
  count = int(gs.sum())
  a16 = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  out = tokamax_amd.ragged_dot(a16, rhs, gst, preferred_element_type=torch.float32)
  _check(out, O.ragged_dot(_np(a16), rhs_f, gs, acc_dtype=np.float64, out_dtype="f64"), TOL["int8"], rows=count)
  a8 = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.float8_e4m3fn)
  a_scale = torch.tensor(rng.uniform(0.5, 1.5, (m, 1)).astype(np.float32), device=device)
  lhs_f = O.dequantize(O.e4m3fn_decode(a8.view(torch.uint8).cpu().numpy()).astype(np.float64), _np(a_scale))
  out = tokamax_amd.ragged_dot(tokamax_amd.QArray(a8, a_scale), rhs, gst, preferred_element_type=torch.float32)
  _check(out, O.ragged_dot(lhs_f, rhs_f, gs, acc_dtype=np.float64, out_dtype="f64"), TOL["fp8"], rows=count)


@pytest.mark.parametrize("m,blocks", [(300, 4), (24, 8), (1100, 2)])
def test_int8_weights_with_sub_channel_scales(m, blocks, device):
  """Scale tile (1, t_k, 1) with t_k < k (pallas_mosaic_gpu_kernel_sm90_quant.py:91-97): the weights are
  widened to bf16 by `tkx_dequantize_weights` (bit-exact against the oracle's dequantisation rounded to
  bf16) and the result matches the oracle on the dequantised weights."""
  rng = np.random.default_rng(m + blocks)
  G, k, n = 5, 1024, 208
  gs = rng.multinomial(m - 7, [0.3, 0.0, 0.4, 0.1, 0.2]).astype(np.int32)
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((np.abs(rng.normal(0, 0.01, (G, blocks, n))) + 1e-3).astype(np.float32), device=device)
  deq = O.dequantize(q.cpu().numpy(), _np(scale))
  wide = hip_ops.dequantize_weights(q, scale)
  assert wide.dtype == torch.bfloat16 and np.array_equal(_np(wide), O.round_to_bf16(deq.astype(np.float32)))
  out = tokamax_amd.HipRaggedDot()(lhs, tokamax_amd.QArray(q, scale), group_sizes=gst, preferred_element_type=torch.float32)
  _check(out, O.ragged_dot(_np(lhs), _np(wide), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 1e-5)
  _check(out, O.ragged_dot(_np(lhs), deq, gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 3e-2)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  with pytest.raises(NotImplementedError):  # a scale that does not tile k
    tokamax_amd.HipRaggedDot()(lhs, tokamax_amd.QArray(q, torch.ones(G, 3, n, device=device)), group_sizes=gst)


@pytest.mark.parametrize("blocks,depth", [(2, 2), (8, 2), (32, 4), (4, 8)])
def test_small_m_int8_kernel_with_sub_channel_scales(blocks, depth, device):
  """The streaming small-m kernel scales int8 weights per k-block while it widens them: same result as
  the oracle on the weights dequantised and rounded to bf16; the op picks this path for small groups."""
  rng = np.random.default_rng(blocks)
  k, n = 1024, 208
  gs = np.array([3, 0, 0, 17, 1, 0, 16, 2], np.int32)
  G, m = len(gs), int(gs.sum()) + 5
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
  scale = torch.tensor((np.abs(rng.normal(0, 0.01, (G, blocks, n))) + 1e-3).astype(np.float32), device=device)
  wide = O.round_to_bf16(O.dequantize(q.cpu().numpy(), _np(scale)).astype(np.float32))
  want = O.ragged_dot(_np(lhs), wide, gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, depth)
  out = hip_ops.ragged_dot_fwd(lhs, q, gst, config=cfg, out_dtype=torch.float32, rhs_scale=scale)
  _check(out, want, 1e-5)
  assert torch.count_nonzero(out[int(gs.sum()):]) == 0
  with pytest.raises(NotImplementedError):  # the tiled kernels take one scale per (group, column)
    hip_ops.ragged_dot_fwd(lhs, q, gst, config=hip_ops.KernelConfig(32, 128, 64, 1, 4, 4), out_dtype=torch.float32,
                           rhs_scale=scale)
  op = tokamax_amd.HipRaggedDot()
  small = np.array([3, 0, 0, 7, 1, 0, 6, 2], np.int32)
  sgs = torch.tensor(small, device=device)
  assert op.bind(lhs[:19], tokamax_amd.QArray(q, scale), group_sizes=sgs).default_config.block_m == 16
  _check(op(lhs[:19], tokamax_amd.QArray(q, scale), group_sizes=sgs, preferred_element_type=torch.float32),
         O.ragged_dot(_np(lhs[:19]), wide, small, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64"), 1e-5)


@pytest.mark.parametrize("dtype", [torch.bfloat16])
@pytest.mark.parametrize("shape", [((3, 70), 256, 192), ((1100,), 512, 1024), ((2, 2, 9), 128, 72)])
def test_gated_linear_unit(shape, dtype, device):
  """`gated_linear_unit` (gated_linear_unit/base.py:60-120) = the gate-up fused kernel with one group:
  fused and unfused weights, the in-kernel activations, no activation, and a callable with no
  in-kernel twin."""
  lead, k, n = shape
  rng = np.random.default_rng(k + n)
  x = torch.tensor(rng.normal(0, 1, (*lead, k)).astype(np.float32), device=device).to(dtype)
  w = torch.tensor(rng.normal(0, k ** -0.5, (k, 2, n)).astype(np.float32), device=device).to(dtype)
  F = torch.nn.functional
  acts = [(F.silu, O.silu), (torch.sigmoid, lambda v: 1 / (1 + np.exp(-v))), (torch.relu, lambda v: np.maximum(v, 0)),
          (torch.tanh, np.tanh), (None, None), (F.softplus, lambda v: np.log1p(np.exp(v)))]
  for act, ref_act in acts:
    out = tokamax_amd.gated_linear_unit(x, w, activation=act)
    assert out.shape == (*lead, n) and out.dtype == dtype
    _check(out, O.gated_linear_unit(_np(x), _np(w), ref_act), 3e-3)
  pair = (w[:, 0].contiguous(), w[:, 1].contiguous())
  assert torch.equal(tokamax_amd.gated_linear_unit(x, pair, activation=F.silu), tokamax_amd.gated_linear_unit(x, w, activation=F.silu))
  with pytest.raises(NotImplementedError):
    tokamax_amd.gated_linear_unit(x, w.float(), activation=F.silu)


@pytest.mark.parametrize("dtype", [torch.bfloat16, torch.float32, torch.float16])
def test_row_movement_ops(dtype, device):
  """ragged_gather, ragged_scatter (bit-exact copies / zeros) and ragged_gather_reduce (f32 sums, one
  rounding) against the oracle; the token permute -> ragged dot -> weighted un-permute round trip."""
  rng = np.random.default_rng(21)
  rows, hidden, n_out, R = 300, 264, 1040, 4
  x = torch.tensor(rng.normal(0, 1, (rows, hidden)).astype(np.float32), device=device).to(dtype)
  idx = torch.tensor(rng.integers(0, rows, n_out).astype(np.int32), device=device)
  got = tokamax_amd.ragged_gather(x, idx, torch.tensor([0], device=device), torch.tensor([rows], device=device))
  assert torch.equal(got, x[idx.long()])
  start, end = 40, 211
  got = tokamax_amd.ragged_scatter(x, idx, torch.tensor([start], device=device), torch.tensor(end, device=device))
  want = O.ragged_scatter(_np(x), idx.cpu().numpy(), start, end)
  assert np.array_equal(_np(got), want)
  w = torch.tensor(rng.uniform(0, 1, n_out).astype(np.float32), device=device)
  valid = torch.tensor(rng.integers(0, 4, n_out) > 0, device=device)
  got = tokamax_amd.ragged_gather_reduce(x, idx, w, valid, R)
  want = O.ragged_gather_reduce(_np(x), idx.cpu().numpy(), _np(w), valid.cpu().numpy(), R)
  assert got.shape == (n_out // R, hidden) and got.dtype == dtype
  _check(got, want, 1e-6 if dtype == torch.float32 else 3e-3)
  got = tokamax_amd.ragged_gather_reduce(x, idx, w, valid, 13)  # more rows per output row than the kernel keeps in registers
  _check(got, O.ragged_gather_reduce(_np(x), idx.cpu().numpy(), _np(w), valid.cpu().numpy(), 13),
         1e-6 if dtype == torch.float32 else 3e-3)
  if dtype == torch.float32:
    return
  # MoE round trip: sort tokens by expert, ragged dot, weighted top-2 combine
  tokens, k, n, G = 64, 128, 256, 4
  h = torch.tensor(rng.normal(0, 1, (tokens, k)).astype(np.float32), device=device).to(dtype)
  wts = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(dtype)
  expert = torch.tensor(np.stack([rng.permutation(G)[:2] for _ in range(tokens)]).astype(np.int64), device=device)
  flat = expert.reshape(-1)
  order = torch.argsort(flat, stable=True)
  gs = torch.bincount(flat, minlength=G).to(torch.int32)
  permuted = tokamax_amd.ragged_gather(h, (order // 2).to(torch.int32), 0, tokens)
  y = tokamax_amd.HipRaggedDot()(permuted, wts, group_sizes=gs)
  gate = torch.tensor(rng.uniform(0, 1, tokens * 2).astype(np.float32), device=device)
  inverse = torch.argsort(order).to(torch.int32)
  combined = tokamax_amd.ragged_gather_reduce(y, inverse, gate, torch.ones(tokens * 2, dtype=torch.bool, device=device), 2)
  want = np.zeros((tokens, n), np.float64)
  hn, wn, gn, en = _np(h).astype(np.float64), _np(wts).astype(np.float64), _np(gate), expert.cpu().numpy()
  for t in range(tokens):
    for s in range(2):
      want[t] += gn[2 * t + s] * (hn[t] @ wn[en[t, s]])
  _check(combined, want, 6e-3)


def test_row_lookup_outside_the_array(device):
  """Indices outside [0, rows): negative ones count from the end, the rest is clamped (the reference's `x[indices]`)."""
  rows, hidden = 37, 64
  rng = np.random.default_rng(5)
  x = torch.tensor(rng.normal(0, 1, (rows, hidden)).astype(np.float32), device=device).to(torch.bfloat16)
  idx_np = np.array([-1, -37, -38, -1000, 36, 37, 5000, 0, -2, 3, 2 ** 31 - 1, -2 ** 31], np.int64).astype(np.int32)
  idx = torch.tensor(idx_np, device=device)
  got = tokamax_amd.ragged_gather(x, idx, 0, rows)
  assert np.array_equal(_np(got), O.ragged_gather(_np(x), idx_np))
  got = tokamax_amd.ragged_scatter(x, idx, torch.tensor([0], device=device), torch.tensor([rows], device=device))
  assert np.array_equal(_np(got), O.ragged_scatter(_np(x), idx_np, 0, rows))
  w = torch.tensor(rng.uniform(0, 1, 12).astype(np.float32), device=device)
  got = tokamax_amd.ragged_gather_reduce(x, idx, w, torch.ones(12, dtype=torch.bool, device=device), 3)
  _check(got, O.ragged_gather_reduce(_np(x), idx_np, _np(w), np.ones(12, bool), 3), 3e-3)


@pytest.mark.parametrize("cfg", [hip_ops.KernelConfig(128, 128, 64, 2, 2, 4, grid_tile_width=4),
                                 hip_ops.KernelConfig(256, 256, 32, 2, 4, 4, grid_tile_width=8),
                                 hip_ops.KernelConfig(32, 128, 64, 1, 4, 4, grid_tile_width=2),
                                 hip_ops.KernelConfig(16, 128, 32, 1, 4, 2)])
@pytest.mark.parametrize("gs", [(300, 300, 300, 300), (5, 2000, 7, 1), (0, 0, 5000, 0), (129, 129, 129, 300)])
def test_group_sizes_that_add_up_to_more_than_m(cfg, gs, device):
  """Unchecked group sizes (checkify is off by default, base.py:223) whose sum exceeds m: the rows below m match
  the oracle, nothing is written past the output (guard rows around it stay as they were) and the call returns."""
  G, m, k, n = 4, 520, 1024, 256
  rng = np.random.default_rng(sum(gs))
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
  gs_t = torch.tensor(gs, dtype=torch.int32, device=device)
  lib = _lib.load()
  guard = 64
  buf = torch.full((m + 2 * guard, n), 7.0, dtype=torch.bfloat16, device=device)
  out = buf[guard:guard + m]
  ws = hip_ops.workspace(m, G, cfg.block_m, device)
  ws_guarded = torch.full((ws.numel() + 512,), -12345, dtype=torch.int32, device=device)
  c = cfg.to_c()
  import ctypes
  for mode, a, b_, cols in ((0, lhs, rhs, n), (1, torch.tensor(rng.normal(0, 1, (m, n)).astype(np.float32), device=device).to(torch.bfloat16), rhs, k)):
    if mode == 1 and cfg.block_m == 16:
      continue
    obuf = torch.full((m + 2 * guard, cols), 7.0, dtype=torch.bfloat16, device=device)
    o = obuf[guard:guard + m]
    st = lib.tkx_ragged_dot_fwd(a.data_ptr(), b_.data_ptr(), gs_t.data_ptr(), None, None, o.data_ptr(),
                                ws_guarded[256:].data_ptr(), m, k, n, G, _lib.TKX_BF16, _lib.TKX_BF16, _lib.TKX_BF16, mode, 0,
                                ctypes.byref(c), torch.cuda.current_stream().cuda_stream)
    _lib.check(st)
    torch.cuda.synchronize()
    assert (obuf[:guard] == 7.0).all() and (obuf[guard + m:] == 7.0).all()
    assert (ws_guarded[:256] == -12345).all() and (ws_guarded[256 + ws.numel():] == -12345).all()
    want = O.ragged_dot(_np(a), _np(rhs), np.array(gs), O.DEFAULT if mode == 0 else O.TRANS_RHS, acc_dtype=np.float64,
                        out_dtype="f64")
    _check(o, want, 2e-3)
  del buf, out


def test_hip_graph_replays_follow_new_inputs_and_group_sizes(device):
  """The entry points allocate nothing, synchronise nothing and schedule on the device, so a captured
  HIP graph stays valid when the contents of lhs, the weights and even group_sizes change between
  replays. One graph holds a tiled forward, a streaming small-m forward, a dlhs and a drhs; every
  replay is checked against the oracle on the inputs of that replay."""
  rng = np.random.default_rng(11)
  G, m, k, n = 6, 640, 256, 384
  f32 = torch.float32
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device).to(torch.bfloat16)
  lhs, rhs, dout = mk((m, k), 1.0), mk((G, k, n), k ** -0.5), mk((m, n), 1.0)
  gs = torch.tensor([100, 0, 257, 9, 130, 80], dtype=torch.int32, device=device)
  small_lhs, small_rhs = mk((40, 1024), 1.0), mk((G, 1024, 256), 1 / 32)
  small_gs = torch.tensor([3, 0, 16, 1, 7, 2], dtype=torch.int32, device=device)
  tiled = hip_ops.KernelConfig(128, 128, 64, 2, 2, 4, grid_tile_width=3)
  stream_cfg = hip_ops.KernelConfig(16, 128, 32, 1, 4, 2)
  drhs_cfg = hip_ops.KernelConfig(128, 128, 64, 2, 2, 4)

  def run():
    return (hip_ops.ragged_dot_fwd(lhs, rhs, gs, config=tiled, out_dtype=f32),
            hip_ops.ragged_dot_fwd(small_lhs, small_rhs, small_gs, config=stream_cfg, out_dtype=f32),
            hip_ops.ragged_dot_fwd(dout, rhs, gs, config=tiled, out_dtype=f32, trans_rhs=True),
            hip_ops.ragged_dot_drhs(lhs, dout, gs, G, config=drhs_cfg, out_dtype=f32))

  def check(outs):
    g, sg = gs.cpu().numpy(), small_gs.cpu().numpy()
    _check(outs[0], _ref(lhs, rhs, g), 1e-5)
    assert torch.count_nonzero(outs[0][int(g.sum()):]) == 0
    _check(outs[1], _ref(small_lhs, small_rhs, sg), 1e-5)
    assert torch.count_nonzero(outs[1][int(sg.sum()):]) == 0
    _check(outs[2], _ref(dout, rhs, g, O.TRANS_RHS), 1e-5)
    _check(outs[3], _ref(lhs, dout, g, O.RAGGED_CONTRACTING), 1e-5)

  side = torch.cuda.Stream()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.stream(side):
    run()
    side.synchronize()
    with torch.cuda.graph(graph, stream=side):
      outs = run()
  torch.cuda.synchronize()
  new_sizes = [[100, 0, 257, 9, 130, 80], [0, 300, 1, 0, 200, 139], [640, 0, 0, 0, 0, 0]]
  new_small = [[3, 0, 16, 1, 7, 2], [0, 0, 0, 0, 0, 0], [16, 1, 0, 12, 0, 11]]
  for sizes, ssizes in zip(new_sizes, new_small):
    gs.copy_(torch.tensor(sizes, dtype=torch.int32))
    small_gs.copy_(torch.tensor(ssizes, dtype=torch.int32))
    lhs.copy_(mk((m, k), 1.0))
    small_rhs.copy_(mk((G, 1024, 256), 1 / 32))
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    check(outs)
    check(run())  # eager work between the replays


def test_unsupported_inputs_are_declined(device):
  a = torch.zeros(64, 100, dtype=torch.bfloat16, device=device)  # k not a multiple of any block_k
  b = torch.zeros(2, 100, 64, dtype=torch.bfloat16, device=device)
  gs = torch.tensor([32, 32], dtype=torch.int32, device=device)
  with pytest.raises(NotImplementedError):
    tokamax_amd.ragged_dot(a, b, gs)
  with pytest.raises(NotImplementedError):  # mixed dtypes have no kernel
    tokamax_amd.ragged_dot(torch.zeros(64, 128, device=device), torch.zeros(2, 128, 64, dtype=torch.bfloat16, device=device), gs)
  calls = []
  fallback = lambda lhs, rhs, **kw: calls.append(1) or "fallback"
  assert tokamax_amd.ragged_dot(a, b, gs, implementation=["hip", fallback]) == "fallback" and calls


def test_autotune_on_device(device):
  a, b, gs = _inputs("test_autotune", 8, 1024, 128, 256, torch.bfloat16, device)
  ba = OP.bind(a, b, group_sizes=torch.tensor(gs, device=device))
  configs = {c for c in ba.autotuning_configs if c.grid_tile_width in (1, 8)}
  bad = hip.Config(block_m=8, block_n=8, block_k=8)  # names no compiled kernel: recorded, not raised
  data = ba.autotune(configs | {bad}, cache_results=False)
  assert isinstance(data[bad], NotImplementedError)
  best = data.fastest_config
  assert best in configs and data[best].median_evaluation_time_ms > 0
  res = tokamax_amd.AutotuningResult(tokamax_amd.op.device_kind(), ((ba, data),))
  with res:
    assert ba.default_config == best
  assert tokamax_amd.op.device_kind() == "AMD Instinct MI355X"


def test_autotune_of_a_function_on_device(device):
  """`tokamax_amd.autotune(f, *args)` (autotuning/api.py:322-418) on a function that calls the ragged dot twice with
  different shapes and once through `jax.grad`'s counterpart: each distinct call is found, tuned on the device and
  served from the result when it is used as an overlay."""
  a, b, gs = _inputs("test_autotune_fn", 8, 1024, 128, 256, torch.bfloat16, device)
  gst = torch.tensor(gs, device=device)
  a2, b2 = a[:512, :64].contiguous(), b[:, :64, :128].contiguous()
  gs2 = torch.tensor(gs // 2, device=device)

  def layer(x, w, x2, w2):
    y = tokamax_amd.ragged_dot(x, w, gst)
    y2 = tokamax_amd.ragged_dot(x2, w2, gs2)
    return y, y2, tokamax_amd.ragged_dot(x, w, gst)  # (a repeated call: one entry)

  found = tokamax_amd.get_bound_args(layer, a, b, a2, b2)
  assert [tuple(ba.arguments["lhs"].shape) for ba in found] == [(1024, 128), (512, 64)]
  res = tokamax_amd.autotune(layer, a, b, a2, b2, autotuner=tokamax_amd.autotuning.autotuner.Autotuner(iterations=2, warmup=1))
  assert res.device_kind == "AMD Instinct MI355X" and len(res.data) == 2
  want = layer(a, b, a2, b2)
  with res:
    for ba, data in res.data:
      assert ba.default_config == data.fastest_config
      assert data[data.fastest_config].median_evaluation_time_ms > 0
    got = layer(a, b, a2, b2)
  for g, w_ in zip(got, want):
    _check(g, _np(w_), 2e-3)
  back = tokamax_amd.AutotuningResult.loads(res.dumps(), {"HipRaggedDot": OP})
  assert [d.fastest_config for _, d in back.data] == [d.fastest_config for _, d in res.data]


# ---- quantisation on the fly (AsQArray), zero points, fp8 output -----------------------------------
_QNAME = {torch.int8: "int8", torch.int4: "int4", torch.float8_e4m3fn: "fp8"}


def _oracle_qarray(x, qtype, tile):
  """`QArray` holding what the oracle's absmax quantisation makes of `x`."""
  q, s = O.quantize_absmax(_np(x), _QNAME[qtype], tile)
  qv = torch.tensor(q, device=x.device)
  if qtype == torch.float8_e4m3fn:
    qv = qv.view(torch.float8_e4m3fn)
  return tokamax_amd.QArray(qv, torch.tensor(s, device=x.device), None, qtype)


def _dequantized(q):
  vals = q.qvalue.view(torch.uint8).cpu().numpy() if q.qvalue.dtype == torch.float8_e4m3fn else q.qvalue.cpu().numpy()
  vals = O.e4m3fn_decode(vals) if q.qvalue.dtype == torch.float8_e4m3fn else vals
  return O.dequantize(vals, _np(q.scale))


@pytest.mark.parametrize("xdtype", [torch.bfloat16, torch.float32, torch.float16])
@pytest.mark.parametrize("qtype", [torch.int8, torch.int4, torch.float8_e4m3fn])
@pytest.mark.parametrize("shape,tile", [((96, 256), (1, 128)), ((96, 256), (1, 16)), ((96, 256), (1, 256)), ((300, 4096), (1, 4096)),
                                        ((512, 256), (256, 1)), ((512, 256), (16, 1)), ((256, 384), (128, 128)),
                                        ((8, 256, 512), (1, 256, 1)), ((8, 256, 512), (1, 16, 1)), ((8, 256, 512), (1, 1, 16)),
                                        ((3, 128, 264), (1, 128, 8)), ((40, 2880), (1, 2880)), ((64, 8), (1, 8)),
                                        # tiles several rows tall that one workgroup does not reduce: one scale per tensor,
                                        # 512-column and 96-column blocks, whole groups of a weight array, all of it
                                        ((96, 512), (96, 512)), ((64, 1024), (32, 512)), ((96, 384), (48, 96)),
                                        ((4, 64, 768), (2, 64, 384)), ((4, 64, 384), (4, 64, 384))])
def test_quantize_kernel_bit_exact(shape, tile, qtype, xdtype, device):
  """`tkx_quantize` against the oracle's absmax quantisation: the same values and the same scales, bit for bit, for the
  tile shapes of the reference's quantised tests (test_base.py:187-192) and a few more; an all-zero tile included."""
  rng = np.random.default_rng(sum(shape) * 3 + sum(tile))
  x = rng.normal(0, 0.1, shape).astype(np.float32)
  x[tuple(slice(0, t) for t in tile)] = 0.0  # the first tile is all zero: scale 1, values 0
  xt = torch.tensor(x, device=device).to(xdtype)
  qv, scale = hip_ops.quantize(xt, qtype, tile)
  want_q, want_s = O.quantize_absmax(_np(xt), _QNAME[qtype], tile)
  assert scale.dtype == torch.float32 and tuple(scale.shape) == want_s.shape
  assert np.array_equal(scale.cpu().numpy(), want_s)
  got_q = qv.view(torch.uint8).cpu().numpy() if qtype == torch.float8_e4m3fn else qv.cpu().numpy()
  assert np.array_equal(got_q, want_q)
  as_q = tokamax_amd.AsQArray(xt, qtype, tiled_axes=dict(enumerate(tile))).as_qarray()
  assert torch.equal(as_q.scale, scale) and as_q.qtype == qtype and as_q.zero_point is None
  assert torch.equal(as_q.qvalue.view(torch.uint8), qv.view(torch.uint8))


@pytest.mark.parametrize("qtype,bound", [(torch.int8, 127.5), (torch.int4, 7.5), (torch.int8, 128.0), (torch.int8, 127.0)])
@pytest.mark.parametrize("shape,tile", [((96, 256), (1, 128)), ((512, 128), (64, 1)), ((2, 128, 256), (1, 128, 128))])
def test_quantize_kernel_with_another_bound(shape, tile, qtype, bound, device):
  """`tkx_quantize(..., qmax, bound)`: scale = absmax / bound and, with a bound above qmax, the type's most negative
  value in range: bit for bit the oracle's quantisation with that bound (127.5 / 7.5 is the convention of symmetric
  integer quantisers that use the type's full range; the default stays absmax / qmax). Bounds outside
  [qmax, qmax + 1], and a bound above qmax for fp8, are `ValueError`."""
  rng = np.random.default_rng(sum(shape) + int(bound))
  x = rng.normal(0, 0.1, shape).astype(np.float32)
  xt = torch.tensor(x, device=device)
  qv, scale = hip_ops.quantize(xt, qtype, tile, bound=bound)
  want_q, want_s = O.quantize_absmax(x, _QNAME[qtype], tile, bound=bound)
  assert np.array_equal(scale.cpu().numpy(), want_s) and np.array_equal(qv.cpu().numpy(), want_q)
  qmax = 127 if qtype == torch.int8 else 7
  if bound > qmax:
    assert int(qv.min()) == -qmax - 1 or int(qv.max()) == qmax  # the extreme of every tile rounds to an end of the range
    plain_q, plain_s = hip_ops.quantize(xt, qtype, tile)
    assert not torch.equal(plain_s, scale)
  with pytest.raises(ValueError):
    hip_ops.quantize(xt, qtype, tile, bound=qmax + 1.5)
  with pytest.raises(ValueError):
    hip_ops.quantize(xt, qtype, tile, bound=qmax - 1.0)
  with pytest.raises(ValueError):
    hip_ops.quantize(xt, torch.float8_e4m3fn, tile, bound=448.5)


@pytest.mark.parametrize("activation", [None, torch.relu, torch.tanh])
@pytest.mark.parametrize("use_as_qarray", [True, False])
@pytest.mark.parametrize("b_tile_shape", [(1, 1, 16), (1, 1, 128), (1, 256, 1), (1, 16, 1)])
@pytest.mark.parametrize("a_tile_shape", [None, (1, 128), (1, 16), (256, 1), (16, 1)])
@pytest.mark.parametrize("qtype", [torch.int8, torch.int4])
def test_quantized(qtype, a_tile_shape, b_tile_shape, use_as_qarray, activation, device):
  """The reference's `test_quantized` (test_base.py:187-242), parametrised as there: both operands quantised with the
  given tile shapes, handed over as `AsQArray` (quantised on the fly) or as `QArray`; the expected value contracts
  the dequantised operands in f32; atol 0.01, rtol 0.005 on the first sum(group_sizes) rows."""
  G, m, k, n = 8, 512, 256, 512
  a, b, gs = _inputs("test_quantized", G, m, k, n, torch.bfloat16, device, random_groups=True)
  if use_as_qarray:
    wrap = lambda x, t: tokamax_amd.AsQArray(x, qtype, tiled_axes=dict(enumerate(t)))
  else:
    wrap = lambda x, t: _oracle_qarray(x, qtype, t)
  a_in = a if a_tile_shape is None else wrap(a, a_tile_shape)
  b_in = wrap(b, b_tile_shape)
  a_f = _np(a) if a_tile_shape is None else _dequantized(_oracle_qarray(a, qtype, a_tile_shape))
  b_f = _dequantized(_oracle_qarray(b, qtype, b_tile_shape))
  want = O.ragged_dot(a_f, b_f, gs, acc_dtype=np.float32, out_dtype="f32")
  if activation is not None:
    want = activation(torch.tensor(want)).numpy()
  got = OP(a_in, b_in, group_sizes=torch.tensor(gs, device=device), activation=activation)
  count = int(gs.sum())
  np.testing.assert_allclose(_np(got)[:count], want[:count], atol=0.01, rtol=0.005)


@pytest.mark.parametrize("side", ["rhs", "lhs", "both"])
def test_operands_with_a_zero_point(side, device):
  """Quantised operands that carry a zero point are dequantised first, `(q - zero_point) * scale`
  (quantization.py:85-93), and then take the bf16 kernels."""
  rng = np.random.default_rng(31)
  G, m, k, n = 4, 200, 128, 256
  gs = np.array([60, 0, 90, 40], np.int32)
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device)
  lhs, rhs = mk((m, k), 1.0).to(torch.bfloat16), mk((G, k, n), k ** -0.5).to(torch.bfloat16)
  lhs_f, rhs_f = _np(lhs), _np(rhs)
  if side in ("rhs", "both"):
    q = torch.tensor(rng.integers(-128, 128, (G, k, n)).astype(np.int8), device=device)
    scale, zp = mk((G, 4, n), 0.01).abs() + 1e-3, torch.tensor(rng.integers(-20, 20, (G, 4, n)).astype(np.float32), device=device)
    rhs = tokamax_amd.QArray(q, scale, zp)
    rhs_f = O.round_to_bf16(O.dequantize_zero_point(q.cpu().numpy(), _np(scale), _np(zp)))
  if side in ("lhs", "both"):
    q = torch.tensor(rng.integers(-128, 128, (m, k)).astype(np.int8), device=device)
    scale, zp = mk((m, 1), 0.02).abs() + 1e-3, torch.tensor(rng.integers(-9, 9, (m, 1)).astype(np.float32), device=device)
    lhs = tokamax_amd.QArray(q, scale, zp)
    lhs_f = O.round_to_bf16(O.dequantize_zero_point(q.cpu().numpy(), _np(scale), _np(zp)))
  got = OP(lhs, rhs, group_sizes=torch.tensor(gs, device=device), preferred_element_type=torch.float32)
  _check(got, O.ragged_dot(lhs_f, rhs_f, gs, acc_dtype=np.float64, out_dtype="f64"), 1e-5)
  assert torch.count_nonzero(got[int(gs.sum()):]) == 0


@pytest.mark.parametrize("activation", [None, torch.relu, torch.nn.functional.silu])
def test_fp8_output_quantisation(activation, device):
  """`enable_fused_epilogue_quant` with an fp8 `preferred_element_type` returns the result quantised per (row, 128
  columns) as a QArray (pallas_mosaic_gpu_common.py:63-68; test of pallas_mosaic_gpu_kernel_sm100_fp8_quant_test.py:
  237-279: dequantised result within atol 0.06, rtol 0.1 of the reference, second run bit-identical). Without the
  switch the fp8 request is widened to the weights' type (pallas_mosaic_gpu.py:197-205)."""
  G, m, k, n = 8, 512, 256, 512
  a, b, gs = _inputs("test_epilogue_quant", G, m, k, n, torch.bfloat16, device, random_groups=True)
  gst = torch.tensor(gs, device=device)
  op_q = hip.HipRaggedDot(enable_fused_epilogue_quant=True)
  out = op_q(a, b, group_sizes=gst, preferred_element_type=torch.float8_e4m3fn, activation=activation)
  assert isinstance(out, tokamax_amd.QArray) and out.qvalue.dtype == torch.float8_e4m3fn
  assert tuple(out.qvalue.shape) == (m, n) and tuple(out.scale.shape) == (m, n // 128)
  want = O.ragged_dot(_np(a), _np(b), gs, acc_dtype=np.float32, out_dtype="f32")
  if activation is not None:
    want = activation(torch.tensor(want)).numpy()
  count = int(gs.sum())
  np.testing.assert_allclose(_dequantized(out)[:count], want[:count], atol=0.06, rtol=0.1)
  # exactly the absmax quantisation of the f32 result of the same call
  dense = OP(a, b, group_sizes=gst, preferred_element_type=torch.float32, activation=activation)
  q, s = O.quantize_absmax(_np(dense), "fp8", (1, 128))
  assert np.array_equal(out.qvalue.view(torch.uint8).cpu().numpy(), q) and np.array_equal(_np(out.scale), s)
  again = op_q(a, b, group_sizes=gst, preferred_element_type=torch.float8_e4m3fn, activation=activation)
  assert torch.equal(again.qvalue.view(torch.uint8), out.qvalue.view(torch.uint8)) and torch.equal(again.scale, out.scale)
  assert OP(a, b, group_sizes=gst, preferred_element_type=torch.float8_e4m3fn).dtype == torch.bfloat16


def test_ceiling_probes_run_and_give_plausible_figures(device):
  """The probes bench.py times beside the operator (libtkx_microbench.so): the matrix cores alone are faster on
  constant operands than on random ones and stay below the published peak; a panel shared by 32 workgroups of an XCD
  streams into LDS several times faster than one nobody shares."""
  from tokamax_amd import microbench
  zeros = microbench.mfma_bf16_tflops("zeros", device, iters=4000)
  random = microbench.mfma_bf16_tflops("random", device, iters=4000)
  assert 800 < random < zeros < 2600, (random, zeros)
  alone = microbench.operand_stream_tbs(1, device)    # 1 GB of panels: past the 256 MB memory-side cache
  shared = microbench.operand_stream_tbs(32, device)
  assert 1.0 < alone < 9.0 and shared > 2 * alone, (alone, shared)


def test_repeated_eager_calls_take_the_remembered_launch(device):
  """The operator's shortcut for repeated eager calls: same bits as the full path, taken only for calls that are one
  forward launch on the caller's own tensors, and never when a gradient is wanted."""
  rng = np.random.default_rng(11)
  G, m, k, n = 8, 64, 1024, 256
  gs = np.array([3, 0, 9, 1, 0, 20, 7, 5], np.int32)
  gst = torch.tensor(gs, device=device)
  lhs = torch.tensor(rng.normal(0, 1, (m, k)).astype(np.float32), device=device).to(torch.bfloat16)
  q = tokamax_amd.QArray(torch.tensor(rng.integers(-127, 128, (G, k, n)).astype(np.int8), device=device),
                         torch.tensor((rng.random((G, 1, n)) * 0.01 + 0.001).astype(np.float32), device=device))
  op = tokamax_amd.HipRaggedDot()
  first = op(lhs, q, group_sizes=gst, preferred_element_type=torch.bfloat16)
  plans = op.__dict__["_plans"]
  assert len(plans) == 1
  again = op(lhs, q, group_sizes=gst, preferred_element_type=torch.bfloat16)
  assert torch.equal(again, first) and again.data_ptr() != first.data_ptr() and len(plans) == 1
  want = O.ragged_dot(_np(lhs), O.dequantize(q.qvalue.cpu().numpy(), _np(q.scale)), gs, acc_dtype=np.float64, out_dtype="f64")
  _check(again, want, 3e-3)
  # other buffers of the same shapes, and group sizes updated in place: the launch reads what it is given
  lhs2 = (lhs.float() * 0.5).to(torch.bfloat16)
  gst.copy_(torch.tensor(gs[::-1].copy(), device=device))
  out2 = op(lhs2, q, group_sizes=gst, preferred_element_type=torch.bfloat16)
  fresh = tokamax_amd.HipRaggedDot()(lhs2, q, group_sizes=gst, preferred_element_type=torch.bfloat16)
  assert torch.equal(out2, fresh) and len(plans) == 1
  # another shape, another output type: plans of their own
  op(lhs[:32], q, group_sizes=torch.tensor(gs // 2, device=device), preferred_element_type=torch.bfloat16)
  op(lhs, q, group_sizes=gst, preferred_element_type=torch.float32)
  assert len(plans) == 3
  # calls that are more than one launch on the caller's tensors are not remembered: int64 group sizes (converted),
  # scales per k-block that need widening first, an activation given as a callable
  n_before = len(plans)
  a = op(lhs2, q, group_sizes=gst.to(torch.int64), preferred_element_type=torch.bfloat16)
  assert torch.equal(a, out2)
  blocks = tokamax_amd.QArray(q.qvalue, q.scale.expand(G, 4, n).contiguous() * torch.arange(1, 5, device=device).view(1, 4, 1))
  big = torch.tensor(rng.normal(0, 1, (2048, k)).astype(np.float32), device=device).to(torch.bfloat16)
  gs_big = torch.full((G,), 256, dtype=torch.int32, device=device)
  b1 = op(big, blocks, group_sizes=gs_big, preferred_element_type=torch.bfloat16)
  b2 = op(big, blocks, group_sizes=gs_big, preferred_element_type=torch.bfloat16)
  assert torch.equal(b1, b2)
  c = op(lhs2, q, group_sizes=gst, preferred_element_type=torch.bfloat16, activation=torch.relu)
  assert torch.equal(c, torch.relu(out2))
  assert len(plans) <= n_before + 1  # (the k-block call may be one launch of a variant of its own; the others are not)
  # a gradient: the full path with its custom VJP
  lhs_g = lhs.float().clone().to(torch.bfloat16).requires_grad_(True)
  w = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(torch.bfloat16)
  op(lhs_g.detach(), w, group_sizes=gst)
  op(lhs_g.detach(), w, group_sizes=gst)  # remembered
  out = op(lhs_g, w, group_sizes=gst)
  out.backward(torch.ones_like(out))
  assert lhs_g.grad is not None and torch.count_nonzero(lhs_g.grad) > 0
  with torch.no_grad():
    assert torch.equal(op(lhs_g, w, group_sizes=gst), out)
  # a change of the cached autotuning data forgets nothing but asks again
  from tokamax_amd import op as op_lib
  key_before = op._plan_key(lhs, q, dict(group_sizes=gst, preferred_element_type=torch.bfloat16))
  op_lib.bump_config_epoch()
  assert op._plan_key(lhs, q, dict(group_sizes=gst, preferred_element_type=torch.bfloat16)) != key_before
  assert torch.equal(op(lhs2, q, group_sizes=gst, preferred_element_type=torch.bfloat16), out2)
  # while an autotuning run records the ops a function calls, every call is a full one
  token = op_lib.OP_CALL_RECORDER.set([])
  try:
    assert op._plan_key(lhs, q, dict(group_sizes=gst)) is None
  finally:
    op_lib.OP_CALL_RECORDER.reset(token)
  # the public entry point goes through the same op objects
  r1 = tokamax_amd.ragged_dot(lhs, w, gst)
  r2 = tokamax_amd.ragged_dot(lhs, w, gst)
  assert torch.equal(r1, r2)


def test_split_workspace_is_never_released_when_a_call_needs_a_larger_one(device):
  """A HIP graph captured earlier holds the address of the workspace its split call used: when a later call on the
  same stream needs more room, the old buffer stays referenced (and keeps its address) next to the new one."""
  stream = torch.cuda.Stream(device)  # a stream of its own, so that no other test's workspace is in the way
  with torch.cuda.stream(stream):
    small = hip_ops.split_workspace(16, 1024, 4, device)
    assert hip_ops.split_workspace(16, 1024, 2, device) is small  # room enough: the same buffer
    address, words = small.data_ptr(), small.numel()
    assert torch.count_nonzero(small) == 0  # the arrival counters start at zero
    big = hip_ops.split_workspace(16, 1024, 1, device, persistent=1)
    assert big is not small and big.numel() * 4 >= _lib.load().tkx_ragged_dot_decode_persistent_workspace_bytes()
    assert any(t is small for t in hip_ops._SUPERSEDED_WORKSPACES)
    assert small.data_ptr() == address and small.numel() == words
    assert hip_ops.split_workspace(16, 1024, 4, device) is big  # later calls share the larger one
  stream.synchronize()


def test_timing_tool_collects_every_kind_of_problem(tmp_path, device):
  """The tool behind the heuristics' thresholds (`tokamax_amd/data/autotuning/tile_cost.py collect`) times every
  variant of a small problem of each kind it knows, writes entries `check` can read back, and finds the heuristics'
  config among the timed ones."""
  from tokamax_amd.data.autotuning import tile_cost
  path = str(tmp_path / "timings.json")
  kinds = ["", ",dlhs", ",drhs", ",int8", ",int4", ",fp8", ",fp8i4", ",fp8i4k", ",fp8i4glu", ",int8i4", ",int8i4k", ",int8i4glu", ",int8x8", ",glu",
           ",int8k", ",f32"]
  tile_cost.collect(["768,256,512,4" + k for k in kinds], 2, path=path)
  entries = tile_cost.load(path)
  assert len(entries) == len(kinds) and all(e["timings"] and e["timings"][0][7] > 0 for e in entries)
  assert {e.get("rhs", "bf16") for e in entries} == {"bf16", "int8", "int4", "fp8", "fp8i4", "fp8i4k", "fp8i4glu", "int8i4", "int8i4k",
                                                     "int8i4glu", "int8x8", "glu", "int8k", "f32"}
  assert sorted(e["mode"] for e in entries) == [0] * 14 + [1, 2]
  for e in entries:
    assert 1.0 <= tile_cost.heuristics_gap(e) < 3.0, e["shape"]
