"""The entry point that allocates nothing (tkx_ragged_dot_fwd_static_workspace) against tkx_ragged_dot_fwd.

It runs the same kernels with the schedule arrays in a device array inside the library instead of a workspace
the caller allocated, so its results must equal tkx_ragged_dot_fwd's bit for bit: on two calls in a row (the
second smaller, so that words the first call left in the shared array lie behind the second call's schedule),
for a tiled variant, the transposed-rhs mode and the streaming small-m kernel, and the size limit is reported
as "unsupported".
"""

import ctypes

import numpy as np
import pytest
import torch

from oracle import ragged_dot_oracle as O
from tokamax_amd import _lib
from tokamax_amd.ragged_dot import hip_ops

pytestmark = pytest.mark.gpu


def _call(entry, lhs, rhs, gs, out, cfg, mode, ws=None):
  lib = _lib.load()
  G, k, n = rhs.shape
  m = lhs.shape[0]
  c = cfg.to_c()
  stream = torch.cuda.current_stream().cuda_stream
  code = {torch.bfloat16: _lib.TKX_BF16, torch.float32: _lib.TKX_F32}[lhs.dtype]
  if entry == "static":
    st = lib.tkx_ragged_dot_fwd_static_workspace(lhs.data_ptr(), rhs.data_ptr(), gs.data_ptr(), None, None, out.data_ptr(),
                                                 m, k, n, G, code, code, code, mode, 0, ctypes.byref(c), stream)
  else:
    st = lib.tkx_ragged_dot_fwd(lhs.data_ptr(), rhs.data_ptr(), gs.data_ptr(), None, None, out.data_ptr(), ws.data_ptr(),
                                m, k, n, G, code, code, code, mode, 0, ctypes.byref(c), stream)
  _lib.check(st)


CASES = [  # (config, mode, dtype, (G, m, k, n) of the first call, of the second call)
    (hip_ops.KernelConfig(128, 128, 64, 2, 2, 4, grid_tile_width=4), 0, torch.bfloat16, (6, 1500, 256, 384), (3, 300, 128, 256)),
    (hip_ops.KernelConfig(256, 256, 32, 2, 4, 4, grid_tile_width=8), 0, torch.bfloat16, (8, 2100, 512, 512), (2, 520, 512, 256)),
    (hip_ops.KernelConfig(128, 128, 64, 2, 2, 4, grid_tile_width=2), 1, torch.bfloat16, (5, 1000, 256, 384), (5, 90, 256, 128)),
    (hip_ops.KernelConfig(16, 128, 32, 1, 4, 2), 0, torch.bfloat16, (12, 40, 1024, 256), (4, 9, 1024, 128)),
    (hip_ops.KernelConfig(64, 128, 32, 2, 2, 4, grid_tile_width=4), 0, torch.float32, (4, 700, 96, 136), (4, 130, 64, 72)),
]


@pytest.mark.parametrize("cfg,mode,dtype,first,second", CASES)
def test_static_workspace_entry_matches_the_workspace_entry(cfg, mode, dtype, first, second, device):
  rng = np.random.default_rng(17)
  for G, m, k, n in (first, second):  # two calls in a row on the same device array, the second smaller
    inner = n if mode == 1 else k
    lhs = torch.tensor(rng.normal(0, 1, (m, inner)).astype(np.float32), device=device).to(dtype)
    rhs = torch.tensor(rng.normal(0, k ** -0.5, (G, k, n)).astype(np.float32), device=device).to(dtype)
    sizes = rng.multinomial(m - m // 10, np.ones(G) / G).astype(np.int32)
    sizes[rng.integers(0, G)] = 0  # an empty group, and a tail of rows that belong to no group
    gs = torch.tensor(sizes, device=device)
    cols = k if mode == 1 else n
    want = torch.full((m, cols), 3.0, dtype=dtype, device=device)
    got = torch.full((m, cols), 5.0, dtype=dtype, device=device)
    ws = hip_ops.workspace(m, G, cfg.block_m, device)
    _call("workspace", lhs, rhs, gs, want, cfg, mode, ws)
    _call("static", lhs, rhs, gs, got, cfg, mode)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16 if dtype == torch.bfloat16 else torch.int32),
                       want.view(torch.int16 if dtype == torch.bfloat16 else torch.int32))
    ref = O.ragged_dot(lhs.float().cpu().numpy(), rhs.float().cpu().numpy(), sizes, O.TRANS_RHS if mode == 1 else O.DEFAULT,
                       acc_dtype=np.float64, out_dtype="f64")
    assert O.rel_l2(got.float().cpu().numpy(), ref) <= (2e-3 if dtype == torch.bfloat16 else 1e-5)


def test_static_workspace_entry_rejects_schedules_beyond_its_array(device):
  lib = _lib.load()
  cfg = hip_ops.KernelConfig(32, 128, 64, 1, 4, 4)
  m, G = 32 * 9000, 8  # cdiv(m, 32) + G - 1 task slots x 8 arrays > 65536 words
  assert lib.tkx_ragged_dot_workspace_bytes(m, G, cfg.block_m) > 256 * 1024
  t = torch.zeros(16, dtype=torch.bfloat16, device=device)  # never touched: the size check comes first
  gs = torch.zeros(G, dtype=torch.int32, device=device)
  c = cfg.to_c()
  st = lib.tkx_ragged_dot_fwd_static_workspace(t.data_ptr(), t.data_ptr(), gs.data_ptr(), None, None, t.data_ptr(), m, 64, 128, G,
                                               _lib.TKX_BF16, _lib.TKX_BF16, _lib.TKX_BF16, 0, 0, ctypes.byref(c),
                                               torch.cuda.current_stream().cuda_stream)
  assert st == _lib.TKX_ERR_UNSUPPORTED and "built-in workspace" in _lib.last_error()


def test_static_workspace_entry_rejects_a_split_contraction(device):
  """split_k > 1 keeps arrival counters in a workspace that must be zero on entry; the built-in array holds the last
  call's schedule, so the entry point declines instead of reading it."""
  lib = _lib.load()
  c = hip_ops.KernelConfig(16, 128, 32, 1, 4, 2, split_k=2).to_c()
  t = torch.zeros(16, dtype=torch.bfloat16, device=device)  # never touched: the check comes first
  gs = torch.zeros(4, dtype=torch.int32, device=device)
  st = lib.tkx_ragged_dot_fwd_static_workspace(t.data_ptr(), t.data_ptr(), gs.data_ptr(), None, None, t.data_ptr(), 8, 1024, 128, 4,
                                               _lib.TKX_BF16, _lib.TKX_BF16, _lib.TKX_BF16, 0, 0, ctypes.byref(c),
                                               torch.cuda.current_stream().cuda_stream)
  assert st == _lib.TKX_ERR_UNSUPPORTED and "split contraction" in _lib.last_error()


def test_static_workspace_entry_under_graph_capture_allocates_nothing(device):
  """The use the entry point is for: one eager call (the first on a device looks the array's address up and raises the
  kernel's LDS limit), then the same call recorded into a HIP graph and replayed with new operands written into the
  captured tensors. Every replay equals the eager result of the workspace entry point bit for bit, and the device's free
  memory is the same before and after eager calls: nothing was allocated. (The graph object itself is torch's.)"""
  cfg = hip_ops.KernelConfig(128, 128, 64, 2, 2, 4, grid_tile_width=4)
  rng = np.random.default_rng(23)
  G, m, k, n = 5, 900, 256, 384
  mk = lambda shape, std: torch.tensor(rng.normal(0, std, shape).astype(np.float32), device=device).to(torch.bfloat16)
  lhs, rhs = mk((m, k), 1.0), mk((G, k, n), k ** -0.5)
  gs = torch.tensor(np.array([200, 0, 310, 150, 180], np.int32), device=device)
  got = torch.zeros((m, n), dtype=torch.bfloat16, device=device)
  want = torch.zeros_like(got)
  ws = hip_ops.workspace(m, G, cfg.block_m, device)
  all_sizes = ([200, 0, 310, 150, 180], [90, 400, 0, 0, 300], [0, 0, 0, 0, 7])
  # (every tensor the loop below needs exists before the memory reading is taken)
  new_lhs = [mk((m, k), 1.0) for _ in all_sizes]
  new_gs = [torch.tensor(np.array(sizes, np.int32), device=device) for sizes in all_sizes]
  side = torch.cuda.Stream()
  with torch.cuda.stream(side):
    _call("static", lhs, rhs, gs, got, cfg, 0)  # eager, outside capture
    side.synchronize()
    torch.cuda.synchronize()
    free_before, _ = torch.cuda.mem_get_info()
    for _ in range(3):
      _call("static", lhs, rhs, gs, got, cfg, 0)
    side.synchronize()
    assert torch.cuda.mem_get_info()[0] == free_before  # three calls later: nothing was allocated
    graph = torch.cuda.CUDAGraph()
    with torch.cuda.graph(graph, stream=side):
      _call("static", lhs, rhs, gs, got, cfg, 0)
  torch.cuda.synchronize()
  for sizes, l, g in zip(all_sizes, new_lhs, new_gs):
    lhs.copy_(l)
    gs.copy_(g)
    torch.cuda.synchronize()
    graph.replay()
    torch.cuda.synchronize()
    _call("workspace", lhs, rhs, gs, want, cfg, 0, ws)
    torch.cuda.synchronize()
    assert torch.equal(got.view(torch.int16), want.view(torch.int16)), sizes
