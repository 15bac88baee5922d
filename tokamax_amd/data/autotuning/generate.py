"""Regenerates the shipped autotuning cache for the device this runs on.

Times every compiled kernel variant on the benchmark workloads (the prefill shapes, the fp8 shape, both
VJP products, the gate-up fused FFN shape, int8 and packed int4 weights at the prefill shape, the small-m decode shape
with int8 and with bf16 weights, whose
calls are short enough to be timed inside a captured graph, and the "primary" shapes of the reference's own
benchmark list) and writes
`tokamax_amd/data/autotuning/<device kind>/hip_ragged_dot.json`, the file `Op.get_autotuning_cache`
reads (layout of the reference's tokamax/data/autotuning/<device>/<op>.json).

  python -m tokamax_amd.data.autotuning.generate [--iterations N] [--only NAME]
"""

from __future__ import annotations

import argparse
import os

import torch

import tokamax_amd
from tokamax_amd import op as op_lib
from tokamax_amd.autotuning import autotuner as autotuner_lib
from tokamax_amd.autotuning import cache as cache_lib
from tokamax_amd.ragged_dot import arg_specs
from tokamax_amd.ragged_dot import base
from tokamax_amd.ragged_dot import workloads


def bound_arguments(op, device):
  """Yields (name, BoundArguments) one at a time (each holds its workload's tensors)."""
  w = workloads.make("mixtral", device)
  gs = torch.tensor(w.group_sizes, device=device)
  yield "mixtral", op.bind(w.lhs, w.rhs, group_sizes=gs)
  n = w.n
  rhs2 = torch.cat([w.rhs, w.rhs], dim=2)
  yield "mixtral gate-up", op.bind(w.lhs, rhs2, group_sizes=gs, fuse_gateup_activation="silu")
  del w, rhs2, n
  w = workloads.make("deepseek", device)
  gs = torch.tensor(w.group_sizes, device=device)
  yield "deepseek", op.bind(w.lhs, w.rhs, group_sizes=gs)
  del w
  w = workloads.make("fp8", device)
  gs = torch.tensor(w.group_sizes, device=device)
  yield "fp8", op.bind(tokamax_amd.QArray(w.lhs, w.lhs_scale), tokamax_amd.QArray(w.rhs, w.rhs_scale), group_sizes=gs,
                       preferred_element_type=torch.bfloat16)
  del w
  w = workloads.make("vjp", device)
  gs = torch.tensor(w.group_sizes, device=device)
  yield "dlhs", op.bind(w.dout, w.rhs, group_sizes=gs, ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS)
  yield "drhs", op.bind(w.lhs, w.dout, group_sizes=gs,
                        ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS)
  del w
  w = workloads.make("decode", device)
  gs = torch.tensor(w.group_sizes, device=device)
  yield "decode int8", op.bind(w.lhs, tokamax_amd.QArray(w.rhs, w.rhs_scale), group_sizes=gs,
                               preferred_element_type=torch.bfloat16)
  dense = (w.rhs.to(torch.float32) * w.rhs_scale).to(torch.bfloat16)
  yield "decode bf16", op.bind(w.lhs, dense, group_sizes=gs)
  del w, dense
  # The Mixtral shape with int8 weights (one scale per (group, column)) under a bf16 lhs, and int8 x int8.
  w = workloads.make("mixtral", device)
  gs = torch.tensor(w.group_sizes, device=device)
  gen = torch.Generator(device=device).manual_seed(1)
  q8 = tokamax_amd.QArray(torch.randint(-127, 128, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen),
                          (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen) + 0.5) / (127 * w.k ** 0.5))
  yield "mixtral int8 weights", op.bind(w.lhs, q8, group_sizes=gs, preferred_element_type=torch.bfloat16)
  a8 = tokamax_amd.QArray(torch.randint(-127, 128, (w.m, w.k), device=device, dtype=torch.int8, generator=gen),
                          (torch.rand(w.m, 1, device=device, generator=gen) + 0.5) / 127)
  yield "mixtral int8 x int8", op.bind(a8, q8, group_sizes=gs, preferred_element_type=torch.bfloat16)
  q4 = tokamax_amd.pack_int4(tokamax_amd.QArray(
      torch.randint(-8, 8, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen),
      (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen) + 0.5) / (7 * w.k ** 0.5), None,
      getattr(torch, "int4", torch.int8)))
  yield "mixtral int4 packed weights", op.bind(w.lhs, q4, group_sizes=gs, preferred_element_type=torch.bfloat16)
  # ... and quantised activations over them: the int8 and fp8 MFMAs on the nibbles
  yield "mixtral int8 x int4 packed", op.bind(a8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16)
  from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
  f8 = tokamax_amd.QArray(*hip_ops.quantize(w.lhs, torch.float8_e4m3fn, (1, w.k)))
  yield "mixtral fp8 x int4 packed", op.bind(f8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16)
  del w, q8, a8, q4, f8
  # The reference's own benchmark list (tokamax/_src/ops/ragged_dot/arg_specs.py): its "primary" shapes.
  for spec in arg_specs.ARG_SPECS:
    if "primary" not in spec.tags:
      continue
    args = arg_specs.random_initialize(spec.args, device)
    yield spec.full_name, op.bind(args["lhs"], args["rhs"], group_sizes=args["group_sizes"])
    del args


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--iterations", type=int, default=10)
  ap.add_argument("--only", default="", help="tune only the workloads whose name contains this; the other keys of the"
                  " shipped file are kept as they are")
  args = ap.parse_args()
  device = torch.device("cuda:0")
  op = tokamax_amd.HipRaggedDot()
  tuner = autotuner_lib.Autotuner(iterations=args.iterations, warmup=2)
  for name, ba in bound_arguments(op, device):
    if args.only not in name:
      continue
    # The span width stays at the heuristics' value: widths 4..16 time within 1% of each other and the
    # heuristics' width moves the fewest bytes past L2.
    width = ba.heuristics_config.grid_tile_width
    configs = {c for c in ba.autotuning_configs if c.grid_tile_width == width}
    if len(configs) < 2:  # drhs has no tile order to choose: its configs all carry width 1
      configs = ba.autotuning_configs
    data = ba.autotune(configs, autotuner=tuner, cache_results=True)
    best = data.fastest_config
    print(f"{name}: {len(data)} configs, fastest {best} {min(data[best].evaluation_times_ms):.4f} ms", flush=True)
    del ba, data
    torch.cuda.empty_cache()
  kind = op_lib.device_kind()
  path = cache_lib.cache_file(op.replace(vjp=None), kind)
  os.makedirs(os.path.dirname(path), exist_ok=True)
  with open(path, "w", encoding="utf-8") as f:
    f.write(cache_lib.dumps(op, op.get_autotuning_cache(kind)))
  print("wrote", path)


if __name__ == "__main__":
  main()
