"""Benchmark of the hip ragged dot on one MI355X.

  python bench.py [--gpus 1] [--steps K] [--warmup W] [--no-extras] [--no-cpu] [--calibration-copy]

Prints ONE JSON line. A step is one pass of the hot path (scheduler kernel + grouped-GEMM kernel)
over one seeded synthetic batch that is already resident in HBM. The headline workload is the
Mixtral-8x7B-shaped prefill grouped GEMM (m=16384, k=4096, n=14336, G=8, bf16, top-2 router group
sizes); `value` is its throughput in TFLOP/s with FLOPs = 2 * sum(group_sizes) * k * n.

`roofline` describes the dominant kernel of a step, the grouped GEMM: its average launch duration is
the HIP-event time of a step (events recorded on the launch stream) minus the separately measured
duration of the scheduler kernel, the only other kernel in a step. The other measured
configurations (DeepSeek-V3 shape, int8-weight decode, fp8, bf16 VJP) are reported under "extras"
with their own roofline figures; the decode kernel runs for tens of microseconds, less than the
host needs to issue a launch, so it is timed as a HIP graph of back-to-back launches over rotating
weight copies. `cpu_baseline` times the CPU oracle (per-group f32 GEMM through NumPy's BLAS) on this
box's host cores; it is a reported baseline, not the thing measured.
"""

from __future__ import annotations

import argparse
import dataclasses
import json
import os
import statistics
import sys
import time

import numpy as np
import torch

ROOT = os.path.dirname(os.path.abspath(__file__))
if ROOT not in sys.path:
  sys.path.insert(0, ROOT)

# MI355X published peaks (dense).
PEAK_TFLOPS = {"bf16": 2500.0, "fp8": 5000.0, "int8": 5000.0, "f32": 157.3}  # (int8: TOP/s)
PEAK_HBM_GBS = 8000.0

TRAFFIC_PROFILE = os.path.join(ROOT, "profiles", "bench_all_workloads.hbm_traffic_pmc.txt")


def _measured_traffic(kernel_prefix, workload_prefix):
  """HBM-side bytes per launch (read + written) of a kernel on a workload, from the committed summary of the
  rocprofv3 --pmc FETCH_SIZE / WRITE_SIZE runs of this script (each counter scaled by what it reads for a copy kernel
  of known size). The row is found by the kernel's template arguments and the workload's name: None when the summary
  has no row for the kernel the current config selects (a changed kernel must not inherit an old figure)."""
  try:
    with open(TRAFFIC_PROFILE) as f:
      lines = f.read().splitlines()
  except OSError:
    return None
  for line in lines:
    cols = [c for c in line.split("  ") if c.strip()]
    if len(cols) < 9 or not cols[0].strip().startswith(kernel_prefix) or not cols[1].strip().startswith(workload_prefix):
      continue
    try:
      read_mb, write_mb = float(cols[4]), float(cols[7])
    except ValueError:
      continue
    return (read_mb + write_mb) * 1e6
  return None


def _gemm_kernel_prefix(mode, lhs_code, rhs_code, cfg):
  return (f"GemmKernel<{mode}, {lhs_code}, {rhs_code}, {cfg.block_m}, {cfg.block_n}, {cfg.block_k}, {cfg.waves_m}, "
          f"{cfg.waves_n}, {cfg.num_stages},")


def _time_steps(fn, steps, warmup, stream):
  """Total and per-step device time (ms) of `steps` calls, HIP events on the launch stream."""
  for _ in range(warmup):
    fn()
  stream.synchronize()
  torch.cuda.synchronize()
  starts = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
  ends = [torch.cuda.Event(enable_timing=True) for _ in range(steps)]
  t0 = time.perf_counter()
  for i in range(steps):
    starts[i].record(stream)
    fn()
    ends[i].record(stream)
  stream.synchronize()
  torch.cuda.synchronize()
  wall_ms = (time.perf_counter() - t0) * 1e3
  per = [s.elapsed_time(e) for s, e in zip(starts, ends)]
  total = starts[0].elapsed_time(ends[-1])
  return total, per, wall_ms


def _roofline(bound, flops, nbytes, ms, dtype_key, traffic=None):
  """Roofline record of one kernel launch of `ms` milliseconds; `traffic` = measured HBM bytes per launch."""
  if bound == "mfma":
    achieved = flops / ms / 1e9
    peak = PEAK_TFLOPS[dtype_key]
    return dict(bound="mfma", achieved=round(achieved, 2), peak=peak, unit="TFLOP/s", frac=round(achieved / peak, 4),
                traffic=traffic, kernel_ms=round(ms, 5))
  achieved = nbytes / ms / 1e6
  return dict(bound="hbm", achieved=round(achieved, 2), peak=PEAK_HBM_GBS, unit="GB/s",
              frac=round(achieved / PEAK_HBM_GBS, 4), traffic=traffic, kernel_ms=round(ms, 5))


def _time_graph(calls, launches, stream_unused=None):
  """Average device time (ms) of one call when `launches` of them run back to back in a HIP graph.

  `calls` is a list of zero-argument functions used round-robin (rotating weight copies). The graph
  is replayed once untimed, then twice between two events."""
  del stream_unused
  side = torch.cuda.Stream()
  graph = torch.cuda.CUDAGraph()
  with torch.cuda.stream(side):
    for c in calls:
      c()
    side.synchronize()
    with torch.cuda.graph(graph, stream=side):
      for i in range(launches):
        calls[i % len(calls)]()
  torch.cuda.synchronize()
  graph.replay()
  torch.cuda.synchronize()
  e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
  e0.record()
  graph.replay()
  graph.replay()
  e1.record()
  torch.cuda.synchronize()
  return e0.elapsed_time(e1) / (2 * launches)


def _cpu_baseline(w):
  """Times the CPU oracle (per-group f32 GEMM, NumPy BLAS) on the full Mixtral workload."""
  from oracle import ragged_dot_oracle as O

  lhs = w.lhs.float().cpu().numpy()
  rhs = w.rhs.float().cpu().numpy()
  gs = w.group_sizes
  O.ragged_dot(lhs[:256], rhs, np.minimum(gs, 32), acc_dtype=np.float32)  # warm the BLAS threads
  times = []
  t_all = time.perf_counter()
  while len(times) < 3 or (time.perf_counter() - t_all < 10.0 and len(times) < 10):
    t0 = time.perf_counter()
    O.ragged_dot(lhs, rhs, gs, acc_dtype=np.float32, out_dtype="f32")
    times.append(time.perf_counter() - t0)
  try:
    from threadpoolctl import threadpool_info

    cores = max([p.get("num_threads", 1) for p in threadpool_info()] or [1])
  except Exception:  # pylint: disable=broad-exception-caught
    cores = os.cpu_count() or 1
  sec = statistics.median(times)
  return dict(value=round(w.flops / sec / 1e12, 4), unit="TFLOP/s", cores=int(cores), kind="port",
              sample=f"full {w.name} workload (m={w.m}, k={w.k}, n={w.n}, G={w.num_groups}), f32 NumPy-BLAS per-group "
                     f"GEMM, median of {len(times)} runs, {sec:.3f} s each")


def main():
  ap = argparse.ArgumentParser()
  ap.add_argument("--gpus", type=int, default=1)
  ap.add_argument("--steps", type=int, default=20)
  ap.add_argument("--warmup", type=int, default=5)
  ap.add_argument("--no-extras", action="store_true", help="headline workload only")
  ap.add_argument("--no-cpu", action="store_true", help="skip the CPU baseline leg")
  ap.add_argument("--calibration-copy", action="store_true",
                  help="also run one elementwise copy of 1 GiB (reads 1 GiB, writes 1 GiB), the known-size kernel "
                       "that hardware byte counters are scaled by")
  args = ap.parse_args()
  if args.gpus != 1 or int(os.environ.get("WORLD_SIZE", "1")) != 1:
    print("bench.py: ragged_dot is a single-device operator and this build measures ONE GPU; "
          "run with --gpus 1 (no multi-GPU figure exists).", file=sys.stderr)
    sys.exit(2)
  if not torch.cuda.is_available():
    print("bench.py: no GPU visible; the hip implementation has no CPU fallback.", file=sys.stderr)
    sys.exit(2)

  import tokamax_amd
  from tokamax_amd.ragged_dot import base, workloads

  device = torch.device("cuda:0")
  torch.cuda.set_device(device)
  stream = torch.cuda.current_stream(device)
  op = tokamax_amd.HipRaggedDot()

  if args.calibration_copy:
    src = torch.zeros(1 << 28, dtype=torch.int32, device=device)
    dst = torch.empty_like(src)
    torch.add(src, 1, out=dst)  # one elementwise kernel: 2^30 bytes in, 2^30 bytes out
    torch.cuda.synchronize()
    del src, dst

  # ---- headline: Mixtral prefill ----------------------------------------------------------------
  w = workloads.make("mixtral", device, seed=0)
  gs = torch.tensor(w.group_sizes, device=device)
  config = op.bind(w.lhs, w.rhs, group_sizes=gs).default_config
  run = lambda: op(w.lhs, w.rhs, group_sizes=gs)
  total_ms, per, wall_ms = _time_steps(run, args.steps, args.warmup, stream)
  ms = total_ms / args.steps
  # The scheduler kernel alone (the only other kernel of a step), as a graph of back-to-back launches.
  from tokamax_amd.ragged_dot import hip_ops
  sched_ms = _time_graph([lambda: hip_ops.schedule(gs, w.m, config.block_m, config.align_tile)], 20)
  gemm_ms = statistics.mean(per) - sched_ms
  result = {
      "metric": "ragged_dot TFLOP/s (% MFMA peak) prefill; GB/s (% HBM peak) decode, 1 GPU",
      "value": round(w.flops / ms / 1e9, 2),
      "unit": "TFLOP/s",
      "n_gpus": 1,
      "steps": args.steps,
      "warmup": args.warmup,
      "ms_per_step": round(ms, 5),
      "higher_is_better": True,
      "scaling": "weak",
      "vs_baseline": None,
      "dtype": "bf16",
      "data": "synthetic",
      "config": {
          "workload": "mixtral-8x7b prefill grouped GEMM: m=16384 (8192 tokens x top-2), k=4096, n=14336, G=8, "
                      "bf16 in / f32 accumulate / bf16 out, group_sizes from a top-2 router over Gaussian logits",
          "group_sizes": w.group_sizes.tolist(),
          "seed": 0,
          "kernel_config": {k: getattr(config, k) for k in ("block_m", "block_n", "block_k", "waves_m", "waves_n",
                                                            "grid_tile_width")},
      },
      "roofline": _roofline("mfma", w.flops, w.algorithmic_bytes(), gemm_ms, "bf16",
                            traffic=_measured_traffic(_gemm_kernel_prefix(0, 1, 1, config), "Mixtral prefill bf16 fwd")),
      "schedule_kernel_ms": round(sched_ms, 5),
      "ms_median_step": round(statistics.median(per), 5),
      "ms_min_step": round(min(per), 5),
      "wall_ms_per_step": round(wall_ms / args.steps, 5),
      "pct_mfma_peak": round(100 * w.flops / ms / 1e9 / PEAK_TFLOPS["bf16"], 2),
      "device": tokamax_amd.op.device_kind(),
  }

  if not args.no_cpu:
    result["cpu_baseline"] = _cpu_baseline(w)
  del w

  # ---- the other measured configurations ----------------------------------------------------------
  if not args.no_extras:
    extras = {}
    steps, warm = max(5, args.steps), max(2, args.warmup)

    def measure(name, fn, flops, nbytes, bound, dtype_key, cfg):
      t, p, _ = _time_steps(fn, steps, warm, stream)
      m_ = t / steps
      extras[name] = dict(ms_per_step=round(m_, 5), ms_min_step=round(min(p), 5), tflops=round(flops / m_ / 1e9, 2),
                          gbs=round(nbytes / m_ / 1e6, 2), roofline=_roofline(bound, flops, nbytes, m_, dtype_key),
                          kernel_config=None if cfg is None else
                          [cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.grid_tile_width])

    w = workloads.make("deepseek", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    cfg = op.bind(w.lhs, w.rhs, group_sizes=gs).default_config
    measure("deepseek_v3_prefill_bf16", lambda: op(w.lhs, w.rhs, group_sizes=gs), w.flops, w.algorithmic_bytes(),
            "hbm", "bf16", cfg)
    extras["deepseek_v3_prefill_bf16"]["roofline"]["traffic"] = _measured_traffic(
        _gemm_kernel_prefix(0, 1, 1, cfg), "DeepSeek-V3 prefill bf16 fwd")
    extras["deepseek_v3_prefill_bf16"]["pct_mfma_peak"] = round(
        100 * extras["deepseek_v3_prefill_bf16"]["tflops"] / PEAK_TFLOPS["bf16"], 2)
    # The same activations and group sizes over int4 weights packed two to a byte (one scale per (group, column)): this
    # workload is bound by the weights' way from HBM, and theirs is a quarter as long.
    from tokamax_amd.ragged_dot import hip_ops  # pylint: disable=g-import-not-at-top
    gen4 = torch.Generator(device=device).manual_seed(2)
    q4 = torch.empty((w.num_groups, w.k // 2, w.n), dtype=torch.uint8, device=device)
    for g0 in range(0, w.num_groups, 32):  # (packed in slices: the int8 form of all 256 experts would be 3.8 GB)
      q4[g0:g0 + 32] = hip_ops.pack_int4(torch.randint(-8, 8, (min(32, w.num_groups - g0), w.k, w.n), device=device,
                                                       dtype=torch.int8, generator=gen4))
    q4 = tokamax_amd.QArray(q4, (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen4) + 0.5) / (7 * w.k ** 0.5),
                            None, tokamax_amd.quantization.PACKED_INT4)
    cfg4 = op.bind(w.lhs, q4, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    nonempty = int((w.group_sizes > 0).sum())
    measure("deepseek_v3_prefill_int4_packed_weights",
            lambda: op(w.lhs, q4, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k * 2 + nonempty * w.k * w.n // 2 + w.m * w.n * 2, "hbm", "bf16", cfg4)
    # ... and with the activations quantised to fp8 per row as well (the fp8 MFMAs on the nibbles; the call includes the
    # pass that sums the activation rows)
    lhs8 = tokamax_amd.QArray(*hip_ops.quantize(w.lhs, torch.float8_e4m3fn, (1, w.k)))
    cfg48 = op.bind(lhs8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("deepseek_v3_prefill_fp8_activations_int4_packed_weights",
            lambda: op(lhs8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k + nonempty * w.k * w.n // 2 + w.m * w.n * 2, "hbm", "fp8", cfg48)
    del w, q4, lhs8

    # decode: 6 rotating copies of the weights defeat the 256 MB last-level cache ("cold"); the same
    # copy every launch is the "warm" figure.
    w = workloads.make("decode", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    copies = [tokamax_amd.QArray(w.rhs.clone(), w.rhs_scale.clone()) for _ in range(6)]
    cfg = op.bind(w.lhs, copies[0], group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    def decode_call(q):
      return lambda: op(w.lhs, q, group_sizes=gs, preferred_element_type=torch.bfloat16)

    def measure_graph(name, calls, traffic=None):
      m_ = _time_graph(calls, 24)
      extras[name] = dict(ms_per_step=round(m_, 5), tflops=round(w.flops / m_ / 1e9, 2),
                          gbs=round(w.algorithmic_bytes() / m_ / 1e6, 2), timing="HIP graph of 24 back-to-back launches",
                          roofline=_roofline("hbm", w.flops, w.algorithmic_bytes(), m_, "bf16", traffic=traffic),
                          kernel_config=[cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages])

    measure_graph("decode_int8_cold", [decode_call(q) for q in copies],
                  _measured_traffic(f"decode_kernel<4, {cfg.num_stages},", "int8-weight decode") if not cfg.persistent else None)
    measure_graph("decode_int8_warm", [decode_call(copies[0])])
    t, p, wall = _time_steps(decode_call(copies[0]), steps, warm, stream)
    extras["decode_int8_cold"]["eager_wall_ms_per_call"] = round(wall / steps, 5)  # host dispatch included
    extras["decode_int8_cold"]["algorithmic_bytes"] = int(w.algorithmic_bytes())
    extras["decode_int8_cold"]["touched_experts"] = w.nonempty_groups
    del w, copies

    w = workloads.make("fp8", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    ql, qr = tokamax_amd.QArray(w.lhs, w.lhs_scale), tokamax_amd.QArray(w.rhs, w.rhs_scale)
    cfg = op.bind(ql, qr, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_fp8", lambda: op(ql, qr, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.algorithmic_bytes(), "mfma", "fp8", cfg)
    # the same operands with one scale per (row, 128 k) and per (group, 128 k, column): folded in after every k-block
    genk = torch.Generator(device=device).manual_seed(2)
    kb = w.k // 128
    qlk = tokamax_amd.QArray(w.lhs, torch.rand(w.m, kb, device=device, generator=genk) + 0.5)
    qrk = tokamax_amd.QArray(w.rhs, (torch.rand(w.num_groups, kb, w.n, device=device, generator=genk) + 0.5) / w.k ** 0.5)
    cfg = op.bind(qlk, qrk, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_fp8_k_block_scales", lambda: op(qlk, qrk, group_sizes=gs, preferred_element_type=torch.bfloat16),
            w.flops, w.algorithmic_bytes() + (w.m * kb + w.nonempty_groups * kb * w.n) * 4, "mfma", "fp8", cfg)
    # fp8 x fp8 with the result quantised to fp8 per (row, 128 columns) in the kernel's epilogue, against the same
    # GEMM with an f32 result followed by the standalone quantisation pass
    from tokamax_amd.ragged_dot import hip as hip_backend, hip_ops  # pylint: disable=g-import-not-at-top
    op_q = hip_backend.HipRaggedDot(enable_fused_epilogue_quant=True)
    cfg = op.bind(ql, qr, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_fp8_quantised_output", lambda: op_q(ql, qr, group_sizes=gs, preferred_element_type=torch.float8_e4m3fn),
            w.flops, w.m * w.k + w.nonempty_groups * w.k * w.n + w.m * w.n + w.m * (w.n // 128) * 4, "mfma", "fp8", cfg)
    def two_passes():
      dense = op(ql, qr, group_sizes=gs, preferred_element_type=torch.float32)
      return hip_ops.quantize(dense, torch.float8_e4m3fn, (1, 128))
    t2, _, _ = _time_steps(two_passes, steps, warm, stream)
    extras["mixtral_prefill_fp8_quantised_output"]["ms_per_step_gemm_then_quantise_pass"] = round(t2 / steps, 5)
    # the same fp8 activations over int4 weights packed two to a byte along k: the nibbles go to the fp8 MFMAs as fp8
    # bytes; the call includes the pass that sums the activation rows for the kernel's epilogue
    gen4f = torch.Generator(device=device).manual_seed(3)
    q4f = tokamax_amd.pack_int4(tokamax_amd.QArray(
        torch.randint(-8, 8, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen4f),
        (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen4f) + 0.5) / (7 * w.k ** 0.5), None,
        getattr(torch, "int4", torch.int8)))
    cfg = op.bind(ql, q4f, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_fp8_activations_int4_packed_weights",
            lambda: op(ql, q4f, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k + w.nonempty_groups * w.k * w.n // 2 + w.m * w.n * 2, "mfma", "fp8", cfg)
    # ... and with the usual scales of int4 weights, one per (group, 128 k rows, column): every k-step's products are
    # folded in with its scales and the row sums of its own 128 activation columns
    q4fk = tokamax_amd.QArray(q4f.qvalue, (torch.rand(w.num_groups, kb, w.n, device=device, generator=gen4f) + 0.5)
                              / (7 * w.k ** 0.5), None, q4f.qtype)
    cfg = op.bind(ql, q4fk, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_fp8_activations_int4_packed_weights_k_block_scales",
            lambda: op(ql, q4fk, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k + w.nonempty_groups * (w.k * w.n // 2 + kb * w.n * 4) + w.m * kb * 8 + w.m * w.n * 2, "mfma", "fp8", cfg)
    del w, ql, qr, qlk, qrk, q4f, q4fk

    # the Mixtral shape with int8 weights (one f32 scale per (group, column)): the weight stream into LDS is half of bf16's
    w = workloads.make("mixtral", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    gen8 = torch.Generator(device=device).manual_seed(1)
    q8 = tokamax_amd.QArray(torch.randint(-127, 128, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen8),
                            (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen8) + 0.5) / (127 * w.k ** 0.5))
    cfg = op.bind(w.lhs, q8, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    nb = w.m * w.k * 2 + w.nonempty_groups * w.k * w.n + w.m * w.n * 2
    measure("mixtral_prefill_int8_weights", lambda: op(w.lhs, q8, group_sizes=gs, preferred_element_type=torch.bfloat16),
            w.flops, nb, "mfma", "bf16", cfg)
    # the same weights with a scale per (group, block of 128 k rows, column): scaled while widened, in the kernel
    q8k = tokamax_amd.QArray(q8.qvalue, (torch.rand(w.num_groups, w.k // 128, w.n, device=device, generator=gen8) + 0.5)
                             / (127 * w.k ** 0.5))
    cfg = op.bind(w.lhs, q8k, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int8_weights_k_block_scales", lambda: op(w.lhs, q8k, group_sizes=gs, preferred_element_type=torch.bfloat16),
            w.flops, nb + w.nonempty_groups * (w.k // 128) * w.n * 4, "mfma", "bf16", cfg)
    # int8 activations x the same int8 weights, one scale per row and per (group, column): the int8 MFMAs
    a8 = tokamax_amd.QArray(torch.randint(-127, 128, (w.m, w.k), device=device, dtype=torch.int8, generator=gen8),
                            (torch.rand(w.m, 1, device=device, generator=gen8) + 0.5) / 127)
    cfg = op.bind(a8, q8, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int8_int8", lambda: op(a8, q8, group_sizes=gs, preferred_element_type=torch.bfloat16),
            w.flops, w.m * w.k + w.nonempty_groups * w.k * w.n + w.m * w.n * 2, "mfma", "int8", cfg)
    # int4 weights packed two to a byte along k, read as they are by the tiled kernels (a quarter of bf16's weight stream)
    int4 = getattr(torch, "int4", torch.int8)
    q4 = tokamax_amd.pack_int4(tokamax_amd.QArray(
        torch.randint(-8, 8, tuple(w.rhs.shape), device=device, dtype=torch.int8, generator=gen8),
        (torch.rand(w.num_groups, 1, w.n, device=device, generator=gen8) + 0.5) / (7 * w.k ** 0.5), None, int4))
    cfg = op.bind(w.lhs, q4, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int4_packed_weights", lambda: op(w.lhs, q4, group_sizes=gs, preferred_element_type=torch.bfloat16),
            w.flops, w.m * w.k * 2 + w.nonempty_groups * w.k * w.n // 2 + w.m * w.n * 2, "mfma", "bf16", cfg)
    # the same weights with a scale per (group, block of 128 k rows, column), the usual form of int4 weights
    q4k = tokamax_amd.QArray(q4.qvalue, (torch.rand(w.num_groups, w.k // 128, w.n, device=device, generator=gen8) + 0.5)
                             / (7 * w.k ** 0.5), None, q4.qtype)
    cfg = op.bind(w.lhs, q4k, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int4_packed_weights_k_block_scales",
            lambda: op(w.lhs, q4k, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k * 2 + w.nonempty_groups * (w.k * w.n // 2 + (w.k // 128) * w.n * 4) + w.m * w.n * 2, "mfma", "bf16", cfg)
    # int8 activations over the packed int4 weights: the int8 MFMAs on the nibbles, exact int32 sums
    cfg = op.bind(a8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int8_activations_int4_packed_weights",
            lambda: op(a8, q4, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k + w.nonempty_groups * w.k * w.n // 2 + w.m * w.n * 2, "mfma", "int8", cfg)
    cfg = op.bind(a8, q4k, group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_prefill_int8_activations_int4_packed_weights_k_block_scales",
            lambda: op(a8, q4k, group_sizes=gs, preferred_element_type=torch.bfloat16), w.flops,
            w.m * w.k + w.nonempty_groups * (w.k * w.n // 2 + (w.k // 128) * w.n * 4) + w.m * (w.k // 128) * 4 + w.m * w.n * 2,
            "mfma", "int8", cfg)
    del w, q8, q8k, a8, q4, q4k

    w = workloads.make("vjp", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    cfg = op.bind(w.dout, w.rhs, group_sizes=gs, ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS).default_config
    nb = (w.m * w.n + w.nonempty_groups * w.k * w.n + w.m * w.k) * 2
    measure("vjp_dlhs_bf16", lambda: op(w.dout, w.rhs, group_sizes=gs, ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS),
            w.flops, nb, "mfma", "bf16", cfg)
    cfg = op.bind(w.lhs, w.dout, group_sizes=gs, ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS).default_config
    nb = (w.m * w.k + w.m * w.n + w.num_groups * w.k * w.n) * 2
    measure("vjp_drhs_bf16", lambda: op(w.lhs, w.dout, group_sizes=gs, ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS),
            w.flops, nb, "mfma", "bf16", cfg)
    del w

    # Mixtral FFN-1 with the gate and up projections in one call (weights [G, k, 2n]) and
    # silu(gate) * up applied in the kernel's epilogue; also the 16-bit-weight small-m kernel.
    gsz = workloads.router_top2_group_sizes(8192, 8, 0)
    gs = torch.tensor(gsz, device=device)
    gen = torch.Generator(device=device).manual_seed(0)
    m_, k_, n_ = int(gsz.sum()), 4096, 14336
    lhs = torch.randn(m_, k_, device=device, dtype=torch.bfloat16, generator=gen)
    rhs = (torch.randn(8, k_, 2 * n_, device=device, dtype=torch.float32, generator=gen) * k_ ** -0.5).to(torch.bfloat16)
    cfg = op.bind(lhs, rhs, group_sizes=gs, fuse_gateup_activation="silu").default_config
    nb = (m_ * k_ + 8 * k_ * 2 * n_ + m_ * n_) * 2
    measure("mixtral_gateup_silu_bf16", lambda: op(lhs, rhs, group_sizes=gs, fuse_gateup_activation="silu"),
            2 * m_ * k_ * 2 * n_, nb, "mfma", "bf16", cfg)
    # the same call over int4 weights packed two to a byte (one scale per (group, column))
    q4g = tokamax_amd.pack_int4(tokamax_amd.QArray(
        torch.randint(-8, 8, (8, k_, 2 * n_), device=device, dtype=torch.int8, generator=gen),
        (torch.rand(8, 1, 2 * n_, device=device, generator=gen) + 0.5) / (7 * k_ ** 0.5), None, getattr(torch, "int4", torch.int8)))
    cfg4 = op.bind(lhs, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_gateup_silu_int4_packed_weights",
            lambda: op(lhs, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16),
            2 * m_ * k_ * 2 * n_, (m_ * k_ + m_ * n_) * 2 + 8 * k_ * n_, "mfma", "bf16", cfg4)
    # ... and with the activations quantised to fp8 per row on top: the fp8 MFMAs on the nibbles (the row-sum pass is
    # part of the call)
    from tokamax_amd.ragged_dot import hip_ops as _ops  # pylint: disable=g-import-not-at-top
    lhs8 = tokamax_amd.QArray(*_ops.quantize(lhs, torch.float8_e4m3fn, (1, k_)))
    cfg48 = op.bind(lhs8, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_gateup_silu_fp8_activations_int4_packed_weights",
            lambda: op(lhs8, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16),
            2 * m_ * k_ * 2 * n_, m_ * k_ + m_ * n_ * 2 + 8 * k_ * n_, "mfma", "fp8", cfg48)
    # ... or to int8: the int8 MFMAs
    lhsi8 = tokamax_amd.QArray(*_ops.quantize(lhs, torch.int8, (1, k_)))
    cfg4i = op.bind(lhsi8, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16).default_config
    measure("mixtral_gateup_silu_int8_activations_int4_packed_weights",
            lambda: op(lhsi8, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16),
            2 * m_ * k_ * 2 * n_, m_ * k_ + m_ * n_ * 2 + 8 * k_ * n_, "mfma", "int8", cfg4i)
    del lhs8, lhsi8
    # The whole expert FFN of a Mixtral layer around those two products, as a caller strings it together: tokens
    # permuted into expert order (ragged_gather), gate-up product with silu(gate) * up in the epilogue, down
    # projection, weighted top-2 combine back into token order (ragged_gather_reduce). 8192 tokens, top 2 of 8 experts.
    tokens = m_ // 2
    h = torch.randn(tokens, k_, device=device, dtype=torch.bfloat16, generator=gen)
    down = (torch.randn(8, n_, k_, device=device, dtype=torch.float32, generator=gen) * n_ ** -0.5).to(torch.bfloat16)
    expert_of_slot = torch.repeat_interleave(torch.arange(8, device=device), gs.long())[torch.randperm(m_, device=device, generator=gen)]
    order = torch.argsort(expert_of_slot, stable=True)             # slot (token, choice) -> position in expert order
    token_of_row = (order // 2).to(torch.int32)
    inverse = torch.argsort(order).to(torch.int32)
    gate_w = torch.rand(m_, device=device, generator=gen)
    valid = torch.ones(m_, dtype=torch.bool, device=device)

    def ffn_block():
      x = tokamax_amd.ragged_gather(h, token_of_row, 0, tokens)
      y = op(x, rhs, group_sizes=gs, fuse_gateup_activation="silu")
      z = op(y, down, group_sizes=gs)
      return tokamax_amd.ragged_gather_reduce(z, inverse, gate_w, valid, 2)

    block_flops = 3 * 2 * m_ * k_ * n_
    block_bytes = (tokens * k_ * 2 + 8 * k_ * 3 * n_) * 2  # tokens in and out, the three weight matrices of every expert
    measure("moe_ffn_block_mixtral_bf16", ffn_block, block_flops, block_bytes, "mfma", "bf16", cfg)
    extras["moe_ffn_block_mixtral_bf16"]["steps"] = "ragged_gather, gate-up ragged_dot (silu fused), down ragged_dot, ragged_gather_reduce (top-2 combine)"
    del down
    # The same block with int4 weights packed two to a byte and the activations of both products quantised to fp8 per
    # row on the way (two quantisation passes): the fp8 MFMAs on the nibbles.
    q4d = tokamax_amd.pack_int4(tokamax_amd.QArray(
        torch.randint(-8, 8, (8, n_, k_), device=device, dtype=torch.int8, generator=gen),
        (torch.rand(8, 1, k_, device=device, generator=gen) + 0.5) / (7 * n_ ** 0.5), None, getattr(torch, "int4", torch.int8)))
    f8 = torch.float8_e4m3fn

    def ffn_block_w4a8():
      x = tokamax_amd.ragged_gather(h, token_of_row, 0, tokens)
      xq = tokamax_amd.QArray(*_ops.quantize(x, f8, (1, k_)))
      y = op(xq, q4g, group_sizes=gs, fuse_gateup_activation="silu", preferred_element_type=torch.bfloat16)
      yq = tokamax_amd.QArray(*_ops.quantize(y, f8, (1, n_)))
      z = op(yq, q4d, group_sizes=gs, preferred_element_type=torch.bfloat16)
      return tokamax_amd.ragged_gather_reduce(z, inverse, gate_w, valid, 2)

    measure("moe_ffn_block_mixtral_fp8_activations_int4_packed_weights", ffn_block_w4a8, block_flops,
            tokens * k_ * 2 * 2 + 8 * k_ * 3 * n_ // 2, "mfma", "fp8", cfg48)
    extras["moe_ffn_block_mixtral_fp8_activations_int4_packed_weights"]["steps"] = (
        "ragged_gather, quantise rows to fp8, gate-up ragged_dot (silu fused), quantise rows to fp8, down ragged_dot,"
        " ragged_gather_reduce (top-2 combine)")
    del lhs, rhs, h, q4g, q4d

    # The reference's own benchmark shapes with published timings on other hardware (tokamax/_src/ops/ragged_dot/
    # arg_specs.py:23-60; standard-normal inputs and representative group sizes as its benchmarks make them):
    # `8x7b` (B200: 0.734 ms Triton, 1.050 ms Mosaic), `compute_bound` (B200: 0.105 ms Triton) and `memory_bound`
    # (one row per group over 268 MB of bf16 weights; B200: 0.0418 ms Triton), the last timed as a graph.
    from tokamax_amd.ragged_dot import arg_specs
    for spec in arg_specs.ARG_SPECS:
      if spec.name not in ("8x7b", "compute_bound", "memory_bound"):
        continue
      kw = arg_specs.random_initialize(spec.args, device)
      lhs_, rhs_, gs_ = kw["lhs"], kw["rhs"], kw["group_sizes"]
      sizes = spec.args["group_sizes"].representative_value
      rows_, touched = int(sum(sizes)), sum(1 for x in sizes if x > 0)
      cfg = op.bind(lhs_, rhs_, group_sizes=gs_).default_config
      fl = arg_specs.flops(**spec.args)
      nb = (rows_ * rhs_.shape[1] + touched * rhs_.shape[1] * rhs_.shape[2] + lhs_.shape[0] * rhs_.shape[2]) * 2
      key = "arg_spec_" + spec.full_name
      if spec.name == "memory_bound":
        copies_ = [rhs_] + [rhs_.clone() for _ in range(2)]  # 3 x 268 MB defeat the 256 MB last-level cache
        m_ = _time_graph([(lambda r=r: op(lhs_, r, group_sizes=gs_)) for r in copies_], 24)
        extras[key] = dict(ms_per_step=round(m_, 5), gbs=round(nb / m_ / 1e6, 2), timing="HIP graph of 24 back-to-back launches",
                           roofline=_roofline("hbm", fl, nb, m_, "bf16"),
                           kernel_config=[cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages])
        del copies_
      else:
        measure(key, lambda: op(lhs_, rhs_, group_sizes=gs_), fl, nb, "mfma", "bf16", cfg)
      del kw, lhs_, rhs_, gs_

    # Stated ceilings of this box, same run, same kind of data (context for the fractions above, not product code):
    # the vendor library's dense bf16 GEMM on one expert's worth of the Mixtral shape in the layout the forward pass
    # has (NN: weights [k, n]) and in the transposed one (NT), and an elementwise copy of 1 GiB.
    a_ = torch.randn(16384, 4096, device=device, dtype=torch.bfloat16, generator=gen)
    b_nn = (torch.randn(4096, 14336, device=device, dtype=torch.float32, generator=gen) * 4096 ** -0.5).to(torch.bfloat16)
    b_nt = b_nn.t().contiguous()
    c_ = torch.empty(16384, 14336, device=device, dtype=torch.bfloat16)
    dense_flops = 2 * 16384 * 4096 * 14336
    t_nn, _, _ = _time_steps(lambda: torch.matmul(a_, b_nn, out=c_), steps, warm, stream)
    t_nt, _, _ = _time_steps(lambda: torch.matmul(a_, b_nt.t(), out=c_), steps, warm, stream)
    src_ = torch.zeros(1 << 28, dtype=torch.int32, device=device)
    dst_ = torch.empty_like(src_)
    t_cp, _, _ = _time_steps(lambda: dst_.copy_(src_), steps, warm, stream)
    ceilings = dict(
        dense_bf16_matmul_nn_tflops=round(dense_flops / (t_nn / steps) / 1e9, 1),
        dense_bf16_matmul_nt_tflops=round(dense_flops / (t_nt / steps) / 1e9, 1),
        copy_1gib_read_plus_write_gbs=round(2 * (1 << 30) / (t_cp / steps) / 1e6, 1),
        note="torch.matmul [16384,4096] x [4096,14336] bf16 (random normal data) and torch copy_ of 1 GiB, HIP-event timed")
    # This library's kernels on the same dense problem (one group holding every row), in both layouts: the forward
    # kernel on the [k, n] weights and the TRANS_RHS kernel on the k-contiguous ones.
    one_group = torch.tensor([16384], dtype=torch.int32, device=device)
    t_own_nn, _, _ = _time_steps(lambda: op(a_, b_nn[None], group_sizes=one_group), steps, warm, stream)
    t_own_nt, _, _ = _time_steps(lambda: op(a_, b_nt[None], group_sizes=one_group,
                                            ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS), steps, warm, stream)
    ceilings["this_library_same_problem_nn_tflops"] = round(dense_flops / (t_own_nn / steps) / 1e9, 1)
    ceilings["this_library_same_problem_nt_tflops"] = round(dense_flops / (t_own_nt / steps) / 1e9, 1)
    del b_nn, c_, src_, dst_
    # The vendor's dense fp8 GEMM (e4m3fn x e4m3fn -> bf16, one scale per tensor) at the same shape, where this torch
    # build has it for the device; it takes the weights k-contiguous (the NT layout).
    try:
      a8, b8 = a_.to(torch.float8_e4m3fn), b_nt.to(torch.float8_e4m3fn)
      one = torch.ones((), device=device, dtype=torch.float32)
      f8 = lambda: torch._scaled_mm(a8, b8.t(), scale_a=one, scale_b=one, out_dtype=torch.bfloat16)
      t_f8, _, _ = _time_steps(f8, steps, warm, stream)
      ceilings["dense_fp8_scaled_mm_nt_tflops"] = round(dense_flops / (t_f8 / steps) / 1e9, 1)
      del a8, b8
    except Exception as e:  # (not built for this device, or another signature: the ceiling is simply not reported)
      ceilings["dense_fp8_scaled_mm_nt_tflops"] = None
      ceilings["dense_fp8_note"] = f"torch._scaled_mm not usable here: {type(e).__name__}"
    del a_, b_nt
    # The chip's own ceilings by the probes of libtkx_microbench.so: the matrix cores on a register-resident MFMA
    # loop (the clock they settle at depends on the operand bits), and the operand stream of a tiled GEMM without
    # arithmetic, by how many workgroups of an XCD share a panel.
    try:
      from tokamax_amd import microbench
      ceilings["mfma_only_bf16_zeros_tflops"] = round(microbench.mfma_bf16_tflops("zeros", device), 1)
      ceilings["mfma_only_bf16_random_tflops"] = round(microbench.mfma_bf16_tflops("random", device), 1)
      ceilings["mfma_only_fp8_random_tflops"] = round(microbench.mfma_fp8_tflops("random", device), 1)
      for share in (1, 8, 32):
        ceilings[f"operand_stream_into_lds_share{share}_tbs"] = round(microbench.operand_stream_tbs(share, device), 2)
    except (RuntimeError, OSError) as e:
      ceilings["microbench_note"] = f"libtkx_microbench.so not usable: {e}"
    extras["ceilings_same_box"] = ceilings

    w = workloads.make("decode", device, seed=0)
    gs = torch.tensor(w.group_sizes, device=device)
    copies = [(torch.randn(w.num_groups, w.k, w.n, device=device, dtype=torch.float32, generator=gen) * w.k ** -0.5)
              .to(torch.bfloat16) for _ in range(3)]
    cfg = op.bind(w.lhs, copies[0], group_sizes=gs).default_config
    nb16 = (w.nonempty_groups * w.k * w.n + w.m * w.k + w.m * w.n) * 2
    m16 = _time_graph([(lambda r=r: op(w.lhs, r, group_sizes=gs)) for r in copies], 24)
    extras["decode_bf16_weights_cold"] = dict(
        ms_per_step=round(m16, 5), gbs=round(nb16 / m16 / 1e6, 2), timing="HIP graph of 24 back-to-back launches",
        roofline=_roofline("hbm", w.flops, nb16, m16, "bf16"),
        kernel_config=[cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages])
    del copies

    # the decode shape with int4 weights packed two to a byte along k (half the weight bytes of int8)
    packed = []
    for _ in range(6):
      q4 = torch.randint(-8, 8, (w.num_groups, w.k, w.n), device=device, dtype=torch.int8, generator=gen)
      packed.append(tokamax_amd.pack_int4(tokamax_amd.QArray(q4, w.rhs_scale.clone(), None, torch.int4)))
    del q4
    cfg = op.bind(w.lhs, packed[0], group_sizes=gs, preferred_element_type=torch.bfloat16).default_config
    nb4 = w.nonempty_groups * (w.k * w.n // 2 + w.n * 4) + (w.m * w.k + w.m * w.n) * 2
    m4 = _time_graph([(lambda r=r: op(w.lhs, r, group_sizes=gs, preferred_element_type=torch.bfloat16)) for r in packed], 24)
    extras["decode_int4_packed_cold"] = dict(
        ms_per_step=round(m4, 5), gbs=round(nb4 / m4 / 1e6, 2), timing="HIP graph of 24 back-to-back launches",
        roofline=_roofline("hbm", w.flops, nb4, m4, "bf16"),
        kernel_config=[cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages, cfg.split_k])
    del w, packed

    # few (group, column tile) pairs: 8 experts x 1024 columns, int8 weights, 2 rows per expert. Unsplit that is 64
    # workgroups on 256 CUs; the heuristics split the contraction 4 ways.
    G_, k_, n_ = 8, 8192, 1024
    lhs_ = torch.randn(2 * G_, k_, device=device, generator=gen).to(torch.bfloat16)
    gs_ = torch.full((G_,), 2, dtype=torch.int32, device=device)
    few = [tokamax_amd.QArray(torch.randint(-127, 128, (G_, k_, n_), device=device, dtype=torch.int8, generator=gen),
                              torch.rand(G_, 1, n_, device=device, generator=gen) / 127) for _ in range(6)]
    nbf = G_ * (k_ * n_ + n_ * 4) + 2 * G_ * (k_ + n_) * 2
    cfg = op.bind(lhs_, few[0], group_sizes=gs_, preferred_element_type=torch.bfloat16).default_config
    unsplit = tokamax_amd.HipRaggedDot(config=dataclasses.replace(cfg, split_k=1))
    t_split = _time_graph([(lambda r=r: op(lhs_, r, group_sizes=gs_, preferred_element_type=torch.bfloat16)) for r in few], 24)
    t_unsplit = _time_graph([(lambda r=r: unsplit(lhs_, r, group_sizes=gs_, preferred_element_type=torch.bfloat16)) for r in few], 24)
    extras["decode_few_tiles_split_k"] = dict(
        shape=dict(m=2 * G_, k=k_, n=n_, num_groups=G_), ms_per_step=round(t_split, 5), ms_per_step_unsplit=round(t_unsplit, 5),
        gbs=round(nbf / t_split / 1e6, 2), timing="HIP graph of 24 back-to-back launches",
        roofline=_roofline("hbm", 2 * 2 * G_ * k_ * n_, nbf, t_split, "bf16"),
        kernel_config=[cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages, cfg.split_k])
    del lhs_, gs_, few
    result["extras"] = extras

  print(json.dumps(result), flush=True)


if __name__ == "__main__":
  main()
