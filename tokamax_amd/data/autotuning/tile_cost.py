"""The timings behind the tile cost model of `HipRaggedDot`'s heuristics, and the fit of its constants.

`<device kind>/tile_cost_timings.json` holds, per shape, the measured time of every compiled tiled variant (with and
without the split of the last round): entries `{"shape": [rows, contraction, cols, groups], "mode": 0 forward | 1 dlhs,
"streaming_best_us": fastest small-m streaming variant or null, "timings": [[block_m, block_n, block_k, waves_m,
waves_n, num_stages, split_k, microseconds], ...]}`; entries of bf16 activations over quantised weights (one scale per
(group, column)) carry `"rhs": "int8"` or `"int4"` (packed two to a byte), fp8 x fp8 entries `"rhs": "fp8"`, int8 x int8
entries `"rhs": "int8x8"`, fp8 activations over packed int4 weights `"fp8i4"` (`"fp8i4k"`: weight scales per 128 k rows, `"fp8i4glu"`: gate-up fusion), int8 activations over them `"int8i4"` / `"int8i4k"` / `"int8i4glu"`, bf16 gate-up fusion `"glu"`, int8 weights with scales per 128 k rows `"int8k"`, f32 operands `"f32"`; mode 2 is
drhs with `"shape": [m, k, n, groups]`. The constants are fitted to the bf16 entries;
the others are what the rules for quantised weights in `HipRaggedDot._get_heuristics_config` were set by and are
checked against.

  python -m tokamax_amd.data.autotuning.tile_cost check              # how far the model's pick is from the fastest
  python -m tokamax_amd.data.autotuning.tile_cost fit [--iterations N]  # refit; prints the constants to paste
  python -m tokamax_amd.data.autotuning.tile_cost collect M,K,N,G[,dlhs|drhs|int8|int4|fp8|fp8i4|fp8i4k|fp8i4glu|int8i4|int8i4k|int8i4glu|int8x8|glu|int8k|f32] ...   # time shapes on this GPU and add them

`check` and `fit` need no GPU.
"""

from __future__ import annotations

import argparse
import json
import math
import os
import random

from tokamax_amd.ragged_dot import hip


def timings_path(device_kind: str = "amd_instinct_mi355x") -> str:
  return os.path.join(os.path.dirname(__file__), device_kind, "tile_cost_timings.json")


def load(path: str | None = None) -> list[dict]:
  with open(path or timings_path()) as f:
    return json.load(f)


def save(entries: list[dict], path: str | None = None) -> None:
  with open(path or timings_path(), "w") as f:
    f.write("[\n" + ",\n".join(json.dumps(e, separators=(",", ":")) for e in entries) + "\n]\n")


_RHS_BYTES = {"bf16": 2.0, "int8": 1.0, "int4": 0.5, "fp8i4": 0.5, "fp8i4k": 0.5, "fp8i4glu": 0.5, "int8i4": 0.5, "int8i4k": 0.5, "int8i4glu": 0.5}


def estimate(entry: dict, timing: list, fit: dict) -> float:
  rows, contraction, cols, groups = entry["shape"]
  return hip._tile_cost(tuple(timing[:6]), timing[6], rows, cols, contraction, groups, entry["mode"], fit,  # pylint: disable=protected-access
                        _RHS_BYTES[entry.get("rhs", "bf16")])


def pick(entry: dict, fit: dict) -> list:
  """The timing row the heuristics' ranking would choose (ties: longer k-step, deeper pipeline, no split)."""
  return min(entry["timings"], key=lambda t: (round(estimate(entry, t, fit), 3), -t[2], -t[5], t[6]))


def gaps(entries: list[dict], fit: dict) -> list[float]:
  """Per shape: time of the picked variant / time of the fastest tiled variant."""
  return [pick(e, fit)[7] / min(t[7] for t in e["timings"]) for e in entries]


def arguments(entry: dict, array):
  """(lhs, rhs, keyword arguments) of the entry's problem. `array(shape, dtype, top)` makes one array (abstract, or
  on the GPU with values of magnitude `top`)."""
  import torch  # pylint: disable=g-import-not-at-top
  import tokamax_amd  # pylint: disable=g-import-not-at-top
  from tokamax_amd.ragged_dot import base  # pylint: disable=g-import-not-at-top

  kind, mode = entry.get("rhs", "bf16"), entry["mode"]
  bf16, f32 = torch.bfloat16, torch.float32
  if mode == 2:  # drhs: shape = [m, k, n, groups], out[g, k, n] = lhs[rows of g, k]^T . dout[rows of g, n]
    m, k, n, groups = entry["shape"]
    return array((m, k), bf16, 1.0), array((m, n), bf16, 1.0), dict(
        ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS)
  rows, contraction, cols, groups = entry["shape"]
  kwargs = {} if mode == 0 else dict(ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS)
  shape = (groups, contraction, cols) if mode == 0 else (groups, cols, contraction)
  lhs = array((rows, contraction), bf16, 1.0)
  if kind == "bf16":
    return lhs, array(shape, bf16, contraction**-0.5), kwargs
  if kind == "f32":
    return array((rows, contraction), f32, 1.0), array(shape, f32, contraction**-0.5), kwargs
  if kind == "glu":  # bf16 gate-up fusion: `cols` output columns from weights [gate | up] of twice as many
    return lhs, array((groups, contraction, 2 * cols), bf16, contraction**-0.5), dict(kwargs, fuse_gateup_activation="silu")
  if kind == "int8k":  # bf16 activations over int8 weights with one scale per (group, 128 k rows, column)
    rhs = tokamax_amd.QArray(array(shape, torch.int8, 127),
                             array((groups, contraction // 128, cols), f32, 1.0 / (127 * contraction**0.5)))
    return lhs, rhs, dict(kwargs, preferred_element_type=bf16)
  if kind == "fp8":  # both operands e4m3fn, one scale per row and per (group, column)
    f8 = torch.float8_e4m3fn
    lhs = tokamax_amd.QArray(array((rows, contraction), f8, 1.0), array((rows, 1), f32, 1.0))
    return lhs, tokamax_amd.QArray(array(shape, f8, 1.0), array((groups, 1, cols), f32, contraction**-0.5)), dict(
        kwargs, preferred_element_type=bf16)
  if kind == "int8x8":  # int8 activations (one scale per row) over int8 weights (one per (group, column)): the int8 MFMAs
    lhs = tokamax_amd.QArray(array((rows, contraction), torch.int8, 127), array((rows, 1), f32, 1 / 127))
    rhs = tokamax_amd.QArray(array(shape, torch.int8, 127), array((groups, 1, cols), f32, 1.0 / (127 * contraction**0.5)))
    return lhs, rhs, dict(kwargs, preferred_element_type=bf16)
  top = 127 if kind == "int8" else 7
  if kind in ("fp8i4glu", "int8i4glu"):  # (`cols` output columns from weights [gate | up] of twice as many)
    shape, kwargs = (groups, contraction, 2 * cols), dict(kwargs, fuse_gateup_activation="silu")
  blocks = contraction // 128 if kind in ("fp8i4k", "int8i4k") else 1
  rhs = tokamax_amd.QArray(array(shape, torch.int8, top), array((groups, blocks, shape[2]), f32, 1.0 / (top * contraction**0.5)),
                           None, None if kind == "int8" else getattr(torch, "int4", torch.int8))
  if kind.startswith("fp8i4"):  # fp8 activations (one scale per row) over packed int4 weights: nibbles to the fp8 MFMAs
    lhs = tokamax_amd.QArray(array((rows, contraction), torch.float8_e4m3fn, 1.0), array((rows, 1), f32, 1.0))
  if kind.startswith("int8i4"):  # int8 activations (one scale per row) over packed int4 weights: the int8 MFMAs
    lhs = tokamax_amd.QArray(array((rows, contraction), torch.int8, 127), array((rows, 1), f32, 1 / 127))
  if kind == "int4" or kind.startswith("fp8i4") or kind.startswith("int8i4"):
    if isinstance(rhs.qvalue, torch.Tensor):
      rhs = tokamax_amd.pack_int4(rhs)
    else:
      rhs = tokamax_amd.QArray(array((groups, contraction // 2, shape[2]), torch.uint8, 0), rhs.scale, None, rhs.qtype)
  return lhs, rhs, dict(kwargs, preferred_element_type=bf16)


def heuristics_gap(entry: dict) -> float:
  """Time of the config `HipRaggedDot`'s heuristics choose for the entry's problem (on abstract arguments: no GPU) /
  time of the fastest variant, tiled or streaming."""
  import torch  # pylint: disable=g-import-not-at-top
  from tokamax_amd.serialization import ShapeDtype  # pylint: disable=g-import-not-at-top

  lhs, rhs, kwargs = arguments(entry, lambda shape, dtype, top: ShapeDtype(shape, dtype))
  op = hip.HipRaggedDot()
  c = op._get_heuristics_config(  # pylint: disable=protected-access
      op.bind(lhs, rhs, group_sizes=ShapeDtype((entry["shape"][3],), torch.int32), **kwargs))
  chosen = [c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages, c.split_k]
  fastest = min([t[7] for t in entry["timings"]] + [entry["streaming_best_us"] or math.inf])
  if c.block_m == 16:
    return entry["streaming_best_us"] / fastest
  return next(t[7] for t in entry["timings"] if t[:7] == chosen) / fastest


def summary(ratios: list[float]) -> tuple[float, float]:
  return math.exp(sum(math.log(r) for r in ratios) / len(ratios)) - 1, max(ratios) - 1


def log_error(entries: list[dict], fit: dict, launch_us: float) -> float:
  """Mean squared log ratio of estimate (+ a launch's fixed time, which does not rank variants) to measurement."""
  total, count = 0.0, 0
  for e in entries:
    for t in e["timings"]:
      total += math.log((estimate(e, t, fit) + launch_us) / t[7]) ** 2
      count += 1
  return total / count


def refit(entries: list[dict], start: dict, iterations: int, seed: int = 0) -> dict:
  """Random search from `start`: two constants at a time, scaled by exp(N(0, 0.12)), kept when the score (log error
  of the estimates plus twice the mean gap of the picks plus a tenth of the worst gap) falls."""
  rng = random.Random(seed)

  def score(p):
    mean, worst = summary(gaps(entries, p))
    return log_error(entries, p, p["launch_us"]) + 2.0 * mean + 0.1 * worst

  best = dict(start)
  best_score = score(best)
  for _ in range(iterations):
    trial = dict(best)
    for name in rng.sample(list(trial), 2):
      trial[name] *= math.exp(rng.gauss(0, 0.12))
    s = score(trial)
    if s < best_score:
      best, best_score = trial, s
  return best


def collect(specs: list[str], iterations: int, path: str | None = None) -> None:
  """Times every tiled and streaming variant on the problems `specs` name and adds the entries to the timings file of
  this device (or to `path`)."""
  import numpy as np  # pylint: disable=g-import-not-at-top
  import torch  # pylint: disable=g-import-not-at-top
  import tokamax_amd  # pylint: disable=g-import-not-at-top
  from tokamax_amd import op as op_lib  # pylint: disable=g-import-not-at-top
  from tokamax_amd.autotuning import autotuner as autotuner_lib  # pylint: disable=g-import-not-at-top
  from tokamax_amd.autotuning import cache as cache_lib  # pylint: disable=g-import-not-at-top
  from tokamax_amd.ragged_dot import base  # pylint: disable=g-import-not-at-top

  device = torch.device("cuda:0")
  path = path or timings_path(cache_lib.device_dir_name(op_lib.device_kind(device)))
  os.makedirs(os.path.dirname(path), exist_ok=True)
  entries = load(path) if os.path.exists(path) else []
  tuner = autotuner_lib.Autotuner(iterations=iterations, warmup=2)
  op = tokamax_amd.HipRaggedDot()
  gen = torch.Generator(device=device).manual_seed(1)
  def array(shape, dtype, top):
    if dtype in (torch.int8, torch.uint8):
      return torch.randint(-top, top + 1, shape, device=device, dtype=torch.int8, generator=gen)
    if dtype == torch.float32:
      return (torch.rand(shape, device=device, generator=gen) + 0.5) * top
    return (torch.randn(shape, device=device, generator=gen) * top).to(dtype)

  for spec in specs:
    parts = spec.split(",")
    tag = parts[4] if parts[4:] else ""
    mode = {"dlhs": 1, "drhs": 2}.get(tag, 0)
    kind = tag if tag in ("int8", "int4", "fp8", "fp8i4", "fp8i4k", "fp8i4glu", "int8i4", "int8i4k", "int8i4glu", "int8x8", "glu", "int8k", "f32") else "bf16"
    dims = [int(x) for x in parts[:4]]
    rng = np.random.default_rng(sum(dims))
    sizes = rng.multinomial(dims[0], rng.dirichlet(np.ones(dims[3]) * 4)).astype(np.int32)
    group_sizes = torch.tensor(sizes, device=device)
    entry = dict(shape=dims, mode=mode, **({} if kind == "bf16" else {"rhs": kind}))
    lhs, rhs, kwargs = arguments(entry, array)
    bound = op.bind(lhs, rhs, group_sizes=group_sizes, **kwargs)
    configs = {c for c in bound.autotuning_configs if c.block_m == 16 or c.grid_tile_width == 8}
    data = tuner.autotune(
        lambda c: (lambda: tokamax_amd.HipRaggedDot(config=c)(lhs, rhs, group_sizes=group_sizes, **kwargs)), configs
    )
    us = {c: d.median_evaluation_time_ms * 1e3 for c, d in data.items() if hasattr(d, "median_evaluation_time_ms")}
    streaming = [t for c, t in us.items() if c.block_m == 16]
    entry.update(
        streaming_best_us=round(min(streaming), 2) if streaming else None,
        timings=sorted(
            (
                [c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages, c.split_k, round(t, 2)]
                for c, t in us.items()
                if c.block_m != 16
            ),
            key=lambda t: t[7],
        ),
    )
    same = lambda e: (e["shape"], e["mode"], e.get("rhs", "bf16")) == (dims, mode, kind)
    entries = [e for e in entries if not same(e)] + [entry]
    save(entries, path)
    print(spec, "fastest", entry["timings"][0], f"heuristics {100 * (heuristics_gap(entry) - 1):.0f} % behind", flush=True)
    del lhs, rhs, bound


def main() -> None:
  parser = argparse.ArgumentParser(description=__doc__, formatter_class=argparse.RawDescriptionHelpFormatter)
  parser.add_argument("command", choices=("check", "fit", "collect"))
  parser.add_argument("shapes", nargs="*")
  parser.add_argument("--iterations", type=int, default=None)
  args = parser.parse_args()
  current = dict(hip._TILE_COST_FIT)  # pylint: disable=protected-access
  if args.command == "collect":
    collect(args.shapes, args.iterations or 6)
    return
  entries = load()
  label = lambda e: "drhs" if e["mode"] == 2 else e.get("rhs", "bf16")
  others = [e for e in entries if label(e) != "bf16"]
  entries = [e for e in entries if label(e) == "bf16"]  # (what the model is fitted to: forward and dlhs of bf16 operands)
  if args.command == "fit":
    fitted = refit(entries, dict(current, launch_us=7.0), args.iterations or 3000)
    fitted.pop("launch_us")
    print("_TILE_COST_FIT = dict(")
    for name, value in fitted.items():
      print(f"    {name}={float('%.4g' % value)!r},")
    print(")")
    current = {name: float("%.4g" % value) for name, value in fitted.items()}
  mean, worst = summary(gaps(entries, current))
  print(f"{len(entries)} shapes, {sum(len(e['timings']) for e in entries)} timings: the model's pick is "
        f"{100 * mean:.1f} % above the fastest variant on average, {100 * worst:.0f} % at worst")
  for kind in ["bf16"] + sorted({label(e) for e in others}):
    some = [e for e in others if label(e) == kind] if kind != "bf16" else entries
    mean, worst = summary([heuristics_gap(e) for e in some])
    print(f"the heuristics' config on the {len(some)} {kind} shapes: {100 * mean:.1f} % above the fastest "
          f"variant on average, {100 * worst:.0f} % at worst")


if __name__ == "__main__":
  main()
