"""Writes the golden fixtures of tests/golden/.

  scheduler_kat.json   the literal known-answer vectors held by the reference's own test
                       (tokamax/_src/ops/ragged_dot/pallas_mosaic_gpu_common_test.py:27-84), typed in
                       as data: inputs (group_sizes, tile, tid_size, align_tile) and the six expected arrays.
  ragged_dot_small.npz small seeded inputs with float64 outputs of the NumPy oracle for the three
                       dimension-number sets, an int8-dequant case and an fp8 case. The reference's
                       tests store no floating-point outputs (they compare against JAX live) and JAX is
                       not installed, so these vectors come from the oracle after it has been pinned by
                       tests/test_oracle.py (brute force, library GEMM special cases, autograd).

Run from the repository root:  python tests/golden/make_golden.py
"""

import json
import os
import sys

import numpy as np

HERE = os.path.dirname(os.path.abspath(__file__))
sys.path.insert(0, os.path.dirname(os.path.dirname(HERE)))

from oracle import ragged_dot_oracle as O  # noqa: E402


def scheduler_kat():
  cases = []
  for tid_size in (3, 5, 100):
    tail = [48 + 32 * (i + 1) for i in range(tid_size - 3)]
    cases.append(dict(
        name=f"create_aligned_tid{tid_size}", group_sizes=[17, 31, 24], tile=32, tid_size=tid_size, align_tile=8,
        group_id=[0, 1, 2] + [2] * (tid_size - 3),
        block_start=[0, 16, 48] + tail,
        actual_start=[0, 17, 48] + tail,
        actual_end=[17, 48, 72] + [72] * (tid_size - 3),
        start_within_block=[0, 1, 0] + [0] * (tid_size - 3),
        actual_size=[17, 31, 24] + [0] * (tid_size - 3),
    ))
  cases.append(dict(
      name="empty_groups", group_sizes=[17, 0, 31], tile=32, tid_size=5, align_tile=8,
      group_id=[0, 2, 2, 2, 2], block_start=[0, 16, 48, 80, 112], actual_start=[0, 17, 48, 80, 112],
      actual_end=[17, 48, 48, 48, 48], start_within_block=[0, 1, 0, 0, 0], actual_size=[17, 31, 0, 0, 0],
  ))
  cases.append(dict(
      name="multiple_blocks_per_group", group_sizes=[41, 32, 33], tile=32, tid_size=6, align_tile=8,
      group_id=[0, 0, 1, 1, 2, 2], block_start=[0, 32, 40, 72, 72, 104], actual_start=[0, 32, 41, 72, 73, 104],
      actual_end=[32, 41, 72, 73, 104, 106], start_within_block=[0, 0, 1, 0, 1, 0], actual_size=[32, 9, 31, 1, 31, 2],
  ))
  cases.append(dict(
      name="multiple_blocks_per_group_aligned", group_sizes=[40, 32, 33], tile=32, tid_size=6, align_tile=8,
      group_id=[0, 0, 1, 2, 2, 2], block_start=[0, 32, 40, 72, 104, 136], actual_start=[0, 32, 40, 72, 104, 136],
      actual_end=[32, 40, 72, 104, 105, 105], start_within_block=[0, 0, 0, 0, 0, 0], actual_size=[32, 8, 32, 32, 1, 0],
  ))
  return cases


def small_cases():
  rng = np.random.default_rng(20250101)
  out = {}
  G, m, k, n = 4, 96, 64, 48
  gs = np.array([23, 0, 41, 19], np.int32)  # sum 83 < m, one empty group, straddles 8-row boundaries
  lhs = O.round_to_bf16(rng.normal(0, 1, (m, k)).astype(np.float32))
  rhs = O.round_to_bf16(rng.normal(0, 1 / np.sqrt(k), (G, k, n)).astype(np.float32))
  dout = O.round_to_bf16(rng.normal(0, 1, (m, n)).astype(np.float32))
  out.update(gs=gs, lhs=lhs, rhs=rhs, dout=dout)
  out["fwd"] = O.ragged_dot(lhs, rhs, gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  out["dlhs"] = O.ragged_dot(dout, rhs, gs, O.TRANS_RHS, acc_dtype=np.float64, out_dtype="f64")
  out["drhs"] = O.ragged_dot(lhs, dout, gs, O.RAGGED_CONTRACTING, acc_dtype=np.float64, out_dtype="f64")
  # int8 weights with per-(group, column) scales
  q = rng.integers(-127, 128, (G, k, n)).astype(np.int8)
  sc = (rng.uniform(0.5, 1.5, (G, 1, n)) / 127).astype(np.float32)
  out.update(q8=q, q8_scale=sc)
  out["fwd_q8"] = O.ragged_dot(lhs, O.dequantize(q, sc), gs, O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  # fp8 e4m3fn both sides, per-row / per-(group, column) scales
  x = rng.normal(0, 1, (m, k)).astype(np.float32)
  w = rng.normal(0, 1 / np.sqrt(k), (G, k, n)).astype(np.float32)
  xs = (np.abs(x).max(1, keepdims=True) / 448).astype(np.float32)
  ws = (np.abs(w).max(1, keepdims=True) / 448).astype(np.float32)
  xq, wq = O.e4m3fn_encode(x / xs), O.e4m3fn_encode(w / ws)
  out.update(x8=xq, x8_scale=xs, w8=wq, w8_scale=ws)
  out["fwd_f8"] = O.ragged_dot(O.dequantize(O.e4m3fn_decode(xq), xs), O.dequantize(O.e4m3fn_decode(wq), ws), gs,
                               O.DEFAULT, acc_dtype=np.float64, out_dtype="f64")
  return out


def main():
  with open(os.path.join(HERE, "scheduler_kat.json"), "w") as f:
    json.dump(scheduler_kat(), f, indent=1)
  np.savez_compressed(os.path.join(HERE, "ragged_dot_small.npz"), **small_cases())
  print("wrote fixtures with numpy", np.__version__)


if __name__ == "__main__":
  main()
