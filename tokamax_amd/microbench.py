"""ctypes binding of libtkx_microbench.so (include/tkx_microbench.h): ceiling probes that bench.py times on the box.

Not part of the operator: nothing under `tokamax_amd.ragged_dot` imports this module.
"""

from __future__ import annotations

import ctypes
import os

import torch

LIB_PATH = os.path.join(os.path.dirname(os.path.abspath(__file__)), "lib", "libtkx_microbench.so")
EXPORTED_SYMBOLS = ("tkxmb_mfma_bf16", "tkxmb_mfma_bf16_flops", "tkxmb_mfma_fp8", "tkxmb_mfma_fp8_flops", "tkxmb_operand_stream", "tkxmb_operand_stream_bytes")

_lib = None


def load():
  global _lib
  if _lib is None:
    if not os.path.exists(LIB_PATH):
      raise RuntimeError(f"{LIB_PATH} not found: build it with `make -C tokamax_amd/csrc`")
    lib = ctypes.CDLL(LIB_PATH)
    i32, i64, vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
    lib.tkxmb_mfma_bf16.restype, lib.tkxmb_mfma_bf16.argtypes = i32, [vp, i32, vp, vp]
    lib.tkxmb_mfma_bf16_flops.restype, lib.tkxmb_mfma_bf16_flops.argtypes = i64, [i32]
    lib.tkxmb_mfma_fp8.restype, lib.tkxmb_mfma_fp8.argtypes = i32, [vp, i32, vp, vp]
    lib.tkxmb_mfma_fp8_flops.restype, lib.tkxmb_mfma_fp8_flops.argtypes = i64, [i32]
    lib.tkxmb_operand_stream.restype, lib.tkxmb_operand_stream.argtypes = i32, [vp, i64, i32, i32, vp]
    lib.tkxmb_operand_stream_bytes.restype, lib.tkxmb_operand_stream_bytes.argtypes = i64, [i64]
    _lib = lib
  return _lib


def _timed(launch, repeats: int) -> float:
  """Median HIP-event time (ms) of `repeats` launches on the current stream, after one untimed launch."""
  launch()
  torch.cuda.synchronize()
  times = []
  for _ in range(repeats):
    e0, e1 = torch.cuda.Event(enable_timing=True), torch.cuda.Event(enable_timing=True)
    e0.record()
    launch()
    e1.record()
    torch.cuda.synchronize()
    times.append(e0.elapsed_time(e1))
  return sorted(times)[len(times) // 2]


def mfma_bf16_tflops(data: str, device, iters: int = 20000, repeats: int = 3) -> float:
  """TFLOP/s of the register-resident bf16 MFMA loop on operands that are all `"zeros"` or `"random"` (normal)."""
  lib = load()
  gen = torch.Generator(device=device).manual_seed(0)
  operands = (torch.zeros(32768, device=device, dtype=torch.bfloat16) if data == "zeros"
              else torch.randn(32768, device=device, generator=gen).to(torch.bfloat16))
  sink = torch.zeros(16, device=device, dtype=torch.float32)
  stream = torch.cuda.current_stream(device).cuda_stream

  def launch():
    if lib.tkxmb_mfma_bf16(operands.data_ptr(), iters, sink.data_ptr(), stream) != 0:
      raise RuntimeError("tkxmb_mfma_bf16 failed")

  return lib.tkxmb_mfma_bf16_flops(iters) / _timed(launch, repeats) / 1e9


def mfma_fp8_tflops(data: str, device, iters: int = 10000, repeats: int = 3) -> float:
  """TFLOP/s of the register-resident fp8 (e4m3fn) MFMA loop on operands that are all `"zeros"` or `"random"`."""
  lib = load()
  gen = torch.Generator(device=device).manual_seed(0)
  operands = (torch.zeros(65536, device=device, dtype=torch.uint8) if data == "zeros"
              else torch.randn(65536, device=device, generator=gen).to(torch.float8_e4m3fn).view(torch.uint8))
  sink = torch.zeros(16, device=device, dtype=torch.float32)
  stream = torch.cuda.current_stream(device).cuda_stream

  def launch():
    if lib.tkxmb_mfma_fp8(operands.data_ptr(), iters, sink.data_ptr(), stream) != 0:
      raise RuntimeError("tkxmb_mfma_fp8 failed")

  return lib.tkxmb_mfma_fp8_flops(iters) / _timed(launch, repeats) / 1e9


def operand_stream_tbs(share: int, device, region_bytes: int = 2 << 20, regions: int = 512, repeats: int = 3) -> float:
  """TB/s into LDS when `share` workgroups of an XCD stream the same 2 MB region at a time (1 GB of regions in all)."""
  lib = load()
  src = torch.ones(region_bytes * regions // 4, device=device, dtype=torch.int32)
  stream = torch.cuda.current_stream(device).cuda_stream

  def launch():
    if lib.tkxmb_operand_stream(src.data_ptr(), region_bytes, regions, share, stream) != 0:
      raise RuntimeError("tkxmb_operand_stream failed")

  return lib.tkxmb_operand_stream_bytes(region_bytes) / _timed(launch, repeats) / 1e9
