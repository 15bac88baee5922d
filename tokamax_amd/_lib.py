"""ctypes binding of libtkx_ragged_dot.so (the C ABI declared in include/tkx_ragged_dot.h).

The library is the only compute path of this package: if it is missing or fails to load, every
operator raises `HipLibraryError` -- there is no CPU or PyTorch fallback.
"""

from __future__ import annotations

import ctypes
import os
import threading

_HERE = os.path.dirname(os.path.abspath(__file__))
LIB_PATH = os.path.join(_HERE, "lib", "libtkx_ragged_dot.so")

TKX_OK, TKX_ERR_INVALID, TKX_ERR_UNSUPPORTED, TKX_ERR_RUNTIME = 0, 1, 2, 3
TKX_F32, TKX_BF16, TKX_F16, TKX_F8E4M3FN, TKX_I8, TKX_I4X2 = 0, 1, 2, 3, 4, 5
TKX_MODE_DEFAULT, TKX_MODE_TRANS_RHS = 0, 1
ACTIVATIONS = {None: 0, "relu": 1, "tanh": 2, "silu": 3, "gelu_tanh": 4, "sigmoid": 5,
               "swigluoai": 6, "silu_and_mul_with_clamp": 7}  # the last two: gate-up fusion only

# Names of every symbol include/tkx_ragged_dot.h declares.
EXPORTED_SYMBOLS = (
    "tkx_version",
    "tkx_last_error",
    "tkx_ragged_dot_tid_size",
    "tkx_ragged_dot_workspace_bytes",
    "tkx_ragged_dot_split_workspace_bytes",
    "tkx_ragged_dot_workspace_offset",
    "tkx_ragged_dot_schedule",
    "tkx_ragged_dot_fwd",
    "tkx_ragged_dot_fwd_static_workspace",
    "tkx_ragged_dot_fwd_fused",
    "tkx_ragged_dot_drhs",
    "tkx_dequantize_weights",
    "tkx_dequantize",
    "tkx_dequantize_zero_point",
    "tkx_quantize",
    "tkx_ragged_gather_rows",
    "tkx_ragged_dot_num_variants",
    "tkx_ragged_dot_variant",
    "tkx_ragged_dot_decode_workspace_bytes",
    "tkx_ragged_dot_decode_counter_bytes",
    "tkx_ragged_dot_decode_persistent_workspace_bytes",
    "tkx_ragged_dot_decode_clear_counters",
    "tkx_unpack_int4",
    "tkx_pack_int4",
    "tkx_row_sums_fp8",
    "tkx_ragged_dot_fwd_fp8_out",
)


class HipLibraryError(RuntimeError):
  """The HIP library is missing, failed to load, or reported a runtime failure."""


class TkxConfig(ctypes.Structure):
  _fields_ = [
      ("block_m", ctypes.c_int32),
      ("block_n", ctypes.c_int32),
      ("block_k", ctypes.c_int32),
      ("waves_m", ctypes.c_int32),
      ("waves_n", ctypes.c_int32),
      ("grid_tile_width", ctypes.c_int32),
      ("align_tile", ctypes.c_int32),
      ("num_stages", ctypes.c_int32),
      ("split_k", ctypes.c_int32),
      ("persistent", ctypes.c_int32),
  ]


_lock = threading.Lock()
_lib = None


def _declare(lib):
  i32, i64, vp = ctypes.c_int32, ctypes.c_int64, ctypes.c_void_p
  cfgp = ctypes.POINTER(TkxConfig)
  lib.tkx_version.restype = i32
  lib.tkx_version.argtypes = []
  lib.tkx_ragged_dot_decode_workspace_bytes.restype = i64
  lib.tkx_ragged_dot_decode_workspace_bytes.argtypes = [i64, i64, i32]
  lib.tkx_ragged_dot_decode_persistent_workspace_bytes.restype = i64
  lib.tkx_ragged_dot_decode_persistent_workspace_bytes.argtypes = []
  lib.tkx_ragged_dot_decode_clear_counters.restype = i32
  lib.tkx_ragged_dot_decode_clear_counters.argtypes = [vp, vp]
  lib.tkx_ragged_dot_decode_counter_bytes.restype = i64
  lib.tkx_ragged_dot_decode_counter_bytes.argtypes = [i32]
  lib.tkx_ragged_dot_fwd_fp8_out.restype = i32
  lib.tkx_ragged_dot_fwd_fp8_out.argtypes = [vp] * 8 + [i64] * 4 + [i32] * 3 + [cfgp, vp]
  for fn in (lib.tkx_unpack_int4, lib.tkx_pack_int4):
    fn.restype = i32
    fn.argtypes = [vp, vp, i64, i64, vp]
  lib.tkx_row_sums_fp8.restype = i32
  lib.tkx_row_sums_fp8.argtypes = [vp, vp, i64, i64, i64, vp]
  lib.tkx_last_error.restype = ctypes.c_char_p
  lib.tkx_last_error.argtypes = []
  lib.tkx_ragged_dot_tid_size.restype = i64
  lib.tkx_ragged_dot_tid_size.argtypes = [i64, i64, i32]
  lib.tkx_ragged_dot_workspace_bytes.restype = i64
  lib.tkx_ragged_dot_workspace_bytes.argtypes = [i64, i64, i32]
  lib.tkx_ragged_dot_split_workspace_bytes.restype = i64
  lib.tkx_ragged_dot_split_workspace_bytes.argtypes = [i64, i64, i32, i32]
  lib.tkx_ragged_dot_workspace_offset.restype = i64
  lib.tkx_ragged_dot_workspace_offset.argtypes = [i64, i64, i32, i32]
  lib.tkx_ragged_dot_schedule.restype = i32
  lib.tkx_ragged_dot_schedule.argtypes = [vp, i64, i64, i32, i32, vp, vp]
  lib.tkx_ragged_dot_fwd.restype = i32
  lib.tkx_ragged_dot_fwd.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, i32, i32, i32, i32, cfgp, vp]
  lib.tkx_ragged_dot_fwd_static_workspace.restype = i32
  lib.tkx_ragged_dot_fwd_static_workspace.argtypes = [vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, i32, i32, i32, i32, cfgp, vp]
  lib.tkx_ragged_dot_fwd_fused.restype = i32
  lib.tkx_ragged_dot_fwd_fused.argtypes = [vp, vp, vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i64, i64, i32, i32,
                                           i32, i32, i32, cfgp, vp]
  lib.tkx_ragged_dot_drhs.restype = i32
  lib.tkx_ragged_dot_drhs.argtypes = [vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, i32, cfgp, vp]
  lib.tkx_dequantize_weights.restype = i32
  lib.tkx_dequantize_weights.argtypes = [vp, vp, vp, i64, i64, i64, i64, i32, i32, vp]
  lib.tkx_dequantize.restype = i32
  lib.tkx_dequantize.argtypes = [vp, vp, vp, i64, i64, i64, i64, i32, i32, vp]
  lib.tkx_dequantize_zero_point.restype = i32
  lib.tkx_dequantize_zero_point.argtypes = [vp, vp, vp, vp, i64, i64, i64, i64, i32, i32, vp]
  lib.tkx_quantize.restype = i32
  lib.tkx_quantize.argtypes = [vp, vp, vp, i64, i64, i64, i64, i32, i32, ctypes.c_float, ctypes.c_float, vp]
  lib.tkx_ragged_gather_rows.restype = i32
  lib.tkx_ragged_gather_rows.argtypes = [vp, vp, vp, vp, vp, vp, vp, i64, i64, i64, i64, i32, vp]
  lib.tkx_ragged_dot_num_variants.restype = i32
  lib.tkx_ragged_dot_num_variants.argtypes = [i32]
  lib.tkx_ragged_dot_variant.restype = i32
  lib.tkx_ragged_dot_variant.argtypes = [i32, i32, cfgp, ctypes.POINTER(i32), ctypes.POINTER(i32), ctypes.POINTER(i32)]


def load():
  """Returns the loaded library, or raises `HipLibraryError`."""
  global _lib
  if _lib is not None:
    return _lib
  with _lock:
    if _lib is None:
      if not os.path.exists(LIB_PATH):
        raise HipLibraryError(
            f"{LIB_PATH} not found: build it with `python -c 'import __graft_entry__ as g; g.build()'` "
            "or `make -C tokamax_amd/csrc`. There is no fallback implementation."
        )
      try:
        lib = ctypes.CDLL(LIB_PATH)
      except OSError as e:
        raise HipLibraryError(f"failed to load {LIB_PATH}: {e}") from e
      _declare(lib)
      _lib = lib
  return _lib


def last_error() -> str:
  return load().tkx_last_error().decode("utf-8", "replace")


def check(status: int) -> None:
  """Maps a C status to the exception type the reference's Python API raises."""
  if status == TKX_OK:
    return
  msg = last_error()
  if status == TKX_ERR_UNSUPPORTED:
    raise NotImplementedError(msg)
  if status == TKX_ERR_INVALID:
    raise ValueError(msg)
  raise HipLibraryError(msg)


def variants(kind: int):
  """Lists compiled kernel variants: dicts with tile fields, dtypes and mode."""
  lib = load()
  out = []
  for i in range(lib.tkx_ragged_dot_num_variants(kind)):
    cfg = TkxConfig()
    a, b, mode = ctypes.c_int32(), ctypes.c_int32(), ctypes.c_int32()
    check(lib.tkx_ragged_dot_variant(kind, i, ctypes.byref(cfg), ctypes.byref(a), ctypes.byref(b), ctypes.byref(mode)))
    out.append(dict(block_m=cfg.block_m, block_n=cfg.block_n, block_k=cfg.block_k, waves_m=cfg.waves_m,
                    waves_n=cfg.waves_n, num_stages=cfg.num_stages, lhs_dtype=a.value, rhs_dtype=b.value, mode=mode.value))
  return out
