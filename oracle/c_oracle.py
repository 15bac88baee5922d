"""ctypes access to the plain-C oracle (`libragged_dot_oracle.so`). Test infrastructure only."""

from __future__ import annotations

import ctypes
import os
import subprocess

import numpy as np

_DIR = os.path.dirname(os.path.abspath(__file__))
_SO = os.path.join(_DIR, "libragged_dot_oracle.so")
_lib = None


def build() -> str:
  subprocess.check_call(["make", "-s", "-B", "-C", _DIR, "libragged_dot_oracle.so"])
  return _SO


def lib():
  global _lib
  if _lib is None:
    if not os.path.exists(_SO):
      build()
    _lib = ctypes.CDLL(_SO)
    _lib.oracle_create_aligned.restype = ctypes.c_int32
  return _lib


def _p(a):
  return a.ctypes.data_as(ctypes.c_void_p)


def group_offsets(group_sizes) -> np.ndarray:
  gs = np.ascontiguousarray(group_sizes, np.int32)
  out = np.zeros(gs.size + 1, np.int32)
  lib().oracle_group_offsets(_p(gs), ctypes.c_int64(gs.size), _p(out))
  return out


def create_aligned(group_sizes, tile, tid_size, align_tile=8):
  gs = np.ascontiguousarray(group_sizes, np.int32)
  out = np.zeros((6, tid_size), np.int32)
  n = lib().oracle_create_aligned(_p(gs), ctypes.c_int64(gs.size), ctypes.c_int32(tile),
                                  ctypes.c_int32(tid_size), ctypes.c_int32(align_tile), _p(out))
  names = ("group_id", "block_start", "actual_start", "actual_end", "start_within_block", "actual_size")
  d = {k: out[i].copy() for i, k in enumerate(names)}
  d["num_tasks"] = int(n)
  return d


def ragged_dot_f32(lhs, rhs, group_sizes, mode: int) -> np.ndarray:
  lhs = np.ascontiguousarray(lhs, np.float32)
  rhs = np.ascontiguousarray(rhs, np.float32)
  gs = np.ascontiguousarray(group_sizes, np.int32)
  G = gs.size
  if mode == 0:
    m, k = lhs.shape
    n = rhs.shape[2]
    out = np.empty((m, n), np.float32)
  elif mode == 1:
    m, n = lhs.shape
    k = rhs.shape[1]
    out = np.empty((m, k), np.float32)
  else:
    m, k = lhs.shape
    n = rhs.shape[1]
    out = np.empty((G, k, n), np.float32)
  lib().oracle_ragged_dot_f32(_p(lhs), _p(rhs), _p(gs), _p(out), ctypes.c_int64(m), ctypes.c_int64(k),
                              ctypes.c_int64(n), ctypes.c_int64(G), ctypes.c_int32(mode))
  return out
