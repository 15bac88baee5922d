"""JSON autotuning cache, one file per (device kind, op class).

Follows tokamax/_src/autotuning/cache.py: files live under
`data/autotuning/<device_kind.lower().replace(" ", "_")>/<snake_case(OpClassName)>.json` (:34,:81-93),
map the JSON of an argument spec to `{config JSON: BenchmarkData}`, are read lazily on first
access per device kind (:62-64), and a file that fails to parse is logged and skipped (:106-109).
"""

from __future__ import annotations

import dataclasses
import json
import logging
import os
import re
from typing import Any

from tokamax_amd import benchmarking
from tokamax_amd import config as config_lib
from tokamax_amd.autotuning import autotuner

AutotuningData = autotuner.AutotuningData
logger = logging.getLogger("tokamax_amd")

CACHE_PATH = "data/autotuning"
_PACKAGE_DIR = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def op_file_name(op) -> str:
  return re.sub(r"(?!^)([A-Z])", r"_\1", type(op).__name__).lower() + ".json"


def device_dir_name(device_kind: str) -> str:
  return device_kind.lower().replace(" ", "_")


def cache_file(op, device_kind: str, base_dir: str = CACHE_PATH) -> str:
  return os.path.join(_PACKAGE_DIR, base_dir, device_dir_name(device_kind), op_file_name(op))


def config_to_json(config) -> str:
  return json.dumps(dataclasses.asdict(config), separators=(",", ":"))


def dumps(op, data: dict) -> str:
  """Serialises {cache key: AutotuningData} for `op`; exceptions are dropped (not serialisable)."""
  del op
  out = {}
  for key, tuning in data.items():
    entry = {}
    for config, bench in tuning.items():
      if isinstance(bench, benchmarking.BenchmarkData):
        entry[config_to_json(config)] = bench.to_json_dict()
    out[key.to_json()] = entry
  return json.dumps(out, indent=2)


def loads(op, json_data: str) -> dict:
  """Parses a cache file body into {cache key: AutotuningData} for `op`."""
  raw = json.loads(json_data or "{}")
  out = {}
  for key_json, entry in raw.items():
    spec = op.arg_spec_from_json(json.loads(key_json))
    key = op.bind(**spec).autotuning_cache_key
    tuning = {}
    for config_json, bench in entry.items():
      config = op.config_cls(**json.loads(config_json))
      tuning[config] = benchmarking.BenchmarkData.from_json_dict(bench)
    out[key] = AutotuningData(tuning)
  return out


class AutotuningCache(dict):
  """{device kind: {cache key: AutotuningData}}, files read on first access."""

  def __init__(self, op, paths=(CACHE_PATH,)):
    super().__init__()
    self.op = op
    self.cache_paths = tuple(paths)

  def __missing__(self, device_kind: str) -> dict:
    self[device_kind] = cache = self._load_cache(device_kind)
    return cache

  def _load_cache(self, device_kind: str) -> dict:
    out: dict[Any, Any] = {}
    for base_dir in self.cache_paths:
      if config_lib.ignore_autotuning_cache.value and base_dir == CACHE_PATH:
        continue
      path = cache_file(self.op, device_kind, base_dir)
      try:
        with open(path, "r", encoding="utf-8") as f:
          json_data = f.read()
      except FileNotFoundError:
        logger.info("Autotuning cache file not found: %s", path)
        continue
      try:
        out.update(loads(self.op, json_data))
      except Exception:  # pylint: disable=broad-except
        logger.exception("Failed to parse autotuning cache file: %s", path)
    return out
