"""Host-side logic of the operator API and the C-ABI library surface (no GPU needed).

Semantics follow the reference's own tests: dispatcher fallback (ragged_dot/api.py:204-240,
api_test.py), config resolution order (ops/op_test.py:109-144), autotuner failure handling
(autotuning/api_test.py:230-241,406-426), cache file naming and JSON key format
(autotuning/cache_test.py:31-36,86-92), config options (_src/config_test.py:28-47).
"""

import ctypes
import dataclasses
import json
import os
import re

import pytest
import torch
from exceptiongroup import ExceptionGroup

import tokamax_amd
from tokamax_amd import _lib
from tokamax_amd import benchmarking
from tokamax_amd import config as config_lib
from tokamax_amd import op as op_lib
from tokamax_amd import precision as precision_lib
from tokamax_amd.autotuning import autotuner as autotuner_lib
from tokamax_amd.autotuning import cache as cache_lib
from tokamax_amd.ragged_dot import api, arg_specs, base, hip
from tokamax_amd.serialization import ShapeDtype

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


# ---- C ABI surface ------------------------------------------------------------------------------
def test_library_loads_and_exports_every_declared_symbol():
  header = open(os.path.join(ROOT, "include", "tkx_ragged_dot.h")).read()
  declared = set(re.findall(r"\b(tkx_[a-z_0-9]+)\s*\(", header))
  assert declared == set(_lib.EXPORTED_SYMBOLS)
  lib = ctypes.CDLL(_lib.LIB_PATH)
  for name in declared:
    assert hasattr(lib, name), name
  assert _lib.load().tkx_version() == 2000  # 2000: TkxConfig.persistent (1001: split_k)


def test_probe_library_loads_and_exports_every_declared_symbol():
  """The ceiling probes bench.py times (a library of their own: nothing of the operator depends on it)."""
  from tokamax_amd import microbench
  header = open(os.path.join(ROOT, "include", "tkx_microbench.h")).read()
  declared = set(re.findall(r"\b(tkxmb_[a-z_0-9]+)\s*\(", header))
  assert declared == set(microbench.EXPORTED_SYMBOLS)
  lib = ctypes.CDLL(microbench.LIB_PATH)
  for name in declared:
    assert hasattr(lib, name), name
  assert microbench.load().tkxmb_operand_stream_bytes(2 << 20) == 2048 * (2 << 20)
  for module in ("hip", "hip_ops", "api", "base"):
    assert "microbench" not in open(os.path.join(ROOT, "tokamax_amd", "ragged_dot", module + ".py")).read()


def test_workspace_layout_queries():
  lib = _lib.load()
  assert lib.tkx_ragged_dot_tid_size(1024, 8, 128) == 1024 // 128 + 8 - 1
  assert lib.tkx_ragged_dot_tid_size(65536, 256, 128) == 767  # cdiv(m, block_m) + G - 1
  nbytes = lib.tkx_ragged_dot_workspace_bytes(1024, 8, 128)
  offs = [lib.tkx_ragged_dot_workspace_offset(1024, 8, 128, w) for w in range(11)]
  assert offs[0] == 0 and offs[1] == 1 and offs == sorted(offs) and offs[-1] * 4 + 15 * 4 <= nbytes
  assert lib.tkx_ragged_dot_workspace_offset(1024, 8, 128, 11) == -1
  assert lib.tkx_ragged_dot_workspace_bytes(-1, 8, 128) == -1


def test_variant_enumeration_matches_config_space():
  fwd = _lib.variants(0)
  drhs = _lib.variants(1)
  assert fwd and drhs
  assert {v["mode"] for v in fwd} == {0, 1, 3, 4} and {v["mode"] for v in drhs} == {2}  # 3 = gate-up fusion, 4 = k-block scales
  assert all(v["block_n"] // (32 * v["waves_n"]) % 2 == 0 for v in fwd if v["mode"] == 3)  # gate/up halves pair up
  pairs = {(v["lhs_dtype"], v["rhs_dtype"]) for v in fwd}
  assert {(_lib.TKX_BF16, _lib.TKX_BF16), (_lib.TKX_F32, _lib.TKX_F32), (_lib.TKX_F8E4M3FN, _lib.TKX_F8E4M3FN),
          (_lib.TKX_BF16, _lib.TKX_I8)} <= pairs
  for v in fwd + drhs:
    if v["block_m"] == 16:
      continue  # the streaming small-m kernel is not a 32x32-atom tile variant
    assert v["block_m"] % (32 * v["waves_m"]) == 0 and v["block_n"] % (32 * v["waves_n"]) == 0


def test_c_abi_argument_errors_without_gpu():
  lib = _lib.load()
  cfg = _lib.TkxConfig(128, 128, 64, 2, 2, 1, 8, 2)
  st = lib.tkx_ragged_dot_fwd(None, None, None, None, None, None, None, 8, 8, 8, 1, 1, 1, 1, 0, 0, ctypes.byref(cfg), None)
  assert st == _lib.TKX_ERR_INVALID and "null" in _lib.last_error()
  with pytest.raises(ValueError):
    _lib.check(st)
  st = lib.tkx_ragged_dot_fwd_fused(None, None, None, None, None, None, None, None, None, 8, 8, 8, 1, 1, 1, 1, 1, 1, 0,
                                    2, ctypes.byref(cfg), None)
  assert st == _lib.TKX_ERR_INVALID and "gateup" in _lib.last_error()
  with pytest.raises(NotImplementedError):
    _lib.check(_lib.TKX_ERR_UNSUPPORTED)
  with pytest.raises(_lib.HipLibraryError):
    _lib.check(_lib.TKX_ERR_RUNTIME)


def test_missing_library_fails_loudly(monkeypatch):
  monkeypatch.setattr(_lib, "_lib", None)
  monkeypatch.setattr(_lib, "LIB_PATH", "/nonexistent/libtkx_ragged_dot.so")
  with pytest.raises(_lib.HipLibraryError, match="no fallback"):
    _lib.load()


def test_no_cpu_fallback_for_cpu_tensors():
  lhs = torch.zeros(16, 64, dtype=torch.bfloat16)
  rhs = torch.zeros(2, 64, 64, dtype=torch.bfloat16)
  if torch.cuda.is_available():
    pytest.skip("checks the CPU-only refusal")
  with pytest.raises(NotImplementedError, match="Not supported on"):
    tokamax_amd.ragged_dot(lhs, rhs, torch.tensor([8, 8], dtype=torch.int32))


# ---- dispatcher ---------------------------------------------------------------------------------
def _args():
  return torch.zeros(16, 64), torch.zeros(2, 64, 64), torch.tensor([8, 8], dtype=torch.int32)


def test_registry_and_unknown_implementation():
  assert set(api.IMPLEMENTATIONS) == {"hip"}
  assert isinstance(api.IMPLEMENTATIONS["hip"], hip.HipRaggedDot)
  with pytest.raises(TypeError):
    api.IMPLEMENTATIONS["x"] = 1  # read-only, like the reference's immutabledict
  lhs, rhs, gs = _args()
  with pytest.raises(ValueError, match="Unknown implementation"):
    api.ragged_dot(lhs, rhs, gs, implementation="mosaic")
  with pytest.raises(ValueError, match="empty sequence"):
    api.ragged_dot(lhs, rhs, gs, implementation=())
  with pytest.raises(NotImplementedError, match="group_offset"):
    api.ragged_dot(lhs, rhs, gs, group_offset=torch.zeros(1), implementation="hip")
  with pytest.raises(ValueError, match="reduction dimension"):
    api.ragged_dot(torch.zeros(16, 32), rhs, gs, implementation="hip")


def test_fallback_only_on_not_implemented():
  lhs, rhs, gs = _args()
  calls = []

  def unsupported(*a, **kw):
    calls.append("unsupported")
    raise NotImplementedError("nope")

  def works(lhs, rhs, *, group_sizes, **kw):
    calls.append("works")
    assert kw["ragged_dot_dimension_numbers"] == base.DEFAULT_RAGGED_DOT_DIM_NUMS
    assert "manual_axis_type" not in kw  # forwarded only when set (api.py:219-223)
    return "result"

  def broken(*a, **kw):
    raise RuntimeError("boom")

  assert api.ragged_dot(lhs, rhs, gs, implementation=[unsupported, works]) == "result"
  assert calls == ["unsupported", "works"]
  with pytest.raises(NotImplementedError, match="nope"):  # a single implementation re-raises
    api.ragged_dot(lhs, rhs, gs, implementation=[unsupported])
  with pytest.raises(ExceptionGroup, match="all implementations failed") as ei:
    api.ragged_dot(lhs, rhs, gs, implementation=[unsupported, unsupported])
  assert len(ei.value.exceptions) == 2
  with pytest.raises(RuntimeError, match="boom"):  # other errors are not swallowed
    api.ragged_dot(lhs, rhs, gs, implementation=[broken, works])
  seen = {}

  def capture(lhs, rhs, **kw):
    seen.update(kw)
    return 0

  api.ragged_dot(lhs, rhs, gs, manual_axis_type="x", implementation=[capture])
  assert seen["manual_axis_type"] == "x"


# ---- bind / GroupSizes / precision ---------------------------------------------------------------
def test_bind_canonicalises_arguments():
  op = hip.HipRaggedDot()
  lhs, rhs, gs = _args()
  ba = op.bind(lhs, rhs, group_sizes=gs, preferred_element_type="bfloat16")
  a = ba.arguments
  assert isinstance(a["group_sizes"], base.GroupSizes) and a["group_sizes"].repr_value_or_total_size == 16
  assert a["ragged_dot_dimension_numbers"] == base.DEFAULT_RAGGED_DOT_DIM_NUMS
  assert a["precision"] == (precision_lib.Precision.DEFAULT,) * 2
  assert a["preferred_element_type"] == torch.bfloat16 and a["zero_initialize"] is True
  ba2 = op.bind(lhs, rhs, group_sizes=[8, 8])  # a sequence becomes its own representative value
  assert ba2.arguments["group_sizes"].repr_value_or_total_size == (8, 8)
  ba3 = op.bind(lhs, torch.zeros(16, 64), group_sizes=gs, ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS)
  assert isinstance(ba3.arguments["group_sizes"], torch.Tensor)  # wrapped only for the default dims (base.py:254-260)
  with pytest.raises(ValueError, match="Negative"):
    dataclasses.replace(op, checkify_group_sizes=True).bind(lhs, rhs, group_sizes=torch.tensor([2, -1]))
  with pytest.raises(ValueError, match="sum"):
    dataclasses.replace(op, checkify_group_sizes=True).bind(lhs, rhs, group_sizes=torch.tensor([15, 2]))


def test_group_sizes_wrapper():
  gs = base.GroupSizes(torch.tensor([3, 5], dtype=torch.int32), 8)
  same = base.GroupSizes(torch.tensor([1, 7], dtype=torch.int32), 8)
  assert gs == same and hash(gs) == hash(same)  # values are ignored (base.py:124-132)
  assert gs != base.GroupSizes(torch.tensor([3, 5], dtype=torch.int32), (3, 5))
  with pytest.raises(ValueError, match="integers"):
    base.GroupSizes(torch.zeros(2), 8)
  with pytest.raises(ValueError, match="same length"):
    base.GroupSizes(torch.tensor([3, 5]), (1, 2, 3))
  abstract = base.GroupSizes(ShapeDtype((8,), torch.int32), 1024)
  assert len(abstract.representative_value) == 8 and sum(abstract.representative_value) == 1024
  assert abstract.representative_value == base.generate_group_sizes(m=1024, num_groups=8)
  assert abstract._to_jsonable() == dict(num_groups=8, total_size=1024)
  assert base.GroupSizes(ShapeDtype((2,), torch.int32), (3, 5))._to_jsonable() == [3, 5]
  assert base.GroupSizes.from_json(dict(num_groups=8, total_size=1024)) == abstract


def test_precision_canonicalisation():
  P, D = precision_lib.Precision, precision_lib.DotAlgorithmPreset
  c = precision_lib.canonicalize_precision
  assert c(None) == (P.DEFAULT, P.DEFAULT) and c("highest") == (P.HIGHEST, P.HIGHEST)
  assert c("BF16_BF16_F32") is D.BF16_BF16_F32 and c(P.HIGH) == (P.HIGH, P.HIGH)
  assert c(("default", "highest")) == (P.DEFAULT, P.HIGHEST)
  with pytest.raises(ValueError):
    c("nonsense")
  assert precision_lib.is_default(torch.float32, torch.float32, (P.HIGHEST, P.HIGHEST))
  assert not precision_lib.is_default(torch.bfloat16, torch.bfloat16, D.F32_F32_F32)


# ---- config selection, cache, autotuning (fake op, as ops/op_test.py:73-96 does) ----------------
@dataclasses.dataclass(frozen=True)
class _FakeConfig:
  foo: int


@dataclasses.dataclass(frozen=True)
class _FakeOp(op_lib.Op):
  config_cls = _FakeConfig

  def _fwd(self, x, y, *, return_residuals, config):
    if config.foo == 13:
      raise RuntimeError("unlucky config")
    return x + y, None

  def _get_heuristics_config(self, ba):
    return _FakeConfig(foo=42)

  def _get_autotuning_configs(self, ba):
    return {_FakeConfig(1), _FakeConfig(2), _FakeConfig(13)}

  def arg_spec_from_json(self, spec):
    from tokamax_amd import serialization
    return {k: serialization.array_spec_from_json(v) for k, v in spec.items()}


def _bench(ms):
  return benchmarking.BenchmarkData(compile_time_ms=0.0, lower_time_ms=0.0, evaluation_times_ms=(ms,))


def test_config_resolution_order():
  x = torch.zeros(3)
  assert _FakeOp(config=_FakeConfig(7)).bind(x, x).default_config == _FakeConfig(7)  # explicit wins
  ba = _FakeOp().bind(x, x)
  assert ba.default_config == _FakeConfig(42)  # heuristics by default
  assert ba.autotuning_configs == {_FakeConfig(42), _FakeConfig(1), _FakeConfig(2), _FakeConfig(13)}
  with config_lib.autotuning_cache_miss_fallback("error"):
    with pytest.raises(ValueError, match="No config found"):
      _ = ba.default_config
  data = autotuner_lib.AutotuningData({_FakeConfig(1): _bench(3.0), _FakeConfig(2): _bench(1.0)})
  outer = tokamax_amd.AutotuningResult(op_lib.device_kind(), ((ba, data),))
  inner = tokamax_amd.AutotuningResult(
      op_lib.device_kind(), ((ba, autotuner_lib.AutotuningData({_FakeConfig(5): _bench(9.0)})),))
  with outer:
    assert ba.default_config == _FakeConfig(2)  # fastest by median
    with inner:
      assert ba.default_config == _FakeConfig(5)  # innermost overlay first
    with config_lib.ignore_autotuning_cache(True):
      assert ba.default_config == _FakeConfig(42)
  assert ba.default_config == _FakeConfig(42)


def test_config_memo_is_dropped_when_its_inputs_change():
  """`default_config` of identical calls is answered from a per-op memo; a new shape, a config option, an
  overlay or newly cached autotuning data each lead to a fresh resolution."""
  calls = []

  class _Counting(_FakeOp):
    def _get_heuristics_config(self, ba):
      calls.append(1)
      return _FakeConfig(42)

  op = _Counting()
  x, y = torch.zeros(3), torch.zeros(4)
  assert op.bind(x, x).default_config == _FakeConfig(42) and len(calls) == 1
  assert op.bind(torch.ones(3), torch.ones(3)).default_config == _FakeConfig(42) and len(calls) == 1  # same shapes: memo
  assert op.bind(y, y).default_config == _FakeConfig(42) and len(calls) == 2                          # new shape
  ba = op.bind(x, x)
  data = autotuner_lib.AutotuningData({_FakeConfig(1): _bench(3.0), _FakeConfig(2): _bench(1.0)})
  with tokamax_amd.AutotuningResult(op_lib.device_kind(), ((ba, data),)):
    assert op.bind(x, x).default_config == _FakeConfig(2)
    with config_lib.ignore_autotuning_cache(True):
      assert op.bind(x, x).default_config == _FakeConfig(42)
  assert op.bind(x, x).default_config == _FakeConfig(42)
  with config_lib.autotuning_cache_miss_fallback("error"):
    with pytest.raises(ValueError, match="No config found"):
      _ = op.bind(x, x).default_config
  # data written to the op's cache (what `autotune(cache_results=True)` does) is seen by the next call
  op.get_autotuning_cache()[ba.autotuning_cache_key] = data
  op_lib.bump_config_epoch()
  try:
    assert op.bind(x, x).default_config == _FakeConfig(2)
  finally:
    del op.get_autotuning_cache()[ba.autotuning_cache_key]
    op_lib.bump_config_epoch()
  assert op.bind(x, x).default_config == _FakeConfig(42)


def test_autotuner_records_failures_and_picks_fastest():
  x = torch.zeros(3)
  ba = _FakeOp().bind(x, x)

  class _Timer(autotuner_lib.Autotuner):
    def autotune(self, fn_factory, configs, *args, timeout=None, **kwargs):
      out = {}
      for c in configs:
        try:
          fn_factory(c)(*args, **kwargs)
          out[c] = _bench(float(c.foo))
        except Exception as e:  # pylint: disable=broad-exception-caught
          out[c] = e
      return autotuner_lib.AutotuningData(out)

  data = ba.autotune(autotuner=_Timer(), cache_results=False)
  assert isinstance(data[_FakeConfig(13)], RuntimeError)  # stored, not raised
  assert data.fastest_config == _FakeConfig(1)
  assert set(data.prune()) == {_FakeConfig(1)} and _FakeConfig(13) not in data.prune_errors()
  with pytest.raises(ExceptionGroup, match="All configs failed"):
    _ = autotuner_lib.AutotuningData({_FakeConfig(13): RuntimeError("x")}).fastest_config
  with pytest.raises(ValueError, match="empty"):
    _ = autotuner_lib.AutotuningData().fastest_config
  with config_lib.autotuning_cache_miss_fallback("autotune"):
    # the real autotuner needs a GPU timer; check only that `AUTO` is what default_config asks for
    called = {}
    orig = op_lib.BoundArguments.autotune
    try:
      op_lib.BoundArguments.autotune = lambda self, configs=op_lib.AUTO, **kw: called.setdefault("configs", configs) and data or data
      assert ba.default_config == _FakeConfig(1) and called["configs"] is op_lib.AUTO
    finally:
      op_lib.BoundArguments.autotune = orig


def test_config_options():
  assert config_lib.autotuning_cache_miss_fallback.value == "heuristics"
  with config_lib.autotuning_cache_miss_fallback("autotune"):
    assert config_lib.autotuning_cache_miss_fallback.value == "autotune"
  with pytest.raises(ValueError, match="Invalid value"):
    with config_lib.autotuning_cache_miss_fallback("bogus"):
      pass
  assert config_lib.cross_compile.value is False
  with config_lib.cross_compile("true"):
    assert config_lib.cross_compile.value is True
  os.environ["TOKAMAX_IGNORE_AUTOTUNING_CACHE"] = "1"
  try:
    assert config_lib.ignore_autotuning_cache.value is True
  finally:
    del os.environ["TOKAMAX_IGNORE_AUTOTUNING_CACHE"]


def test_shipped_mi355x_cache_parses_and_names_compiled_variants():
  """data/autotuning/amd_instinct_mi355x/hip_ragged_dot.json (written by data/autotuning/generate.py on
  an MI355X): every key binds again, and every timed config is a compiled kernel variant."""
  op = tokamax_amd.HipRaggedDot()
  path = cache_lib.cache_file(op.replace(vjp=None), "AMD Instinct MI355X")
  with open(path, encoding="utf-8") as f:
    loaded = cache_lib.loads(op, f.read())
  assert len(loaded) >= 20  # the bench workloads and the reference's "primary" arg specs
  compiled = {(v["block_m"], v["block_n"], v["block_k"], v["waves_m"], v["waves_n"], v["num_stages"])
              for kind in (0, 1) for v in _lib.variants(kind)}
  for key, data in loaded.items():
    assert len(data) >= 4, key
    for cfg in data:
      assert (cfg.block_m, cfg.block_n, cfg.block_k, cfg.waves_m, cfg.waves_n, cfg.num_stages) in compiled
    spec = json.loads(key.to_json())
    lhs = spec["lhs"]["qvalue"] if isinstance(spec["lhs"], dict) else spec["lhs"]
    rows = int(lhs[lhs.index("[") + 1:lhs.index(",")])
    groups = spec["group_sizes"]["num_groups"] if isinstance(spec["group_sizes"], dict) else 8
    small_m = rows <= 8 * groups  # a few rows per group: the streaming kernel; the others are large shapes
    assert (data.fastest_config.block_m == 16) if small_m else (data.fastest_config.block_m >= 128)


def test_cache_file_name_and_json_round_trip(tmp_path):
  op = hip.HipRaggedDot()
  assert cache_lib.op_file_name(op) == "hip_ragged_dot.json"
  assert cache_lib.device_dir_name("AMD Instinct MI355X") == "amd_instinct_mi355x"
  spec = arg_specs.ARG_SPECS[0].args
  ba = op.bind(**spec)
  key_json = ba.autotuning_cache_key.to_json()
  parsed = json.loads(key_json)
  # same schema as the reference's shipped caches
  assert parsed["lhs"] == "bf16[131072,7168]" and parsed["rhs"] == "bf16[256,7168,1024]"
  assert parsed["group_sizes"] == {"num_groups": 256, "total_size": 131072}
  assert parsed["ragged_dot_dimension_numbers"]["dot_dimension_numbers"] == [[[1], [1]], [[], []]]
  assert parsed["precision"] == ["DEFAULT", "DEFAULT"] and parsed["preferred_element_type"] is None
  cfg = hip.Config(block_m=128, block_n=256, block_k=64, waves_m=2, waves_n=4, num_stages=3)
  text = cache_lib.dumps(op, {ba.autotuning_cache_key: autotuner_lib.AutotuningData({cfg: _bench(1.5), hip.Config(64, 128, 64): RuntimeError("x")})})
  loaded = cache_lib.loads(op, text)
  assert list(loaded) == [ba.autotuning_cache_key]
  assert loaded[ba.autotuning_cache_key].fastest_config == cfg
  # a reference-format key (as in its shipped JSON) parses into the same cache key
  ref_key = ('{"lhs":"bf16[131072,7168]","rhs":"bf16[256,7168,1024]","group_sizes":{"num_groups":256,"total_size":131072},'
             '"ragged_dot_dimension_numbers":{"dot_dimension_numbers":[[[1],[1]],[[],[]]],"lhs_ragged_dimensions":[0],'
             '"rhs_group_dimensions":[0]},"precision":["DEFAULT","DEFAULT"],"preferred_element_type":null,'
             '"return_residuals":false,"activation":null,"manual_axis_type":null,"group_offset":null,"rhs_scale":null,'
             '"rhs_bias":null,"maybe_quantize_lhs":false,"zero_initialize":true,"fuse_gateup_activation":null,'
             '"lhs_quantization_dtype":null,"rhs_quantization_dtype":null}')
  assert op.bind(**op.arg_spec_from_json(json.loads(ref_key))).autotuning_cache_key == ba.autotuning_cache_key
  # shipped cache for MI355X parses and every config in it names a compiled kernel variant
  shipped = cache_lib.cache_file(op, "AMD Instinct MI355X")
  if os.path.exists(shipped):
    entries = cache_lib.loads(op, open(shipped).read())
    assert entries
    table = hip._variant_table()
    tiles = {v for vs in table.values() for v in vs}
    for data in entries.values():
      for c in data:
        assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages) in tiles


def test_autotune_discovers_the_ops_a_function_calls():
  """`get_bound_args(f, *args, **kwargs)` and `autotune(f, *args)` (autotuning/api.py:202-239, :322-418; test pattern of
  autotuning/api_test.py:42-60): the ops a function calls are found by running it, unique by (op, cache key), in call
  order, without the config of the call; a list of bound arguments is taken as it is."""
  class _Timer(autotuner_lib.Autotuner):
    def autotune(self, fn_factory, configs, *args, timeout=None, **kwargs):
      out = {}
      for c in configs:
        try:
          fn_factory(c)(*args, **kwargs)
          out[c] = _bench(float(c.foo))
        except Exception as e:  # pylint: disable=broad-exception-caught
          out[c] = e
      return autotuner_lib.AutotuningData(out)

  op = _FakeOp()

  def f(x, y, scale=1.0):
    a = op(x, y)                               # [3] + [3]
    b = _FakeOp(config=_FakeConfig(7))(a, a)   # the same op and shapes again, with an explicit config: one entry
    c = op(torch.zeros(5), torch.zeros(5))     # another shape: a second entry
    return b * scale, c

  x = torch.zeros(3)
  found = tokamax_amd.get_bound_args(f, x, x, scale=2.0)
  assert [tuple(ba.arguments["x"].shape) for ba in found] == [(3,), (5,)]
  assert all(ba.op.config is None for ba in found)
  assert op_lib.OP_CALL_RECORDER.get() is None  # nothing is recorded outside
  assert tokamax_amd.get_bound_args(list(found)) == found
  with pytest.raises(ValueError, match="only supported if `f` is callable"):
    tokamax_amd.get_bound_args(list(found), x)
  with pytest.raises(TypeError):
    tokamax_amd.get_bound_args(3)

  res = tokamax_amd.autotune(f, x, x, autotuner=_Timer())
  assert isinstance(res, tokamax_amd.AutotuningResult) and len(res.data) == 2
  assert res.device_kind == op_lib.device_kind()
  for ba, data in res.data:
    assert data.fastest_config == _FakeConfig(1) and isinstance(data[_FakeConfig(13)], RuntimeError)
  assert [ba for ba, _ in res.data] == list(found)
  with res:  # the result works as an overlay: the next call of `f` runs with the tuned config
    assert op.bind(x, x).default_config == _FakeConfig(1)
  assert op.bind(x, x).default_config == _FakeConfig(42)
  # from a list of bound arguments; ops that already have cached data are skipped unless ignore_cache
  assert len(tokamax_amd.autotune(list(found), autotuner=_Timer()).data) == 2
  with res:
    assert len(tokamax_amd.autotune(f, x, x, autotuner=_Timer()).data) == 0
    assert len(tokamax_amd.autotune(f, x, x, autotuner=_Timer(), ignore_cache=True).data) == 2

  # an op that cannot be tuned is logged and left out, the others still come back (api.py:403-416)
  class _Broken(autotuner_lib.Autotuner):
    def autotune(self, fn_factory, configs, *args, timeout=None, **kwargs):
      if args[0].shape == (5,):
        raise RuntimeError("no timer")
      return _Timer().autotune(fn_factory, configs, *args, timeout=timeout, **kwargs)

  assert [tuple(ba.arguments["x"].shape) for ba, _ in tokamax_amd.autotune(f, x, x, autotuner=_Broken()).data] == [(3,)]


def test_bound_args_and_autotuning_result_round_trip():
  op = hip.HipRaggedDot()
  for spec in arg_specs.ARG_SPECS:  # ops/op_test.py:201-237 does this over all arg specs
    ba = op.bind(**spec.args)
    d = ba.to_json_dict()
    assert d["op"]["__class__"] == "HipRaggedDot"
    ba2 = op.bind(**op.arg_spec_from_json(json.loads(json.dumps(d["arguments"]))))
    assert ba2 == ba and hash(ba2) == hash(ba)
  ba = op.bind(**arg_specs.ARG_SPECS[-1].args)
  res = tokamax_amd.AutotuningResult("AMD Instinct MI355X", ((ba, autotuner_lib.AutotuningData({hip.Config(128, 128, 64): _bench(2.0)})),))
  back = tokamax_amd.AutotuningResult.loads(res.dumps(), {"HipRaggedDot": op})
  assert back.device_kind == res.device_kind and back.data[0][0] == ba
  assert back.data[0][1].fastest_config == hip.Config(128, 128, 64)


def test_hip_config_validation_and_heuristics():
  with pytest.raises(ValueError, match="multiple of 8"):
    hip.Config(block_m=12, block_n=128, block_k=64)
  with pytest.raises(ValueError, match="positive"):
    hip.Config(block_m=16, block_n=0, block_k=64)
  op = hip.HipRaggedDot()
  table = hip._variant_table()
  for spec in arg_specs.ARG_SPECS:
    ba = op.bind(**spec.args)
    c = ba.heuristics_config
    assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages) in table[(0, _lib.TKX_BF16, _lib.TKX_BF16)]
    configs = ba.autotuning_configs
    assert c in configs and len(configs) > 10
  # decode-like int8 weights pick a short m-tile; unsupported dtypes raise NotImplementedError
  q = tokamax_amd.QArray(ShapeDtype((128, 2048, 768), torch.int8), ShapeDtype((128, 1, 768), torch.float32))
  ba = op.bind(ShapeDtype((256, 2048), torch.bfloat16), q, group_sizes=base.GroupSizes(ShapeDtype((128,), torch.int32), 256))
  assert ba.heuristics_config.block_m == 16  # the streaming small-m kernel
  assert ba.heuristics_config.block_n == 128  # 128 x 3 wide workgroups would fill 256 CUs unevenly
  q = tokamax_amd.QArray(ShapeDtype((128, 2048, 1024), torch.int8), ShapeDtype((128, 1, 1024), torch.float32))
  ba = op.bind(ShapeDtype((256, 2048), torch.bfloat16), q, group_sizes=base.GroupSizes(ShapeDtype((128,), torch.int32), 256))
  assert (ba.heuristics_config.block_m, ba.heuristics_config.block_n) == (16, 256)  # 512 wide workgroups: two per CU
  with pytest.raises(NotImplementedError):
    _ = op.bind(ShapeDtype((256, 2048), torch.float64), ShapeDtype((8, 2048, 768), torch.float64),
                group_sizes=base.GroupSizes(ShapeDtype((8,), torch.int32), 256)).heuristics_config


def test_quantised_operand_routes():
  """Which kernels a pair of quantised operands takes (mode, lhs kind, rhs kind of the variant key), decided on
  shapes alone: epilogue scales, scales folded in per k-block, weights scaled while widened, or the widening pass."""
  op = hip.HipRaggedDot()
  f8, i8, bf, f32 = torch.float8_e4m3fn, torch.int8, torch.bfloat16, torch.float32
  F8, I8, BF = _lib.TKX_F8E4M3FN, _lib.TKX_I8, _lib.TKX_BF16
  m, k, n, G = 4096, 1024, 512, 8
  q = lambda shape, dt, sshape: tokamax_amd.QArray(ShapeDtype(shape, dt), ShapeDtype(sshape, f32))
  gsz = base.GroupSizes(ShapeDtype((G,), torch.int32), m)
  def key(lhs, rhs):
    return op._problem(op.bind(lhs, rhs, group_sizes=gsz))[1]
  lhs16 = ShapeDtype((m, k), bf)
  assert key(q((m, k), f8, (m, 1)), q((G, k, n), f8, (G, 1, n))) == (0, F8, F8)              # epilogue scales
  assert key(q((m, k), f8, (1, 1)), q((G, k, n), f8, (1, 1, 1))) == (0, F8, F8)              # one scale per tensor
  assert key(q((m, k), f8, (m, k // 128)), q((G, k, n), f8, (G, k // 128, n))) == (4, F8, F8)        # folded per k-block
  assert key(q((m, k), f8, (m, k // 128)), q((G, k, n), f8, (G, k // 128, n // 128))) == (4, F8, F8)  # 128 x 128 blocks
  assert key(q((m, k), i8, (m, 1)), q((G, k, n), i8, (G, 1, n))) == (0, I8, I8)              # int8 MFMAs, epilogue scales
  assert key(q((m, k), i8, (m, k // 64)), q((G, k, n), i8, (G, k // 64, n))) == (4, I8, I8)
  assert key(lhs16, q((G, k, n), i8, (G, 1, n))) == (0, BF, I8)
  assert key(lhs16, q((G, k, n), i8, (G, k // 128, n))) == (4, BF, I8)                       # scaled while widened
  assert key(lhs16, q((G, k, n), f8, (G, 1, n))) == (4, BF, F8)
  assert key(q((m, k), f8, (m, 1)), q((G, k, n), f8, (G, k // 128, n))) == (4, BF, F8)       # lhs widened for it
  assert key(lhs16, q((G, k, n), i8, (G, k // 32, n))) == (0, BF, BF)                        # t_k = 32: the widening pass
  assert key(q((m, k), f8, (m, k // 32)), q((G, k, n), f8, (G, k // 32, n))) == (0, BF, BF)
  assert key(lhs16, q((G, k, n), i8, (G // 2, 1, n))) == (0, BF, I8)                        # shared by pairs of groups: repeated
  with pytest.raises(NotImplementedError):
    key(lhs16, q((G, k, n), i8, (3, 1, n)))                                                   # a scale array that tiles nothing
  # the k-step of the chosen variant divides the rows of a scale block
  ba = op.bind(q((m, k), i8, (m, k // 64)), q((G, k, n), i8, (G, k // 64, n)), group_sizes=gsz)
  assert 64 % ba.heuristics_config.block_k == 0


def test_arg_specs_and_flops():
  names = {s.full_name for s in arg_specs.ARG_SPECS}
  assert {"compute_bound", "memory_bound", "mixtral_8x7b"} <= names
  s = next(s for s in arg_specs.ARG_SPECS if s.name == "8x7b")
  assert arg_specs.flops(**s.args) == 2 * 8192 * 4096 * 14336  # bench.py:52-56


def test_uint8_storage_is_packed_int4_and_nothing_else():
  """A uint8 `qvalue` is two int4 per byte only under a 4-bit `qtype`; any other uint8 quantised array is declined when
  it is made, instead of being read as nibbles."""
  from tokamax_amd import quantization
  q = ShapeDtype((4, 64, 32), torch.uint8)
  scale = ShapeDtype((4, 1, 32), torch.float32)
  packed = quantization.QArray(q, scale, None, torch.int4)
  assert packed.packed and packed.shape == (4, 128, 32)
  for qtype in (None, torch.uint8, torch.int8):
    with pytest.raises(NotImplementedError):
      quantization.QArray(q, scale, None, qtype)
  plain = quantization.QArray(ShapeDtype((4, 64, 32), torch.int8), scale, None, torch.int4)
  assert not plain.packed and plain.shape == (4, 64, 32)


def test_ffi_shim_compiles_to_its_stub_without_the_xla_header(tmp_path):
  """tokamax_amd/csrc/ffi_shim.cc holds the XLA FFI handlers behind `__has_include("xla/ffi/api/ffi.h")`; without the
  header (this image has no jaxlib) it must still compile, to a stub that says so."""
  import shutil
  import subprocess
  cxx = shutil.which("g++") or shutil.which("c++")
  if cxx is None:
    pytest.skip("no host C++ compiler")
  src = os.path.join(ROOT, "tokamax_amd", "csrc", "ffi_shim.cc")
  out = tmp_path / "libshim.so"
  subprocess.check_call([cxx, "-std=c++17", "-shared", "-fPIC", "-I", os.path.join(ROOT, "include"), src, "-o", str(out)])
  lib = ctypes.CDLL(str(out))
  lib.tkx_ffi_shim_available.restype = ctypes.c_int32
  assert lib.tkx_ffi_shim_available() == 0
  text = open(src).read()
  for symbol in ("TkxRaggedDotFwd", "TkxRaggedDotFwdFused", "TkxRaggedDotFwdFp8Out", "TkxRaggedDotDrhs"):
    assert f"XLA_FFI_DEFINE_HANDLER_SYMBOL({symbol}," in text
    assert text.count("TKX_CONFIG_ATTRS") >= 5  # the definition and one use per handler
  # Every field of TkxConfig travels as an attribute of its name and is assigned by name (no positional initialiser
  # that a new trailing field would silently leave out).
  for name, _ in _lib.TkxConfig._fields_:
    assert f'.Attr<int32_t>("{name}")' in text, name
    assert f"cfg.{name} = {name};" in text, name
  assert "const TkxConfig cfg{" not in text
  header = open(os.path.join(ROOT, "include", "tkx_ragged_dot.h")).read()
  struct = header[header.index("typedef struct TkxConfig {"):header.index("} TkxConfig;")]
  declared = [line.split()[1].rstrip(";") for line in struct.splitlines() if line.strip().startswith("int32_t ")]
  assert declared == [name for name, _ in _lib.TkxConfig._fields_]


def test_heuristics_on_abstract_arguments_split_and_packed_int4():
  """Config choice needs no GPU: shapes and types only. A launch of the streaming kernel with fewer (group, column
  tile) pairs than CUs gets its contraction split (8 ways at most, and only as far as k divides); packed int4 weights
  stay packed (their own variant key) where a kernel reads them as they are and count as int8 storage otherwise; a QArray
  of packed int4 reports the shape of its values."""
  op = hip.HipRaggedDot()
  bf16, f32, i8, u8 = torch.bfloat16, torch.float32, torch.int8, torch.uint8

  def config(m, k, n, groups, rhs_dtype=bf16, packed=False):
    lhs = ShapeDtype((m, k), bf16)
    gs = ShapeDtype((groups,), torch.int32)
    if rhs_dtype == bf16:
      rhs = ShapeDtype((groups, k, n), bf16)
    else:
      rhs = tokamax_amd.QArray(ShapeDtype((groups, k // 2 if packed else k, n), rhs_dtype), ShapeDtype((groups, 1, n), f32),
                               None, getattr(torch, "int4", i8) if packed else None)
    return op._get_heuristics_config(op.bind(lhs, rhs, group_sizes=gs))

  assert hip._streaming_split(768, 2048, 128, 2) == 1     # a tile or more per CU: never split
  assert hip._streaming_split(64, 8192, 128, 2) == 4      # up to 256 workgroups
  assert hip._streaming_split(16, 16384, 128, 4) == 8     # 8 ways at most
  assert hip._streaming_split(16, 1024, 128, 2) == 4      # as far as k divides: 1024 % (128 * 8 * 2) != 0
  assert hip._streaming_split(16, 16384, 256, 2) == 1     # the wide form has no split
  c = config(16, 8192, 1024, 8, i8)
  assert (c.block_m, c.block_n, c.split_k) == (16, 128, 4)
  c = config(256, 2048, 768, 128, i8)
  assert (c.block_m, c.split_k) == (16, 1)
  packed = tokamax_amd.QArray(ShapeDtype((8, 512, 256), u8), ShapeDtype((8, 1, 256), f32), None, getattr(torch, "int4", i8))
  assert packed.packed and packed.shape == (8, 1024, 256) and packed.scale_tile_shape == (1, 1024, 1)
  assert packed.unpacked().qvalue.shape == (8, 1024, 256) and packed.unpacked().qvalue.dtype == i8
  c = config(16, 1024, 256, 8, u8, packed=True)          # 2 rows per group: the streaming kernel reads the bytes
  assert c.block_m == 16
  c = config(4096, 1024, 4096, 8, u8, packed=True)       # 512 rows per group: a tiled kernel reads the bytes too,
  assert (c.block_m, c.block_n, c.waves_m, c.waves_n) == (128, 256, 1, 8)  # the one whose workgroups share a CU in pairs
  c = config(4096, 1024, 4096, 8, i8)                    # ... as for int8 weights (two stages: 64 KB of LDS)
  assert (c.block_m, c.block_n, c.waves_m, c.waves_n, c.num_stages) == (128, 256, 1, 8, 2)
  c = config(4096, 1024, 256, 8, u8, packed=True)        # ... a smaller tile where 256 x 256 would leave most CUs idle
  assert c.block_m in (32, 64)
  lhs, gs = ShapeDtype((4096, 1024), bf16), ShapeDtype((8,), torch.int32)
  route = lambda rhs, **kw: op._problem(op.bind(lhs, rhs, group_sizes=gs, **kw))[1]
  assert route(packed)[2] == _lib.TKX_I4X2
  # ... also with a bias, with gate-up fusion, and with scale blocks of a power of two >= 64 rows along k (the forms
  # the tiled kernels have for int8 weights); unpacked first for gate-up fusion over scale blocks, blocks of 32
  # rows, a contraction that is not a multiple of the k-step
  assert route(packed, rhs_bias=ShapeDtype((8, 1, 256), f32))[2] == _lib.TKX_I4X2
  assert route(packed, fuse_gateup_activation="silu")[::2] == (3, _lib.TKX_I4X2)
  int4 = getattr(torch, "int4", i8)
  blocks = tokamax_amd.QArray(ShapeDtype((8, 512, 256), u8), ShapeDtype((8, 4, 256), f32), None, int4)
  assert route(blocks)[::2] == (4, _lib.TKX_I4X2)
  assert op._get_heuristics_config(op.bind(lhs, blocks, group_sizes=gs)).block_n == 256
  assert route(blocks, fuse_gateup_activation="silu")[2] != _lib.TKX_I4X2
  small_blocks = tokamax_amd.QArray(ShapeDtype((8, 512, 256), u8), ShapeDtype((8, 32, 256), f32), None, int4)
  assert route(small_blocks)[2] != _lib.TKX_I4X2
  few_rows = op.bind(ShapeDtype((16, 1024), bf16), small_blocks, group_sizes=gs)   # ... which the streaming kernel takes
  assert op._problem(few_rows)[1][::2] == (4, _lib.TKX_I4X2) and op._get_heuristics_config(few_rows).block_m == 16
  assert {x.block_m for x in op._get_autotuning_configs(few_rows)} == {16}
  odd = tokamax_amd.QArray(ShapeDtype((8, 48, 256), u8), ShapeDtype((8, 1, 256), f32), None, int4)
  assert op._problem(op.bind(ShapeDtype((4096, 96), bf16), odd, group_sizes=gs))[1][2] == _lib.TKX_I8
  space = op._get_autotuning_configs(op.bind(lhs, packed, group_sizes=gs))
  assert {x.block_m for x in space} >= {16, 32, 128, 256}
  # fp8 activations with one scale per row (or per run of rows): the packed weights stay packed for the kernels that
  # feed the nibbles to the fp8 MFMAs (one row of waves: each nibble becomes an fp8 byte once per workgroup); with scale
  # fp8 activations over int8 storage are widened to bf16; gate-up fusion has kernels of the same kind
  f8 = torch.float8_e4m3fn
  x8 = tokamax_amd.QArray(ShapeDtype((4096, 1024), f8), ShapeDtype((4096, 1), f32))
  route8 = lambda x, rhs, **kw: op._problem(op.bind(x, rhs, group_sizes=gs, **kw))[1]
  assert route8(x8, packed) == (0, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  assert route8(x8, packed, rhs_bias=ShapeDtype((8, 1, 256), f32)) == (0, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  shared = tokamax_amd.QArray(ShapeDtype((4096, 1024), f8), ShapeDtype((16, 1), f32))
  assert route8(shared, packed) == (0, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  wide = tokamax_amd.QArray(ShapeDtype((8, 512, 4096), u8), ShapeDtype((8, 1, 4096), f32), None, int4)
  # 512 rows per group, and 128: the 128-row tile on one row of four waves, whose workgroups share a CU in pairs
  c = op._get_heuristics_config(op.bind(x8, wide, group_sizes=gs))
  assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages) == (128, 256, 128, 1, 4, 2)
  fewer = tokamax_amd.QArray(ShapeDtype((1024, 1024), f8), ShapeDtype((1024, 1), f32))
  c = op._get_heuristics_config(op.bind(fewer, wide, group_sizes=gs))
  assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n) == (128, 256, 128, 1, 4)
  c = op._get_heuristics_config(op.bind(x8, wide, group_sizes=gs, fuse_gateup_activation="silu"))
  assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n) == (128, 256, 128, 1, 4)
  assert {x.block_k for x in op._get_autotuning_configs(op.bind(x8, wide, group_sizes=gs))} == {128}
  # scale blocks of a power of two >= 128 rows along k (lhs scales per row or per (row, same block)): kernels of the
  # same kind that fold every k-step's products in with its scales; smaller blocks are unpacked and widened
  assert route8(x8, blocks) == (4, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  c = op._get_heuristics_config(op.bind(x8, blocks, group_sizes=gs))
  assert (c.block_n, c.block_k) == (256, 128)
  x8_same = tokamax_amd.QArray(ShapeDtype((4096, 1024), f8), ShapeDtype((4096, 4), f32))
  assert route8(x8_same, blocks) == (4, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  assert route8(x8, small_blocks)[2] != _lib.TKX_I4X2
  assert route8(x8, packed, fuse_gateup_activation="silu") == (3, _lib.TKX_F8E4M3FN, _lib.TKX_I4X2)
  assert route8(x8, blocks, fuse_gateup_activation="silu") == (3, _lib.TKX_BF16, _lib.TKX_BF16)
  assert route8(x8, packed.unpacked()) == (0, _lib.TKX_BF16, _lib.TKX_I8)
  # int8 activations: the int8 MFMAs on the nibbles; again the tile whose 4-wave workgroups share a CU in pairs
  xi8 = tokamax_amd.QArray(ShapeDtype((4096, 1024), i8), ShapeDtype((4096, 1), f32))
  assert route8(xi8, packed) == (0, _lib.TKX_I8, _lib.TKX_I4X2) and route8(xi8, blocks) == (4, _lib.TKX_I8, _lib.TKX_I4X2)
  assert route8(xi8, packed, fuse_gateup_activation="silu") == (3, _lib.TKX_I8, _lib.TKX_I4X2)
  assert route8(xi8, blocks, fuse_gateup_activation="silu")[2] != _lib.TKX_I4X2
  c = op._get_heuristics_config(op.bind(xi8, wide, group_sizes=gs))
  assert (c.block_m, c.block_n, c.block_k, c.waves_m, c.waves_n, c.num_stages) == (128, 256, 128, 1, 4, 2)
  x8_blocks = tokamax_amd.QArray(ShapeDtype((4096, 1024), f8), ShapeDtype((4096, 8), f32))
  assert route8(x8_blocks, packed)[1:] == (_lib.TKX_BF16, _lib.TKX_I8)
  # the key of an autotuning cache entry names the 4-bit type and comes back as the same abstract QArray
  from tokamax_amd import serialization
  spec = serialization.to_jsonable(packed)
  assert spec["qvalue"] == "u8[8,512,256]" and spec["qtype"].endswith("int4" if hasattr(torch, "int4") else "int8")
  assert serialization.array_spec_from_json(json.loads(json.dumps(spec))) == packed


def test_heuristics_split_the_last_round_of_tiled_launches_with_few_rounds():
  """A tiled forward / dlhs launch of fewer than 8 rounds of 256 workgroups gets `split_k` = 4 (the kernel cuts only
  the tiles of a partial last round, and decides into how many parts); longer launches, drhs, gate-up fusion and tiles
  of fewer than 128 rows do not; the search space offers both forms where the heuristics split."""
  op = hip.HipRaggedDot()
  bf16 = torch.bfloat16
  gs = lambda groups: ShapeDtype((groups,), torch.int32)
  assert hip._tiled_split_pays(1, 128, 256, 4096, 4096, 8) and not hip._tiled_split_pays(0, 256, 256, 16384, 14336, 8)
  assert not hip._tiled_split_pays(2, 256, 256, 4096, 4096, 8) and not hip._tiled_split_pays(0, 64, 128, 512, 512, 8)
  vjp_dlhs = op.bind(ShapeDtype((4096, 14336), bf16), ShapeDtype((8, 4096, 14336), bf16), group_sizes=gs(8),
                     ragged_dot_dimension_numbers=base.TRANS_RHS_RAGGED_DOT_DIM_NUMS)
  c = op._get_heuristics_config(vjp_dlhs)
  assert c.block_m >= 128 and c.split_k == 4
  space = op._get_autotuning_configs(vjp_dlhs)
  assert any(x.split_k == 4 for x in space) and any(x.split_k == 1 and x.block_m == c.block_m for x in space)
  assert all(x.split_k == 1 for x in space if x.block_m < 128)
  mixtral = op.bind(ShapeDtype((16384, 4096), bf16), ShapeDtype((8, 4096, 14336), bf16), group_sizes=gs(8))
  assert op._get_heuristics_config(mixtral).split_k == 1
  assert all(x.split_k == 1 for x in op._get_autotuning_configs(mixtral) if x.block_m != 16)
  drhs = op.bind(ShapeDtype((4096, 4096), bf16), ShapeDtype((4096, 14336), bf16), group_sizes=gs(8),
                 ragged_dot_dimension_numbers=base.RAGGED_CONTRACTING_DOT_DIM_NUMS)
  assert op._get_heuristics_config(drhs).split_k == 1
  glu = op.bind(ShapeDtype((2048, 1024), bf16), ShapeDtype((8, 1024, 2048), bf16), group_sizes=gs(8),
                fuse_gateup_activation="silu")
  assert op._get_heuristics_config(glu).split_k == 1


def test_tile_cost_model_picks_near_the_fastest_measured_variant():
  """The heuristics rank tiled variants of 16-bit forward / dlhs launches by `_tile_cost`. On the shipped timings (every
  variant on 122 shapes of bf16 operands) its pick stays within 6 % of the fastest variant on average and 35 % at worst, and its time
  estimates follow the form of the data: more rows or a longer contraction never cost less, and a launch with a sliver
  of a last round gains from the split while one without a partial round does not."""
  from tokamax_amd.data.autotuning import tile_cost
  entries = [e for e in tile_cost.load() if e.get("rhs", "bf16") == "bf16" and e["mode"] != 2]
  assert len(entries) >= 100 and all(len(e["timings"]) >= 10 for e in entries)
  mean, worst = tile_cost.summary(tile_cost.gaps(entries, hip._TILE_COST_FIT))
  assert mean < 0.06 and worst < 0.35, (mean, worst)
  # the config the heuristics hand out for those problems (model, rules for the streaming kernel, split decision), and
  # for quantised operands and drhs, where rules on rows per group and on the fill of the chip choose the tile
  label = lambda e: "drhs" if e["mode"] == 2 else e.get("rhs", "bf16")
  for kind, count, most in (("bf16", 122, 0.06), ("int8", 26, 0.08), ("int4", 26, 0.06), ("fp8", 26, 0.03), ("fp8i4", 43, 0.04), ("fp8i4k", 26, 0.02), ("fp8i4glu", 26, 0.05), ("int8i4", 26, 0.04), ("int8i4k", 26, 0.03), ("int8i4glu", 26, 0.03),
                            ("int8x8", 12, 0.03), ("drhs", 26, 0.03), ("glu", 26, 0.06), ("int8k", 26, 0.04), ("f32", 12, 0.01)):
    some = [e for e in tile_cost.load() if label(e) == kind]
    mean, worst = tile_cost.summary([tile_cost.heuristics_gap(e) for e in some])
    assert len(some) >= count and mean < most and worst < 0.4, (kind, mean, worst)
  v = (256, 256, 64, 2, 2, 2)
  costs = [hip._tile_cost(v, 1, rows, 4096, 4096, 8) for rows in (1024, 4096, 16384, 65536, 262144)]
  assert costs == sorted(costs) and costs[-1] > 30 * costs[1]
  assert hip._tile_cost(v, 1, 16384, 4096, 8192, 8) > 1.8 * hip._tile_cost(v, 1, 16384, 4096, 4096, 8)
  # 4096 x 14336 x 4096 in 8 groups of 512 rows: 16 * 56 = 896 tiles = 3.5 rounds of 256
  assert hip._tile_cost((256, 256, 64, 2, 4, 3), 4, 4096, 14336, 4096, 8) < hip._tile_cost((256, 256, 64, 2, 4, 3), 1, 4096, 14336, 4096, 8)
  # ... and 16 * 64 = 1024 tiles = 4 full rounds: nothing to split
  assert hip._tile_cost((256, 256, 64, 2, 4, 3), 4, 4096, 16384, 4096, 8) == hip._tile_cost((256, 256, 64, 2, 4, 3), 1, 4096, 16384, 4096, 8)
  # the bound launch asks the same model: the headline prefill shape gets the 256 x 256 tile, 64 rows per group a 128-row one
  # (both the fastest measured)
  op = hip.HipRaggedDot()
  bf16 = torch.bfloat16
  big = op.bind(ShapeDtype((16384, 4096), bf16), ShapeDtype((8, 4096, 14336), bf16), group_sizes=ShapeDtype((8,), torch.int32))
  c = op._get_heuristics_config(big)
  assert (c.block_m, c.block_n) == (256, 256)
  small = op.bind(ShapeDtype((3584, 1536), bf16), ShapeDtype((56, 1536, 9216), bf16), group_sizes=ShapeDtype((56,), torch.int32))
  assert op._get_heuristics_config(small).block_m == 128


def test_bind_without_inspect_matches_the_signature_path():
  """`RaggedDot.bind` names every parameter of `_fwd` itself and skips `inspect`; the result is the one
  `Signature.bind` + `apply_defaults` gives, in signature order, and unknown or missing names still fail."""
  op = hip.HipRaggedDot()
  lhs, rhs = ShapeDtype((64, 128), torch.bfloat16), ShapeDtype((4, 128, 256), torch.bfloat16)
  gs = ShapeDtype((4,), torch.int32)
  ba = op.bind(lhs, rhs, group_sizes=gs, preferred_element_type=torch.float32)
  names = list(op._fwd_signature.parameters)
  assert list(ba.arguments) == names
  slow = op_lib.Op.bind(op, **dict(ba.arguments))
  assert list(slow.arguments) == names and all(slow.arguments[n] is ba.arguments[n] or slow.arguments[n] == ba.arguments[n]
                                                for n in names)
  with pytest.raises(TypeError):
    op._bind_all(lhs=lhs, rhs=rhs, group_sizes=gs, no_such_parameter=1)
  with pytest.raises(TypeError):
    op._bind_all(lhs=lhs, rhs=rhs)


def test_config_json_without_split_k_loads_with_the_default():
  """Cache files written before `split_k` existed name configs without it; they load as split_k = 1."""
  cfg = hip.Config(**json.loads('{"block_m":16,"block_n":128,"block_k":32,"waves_m":1,"waves_n":4,"num_stages":2,'
                                '"grid_tile_width":1,"align_tile":8}'))
  assert cfg.split_k == 1 and cfg.to_kernel_config().split_k == 1
  assert json.loads(cache_lib.config_to_json(hip.Config(16, 128, 32, 1, 4, 2, 1, 8, 4)))["split_k"] == 4
  c = cfg.to_kernel_config().to_c()
  assert cfg.persistent == 0 and json.loads(cache_lib.config_to_json(hip.Config(16, 128, 32, 1, 4, 2, 1, 8, 1, 3)))["persistent"] == 3
  assert ctypes.sizeof(c) == 10 * 4 and c.split_k == 1 and c.persistent == 0
  with pytest.raises(ValueError):
    hip.Config(16, 128, 32, 1, 4, 2, 1, 8, 1, -1)
