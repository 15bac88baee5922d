"""Register budget of the compiled kernels, read from the metadata of the library's gfx950 code objects.

A kernel that spills keeps a scratch allocation per lane (`.private_segment_fixed_size` in the code object's
kernel metadata, the figure hipcc prints as ScratchSize under -Rpass-analysis=kernel-resource-usage): every tile's
accumulators then make a round trip through memory, and a launch pays for the scratch set-up. No kernel of the
library may have one.
"""

import os
import re
import shutil
import subprocess

import pytest

from tokamax_amd import _lib

LLVM = "/opt/rocm/llvm/bin"
TOOLS = [os.path.join(LLVM, t) for t in ("llvm-objcopy", "clang-offload-bundler", "llvm-readelf")]
TARGET = "hipv4-amdgcn-amd-amdhsa--gfx950"


def _kernel_metadata(tmp_path):
  """[(mangled kernel name, scratch bytes per lane, vgprs)] over every code object bundled into the library."""
  fat = tmp_path / "fatbin"
  subprocess.run([TOOLS[0], "-O", "binary", "--only-section=.hip_fatbin", _lib.LIB_PATH, str(fat)], check=True)
  blob = fat.read_bytes()
  starts = [m.start() for m in re.finditer(rb"__CLANG_OFFLOAD_BUNDLE__", blob)]  # one bundle per source file
  rows = []
  for n, first in enumerate(starts):
    part, code = tmp_path / f"bundle{n}", tmp_path / f"bundle{n}.co"
    part.write_bytes(blob[first:starts[n + 1] if n + 1 < len(starts) else len(blob)])
    subprocess.run([TOOLS[1], "--unbundle", "--type=o", f"--input={part}", f"--targets={TARGET}", f"--output={code}"], check=True)
    notes = subprocess.run([TOOLS[2], "--notes", str(code)], check=True, capture_output=True, text=True).stdout
    name = scratch = None
    for line in notes.splitlines():
      if m := re.match(r"\s+\.name:\s+(\S+)", line):
        name = m.group(1)
      elif m := re.match(r"\s+\.private_segment_fixed_size:\s+(\d+)", line):
        scratch = int(m.group(1))
      elif m := re.match(r"\s+\.vgpr_count:\s+(\d+)", line):
        rows.append((name, scratch, int(m.group(1))))
  return rows


@pytest.mark.skipif(not all(os.path.exists(t) for t in TOOLS), reason="ROCm's LLVM tools are not installed")
def test_no_kernel_of_the_library_uses_scratch_memory(tmp_path):
  assert os.path.exists(_lib.LIB_PATH), "build the library first"
  rows = _kernel_metadata(tmp_path)
  names = [r[0] for r in rows]
  # every source file's kernels were seen: the tiled GEMM entries (plain, quantising, split last round), the
  # streaming small-m kernels and their persistent form, the scheduler
  for piece in ("gemm_entry", "gemm_entry_fp8_out", "gemm_entry_split", "decode_kernel", "decode_persistent_kernel", "schedule"):
    assert any(piece in n for n in names), piece
  assert len(rows) >= 200
  # (The fp8 256 x 256 x 128 tile, 32-byte fragments next to 128 accumulators, keeps a few lane constants of the loops
  # that drain the pipeline in scratch, written and read once per tile, outside the steady-state loop.)
  # (Likewise the two tiles on one row of waves of packed int4 weights with scales per k-block: the 256-row one keeps
  # eight lhs fragments double-buffered next to 128 accumulators, the 128-row one lives in 128 registers so that two
  # workgroups share a CU; five to seven lane constants, stored before the k loop and reloaded after it.)
  # (And the 128 x 256 x 128 tile on one row of waves of fp8 activations over packed int4 weights with scales per k-block:
  # 64 accumulators, 64 partial ones and double-buffered 32-byte lhs fragments; eight lane constants, likewise stored
  # before the k loops and reloaded after them.)
  allowed = lambda name: (24 if "GemmKernelILi0ELi3ELi3ELi256ELi256ELi128E" in name else
                          24 if "GemmKernelILi4ELi1ELi5ELi256ELi256ELi64ELi1ELi8E" in name else
                          32 if "GemmKernelILi4ELi1ELi5ELi128ELi256ELi64ELi1ELi8E" in name else
                          32 if "GemmKernelILi4ELi3ELi5ELi128ELi256ELi128ELi1ELi8E" in name else 0)
  spilling = [(n, s) for n, s, _ in rows if s > allowed(n)]
  if spilling and shutil.which("c++filt"):
    spilling = [(subprocess.run(["c++filt", n], capture_output=True, text=True).stdout.strip(), s) for n, s in spilling]
  assert not spilling, spilling
  # the 8-wave tiles run two waves per SIMD: 256 registers each
  headline = [v for n, _, v in rows if "GemmKernelILi0ELi1ELi1ELi256ELi256ELi64ELi2ELi4E" in n]
  assert len(headline) >= 6 and max(headline) <= 256
