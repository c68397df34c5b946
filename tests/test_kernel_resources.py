"""Host-side check of the persistent stream kernels' machine code (no GPU needed: hipcc cross-compiles).

A register that the compiler parks in scratch memory and reloads INSIDE a stream kernel's main loop costs far more than
a reload elsewhere: the reload waits for every global -> LDS request in flight, i.e. a full memory latency per loop
iteration (the int4 kernel once ran 1.5x slower for exactly this reason, with every parity test green).  The check
compiles each stream kernel to assembly and fails if a scratch access sits in a loop nested inside the tile loop.
"""

import os
import re
import shutil
import subprocess
from concurrent.futures import ThreadPoolExecutor

import pytest

from maxtext_amd import build

STREAM_KERNELS = ["moe_gmm_dls.hip", "moe_gmm_dlw.hip", "moe_gmm_f8s.hip"]


def _assembly(src, tmp):
  hipcc = shutil.which("hipcc") or "/opt/rocm/bin/hipcc"
  flags = [f for f in build.HIPCC_FLAGS if f != "-shared"]
  out = os.path.join(tmp, src.replace(".hip", ".s"))
  cmd = [hipcc] + flags + ["-I", build.INCLUDE, "-I", build.CSRC, "-S", "--cuda-device-only", os.path.join(build.CSRC, src), "-o", out]
  res = subprocess.run(cmd, capture_output=True, text=True)
  assert res.returncode == 0, res.stderr[-2000:]
  return open(out).read()


def _scratch_in_inner_loops(asm):
  """-> {kernel: scratch accesses in blocks the compiler marks as nested loops (Depth >= 2)}"""
  found = {}
  parts = re.split(r"\n(_ZN3moe\w+):", asm)
  for i in range(1, len(parts), 2):
    name, body = parts[i], parts[i + 1].split(".end_amdhsa_kernel")[0]
    if "_kernel" not in name:
      continue
    depth, count = 0, 0
    for line in body.split("\n"):
      if line.startswith(".LBB"):
        m = re.search(r"Depth=(\d+)", line)
        depth = int(m.group(1)) if m else 0
      if "scratch_" in line and depth >= 2:
        count += 1
    found[name] = count
  return found


@pytest.mark.skipif(not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")), reason="needs hipcc")
def test_stream_kernels_keep_their_main_loops_free_of_scratch_accesses(tmp_path):
  with ThreadPoolExecutor(max_workers=3) as pool:
    texts = list(pool.map(lambda s: _assembly(s, str(tmp_path)), STREAM_KERNELS))
  kernels = {}
  for text in texts:
    kernels.update(_scratch_in_inner_loops(text))
  assert len(kernels) >= 12, sorted(kernels)  # 4 + 6 + 2 instantiations
  bad = {k: v for k, v in kernels.items() if v}
  assert not bad, f"scratch accesses inside the main loop: {bad}"
