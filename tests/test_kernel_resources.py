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


@pytest.mark.skipif(not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")), reason="needs hipcc")
def test_lds_streamed_decode_kernel_uses_no_scratch_and_waits_only_where_written(tmp_path):
  """The persistent int4 decode kernel keeps a tile's activations in registers across work items: every instantiation must
  fit its registers (no scratch at all: a reload would wait for the copies in flight), and inside its item loop the only
  waits on the vector-memory counter are the three explicit ones per segment (8, 4 or 0 copies of younger segments
  outstanding) and those of the side block that loads a new tile's state; a wait the compiler added for a load of its own
  would drain the copies on every item."""
  asm = _assembly("moe_gmm_wqs.hip", str(tmp_path))
  sizes = re.findall(r"\.name:\s+(_ZN3moe14gmm_wqs_kernel\w+)\n\s+\.private_segment_fixed_size:\s+(\d+)", asm)
  assert len(sizes) == 12, sizes  # 2 formats x 3 segment counts x with / without the second projection
  assert all(int(b) == 0 for _, b in sizes), sizes
  parts = re.split(r"\n(_ZN3moe14gmm_wqs_kernel\w+):", asm)
  for i in range(1, len(parts), 2):
    body = parts[i + 1].split(".end_amdhsa_kernel")[0]
    barriers = [m.start() for m in re.finditer(r"s_barrier", body)]
    assert len(barriers) >= 2
    # between the first segment barrier and the last barrier of the loop body: waits are vmcnt(8/4/0) chosen by branches
    loop = body[barriers[0]:barriers[-1]]
    waits = re.findall(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", loop)
    assert set(waits) <= {"8", "4", "0"}, (parts[i], waits)


@pytest.mark.skipif(not (shutil.which("hipcc") or os.path.exists("/opt/rocm/bin/hipcc")), reason="needs hipcc")
def test_lds_streamed_fp8_decode_kernel_uses_no_scratch_and_waits_only_where_written(tmp_path):
  """The persistent fp8 decode kernel follows the same rules: up to 112 registers of activations stay resident per lane, so
  every instantiation must fit its registers, and between the barriers of its item loop the only waits on the
  vector-memory counter are the explicit ones per segment."""
  asm = _assembly("moe_gmm_f8d.hip", str(tmp_path))
  sizes = re.findall(r"\.name:\s+(_ZN3moe14gmm_f8d_kernel\w+)\n\s+\.private_segment_fixed_size:\s+(\d+)", asm)
  assert len(sizes) == 28, sizes  # 14 row lengths (K = 512 .. 7168) x with / without the second projection
  assert all(int(b) == 0 for _, b in sizes), sizes
  parts = re.split(r"\n(_ZN3moe14gmm_f8d_kernel\w+):", asm)
  assert len(parts) == 57
  for i in range(1, len(parts), 2):
    body = parts[i + 1].split(".end_amdhsa_kernel")[0]
    barriers = [m.start() for m in re.finditer(r"s_barrier", body)]
    assert len(barriers) >= 2
    loop = body[barriers[0]:barriers[-1]]
    waits = re.findall(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", loop)
    assert set(waits) <= {"8", "4", "0"}, (parts[i], waits)
    assert "nt lds" in loop and re.search(r"offen lds", loop)  # weights read once stream past the caches, shared ones do not
  # the kernel of the per-row x per-channel scales (activations copied beside the weights): twelve instantiations (16-, 32-
  # and 64-row tiles), no scratch, waits of 5, 6 or 8 (the copies of the segments after it may be outstanding) or 0 between its
  # barriers
  asm = _assembly("moe_gmm_f8l.hip", str(tmp_path))
  sizes = re.findall(r"\.name:\s+(_ZN3moe14gmm_f8l_kernel\w+)\n\s+\.private_segment_fixed_size:\s+(\d+)", asm)
  assert len(sizes) == 12 and all(int(b) == 0 for _, b in sizes), sizes
  parts = re.split(r"\n(_ZN3moe14gmm_f8l_kernel\w+):", asm)
  assert len(parts) == 25
  for i in range(1, len(parts), 2):
    body = parts[i + 1].split(".end_amdhsa_kernel")[0]
    barriers = [m.start() for m in re.finditer(r"s_barrier", body)]
    assert len(barriers) >= 2
    waits = re.findall(r"s_waitcnt[^\n]*vmcnt\((\d+)\)", body[barriers[0]:barriers[-1]])
    assert set(waits) <= {"5", "6", "8", "0"}, (parts[i], waits)

