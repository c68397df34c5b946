"""The C-ABI library loads without a GPU and exports every symbol include/moe_mi355x.h declares."""

import ctypes
import os
import re
import subprocess

import pytest

from maxtext_amd import _lib

ROOT = os.path.dirname(os.path.dirname(os.path.abspath(__file__)))


def _declared_symbols():
  text = open(os.path.join(ROOT, "include", "moe_mi355x.h")).read()
  return sorted(set(re.findall(r"MOE_API\s+[\w\s\*]+?\b(moe_\w+)\s*\(", text)))


def test_header_declares_the_expected_entry_points():
  names = _declared_symbols()
  for must in ("moe_route_topk", "moe_sort_by_expert", "moe_gather_rows", "moe_gmm", "moe_unpermute_combine",
               "moe_gmm_workspace_bytes", "moe_gmm_rhs_kn_supported", "moe_gmm_tuned", "moe_sort_workspace_bytes", "moe_transpose_rhs", "moe_last_error"):
    assert must in names


def test_library_exports_every_declared_symbol():
  if not os.path.exists(_lib.LIB_PATH):
    pytest.fail(f"{_lib.LIB_PATH} has not been built (python -m maxtext_amd.build)")
  lib = ctypes.CDLL(_lib.LIB_PATH)
  for name in _declared_symbols():
    assert hasattr(lib, name), f"{name} declared in the header but not exported"
  assert set(_lib.SIGNATURES) == set(_declared_symbols())


def test_size_queries_and_struct_layout_without_gpu():
  lib = _lib.load()
  assert lib.moe_abi_version() == 3
  assert lib.moe_sort_workspace_bytes(2048, 2, 8) >= (4 * 4 * 8 + 8) * 4
  assert lib.moe_gmm_workspace_bytes(4096, 8) >= 16 + (4096 // 16 + 9) * 16


def test_struct_layout_matches_the_header(tmp_path):
  # the C compiler's view of moe_gmm_args (size and a few offsets) must equal the ctypes mirror
  src = tmp_path / "layout.c"
  src.write_text('#include <stdio.h>\n#include <stddef.h>\n#include "moe_mi355x.h"\n'
                 'int main(void){printf("%zu %zu %zu %zu %zu %zu %zu %zu\\n", sizeof(moe_gmm_args), offsetof(moe_gmm_args, workspace_bytes),'
                 ' offsetof(moe_gmm_args, M), offsetof(moe_gmm_args, act), offsetof(moe_gmm_args, act_limit),'
                 ' offsetof(moe_gmm_args, out_dtype), offsetof(moe_gmm_args, rhs_bias), offsetof(moe_gmm_args, out_row_scale));return 0;}\n')
  exe = tmp_path / "layout"
  subprocess.run(["gcc", "-I", os.path.join(ROOT, "include"), str(src), "-o", str(exe)], check=True)
  got = [int(v) for v in subprocess.run([str(exe)], capture_output=True, text=True, check=True).stdout.split()]
  g = _lib.GmmArgs
  assert got == [ctypes.sizeof(g), g.workspace_bytes.offset, g.M.offset, g.act.offset, g.act_limit.offset, g.out_dtype.offset,
                 g.rhs_bias.offset, g.out_row_scale.offset]


def test_argument_errors_are_reported_not_launched():
  lib = _lib.load()
  st = lib.moe_route_topk(None, None, 4, 8, 2, 0, 0, 1, 1.0, -1, -1, None, None, None)
  assert st == -1 and b"NULL" in lib.moe_last_error()
  a = _lib.GmmArgs()
  a.struct_size = 3
  assert lib.moe_gmm(ctypes.byref(a), None) == -1


def test_stream_kernel_offset_guards():
  """The persistent stream kernels form 32-bit byte offsets (lane row x row pitch, up to 255 rows past the last n-tile's
  first row); the shape predicate must refuse every shape in which such a sum could reach 2^32 and wrap around."""
  lib = _lib.load()
  takes = lib.moe_gmm_stream_kernel_takes
  I8, BF16, F8, E5M2, I4 = _lib.MOE_INT8, _lib.MOE_BF16, _lib.MOE_FP8_E4M3, _lib.MOE_FP8_E5M2, _lib.MOE_INT4
  assert takes(I8, I8, 4096, 28672, 0) == 1 and takes(BF16, BF16, 4096, 14336, 0) == 1 and takes(F8, F8, 4096, 14336, 0) == 1
  assert takes(E5M2, F8, 14336, 4096, 0) == 1 and takes(BF16, I4, 2880, 2880, 0) == 1
  # whole stages, three or more
  assert takes(I8, I8, 4096 + 64, 1024, 0) == 0 and takes(I8, I8, 256, 1024, 0) == 0 and takes(BF16, BF16, 128, 1024, 0) == 0
  # weights: (N + 256) * pitch must stay below 2^32
  k = 16384
  n_ok = (1 << 32) // k - 257
  assert takes(I8, I8, k, n_ok, 0) == 1 and takes(I8, I8, k, n_ok + 1, 0) == 0
  assert takes(BF16, BF16, k, n_ok // 2 - 128, 0) == 1 and takes(BF16, BF16, k, n_ok // 2 + 1, 0) == 0
  # indexed activations: (rows + 256) * pitch likewise
  rows_ok = (1 << 32) // 4096 - 257
  assert takes(I8, I8, 4096, 1024, rows_ok) == 1 and takes(I8, I8, 4096, 1024, rows_ok + 1) == 0
  assert takes(BF16, I4, 4096, 1024, (1 << 32) // 8192 - 257) == 1 and takes(BF16, I4, 4096, 1024, (1 << 32) // 8192 - 256) == 0
  assert takes(I8, BF16, 4096, 1024, 0) == 0
