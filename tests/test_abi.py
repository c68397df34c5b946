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
  assert lib.moe_abi_version() == 2
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
