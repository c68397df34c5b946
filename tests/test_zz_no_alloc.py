"""moe_gmm_static_ws: the entry point that allocates nothing (its m-tile list lives in an array the library holds on
the device) against moe_gmm on the same operands, through the C ABI.  Two calls in a row, the second with a smaller
input, each bit for bit equal to moe_gmm's result; a request beyond the array's capacity is refused."""

import ctypes

import numpy as np
import pytest
import torch

from maxtext_amd import _lib

pytestmark = pytest.mark.gpu


def _args(lhs, lhs_scale, rhs, rhs_scale, gs, out, ws):
  a = _lib.GmmArgs()
  a.struct_size = ctypes.sizeof(_lib.GmmArgs)
  a.lhs, a.lhs_scale, a.rhs, a.rhs_scale = lhs.data_ptr(), lhs_scale.data_ptr(), rhs.data_ptr(), rhs_scale.data_ptr()
  a.group_sizes, a.out = gs.data_ptr(), out.data_ptr()
  a.workspace, a.workspace_bytes = (ws.data_ptr(), ws.numel()) if ws is not None else (None, 0)
  a.M, a.K, a.N = lhs.shape[0], lhs.shape[1], rhs.shape[1]
  a.num_groups_total = a.num_groups_local = gs.numel()
  a.lhs_dtype = a.rhs_dtype = _lib.MOE_INT8
  a.rhs_scale_block_n = 1
  return a


def _operands(m, k, n, sizes, seed):
  g = torch.Generator().manual_seed(seed)
  lhs = torch.randint(-127, 128, (m, k), generator=g).to(torch.int8).cuda()
  ls = (torch.rand(m, generator=g) * 0.02 + 0.005).cuda()
  rhs = torch.randint(-127, 128, (len(sizes), n, k), generator=g).to(torch.int8).cuda()
  rs = (torch.rand(len(sizes), n, generator=g) * 0.01 + 0.002).cuda()
  return lhs, ls, rhs, rs, torch.tensor(sizes, dtype=torch.int32).cuda()


def test_static_workspace_entry_point_matches_moe_gmm_on_two_calls():
  lib = _lib.load()
  assert lib.moe_init() == 0, lib.moe_last_error()
  stream = _lib.current_stream()
  # first call: a prefill-sized problem (persistent 256 x 256 kernel); second: a smaller, ragged one (64-row tiles), so
  # that the second tile list is shorter than what the first call left in the array
  # then two decode-sized ones that the LDS-streamed persistent kernel takes (16-row tiles, 64-row tiles)
  for m, k, n, sizes, seed in ((2100, 512, 512, [700, 0, 800, 500], 1), (90, 256, 128, [30, 0, 45, 10], 2),
                               (70, 1024, 256, [5, 0, 9, 14, 3, 11, 2, 16], 3), (210, 512, 256, [40] * 5, 4)):
    lhs, ls, rhs, rs, gs = _operands(m, k, n, sizes, seed)
    ws = torch.empty((lib.moe_gmm_workspace_bytes(m, len(sizes)),), dtype=torch.uint8, device="cuda")
    want = torch.full((m, n), 7.0, dtype=torch.bfloat16, device="cuda")
    got = torch.full((m, n), -3.0, dtype=torch.bfloat16, device="cuda")
    a = _args(lhs, ls, rhs, rs, gs, want, ws)
    _lib.check(lib.moe_gmm(ctypes.byref(a), stream), "moe_gmm")
    b = _args(lhs, ls, rhs, rs, gs, got, None)  # no workspace pointer at all
    before = torch.cuda.memory_allocated()
    _lib.check(lib.moe_gmm_static_ws(ctypes.byref(b), stream), "moe_gmm_static_ws")
    torch.cuda.synchronize()
    assert torch.cuda.memory_allocated() == before
    assert torch.equal(got, want)
    assert torch.all(got[sum(sizes):] == 0) and float(got[: sum(sizes)].float().abs().max()) > 0


def test_static_workspace_with_the_same_groups_flag():
  """MOE_GMM_SAME_GROUPS on the library's own array: a flagged second product of the same tile height reuses the list, one
  of another height or of another problem in between rebuilds it; every result bit for bit moe_gmm's."""
  lib = _lib.load()
  stream = _lib.current_stream()
  m, k, n, sizes = 2100, 512, 512, [700, 0, 800, 500]
  lhs, ls, rhs, rs, gs = _operands(m, k, n, sizes, 3)
  ws = torch.empty((lib.moe_gmm_workspace_bytes(m, len(sizes)),), dtype=torch.uint8, device="cuda")

  def both(lhs_, ls_, rhs_, rs_, gs_, flagged):
    rows, nn = lhs_.shape[0], rhs_.shape[1]
    want = torch.full((rows, nn), 7.0, dtype=torch.bfloat16, device="cuda")
    got = torch.full((rows, nn), -3.0, dtype=torch.bfloat16, device="cuda")
    w2 = torch.empty((lib.moe_gmm_workspace_bytes(rows, gs_.numel()),), dtype=torch.uint8, device="cuda")
    _lib.check(lib.moe_gmm(ctypes.byref(_args(lhs_, ls_, rhs_, rs_, gs_, want, w2)), stream), "moe_gmm")
    b = _args(lhs_, ls_, rhs_, rs_, gs_, got, None)
    b.flags = _lib.MOE_GMM_SAME_GROUPS if flagged else 0
    _lib.check(lib.moe_gmm_static_ws(ctypes.byref(b), stream), "moe_gmm_static_ws")
    torch.cuda.synchronize()
    assert torch.equal(got, want)

  both(lhs, ls, rhs, rs, gs, False)          # maps 256-row tiles
  both(lhs, ls, rhs, rs, gs, True)           # same height: the list is used again
  # the same groups at 40 rows: a 64-row tile list; flagged, it must not read the 256-row list left above
  small = torch.tensor([12, 0, 20, 8], dtype=torch.int32).cuda()
  both(lhs[:40].contiguous(), ls[:40].contiguous(), rhs, rs, small, True)
  # back to the first problem, flagged: the record now names another problem, so the list is rebuilt
  both(lhs, ls, rhs, rs, gs, True)
  # another group_sizes buffer with other contents at the same sizes, flagged: rebuilt again
  other = torch.tensor([100, 900, 600, 500], dtype=torch.int32).cuda()
  both(lhs, ls, rhs, rs, other, True)


def test_static_workspace_entry_point_rejects_what_does_not_fit():
  lib = _lib.load()
  cap = lib.moe_gmm_static_ws_capacity()
  assert cap == 1 << 20
  a = _lib.GmmArgs()
  a.struct_size = ctypes.sizeof(_lib.GmmArgs)
  a.M, a.num_groups_total = 2_000_000, 8
  assert lib.moe_gmm_workspace_bytes(a.M, 8) > cap
  assert lib.moe_gmm_static_ws(ctypes.byref(a), None) == -3
  assert b"static workspace" in lib.moe_last_error()
