"""GPU parity of the expert-parallel dispatch bookkeeping (moe_local_expert_keys, moe_all_to_all_params and the
local_permute built on them) against the CPU oracle: integer results, compared bit-exactly; rows are copies."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O

pytestmark = pytest.mark.gpu


def gmm_bf16(*args, **kwargs):
  """megablox.gmm with the layer dtype as preferred_element_type, as the reference's layer calls it (moe.py:1549)."""
  from maxtext_amd import megablox

  kwargs.setdefault("preferred_element_type", torch.bfloat16)
  return megablox.gmm(*args, **kwargs)


@pytest.fixture(scope="module")
def M():
  from maxtext_amd import moe

  assert torch.cuda.is_available()
  return moe.RoutedMoE


def cuda_i32(a):
  return torch.from_numpy(np.ascontiguousarray(a, dtype=np.int32)).cuda()


def check_local_permute(M, g, l, shard, rows, d, seed, offset=False, factor=-1.0, ragged=False):
  rng = np.random.default_rng(seed)
  x = torch.from_numpy(rng.standard_normal((rows, d)).astype(np.float32)).to(torch.bfloat16)
  gse = None
  if offset:
    gse = np.repeat(np.arange(g.shape[1]), g.sum(0))[:rows]
    gse = np.concatenate([gse, np.full(rows - gse.shape[0], g.shape[1] - 1)]).astype(np.int32)
  want = O.local_permute(x, g, l, shard, is_offset=offset, global_sorted_experts=gse, ragged_buffer_factor=factor)
  got = M.local_permute(x.cuda(), cuda_i32(g), l, shard, is_offset=offset, global_sorted_experts=None if gse is None else cuda_i32(gse),
                        use_ragged_sort=ragged, ragged_buffer_factor=factor)
  np.testing.assert_array_equal(got[1].cpu().numpy(), want[1])
  np.testing.assert_array_equal(got[2].cpu().numpy(), want[2])
  np.testing.assert_array_equal(got[3].cpu().numpy(), want[3])
  valid = int(want[2].sum()) if ragged else rows
  assert torch.equal(got[0].cpu()[:valid].view(torch.int16), want[0][:valid].view(torch.int16))
  if ragged:
    assert not got[0].cpu()[valid:].any()


def test_local_permute_reference_cases(M):
  # the cases of tests/unit/moe_test.py:1174-1336
  sizes = np.arange(8, dtype=np.int32)[None, :]
  for shard, rows in enumerate([1, 6, 12, 18]):
    check_local_permute(M, sizes, 2, shard, rows, 8, seed=shard)
  for counts in (np.arange(8), np.array([0, 0, 1, 1, 2, 0, 2, 2])):
    for shard in range(4):
      check_local_permute(M, counts[None, :].astype(np.int32), 2, shard, int(counts.sum()), 8, seed=10 + shard, offset=True)


@pytest.mark.parametrize("seed", range(12))
def test_local_permute_random(M, seed):
  rng = np.random.default_rng(100 + seed)
  s = int(rng.choice([1, 2, 4, 8, 64]))
  l = int(rng.choice([1, 2, 8, 32]))
  shards = int(rng.choice([1, 2, 8]))
  shard = int(rng.integers(0, shards))
  hi = int(rng.choice([1, 4, 40, 300]))
  g = rng.integers(0, hi + 1, size=(s, l * shards)).astype(np.int32)
  if seed % 3 == 0:
    g[rng.random(g.shape) < 0.5] = 0  # empty segments share their start with the next one
  received = int(g[:, shard * l:(shard + 1) * l].sum())
  mode = seed % 4
  if mode == 0:      # exact buffer
    check_local_permute(M, g, l, shard, max(received, 1), 64, seed)
  elif mode == 1:    # worst-case buffer with an unused tail, only the valid prefix moved
    check_local_permute(M, g, l, shard, received + 1 + received // 3, 64, seed, ragged=True)
  elif mode == 2:    # capacity below what was routed here: sizes cut in (batch shard, expert) order
    check_local_permute(M, g, l, shard, max(received * 2 // 3, 1), 64, seed, factor=1.0)
  else:              # replicated batch sorted by global expert
    check_local_permute(M, g[:1], l, shard, max(int(g[:1].sum()), 1), 64, seed, offset=True)


def test_local_permute_deepseek_shard_at_size(M):
  # one of 8 expert shards of DeepSeek-V3 (32 local experts) receiving from 8 batch shards, 64k rows of d = 7168
  rng = np.random.default_rng(7)
  g = rng.multinomial(16384 * 8 // 8, np.ones(256) / 256, size=8).astype(np.int32)
  rows = int(g[:, 96:128].sum())
  check_local_permute(M, g, 32, 3, rows + 4096, 7168, seed=7, ragged=True)


@pytest.mark.parametrize("seed", range(10))
def test_all_to_all_params(M, seed):
  rng = np.random.default_rng(200 + seed)
  p = int(rng.choice([1, 2, 4, 8, 64, 256]))
  m = rng.integers(0, 1000, size=(p, p)).astype(np.int32)
  cap = int(m.sum(0).mean() * rng.choice([0.3, 0.8, 1.5]))
  for shard in {0, p // 2, p - 1}:
    for dispatch in (True, False):
      for factor in (-1.0, 1.0):
        want = O.get_all_to_all_params(m, shard, p, True, factor, cap, dispatch)
        got = M.get_all_to_all_params(cuda_i32(m), shard, p, True, factor, cap, dispatch)
        for gt, w in zip(got, want):
          np.testing.assert_array_equal(gt.cpu().numpy(), w)
    want = O.get_all_to_all_params(m[0], shard, p, False)
    got = M.get_all_to_all_params(cuda_i32(m[0]), shard, p, False)
    for gt, w in zip(got, want):
      np.testing.assert_array_equal(gt.cpu().numpy(), w)


def test_all_to_all_params_reference_cases(M):
  # tests/unit/moe_test.py:1338-1442
  a = np.array([[1, 2, 0, 3], [4, 0, 1, 2], [0, 3, 2, 1], [2, 1, 4, 0]], dtype=np.int32)
  in_off = [[0, 1, 3, 3], [0, 4, 4, 5], [0, 0, 3, 5], [0, 2, 3, 7]]
  out_off = [[0, 0, 0, 0], [1, 2, 0, 3], [5, 2, 1, 5], [5, 5, 3, 6]]
  recv = [[1, 4, 0, 2], [2, 0, 3, 1], [0, 1, 2, 4], [3, 2, 1, 0]]
  for s in range(4):
    got = M.get_all_to_all_params(cuda_i32(a), s, 4, is_batch_sharded=True)
    for g, w in zip(got, (in_off[s], a[s], out_off[s], recv[s])):
      np.testing.assert_array_equal(g.cpu().numpy(), w)
  g1 = np.array([6, 7, 6, 7], dtype=np.int32)
  for s in range(4):
    got = M.get_all_to_all_params(cuda_i32(g1), s, 4, is_batch_sharded=False)
    for g, w in zip(got, ([0, 0, 0, 0], [g1[s]] * 4, [[0, 6, 13, 19][s]] * 4, g1)):
      np.testing.assert_array_equal(g.cpu().numpy(), w)


def test_ragged_buffer_size(M):
  # tests/unit/moe_test.py:1444-1494
  assert M.get_ragged_buffer_size(32768, 4, 256, 8, 1.0) == 32768
  assert M.get_ragged_buffer_size(32768, 4, 256, 8, 2.0) == 65536
  assert M.get_ragged_buffer_size(32768, 4, 256, 8, -1.0) == 131072
  assert M.get_ragged_buffer_size(32768, 128, 256, 8, -1.0) == 1048576


def test_dispatch_argument_errors(M):
  from maxtext_amd import kernels

  g = cuda_i32(np.ones((2, 8)))
  with pytest.raises(RuntimeError):
    kernels.local_expert_keys(g, 4, 2, 16)  # shard 2 of 4 experts each lies outside 8 experts
  with pytest.raises(ValueError):
    M.local_permute(torch.zeros((4, 8), dtype=torch.bfloat16, device="cuda"), g, 4, 0, is_offset=True)
  with pytest.raises(RuntimeError):
    kernels.all_to_all_params(cuda_i32(np.ones(4)), 0, 4, is_batch_sharded=False, buffer_size=8)


def _shard_layer(moe, cfg, ws, x, logits):
  return moe.RoutedMoE(cfg, *ws).sparse_matmul(x, logits, None, *ws)[0]


def test_ragged_all_to_all_flow_on_one_gpu_matches_the_single_device_layer():
  # ra2a_and_route + unsort_output_and_ra2a (moe.py:1757-1856, :2022-2087) with 4 batch shards and 4 expert shards played
  # one after the other on this GPU; the collective is copied by hand from the offsets and sizes this library computes
  # (ragged_all_to_all: piece j of the sender's operand goes to peer j at the output offset the sender names).
  from maxtext_amd import kernels, megablox, moe
  from tolerances import relerr

  p, e, k, d, f, tb = 4, 16, 2, 128, 256, 96
  l = e // p
  cfg = moe.MoEConfig(e, k, d, f)
  g = torch.Generator(device="cuda").manual_seed(11)
  w0, w1 = [(torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16) for _ in range(2)]
  wo = (torch.randn((e, d, f), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  block = moe.RoutedMoE(cfg, w0, w1, wo)
  xs = [torch.randn((1, tb, d), generator=g, device="cuda").to(torch.bfloat16) for _ in range(p)]
  # skewed logits: expert shards receive different loads, some experts nothing
  lg = [torch.randn((1, tb, e), generator=g, device="cuda") - 0.4 * torch.arange(e, device="cuda") for _ in range(p)]

  routed = [block.permute(xs[b], lg[b]) for b in range(p)]  # (sorted x, perm, weights, group_size, ...)
  group_sizes = torch.stack([r[3] for r in routed]).contiguous()            # all_gather(group_sizes): [P, E]
  traffic = group_sizes.reshape(p, p, l).sum(-1).to(torch.int32).contiguous()  # all_shards_group_sizes [P, P]
  rows = tb * k
  buffer_size = moe.RoutedMoE.get_ragged_buffer_size(rows, p, e, k, -1.0)
  assert buffer_size == rows * p

  # dispatch
  buffers = [torch.full((buffer_size, d), float("nan"), dtype=torch.bfloat16, device="cuda") for _ in range(p)]
  for s in range(p):
    in_off, send, out_off, recv = [v.cpu().numpy() for v in moe.RoutedMoE.get_all_to_all_params(traffic, s, p)]
    np.testing.assert_array_equal(recv, traffic[:, s].cpu().numpy())
    for j in range(p):
      buffers[j][out_off[j]:out_off[j] + send[j]] = routed[s][0][in_off[j]:in_off[j] + send[j]]

  # every expert shard: local permute, its own experts' three matmuls, local unsort
  returned = []
  for j in range(p):
    xj, local_idx, local_sizes, ids = moe.RoutedMoE.local_permute(buffers[j], group_sizes, l, j, use_ragged_sort=True)
    n = int(local_sizes.sum())
    assert n == int(traffic[:, j].sum()) and not torch.isnan(xj[:n].float()).any()
    np.testing.assert_array_equal(ids[:n].cpu().numpy(), np.repeat(np.arange(l), local_sizes.cpu().numpy()))
    sl = slice(j * l, (j + 1) * l)
    h = gmm_bf16(xj, w0[sl].contiguous(), local_sizes, transpose_rhs=True, rhs_up=w1[sl].contiguous(), fuse_act="silu")
    y = gmm_bf16(h, wo[sl].contiguous(), local_sizes, transpose_rhs=True)
    returned.append(kernels.unpermute_combine(y.contiguous(), None, k=1, perm=local_idx))  # rows back in arrival order

  # the way back, then each batch shard's unpermute with its routing weights
  for b in range(p):
    got_rows = torch.zeros((rows, d), dtype=torch.bfloat16, device="cuda")
    for j in range(p):
      in_off, send, out_off, recv = [v.cpu().numpy() for v in moe.RoutedMoE.get_all_to_all_params(traffic, j, p, is_dispatch=False)]
      got_rows[out_off[b]:out_off[b] + send[b]] = returned[j][in_off[b]:in_off[b] + send[b]]
    out = block.unpermute(got_rows, routed[b][1], routed[b][2], 1, tb)
    want = _shard_layer(moe, cfg, (w0, w1, wo), xs[b], lg[b])
    assert relerr(out.float().cpu(), want.float().cpu()) <= 1e-2


def test_ring_of_experts_flow_on_one_gpu_matches_the_single_device_layer():
  # roe_ag_and_route (moe.py:1709-1755): every expert shard sees all tokens, sorts them with its own experts first
  # (roll_to_expert_id), multiplies only its experts' rows (group_offset 0, the local experts' weights) and the shards'
  # partial outputs add up (the reduce-scatter of moe.py:2266) to the single-device layer
  from maxtext_amd import megablox, moe
  from tolerances import relerr

  p, e, k, d, f, t = 4, 16, 2, 128, 256, 200
  l = e // p
  cfg = moe.MoEConfig(e, k, d, f)
  g = torch.Generator(device="cuda").manual_seed(12)
  w0, w1 = [(torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16) for _ in range(2)]
  wo = (torch.randn((e, d, f), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  block = moe.RoutedMoE(cfg, w0, w1, wo)
  x = torch.randn((1, t, d), generator=g, device="cuda").to(torch.bfloat16)
  logits = torch.randn((1, t, e), generator=g, device="cuda")
  total = torch.zeros((t, d), dtype=torch.float32, device="cuda")
  for j in range(p):
    sx, perm, weights, group_size, sorted_experts, _, _, _ = block.permute(x, logits, roll_to_expert_id=j * l)
    sl = slice(j * l, (j + 1) * l)
    # rolled ids: this shard's experts are groups 0 .. l-1 of the rolled order; rows of the other groups come back as zeros
    h = gmm_bf16(sx, w0[sl].contiguous(), group_size, transpose_rhs=True, rhs_up=w1[sl].contiguous(), fuse_act="silu", group_offset=0)
    y = gmm_bf16(h, wo[sl].contiguous(), group_size, transpose_rhs=True, group_offset=0)
    n = int(group_size[:l].sum())
    assert not y[n:].any()
    total += block.unpermute(y, perm, weights, 1, t).reshape(t, d).float()
  want = _shard_layer(moe, cfg, (w0, w1, wo), x, logits)
  assert relerr(total.cpu(), want.reshape(t, d).float().cpu()) <= 1e-2


@pytest.mark.parametrize("seed", range(8))
def test_ring_ragged_sort_unsort(seed):
  # kernels/ragged/ragged_sort.py:23-451 (forward passes) against the oracle: indices bit-exact, rows are copies, the
  # weighted sum within the output tolerance
  from maxtext_amd import ragged_sort
  from tolerances import relerr

  rng = np.random.default_rng(300 + seed)
  ep = int(rng.choice([1, 2, 4, 8]))
  e = ep * int(rng.choice([1, 2, 4, 16]))
  k = int(rng.integers(1, min(e, 8) + 1))
  t = int(rng.choice([1, 5, 64, 700]))
  d = int(rng.choice([8, 64, 512]))
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(torch.bfloat16)
  w = torch.from_numpy(rng.random((t, k)).astype(np.float32))
  n = t * k
  for shard in sorted({0, ep - 1, ep // 2}):
    for buf in (None, n + 3, max(n // (2 * ep), 1)):
      want_x, want_gs, want_rev = O.ring_ragged_sort(x, sel, e, k, shard, ep, buffer_size=buf)
      got_x, got_gs, got_rev = ragged_sort.ring_ragged_sort(x.cuda(), cuda_i32(sel), e, k, shard, ep, buffer_size=buf)
      np.testing.assert_array_equal(got_gs.cpu().numpy(), want_gs)
      np.testing.assert_array_equal(got_rev.cpu().numpy(), want_rev)
      # the reference returns T*k rows when the buffer is larger; this library returns min(buffer, T*k) rows likewise
      assert got_x.shape == want_x.shape
      assert torch.equal(got_x.cpu().view(torch.int16), want_x.view(torch.int16))
      y = torch.from_numpy(rng.standard_normal(tuple(want_x.shape)).astype(np.float32)).to(torch.bfloat16)
      want_o = O.ring_ragged_unsort(y, want_gs, want_rev, k, e // ep, shard, w)
      got_o = ragged_sort.ring_ragged_unsort(y.cuda(), got_gs, got_rev, k, e // ep, shard, w.cuda())
      assert got_o.shape == want_o.shape
      if want_o.abs().max() > 0:
        assert relerr(got_o.float().cpu(), want_o.float()) <= 1e-2
      else:
        assert not got_o.any()


def test_a2a_ragged_sort_unsort():
  from maxtext_amd import ragged_sort

  rng = np.random.default_rng(9)
  n, d = 1000, 256
  x = torch.from_numpy(rng.standard_normal((n, d)).astype(np.float32)).to(torch.bfloat16)
  idx = rng.permutation(n).astype(np.int32)
  for valid in (0, 1, 617, n):
    want = O.a2a_ragged_sort(x, idx, valid)
    assert torch.equal(ragged_sort.a2a_ragged_sort(x.cuda(), cuda_i32(idx), valid).cpu(), want)
    assert torch.equal(ragged_sort.a2a_ragged_unsort(x.cuda(), cuda_i32(idx), torch.tensor(valid, device="cuda")).cpu(), want)
  # unsort(sort(x)) restores the valid prefix when the permutation keeps it in place
  keep = np.concatenate([rng.permutation(600), np.arange(600, n)]).astype(np.int32)
  s = ragged_sort.a2a_ragged_sort(x.cuda(), cuda_i32(keep), 600)
  back = ragged_sort.a2a_ragged_unsort(s, cuda_i32(np.argsort(keep).astype(np.int32)), 600)
  assert torch.equal(back[:600].cpu(), x[:600]) and not back[600:].any()


@pytest.mark.parametrize("seed", range(6))
def test_ring_ragged_sort_unsort_gradients(seed):
  """The custom VJPs of ring_ragged_sort / ring_ragged_unsort (kernels/ragged/ragged_sort.py:155-224, :364-441) against
  torch autograd through a plain restatement of the forward passes (index_select + mask), full and packed buffers."""
  from maxtext_amd import ragged_sort
  from tolerances import relerr

  rng = np.random.default_rng(500 + seed)
  ep = int(rng.choice([1, 2, 4]))
  e = ep * int(rng.choice([2, 4, 16]))
  k = int(rng.integers(1, min(e, 6) + 1))
  t = int(rng.choice([5, 64, 300]))
  d = int(rng.choice([8, 64, 256]))
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  n = t * k
  flat = sel.reshape(-1)
  perm = np.argsort(flat, kind="stable")
  gs = np.bincount(flat, minlength=e)
  local = e // ep
  x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(torch.bfloat16)
  w = torch.from_numpy(rng.random((t, k)).astype(np.float32))
  for shard in sorted({0, ep - 1}):
    start = int(gs[: shard * local].sum())
    end = start + int(gs[shard * local:(shard + 1) * local].sum())
    for buf in (None, max(n // (2 * ep), 1)):
      rows = n if buf is None or buf >= n else buf
      # positions of the buffer that hold a row, and the flat slot each of them copies
      if rows == n:
        pos = np.arange(start, end)
        slots = perm[start:end]
      else:
        cnt = min(end - start, rows)
        pos = np.arange(cnt)
        slots = perm[start:start + cnt]
      pos_t, tok_t = torch.from_numpy(pos).long(), torch.from_numpy(slots // k).long()
      # sort: x_sorted[pos] = hidden[token of the slot]
      g_x = torch.from_numpy(rng.standard_normal((rows, d)).astype(np.float32)).to(torch.bfloat16)
      h = x.double().requires_grad_()
      ref = torch.zeros((rows, d), dtype=torch.float64).index_put((pos_t,), h[tok_t])
      (ref * g_x.double()).sum().backward()
      hg = x.cuda().requires_grad_()
      got_x, got_gs, got_rev = ragged_sort.ring_ragged_sort(hg, cuda_i32(sel), e, k, shard, ep, buffer_size=buf)
      assert torch.equal(got_x.detach().cpu().float(), ref.detach().float())
      got_x.backward(g_x.cuda())
      if h.grad.abs().max() > 0:
        assert relerr(hg.grad, h.grad) <= 1e-2
      else:
        assert not hg.grad.any()
      # unsort: out[token] = sum over its slots in the buffer of w[slot] * y[pos]
      y = torch.from_numpy(rng.standard_normal((rows, d)).astype(np.float32)).to(torch.bfloat16)
      g_o = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(torch.bfloat16)
      yd = y.double().requires_grad_()
      contrib = yd[pos_t] * w.reshape(-1).double()[torch.from_numpy(slots).long()][:, None]
      ref_o = torch.zeros((t, d), dtype=torch.float64).index_add(0, tok_t, contrib)
      (ref_o * g_o.double()).sum().backward()
      yg = y.cuda().requires_grad_()
      got_o = ragged_sort.ring_ragged_unsort(yg, got_gs, got_rev, k, local, shard, w.cuda())
      if ref_o.abs().max() > 0:
        assert relerr(got_o, ref_o) <= 1e-2
      got_o.backward(g_o.cuda())
      if yd.grad.abs().max() > 0:
        assert relerr(yg.grad, yd.grad) <= 1e-2
      else:
        assert not yg.grad.any()


def test_a2a_ragged_sort_unsort_gradients():
  """The custom VJPs of a2a_ragged_sort / a2a_ragged_unsort (ragged_sort.py:515-537, :596-616) and of
  local_permute(use_ragged_sort=True) against torch autograd through out = where(i < end, x[idx[i]], 0)."""
  from maxtext_amd import moe, ragged_sort

  rng = np.random.default_rng(11)
  n, d = 700, 128
  x = torch.from_numpy(rng.standard_normal((n, d)).astype(np.float32)).to(torch.bfloat16)
  g = torch.from_numpy(rng.standard_normal((n, d)).astype(np.float32)).to(torch.bfloat16)
  for valid in (0, 1, 400, n):
    # a permutation that keeps the valid prefix in place as a set (the case the reference's unsort rule is exact for)
    idx = np.concatenate([rng.permutation(valid), valid + rng.permutation(n - valid)]).astype(np.int32)
    mask = (torch.arange(n) < valid)[:, None]
    xd = x.double().requires_grad_()
    (torch.where(mask, xd[torch.from_numpy(idx).long()], torch.zeros((), dtype=torch.float64)) * g.double()).sum().backward()
    for fn in (ragged_sort.a2a_ragged_sort, ragged_sort.a2a_ragged_unsort):
      xg = x.cuda().requires_grad_()
      out = fn(xg, cuda_i32(idx), valid)
      out.backward(g.cuda())
      assert torch.equal(xg.grad.cpu().double(), xd.grad)  # a permutation of rows: exact
  # a2a_ragged_sort alone is exact for any permutation
  idx = rng.permutation(n).astype(np.int32)
  xd = x.double().requires_grad_()
  (torch.where((torch.arange(n) < 250)[:, None], xd[torch.from_numpy(idx).long()], torch.zeros((), dtype=torch.float64)) * g.double()).sum().backward()
  xg = x.cuda().requires_grad_()
  ragged_sort.a2a_ragged_sort(xg, cuda_i32(idx), 250).backward(g.cuda())
  assert torch.equal(xg.grad.cpu().double(), xd.grad)
  # local_permute with the ragged sort, under grad: rows past the received total get no gradient
  sizes = np.array([[3, 0, 5, 2], [1, 4, 0, 6]], np.int32)  # 2 batch shards x 4 experts; this shard owns experts 2, 3
  rows = 20
  buf = torch.from_numpy(rng.standard_normal((rows, d)).astype(np.float32)).to(torch.bfloat16)
  bg = buf.cuda().requires_grad_()
  sorted_inputs, sorted_indices, local_sizes, _ = moe.RoutedMoE.local_permute(bg, cuda_i32(sizes), 2, 1, use_ragged_sort=True)
  total = int(local_sizes.sum())
  assert total == 5 + 2 + 0 + 6
  gg = torch.ones_like(sorted_inputs)
  sorted_inputs.backward(gg)
  got = bg.grad.cpu().float()
  want = torch.zeros(rows, d)
  want[sorted_indices.cpu().long()[:total]] = 1.0
  assert torch.equal(got, want)
