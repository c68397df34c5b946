"""Shard-dependent scalars held on the device (the reference derives group_offset and roll_to_expert_id from
jax.lax.axis_index, moe.py:2014-2019, backend.py:340-345: device values a custom call receives as buffers), and the
dynamic per-tensor scales of disable_channelwise_axes (kernels/megablox/ops.py:245, :258)."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tolerances import relerr

pytestmark = pytest.mark.gpu

TOL = 1e-2


@pytest.fixture(scope="module")
def K():
  from maxtext_amd import kernels

  assert torch.cuda.is_available()
  return kernels


def cuda(x):
  if isinstance(x, np.ndarray):
    x = torch.from_numpy(x)
  return x.cuda().contiguous()


@pytest.mark.parametrize("m,k,n,sizes", [(900, 384, 200, [130, 300, 0, 270, 150]), (4200, 512, 2048, [1500, 0, 700, 1900, 50])])
@pytest.mark.parametrize("offset,g_local", [(0, 2), (1, 3), (3, 2)])
def test_group_offset_from_a_device_buffer(K, m, k, n, sizes, offset, g_local):
  """moe_gmm with the first local group in a device buffer: bit-equal to the same call with the offset by value
  (zero-filled rows of the other groups included), with and without kept rows, and with a value field that disagrees
  (the device value wins)."""
  g = torch.Generator().manual_seed(m + offset)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(len(sizes), n, k, generator=g) * 0.05).to(torch.bfloat16)
  gs = cuda(np.asarray(sizes, np.int32))
  off_dev = torch.tensor([offset], dtype=torch.int32, device="cuda")
  wl = cuda(w[offset:offset + g_local])
  by_value = K.gmm_raw(cuda(lhs), wl, gs, group_offset=offset)
  by_dev = K.gmm_raw(cuda(lhs), wl, gs, group_offset=0 if offset else 2, group_offset_dev=off_dev)
  assert torch.equal(by_value, by_dev)
  want = O.gmm(lhs, w[offset:offset + g_local], sizes, transpose_rhs=True, group_offset=offset)
  assert relerr(by_dev, want) <= TOL
  buf_a = torch.full((m, n), 3.0, dtype=torch.bfloat16, device="cuda")
  buf_b = buf_a.clone()
  K.gmm_raw(cuda(lhs), wl, gs, group_offset=offset, out=buf_a, keep_other_rows=True)
  K.gmm_raw(cuda(lhs), wl, gs, group_offset_dev=off_dev, out=buf_b, keep_other_rows=True)
  assert torch.equal(buf_a, buf_b)


def test_megablox_gmm_takes_a_device_group_offset_without_reading_it():
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(4)
  m, k, n, sizes = 700, 256, 256, [100, 200, 0, 300, 100]
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(5, k, n, generator=g) * 0.05).to(torch.bfloat16)
  gs = cuda(np.asarray(sizes, np.int32))
  off = torch.tensor(1, dtype=torch.int32, device="cuda")  # ()-shaped, as the reference's (backend.py:340-345)
  got = megablox.gmm(cuda(lhs), cuda(w[1:4]), gs, torch.bfloat16, group_offset=off)
  assert torch.equal(got, megablox.gmm(cuda(lhs), cuda(w[1:4]), gs, torch.bfloat16, group_offset=1))
  with pytest.raises(ValueError):
    megablox.gmm(cuda(lhs), cuda(w[1:4]), gs, torch.bfloat16, group_offset=torch.tensor([1], device="cuda"))


@pytest.mark.parametrize("t,e,k,roll", [(300, 8, 2, 3), (5000, 64, 4, 48), (17, 16, 4, -5)])
def test_rolled_sort_with_the_roll_on_the_device(K, t, e, k, roll):
  rng = np.random.default_rng(t)
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  want = K.sort_by_expert(cuda(sel), e, roll_to_expert_id=roll % e)
  got = K.sort_by_expert(cuda(sel), e, roll_to_expert_id=torch.tensor([roll], dtype=torch.int32, device="cuda"))
  for a, b in zip(got, want):
    assert torch.equal(a, b)
  keys = (sel.reshape(-1) - roll) % e
  np.testing.assert_array_equal(got[0].cpu().numpy(), np.argsort(keys, kind="stable"))


@pytest.mark.parametrize("qname", ["int8", "fp8"])
def test_dynamic_per_tensor_scales(K, qname):
  """disable_channelwise_axes: one absmax scale for the activations and one for the weights (channelwise_axes=[]),
  against the host statement of the same rule, bit for bit, and through gmm against the dequantised product."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  qdt = torch.int8 if qname == "int8" else torch.float8_e4m3fn
  qmax = 127.0 if qname == "int8" else 448.0
  g = torch.Generator().manual_seed(19)
  m, k, n, sizes = 260, 256, 136, [100, 0, 160]
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(3, k, n, generator=g) * 0.05).to(torch.bfloat16)  # [g, k, n]
  ls = lhs.float().abs().max() / qmax
  rs = w.float().abs().max() / qmax
  cast = (lambda y: torch.round(y).clamp(-qmax, qmax).to(qdt)) if qname == "int8" else (lambda y: y.clamp(-qmax, qmax).to(qdt))
  want_l, want_r = cast(lhs.float() / ls), cast(w.float() / rs)
  dl = megablox.quantize_lhs(cuda(lhs), qname, per_tensor=True)
  dr = megablox.quantize_rhs(cuda(w.transpose(1, 2).contiguous()), qname, per_tensor=True)
  assert float(dl.scale) == float(ls) and float(dr.scale) == float(rs)
  assert torch.equal(dl.qvalue.cpu().float(), want_l.float()) and torch.equal(dr.qvalue.cpu().float().transpose(1, 2), want_r.float())
  rule = QtRule(weight_qtype=qname, act_qtype=qname, disable_channelwise_axes=True)
  out = megablox.gmm(cuda(lhs), cuda(w), cuda(np.asarray(sizes, np.int32)), torch.bfloat16, use_qwix_quantization=True, qwix_rule=rule)
  want = O.gmm(want_l.float(), want_r.float(), sizes, lhs_scale=ls.reshape(1, 1), rhs_scale=rs.reshape(1, 1).expand(1, n))
  assert relerr(out, want) <= TOL
  assert float(K.tensor_scale(torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda"), qmax)) == 0.0


def test_dispatch_bookkeeping_with_the_shard_index_on_the_device(K):
  """moe_local_expert_keys / moe_all_to_all_params / moe_ring_ragged_indices with the shard's index in a device buffer
  (jax.lax.axis_index of moe.py:1134, :1709-1712): bit-equal to the by-value calls for every shard, and a value past the
  last shard is clamped to it."""
  rng = np.random.default_rng(5)
  shards, experts, local = 4, 16, 4
  ggs = rng.integers(0, 40, size=(shards, experts)).astype(np.int32)
  rows = int(ggs.sum()) + 7
  sorted_experts = np.sort(rng.integers(0, experts, size=rows)).astype(np.int32)
  traffic = rng.integers(0, 50, size=(shards, shards)).astype(np.int32)
  topk_idx = rng.integers(0, experts, size=(96, 2)).astype(np.int32)
  perm, inv, gs, _ = K.sort_by_expert(cuda(topk_idx), experts, want_sorted_experts=False)
  for shard in range(shards + 1):
    ref = min(shard, shards - 1)
    dev = torch.tensor([shard], dtype=torch.int32, device="cuda")
    for offset_mode in (False, True):
      kw = dict(global_sorted_experts=cuda(sorted_experts) if offset_mode else None, truncate=not offset_mode)
      a = K.local_expert_keys(cuda(ggs), local, ref, rows, **kw)
      b = K.local_expert_keys(cuda(ggs), local, dev, rows, **kw)
      assert all(torch.equal(x, y) for x, y in zip(a, b))
    for dispatch in (True, False):
      a = K.all_to_all_params(cuda(traffic), ref, shards, buffer_size=60, is_dispatch=dispatch)
      b = K.all_to_all_params(cuda(traffic), dev, shards, buffer_size=60, is_dispatch=dispatch)
      assert all(torch.equal(x, y) for x, y in zip(a, b))
    a = K.all_to_all_params(cuda(traffic[0]), ref, shards, is_batch_sharded=False)
    b = K.all_to_all_params(cuda(traffic[0]), dev, shards, is_batch_sharded=False)
    assert all(torch.equal(x, y) for x, y in zip(a, b))
    for unsort, idx, buf in ((False, perm, None), (False, perm, 40), (True, inv, None), (True, inv, 40)):
      a = K.ring_ragged_indices(idx, gs, ref * local, local, buffer_size=buf, unsort=unsort)
      b = K.ring_ragged_indices(idx, gs, 0, local, buffer_size=buf, unsort=unsort, shard_index=dev)
      assert all(torch.equal(x, y) for x, y in zip(a, b))


def test_ring_ragged_sort_with_a_device_shard_index():
  """ring_ragged_sort / _unsort with the shard index as a tensor: same rows, sizes and gradient as with the integer."""
  from maxtext_amd import ragged_sort

  g = torch.Generator().manual_seed(11)
  t, d, e, k, ep = 64, 128, 8, 2, 4
  x = torch.randn(t, d, generator=g).to(torch.bfloat16).cuda()
  idx = torch.randint(0, e, (t, k), generator=g, dtype=torch.int32).cuda()
  w = torch.rand(t, k, generator=g).cuda()
  for shard in range(ep):
    outs = []
    for s in (shard, torch.tensor(shard, device="cuda")):
      xi = x.clone().requires_grad_(True)
      rows, gs, inv = ragged_sort.ring_ragged_sort(xi, idx, e, k, s, ep)
      y = ragged_sort.ring_ragged_unsort(rows * 2, gs, inv, k, e // ep, s, w)
      y.float().square().sum().backward()
      outs.append((rows.detach(), gs, inv, y.detach(), xi.grad))
    assert all(torch.equal(a, b) for a, b in zip(*outs))
