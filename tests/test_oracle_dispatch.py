"""Pins the oracle's expert-parallel dispatch bookkeeping (integer work) against the expected arrays the reference's
own tests hold and against brute-force formulations."""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


def test_local_permute_no_offset_known_answer():
  # tests/unit/moe_test.py:1174-1261: 8 experts on 4 shards, expert e holds e rows; every shard's rows arrive in
  # expert order, so the permutation is the identity and the keys repeat each local expert by its count.  The slices
  # that test cuts (start = cumsum[:-2:2], end = cumsum[1::2]) are longer than the shard's rows for shards 1 to 3, and
  # its expected keys come from jnp.repeat(..., total_repeat_length=rows): the surplus rows carry the last expert's key
  sizes = np.arange(8, dtype=np.int32)
  total = int(sizes.sum())
  x = torch.arange(total * 5, dtype=torch.int32).reshape(total, 5)
  c = np.cumsum(sizes)
  starts = np.concatenate([[0], c[:-2:2]])
  ends = c[1::2]
  for shard in range(4):
    xs = x[starts[shard]:ends[shard]]
    si, idx, lgs, ids = O.local_permute(xs, sizes[None, :], 2, shard, is_offset=False)
    want_sizes = sizes[2 * shard:2 * shard + 2]
    assert torch.equal(si, xs)
    np.testing.assert_array_equal(idx, np.arange(ends[shard] - starts[shard]))
    np.testing.assert_array_equal(lgs, want_sizes)
    rows = int(ends[shard] - starts[shard])
    assert rows == [1, 6, 12, 18][shard]
    np.testing.assert_array_equal(ids, np.concatenate([np.repeat(np.arange(2), want_sizes), np.full(rows - int(want_sizes.sum()), 1)]))


@pytest.mark.parametrize("counts", [list(range(8)), [0, 0, 1, 1, 2, 0, 2, 2]])
def test_local_permute_offset_known_answer(counts):
  # tests/unit/moe_test.py:1263-1336: all routed rows sorted by global expert; a shard's rows come first, in order
  counts = np.array(counts, dtype=np.int32)
  n = int(counts.sum())
  x = torch.arange(1, n + 1, dtype=torch.int32).reshape(-1, 1).repeat(1, 5)
  per_shard = counts.reshape(4, 2).sum(-1)
  assign = np.repeat(np.arange(8), counts)
  offs = np.concatenate([[0], np.cumsum(per_shard)[:-1]])
  for shard in range(4):
    px, idx, lgs, ids = O.local_permute(x, counts[None, :], 2, shard, is_offset=True, global_sorted_experts=assign)
    m = per_shard[shard]
    assert torch.equal(px[:m], x[offs[shard]:offs[shard] + m])
    np.testing.assert_array_equal(idx[:m], np.arange(offs[shard], offs[shard] + m))
    np.testing.assert_array_equal(lgs, counts[2 * shard:2 * shard + 2])
    np.testing.assert_array_equal(ids[:m], assign[offs[shard]:offs[shard] + m] % 2)
    assert (ids[m:] == 2).all()  # rows of other shards carry the key local_expert_size (moe.py:1169-1172)


def test_all_to_all_params_sharded_known_answer():
  # tests/unit/moe_test.py:1338-1390
  a = np.array([[1, 2, 0, 3], [4, 0, 1, 2], [0, 3, 2, 1], [2, 1, 4, 0]], dtype=np.int32)
  in_off = [[0, 1, 3, 3], [0, 4, 4, 5], [0, 0, 3, 5], [0, 2, 3, 7]]
  out_off = [[0, 0, 0, 0], [1, 2, 0, 3], [5, 2, 1, 5], [5, 5, 3, 6]]
  recv = [[1, 4, 0, 2], [2, 0, 3, 1], [0, 1, 2, 4], [3, 2, 1, 0]]
  for s in range(4):
    got = O.get_all_to_all_params(a, s, 4, is_batch_sharded=True)
    for g, w in zip(got, (in_off[s], a[s], out_off[s], recv[s])):
      np.testing.assert_array_equal(g, w)


def test_all_to_all_params_unsharded_known_answer():
  # tests/unit/moe_test.py:1392-1442
  g = np.array([6, 7, 6, 7], dtype=np.int32)
  for s in range(4):
    got = O.get_all_to_all_params(g, s, 4, is_batch_sharded=False)
    for x, w in zip(got, ([0, 0, 0, 0], [g[s]] * 4, [[0, 6, 13, 19][s]] * 4, g)):
      np.testing.assert_array_equal(x, w)


def test_ragged_buffer_size_known_answers():
  # tests/unit/moe_test.py:1444-1494
  assert O.get_ragged_buffer_size(32768, 4, 256, 8, 1.0) == 32768
  assert O.get_ragged_buffer_size(32768, 4, 256, 8, 2.0) == 65536
  assert O.get_ragged_buffer_size(32768, 4, 256, 8, -1.0) == 131072
  assert O.get_ragged_buffer_size(32768, 128, 256, 8, -1.0) == 1048576


def test_truncate_matrix_by_hand_and_invariants():
  # column 0 receives 3 + 4 + 5: with room for 6 the first sender keeps 3, the second 3 of 4, the third nothing
  a = np.array([[3, 1], [4, 0], [5, 2]], dtype=np.int32)
  np.testing.assert_array_equal(O.truncate_matrix(a, 6), [[3, 1], [3, 0], [0, 2]])
  np.testing.assert_array_equal(O.truncate_matrix(a, 100), a)
  np.testing.assert_array_equal(O.truncate_matrix(a, 0), np.zeros_like(a))
  rng = np.random.default_rng(0)
  for _ in range(50):
    p = int(rng.integers(1, 9))
    m = rng.integers(0, 20, size=(p, p)).astype(np.int32)
    cap = int(rng.integers(0, 60))
    t = O.truncate_matrix(m, cap)
    assert (t >= 0).all() and (t <= m).all()
    np.testing.assert_array_equal(t.sum(0), np.minimum(m.sum(0), cap))
    # senders are served in order: a sender is cut only once every earlier one got its full share or the room is gone
    for j in range(p):
      room = cap
      for i in range(p):
        assert t[i, j] == min(m[i, j], room)
        room -= t[i, j]


def test_truncated_local_group_size_by_hand():
  # two batch shards x two local experts, flattened order (s0 e0, s0 e1, s1 e0, s1 e1) = 3, 2, 4, 1, room for 6:
  # kept 3, 2, 1, 0 -> per expert 3 + 1 and 2 + 0
  a = np.array([[3, 2], [4, 1]], dtype=np.int32)
  np.testing.assert_array_equal(O.maybe_truncate_local_group_size(a, 6, 1.0), [4, 2])
  np.testing.assert_array_equal(O.maybe_truncate_local_group_size(a, 6, -1.0), [7, 3])
  np.testing.assert_array_equal(O.maybe_truncate_local_group_size(a, 100, 1.0), [7, 3])


def test_all_to_all_params_truncated_are_consistent():
  # what shard i sends to shard j on dispatch is what j receives from i, receive offsets stack the received pieces
  # without gaps inside the capacity, and the way back returns every piece to the offset it was sent from
  rng = np.random.default_rng(1)
  for _ in range(30):
    p = int(rng.integers(2, 7))
    m = rng.integers(0, 12, size=(p, p)).astype(np.int32)
    cap = int(rng.integers(1, 40))
    d = [O.get_all_to_all_params(m, s, p, True, 1.0, cap, True) for s in range(p)]
    c = [O.get_all_to_all_params(m, s, p, True, 1.0, cap, False) for s in range(p)]
    t = O.truncate_matrix(m, cap)
    for i in range(p):
      for j in range(p):
        assert d[i][1][j] == d[j][3][i] == t[i, j]            # send i->j == recv at j from i
        assert d[i][2][j] == t[:i, j].sum()                     # lands behind the earlier senders' pieces
        assert d[i][2][j] + d[i][1][j] <= cap
        assert d[i][0][j] == m[i, :j].sum()                     # read from the sender's uncut layout
        assert c[j][1][i] == t[i, j] == c[i][3][j]              # the way back carries the same piece
        assert c[j][0][i] == d[i][2][j]                         # read where dispatch put it
        assert c[j][2][i] == d[i][0][j]                         # written where dispatch read it


def test_local_keys_brute_force_and_padding():
  rng = np.random.default_rng(2)
  for _ in range(40):
    s, l, shards = int(rng.integers(1, 5)), int(rng.integers(1, 6)), int(rng.integers(1, 4))
    shard = int(rng.integers(0, shards))
    g = rng.integers(0, 5, size=(s, l * shards)).astype(np.int32)
    local = g[:, shard * l:(shard + 1) * l]
    received = int(local.sum())
    rows = received + int(rng.integers(0, 4))
    x = torch.arange(rows, dtype=torch.int32).reshape(rows, 1)
    _, idx, lgs, ids = O.local_permute(x, g, l, shard)
    keys = []  # row by row: batch shards in order, each with its local experts in order
    for bs in range(s):
      for e in range(l):
        keys += [e] * int(local[bs, e])
    keys += [l - 1] * (rows - received)  # jnp.repeat pads with the last value
    keys = np.array(keys[:rows], dtype=np.int64)
    want = sorted(range(rows), key=lambda r: (keys[r], r))
    np.testing.assert_array_equal(idx, want)
    np.testing.assert_array_equal(ids, keys[want])
    np.testing.assert_array_equal(lgs, local.sum(0))


@pytest.mark.parametrize("buffered", [False, True])
def test_ring_ragged_sort_unsort_row_by_row(buffered):
  # kernels/ragged/ragged_sort.py:23-451 (forward): every sorted position that belongs to the shard's experts holds its
  # token's row (at the same position, or packed from 0 in a small buffer, where rows beyond the buffer are dropped)
  rng = np.random.default_rng(3)
  t, k, e, ep, d = 23, 3, 8, 4, 4
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  x = torch.arange(t * d, dtype=torch.float32).reshape(t, d).to(torch.bfloat16) + 1
  w = torch.from_numpy(rng.random((t, k)).astype(np.float32))
  flat = sel.reshape(-1)
  order = sorted(range(t * k), key=lambda i: (flat[i], i))
  total = torch.zeros(t, d)
  for shard in range(ep):
    buf = 7 if buffered else None
    xs, gs, revert = O.ring_ragged_sort(x, sel, e, k, shard, ep, buffer_size=buf)
    np.testing.assert_array_equal(gs, np.bincount(flat, minlength=e))
    np.testing.assert_array_equal(revert, np.argsort(np.array(order), kind="stable"))
    mine = [p for p, i in enumerate(order) if flat[i] // (e // ep) == shard]
    want = torch.zeros((buf if buffered else t * k, d), dtype=torch.bfloat16)
    for slot, p in enumerate(mine):
      if buffered and slot < buf:
        want[slot] = x[order[p] // k]
      elif not buffered:
        want[p] = x[order[p] // k]
    assert torch.equal(xs, want)
    out = O.ring_ragged_unsort(xs, gs, revert, k, e // ep, shard, w)
    kept = mine[:buf] if buffered else mine
    want_out = torch.zeros(t, d)
    for p in kept:
      want_out[order[p] // k] += w.reshape(-1)[order[p]] * x[order[p] // k].float()
    assert torch.allclose(out.float(), want_out.to(torch.bfloat16).float(), rtol=1e-2, atol=1e-2)
    total += out.float()
  if not buffered:  # nothing dropped: the shards' outputs add up to (sum of a token's weights) * x
    assert torch.allclose(total, w.sum(1, keepdim=True) * x.float(), rtol=2e-2, atol=2e-2)


def test_a2a_ragged_sort_by_hand():
  x = torch.arange(12, dtype=torch.float32).reshape(6, 2).to(torch.bfloat16)
  out = O.a2a_ragged_sort(x, np.array([2, 0, 1, 5, 4, 3]), 3)
  assert torch.equal(out, torch.tensor([[4, 5], [0, 1], [2, 3], [0, 0], [0, 0], [0, 0]], dtype=torch.bfloat16))
