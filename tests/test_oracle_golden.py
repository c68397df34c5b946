"""Pins the CPU oracle against the reference's own known answers and against
independent formulations (brute force, closed forms, second code paths)."""

import math

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O


# ---- known answers held by the reference's tests ---------------------------


def test_deepseek_group_routing_known_answer():
  # tests/unit/moe_test.py:293-326 (16 experts, 4 groups, top-2 groups, top-4)
  gate = np.array(
      [[[0.20, 0.10, 0.05, 0.10, 0.10, 0.60, 0.30, 0.10, 0.80, 0.01, 0.01, 0.01, 0.05, 0.80, 0.20, 0.10],
        [0.68, 0.20, 0.06, 0.03, 0.32, 0.10, 0.05, 0.02, 0.65, 0.20, 0.04, 0.01, 0.32, 0.10, 0.05, 0.02]]],
      dtype=np.float32)
  pre = gate - 0.5
  w, idx = O.deepseek_routing(gate, pre, 4, n_routing_groups=4, topk_routing_group=2)
  expect = np.array([[[13, 5, 6, 14], [0, 8, 1, 9]]])
  np.testing.assert_array_equal(idx, expect)
  np.testing.assert_allclose(w, np.take_along_axis(pre, expect, -1), rtol=1e-5, atol=1e-5)


def test_load_balance_updates_known_answer():
  # tests/unit/moe_test.py:328-341
  idx = np.array([[[0, 1], [3, 0], [3, 1], [1, 0]], [[0, 3], [2, 0], [1, 2], [2, 3]]])
  np.testing.assert_allclose(O.calculate_load_balance_updates(idx, 4, 0.01), [-0.01, 0.0, 0.01, 0.0])


def test_static_scale_known_answer():
  # tests/unit/quantizations_test.py:723-743
  assert abs(O.get_static_scale(O.FP8_E4M3_MAX, "fixed,224.0") - 0.5) < 1e-6
  assert abs(O.get_static_scale(O.FP8_E4M3_MAX, "fixed,-224,224") - 0.5) < 1e-6
  for bad in ("fixed,1,2,3", "fixed,-200.0,224.0", "fixed", "absmax"):
    with pytest.raises(ValueError):
      O.get_static_scale(O.FP8_E4M3_MAX, bad)
  assert float(torch.finfo(torch.float8_e4m3fn).max) == O.FP8_E4M3_MAX


def test_int4_pack_format_known_answers():
  # tests/unit/dequantize_pack_quantized_int4_test.py:61-127 (cases restated:
  # pack_to_int32 of compressed_tensors is not installed; its layout is
  # "weight k in bits [4k,4k+4) of the int32", i.e. low nibble first).
  torch.manual_seed(0)
  w = torch.randn(64, 128) * 0.1
  q, scale = O.quantize_int4_groups(w, group=32)
  packed = O.pack_int4(q)
  assert packed.shape == (64, 64)
  # int32 view: weight k lives in bits [4k, 4k+4)
  as_i32 = packed.contiguous().view(torch.int32)
  shifts = torch.arange(8, dtype=torch.int32) * 4
  nib = ((as_i32.unsqueeze(-1) >> shifts) & 0xF) - 8
  assert torch.equal(nib.reshape(64, 128).to(torch.int8), q)
  assert torch.equal(O.unpack_int4(packed), q)
  # full dequant == (int * bf16 scale).bf16 bit for bit
  sb = scale.to(torch.bfloat16)
  ref = (q.reshape(64, 4, 32).float() * sb.float().unsqueeze(-1)).reshape(64, 128).to(torch.bfloat16)
  assert torch.equal(O.dequantize_int4(packed, sb, group=32), ref)
  # boundary values and zero groups
  ones = torch.ones(16, 2, dtype=torch.bfloat16)
  for v in (-8, 7):
    p = O.pack_int4(torch.full((16, 64), v, dtype=torch.int8))
    assert torch.all(O.dequantize_int4(p, ones, group=32).float() == float(v))
  p = O.pack_int4(torch.zeros(8, 64, dtype=torch.int8))
  assert torch.all(O.dequantize_int4(p, torch.full((8, 2), 0.123, dtype=torch.bfloat16), group=32) == 0)


def test_fp8_block_dequant_formula():
  # deepseek_dequantize.py:42-68: reshape/broadcast branch vs element loop
  torch.manual_seed(1)
  x = (torch.randn(256, 384) * 3).to(torch.float8_e4m3fn)
  s = torch.rand(2, 3) + 0.5
  got = O.dequantize_fp8_blocks(x, s, 128)
  for (i, j) in [(0, 0), (127, 127), (128, 128), (255, 383), (200, 130)]:
    assert got[i, j] == (x[i, j].float() * s[i // 128, j // 128]).to(torch.bfloat16)
  # ragged shape branch (:57-62)
  xr = x[:200, :300]
  gr = O.dequantize_fp8_blocks(xr, s, 128)
  assert torch.equal(gr, got[:200, :300])


def test_gmm_int8_small_known_tolerance():
  # tests/unit/quantizations_test.py:607-653: groups [3,5], k=6, n=4, int8 on
  # both sides, mean relative error below 0.2 versus the unquantised product.
  g = torch.Generator().manual_seed(0)
  gs = np.array([3, 5], np.int32)
  lhs = torch.randn(8, 6, generator=g)
  rhs = torch.randn(2, 6, 4, generator=g)
  base = O.gmm(lhs, rhs, gs, out_dtype=torch.float32)
  ql, sl = O.quantize_rows_int8(lhs)
  qr, sr = O.quantize_weight_int8(rhs, per_expert=False)
  quant = O.gmm(ql, qr, gs, lhs_scale=sl, rhs_scale=sr, out_dtype=torch.float32)
  assert (quant - base).abs().mean() / base.abs().mean() < 0.2


# ---- brute force / invariants / independent second paths -------------------


def test_top_k_brute_force_and_ties():
  rng = np.random.default_rng(0)
  x = rng.standard_normal((50, 37)).astype(np.float32)
  vals, idx = O.top_k(x, 5)
  for r in range(50):
    row = list(x[r])
    picked = []
    for _ in range(5):
      best = max(range(37), key=lambda j: (row[j], -j) if j not in picked else (-np.inf, -j))
      picked.append(best)
    assert picked == list(idx[r])
    assert np.all(np.diff(vals[r]) <= 0)
  # ties: lower index first
  t = np.array([[1.0, 3.0, 3.0, 2.0, 3.0]], np.float32)
  assert list(O.top_k(t, 4)[1][0]) == [1, 2, 4, 3]


def test_softmax_topk_weights_closed_form():
  rng = np.random.default_rng(1)
  x = rng.standard_normal((64, 8)).astype(np.float32)
  w, idx = O.get_topk(x, k=2, weight_dtype="f32")
  a = np.take_along_axis(x, idx, -1).astype(np.float64)
  # two-way softmax == logistic of the difference
  np.testing.assert_allclose(w[:, 0], 1 / (1 + np.exp(a[:, 1] - a[:, 0])), rtol=1e-6)
  np.testing.assert_allclose(w.sum(-1), 1.0, rtol=1e-6)
  wb, _ = O.get_topk(x, k=2)
  assert np.max(np.abs(wb - w) / w) <= 2.0**-8
  wn, _ = O.get_topk(x, k=2, norm_topk_prob=True)
  np.testing.assert_allclose(wn.sum(-1), 1.0, atol=2e-2)


def test_llama4_and_gemma4_weight_rules_closed_form():
  """moe.py:742-753: Gemma4 reads softmax(all experts) at the top-k indices, Llama4 keeps the logits themselves."""
  rng = np.random.default_rng(11)
  x = rng.standard_normal((50, 12)).astype(np.float32)
  w, idx = O.get_topk(x, k=3, mode="topk_raw", weight_dtype="f32")
  np.testing.assert_array_equal(w, -np.sort(-x, axis=-1)[:, :3])
  w, idx2 = O.get_topk(x, k=3, mode="softmax_all", weight_dtype="f32")
  np.testing.assert_array_equal(idx, idx2)
  # with k == E the rule is the plain softmax, which sums to one; the selected ones are its largest entries
  wall, iall = O.get_topk(x, k=12, mode="softmax_all", weight_dtype="f32")
  np.testing.assert_allclose(wall.sum(-1), 1.0, rtol=1e-6)
  np.testing.assert_allclose(w, wall[:, :3], rtol=1e-6)
  # ratio of two entries == exp of the logit difference (fails for a softmax over the top-k only if k changes it: it does not,
  # so also check the absolute value against f64)
  z = np.exp(x.astype(np.float64))
  np.testing.assert_allclose(w, np.take_along_axis(z / z.sum(-1, keepdims=True), idx, -1), rtol=1e-5)
  wn, _ = O.get_topk(x, k=3, mode="softmax_all", norm_topk_prob=True, weight_dtype="f32")
  np.testing.assert_allclose(wn.sum(-1), 1.0, rtol=1e-5)


def test_deepseek_weights_closed_form():
  rng = np.random.default_rng(2)
  logits = rng.standard_normal((32, 64)).astype(np.float32)
  scores = (1 / (1 + np.exp(-logits))).astype(np.float32)
  bias = (rng.standard_normal(64) * 0.1).astype(np.float32)
  w, idx = O.get_topk(scores + bias, scores, k=8, mode="deepseek", routed_scaling_factor=2.5)
  np.testing.assert_allclose(w.sum(-1), 2.5, rtol=1e-5)
  # selection uses biased scores, weights use unbiased ones
  sel = np.argsort(-(scores + bias), -1, kind="stable")[:, :8]
  np.testing.assert_array_equal(idx, sel)
  raw = np.take_along_axis(scores, idx, -1)
  np.testing.assert_allclose(w, raw / raw.sum(-1, keepdims=True) * 2.5, rtol=1e-5)


def test_permute_invariants_and_bruteforce():
  rng = np.random.default_rng(3)
  t, k, e, d = 97, 3, 11, 16
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  sel[sel == 7] = 6  # leave expert 7 empty, duplicates across tokens only
  x = torch.randn(t, d).to(torch.bfloat16)
  sx, perm, gs, se = O.permute(x, sel, e)
  flat = sel.reshape(-1)
  assert sorted(perm.tolist()) == list(range(t * k))
  assert np.all(np.diff(flat[perm]) >= 0)
  for i in range(1, t * k):
    if flat[perm[i]] == flat[perm[i - 1]]:
      assert perm[i] > perm[i - 1]
  assert gs.sum() == t * k and gs[7] == 0
  for ee in range(e):
    assert gs[ee] == int((flat == ee).sum())
  np.testing.assert_array_equal(se, flat[perm])
  for i in range(t * k):
    assert torch.equal(sx[i], x[perm[i] // k])


def test_unpermute_bruteforce_and_identity():
  rng = np.random.default_rng(4)
  t, k, e, d = 40, 4, 9, 8
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  x = torch.randn(t, d).to(torch.bfloat16)
  sx, perm, _, _ = O.permute(x, sel, e)
  # identity experts, weights one: output == k * x
  out = O.unpermute(sx, perm, np.ones((t, k), np.float32), k)
  assert torch.equal(out, (x.float() * k).to(torch.bfloat16))
  # brute force with random weights and random intermediate
  inter = torch.randn(t * k, d).to(torch.bfloat16)
  w = rng.random((t, k)).astype(np.float32)
  out = O.unpermute(inter, perm, w, k, out_dtype=torch.float32)
  pos = {int(p): i for i, p in enumerate(perm)}
  for tt in range(t):
    acc = np.zeros(d, np.float64)
    for s in range(k):
      acc += float(w[tt, s]) * inter[pos[tt * k + s]].double().numpy()
    np.testing.assert_allclose(out[tt].numpy(), acc, rtol=1e-5, atol=1e-6)
  # unweighted unroute (sort_activations.py:98-121)
  un = O.unroute_sum(inter.float(), sel)
  np.testing.assert_allclose(un.numpy(), O.unpermute(inter, perm, np.ones((t, k), np.float32), k, torch.float32).numpy(), rtol=1e-6)


def test_gmm_special_cases():
  g = torch.Generator().manual_seed(5)
  m, k, n, e = 64, 48, 40, 5
  lhs = torch.randn(m, k, generator=g)
  rhs = torch.randn(e, k, n, generator=g)
  # one group holds everything -> plain matmul
  gs = np.array([0, 0, m, 0, 0], np.int32)
  np.testing.assert_allclose(O.gmm(lhs, rhs, gs, out_dtype=torch.float32), lhs @ rhs[2], rtol=1e-5, atol=1e-5)
  # ragged groups with an empty one, rows past the sum are zero
  gs = np.array([7, 0, 20, 1, 30], np.int32)
  out = O.gmm(lhs, rhs, gs, out_dtype=torch.float32)
  off = np.concatenate([[0], np.cumsum(gs)])
  for ee in range(e):
    np.testing.assert_allclose(out[off[ee]:off[ee + 1]], lhs[off[ee]:off[ee + 1]] @ rhs[ee], rtol=1e-5, atol=1e-5)
  assert torch.all(out[off[-1]:] == 0)
  # transpose_rhs
  np.testing.assert_allclose(O.gmm(lhs, rhs.transpose(1, 2).contiguous(), gs, transpose_rhs=True, out_dtype=torch.float32), out)
  # group_offset: only local groups computed, others zero (reference_gmm :111-141)
  out2 = O.gmm(lhs, rhs[2:4], gs, group_offset=2, out_dtype=torch.float32)
  assert torch.all(out2[:off[2]] == 0) and torch.all(out2[off[4]:] == 0)
  np.testing.assert_allclose(out2[off[2]:off[4]], out[off[2]:off[4]])
  # bias + partial_sum
  bias = torch.randn(e, 1, n, generator=g)
  ps = torch.randn(m, n, generator=g)
  out3 = O.gmm(lhs, rhs, gs, rhs_bias=bias, partial_sum=ps, out_dtype=torch.float32)
  np.testing.assert_allclose(out3[:7], lhs[:7] @ rhs[0] + bias[0] + ps[:7], rtol=1e-5, atol=1e-5)


def test_gmm_int8_exact_on_integers():
  g = torch.Generator().manual_seed(6)
  m, k, n, e = 33, 512, 24, 3
  lq = torch.randint(-127, 128, (m, k), generator=g, dtype=torch.int8)
  rq = torch.randint(-127, 128, (e, k, n), generator=g, dtype=torch.int8)
  gs = np.array([10, 3, 20], np.int32)
  out = O.gmm(lq, rq, gs, out_dtype=torch.float64)
  off = [0, 10, 13, 33]
  for ee in range(e):
    want = lq[off[ee]:off[ee + 1]].to(torch.int64) @ rq[ee].to(torch.int64)
    assert torch.equal(out[off[ee]:off[ee + 1]].to(torch.int64), want)


def test_gmm_block_scales_equal_dequantised_matmul():
  g = torch.Generator().manual_seed(7)
  m, k, n, e = 24, 384, 256, 2
  a = torch.randn(m, k, generator=g)
  w = torch.randn(e, n, k, generator=g) * 0.02  # [g, n, k]
  aq, asc = O.quantize_fp8_blocks(a, 1, 128)
  wq, wsc = O.quantize_fp8_blocks(w, 128, 128)  # scale [e, n/128, k/128]
  gs = np.array([10, 14], np.int32)
  rhs_scale = torch.repeat_interleave(wsc.permute(0, 2, 1), 128, dim=2)[:, :, None, :]  # v2 format [g, nb, 1, n]
  out = O.gmm(aq, wq, gs, lhs_scale=asc, rhs_scale=rhs_scale, transpose_rhs=True, quant_block=128, out_dtype=torch.float32)
  a_deq = aq.float() * torch.repeat_interleave(asc, 128, dim=1)
  w_deq = wq.float() * torch.repeat_interleave(torch.repeat_interleave(wsc, 128, 1), 128, 2)
  want = torch.cat([a_deq[:10] @ w_deq[0].T, a_deq[10:] @ w_deq[1].T])
  np.testing.assert_allclose(out, want, rtol=1e-4, atol=1e-5)
  # quantisation error itself is small
  full = torch.cat([a[:10] @ w[0].T, a[10:] @ w[1].T])
  assert (out - full).norm() / full.norm() < 0.06


def test_quantisers_closed_form():
  x = torch.tensor([[0.0, 0.0, 0.0, 0.0], [1.0, -2.0, 0.5, 127.0], [-254.0, 1.0, 3.0, 5.0]])
  q, s = O.quantize_rows_int8(x)
  assert s.tolist() == [0.0, 1.0, 2.0]
  assert q.tolist() == [[0, 0, 0, 0], [1, -2, 0, 127], [-127, 0, 2, 2]]  # 0.5->0, 1.5->2, 2.5->2 (half to even)
  w = torch.randn(3, 16, 5)
  qw, sw = O.quantize_weight_int8(w)
  assert sw.shape == (3, 5) and torch.allclose(sw, w.abs().amax(1) / 127)
  assert (qw.float() * sw[:, None, :] - w).abs().max() <= sw.max() * 0.5 + 1e-7
  qs, ss = O.quantize_weight_int8(w, per_expert=False)
  assert torch.all(ss == ss[0])
  q4, s4 = O.quantize_int4_groups(torch.randn(4, 2880), group=128)
  assert s4.shape == (4, 23) and q4.min() >= -8 and q4.max() <= 7


def test_activation_closed_forms():
  h0 = torch.tensor([-3.0, 0.0, 2.0, 9.0])
  h1 = torch.tensor([1.0, 2.0, -8.0, 0.5])
  a = O.apply_ffn_activation(h0, h1, "silu", out_dtype=torch.float32)
  np.testing.assert_allclose(a, (h0 / (1 + torch.exp(-h0))) * h1, rtol=1e-6)
  b = O.apply_ffn_activation(h0, h1, "swigluoai", out_dtype=torch.float32)
  g = torch.tensor([-3.0, 0.0, 2.0, 7.0])
  u = torch.tensor([1.0, 2.0, -7.0, 0.5])
  np.testing.assert_allclose(b, g / (1 + torch.exp(-1.702 * g)) * (u + 1), rtol=1e-6)
  # DeepSeek-V4 clipped SwiGLU (moe.py:854-866): gate clipped from above only, up clipped on both sides, plain silu, no
  # "+ 1" and no 1.702: each of these would fail one of the four columns (9 -> 7; -8 -> -7; -3 stays; factor 1)
  c = O.apply_ffn_activation(h0, h1, "silu_clip", out_dtype=torch.float32)
  np.testing.assert_allclose(c, (g / (1 + torch.exp(-g))) * u, rtol=1e-6)
  assert float(c[0]) == pytest.approx(-3.0 / (1 + np.exp(3.0)) * 1.0, rel=1e-6)  # a gate below -limit is NOT clipped
  assert float(O.apply_ffn_activation(torch.tensor([2.0]), torch.tensor([3.0]), "silu_clip", limit=1.0, out_dtype=torch.float32)) == pytest.approx(
      1.0 / (1 + np.exp(-1.0)) * 1.0, rel=1e-6)  # the limit is the argument, not a constant


def test_quantize_int4_groups_hand_case():
  """_quantize_per_group of tests/unit/dequantize_pack_quantized_int4_test.py:46-53 restated: scale = absmax / 7 clamped
  at 1e-12, q = round(w / scale) clamped to [-8, 7]; values on and between grid points, an all-zero group (the clamp),
  and the ragged 64-wide last group of K = 2880."""
  w = torch.zeros(2, 8)
  w[0] = torch.tensor([7.0, -7.0, 3.0, 3.5, 2.5, -0.4, 0.6, 0.0])  # scale 1: 3.5 -> 4, 2.5 -> 2 (half to even), -0.4 -> 0, 0.6 -> 1
  w[1, :4] = torch.tensor([14.0, -16.0, 1.0, 15.0])  # group of 4: scale 16/7; -16 -> -7, 14 -> round(6.125) = 6, 15 -> round(6.5625) = 7
  q, s = O.quantize_int4_groups(w, group=4)
  assert s.shape == (2, 2)
  assert s[0].tolist() == [1.0, pytest.approx(2.5 / 7)]
  assert q[0, :4].tolist() == [7, -7, 3, 4]
  assert q[0, 4:].tolist() == [7, -1, 2, 0]  # second group of row 0: scale 2.5/7: 2.5 -> 7, -0.4 -> -1.12 -> -1, 0.6 -> 1.68 -> 2
  assert float(s[1, 0]) == pytest.approx(16.0 / 7) and q[1, :4].tolist() == [6, -7, 0, 7]
  assert float(s[1, 1]) == pytest.approx(1e-12) and q[1, 4:].tolist() == [0, 0, 0, 0]  # zero group: clamped scale, zeros
  # K = 2880 with groups of 128: 22 full groups and one of 64; the tail's scale comes from its 64 values only
  g = torch.Generator().manual_seed(3)
  big = torch.randn(3, 2880, generator=g)
  big[:, 2816:] *= 0.01
  qb, sb = O.quantize_int4_groups(big, group=128)
  assert qb.shape == (3, 2880) and sb.shape == (3, 23)
  np.testing.assert_allclose(sb[:, 22], big[:, 2816:].abs().amax(1) / 7, rtol=1e-6)
  np.testing.assert_allclose(sb[:, 5], big[:, 640:768].abs().amax(1) / 7, rtol=1e-6)
  assert int(qb[:, 2816:].abs().max()) == 7  # the small tail still uses the full grid
  deq = O.dequantize_int4(O.pack_int4(qb), sb.to(torch.bfloat16), 128).float()
  assert float((deq - big).abs().max()) <= float(sb.max()) * 0.51 + 0.02


def test_quantize_rows_fp8_hand_case():
  """Per-row float8_e4m3fn under this build's v1 rule: scale = absmax / 448, values divided by it and rounded to nearest
  even on the e4m3 grid (3 mantissa bits: between 16 and 32 the grid step is 2, between 256 and 448 it is 32)."""
  x = torch.tensor([[448.0, -224.0, 17.0, 19.0, 1.0, 0.0],  # scale 1: 17 -> 16 (tie to even mantissa), 19 -> 20 (tie to even)
                    [896.0, 100.0, -34.0, 38.0, 2.0, 600.0],  # scale 2: 50 -> 48 (tie: 48 even, 52 odd), -17 -> -16, 19 -> 20, 300 -> 288 (nearer than 320)
                    [0.0, 0.0, 0.0, 0.0, 0.0, 0.0]])
  q, s = O.quantize_rows_fp8(x)
  assert q.dtype == torch.float8_e4m3fn and s.tolist() == [1.0, 2.0, 0.0]
  assert q.float()[0].tolist() == [448.0, -224.0, 16.0, 20.0, 1.0, 0.0]
  assert q.float()[1].tolist() == [448.0, 48.0, -16.0, 20.0, 1.0, 288.0]
  assert q.float()[2].tolist() == [0.0] * 6


def _layer_fixture(seed=8, t=60, d=32, f=48, e=6, k=2):
  g = torch.Generator().manual_seed(seed)
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  w0 = (torch.randn(e, d, f, generator=g) * 0.1).to(torch.bfloat16)
  w1 = (torch.randn(e, d, f, generator=g) * 0.1).to(torch.bfloat16)
  wo = (torch.randn(e, f, d, generator=g) * 0.1).to(torch.bfloat16)
  logits = torch.randn(t, e, generator=g).numpy()
  return x, w0, w1, wo, logits


def test_sparse_layer_equals_loop_and_dense():
  x, w0, w1, wo, logits = _layer_fixture()
  e, k = 6, 2
  wts, idx = O.get_topk(logits, k=k)

  def expert_fn(rows, gs):
    h0 = O.gmm(rows, w0, gs)
    h1 = O.gmm(rows, w1, gs)
    return O.gmm(O.apply_ffn_activation(h0, h1), wo, gs)

  sparse = O.moe_layer_sparse(x, wts, idx, e, expert_fn)

  def mlp(ee, rows):
    h0 = (rows.double() @ w0[ee].double()).to(torch.bfloat16)
    h1 = (rows.double() @ w1[ee].double()).to(torch.bfloat16)
    a = O.apply_ffn_activation(h0, h1)
    return (a.double() @ wo[ee].double()).to(torch.bfloat16)

  loop = O.moe_layer_loop(x, wts, idx, e, mlp)
  assert (sparse.float() - loop.float()).abs().max() <= 2e-2 * loop.float().abs().max()
  # dense all-experts formulation (moe.py:2996-3039): "BSM,EMH->BSEH" then
  # "BSEM,BSE->BSM" with a scattered weight matrix
  dense_w = torch.zeros(x.shape[0], e)
  dense_w.scatter_(1, torch.from_numpy(idx.astype(np.int64)), torch.from_numpy(wts))
  h0 = torch.einsum("tm,emh->teh", x.float(), w0.float()).to(torch.bfloat16)
  h1 = torch.einsum("tm,emh->teh", x.float(), w1.float()).to(torch.bfloat16)
  a = O.apply_ffn_activation(h0, h1)
  y = torch.einsum("teh,ehm->tem", a.float(), wo.float()).to(torch.bfloat16)
  dense = torch.einsum("tem,te->tm", y.float(), dense_w).to(torch.bfloat16)
  assert (sparse.float() - dense.float()).abs().max() <= 2e-2 * dense.float().abs().max()


def test_tgmm_equals_autograd_of_grouped_matmul_and_hand_case():
  """tgmm is the weight gradient of gmm: d/d rhs of sum(gmm(lhs, rhs) * dout), here taken by torch
  autograd through an independent per-group matmul; plus a hand-computed 2-group case and the
  group_offset / num_actual_groups window."""
  g = torch.Generator().manual_seed(0)
  m, k, n, e = 50, 16, 24, 4
  lhs = torch.randn(m, k, generator=g, dtype=torch.float64)
  rhs = torch.randn(e, k, n, generator=g, dtype=torch.float64, requires_grad=True)
  dout = torch.randn(m, n, generator=g, dtype=torch.float64)
  gs = np.array([10, 0, 25, 15], np.int32)
  off = np.concatenate([[0], np.cumsum(gs)])
  out = torch.cat([lhs[off[i] : off[i + 1]] @ rhs[i] for i in range(e)])
  (out * dout).sum().backward()
  got = O.tgmm(lhs, dout, gs, out_dtype=torch.float64)
  assert torch.allclose(got, rhs.grad, rtol=1e-12, atol=1e-12)
  assert torch.all(got[1] == 0)  # empty group -> zero gradient
  win = O.tgmm(lhs, dout, gs, num_actual_groups=2, group_offset=2, out_dtype=torch.float64)
  assert torch.equal(win, got[2:4])
  # hand case: rows [1,2],[3,4] | [5,6];  dout rows [1],[10] | [100]
  lhs2 = torch.tensor([[1.0, 2.0], [3.0, 4.0], [5.0, 6.0]])
  d2 = torch.tensor([[1.0], [10.0], [100.0]])
  t2 = O.tgmm(lhs2, d2, np.array([2, 1], np.int32), out_dtype=torch.float32)
  assert t2.tolist() == [[[31.0], [42.0]], [[500.0], [600.0]]]
  # existing_out joins the accumulator before the one rounding (backend.py:733-734): 256 + 1 + 0.5 rounds to 258 in
  # bf16 (8 bits of mantissa: spacing 2 above 256), while bf16(256 + 1) + 0.5 would have stayed at 256
  lhs3, d3 = torch.tensor([[16.0], [1.0]]), torch.tensor([[16.0], [1.0]])
  ex = torch.tensor([[[0.5]]])
  assert O.tgmm(lhs3, d3, np.array([2], np.int32), out_dtype=torch.bfloat16, existing_out=ex).tolist() == [[[258.0]]]
  assert O.tgmm(lhs3, d3, np.array([0, 2], np.int32), out_dtype=torch.float32, existing_out=torch.tensor([[[0.5]], [[1.0]]])).tolist() == [[[0.5]], [[258.0]]]


def test_gate_logits_special_cases():
  """GateLogit: a zero kernel gives sigmoid(0) = 0.5 everywhere (+ bias, with pre_bias untouched); a kernel
  whose columns are unit vectors copies input features; the bf16 gate rounds once at the end."""
  g = torch.Generator().manual_seed(1)
  x = torch.randn(5, 8, generator=g).to(torch.bfloat16)
  bias = torch.tensor([0.25, -1.0, 0.0, 2.0])
  out, pre = O.gate_logits(x, torch.zeros(8, 4), bias, score_func="sigmoid", deepseek=True)
  assert np.all(pre == 0.5) and np.array_equal(out, np.broadcast_to(0.5 + bias.numpy(), (5, 4)))
  sel = torch.zeros(8, 4)
  for e, f in enumerate((6, 0, 3, 3)):
    sel[f, e] = 1.0
  out, pre = O.gate_logits(x, sel)
  assert pre is None and np.array_equal(out, x.float().numpy()[:, [6, 0, 3, 3]])
  w = torch.randn(8, 4, generator=g)
  out16, _ = O.gate_logits(x, w, float32_gate_logits=False)
  want = (x.double() @ w.to(torch.bfloat16).double()).to(torch.bfloat16).float().numpy()
  assert np.array_equal(out16, want)


def test_mxfp4_dequantize_code_points_and_layout():
  """MXFP4: every e2m1 code against the OCP MX value table (restated independently from the bit fields:
  sign, 2-bit exponent with bias 1, 1 mantissa bit, subnormal 0.5), low nibble first, scale 2^(s-127)."""
  want = []
  for code in range(16):
    sign = -1.0 if code & 8 else 1.0
    e, m = (code >> 1) & 3, code & 1
    want.append(sign * (0.5 * m if e == 0 else (1.0 + 0.5 * m) * 2.0 ** (e - 1)))
  assert np.array_equal(O.E2M1_VALUES, np.array(want, np.float32))
  blocks = torch.zeros(1, 2, 16, dtype=torch.uint8)
  blocks[0, 0, 0] = 0x52  # first value code 2 (1.0), second value code 5 (3.0)
  blocks[0, 0, 15] = 0xF7  # 31st value code 7 (6.0), 32nd code 15 (-6.0)
  blocks[0, 1, 1] = 0x0B  # block 1: third value code 11 (-1.5)
  scales = torch.tensor([[127, 124]], dtype=torch.uint8)  # 2^0, 2^-3
  out = O.dequantize_mxfp4(blocks, scales)
  assert out.shape == (1, 64)
  assert out[0, 0] == 1.0 and out[0, 1] == 3.0 and out[0, 30] == 6.0 and out[0, 31] == -6.0
  assert out[0, 34] == -1.5 / 8 and out[0, 35] == 0.0
  # quantise -> dequantise is the identity on representable inputs
  g = torch.Generator().manual_seed(3)
  codes = torch.randint(0, 16, (4, 96), generator=g)
  exps = torch.randint(-6, 5, (4, 3), generator=g).float()
  x = torch.from_numpy(O.E2M1_VALUES)[codes].reshape(4, 3, 32) * torch.exp2(exps)[..., None]
  x[:, :, 0] = 6.0 * torch.exp2(exps)  # pin the block maximum so the shared exponent is the one used above
  b, s_ = O.quantize_mxfp4(x.reshape(4, 96))
  assert torch.equal(O.dequantize_mxfp4(b, s_), x.reshape(4, 96))


def test_product_mxfp4_quantiser_agrees_with_oracle_generator():
  """The package's mxfp4 quantiser (used for synthetic weights) and the oracle's test-data generator are written
  independently (threshold chain vs nearest-grid search); they must produce the same bytes."""
  from maxtext_amd import quantizations as Q

  g = torch.Generator().manual_seed(5)
  w = torch.randn(2, 6, 96, generator=g) * 0.02
  w[0, 0, :32] = 0.0  # an all-zero block
  qa = Q.quantize_weight_mxfp4(w)
  blocks, scales = O.quantize_mxfp4(w)
  assert torch.equal(qa.qvalue.reshape(2, 6, 3, 16), blocks) and torch.equal(qa.scale, scales)


def test_quantized_backward_equals_autograd_through_dequantised_operands():
  """ops.py:530-604: folding the scale of the contracted axis into the gradient is exact algebra, so without
  gradient quantisation the result equals autograd through the dequantised operands; the e5m2 quantiser keeps
  one absmax scale per row / column and its values lie on the e5m2 grid."""
  g = torch.Generator().manual_seed(4)
  m, k, n, gs = 50, 16, 24, [20, 0, 30]
  lhs_q = torch.randint(-127, 128, (m, k), generator=g).to(torch.int8)
  rhs_q = torch.randint(-127, 128, (3, k, n), generator=g).to(torch.int8)
  ls, rs = torch.rand(m, generator=g) + 0.5, torch.rand(n, generator=g) + 0.5
  grad = torch.randn(m, n, generator=g)
  dl, dr = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs, gs, grad_dtype=torch.float64)
  L = (lhs_q.double() * ls.double()[:, None]).requires_grad_(True)
  R = (rhs_q.double() * rs.double()[None, None, :]).requires_grad_(True)
  torch.cat([L[:20] @ R[0], L[20:] @ R[2]]).backward(grad.double())
  # d/dL of sum(grad * L R) = grad R^T: the reference's dlhs.  drhs is the gradient w.r.t. the value lhs_scale * lhs_q
  # multiplies, i.e. R.grad with L replaced by lhs_q * lhs_scale: the same thing.
  assert float((dl - L.grad).abs().max()) <= 1e-3
  assert float((dr - R.grad).abs().max()) <= 1e-3 and float(dr[1].abs().max()) == 0.0
  # per-expert scales [g, n] reduce to the shared case when all rows are equal
  dl2, dr2 = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs[None].expand(3, n).contiguous(), gs, grad_dtype=torch.float64)
  assert torch.equal(dl, dl2) and torch.equal(dr, dr2)
  # e5m2 quantiser: closed-form scale, grid membership, and a backward that stays within the format's 2^-3 steps
  q, s = O.quantize_e5m2(grad, dim=1)
  np.testing.assert_allclose(s[:, 0].numpy(), grad.abs().amax(1).numpy() / 57344.0, rtol=1e-6)
  assert torch.equal(q, q.to(torch.float8_e5m2).to(torch.float32)) and float(q.abs().max()) == 57344.0
  assert float(((q * s) - grad).abs().max() / grad.abs().max()) <= 2.0**-3
  dlq, drq = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs, gs, bwd_qtype="e5m2", grad_dtype=torch.float64)
  assert float((dlq - dl).abs().max() / dl.abs().max()) <= 0.1 and float((drq - dr).abs().max() / dr.abs().max()) <= 0.1


def test_quantized_backward_with_per_tensor_scales():
  """ops.py:568-601 with disable_channelwise_axes: scalar operand scales and one e5m2 scale per gradient.  Without
  gradient quantisation the result is the channelwise backward on constant scale vectors (the same algebra); with it, a
  hand case: the tensor's largest magnitude lands on 57344, a value at a quarter of it on 14336, and one scale serves
  rows whose own maxima differ by 2^10 (per row each would reach 57344)."""
  g = torch.Generator().manual_seed(6)
  m, k, n, gs = 30, 8, 16, [10, 0, 20]
  lhs_q = torch.randint(-127, 128, (m, k), generator=g).to(torch.int8)
  rhs_q = torch.randint(-127, 128, (3, k, n), generator=g).to(torch.int8)
  ls, rs = torch.full((m,), 0.75), torch.full((n,), 1.5)
  grad = torch.randn(m, n, generator=g)
  a = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs, gs, grad_dtype=torch.float64, per_tensor=True)
  b = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs, gs, grad_dtype=torch.float64)
  assert torch.equal(a[0], b[0]) and torch.equal(a[1], b[1])
  x = torch.tensor([[8.0, -2.0, 0.5], [2.0**-7, 2.0**-8, 0.0]])
  q, s = O.quantize_e5m2(x, dim=(0, 1))
  assert tuple(s.shape) == (1, 1) and float(s) == float(np.float32(8.0) / np.float32(57344.0))
  np.testing.assert_array_equal(q.numpy(), [[57344.0, -14336.0, 3584.0], [56.0, 28.0, 0.0]])
  q_row, s_row = O.quantize_e5m2(x, dim=1)
  assert float(q_row[1, 0]) == 57344.0 and float(s_row[1, 0]) == float(np.float32(2.0**-7) / np.float32(57344.0))
  # the quantised backward with ONE scale equals the products of the dequantised gradients
  dlq, drq = O.gmm_bwd_quantized(grad, lhs_q, ls, rhs_q, rs, gs, bwd_qtype="e5m2", grad_dtype=torch.float64, per_tensor=True)
  q1, s1 = O.quantize_e5m2(grad * 1.5, dim=(0, 1))
  q2, s2 = O.quantize_e5m2(grad * 0.75, dim=(0, 1))
  want_dl = O.gmm(q1 * s1, rhs_q.float().transpose(1, 2), gs, out_dtype=torch.float64)
  want_dr = O.tgmm(lhs_q.float(), q2 * s2, gs, out_dtype=torch.float64)
  assert float((dlq - want_dl).abs().max()) <= 1e-3 * float(want_dl.abs().max())
  assert float((drq - want_dr).abs().max()) <= 1e-3 * float(want_dr.abs().max())


def test_hash_routing_is_a_table_lookup():
  """moe.py:729-738: a hand case (two tokens, k = 2) and the invariants of the scaling (moe.py:767-773)."""
  scores = np.array([[0.1, 0.2, 0.3, 0.4], [0.4, 0.3, 0.2, 0.1]], np.float32)
  table = np.array([[0, 1], [2, 3], [3, 0]], np.float32)  # stored as f32 (moe.py:448-454)
  w, idx = O.hash_routing(scores, table, np.array([2, 1]), routed_scaling_factor=2.0)
  np.testing.assert_array_equal(idx, [[3, 0], [2, 3]])
  np.testing.assert_allclose(w, [[2 * 0.4 / 0.5, 2 * 0.1 / 0.5], [2 * 0.2 / 0.3, 2 * 0.1 / 0.3]], rtol=1e-6)
  w2, _ = O.hash_routing(scores, table, np.array([2, 1]), routed_score_func="", routed_scaling_factor=1.0)
  np.testing.assert_allclose(w2, [[0.4, 0.1], [0.2, 0.1]], rtol=1e-7)


# ---- the in-tree quantisers (gmm_v2's activation quantiser, manual_quantize), pinned in exact arithmetic ----
#
# The helpers below do IEEE arithmetic with python Fractions: every operation is carried out exactly and then
# rounded (nearest, ties to even) to a significand of `p` bits (24 = float32, 8 = bfloat16).  They share no code
# with the oracle (no torch, no numpy float types).


def _rne(x, p):
  from fractions import Fraction

  x = Fraction(x)
  if x == 0:
    return x
  sign = -1 if x < 0 else 1
  a = abs(x)
  e = 0
  while a >= 2:
    a /= 2
    e += 1
  while a < 1:
    a *= 2
    e -= 1
  scaled = a * 2 ** (p - 1)  # in [2^(p-1), 2^p)
  n = int(scaled)  # floor
  rem = scaled - n
  if rem > Fraction(1, 2) or (rem == Fraction(1, 2) and n % 2 == 1):
    n += 1
  return sign * Fraction(n, 2 ** (p - 1)) * Fraction(2) ** e


def _op(x, dt):
  """One JAX op whose result has dtype dt: float32 rounds once; bfloat16 is carried in float32 and rounded again."""
  return _rne(x, 24) if dt == "f32" else _rne(_rne(x, 24), 8)


def _trunc(x):
  return int(x) if x >= 0 else -int(-x)


def _v2_int8_row(row, dt):
  """pallas_mosaic_tpu_v2_gmm_kernel.py:533-542 on one row (= one quant block) with Fractions."""
  from fractions import Fraction

  row = [Fraction(v) for v in row]
  amax = max(abs(v) for v in row)
  scale = _op(amax / 127, dt)
  inv = Fraction(0) if scale == 0 else _op(1 / scale, dt)
  return [_trunc(_op(v * inv, dt)) for v in row], scale


def _bf16_exact(vals):
  t = torch.tensor(vals, dtype=torch.float32)
  assert torch.equal(t, t.to(torch.bfloat16).float()), "test inputs must be exact in bf16"
  return t


def test_v2_quantiser_int8_matches_exact_arithmetic():
  # rows chosen so that the rule's ingredients matter: fractions of the scale, negative values, an all-zero row
  rows = [[1.0, 0.703125, -0.5, 0.25, 0.00390625, -0.99609375, 0.33203125, 0.66796875],
          [1.5, -1.4921875, 0.75, 0.375, 0.01171875, 1.0, -0.1875, 0.5],
          [3.0, 2.984375, -2.96875, 1.0, 0.5, 0.25, -3.0, 0.0234375],
          [0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0, 0.0],
          [100.0, 99.5, -37.25, 12.125, 0.78125, -100.0, 50.0, 25.0]]
  for dt, tdt in (("bf16", torch.bfloat16), ("f32", torch.float32)):
    x = _bf16_exact(rows).to(tdt)
    q, s = O.quantize_lhs_v2(x, torch.int8, quant_block=8)
    for r, row in enumerate(rows):
      want_q, want_s = _v2_int8_row(row, dt)
      assert q[r].tolist() == want_q, (dt, r)
      assert float(s[r, 0]) == float(want_s), (dt, r)
  # zero row: scale 0, inverse forced to 0 (:537-540), q = 0
  assert q[3].abs().max() == 0 and float(s[3, 0]) == 0.0


def test_v2_quantiser_hand_cases_separate_the_alternatives():
  from fractions import Fraction as F

  # (1) truncation vs rounding.  f32 row [1, 0.703125]: scale = f32(1/127), inv = f32(1/scale) = 127 exactly
  #     (1/127 rounds to 0x3C010204 = 0.007874015718698502; its reciprocal is 127.0000000486, which rounds to 127),
  #     0.703125 * 127 = 89.296875 -> truncation gives 89, and 0.99609375 * 127 = 126.50390625 -> 126 (rounding: 127).
  x = torch.tensor([[1.0, 0.703125, 0.99609375, -0.99609375]], dtype=torch.float32)
  q, s = O.quantize_lhs_v2(x, torch.int8, quant_block=4)
  assert float(s[0, 0]) == float(_rne(F(1, 127), 24)) == 0.007874015718698502
  assert q[0].tolist() == [127, 89, 126, -126]
  assert torch.round(x * 127.0)[0].tolist() == [127.0, 89.0, 127.0, -127.0]  # what any rounding rule would give
  # (2) half-even vs half-away cannot be told apart once truncation is in place; the product rule (rint) is pinned
  #     separately in test_quantisers_closed_form.  What can be told apart is x * (1/scale) from x / scale:
  #     bf16 row with absmax 1.5: scale = bf16(f32(1.5/127)) = 0.0118408203125 (1.515625 * 2^-7),
  #     inv = bf16(84.4536...) = 84.5; 1.4921875 * 84.5 = 126.08984375 -> bf16 126.0 -> 126, while
  #     1.4921875 / 0.0118408203125 = 126.02 -> 126 too, but 0.75 * 84.5 = 63.375 -> bf16 63.5 -> 63 against
  #     0.75 / scale = 63.34 -> bf16 63.25 -> 63; the separating element is 1.5 itself:
  #     1.5 * 84.5 = 126.75 -> bf16 (tie between 126.5 and 127.0, even significand) 127.0 -> 127, and
  #     1.5 / scale = 126.68 -> bf16 126.5 -> 126.
  xb = torch.tensor([[1.5, 1.4921875, 0.75]], dtype=torch.bfloat16)
  q, s = O.quantize_lhs_v2(xb, torch.int8, quant_block=3)
  assert float(s[0, 0]) == 0.0118408203125
  assert q[0].tolist() == [127, 126, 63]
  div = [_trunc(_op(F(v) / F(0.0118408203125), "bf16")) for v in (1.5, 1.4921875, 0.75)]
  assert div == [126, 126, 63]  # the x / scale rule differs on the first element
  # (3) bf16 vs f32 intermediate arithmetic: the same values as f32 input give scale = f32(1.5/127) and
  #     inv = f32(84.666...): 1.4921875 * inv = 126.338... -> 126, 0.75 * inv = 63.4999... -> 63, 1.5 * inv -> 126 or 127
  q32, s32 = O.quantize_lhs_v2(xb.float(), torch.int8, quant_block=3)
  assert float(s32[0, 0]) == float(_rne(F(3, 2) / 127, 24)) != float(s[0, 0])
  assert q32[0].tolist() == _v2_int8_row([1.5, 1.4921875, 0.75], "f32")[0]
  # (4) per-block scales: two blocks of one row are quantised independently
  x2 = torch.tensor([[1.0, 0.5, 8.0, 4.0]], dtype=torch.bfloat16)
  q, s = O.quantize_lhs_v2(x2, torch.int8, quant_block=2)
  assert s.shape == (1, 2) and q[0].tolist() == _v2_int8_row([1.0, 0.5], "bf16")[0] + _v2_int8_row([8.0, 4.0], "bf16")[0]


def test_v2_quantiser_fp8_and_static_scale():
  from fractions import Fraction as F

  # e4m3fn grid near the top: 448 = max, spacing 32 above 256, 16 in [128, 256)
  # dynamic, f32 row [448, 300, 17, -1.0625]: scale = 1, inv = 1 -> q = RNE to e4m3: 448, 288|320 -> 300 is 288 + 12 -> 288,
  # 17 -> 16|18 (spacing 2 in [16,32)) tie -> even significand: 16 = 1.000b * 2^4, 18 = 1.001b * 2^4 -> 16;
  # -1.0625 -> spacing 0.125 in [1,2): tie between -1.0 and -1.125 -> -1.0
  x = torch.tensor([[448.0, 300.0, 17.0, -1.0625]], dtype=torch.float32)
  q, s = O.quantize_lhs_v2(x, torch.float8_e4m3fn, quant_block=4)
  assert float(s[0, 0]) == 1.0 and q[0].float().tolist() == [448.0, 288.0, 16.0, -1.0]
  # static scale of tests/integration/tokamax_test.py:113-114 ("fixed,-224,224" -> 0.5, quantizations_test.py:723):
  # inv = 2 exactly, values beyond +-224 are clipped to +-448 BEFORE the cast (no NaN), :531
  st = O.get_static_scale(448.0, "fixed,-224,224")
  x = torch.tensor([[1.0, 223.0, 224.0, 300.0, -1000.0, 0.51171875]], dtype=torch.bfloat16)
  q, s = O.quantize_lhs_v2(x, torch.float8_e4m3fn, static_scale=st)
  assert s.shape == (1, 1) and float(s) == 0.5
  # 1.0234375 -> e4m3 spacing 0.125 in [1, 2) -> 1.0
  assert q[0].float().tolist() == [2.0, 448.0, 448.0, 448.0, -448.0, 1.0]
  # a static int8 scale that is not a power of two: "fixed,3" -> 3/127; bf16(3/127) = 0.0236816..., inverse in bf16
  st = O.get_static_scale(127.0, "fixed,3")
  sb = _op(F(st), "bf16")
  inv = _op(1 / sb, "bf16")
  vals = [3.0, 2.984375, -1.0, 0.01171875, 10.0, -10.0]
  q, s = O.quantize_lhs_v2(_bf16_exact([vals]).to(torch.bfloat16), torch.int8, static_scale=st)
  want = [_trunc(max(F(-127), min(F(127), _op(F(v) * inv, "bf16")))) for v in vals]
  assert q[0].tolist() == want and float(s) == float(sb)
  assert want[4] == 127 and want[5] == -127  # clipped, then cast
  # with an f32 accumulator dtype the inverse and the product are f32 (promotion of bf16 * f32)
  q32, s32 = O.quantize_lhs_v2(_bf16_exact([vals]).to(torch.bfloat16), torch.int8, static_scale=st, acc_dtype=torch.float32)
  inv32 = _op(1 / _op(F(st), "f32"), "f32")
  assert q32[0].tolist() == [_trunc(max(F(-127), min(F(127), _op(F(v) * inv32, "f32")))) for v in vals]


def test_manual_quantize_matches_exact_arithmetic():
  from fractions import Fraction as F

  # layers/quantizations.py:961-991 with "fixed,-224,224" (scale 0.5, exact in bf16): q = clip(w / 0.5).astype(e4m3)
  w = torch.tensor([[0.25, -0.28125, 300.0, 1.0625]], dtype=torch.bfloat16)
  q, s = O.manual_quantize(w, torch.float8_e4m3fn, "fixed,-224,224")
  assert float(s) == 0.5 and q[0].float().tolist() == [0.5, -0.5625, 448.0, 2.0]  # 2.125 -> tie 2.0|2.25 -> 2.0
  # a scale that bf16 cannot hold: "fixed,3" for int8: the division uses the bf16-rounded scale tensor
  wv = [3.0, -2.984375, 1.0, 0.01171875]
  q, s = O.manual_quantize(_bf16_exact([wv]).to(torch.bfloat16), torch.int8, "fixed,3")
  sb = _op(F(3, 127), "bf16")
  assert q[0].tolist() == [_trunc(max(F(-127), min(F(127), _op(F(v) / sb, "bf16")))) for v in wv]
  assert float(s) == float(sb)


def test_gmm_with_v2_scale_layouts_equals_dequantised_matmul():
  # lhs scales per row per 512-block (in-kernel quantiser), rhs scales [g, nb, 1, n] with another block size, a scale
  # shared by all experts ([1, 1, 1, n], ops.py:250-260) and a static [1, 1] lhs scale: all equal the plain matmul of the
  # dequantised operands, group by group
  g0 = torch.Generator().manual_seed(11)
  m, k, n, g = 24, 1024, 16, 3
  gs = np.array([7, 0, 17], np.int32)
  lq = torch.randint(-127, 128, (m, k), generator=g0).to(torch.int8)
  rq = torch.randint(-127, 128, (g, k, n), generator=g0).to(torch.int8)
  ls = torch.rand((m, 2), generator=g0) + 0.5
  rs = torch.rand((g, 4, 1, n), generator=g0) + 0.5
  ld = lq.double() * torch.repeat_interleave(ls.double(), 512, dim=1)
  rd = rq.double() * torch.repeat_interleave(rs[:, :, 0, :].double(), 256, dim=1)
  want = torch.zeros((m, n), dtype=torch.float64)
  want[:7] = ld[:7] @ rd[0]
  want[7:] = ld[7:] @ rd[2]
  got = O.gmm(lq, rq, gs, lhs_scale=ls, rhs_scale=rs, quant_block=(512, 256), out_dtype=torch.float64)
  torch.testing.assert_close(got, want, rtol=1e-12, atol=1e-9)
  shared = rs[:1, :1]
  got = O.gmm(lq, rq, gs, lhs_scale=torch.tensor([[0.25]]), rhs_scale=shared, out_dtype=torch.float64)
  want = torch.zeros((m, n), dtype=torch.float64)
  want[:7] = lq[:7].double() @ rq[0].double()
  want[7:] = lq[7:].double() @ rq[2].double()
  torch.testing.assert_close(got, want * 0.25 * shared[0, 0].double(), rtol=1e-12, atol=1e-9)


def test_gate_logits_sqrtsoftplus_closed_forms():
  """sqrt(softplus(x)) (linears.py:51-53): sqrt(ln 2) at 0, sqrt(x) far above, exp(x / 2) far below."""
  x = torch.tensor([[1.0, 0.0, 0.0]]).to(torch.bfloat16)
  kernel = torch.tensor([[0.0, 50.0, -50.0], [0.0, 0.0, 0.0], [0.0, 0.0, 0.0]])
  out, pre = O.gate_logits(x, kernel, score_func="sqrtsoftplus", deepseek=True)
  np.testing.assert_allclose(out[0], [math.sqrt(math.log(2.0)), math.sqrt(50.0), math.exp(-25.0)], rtol=1e-6)
  assert np.array_equal(out, pre)


def test_ragged_variants_hand_cases():
  """ragged_gather (ragged_gather.py:310-320), ragged_gather_reduce (ragged_gather_reduce_v2.py:170-182) and the
  weight-before-wo rule (deepseek_batchsplit_fp8.py:1048-1049) on rows worked out by hand."""
  x = torch.tensor([[1.0, 2.0], [10.0, 20.0], [100.0, 200.0], [float("nan"), 7.0]]).to(torch.bfloat16)
  # gather with weights: row i of the output is x[indices[i]] * weights[i]
  got = O.ragged_gather(x, np.array([2, 0, 0, 1]), weights=torch.tensor([0.5, 2.0, 1.0, 0.25]).to(torch.bfloat16))
  assert got.dtype == torch.bfloat16 and got.tolist() == [[50.0, 100.0], [2.0, 4.0], [1.0, 2.0], [2.5, 5.0]]
  # rows outside [start, end) come back as zeros, NaN source rows included
  got = O.ragged_gather(x, np.array([3, 1, 2, 3]), start=1, end=3)
  assert got.tolist() == [[0.0, 0.0], [10.0, 20.0], [100.0, 200.0], [0.0, 0.0]]
  # gather-reduce: groups of 2; the NaN row sits behind a cleared mask bit; group 2 has no valid row
  idx = np.array([0, 1, 3, 2, 3, 3])
  w = torch.tensor([1.0, 0.5, 9.0, 0.25, 1.0, 1.0])
  mask = np.array([1, 1, 0, 1, 0, 0], bool)
  got = O.ragged_gather_reduce(x, idx, w, mask, 2)
  assert got.dtype == torch.bfloat16 and got.tolist() == [[6.0, 12.0], [25.0, 50.0], [0.0, 0.0]]
  # one rounding at the end: 256 + 1 + 1 = 258 in f32 -> bf16 258, where rounding after every addition would stay at 256
  x2 = torch.tensor([[256.0], [1.0]]).to(torch.bfloat16)
  got = O.ragged_gather_reduce(x2, np.array([0, 1, 1]), torch.ones(3), np.ones(3, bool), 3)
  assert got.tolist() == [[258.0]]
  # with every row valid it is unpermute (moe.py:1039-1063) under another name
  g = torch.Generator().manual_seed(3)
  t, k, d = 7, 3, 16
  y = torch.randn(t * k, d, generator=g).to(torch.bfloat16)
  perm = np.random.default_rng(0).permutation(t * k).astype(np.int32)
  wts = torch.rand(t, k, generator=g)
  inv = np.argsort(perm, kind="stable")
  a = O.ragged_gather_reduce(y, inv, wts.reshape(-1), np.ones(t * k, bool), k)
  assert torch.equal(a, O.unpermute(y, perm, wts.numpy(), k))
  # weight before wo: silu(33) = 33 in f32, 33 * 1.015625 = 33.515625 -> bf16 33.5; 33.5 * 1.75 = 58.625 is a tie ->
  # 58.5 (even); a single rounding of 33.515625 * 1.75 = 58.652... would have given 58.75
  h0 = torch.tensor([[33.0]]).to(torch.bfloat16)
  h1 = torch.tensor([[1.015625]]).to(torch.bfloat16)
  got = O.weighted_intermediate(h0, h1, torch.tensor([1.75]))
  assert got.tolist() == [[58.5]]


def test_permute_roll_is_a_rotation_of_the_plain_order():
  # (id - roll) % E keeps the order inside an expert and moves the experts below `roll` behind all others (moe.py:953-954)
  rng = np.random.default_rng(5)
  t, k, e, roll = 37, 3, 8, 3
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  x = torch.arange(t, dtype=torch.float32).reshape(t, 1).to(torch.bfloat16)
  _, perm0, gs0, _ = O.permute(x, sel, e)
  si, perm, gs, se = O.permute(x, sel, e, roll_to_expert_id=roll)
  ahead = int(gs0[:roll].sum())
  np.testing.assert_array_equal(perm, np.roll(perm0, -ahead))
  np.testing.assert_array_equal(gs, np.roll(gs0, -roll))
  np.testing.assert_array_equal(se, np.repeat(np.arange(e), np.roll(gs0, -roll)))
  # brute force: rows listed expert by expert starting at expert `roll`, tokens in order
  want = [i for ex in list(range(roll, e)) + list(range(roll)) for i in range(t * k) if sel.reshape(-1)[i] == ex]
  np.testing.assert_array_equal(perm, want)
  assert torch.equal(si, x[torch.tensor(want) // k])
