"""GPU parity: every C-ABI entry point against the CPU oracle on identical seeded inputs.

Index outputs (top-k indices, perm, group_sizes, sorted_experts, quantised values) are compared
bit-exactly; floating-point outputs with max|got-want| / max|want| <= 1e-2 (bf16 outputs, f32
accumulation), the tolerance this path is specified to.
"""

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

TOL = 1e-2
# kernel families of moe_gmm_tuned the block-scaled fp8 tests run: picked by shape / streaming / 128 x 128 tiles / 256 x 256 tiles
FP8_KERNELS = {0: None, 1: "stream", 2: "tiled", 3: "big"}


from tolerances import ELEM_ATOL_RMS_CHAINED, relerr  # noqa: E402  (max-norm error; also enforces the elementwise criterion)


@pytest.fixture(scope="module")
def K():
  from maxtext_amd import kernels

  assert torch.cuda.is_available()
  return kernels


def cuda(x):
  if isinstance(x, np.ndarray):
    x = torch.from_numpy(x)
  return x.cuda().contiguous()


# ---------------------------------------------------------------- routing


@pytest.mark.parametrize("t,e,k", [(1, 8, 2), (257, 8, 2), (100, 128, 8), (64, 256, 8), (33, 32, 4), (5, 512, 16), (19, 60, 6)])
def test_route_softmax_topk(K, t, e, k):
  rng = np.random.default_rng(t * 1000 + e)
  logits = rng.standard_normal((t, e)).astype(np.float32)
  for norm in (False, True):
    w, idx = K.route_topk(cuda(logits), k=k, norm_topk_prob=norm)
    ow, oidx = O.get_topk(logits, k=k, norm_topk_prob=norm)
    np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
    # weights are bf16-rounded: a 1-ulp f32 difference in exp may move a value by one bf16 ulp
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2.0**-7, atol=1e-6)


def test_route_ties_lower_index_first(K):
  logits = np.zeros((4, 16), np.float32)
  logits[1, [3, 9, 12]] = 2.0
  logits[2] = -np.inf
  logits[3, 5] = np.inf
  w, idx = K.route_topk(cuda(logits), k=4)
  _, oidx = O.get_topk(logits, k=4)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
  assert idx[0].tolist() == [0, 1, 2, 3] and idx[1].tolist() == [3, 9, 12, 0]


@pytest.mark.parametrize("t,e,k,groups,topg", [(256, 256, 8, -1, -1), (64, 64, 6, 8, 3), (2, 16, 4, 4, 2)])
def test_route_deepseek(K, t, e, k, groups, topg):
  rng = np.random.default_rng(7 + e)
  raw = rng.standard_normal((t, e)).astype(np.float32)
  scores = (1.0 / (1.0 + np.exp(-raw))).astype(np.float32)
  bias = (rng.standard_normal(e) * 0.1).astype(np.float32)
  gate = (scores + bias).astype(np.float32)
  w, idx = K.route_topk(cuda(gate), cuda(scores), k=k, mode="deepseek", norm_topk_prob=True, routed_scaling_factor=2.5,
                        n_routing_groups=groups, topk_routing_group=topg)
  ow, oidx = O.get_topk(gate, scores, k=k, mode="deepseek", routed_scaling_factor=2.5, n_routing_groups=groups,
                        topk_routing_group=topg)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
  np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=1e-5)


def test_route_deepseek_reference_known_answer(K):
  # tests/unit/moe_test.py:293-326
  gate = np.array(
      [[0.20, 0.10, 0.05, 0.10, 0.10, 0.60, 0.30, 0.10, 0.80, 0.01, 0.01, 0.01, 0.05, 0.80, 0.20, 0.10],
       [0.68, 0.20, 0.06, 0.03, 0.32, 0.10, 0.05, 0.02, 0.65, 0.20, 0.04, 0.01, 0.32, 0.10, 0.05, 0.02]], np.float32)
  pre = gate - 0.5
  w, idx = K.route_topk(cuda(gate), cuda(pre), k=4, mode="deepseek", norm_topk_prob=False, routed_scaling_factor=1.0,
                        n_routing_groups=4, topk_routing_group=2)
  expect = np.array([[13, 5, 6, 14], [0, 8, 1, 9]])
  np.testing.assert_array_equal(idx.cpu().numpy(), expect)
  np.testing.assert_allclose(w.cpu().numpy(), np.take_along_axis(pre, expect, -1), rtol=1e-6)


# ---------------------------------------------------------------- sort / permute


def _zipf_selection(rng, t, e, k, s=1.2):
  logits = rng.standard_normal((t, e)) - s * np.log(np.arange(1, e + 1)) * 3.0
  return np.argsort(-logits, -1, kind="stable")[:, :k].astype(np.int32)


@pytest.mark.parametrize("t,e,k", [(1, 8, 2), (7, 8, 2), (128, 8, 2), (512, 8, 2), (128, 256, 8), (341, 512, 3), (1000, 128, 8), (4099, 256, 8), (2048, 32, 4), (513, 512, 3)])
def test_sort_by_expert_bit_exact(K, t, e, k):
  rng = np.random.default_rng(e + t)
  sel = _zipf_selection(rng, t, e, k) if e >= 32 else np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  perm, inv, gs, se = K.sort_by_expert(cuda(sel), e)
  x = torch.zeros(t, 8, dtype=torch.bfloat16)
  _, operm, ogs, ose = O.permute(x, sel, e)
  np.testing.assert_array_equal(perm.cpu().numpy(), operm)
  np.testing.assert_array_equal(gs.cpu().numpy(), ogs)
  np.testing.assert_array_equal(se.cpu().numpy(), ose)
  np.testing.assert_array_equal(inv.cpu().numpy(), np.argsort(operm, kind="stable").astype(np.int32))
  if e >= 128:
    assert (ogs == 0).any()  # the skewed selection leaves experts empty


@pytest.mark.parametrize("t,e,k,roll", [(7, 8, 2, 2), (128, 8, 2, 6), (1000, 128, 8, 96), (4099, 256, 8, 32), (2048, 32, 4, 31), (513, 512, 3, 64)])
def test_sort_by_expert_rolled_bit_exact(K, t, e, k, roll):
  # permute(roll_to_expert_id=...) (moe.py:953-954): the ids are sorted as (id - roll) % E
  rng = np.random.default_rng(e + t + roll)
  sel = _zipf_selection(rng, t, e, k) if e >= 32 else np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  perm, inv, gs, se = K.sort_by_expert(cuda(sel), e, roll_to_expert_id=roll)
  _, operm, ogs, ose = O.permute(torch.zeros(t, 8, dtype=torch.bfloat16), sel, e, roll_to_expert_id=roll)
  np.testing.assert_array_equal(perm.cpu().numpy(), operm)
  np.testing.assert_array_equal(gs.cpu().numpy(), ogs)
  np.testing.assert_array_equal(se.cpu().numpy(), ose)
  np.testing.assert_array_equal(inv.cpu().numpy(), np.argsort(operm, kind="stable").astype(np.int32))
  # the rolled order is the plain order of the ids rotated by the rows of the first `roll` experts
  plain = K.sort_by_expert(cuda(sel), e)
  ahead = int(plain[2][:roll].sum())
  np.testing.assert_array_equal(perm.cpu().numpy(), np.roll(plain[0].cpu().numpy(), -ahead))
  with pytest.raises(RuntimeError):
    K.sort_by_expert(cuda(sel), e, roll_to_expert_id=e)


@pytest.mark.parametrize("d", [8, 512, 2048, 4096, 7168, 14336])
def test_gather_rows_copy_bit_exact(K, d):
  rng = np.random.default_rng(d)
  t, k, e = 50, 4, 16
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  x = torch.randn(t, d, generator=torch.Generator().manual_seed(d)).to(torch.bfloat16)
  perm, _, _, _ = K.sort_by_expert(cuda(sel), e)
  got = K.gather_rows(cuda(x), perm, k)
  want, _, _, _ = O.permute(x, sel, e)
  assert torch.equal(got.cpu(), want)


@pytest.mark.parametrize("d", [64, 512, 4096, 14336])
def test_gather_rows_int8_quant(K, d):
  g = torch.Generator().manual_seed(d + 1)
  x = torch.randn(37, d, generator=g).to(torch.bfloat16)
  x[3] = 0
  idx = torch.randint(0, 37, (80,), generator=g).to(torch.int32)
  q, s = K.gather_rows(cuda(x), cuda(idx), 1, out_dtype=torch.int8)
  oq, os_ = O.quantize_rows_int8(x[idx.long()])
  assert torch.equal(s.cpu(), os_)
  assert torch.equal(q.cpu(), oq)


def test_gather_rows_int8_quant_next_to_rounding_boundaries(K):
  """Rows whose quotients x / scale sit on and right beside k + 1/2: the values are bf16((k + 1/2) * scale) for random k
  and row maxima, so the quotients scatter within 2^-9 of the boundaries, thousands exactly on them, hundreds beside them
  by less than 1e-4; the quantised values must equal the oracle's rint(x / scale) on every one
  (the kernel multiplies by 1 / scale and divides only next to a boundary), also with a per-tensor static scale and
  with a scale per 128-wide block."""
  rng = np.random.default_rng(73)
  rows, d = 96, 1024
  amax = torch.from_numpy(np.concatenate([[127.0, 254.0, 63.5, 1e-3, 3e4], rng.uniform(0.01, 300.0, rows - 5)]).astype(np.float32)).to(torch.bfloat16).float()
  scale = amax / 127.0
  k = torch.from_numpy(rng.integers(-127, 127, (rows, d)).astype(np.float32)) + 0.5
  x = (k * scale[:, None]).to(torch.bfloat16)
  x[:, 0] = amax.to(torch.bfloat16)  # the row maximum itself, so that the scale is the intended one
  oq, os_ = O.quantize_rows_int8(x)
  assert torch.equal(os_, scale)
  frac = (x.float() / os_[:, None]).double() % 1.0
  assert int(((frac - 0.5).abs() < 1e-4).sum()) > 1000 and int((frac == 0.5).sum()) > 100  # the cases meant are there
  q, s = K.gather_rows(cuda(x), None, 1, out_dtype=torch.int8)
  assert torch.equal(s.cpu(), os_) and torch.equal(q.cpu(), oq)
  qb, sb = K.gather_rows(cuda(x), None, 1, out_dtype=torch.int8, block_k=128)
  ob, osb = O.quantize_rows_int8(x.reshape(rows * (d // 128), 128))
  assert torch.equal(sb.cpu().reshape(-1), osb) and torch.equal(qb.cpu().reshape(-1, 128), ob)
  static = torch.tensor([0.37], dtype=torch.float32)
  xs = ((k[:8] * 0.37).clamp(-60, 60)).to(torch.bfloat16)
  qs, _ = K.gather_rows(cuda(xs), None, 1, out_dtype=torch.int8, static_scale=cuda(static))
  want = torch.clamp(torch.round(xs.float() / static), -127, 127).to(torch.int8)
  assert torch.equal(qs.cpu(), want)


@pytest.mark.parametrize("d", [128, 2048, 7168, 2880])
def test_gather_rows_fp8_block_quant(K, d):
  g = torch.Generator().manual_seed(d + 2)
  x = (torch.randn(29, d, generator=g) * 3).to(torch.bfloat16)
  x[5, 128:256] = 0 if d > 256 else x[5, 128:256]
  q, s = K.gather_rows(cuda(x), None, 1, out_dtype=torch.float8_e4m3fn, block_k=128)
  oq, os_ = O.quantize_fp8_blocks(x, 1, 128)
  assert torch.equal(s.cpu(), os_)
  assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))


def _v2_inputs(d, seed):
  g = torch.Generator().manual_seed(seed)
  x = (torch.randn(41, d, generator=g) * torch.logspace(-3, 2, 41)[:, None]).to(torch.bfloat16)
  x[3] = 0
  if d >= 8:
    # the hand cases of tests/test_oracle_golden.py (truncation, x * (1/scale) against x / scale) in two rows
    x[4] = 0
    x[4, :4] = torch.tensor([1.0, 0.703125, 0.99609375, -0.99609375])
    x[6] = 0
    x[6, :3] = torch.tensor([1.5, 1.4921875, 0.75])
  return x


@pytest.mark.parametrize("qdtype", [torch.int8, torch.float8_e4m3fn])
@pytest.mark.parametrize("d,block_k", [(512, 0), (4096, 0), (14336, 0), (2048, 512), (7168, 512), (4096, 256), (7168, 128), (2880, 128), (1000, 512)])
def test_gather_rows_v2_rule_bit_exact(K, qdtype, d, block_k):
  """The quantiser of gmm_v2 (pallas_mosaic_tpu_v2_gmm_kernel.py:533-542): values and scales bit for bit."""
  x = _v2_inputs(d, d + block_k)
  idx = torch.randint(0, x.shape[0], (90,), generator=torch.Generator().manual_seed(5)).to(torch.int32)
  q, s = K.gather_rows(cuda(x), cuda(idx), 1, out_dtype=qdtype, block_k=block_k, rule="v2")
  oq, os_ = O.quantize_lhs_v2(x[idx.long()], qdtype, quant_block=block_k if block_k else d)
  assert torch.equal(s.cpu().reshape(os_.shape), os_)
  assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))
  if qdtype == torch.int8 and block_k == 0:
    rows = q.cpu()[(idx == 4).nonzero().flatten()]
    assert all(r[:4].tolist() == [127, 89, 126, -126] for r in rows)  # truncation, not rounding
    rows = q.cpu()[(idx == 6).nonzero().flatten()]
    assert all(r[:3].tolist() == [127, 126, 63] for r in rows)  # bf16 arithmetic, reciprocal multiply


@pytest.mark.parametrize("qdtype,method", [(torch.float8_e4m3fn, "fixed,-224,224"), (torch.int8, "fixed,3"), (torch.int8, "fixed,-1,1"),
                                           (torch.float8_e4m3fn, "fixed,100")])
def test_gather_rows_static_scale_bit_exact(K, qdtype, method):
  """Per-tensor static activation scale (v2 kernel :528-531; get_static_scale, layers/quantizations.py:928-958)."""
  from maxtext_amd import quantizations

  x = _v2_inputs(2048, 77)
  qmax = O.qdtype_max(qdtype)
  st = quantizations.get_static_scale(qmax, method)
  assert st == O.get_static_scale(qmax, method)
  q, s = K.gather_rows(cuda(x), None, 1, out_dtype=qdtype, rule="v2", static_scale=torch.tensor([st], dtype=torch.float32, device="cuda"))
  oq, os_ = O.quantize_lhs_v2(x, qdtype, static_scale=st)
  assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8))
  assert float(s) == float(np.float32(st))  # the caller's scale comes back; the kernel multiplies by bf16(1 / bf16(scale))


def test_gather_rows_out_of_range_index_gives_zero_row(K):
  x = torch.randn(8, 64).to(torch.bfloat16)
  idx = torch.tensor([0, 7, 8, -1, 100000, 3], dtype=torch.int32)
  got = K.gather_rows(cuda(x), cuda(idx), 1).cpu()
  assert torch.equal(got[[0, 1, 5]], x[[0, 7, 3]]) and got[[2, 3, 4]].abs().max() == 0
  with pytest.raises(ValueError):
    K.gather_rows(cuda(x), None, 1, out_dtype=torch.float8_e4m3fn, block_k=64)


@pytest.mark.parametrize("t,k,d", [(1, 2, 512), (300, 2, 4096), (64, 8, 7168), (100, 4, 2880), (33, 9, 64)])
def test_unpermute_combine(K, t, k, d):
  rng = np.random.default_rng(t + d)
  e = 16
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  y = torch.randn(t * k, d, generator=torch.Generator().manual_seed(t)).to(torch.bfloat16)
  w = rng.random((t, k)).astype(np.float32)
  perm, inv, _, _ = K.sort_by_expert(cuda(sel), e)
  want = O.unpermute(y, perm.cpu().numpy(), w, k)
  got = K.unpermute_combine(cuda(y), cuda(w), k=k, inv_perm=inv)
  assert relerr(got, want) <= 2.0**-8
  got2 = K.unpermute_combine(cuda(y), cuda(w), k=k, perm=perm)  # inverse rebuilt from perm
  assert torch.equal(got, got2)
  # unweighted sum (sort_activations.py:98-121)
  got3 = K.unpermute_combine(cuda(y), None, k=k, inv_perm=inv)
  assert relerr(got3, O.unroute_sum(y.float(), sel)) <= 2.0**-8


def test_gather_rows_weighted_and_ranged(K):
  """The weighted ragged gather (ragged_gather.py:310-320) and its [start, end) window, bit for bit."""
  g = torch.Generator().manual_seed(12)
  r_in, r_out, d = 300, 700, 1024
  x = torch.randn(r_in, d, generator=g).to(torch.bfloat16)
  x[5] = float("nan")
  idx = torch.randint(0, r_in, (r_out,), generator=g).to(torch.int32)
  idx[10], idx[650] = 5, 5  # the NaN row: once inside the window, once outside
  w = torch.rand(r_out, generator=g).to(torch.bfloat16)
  def same_bits(a, b):  # NaN payloads are not part of the contract: NaN where NaN is expected, identical bits elsewhere
    return torch.equal(torch.isnan(a), torch.isnan(b)) and torch.equal(torch.nan_to_num(a).view(torch.int16), torch.nan_to_num(b).view(torch.int16))

  want = O.ragged_gather(x, idx.numpy(), weights=w)
  got = K.gather_rows(cuda(x), cuda(idx), 1, row_weight=cuda(w.float())).cpu()
  assert got.dtype == torch.bfloat16 and same_bits(got, want)
  rng_ = torch.tensor([9, 600], dtype=torch.int32)
  want = O.ragged_gather(x, idx.numpy(), 9, 600, weights=w)
  got = K.gather_rows(cuda(x), cuda(idx), 1, row_weight=cuda(w.float()), row_range=cuda(rng_)).cpu()
  assert same_bits(got, want)
  assert got[:9].abs().max() == 0 and got[600:].abs().max() == 0 and torch.isnan(got[10]).all()
  # the window applies before quantisation too: rows outside it quantise to zeros with a zero scale
  q, sc = K.gather_rows(cuda(x), cuda(idx), 1, out_dtype=torch.int8, row_range=cuda(rng_))
  assert q[600:].abs().max() == 0 and sc[600:].abs().max() == 0


@pytest.mark.parametrize("t,k,d", [(64, 8, 512), (300, 2, 4096), (33, 9, 64)])
def test_combine_valid_rows_mask(K, t, k, d):
  """Gather-reduce with a mask of valid rows (ragged_gather_reduce_v2.py:170-182): masked rows are left out whatever
  they hold; integer data keeps the f32 sums exact."""
  rng = np.random.default_rng(t * k)
  e = 16
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  y = torch.from_numpy(rng.integers(-8, 9, (t * k, d)).astype(np.float32)).to(torch.bfloat16)
  w = rng.integers(0, 3, (t, k)).astype(np.float32)
  mask = rng.random((t, k)) < 0.7
  mask[0] = False  # a token with no valid row at all
  perm, inv, _, _ = K.sort_by_expert(cuda(sel), e)
  inv_h = inv.cpu().numpy()
  y[inv_h[~mask.reshape(-1)]] = float("nan")  # every masked row holds NaN
  want = O.ragged_gather_reduce(y, inv_h, torch.from_numpy(w).reshape(-1), mask.reshape(-1), k)
  got = K.unpermute_combine(cuda(y), cuda(w), k=k, inv_perm=inv, valid_rows_mask=cuda(torch.from_numpy(mask)))
  assert torch.equal(got.cpu(), want) and got[0].abs().max() == 0
  # gradient: masked rows get zeros, the others w * dout; dweights of masked entries are zero
  dout = torch.from_numpy(rng.integers(-4, 5, (t, d)).astype(np.float32)).to(torch.bfloat16)
  dy, dw = K.unpermute_combine_bwd(cuda(dout), cuda(y), cuda(w), k=k, inv_perm=inv, valid_rows_mask=cuda(torch.from_numpy(mask)))
  rows = torch.from_numpy(inv_h.astype(np.int64))
  want_dy = torch.zeros(t * k, d)
  want_dy[rows] = (torch.from_numpy(w * mask).reshape(-1, 1) * dout.float().repeat_interleave(k, 0))
  assert torch.equal(dy.cpu().float(), want_dy)
  y0 = torch.nan_to_num(y.float(), nan=0.0)
  want_dw = (y0[rows].reshape(t, k, d) * dout.float()[:, None, :]).sum(-1) * torch.from_numpy(mask)
  assert torch.equal(dw.cpu(), want_dw)


def test_gmm_weight_before_wo(K):
  """The batch-split rule (deepseek_batchsplit_fp8.py:1048-1049): the routing weight multiplies the finished bf16
  activation inside the first matmul's epilogue; against the oracle's gmm + weighted_intermediate."""
  g = torch.Generator().manual_seed(8)
  m, k, n = 640, 512, 384
  gs = np.array([300, 0, 211, 100], np.int32)  # 29 rows in no group
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w0 = (torch.randn(4, n, k, generator=g) * 0.05).to(torch.bfloat16)
  w1 = (torch.randn(4, n, k, generator=g) * 0.05).to(torch.bfloat16)
  rw = (torch.rand(m, generator=g) * 2.5).to(torch.bfloat16)
  h0 = O.gmm(lhs, w0.transpose(1, 2), gs, out_dtype=torch.bfloat16)
  h1 = O.gmm(lhs, w1.transpose(1, 2), gs, out_dtype=torch.bfloat16)
  want = O.weighted_intermediate(h0, h1, rw)
  got = K.gmm_raw(cuda(lhs), cuda(w0), cuda(gs), rhs_up=cuda(w1), act="silu", out_row_scale=cuda(rw.float()))
  assert relerr(got, want) <= TOL
  plain = K.gmm_raw(cuda(lhs), cuda(w0), cuda(gs), rhs_up=cuda(w1), act="silu")
  assert torch.equal(got, (plain.float() * cuda(rw.float())[:, None]).to(torch.bfloat16))


def test_combine_exact_on_integers(K):
  # integer-valued bf16 inputs make the f32 accumulation exact (trick of tests/gather_reduce_sc_test.py:68)
  rng = np.random.default_rng(0)
  t, k, d, e = 200, 8, 256, 64
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  y = torch.from_numpy(rng.integers(-8, 9, (t * k, d)).astype(np.float32)).to(torch.bfloat16)
  w = rng.integers(0, 3, (t, k)).astype(np.float32)
  perm, inv, _, _ = K.sort_by_expert(cuda(sel), e)
  got = K.unpermute_combine(cuda(y), cuda(w), k=k, inv_perm=inv)
  assert torch.equal(got.cpu(), O.unpermute(y, perm.cpu().numpy(), w, k))


def test_transpose_rhs(K):
  w = torch.randint(-128, 128, (3, 200, 136), dtype=torch.int8)
  assert torch.equal(K.transpose_rhs(cuda(w)).cpu(), w.transpose(1, 2).contiguous())
  for shape in ((2, 208, 144), (3, 128, 128), (1, 16, 16), (2, 1040, 400), (2, 128, 2064)):  # 1-byte, 16-byte path, ragged 128 x 128 tiles
    w8 = torch.randint(-128, 128, shape, dtype=torch.int8)
    assert torch.equal(K.transpose_rhs(cuda(w8)).cpu(), w8.transpose(1, 2).contiguous()), shape
    f8 = torch.randn(*shape).to(torch.float8_e4m3fn)
    assert torch.equal(K.transpose_rhs(cuda(f8)).cpu().view(torch.uint8), f8.transpose(1, 2).contiguous().view(torch.uint8)), shape
  wb = torch.randn(2, 70, 264).to(torch.bfloat16)  # K % 8 != 0: element-wise kernel
  assert torch.equal(K.transpose_rhs(cuda(wb)).cpu(), wb.transpose(1, 2).contiguous())
  for shape in ((2, 72, 264), (3, 128, 64), (1, 200, 136), (2, 8, 8), (1, 1024, 520)):  # 16-byte path, ragged tiles
    wb = torch.randn(*shape).to(torch.bfloat16)
    assert torch.equal(K.transpose_rhs(cuda(wb)).cpu(), wb.transpose(1, 2).contiguous()), shape


# ---------------------------------------------------------------- grouped matmul

# (M, K, N, group_sizes): small-tile (rows/expert < 128) and big-tile (>= 128) dispatch, empty groups,
# ragged boundaries, rows past the sum, K and N that are not multiples of the tile.
GMM_SHAPES = [
    (300, 256, 128, [7, 0, 120, 1, 100, 60]),
    (64, 512, 264, [64]),
    (1024, 320, 200, [300, 0, 500, 200]),
    (1500, 1024, 512, [256, 257, 255, 700]),
    (520, 2880, 96, [500, 20]),
    (1010, 256, 264, [300, 20, 0, 130, 250, 40, 160, 100, 0, 10]),  # 128-row tiles, groups of one to three tiles
    (400, 256, 264, [90, 0, 30, 45, 17, 60, 33, 50, 75]),  # 44 rows per group: group-128 int4 streams with up to six 16-row tiles per group
]


def _gmm_inputs(m, k, n, gs, seed):
  g = torch.Generator().manual_seed(seed)
  e = len(gs)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = torch.randn(e, k, n, generator=g) * 0.05  # [g, k, n] f32
  w_up = torch.randn(e, k, n, generator=g) * 0.05
  return lhs, w, w_up, np.asarray(gs, np.int32)


def native(w_gkn):
  return w_gkn.transpose(1, 2).contiguous()


@pytest.mark.parametrize("m,k,n,gs", GMM_SHAPES)
def test_gmm_bf16(K, m, k, n, gs):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 1)
  wb, ub = w.to(torch.bfloat16), w_up.to(torch.bfloat16)
  got = K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs))
  want = O.gmm(lhs, wb, gs)
  assert relerr(got, want) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  got = K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), rhs_up=cuda(native(ub)), act="silu")
  want = O.apply_ffn_activation(O.gmm(lhs, wb, gs, out_dtype=torch.float32), O.gmm(lhs, ub, gs, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


RHS_KN_SHAPES = [
    (1065, 192, 3328, [300, 0, 700, 65]),  # three k stages, an empty group, ragged m-tiles
    (2100, 1024, 2560, [1000, 500, 436, 64]),  # 100 rows belong to no group
]


@pytest.mark.parametrize("m,k,n,gs", RHS_KN_SHAPES)
def test_gmm_bf16_rhs_kn(K, m, k, n, gs):
  """[G, K, N] weights (the reference's default layout, ops.py:47-52) read as they are against the oracle and against
  the same product on re-laid-out [G, N, K] weights, whole and through a window of local groups."""
  lhs, w, _, gs = _gmm_inputs(m, k, n, gs, 1)
  wb = w.to(torch.bfloat16)
  assert K.gmm_rhs_kn_supported(m, k, n, len(gs))
  got = K.gmm_raw(cuda(lhs), cuda(wb), cuda(gs), rhs_kn=True)
  want = O.gmm(lhs, wb, gs)
  assert relerr(got, want) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  assert torch.equal(got, K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs)))  # the same k order in both kernels
  win = K.gmm_raw(cuda(lhs), cuda(wb[1:3].contiguous()), cuda(gs), rhs_kn=True, group_offset=1)
  lo, hi = int(gs[0]), int(gs[:3].sum())
  assert torch.equal(win[lo:hi], got[lo:hi]) and torch.all(win[:lo] == 0) and torch.all(win[hi:] == 0)


def test_gmm_rhs_kn_rejects_other_shapes_and_formats(K):
  gs = torch.tensor([64, 64], dtype=torch.int32, device="cuda")
  lhs = torch.zeros(128, 64, dtype=torch.bfloat16, device="cuda")
  assert not K.gmm_rhs_kn_supported(128, 64, 256, 2)  # too few rows per group
  assert not K.gmm_rhs_kn_supported(4096, 96, 4096, 2) and not K.gmm_rhs_kn_supported(4096, 128, 4224, 2)
  with pytest.raises(RuntimeError, match="moe_gmm_rhs_kn_supported"):
    K.gmm_raw(lhs, torch.zeros(2, 64, 256, dtype=torch.bfloat16, device="cuda"), gs, rhs_kn=True)
  big = torch.zeros(4096, 128, dtype=torch.int8, device="cuda")
  gs2 = torch.tensor([2048, 2048], dtype=torch.int32, device="cuda")
  with pytest.raises(RuntimeError, match="moe_gmm_rhs_kn_supported"):
    K.gmm_raw(big, torch.zeros(2, 128, 4096, dtype=torch.int8, device="cuda"), gs2, rhs_kn=True,
              lhs_scale=torch.ones(4096, device="cuda"), rhs_scale=torch.ones(2, 4096, device="cuda"))


@pytest.mark.parametrize("m,k,n,gs", GMM_SHAPES)
def test_gmm_int8_weight_only(K, m, k, n, gs):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 2)
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  got = K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s))
  want = O.gmm(lhs, q, gs, rhs_scale=s)
  assert relerr(got, want) <= TOL
  got = K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su), act="silu")
  want = O.apply_ffn_activation(O.gmm(lhs, q, gs, rhs_scale=s, out_dtype=torch.float32), O.gmm(lhs, qu, gs, rhs_scale=su, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


@pytest.mark.parametrize("m,k,n,gs", GMM_SHAPES)
def test_gmm_int8_int8(K, m, k, n, gs):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 3)
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  lq, ls = O.quantize_rows_int8(lhs)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s))
  want = O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s)
  assert relerr(got, want) <= TOL
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s), rhs_up=cuda(native(qu)),
                  rhs_up_scale=cuda(su), act="silu")
  want = O.apply_ffn_activation(O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s, out_dtype=torch.float32),
                                O.gmm(lq, qu, gs, lhs_scale=ls, rhs_scale=su, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


@pytest.mark.parametrize("m,k,n,gs", [(40, 1024, 128, [7, 0, 12, 1, 20]), (90, 3584, 328, [10, 25, 1, 16, 17, 9, 12]), (420, 512, 256, [1] * 300 + [100]),
                                      (60, 4096, 256, [5, 0, 9, 14, 3, 11, 2, 16]),
                                      # rows past 7168 values: the variant whose activations travel beside the weights
                                      (45, 7680, 136, [7, 0, 12, 1, 20]), (70, 14336, 256, [5, 0, 9, 14, 3, 11, 2, 16, 1]),
                                      # 15 to 28 rows per expert on average: 32-row tiles, two row tiles per weight segment
                                      (100, 2048, 200, [32, 0, 17, 5, 31, 1]), (310, 1024, 128, [25] * 12), (130, 8192, 264, [33, 20, 64, 1, 0]),
                                      # 25 to 48: 64-row tiles on segments of two k-blocks
                                      (160, 2048, 200, [64, 0, 17, 5, 63, 1]), (380, 1024, 128, [37] * 10), (200, 512, 256, [40] * 5),
                                      (200, 8192, 264, [65, 30, 64, 1, 0, 30])])
def test_gmm_int8_int8_at_decode_sizes(K, m, k, n, gs):
  """int8 x int8 with per-row x per-channel scales at a handful of rows per expert: the LDS-streamed persistent kernel
  (int32 sums, scales applied once) against the oracle and against the LDS-tiled kernel on the same operands; both
  projections with an activation, biases, partial sums, f32 output and rows read through an index."""
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 33)
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  lq, ls = O.quantize_rows_int8(lhs)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s))
  assert relerr(got, O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s)) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  other = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s), kernel="tiled")
  assert relerr(got, other.cpu()) <= 4e-3  # the same exact integer sums: at most the scale product's rounding apart, in bf16
  g = torch.Generator().manual_seed(34)
  b0, b1 = torch.randn(len(gs), n, generator=g), torch.randn(len(gs), n, generator=g)
  p0, p1 = (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16), (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su),
                  rhs_bias=cuda(b0), rhs_up_bias=cuda(b1), partial_sum=cuda(p0), partial_sum_up=cuda(p1), act="swigluoai", act_limit=7.0,
                  out_dtype=torch.float32)
  h0 = O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s, rhs_bias=b0[:, None, :], out_dtype=torch.float32) + p0.float()
  h1 = O.gmm(lq, qu, gs, lhs_scale=ls, rhs_scale=su, rhs_bias=b1[:, None, :], out_dtype=torch.float32) + p1.float()
  want = O.apply_ffn_activation(h0, h1, "swigluoai", 7.0, out_dtype=torch.float32)
  want[int(gs.sum()):] = 0
  assert got.dtype == torch.float32 and relerr(got, want) <= TOL
  t_rows = max(m // 3, 1)
  idx = torch.randint(0, t_rows * 3, (m,), generator=g, dtype=torch.int32)
  rows = (idx // 3).long()
  got = K.gmm_raw(cuda(lq[:t_rows]), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls[:t_rows]), rhs_scale=cuda(s), rhs_up=cuda(native(qu)),
                  rhs_up_scale=cuda(su), act="silu", lhs_row_idx=cuda(idx), lhs_row_idx_div=3)
  want = O.apply_ffn_activation(O.gmm(lq[rows], q, gs, lhs_scale=ls[rows], rhs_scale=s, out_dtype=torch.float32),
                                O.gmm(lq[rows], qu, gs, lhs_scale=ls[rows], rhs_scale=su, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


def test_gmm_int8_exact_with_unit_scales(K):
  # integer operands, unit scales, |sum| < 256: the bf16 output must equal the integer product exactly
  g = torch.Generator().manual_seed(4)
  m, k, n = 400, 64, 128
  gs = np.array([100, 0, 300], np.int32)
  lq = torch.randint(-1, 2, (m, k), generator=g, dtype=torch.int8)
  q = torch.randint(-2, 3, (3, k, n), generator=g, dtype=torch.int8)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(torch.ones(m)), rhs_scale=cuda(torch.ones(3, n)))
  want = O.gmm(lq, q, gs, out_dtype=torch.float32)
  assert want.abs().max() < 256
  assert torch.equal(got.float().cpu(), want)


@pytest.mark.parametrize("m,k,n,gs", [(300, 256, 128, [7, 0, 120, 1, 100, 60]), (520, 2880, 96, [500, 20]), (1024, 320 + 64, 200, [300, 0, 500, 200])])
def test_gmm_int4_weight_only(K, m, k, n, gs):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 5)
  q, s = O.quantize_int4_groups(native(w), 128)  # along K: q [g,n,k], scale [g,n,ceil(k/128)]
  qu, su = O.quantize_int4_groups(native(w_up), 128)
  s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
  from maxtext_amd._lib import MOE_INT4
  got = K.gmm_raw(cuda(lhs), cuda(O.pack_int4(q)), cuda(gs), rhs_scale=cuda(s), rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
  rhs_scale_v2 = s.float().permute(0, 2, 1)[:, :, None, :]  # [g, nb, 1, n]
  want = O.gmm(lhs, q.transpose(1, 2), gs, rhs_scale=rhs_scale_v2, quant_block=128)
  assert relerr(got, want) <= TOL
  got = K.gmm_raw(cuda(lhs), cuda(O.pack_int4(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(O.pack_int4(qu)), rhs_up_scale=cuda(su),
                  rhs_dtype=MOE_INT4, rhs_scale_block_k=128, act="silu")
  up_scale_v2 = su.float().permute(0, 2, 1)[:, :, None, :]
  want = O.apply_ffn_activation(O.gmm(lhs, q.transpose(1, 2), gs, rhs_scale=rhs_scale_v2, quant_block=128, out_dtype=torch.float32),
                                O.gmm(lhs, qu.transpose(1, 2), gs, rhs_scale=up_scale_v2, quant_block=128, out_dtype=torch.float32))
  # the LDS-tiled kernel multiplies the dequantised weights rounded to bf16 (what the reference's converter stores,
  # convert_deepseek_family_ckpt.py:56-84); the oracle keeps q * scale exact
  assert relerr(got, want, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL


# few rows per expert: the streaming (decode) kernels for weight-only int8 / int4
DECODE_SHAPES = [
    (40, 256, 128, [7, 0, 12, 1, 20]),       # <= 16 rows per expert on average, one group above 16
    (4, 2880, 2880, [1, 0, 1, 0, 1, 0, 0, 1]),  # a single token, top-4 of 8 experts, ragged last K group
    (200, 512, 200, [30, 25, 60, 5, 40, 20, 20]),  # 17..32 rows per expert on average
    (64, 384, 264, [16, 16, 16, 16]),
]


@pytest.mark.parametrize("m,k,n,gs", DECODE_SHAPES)
def test_gmm_decode_int8_weight_only(K, m, k, n, gs):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 12)
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  got = K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s))
  assert relerr(got, O.gmm(lhs, q, gs, rhs_scale=s)) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  got = K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su), act="silu")
  want = O.apply_ffn_activation(O.gmm(lhs, q, gs, rhs_scale=s, out_dtype=torch.float32), O.gmm(lhs, qu, gs, rhs_scale=su, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL
  # the tiled kernel must agree with the streaming kernel on the same operands
  tiled = K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su), act="silu", kernel="tiled")
  assert relerr(tiled, want) <= TOL


@pytest.mark.parametrize("m,k,n,gs", DECODE_SHAPES)
def test_gmm_decode_int4_weight_only(K, m, k, n, gs):
  from maxtext_amd._lib import MOE_INT4
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 13)
  q, s = O.quantize_int4_groups(native(w), 128)
  qu, su = O.quantize_int4_groups(native(w_up), 128)
  s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
  v2 = lambda sc: sc.float().permute(0, 2, 1)[:, :, None, :]
  got = K.gmm_raw(cuda(lhs), cuda(O.pack_int4(q)), cuda(gs), rhs_scale=cuda(s), rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
  assert relerr(got, O.gmm(lhs, q.transpose(1, 2), gs, rhs_scale=v2(s), quant_block=128)) <= TOL
  got = K.gmm_raw(cuda(lhs), cuda(O.pack_int4(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(O.pack_int4(qu)), rhs_up_scale=cuda(su),
                  rhs_dtype=MOE_INT4, rhs_scale_block_k=128, act="swigluoai")
  want = O.apply_ffn_activation(O.gmm(lhs, q.transpose(1, 2), gs, rhs_scale=v2(s), quant_block=128, out_dtype=torch.float32),
                                O.gmm(lhs, qu.transpose(1, 2), gs, rhs_scale=v2(su), quant_block=128, out_dtype=torch.float32), "swigluoai")
  assert relerr(got, want) <= TOL


WQS_SHAPES = [
    # m, k, n, group sizes, first local group, local groups
    (40, 256, 128, [7, 0, 12, 1, 20], 0, 5),          # one segment of K; four channel groups with SwiGLU (the minimum)
    (150, 1536, 264, [16, 3, 33, 0, 50, 48], 0, 6),    # two segments; a channel tail (264 = 8 x 32 + 8); groups of 1..4 tiles
    (90, 2880, 320, [10, 25, 1, 16, 17, 9, 12], 2, 3),  # three segments with a ragged last k-block; a shard of the experts
    (700, 3072, 160, [40] * 16 + [60], 0, 17),        # many tiles per block: runs that cross tiles; 40 rows per expert
]


@pytest.mark.parametrize("fmt", ["int4", "mxfp4"])
@pytest.mark.parametrize("m,k,n,gs,off,g_local", WQS_SHAPES)
def test_gmm_4bit_lds_streamed_kernel(K, m, k, n, gs, off, g_local, fmt):
  """The persistent decode kernel for group-128 int4 and MXFP4 (weights copied global -> LDS three segments ahead,
  activations resident in registers): both projections with SwiGLU and the plain product, against the oracle and against
  the register-staged streaming kernel on the same operands; per-expert biases, partial sums, f32 output, activation rows
  read through an index, and rows of experts outside the local shard (zeros)."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 23)
  lo, hi = off, off + g_local
  if fmt == "int4":
    q, s = O.quantize_int4_groups(native(w), 128)
    qu, su = O.quantize_int4_groups(native(w_up), 128)
    s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
    v2 = lambda sc: sc.float().permute(0, 2, 1)[:, :, None, :]
    pk, pku = O.pack_int4(q), O.pack_int4(qu)
    kw = dict(rhs_dtype=MOE_INT4, rhs_scale_block_k=128, group_offset=off)
    ogmm = lambda x, up, **o: O.gmm(x, (qu if up else q).transpose(1, 2)[lo:hi], gs, rhs_scale=v2((su if up else s)[lo:hi]), quant_block=128,
                                    group_offset=off, **o)
  else:
    blocks, s = O.quantize_mxfp4(native(w))  # [g, n, k/32, 16], [g, n, k/32]
    ublocks, su = O.quantize_mxfp4(native(w_up))
    deq, udeq = O.dequantize_mxfp4(blocks, s).to(torch.bfloat16), O.dequantize_mxfp4(ublocks, su).to(torch.bfloat16)
    pk, pku = blocks.reshape(len(gs), n, k // 2), ublocks.reshape(len(gs), n, k // 2)
    kw = dict(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32, group_offset=off)
    ogmm = lambda x, up, **o: O.gmm(x, (udeq if up else deq)[lo:hi], gs, transpose_rhs=True, group_offset=off, **o)
  # plain product
  got = K.gmm_raw(cuda(lhs), cuda(pk[lo:hi]), cuda(gs), rhs_scale=cuda(s[lo:hi]), **kw)
  assert relerr(got, ogmm(lhs, False)) <= TOL
  old = K.gmm_raw(cuda(lhs), cuda(pk[lo:hi]), cuda(gs), rhs_scale=cuda(s[lo:hi]), kernel="stream", **kw)
  assert relerr(got, old.cpu()) <= 8e-3  # the same products summed over K in another order: at most one bf16 step of the result
  ends = np.cumsum(gs)
  first, last = (int(ends[lo - 1]) if lo else 0), int(ends[hi - 1])
  assert torch.all(got[:first] == 0) and torch.all(got[last:] == 0)
  # SwiGLU with biases, partial sums and f32 output
  g = torch.Generator().manual_seed(24)
  b0, b1 = torch.randn(len(gs), n, generator=g), torch.randn(len(gs), n, generator=g)
  p0, p1 = (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16), (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16)
  got = K.gmm_raw(cuda(lhs), cuda(pk[lo:hi]), cuda(gs), rhs_scale=cuda(s[lo:hi]), rhs_up=cuda(pku[lo:hi]), rhs_up_scale=cuda(su[lo:hi]),
                  rhs_bias=cuda(b0[lo:hi]), rhs_up_bias=cuda(b1[lo:hi]), partial_sum=cuda(p0), partial_sum_up=cuda(p1), act="swigluoai",
                  act_limit=7.0, out_dtype=torch.float32, **kw)
  h0 = ogmm(lhs, False, rhs_bias=b0[lo:hi, None, :], out_dtype=torch.float32) + p0.float()
  h1 = ogmm(lhs, True, rhs_bias=b1[lo:hi, None, :], out_dtype=torch.float32) + p1.float()
  want = O.apply_ffn_activation(h0, h1, "swigluoai", 7.0, out_dtype=torch.float32)
  want[:first] = 0
  want[last:] = 0
  assert got.dtype == torch.float32 and relerr(got, want) <= TOL
  # the fused permute: m product rows read the rows of a shorter activation matrix through an index
  t_rows = max(m // 3, 1)
  idx = torch.randint(0, t_rows * 3, (m,), generator=g, dtype=torch.int32)
  x = lhs[:t_rows].contiguous()
  got = K.gmm_raw(cuda(x), cuda(pk[lo:hi]), cuda(gs), rhs_scale=cuda(s[lo:hi]), rhs_up=cuda(pku[lo:hi]), rhs_up_scale=cuda(su[lo:hi]),
                  act="silu", lhs_row_idx=cuda(idx), lhs_row_idx_div=3, **kw)
  rows = x[(idx // 3).long()]
  want = O.apply_ffn_activation(ogmm(rows, False, out_dtype=torch.float32), ogmm(rows, True, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


@pytest.mark.parametrize("fmt", ["int4", "mxfp4"])
@pytest.mark.parametrize("regime", ["tiles256", "tiles128"])
def test_gmm_4bit_prefill_hands_short_group_tails_to_the_decode_kernel(K, fmt, regime):
  """4-bit weights at prefill sizes: a group's remainder of at most 48 rows past its 256- (or 128-) row tiles runs as
  16-row tiles on the decode kernel in a second launch, everything else on the persistent kernel.  Remainders on both
  sides of every boundary (0, 1, 16, 17, 48, 49, a full tile less one), an empty group, rows in no group, a shard of
  the experts with the other rows kept; against the oracle, and every row written exactly once."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4
  bm = 256 if regime == "tiles256" else 128
  rem = [0, 1, 16, 17, 48, 49, bm - 1, 5]
  gs = np.asarray([bm * (1 + i % 2) + r for i, r in enumerate(rem)] + [0, 33], np.int32)  # the last group: a tail and nothing else
  if regime == "tiles128":
    gs = np.asarray([(bm if i % 3 == 0 else 0) + r for i, r in enumerate(rem)] + [0, 33, 130, 128], np.int32)  # 50-odd rows per expert
  e = len(gs)
  m, k, n = int(gs.sum()) + 40, 320, 160
  lhs, w, w_up, _ = _gmm_inputs(m, k, n, gs.tolist(), 31)
  if fmt == "int4":
    q, s = O.quantize_int4_groups(native(w), 128)
    qu, su = O.quantize_int4_groups(native(w_up), 128)
    s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
    v2 = lambda sc: sc.float().permute(0, 2, 1)[:, :, None, :]
    pk, pku, kw = O.pack_int4(q), O.pack_int4(qu), dict(rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
    ogmm = lambda up, lo, hi, **o: O.gmm(lhs, (qu if up else q).transpose(1, 2)[lo:hi], gs, rhs_scale=v2((su if up else s)[lo:hi]), quant_block=128, **o)
  else:
    blocks, s = O.quantize_mxfp4(native(w))
    ublocks, su = O.quantize_mxfp4(native(w_up))
    deq, udeq = O.dequantize_mxfp4(blocks, s).to(torch.bfloat16), O.dequantize_mxfp4(ublocks, su).to(torch.bfloat16)
    pk, pku, kw = blocks.reshape(e, n, k // 2), ublocks.reshape(e, n, k // 2), dict(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
    ogmm = lambda up, lo, hi, **o: O.gmm(lhs, (udeq if up else deq)[lo:hi], gs, transpose_rhs=True, **o)
  total = int(gs.sum())
  got = K.gmm_raw(cuda(lhs), cuda(pk), cuda(gs), rhs_scale=cuda(s), **kw)
  assert relerr(got, ogmm(False, 0, e)) <= TOL and torch.all(got[total:] == 0)
  got = K.gmm_raw(cuda(lhs), cuda(pk), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(pku), rhs_up_scale=cuda(su), act="silu", **kw)
  want = O.apply_ffn_activation(ogmm(False, 0, e, out_dtype=torch.float32), ogmm(True, 0, e, out_dtype=torch.float32))
  # (the persistent kernel multiplies int4 weights dequantised to bf16, as the reference's converter stores them; the oracle
  # keeps q * scale exact: the chained tolerance of test_gmm_int4_weight_only)
  assert relerr(got, want, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL
  # experts 2 .. 6 only, into a buffer whose other rows stay as they are
  lo, hi = 2, 7
  ends = np.cumsum(gs)
  first, last = int(ends[lo - 1]), int(ends[hi - 1])
  buf = torch.full((m, n), 3.0, dtype=torch.bfloat16, device="cuda")
  K.gmm_raw(cuda(lhs), cuda(pk[lo:hi]), cuda(gs), rhs_scale=cuda(s[lo:hi]), group_offset=lo, out=buf, keep_other_rows=True, **kw)
  assert torch.all(buf[:first] == 3.0) and torch.all(buf[last:] == 3.0)
  assert relerr(buf[first:last], ogmm(False, lo, hi, group_offset=lo)[first:last]) <= TOL


FP8_SHAPES = [
    (40, 256, 128, [7, 0, 12, 1, 20]),
    (256, 1024, 384, [8] * 32),
    (200, 512, 200, [100, 60, 40]),
    (300, 384, 256, [5, 290]),
    (1500, 640, 456, [700, 0, 333, 300, 1, 166]),
]


# 0: the kernel the library picks for the shape; 1: streaming kernel; 2 / 3: LDS-tiled kernels with 128 x 128 / 256 x 256 tiles
@pytest.mark.parametrize("variant", [0, 1, 2, 3])
@pytest.mark.parametrize("m,k,n,gs", FP8_SHAPES)
def test_gmm_fp8_block_scaled(K, m, k, n, gs, variant):
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 6)
  aq, asc = O.quantize_fp8_blocks(lhs, 1, 128)
  wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)  # [g, n, k], scale [g, n/128, k/128]
  uq, usc = O.quantize_fp8_blocks(native(w_up), 128, 128)

  def v2(sc):  # -> [g, nb, 1, n]
    return torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]

  got = K.gmm_raw(cuda(aq), cuda(wq), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc), lhs_scale_block_k=128,
                  rhs_scale_block_n=128, rhs_scale_block_k=128, kernel=FP8_KERNELS[variant])
  want = O.gmm(aq, wq, gs, lhs_scale=asc, rhs_scale=v2(wsc), transpose_rhs=True, quant_block=128)
  assert relerr(got, want) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  got = K.gmm_raw(cuda(aq), cuda(wq), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc), rhs_up=cuda(uq), rhs_up_scale=cuda(usc),
                  lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128, act="silu", kernel=FP8_KERNELS[variant])
  want = O.apply_ffn_activation(
      O.gmm(aq, wq, gs, lhs_scale=asc, rhs_scale=v2(wsc), transpose_rhs=True, quant_block=128, out_dtype=torch.float32),
      O.gmm(aq, uq, gs, lhs_scale=asc, rhs_scale=v2(usc), transpose_rhs=True, quant_block=128, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


F8D_SHAPES = [
    # m, k, n, group sizes, first local group, local groups (the library takes this kernel up to 14 rows per group on average)
    (40, 1024, 128, [7, 0, 12, 1, 20], 0, 5),            # two segments of K; four channel groups with SwiGLU (the minimum)
    (30, 512, 256, [3, 16, 0, 11], 0, 4),                # one segment: the scales of four items in flight
    (80, 2048, 264, [16, 3, 33, 0, 2, 17], 0, 6),        # four segments; a channel tail (264 = 8 x 32 + 8); groups of 1..3 tiles
    (90, 7168, 320, [10, 25, 1, 16, 17, 9, 12], 2, 3),   # the longest rows the kernel takes; a shard of the experts
    (450, 3584, 160, [12] * 32 + [52], 0, 33),           # an odd number of segments; many tiles per block: runs that cross tiles
    # a last expert of several tiles where a tile is about one block's share of the work (the shared expert of a
    # DeepSeek layer): its tiles go one each to blocks of one XCD, the other blocks split the rest
    (420, 1024, 192, [1] * 300 + [100], 0, 301),
]


@pytest.mark.parametrize("m,k,n,gs,off,g_local", F8D_SHAPES)
def test_gmm_fp8_lds_streamed_decode_kernel(K, m, k, n, gs, off, g_local):
  """The persistent decode kernel for block-scaled fp8 (e4m3 activations with 1 x 128 scales, e4m3 weights with 128 x 128
  scales; weights copied global -> LDS three segments ahead, activations resident in registers): both projections with
  SwiGLU and the plain product, against the oracle and against the register-staged streaming kernel on the same
  operands; per-expert biases, partial sums, f32 output, activation rows read through an index, and rows of experts
  outside the local shard (zeros)."""
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 29)
  lo, hi = off, off + g_local
  aq, asc = O.quantize_fp8_blocks(lhs, 1, 128)
  wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)  # [g, n, k], scale [g, n/128, k/128]
  uq, usc = O.quantize_fp8_blocks(native(w_up), 128, 128)
  v2 = lambda sc: torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]  # -> [g, nb, 1, n]
  kw = dict(lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128, group_offset=off)
  ogmm = lambda x, xs, up, **o: O.gmm(x, (uq if up else wq)[lo:hi], gs, lhs_scale=xs, rhs_scale=v2((usc if up else wsc)[lo:hi]), transpose_rhs=True,
                                      quant_block=128, group_offset=off, **o)
  # plain product
  got = K.gmm_raw(cuda(aq), cuda(wq[lo:hi]), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc[lo:hi]), **kw)
  assert relerr(got, ogmm(aq, asc, False)) <= TOL
  old = K.gmm_raw(cuda(aq), cuda(wq[lo:hi]), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc[lo:hi]), kernel="stream", **kw)
  assert relerr(got, old.cpu()) <= 8e-3  # the same products summed over K in another order: at most one bf16 step of the result
  ends = np.cumsum(gs)
  first, last = (int(ends[lo - 1]) if lo else 0), int(ends[hi - 1])
  assert torch.all(got[:first] == 0) and torch.all(got[last:] == 0)
  # SwiGLU with biases, partial sums and f32 output
  g = torch.Generator().manual_seed(30)
  b0, b1 = torch.randn(len(gs), n, generator=g), torch.randn(len(gs), n, generator=g)
  p0, p1 = (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16), (torch.randn(m, n, generator=g) * 0.5).to(torch.bfloat16)
  got = K.gmm_raw(cuda(aq), cuda(wq[lo:hi]), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc[lo:hi]), rhs_up=cuda(uq[lo:hi]),
                  rhs_up_scale=cuda(usc[lo:hi]), rhs_bias=cuda(b0[lo:hi]), rhs_up_bias=cuda(b1[lo:hi]), partial_sum=cuda(p0), partial_sum_up=cuda(p1),
                  act="swigluoai", act_limit=7.0, out_dtype=torch.float32, **kw)
  h0 = ogmm(aq, asc, False, rhs_bias=b0[lo:hi, None, :], out_dtype=torch.float32) + p0.float()
  h1 = ogmm(aq, asc, True, rhs_bias=b1[lo:hi, None, :], out_dtype=torch.float32) + p1.float()
  want = O.apply_ffn_activation(h0, h1, "swigluoai", 7.0, out_dtype=torch.float32)
  want[:first] = 0
  want[last:] = 0
  assert got.dtype == torch.float32 and relerr(got, want) <= TOL
  same = K.gmm_raw(cuda(aq), cuda(wq[lo:hi]), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(wsc[lo:hi]), rhs_up=cuda(uq[lo:hi]),
                   rhs_up_scale=cuda(usc[lo:hi]), rhs_bias=cuda(b0[lo:hi]), rhs_up_bias=cuda(b1[lo:hi]), partial_sum=cuda(p0), partial_sum_up=cuda(p1),
                   act="swigluoai", act_limit=7.0, out_dtype=torch.float32, kernel="stream", **kw)
  assert relerr(got, same.cpu()) <= 1e-4  # f32 results of the two kernels: only the order of the K sum differs
  # the fused permute: m product rows read the rows of a shorter activation matrix (and its scales) through an index
  t_rows = max(m // 3, 1)
  idx = torch.randint(0, t_rows * 3, (m,), generator=g, dtype=torch.int32)
  x, xs = aq[:t_rows].contiguous(), asc[:t_rows].contiguous()
  got = K.gmm_raw(cuda(x), cuda(wq[lo:hi]), cuda(gs), lhs_scale=cuda(xs), rhs_scale=cuda(wsc[lo:hi]), rhs_up=cuda(uq[lo:hi]),
                  rhs_up_scale=cuda(usc[lo:hi]), act="silu", lhs_row_idx=cuda(idx), lhs_row_idx_div=3, **kw)
  rows, rscales = x[(idx // 3).long()], xs[(idx // 3).long()]
  want = O.apply_ffn_activation(ogmm(rows, rscales, False, out_dtype=torch.float32), ogmm(rows, rscales, True, out_dtype=torch.float32))
  assert relerr(got, want) <= TOL


def test_gmm_group_offset_and_nan_isolation(K):
  # non-local groups produce zeros (v2 kernel test :939); a NaN row must not leak into other experts' rows (:592)
  lhs, w, _, gs = _gmm_inputs(600, 256, 128, [100, 200, 150, 100], 8)
  wb = w.to(torch.bfloat16)
  got = K.gmm_raw(cuda(lhs), cuda(native(wb[1:3])), cuda(gs), group_offset=1)
  want = O.gmm(lhs, wb[1:3], gs, group_offset=1)
  assert relerr(got, want) <= TOL
  assert torch.all(got[:100] == 0) and torch.all(got[450:] == 0)
  lhs_nan = lhs.clone()
  lhs_nan[100:300] = float("nan")
  clean = K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs))
  dirty = K.gmm_raw(cuda(lhs_nan), cuda(native(wb)), cuda(gs))
  assert torch.equal(clean[:100], dirty[:100]) and torch.equal(clean[300:], dirty[300:])
  assert torch.isnan(dirty[100:300].float()).all()


def test_gmm_argument_errors(K):
  lhs = torch.zeros(16, 64, dtype=torch.bfloat16).cuda()
  rhs = torch.zeros(2, 24, 64, dtype=torch.bfloat16).cuda()
  gs = torch.tensor([8, 8], dtype=torch.int32).cuda()
  with pytest.raises(RuntimeError):
    K.gmm_raw(lhs, rhs[:, :20].contiguous(), gs)  # N % 8 != 0
  with pytest.raises(RuntimeError):
    K.gmm_raw(lhs, rhs, gs, act="silu")  # activation without rhs_up
  with pytest.raises(ValueError):
    K.gmm_raw(lhs.cpu(), rhs, gs)


# ---------------------------------------------------------------- backward: tgmm, dlhs, autograd

TGMM_SHAPES = [
    (300, 128, 128, [100, 0, 150, 50]),
    (1000, 256, 384, [1, 31, 32, 33, 400, 0, 503]),
    (520, 200, 72, [500, 20]),  # K, N not multiples of the 128 tile
    (64, 2880, 96, [7, 57]),
    (700, 128, 256, [300, 200]),  # rows past sum(group_sizes) belong to no group
    # 256 x 256 tiles on the direct-to-LDS pipeline (K, N multiples of 256, 128 rows per group on average, 128 tiles):
    (1065, 1024, 2048, [300, 0, 700, 65]),  # ragged last stages (44 and 1 rows), an empty group
    (2100, 512, 4096, [1000, 500, 436, 64]),  # a group of exactly one stage; 100 rows belong to no group
]


@pytest.mark.parametrize("m,k,n,gs", TGMM_SHAPES)
@pytest.mark.parametrize("out_dtype", [torch.bfloat16, torch.float32])
def test_tgmm(K, m, k, n, gs, out_dtype):
  g = torch.Generator().manual_seed(5)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  gs = np.asarray(gs, np.int32)
  got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=out_dtype)  # [G, N, K]
  want = O.tgmm(lhs, dout, gs, out_dtype=out_dtype).transpose(1, 2)
  assert got.shape == want.shape and got.dtype == out_dtype
  assert relerr(got, want) <= TOL
  for i, sz in enumerate(gs):
    if sz == 0:
      assert torch.all(got[i] == 0)
    else:  # per-group bound too, so a small group next to a big one is not hidden by the global max
      assert relerr(got[i], want[i]) <= TOL


def test_tgmm_exact_on_small_integers_and_group_window(K):
  rng = np.random.default_rng(3)
  m, k, n = 333, 136, 264
  gs = np.array([40, 0, 100, 93, 100], np.int32)
  lhs = torch.from_numpy(rng.integers(-3, 4, (m, k)).astype(np.float32)).to(torch.bfloat16)
  dout = torch.from_numpy(rng.integers(-3, 4, (m, n)).astype(np.float32)).to(torch.bfloat16)
  want = O.tgmm(lhs, dout, gs, out_dtype=torch.float32).transpose(1, 2)
  got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.float32)
  assert torch.equal(got.cpu(), want)  # sums of at most 100 products of magnitude <= 9 are exact in f32
  win = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), num_groups_local=3, group_offset=1, out_dtype=torch.float32)
  assert torch.equal(win.cpu(), want[1:4])
  # NaN rows outside the window must not leak into it
  lhs_nan = lhs.clone()
  lhs_nan[:40] = float("nan")
  win = K.tgmm(cuda(lhs_nan), cuda(dout), cuda(gs), num_groups_local=3, group_offset=1, out_dtype=torch.float32)
  assert torch.equal(win.cpu(), want[1:4])


def test_tgmm_big_tiles_exact_on_small_integers_and_group_window(K):
  """The same on a shape that takes the 256 x 256 kernel, whose rows past a group's end come from a row of zeros."""
  rng = np.random.default_rng(4)
  m, k, n = 700, 1024, 3072
  gs = np.array([140, 0, 199, 193, 100], np.int32)  # 68 rows belong to no group
  lhs = torch.from_numpy(rng.integers(-3, 4, (m, k)).astype(np.float32)).to(torch.bfloat16)
  dout = torch.from_numpy(rng.integers(-3, 4, (m, n)).astype(np.float32)).to(torch.bfloat16)
  want = O.tgmm(lhs, dout, gs, out_dtype=torch.float32).transpose(1, 2)
  got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.float32)
  assert torch.equal(got.cpu(), want)  # sums of at most 199 products of magnitude <= 9 are exact in f32
  lhs_nan = lhs.clone()
  lhs_nan[:140] = float("nan")
  lhs_nan[632:] = float("nan")
  win = K.tgmm(cuda(lhs_nan), cuda(dout), cuda(gs), num_groups_local=3, group_offset=1, out_dtype=torch.float32)
  assert torch.equal(win.cpu(), want[1:4])  # NaN rows of other groups and of no group do not leak into the window
  got16 = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.bfloat16)
  assert torch.equal(got16.cpu(), want.to(torch.bfloat16))


@pytest.mark.parametrize("m,k,n,gs", [(333, 136, 264, [40, 0, 100, 93, 100]), (700, 1024, 3072, [140, 0, 199, 193, 100])])
@pytest.mark.parametrize("existing_dtype,out_dtype", [(torch.float32, torch.float32), (torch.bfloat16, torch.bfloat16), (torch.bfloat16, torch.float32)])
def test_tgmm_existing_out_is_added_before_rounding(K, m, k, n, gs, existing_dtype, out_dtype):
  """existing_out joins the f32 accumulator (backend.py:733-734), also for groups without rows, also when it is the
  output buffer's own dtype; integer data keeps every sum exact, so the comparison is bit for bit."""
  from maxtext_amd import megablox

  rng = np.random.default_rng(31)
  gs = np.array(gs, np.int32)
  lhs = torch.from_numpy(rng.integers(-3, 4, (m, k)).astype(np.float32)).to(torch.bfloat16)
  dout = torch.from_numpy(rng.integers(-3, 4, (m, n)).astype(np.float32)).to(torch.bfloat16)
  # halves make the bf16 output round: rounding the products first and adding afterwards would give other bits
  existing = torch.from_numpy(rng.integers(-9, 10, (3, k, n)).astype(np.float32) * 0.5).to(existing_dtype)
  want = O.tgmm(lhs, dout, gs, num_actual_groups=3, group_offset=1, out_dtype=out_dtype, existing_out=existing)
  got = megablox.tgmm(cuda(lhs).t(), cuda(dout), cuda(gs), preferred_element_type=out_dtype, group_offset=1, num_actual_groups=3,
                      existing_out=cuda(existing))
  assert got.shape == want.shape and got.dtype == out_dtype
  assert torch.equal(got.cpu(), want)
  assert torch.equal(got[0].cpu(), existing[0].to(out_dtype))  # group 1 has no rows: its slice is existing_out alone
  # accumulating in place: the kernel's [G, N, K] result of one call is the existing_out of the next
  first = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.float32)
  twice = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.float32, existing_out=first)
  assert torch.equal(twice, 2 * first)
  with pytest.raises(ValueError):
    megablox.tgmm(cuda(lhs).t(), cuda(dout), cuda(gs), existing_out=cuda(existing))  # 3 groups given, 5 expected


@pytest.mark.parametrize("m,k,n,gs", [(333, 136, 264, [40, 0, 100, 93, 100]), (700, 1024, 3072, [140, 0, 199, 193, 100])])
@pytest.mark.parametrize("out_dtype", [torch.float32, torch.bfloat16])
def test_tgmm_row_scale_goes_on_before_existing_out_and_rounding(K, m, k, n, gs, out_dtype):
  """out[g, n, :] = f32 products * out_row_scale[n] (+ existing_out), rounded once (the column scales of an e5m2 gradient,
  ops.py:590-603): integer data keeps the sums exact, odd multiples of 1/8 as scales make the bf16 result round, so
  the comparison with the oracle's unscaled f32 product, scaled and rounded here, is bit for bit."""
  rng = np.random.default_rng(47)
  gs = np.array(gs, np.int32)
  lhs = torch.from_numpy(rng.integers(-3, 4, (m, k)).astype(np.float32)).to(torch.bfloat16)
  dout = torch.from_numpy(rng.integers(-31, 32, (m, n)).astype(np.float32)).to(torch.bfloat16)  # sums beyond bf16's 8 bits
  scale = torch.from_numpy((2 * rng.integers(1, 40, n) + 1).astype(np.float32) / 8)
  existing = torch.from_numpy(rng.integers(-9, 10, (3, n, k)).astype(np.float32) * 0.5)
  plain = O.tgmm(lhs, dout, gs, num_actual_groups=3, group_offset=1, out_dtype=torch.float32).transpose(1, 2)  # [g, n, k] f32, exact
  want = plain * scale.reshape(1, n, 1)
  got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), num_groups_local=3, group_offset=1, out_dtype=out_dtype, out_row_scale=cuda(scale))
  assert got.dtype == out_dtype and torch.equal(got.cpu(), want.to(out_dtype))
  if out_dtype == torch.bfloat16:  # (rounding the products before the scaling would give other bits)
    assert not torch.equal(want.to(out_dtype), (plain.to(out_dtype) * scale.reshape(1, n, 1)).to(out_dtype))
  got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), num_groups_local=3, group_offset=1, out_dtype=out_dtype, out_row_scale=cuda(scale),
               existing_out=cuda(existing))
  assert torch.equal(got.cpu(), (want + existing).to(out_dtype))
  with pytest.raises(ValueError):
    K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_row_scale=cuda(scale[:-1]))


def test_tgmm_argument_errors(K):
  a = torch.zeros(16, 64, dtype=torch.bfloat16, device="cuda")
  gs = torch.tensor([16], dtype=torch.int32, device="cuda")
  with pytest.raises(ValueError):
    K.tgmm(a, torch.zeros(8, 64, dtype=torch.bfloat16, device="cuda"), gs)
  with pytest.raises(RuntimeError, match="multiples of 8"):
    K.tgmm(a, torch.zeros(16, 12, dtype=torch.bfloat16, device="cuda"), gs)
  with pytest.raises(TypeError):
    K.tgmm(a.float(), a, gs)


# the second shape is large enough for the 256 x 256 kernels: [g, k, n] weights read as they are (the forward of
# transpose_rhs=False, dlhs of transpose_rhs=True) and the big-tile weight gradient
@pytest.mark.parametrize("m,k,n,gs", [(450, 256, 192, [200, 0, 70, 150]), (1100, 3328, 3328, [500, 0, 170, 400])])
@pytest.mark.parametrize("transpose_rhs", [False, True])
def test_gmm_autograd_matches_torch_autograd(transpose_rhs, m, k, n, gs):
  """dlhs and drhs of megablox.gmm against torch autograd through a per-group f64 matmul (the custom
  VJP of ops.py:438-527: dlhs = gmm(dout, rhs^T), drhs = tgmm(lhs^T, dout))."""
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(9)
  gs = np.array(gs, np.int32)  # 30 trailing rows in no group
  e = len(gs)
  lhs = (torch.randn(m, k, generator=g)).to(torch.bfloat16)
  w = (torch.randn(e, k, n, generator=g) * 0.05).to(torch.bfloat16)  # [g, k, n]
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  lhs64 = lhs.double().requires_grad_()
  w64 = w.double().requires_grad_()
  off = np.concatenate([[0], np.cumsum(gs)])
  ref = torch.cat([lhs64[off[i] : off[i + 1]] @ w64[i] for i in range(e)] + [torch.zeros(m - off[-1], n, dtype=torch.float64)])
  (ref * dout.double()).sum().backward()

  lhs_g = cuda(lhs).requires_grad_()
  rhs_g = cuda(w.transpose(1, 2) if transpose_rhs else w).requires_grad_()
  out = gmm_bf16(lhs_g, rhs_g, cuda(gs), transpose_rhs=transpose_rhs)
  assert relerr(out, ref) <= TOL
  out.backward(cuda(dout))
  assert lhs_g.grad.shape == lhs.shape and rhs_g.grad.shape == rhs_g.shape
  assert relerr(lhs_g.grad, lhs64.grad) <= TOL
  assert torch.all(lhs_g.grad[int(off[-1]) :] == 0)
  want_drhs = w64.grad.transpose(1, 2) if transpose_rhs else w64.grad
  assert relerr(rhs_g.grad, want_drhs) <= TOL
  assert torch.all(rhs_g.grad[1] == 0)


def test_gmm_autograd_through_fused_activation():
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(10)
  m, k, n = 256, 128, 128
  gs = np.array([100, 156], np.int32)
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w0 = (torch.randn(2, n, k, generator=g) * 0.1).to(torch.bfloat16)
  w1 = (torch.randn(2, n, k, generator=g) * 0.1).to(torch.bfloat16)
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  a, b0, b1 = lhs.double().requires_grad_(), w0.double().requires_grad_(), w1.double().requires_grad_()
  off = [0, 100, 256]
  h0 = torch.cat([a[off[i] : off[i + 1]] @ b0[i].T for i in range(2)])
  h1 = torch.cat([a[off[i] : off[i + 1]] @ b1[i].T for i in range(2)])
  (torch.nn.functional.silu(h0) * h1 * dout.double()).sum().backward()
  la, r0, r1 = cuda(lhs).requires_grad_(), cuda(w0).requires_grad_(), cuda(w1).requires_grad_()
  out = gmm_bf16(la, r0, cuda(gs), transpose_rhs=True, rhs_up=r1, fuse_act="silu")
  out.backward(cuda(dout))
  # bf16 intermediates (h0, h1 and their gradients are rounded to bf16) -> 2e-2 on the gradients
  assert relerr(la.grad, a.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(r0.grad, b0.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(r1.grad, b1.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2


@pytest.mark.parametrize("quant", [None, "int8", "fp8"])
@pytest.mark.parametrize("with_inverse", [True, False])
def test_gmm_autograd_with_row_index(quant, with_inverse):
  """The fused permute under grad: lhs holds the T token rows, row i of the product reads row perm[i] // k.  dlhs is the sum
  of each token's k row gradients (a deterministic sum through the inverse permutation, or a scatter-add when the index
  is not a permutation), drhs reads the rows through the index again; against torch autograd in f64 (unquantised) or the
  same call on the gathered copy (quantised forward with its quantised backward)."""
  from maxtext_amd import megablox
  from maxtext_amd.quantizations import QtRule

  g = torch.Generator().manual_seed(15)
  t, k, kd, n = 300, 2, 256, 192
  m = t * k
  gs = np.array([250, 0, 200, 120], np.int32)  # 30 trailing rows in no group
  x = torch.randn(t, kd, generator=g).to(torch.bfloat16)
  w = (torch.randn(4, kd, n, generator=g) * 0.05).to(torch.bfloat16)
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  if with_inverse:
    perm = torch.randperm(m, generator=g).to(torch.int32)
    inv = torch.empty_like(perm)
    inv[perm.long()] = torch.arange(m, dtype=torch.int32)
  else:
    perm = torch.randint(0, m, (m,), generator=g).to(torch.int32)  # tokens read any number of times
    inv = None
  rows = (perm // k).long()
  kw = {}
  if quant is not None:
    kw = dict(use_qwix_quantization=True, qwix_rule=QtRule(weight_qtype=quant, act_qtype=quant, bwd_qtype="float8_e5m2"))
  xg, wg = cuda(x).requires_grad_(), cuda(w).requires_grad_()
  out = gmm_bf16(xg, wg, cuda(gs), lhs_row_idx=cuda(perm), lhs_row_idx_div=k, lhs_row_inv=None if inv is None else cuda(inv), **kw)
  out.backward(cuda(dout))
  if quant is None:
    x64, w64 = x.double().requires_grad_(), w.double().requires_grad_()
    lhs64 = x64[rows]
    off = np.concatenate([[0], np.cumsum(gs)])
    ref = torch.cat([lhs64[off[i]:off[i + 1]] @ w64[i] for i in range(4)] + [torch.zeros(m - off[-1], n, dtype=torch.float64)])
    (ref * dout.double()).sum().backward()
    assert relerr(out, ref) <= TOL
    assert relerr(xg.grad, x64.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL and relerr(wg.grad, w64.grad) <= TOL
  else:
    # the same products on the gathered copy: per-row quantisation commutes with the gather, so forward and weight
    # gradient are bit-equal and the token gradient is the sum of the copy's row gradients
    x2 = cuda(x).requires_grad_()
    w2 = cuda(w).requires_grad_()
    gathered = x2[cuda(rows)]
    out2 = gmm_bf16(gathered, w2, cuda(gs), **kw)
    assert torch.equal(out, out2)
    out2.backward(cuda(dout))
    assert torch.equal(wg.grad, w2.grad)
    assert relerr(xg.grad, x2.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL


def test_gmm_autograd_partial_sum_existing_out_and_row_scale():
  """The remaining differentiable arguments: partial_sum and existing_out receive the incoming gradient (ops.py:524-527),
  out_row_scale multiplies the finished rows (its gradient is the row's inner product with the incoming gradient)."""
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(16)
  m, kd, n = 420, 128, 136
  gs = np.array([200, 0, 220], np.int32)
  lhs = torch.randn(m, kd, generator=g).to(torch.bfloat16)
  w = (torch.randn(3, kd, n, generator=g) * 0.05).to(torch.bfloat16)
  ps = torch.randn(m, n, generator=g).to(torch.bfloat16)
  scale = torch.rand(m, generator=g) + 0.5
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  a, b, p64, s64 = lhs.double().requires_grad_(), w.double().requires_grad_(), ps.double().requires_grad_(), scale.double().requires_grad_()
  off = [0, 200, 200, 420]
  ref = (torch.cat([a[off[i]:off[i + 1]] @ b[i] for i in range(3)]) + p64) * s64[:, None]
  (ref * dout.double()).sum().backward()
  la, wa, pa, sa = cuda(lhs).requires_grad_(), cuda(w).requires_grad_(), cuda(ps).requires_grad_(), cuda(scale).requires_grad_()
  out = gmm_bf16(la, wa, cuda(gs), partial_sum=pa, out_row_scale=sa)
  assert relerr(out, ref) <= TOL
  out.backward(cuda(dout))
  assert relerr(la.grad, a.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL and relerr(wa.grad, b.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL
  assert relerr(pa.grad, p64.grad) <= TOL and relerr(sa.grad, s64.grad) <= TOL
  # existing_out: two shards of the experts write their rows into one buffer; its gradient is the incoming gradient
  gs5 = np.array([100, 60, 0, 160, 100], np.int32)
  w5 = (torch.randn(5, kd, n, generator=g) * 0.05).to(torch.bfloat16)
  la = cuda(lhs).requires_grad_()
  w_lo, w_hi = cuda(w5[:2]).requires_grad_(), cuda(w5[2:]).requires_grad_()
  buf = torch.zeros((m, n), dtype=torch.bfloat16, device="cuda").requires_grad_()
  first = gmm_bf16(la, w_lo, cuda(gs5), existing_out=buf.clone(), group_offset=0)
  both = gmm_bf16(la, w_hi, cuda(gs5), existing_out=first, group_offset=2)
  both.backward(cuda(dout))
  a, b = lhs.double().requires_grad_(), w5.double().requires_grad_()
  off = np.concatenate([[0], np.cumsum(gs5)])
  ref = torch.cat([a[off[i]:off[i + 1]] @ b[i] for i in range(5)])
  (ref * dout.double()).sum().backward()
  assert relerr(both, ref) <= TOL
  assert relerr(la.grad, a.grad) <= TOL
  assert relerr(torch.cat([w_lo.grad, w_hi.grad]), b.grad) <= TOL
  assert torch.equal(buf.grad, cuda(dout))


# ---------------------------------------------------------------- router: gate matmul + top-k in one call


def _margin_ok(scores, k, eps):
  """Tokens whose k+1 best scores are pairwise separated by more than eps (ties are where a different
  summation order may legitimately pick another expert)."""
  s = np.sort(scores.astype(np.float64), axis=-1)[:, ::-1][:, : k + 1]
  return np.all(s[:, :-1] - s[:, 1:] > eps, axis=-1)


@pytest.mark.parametrize("t,d,e,k", [(2048, 4096, 8, 2), (256, 7168, 256, 8), (3, 7168, 256, 8), (1, 2880 // 64 * 64, 32, 4), (77, 512, 128, 8)])
def test_gate_route_softmax_f32(K, t, d, e, k):
  from maxtext_amd.quantizations import split_gate_kernel

  g = torch.Generator().manual_seed(31)
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  wg = torch.randn(d, e, generator=g) * 0.02
  w, idx, logits, pre = K.gate_route(cuda(x), cuda(split_gate_kernel(wg)), k=k, return_logits=True)
  want_logits, _ = O.gate_logits(x, wg)
  scale = np.abs(want_logits).max()
  assert np.abs(logits.cpu().numpy() - want_logits).max() <= 2e-6 * scale  # f32 products, f32 accumulation over d
  assert torch.equal(pre, logits)
  ow, oidx = O.get_topk(want_logits, k=k)
  ok = _margin_ok(want_logits, k, 1e-5 * scale)
  assert ok.mean() > 0.9
  np.testing.assert_array_equal(idx.cpu().numpy()[ok], oidx[ok])
  np.testing.assert_allclose(w.cpu().numpy()[ok], ow[ok], rtol=2.0**-7, atol=1e-6)
  # and bit-exact against the top-k of the logits the kernel itself produced, ties included
  ow2, oidx2 = O.get_topk(logits.cpu().numpy(), k=k)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx2)
  np.testing.assert_array_equal(w.cpu().numpy(), ow2)


def test_gate_route_exact_on_integers(K):
  """Small-integer activations and gate weights make every partial sum exact in f32, so logits and indices
  must match the oracle bit for bit whatever the summation order (and the mid / lo terms are zero)."""
  from maxtext_amd.quantizations import split_gate_kernel

  rng = np.random.default_rng(7)
  t, d, e, k = 513, 1024, 64, 6
  x = torch.from_numpy(rng.integers(-4, 5, (t, d)).astype(np.float32)).to(torch.bfloat16)
  wg = torch.from_numpy(rng.integers(-8, 9, (d, e)).astype(np.float32)) / 16.0
  terms = split_gate_kernel(wg)
  assert torch.all(terms[1] == 0) and torch.all(terms[2] == 0)
  w, idx, logits, _ = K.gate_route(cuda(x), cuda(terms), k=k, norm_topk_prob=True, return_logits=True)
  want_logits, _ = O.gate_logits(x, wg)
  np.testing.assert_array_equal(logits.cpu().numpy(), want_logits)
  ow, oidx = O.get_topk(want_logits, k=k, norm_topk_prob=True)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)  # integer logits: many exact ties, lower index first
  np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2.0**-6, atol=1e-6)


@pytest.mark.parametrize("groups", [(-1, -1), (8, 4)])
def test_gate_route_deepseek_sigmoid_bias(K, groups):
  from maxtext_amd.quantizations import split_gate_kernel

  g = torch.Generator().manual_seed(33)
  t, d, e, k = 200, 1024, 256, 8
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  wg = torch.randn(d, e, generator=g) * 0.05
  bias = torch.randn(e, generator=g) * 0.1
  w, idx, logits, pre = K.gate_route(cuda(x), cuda(split_gate_kernel(wg)), cuda(bias), k=k, score_func="sigmoid", mode="deepseek",
                                     norm_topk_prob=True, routed_scaling_factor=2.5, n_routing_groups=groups[0],
                                     topk_routing_group=groups[1], return_logits=True)
  want_logits, want_pre = O.gate_logits(x, wg, bias, score_func="sigmoid", deepseek=True)
  assert np.abs(pre.cpu().numpy() - want_pre).max() <= 1e-6
  assert np.abs(logits.cpu().numpy() - want_logits).max() <= 1e-6
  # routing on the kernel's own scores must equal the oracle's routing on the same scores, bit for bit
  ow, oidx = O.get_topk(logits.cpu().numpy(), pre.cpu().numpy(), k=k, mode="deepseek", routed_scaling_factor=2.5,
                        n_routing_groups=groups[0], topk_routing_group=groups[1])
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
  np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=1e-5)


def test_gate_route_sqrtsoftplus(K):
  """The DeepSeek-V4 router's score function sqrt(softplus(x)) (linears.py:51-53) inside moe_gate_route."""
  from maxtext_amd.quantizations import split_gate_kernel

  g = torch.Generator().manual_seed(35)
  t, d, e, k = 300, 1024, 64, 6
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  x[0] *= 40.0  # logits far out on both sides: sqrt(x) above, exp(x / 2) below
  wg = torch.randn(d, e, generator=g) * 0.05
  w, idx, logits, pre = K.gate_route(cuda(x), cuda(split_gate_kernel(wg)), k=k, score_func="sqrtsoftplus", mode="deepseek",
                                     norm_topk_prob=True, routed_scaling_factor=1.5, return_logits=True)
  want_logits, want_pre = O.gate_logits(x, wg, score_func="sqrtsoftplus", deepseek=True)
  np.testing.assert_allclose(pre.cpu().numpy(), want_pre, rtol=2e-5, atol=1e-30)
  assert torch.equal(logits, pre)  # no bias
  ow, oidx = O.get_topk(logits.cpu().numpy(), pre.cpu().numpy(), k=k, mode="deepseek", routed_score_func="sqrtsoftplus",
                        routed_scaling_factor=1.5)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
  np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=1e-5)


def test_gate_route_bf16_gate_and_errors(K):
  from maxtext_amd.quantizations import split_gate_kernel

  g = torch.Generator().manual_seed(34)
  t, d, e, k = 100, 512, 16, 2
  x = torch.randn(t, d, generator=g).to(torch.bfloat16)
  wg = torch.randn(d, e, generator=g) * 0.05
  w, idx, logits, _ = K.gate_route(cuda(x), cuda(split_gate_kernel(wg, 1)), k=k, gate_round_bf16=True, return_logits=True)
  want, _ = O.gate_logits(x, wg, float32_gate_logits=False)
  got = logits.cpu().numpy()
  # f32 accumulation order may move a sum across a bf16 rounding boundary: allow one bf16 ulp on a few values
  assert np.mean(got != want) < 0.02 and np.abs(got - want).max() <= 2.0**-7 * np.abs(want).max()
  with pytest.raises(RuntimeError, match="d % 64"):
    K.gate_route(cuda(x[:, :72].contiguous()), cuda(split_gate_kernel(wg[:72], 1)), k=k)
  with pytest.raises(ValueError):
    K.gate_route(cuda(x), cuda(split_gate_kernel(wg[:256], 1)), k=k)


# ---------------------------------------------------------------- per-expert bias (mlp_bias models)


def _bias(e, n, seed):
  g = torch.Generator().manual_seed(seed)
  return torch.randn(e, n, generator=g) * 0.5, torch.randn(e, n, generator=g) * 0.5


@pytest.mark.parametrize("m,k,n,gs", [GMM_SHAPES[0], GMM_SHAPES[3], DECODE_SHAPES[0], DECODE_SHAPES[2]])
def test_gmm_bias_every_kernel_family(K, m, k, n, gs):
  """rhs_bias / rhs_up_bias through each kernel family: bf16 tiles (small / large), int8 x int8, weight-only int8
  (tiled or streaming by shape), int4, block-scaled fp8.  Bias enters before the activation (moe.py:1952-1981)
  and rows that belong to no group stay zero."""
  from maxtext_amd._lib import MOE_INT4

  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 17)
  e = len(gs)
  b0, b1 = _bias(e, n, 18)
  ob0, ob1 = b0[:, None, :], b1[:, None, :]
  act = lambda h0, h1: O.apply_ffn_activation(h0, h1, "swigluoai")
  used = int(gs.sum())

  def check(got, want):
    assert relerr(got, want) <= TOL
    assert torch.all(got[used:] == 0)

  # bf16 x bf16
  wb, ub = w.to(torch.bfloat16), w_up.to(torch.bfloat16)
  check(K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), rhs_bias=cuda(b0)), O.gmm(lhs, wb, gs, rhs_bias=ob0))
  check(K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), rhs_up=cuda(native(ub)), act="swigluoai", rhs_bias=cuda(b0), rhs_up_bias=cuda(b1)),
        act(O.gmm(lhs, wb, gs, rhs_bias=ob0, out_dtype=torch.float32), O.gmm(lhs, ub, gs, rhs_bias=ob1, out_dtype=torch.float32)))
  # weight-only int8 and int8 x int8
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  want_glu = act(O.gmm(lhs, q, gs, rhs_scale=s, rhs_bias=ob0, out_dtype=torch.float32), O.gmm(lhs, qu, gs, rhs_scale=su, rhs_bias=ob1, out_dtype=torch.float32))
  check(K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su), act="swigluoai",
                  rhs_bias=cuda(b0), rhs_up_bias=cuda(b1)), want_glu)
  aq, asc = O.quantize_rows_int8(lhs.float())
  check(K.gmm_raw(cuda(aq), cuda(native(q)), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(s), rhs_bias=cuda(b0)),
        O.gmm(aq, q, gs, lhs_scale=asc[:, None], rhs_scale=s, rhs_bias=ob0))
  # int4
  if k % 32 == 0:
    q4, s4 = O.quantize_int4_groups(native(w), 128)
    s4 = s4.to(torch.bfloat16)
    v2 = lambda sc: sc.float().permute(0, 2, 1)[:, :, None, :]
    check(K.gmm_raw(cuda(lhs), cuda(O.pack_int4(q4)), cuda(gs), rhs_scale=cuda(s4), rhs_dtype=MOE_INT4, rhs_scale_block_k=128, rhs_bias=cuda(b0)),
          O.gmm(lhs, q4.transpose(1, 2), gs, rhs_scale=v2(s4), quant_block=128, rhs_bias=ob0))
  # fp8 block scaled
  if k % 128 == 0:
    fq, fsc = O.quantize_fp8_blocks(lhs, 1, 128)
    wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)
    uq, usc = O.quantize_fp8_blocks(native(w_up), 128, 128)
    v2f = lambda sc: torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
    fkw = dict(lhs_scale=cuda(fsc), lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128)
    okw = dict(lhs_scale=fsc, transpose_rhs=True, quant_block=128, out_dtype=torch.float32)
    for variant in (0, 1, 2, 3):  # picked by shape / streaming / LDS-tiled with 128- and 256-row tiles
      check(K.gmm_raw(cuda(fq), cuda(wq), cuda(gs), rhs_scale=cuda(wsc), rhs_up=cuda(uq), rhs_up_scale=cuda(usc), act="swigluoai",
                      rhs_bias=cuda(b0), rhs_up_bias=cuda(b1), kernel=FP8_KERNELS[variant], **fkw),
            act(O.gmm(fq, wq, gs, rhs_scale=v2f(wsc), rhs_bias=ob0, **okw), O.gmm(fq, uq, gs, rhs_scale=v2f(usc), rhs_bias=ob1, **okw)))


def test_gmm_bias_argument_errors(K):
  lhs, w, _, gs = _gmm_inputs(64, 128, 64, [64], 19)
  wb = cuda(native(w.to(torch.bfloat16)))
  with pytest.raises(ValueError):
    K.gmm_raw(cuda(lhs), wb, cuda(gs), rhs_bias=torch.zeros(1, 32, device="cuda"))
  with pytest.raises(ValueError):
    K.gmm_raw(cuda(lhs), wb, cuda(gs), rhs_up_bias=torch.zeros(1, 64, device="cuda"))


# ---------------------------------------------------------------- stand-alone gated activation and its gradient


@pytest.mark.parametrize("act", ["silu", "swigluoai", "silu_clip"])
def test_glu_act_forward_and_gradient(K, act):
  g = torch.Generator().manual_seed(60)
  h0 = (torch.randn(300, 264, generator=g) * 4).to(torch.bfloat16)  # |x| reaches past the clip limit of 7
  h1 = (torch.randn(300, 264, generator=g) * 4).to(torch.bfloat16)
  dy = torch.randn(300, 264, generator=g).to(torch.bfloat16)
  got = K.glu_act(cuda(h0), cuda(h1), act, 7.0)
  want = O.apply_ffn_activation(h0, h1, act, 7.0)
  assert relerr(got, want) <= 2.0**-7
  a, b = h0.double().requires_grad_(), h1.double().requires_grad_()
  if act == "silu":
    y = torch.nn.functional.silu(a) * b
  elif act == "swigluoai":
    gc, uc = a.clamp(max=7.0), b.clamp(-7.0, 7.0)
    y = gc * torch.sigmoid(1.702 * gc) * (uc + 1.0)
  else:
    y = torch.nn.functional.silu(a.clamp(max=7.0)) * b.clamp(-7.0, 7.0)
  (y * dy.double()).sum().backward()
  d0, d1 = K.glu_act_bwd(cuda(h0), cuda(h1), cuda(dy), act, 7.0)
  assert relerr(d0, a.grad) <= 2.0**-7 and relerr(d1, b.grad) <= 2.0**-7
  if act != "silu":  # no gradient outside the clip range
    assert torch.all(d0.cpu()[h0.float() > 7.0] == 0) and torch.all(d1.cpu()[h1.float().abs() > 7.0] == 0)
    assert (h0.float() > 7.0).any() and (h1.float().abs() > 7.0).any()


# ---------------------------------------------------------------- MXFP4 weights (GPT-OSS checkpoint format)


@pytest.mark.parametrize("m,k,n,gs", DECODE_SHAPES + [GMM_SHAPES[0], GMM_SHAPES[3], (520, 2880, 96, [500, 20])])
def test_gmm_mxfp4_weight_only(K, m, k, n, gs):
  """bf16 activations x MXFP4 weights consumed as stored (e2m1 pairs + e8m0 block scales): the dequantised
  weights are exact in bf16, so the oracle is its plain bf16 gmm on dequantize_mxfp4 of the same bytes."""
  from maxtext_amd._lib import MOE_MXFP4

  if k % 32:
    pytest.skip("MXFP4 blocks hold 32 values")
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 70)
  blocks, scales = O.quantize_mxfp4(native(w))  # [g, n, k/32, 16], [g, n, k/32]
  ublocks, uscales = O.quantize_mxfp4(native(w_up))
  deq = O.dequantize_mxfp4(blocks, scales).to(torch.bfloat16)  # [g, n, k]
  udeq = O.dequantize_mxfp4(ublocks, uscales).to(torch.bfloat16)
  assert torch.equal(deq.float(), O.dequantize_mxfp4(blocks, scales))  # exact in bf16
  e = len(gs)
  q = blocks.reshape(e, n, k // 2)
  uq = ublocks.reshape(e, n, k // 2)
  kw = dict(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
  got = K.gmm_raw(cuda(lhs), cuda(q), cuda(gs), rhs_scale=cuda(scales), **kw)
  want = O.gmm(lhs, deq, gs, transpose_rhs=True)
  assert relerr(got, want) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  got = K.gmm_raw(cuda(lhs), cuda(q), cuda(gs), rhs_scale=cuda(scales), rhs_up=cuda(uq), rhs_up_scale=cuda(uscales), act="swigluoai", **kw)
  want = O.apply_ffn_activation(O.gmm(lhs, deq, gs, transpose_rhs=True, out_dtype=torch.float32),
                                O.gmm(lhs, udeq, gs, transpose_rhs=True, out_dtype=torch.float32), "swigluoai")
  assert relerr(got, want) <= TOL
  # tiled and streaming kernels agree on the same operands
  tiled = K.gmm_raw(cuda(lhs), cuda(q), cuda(gs), rhs_scale=cuda(scales), rhs_up=cuda(uq), rhs_up_scale=cuda(uscales), act="swigluoai",
                    kernel="tiled", **kw)
  assert relerr(tiled, want) <= TOL


def test_gmm_mxfp4_exact_on_small_integers(K):
  """Integer activations and weights from the e2m1 grid with power-of-two scales: every product and partial sum
  is exact in f32, so the result must equal the oracle bit for bit (catches a swapped nibble or a scale off by one)."""
  from maxtext_amd._lib import MOE_MXFP4

  rng = np.random.default_rng(11)
  m, k, n, gs = 48, 256, 64, np.array([20, 0, 28], np.int32)
  lhs = torch.from_numpy(rng.integers(-3, 4, (m, k)).astype(np.float32)).to(torch.bfloat16)
  blocks = torch.from_numpy(rng.integers(0, 256, (3, n, k // 32, 16)).astype(np.uint8))
  scales = torch.from_numpy(rng.integers(124, 131, (3, n, k // 32)).astype(np.uint8))
  deq = O.dequantize_mxfp4(blocks, scales).to(torch.bfloat16)
  got = K.gmm_raw(cuda(lhs), cuda(blocks.reshape(3, n, k // 2)), cuda(gs), rhs_scale=cuda(scales), rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
  want = O.gmm(lhs, deq, gs, transpose_rhs=True)
  assert torch.equal(got.cpu(), want)


# ---------------------------------------------------------------- randomised shapes, every operand family


def _random_case(rng, k_mult):
  e = int(rng.integers(1, 9))
  k = int(rng.integers(1, 9)) * k_mult
  n = int(rng.integers(1, 40)) * 8
  # few rows per expert (streaming kernels), medium, many (256-row tiles), skewed (one hot expert among cold ones: the
  # tile height follows the average, so the hot expert spans many small tiles or the cold ones sit in big tiles)
  regime = rng.integers(0, 4)
  if regime == 3:
    gs = rng.integers(0, 7, e)
    gs[rng.integers(0, e)] = rng.integers(150, 700)
  else:
    hi = (12, 90, 400)[regime]
    gs = rng.integers(0, hi, e)
    gs[rng.integers(0, e)] = 0 if e > 1 and rng.random() < 0.5 else gs[rng.integers(0, e)]
  m = int(gs.sum()) + int(rng.integers(0, 20))  # trailing rows that belong to no group
  return max(m, 1), k, n, gs.astype(np.int32)


@pytest.mark.parametrize("family", ["bf16", "w8", "i8", "int4", "mxfp4", "fp8"])
def test_gmm_random_shapes(K, family):
  """20 random (M, K, N, group_sizes) per operand family against the oracle: ragged groups, empty groups, skewed
  groups, rows past the last group, K and N at every supported granularity, with and without the fused activation and bias."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4

  rng = np.random.default_rng({"bf16": 1, "w8": 2, "i8": 3, "int4": 4, "mxfp4": 5, "fp8": 6}[family])
  k_mult = {"bf16": 8, "w8": 16, "i8": 16, "int4": 32, "mxfp4": 32, "fp8": 128}[family]
  for case in range(20):
    m, k, n, gs = _random_case(rng, k_mult)
    lhs, w, w_up, _ = _gmm_inputs(m, k, n, list(gs), 1000 + case)
    e = len(gs)
    glu = bool(case % 2)
    bias = _bias(e, n, case) if case % 3 == 0 else (None, None)
    kw, okw, lhs_g, lhs_o = {}, {}, lhs, lhs
    if family == "bf16":
      wq, uq = w.to(torch.bfloat16), w_up.to(torch.bfloat16)
      rhs, rhs_up, orhs, orhs_up = native(wq), native(uq), wq, uq
    elif family in ("w8", "i8"):
      (q, s), (qu, su) = O.quantize_weight_int8(w), O.quantize_weight_int8(w_up)
      rhs, rhs_up, orhs, orhs_up = native(q), native(qu), q, qu
      kw.update(rhs_scale=cuda(s), rhs_up_scale=cuda(su))
      okw.update(rhs_scale=s)
      oup = dict(rhs_scale=su)
      if family == "i8":
        aq, asc = O.quantize_rows_int8(lhs.float())
        lhs_g, lhs_o = aq, aq
        kw.update(lhs_scale=cuda(asc))
        okw.update(lhs_scale=asc[:, None])
        oup.update(lhs_scale=asc[:, None])
    elif family == "int4":
      (q, s), (qu, su) = O.quantize_int4_groups(native(w), 128), O.quantize_int4_groups(native(w_up), 128)
      s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
      v2 = lambda sc: sc.float().permute(0, 2, 1)[:, :, None, :]
      rhs, rhs_up, orhs, orhs_up = O.pack_int4(q), O.pack_int4(qu), q.transpose(1, 2), qu.transpose(1, 2)
      kw.update(rhs_scale=cuda(s), rhs_up_scale=cuda(su), rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
      okw.update(rhs_scale=v2(s), quant_block=128)
      oup = dict(rhs_scale=v2(su), quant_block=128)
    elif family == "mxfp4":
      (b, s), (bu, su) = O.quantize_mxfp4(native(w)), O.quantize_mxfp4(native(w_up))
      rhs, rhs_up = b.reshape(e, n, k // 2), bu.reshape(e, n, k // 2)
      orhs = O.dequantize_mxfp4(b, s).to(torch.bfloat16).transpose(1, 2)
      orhs_up = O.dequantize_mxfp4(bu, su).to(torch.bfloat16).transpose(1, 2)
      kw.update(rhs_scale=cuda(s), rhs_up_scale=cuda(su), rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
    else:  # fp8 block scaled
      aq, asc = O.quantize_fp8_blocks(lhs, 1, 128)
      (q, s), (qu, su) = O.quantize_fp8_blocks(native(w), 128, 128), O.quantize_fp8_blocks(native(w_up), 128, 128)
      v2f = lambda sc: torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
      lhs_g, lhs_o = aq, aq
      rhs, rhs_up, orhs, orhs_up = q, qu, q.transpose(1, 2), qu.transpose(1, 2)
      kw.update(lhs_scale=cuda(asc), rhs_scale=cuda(s), rhs_up_scale=cuda(su), lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128)
      okw.update(lhs_scale=asc, rhs_scale=v2f(s), quant_block=128)
      oup = dict(lhs_scale=asc, rhs_scale=v2f(su), quant_block=128)
    if family in ("bf16", "mxfp4"):
      oup = {}
    if not glu:
      kw.pop("rhs_up_scale", None)
    ob0 = None if bias[0] is None else bias[0][:, None, :]
    ob1 = None if bias[1] is None else bias[1][:, None, :]
    tag = f"{family} case {case}: m={m} k={k} n={n} gs={list(gs)} glu={glu} bias={bias[0] is not None}"
    if glu:
      got = K.gmm_raw(cuda(lhs_g), cuda(rhs), cuda(gs), rhs_up=cuda(rhs_up), act="silu", rhs_bias=None if bias[0] is None else cuda(bias[0]),
                      rhs_up_bias=None if bias[1] is None else cuda(bias[1]), **kw)
      want = O.apply_ffn_activation(O.gmm(lhs_o, orhs, gs, out_dtype=torch.float32, rhs_bias=ob0, **okw),
                                    O.gmm(lhs_o, orhs_up, gs, out_dtype=torch.float32, rhs_bias=ob1, **{**okw, **oup}))
    else:
      got = K.gmm_raw(cuda(lhs_g), cuda(rhs), cuda(gs), rhs_bias=None if bias[0] is None else cuda(bias[0]), **kw)
      want = O.gmm(lhs_o, orhs, gs, rhs_bias=ob0, **okw)
    used = int(gs.sum())
    assert torch.isfinite(got.float()).all(), tag
    assert torch.all(got[used:] == 0), tag
    if used:
      assert relerr(got, want, atol_rms=ELEM_ATOL_RMS_CHAINED if family == "int4" else 1e-2) <= TOL, tag


def test_route_sort_gather_combine_random_sizes(K):
  """Random (T, E, k, d): the integer half of the path bit-exact against numpy, gathers and the weighted combine
  against brute force, for sizes around the kernels' internal chunk boundaries."""
  rng = np.random.default_rng(77)
  for case in range(24):
    e = int(rng.choice([1, 2, 7, 8, 32, 60, 64, 65, 128, 200, 256, 384, 512]))
    k = int(rng.integers(1, min(e, 8) + 1))
    t = int(rng.choice([1, 2, 63, 64, 65, 255, 256, 257, 1000, 1023, 1024, 1025, 4097, 9000]))
    d = int(rng.integers(1, 40)) * 8
    logits = rng.standard_normal((t, e)).astype(np.float32)
    if case % 4 == 0:
      logits = np.round(logits * 2) / 2  # many exact ties
    w, idx = K.route_topk(cuda(logits), k=k, norm_topk_prob=bool(case % 2))
    ow, oidx = O.get_topk(logits, k=k, norm_topk_prob=bool(case % 2))
    tag = f"case {case}: t={t} e={e} k={k} d={d}"
    np.testing.assert_array_equal(idx.cpu().numpy(), oidx, err_msg=tag)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2.0**-6, atol=1e-6, err_msg=tag)
    perm, inv, gs, se = K.sort_by_expert(idx, e)
    flat = oidx.reshape(-1)
    operm = np.argsort(flat, kind="stable").astype(np.int32)
    np.testing.assert_array_equal(perm.cpu().numpy(), operm, err_msg=tag)
    np.testing.assert_array_equal(gs.cpu().numpy(), np.bincount(flat, minlength=e), err_msg=tag)
    np.testing.assert_array_equal(se.cpu().numpy(), flat[operm], err_msg=tag)
    np.testing.assert_array_equal(inv.cpu().numpy()[operm], np.arange(t * k), err_msg=tag)
    x = torch.from_numpy(rng.standard_normal((t, d)).astype(np.float32)).to(torch.bfloat16)
    rows = K.gather_rows(cuda(x), perm, k)
    assert torch.equal(rows.cpu(), x[torch.from_numpy(operm.astype(np.int64) // k)]), tag
    out = K.unpermute_combine(rows, w, k=k, inv_perm=inv)
    want = (x.float() * torch.from_numpy(ow).sum(-1, keepdim=True)).to(torch.bfloat16)  # every copy of a token is the token itself
    assert relerr(out, want) <= 2.0**-7, tag


def test_tgmm_random_shapes(K):
  rng = np.random.default_rng(78)
  for case in range(16):
    e = int(rng.integers(1, 7))
    k, n = int(rng.integers(1, 50)) * 8, int(rng.integers(1, 50)) * 8
    gs = rng.integers(0, (5, 40, 300)[case % 3], e).astype(np.int32)
    m = max(int(gs.sum()) + int(rng.integers(0, 10)), 1)
    g = torch.Generator().manual_seed(case)
    lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
    dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
    got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), out_dtype=torch.float32)
    want = O.tgmm(lhs, dout, gs, out_dtype=torch.float32).transpose(1, 2)
    tag = f"case {case}: m={m} k={k} n={n} gs={list(gs)}"
    for i, sz in enumerate(gs):
      if sz == 0:
        assert torch.all(got[i] == 0), tag
      else:
        assert relerr(got[i], want[i]) <= TOL, tag


def test_tgmm_random_shapes_big_tiles(K):
  """Random group sizes on shapes that take the 256 x 256 kernel (K, N multiples of 256, 128 rows per group on average,
  at least 128 tiles): empty groups, groups shorter than one 64-row stage, ragged last stages, rows of no group, windows."""
  rng = np.random.default_rng(79)
  for case in range(6):
    e = int(rng.integers(2, 7))
    off = int(rng.integers(0, 2))
    loc = e - off if case % 2 == 0 else max(1, e - off - 1)
    tk, tn = int(rng.integers(1, 5)), int(rng.integers(1, 5))
    while tk * tn * loc < 128:
      tk, tn = (tk + 1, tn) if tk <= tn else (tk, tn + 1)
    k, n = tk * 256, tn * 256
    gs = rng.integers(0, 520, e).astype(np.int32)
    gs[int(rng.integers(0, e))] = (0, 1, 63, 64, 65, 129)[case]
    need = 128 * e - int(gs.sum())
    if need > 0:
      gs[int(np.argmax(gs))] += need
    m = int(gs.sum()) + int(rng.integers(0, 70))
    g = torch.Generator().manual_seed(100 + case)
    lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
    dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
    want = O.tgmm(lhs, dout, gs, out_dtype=torch.float32).transpose(1, 2)
    got = K.tgmm(cuda(lhs), cuda(dout), cuda(gs), num_groups_local=loc, group_offset=off, out_dtype=torch.float32)
    tag = f"case {case}: m={m} k={k} n={n} gs={list(gs)} window=({off},{loc})"
    assert got.shape == (loc, n, k), tag
    for i in range(loc):
      if gs[off + i] == 0:
        assert torch.all(got[i] == 0), tag
      else:
        assert relerr(got[i], want[off + i]) <= TOL, tag


@pytest.mark.parametrize("m,k,n,gs", DECODE_SHAPES + [GMM_SHAPES[0], GMM_SHAPES[3]])
def test_gmm_int4_group32(K, m, k, n, gs):
  """int4 with one scale per 32 values (Kimi-K2 checkpoints): the reference dequantises to bf16 first
  (convert_deepseek_family_ckpt.py:56-84), so the oracle is its bf16 gmm on dequantize_int4(..., 32)."""
  from maxtext_amd._lib import MOE_INT4

  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 80)
  q, s = O.quantize_int4_groups(native(w), 32)
  qu, su = O.quantize_int4_groups(native(w_up), 32)
  s, su = s.to(torch.bfloat16), su.to(torch.bfloat16)
  pq, pu = O.pack_int4(q), O.pack_int4(qu)
  deq, udeq = O.dequantize_int4(pq, s, 32), O.dequantize_int4(pu, su, 32)  # [g, n, k] bf16
  kw = dict(rhs_dtype=MOE_INT4, rhs_scale_block_k=32)
  got = K.gmm_raw(cuda(lhs), cuda(pq), cuda(gs), rhs_scale=cuda(s), **kw)
  assert relerr(got, O.gmm(lhs, deq, gs, transpose_rhs=True)) <= TOL
  assert torch.all(got[int(gs.sum()):] == 0)
  want = O.apply_ffn_activation(O.gmm(lhs, deq, gs, transpose_rhs=True, out_dtype=torch.float32),
                                O.gmm(lhs, udeq, gs, transpose_rhs=True, out_dtype=torch.float32))
  got = K.gmm_raw(cuda(lhs), cuda(pq), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(pu), rhs_up_scale=cuda(su), act="silu", **kw)
  assert relerr(got, want) <= TOL
  tiled = K.gmm_raw(cuda(lhs), cuda(pq), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(pu), rhs_up_scale=cuda(su), act="silu", kernel="tiled", **kw)
  assert relerr(tiled, want) <= TOL


@pytest.mark.parametrize("m,k,n,gs", [GMM_SHAPES[0], GMM_SHAPES[3], DECODE_SHAPES[0]])
def test_gmm_partial_sum_every_kernel_family(K, m, k, n, gs):
  """partial_sum (ops.py:77; v2 kernel :576-578): added after the bias and before the activation, only to rows of
  local groups; rows that belong to no group stay zero.  Exercised with bf16 (tiled / direct-to-LDS), int8 x int8,
  weight-only int8 (tiled or streaming by shape) and block-scaled fp8."""
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 90)
  g = torch.Generator().manual_seed(91)
  ps = torch.randn(m, n, generator=g).to(torch.bfloat16)
  ps_up = torch.randn(m, n, generator=g).to(torch.bfloat16)
  used = int(gs.sum())
  act = lambda h0, h1: O.apply_ffn_activation(h0, h1, "silu")

  def check(got, want):
    assert relerr(got, want) <= TOL
    assert torch.all(got[used:] == 0)

  wb, ub = w.to(torch.bfloat16), w_up.to(torch.bfloat16)
  check(K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), partial_sum=cuda(ps)), O.gmm(lhs, wb, gs, partial_sum=ps))
  check(K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), rhs_up=cuda(native(ub)), act="silu", partial_sum=cuda(ps), partial_sum_up=cuda(ps_up)),
        act(O.gmm(lhs, wb, gs, partial_sum=ps, out_dtype=torch.float32), O.gmm(lhs, ub, gs, partial_sum=ps_up, out_dtype=torch.float32)))
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  check(K.gmm_raw(cuda(lhs), cuda(native(q)), cuda(gs), rhs_scale=cuda(s), rhs_up=cuda(native(qu)), rhs_up_scale=cuda(su), act="silu",
                  partial_sum=cuda(ps), partial_sum_up=cuda(ps_up)),
        act(O.gmm(lhs, q, gs, rhs_scale=s, partial_sum=ps, out_dtype=torch.float32), O.gmm(lhs, qu, gs, rhs_scale=su, partial_sum=ps_up, out_dtype=torch.float32)))
  aq, asc = O.quantize_rows_int8(lhs.float())
  check(K.gmm_raw(cuda(aq), cuda(native(q)), cuda(gs), lhs_scale=cuda(asc), rhs_scale=cuda(s), partial_sum=cuda(ps)),
        O.gmm(aq, q, gs, lhs_scale=asc[:, None], rhs_scale=s, partial_sum=ps))
  if k % 128 == 0:
    fq, fsc = O.quantize_fp8_blocks(lhs, 1, 128)
    wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)
    v2f = lambda sc: torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
    for variant in (0, 1, 2, 3):
      check(K.gmm_raw(cuda(fq), cuda(wq), cuda(gs), lhs_scale=cuda(fsc), rhs_scale=cuda(wsc), lhs_scale_block_k=128, rhs_scale_block_n=128,
                      rhs_scale_block_k=128, partial_sum=cuda(ps), kernel=FP8_KERNELS[variant]),
            O.gmm(fq, wq, gs, lhs_scale=fsc, rhs_scale=v2f(wsc), transpose_rhs=True, quant_block=128, partial_sum=ps))
  with pytest.raises(ValueError):
    K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), partial_sum_up=cuda(ps_up))


def test_megablox_gmm_partial_sum_accumulates_k_chunks():
  """The way the reference uses partial_sum (moe.py:1962-1980): the contraction is split into chunks of the embedding
  dimension and each call adds the previous chunks' result; the chunked result must match the one-shot call."""
  from maxtext_amd import megablox

  lhs, w, _, gs = _gmm_inputs(600, 512, 256, [100, 0, 300, 200], 92)
  wb = cuda(w.to(torch.bfloat16))  # [g, k, n]
  lhs_d, gs_d = cuda(lhs), cuda(gs)
  acc = None
  for c in range(4):
    sl = slice(c * 128, (c + 1) * 128)
    acc = gmm_bf16(lhs_d[:, sl].contiguous(), wb[:, sl].contiguous(), gs_d, partial_sum=acc)
  full = gmm_bf16(lhs_d, wb, gs_d)
  assert relerr(acc, full, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2  # three extra bf16 roundings of the running sum


def test_gmm_existing_out_keeps_rows_of_other_groups():
  """existing_out (ops.py:51): two calls, each holding half of the groups, fill one buffer; rows of the other
  half and rows past the last group keep what the buffer held (here a sentinel), bit for bit."""
  from maxtext_amd import megablox

  lhs, w, _, gs = _gmm_inputs(700, 256, 128, [150, 0, 250, 100, 120], 95)  # 80 trailing rows in no group
  wb = w.to(torch.bfloat16)
  full = O.gmm(lhs, wb, gs)
  buf = torch.full((700, 128), 7.0, dtype=torch.bfloat16, device="cuda")
  out = gmm_bf16(cuda(lhs), cuda(wb[:2]), cuda(gs), existing_out=buf, group_offset=0)
  assert out.data_ptr() == buf.data_ptr()
  assert torch.all(buf[150:] == 7.0) and relerr(buf[:150], full[:150]) <= TOL
  gmm_bf16(cuda(lhs), cuda(wb[2:]), cuda(gs), existing_out=buf, group_offset=2)
  assert relerr(buf[:620], full[:620]) <= TOL and torch.all(buf[620:] == 7.0)
  # without existing_out the same call zeroes the rows it does not own
  plain = gmm_bf16(cuda(lhs), cuda(wb[2:]), cuda(gs), group_offset=2)
  assert torch.all(plain[:150] == 0) and torch.all(plain[620:] == 0)
  # the few-rows (streaming) kernels take the same tile list
  lhs2, w2, _, gs2 = _gmm_inputs(60, 256, 128, [10, 20, 5, 15], 96)
  q, s = O.quantize_weight_int8(w2)
  buf2 = torch.full((60, 128), -3.0, dtype=torch.bfloat16, device="cuda")
  K = __import__("maxtext_amd.kernels", fromlist=["x"])
  K.gmm_raw(cuda(lhs2), cuda(native(q[1:3])), cuda(gs2), rhs_scale=cuda(s[1:3]), group_offset=1, out=buf2, keep_other_rows=True)
  want = O.gmm(lhs2, q, gs2, rhs_scale=s)
  assert torch.all(buf2[:10] == -3.0) and torch.all(buf2[35:] == -3.0) and relerr(buf2[10:35], want[10:35]) <= TOL


@pytest.mark.parametrize("mode", ["topk_raw", "softmax_all"])
@pytest.mark.parametrize("t,e,k", [(300, 16, 1), (1000, 128, 8), (77, 200, 4)])
def test_route_llama4_and_gemma4_weight_rules(K, mode, t, e, k):
  """Llama4 keeps the selected logits as weights; Gemma4 reads a softmax over all experts at the selected
  indices (moe.py:742-753).  Indices bit-exact, weights against the closed forms."""
  rng = np.random.default_rng(8)
  logits = rng.standard_normal((t, e)).astype(np.float32) * 2
  for norm in (False, True):
    w, idx = K.route_topk(cuda(logits), k=k, mode=mode, norm_topk_prob=norm)
    ow, oidx = O.get_topk(logits, k=k, mode=mode, norm_topk_prob=norm)
    np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
    np.testing.assert_allclose(w.cpu().numpy(), ow, rtol=2.0**-6, atol=1e-6)
  # independent closed forms in f64
  w, idx = K.route_topk(cuda(logits), k=k, mode=mode, weights_round_bf16=False)
  sel = np.take_along_axis(logits.astype(np.float64), idx.cpu().numpy().astype(np.int64), -1)
  if mode == "topk_raw":
    want = sel
  else:
    z = np.exp(logits.astype(np.float64) - logits.max(-1, keepdims=True))
    want = np.exp(sel - logits.max(-1, keepdims=True)) / z.sum(-1, keepdims=True)
  np.testing.assert_allclose(w.cpu().numpy(), want, rtol=1e-5, atol=1e-7)


@pytest.mark.parametrize("variant", [0, 1, 2, 3])
def test_gmm_fp8_group_offset_and_kept_rows(K, variant):
  """Block-scaled fp8 with a shard of the experts (group_offset, ops.py:50): rows of other groups are zero-filled, or keep
  the buffer's contents with existing_out, in the streaming and in the LDS-tiled kernel."""
  lhs, w, _, gs = _gmm_inputs(900, 384, 200, [130, 300, 0, 270, 150], 33)
  aq, asc = O.quantize_fp8_blocks(lhs, 1, 128)
  wq, wsc = O.quantize_fp8_blocks(native(w), 128, 128)
  v2 = lambda sc: torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :200]
  kw = dict(lhs_scale=cuda(asc), lhs_scale_block_k=128, rhs_scale_block_n=128, rhs_scale_block_k=128, kernel=FP8_KERNELS[variant])
  got = K.gmm_raw(cuda(aq), cuda(wq[1:4]), cuda(gs), rhs_scale=cuda(wsc[1:4]), group_offset=1, **kw)
  want = O.gmm(aq, wq[1:4], gs, lhs_scale=asc, rhs_scale=v2(wsc[1:4]), transpose_rhs=True, quant_block=128, group_offset=1)
  assert relerr(got, want) <= TOL
  assert torch.all(got[:130] == 0) and torch.all(got[700:] == 0)
  buf = torch.full((900, 200), 3.0, dtype=torch.bfloat16, device="cuda")
  K.gmm_raw(cuda(aq), cuda(wq[1:4]), cuda(gs), rhs_scale=cuda(wsc[1:4]), group_offset=1, out=buf, keep_other_rows=True, **kw)
  assert torch.all(buf[:130] == 3.0) and torch.all(buf[700:] == 3.0)
  assert torch.equal(buf[130:700], got[130:700])


@pytest.mark.parametrize("bwd_q", [None, "float8_e5m2"])
@pytest.mark.parametrize("transpose_rhs", [False, True])
def test_gmm_quantized_backward(transpose_rhs, bwd_q):
  """int8 x int8 forward with the reference's backward (ops.py:530-604): quantised residuals, the scale of the
  contracted axis folded into the gradient, optional e5m2 quantisation of the gradient per row / per column.
  Compared with the oracle on the oracle's own quantised operands."""
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(12)
  m, k, n = 450, 256, 192
  gs = np.array([200, 0, 70, 150], np.int32)  # an empty group and 30 trailing rows in no group
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = (torch.randn(4, k, n, generator=g) * 0.05).to(torch.bfloat16)  # [g, k, n]
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  lq, ls = O.quantize_rows_int8(lhs.float())
  rq, rs = O.quantize_weight_int8(w.float(), per_expert=False)  # one [n] scale shared by the experts (ops.py:250-260)
  want_dl, want_dr = O.gmm_bwd_quantized(dout, lq, ls, rq, rs[0], gs, bwd_qtype=None if bwd_q is None else "e5m2")
  want_out = O.gmm(lq, rq, gs, lhs_scale=ls[:, None], rhs_scale=rs)

  lhs_g = cuda(lhs).requires_grad_()
  rhs_g = cuda(w.transpose(1, 2).contiguous() if transpose_rhs else w).requires_grad_()
  out = gmm_bf16(lhs_g, rhs_g, cuda(gs), transpose_rhs=transpose_rhs, lhs_quantize_dtype="int8", rhs_quantize_dtype="int8",
                     bwd_quantize_dtype=bwd_q)
  assert relerr(out, want_out) <= TOL
  out.backward(cuda(dout))
  tol = TOL if bwd_q is None else 2e-2  # a gradient value next to an e5m2 rounding boundary may land on either side
  assert relerr(lhs_g.grad, want_dl) <= tol
  assert torch.all(lhs_g.grad[420:] == 0)
  got_dr = rhs_g.grad.transpose(1, 2) if transpose_rhs else rhs_g.grad
  assert got_dr.shape == want_dr.shape and relerr(got_dr, want_dr) <= tol
  assert torch.all(got_dr[1] == 0)
  with pytest.raises(NotImplementedError):
    gmm_bf16(lhs_g, rhs_g, cuda(gs), transpose_rhs=transpose_rhs, bwd_quantize_dtype="float8_e5m2")


@pytest.mark.parametrize("quantize", [False, True])
@pytest.mark.parametrize("n", [192, 2056])
def test_bwd_scale_grad_bit_exact(K, n, quantize):
  """The gradient preparation of the quantised backward (ops.py:530-604) against the oracle's e5m2 quantiser on the
  same scaled gradient: per row with the weights' channel scales of each row's expert (an empty group, rows past the
  last group, a group offset), per column with the activations' row scales; values and scales bit for bit."""
  g = torch.Generator().manual_seed(31)
  m = 333
  gs = np.array([40, 100, 0, 70, 93], np.int32)  # 30 trailing rows in no group
  offset, g_local = 1, 3
  dout = (torch.randn(m, n, generator=g) * torch.rand(m, 1, generator=g) * 8).to(torch.bfloat16)
  dout[5, 7] = 0.0
  dout[17] = 0.0  # a zero row: scale 0, values 0
  dout[:, 11] = 0.0  # a zero column
  rs = torch.rand(g_local, n, generator=g) * 0.02 + 1e-4
  ls = torch.rand(m, generator=g) * 0.05 + 1e-4
  ends = np.cumsum(gs)
  local = np.clip(np.searchsorted(ends, np.arange(m), side="right") - offset, 0, g_local - 1)
  d_rows = dout * rs.to(torch.bfloat16)[torch.from_numpy(local)]
  d_cols = dout * ls.to(torch.bfloat16)[:, None]
  got_r, s_r = K.bwd_scale_grad(cuda(dout), cuda(rs), mode="dlhs", quantize=quantize, group_sizes=cuda(gs), num_groups_local=g_local,
                                group_offset=offset)
  got_c, s_c = K.bwd_scale_grad(cuda(dout), cuda(ls), mode="drhs", quantize=quantize)
  if not quantize:
    assert s_r is None and s_c is None
    assert torch.equal(got_r.cpu(), d_rows) and torch.equal(got_c.cpu(), d_cols)
    return
  want_r, want_sr = O.quantize_e5m2(d_rows, dim=1)
  want_c, want_sc = O.quantize_e5m2(d_cols, dim=0)
  assert torch.equal(s_r.cpu(), want_sr[:, 0]) and torch.equal(s_c.cpu(), want_sc[0])
  assert torch.equal(got_r.cpu().float(), want_r) and torch.equal(got_c.cpu().float(), want_c)
  assert float(s_r[17]) == 0.0 and torch.all(got_r[17] == 0) and float(s_c[11]) == 0.0


@pytest.mark.parametrize("as_fp8", [False, True])
@pytest.mark.parametrize("n", [192, 2056])
def test_bwd_scale_grad_per_tensor_bit_exact(K, n, as_fp8):
  """disable_channelwise_axes in the backward (ops.py:568, :594, :601: channelwise_axes=[]): the gradient times the one
  scale of an operand quantised per tensor, then ONE absmax scale for the whole gradient; values and scale bit for bit
  against the oracle's e5m2 quantiser over both axes, as bf16 values and as float8_e5m2 bytes; a NaN-free all-zero
  gradient gives scale 0 and zeros."""
  g = torch.Generator().manual_seed(33)
  m = 333
  dout = (torch.randn(m, n, generator=g) * torch.rand(m, 1, generator=g) * 8).to(torch.bfloat16)
  dout[17] = 0.0
  dout[:, 11] = 0.0
  f = torch.tensor([0.0173])
  d = dout * f.to(torch.bfloat16)
  plain, none = K.bwd_scale_grad(cuda(dout), cuda(f), mode="tensor", quantize=False)
  assert none is None and torch.equal(plain.cpu(), d)
  want, want_s = O.quantize_e5m2(d, dim=(0, 1))
  got, s = K.bwd_scale_grad(cuda(dout), cuda(f), mode="tensor", quantize=True, as_fp8=as_fp8)
  assert got.dtype == (torch.float8_e5m2 if as_fp8 else torch.bfloat16)
  assert tuple(s.shape) == (n,) and torch.all(s.cpu() == want_s.reshape(())) and float(want_s) == float(np.float32(float(d.float().abs().max())) / np.float32(57344.0))
  assert torch.equal(got.cpu().float(), want)
  assert float(got.float().abs().max()) == 57344.0  # the tensor's largest value sits on the format's largest
  zero, s0 = K.bwd_scale_grad(cuda(torch.zeros_like(dout)), cuda(f), mode="tensor", quantize=True, as_fp8=as_fp8)
  assert torch.all(s0 == 0) and torch.all(zero.float() == 0)
  with pytest.raises(ValueError):
    K.bwd_scale_grad(cuda(dout), cuda(torch.ones(m)), mode="tensor", quantize=True)


def test_gmm_autograd_with_expert_bias():
  """Per-expert mlp_bias on the differentiable path (moe.py:1952-1957): forward equals the epilogue bias of the
  inference path; gradients of lhs, both weights and both biases against torch autograd in f64."""
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(14)
  m, k, n = 300, 128, 128
  gs = np.array([100, 0, 156], np.int32)  # 44 trailing rows
  off = [0, 100, 100, 256]
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w0 = (torch.randn(3, n, k, generator=g) * 0.1).to(torch.bfloat16)
  w1 = (torch.randn(3, n, k, generator=g) * 0.1).to(torch.bfloat16)
  b0, b1 = torch.randn(3, n, generator=g), torch.randn(3, n, generator=g)
  dout = torch.randn(m, n, generator=g).to(torch.bfloat16)
  a, r0, r1, c0, c1 = (t.double().requires_grad_() for t in (lhs, w0, w1, b0, b1))
  h0 = torch.cat([a[off[i] : off[i + 1]] @ r0[i].T + c0[i] for i in range(3)])
  h1 = torch.cat([a[off[i] : off[i + 1]] @ r1[i].T + c1[i] for i in range(3)])
  ref = torch.cat([torch.nn.functional.silu(h0) * h1, torch.zeros(44, n, dtype=torch.float64)])
  (ref * dout.double()).sum().backward()
  la, q0, q1, d0, d1 = (cuda(t).requires_grad_() for t in (lhs, w0, w1, b0, b1))
  out = gmm_bf16(la, q0, cuda(gs), transpose_rhs=True, rhs_up=q1, fuse_act="silu", rhs_bias=d0, rhs_up_bias=d1)
  with torch.no_grad():
    fused = gmm_bf16(cuda(lhs), cuda(w0), cuda(gs), transpose_rhs=True, rhs_up=cuda(w1), fuse_act="silu", rhs_bias=cuda(b0), rhs_up_bias=cuda(b1))
  assert relerr(out, ref, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2 and relerr(out, fused, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2 and torch.all(out[256:] == 0)
  out.backward(cuda(dout))
  assert relerr(la.grad, a.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(q0.grad, r0.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2 and relerr(q1.grad, r1.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert relerr(d0.grad, c0.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2 and relerr(d1.grad, c1.grad, atol_rms=ELEM_ATOL_RMS_CHAINED) <= 2e-2
  assert torch.all(d0.grad[1] == 0)


# Shapes large enough for the persistent direct-to-LDS kernel (at least 128 tiles of 256 x 256, 128 rows per
# expert): K = 128 (one stage), 384 (three 128-byte stages), 320 and 192 (K * elem only a multiple of 64: the
# 64-byte pipeline for int8; for bf16 both are multiples of 128 bytes), ragged groups with an empty one and
# trailing rows that belong to no group.
DL_SHAPES = [(4200, 128, 2048), (4200, 384, 2048), (4200, 320, 2048), (4200, 192, 2304)]


@pytest.mark.parametrize("m,k,n", DL_SHAPES)
def test_gmm_direct_to_lds_pipelines_int8(K, m, k, n):
  gs = np.array([1000, 0, 2000, 1096], np.int32)
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 41)
  q, s = O.quantize_weight_int8(w)
  qu, su = O.quantize_weight_int8(w_up)
  lq, ls = O.quantize_rows_int8(lhs)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s), rhs_up=cuda(native(qu)),
                  rhs_up_scale=cuda(su), act="silu")
  want = O.apply_ffn_activation(O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s, out_dtype=torch.float32, acc_dtype=torch.float32),
                                O.gmm(lq, qu, gs, lhs_scale=ls, rhs_scale=su, out_dtype=torch.float32, acc_dtype=torch.float32))
  assert relerr(got, want) <= TOL and torch.all(got[4096:] == 0)
  got = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s))
  want = O.gmm(lq, q, gs, lhs_scale=ls, rhs_scale=s, acc_dtype=torch.float32)
  assert relerr(got, want) <= TOL and torch.all(got[4096:] == 0)
  # the 64-byte pipeline on the same operands (the "dl64" kernel family) agrees bit for bit: integer accumulation
  if k % 128 == 0:
    other = K.gmm_raw(cuda(lq), cuda(native(q)), cuda(gs), lhs_scale=cuda(ls), rhs_scale=cuda(s), kernel="dl64")
    assert torch.equal(got, other)


@pytest.mark.parametrize("m,k,n", DL_SHAPES[:3])
def test_gmm_direct_to_lds_pipelines_bf16(K, m, k, n):
  gs = np.array([1000, 0, 2000, 1096], np.int32)
  lhs, w, w_up, gs = _gmm_inputs(m, k, n, gs, 42)
  wb, ub = w.to(torch.bfloat16), w_up.to(torch.bfloat16)
  got = K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs), rhs_up=cuda(native(ub)), act="silu")
  want = O.apply_ffn_activation(O.gmm(lhs, wb, gs, out_dtype=torch.float32, acc_dtype=torch.float32),
                                O.gmm(lhs, ub, gs, out_dtype=torch.float32, acc_dtype=torch.float32))
  assert relerr(got, want) <= TOL and torch.all(got[4096:] == 0)
  got = K.gmm_raw(cuda(lhs), cuda(native(wb)), cuda(gs))
  assert relerr(got, O.gmm(lhs, wb, gs, acc_dtype=torch.float32)) <= TOL


# ---------------------------------------------------------------- degenerate sizes


def test_gmm_degenerate_group_sizes(K):
  """All groups empty (every row is written as zero), a single row, group sizes that overrun the rows (clipped to m as
  reference_gmm does, tests/unit/pallas_mosaic_tpu_v2_kernel_test.py:139-141), the smallest K and N the kernels take."""
  g = torch.Generator().manual_seed(41)
  lhs = torch.randn(37, 64, generator=g).to(torch.bfloat16)
  w = (torch.randn(3, 24, 64, generator=g) * 0.1).to(torch.bfloat16)  # [g, n, k]
  out = K.gmm_raw(cuda(lhs), cuda(w), cuda(np.array([0, 0, 0], np.int32)))
  assert out.shape == (37, 24) and torch.all(out == 0)
  one = K.gmm_raw(cuda(lhs[:1]), cuda(w), cuda(np.array([0, 1, 0], np.int32)))
  assert relerr(one, lhs[:1].float() @ w[1].float().T) <= TOL
  over = K.gmm_raw(cuda(lhs), cuda(w), cuda(np.array([20, 30, 50], np.int32)))  # 100 rows announced, 37 exist
  want = torch.cat([lhs[:20].float() @ w[0].float().T, lhs[20:].float() @ w[1].float().T])
  assert relerr(over, want) <= TOL
  tiny = K.gmm_raw(cuda(lhs[:, :16].contiguous()), cuda(w[:, :8, :16].contiguous()), cuda(np.array([10, 20, 7], np.int32)))
  gs = [10, 20, 7]
  off = np.concatenate([[0], np.cumsum(gs)])
  want = torch.cat([lhs[off[i]:off[i + 1], :16].float() @ w[i, :8, :16].float().T for i in range(3)])
  assert relerr(tiny, want) <= TOL


@pytest.mark.parametrize("fmt", ["int4", "mxfp4"])
def test_gmm_4bit_decode_degenerate_group_sizes(K, fmt):
  """The LDS-streamed decode kernel on all-empty groups (every row zero), a single row, and group sizes that overrun the
  rows (clipped to m): the cases of test_gmm_degenerate_group_sizes on 4-bit weights."""
  from maxtext_amd._lib import MOE_INT4, MOE_MXFP4
  g = torch.Generator().manual_seed(43)
  m, k, n = 37, 256, 128
  lhs = torch.randn(m, k, generator=g).to(torch.bfloat16)
  w = torch.randn(3, n, k, generator=g) * 0.1  # [g, n, k]
  if fmt == "int4":
    q, s = O.quantize_int4_groups(w, 128)
    s = s.to(torch.bfloat16)
    deq = (q.float().reshape(3, n, k // 128, 128) * s.float()[..., None]).reshape(3, n, k)
    pk, kw = O.pack_int4(q), dict(rhs_dtype=MOE_INT4, rhs_scale_block_k=128)
  else:
    blocks, s = O.quantize_mxfp4(w)
    deq = O.dequantize_mxfp4(blocks, s)
    pk, kw = blocks.reshape(3, n, k // 2), dict(rhs_dtype=MOE_MXFP4, rhs_scale_block_k=32)
  up = dict(rhs_up=cuda(pk), rhs_up_scale=cuda(s), act="silu")  # (with the second projection the kernel takes 128 channels)
  out = K.gmm_raw(cuda(lhs), cuda(pk), cuda(np.array([0, 0, 0], np.int32)), rhs_scale=cuda(s), **up, **kw)
  assert out.shape == (m, n) and torch.all(out == 0)
  h = lambda x, e: x.float() @ deq[e].float().T
  act = lambda y: torch.nn.functional.silu(y) * y
  one = K.gmm_raw(cuda(lhs[:1]), cuda(pk), cuda(np.array([0, 1, 0], np.int32)), rhs_scale=cuda(s), **up, **kw)
  assert relerr(one, act(h(lhs[:1], 1))) <= TOL
  over = K.gmm_raw(cuda(lhs), cuda(pk), cuda(np.array([20, 30, 50], np.int32)), rhs_scale=cuda(s), **up, **kw)  # 100 rows announced, 37 exist
  assert relerr(over, torch.cat([act(h(lhs[:20], 0)), act(h(lhs[20:], 1))])) <= TOL


def test_route_sort_combine_single_token(K):
  """One token: routing, sort, gather and combine on the smallest input (k of E selections, all in different groups)."""
  g = torch.Generator().manual_seed(42)
  logits = torch.randn(1, 8, generator=g)
  w, idx = K.route_topk(cuda(logits), k=2)
  want_w, want_idx = O.get_topk(logits, k=2)
  assert torch.equal(idx.cpu(), torch.from_numpy(np.asarray(want_idx)).to(torch.int32))
  assert torch.equal(w.cpu(), torch.from_numpy(np.asarray(want_w, np.float32)))
  perm, inv, gs, _ = K.sort_by_expert(idx, 8)
  assert int(gs.sum()) == 2 and sorted(perm.cpu().tolist()) == [0, 1]
  x = torch.randn(1, 32, generator=g).to(torch.bfloat16)
  rows = K.gather_rows(cuda(x), perm, 2)
  rows = rows[0] if isinstance(rows, tuple) else rows
  assert torch.equal(rows.cpu(), x.expand(2, 32))
  y = K.unpermute_combine(rows, w, k=2, perm=perm, inv_perm=inv)
  want = (x.float() * float(w.sum())).to(torch.bfloat16)
  assert relerr(y, want) <= TOL


@pytest.mark.parametrize("t,e,k", [(1, 32, 4), (16, 32, 4), (128, 32, 4), (256, 256, 8), (1024, 8, 2), (1025, 8, 4)])
def test_sort_leaves_the_tile_list_for_the_matmuls(K, t, e, k):
  # moe_sort_by_expert_mapped: same sort results; the grouped matmul that follows on the same workspace, flagged
  # MOE_GMM_SAME_GROUPS, gives the result of a call that maps for itself (bit for bit), whether it picks 16-row tiles
  # (weight-only int8 at decode sizes) or another height (bf16: list rebuilt); above 4096 rows nothing is mapped
  rng = np.random.default_rng(t + e)
  sel = np.stack([rng.permutation(e)[:k] for _ in range(t)]).astype(np.int32)
  m = t * k
  ws = K.gmm_workspace(m, e, "cuda")
  perm, inv, gs, se = K.sort_by_expert(cuda(sel), e, gmm_workspace=ws)
  perm0, inv0, gs0, se0 = K.sort_by_expert(cuda(sel), e)
  for a, b in ((perm, perm0), (inv, inv0), (gs, gs0), (se, se0)):
    assert torch.equal(a, b)
  g = torch.Generator(device="cuda").manual_seed(t)
  d, f = 128, 256
  x = torch.randn((m, d), generator=g, device="cuda").to(torch.bfloat16)
  wq = torch.randint(-127, 128, (e, f, d), generator=g, device="cuda", dtype=torch.int8)
  sc = torch.rand((e, f), generator=g, device="cuda") * 0.01
  wb = (torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  y = K.gmm_raw(x, wq, gs, rhs_scale=sc, workspace=ws, same_groups=True)
  assert torch.equal(y, K.gmm_raw(x, wq, gs0, rhs_scale=sc))
  yb = K.gmm_raw(x, wb, gs, workspace=ws, same_groups=True)
  assert torch.equal(yb, K.gmm_raw(x, wb, gs0))
  y2 = K.gmm_raw(x, wq, gs, rhs_scale=sc, workspace=ws, same_groups=True)
  assert torch.equal(y2, y)


@pytest.mark.parametrize("t,e,k,mode", [(1, 32, 4, "softmax_topk"), (16, 32, 4, "softmax_topk"), (3, 128, 5, "topk_raw"), (13, 256, 8, "deepseek"),
                                        (4, 8, 2, "softmax_all"), (5, 8, 2, "softmax_all"), (17, 32, 4, "softmax_topk"), (300, 32, 4, "softmax_topk")])
def test_route_and_sort_in_one_call(K, t, e, k, mode):
  """moe_route_sort_mapped: the weights and indices of moe_route_topk and the permutation, group sizes and tile list of
  moe_sort_by_expert_mapped on those indices, bit for bit, as one launch (up to 16 tokens, with 4 or 16 waves) or as the
  two calls (the last two cases); the flagged grouped matmul that follows equals one that maps for itself."""
  g = torch.Generator(device="cuda").manual_seed(t * e + k)
  logits = torch.randn((t, e), generator=g, device="cuda")
  pre = torch.sigmoid(logits) if mode == "deepseek" else None
  kw = dict(k=k, mode=mode, norm_topk_prob=mode != "topk_raw", routed_scaling_factor=2.5 if mode == "deepseek" else 1.0)
  w0, idx0 = K.route_topk(logits, pre, **kw)
  perm0, inv0, gs0, _ = K.sort_by_expert(idx0, e, want_sorted_experts=False)
  ws = K.gmm_workspace(t * k, e, "cuda")
  w, idx, perm, inv, gs = K.route_sort(logits, pre, gmm_workspace=ws, **kw)
  for a, b in ((w, w0), (idx, idx0), (perm, perm0), (inv, inv0), (gs, gs0)):
    assert torch.equal(a, b)
  d, f = 128, 256
  x = torch.randn((t * k, d), generator=g, device="cuda").to(torch.bfloat16)
  wq = torch.randint(-127, 128, (e, f, d), generator=g, device="cuda", dtype=torch.int8)
  sc = torch.rand((e, f), generator=g, device="cuda") * 0.01
  y = K.gmm_raw(x, wq, gs, rhs_scale=sc, workspace=ws, same_groups=True)
  assert torch.equal(y, K.gmm_raw(x, wq, gs0, rhs_scale=sc))


def test_flagged_matmuls_after_a_sort_that_maps_nothing_use_the_new_groups(K):
  """Two steps on the SAME group_sizes / workspace buffers above 4096 routed rows (where the sort maps nothing), each a
  sort followed by two grouped matmuls flagged MOE_GMM_SAME_GROUPS, as a serving loop with persistent buffers issues
  them: the second step's first matmul finds a record that matches in every field (same workspace, same group_sizes
  pointer, same sizes and tile height) and must still map the new routing."""
  e, k, t, d, f = 8, 2, 4096, 256, 512
  m = t * k
  ws = K.gmm_workspace(m, e, "cuda")
  g = torch.Generator(device="cuda").manual_seed(7)
  x = torch.randn((m, d), generator=g, device="cuda").to(torch.bfloat16)
  w1 = (torch.randn((e, f, d), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  w2 = (torch.randn((e, d, f), generator=g, device="cuda") * 0.05).to(torch.bfloat16)
  bufs = None
  for step, skew in enumerate((0.0, 3.0)):
    rng = np.random.default_rng(100 + step)
    p = np.exp(-skew * np.arange(e) / e)
    sel = np.stack([rng.choice(e, size=k, replace=False, p=p / p.sum()) for _ in range(t)]).astype(np.int32)
    bufs = K.sort_by_expert(cuda(sel), e, gmm_workspace=ws, out=bufs)
    gs = bufs[2]
    h = K.gmm_raw(x, w1, gs, workspace=ws, same_groups=True)
    y = K.gmm_raw(h, w2, gs, workspace=ws, same_groups=True)
    fresh = gs.clone()
    h0 = K.gmm_raw(x, w1, fresh)
    assert torch.equal(h, h0) and torch.equal(y, K.gmm_raw(h0, w2, fresh))
    assert torch.equal(gs.cpu(), torch.from_numpy(np.bincount(sel.reshape(-1), minlength=e).astype(np.int32)))


@pytest.mark.parametrize("m,n,sizes,offset,g_local", [(40, 64, [7, 0, 12, 1, 20], 0, 5), (300, 2880, [100, 0, 37, 63, 50], 1, 3), (64, 8, [70], 0, 1),
                                                     (513, 512, [3] * 100 + [0] * 28, 64, 64)])
def test_add_group_bias_bit_exact(K, m, n, sizes, offset, g_local):
  # bf16(h + bias[group of the row - offset]) on the rows of the local groups; rows of other groups and rows in no
  # group are copied (moe.py:1952-1957 as the differentiable path applies it)
  g = torch.Generator().manual_seed(m + n)
  h = torch.randn((m, n), generator=g).to(torch.bfloat16)
  bias = torch.randn((g_local, n), generator=g)
  gs = np.array(sizes, np.int32)
  ends = np.cumsum(gs)
  want = h.clone()
  for r in range(m):
    grp = int(np.searchsorted(ends, r, side="right"))
    if grp < len(sizes) and 0 <= grp - offset < g_local:
      want[r] = (h[r].float() + bias[grp - offset]).to(torch.bfloat16)
  got = K.add_group_bias(h.cuda(), bias.cuda(), cuda(gs), group_offset=offset)
  assert torch.equal(got.cpu().view(torch.int16), want.view(torch.int16))
