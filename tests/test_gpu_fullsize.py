"""GPU parity at the full sizes of the benchmark configurations.

The integer half of the path (top-k indices, perm, group_sizes) is compared bit-exactly against the
oracle over ALL tokens.  The floating-point half is checked three ways: (a) the WHOLE layer output of the
Mixtral, Qwen3 and GPT-OSS configurations against the whole-layer oracle (f32 accumulation on the host
cores; a few seconds each on the GPU box), (b) on a random sample of sorted rows, each recomputed by the
oracle's formula in f64 from the same quantised operands (per-row matmul against its expert's weights),
both stages of the expert MLP separately, and (c) through size-independent properties of the whole output
(finite, routing round trip, zero rows stay zero).
Tolerances: max|got-want| / max|want| <= 1e-2 and the elementwise rule of tests/tolerances.py.
"""

import numpy as np
import pytest
import torch

from oracle import moe_oracle as O
from tolerances import ELEM_ATOL_RMS_CHAINED, relerr

pytestmark = pytest.mark.gpu


def gmm_bf16(*args, **kwargs):
  """megablox.gmm with the layer dtype as preferred_element_type, as the reference's layer calls it (moe.py:1549)."""
  from maxtext_amd import megablox

  kwargs.setdefault("preferred_element_type", torch.bfloat16)
  return megablox.gmm(*args, **kwargs)
TOL = 1e-2
N_SAMPLE = 40


def _routing(wl, L):
  from maxtext_amd import moe

  cfg = wl.cfg
  r = moe.RoutedMoE(cfg, L["wi_0"], L["wi_1"], L["wo"])
  w, idx = r.get_topk(L["gate_logits"], L["pre_bias_logits"])
  k, e = cfg.num_experts_per_tok, cfg.num_experts
  logits = L["gate_logits"].cpu().numpy().reshape(-1, e)
  if cfg.is_deepseek:
    pre = L["pre_bias_logits"].cpu().numpy().reshape(-1, e)
    ow, oidx = O.get_topk(logits, pre, k=k, mode="deepseek", routed_scaling_factor=cfg.routed_scaling_factor)
    np.testing.assert_allclose(w.reshape(-1, k).cpu().numpy(), ow, rtol=1e-5)
  else:
    ow, oidx = O.get_topk(logits, k=k, norm_topk_prob=cfg.norm_topk_prob)
    np.testing.assert_allclose(w.reshape(-1, k).cpu().numpy(), ow, rtol=2.0**-6, atol=1e-6)
  np.testing.assert_array_equal(idx.reshape(-1, k).cpu().numpy(), oidx)
  return r, w, idx, oidx


def _dequant_rows(qa, expert, n_rows=None):
  """Rows [N, K] of one expert's weights as f64 with scales applied where they are not separable."""
  q = qa.qvalue[expert].cpu()
  if qa.qtype == "int8":
    return q.double(), qa.scale[expert].cpu().double()  # per-channel scale applied after the dot
  if qa.qtype == "int4":
    w = O.unpack_int4(q).double()
    s = torch.repeat_interleave(qa.scale[expert].cpu().double(), 128, dim=-1)[:, : w.shape[1]]
    return w * s, None
  raise ValueError(qa.qtype)


def _check_sampled_rows(wl, L, rows_q, rows_scale, inter, y, group_sizes, act_quant):
  """Recomputes `inter` (after wi_0/wi_1 + SwiGLU) and `y` (after wo) for a sample of sorted rows."""
  gs = group_sizes.cpu().numpy()
  offs = np.concatenate([[0], np.cumsum(gs)])
  m = int(offs[-1])
  rng = np.random.default_rng(0)
  bounds = np.concatenate([offs[:-1][gs > 0][:4], offs[1:][gs > 0][:4] - 1])  # first / last rows of groups
  picks = np.unique(np.concatenate([bounds, rng.integers(0, m, N_SAMPLE)]))[:N_SAMPLE]
  experts = np.searchsorted(offs, picks, side="right") - 1
  got_i, want_i, got_y, want_y = [], [], [], []
  cache = {}
  order = np.argsort(experts, kind="stable")  # one expert's weights at a time (a Mixtral expert is 1.4 GB in f64)
  for r, e in zip(picks[order], experts[order]):
    if e not in cache:
      cache.clear()
      cache[e] = (_dequant_rows(L["wi_0"], e), _dequant_rows(L["wi_1"], e), _dequant_rows(L["wo"], e))
    (w0, s0), (w1, s1), (wo, so) = cache[e]
    a = rows_q[r].cpu().double()
    a_s = 1.0 if rows_scale is None else float(rows_scale[r])
    h0 = (w0 @ a) * a_s * (s0 if s0 is not None else 1.0)
    h1 = (w1 @ a) * a_s * (s1 if s1 is not None else 1.0)
    want_i.append(O.apply_ffn_activation(h0.float(), h1.float(), wl.cfg.activation))
    got_i.append(inter[r].cpu())
    # the second matmul consumes the GPU's own intermediate row (re-quantised as the path does)
    b = inter[r].cpu()
    if act_quant == "int8":
      bq, bs = O.quantize_rows_int8(b[None].float())
      b, b_s = bq[0].double(), float(bs[0])
    else:
      b, b_s = b.double(), 1.0
    want_y.append(((wo @ b) * b_s * (so if so is not None else 1.0)).to(torch.bfloat16))
    got_y.append(y[r].cpu())
  gi, wi = torch.stack(got_i).float(), torch.stack(want_i).float()
  gy, wy = torch.stack(got_y).float(), torch.stack(want_y).float()
  assert float((gi - wi).abs().max() / wi.abs().max()) <= TOL
  assert float((gy - wy).abs().max() / wy.abs().max()) <= TOL
  return len(got_i)


@pytest.mark.parametrize("name", ["c2", "c4", "c5"])
def test_fullsize_int_weight_layers(name):
  from maxtext_amd import kernels, megablox, synthetic
  from maxtext_amd.quantizations import QArray

  wl = synthetic.workload(name)
  cfg = wl.cfg
  L = synthetic.make_layer(wl, device="cuda")
  r, w, idx, oidx = _routing(wl, L)
  k, e, d = cfg.num_experts_per_tok, cfg.num_experts, cfg.emb_dim
  t = wl.tokens
  # perm / group_sizes over all M rows, bit-exact against the stable argsort
  perm, inv, gs, se = kernels.sort_by_expert(idx.reshape(t, k).contiguous(), e)
  flat = oidx.reshape(-1)
  operm = np.argsort(flat, kind="stable").astype(np.int32)
  np.testing.assert_array_equal(perm.cpu().numpy(), operm)
  np.testing.assert_array_equal(gs.cpu().numpy(), np.bincount(flat, minlength=e).astype(np.int32))
  np.testing.assert_array_equal(se.cpu().numpy(), flat[operm])
  if name == "c4":
    assert (gs == 0).any().item(), "the Zipf workload must leave experts empty"
  x2d = L["x"].reshape(t, d)
  if cfg.act_quant == "int8":
    q, sc = kernels.gather_rows(x2d, perm, k, out_dtype=torch.int8)
    oq, osc = O.quantize_rows_int8(x2d.cpu()[torch.from_numpy(operm[:4096].astype(np.int64) // k)])
    assert torch.equal(q[:4096].cpu(), oq) and torch.equal(sc[:4096].cpu(), osc)
    rows, rows_q, rows_scale = QArray(q, sc, "int8"), q, sc.cpu().numpy()
  else:
    rows = kernels.gather_rows(x2d, perm, k)
    assert torch.equal(rows[:4096].cpu(), x2d.cpu()[torch.from_numpy(operm[:4096].astype(np.int64) // k)])
    rows_q, rows_scale = rows, None
  inter = gmm_bf16(rows, L["wi_0"], gs, transpose_rhs=True, rhs_up=L["wi_1"], fuse_act=cfg.activation)
  inter_in = megablox.quantize_lhs(inter, "int8") if cfg.act_quant == "int8" else inter
  y = gmm_bf16(inter_in, L["wo"], gs, transpose_rhs=True)
  assert torch.isfinite(inter.float()).all() and torch.isfinite(y.float()).all()
  n = _check_sampled_rows(wl, L, rows_q, rows_scale, inter, y, gs, cfg.act_quant)
  assert n >= 16
  # combine: with unit weights and y := sorted inputs the layer returns k * x (routing round trip)
  back = kernels.unpermute_combine(kernels.gather_rows(x2d, perm, k), torch.ones((t, k), device="cuda"), k=k, inv_perm=inv)
  assert torch.equal(back, (x2d.float() * k).to(torch.bfloat16))
  # and the real combine equals the f32 weighted sum of the rows it gathers, on a sample of tokens
  out = kernels.unpermute_combine(y, w.reshape(t, k).contiguous(), k=k, inv_perm=inv)
  toks = np.random.default_rng(1).integers(0, t, 64)
  invc, wc = inv.cpu().numpy().reshape(t, k), w.reshape(t, k).cpu().numpy()
  for tok in toks:
    want = sum(float(wc[tok, s]) * y[int(invc[tok, s])].float().cpu() for s in range(k)).to(torch.bfloat16)
    assert float((out[tok].float().cpu() - want.float()).abs().max()) <= 2.0**-7 * float(want.float().abs().max()) + 1e-6


@pytest.mark.parametrize("tokens", [None, 4096])
def test_fullsize_deepseek_fp8(tokens):
  """C3 at full size: 256 routed experts + shared expert resident, fp8 128x128 weights; at its own 256 tokens (9 rows per
  expert: the streaming kernel) and at 4096 tokens (143 rows per expert: the persistent 256 x 256 stream kernel)."""
  from maxtext_amd import kernels, megablox, synthetic
  from maxtext_amd.quantizations import QArray

  wl = synthetic.workload("c3", tokens)
  cfg = wl.cfg
  L = synthetic.make_layer(wl, device="cuda")
  r, w, idx, oidx = _routing(wl, L)
  k, e, d, f, t = cfg.num_experts_per_tok, cfg.num_experts, cfg.emb_dim, cfg.moe_mlp_dim, wl.tokens
  sel = torch.cat([idx.reshape(t, k), torch.full((t, 1), e, dtype=torch.int32, device="cuda")], 1).contiguous()
  perm, inv, gs, _ = kernels.sort_by_expert(sel, e + 1)
  flat = np.concatenate([oidx, np.full((t, 1), e, np.int32)], 1).reshape(-1)
  operm = np.argsort(flat, kind="stable").astype(np.int32)
  np.testing.assert_array_equal(perm.cpu().numpy(), operm)
  np.testing.assert_array_equal(gs.cpu().numpy(), np.bincount(flat, minlength=e + 1).astype(np.int32))
  x2d = L["x"].reshape(t, d)
  q, sc = kernels.gather_rows(x2d, perm, k + 1, out_dtype=torch.float8_e4m3fn, block_k=128)
  oq, osc = O.quantize_fp8_blocks(x2d.cpu()[torch.from_numpy(operm.astype(np.int64) // (k + 1))], 1, 128)
  assert torch.equal(q.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(sc.cpu(), osc)
  inter = gmm_bf16(QArray(q, sc, "fp8"), L["wi_0"], gs, transpose_rhs=True, rhs_up=L["wi_1"], fuse_act="silu")
  y = gmm_bf16(megablox.quantize_lhs(inter, "fp8", blocks=128), L["wo"], gs, transpose_rhs=True)
  assert torch.isfinite(y.float()).all()
  # sampled rows against the oracle's block-scaled formula (including rows of the shared expert)
  gsn = gs.cpu().numpy()
  offs = np.concatenate([[0], np.cumsum(gsn)])
  rng = np.random.default_rng(2)
  picks = np.concatenate([rng.integers(0, offs[-2], 24), rng.integers(offs[-2], offs[-1], 8)])
  got, want = [], []
  for rr in picks:
    ex = int(np.searchsorted(offs, rr, side="right") - 1)
    a = q[rr].cpu()[None]
    a_s = sc[rr].cpu()[None]
    one = np.array([1], np.int32)

    def proj(qa, lhs, lhs_s):
      wq = qa.qvalue[ex].cpu()[None]  # [1, n, k]
      n = wq.shape[1]
      ws = torch.repeat_interleave(qa.scale[ex].cpu()[None].permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
      return O.gmm(lhs, wq, one, lhs_scale=lhs_s, rhs_scale=ws, transpose_rhs=True, quant_block=128, out_dtype=torch.float32)

    it = O.apply_ffn_activation(proj(L["wi_0"], a, a_s), proj(L["wi_1"], a, a_s))
    got.append(inter[rr].cpu().float())
    want.append(it[0].float())
    bq, bs = O.quantize_fp8_blocks(inter[rr].cpu()[None], 1, 128)
    got.append(y[rr].cpu().float())
    want.append(proj(L["wo"], bq, bs)[0].to(torch.bfloat16).float())
  for g_, w_ in zip(got, want):
    assert float((g_ - w_).abs().max() / w_.abs().max().clamp_min(1e-30)) <= TOL


def test_fullsize_deepseek_whole_layer_output_against_oracle():
  """C3 as BASELINE states it (256 tokens, 256 routed experts top-8 + the shared expert, d 7168, f 2048, fp8 128 x 128
  weights, 1 x 128 activation scales): every element of the layer output, routed sum plus shared expert, against the CPU
  oracle on the identical quantised weights (generated on the GPU and copied; the oracle dequantises one expert and
  one K block at a time), and the integer half of the path over all rows."""
  from maxtext_amd import moe, synthetic
  from oracle.layer import oracle_layer

  wl = synthetic.workload("c3")
  cfg = wl.cfg
  L = synthetic.make_layer(wl, device="cuda")
  block = moe.RoutedAndSharedMoE(cfg, L["wi_0"], L["wi_1"], L["wo"])
  out, _, _ = block.sparse_matmul(L["x"], L["gate_logits"], L["pre_bias_logits"])
  torch.cuda.synchronize()
  trip = lambda qa: (qa.qvalue.cpu(), qa.scale.cpu(), qa.qtype)
  want, oidx, operm, ogs = oracle_layer(
      L["x"].cpu(), L["gate_logits"].cpu(), L["pre_bias_logits"].cpu(), trip(L["wi_0"]), trip(L["wi_1"]), trip(L["wo"]),
      num_experts=cfg.num_experts, k=cfg.num_experts_per_tok, emb_dim=cfg.emb_dim, mlp_dim=cfg.moe_mlp_dim, deepseek=True,
      routed_scaling_factor=cfg.routed_scaling_factor, shared_experts=cfg.shared_experts, act_quant=cfg.act_quant,
      activation=cfg.activation, acc_dtype=torch.float32)
  assert want.shape == (wl.tokens, cfg.emb_dim) and ogs.shape == (cfg.num_experts + 1,) and int(ogs[-1]) == wl.tokens
  got = out.reshape(want.shape)
  assert torch.isfinite(got.float()).all()
  # the second matmul of the two pipelines sees fp8 inputs that differ by one e4m3 step wherever the bf16 intermediates
  # differ by an ulp (the allowance the Mixtral layer's re-quantised activations get below)
  assert relerr(got, want, atol_rms=4e-2) <= TOL


@pytest.mark.parametrize("name", ["c2", "c4", "c5"])
def test_fullsize_whole_layer_output_against_oracle(name):
  """Every element of the layer output at BASELINE's full size (C2: 8192 x 4096, C4: 16384 x 2048, C5: 4096 x 2880) against
  the CPU oracle run on the identical quantised weights, plus the integer half of the path over all rows."""
  from maxtext_amd import moe, synthetic
  from maxtext_amd.quantizations import QArray
  from oracle.layer import oracle_layer

  wl = synthetic.workload(name)
  cfg = wl.cfg
  layer = synthetic.make_layer(wl, device="cpu")
  trip = synthetic.as_triple
  want, oidx, operm, ogs = oracle_layer(
      layer["x"], layer["gate_logits"], layer["pre_bias_logits"], trip(layer["wi_0"]), trip(layer["wi_1"]), trip(layer["wo"]),
      num_experts=cfg.num_experts, k=cfg.num_experts_per_tok, emb_dim=cfg.emb_dim, mlp_dim=cfg.moe_mlp_dim,
      norm_topk_prob=cfg.norm_topk_prob, act_quant=cfg.act_quant, activation=cfg.activation, acc_dtype=torch.float32)
  import dataclasses

  dev = lambda v: dataclasses.replace(v, qvalue=v.qvalue.cuda(), scale=v.scale.cuda()) if isinstance(v, QArray) else v.cuda()
  wi_0, wi_1, wo = dev(layer["wi_0"]), dev(layer["wi_1"]), dev(layer["wo"])
  block = moe.RoutedMoE(cfg, wi_0, wi_1, wo)
  x, logits = layer["x"].cuda(), layer["gate_logits"].cuda()
  out, _, _ = block.sparse_matmul(x, logits, None, wi_0, wi_1, wo)
  _, perm, _, gs, _, _, _, _ = block.permute(x, logits)
  np.testing.assert_array_equal(perm.cpu().numpy(), operm)
  np.testing.assert_array_equal(gs.cpu().numpy(), ogs)
  got = out.reshape(want.shape)
  assert torch.isfinite(got.float()).all()
  # With re-quantised activations (C2) the second matmul of the two pipelines sees int8 inputs that differ by one step
  # wherever the bf16 intermediates differ by an ulp: a noise of about 0.6 % of the output's rms per element, whose
  # maximum over 33 million elements reaches 3.3 %
  assert relerr(got, want, atol_rms=4e-2 if cfg.act_quant else ELEM_ATOL_RMS_CHAINED) <= TOL


def test_fullsize_fp8_row_by_channel_layer_stage_by_stage():
  """The forward of the fp8_full recipe at the Mixtral shape (8192 tokens, e4m3 rows x e4m3 channels on the stream kernel),
  every element of every stage against the CPU oracle.  An e4m3 re-quantisation in the middle of the chain makes two
  pipelines diverge by whole fp8 steps wherever their bf16 intermediates differ by an ulp (about 70 of a row's 14336
  values, 7 % of the output's rms at the worst of 33 million), so each oracle stage is fed the GPU's previous stage and the
  quantisers are compared bit for bit; the end-to-end output is then held to the max-norm bound only."""
  from maxtext_amd import kernels, megablox, synthetic

  wl = synthetic.workload("c2f8")
  cfg = wl.cfg
  L = synthetic.make_layer(wl, device="cuda")
  t, k, e, d = wl.tokens, cfg.num_experts_per_tok, cfg.num_experts, cfg.emb_dim
  w, idx = kernels.route_topk(L["gate_logits"].reshape(t, e).float().contiguous(), k=k, norm_topk_prob=cfg.norm_topk_prob)
  perm, inv, gs, _ = kernels.sort_by_expert(idx, e)
  x2d = L["x"].reshape(t, d)
  # stage 0: the activation quantiser, one scale per token row, bit for bit
  xq = megablox.quantize_lhs(x2d, "fp8")
  oq, osc = O.quantize_rows_fp8(x2d.cpu())
  assert torch.equal(xq.qvalue.cpu().view(torch.uint8), oq.view(torch.uint8)) and torch.equal(xq.scale.cpu(), osc)
  # stage 1: both first projections + SwiGLU, the rows read through the permutation
  inter = gmm_bf16(xq, L["wi_0"], gs, transpose_rhs=True, rhs_up=L["wi_1"], fuse_act=cfg.activation, lhs_row_idx=perm, lhs_row_idx_div=k)
  rows = torch.from_numpy(perm.cpu().numpy().astype(np.int64) // k)
  ogs = gs.cpu().numpy()
  kw = dict(lhs_scale=osc[rows], out_dtype=torch.float32, acc_dtype=torch.float32)
  tr = lambda qa: qa.qvalue.cpu().transpose(1, 2)
  h0 = O.gmm(oq[rows], tr(L["wi_0"]), ogs, rhs_scale=L["wi_0"].scale.cpu(), **kw)
  h1 = O.gmm(oq[rows], tr(L["wi_1"]), ogs, rhs_scale=L["wi_1"].scale.cpu(), **kw)
  assert relerr(inter, O.apply_ffn_activation(h0, h1, cfg.activation)) <= TOL
  del h0, h1
  # stage 2: the intermediate's quantiser bit for bit, then the second projection on the GPU's own intermediate
  iq = megablox.quantize_lhs(inter, "fp8")
  oiq, oisc = O.quantize_rows_fp8(inter.cpu())
  assert torch.equal(iq.qvalue.cpu().view(torch.uint8), oiq.view(torch.uint8)) and torch.equal(iq.scale.cpu(), oisc)
  y = gmm_bf16(iq, L["wo"], gs, transpose_rhs=True)
  want_y = O.gmm(oiq, tr(L["wo"]), ogs, rhs_scale=L["wo"].scale.cpu(), lhs_scale=oisc, acc_dtype=torch.float32)
  assert relerr(y, want_y) <= TOL
  # stage 3: the combine on the GPU's rows
  out = kernels.unpermute_combine(y, w, k=k, inv_perm=inv)
  want_out = O.unpermute(y.cpu(), perm.cpu().numpy(), w.cpu().numpy(), k)
  assert relerr(out, want_out) <= TOL
  # and the layer mirror gives these very values end to end
  from maxtext_amd import moe

  block = moe.RoutedMoE(cfg, L["wi_0"], L["wi_1"], L["wo"])
  full, _, _ = block.sparse_matmul(L["x"], L["gate_logits"], None, L["wi_0"], L["wi_1"], L["wo"])
  assert torch.equal(full.reshape(t, d), out)


@pytest.mark.parametrize("name,tokens", [("c4", 768), ("c5", 384), ("c5", 880), ("c5mx", 512)])
def test_mid_sized_weight_only_layers_against_oracle(name, tokens):
  """The token counts between decode and prefill (20 to 104 rows per expert), where the weight-only formats run the stream
  kernel on 128-row tiles with the permute fused in through the row index: every element against the CPU oracle."""
  from maxtext_amd import moe, synthetic
  from maxtext_amd.quantizations import QArray
  from oracle.layer import oracle_layer

  wl = synthetic.workload(name, tokens)
  cfg = wl.cfg
  layer = synthetic.make_layer(wl, device="cpu")
  trip = lambda qa: (qa.qvalue, qa.scale, qa.qtype)
  want, _, operm, ogs = oracle_layer(
      layer["x"], layer["gate_logits"], layer["pre_bias_logits"], trip(layer["wi_0"]), trip(layer["wi_1"]), trip(layer["wo"]),
      num_experts=cfg.num_experts, k=cfg.num_experts_per_tok, emb_dim=cfg.emb_dim, mlp_dim=cfg.moe_mlp_dim,
      norm_topk_prob=cfg.norm_topk_prob, act_quant=cfg.act_quant, activation=cfg.activation, acc_dtype=torch.float32)
  rows_per_expert = tokens * cfg.num_experts_per_tok / cfg.num_experts
  assert 16 < rows_per_expert < 112  # the regime
  if name == "c4":
    assert ogs.max() > 128  # skewed routing: groups that need a second tile
  dev = lambda v: QArray(v.qvalue.cuda(), v.scale.cuda(), v.qtype) if isinstance(v, QArray) else v.cuda()
  wi_0, wi_1, wo = dev(layer["wi_0"]), dev(layer["wi_1"]), dev(layer["wo"])
  block = moe.RoutedMoE(cfg, wi_0, wi_1, wo)
  out, _, _ = block.sparse_matmul(layer["x"].cuda(), layer["gate_logits"].cuda(), None, wi_0, wi_1, wo)
  got = out.reshape(want.shape)
  assert torch.isfinite(got.float()).all()
  assert relerr(got, want, atol_rms=ELEM_ATOL_RMS_CHAINED) <= TOL
