"""GPU parity of the whole expert path (route -> permute -> gmm x3 + SwiGLU -> combine) against
the oracle, on the benchmark configurations (C1 at full size, C2..C5 at reduced dims so the
CPU oracle finishes in seconds) plus size-independent properties at larger sizes.

Routing indices, perm and group sizes must match bit-exactly; outputs within
max|got-want| / max|want| <= 1e-2.
"""

import dataclasses

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


import functools

import tolerances

# whole layers are chains of three matmuls with bf16 (or re-quantised) intermediates
relerr = functools.partial(tolerances.relerr, atol_rms=tolerances.ELEM_ATOL_RMS_CHAINED)


def _small(name, tokens, **dims):
  from maxtext_amd import synthetic

  wl = synthetic.workload(name, tokens)
  return dataclasses.replace(wl, cfg=dataclasses.replace(wl.cfg, **dims))


def oracle_layer(wl, layer):
  """The same pipeline with oracle functions, consuming the identical quantised weights."""
  from oracle.layer import oracle_layer as run

  cfg = wl.cfg
  # (the oracle names fp8 weights with one scale per output channel "fp8c"; "fp8" there is the 128 x 128 block layout)
  trip = lambda qa: (qa.qvalue, qa.scale, "fp8c" if qa.qtype == "fp8" and qa.scale.dim() == 2 else qa.qtype)
  return run(layer["x"], layer["gate_logits"], layer["pre_bias_logits"], trip(layer["wi_0"]), trip(layer["wi_1"]), trip(layer["wo"]),
             num_experts=cfg.num_experts, k=cfg.num_experts_per_tok, emb_dim=cfg.emb_dim, mlp_dim=cfg.moe_mlp_dim,
             deepseek=cfg.is_deepseek, routed_scaling_factor=cfg.routed_scaling_factor, norm_topk_prob=cfg.norm_topk_prob,
             shared_experts=cfg.shared_experts, act_quant=cfg.act_quant, activation=cfg.activation)


def run_gpu(wl, layer_cpu):
  from maxtext_amd import moe
  from maxtext_amd.quantizations import QArray

  def dev(v):
    if isinstance(v, QArray):
      return dataclasses.replace(v, qvalue=v.qvalue.cuda(), scale=v.scale.cuda())
    return None if v is None else v.cuda()

  L = {k: dev(v) for k, v in layer_cpu.items()}
  cls = moe.RoutedAndSharedMoE if wl.cfg.shared_experts else moe.RoutedMoE
  block = cls(wl.cfg, L["wi_0"], L["wi_1"], L["wo"])
  if wl.cfg.shared_experts:
    out, _, _ = block.sparse_matmul(L["x"], L["gate_logits"], L["pre_bias_logits"])
  else:
    out, _, _ = block.sparse_matmul(L["x"], L["gate_logits"], L["pre_bias_logits"], L["wi_0"], L["wi_1"], L["wo"])
  return out, block, L


CASES = {
    "c1_full": lambda: _small("c1", 2048),
    "c2_small": lambda: _small("c2", 1024, emb_dim=1024, moe_mlp_dim=2048),
    # decode sizes of the 8-bit x 8-bit layers: 4, 24 and 40 rows per expert (the LDS-streamed kernel on 16-, 32- and 64-row tiles)
    "c2_t16": lambda: _small("c2", 16, emb_dim=1024, moe_mlp_dim=2048),
    "c2_t96": lambda: _small("c2", 96, emb_dim=1024, moe_mlp_dim=2048),
    "c2_t160": lambda: _small("c2", 160, emb_dim=1024, moe_mlp_dim=2048),
    "c2f8_t16": lambda: _small("c2f8", 16, emb_dim=1024, moe_mlp_dim=2048),
    "c2f8_t160": lambda: _small("c2f8", 160, emb_dim=1024, moe_mlp_dim=2048),
    "c3_small": lambda: _small("c3", 64, emb_dim=1024, moe_mlp_dim=512, num_experts=32),
    "c3_t32": lambda: _small("c3", 32, emb_dim=1024, moe_mlp_dim=512, num_experts=32),  # (8 rows per expert: the block-scaled decode kernel)
    "c4_small": lambda: _small("c4", 2048, emb_dim=512, moe_mlp_dim=256),
    # the GPT-OSS shape at its full dimensions (32 experts, d = f = 2880) over the token sweep; 4096 tokens run in
    # tests/test_gpu_fullsize.py
    "c5_t1": lambda: _small("c5", 1),
    "c5_t16": lambda: _small("c5", 16),
    "c5_t128": lambda: _small("c5", 128),
    "c5_t1024": lambda: _small("c5", 1024),
    "c5mx_t16": lambda: _small("c5mx", 16, num_experts=8),
    "c5mx_t1024": lambda: _small("c5mx", 1024, num_experts=4, moe_mlp_dim=1024),
}


@pytest.mark.parametrize("case", list(CASES))
def test_layer_matches_oracle(case):
  from maxtext_amd import synthetic

  wl = CASES[case]()
  layer = synthetic.make_layer(wl, device="cpu")
  want, oidx, operm, ogs = oracle_layer(wl, layer)
  got, block, L = run_gpu(wl, layer)
  # the integer half of the path, bit-exact
  r = block.routed if wl.cfg.shared_experts else block
  _, idx = r.get_topk(L["gate_logits"], L["pre_bias_logits"])
  k = wl.cfg.num_experts_per_tok
  np.testing.assert_array_equal(idx.reshape(-1, k).cpu().numpy(), oidx[:, :k])
  if not wl.cfg.shared_experts:
    _, perm, _, gs, _, _, _, _ = r.permute(L["x"], L["gate_logits"], L["pre_bias_logits"])
    np.testing.assert_array_equal(perm.cpu().numpy(), operm)
    np.testing.assert_array_equal(gs.cpu().numpy(), ogs)
  assert got.shape == layer["x"].shape and got.dtype == torch.bfloat16
  assert relerr(got.reshape(want.shape), want) <= TOL


def test_permute_unpermute_api_roundtrip():
  # unpermute(permute(x)) with unit weights returns k*x exactly (property, any size)
  from maxtext_amd import moe

  t, d, e, k = 4096, 1024, 64, 4
  cfg = moe.MoEConfig(e, k, d, 128)
  block = moe.RoutedMoE(cfg, None, None, None)
  g = torch.Generator(device="cuda").manual_seed(3)
  x = torch.randn((1, t, d), generator=g, device="cuda").to(torch.bfloat16)
  logits = torch.randn((1, t, e), generator=g, device="cuda")
  sorted_inputs, perm, weights, group_size, sorted_experts, _, _, _ = block.permute(x, logits)
  assert int(group_size.sum()) == t * k
  assert torch.equal(torch.sort(perm.long())[0], torch.arange(t * k, device="cuda"))
  assert torch.all(sorted_experts[1:] >= sorted_experts[:-1])
  assert torch.equal(torch.bincount(sorted_experts.long(), minlength=e).int(), group_size)
  out = block.unpermute(sorted_inputs, perm, torch.ones_like(weights), 1, t)
  assert torch.equal(out, (x.float() * k).to(torch.bfloat16))


def test_permute_roll_to_expert_id():
  # permute(roll_to_expert_id=r) (moe.py:953-954): rows of experts r, r+1, ... come first; against the oracle's permute
  from maxtext_amd import moe

  t, d, e, k, roll = 257, 64, 16, 2, 12
  cfg = moe.MoEConfig(e, k, d, 128)
  block = moe.RoutedMoE(cfg, None, None, None)
  g = torch.Generator(device="cuda").manual_seed(4)
  x = torch.randn((1, t, d), generator=g, device="cuda").to(torch.bfloat16)
  logits = torch.randn((1, t, e), generator=g, device="cuda")
  sorted_inputs, perm, weights, group_size, sorted_experts, _, _, _ = block.permute(x, logits, roll_to_expert_id=roll)
  _, sel = block.get_topk(logits)
  want = O.permute(x[0].cpu(), sel.reshape(t, k).cpu().numpy(), e, roll_to_expert_id=roll)
  assert torch.equal(sorted_inputs.cpu(), want[0])
  np.testing.assert_array_equal(perm.cpu().numpy(), want[1])
  np.testing.assert_array_equal(group_size.cpu().numpy(), want[2])
  np.testing.assert_array_equal(sorted_experts.cpu().numpy(), want[3])
  out = block.unpermute(sorted_inputs, perm, torch.ones_like(weights), 1, t)
  assert torch.equal(out, (x.float() * k).to(torch.bfloat16))


def test_megablox_gmm_api():
  from maxtext_amd import megablox

  g = torch.Generator().manual_seed(11)
  m, kd, n, e = 512, 256, 384, 4
  lhs = torch.randn(m, kd, generator=g).to(torch.bfloat16)
  rhs = (torch.randn(e, kd, n, generator=g) * 0.05).to(torch.bfloat16)  # reference default layout [g, k, n]
  gs = np.array([100, 0, 312, 100], np.int32)
  want = O.gmm(lhs, rhs, gs)
  got = gmm_bf16(lhs.cuda(), rhs.cuda(), torch.from_numpy(gs).cuda())
  assert relerr(got, want) <= TOL
  got_t = gmm_bf16(lhs.cuda(), rhs.transpose(1, 2).contiguous().cuda(), torch.from_numpy(gs).cuda(), transpose_rhs=True)
  assert torch.equal(got, got_t)
  # the default result type is the reference's float32 (ops.py:50), with and without gradients
  dflt = megablox.gmm(lhs.cuda(), rhs.cuda(), torch.from_numpy(gs).cuda())
  assert dflt.dtype == torch.float32 and relerr(dflt, O.gmm(lhs, rhs, gs, out_dtype=torch.float32)) <= 1e-3
  lg = lhs.cuda().requires_grad_()
  dg = megablox.gmm(lg, rhs.cuda(), torch.from_numpy(gs).cuda())
  assert dg.dtype == torch.float32
  dg.sum().backward()
  assert lg.grad is not None and lg.grad.dtype == torch.bfloat16
  # dynamic int8 on both sides (ops.py:232-267): close to the unquantised product (quantizations_test.py:653: < 0.2)
  got_q = gmm_bf16(lhs.cuda(), rhs.cuda(), torch.from_numpy(gs).cuda(), lhs_quantize_dtype="int8", rhs_quantize_dtype="int8")
  assert (got_q.float().cpu() - want.float()).abs().mean() / want.float().abs().mean() < 0.2
  with pytest.raises(ValueError):
    gmm_bf16(lhs.cuda(), rhs.cuda(), torch.from_numpy(gs.astype(np.int64)).cuda())
  with pytest.raises(ValueError):
    gmm_bf16(lhs.cuda()[None], rhs.cuda(), torch.from_numpy(gs).cuda())


def test_layer_linearity_at_benchmark_width():
  # property at C2's real width (d 4096, f 14336): with bf16 activations and int8 weights the layer is
  # positively homogeneous in the wo weights' scales: doubling wo's scales doubles the output exactly.
  from maxtext_amd import moe, synthetic
  from maxtext_amd.quantizations import QArray

  wl = _small("c2", 512, act_quant=None)
  layer = synthetic.make_layer(wl, device="cuda")
  block = moe.RoutedMoE(wl.cfg, layer["wi_0"], layer["wi_1"], layer["wo"])
  out1, _, _ = block.sparse_matmul(layer["x"], layer["gate_logits"], None, layer["wi_0"], layer["wi_1"], layer["wo"])
  wo2 = QArray(layer["wo"].qvalue, layer["wo"].scale * 2, "int8")
  out2, _, _ = block.sparse_matmul(layer["x"], layer["gate_logits"], None, layer["wi_0"], layer["wi_1"], wo2)
  assert torch.isfinite(out1.float()).all()
  assert torch.equal(out2.float(), out1.float() * 2)


# ---------------------------------------------------------------- training: gradients of the whole layer


def test_combine_bwd_matches_bruteforce():
  from maxtext_amd import kernels

  g = torch.Generator().manual_seed(4)
  t, k, d = 37, 3, 264
  y = torch.randn(t * k, d, generator=g).to(torch.bfloat16)
  dout = torch.randn(t, d, generator=g).to(torch.bfloat16)
  w = torch.rand(t, k, generator=g)
  inv = torch.randperm(t * k, generator=g).to(torch.int32)
  dy, dw = kernels.unpermute_combine_bwd(dout.cuda(), y.cuda(), w.cuda(), k=k, inv_perm=inv.cuda())
  rows = inv.long().reshape(t, k)
  want_dy = torch.zeros(t * k, d)
  want_dy[rows.reshape(-1)] = (w[:, :, None] * dout.float()[:, None, :]).reshape(t * k, d)
  want_dw = (y.float()[rows] * dout.float()[:, None, :]).sum(-1)
  assert torch.equal(dy.cpu(), want_dy.to(torch.bfloat16))  # one rounding of an exact f32 product
  assert relerr(dw, want_dw) <= 1e-5
  dy1, none = kernels.unpermute_combine_bwd(dout.cuda(), None, None, k=k, inv_perm=inv.cuda(), need_dweights=False)
  assert none is None
  want1 = torch.zeros(t * k, d, dtype=torch.bfloat16)
  want1[rows.reshape(-1)] = dout[:, None, :].expand(t, k, d).reshape(t * k, d)
  assert torch.equal(dy1.cpu(), want1)


@pytest.mark.parametrize("norm_topk_prob", [False, True])
def test_layer_gradients_match_torch_autograd(norm_topk_prob):
  """Forward + backward of RoutedMoE with bf16 weights (gate -> top-k -> permute -> gmm x3 -> combine)
  against torch autograd through the per-token formulation of tests/unit/moe_test.py:344-411
  (sum over the selected experts of weight * MLP_e(x)) in f64, on the indices the GPU selected."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(21)
  t, d, f, e, k = 192, 128, 256, 4, 2
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  wg = (torch.randn(d, e, generator=g) * 0.1)
  w0 = (torch.randn(e, f, d, generator=g) * 0.08).to(torch.bfloat16)
  w1 = (torch.randn(e, f, d, generator=g) * 0.08).to(torch.bfloat16)
  wo = (torch.randn(e, d, f, generator=g) * 0.08).to(torch.bfloat16)
  dout = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, norm_topk_prob=norm_topk_prob)
  leaves = [v.cuda().requires_grad_() for v in (x, wg, w0, w1, wo)]
  xg, wgg, w0g, w1g, wog = leaves
  block = moe.RoutedMoE(cfg, w0g, w1g, wog, gate_kernel=wgg)
  out, _, _ = block(xg)
  out.backward(dout.cuda())
  # the indices the kernel chose (no gradient flows through them)
  with torch.no_grad():
    logits, _ = block.gate(xg.reshape(t, d))
    _, idx = block.get_topk(logits)
  idx = idx.reshape(t, k).cpu().long()

  r = [v.double().requires_grad_() for v in (x, wg, w0, w1, wo)]
  xr, wgr, w0r, w1r, wor = r
  x2 = xr.reshape(t, d)
  lg = x2 @ wgr
  wts = torch.softmax(torch.gather(lg, -1, idx), -1)
  if norm_topk_prob:
    wts = wts / wts.sum(-1, keepdim=True)
  ref = torch.zeros(t, d, dtype=torch.float64)
  for s in range(k):
    ex = idx[:, s]
    h0 = torch.einsum("td,tfd->tf", x2, w0r[ex])
    h1 = torch.einsum("td,tfd->tf", x2, w1r[ex])
    y = torch.einsum("tf,tdf->td", torch.nn.functional.silu(h0) * h1, wor[ex])
    ref = ref + wts[:, s : s + 1] * y
  (ref * dout.double().reshape(t, d)).sum().backward()
  assert relerr(out.reshape(t, d), ref) <= 2e-2
  # bf16 intermediates on the way back (dy, d inter, d h0/h1 are each rounded to bf16): 3e-2 of the max
  for got, want, name in zip(leaves, r, ("x", "gate", "wi_0", "wi_1", "wo")):
    assert got.grad is not None and got.grad.shape == got.shape, name
    # (each gradient is a sum of products of values that were rounded to bf16 two or three times on the way back)
    assert relerr(got.grad, want.grad, atol_rms=5e-2) <= 3e-2, name


def test_layer_gradients_with_int8_quantised_forward():
  """With act_quant="int8" the forward quantises both operands of each GEMM and the backward runs on the quantised
  residuals with the scales folded into the gradient (ops.py:530-580): gradients stay within the quantisation
  noise of the bf16 run."""
  import dataclasses as dc

  from maxtext_amd import moe

  g = torch.Generator().manual_seed(22)
  t, d, f, e, k = 128, 128, 128, 4, 2
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  logits = torch.randn(1, t, e, generator=g)
  ws = [(torch.randn(e, n_, k_, generator=g) * 0.08).to(torch.bfloat16) for n_, k_ in ((f, d), (f, d), (d, f))]
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f)
  grads = {}
  for q in (None, "int8"):
    leaves = [v.cuda().requires_grad_() for v in [x] + ws]
    block = moe.RoutedMoE(dc.replace(cfg, act_quant=q), *leaves[1:])
    out, _, _ = block.sparse_matmul(leaves[0], logits.cuda(), None, *leaves[1:])
    out.float().square().sum().backward()
    grads[q] = [v.grad for v in leaves]
  for a, b in zip(grads[None], grads["int8"]):
    # two different computations (quantised against unquantised forward): only the max-norm criterion applies
    assert relerr(b, a, elementwise=False) <= 5e-2


def test_layer_gradients_with_expert_biases():
  """mlp_bias layer (GPT-OSS, moe.py:617-637): gradients of the inputs, the three weights and the three per-expert
  biases against torch autograd through the per-token loop in f64, on the GPU's routing."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(23)
  t, d, f, e, k = 160, 128, 128, 4, 2
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  logits = torch.randn(1, t, e, generator=g)
  w0, w1, wo = [(torch.randn(e, n_, k_, generator=g) * 0.08).to(torch.bfloat16) for n_, k_ in ((f, d), (f, d), (d, f))]
  b0, b1, bo = torch.randn(e, f, generator=g) * 0.5, torch.randn(e, f, generator=g) * 0.5, torch.randn(e, d, generator=g) * 0.5
  dout = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f)
  leaves = [v.cuda().requires_grad_() for v in (x, w0, w1, wo, b0, b1, bo)]
  block = moe.RoutedMoE(cfg, *leaves[1:4])
  out, _, _ = block.sparse_matmul(leaves[0], logits.cuda(), None, *leaves[1:4], *leaves[4:])
  out.backward(dout.cuda())
  with torch.no_grad():
    wts, idx = block.get_topk(logits.cuda())
  idx, wts = idx.reshape(t, k).cpu().long(), wts.reshape(t, k).cpu().double()
  r = [v.double().requires_grad_() for v in (x, w0, w1, wo, b0, b1, bo)]
  xr, w0r, w1r, wor, b0r, b1r, bor = r
  x2 = xr.reshape(t, d)
  ref = torch.zeros(t, d, dtype=torch.float64)
  for s_ in range(k):
    ex = idx[:, s_]
    h0 = torch.einsum("td,tfd->tf", x2, w0r[ex]) + b0r[ex]
    h1 = torch.einsum("td,tfd->tf", x2, w1r[ex]) + b1r[ex]
    ref = ref + wts[:, s_ : s_ + 1] * (torch.einsum("tf,tdf->td", torch.nn.functional.silu(h0) * h1, wor[ex]) + bor[ex])
  (ref * dout.double().reshape(t, d)).sum().backward()
  assert relerr(out.reshape(t, d), ref) <= 2e-2
  for got, want, name in zip(leaves, r, ("x", "wi_0", "wi_1", "wo", "b0", "b1", "bo")):
    assert got.grad is not None and got.grad.shape == got.shape, name
    # (each gradient is a sum of products of values that were rounded to bf16 two or three times on the way back)
    assert relerr(got.grad, want.grad, atol_rms=5e-2) <= 3e-2, name


# ---------------------------------------------------------------- graph replay


@pytest.mark.parametrize("case", ["c1_full", "c3_small", "c5_t16", "c2_t16", "c2_t160", "c2f8_t16", "c3_t32"])
def test_graph_replay_equals_eager(case):
  """A captured layer call replayed several times, with eager work and synchronisations in between and new
  inputs each time, must reproduce the eager result bit for bit."""
  from maxtext_amd import graph, synthetic

  wl = CASES[case]()
  layer = synthetic.make_layer(wl, device="cpu")
  _, block, L = run_gpu(wl, layer)
  x, logits, pre = L["x"], L["gate_logits"], L["pre_bias_logits"]
  g = graph.GraphedLayer(block, x, logits, pre)
  gen = torch.Generator(device="cuda").manual_seed(3)
  for it in range(4):
    xi = (torch.randn(x.shape, device="cuda", generator=gen)).to(torch.bfloat16)
    li = torch.randn(logits.shape, device="cuda", generator=gen)
    pi = None if pre is None else torch.sigmoid(li)
    if pre is not None:
      li = pi + 0.01 * torch.randn(logits.shape, device="cuda", generator=gen)
    if wl.cfg.shared_experts:
      want = block.sparse_matmul(xi, li, pi)[0]
    else:
      want = block.sparse_matmul(xi, li, pi, L["wi_0"], L["wi_1"], L["wo"])[0]
    torch.cuda.synchronize()
    got = g(xi, li, pi).clone()
    torch.cuda.synchronize()
    assert torch.equal(got, want), f"replay {it}"
    _ = (xi.float() @ xi.float().transpose(-1, -2)).sum().item()  # unrelated eager work between replays


# ---------------------------------------------------------------- router inside the layer call


@pytest.mark.parametrize("deepseek", [False, True])
def test_layer_call_routes_through_gate_route(deepseek):
  """block(x) computes the gate inside the HIP path; it must equal sparse_matmul fed with the logits that
  the same entry point reports (identical routing by construction), and the torch gate within tolerance."""
  from maxtext_amd import moe, quantizations

  g = torch.Generator().manual_seed(40)
  t, d, f, e, k = 300, 256, 512, 16, 4
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16).cuda()
  wg = (torch.randn(d, e, generator=g) * 0.1).cuda()
  bias = (torch.randn(e, generator=g) * 0.1).cuda() if deepseek else None
  ws = [(torch.randn(e + (1 if deepseek else 0), n_, k_, generator=g) * 0.05).to(torch.bfloat16).cuda() for n_, k_ in ((f, d), (f, d), (d, f))]
  if deepseek:
    cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, model_name="deepseek3-test",
                        routed_score_func="sigmoid", routed_bias=True, routed_scaling_factor=2.5, shared_experts=1)
    block = moe.RoutedAndSharedMoE(cfg, *ws, gate_kernel=wg, gate_bias=bias)
    routed = block.routed
  else:
    cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f)
    block = routed = moe.RoutedMoE(cfg, *ws, gate_kernel=wg)
  out, _, _ = block(x)
  w, idx, logits, pre = routed.gate_and_route(x.reshape(t, d), return_logits=True)
  if deepseek:
    want, _, _ = block.sparse_matmul(x, logits.reshape(1, t, e), pre.reshape(1, t, e))
  else:
    want, _, _ = block.sparse_matmul(x, logits.reshape(1, t, e), None, *ws)
  assert torch.equal(out, want)
  tl, tp = routed.gate(x.reshape(t, d))
  assert float((tl - logits).abs().max()) <= 1e-4 * float(tl.abs().max())


def test_gpt_oss_style_layer_with_mlp_bias():
  """GPT-OSS variant (gpt-oss-20b.yml:44-49): clipped swigluoai activation and per-expert biases on all three
  projections, against the per-token loop formulation in f64 on the GPU's own routing."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(50)
  t, d, f, e, k = 160, 192, 320, 8, 4
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  logits = torch.randn(1, t, e, generator=g)
  w0, w1 = [(torch.randn(e, f, d, generator=g) * 0.1).to(torch.bfloat16) for _ in range(2)]
  wo = (torch.randn(e, d, f, generator=g) * 0.1).to(torch.bfloat16)
  b0, b1, bo = torch.randn(e, f, generator=g) * 0.3, torch.randn(e, f, generator=g) * 0.3, torch.randn(e, d, generator=g) * 0.3
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, decoder_block="gpt_oss", mlp_activations_limit=7.0)
  block = moe.RoutedMoE(cfg, w0.cuda(), w1.cuda(), wo.cuda())
  out, _, _ = block.sparse_matmul(x.cuda(), logits.cuda(), None, w0.cuda(), w1.cuda(), wo.cuda(), b0.cuda(), b1.cuda(), bo.cuda())
  w, idx = block.get_topk(logits.cuda())
  w, idx = w.reshape(t, k).cpu().double(), idx.reshape(t, k).cpu().long()
  x2 = x.reshape(t, d).double()
  want = torch.zeros(t, d, dtype=torch.float64)
  for s_ in range(k):
    ex = idx[:, s_]
    h0 = torch.einsum("td,tfd->tf", x2, w0.double()[ex]) + b0.double()[ex]
    h1 = torch.einsum("td,tfd->tf", x2, w1.double()[ex]) + b1.double()[ex]
    a = O.apply_ffn_activation(h0.float(), h1.float(), "swigluoai", 7.0).double()
    want += w[:, s_ : s_ + 1] * (torch.einsum("tf,tdf->td", a, wo.double()[ex]) + bo.double()[ex])
  assert relerr(out.reshape(t, d), want) <= TOL


def test_auxiliary_outputs_match_reference_formulas():
  """lb_loss (moe.py:2662-2687) and bias_updates (moe.py:215-236, known answer of tests/unit/moe_test.py:328-341)
  as returned by sparse_matmul / __call__."""
  import dataclasses as dc

  from maxtext_amd import moe

  # the reference's own vector: 4 experts, indices [[0,1],[0,2],[0,3]] -> sign(1.5 - [3,1,1,1]) * rate
  upd = moe.calculate_load_balance_updates(torch.tensor([[[0, 1], [0, 2], [0, 3]]]), 4, 0.1)
  assert torch.allclose(upd, torch.tensor([-0.1, 0.1, 0.1, 0.1]))
  assert np.allclose(O.calculate_load_balance_updates(np.array([[[0, 1], [0, 2], [0, 3]]]), 4, 0.1), upd.numpy())

  g = torch.Generator().manual_seed(61)
  b, s_, d, f, e, k = 2, 96, 128, 128, 8, 2
  x = torch.randn(b, s_, d, generator=g).to(torch.bfloat16).cuda()
  logits = torch.randn(b, s_, e, generator=g).cuda()
  ws = [(torch.randn(e, n_, k_, generator=g) * 0.05).to(torch.bfloat16).cuda() for n_, k_ in ((f, d), (f, d), (d, f))]
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, load_balance_loss_weight=0.01,
                      routed_bias=True, routed_bias_update_rate=0.001)
  block = moe.RoutedMoE(cfg, *ws)
  out, lb, upd = block.sparse_matmul(x, logits, None, *ws)
  _, idx = block.get_topk(logits)
  idx = idx.cpu().long()
  # brute force per sequence
  probs = torch.softmax(logits.cpu().float(), -1).to(torch.bfloat16).float()
  want = 0.0
  for bi in range(b):
    dens = torch.bincount(idx[bi].reshape(-1), minlength=e).float() / s_
    want += float((dens * probs[bi].mean(0)).mean())
  want = want / b * e * e * 0.01
  assert abs(float(lb) - want) <= 1e-4 * abs(want)
  cnt = torch.bincount(idx.reshape(-1), minlength=e).float()
  assert torch.equal(upd.cpu(), torch.sign(b * s_ * k / e - cnt) * 0.001)
  # without the config keys nothing is returned
  _, lb0, upd0 = moe.RoutedMoE(dc.replace(cfg, load_balance_loss_weight=0.0, routed_bias_update_rate=0.0), *ws).sparse_matmul(x, logits, None, *ws)
  assert lb0 is None and upd0 is None


def test_llama4_and_gemma4_style_layers():
  """Llama4: top-1, token scaled by sigmoid(router logit) before the expert, combine with ones (moe.py:902-906, :1051).
  Gemma4: weights = softmax over all experts at the top-k, renormalised, times a per-expert scale (moe.py:742-763).
  Both against the per-token loop in f64 on the GPU's routing."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(70)
  t, d, f, e = 200, 128, 256, 8
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  logits = torch.randn(1, t, e, generator=g)
  ws = [(torch.randn(e, n_, k_, generator=g) * 0.08).to(torch.bfloat16) for n_, k_ in ((f, d), (f, d), (d, f))]
  scale = torch.rand(e, generator=g) + 0.5

  def expert(xrow, ex):
    h0 = torch.einsum("td,tfd->tf", xrow, ws[0].double()[ex])
    h1 = torch.einsum("td,tfd->tf", xrow, ws[1].double()[ex])
    return torch.einsum("tf,tdf->td", torch.nn.functional.silu(h0) * h1, ws[2].double()[ex])

  # Llama4
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=1, emb_dim=d, moe_mlp_dim=f, decoder_block="llama4")
  block = moe.RoutedMoE(cfg, *[w.cuda() for w in ws])
  out, _, _ = block.sparse_matmul(x.cuda(), logits.cuda(), None, *[w.cuda() for w in ws])
  top = logits.reshape(t, e).max(-1)
  xs = (x.reshape(t, d).float() * torch.sigmoid(top.values.float())[:, None]).to(torch.bfloat16).double()
  want = expert(xs, top.indices)
  assert relerr(out.reshape(t, d), want) <= TOL
  # Gemma4
  k = 2
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, decoder_block="gemma4", norm_topk_prob=True)
  block = moe.RoutedMoE(cfg, *[w.cuda() for w in ws])
  block.per_expert_scale = scale.cuda()
  out, _, _ = block.sparse_matmul(x.cuda(), logits.cuda(), None, *[w.cuda() for w in ws])
  w_gpu, idx = block.get_topk(logits.cuda())
  idx = idx.reshape(t, k).cpu().long()
  probs = torch.softmax(logits.reshape(t, e).double(), -1)
  wsel = torch.gather(probs, -1, idx)
  wsel = wsel / wsel.sum(-1, keepdim=True) * scale.double()[idx]  # normalised first, then scaled (moe.py:755-763)
  assert relerr(w_gpu.reshape(t, k), wsel) <= 2.0**-6
  x2 = x.reshape(t, d).double()
  want = sum(wsel[:, s_ : s_ + 1] * expert(x2, idx[:, s_]) for s_ in range(k))
  assert relerr(out.reshape(t, d), want) <= 2e-2


def test_hash_routed_layer():
  """DeepSeek-V4 hash routing (moe.py:729-738) with the sqrtsoftplus router score (linears.py:51-53): experts come from
  the token-id table, weights from the scores at those experts; the layer output against the per-token loop in f64."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(71)
  t, d, f, e, k, vocab = 96, 128, 128, 8, 2, 50
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  wg = torch.randn(d, e, generator=g) * 0.1
  ws = [(torch.randn(e, n_, k_, generator=g) * 0.08).to(torch.bfloat16) for n_, k_ in ((f, d), (f, d), (d, f))]
  table = torch.stack([torch.randperm(e, generator=g)[:k] for _ in range(vocab)]).float()
  ids = torch.randint(0, vocab, (1, t), generator=g)
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, model_name="deepseek4", decoder_block="deepseek4",
                      routed_score_func="sqrtsoftplus", routed_scaling_factor=1.5)
  assert cfg.is_deepseek
  block = moe.RoutedMoE(cfg, *[w.cuda() for w in ws], gate_kernel=wg.cuda())
  block.tid2eid = table.cuda()
  out, _, _ = block(x.cuda(), input_ids=ids.cuda())
  scores = torch.sqrt(torch.nn.functional.softplus(x.reshape(t, d).float() @ wg))
  ow, oidx = O.hash_routing(scores.numpy(), table.numpy(), ids.reshape(t).numpy(), routed_score_func="sqrtsoftplus", routed_scaling_factor=1.5)
  w_gpu, idx_gpu = block.get_topk(scores.reshape(1, t, e).cuda(), scores.reshape(1, t, e).cuda(), input_ids=ids.cuda())
  np.testing.assert_array_equal(idx_gpu.reshape(t, k).cpu().numpy(), oidx)
  np.testing.assert_allclose(w_gpu.reshape(t, k).cpu().numpy(), ow, rtol=1e-5)
  x2 = x.reshape(t, d).double()
  want = torch.zeros(t, d, dtype=torch.float64)
  for s_ in range(k):
    ex = torch.as_tensor(oidx[:, s_]).long()
    h0 = torch.einsum("td,tfd->tf", x2, ws[0].double()[ex])
    h1 = torch.einsum("td,tfd->tf", x2, ws[1].double()[ex])
    want += torch.as_tensor(ow[:, s_ : s_ + 1]).double() * torch.einsum("tf,tdf->td", torch.nn.functional.silu(h0) * h1, ws[2].double()[ex])
  assert relerr(out.reshape(t, d), want) <= 2e-2


def test_routed_and_shared_block_with_two_shared_experts_gate_inputs_and_aux_outputs():
  """RoutedAndSharedMoE.__call__ (moe.py:3338-3371): the shared MLP of width shared_experts * mlp_dim as that many
  stacked slices, the gate reading gate_inputs, and the routed block's auxiliary outputs handed through.  Expected
  value: the routed layer of the oracle plus a dense gated MLP of width 2 f in f64."""
  from maxtext_amd import moe

  g = torch.Generator().manual_seed(90)
  t, d, f, e, k, sh = 192, 256, 128, 8, 2, 2
  x = torch.randn(1, t, d, generator=g).to(torch.bfloat16)
  gate_in = torch.randn(1, t, d, generator=g).to(torch.bfloat16)  # the router looks at other activations than the experts
  wg = torch.randn(d, e, generator=g) * 0.1
  bias = torch.randn(e, generator=g) * 0.1
  ws = [(torch.randn(e + sh, n_, k_, generator=g) * 0.05).to(torch.bfloat16) for n_, k_ in ((f, d), (f, d), (d, f))]
  cfg = moe.MoEConfig(float32_gate_logits=True, num_experts=e, num_experts_per_tok=k, emb_dim=d, moe_mlp_dim=f, model_name="deepseek3-test",
                      routed_score_func="sigmoid", routed_bias=True, routed_scaling_factor=2.5, shared_experts=sh,
                      load_balance_loss_weight=0.01, routed_bias_update_rate=0.001)
  block = moe.RoutedAndSharedMoE(cfg, *[w.cuda() for w in ws], gate_kernel=wg.cuda(), gate_bias=bias.cuda())
  out, lb, upd = block(x.cuda(), gate_inputs=gate_in.cuda())
  # routing as the block saw it, from gate_inputs
  w_r, idx, logits, pre = block.routed.gate_and_route(gate_in.cuda().reshape(t, d), return_logits=True)
  want_logits, want_pre = O.gate_logits(gate_in.reshape(t, d), wg, bias, score_func="sigmoid", deepseek=True)
  assert np.abs(logits.cpu().numpy() - want_logits).max() <= 1e-5
  from oracle.layer import oracle_layer as run_oracle

  trip = lambda w: (w[:e], None, "bf16")
  routed, oidx, _, _ = run_oracle(x, logits.cpu(), pre.cpu(), trip(ws[0]), trip(ws[1]), trip(ws[2]), num_experts=e, k=k, emb_dim=d, mlp_dim=f,
                                    deepseek=True, routed_scaling_factor=2.5)
  np.testing.assert_array_equal(idx.cpu().numpy(), oidx)
  x64 = x.reshape(t, d).double()
  w0s, w1s, wos = ws[0][e:].double().reshape(sh * f, d), ws[1][e:].double().reshape(sh * f, d), ws[2][e:].double()
  inter = torch.nn.functional.silu(x64 @ w0s.T) * (x64 @ w1s.T)  # [t, sh * f]: one MLP of width 2 f
  shared = inter @ torch.cat([wos[i] for i in range(sh)], 1).T
  want = routed.double() + shared
  assert relerr(out.reshape(t, d), want) <= 2e-2
  # auxiliary outputs are the routed block's own
  _, lb_r, upd_r = block.routed.sparse_matmul(x.cuda(), logits.reshape(1, t, e), pre.reshape(1, t, e), *[w.cuda()[:e].contiguous() for w in ws])
  assert lb is not None and upd is not None and torch.equal(lb, lb_r) and torch.equal(upd, upd_r)
  with pytest.raises(ValueError):
    moe.RoutedAndSharedMoE(cfg, *[w.cuda()[: e + 1] for w in ws])
