"""Whole-layer CPU oracle: the sparse MoE expert path on already-quantised weights.

TEST INFRASTRUCTURE ONLY (see oracle/moe_oracle.py).  Follows _moe_body of
src/maxtext/layers/moe.py:2186-2294: route -> permute -> gmm(w0), gmm(w1) -> activation ->
gmm(wo) -> unpermute, with the activation quantisers placed where the kernels place them
(before each grouped matmul).  Takes plain tensors so it imports nothing from the product.
"""

from __future__ import annotations

import numpy as np
import torch

from oracle import moe_oracle as O


def oracle_rhs(qvalue: torch.Tensor, scale: torch.Tensor, qtype: str, n: int):
  """Weights in the kernels' HBM layout ([G,N,K] K-contiguous; scales [G,N] / [G,N/128,K/128] /
  [G,N,K/128]) -> (rhs [g,k,n], rhs_scale in the reference's v2 layout [g,nb,1,n], quant_block)."""
  if qtype == "bf16":  # unquantised weights [G, N, K]
    return qvalue.cpu().transpose(1, 2), None, None
  qv, sc = qvalue.cpu(), scale.cpu()
  if qtype in ("int8", "fp8c"):  # one scale per output channel [G, N] (fp8c: float8_e4m3fn values)
    return qv.transpose(1, 2), sc, None
  if qtype == "fp8":
    s = torch.repeat_interleave(sc.permute(0, 2, 1), 128, dim=2)[:, :, None, :n]
    return qv.transpose(1, 2), s, 128
  if qtype == "int4":
    return O.unpack_int4(qv).transpose(1, 2), sc.float().permute(0, 2, 1)[:, :, None, :], 128
  if qtype == "mxfp4":
    g, nn, kb = qv.shape
    deq = O.dequantize_mxfp4(qv.reshape(g, nn, kb // 16, 16), sc).to(torch.bfloat16)  # exact: e2m1 * 2^e fits bf16
    return deq.transpose(1, 2), None, None
  raise ValueError(qtype)


def oracle_layer(x, gate_logits, pre_bias_logits, wi_0, wi_1, wo, *, num_experts, k, emb_dim, mlp_dim, deepseek=False,
                 routed_scaling_factor=1.0, norm_topk_prob=False, shared_experts=0, act_quant=None, activation="silu",
                 acc_dtype=torch.float64):
  """wi_0 / wi_1 / wo are (qvalue, scale, qtype) triples.  -> (out [T,d] bf16, idx, perm, group_sizes)."""
  e, d, f = num_experts, emb_dim, mlp_dim
  x = x.cpu().reshape(-1, d)
  logits = gate_logits.cpu().numpy().reshape(-1, e)
  if deepseek:
    pre = pre_bias_logits.cpu().numpy().reshape(-1, e)
    w, idx = O.get_topk(logits, pre, k=k, mode="deepseek", routed_scaling_factor=routed_scaling_factor)
  else:
    w, idx = O.get_topk(logits, k=k, norm_topk_prob=norm_topk_prob)
  n_exp = e
  if shared_experts:
    # the shared MLP (moe.py:3317-3321, :3360-3371), width shared_experts * mlp_dim, as shared_experts slices of width
    # mlp_dim: each is one more group owning every token with weight 1
    t_ = idx.shape[0]
    idx = np.concatenate([idx, np.broadcast_to(np.arange(e, e + shared_experts, dtype=np.int32), (t_, shared_experts))], 1)
    w = np.concatenate([w, np.ones((t_, shared_experts), np.float32)], 1)
    n_exp, k = e + shared_experts, k + shared_experts
  r0, s0, qb = oracle_rhs(*wi_0, f)
  r1, s1, _ = oracle_rhs(*wi_1, f)
  ro, so, _ = oracle_rhs(*wo, d)

  def quant(rows):
    if act_quant == "int8":
      return O.quantize_rows_int8(rows)
    if act_quant == "fp8":
      return O.quantize_fp8_blocks(rows, 1, 128)
    if act_quant == "fp8_row":
      return O.quantize_rows_fp8(rows)
    return rows, None

  def expert_fn(rows, gs):
    a, a_s = quant(rows)
    kw = dict(lhs_scale=a_s, quant_block=qb, out_dtype=torch.float32, acc_dtype=acc_dtype)
    h0 = O.gmm(a, r0, gs, rhs_scale=s0, **kw)
    h1 = O.gmm(a, r1, gs, rhs_scale=s1, **kw)
    inter = O.apply_ffn_activation(h0, h1, activation)
    b, b_s = quant(inter)
    return O.gmm(b, ro, gs, rhs_scale=so, lhs_scale=b_s, quant_block=qb, acc_dtype=acc_dtype)

  sorted_inputs, perm, gs, _ = O.permute(x, idx, n_exp)
  out = O.unpermute(expert_fn(sorted_inputs, gs), perm, w, k)
  return out, idx, perm, gs
