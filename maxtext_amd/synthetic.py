"""Seeded synthetic MoE layers for the five benchmark / parity configurations.

Tensors are created on the requested device with a generator seeded from the configuration, so
the CPU (parity tests, CPU baseline) and the GPU (benchmark) can each build the same recipe;
tests that compare bit-for-bit build on the CPU and copy.

  c1  tiny:      T 2048,  d 512,  f 1024,  E 8,   k 2, int8 per-channel weights, bf16 activations,
                 router weights f32 ~N(0, 0.02), softmax top-2
  c2  mixtral:   T 8192,  d 4096, f 14336, E 8,   k 2, int8 weights + int8 per-token activations
  c3  deepseek:  T 256,   d 7168, f 2048,  E 256, k 8 (+1 shared), fp8 128x128 weights, 1x128
                 activations, sigmoid scores with renormalisation x 2.5
  c4  qwen3:     T 16384, d 2048, f 768,   E 128, k 8, int8 weights, bf16 activations, router
                 logits biased by -1.2*log(rank) (Zipf popularity, some experts empty)
  c5  gpt-oss:   d 2880,  f 2880, E 32,    k 4, int4 group-128 weights, T in {1,16,128,1024,4096}
  c2f8           the c2 shape with float8_e4m3fn weights (one scale per output channel) and activations (one scale per
                 token): the operand layout of the fp8_full recipe (kernels/megablox/ops.py:232-267)
"""

from __future__ import annotations

import dataclasses
import math
from typing import Optional

import torch

from maxtext_amd import quantizations as Q
from maxtext_amd.moe import MoEConfig


@dataclasses.dataclass
class Workload:
  name: str
  tokens: int
  cfg: MoEConfig
  weight_quant: str  # "int8" | "fp8" (128 x 128 blocks) | "fp8c" (per channel) | "int4" | "mxfp4"
  seed: int
  zipf_s: float = 0.0
  router_from_weights: bool = False


def workload(name: str, tokens: Optional[int] = None) -> Workload:
  name = name.lower()
  if name == "c1":
    cfg = MoEConfig(8, 2, 512, 1024, model_name="tiny")
    return Workload("c1", tokens or 2048, cfg, "int8", 1235, router_from_weights=True)
  if name == "c2":
    cfg = MoEConfig(8, 2, 4096, 14336, model_name="mixtral-8x7b", act_quant="int8")
    return Workload("c2", tokens or 8192, cfg, "int8", 1236)
  if name == "c2f8":
    cfg = MoEConfig(8, 2, 4096, 14336, model_name="mixtral-8x7b", act_quant="fp8_row")
    return Workload("c2f8", tokens or 8192, cfg, "fp8c", 1241)
  if name == "c3":
    cfg = MoEConfig(256, 8, 7168, 2048, model_name="deepseek3-671b", decoder_block="deepseek", routed_scaling_factor=2.5,
                    routed_score_func="sigmoid", routed_bias=True, shared_experts=1, act_quant="fp8")
    return Workload("c3", tokens or 256, cfg, "fp8", 1237)
  if name == "c4":
    cfg = MoEConfig(128, 8, 2048, 768, model_name="qwen3-30b-a3b", decoder_block="qwen3_moe", norm_topk_prob=True)
    return Workload("c4", tokens or 16384, cfg, "int8", 1238, zipf_s=1.2)
  if name == "c5":
    cfg = MoEConfig(32, 4, 2880, 2880, model_name="gpt-oss-20b", decoder_block="mixtral")
    return Workload("c5", tokens or 4096, cfg, "int4", 1239)
  if name == "c5mx":  # the C5 shape with the weights in the format GPT-OSS checkpoints are stored in
    cfg = MoEConfig(32, 4, 2880, 2880, model_name="gpt-oss-20b", decoder_block="mixtral")
    return Workload("c5mx", tokens or 4096, cfg, "mxfp4", 1240)
  raise ValueError(f"unknown workload {name}")


def _quantize(w_gnk: torch.Tensor, kind: str) -> Q.QArray:
  if kind == "int8":
    return Q.quantize_weight_int8(w_gnk)
  if kind == "fp8":
    return Q.quantize_weight_fp8_blocks(w_gnk)
  if kind == "fp8c":
    return Q.quantize_weight_fp8_channel(w_gnk, share_across_experts=False)
  if kind == "int4":
    return Q.quantize_weight_int4(w_gnk)
  if kind == "mxfp4":
    return Q.quantize_weight_mxfp4(w_gnk)
  raise ValueError(kind)


def _expert_weights(gen, n_experts, n, k, kind, device, chunk=8) -> Q.QArray:
  """N(0, 0.02) weights [E, N, K], quantised `chunk` experts at a time to bound memory."""
  qs, ss = [], []
  for e0 in range(0, n_experts, chunk):
    e1 = min(e0 + chunk, n_experts)
    w = torch.randn((e1 - e0, n, k), generator=gen, device=device, dtype=torch.float32) * 0.02
    qa = _quantize(w, kind)
    qs.append(qa.qvalue)
    ss.append(qa.scale)
    del w
  if kind == "fp8c":
    return Q.QArray(torch.cat(qs), torch.cat(ss), "fp8", block_n=1, block_k=0)
  return Q.QArray(torch.cat(qs), torch.cat(ss), kind)


def make_layer(wl: Workload, device="cuda"):
  """-> dict(x [1,T,d] bf16, gate_logits [1,T,E] f32, pre_bias_logits or None, wi_0, wi_1, wo)."""
  cfg = wl.cfg
  dev = torch.device(device)
  gen = torch.Generator(device=dev).manual_seed(wl.seed)
  t, d, f, e = wl.tokens, cfg.emb_dim, cfg.moe_mlp_dim, cfg.num_experts
  x = torch.randn((t, d), generator=gen, device=dev, dtype=torch.float32).to(torch.bfloat16)
  pre_bias = None
  if wl.router_from_weights:
    wg = torch.randn((d, e), generator=gen, device=dev, dtype=torch.float32) * 0.02
    logits = x.float() @ wg
  else:
    logits = torch.randn((t, e), generator=gen, device=dev, dtype=torch.float32)
  if wl.zipf_s > 0:
    rank = torch.arange(1, e + 1, device=dev, dtype=torch.float32)
    logits = logits - wl.zipf_s * torch.log(rank) * 2.0
  if cfg.is_deepseek:
    pre_bias = torch.sigmoid(logits)
    bias = torch.randn((e,), generator=gen, device=dev, dtype=torch.float32) * 0.01
    logits = pre_bias + bias
  n_stack = e + (1 if cfg.shared_experts else 0)
  chunk = max(1, min(8, (1 << 28) // (d * f)))
  wi_0 = _expert_weights(gen, n_stack, f, d, wl.weight_quant, dev, chunk)
  wi_1 = _expert_weights(gen, n_stack, f, d, wl.weight_quant, dev, chunk)
  wo = _expert_weights(gen, n_stack, d, f, wl.weight_quant, dev, chunk)
  return dict(x=x.reshape(1, t, d), gate_logits=logits.reshape(1, t, e).contiguous(),
              pre_bias_logits=None if pre_bias is None else pre_bias.reshape(1, t, e).contiguous(),
              wi_0=wi_0, wi_1=wi_1, wo=wo)


def as_triple(qa: Q.QArray):
  """(qvalue, scale, kind) of a weight QArray, `kind` naming the scale layout as well: "fp8c" for float8 values with one
  scale per output channel ("fp8" alone means 128 x 128 blocks)."""
  kind = "fp8c" if qa.qtype == "fp8" and qa.block_n == 1 else qa.qtype
  return qa.qvalue, qa.scale, kind


def layer_flops(wl: Workload) -> float:
  """2*M*d*f per projection, three projections (+ the shared expert over all T rows)."""
  cfg = wl.cfg
  rows = wl.tokens * (cfg.num_experts_per_tok + (1 if cfg.shared_experts else 0))
  return 6.0 * rows * cfg.emb_dim * cfg.moe_mlp_dim


def weight_bytes_per_expert(wl: Workload) -> float:
  per = {"int8": 1.0, "fp8": 1.0, "fp8c": 1.0, "int4": 0.5, "mxfp4": 0.5}[wl.weight_quant]
  return 3.0 * wl.cfg.emb_dim * wl.cfg.moe_mlp_dim * per
