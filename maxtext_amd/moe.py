"""Host-side mirror of the reference's sparse MoE expert path, driving the HIP kernels.

Mirrors the method surface of RoutedMoE in src/maxtext/layers/moe.py: get_topk (:717),
permute (:872), unpermute (:1004), apply_ffn_activation (:841, fused into the first GEMM),
sparse_matmul (:1403) and __call__ (:3143), plus RoutedAndSharedMoE (:3259).  Only the
single-device dropless `sparse_matmul=True` branch exists here; arrays are torch CUDA tensors.
"""

from __future__ import annotations

import dataclasses
from typing import Optional

import torch

from maxtext_amd import kernels, megablox
from maxtext_amd.quantizations import QArray


@dataclasses.dataclass
class MoEConfig:
  """The MoE keys of src/maxtext/configs/base.yml:212-298 that the expert path reads."""

  num_experts: int
  num_experts_per_tok: int
  emb_dim: int
  moe_mlp_dim: int
  model_name: str = "mixtral-8x7b"  # "deepseek3-*" selects DeepSeek routing (moe.py:744)
  decoder_block: str = "mixtral"  # "gpt_oss" selects the clipped activation (moe.py:844)
  norm_topk_prob: bool = False
  routed_scaling_factor: float = 1.0
  routed_score_func: str = ""  # "sigmoid" for DeepSeek-V3
  routed_bias: bool = False
  n_routing_groups: int = -1
  topk_routing_group: int = -1
  mlp_activations_limit: float = -1.0
  float32_weight_sum: bool = True
  float32_gate_logits: bool = False  # configs/base.yml:198
  shared_experts: int = 0
  # activation quantisation for the grouped GEMMs: None | "int8" (one scale per row) | "fp8" (the DeepSeek recipe: one
  # scale per row and 128 values of K, against 128 x 128 weight blocks) | "fp8_row" (one scale per row, against per-channel
  # weight scales: what gmm() quantises to, kernels/megablox/ops.py:241-260)
  act_quant: Optional[str] = None
  # the reference's quantisation keys that reach the grouped matmuls (configs/base.yml; moe.py:1554-1556): only
  # quantization == "fp8_full" together with use_qwix_quantization quantises them, by the rule of
  # layers/quantizations.py:798-855 (e4m3 weights and activations, e5m2 gradients, the three calibration methods)
  quantization: str = ""
  use_qwix_quantization: bool = False
  weight_quantization_calibration_method: str = "absmax"
  act_quantization_calibration_method: str = "absmax"
  bwd_quantization_calibration_method: str = "absmax"
  load_balance_loss_weight: float = 0.0  # > 0: permute / sparse_matmul return the auxiliary loss (moe.py:888-891)
  routed_bias_update_rate: float = 0.0  # > 0 with routed_bias: return the loss-free balancing update (moe.py:893-898)

  @property
  def gmm_quantization_rule(self):
    """The QtRule the grouped matmuls run under, or None (get_fp8_full_qwix_rule_w_sparsity,
    layers/quantizations.py:798-821; only "fp8_full" names "gmm" among its op_names)."""
    if self.quantization != "fp8_full" or not self.use_qwix_quantization:
      return None
    from maxtext_amd.quantizations import QtRule

    return QtRule(weight_qtype="float8_e4m3fn", act_qtype="float8_e4m3fn", bwd_qtype="float8_e5m2",
                  weight_calibration_method=self.weight_quantization_calibration_method,
                  act_calibration_method=self.act_quantization_calibration_method,
                  bwd_calibration_method=self.bwd_quantization_calibration_method)

  @property
  def is_deepseek(self) -> bool:
    return self.model_name.startswith(("deepseek3", "deepseek4"))

  @property
  def route_mode(self) -> str:
    """Weight rule of get_topk (moe.py:738-756)."""
    if self.is_deepseek:
      return "deepseek"
    if self.decoder_block == "llama4":
      return "topk_raw"  # raw top-k logits; sigmoid of them scales the inputs in permute (moe.py:902-906)
    if self.decoder_block == "gemma4":
      return "softmax_all"  # softmax over all experts read at the top-k indices (moe.py:742-745)
    return "softmax_topk"

  @property
  def activation(self) -> str:
    if self.decoder_block == "gpt_oss":
      return "swigluoai"
    if self.is_deepseek and self.mlp_activations_limit > 0.0:
      return "silu_clip"
    return "silu"


def calculate_load_balance_updates(top_k_indices: torch.Tensor, num_experts: int, rate: float) -> torch.Tensor:
  """Bias adjustment sign(average_load - expert_load) * rate, shape [num_experts] (moe.py:215-236)."""
  flat = top_k_indices.reshape(-1).long()
  counts = torch.bincount(flat, minlength=num_experts).float()
  return torch.sign(flat.numel() / num_experts - counts) * rate


class _GatherRowsFn(torch.autograd.Function):
  """Row gather sorted[i] = x[perm[i] // k] with the custom VJP of moe.py:154-171: the gradient of a
  token is the sum of the gradients of its k copies, gathered through the inverse permutation."""

  @staticmethod
  def forward(ctx, x2d, perm, inv_perm, k):
    ctx.save_for_backward(inv_perm)
    ctx.k = k
    return kernels.gather_rows(x2d, perm, k)

  @staticmethod
  def backward(ctx, dsorted):
    (inv_perm,) = ctx.saved_tensors
    return kernels.unpermute_combine(dsorted.contiguous(), None, k=ctx.k, inv_perm=inv_perm), None, None, None


class _CombineFn(torch.autograd.Function):
  """unpermute + weighted sum (moe.py:1039-1062) with gradients for the expert outputs and the weights."""

  @staticmethod
  def forward(ctx, y, weights, inv_perm, k):
    ctx.save_for_backward(y, weights, inv_perm)
    ctx.k = k
    return kernels.unpermute_combine(y, weights, k=k, inv_perm=inv_perm)

  @staticmethod
  def backward(ctx, dout):
    y, weights, inv_perm = ctx.saved_tensors
    dy, dw = kernels.unpermute_combine_bwd(dout.contiguous(), y, weights, k=ctx.k, inv_perm=inv_perm,
                                           need_dweights=ctx.needs_input_grad[1])
    return dy, dw, None, None


class RoutedMoE:
  """Routed experts: top-k routing, permute, three grouped GEMMs with fused SwiGLU, combine.

  Expert weights are held in the kernels' layout [E, N, K] (K contiguous): `wi_0`, `wi_1` are
  [E, moe_mlp_dim, emb_dim] and `wo` is [E, emb_dim, moe_mlp_dim], each a bf16 tensor or a
  quantizations.QArray.  `gate_kernel` is [emb_dim, E] (GateLogit, moe.py:247); `gate_bias` [E].
  """

  def __init__(self, config: MoEConfig, wi_0, wi_1, wo, gate_kernel=None, gate_bias=None):
    self.config = config
    self.num_experts = config.num_experts
    self.num_experts_per_tok = config.num_experts_per_tok
    self.wi_0, self.wi_1, self.wo = wi_0, wi_1, wo
    self.gate_kernel, self.gate_bias = gate_kernel, gate_bias
    self._gate_terms = None  # [S, E, d] bf16 form of gate_kernel for moe_gate_route, built on first use
    self.per_expert_scale = None  # [E] f32, Gemma4: multiplies the routing weights (moe.py:758-763)
    self.tid2eid = None  # [vocab, k] token id -> expert ids: DeepSeek-V4 hash routing (moe.py:443-454, :729-738)
    # when set to a list, _experts appends (stage, start_event, end_event) recorded on the launch stream
    self.profile_events = None

  # -- GateLogit.__call__ (moe.py:353-392): upstream of the kernels' boundary -----------------
  def gate(self, inputs_2d: torch.Tensor):
    cfg = self.config
    x = inputs_2d.float() if cfg.float32_gate_logits else inputs_2d
    out = (x @ self.gate_kernel.to(x.dtype)).float()
    if cfg.routed_score_func == "sigmoid":
      out = torch.sigmoid(out)
    elif cfg.routed_score_func == "sqrtsoftplus":  # DeepSeek-V4 router (linears.py:51-53)
      out = torch.sqrt(torch.nn.functional.softplus(out))
    elif cfg.routed_score_func:
      raise NotImplementedError(cfg.routed_score_func)
    pre_bias = out if cfg.is_deepseek else None
    if self.gate_bias is not None and self.tid2eid is None:  # a hash-routed layer has no gate bias (moe.py:499)
      out = out + self.gate_bias.float()
    return out.contiguous(), pre_bias

  # -- GateLogit.__call__ + get_topk through one entry point (no [T, E] round trip through torch) ---------
  def gate_and_route(self, inputs_2d: torch.Tensor, return_logits: bool = False):
    """-> (weights [T,k] f32, indices [T,k] int32[, gate_logits, pre_bias_logits])."""
    cfg = self.config
    if cfg.routed_score_func not in ("", "sigmoid", "sqrtsoftplus"):
      raise NotImplementedError(cfg.routed_score_func)
    if self._gate_terms is None or self._gate_terms.device != inputs_2d.device:
      from maxtext_amd.quantizations import split_gate_kernel

      self._gate_terms = split_gate_kernel(self.gate_kernel, 3 if cfg.float32_gate_logits else 1).to(inputs_2d.device)
    bias = None if self.gate_bias is None else self.gate_bias.float().contiguous()
    common = dict(k=self.num_experts_per_tok, score_func=cfg.routed_score_func, gate_round_bf16=not cfg.float32_gate_logits,
                  return_logits=return_logits)
    x = inputs_2d.to(torch.bfloat16).contiguous()
    if cfg.is_deepseek:
      return kernels.gate_route(x, self._gate_terms, bias, mode="deepseek",
                                norm_topk_prob=cfg.routed_score_func in ("sigmoid", "sqrtsoftplus"),
                                routed_scaling_factor=cfg.routed_scaling_factor, n_routing_groups=cfg.n_routing_groups,
                                topk_routing_group=cfg.topk_routing_group, **common)
    r = kernels.gate_route(x, self._gate_terms, bias, mode=cfg.route_mode, norm_topk_prob=cfg.norm_topk_prob,
                           weights_round_bf16=cfg.route_mode != "topk_raw", **common)
    return (self._scale_per_expert(r[0], r[1]),) + tuple(r[1:])

  def _scale_per_expert(self, w, idx):
    if self.per_expert_scale is None:
      return w
    return w * self.per_expert_scale.float()[idx.long()]

  # -- auxiliary outputs of permute (moe.py:886-900) ------------------------------------------
  def load_balance_loss(self, top_k_indices: torch.Tensor, probs: torch.Tensor) -> torch.Tensor:
    """Sequence-wise load-balance loss (moe.py:2662-2687): per sequence, token density per expert times mean
    routing probability per expert, averaged, times E^2 * load_balance_loss_weight.  top_k_indices [B,S,k],
    probs [B,S,E]."""
    e = self.num_experts
    b, s_, k = top_k_indices.shape
    counts = torch.zeros((b, e), dtype=torch.float32, device=probs.device)
    counts.scatter_add_(1, top_k_indices.reshape(b, s_ * k).long(), torch.ones((b, s_ * k), dtype=torch.float32, device=probs.device))
    density = counts / s_
    density_prob = probs.float().mean(dim=1)
    return (density * density_prob).mean() * (e**2) * self.config.load_balance_loss_weight

  def _aux_outputs(self, gate_logits, selected):
    cfg = self.config
    lb_loss = bias_updates = None
    if cfg.load_balance_loss_weight > 0.0 and gate_logits is not None:
      probs = torch.softmax(gate_logits.float(), dim=-1).to(torch.bfloat16)
      lb_loss = self.load_balance_loss(selected, probs)
    if cfg.routed_bias and cfg.routed_bias_update_rate > 0.0:
      bias_updates = calculate_load_balance_updates(selected, self.num_experts, cfg.routed_bias_update_rate)
    return lb_loss, bias_updates

  # -- get_topk (moe.py:717-765) ------------------------------------------------------------
  def get_topk(self, gate_logits: torch.Tensor, pre_bias_logits: Optional[torch.Tensor] = None, input_ids=None):
    cfg = self.config
    if self.tid2eid is not None:
      return self._hash_routing(pre_bias_logits if pre_bias_logits is not None else gate_logits, input_ids)
    shape = gate_logits.shape[:-1]
    g2 = gate_logits.reshape(-1, gate_logits.shape[-1]).float().contiguous()
    if cfg.is_deepseek:
      p2 = pre_bias_logits.reshape(g2.shape).float().contiguous()
      w, idx = kernels.route_topk(
          g2, p2, k=self.num_experts_per_tok, mode="deepseek",
          norm_topk_prob=cfg.routed_score_func in ("sigmoid", "sqrtsoftplus"),
          routed_scaling_factor=cfg.routed_scaling_factor, n_routing_groups=cfg.n_routing_groups,
          topk_routing_group=cfg.topk_routing_group)
    else:
      # Llama4's raw logits skip the cast to the layer dtype (moe.py:752-753): they keep the gate's dtype
      w, idx = kernels.route_topk(g2, k=self.num_experts_per_tok, mode=cfg.route_mode, norm_topk_prob=cfg.norm_topk_prob,
                                  weights_round_bf16=cfg.route_mode != "topk_raw")
      w = self._scale_per_expert(w, idx)
    k = self.num_experts_per_tok
    if torch.is_grad_enabled() and (gate_logits.requires_grad or (pre_bias_logits is not None and pre_bias_logits.requires_grad)):
      w = self._weights_with_grad(gate_logits, pre_bias_logits, idx.reshape(*shape, k))
    return w.reshape(*shape, k), idx.reshape(*shape, k)

  def _get_topk_sorted(self, gate_logits, pre_bias_logits, ws):
    """get_topk and the sort of permute through one library call (one launch at decode sizes): -> (weights [..., k],
    indices [..., k], perm, inv_perm, group_sizes).  For calls without hash routing and without gradients."""
    cfg = self.config
    shape, k = gate_logits.shape[:-1], self.num_experts_per_tok
    g2 = gate_logits.reshape(-1, gate_logits.shape[-1]).float().contiguous()
    if cfg.is_deepseek:
      p2 = pre_bias_logits.reshape(g2.shape).float().contiguous()
      w, idx, perm, inv, gs = kernels.route_sort(
          g2, p2, k=k, gmm_workspace=ws, mode="deepseek", norm_topk_prob=cfg.routed_score_func in ("sigmoid", "sqrtsoftplus"),
          routed_scaling_factor=cfg.routed_scaling_factor, n_routing_groups=cfg.n_routing_groups, topk_routing_group=cfg.topk_routing_group)
    else:
      w, idx, perm, inv, gs = kernels.route_sort(g2, k=k, gmm_workspace=ws, mode=cfg.route_mode, norm_topk_prob=cfg.norm_topk_prob,
                                                 weights_round_bf16=cfg.route_mode != "topk_raw")
      w = self._scale_per_expert(w, idx)
    return w.reshape(*shape, k), idx.reshape(*shape, k), perm, inv, gs

  def _hash_routing(self, scores, input_ids):
    """Hash routing (moe.py:729-738): the experts of a token are read from a table indexed by its id, the weights are
    the scores at those experts, scaled as for DeepSeek (moe.py:767-773).  A table lookup and a gather: torch ops,
    differentiable in the scores."""
    cfg = self.config
    if input_ids is None:
      raise ValueError("input_ids cannot be None when is_hash_routing is True")
    idx = self.tid2eid.to(torch.int32)[input_ids.long()]  # [..., k]
    w = torch.gather(scores.float(), -1, idx.long())
    if cfg.is_deepseek:
      if cfg.routed_score_func in ("sigmoid", "sqrtsoftplus"):
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
      w = w * cfg.routed_scaling_factor
    else:
      w = torch.softmax(w, -1).to(torch.bfloat16).float()
      if cfg.norm_topk_prob:
        w = w / w.sum(-1, keepdim=True)
    return w, idx.contiguous()

  def _weights_with_grad(self, gate_logits, pre_bias_logits, idx):
    """The weight half of get_topk in differentiable torch ops, on the indices the kernel selected
    (moe.py:747-756 and :767-773, :838); top-k indices carry no gradient."""
    cfg = self.config
    gi = idx.long()
    if cfg.is_deepseek:
      w = torch.gather(pre_bias_logits.float(), -1, gi)
      if cfg.routed_score_func in ("sigmoid", "sqrtsoftplus"):
        w = w / (w.sum(-1, keepdim=True) + 1e-20)
      return w * cfg.routed_scaling_factor
    if cfg.route_mode == "topk_raw":
      w = torch.gather(gate_logits.float(), -1, gi)  # no cast to the layer dtype for Llama4 (moe.py:752-753)
    elif cfg.route_mode == "softmax_all":
      w = torch.gather(torch.softmax(gate_logits.float(), -1), -1, gi).to(torch.bfloat16)
    else:
      w = torch.softmax(torch.gather(gate_logits.float(), -1, gi), -1).to(torch.bfloat16)
    if cfg.norm_topk_prob:
      w = w / w.sum(-1, keepdim=True)
    if self.per_expert_scale is not None:
      w = w * self.per_expert_scale.to(w.dtype)[gi]
    return w.float()

  def _scale_inputs_by_router_score(self, x2d, weights):
    """Llama4 scales each token by sigmoid(router score) before the experts (moe.py:902-906); the reference's
    broadcast of [T, d] * [T, k] only exists for top-1."""
    if self.config.decoder_block != "llama4":
      return x2d
    if self.num_experts_per_tok != 1:
      raise NotImplementedError("Llama4 routing scales the token by its single router score (num_experts_per_tok == 1)")
    return (x2d.float() * torch.sigmoid(weights.reshape(-1, 1).float())).to(x2d.dtype)

  # -- permute (moe.py:872-1002), non-ragged branch -----------------------------------------
  def permute(self, inputs, gate_logits, pre_bias_logits=None, use_custom_sort_vjp=True, rngs=None,
              roll_to_expert_id=None, input_ids=None):
    """-> (sorted_inputs, sorted_selected_experts, weights, group_size, sorted_experts,
    lb_loss, bias_updates, local_group_size), as moe.py:993-1002."""
    b, s, d = inputs.shape
    x2d = inputs.reshape(b * s, d).contiguous()
    weights, selected = self.get_topk(gate_logits, pre_bias_logits, input_ids=input_ids)
    x2d = self._scale_inputs_by_router_score(x2d, weights)
    sel2d = selected.reshape(b * s, -1).contiguous()
    # roll_to_expert_id (a host integer here; the reference passes shard index * experts per shard): ids are sorted as
    # (id - roll) mod E, so that the calling shard's experts come first (moe.py:953-954)
    roll = 0 if roll_to_expert_id is None else int(roll_to_expert_id) % self.num_experts
    perm, inv, group_size, sorted_experts = kernels.sort_by_expert(sel2d, self.num_experts, roll_to_expert_id=roll)
    if torch.is_grad_enabled() and x2d.requires_grad:
      sorted_inputs = _GatherRowsFn.apply(x2d, perm, inv, self.num_experts_per_tok)
    else:
      sorted_inputs = kernels.gather_rows(x2d, perm, self.num_experts_per_tok)
    self._last_inv_perm = inv
    lb_loss, bias_updates = self._aux_outputs(gate_logits, selected)
    return sorted_inputs, perm, weights, group_size, sorted_experts, lb_loss, bias_updates, None

  # -- expert-parallel dispatch bookkeeping on one shard (moe.py:1066-1401): the exchange itself is a collective ----
  @staticmethod
  def local_permute(inputs, global_group_sizes, local_expert_size, shard_index, is_offset=False, global_sorted_experts=None,
                    use_custom_sort_vjp=True, use_ragged_sort=False, ragged_buffer_factor=-1.0, use_single_sparsecore=False):
    """-> (sorted_inputs, sorted_indices, local_group_size, sorted_experts_ids), as moe.py:1091-1200.
    inputs [rows, emb_dim] bf16; global_group_sizes [batch shards, num_experts] int32 on the device.
    use_ragged_sort moves only the rows that carry tokens (the first sum(local_group_size)); the rest of
    sorted_inputs is zeros (a2a_ragged_sort leaves it unspecified)."""
    rows = inputs.shape[0]
    if is_offset and global_sorted_experts is None:
      raise ValueError("is_offset=True needs global_sorted_experts")
    keys, local_group_size = kernels.local_expert_keys(
        global_group_sizes, local_expert_size, shard_index, rows,
        global_sorted_experts=global_sorted_experts if is_offset else None, truncate=ragged_buffer_factor > 0.0)
    sorted_indices, inv, _, sorted_experts_ids = kernels.sort_by_expert(keys.reshape(rows, 1), local_expert_size + 1)
    row_range = None
    if use_ragged_sort:
      row_range = torch.stack([torch.zeros((), dtype=torch.int32, device=inputs.device), local_group_size.sum().to(torch.int32)])
    if torch.is_grad_enabled() and inputs.requires_grad:
      if row_range is not None:  # a2a_ragged_sort with its custom VJP (kernels/ragged/ragged_sort.py:454-537)
        from maxtext_amd import ragged_sort

        sorted_inputs = ragged_sort._A2aSortFn.apply(inputs, sorted_indices, row_range)
      else:
        sorted_inputs = _GatherRowsFn.apply(inputs, sorted_indices, inv, 1)
    else:
      sorted_inputs = kernels.gather_rows(inputs.contiguous(), sorted_indices, 1, row_range=row_range)
    return sorted_inputs, sorted_indices, local_group_size, sorted_experts_ids

  @staticmethod
  def get_all_to_all_params(all_shards_group_sizes, shard_id, num_expert_parallelism, is_batch_sharded=True,
                            ragged_buffer_factor=-1.0, buffer_size=None, is_dispatch=True):
    """-> (input_offsets, send_sizes, output_offsets, recv_sizes) for ragged_all_to_all, as moe.py:1202-1349."""
    if ragged_buffer_factor > 0.0 and buffer_size is None:
      raise ValueError("ragged_buffer_factor > 0 needs buffer_size")
    return kernels.all_to_all_params(all_shards_group_sizes, shard_id, num_expert_parallelism, is_batch_sharded=is_batch_sharded,
                                     buffer_size=buffer_size if ragged_buffer_factor > 0.0 else None, is_dispatch=is_dispatch)

  @staticmethod
  def get_ragged_buffer_size(local_batch, ep_degree, global_experts, top_k, ragged_buffer_factor):
    """Rows of the ragged receive buffer (moe.py:1368-1401): the balanced share times the factor (tokens beyond it are
    dropped), or the worst case: min(ep_degree, global_experts / top_k) times the share."""
    if ragged_buffer_factor > 0.0:
      return int(local_batch * ragged_buffer_factor)
    return int(local_batch * min(ep_degree, global_experts / top_k))

  # -- unpermute (moe.py:1004-1063), non-ragged branch --------------------------------------
  def unpermute(self, intermediate, sorted_selected_experts, weights, batch_size, sequence_length,
                use_custom_sort_vjp=True, group_sizes=None, inv_perm=None):
    k = self.num_experts_per_tok
    w = weights.reshape(-1, k).float().contiguous()
    if not self.config.float32_weight_sum:
      # moe.py:1053-1061 without the casts: a bf16 x bf16 einsum, whose products are exact in the f32 accumulator and whose
      # result is rounded once -- the same kernel, fed with the weights as the layer dtype holds them
      w = w.to(torch.bfloat16).float()
    if self.config.decoder_block == "llama4":
      w = torch.ones_like(w)  # the router score already scaled the inputs (moe.py:1051-1052)
    if torch.is_grad_enabled() and (intermediate.requires_grad or w.requires_grad):
      if inv_perm is None:
        inv_perm = torch.empty_like(sorted_selected_experts)
        inv_perm[sorted_selected_experts.long()] = torch.arange(inv_perm.numel(), dtype=torch.int32, device=inv_perm.device)
      out = _CombineFn.apply(intermediate.contiguous(), w, inv_perm, k)
    else:
      out = kernels.unpermute_combine(intermediate.contiguous(), w, k=k,
                                      perm=None if inv_perm is not None else sorted_selected_experts,
                                      inv_perm=inv_perm)
    return out.reshape(batch_size, sequence_length, -1)

  # -- the three grouped GEMMs: gmm_up + apply_ffn_activation + wo (moe.py:1932-1986, :841, :2226)
  def _experts(self, sorted_inputs, group_size, w0, w1, wo, w0_bias=None, w1_bias=None, wo_bias=None, row_idx=None, row_idx_div=1,
               workspace=None, row_inv=None):
    """row_idx / row_idx_div: `sorted_inputs` holds the T token rows (plain or quantised) and row i of the first product
    reads row row_idx[i] // row_idx_div of it: the permute fused into the matmul, no [M, d] copy."""
    cfg = self.config
    act, limit = cfg.activation, (cfg.mlp_activations_limit if cfg.mlp_activations_limit > 0 else 7.0)
    bf16 = torch.bfloat16  # preferred_element_type=self.dtype of the reference's calls (moe.py:1549)
    ev = self.profile_events
    marks = [torch.cuda.Event(enable_timing=True) for _ in range(4)] if ev is not None else None
    if marks:
      marks[0].record()
    training = torch.is_grad_enabled() and any(isinstance(t, torch.Tensor) and t.requires_grad for t in (sorted_inputs, w0, w1, wo))
    if training:
      # differentiable path: bf16 operands; with act_quant both operands of each GEMM are quantised
      # inside its forward (ops.py:232-267); the backward of the int8 path is the reference's quantised one, an fp8
      # forward is differentiated through its quantisers unchanged; the activation is applied unfused so that its
      # inputs are kept for the backward pass; per-expert biases are added (and differentiated) after each GEMM
      if any(isinstance(t, QArray) for t in (sorted_inputs, w0, w1, wo)):
        raise NotImplementedError("gradients need bf16 weights; QArray weights are an inference format")
      rule = cfg.gmm_quantization_rule
      if rule is not None:  # fp8_full: the qwix rule decides types and calibration (moe.py:1554-1556)
        qkw = dict(use_qwix_quantization=True, qwix_rule=rule)
      else:
        q = "fp8" if cfg.act_quant == "fp8_row" else cfg.act_quant
        qkw = dict(lhs_quantize_dtype=q, rhs_quantize_dtype=q)
      inter = megablox.gmm(sorted_inputs, w0, group_size, bf16, transpose_rhs=True, rhs_up=w1, fuse_act=act, act_limit=limit,
                           rhs_bias=w0_bias, rhs_up_bias=w1_bias, lhs_row_idx=row_idx, lhs_row_idx_div=row_idx_div, lhs_row_inv=row_inv, **qkw)
      return megablox.gmm(inter, wo, group_size, bf16, transpose_rhs=True, rhs_bias=wo_bias, **qkw)
    # one tile-list buffer for both products: the second reuses the first one's list when its tile height agrees
    rows = row_idx.shape[0] if row_idx is not None else (sorted_inputs.qvalue if isinstance(sorted_inputs, QArray) else sorted_inputs).shape[0]
    # (`workspace`: one the sort already left a tile list in, for these group sizes)
    ws = workspace if workspace is not None else kernels.gmm_workspace(rows, group_size.numel(), group_size.device)
    inter = megablox.gmm(sorted_inputs, w0, group_size, bf16, transpose_rhs=True, rhs_up=w1, fuse_act=act, act_limit=limit,
                         rhs_bias=w0_bias, rhs_up_bias=w1_bias, lhs_row_idx=row_idx, lhs_row_idx_div=row_idx_div, workspace=ws,
                         same_groups=workspace is not None)
    if marks:
      marks[1].record()
    if cfg.act_quant is not None:
      # "fp8" is the DeepSeek recipe: 128 x 128 weight blocks with 1 x 128 activation scales
      inter = megablox.quantize_lhs(inter, "fp8" if cfg.act_quant == "fp8_row" else cfg.act_quant, blocks=128 if cfg.act_quant == "fp8" else None)
    if marks:
      marks[2].record()
    out = megablox.gmm(inter, wo, group_size, bf16, transpose_rhs=True, rhs_bias=wo_bias, workspace=ws, same_groups=True)
    if marks:
      marks[3].record()
      ev.append(("wi_glu", marks[0], marks[1]))
      ev.append(("wo", marks[2], marks[3]))
    return out

  # -- sparse_matmul (moe.py:1403), single device -------------------------------------------
  def sparse_matmul(self, inputs, gate_logits, pre_bias_logits, w0_kernel, w1_kernel, wo_kernel,
                    w0_bias=None, w1_bias=None, wo_bias=None, input_ids=None, routing=None):
    """-> (output [B,S,d], lb_loss, bias_updates).  `routing` = (weights, indices) skips get_topk.
    w0_bias / w1_bias [E, moe_mlp_dim] and wo_bias [E, emb_dim] are the per-expert biases of mlp_bias models
    (moe.py:617-637): every routed row gets the bias of its expert (transform_bias, moe.py:1363)."""
    cfg = self.config
    b, s, d = inputs.shape
    k = self.num_experts_per_tok
    x2d = inputs.reshape(b * s, d).contiguous()
    # decode-sized calls: the sort leaves the tile list of the streaming matmul kernels (16-row tiles) behind, one launch less
    # (up to 16 rows per expert on average, where moe_gmm takes those kernels, and 4096 rows, the sort's one-launch limit)
    ws = kernels.gmm_workspace(b * s * k, self.num_experts, x2d.device) if b * s * k <= min(4096, 16 * self.num_experts) else None
    no_grad = not (torch.is_grad_enabled() and any(t is not None and t.requires_grad for t in (gate_logits, pre_bias_logits)))
    if routing is None and ws is not None and self.tid2eid is None and no_grad and gate_logits is not None:
      # ... and the routing runs in the sort's launch (one block does both up to 16 tokens)
      weights, selected, perm, inv, group_size = self._get_topk_sorted(gate_logits, pre_bias_logits, ws)
      x2d = self._scale_inputs_by_router_score(x2d, weights)
    else:
      weights, selected = routing if routing is not None else self.get_topk(gate_logits, pre_bias_logits, input_ids=input_ids)
      x2d = self._scale_inputs_by_router_score(x2d, weights)
      perm, inv, group_size, _ = kernels.sort_by_expert(selected.reshape(b * s, k).contiguous(), self.num_experts,
                                                        want_sorted_experts=False, gmm_workspace=ws)
    training = torch.is_grad_enabled() and any(
        isinstance(t, torch.Tensor) and t.requires_grad for t in (x2d, weights, w0_kernel, w1_kernel, wo_kernel))
    if training:
      # the permute stays fused under grad: the first products read the token rows through perm, their input gradient is
      # summed over each token's k copies through inv (the custom VJP of moe.py:154-171), and no [M, d] copy is kept
      inter = self._experts(x2d, group_size, w0_kernel, w1_kernel, wo_kernel, w0_bias, w1_bias, wo_bias, row_idx=perm, row_idx_div=k,
                            row_inv=inv)
    else:
      # the permute is fused into the first grouped matmul: the T token rows are quantised once (not their M = T * k
      # copies) and the matmul reads row perm[i] // k for its row i, so the [M, d] gathered copy is never written
      inter = self._experts(_quantize_tokens(x2d, cfg.act_quant), group_size, w0_kernel, w1_kernel, wo_kernel, w0_bias, w1_bias, wo_bias,
                            row_idx=perm, row_idx_div=k, workspace=ws)
    out = self.unpermute(inter, perm, weights, b, s, inv_perm=inv)
    lb_loss, bias_updates = self._aux_outputs(gate_logits, selected.reshape(b, s, k))
    return out, lb_loss, bias_updates

  def __call__(self, inputs, input_ids=None, gate_inputs=None, out_sharding=None):
    """-> (output, lb_loss, bias_updates), as moe.py:3143."""
    b, s, d = inputs.shape
    routing_inputs = inputs if gate_inputs is None else gate_inputs
    needs_grad = torch.is_grad_enabled() and any(
        isinstance(t, torch.Tensor) and t.requires_grad for t in (routing_inputs, self.gate_kernel, self.gate_bias))
    fused_router = self.tid2eid is None and self.config.routed_score_func in ("", "sigmoid", "sqrtsoftplus")
    if fused_router and not needs_grad and routing_inputs.dtype == torch.bfloat16 and routing_inputs.shape[-1] % 64 == 0 and self.num_experts % 4 == 0:
      want_logits = self.config.load_balance_loss_weight > 0.0  # the auxiliary loss needs the full distribution
      r = self.gate_and_route(routing_inputs.reshape(b * s, -1), return_logits=want_logits)
      logits = r[2].reshape(b, s, -1) if want_logits else None
      return self.sparse_matmul(inputs, logits, None, self.wi_0, self.wi_1, self.wo, routing=(r[0], r[1]))
    gate_logits, pre_bias = self.gate(routing_inputs.reshape(b * s, -1))
    gate_logits = gate_logits.reshape(b, s, -1)
    pre_bias = None if pre_bias is None else pre_bias.reshape(b, s, -1)
    return self.sparse_matmul(inputs, gate_logits, pre_bias, self.wi_0, self.wi_1, self.wo, input_ids=input_ids)


def _quantize_tokens(x2d, act_quant):
  """The activation quantiser of the first grouped matmul on the token rows: int8 with one scale per row, fp8 with
  one scale per row and 128 values (the DeepSeek recipe) or per row; None leaves the bf16 rows as they are."""
  if act_quant == "int8":
    q, sc = kernels.gather_rows(x2d, out_dtype=torch.int8)
    return QArray(q, sc, "int8")
  if act_quant == "fp8":
    q, sc = kernels.gather_rows(x2d, out_dtype=torch.float8_e4m3fn, block_k=128)
    return QArray(q, sc, "fp8")
  if act_quant == "fp8_row":
    q, sc = kernels.gather_rows(x2d, out_dtype=torch.float8_e4m3fn)
    return QArray(q, sc, "fp8", block_k=0)
  return x2d


class RoutedAndSharedMoE:
  """Routed experts plus always-on shared experts (moe.py:3259-3371).

  The reference's shared block is one gated MLP of width shared_experts * mlp_dim (moe.py:3317-3321).  Such an MLP is
  the sum of shared_experts MLPs of width mlp_dim (the activation acts per intermediate channel, `wo` sums over them),
  so each slice is one more group that owns every token: the stacked [E + S, N, K] tensors hold the routed experts
  followed by the S slices, every token gets them as selections k .. k + S - 1 with combine weight 1, and the whole
  layer runs through the same three grouped-GEMM launches.
  """

  def __init__(self, config: MoEConfig, wi_0, wi_1, wo, gate_kernel=None, gate_bias=None):
    if config.shared_experts < 1:
      raise ValueError("RoutedAndSharedMoE needs shared_experts >= 1")
    self.config = config
    self.routed = RoutedMoE(config, wi_0, wi_1, wo, gate_kernel, gate_bias)
    n_stacked = (wi_0.qvalue if isinstance(wi_0, QArray) else wi_0).shape[0]
    if n_stacked != config.num_experts + config.shared_experts:
      raise ValueError("expert tensors must hold num_experts routed experts followed by shared_experts slices of the shared MLP")

  @property
  def routed_moe(self):
    return self.routed

  def sparse_matmul(self, inputs, gate_logits, pre_bias_logits, routing=None, input_ids=None):
    """-> (routed + shared output [B,S,d], lb_loss, bias_updates); the last two are the routed block's (moe.py:3355-3370)."""
    cfg, r = self.config, self.routed
    b, s, d = inputs.shape
    t, k, e, sh = b * s, cfg.num_experts_per_tok, cfg.num_experts, cfg.shared_experts
    x2d = inputs.reshape(t, d).contiguous()
    w, sel = routing if routing is not None else r.get_topk(gate_logits, pre_bias_logits, input_ids=input_ids)
    routed_sel = sel.reshape(b, s, k)
    shared_ids = torch.arange(e, e + sh, dtype=torch.int32, device=sel.device).expand(t, sh)
    sel = torch.cat([sel.reshape(t, k), shared_ids], 1).contiguous()
    w = torch.cat([w.reshape(t, k).float(), torch.ones((t, sh), dtype=torch.float32, device=w.device)], 1).contiguous()
    ws = kernels.gmm_workspace(t * (k + sh), e + sh, x2d.device) if t * (k + sh) <= min(4096, 16 * (e + sh)) else None
    perm, inv, group_size, _ = kernels.sort_by_expert(sel, e + sh, want_sorted_experts=False, gmm_workspace=ws)
    inter = r._experts(_quantize_tokens(x2d, cfg.act_quant), group_size, r.wi_0, r.wi_1, r.wo, row_idx=perm, row_idx_div=k + sh, workspace=ws)
    out = kernels.unpermute_combine(inter, w, k=k + sh, inv_perm=inv)
    lb_loss, bias_updates = r._aux_outputs(gate_logits, routed_sel)
    return out.reshape(b, s, d), lb_loss, bias_updates

  def __call__(self, inputs, original_inputs=None, gate_inputs=None, intermediate_sharding=None, out_sharding=None, input_ids=None):
    """-> (output, lb_loss, bias_updates), as moe.py:3338-3371: the gate reads gate_inputs when given, hash routing
    (a RoutedMoE with tid2eid set) reads input_ids."""
    del original_inputs, intermediate_sharding, out_sharding
    r = self.routed
    b, s, d = inputs.shape
    routing_inputs = inputs if gate_inputs is None else gate_inputs
    fused = r.tid2eid is None and routing_inputs.dtype == torch.bfloat16 and routing_inputs.shape[-1] % 64 == 0 and cfg_ok(self.config)
    if fused:
      want_logits = self.config.load_balance_loss_weight > 0.0  # the auxiliary loss needs the full distribution
      g = r.gate_and_route(routing_inputs.reshape(b * s, -1), return_logits=want_logits)
      logits = g[2].reshape(b, s, -1) if want_logits else None
      return self.sparse_matmul(inputs, logits, None, routing=(g[0], g[1]))
    gate_logits, pre_bias = r.gate(routing_inputs.reshape(b * s, -1))
    pre_bias = None if pre_bias is None else pre_bias.reshape(b, s, -1)
    return self.sparse_matmul(inputs, gate_logits.reshape(b, s, -1), pre_bias, input_ids=input_ids)


def cfg_ok(cfg: MoEConfig) -> bool:
  """Whether moe_gate_route covers this configuration's router."""
  return cfg.num_experts % 4 == 0 and cfg.routed_score_func in ("", "sigmoid", "sqrtsoftplus")
