"""CPU restatement of the reference's quantized MoE expert path.

TEST INFRASTRUCTURE ONLY -- this file is the checker, never the product.  Only
``tests/``, ``__graft_entry__.smoke()`` and the ``cpu_baseline`` leg of
``bench.py`` may import it.

Every function cites the reference lines (paths relative to the reference
checkout) whose behaviour it restates.  Index/integer work is numpy; floating
point work uses torch on the CPU because numpy has no bfloat16 / float8.

How each function is pinned (see tests/test_oracle_*.py):

  gate_logits
      zero kernel -> sigmoid(0) = 0.5 (+ bias); one-hot kernel columns copy input features.
  top_k, deepseek_routing, expert_group_mask
      hand-computed case of tests/unit/moe_test.py:293-326; brute force.
  calculate_load_balance_updates
      hand-computed case of tests/unit/moe_test.py:328-341.
  permute / unpermute
      permutation invariants, brute-force loops, k*x identity.
  tgmm
      per-group python loop; autograd of the gmm oracle (d/d rhs of sum(gmm * dout)).
  gmm
      per-expert python loop, E=1 == plain matmul, int8 path exact on
      integer inputs, the [3,5]-group case of quantizations_test.py:607-653.
  moe_layer (sparse path)
      independent dense all-experts formulation (moe.py:2986-3040) and the
      per-expert loop block of tests/unit/moe_test.py:344-411.
  get_static_scale
      quantizations_test.py:723-726 (224 -> 0.5 for e4m3fn).
  unpack_int4 / dequantize_int4 / dequantize_fp8_blocks
      tests/unit/dequantize_pack_quantized_int4_test.py:61-127 cases.
  dequantize_mxfp4
      the 16 e2m1 code points of the OCP MX specification (0, 0.5, 1, 1.5, 2, 3, 4, 6 and negatives), the
      nibble order and 2^(s-127) scaling on hand-made blocks; quantize_mxfp4 (a test-data generator only) by
      dequantize(quantize(x)) == x on representable inputs.

  ring_ragged_sort / ring_ragged_unsort / a2a_ragged_sort
      compositions of ragged_gather / ragged_gather_reduce (pinned below) with index arithmetic; checked against
      row-by-row loops (which sorted positions belong to the shard, where they sit in a packed buffer) and by the
      identity sum over shards of unsort(sort(x)) == sum of the routing weights times x.

  ragged_gather / ragged_gather_reduce / weighted_intermediate
      hand-made rows: a NaN row behind a cleared mask bit stays out of the sum, a group with every row masked
      gives zeros, the f32 sum rounds once (a case where rounding each term first gives another result), equality
      with unpermute when every row is valid, double rounding of the weighted activation on a value that
      separates it from a single rounding.

  quantize_lhs_v2 / manual_quantize (the quantisers whose source IS in the reference tree)
      hand cases worked out in exact rational arithmetic (python Fractions with an explicit round-to-nearest-even
      to the 8-bit / 24-bit significand) that separate truncation from round-half-even and round-half-away,
      x * (1 / scale) from x / scale, and bf16 from f32 intermediate arithmetic; the closed forms
      q * scale == x on inputs that are exact multiples of the scale; zero rows.

  truncate_matrix / maybe_truncate_local_group_size / local_permute / get_all_to_all_params / get_ragged_buffer_size
      (the bookkeeping of the expert-parallel dispatch, all integer): the expected arrays of
      tests/unit/moe_test.py:1174-1336 (local_permute with and without offset), :1338-1442 (the four parameter
      vectors, batch sharded and replicated), :1444-1494 (buffer sizes); conservation laws for the truncation
      (column sums never exceed the buffer, rows are cut in shard order, nothing changes below the capacity);
      brute-force loops over rows for the keys.  The fill of rows past the received total follows
      jax.numpy.repeat(total_repeat_length=...), which pads with the last value; moe_test.py:1174-1261 reaches it (its
      slices are longer than the shards' rows) with jnp.repeat on both sides, so it pins the use of that rule, and the
      rule itself is jax's documented one (those rows carry no tokens and no result depends on them).

PARITY UNPINNED (third-party arithmetic whose source is not in the reference
tree, and which no reference test pins):
  * quantize_rows_int8 / quantize_weight_int8 / quantize_fp8_blocks / quantize_e5m2: rounding mode and
    zero-scale handling of qwix.pallas.quantize (qwix >= 0.1.8), the quantiser of the v1 path
    (ops.py:241-260, :563-571, :590-603).  Adopted: scale = absmax / qmax, q = clip(rint(x / scale)),
    zero absmax -> q = 0.  GEMM parity is therefore asserted on identical already-quantized operands.
    (The v2 path's in-kernel quantiser and manual_quantize are restated exactly, see above.)
  * tie order of jax.lax.top_k and stability of jnp.argsort (jax >= 0.10.2).
    Adopted: larger value first, lower index first on ties; stable sort.
  * bf16 rounding of the norm_topk_prob renormalisation (moe.py:756).
  * the value an out-of-range float -> int8 conversion yields in XLA (implementation defined); unreachable from
    quantize_lhs_v2 (|x * inv| <= 127.5 before truncation), clamped here.
"""

from __future__ import annotations

import math

import numpy as np
import torch

FP8_E4M3_MAX = 448.0
INT8_MAX = 127.0
INT4_MAX = 7.0


# --------------------------------------------------------------------------
# Routing  (src/maxtext/layers/moe.py:717-839)
# --------------------------------------------------------------------------


def top_k(x: np.ndarray, k: int):
  """jax.lax.top_k semantics as adopted here: descending values, lower index
  first among equal values (moe.py:747, :834).  Brute force via stable sort."""
  x = np.asarray(x)
  idx = np.argsort(-x.astype(np.float64), axis=-1, kind="stable")[..., :k].astype(np.int32)
  vals = np.take_along_axis(x, idx, axis=-1)
  return vals, idx


def expert_group_mask(gate_logits: np.ndarray, n_routing_groups: int, topk_routing_group: int) -> np.ndarray:
  """moe.py:775-811: keep experts of the top groups; group score = sum of the
  group's top-2 expert scores (f32)."""
  e = gate_logits.shape[-1]
  grouped = gate_logits.reshape(gate_logits.shape[:-1] + (n_routing_groups, e // n_routing_groups))
  top2, _ = top_k(grouped, 2)
  group_scores = top2.astype(np.float32).sum(-1)
  _, group_idx = top_k(group_scores, topk_routing_group)
  group_mask = np.zeros(group_scores.shape, np.float32)
  np.put_along_axis(group_mask, group_idx, 1.0, axis=-1)
  mask = np.repeat(group_mask, e // n_routing_groups, axis=-1)
  return mask


def deepseek_routing(gate_logits, pre_bias_logits, k, n_routing_groups=-1, topk_routing_group=-1):
  """moe.py:813-839: select on post-bias scores (optionally group-limited),
  return the pre-bias scores of the selected experts as weights."""
  gate_logits = np.asarray(gate_logits)
  if n_routing_groups == -1:
    masked = gate_logits
  else:
    mask = expert_group_mask(gate_logits, n_routing_groups, topk_routing_group)
    masked = np.where(mask > 0, gate_logits, -np.inf)
  _, idx = top_k(masked, k)
  weights = np.take_along_axis(np.asarray(pre_bias_logits), idx, axis=-1)
  return weights, idx


def gate_logits(x: torch.Tensor, kernel: torch.Tensor, bias=None, *, score_func: str = "", deepseek: bool = False,
                float32_gate_logits: bool = True):
  """GateLogit.__call__ (moe.py:353-392): inputs and kernel cast to the gate dtype (f32 when
  float32_gate_logits, moe.py:494), output = inputs @ kernel [d, E], optional score function, pre_bias_logits =
  output for DeepSeek-V3/V4 (:385-386), output += bias (:388-390).  Returns float32 ndarrays (logits, pre_bias
  or None).  The f32 matmul is carried in f64 and rounded once."""
  if float32_gate_logits:
    out = (x.double() @ kernel.double()).float()
  else:
    out = (x.to(torch.bfloat16).double() @ kernel.to(torch.bfloat16).double()).to(torch.bfloat16).float()
  if score_func == "sigmoid":
    out = torch.sigmoid(out)
  elif score_func == "sqrtsoftplus":  # linears.py:51-53: jnp.sqrt(jax.nn.softplus(x)), softplus = logaddexp(x, 0)
    out = torch.from_numpy(np.sqrt(np.logaddexp(out.numpy(), np.float32(0))).astype(np.float32))
  elif score_func:
    raise ValueError(score_func)
  pre = out.clone() if deepseek else None
  if bias is not None:
    out = out + bias.float()
  return out.numpy(), None if pre is None else pre.numpy()


def _softmax_f32(x: np.ndarray) -> np.ndarray:
  x = x.astype(np.float32)
  m = x.max(-1, keepdims=True)
  e = np.exp(x - m, dtype=np.float32)
  return (e / e.sum(-1, keepdims=True, dtype=np.float32)).astype(np.float32)


def _round_bf16(x: np.ndarray) -> np.ndarray:
  return torch.from_numpy(np.ascontiguousarray(x, dtype=np.float32)).to(torch.bfloat16).to(torch.float32).numpy()


def get_topk(
    gate_logits,
    pre_bias_logits=None,
    *,
    k: int,
    mode: str = "softmax_topk",
    norm_topk_prob: bool = False,
    routed_scaling_factor: float = 1.0,
    routed_score_func: str = "sigmoid",
    n_routing_groups: int = -1,
    topk_routing_group: int = -1,
    weight_dtype: str = "bf16",
):
  """moe.py:717-765.  Returns (weights f32 ndarray holding values already
  rounded to `weight_dtype`, indices int32).

  mode "softmax_topk": lax.top_k -> softmax over the k values in f32 -> cast to
  the layer dtype (:747, :753) -> optional renormalisation in that dtype (:756).
  mode "deepseek": deepseek_routing (:744) then deepseek_scale_weights (:767-773);
  weights keep the gate dtype (f32).
  """
  gate_logits = np.asarray(gate_logits)
  if mode == "deepseek":
    w, idx = deepseek_routing(gate_logits, pre_bias_logits, k, n_routing_groups, topk_routing_group)
    w = w.astype(np.float32)
    if routed_score_func in ("sigmoid", "sqrtsoftplus"):
      w = w / (w.sum(-1, keepdims=True, dtype=np.float32) + np.float32(1e-20))
    w = (w * np.float32(routed_scaling_factor)).astype(np.float32)
    return w, idx
  if mode not in ("softmax_topk", "topk_raw", "softmax_all"):
    raise ValueError(f"unknown routing mode {mode}")
  vals, idx = top_k(gate_logits, k)
  if mode == "topk_raw":
    # Llama4: the selected logits themselves; the softmax and its cast to the layer dtype (moe.py:753) are skipped, so
    # the weights keep the gate's dtype, i.e. the values handed in stay as they are
    w = vals.astype(np.float32)
    weight_dtype = "gate"
  elif mode == "softmax_all":  # Gemma4: softmax over all experts, gathered at the indices (moe.py:742-745)
    w = np.take_along_axis(_softmax_f32(gate_logits), idx, axis=-1)
  else:
    w = _softmax_f32(vals)
  if weight_dtype == "bf16":
    w = _round_bf16(w)
  if norm_topk_prob:
    s = w.sum(-1, keepdims=True, dtype=np.float32)
    if weight_dtype == "bf16":
      s = _round_bf16(s)
      w = _round_bf16(w / s)
    else:
      w = (w / s).astype(np.float32)
  return w, idx


def hash_routing(scores: np.ndarray, tid2eid: np.ndarray, input_ids: np.ndarray, *, deepseek: bool = True,
                 routed_score_func: str = "sigmoid", routed_scaling_factor: float = 1.0):
  """DeepSeek-V4 hash routing (moe.py:729-738 then :749-751, :767-773): indices = tid2eid[input_ids]
  (the table is stored as f32 and cast to int32), weights = scores at those indices, divided by their sum
  (+1e-20) for the sigmoid / sqrtsoftplus score functions and multiplied by routed_scaling_factor."""
  assert deepseek, "only DeepSeek-V4 layers are hash routed"
  idx = np.asarray(tid2eid).astype(np.int32)[np.asarray(input_ids).astype(np.int32)]
  w = np.take_along_axis(np.asarray(scores, np.float32), idx.astype(np.int64), axis=-1)
  if routed_score_func in ("sigmoid", "sqrtsoftplus"):
    w = w / (w.sum(-1, keepdims=True) + np.float32(1e-20))
  return (w * np.float32(routed_scaling_factor)).astype(np.float32), idx


def calculate_load_balance_updates(top_k_indices, num_experts: int, rate: float):
  """moe.py:215-236."""
  flat = np.asarray(top_k_indices).ravel()
  counts = np.bincount(flat, minlength=num_experts)
  average = flat.size / num_experts
  return np.sign(average - counts) * rate


# --------------------------------------------------------------------------
# Permute / unpermute  (moe.py:950-960, :986-991, :1039-1063)
# --------------------------------------------------------------------------


def permute(inputs_2d: torch.Tensor, selected_experts: np.ndarray, num_experts: int, roll_to_expert_id=None):
  """moe.py:950-960, :986-991 (non-ragged branch); roll_to_expert_id: ids become (id - roll) % E first (:953-954).

  Returns (sorted_inputs [M,d], sorted_selected_experts [M] int32 -- the stable
  argsort of the flattened expert ids, group_size [E] int32, sorted_experts [M]).
  Row i of sorted_inputs is token perm[i] // k (repeat(x, k)[perm])."""
  t, k = selected_experts.shape
  flat = np.asarray(selected_experts).reshape(-1)
  if roll_to_expert_id is not None:
    flat = (flat - roll_to_expert_id) % num_experts
  perm = np.argsort(flat, kind="stable").astype(np.int32)
  sorted_inputs = inputs_2d[torch.from_numpy((perm // k).astype(np.int64))]
  group_size = np.bincount(flat, minlength=num_experts).astype(np.int32)
  sorted_experts = np.repeat(np.arange(num_experts, dtype=np.int32), group_size)
  return sorted_inputs, perm, group_size, sorted_experts


def unpermute(intermediate: torch.Tensor, perm: np.ndarray, weights: np.ndarray, k: int, out_dtype=torch.bfloat16):
  """moe.py:1039-1063 with float32_weight_sum=True: gather by argsort(perm),
  reshape [T,k,d], f32 einsum "BKE,BK->BE", cast to the layer dtype."""
  inv = np.argsort(perm, kind="stable")
  un = intermediate[torch.from_numpy(inv.astype(np.int64))].to(torch.float32)
  w = torch.from_numpy(np.ascontiguousarray(weights, dtype=np.float32)).reshape(-1, k)
  un = un.reshape(w.shape[0], k, -1)
  out = torch.einsum("bke,bk->be", un, w)
  return out.to(out_dtype)


# --------------------------------------------------------------------------
# Expert-parallel dispatch bookkeeping  (moe.py:103-120, :1066-1349, :1368-1401)
# --------------------------------------------------------------------------


def truncate_matrix(all_shards_group_sizes: np.ndarray, buffer_size: int) -> np.ndarray:
  """moe.py:103-120: the traffic matrix [sender, receiver] cut so that no receiver gets more than buffer_size rows;
  senders are served in order (prefix sum over axis 0, clamped, differenced)."""
  a = np.asarray(all_shards_group_sizes)
  c = np.minimum(np.cumsum(a, axis=0), buffer_size)
  return np.diff(np.concatenate([np.zeros((1, a.shape[1]), dtype=c.dtype), c], axis=0), axis=0).astype(a.dtype)


def maybe_truncate_local_group_size(all_shard_local_sizes: np.ndarray, buffer_size: int, ragged_buffer_factor: float) -> np.ndarray:
  """moe.py:1066-1089: rows per local expert summed over the batch shards; with ragged_buffer_factor > 0 the flattened
  [shard, local expert] sizes are first cut at buffer_size in that order."""
  a = np.asarray(all_shard_local_sizes)
  if ragged_buffer_factor > 0.0:
    flat = a.reshape(-1)
    c = np.minimum(np.cumsum(flat), buffer_size)
    a = np.diff(np.concatenate([np.zeros((1,), dtype=c.dtype), c])).reshape(a.shape)
  return a.sum(axis=0).astype(np.int32)


def _repeat_total(values: np.ndarray, repeats: np.ndarray, total: int) -> np.ndarray:
  """jax.numpy.repeat(values, repeats, total_repeat_length=total): output position p takes values[i] for the largest
  i whose start (exclusive prefix sum of repeats) is <= p, so a short sum is padded with the last value and a long
  one is cut."""
  starts = np.concatenate([[0], np.cumsum(repeats)[:-1]])
  idx = np.searchsorted(starts, np.arange(total), side="right") - 1
  return np.asarray(values)[idx]


def local_permute(inputs: torch.Tensor, global_group_sizes: np.ndarray, local_expert_size: int, shard_index: int,
                  is_offset: bool = False, global_sorted_experts=None, ragged_buffer_factor: float = -1.0):
  """moe.py:1091-1200 -> (sorted_inputs, sorted_indices, local_group_size, sorted_experts_ids).

  global_group_sizes [batch shards, E].  Without offset the rows arrive grouped by (batch shard, local expert) and the
  key of a row is its local expert; with offset the rows are all routed rows sorted by global expert and rows of other
  shards get the key local_expert_size, which sorts them behind this shard's."""
  g = np.asarray(global_group_sizes)
  all_shard_local = g[:, shard_index * local_expert_size:(shard_index + 1) * local_expert_size]
  local_sizes = all_shard_local.reshape(-1)
  rows = inputs.shape[0]
  local_group_size = maybe_truncate_local_group_size(all_shard_local, rows, ragged_buffer_factor)
  if is_offset:
    gse = np.asarray(global_sorted_experts)
    keys = np.where(gse // local_expert_size == shard_index, gse % local_expert_size, local_expert_size)
  else:
    base = np.arange(local_sizes.shape[0]) % local_expert_size
    keys = _repeat_total(base, local_sizes, rows)
  sorted_indices = np.argsort(keys, kind="stable").astype(np.int32)
  sorted_inputs = inputs[torch.from_numpy(sorted_indices.astype(np.int64))]
  return sorted_inputs, sorted_indices, local_group_size, keys[sorted_indices].astype(np.int32)


def get_all_to_all_params(all_shards_group_sizes: np.ndarray, shard_id: int, num_expert_parallelism: int,
                          is_batch_sharded: bool = True, ragged_buffer_factor: float = -1.0, buffer_size=None,
                          is_dispatch: bool = True):
  """moe.py:1202-1349 -> (input_offsets, send_sizes, output_offsets, recv_sizes) of ragged_all_to_all."""
  a = np.asarray(all_shards_group_sizes)

  def input_offset(m):
    if is_batch_sharded:
      return np.concatenate([[0], np.cumsum(m[shard_id])[:-1]]).astype(m.dtype)
    return np.zeros(num_expert_parallelism, dtype=m.dtype)

  def send_size(m):
    return m[shard_id] if is_batch_sharded else np.repeat(m[shard_id], num_expert_parallelism)

  def output_offset(m):
    if is_batch_sharded:
      return np.cumsum(np.concatenate([np.zeros((1,) + m.shape[1:], dtype=m.dtype), m], axis=0), axis=0, dtype=m.dtype)[shard_id]
    return np.repeat(np.concatenate([[0], np.cumsum(m[:-1])])[shard_id], num_expert_parallelism).astype(m.dtype)

  def recv_size(m):
    return m[:, shard_id] if is_batch_sharded else m

  if ragged_buffer_factor > 0.0:
    assert buffer_size is not None
    t = truncate_matrix(a, buffer_size)
    if is_dispatch:  # the sender still holds every row; sizes and receive offsets follow the cut matrix
      return input_offset(a), send_size(t), output_offset(t), recv_size(t)
    at, tt = a.T, t.T  # combine: the packed (cut) buffer is sent back to the rows' original positions
    return input_offset(tt), send_size(tt), output_offset(at), recv_size(tt)
  m = a if is_dispatch else a.T
  return input_offset(m), send_size(m), output_offset(m), recv_size(m)


def get_ragged_buffer_size(local_batch: int, ep_degree: int, global_experts: int, top_k: int, ragged_buffer_factor: float) -> int:
  """moe.py:1368-1401: rows of the receive buffer: the balanced share times the factor, or the worst case
  min(ep_degree, global_experts / top_k) times the share."""
  if ragged_buffer_factor > 0.0:
    return int(local_batch * ragged_buffer_factor)
  return int(local_batch * min(ep_degree, global_experts / top_k))


def unroute_sum(tokens: torch.Tensor, selected_experts: np.ndarray):
  """kernels/sort_activations.py:98-121: gather by argsort(argsort) and sum
  over k without weights (batch-split DeepSeek variant)."""
  t, k = selected_experts.shape
  inds = np.argsort(np.argsort(selected_experts.reshape(-1), kind="stable"), kind="stable")
  g = tokens[torch.from_numpy(inds.astype(np.int64))]
  return g.reshape(t, k, -1).sum(1)


def ragged_gather(x: torch.Tensor, indices: np.ndarray, start=None, end=None, weights=None):
  """kernels/ragged/ragged_gather.py:310-320: out = x[indices], times weights[:, None] when given (the product
  is formed in the promoted type of the two and returned in it; callers keep bf16 by passing bf16 weights).
  [start, end) (ragged_gather.py:357-376) names the output rows a caller will use; the reference leaves the
  others unspecified, this restatement writes zeros there."""
  out = x[torch.from_numpy(np.asarray(indices, dtype=np.int64))]
  if weights is not None:
    out = out * weights[:, None]
  if start is not None:
    rows = torch.arange(out.shape[0])
    out = torch.where(((rows >= int(start)) & (rows < int(end)))[:, None], out, torch.zeros_like(out))
  return out


def ragged_gather_reduce(x: torch.Tensor, indices: np.ndarray, topk_weights: torch.Tensor, valid_rows_mask: np.ndarray,
                         reduce_group_size: int):
  """kernels/ragged/ragged_gather_reduce_v2.py:170-182: gather, weight in f32, zero the rows that are not valid,
  sum each run of reduce_group_size consecutive rows in f32, round once to bf16.  (`where` drops a masked row
  whatever it holds, NaN included.)"""
  out = x[torch.from_numpy(np.asarray(indices, dtype=np.int64))].to(torch.float32) * topk_weights.to(torch.float32)[:, None]
  out = torch.where(torch.from_numpy(np.asarray(valid_rows_mask, dtype=bool))[:, None], out, torch.zeros_like(out))
  out = out.reshape(-1, reduce_group_size, out.shape[-1])
  return out.sum(1).to(torch.bfloat16)


def _shard_rows(group_sizes: np.ndarray, num_experts: int, shard_idx: int, ep_size: int):
  """Positions [start, end) of a shard's experts in the order sorted by expert (ragged_sort.py:102-107)."""
  offs = np.concatenate([[0], np.cumsum(group_sizes)])
  local = num_experts // ep_size
  return int(offs[shard_idx * local]), int(offs[(shard_idx + 1) * local])


def ring_ragged_sort(hidden: torch.Tensor, topk_indices: np.ndarray, num_experts: int, topk: int, shard_idx: int, ep_size: int,
                     buffer_size=None):
  """kernels/ragged/ragged_sort.py:84-151 (forward) -> (x, group_sizes [E], topk_argsort_revert_indices [T*k])."""
  t = hidden.shape[0]
  flat = np.asarray(topk_indices).reshape(-1)
  order = np.argsort(flat, kind="stable")
  token_sorted = np.repeat(np.arange(t), topk)[order]
  group_sizes = np.bincount(flat, minlength=num_experts).astype(np.int32)
  revert = np.argsort(order, kind="stable").astype(np.int32)
  start, end = _shard_rows(group_sizes, num_experts, shard_idx, ep_size)
  n = t * topk
  if buffer_size is None or buffer_size >= n:
    x = ragged_gather(hidden, token_sorted, start, end)
  else:
    sliced = np.pad(token_sorted, (0, buffer_size))[start:start + buffer_size]
    x = ragged_gather(hidden, sliced, 0, min(end - start, buffer_size))
  return x, group_sizes, revert


def ring_ragged_unsort(sorted_tokens: torch.Tensor, group_sizes: np.ndarray, revert: np.ndarray, topk: int, local_num_experts: int,
                       shard_idx: int, topk_weights: torch.Tensor):
  """kernels/ragged/ragged_sort.py:294-351 (forward) -> [T, hidden]."""
  offs = np.concatenate([[0], np.cumsum(group_sizes)])
  start, end = int(offs[shard_idx * local_num_experts]), int(offs[(shard_idx + 1) * local_num_experts])
  revert = np.asarray(revert, dtype=np.int64)
  buffer_size, n = sorted_tokens.shape[0], revert.shape[0]
  w = topk_weights.reshape(-1).to(torch.float32)
  if buffer_size >= n:
    mask = (revert >= start) & (revert < end)
    return ragged_gather_reduce(sorted_tokens, revert, w, mask, topk)
  shifted = revert - start
  mask = (shifted >= 0) & (shifted < min(end - start, buffer_size))
  return ragged_gather_reduce(sorted_tokens, np.where(mask, shifted, 0), w, mask, topk)


def a2a_ragged_sort(inputs: torch.Tensor, sort_indices: np.ndarray, valid_end: int):
  """kernels/ragged/ragged_sort.py:497-512 (and, with revert indices, :592-606): rows below valid_end are gathered,
  the rest are zeros."""
  return ragged_gather(inputs, sort_indices, 0, int(valid_end))


def weighted_intermediate(h0: torch.Tensor, h1: torch.Tensor, weights: torch.Tensor, kind: str = "silu", limit: float = 7.0):
  """models/deepseek_batchsplit_fp8.py:1048-1049: the routing weight of each sorted row multiplies the finished
  bf16 activation before `wo` (the combine after it is then an unweighted sum): bf16(bf16(act(h0, h1)) * w)."""
  act = apply_ffn_activation(h0, h1, kind, limit, out_dtype=torch.bfloat16)
  return (act.to(torch.float32) * weights.to(torch.float32)[:, None]).to(torch.bfloat16)


# --------------------------------------------------------------------------
# Activation  (moe.py:841-870; pallas_mosaic_tpu_v2_gmm_kernel.py:33-73)
# --------------------------------------------------------------------------


def apply_ffn_activation(h0: torch.Tensor, h1: torch.Tensor, kind: str = "silu", limit: float = 7.0, out_dtype=torch.bfloat16):
  """kind "silu": silu(h0)*h1 (moe.py:868-869); "swigluoai": GPT-OSS clipped
  variant (moe.py:844-853 == v2 kernel :33-40); "silu_clip": DeepSeek-V4
  (moe.py:854-866).  Computed in f32, cast to the layer dtype (:870)."""
  h0 = h0.to(torch.float32)
  h1 = h1.to(torch.float32)
  if kind == "silu":
    out = torch.nn.functional.silu(h0) * h1
  elif kind == "swigluoai":
    g = torch.clamp(h0, max=limit)
    u = torch.clamp(h1, min=-limit, max=limit)
    out = g * torch.sigmoid(1.702 * g) * (u + 1.0)
  elif kind == "silu_clip":
    g = torch.clamp(h0, max=limit)
    u = torch.clamp(h1, min=-limit, max=limit)
    out = torch.nn.functional.silu(g) * u
  else:
    raise ValueError(kind)
  return out.to(out_dtype)


# --------------------------------------------------------------------------
# Grouped matmul
#   tests/unit/pallas_mosaic_tpu_v2_kernel_test.py:92-153 (reference_gmm),
#   kernels/megablox/backend.py:316-333, moe.py:1450-1459 (per-expert scale)
# --------------------------------------------------------------------------


def _to_f(x: torch.Tensor, dt):
  return x.to(dt)


def gmm(
    lhs: torch.Tensor,  # [m, k]  bf16 / int8 / float8_e4m3fn
    rhs: torch.Tensor,  # [g, k, n] (or [g, n, k] with transpose_rhs)
    group_sizes,  # [G_total] int32
    *,
    rhs_scale: torch.Tensor | None = None,  # [g, nb, 1, n] f32 (v2 format) or [g, n]; g may be 1 (shared by all experts)
    lhs_scale: torch.Tensor | None = None,  # [m] / [m,1] per row, [m, nb] per K-block, or [1, 1] (static per-tensor)
    rhs_bias: torch.Tensor | None = None,  # [g, 1, n]
    partial_sum: torch.Tensor | None = None,  # [m, n]
    group_offset: int = 0,
    quant_block=None,  # K-block size when scales are block-wise (ragged tail allowed); (lhs_block, rhs_block) when they differ
    transpose_rhs: bool = False,
    out_dtype=torch.bfloat16,
    acc_dtype=torch.float64,
) -> torch.Tensor:
  """out[rows of group g] = lhs[rows] @ rhs[g - group_offset], accumulating
  per K-block and applying the block's scales to the partial sum
  (reference_gmm :121-135); rows of non-local groups and rows past
  sum(group_sizes) are zero (:139-141; v2 kernel :753-826)."""
  if transpose_rhs:
    rhs = rhs.transpose(1, 2)
  m, k = lhs.shape
  g, k2, n = rhs.shape
  assert k == k2
  group_sizes = np.asarray(group_sizes, dtype=np.int64)
  out = torch.zeros((m, n), dtype=acc_dtype)

  if rhs_scale is not None and rhs_scale.dim() == 2:
    rhs_scale = rhs_scale[:, None, None, :]
  nb_r = rhs_scale.shape[1] if rhs_scale is not None else 1
  if lhs_scale is not None and lhs_scale.dim() == 1:
    lhs_scale = lhs_scale[:, None]
  nb_l = lhs_scale.shape[1] if lhs_scale is not None else 1
  # K-block of each side's scales (quant_block: the common one, or a (lhs, rhs) pair when they differ, as in gmm_v2
  # where the activation block is 512 and the weight block comes with the checkpoint); the sum runs over the common
  # refinement of the two grids
  if isinstance(quant_block, (tuple, list)):
    qb_l, qb_r = quant_block
  else:
    qb_l = qb_r = quant_block
  qb_l = k if nb_l == 1 else (qb_l if qb_l is not None else k // nb_l)
  qb_r = k if nb_r == 1 else (qb_r if qb_r is not None else k // nb_r)
  assert math.ceil(k / qb_l) == nb_l and math.ceil(k / qb_r) == nb_r, (k, qb_l, nb_l, qb_r, nb_r)
  cuts = sorted(set(range(0, k, qb_l)) | set(range(0, k, qb_r)) | {k})

  start = 0
  for gg in range(group_sizes.size):
    end = min(start + int(group_sizes[gg]), m)
    loc = gg - group_offset
    if 0 <= loc < g and end > start:
      acc = torch.zeros((end - start, n), dtype=acc_dtype)
      for ks, ke in zip(cuts[:-1], cuts[1:]):
        part = lhs[start:end, ks:ke].to(acc_dtype) @ rhs[loc, ks:ke, :].to(acc_dtype)
        if rhs_scale is not None:
          part = part * rhs_scale[loc if rhs_scale.shape[0] > 1 else 0, ks // qb_r].to(acc_dtype)
        if lhs_scale is not None:
          rows = slice(start, end) if lhs_scale.shape[0] > 1 else slice(0, 1)  # [1, 1]: one static scale for all rows
          part = part * lhs_scale[rows, ks // qb_l].to(acc_dtype)[:, None]
        acc += part
      if rhs_bias is not None:
        acc = acc + rhs_bias[loc].to(acc_dtype)
      if partial_sum is not None:
        acc = acc + partial_sum[start:end].to(acc_dtype)
      out[start:end] = acc
    start = end
  return out.to(out_dtype)


def tgmm(lhs: torch.Tensor, dout: torch.Tensor, group_sizes, *, num_actual_groups=None, group_offset: int = 0,
         out_dtype=torch.bfloat16, existing_out=None) -> torch.Tensor:
  """Transposed grouped matmul, the weight gradient of gmm
  (tests/unit/pallas_mosaic_tpu_v2_kernel_test.py:156-186 reference_tgmm; backend.py:587):
  out[g] = lhs[rows of group g]^T @ dout[rows of group g], shape [groups, k, n]; only the
  num_actual_groups groups starting at group_offset are produced.  existing_out ([groups, k, n]) joins the
  accumulator before the rounding to out_dtype (backend.py:731-735)."""
  group_sizes = np.asarray(group_sizes, dtype=np.int64)
  m = lhs.shape[0]
  g = group_sizes.size - group_offset if num_actual_groups is None else num_actual_groups
  outs = []
  start = 0
  for gg in range(group_sizes.size):
    end = min(start + int(group_sizes[gg]), m)
    loc = gg - group_offset
    if 0 <= loc < g:
      acc = lhs[start:end].double().T @ dout[start:end].double()
      if existing_out is not None:
        acc = acc + existing_out[loc].double()
      outs.append(acc.to(out_dtype))
    start = end
  return torch.stack(outs)


E5M2_MAX = 57344.0  # largest finite float8_e5m2


def quantize_e5m2(x: torch.Tensor, dim):
  """Gradient quantiser of the backward pass (ops.py:583-604): symmetric absmax scale along `dim`
  (channelwise_axes=[0] keeps one scale per row -> dim=1; [1] one per column -> dim=0; [] one for the tensor, the
  rule's disable_channelwise_axes -> dim=(0, 1)), values cast to
  float8_e5m2.  Returns (values as f32 on the e5m2 grid, scale f32 with `dim` kept).  Rounding mode and the
  zero-scale rule of qwix are not in the reference tree (see module docstring): round-to-nearest-even of the
  torch cast, zero scale -> zeros."""
  x = x.to(torch.float32)
  scale = x.abs().amax(dim=dim, keepdim=True) / E5M2_MAX
  q = torch.where(scale == 0, torch.zeros_like(x), x / scale).to(torch.float8_e5m2).to(torch.float32)
  return q, scale


def gmm_bwd_quantized(grad: torch.Tensor, lhs_q: torch.Tensor, lhs_scale: torch.Tensor, rhs_q: torch.Tensor,
                      rhs_scale: torch.Tensor, group_sizes, *, bwd_qtype: str | None = None, grad_dtype=torch.bfloat16,
                      per_tensor: bool = False):
  """Backward of a quantised gmm as the reference runs it (ops.py:438-527 with _bwd_prepare_inputs :530-580 and
  _bwd_quantize_gradient :583-604), for channelwise scales: lhs_q [m,k] with lhs_scale [m]; rhs_q [g,k,n] with
  rhs_scale [n] (shared, ops.py:250-260) or [g,n] (per expert).

    dlhs_dout = grad * rhs_scale[n]      (the scale of the contracted axis goes onto the gradient, :548-559)
    drhs_dout = grad * lhs_scale[m]      (:575-578)
    both optionally quantised to e5m2, per row / per column (:590-603)
    dlhs = gmm(dlhs_dout, rhs_q^T)       (:612-642)      drhs = tgmm(lhs_q^T, drhs_dout)   (:766-796)

  per_tensor: the rule's disable_channelwise_axes (channelwise_axes=[] at :568, :594, :601): lhs_scale and rhs_scale hold one
  value each (any shape that broadcasts as given above), and each scaled gradient is quantised with ONE absmax scale.

  Scaled gradients are rounded to grad_dtype (the reference multiplies in grad.dtype).  Returns (dlhs [m,k] f64,
  drhs [g,k,n] f64)."""
  group_sizes = np.asarray(group_sizes, dtype=np.int64)
  m, n = grad.shape
  g = rhs_q.shape[0]
  row_group = np.repeat(np.arange(group_sizes.size), group_sizes)[:m]
  rs = rhs_scale.to(torch.float32)
  rs_rows = rs[None, :].expand(m, n) if rs.dim() == 1 else rs[torch.as_tensor(np.minimum(row_group, g - 1))]
  dlhs_dout = (grad.to(grad_dtype) * rs_rows.to(grad_dtype)).to(torch.float32)
  drhs_dout = (grad.to(grad_dtype) * lhs_scale.to(grad_dtype)[:, None]).to(torch.float32)
  s_row = torch.ones((m, 1))
  s_col = torch.ones((1, n))
  if bwd_qtype is not None:
    assert bwd_qtype in ("e5m2", "float8_e5m2")
    dlhs_dout, s_row = quantize_e5m2(dlhs_dout, dim=(0, 1) if per_tensor else 1)
    drhs_dout, s_col = quantize_e5m2(drhs_dout, dim=(0, 1) if per_tensor else 0)
  dlhs = gmm(dlhs_dout, rhs_q.to(torch.float32).transpose(1, 2), group_sizes, out_dtype=torch.float64) * s_row.double()
  drhs = tgmm(lhs_q.to(torch.float32), drhs_dout, group_sizes, out_dtype=torch.float64) * s_col.double()[None]
  return dlhs, drhs


# --------------------------------------------------------------------------
# Quantisers and storage formats
# --------------------------------------------------------------------------


def get_static_scale(qmax: float, calibration_method: str) -> float:
  """layers/quantizations.py:928-958 with qmax = symmetric bound of the dtype
  (448 for float8_e4m3fn, pinned by quantizations_test.py:723-726)."""
  if calibration_method is None or not calibration_method.lower().startswith("fixed"):
    raise ValueError(f"Only static scale quantization is supported, got {calibration_method}")
  args = [float(a) for a in calibration_method.split(",")[1:]]
  if len(args) == 1:
    args = [-args[0], args[0]]
  if len(args) != 2 or args[0] + args[1] != 0 or args[1] <= 0:
    raise ValueError(f"Expected format: 'fixed,max' or 'fixed,-max,max'. Got: {calibration_method}")
  scale = args[1] / qmax
  if scale < np.finfo(np.float32).tiny ** 0.5:
    scale = 1.0
  return scale


def _round_to(x: torch.Tensor, dtype) -> torch.Tensor:
  """f32 values rounded (nearest even) to `dtype`'s grid, returned as f32: one JAX op in that dtype."""
  return x if dtype == torch.float32 else x.to(dtype).to(torch.float32)


def _astype_q(y: torch.Tensor, qdtype) -> torch.Tensor:
  """jnp `.astype(qdtype)` of float values: integers truncate toward zero (XLA ConvertElementType; out-of-range values
  are clamped here), float8_e4m3fn rounds to nearest even (values above 464 become NaN: e4m3fn has no infinity)."""
  if qdtype == torch.int8:
    return torch.trunc(y).clamp(-128, 127).to(torch.int8)
  if qdtype == torch.float8_e4m3fn:
    return y.to(torch.float8_e4m3fn)
  raise ValueError(qdtype)


def qdtype_max(qdtype) -> float:
  """jnp.iinfo(int8).max / jnp.finfo(float8_e4m3fn).max (pallas_mosaic_tpu_v2_gmm_kernel.py:496-501)."""
  return {torch.int8: 127.0, torch.float8_e4m3fn: 448.0}[qdtype]


def quantize_lhs_v2(x: torch.Tensor, qdtype, quant_block: int = 512, static_scale=None, acc_dtype=torch.bfloat16):
  """The activation quantiser inside gmm_v2 (pallas_mosaic_tpu_v2_gmm_kernel.py:489-542), restated op by op.

  Dynamic (static_scale None, :533-542), per row and per `quant_block` values of K, every op in x's dtype (the
  python scalars dtype_max, 0 and 1 are weakly typed, so a bf16 input keeps the arithmetic in bf16):
      block_abs_max   = max |x|                                  (exact)
      block_scale     = block_abs_max / dtype_max
      block_scale_inv = where(block_scale == 0, 0, 1 / block_scale)
      q               = (x * block_scale_inv).astype(qdtype)     (int8: truncation; fp8: nearest even)
  Static (:528-531, scale from get_static_scale as a (1, 1) array, ops.py:333-360): lhs_scale is cast to the
  accumulator dtype (bf16 unless the caller asks otherwise, :1247-1254), lhs_scale_inv = 1.0 / lhs_scale in that
  dtype, q = clip(x * lhs_scale_inv, -dtype_max, dtype_max).astype(qdtype) in the promoted dtype.

  The last block may be ragged (K % quant_block != 0 is rejected by the reference's tiling; allowed here).
  Returns (q [m, k] qdtype, scale f32 [m, ceil(k / quant_block)] holding the values of x's dtype; static: [1, 1])."""
  dt = x.dtype
  assert dt in (torch.bfloat16, torch.float32)
  xf = x.to(torch.float32)
  m, k = xf.shape
  qmax = qdtype_max(qdtype)
  if static_scale is not None:
    wide = torch.float32 if torch.float32 in (dt, acc_dtype) else torch.bfloat16  # jnp promotion of x * lhs_scale_inv
    s = _round_to(torch.tensor([[float(static_scale)]], dtype=torch.float32), acc_dtype)
    inv = _round_to(1.0 / s, acc_dtype)
    y = _round_to(xf * inv, wide).clamp(-qmax, qmax)
    return _astype_q(y, qdtype), s
  nb = math.ceil(k / quant_block)
  q = torch.empty((m, k), dtype=qdtype)
  scale = torch.empty((m, nb), dtype=torch.float32)
  for b in range(nb):
    blk = xf[:, b * quant_block : (b + 1) * quant_block]
    amax = blk.abs().amax(dim=1, keepdim=True)
    s = _round_to(amax / qmax, dt)
    inv = torch.where(s == 0, torch.zeros_like(s), _round_to(1.0 / s, dt))
    q[:, b * quant_block : (b + 1) * quant_block] = _astype_q(_round_to(blk * inv, dt), qdtype)
    scale[:, b] = s[:, 0]
  return q, scale


def manual_quantize(w: torch.Tensor, qdtype, calibration_method: str):
  """layers/quantizations.py:961-991: per-tensor static quantisation of a weight,
  q = clip(w / scale, -qmax, qmax).astype(qdtype) with scale, qmax as bf16 tensors (_make_scale_tensor :923-925:
  dtype=jnp.bfloat16), so w / scale is computed in promote(w.dtype, bf16); the QArray's scale is the python
  float cast to w's dtype, shape [1] * ndim.  Returns (q, scale f32 scalar tensor holding that value)."""
  qmax = qdtype_max(qdtype)
  scale = get_static_scale(qmax, calibration_method)
  s_bf = _round_to(torch.tensor(float(scale)), torch.bfloat16)
  y = _round_to(w.to(torch.float32) / s_bf, w.dtype)
  bound = float(_round_to(torch.tensor(qmax), torch.bfloat16))
  q = _astype_q(y.clamp(-bound, bound), qdtype)
  return q, _round_to(torch.tensor(float(scale)), w.dtype)


def _absmax_scale(x: torch.Tensor, dim, qmax: float):
  absmax = x.abs().to(torch.float32).amax(dim=dim, keepdim=True)
  return absmax / qmax


def _quant_int(x: torch.Tensor, scale: torch.Tensor, qmin: float, qmax: float):
  x = x.to(torch.float32)
  q = torch.where(scale == 0, torch.zeros_like(x), torch.round(x / scale))  # torch.round = half-to-even
  return q.clamp(qmin, qmax)


def quantize_rows_int8(x: torch.Tensor):
  """Per-row (per-token) symmetric int8, scale [m] f32 (ops.py:241-248:
  channelwise_axes=[0]; rounding unpinned, see module docstring)."""
  scale = _absmax_scale(x, -1, INT8_MAX)
  q = _quant_int(x, scale, -INT8_MAX, INT8_MAX).to(torch.int8)
  return q, scale.squeeze(-1)


def quantize_rows_fp8(x: torch.Tensor):
  """Per-row float8_e4m3fn quantisation of activations [m, k]: the [m, 1] scale of qpl.quantize(lhs, float8_e4m3fn,
  channelwise_axes=[0]) (ops.py:241-248) under this build's v1 rule: scale = absmax / 448, q = e4m3(x / scale) rounded
  to nearest even, zero rows give q = 0 and scale 0.  -> (q float8_e4m3fn, scale f32 [m])."""
  x = x.to(torch.float32)
  scale = _absmax_scale(x, 1, 448.0)
  q = torch.where(scale == 0, torch.zeros_like(x), x / scale).clamp(-448.0, 448.0).to(torch.float8_e4m3fn)
  return q, scale.squeeze(1)


def quantize_weight_int8(w: torch.Tensor, per_expert: bool = True):
  """w [g, k, n] -> int8 [g,k,n], scale [g, n] f32.  per_expert=True is the
  serve-mode layout gathered per row at moe.py:1450-1459; per_expert=False
  shares one [n] scale across experts and K (ops.py:250-260)."""
  if per_expert:
    scale = _absmax_scale(w, 1, INT8_MAX)  # [g,1,n]
  else:
    scale = _absmax_scale(w, (0, 1), INT8_MAX).expand(w.shape[0], 1, w.shape[2])
  q = _quant_int(w, scale, -INT8_MAX, INT8_MAX).to(torch.int8)
  return q, scale.squeeze(1).contiguous()


def quantize_fp8_blocks(x: torch.Tensor, block_rows: int, block_cols: int):
  """Symmetric float8_e4m3fn with one f32 scale per [block_rows, block_cols]
  block of the last two dims (ragged edge blocks allowed).  1x128 for
  activations, 128x128 for weights (DeepSeek-V3 recipe; storage format follows
  checkpoint_conversion/standalone_scripts/deepseek_dequantize.py:42-68).
  Returns (q float8_e4m3fn same shape, scale [..., ceil(r/br), ceil(c/bc)])."""
  *lead, r, c = x.shape
  nr, nc = math.ceil(r / block_rows), math.ceil(c / block_cols)
  xp = torch.zeros(*lead, nr * block_rows, nc * block_cols, dtype=torch.float32)
  xp[..., :r, :c] = x.to(torch.float32)
  xb = xp.reshape(*lead, nr, block_rows, nc, block_cols)
  absmax = xb.abs().amax(dim=(-3, -1), keepdim=True)
  scale = absmax / FP8_E4M3_MAX
  q = torch.where(scale == 0, torch.zeros_like(xb), xb / scale).clamp(-FP8_E4M3_MAX, FP8_E4M3_MAX)
  q = q.reshape(*lead, nr * block_rows, nc * block_cols)[..., :r, :c].to(torch.float8_e4m3fn)
  return q.contiguous(), scale.reshape(*lead, nr, nc).contiguous()


def dequantize_fp8_blocks(q: torch.Tensor, scale: torch.Tensor, block: int = 128) -> torch.Tensor:
  """deepseek_dequantize.py:42-68 (float scale branch): x * repeat(scale) -> bf16."""
  r, c = q.shape[-2:]
  s = torch.repeat_interleave(torch.repeat_interleave(scale.to(torch.float32), block, dim=-2), block, dim=-1)
  return (q.to(torch.float32) * s[..., :r, :c]).to(torch.bfloat16)


def quantize_int4_groups(w: torch.Tensor, group: int = 128):
  """Symmetric int4 with one scale per `group` consecutive elements of the
  last (contraction) axis; restates _quantize_per_group of
  tests/unit/dequantize_pack_quantized_int4_test.py:46-53 (scale clamped at
  1e-12, round, clamp [-8, 7]) and allows a ragged last group.
  Returns (int8 values in [-8,7] same shape, scale [..., ceil(K/group)] f32)."""
  *lead, kdim = w.shape
  ng = math.ceil(kdim / group)
  wp = torch.zeros(*lead, ng * group, dtype=torch.float32)
  wp[..., :kdim] = w.to(torch.float32)
  wg = wp.reshape(*lead, ng, group)
  scale = (wg.abs().amax(-1, keepdim=True) / INT4_MAX).clamp(min=1e-12)
  q = torch.round(wg / scale).clamp(-8, 7).to(torch.int8).reshape(*lead, ng * group)[..., :kdim]
  return q.contiguous(), scale.squeeze(-1).contiguous()


def pack_int4(q: torch.Tensor) -> torch.Tensor:
  """Two values per byte along the last axis, first value in the low nibble,
  stored as value + 8 -- byte-identical (little endian) to the int32 layout
  described at convert_deepseek_family_ckpt.py:62-66 (weight k in bits
  [4k, 4k+4))."""
  assert q.shape[-1] % 2 == 0
  u = (q.to(torch.int16) + 8).to(torch.uint8)
  return (u[..., 0::2] | (u[..., 1::2] << 4)).contiguous()


def unpack_int4(packed: torch.Tensor) -> torch.Tensor:
  """Inverse of pack_int4 (convert_deepseek_family_ckpt.py:72-74: nibble - 8)."""
  lo = (packed & 0xF).to(torch.int8) - 8
  hi = (packed >> 4).to(torch.int8) - 8
  return torch.stack([lo, hi], dim=-1).reshape(*packed.shape[:-1], packed.shape[-1] * 2)


def dequantize_int4(packed: torch.Tensor, scale: torch.Tensor, group: int = 128) -> torch.Tensor:
  """convert_deepseek_family_ckpt.py:56-84: (nibble-8) * scale per group -> bf16."""
  q = unpack_int4(packed).to(torch.float32)
  kdim = q.shape[-1]
  s = torch.repeat_interleave(scale.to(torch.float32), group, dim=-1)[..., :kdim]
  return (q * s).to(torch.bfloat16)


# --------------------------------------------------------------------------
# Whole layer: sparse path (moe.py:2186-2294) and two independent restatements
# --------------------------------------------------------------------------


def moe_layer_sparse(x: torch.Tensor, weights: np.ndarray, idx: np.ndarray, num_experts: int, expert_fn):
  """permute -> expert_fn(sorted_inputs, group_sizes) -> unpermute.
  expert_fn maps the sorted [M,d] rows to [M,d] outputs (gmm x3 + activation)."""
  k = idx.shape[-1]
  sorted_inputs, perm, group_size, _ = permute(x, idx, num_experts)
  inter = expert_fn(sorted_inputs, group_size)
  return unpermute(inter, perm, weights, k, out_dtype=x.dtype)


def moe_layer_loop(x: torch.Tensor, weights: np.ndarray, idx: np.ndarray, num_experts: int, mlp_fn):
  """Per-expert masked loop, the ground truth of tests/unit/moe_test.py:344-411
  (MoeLoopBlock): out = sum_e mask_e * w * MLP_e(x).  mlp_fn(e, rows)->[r,d]."""
  t, d = x.shape
  out = torch.zeros((t, d), dtype=torch.float32)
  w = torch.from_numpy(np.ascontiguousarray(weights, dtype=np.float32))
  for e in range(num_experts):
    tok, slot = np.nonzero(idx == e)
    if tok.size == 0:
      continue
    y = mlp_fn(e, x[torch.from_numpy(tok)]).to(torch.float32)
    out.index_add_(0, torch.from_numpy(tok), y * w[torch.from_numpy(tok), torch.from_numpy(slot)][:, None])
  return out.to(x.dtype)


# --------------------------------------------------------------------------
# MXFP4 (OCP microscaling fp4, the GPT-OSS checkpoint format)
# --------------------------------------------------------------------------

# e2m1 code -> value: bit 3 sign, bits 2..1 exponent (bias 1), bit 0 mantissa; exponent 0 is subnormal
# (src/maxtext/checkpoint_conversion/standalone_scripts/dequantize_mxfp4.py:46-59).
E2M1_VALUES = np.array([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0, -0.0, -0.5, -1.0, -1.5, -2.0, -3.0, -4.0, -6.0], np.float32)


def dequantize_mxfp4(blocks: torch.Tensor, scales: torch.Tensor) -> torch.Tensor:
  """dequantize_mxfp4.py:62-72: blocks uint8 [..., G, 16] hold 32 e2m1 values each, first value in the low nibble;
  scales uint8 [..., G] are e8m0 exponents, value = e2m1 * 2^(scale - 127).  -> float32 [..., G * 32]."""
  b = blocks.to(torch.int64)
  table = torch.from_numpy(E2M1_VALUES)
  vals = torch.stack([table[b & 0xF], table[b >> 4]], -1)  # [..., G, 16, 2]
  factor = torch.exp2(scales.to(torch.float32) - 127.0)[..., None, None]
  out = vals * factor
  return out.reshape(out.shape[:-3] + (-1,))


def quantize_mxfp4(w: torch.Tensor):
  """Test-data generator (no counterpart in the reference): [..., K] f32 -> (blocks uint8 [..., K/32, 16], scales
  uint8 [..., K/32]) by the OCP MX rule: shared exponent = floor(log2(absmax of the block)) - 2 (2 = exponent of
  the largest e2m1 normal, 6 = 1.5 * 2^2), elements rounded to the nearest e2m1 value (ties to the even code),
  saturating at +-6."""
  k = w.shape[-1]
  assert k % 32 == 0
  x = w.float().reshape(w.shape[:-1] + (k // 32, 32))
  amax = x.abs().amax(-1, keepdim=True)
  exp = torch.where(amax > 0, torch.floor(torch.log2(amax.clamp_min(1e-38))) - 2.0, torch.zeros_like(amax)).clamp(-127, 127)
  y = (x / torch.exp2(exp)).clamp(-6.0, 6.0)
  grid = torch.tensor([0.0, 0.5, 1.0, 1.5, 2.0, 3.0, 4.0, 6.0])
  d = (y.abs()[..., None] - grid).abs()
  # nearest grid point; on a tie prefer the even code (codes 0, 2, 4, 6 have mantissa bit 0)
  tie_break = torch.tensor([0.0, 1e-6, 0.0, 1e-6, 0.0, 1e-6, 0.0, 1e-6])
  code = torch.argmin(d + tie_break, dim=-1)
  code = code + 8 * (y < 0).long()
  blocks = (code[..., 0::2] | (code[..., 1::2] << 4)).to(torch.uint8)
  scales = (exp.squeeze(-1) + 127.0).to(torch.uint8)
  return blocks, scales
