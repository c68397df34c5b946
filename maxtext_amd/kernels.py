"""Thin torch-tensor wrappers over the C ABI (one function per entry point).

Each wrapper checks device, dtype, contiguity and shapes on the host before the launch,
allocates outputs/workspaces with torch and enqueues on torch's current stream.
"""

from __future__ import annotations

import ctypes

import torch

from maxtext_amd import _lib
from maxtext_amd._lib import (MOE_BF16, MOE_FP8_E4M3, MOE_FP8_E5M2, MOE_INT4, MOE_INT8, MOE_MXFP4, MOE_ROUTE_DEEPSEEK, MOE_ROUTE_SOFTMAX_TOPK)

_DTYPE_CODE = {torch.bfloat16: MOE_BF16, torch.int8: MOE_INT8, torch.float8_e4m3fn: MOE_FP8_E4M3}
_LHS_DTYPE_CODE = dict(_DTYPE_CODE)
_LHS_DTYPE_CODE[torch.float8_e5m2] = MOE_FP8_E5M2  # the quantised gradient of the backward; activations only


def _need(t: torch.Tensor, name: str, dtype=None, ndim=None):
  if not isinstance(t, torch.Tensor):
    raise TypeError(f"{name} must be a torch.Tensor")
  if not t.is_cuda:
    raise ValueError(f"{name} must live on the GPU (the MoE path has no CPU implementation)")
  if not t.is_contiguous():
    raise ValueError(f"{name} must be contiguous")
  if dtype is not None and t.dtype != dtype:
    raise TypeError(f"{name} must be {dtype}, got {t.dtype}")
  if ndim is not None and t.dim() != ndim:
    raise ValueError(f"{name} must have {ndim} dims, got shape {tuple(t.shape)}")


def route_topk(gate_logits, pre_bias_logits=None, *, k, mode="softmax_topk", norm_topk_prob=False,
               weights_round_bf16=True, routed_scaling_factor=1.0, n_routing_groups=-1, topk_routing_group=-1):
  """-> (weights [T,k] f32, indices [T,k] int32)."""
  _need(gate_logits, "gate_logits", torch.float32, 2)
  t, e = gate_logits.shape
  if mode not in _lib.ROUTE_BY_NAME:
    raise ValueError(f"unknown routing mode {mode!r}")
  code = _lib.ROUTE_BY_NAME[mode]
  if mode == "deepseek":
    _need(pre_bias_logits, "pre_bias_logits", torch.float32, 2)
    if pre_bias_logits.shape != gate_logits.shape:
      raise ValueError("pre_bias_logits must match gate_logits")
  w = torch.empty((t, k), dtype=torch.float32, device=gate_logits.device)
  idx = torch.empty((t, k), dtype=torch.int32, device=gate_logits.device)
  lib = _lib.load()
  st = lib.moe_route_topk(_lib.ptr(gate_logits), _lib.ptr(pre_bias_logits) if mode == "deepseek" else None, t, e, k, code,
                          int(bool(norm_topk_prob)), int(bool(weights_round_bf16)), float(routed_scaling_factor),
                          int(n_routing_groups), int(topk_routing_group), _lib.ptr(w), _lib.ptr(idx), _lib.current_stream())
  _lib.check(st, "moe_route_topk")
  return w, idx


def route_sort(gate_logits, pre_bias_logits=None, *, k, gmm_workspace, mode="softmax_topk", norm_topk_prob=False, weights_round_bf16=True,
               routed_scaling_factor=1.0, n_routing_groups=-1, topk_routing_group=-1, roll_to_expert_id=0, tile_rows=16):
  """route_topk and sort_by_expert(..., gmm_workspace=...) through one call (one launch up to 16 tokens):
  -> (weights [T,k] f32, indices [T,k] int32, perm [M], inv_perm [M], group_sizes [E]), as those two return them."""
  _need(gate_logits, "gate_logits", torch.float32, 2)
  t, e = gate_logits.shape
  if mode not in _lib.ROUTE_BY_NAME:
    raise ValueError(f"unknown routing mode {mode!r}")
  if mode == "deepseek":
    _need(pre_bias_logits, "pre_bias_logits", torch.float32, 2)
    if pre_bias_logits.shape != gate_logits.shape:
      raise ValueError("pre_bias_logits must match gate_logits")
  _need(gmm_workspace, "gmm_workspace", torch.uint8)
  dev = gate_logits.device
  m = t * k
  w = torch.empty((t, k), dtype=torch.float32, device=dev)
  idx = torch.empty((t, k), dtype=torch.int32, device=dev)
  perm = torch.empty((m,), dtype=torch.int32, device=dev)
  inv = torch.empty((m,), dtype=torch.int32, device=dev)
  gs = torch.empty((e,), dtype=torch.int32, device=dev)
  lib = _lib.load()
  ws = torch.empty((max(lib.moe_sort_workspace_bytes(t, k, e), 16),), dtype=torch.uint8, device=dev)
  st = lib.moe_route_sort_mapped(_lib.ptr(gate_logits), _lib.ptr(pre_bias_logits) if mode == "deepseek" else None, t, e, k, _lib.ROUTE_BY_NAME[mode],
                                 int(bool(norm_topk_prob)), int(bool(weights_round_bf16)), float(routed_scaling_factor), int(n_routing_groups),
                                 int(topk_routing_group), _lib.ptr(w), _lib.ptr(idx), int(roll_to_expert_id), _lib.ptr(perm), _lib.ptr(inv),
                                 _lib.ptr(gs), None, _lib.ptr(ws), ws.numel(), int(tile_rows), e, 0, 0, _lib.ptr(gmm_workspace),
                                 gmm_workspace.numel(), _lib.current_stream())
  _lib.check(st, "moe_route_sort_mapped")
  return w, idx, perm, inv, gs


_SCORE_FUNC_CODE = {"": 0, "sigmoid": 1, "sqrtsoftplus": 2}


def gate_route(x, gate_kernel_terms, gate_bias=None, *, k, score_func="", gate_round_bf16=False, mode="softmax_topk",
               norm_topk_prob=False, weights_round_bf16=True, routed_scaling_factor=1.0, n_routing_groups=-1,
               topk_routing_group=-1, return_logits=False):
  """Gate matmul + score function + bias + top-k.  x [T, d] bf16; gate_kernel_terms [S, E, d] bf16 (S = 1 or 3).
  -> (weights [T,k] f32, indices [T,k] int32[, gate_logits [T,E] f32, pre_bias_logits [T,E] f32])."""
  _need(x, "x", torch.bfloat16, 2)
  _need(gate_kernel_terms, "gate_kernel_terms", torch.bfloat16, 3)
  t, d = x.shape
  s_, e, d2 = gate_kernel_terms.shape
  if d2 != d:
    raise ValueError(f"gate kernel has d={d2}, x has d={d}")
  if gate_bias is not None:
    _need(gate_bias, "gate_bias", torch.float32, 1)
    if gate_bias.numel() != e:
      raise ValueError("gate_bias must have E elements")
  if score_func not in _SCORE_FUNC_CODE:
    raise NotImplementedError(f"score_func {score_func!r}")
  if mode not in _lib.ROUTE_BY_NAME:
    raise ValueError(f"unknown routing mode {mode!r}")
  dev = x.device
  w = torch.empty((t, k), dtype=torch.float32, device=dev)
  idx = torch.empty((t, k), dtype=torch.int32, device=dev)
  logits = torch.empty((t, e), dtype=torch.float32, device=dev) if return_logits else None
  pre = torch.empty((t, e), dtype=torch.float32, device=dev) if return_logits else None
  lib = _lib.load()
  ws = torch.empty((max(lib.moe_gate_route_workspace_bytes(t, d, e), 16),), dtype=torch.uint8, device=dev)
  st = lib.moe_gate_route(_lib.ptr(x), _lib.ptr(gate_kernel_terms), s_, _lib.ptr(gate_bias), t, d, e, k,
                          _SCORE_FUNC_CODE[score_func], int(bool(gate_round_bf16)),
                          _lib.ROUTE_BY_NAME[mode], int(bool(norm_topk_prob)),
                          int(bool(weights_round_bf16)), float(routed_scaling_factor), int(n_routing_groups),
                          int(topk_routing_group), _lib.ptr(w), _lib.ptr(idx), _lib.ptr(logits), _lib.ptr(pre), _lib.ptr(ws),
                          ws.numel(), _lib.current_stream())
  _lib.check(st, "moe_gate_route")
  return (w, idx, logits, pre) if return_logits else (w, idx)


def sort_by_expert(topk_idx, num_experts, *, want_sorted_experts=True, roll_to_expert_id=0, gmm_workspace=None, tile_rows=16, out=None):
  """-> (perm [M], inv_perm [M], group_sizes [E], sorted_experts [M] or None), all int32.
  roll_to_expert_id: the ids are sorted as (id - roll_to_expert_id) mod num_experts (moe.py:953-954).
  gmm_workspace (from gmm_workspace(M, num_experts)): up to 4096 routed rows the sort also leaves the grouped matmuls'
  tile list of height tile_rows there, which gmm_raw(..., workspace=gmm_workspace, same_groups=True) then uses.
  out: (perm, inv_perm, group_sizes, sorted_experts) buffers of an earlier call, written again (a caller with
  persistent buffers)."""
  _need(topk_idx, "topk_idx", torch.int32, 2)
  t, k = topk_idx.shape
  m = t * k
  dev = topk_idx.device
  lib = _lib.load()
  if out is not None:
    perm, inv, gs, se = out
    for name, buf, size in (("perm", perm, m), ("inv_perm", inv, m), ("group_sizes", gs, num_experts)):
      _need(buf, name, torch.int32, 1)
      if buf.numel() != size:
        raise ValueError(f"out: {name} must hold {size} entries")
    if se is not None and se.numel() != m:
      raise ValueError(f"out: sorted_experts must hold {m} entries")
  else:
    perm = torch.empty((m,), dtype=torch.int32, device=dev)
    inv = torch.empty((m,), dtype=torch.int32, device=dev)
    gs = torch.empty((num_experts,), dtype=torch.int32, device=dev)
    se = torch.empty((m,), dtype=torch.int32, device=dev) if want_sorted_experts else None
  nbytes = lib.moe_sort_workspace_bytes(t, k, num_experts)
  ws = torch.empty((max(nbytes, 16),), dtype=torch.uint8, device=dev)
  if gmm_workspace is not None:
    st = lib.moe_sort_by_expert_mapped(_lib.ptr(topk_idx), t, k, num_experts, int(roll_to_expert_id), _lib.ptr(perm), _lib.ptr(inv),
                                       _lib.ptr(gs), _lib.ptr(se), _lib.ptr(ws), ws.numel(), int(tile_rows), num_experts, 0, 0,
                                       _lib.ptr(gmm_workspace), gmm_workspace.numel(), _lib.current_stream())
    _lib.check(st, "moe_sort_by_expert_mapped")
    return perm, inv, gs, se
  if isinstance(roll_to_expert_id, torch.Tensor):  # a device scalar (the reference's comes from jax.lax.axis_index): never read here
    _need(roll_to_expert_id, "roll_to_expert_id", torch.int32)
    if roll_to_expert_id.numel() != 1:
      raise ValueError("roll_to_expert_id must hold one value")
    st = lib.moe_sort_by_expert_rolled_dev(_lib.ptr(topk_idx), t, k, num_experts, _lib.ptr(roll_to_expert_id), _lib.ptr(perm), _lib.ptr(inv),
                                           _lib.ptr(gs), _lib.ptr(se), _lib.ptr(ws), ws.numel(), _lib.current_stream())
    _lib.check(st, "moe_sort_by_expert_rolled_dev")
    return perm, inv, gs, se
  st = lib.moe_sort_by_expert_rolled(_lib.ptr(topk_idx), t, k, num_experts, int(roll_to_expert_id), _lib.ptr(perm), _lib.ptr(inv),
                                     _lib.ptr(gs), _lib.ptr(se), _lib.ptr(ws), ws.numel(), _lib.current_stream())
  _lib.check(st, "moe_sort_by_expert_rolled")
  return perm, inv, gs, se


def gather_rows(x, row_idx=None, idx_div=1, *, out_dtype=torch.bfloat16, block_k=0, num_rows=None, rule="rint_div", static_scale=None,
                row_weight=None, row_range=None):
  """Row gather (+ int8 / fp8 quantisation, one scale per row or per `block_k` values of a row, or one static scale).
  rule: "rint_div" (v1 path) or "v2" (the in-kernel quantiser of gmm_v2).  row_weight [R_out] f32 multiplies each
  gathered row; row_range int32 [2] (start, end) on the device zeroes the output rows outside it.  -> out or (q, scale)."""
  _need(x, "x", torch.bfloat16, 2)
  r_in, d = x.shape
  if row_idx is not None:
    _need(row_idx, "row_idx", torch.int32, 1)
    r_out = row_idx.shape[0]
  else:
    r_out = r_in if num_rows is None else num_rows
  if rule not in _lib.QUANT_RULE_BY_NAME:
    raise ValueError(f"unknown quantisation rule {rule!r}")
  quantised = out_dtype in (torch.int8, torch.float8_e4m3fn)
  if not quantised and out_dtype != torch.bfloat16:
    raise TypeError(f"out_dtype {out_dtype} not supported")
  if quantised and static_scale is None and block_k not in (0, 128, 256, 512):
    raise ValueError(f"block_k must be 0 (one scale per row), 128, 256 or 512, got {block_k}")
  out = torch.empty((r_out, d), dtype=out_dtype, device=x.device)
  scale = None
  if quantised and static_scale is not None:
    _need(static_scale, "static_scale", torch.float32)
    if static_scale.numel() != 1:
      raise ValueError("static_scale must hold one value")
  elif quantised:
    scale = torch.empty((r_out,) if block_k == 0 else (r_out, (d + block_k - 1) // block_k), dtype=torch.float32, device=x.device)
  if row_weight is not None:
    _need(row_weight, "row_weight", torch.float32, 1)
    if row_weight.numel() != r_out:
      raise ValueError("row_weight must have one value per output row")
  if row_range is not None:
    _need(row_range, "row_range", torch.int32, 1)
    if row_range.numel() != 2:
      raise ValueError("row_range must hold (start, end)")
  lib = _lib.load()
  st = lib.moe_gather_rows(_lib.ptr(x), _lib.ptr(row_idx), int(idx_div), r_in, r_out, d, _DTYPE_CODE[out_dtype], int(block_k),
                           _lib.QUANT_RULE_BY_NAME[rule], _lib.ptr(static_scale) if quantised else None, _lib.ptr(row_weight),
                           _lib.ptr(row_range), _lib.ptr(out), _lib.ptr(scale), _lib.current_stream())
  _lib.check(st, "moe_gather_rows")
  if not quantised:
    return out
  return out, (static_scale if static_scale is not None else scale)


def _shard_on_device(shard, name, device):
  """A shard index given as a tensor stays on the device (int32, one element): the `_dev` entry points read it there."""
  if not isinstance(shard, torch.Tensor):
    return None
  if shard.numel() != 1:
    raise ValueError(f"{name} must hold one value")
  return shard.to(device=device, dtype=torch.int32).reshape(1).contiguous()


def local_expert_keys(global_group_sizes, local_expert_size, shard_index, num_rows, *, global_sorted_experts=None, truncate=False):
  """Index half of RoutedMoE.local_permute (moe.py:1091-1200) before its argsort.
  global_group_sizes [batch shards, E] int32 -> (expert_keys [num_rows] int32, local_group_size [local_expert_size] int32).
  shard_index: an int, or a one-element tensor (jax.lax.axis_index of the reference) that is read on the device."""
  _need(global_group_sizes, "global_group_sizes", torch.int32, 2)
  s, e = global_group_sizes.shape
  if global_sorted_experts is not None:
    _need(global_sorted_experts, "global_sorted_experts", torch.int32, 1)
    if global_sorted_experts.shape[0] != num_rows:
      raise ValueError("global_sorted_experts must name the expert of every row")
  dev = global_group_sizes.device
  lib = _lib.load()
  keys = torch.empty((num_rows,), dtype=torch.int32, device=dev)
  sizes = torch.empty((local_expert_size,), dtype=torch.int32, device=dev)
  ws = torch.empty((max(lib.moe_local_expert_keys_workspace_bytes(s, local_expert_size), 16),), dtype=torch.uint8, device=dev)
  shard_dev = _shard_on_device(shard_index, "shard_index", dev)
  if shard_dev is not None:
    st = lib.moe_local_expert_keys_dev(_lib.ptr(global_group_sizes), s, e, int(local_expert_size), _lib.ptr(shard_dev), int(num_rows),
                                       _lib.ptr(global_sorted_experts), int(bool(truncate)), _lib.ptr(keys), _lib.ptr(sizes), _lib.ptr(ws),
                                       ws.numel(), _lib.current_stream())
  else:
    st = lib.moe_local_expert_keys(_lib.ptr(global_group_sizes), s, e, int(local_expert_size), int(shard_index), int(num_rows),
                                   _lib.ptr(global_sorted_experts), int(bool(truncate)), _lib.ptr(keys), _lib.ptr(sizes), _lib.ptr(ws),
                                   ws.numel(), _lib.current_stream())
  _lib.check(st, "moe_local_expert_keys")
  return keys, sizes


def all_to_all_params(all_shards_group_sizes, shard_id, num_expert_parallelism, *, is_batch_sharded=True, buffer_size=None,
                      is_dispatch=True):
  """RoutedMoE.get_all_to_all_params (moe.py:1202-1349) -> (input_offsets, send_sizes, output_offsets, recv_sizes),
  int32 [num_expert_parallelism] each, on the device.  buffer_size: a receiver's capacity, or None."""
  _need(all_shards_group_sizes, "all_shards_group_sizes", torch.int32, 2 if is_batch_sharded else 1)
  p = int(num_expert_parallelism)
  if tuple(all_shards_group_sizes.shape) != ((p, p) if is_batch_sharded else (p,)):
    raise ValueError(f"all_shards_group_sizes has shape {tuple(all_shards_group_sizes.shape)} for {p} shards")
  out = torch.empty((4, p), dtype=torch.int32, device=all_shards_group_sizes.device)
  shard_dev = _shard_on_device(shard_id, "shard_id", all_shards_group_sizes.device)
  tail = (int(bool(is_batch_sharded)), -1 if buffer_size is None else int(buffer_size), int(bool(is_dispatch)), _lib.ptr(out[0]),
          _lib.ptr(out[1]), _lib.ptr(out[2]), _lib.ptr(out[3]), _lib.current_stream())
  if shard_dev is not None:
    st = _lib.load().moe_all_to_all_params_dev(_lib.ptr(all_shards_group_sizes), p, _lib.ptr(shard_dev), *tail)
  else:
    st = _lib.load().moe_all_to_all_params(_lib.ptr(all_shards_group_sizes), p, int(shard_id), *tail)
  _lib.check(st, "moe_all_to_all_params")
  return out[0], out[1], out[2], out[3]


def ring_ragged_indices(indices, group_sizes, experts_start, local_experts, *, buffer_size=None, unsort=False, shard_index=None):
  """Index arrays of ring_ragged_sort / ring_ragged_unsort (kernels/ragged/ragged_sort.py:102-151, :300-350).
  unsort=False: indices = perm -> (row_idx [min(buffer, n)], row_range [2]); unsort=True: indices = inv_perm ->
  (inv_perm into the shard's buffer [n], valid_rows_mask [n] uint8).
  shard_index: a one-element tensor read on the device; the shard then owns experts [shard * local_experts, + local_experts)
  and experts_start is ignored."""
  _need(indices, "indices", torch.int32, 1)
  _need(group_sizes, "group_sizes", torch.int32, 1)
  n = indices.shape[0]
  buf = n if buffer_size is None else int(buffer_size)
  dev = indices.device
  out = torch.empty((n if unsort else min(buf, n),), dtype=torch.int32, device=dev)
  mask = torch.empty((n,), dtype=torch.uint8, device=dev) if unsort else None
  rng = None if unsort else torch.empty((2,), dtype=torch.int32, device=dev)
  shard_dev = _shard_on_device(shard_index, "shard_index", dev)
  tail = (int(local_experts), n, buf, int(bool(unsort)), _lib.ptr(out), _lib.ptr(mask), _lib.ptr(rng), _lib.current_stream())
  if shard_dev is not None:
    st = _lib.load().moe_ring_ragged_indices_dev(_lib.ptr(indices), _lib.ptr(group_sizes), group_sizes.shape[0], _lib.ptr(shard_dev), *tail)
  else:
    st = _lib.load().moe_ring_ragged_indices(_lib.ptr(indices), _lib.ptr(group_sizes), group_sizes.shape[0], int(experts_start), *tail)
  _lib.check(st, "moe_ring_ragged_indices")
  return (out, mask) if unsort else (out, rng)


def _valid_mask(valid_rows_mask, m):
  if valid_rows_mask is None:
    return None
  _need(valid_rows_mask, "valid_rows_mask", None, None)
  if valid_rows_mask.dtype not in (torch.bool, torch.uint8) or valid_rows_mask.numel() != m:
    raise ValueError("valid_rows_mask must hold T*k bool or uint8 entries")
  return valid_rows_mask.view(torch.uint8)


def unpermute_combine(y, weights, *, k, perm=None, inv_perm=None, valid_rows_mask=None, num_tokens=None):
  """out[t] = sum over the valid s of weights[t,s] * y[inv_perm[t*k+s]]  (f32 accumulate, bf16 out).
  num_tokens: T when y is a packed buffer with other than T*k rows (needs inv_perm, whose valid entries index y)."""
  _need(y, "y", torch.bfloat16, 2)
  m, d = y.shape
  if num_tokens is not None:
    if inv_perm is None:
      raise ValueError("num_tokens needs inv_perm")
    m = int(num_tokens) * k
  if m % k:
    raise ValueError("rows of y must be a multiple of k")
  t = m // k
  valid = _valid_mask(valid_rows_mask, m)
  if weights is not None:
    _need(weights, "weights", torch.float32)
    if weights.numel() != m:
      raise ValueError("weights must have T*k elements")
  ws = None
  if inv_perm is None:
    _need(perm, "perm", torch.int32, 1)
    if perm.numel() != m:
      raise ValueError("perm must have T*k elements")
    ws = torch.empty((m,), dtype=torch.int32, device=y.device)
  else:
    _need(inv_perm, "inv_perm", torch.int32, 1)
    if inv_perm.numel() != m:
      raise ValueError("inv_perm must have T*k elements")
  out = torch.empty((t, d), dtype=torch.bfloat16, device=y.device)
  lib = _lib.load()
  st = lib.moe_unpermute_combine(_lib.ptr(y), _lib.ptr(perm), _lib.ptr(inv_perm), _lib.ptr(weights), _lib.ptr(valid), t, k, d, _lib.ptr(out),
                                 _lib.ptr(ws), 0 if ws is None else ws.numel() * 4, _lib.current_stream())
  _lib.check(st, "moe_unpermute_combine")
  return out


def unpermute_combine_bwd(dout, y, weights, *, k, inv_perm, need_dweights=True, valid_rows_mask=None):
  """Gradient of unpermute_combine: -> (dy [M, d] bf16, dweights [T, k] f32 or None)."""
  _need(dout, "dout", torch.bfloat16, 2)
  _need(inv_perm, "inv_perm", torch.int32, 1)
  t, d = dout.shape
  m = t * k
  valid = _valid_mask(valid_rows_mask, m)
  if inv_perm.numel() != m:
    raise ValueError("inv_perm must have T*k elements")
  if weights is not None:
    _need(weights, "weights", torch.float32)
    if weights.numel() != m:
      raise ValueError("weights must have T*k elements")
  dw = None
  if need_dweights:
    _need(y, "y", torch.bfloat16, 2)
    if y.shape != (m, d):
      raise ValueError("y must be [T*k, d]")
    dw = torch.empty((t, k), dtype=torch.float32, device=dout.device)
  dy = torch.empty((m, d), dtype=torch.bfloat16, device=dout.device)
  lib = _lib.load()
  st = lib.moe_unpermute_combine_bwd(_lib.ptr(dout), _lib.ptr(y) if need_dweights else None, _lib.ptr(inv_perm), _lib.ptr(weights),
                                     _lib.ptr(valid), t, k, d, _lib.ptr(dy), _lib.ptr(dw), _lib.current_stream())
  _lib.check(st, "moe_unpermute_combine_bwd")
  return dy, dw


def glu_act(h0, h1, act="silu", act_limit=7.0):
  """act(h0, h1) elementwise on bf16 tensors of one shape -> bf16."""
  _need(h0, "h0", torch.bfloat16)
  _need(h1, "h1", torch.bfloat16)
  if h0.shape != h1.shape:
    raise ValueError("h0 and h1 must have one shape")
  out = torch.empty_like(h0)
  st = _lib.load().moe_glu_act(_lib.ptr(h0), _lib.ptr(h1), h0.numel(), _lib.ACT_BY_NAME[act], float(act_limit), _lib.ptr(out),
                               _lib.current_stream())
  _lib.check(st, "moe_glu_act")
  return out


def glu_act_bwd(h0, h1, dout, act="silu", act_limit=7.0):
  """-> (dh0, dh1), the gradient of glu_act."""
  for name, t in (("h0", h0), ("h1", h1), ("dout", dout)):
    _need(t, name, torch.bfloat16)
  if h0.shape != h1.shape or h0.shape != dout.shape:
    raise ValueError("h0, h1 and dout must have one shape")
  dh0, dh1 = torch.empty_like(h0), torch.empty_like(h0)
  st = _lib.load().moe_glu_act_bwd(_lib.ptr(h0), _lib.ptr(h1), _lib.ptr(dout), h0.numel(), _lib.ACT_BY_NAME[act], float(act_limit),
                                   _lib.ptr(dh0), _lib.ptr(dh1), _lib.current_stream())
  _lib.check(st, "moe_glu_act_bwd")
  return dh0, dh1


def bwd_scale_grad(dout, factor, *, mode, quantize, group_sizes=None, num_groups_local=None, group_offset=0, as_fp8=False):
  """Gradient preparation of the quantised backward (ops.py:530-604): `dout` [m, n] bf16 times the scale of the axis the
  gradient product contracts away, optionally quantised to float8_e5m2.

  mode "dlhs": factor = rhs scales [g_local, n] f32, picked per row by its expert (group_sizes); quantised per row.
  mode "drhs": factor = lhs scales [m] f32; quantised per column.
  mode "tensor": factor = the one scale [1] of an operand quantised per tensor (disable_channelwise_axes, ops.py:568-601);
  one scale for the whole gradient, returned as [n] equal entries (a column scale like any other; [:1] is the scalar).
  -> (d [m, n] bf16, scale): the e5m2 values (exact in bf16) and their f32 scales ([m] or [n]), or (dout * factor, None).
  as_fp8 (with quantize): d is returned as a float8_e5m2 tensor instead, the lhs of gmm_raw against e4m3 weights.
  """
  _need(dout, "dout", torch.bfloat16, 2)
  _need(factor, "factor", torch.float32)
  m, n = dout.shape
  code = {"dlhs": 0, "drhs": 1, "tensor": 2}[mode]
  if code == 0:
    _need(group_sizes, "group_sizes", torch.int32, 1)
    g_local = int(num_groups_local if num_groups_local is not None else factor.shape[0])
    if factor.numel() != g_local * n:
      raise ValueError(f"factor must hold [{g_local}, {n}] scales, got {tuple(factor.shape)}")
    g_total = group_sizes.numel()
  else:
    if factor.numel() != (m if code == 1 else 1):
      raise ValueError(f"factor must hold one scale {'per row (%d)' % m if code == 1 else 'for the tensor'}, got {tuple(factor.shape)}")
    g_total, g_local = 0, 0
  if as_fp8 and not quantize:
    raise ValueError("as_fp8 needs quantize")
  out = torch.empty((m, n), dtype=torch.float8_e5m2, device=dout.device) if as_fp8 else torch.empty_like(dout)
  scale = torch.empty((m if code == 0 else n,), dtype=torch.float32, device=dout.device) if quantize else None
  st = _lib.load().moe_bwd_scale_grad(_lib.ptr(dout), m, n, code, (2 if as_fp8 else 1) if quantize else 0, _lib.ptr(factor), _lib.ptr(group_sizes), g_total,
                                      g_local, int(group_offset), _lib.ptr(out), _lib.ptr(scale), _lib.current_stream())
  _lib.check(st, "moe_bwd_scale_grad")
  return out, scale


def tensor_scale(x, qmax):
  """absmax(x) / qmax of a bf16 matrix as a [1] f32 device tensor: the dynamic per-tensor scale of
  disable_channelwise_axes (ops.py:245), usable as gather_rows' static_scale."""
  _need(x, "x", torch.bfloat16, 2)
  scale = torch.empty((1,), dtype=torch.float32, device=x.device)
  st = _lib.load().moe_tensor_scale(_lib.ptr(x), x.shape[0], x.shape[1], float(qmax), _lib.ptr(scale), _lib.current_stream())
  _lib.check(st, "moe_tensor_scale")
  return scale


def quantize_rhs(w_gnk, out_dtype, *, shared=True, static_scale=None, per_tensor=False):
  """Weight quantiser of the training path (ops.py:250-266): w [G, N, K] bf16 -> (q [G, N, K] int8 / float8_e4m3fn, scale).
  Dynamic: one absmax scale per output channel, shared by the experts (scale [1, N]) or per expert ([G, N]), or one for
  the tensor (per_tensor: scale [1], disable_channelwise_axes);
  static_scale ([1] f32 on the device): manual_quantize's per-tensor rule, scale returned as given."""
  _need(w_gnk, "w", torch.bfloat16, 3)
  if out_dtype not in (torch.int8, torch.float8_e4m3fn):
    raise TypeError(f"out_dtype {out_dtype} not supported")
  g, n, k = w_gnk.shape
  q = torch.empty((g, n, k), dtype=out_dtype, device=w_gnk.device)
  scale = None
  if static_scale is not None:
    _need(static_scale, "static_scale", torch.float32)
    if static_scale.numel() != 1:
      raise ValueError("static_scale must hold one value")
  else:
    scale = torch.empty((1,) if per_tensor else (1, n) if shared else (g, n), dtype=torch.float32, device=w_gnk.device)
  st = _lib.load().moe_quantize_rhs(_lib.ptr(w_gnk), g, n, k, _DTYPE_CODE[out_dtype], 2 if per_tensor else 1 if shared else 0, _lib.ptr(static_scale), _lib.ptr(q),
                                    _lib.ptr(scale), _lib.current_stream())
  _lib.check(st, "moe_quantize_rhs")
  return q, (static_scale if static_scale is not None else scale)


def add_group_bias(h, bias, group_sizes, *, group_offset=0):
  """bf16(h + bias[expert of the row]) for the rows of the local groups (bias [G_local, N] f32), other rows copied."""
  _need(h, "h", torch.bfloat16, 2)
  _need(bias, "bias", torch.float32, 2)
  _need(group_sizes, "group_sizes", torch.int32, 1)
  m, n = h.shape
  if bias.shape[1] != n:
    raise ValueError(f"bias has {bias.shape[1]} channels for {n}")
  out = torch.empty_like(h)
  st = _lib.load().moe_add_group_bias(_lib.ptr(h), m, n, _lib.ptr(bias), _lib.ptr(group_sizes), group_sizes.numel(), bias.shape[0],
                                      int(group_offset), _lib.ptr(out), _lib.current_stream())
  _lib.check(st, "moe_add_group_bias")
  return out


def transpose_rhs(rhs_gkn):
  """[G, K, N] -> [G, N, K] for 1- or 2-byte element types."""
  _need(rhs_gkn, "rhs", None, 3)
  g, k, n = rhs_gkn.shape
  out = torch.empty((g, n, k), dtype=rhs_gkn.dtype, device=rhs_gkn.device)
  lib = _lib.load()
  st = lib.moe_transpose_rhs(_lib.ptr(rhs_gkn), g, k, n, rhs_gkn.element_size(), _lib.ptr(out), _lib.current_stream())
  _lib.check(st, "moe_transpose_rhs")
  return out


def gmm_raw(lhs, rhs, group_sizes, *, lhs_scale=None, rhs_scale=None, rhs_up=None, rhs_up_scale=None,
            rhs_dtype=None, lhs_scale_block_k=0, rhs_scale_block_n=1, rhs_scale_block_k=0, act=None, act_limit=7.0,
            group_offset=0, out=None, kernel=None, raster=0, rhs_bias=None, rhs_up_bias=None, partial_sum=None, partial_sum_up=None,
            keep_other_rows=False, rhs_kn=False, rhs_scale_kmajor=False, rhs_scale_shared=False, out_dtype=torch.bfloat16,
            lhs_row_idx=None, lhs_row_idx_div=1, out_row_scale=None, num_rows=None, workspace=None, same_groups=False,
            group_offset_dev=None):
  """Grouped matmul on native layouts: lhs [M,K], rhs [G,N,K] (INT4 / MXFP4: uint8 [G,N,K/2]).
  rhs_kn: rhs is [G,K,N] instead (bf16 x bf16 on shapes `gmm_rhs_kn_supported` accepts, fp8 x fp8 on shapes
  `gmm_fp8_rhs_kn_supported` accepts; no rhs_up).
  Scale layouts follow include/moe_mi355x.h: lhs_scale_block_k 0 = [M], -1 = [1] (per tensor), b = [M, ceil(K/b)];
  rhs scales [G, ceil(N/bn), ceil(K/bk)], or [G, ceil(K/bk), N] with rhs_scale_kmajor, without the leading G with
  rhs_scale_shared; bn = -1: one scale for all channels.
  lhs_row_idx [M] int32: row i of the product reads lhs row lhs_row_idx[i] // lhs_row_idx_div (lhs then has any number of
  rows); out_row_scale [M] f32 multiplies the result rows.  kernel / raster select a kernel family (moe_gmm_tuned).
  workspace: a caller-held uint8 buffer of moe_gmm_workspace_bytes; same_groups: MOE_GMM_SAME_GROUPS (group_sizes and the
  workspace are those of the previous call, untouched: its tile list is used again when the tile height agrees).
  group_offset_dev: int32 [1] on the device; replaces group_offset without the host ever reading it."""
  _need(lhs, "lhs", None, 2)
  _need(rhs, "rhs", None, 3)
  _need(group_sizes, "group_sizes", torch.int32, 1)
  lhs_rows, kdim = lhs.shape
  if lhs_row_idx is not None:
    _need(lhs_row_idx, "lhs_row_idx", torch.int32, 1)
    m = lhs_row_idx.numel()
  else:
    m = lhs_rows if num_rows is None else int(num_rows)
    if m > lhs_rows:
      raise ValueError("num_rows exceeds the rows of lhs")
  if rhs_kn:
    g_local, kr, n = rhs.shape
  else:
    g_local, n, kr = rhs.shape
  if lhs.dtype not in _LHS_DTYPE_CODE:
    raise TypeError(f"lhs dtype {lhs.dtype} not supported")
  if rhs_dtype is None:
    if rhs.dtype not in _DTYPE_CODE:
      raise TypeError(f"rhs dtype {rhs.dtype} needs an explicit rhs_dtype")
    rhs_dtype = _DTYPE_CODE[rhs.dtype]
  if rhs_dtype in (MOE_INT4, MOE_MXFP4):
    if rhs.dtype != torch.uint8 or kr * 2 != kdim:
      raise ValueError("INT4 / MXFP4 rhs must be uint8 [G, N, K/2]")
  elif kr != kdim:
    raise ValueError(f"rhs K {kr} != lhs K {kdim}")
  for name, t in (("rhs_up", rhs_up),):
    if t is not None:
      _need(t, name, rhs.dtype, 3)
      if t.shape != rhs.shape:
        raise ValueError("rhs_up must match rhs")
  nkb_r = 1 if rhs_scale_block_k == 0 else (kdim + rhs_scale_block_k - 1) // rhs_scale_block_k
  nnb = 1 if rhs_scale_block_n == _lib.MOE_SCALE_PER_TENSOR else (n + rhs_scale_block_n - 1) // rhs_scale_block_n
  for name, t in (("rhs_scale", rhs_scale), ("rhs_up_scale", rhs_up_scale)):
    if t is not None:
      _need(t, name)
      want = torch.bfloat16 if rhs_dtype == MOE_INT4 and not rhs_scale_kmajor else (torch.uint8 if rhs_dtype == MOE_MXFP4 else torch.float32)
      count = (1 if rhs_scale_shared else g_local) * nnb * nkb_r
      if t.dtype != want or t.numel() != count:
        raise ValueError(f"{name} must be {want} with {count} elements, got {t.dtype} {tuple(t.shape)}")
  for name, t in (("rhs_bias", rhs_bias), ("rhs_up_bias", rhs_up_bias)):
    if t is not None:
      _need(t, name, torch.float32, 2)
      if t.shape != (g_local, n):
        raise ValueError(f"{name} must be [{g_local}, {n}] f32")
  if rhs_up_bias is not None and rhs_up is None:
    raise ValueError("rhs_up_bias needs rhs_up")
  for name, t in (("partial_sum", partial_sum), ("partial_sum_up", partial_sum_up)):
    if t is not None:
      _need(t, name, torch.bfloat16, 2)
      if t.shape != (m, n):
        raise ValueError(f"{name} must be [{m}, {n}] bf16")
  if partial_sum_up is not None and rhs_up is None:
    raise ValueError("partial_sum_up needs rhs_up")
  if lhs_scale is not None:
    _need(lhs_scale, "lhs_scale", torch.float32)
    if lhs_scale_block_k == _lib.MOE_SCALE_PER_TENSOR:
      count = 1
    else:
      count = lhs_rows * (1 if lhs_scale_block_k == 0 else (kdim + lhs_scale_block_k - 1) // lhs_scale_block_k)
    if lhs_scale.numel() != count:
      raise ValueError(f"lhs_scale must have {count} elements, got {lhs_scale.numel()}")
  if out_row_scale is not None:
    _need(out_row_scale, "out_row_scale", torch.float32, 1)
    if out_row_scale.numel() != m:
      raise ValueError("out_row_scale must have one value per row of the product")
  if out_dtype not in (torch.bfloat16, torch.float32):
    raise TypeError("out_dtype must be bfloat16 or float32")
  if out is None:
    out = torch.empty((m, n), dtype=out_dtype, device=lhs.device)
  else:
    _need(out, "out", out_dtype, 2)
    if out.shape != (m, n):
      raise ValueError("out must be [M, N]")
  if kernel not in _lib.GMM_KERNEL_BY_NAME:
    raise ValueError(f"unknown kernel family {kernel!r}")
  lib = _lib.load()
  g_total = group_sizes.numel()
  wsb = lib.moe_gmm_workspace_bytes(m, g_total)
  ws = workspace if workspace is not None else torch.empty((max(wsb, 16),), dtype=torch.uint8, device=lhs.device)
  a = _lib.GmmArgs()
  a.struct_size = ctypes.sizeof(_lib.GmmArgs)
  a.lhs, a.lhs_scale = lhs.data_ptr(), (lhs_scale.data_ptr() if lhs_scale is not None else None)
  a.rhs, a.rhs_scale = rhs.data_ptr(), (rhs_scale.data_ptr() if rhs_scale is not None else None)
  a.rhs_up = rhs_up.data_ptr() if rhs_up is not None else None
  a.rhs_up_scale = rhs_up_scale.data_ptr() if rhs_up_scale is not None else None
  a.group_sizes, a.out = group_sizes.data_ptr(), out.data_ptr()
  a.workspace, a.workspace_bytes = ws.data_ptr(), ws.numel() * ws.element_size()
  a.M, a.K, a.N = m, kdim, n
  a.num_groups_total, a.num_groups_local, a.group_offset = g_total, g_local, int(group_offset)
  a.lhs_dtype, a.rhs_dtype = _LHS_DTYPE_CODE[lhs.dtype], rhs_dtype
  a.lhs_scale_block_k, a.rhs_scale_block_n, a.rhs_scale_block_k = int(lhs_scale_block_k), int(rhs_scale_block_n), int(rhs_scale_block_k)
  a.act = _lib.ACT_BY_NAME[act]
  a.act_limit = float(act_limit)
  a.out_dtype = _lib.MOE_BF16 if out_dtype == torch.bfloat16 else _lib.MOE_F32
  a.lhs_row_idx = lhs_row_idx.data_ptr() if lhs_row_idx is not None else None
  a.lhs_row_idx_div, a.lhs_rows = int(lhs_row_idx_div), lhs_rows
  a.out_row_scale = out_row_scale.data_ptr() if out_row_scale is not None else None
  if group_offset_dev is not None:
    _need(group_offset_dev, "group_offset_dev", torch.int32)
    if group_offset_dev.numel() != 1:
      raise ValueError("group_offset_dev must hold one value")
    a.group_offset_dev = group_offset_dev.data_ptr()
  a.rhs_bias = rhs_bias.data_ptr() if rhs_bias is not None else None
  a.rhs_up_bias = rhs_up_bias.data_ptr() if rhs_up_bias is not None else None
  a.partial_sum = partial_sum.data_ptr() if partial_sum is not None else None
  a.partial_sum_up = partial_sum_up.data_ptr() if partial_sum_up is not None else None
  a.flags = ((_lib.MOE_GMM_KEEP_OTHER_ROWS if keep_other_rows else 0) | (_lib.MOE_GMM_RHS_KN if rhs_kn else 0)
             | (_lib.MOE_GMM_RHS_SCALE_KMAJOR if rhs_scale_kmajor else 0) | (_lib.MOE_GMM_RHS_SCALE_SHARED if rhs_scale_shared else 0)
             | (_lib.MOE_GMM_SAME_GROUPS if same_groups and workspace is not None else 0))
  code = _lib.GMM_KERNEL_BY_NAME[kernel]
  if code or raster:
    st = lib.moe_gmm_tuned(ctypes.byref(a), code, int(raster), _lib.current_stream())
  else:
    st = lib.moe_gmm(ctypes.byref(a), _lib.current_stream())
  _lib.check(st, "moe_gmm")
  return out


def gmm_workspace(m, num_groups_total, device):
  """A tile-list buffer for moe_gmm calls on m rows and num_groups_total groups (uint8)."""
  return torch.empty((max(_lib.load().moe_gmm_workspace_bytes(int(m), int(num_groups_total)), 16),), dtype=torch.uint8, device=device)


def gmm_lhs_e5m2_supported(m, k, n, num_groups_total):
  """True when `gmm_raw` takes float8_e5m2 activations (against e4m3 weights) for this shape."""
  return bool(_lib.load().moe_gmm_lhs_e5m2_supported(int(m), int(k), int(n), int(num_groups_total)))


def gmm_fp8_rhs_kn_supported(m, k, n, num_groups_total):
  """True when `gmm_raw(..., rhs_kn=True)` takes [G, K, N] float8_e4m3fn weights of this shape as they are (fp8 activations)."""
  return bool(_lib.load().moe_gmm_fp8_rhs_kn_supported(int(m), int(k), int(n), int(num_groups_total)))


def gmm_rhs_kn_supported(m, k, n, num_groups_total):
  """True when `gmm_raw(..., rhs_kn=True)` takes [G, K, N] bf16 weights of this shape as they are."""
  return bool(_lib.load().moe_gmm_rhs_kn_supported(int(m), int(k), int(n), int(num_groups_total)))


def tgmm(lhs, dout, group_sizes, *, num_groups_local=None, group_offset=0, out_dtype=torch.bfloat16, existing_out=None,
         out_row_scale=None):
  """Weight gradient: out[g, n, k] = sum over rows m of group g of dout[m, n] * lhs[m, k]  ->  [G_local, N, K].

  out_row_scale: [N] f32; the f32 products of output row n are multiplied by out_row_scale[n] first.
  existing_out: [G_local, N, K] bf16 or f32, added to the f32 products before the rounding to out_dtype."""
  _need(lhs, "lhs", torch.bfloat16, 2)
  _need(dout, "dout", torch.bfloat16, 2)
  _need(group_sizes, "group_sizes", torch.int32, 1)
  m, k = lhs.shape
  if dout.shape[0] != m:
    raise ValueError("lhs and dout must have the same number of rows")
  n = dout.shape[1]
  g_total = group_sizes.numel()
  g_local = g_total - int(group_offset) if num_groups_local is None else int(num_groups_local)
  if out_dtype not in (torch.bfloat16, torch.float32):
    raise TypeError("out_dtype must be bfloat16 or float32")
  out = torch.empty((g_local, n, k), dtype=out_dtype, device=lhs.device)
  code = {torch.bfloat16: _lib.MOE_BF16, torch.float32: _lib.MOE_F32}
  if existing_out is not None:
    if existing_out.dtype not in code:
      raise TypeError("existing_out must be bfloat16 or float32")
    _need(existing_out, "existing_out", existing_out.dtype, 3)
    if tuple(existing_out.shape) != (g_local, n, k):
      raise ValueError(f"existing_out must be [{g_local}, {n}, {k}], got {tuple(existing_out.shape)}")
  if out_row_scale is not None:
    _need(out_row_scale, "out_row_scale", torch.float32, 1)
    if out_row_scale.numel() != n:
      raise ValueError(f"out_row_scale must have {n} entries, got {out_row_scale.numel()}")
  lib = _lib.load()
  st = lib.moe_tgmm_scaled(_lib.ptr(lhs), _lib.ptr(dout), _lib.ptr(group_sizes), m, k, n, g_total, g_local, int(group_offset),
                           None if out_row_scale is None else _lib.ptr(out_row_scale),
                           None if existing_out is None else _lib.ptr(existing_out),
                           0 if existing_out is None else code[existing_out.dtype], code[out_dtype], _lib.ptr(out),
                           _lib.current_stream())
  _lib.check(st, "moe_tgmm_scaled")
  return out


def tgmm_fp8_supported(m, k, n, num_groups_total, num_groups_local=None):
  """Whether tgmm_fp8 takes this shape (256 x 256 output tiles, 128 rows per group on average)."""
  g_local = num_groups_total if num_groups_local is None else num_groups_local
  return bool(_lib.load().moe_tgmm_fp8_supported(int(m), int(k), int(n), int(num_groups_total), int(g_local)))


def tgmm_fp8(lhs, dout, group_sizes, *, num_groups_local=None, group_offset=0, out_dtype=torch.bfloat16, existing_out=None,
             out_row_scale=None):
  """tgmm on 1-byte operands as stored: lhs [M, K] float8_e4m3fn, dout [M, N] float8_e5m2 or float8_e4m3fn (the drhs
  product of the fp8_full backward, kernels/megablox/ops.py:590-604) -> [G_local, N, K]."""
  _need(lhs, "lhs", torch.float8_e4m3fn, 2)
  _need(dout, "dout", None, 2)
  if dout.dtype not in (torch.float8_e5m2, torch.float8_e4m3fn):
    raise TypeError("dout must be float8_e5m2 or float8_e4m3fn")
  _need(group_sizes, "group_sizes", torch.int32, 1)
  m, k = lhs.shape
  if dout.shape[0] != m:
    raise ValueError("lhs and dout must have the same number of rows")
  n = dout.shape[1]
  g_total = group_sizes.numel()
  g_local = g_total - int(group_offset) if num_groups_local is None else int(num_groups_local)
  code = {torch.bfloat16: _lib.MOE_BF16, torch.float32: _lib.MOE_F32}
  if out_dtype not in code:
    raise TypeError("out_dtype must be bfloat16 or float32")
  out = torch.empty((g_local, n, k), dtype=out_dtype, device=lhs.device)
  if existing_out is not None:
    if existing_out.dtype not in code:
      raise TypeError("existing_out must be bfloat16 or float32")
    _need(existing_out, "existing_out", existing_out.dtype, 3)
    if tuple(existing_out.shape) != (g_local, n, k):
      raise ValueError(f"existing_out must be [{g_local}, {n}, {k}], got {tuple(existing_out.shape)}")
  if out_row_scale is not None:
    _need(out_row_scale, "out_row_scale", torch.float32, 1)
    if out_row_scale.numel() != n:
      raise ValueError(f"out_row_scale must have {n} entries, got {out_row_scale.numel()}")
  st = _lib.load().moe_tgmm_fp8(_lib.ptr(lhs), _lib.ptr(dout), _lib.MOE_FP8_E5M2 if dout.dtype == torch.float8_e5m2 else _lib.MOE_FP8_E4M3,
                                _lib.ptr(group_sizes), m, k, n, g_total, g_local, int(group_offset),
                                None if out_row_scale is None else _lib.ptr(out_row_scale),
                                None if existing_out is None else _lib.ptr(existing_out),
                                0 if existing_out is None else code[existing_out.dtype], code[out_dtype], _lib.ptr(out),
                                _lib.current_stream())
  _lib.check(st, "moe_tgmm_fp8")
  return out
