"""Host-side mirror of src/maxtext/kernels/ragged/ragged_sort.py: the sorts of the expert-parallel strategies that move
only the rows a shard owns, with the custom VJPs of the reference (:155-224, :364-441, :515-537, :596-616).  Each pass,
forward or backward, is one index kernel plus one row-moving kernel of the library; no size is read back by the host.
`shard_idx` replaces jax.lax.axis_index(ep_name): an integer, or a one-element tensor that only the kernels read."""

from __future__ import annotations

import torch

from maxtext_amd import kernels


def _row_range(valid_end, device):
  if isinstance(valid_end, torch.Tensor):
    end = valid_end.to(device=device, dtype=torch.int32).reshape(())
  else:
    end = torch.tensor(int(valid_end), dtype=torch.int32, device=device)
  return torch.stack([torch.zeros((), dtype=torch.int32, device=device), end])


def _ring_indices(indices, group_sizes, shard_idx, local_experts, **kw):
  if isinstance(shard_idx, torch.Tensor):
    return kernels.ring_ragged_indices(indices, group_sizes, 0, local_experts, shard_index=shard_idx, **kw)
  return kernels.ring_ragged_indices(indices, group_sizes, int(shard_idx) * local_experts, local_experts, **kw)


def _inverse_permutation(p):
  """argsort of a permutation, on the device."""
  inv = torch.empty_like(p)
  inv[p.long()] = torch.arange(p.numel(), dtype=p.dtype, device=p.device)
  return inv


class _RingSortFn(torch.autograd.Function):
  """ring_ragged_sort's row movement with the backward of ragged_sort.py:155-224: the gradient of a token is the sum of
  the gradients of those of its topk copies that lie in the shard's range (a gather-reduce over the revert indices,
  masked; indices shifted into the packed buffer when it is smaller than T * k)."""

  @staticmethod
  def forward(ctx, hidden, row_idx, row_range, inv, group_sizes, topk, shard_idx, local_experts, buffer_rows):
    ctx.save_for_backward(inv, group_sizes)
    ctx.meta = (topk, shard_idx, local_experts, buffer_rows, hidden.shape[0])
    return kernels.gather_rows(hidden.contiguous(), row_idx, topk, row_range=row_range)

  @staticmethod
  def backward(ctx, g_x):
    inv, group_sizes = ctx.saved_tensors
    topk, shard_idx, local_experts, buffer_rows, tokens = ctx.meta
    idx, mask = _ring_indices(inv, group_sizes, shard_idx, local_experts, buffer_size=buffer_rows, unsort=True)
    g = kernels.unpermute_combine(g_x.contiguous(), None, k=topk, inv_perm=idx, valid_rows_mask=mask, num_tokens=tokens)
    return g, None, None, None, None, None, None, None, None


def ring_ragged_sort(hidden_states_local, topk_indices_local, num_experts, topk, shard_idx, ep_size, buffer_size=None):
  """ragged_sort.py:23-226 -> (x [min(buffer_size, T*k), hidden], group_sizes [E], topk_argsort_revert_indices [T*k]).
  Rows [start, end) of x (the shard's experts in the sorted order; [0, min(end - start, buffer_size)) when the buffer is
  smaller than T*k) hold hidden_states_local[token of sorted position i]; all other rows are zeros."""
  t, k = topk_indices_local.shape
  if k != topk:
    raise ValueError(f"topk_indices_local has {k} columns for topk={topk}")
  perm, inv, group_sizes, _ = kernels.sort_by_expert(topk_indices_local.contiguous(), num_experts, want_sorted_experts=False)
  local = num_experts // ep_size
  row_idx, row_range = _ring_indices(perm, group_sizes, shard_idx, local, buffer_size=buffer_size)
  if torch.is_grad_enabled() and hidden_states_local.requires_grad:
    x = _RingSortFn.apply(hidden_states_local, row_idx, row_range, inv, group_sizes, topk, shard_idx, local, row_idx.shape[0])
  else:
    x = kernels.gather_rows(hidden_states_local.contiguous(), row_idx, topk, row_range=row_range)
  return x, group_sizes, inv


class _RingUnsortFn(torch.autograd.Function):
  """ring_ragged_unsort's weighted gather-reduce with the backward of ragged_sort.py:364-441: g_sorted[j] = w[i] *
  g_out[i // topk] for the flat slot i whose sorted position is j, j inside the shard's range (one weighted row gather
  through the inverse of the revert indices; rows outside the range are zeros).  The routing weights get no gradient
  here, as in the reference (:441)."""

  @staticmethod
  def forward(ctx, sorted_tokens, idx, mask, w, revert, group_sizes, topk, shard_idx, local_experts):
    ctx.save_for_backward(w, revert, group_sizes)
    ctx.meta = (topk, shard_idx, local_experts, sorted_tokens.shape[0])
    return kernels.unpermute_combine(sorted_tokens.contiguous(), w, k=topk, inv_perm=idx, valid_rows_mask=mask, num_tokens=revert.shape[0] // topk)

  @staticmethod
  def backward(ctx, g_out):
    w, revert, group_sizes = ctx.saved_tensors
    topk, shard_idx, local_experts, buffer_rows = ctx.meta
    perm = _inverse_permutation(revert)  # sorted position -> flat slot t * topk + s
    row_idx, row_range = _ring_indices(perm, group_sizes, shard_idx, local_experts, buffer_size=buffer_rows)
    w_rows = w[row_idx.long().clamp_(0, w.numel() - 1)].contiguous()  # the slot's weight, row by row of the (packed) buffer
    g = kernels.gather_rows(g_out.contiguous(), row_idx, topk, row_weight=w_rows, row_range=row_range)
    return g, None, None, None, None, None, None, None, None


def ring_ragged_unsort(sorted_tokens_local, group_sizes_local, topk_argsort_revert_indices, topk, local_num_experts, shard_idx, topk_weights):
  """ragged_sort.py:229-451 -> out [T, hidden]: out[t] = sum over the k slots of token t whose sorted position lies in the
  shard's range of w[t, s] * sorted_tokens_local[position] (f32 sum, one rounding); tokens with no such slot get zeros."""
  n = topk_argsort_revert_indices.shape[0]
  revert = topk_argsort_revert_indices.contiguous()
  gs = group_sizes_local.contiguous()
  idx, mask = _ring_indices(revert, gs, shard_idx, local_num_experts, buffer_size=sorted_tokens_local.shape[0], unsort=True)
  w = topk_weights.reshape(-1).float().contiguous()
  if torch.is_grad_enabled() and sorted_tokens_local.requires_grad:
    return _RingUnsortFn.apply(sorted_tokens_local, idx, mask, w.detach(), revert, gs, topk, shard_idx, local_num_experts)
  return kernels.unpermute_combine(sorted_tokens_local.contiguous(), w, k=topk, inv_perm=idx, valid_rows_mask=mask, num_tokens=n // topk)


class _A2aSortFn(torch.autograd.Function):
  """out[i] = inputs[indices[i]] for i < valid_end.  Backward of a2a_ragged_sort (ragged_sort.py:515-537): input row j
  receives the gradient of the one output row i with indices[i] == j when i < valid_end (a masked gather through the
  inverse permutation)."""

  @staticmethod
  def forward(ctx, inputs, indices, row_range):
    ctx.save_for_backward(indices, row_range)
    return kernels.gather_rows(inputs.contiguous(), indices, 1, row_range=row_range)

  @staticmethod
  def backward(ctx, g_out):
    indices, row_range = ctx.saved_tensors
    inv = _inverse_permutation(indices)
    mask = (inv < row_range[1]).to(torch.uint8)
    return kernels.unpermute_combine(g_out.contiguous(), None, k=1, inv_perm=inv, valid_rows_mask=mask), None, None


class _A2aUnsortFn(torch.autograd.Function):
  """out[i] = sorted_tokens[revert[i]] for i < valid_end.  Backward of a2a_ragged_unsort (ragged_sort.py:596-616):
  g_sorted[j] = g_out[argsort(revert)[j]] for the positions j < valid_end, zeros behind."""

  @staticmethod
  def forward(ctx, sorted_tokens, revert, row_range):
    ctx.save_for_backward(revert, row_range)
    return kernels.gather_rows(sorted_tokens.contiguous(), revert, 1, row_range=row_range)

  @staticmethod
  def backward(ctx, g_out):
    revert, row_range = ctx.saved_tensors
    return kernels.gather_rows(g_out.contiguous(), _inverse_permutation(revert), 1, row_range=row_range), None, None


def a2a_ragged_sort(inputs, sort_indices, valid_end):
  """ragged_sort.py:454-533: out[i] = inputs[sort_indices[i]] for i < valid_end, zeros behind."""
  rng = _row_range(valid_end, inputs.device)
  if torch.is_grad_enabled() and inputs.requires_grad:
    return _A2aSortFn.apply(inputs, sort_indices.contiguous(), rng)
  return kernels.gather_rows(inputs.contiguous(), sort_indices.contiguous(), 1, row_range=rng)


def a2a_ragged_unsort(sorted_tokens, revert_indices, valid_end):
  """ragged_sort.py:541-626: out[i] = sorted_tokens[revert_indices[i]] for i < valid_end, zeros behind."""
  rng = _row_range(valid_end, sorted_tokens.device)
  if torch.is_grad_enabled() and sorted_tokens.requires_grad:
    return _A2aUnsortFn.apply(sorted_tokens, revert_indices.contiguous(), rng)
  return kernels.gather_rows(sorted_tokens.contiguous(), revert_indices.contiguous(), 1, row_range=rng)
