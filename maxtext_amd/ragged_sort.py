"""Host-side mirror of src/maxtext/kernels/ragged/ragged_sort.py (forward passes): the sorts of the expert-parallel
strategies that move only the rows a shard owns.  Each is one index kernel plus one row-moving kernel of the library;
no size is read back by the host.  `shard_idx` replaces jax.lax.axis_index(ep_name): a plain integer here."""

from __future__ import annotations

import torch

from maxtext_amd import kernels


def _row_range(valid_end, device):
  if isinstance(valid_end, torch.Tensor):
    end = valid_end.to(device=device, dtype=torch.int32).reshape(())
  else:
    end = torch.tensor(int(valid_end), dtype=torch.int32, device=device)
  return torch.stack([torch.zeros((), dtype=torch.int32, device=device), end])


def ring_ragged_sort(hidden_states_local, topk_indices_local, num_experts, topk, shard_idx, ep_size, buffer_size=None):
  """ragged_sort.py:23-226 -> (x [min(buffer_size, T*k), hidden], group_sizes [E], topk_argsort_revert_indices [T*k]).
  Rows [start, end) of x (the shard's experts in the sorted order; [0, min(end - start, buffer_size)) when the buffer is
  smaller than T*k) hold hidden_states_local[token of sorted position i]; all other rows are zeros."""
  t, k = topk_indices_local.shape
  if k != topk:
    raise ValueError(f"topk_indices_local has {k} columns for topk={topk}")
  perm, inv, group_sizes, _ = kernels.sort_by_expert(topk_indices_local.contiguous(), num_experts, want_sorted_experts=False)
  local = num_experts // ep_size
  row_idx, row_range = kernels.ring_ragged_indices(perm, group_sizes, shard_idx * local, local, buffer_size=buffer_size)
  x = kernels.gather_rows(hidden_states_local.contiguous(), row_idx, topk, row_range=row_range)
  return x, group_sizes, inv


def ring_ragged_unsort(sorted_tokens_local, group_sizes_local, topk_argsort_revert_indices, topk, local_num_experts, shard_idx, topk_weights):
  """ragged_sort.py:229-451 -> out [T, hidden]: out[t] = sum over the k slots of token t whose sorted position lies in the
  shard's range of w[t, s] * sorted_tokens_local[position] (f32 sum, one rounding); tokens with no such slot get zeros."""
  n = topk_argsort_revert_indices.shape[0]
  idx, mask = kernels.ring_ragged_indices(topk_argsort_revert_indices.contiguous(), group_sizes_local.contiguous(), shard_idx * local_num_experts,
                                          local_num_experts, buffer_size=sorted_tokens_local.shape[0], unsort=True)
  w = topk_weights.reshape(-1).float().contiguous()
  return kernels.unpermute_combine(sorted_tokens_local.contiguous(), w, k=topk, inv_perm=idx, valid_rows_mask=mask, num_tokens=n // topk)


def a2a_ragged_sort(inputs, sort_indices, valid_end):
  """ragged_sort.py:454-533: out[i] = inputs[sort_indices[i]] for i < valid_end, zeros behind."""
  return kernels.gather_rows(inputs.contiguous(), sort_indices.contiguous(), 1, row_range=_row_range(valid_end, inputs.device))


def a2a_ragged_unsort(sorted_tokens, revert_indices, valid_end):
  """ragged_sort.py:541-626: out[i] = sorted_tokens[revert_indices[i]] for i < valid_end, zeros behind."""
  return kernels.gather_rows(sorted_tokens.contiguous(), revert_indices.contiguous(), 1, row_range=_row_range(valid_end, sorted_tokens.device))
