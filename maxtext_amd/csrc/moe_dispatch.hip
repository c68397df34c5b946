// Bookkeeping of the expert-parallel dispatch on one expert shard: the keys RoutedMoE.local_permute sorts by, the rows per
// local expert (cut to the receive buffer when it has a fixed capacity) and the four parameter vectors of the ragged
// all-to-all.  All integer work on device-resident sizes, so that nothing waits for the host; the sort itself is
// moe_sort_by_expert on the keys and the row movement moe_gather_rows on the sorted indices.

#include "moe_common.h"

namespace moe {
void note_group_sizes_rewritten(const int32_t* group_sizes);  // moe_gmm.hip: drops a tile list recorded over this buffer
}

#include <climits>

namespace moe {

constexpr int kDispThreads = 1024;
constexpr int kDispMaxParallelism = 1024;

// Inclusive prefix sum of a block's values (one per thread); returns the thread's inclusive sum, *total = the block's sum.
__device__ __forceinline__ long long block_inclusive_scan(long long v, long long* s_buf, long long* total) {
  const int tid = threadIdx.x;
  s_buf[tid] = v;
  __syncthreads();
  for (int o = 1; o < kDispThreads; o <<= 1) {
    const long long add = tid >= o ? s_buf[tid - o] : 0;
    __syncthreads();
    s_buf[tid] += add;
    __syncthreads();
  }
  const long long incl = s_buf[tid];
  *total = s_buf[kDispThreads - 1];
  __syncthreads();
  return incl;
}

// A shard's index as the caller holds it: by value, or in device memory (inside shard_map it is jax.lax.axis_index, which
// only exists on the device); a device value is clamped into [0, hi] so that no table is indexed outside its rows.
__device__ __forceinline__ int resolve_shard(int by_value, const int32_t* dev, int hi) {
  return dev ? min(max(*dev, 0), hi) : by_value;
}

// starts[i], i < S * L: rows that precede segment i = (batch shard i / L, local expert i % L) in the received buffer;
// starts[S * L] = rows received.  local_group_size[l] = sum over the batch shards of segment (s, l), each segment cut
// to what is left of `capacity` rows when the prefix sum reaches it (capacity < 0: no cut).
__global__ __launch_bounds__(kDispThreads) void local_sizes_kernel(const int32_t* __restrict__ global_group_sizes, int S, int E, int L,
                                                                   int shard_index, const int32_t* __restrict__ shard_dev, long long capacity,
                                                                   int32_t* __restrict__ starts, int32_t* __restrict__ local_group_size) {
  __shared__ long long s_buf[kDispThreads];
  shard_index = resolve_shard(shard_index, shard_dev, E / L - 1);
  const int tid = threadIdx.x;
  const int n = S * L;
  long long carry = 0;
  for (int base = 0; base < n; base += kDispThreads) {
    const int i = base + tid;
    long long v = 0;
    if (i < n) v = max(global_group_sizes[(size_t)(i / L) * E + shard_index * L + i % L], 0);
    long long total;
    const long long incl = block_inclusive_scan(v, s_buf, &total) + carry;
    if (i < n) starts[i] = (int32_t)min(incl - v, (long long)INT_MAX);
    carry += total;
  }
  if (tid == 0) starts[n] = (int32_t)min(carry, (long long)INT_MAX);
  __syncthreads();
  __threadfence_block();
  // rows per local expert; starts[] of this block's own writes are visible after the barrier
  for (int l = tid; l < L; l += kDispThreads) {
    long long sum = 0;
    for (int s = 0; s < S; s++) {
      const int i = s * L + l;
      long long lo = starts[i], hi = starts[i + 1];
      if (capacity >= 0) {
        lo = min(lo, capacity);
        hi = min(hi, capacity);
      }
      sum += hi - lo;
    }
    local_group_size[l] = (int32_t)sum;
  }
}

// Key of received row r: the local expert of the segment that holds it, i.e. of the largest i with starts[i] <= r
// (segments without rows share their start with the next one and are skipped; rows past the received total take the
// last segment's expert, which is how jax.numpy.repeat(total_repeat_length=...) pads).
__global__ void local_keys_kernel(const int32_t* __restrict__ starts, int n, int L, int R, int32_t* __restrict__ keys) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  int lo = 0, hi = n - 1;  // invariant: starts[lo] <= r (starts[0] == 0)
  while (lo < hi) {
    const int mid = (lo + hi + 1) >> 1;
    if (starts[mid] <= r) lo = mid;
    else hi = mid - 1;
  }
  keys[r] = lo % L;
}

// Rows sorted by global expert (every routed row of the replicated batch): this shard's rows keep their local expert,
// all others get the key L, which sorts them behind (moe.py:1166-1172).
__global__ void offset_keys_kernel(const int32_t* __restrict__ global_sorted_experts, int L, int shard_index, const int32_t* __restrict__ shard_dev,
                                   int max_shard, int R, int32_t* __restrict__ keys) {
  const int r = blockIdx.x * blockDim.x + threadIdx.x;
  if (r >= R) return;
  shard_index = resolve_shard(shard_index, shard_dev, max_shard);
  const int e = global_sorted_experts[r];
  // floor division and modulus as jnp.floor_divide / jnp.mod define them (a negative id belongs to no shard)
  const int q = e >= 0 ? e / L : -((-e + L - 1) / L);
  keys[r] = q == shard_index ? e - q * L : L;
}

// The four vectors of ragged_all_to_all for one shard (moe.py:1202-1349).  a = all_shards_group_sizes, [P, P] with
// a[i][j] = rows batch shard i sends to expert shard j, or [P] when the batch is replicated.  With a capacity the
// matrix is cut per receiver in sender order (_truncate_matrix, moe.py:103-120); the sum of the cut entries of a
// column up to sender n is min(column prefix, capacity), which is all the sums below need.
__global__ __launch_bounds__(kDispThreads) void all_to_all_params_kernel(const int32_t* __restrict__ a, int P, int shard, const int32_t* __restrict__ shard_dev,
                                                                         int batch_sharded, long long capacity, int dispatch, int32_t* __restrict__ input_offsets,
                                                                         int32_t* __restrict__ send_sizes, int32_t* __restrict__ output_offsets,
                                                                         int32_t* __restrict__ recv_sizes) {
  const int j = threadIdx.x;
  if (j >= P) return;
  shard = resolve_shard(shard, shard_dev, P - 1);
  if (!batch_sharded) {
    long long before = 0;
    for (int i = 0; i < shard; i++) before += a[i];
    input_offsets[j] = 0;
    send_sizes[j] = a[shard];
    output_offsets[j] = (int32_t)before;
    recv_sizes[j] = a[j];
    return;
  }
  auto cut = [&](long long v) { return capacity >= 0 ? min(v, capacity) : v; };
  // prefix of column c over senders 0 .. n (n = -1: nothing)
  auto col_prefix = [&](int n, int c) {
    long long v = 0;
    for (int i = 0; i <= n; i++) v += a[(size_t)i * P + c];
    return v;
  };
  auto cut_entry = [&](int i, int c) {
    const long long hi = col_prefix(i, c);
    return cut(hi) - cut(hi - a[(size_t)i * P + c]);
  };
  if (dispatch) {
    long long off = 0;  // the sender's buffer still holds every row: offsets from the uncut sizes
    for (int c = 0; c < j; c++) off += a[(size_t)shard * P + c];
    input_offsets[j] = (int32_t)off;
    send_sizes[j] = (int32_t)cut_entry(shard, j);
    output_offsets[j] = (int32_t)cut(col_prefix(shard - 1, j));
    recv_sizes[j] = (int32_t)cut_entry(j, shard);
  } else {
    // the way back: the packed (cut) buffer is sent, each piece to the position its rows came from
    input_offsets[j] = (int32_t)cut(col_prefix(j - 1, shard));
    send_sizes[j] = (int32_t)cut_entry(j, shard);
    long long off = 0;
    for (int c = 0; c < shard; c++) off += a[(size_t)j * P + c];
    output_offsets[j] = (int32_t)off;
    recv_sizes[j] = (int32_t)cut_entry(shard, j);
  }
}

// Index arrays of the ring-of-experts ragged sort (kernels/ragged/ragged_sort.py:23-226, :229-365).  The rows of this
// shard's experts are positions [start, end) of the globally sorted order (start / end = sums of group_sizes before /
// through the shard's experts); with a buffer smaller than the n sorted rows they are packed at its front.
//   SORT:   idx_in = the sort permutation.  Unbuffered: idx_out = idx_in, range = [start, end).  Buffered: idx_out[i] =
//           idx_in[start + i] (0 past the end), range = [0, min(end - start, buffer)).
//   UNSORT: idx_in = the inverse permutation.  Unbuffered: idx_out = idx_in, mask[i] = start <= idx_in[i] < end.
//           Buffered: idx_out[i] = idx_in[i] - start where 0 <= that < min(end - start, buffer), else 0 with mask 0.
__global__ __launch_bounds__(256) void ring_ragged_indices_kernel(const int32_t* __restrict__ idx_in, const int32_t* __restrict__ group_sizes,
                                                                  int E, int experts_start, const int32_t* __restrict__ shard_dev, int local_experts,
                                                                  int n, int buffer, int unsort, int32_t* __restrict__ idx_out,
                                                                  uint8_t* __restrict__ mask_out, int32_t* __restrict__ range_out) {
  __shared__ long long s_before[256], s_local[256];
  if (shard_dev) experts_start = resolve_shard(0, shard_dev, E / local_experts - 1) * local_experts;
  long long before = 0, local = 0;
  for (int e = threadIdx.x; e < experts_start + local_experts && e < E; e += 256) {
    const long long g = max(group_sizes[e], 0);
    if (e < experts_start) before += g;
    else local += g;
  }
  s_before[threadIdx.x] = before;
  s_local[threadIdx.x] = local;
  __syncthreads();
  for (int o = 128; o > 0; o >>= 1) {
    if ((int)threadIdx.x < o) {
      s_before[threadIdx.x] += s_before[threadIdx.x + o];
      s_local[threadIdx.x] += s_local[threadIdx.x + o];
    }
    __syncthreads();
  }
  const long long start = min(s_before[0], (long long)n), end = min(s_before[0] + s_local[0], (long long)n);
  const bool buffered = buffer < n;
  const long long limit = min(end - start, (long long)buffer);
  if (blockIdx.x == 0 && threadIdx.x == 0 && range_out) {
    range_out[0] = buffered ? 0 : (int32_t)start;
    range_out[1] = buffered ? (int32_t)limit : (int32_t)end;
  }
  const int out_n = unsort ? n : (buffered ? buffer : n);
  const int i = blockIdx.x * 256 + threadIdx.x;
  if (i >= out_n) return;
  if (!unsort) {
    idx_out[i] = buffered ? (start + i < n ? idx_in[start + i] : 0) : idx_in[i];
  } else {
    const long long v = idx_in[i];
    if (!buffered) {
      idx_out[i] = (int32_t)v;
      mask_out[i] = v >= start && v < end;
    } else {
      const long long sh = v - start;
      const bool ok = sh >= 0 && sh < limit;
      idx_out[i] = ok ? (int32_t)sh : 0;
      mask_out[i] = ok;
    }
  }
}

}  // namespace moe

using namespace moe;

extern "C" {

size_t moe_local_expert_keys_workspace_bytes(int num_batch_shards, int local_expert_size) {
  if (num_batch_shards <= 0 || local_expert_size <= 0) return 0;
  return ((size_t)num_batch_shards * local_expert_size + 1) * sizeof(int32_t);
}

static int local_expert_keys_impl(const int32_t* global_group_sizes, int num_batch_shards, int num_experts, int local_expert_size,
                                  int shard_index, const int32_t* shard_dev, int num_rows, const int32_t* global_sorted_experts, int truncate,
                                  int32_t* expert_keys, int32_t* local_group_size, void* workspace, size_t workspace_bytes, void* stream) {
  if (!global_group_sizes || !expert_keys || !local_group_size || !workspace) return fail(MOE_ERR_INVALID_ARG, "local_expert_keys: NULL pointer");
  if (num_batch_shards <= 0 || num_experts <= 0 || local_expert_size <= 0 || shard_index < 0 || num_rows < 0)
    return fail(MOE_ERR_INVALID_ARG, "local_expert_keys: bad sizes");
  if ((long long)(shard_index + 1) * local_expert_size > num_experts)
    return fail(MOE_ERR_INVALID_ARG, "local_expert_keys: shard %d of %d experts each lies outside %d experts", shard_index, local_expert_size, num_experts);
  if ((long long)num_batch_shards * local_expert_size > (1 << 24)) return fail(MOE_ERR_UNSUPPORTED, "local_expert_keys: more than 2^24 segments");
  if (workspace_bytes < moe_local_expert_keys_workspace_bytes(num_batch_shards, local_expert_size))
    return fail(MOE_ERR_WORKSPACE, "local_expert_keys: workspace too small");
  hipStream_t s = (hipStream_t)stream;
  int32_t* starts = (int32_t*)workspace;
  const int n = num_batch_shards * local_expert_size;
  local_sizes_kernel<<<1, kDispThreads, 0, s>>>(global_group_sizes, num_batch_shards, num_experts, local_expert_size, shard_index, shard_dev,
                                                truncate ? (long long)num_rows : -1LL, starts, local_group_size);
  if (num_rows > 0) {
    const int blocks = cdiv(num_rows, 256);
    if (global_sorted_experts) offset_keys_kernel<<<blocks, 256, 0, s>>>(global_sorted_experts, local_expert_size, shard_index, shard_dev, num_experts / local_expert_size - 1, num_rows, expert_keys);
    else local_keys_kernel<<<blocks, 256, 0, s>>>(starts, n, local_expert_size, num_rows, expert_keys);
  }
  note_group_sizes_rewritten(local_group_size);
  return check_launch("local_expert_keys");
}

int moe_local_expert_keys(const int32_t* global_group_sizes, int num_batch_shards, int num_experts, int local_expert_size,
                          int shard_index, int num_rows, const int32_t* global_sorted_experts, int truncate,
                          int32_t* expert_keys, int32_t* local_group_size, void* workspace, size_t workspace_bytes, void* stream) {
  return local_expert_keys_impl(global_group_sizes, num_batch_shards, num_experts, local_expert_size, shard_index, nullptr, num_rows,
                                global_sorted_experts, truncate, expert_keys, local_group_size, workspace, workspace_bytes, stream);
}

int moe_local_expert_keys_dev(const int32_t* global_group_sizes, int num_batch_shards, int num_experts, int local_expert_size,
                              const int32_t* shard_index_dev, int num_rows, const int32_t* global_sorted_experts, int truncate,
                              int32_t* expert_keys, int32_t* local_group_size, void* workspace, size_t workspace_bytes, void* stream) {
  if (!shard_index_dev) return fail(MOE_ERR_INVALID_ARG, "local_expert_keys_dev: NULL shard index");
  return local_expert_keys_impl(global_group_sizes, num_batch_shards, num_experts, local_expert_size, 0, shard_index_dev, num_rows,
                                global_sorted_experts, truncate, expert_keys, local_group_size, workspace, workspace_bytes, stream);
}

static int all_to_all_params_impl(const int32_t* all_shards_group_sizes, int num_expert_parallelism, int shard_id, const int32_t* shard_dev,
                                  int is_batch_sharded, long long buffer_size, int is_dispatch, int32_t* input_offsets, int32_t* send_sizes,
                                  int32_t* output_offsets, int32_t* recv_sizes, void* stream) {
  if (!all_shards_group_sizes || !input_offsets || !send_sizes || !output_offsets || !recv_sizes)
    return fail(MOE_ERR_INVALID_ARG, "all_to_all_params: NULL pointer");
  if (num_expert_parallelism <= 0 || shard_id < 0 || shard_id >= num_expert_parallelism)
    return fail(MOE_ERR_INVALID_ARG, "all_to_all_params: shard %d of %d", shard_id, num_expert_parallelism);
  if (num_expert_parallelism > kDispMaxParallelism) return fail(MOE_ERR_UNSUPPORTED, "all_to_all_params: more than %d shards", kDispMaxParallelism);
  if (!is_batch_sharded && buffer_size >= 0)
    return fail(MOE_ERR_UNSUPPORTED, "all_to_all_params: a receive capacity needs the batch-sharded traffic matrix");
  all_to_all_params_kernel<<<1, kDispThreads, 0, (hipStream_t)stream>>>(all_shards_group_sizes, num_expert_parallelism, shard_id, shard_dev, is_batch_sharded,
                                                                        buffer_size, is_dispatch, input_offsets, send_sizes, output_offsets, recv_sizes);
  return check_launch("all_to_all_params");
}

int moe_all_to_all_params(const int32_t* all_shards_group_sizes, int num_expert_parallelism, int shard_id, int is_batch_sharded,
                          long long buffer_size, int is_dispatch, int32_t* input_offsets, int32_t* send_sizes,
                          int32_t* output_offsets, int32_t* recv_sizes, void* stream) {
  return all_to_all_params_impl(all_shards_group_sizes, num_expert_parallelism, shard_id, nullptr, is_batch_sharded, buffer_size, is_dispatch,
                                input_offsets, send_sizes, output_offsets, recv_sizes, stream);
}

int moe_all_to_all_params_dev(const int32_t* all_shards_group_sizes, int num_expert_parallelism, const int32_t* shard_id_dev, int is_batch_sharded,
                              long long buffer_size, int is_dispatch, int32_t* input_offsets, int32_t* send_sizes,
                              int32_t* output_offsets, int32_t* recv_sizes, void* stream) {
  if (!shard_id_dev) return fail(MOE_ERR_INVALID_ARG, "all_to_all_params_dev: NULL shard id");
  return all_to_all_params_impl(all_shards_group_sizes, num_expert_parallelism, 0, shard_id_dev, is_batch_sharded, buffer_size, is_dispatch,
                                input_offsets, send_sizes, output_offsets, recv_sizes, stream);
}

static int ring_ragged_indices_impl(const int32_t* indices, const int32_t* group_sizes, int num_experts, int experts_start, const int32_t* shard_dev,
                                    int local_experts, int num_rows, int buffer_size, int unsort, int32_t* indices_out,
                                    uint8_t* valid_rows_mask, int32_t* row_range, void* stream) {
  if (!indices || !group_sizes || !indices_out) return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices: NULL pointer");
  if (unsort ? !valid_rows_mask : !row_range) return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices: NULL output");
  if (num_experts <= 0 || experts_start < 0 || local_experts <= 0 || experts_start + local_experts > num_experts || num_rows < 0)
    return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices: experts %d .. +%d of %d, %d rows", experts_start, local_experts, num_experts, num_rows);
  if (buffer_size < 0) return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices: buffer_size %d", buffer_size);
  const int out_n = unsort ? num_rows : (buffer_size < num_rows ? buffer_size : num_rows);
  const int blocks = out_n > 0 ? cdiv(out_n, 256) : 1;
  ring_ragged_indices_kernel<<<blocks, 256, 0, (hipStream_t)stream>>>(indices, group_sizes, num_experts, experts_start, shard_dev, local_experts, num_rows,
                                                                        buffer_size, unsort, indices_out, valid_rows_mask, row_range);
  return check_launch("ring_ragged_indices");
}

int moe_ring_ragged_indices(const int32_t* indices, const int32_t* group_sizes, int num_experts, int experts_start,
                            int local_experts, int num_rows, int buffer_size, int unsort, int32_t* indices_out,
                            uint8_t* valid_rows_mask, int32_t* row_range, void* stream) {
  return ring_ragged_indices_impl(indices, group_sizes, num_experts, experts_start, nullptr, local_experts, num_rows, buffer_size, unsort,
                                  indices_out, valid_rows_mask, row_range, stream);
}

int moe_ring_ragged_indices_dev(const int32_t* indices, const int32_t* group_sizes, int num_experts, const int32_t* shard_index_dev,
                                int local_experts, int num_rows, int buffer_size, int unsort, int32_t* indices_out,
                                uint8_t* valid_rows_mask, int32_t* row_range, void* stream) {
  if (!shard_index_dev) return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices_dev: NULL shard index");
  if (local_experts <= 0 || num_experts % local_experts != 0)
    return fail(MOE_ERR_INVALID_ARG, "ring_ragged_indices_dev: %d experts do not divide into shards of %d", num_experts, local_experts);
  return ring_ragged_indices_impl(indices, group_sizes, num_experts, 0, shard_index_dev, local_experts, num_rows, buffer_size, unsort,
                                  indices_out, valid_rows_mask, row_range, stream);
}

}  // extern "C"
