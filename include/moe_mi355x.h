/*
 * moe_mi355x.h -- C ABI of libmoe_mi355x.so: the quantized MoE expert path
 * (routing -> permute -> grouped GEMM with fused SwiGLU -> unpermute+combine)
 * as hand-written gfx950 HIP kernels.
 *
 * Conventions
 *   - every pointer is a DEVICE pointer unless the parameter name ends in _host;
 *   - every call is asynchronous on `stream` (a hipStream_t passed as void*; NULL =
 *     the default stream), allocates nothing, never synchronises and never throws;
 *   - the return value is a moe_status (0 = ok, negative = the call enqueued nothing);
 *   - `group_sizes` stays on the device: no entry point reads it on the host;
 *   - inputs are never written; outputs are fully defined (rows that belong to no
 *     local group are written as zeros), so buffers need no pre-clearing;
 *   - calls on different streams with disjoint buffers may overlap; the state the library keeps is per device: values
 *     written once (the CU count, "this kernel may use more than 64 KB of LDS", the address of the static workspace),
 *     set up on the first call that needs them or ahead of time by moe_init() (two host threads that race there repeat
 *     an idempotent query and store the same value), and one host-side record, under a lock, of what the last moe_gmm
 *     call on the device mapped and where, which only calls flagged MOE_GMM_SAME_GROUPS consult.
 *
 * Paths in the citations are relative to the reference (AI-Hypercomputer/maxtext).
 */
#ifndef MOE_MI355X_H_
#define MOE_MI355X_H_

#include <stddef.h>
#include <stdint.h>

#ifdef __cplusplus
extern "C" {
#endif

/* Exported from the shared library (everything else is built with hidden visibility). */
#define MOE_API __attribute__((visibility("default")))

typedef enum {
  MOE_OK = 0,
  MOE_ERR_INVALID_ARG = -1, /* NULL pointer, non-positive size, bad enum            */
  MOE_ERR_UNSUPPORTED = -2, /* valid request the kernels do not cover (see below)   */
  MOE_ERR_WORKSPACE = -3,   /* workspace_bytes smaller than *_workspace_bytes()     */
  MOE_ERR_LAUNCH = -4       /* hipGetLastError() != hipSuccess after a launch       */
} moe_status;

typedef enum {
  MOE_BF16 = 0,
  MOE_INT8 = 1,
  MOE_FP8_E4M3 = 2, /* OCP float8_e4m3fn (max 448), layers/quantizations.py:237      */
  MOE_INT4 = 3,     /* 2 per byte along K, first value in the low nibble, stored +8  */
  MOE_F32 = 4,
  MOE_MXFP4 = 5,   /* OCP MX fp4: e2m1 values, 2 per byte along K (first in the low nibble), one e8m0 scale
                      byte 2^(s-127) per 32 values (dequantize_mxfp4.py:46-72) */
  MOE_FP8_E5M2 = 6 /* OCP float8_e5m2 (max 57344): the gradient type of the fp8_full recipe's backward
                      (bwd_qtype, layers/quantizations.py:234-250, kernels/megablox/ops.py:583-604); lhs of moe_gmm only */
} moe_dtype;

typedef enum {
  MOE_ROUTE_SOFTMAX_TOPK = 0, /* lax.top_k -> softmax over the k values, moe.py:747-753 */
  MOE_ROUTE_DEEPSEEK = 1,     /* deepseek_routing + deepseek_scale_weights, moe.py:767-839 */
  MOE_ROUTE_TOPK_RAW = 2,     /* Llama4: the top-k logits themselves are the weights, moe.py:747, :753 skipped */
  MOE_ROUTE_SOFTMAX_ALL = 3   /* Gemma4: softmax over all experts, read at the top-k indices, moe.py:742-745 */
} moe_route_mode;

typedef enum {
  MOE_ACT_NONE = 0,
  MOE_ACT_SILU = 1,      /* silu(gate) * up, moe.py:868-869; v2 kernel "silu" :64-65   */
  MOE_ACT_SWIGLUOAI = 2, /* GPT-OSS clipped variant, moe.py:844-853; v2 kernel :33-40   */
  MOE_ACT_SILU_CLIP = 3  /* DeepSeek-V4 clipped SwiGLU, moe.py:854-866                  */
} moe_act;

/* Text for the last non-zero status returned on the calling thread. */
MOE_API const char* moe_last_error(void);
/* ABI version; bumped when a struct below changes. */
MOE_API int moe_abi_version(void);

/* ---------------------------------------------------------------------------
 * Routing.  Replaces RoutedMoE.get_topk (src/maxtext/layers/moe.py:717-765),
 * deepseek_routing (:813-839), expert_group_mask (:775-811) and
 * deepseek_scale_weights (:767-773).
 *
 *   gate_logits      [T, E] f32   scores the selection runs on (post-bias for DeepSeek)
 *   pre_bias_logits  [T, E] f32   DeepSeek only: scores the weights are read from
 *   topk_weights     [T, k] f32   out; SOFTMAX_TOPK rounds them to bf16 when
 *                                 weights_round_bf16 != 0 (the cast at moe.py:753)
 *   topk_idx         [T, k] i32   out; descending score, lower index first on ties
 *
 * norm_topk_prob: SOFTMAX_TOPK, TOPK_RAW, SOFTMAX_ALL: divide by the sum of the k weights (moe.py:756);
 *   DEEPSEEK: w /= sum(w) + 1e-20, the sigmoid / sqrtsoftplus branch of moe.py:770-771.
 *   DEEPSEEK always multiplies by routed_scaling_factor (moe.py:772).
 * n_routing_groups / topk_routing_group: DeepSeek group-limited routing; -1 disables.
 * Limits: 1 <= k <= 16, k <= E <= 512, n_routing_groups <= 64 and divides E.
 */
MOE_API int moe_route_topk(const float* gate_logits, const float* pre_bias_logits, int T, int E, int k,
                   int mode, int norm_topk_prob, int weights_round_bf16,
                   float routed_scaling_factor, int n_routing_groups, int topk_routing_group,
                   float* topk_weights, int32_t* topk_idx, void* stream);

/* ---------------------------------------------------------------------------
 * Router: gate matmul + score function + bias + top-k through one call.  Replaces GateLogit.__call__
 * (src/maxtext/layers/moe.py:353-392) followed by RoutedMoE.get_topk (moe.py:717-765):
 *
 *   logits   = x @ Wg                       (f32 accumulation)
 *   scores   = sigmoid(logits) if score_func == 1, sqrt(softplus(logits)) if score_func == 2 (the DeepSeek-V4 router,
 *              layers/linears.py:51-53), else logits;   pre_bias = scores   (moe.py:382-386)
 *   scores  += gate_bias                                                              (moe.py:388-390)
 *   (topk_weights, topk_idx) = moe_route_topk(scores, pre_bias, ...)
 *
 *   x                  [T, d] bf16
 *   gate_kernel_terms  [num_terms, E, d] bf16: Wg^T written as a sum of bf16 terms.  num_terms == 3
 *                      (hi, mid, lo; hi = bf16(w), mid = bf16(w - hi), lo = bf16(w - hi - mid)) reproduces
 *                      the f32 gate (float32_gate_logits, moe.py:494-495): every product is exact in f32;
 *                      num_terms == 1 with gate_round_bf16 = 1 is the bf16 gate.
 *   gate_bias          [E] f32 or NULL
 *   gate_logits_out, pre_bias_logits_out   [T, E] f32 or NULL (the two values GateLogit returns)
 *   workspace          moe_gate_route_workspace_bytes(T, d, E) bytes (K-split partial sums, added in a fixed order)
 * The remaining arguments are those of moe_route_topk.  Limits: d % 64 == 0, E % 4 == 0, E <= 512, k <= 16.
 */
MOE_API size_t moe_gate_route_workspace_bytes(int T, int d, int E);
MOE_API int moe_gate_route(const void* x, const void* gate_kernel_terms, int num_terms, const float* gate_bias, int T,
                           int d, int E, int k, int score_func, int gate_round_bf16, int mode, int norm_topk_prob,
                           int weights_round_bf16, float routed_scaling_factor, int n_routing_groups,
                           int topk_routing_group, float* topk_weights, int32_t* topk_idx, float* gate_logits_out,
                           float* pre_bias_logits_out, void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Sort by expert.  Replaces the index half of RoutedMoE.permute
 * (moe.py:950-954, :960, :986-991): jnp.argsort (stable) of the flattened
 * expert ids, jnp.bincount, and repeat(arange(E), group_size).
 *
 *   topk_idx        [T, k] i32   in
 *   perm            [M] i32      out, M = T*k; == sorted_selected_experts
 *   inv_perm        [M] i32      out (may be NULL); inv_perm[perm[i]] = i == argsort(perm)
 *   group_sizes     [E] i32      out
 *   sorted_experts  [M] i32      out (may be NULL)
 * Limits: E <= 512.
 */
MOE_API size_t moe_sort_workspace_bytes(int T, int k, int E);
MOE_API int moe_sort_by_expert(const int32_t* topk_idx, int T, int k, int E, int32_t* perm,
                       int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, void* stream);
/* The same with the ids rolled first: key = (id - roll_to_expert_id) mod E (permute's roll_to_expert_id,
 * moe.py:953-954, by which a shard of the ring-of-experts strategy brings its own experts to the front);
 * group_sizes and sorted_experts are those of the rolled ids.  0 <= roll_to_expert_id < E. */
MOE_API int moe_sort_by_expert_rolled(const int32_t* topk_idx, int T, int k, int E, int roll_to_expert_id, int32_t* perm,
                       int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, void* stream);
/* The same with the roll read from the device: roll_to_expert_id_dev [1] i32 (taken mod E).  In the reference it is
 * expert_shard_id * local_experts with expert_shard_id = jax.lax.axis_index (moe.py:2014-2019), a device value. */
MOE_API int moe_sort_by_expert_rolled_dev(const int32_t* topk_idx, int T, int k, int E, const int32_t* roll_to_expert_id_dev,
                       int32_t* perm, int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, void* stream);
/* The same, and for up to 4096 routed rows (one launch) the block that sorted also builds the m-tile list of the
 * grouped matmuls that follow: gmm_workspace (moe_gmm_workspace_bytes(T * k, E) bytes) then holds the list for tiles of
 * tile_rows rows over these group_sizes with the given num_groups_local / group_offset / MOE_GMM_KEEP_OTHER_ROWS setting,
 * and a moe_gmm call on that workspace and the group_sizes buffer written here, flagged MOE_GMM_SAME_GROUPS, skips its
 * own mapping launch when it picks that tile height (16 for the streaming kernels of decode-sized calls; any other
 * choice rebuilds the list).  Above 4096 rows nothing is mapped: the sort then drops whatever record the library held
 * of a tile list over this group_sizes buffer (as every entry point does that writes group sizes without mapping), so a
 * following moe_gmm maps as usual, flagged or not. */
MOE_API int moe_sort_by_expert_mapped(const int32_t* topk_idx, int T, int k, int E, int roll_to_expert_id, int32_t* perm,
                       int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, int tile_rows, int num_groups_local, int group_offset,
                       int keep_other_rows, void* gmm_workspace, size_t gmm_workspace_bytes, void* stream);
/* moe_route_topk followed by moe_sort_by_expert_mapped on the indices it wrote (get_topk, moe.py:717-765, then the
 * argsort / bincount of permute, moe.py:950-960), with the arguments and results of both.  Up to 16 tokens (and 1024 routed
 * rows) without routing groups the two run as ONE launch (such a decode step spends as long on a launch as on either piece of work);
 * otherwise this is the two calls one after the other.  topk_idx is both a result and the sort's input. */
MOE_API int moe_route_sort_mapped(const float* gate_logits, const float* pre_bias_logits, int T, int E, int k,
                       int mode, int norm_topk_prob, int weights_round_bf16, float routed_scaling_factor,
                       int n_routing_groups, int topk_routing_group, float* topk_weights, int32_t* topk_idx,
                       int roll_to_expert_id, int32_t* perm, int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, int tile_rows, int num_groups_local, int group_offset,
                       int keep_other_rows, void* gmm_workspace, size_t gmm_workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Expert-parallel dispatch bookkeeping on one expert shard (integer work on device-resident sizes; the exchange
 * itself is a collective and no part of this library).
 *
 * moe_local_expert_keys replaces the index half of RoutedMoE.local_permute (moe.py:1091-1200) up to its argsort:
 *   global_group_sizes     [num_batch_shards, num_experts] i32: rows batch shard s holds for global expert e
 *   local_expert_size      experts per expert shard; this shard owns experts shard_index * local_expert_size ...
 *   num_rows               rows of the buffer local_permute is given (inputs.shape[0])
 *   global_sorted_experts  NULL (is_offset=False): the buffer holds the received rows grouped by (batch shard, local
 *                          expert), moe.py:1176-1178; key of row r = local expert of its segment, rows past the received
 *                          total take the last segment's expert (jnp.repeat's total_repeat_length padding).
 *                          [num_rows] i32 (is_offset=True): the buffer holds every routed row sorted by global expert,
 *                          moe.py:1166-1172; rows of this shard get e % local_expert_size, all others the key
 *                          local_expert_size.
 *   truncate               ragged_buffer_factor > 0: the per-(batch shard, local expert) sizes are cut at num_rows in
 *                          that order before they are summed (_maybe_truncate_local_group_size, moe.py:1066-1089)
 *   expert_keys            [num_rows] i32 out: expert_indices of local_permute; sort them with
 *                          moe_sort_by_expert(expert_keys, T = num_rows, k = 1, E = local_expert_size + 1): perm is
 *                          sorted_indices, sorted_experts is sorted_experts_ids; moe_gather_rows(inputs, perm) moves the rows
 *   local_group_size       [local_expert_size] i32 out
 *   workspace              moe_local_expert_keys_workspace_bytes(num_batch_shards, local_expert_size) bytes
 * Limits: num_batch_shards * local_expert_size <= 2^24.
 *
 * moe_all_to_all_params replaces RoutedMoE.get_all_to_all_params (moe.py:1202-1349): the input offsets, send sizes,
 * output offsets and receive sizes ([num_expert_parallelism] i32 each) that shard_id hands to ragged_all_to_all.
 *   all_shards_group_sizes  is_batch_sharded: [P, P] i32, entry (i, j) = rows batch shard i sends to expert shard j;
 *                           otherwise [P]: rows each expert shard is responsible for (replicated batch)
 *   buffer_size             >= 0: capacity of a receiver (ragged_buffer_factor > 0): the matrix is cut per receiver in
 *                           sender order (_truncate_matrix, moe.py:103-120); < 0: no capacity.  Batch-sharded only.
 *   is_dispatch             1: tokens to experts; 0: the way back (transposed roles, moe.py:1296-1330)
 * Limits: num_expert_parallelism <= 1024.
 *
 * moe_ring_ragged_indices derives the index arrays of ring_ragged_sort / ring_ragged_unsort
 * (kernels/ragged/ragged_sort.py:102-151, :300-350) from the sort's permutation, so that the row movement is one
 * moe_gather_rows (sort) or one moe_unpermute_combine (unsort) and nothing is read back by the host.  The rows of the
 * shard's experts [experts_start, experts_start + local_experts) are positions [start, end) of the sorted order.
 *   unsort = 0  indices = perm [num_rows]; indices_out [min(buffer_size, num_rows)]; row_range [2]:
 *               buffer_size >= num_rows: indices_out = perm, row_range = (start, end); smaller: indices_out[i] =
 *               perm[start + i] (0 past the end), row_range = (0, min(end - start, buffer_size)).  Gather with
 *               idx_div = k and this row_range.
 *   unsort = 1  indices = inv_perm [num_rows]; indices_out, valid_rows_mask [num_rows]: the inverse permutation
 *               (shifted by -start into the packed buffer when buffer_size < num_rows) and which of its entries
 *               point at a row of this shard; the others are 0 with mask 0.
 */
MOE_API size_t moe_local_expert_keys_workspace_bytes(int num_batch_shards, int local_expert_size);
MOE_API int moe_ring_ragged_indices(const int32_t* indices, const int32_t* group_sizes, int num_experts, int experts_start,
                            int local_experts, int num_rows, int buffer_size, int unsort, int32_t* indices_out,
                            uint8_t* valid_rows_mask, int32_t* row_range, void* stream);
MOE_API int moe_local_expert_keys(const int32_t* global_group_sizes, int num_batch_shards, int num_experts,
                          int local_expert_size, int shard_index, int num_rows, const int32_t* global_sorted_experts,
                          int truncate, int32_t* expert_keys, int32_t* local_group_size, void* workspace,
                          size_t workspace_bytes, void* stream);
MOE_API int moe_all_to_all_params(const int32_t* all_shards_group_sizes, int num_expert_parallelism, int shard_id,
                          int is_batch_sharded, long long buffer_size, int is_dispatch, int32_t* input_offsets,
                          int32_t* send_sizes, int32_t* output_offsets, int32_t* recv_sizes, void* stream);
/* The same three calls with the shard's index in device memory (an int32 the kernels read; the host never does): inside
 * shard_map the reference takes it from jax.lax.axis_index (moe.py:1134, :1709-1712, :2014-2019), a traced device value that
 * a custom call receives as a buffer.  Values outside the shards that exist are clamped into them.  In
 * moe_ring_ragged_indices_dev the shard owns experts [shard * local_experts, (shard + 1) * local_experts), so num_experts
 * must be a multiple of local_experts. */
MOE_API int moe_ring_ragged_indices_dev(const int32_t* indices, const int32_t* group_sizes, int num_experts,
                            const int32_t* shard_index_dev, int local_experts, int num_rows, int buffer_size, int unsort,
                            int32_t* indices_out, uint8_t* valid_rows_mask, int32_t* row_range, void* stream);
MOE_API int moe_local_expert_keys_dev(const int32_t* global_group_sizes, int num_batch_shards, int num_experts,
                          int local_expert_size, const int32_t* shard_index_dev, int num_rows,
                          const int32_t* global_sorted_experts, int truncate, int32_t* expert_keys, int32_t* local_group_size,
                          void* workspace, size_t workspace_bytes, void* stream);
MOE_API int moe_all_to_all_params_dev(const int32_t* all_shards_group_sizes, int num_expert_parallelism,
                          const int32_t* shard_id_dev, int is_batch_sharded, long long buffer_size, int is_dispatch,
                          int32_t* input_offsets, int32_t* send_sizes, int32_t* output_offsets, int32_t* recv_sizes, void* stream);

/* ---------------------------------------------------------------------------
 * Row gather with optional quantisation.  Replaces the data half of permute
 * (moe.py:956-959: repeat(x, k)[perm]) fused with the activation quantiser of
 * the grouped GEMM.  Two quantisation rules (moe_quant_rule):
 *
 *   MOE_QUANT_RINT_DIV  scale = absmax / qmax, q = rint(x / scale) clipped to +-qmax, in f32; zero absmax gives
 *                       q = 0, scale = 0.  Serves the v1 path, kernels/megablox/ops.py:241-248 (one scale per row,
 *                       channelwise_axes=[0]); its quantiser is third-party (qwix.pallas.quantize), so the rounding
 *                       rule is this library's choice, not a restatement.
 *   MOE_QUANT_V2        the quantiser inside gmm_v2, pallas_mosaic_tpu_v2_gmm_kernel.py:528-542, op by op in the
 *                       activation dtype (bf16): scale = bf16(absmax / qmax); inv = scale == 0 ? 0 : bf16(1 / scale);
 *                       q = bf16(x * inv) cast as `.astype` does: truncated toward zero for int8, rounded to nearest
 *                       even for fp8.  With static_scale (the per-tensor (1, 1) lhs_scale of :528-531, ops.py:333-360):
 *                       s = bf16(*static_scale), inv = bf16(1 / s), q = clip(bf16(x * inv), +-qmax) cast the same way.
 *
 *   x        [R_in, d] bf16
 *   row_idx  [R_out] i32 or NULL; output row i reads input row row_idx[i] / idx_div
 *            (NULL: row i).  permute passes row_idx = perm, idx_div = k.  An index outside [0, R_in) yields a row of zeros.
 *   out      [R_out, d] of out_dtype: MOE_BF16 (copy), MOE_INT8, MOE_FP8_E4M3 (qmax 127 / 448)
 *   scale    f32 out; block_k == 0: [R_out] one scale per row; block_k in {128, 256, 512}: [R_out, ceil(d/block_k)]
 *            (gmm_v2 uses 512, :1231; the DeepSeek recipe 1 x 128).  Not written when static_scale is given.
 *   static_scale  [1] f32 on the device, or NULL for dynamic (absmax) scales
 *   row_weight    [R_out] f32 or NULL: the gathered row is multiplied by its weight first (x[indices] * weights[:, None],
 *                 the weighted ragged_gather of kernels/ragged/ragged_gather.py:310-320; product rounded to bf16)
 *   row_range     [2] i32 (start, end) on the device, or NULL: output rows outside [start, end) are written as zeros
 *                 (ragged_gather.py:357-376 leaves them unspecified)
 * Limits: d % 8 == 0, d <= 16384.
 */
typedef enum { MOE_QUANT_RINT_DIV = 0, MOE_QUANT_V2 = 1 } moe_quant_rule;
MOE_API int moe_gather_rows(const void* x, const int32_t* row_idx, int idx_div, int R_in, int R_out, int d,
                    int out_dtype, int block_k, int rule, const float* static_scale, const float* row_weight,
                    const int32_t* row_range, void* out, float* scale, void* stream);

/* ---------------------------------------------------------------------------
 * Grouped matmul.  Replaces gmm(lhs, rhs, group_sizes, ...)
 * (src/maxtext/kernels/megablox/ops.py:46-129; backend.gmm backend.py:304-562;
 * gmm_v2 pallas_mosaic_tpu_v2_gmm_kernel.py:1297-1481) and the fused
 * "gmm, gmm, activation" of gmm_up + apply_ffn_activation (moe.py:1932-1986, :841-870).
 *
 *   out[rows of group g, :] = act( lhs[rows] @ rhs[g - group_offset]^T ... )
 *
 * for every g in [group_offset, group_offset + num_groups_local); all other rows of
 * `out` (non-local groups, rows past sum(group_sizes)) are written as zeros
 * (reference_gmm, tests/unit/pallas_mosaic_tpu_v2_kernel_test.py:139-141).
 *
 * Operand layouts in HBM
 *   lhs        [M, K] row-major ([lhs_rows, K] with lhs_row_idx), lhs_dtype in {BF16, INT8, FP8_E4M3, FP8_E5M2}
 *   lhs_scale  f32: NULL (bf16 lhs) | [M] one per row (lhs_scale_block_k == 0; qpl.quantize channelwise_axes=[0],
 *              ops.py:241-248) | [1] one for the tensor (lhs_scale_block_k == MOE_SCALE_PER_TENSOR; the static (1, 1)
 *              lhs_scale of gmm_v2, ops.py:333-360) | [M, ceil(K / b)] one per row and b values of K
 *              (lhs_scale_block_k == b: 128 for the DeepSeek 1 x 128 recipe, 512 for gmm_v2's in-kernel quantiser,
 *              pallas_mosaic_tpu_v2_gmm_kernel.py:1231; any multiple of 128)
 *   rhs        [G_local, N, K], K contiguous ("transpose_rhs" layout, ops.py:52),
 *              rhs_dtype in {BF16, INT8, FP8_E4M3, INT4, MXFP4}; INT4 / MXFP4 rows hold K/2 bytes
 *   rhs_scale  NULL (bf16 rhs), else scales over blocks of bn = rhs_scale_block_n output channels (1 = per channel,
 *              128 = DeepSeek 128 x 128 blocks, MOE_SCALE_PER_TENSOR = one for all channels) and bk = rhs_scale_block_k
 *              values of K (0 = all of K).  With nnb = ceil(N / bn) and nkb = ceil(K / bk) the layout is
 *                [G_local, nnb, nkb]                     by default (DeepSeek fp8 checkpoints, int4 group scales), or
 *                [G_local, nkb, nnb]                     with MOE_GMM_RHS_SCALE_KMAJOR: gmm_v2's [G, nb, 1, N]
 *                                                        (ops.py:310-331; bn == 1, bk a multiple of 128, for INT8 / FP8
 *                                                        lhs; a multiple of 32 for weight-only INT8 / INT4);
 *              MOE_GMM_RHS_SCALE_SHARED drops the leading dimension: one set of scales for all experts (the
 *              [1, 1, n] scale qpl.quantize yields for channelwise_axes=[2], ops.py:250-260, and the per-tensor scale
 *              of manual_quantize, layers/quantizations.py:961-991).  f32; bf16 for INT4 in the default layout;
 *              MXFP4: e8m0 bytes [G_local, N, K/32] (bn = 1, bk = 32)
 *   rhs_up / rhs_up_scale   second projection (wi_1) with the same layout; when non-NULL
 *              the kernel computes act(lhs@rhs^T) * (lhs@rhs_up^T) in one pass
 *   rhs_bias / rhs_up_bias   [G_local, N] f32 or NULL, see the end of the struct
 *   out        [M, N] bf16, or f32 (out_dtype == MOE_F32: preferred_element_type of ops.py:50)
 *
 * Supported operand combinations (others return MOE_ERR_UNSUPPORTED):
 *   BF16 x BF16
 *   BF16 x INT8   per channel or per tensor (bk = 0), or KMAJOR [G, nkb, N]
 *   BF16 x INT4   bf16 [G, N, ceil(K/bk)] with bk = 128 or 32, or f32 KMAJOR [G, nkb, N]
 *   BF16 x MXFP4
 *   INT8 x INT8, FP8 x FP8:
 *     lhs per row or per tensor  x  rhs per channel or per tensor over all of K (what gmm() quantises to, ops.py:232-267)
 *     lhs per row / per tensor / [M, K/b]  x  rhs KMAJOR per channel [G, nkb, N] (gmm_v2's layouts; K % 128 == 0)
 *     FP8 only: lhs [M, K/128]  x  rhs 128 x 128 blocks [G, N/128, K/128] (DeepSeek-V3 checkpoints)
 *   FP8_E5M2 x FP8 (the quantised gradient against the forward's e4m3 weights, ops.py:583-642): lhs per row or per
 *     tensor x rhs per channel or per tensor, without rhs_up, on shapes moe_gmm_lhs_e5m2_supported() accepts
 * Alignment: K % 32 == 0 (INT4, MXFP4), K % 16 == 0 otherwise; N % 8 == 0; pointers 16-byte aligned.
 */
#define MOE_SCALE_PER_TENSOR (-1)

typedef struct {
  size_t struct_size; /* sizeof(moe_gmm_args), checked */
  const void* lhs;
  const float* lhs_scale;
  const void* rhs;
  const void* rhs_scale;
  const void* rhs_up;
  const void* rhs_up_scale;
  const int32_t* group_sizes; /* [num_groups_total] i32, device */
  void* out;
  void* workspace;
  size_t workspace_bytes;
  int32_t M, K, N;
  int32_t num_groups_total; /* length of group_sizes                       */
  int32_t num_groups_local; /* leading dim of rhs                          */
  int32_t group_offset;     /* first global group held by rhs (backend.py:340-347) */
  int32_t lhs_dtype, rhs_dtype;
  int32_t lhs_scale_block_k;
  int32_t rhs_scale_block_n, rhs_scale_block_k;
  int32_t act;     /* moe_act; must be MOE_ACT_NONE when rhs_up == NULL      */
  float act_limit; /* clip for SWIGLUOAI / SILU_CLIP                        */
  int32_t out_dtype;       /* MOE_BF16 (= 0) or MOE_F32                                        */
  int32_t lhs_row_idx_div; /* see lhs_row_idx; values < 1 are read as 1                        */
  int32_t lhs_rows;        /* rows of lhs when lhs_row_idx is given (indices are clamped to it) */
  int32_t reserved;        /* zero */
  /* per-expert bias [G_local, N] f32 added to lhs@rhs^T (and to lhs@rhs_up^T) before the activation:
   * w0_bias / w1_bias / wo_bias of mlp_bias models (moe.py:1952-1981, :2239-2241; rhs_bias of
   * pallas_mosaic_tpu_v2_gmm_kernel.py:573).  NULL = no bias.  Rows that are written as zeros stay zero. */
  const float* rhs_bias;
  const float* rhs_up_bias;
  /* [M, N] bf16 or NULL: added to lhs@rhs^T (to lhs@rhs_up^T) after the bias and before the activation, for rows
   * of local groups only: partial_sum of ops.py:77 / pallas_mosaic_tpu_v2_gmm_kernel.py:576-578, used by the
   * embedding-chunked expert MLP (moe.py:1962-1980).  Must not alias `out`. */
  const void* partial_sum;
  const void* partial_sum_up;
  int32_t flags; /* MOE_GMM_* bits */
  int32_t pad_;
  /* [M] i32 or NULL: row i of the product reads lhs row lhs_row_idx[i] / lhs_row_idx_div, and that row's scales, instead
   * of row i: the permute (moe.py:956-959: repeat(x, k)[perm]; kernels/ragged/ragged_gather.py:310-320) fused into the
   * matmul, so that the [M, K] gathered copy is never written and T token rows are quantised instead of M = T * k copies.
   * permute passes lhs_row_idx = perm, lhs_row_idx_div = k, lhs_rows = T. */
  const int32_t* lhs_row_idx;
  /* [M] f32 or NULL: row i of the result is multiplied by out_row_scale[i] after the activation and before the rounding
   * to out_dtype: the routing weights applied between the activation and wo
   * (models/deepseek_batchsplit_fp8.py:1049, intermediate_layer *= weights[:, None]). */
  const float* out_row_scale;
  /* [1] i32 on the device, or NULL: when given it replaces group_offset (negative values are read as 0).  Inside
   * shard_map the reference's group_offset is a ()-shaped device array derived from jax.lax.axis_index
   * (backend.py:340-345, moe.py:2014-2019), which a custom call receives as a buffer, not as an attribute: the tile-map
   * kernel reads it, so the host never needs the value. */
  const int32_t* group_offset_dev;
} moe_gmm_args;

/* flags: rows that belong to no local group are left as `out` holds them instead of being written as zeros:
 * the existing_out argument of gmm (ops.py:51, backend.py:493-501), where a caller accumulates the shards' rows
 * in one buffer. */
#define MOE_GMM_KEEP_OTHER_ROWS 1
/* flags: rhs is [G_local, K, N] with N contiguous, the reference's default layout (transpose_rhs=False, ops.py:47-52),
 * read as it is: no re-layout pass.  This is how the backward computes dlhs = gmm(dout, rhs, transpose_rhs=True)
 * (ops.py:470-485) from the forward's [G, N, K] weights, whose roles of K and N are then swapped.  BF16 x BF16 without
 * rhs_up, on shapes moe_gmm_rhs_kn_supported() accepts, and fp8 x fp8 (e4m3 weights, e4m3 or e5m2 activations, scales
 * per row / tensor x per channel / tensor, no row index) on shapes moe_gmm_fp8_rhs_kn_supported() accepts; others return
 * MOE_ERR_UNSUPPORTED: re-lay the weights out with moe_transpose_rhs and call without the flag. */
#define MOE_GMM_RHS_KN 2
/* flags: layout of rhs_scale / rhs_up_scale, see "Operand layouts" above. */
#define MOE_GMM_RHS_SCALE_KMAJOR 4
#define MOE_GMM_RHS_SCALE_SHARED 8
/* flags: the caller's promise that group_sizes holds what it held at the previous moe_gmm call on this device (or at
 * the moe_sort_by_expert_mapped call that built the list), that the workspace is the same buffer, untouched since, and
 * that this call is ordered behind that one.  When that call mapped the same M, groups and tile height, its tile list is
 * used again and the mapping launch is skipped (the second and third product of an expert layer: one launch less in a
 * chain of dependent launches, about 4 us at decode sizes); when anything differs the list is rebuilt as usual.  The
 * library keeps one record per device, the last call's, and drops it when one of its own entry points (the sorts,
 * moe_local_expert_keys) writes that group_sizes buffer again without mapping; what the library cannot see is a buffer
 * the caller overwrites itself, or frees and gets back at the same address: that is the promise. */
#define MOE_GMM_SAME_GROUPS 16

/* 1 when moe_gmm takes MOE_GMM_RHS_KN for this shape (K % 64 == 0, N % 256 == 0, 128 rows per group on average and
 * enough 256 x 256 tiles to fill the chip), else 0. */
MOE_API int moe_gmm_rhs_kn_supported(int M, int K, int N, int num_groups_total);
/* 1 when moe_gmm takes MOE_FP8_E5M2 activations for this shape (the persistent 256 x 256 kernel: K % 128 == 0, K >= 384,
 * N * K < 2^32, 128 rows per group on average and enough tiles to fill the chip), else 0: widen the gradient to bf16
 * (moe_bwd_scale_grad with quantize == 1) and the weights with it. */
MOE_API int moe_gmm_lhs_e5m2_supported(int M, int K, int N, int num_groups_total);
/* 1 when moe_gmm takes MOE_GMM_RHS_KN with fp8 operands for this shape (what moe_gmm_lhs_e5m2_supported asks, and
 * N % 256 == 0), else 0. */
MOE_API int moe_gmm_fp8_rhs_kn_supported(int M, int K, int N, int num_groups_total);
/* 1 when the persistent stream kernels take this operand pair at this K and N (whole stages, at least three of them,
 * and every 32-bit byte offset a request can form stays below 2^32), with indexed_lhs_rows = lhs_rows when lhs_row_idx is
 * used, else 0.  moe_gmm falls back to its other kernels otherwise; no counterpart in the reference. */
MOE_API int moe_gmm_stream_kernel_takes(int lhs_dtype, int rhs_dtype, int K, int N, long long indexed_lhs_rows);
MOE_API size_t moe_gmm_workspace_bytes(int M, int num_groups_total);
MOE_API int moe_gmm(const moe_gmm_args* args, void* stream);

/* moe_gmm for callers that cannot allocate device memory for the workspace (code under HIP graph capture, serving
 * loops and harnesses that forbid hipMalloc): no counterpart in the reference.  args->workspace / workspace_bytes are
 * ignored; the m-tile list goes into an array the library holds in device memory (one per GPU, 1 MiB =
 * moe_gmm_static_ws_capacity(), kept until the process ends).  The call allocates nothing.  Requests whose tile list
 * does not fit (moe_gmm_workspace_bytes(M, num_groups_total) above the capacity: about a million rows) return
 * MOE_ERR_WORKSPACE.  Every call on a GPU shares that GPU's array: calls that overlap on one GPU (two streams, two
 * threads) race; calls in stream order are safe, because each call rewrites the part of the list it reads.
 * The first call on a device looks the array's address up and raises the LDS limit of the kernel it launches;
 * moe_init() does both ahead of time for every kernel. */
MOE_API size_t moe_gmm_static_ws_capacity(void);
MOE_API int moe_gmm_static_ws(const moe_gmm_args* args, void* stream);

/* Per-device set-up, for the device that is current: the CU count, the address of the static workspace and the raised
 * LDS limit of every kernel.  Optional: each entry point does its share on first use.  No counterpart in the reference. */
MOE_API int moe_init(void);

/* moe_gmm with the kernel family and the tile raster chosen by the caller instead of by the shape: a tuning and test
 * aid (no counterpart in the reference; the parity tests use it to run every kernel family on small shapes).
 * kernel: MOE_GMM_KERNEL_*; a family that does not take the operands returns MOE_ERR_UNSUPPORTED.
 * raster: > 0 = m-tiles per super-row of the tile order (persistent and fp8 LDS kernels); 0 = default. */
typedef enum {
  MOE_GMM_KERNEL_AUTO = 0,
  MOE_GMM_KERNEL_STREAM = 1,    /* register-staged streaming kernels (fp8 block-scaled, weight-only formats); AUTO
                                   prefers the persistent kernels that stream the weights through LDS where they take
                                   the shape (group-128 int4, MXFP4, 8-bit x 8-bit operands with K % 512 == 0)        */
  MOE_GMM_KERNEL_TILED = 2,     /* LDS-tiled kernels with the m-tile chosen by rows per expert (fp8: 128 x 128)       */
  MOE_GMM_KERNEL_BIG = 3,       /* 256 x 256 tiles: fp8 block-scaled (the persistent stream kernel when K % 512 == 0,
                                   what AUTO picks for prefill-sized groups); int8 x int8 register-staged kernel       */
  MOE_GMM_KERNEL_DL64 = 4,      /* direct-to-LDS persistent kernel with 64-byte stages (int8 x int8, bf16 x bf16)     */
  MOE_GMM_KERNEL_STREAM_NOSPLIT = 5 /* weight-only streaming kernel with every wave walking all of K                   */
} moe_gmm_kernel;
MOE_API int moe_gmm_tuned(const moe_gmm_args* args, int kernel, int raster, void* stream);

/* One-time weight re-layout [G, K, N] -> [G, N, K] (1-byte or 2-byte elements), for
 * callers that hold the reference's default rhs layout (ops.py:47, transpose_rhs=False). */
MOE_API int moe_transpose_rhs(const void* rhs_gkn, int G, int K, int N, int elem_bytes, void* rhs_gnk,
                      void* stream);

/* ---------------------------------------------------------------------------
 * Transposed grouped matmul (weight gradient of gmm).  Replaces tgmm(lhs^T, dout, group_sizes, ...)
 * (src/maxtext/kernels/megablox/backend.py:575-816; called from _gmm_bwd, ops.py:766) for bf16 operands:
 *
 *   out[g - group_offset, n, k] = sum over the rows m of group g of dout[m, n] * lhs[m, k]
 *
 *   lhs   [M, K] bf16   forward activations (the caller does NOT transpose them)
 *   dout  [M, N] bf16   gradient of the forward output
 *   existing_out  NULL, or [G_local, N, K] bf16 or f32 (existing_dtype) added to the f32 products before the
 *         one rounding to out_dtype (backend.py:733-734).  It may be `out` itself when the element types agree
 *         (the reference aliases the two buffers, backend.py:761-766).
 *   out   [G_local, N, K] bf16 or f32 (out_dtype): the layout of the forward weights; groups with no
 *         rows are written as zeros plus existing_out (reference_tgmm,
 *         tests/unit/pallas_mosaic_tpu_v2_kernel_test.py:156-186)
 * The gradient of lhs needs no entry point of its own: it is moe_gmm(dout, rhs re-laid out as [G, K, N]).
 * Limits: K % 8 == 0, N % 8 == 0.
 */
MOE_API int moe_tgmm(const void* lhs, const void* dout, const int32_t* group_sizes, int M, int K, int N,
                     int num_groups_total, int num_groups_local, int group_offset, const void* existing_out,
                     int existing_dtype, int out_dtype, void* out, void* stream);
/* The same with the products of output row n (the channel of dout) multiplied by out_row_scale[n] ([N] f32) before
 * existing_out is added and the result is rounded: the column scales of a float8_e5m2 gradient (ops.py:590-603) go
 * back onto the weight gradient here instead of in a pass over [G, N, K]. */
MOE_API int moe_tgmm_scaled(const void* lhs, const void* dout, const int32_t* group_sizes, int M, int K, int N,
                    int num_groups_total, int num_groups_local, int group_offset, const float* out_row_scale,
                    const void* existing_out, int existing_dtype, int out_dtype, void* out, void* stream);
/* moe_tgmm_scaled on 1-byte operands as they are stored: lhs [M, K] float8_e4m3fn (the quantised activations kept from the
 * forward) and dout [M, N] float8_e5m2 or float8_e4m3fn (dout_dtype; the gradient quantised per column by
 * moe_bwd_scale_grad with quantize = 2), the drhs product of the fp8_full backward (kernels/megablox/ops.py:590-604) on the
 * fp8 MFMA with f32 accumulation.  Same output, out_row_scale and existing_out as above.  Runs on 256 x 256 output tiles only:
 * K % 256 == 0, N % 256 == 0, M >= 128 * num_groups_total, at least 128 tiles (moe_tgmm_fp8_supported says so; other shapes
 * return MOE_ERR_UNSUPPORTED and take the operands widened to bf16, in which fp8 values are exact, through moe_tgmm_scaled). */
MOE_API int moe_tgmm_fp8_supported(int M, int K, int N, int num_groups_total, int num_groups_local);
MOE_API int moe_tgmm_fp8(const void* lhs, const void* dout, int dout_dtype, const int32_t* group_sizes, int M, int K, int N,
                 int num_groups_total, int num_groups_local, int group_offset, const float* out_row_scale,
                 const void* existing_out, int existing_dtype, int out_dtype, void* out, void* stream);

/* ---------------------------------------------------------------------------
 * Unpermute + top-k weighted combine.  Replaces RoutedMoE.unpermute
 * (moe.py:1039-1063, float32_weight_sum=True) and the fused gather-reduce
 * fallback (kernels/ragged/ragged_gather_reduce_v2.py:170-182):
 *
 *   out[t, :] = bf16( sum over the valid s of weights[t, s] * f32(y[inv_perm[t*k + s], :]) )
 *
 *   y        [M, d] bf16     expert outputs in sorted order
 *   perm     [M] i32         sorted_selected_experts; used only when inv_perm == NULL,
 *                            then inv_perm is rebuilt into `workspace` (M * 4 bytes)
 *   weights  [T, k] f32, or NULL for an unweighted sum
 *            (kernels/sort_activations.py:98-121)
 *   valid_rows_mask  [T, k] bytes, or NULL for "all valid": a zero byte takes gathered row (t, s) out of the sum
 *            (valid_rows_mask of ragged_gather_reduce, kernels/ragged/ragged_gather_reduce_v2.py:637-659; the row
 *            is not read, so a NaN in it does not reach the output)
 *   out      [T, d] bf16
 * Limits: d % 8 == 0, k <= 16.
 */
MOE_API int moe_unpermute_combine(const void* y, const int32_t* perm, const int32_t* inv_perm,
                          const float* weights, const uint8_t* valid_rows_mask, int T, int k, int d, void* out,
                          void* workspace, size_t workspace_bytes, void* stream);

/* ---------------------------------------------------------------------------
 * Gradient of moe_unpermute_combine with respect to y and to the weights (the VJP that JAX derives for
 * the gather + einsum of moe.py:1041-1062; its hand-written counterpart for the fused kernel is
 * kernels/sort_activations.py:85-121):
 *
 *   dy[inv_perm[t*k + s], :] = bf16( weights[t, s] * f32(dout[t, :]) )
 *   dweights[t, s]           = sum_d f32(y[inv_perm[t*k + s], d]) * f32(dout[t, d])
 *
 *   dout [T, d] bf16; y [M, d] bf16 (forward input; may be NULL when dweights is NULL);
 *   weights [T, k] f32 or NULL (ones); dy [M, d] bf16 (every row is written: inv_perm is a permutation);
 *   dweights [T, k] f32 or NULL; valid_rows_mask as in the forward pass: a masked (t, s) gets a zero row of dy
 *   and a zero dweights entry.
 * The gradient of the row gather (moe_gather_rows in copy mode; _sort_activations_custom_bwd,
 * moe.py:165-171) is moe_unpermute_combine itself with weights == NULL.
 * Limits: d % 8 == 0, k <= 16.
 */
MOE_API int moe_unpermute_combine_bwd(const void* dout, const void* y, const int32_t* inv_perm, const float* weights,
                                      const uint8_t* valid_rows_mask, int T, int k, int d, void* dy, float* dweights,
                                      void* stream);

/* ---------------------------------------------------------------------------
 * Gated activation as a stand-alone pass and its gradient, for training, where both projections are kept
 * for the backward pass (apply_ffn_activation, moe.py:841-870, and the VJP JAX derives for it):
 *
 *   out = act(h0, h1)                 (as the fused epilogue of moe_gmm computes it, f32 math, bf16 result)
 *   dh0, dh1 = d out / d (h0, h1) * dout; clipped inputs (SWIGLUOAI, SILU_CLIP) pass no gradient outside
 *   their clip range.
 *
 * All tensors are bf16 with n elements (n % 8 == 0), 16-byte aligned.
 */
MOE_API int moe_glu_act(const void* h0, const void* h1, size_t n, int act, float act_limit, void* out, void* stream);
MOE_API int moe_glu_act_bwd(const void* h0, const void* h1, const void* dout, size_t n, int act, float act_limit,
                            void* dh0, void* dh1, void* stream);

/* ---------------------------------------------------------------------------
 * Per-expert bias on finished bf16 rows: out[m, :] = bf16(h[m, :] + bias[g(m), :]) for the rows of the local groups
 * (g(m) = the row's group minus group_offset), all other rows copied.  This is the separate add of the reference's
 * layer (layer_w0 + w0_bias after the matmul has rounded to the activation dtype, moe.py:1952-1957, :2239-2242), which
 * the differentiable path keeps so that its forward rounds twice like the reference's; inference calls pass the bias to
 * moe_gmm (rhs_bias), whose epilogue adds it before the one rounding.
 *   h, out [M, N] bf16 (may be the same buffer);  bias [num_groups_local, N] f32
 * Limits: N % 8 == 0, at most 1024 groups.
 */
MOE_API int moe_add_group_bias(const void* h, int M, int N, const float* bias, const int32_t* group_sizes, int num_groups_total,
                       int num_groups_local, int group_offset, void* out, void* stream);

/* ---------------------------------------------------------------------------
 * Gradient preparation of the quantised backward pass (int8 x int8 or fp8 x fp8 forward with channelwise scales): the incoming
 * gradient times the scale of the axis that the gradient product contracts away (_bwd_prepare_inputs,
 * kernels/megablox/ops.py:530-580), optionally quantised to float8_e5m2 (_bwd_quantize_gradient, ops.py:583-604;
 * symmetric absmax scale = absmax / 57344, values rounded to nearest even, a zero scale gives zeros).
 *
 *   MOE_BWD_FOR_DLHS  d[m, n] = bf16(dout[m, n] * bf16(factor[g(m), n]));  factor = rhs scales [G_local, N] f32, g(m) the
 *                     expert of row m relative to group_offset, clamped to the local experts; quantised per row:
 *                     scale_out [M]
 *   MOE_BWD_FOR_DRHS  d[m, n] = bf16(dout[m, n] * bf16(factor[m]));  factor = lhs scales [M] f32; quantised per column:
 *                     scale_out [N] (group_sizes is not used)
 *   MOE_BWD_PER_TENSOR  d[m, n] = bf16(dout[m, n] * bf16(factor[0]));  factor = the one scale [1] f32 of a tensor quantised
 *                     with channelwise_axes=[] (disable_channelwise_axes, ops.py:568, :594, :601), either operand's; one
 *                     scale for the whole gradient: scale_out [N], every entry holding that scale (the buffer carries the
 *                     column maxima on the way; group_sizes is not used)
 *
 *   dout [M, N] bf16;  out [M, N] bf16: d itself (quantize == 0; scale_out is not touched), or d / scale on the e5m2
 *   grid, whose values are exact in bf16 (quantize == 1), so that moe_gmm / moe_tgmm take it as a bf16 operand;
 *   quantize == 2: out [M, N] holds the same values as float8_e5m2 bytes, the MOE_FP8_E5M2 lhs of moe_gmm.
 * Limits: N % 8 == 0, N <= 16384, at most 1024 groups.
 */
typedef enum { MOE_BWD_FOR_DLHS = 0, MOE_BWD_FOR_DRHS = 1, MOE_BWD_PER_TENSOR = 2 } moe_bwd_mode;
MOE_API int moe_bwd_scale_grad(const void* dout, int M, int N, int mode, int quantize, const float* factor,
                               const int32_t* group_sizes, int num_groups_total, int num_groups_local, int group_offset,
                               void* out, float* scale_out, void* stream);

/* ---------------------------------------------------------------------------
 * Weight quantiser of the training path: what gmm() applies to bf16 weights on every step
 * (_fwd_quantize_activation_and_weight, kernels/megablox/ops.py:250-266).
 *
 *   w       [G, N, K] bf16, K contiguous
 *   q       [G, N, K] out_dtype: MOE_INT8 or MOE_FP8_E4M3
 *   dynamic (static_scale == NULL): qpl.quantize(rhs, qtype, channelwise_axes=[2]) (ops.py:250-260): one scale per output
 *           channel over all of K, shared by the experts (shared != 0: scale [N], the [1, 1, n] of the reference) or per
 *           expert (shared == 0: scale [G, N]); scale = absmax / qmax, q = rint(w / scale) (int8) or the nearest-even
 *           float8 cast of w / scale, zero channels give q = 0 and scale 0.  The third-party quantiser's rounding is not
 *           in the reference tree: this is the library's MOE_QUANT_RINT_DIV rule.
 *   static  (static_scale [1] f32 on the device): manual_quantize (layers/quantizations.py:961-991) for bf16 weights:
 *           q = clip(bf16(w / bf16(scale)), +-qmax) cast as `.astype` does (int8 truncates toward zero, float8 rounds to
 *           nearest even); `scale` is not written.
 *           shared == 2: one scale for the whole tensor (scale [1]): disable_channelwise_axes of the qwix rule
 *           (channelwise_axes=[], ops.py:258).
 * Limits: K % 8 == 0.
 *
 * moe_tensor_scale: scale[0] = max|x| / qmax over x [rows, K] bf16: the dynamic per-tensor activation scale of
 * disable_channelwise_axes (ops.py:245); feed it to moe_gather_rows as static_scale.  `scale` doubles as the
 * reduction's scratch word.
 */
MOE_API int moe_tensor_scale(const void* x, long long rows, int K, float qmax, float* scale, void* stream);
MOE_API int moe_quantize_rhs(const void* w, int G, int N, int K, int out_dtype, int shared, const float* static_scale,
                             void* q, float* scale, void* stream);

#ifdef __cplusplus
}
#endif
#endif /* MOE_MI355X_H_ */
