// Routing, sort-by-expert, row gather (+ activation quantisation), unpermute+combine.
// All of these are HBM/latency-bound integer and byte work: one wavefront per token for
// top-k, a three-launch stable counting sort for the permutation, 16-byte coalesced
// row copies for the gathers.

#include <limits.h>
#include <math.h>
#include <stdarg.h>
#include <stdio.h>

#include "moe_gmm_common.h"

namespace moe {

static thread_local char g_err[256] = "";

int fail(int code, const char* fmt, ...) {
  va_list ap;
  va_start(ap, fmt);
  vsnprintf(g_err, sizeof(g_err), fmt, ap);
  va_end(ap);
  return code;
}

int check_launch(const char* what) {
  hipError_t e = hipGetLastError();
  if (e != hipSuccess) return fail(MOE_ERR_LAUNCH, "%s: %s", what, hipGetErrorString(e));
  return MOE_OK;
}

// ---------------------------------------------------------------------------------------
// Top-k routing: one wavefront per token, lane l owns experts l, l+64, ...
// ---------------------------------------------------------------------------------------

constexpr int kRouteMaxE = 512;
constexpr int kRouteVpl = kRouteMaxE / kWave;  // values per lane
constexpr int kRouteWaves = 4;

// (value, index) order of lax.top_k as adopted here: larger value first, lower index first.
__device__ __forceinline__ bool better(float av, int ai, float bv, int bi) {
  return av > bv || (av == bv && ai < bi);
}

__device__ __forceinline__ void wave_argmax(float& bv, int& bi) {
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) {
    float ov = __shfl_xor(bv, o);
    int oi = __shfl_xor(bi, o);
    if (better(ov, oi, bv, bi)) {
      bv = ov;
      bi = oi;
    }
  }
}

// With GATE the scores are built here from the partial sums of the gate matmul (GateLogit.__call__,
// moe.py:353-392): logits = sum of the K-split partials (in split order, so the result does not depend on
// scheduling), optional bf16 rounding (gate computed in bf16), score function, pre_bias = scores,
// scores += bias.
struct GateEpilogue {
  const float* partials;  // [num_partials, T, E]
  const float* bias;      // [E] or NULL
  float* logits_out;      // [T, E] or NULL
  float* pre_bias_out;    // [T, E] or NULL
  int num_partials;
  int score_func;         // 0 none, 1 sigmoid, 2 sqrt(softplus)
  int round_bf16;         // round the matmul result to bf16 first
};

// One token per wave: token t_raw of T (a wave past the end repeats the last token and writes nothing; every wave of the
// block must make the call, there is a block barrier inside).  s_row_w / s_pre_w: this wave's kRouteMaxE floats of LDS.
template <bool GATE>
__device__ __forceinline__ void route_token(
    const float* __restrict__ logits, const float* __restrict__ pre_bias, int T, int E, int k,
    int mode, int norm, int round_bf16, float scaling, int n_groups, int topk_groups,
    float* __restrict__ w_out, int32_t* __restrict__ idx_out, const GateEpilogue& g, int t_raw, int lane, float* s_row_w, float* s_pre_w) {
  const bool active = t_raw < T;
  const int t = active ? t_raw : T - 1;
  const float* row = logits + (size_t)t * E;

  float v[kRouteVpl];
  unsigned taken = 0;
#pragma unroll
  for (int j = 0; j < kRouteVpl; j++) {
    int e = lane + kWave * j;
    if (GATE) {
      float x = -INFINITY;
      if (e < E) {
        x = 0.f;
        for (int s = 0; s < g.num_partials; s++) x += g.partials[((size_t)s * T + t) * E + e];
        if (g.round_bf16) x = round_bf16_fn(x);
        if (g.score_func == 1) x = 1.0f / (1.0f + expf(-x));
        // sqrt(softplus(x)), softplus as logaddexp(x, 0) = max(x, 0) + log1p(exp(-|x|)) (linears.py:51-53)
        if (g.score_func == 2) x = sqrtf(fmaxf(x, 0.f) + log1pf(expf(-fabsf(x))));
        s_pre_w[e] = x;
        if (active && g.pre_bias_out) g.pre_bias_out[(size_t)t * E + e] = x;
        if (g.bias) x += g.bias[e];
        if (active && g.logits_out) g.logits_out[(size_t)t * E + e] = x;
      }
      v[j] = x;
    } else {
      v[j] = e < E ? row[e] : -INFINITY;
    }
    if (e >= E) taken |= 1u << j;
  }

  if (n_groups > 0) {
    // expert_group_mask: group score = sum of the group's two best scores; keep the best
    // topk_groups groups, everything else becomes -inf (still selectable, as in jnp.where).
    const int gs = E / n_groups;
#pragma unroll
    for (int j = 0; j < kRouteVpl; j++) {
      int e = lane + kWave * j;
      if (e < E) s_row_w[e] = v[j];
    }
    __syncthreads();
    float score = -INFINITY;
    int gi = INT_MAX;
    if (lane < n_groups) {
      float b1 = -INFINITY, b2 = -INFINITY;
      for (int i = 0; i < gs; i++) {
        float x = s_row_w[lane * gs + i];
        if (x > b1) {
          b2 = b1;
          b1 = x;
        } else if (x > b2) {
          b2 = x;
        }
      }
      score = b1 + b2;
      gi = lane;
    }
    unsigned long long sel = 0;
    bool mine_taken = lane >= n_groups;
    for (int r = 0; r < topk_groups; r++) {
      float bv = mine_taken ? -INFINITY : score;
      int bi = mine_taken ? INT_MAX : gi;
      wave_argmax(bv, bi);
      if (bi < n_groups) sel |= 1ull << bi;
      if (bi == lane) mine_taken = true;
    }
#pragma unroll
    for (int j = 0; j < kRouteVpl; j++) {
      int e = lane + kWave * j;
      if (e < E && !((sel >> (e / gs)) & 1ull)) v[j] = -INFINITY;
    }
  }

  float myv = 0.f;
  int myi = 0;
  for (int r = 0; r < k; r++) {
    float bv = -INFINITY;
    int bi = INT_MAX;
#pragma unroll
    for (int j = 0; j < kRouteVpl; j++) {
      if (!((taken >> j) & 1u)) {
        int e = lane + kWave * j;
        if (better(v[j], e, bv, bi)) {
          bv = v[j];
          bi = e;
        }
      }
    }
    wave_argmax(bv, bi);
    if (bi == INT_MAX) bi = 0;  // only reachable with NaN scores
    if (lane == r) {
      myv = bv;
      myi = bi;
    }
    if ((bi & (kWave - 1)) == lane) taken |= 1u << (bi >> 6);
  }

  float w;
  if (mode == MOE_ROUTE_DEEPSEEK) {
    if (GATE)
      w = lane < k ? s_pre_w[myi] : 0.f;  // written by this wave's own lanes above
    else
      w = lane < k ? pre_bias[(size_t)t * E + myi] : 0.f;
    if (norm) {
      float s = wave_sum(w);
      w = w / (s + 1e-20f);
    }
    w *= scaling;
  } else {
    float mx = __shfl(myv, 0);
    if (mode == MOE_ROUTE_TOPK_RAW) {
      w = lane < k ? myv : 0.f;
    } else if (mode == MOE_ROUTE_SOFTMAX_ALL) {
      // softmax over every expert (the best score is the first selected one), read at the selected experts
      float part = 0.f;
#pragma unroll
      for (int j = 0; j < kRouteVpl; j++)
        if (lane + kWave * j < E) part += expf(v[j] - mx);
      const float s = wave_sum(part);
      w = lane < k ? expf(myv - mx) / s : 0.f;
    } else {
      float ex = lane < k ? expf(myv - mx) : 0.f;
      float s = wave_sum(ex);
      w = ex / s;
    }
    if (round_bf16) w = round_bf16_fn(w);
    if (norm) {
      float s2 = wave_sum(lane < k ? w : 0.f);
      if (round_bf16) s2 = round_bf16_fn(s2);
      w = w / s2;
      if (round_bf16) w = round_bf16_fn(w);
    }
  }
  if (active && lane < k) {
    w_out[(size_t)t * k + lane] = w;
    idx_out[(size_t)t * k + lane] = myi;
  }
}

template <bool GATE>
__global__ __launch_bounds__(kRouteWaves* kWave) void route_topk_kernel(
    const float* __restrict__ logits, const float* __restrict__ pre_bias, int T, int E, int k,
    int mode, int norm, int round_bf16, float scaling, int n_groups, int topk_groups,
    float* __restrict__ w_out, int32_t* __restrict__ idx_out, const GateEpilogue g) {
  __shared__ float s_row[kRouteWaves][kRouteMaxE];
  __shared__ float s_pre[GATE ? kRouteWaves : 1][GATE ? kRouteMaxE : 1];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  route_token<GATE>(logits, pre_bias, T, E, k, mode, norm, round_bf16, scaling, n_groups, topk_groups, w_out, idx_out, g,
                    blockIdx.x * kRouteWaves + wave, lane, s_row[wave], s_pre[GATE ? wave : 0]);
}

// ---------------------------------------------------------------------------------------
// Gate matmul x [T, d] bf16  @  Wg [d, E] f32 -> partial logits f32, Wg given as a sum of S bf16 terms
// [S, E, d] (S = 3 reproduces f32 products: 3 x 8 mantissa bits; S = 1 is the bf16 gate).  A block owns
// 32 tokens x 32 experts and one slice of K; its 4 waves split the slice further and add through LDS.
// Operands go straight from global memory into MFMA fragments: within a 64-element chunk of K, lanes
// 0-31 take elements 0-31 of their row and lanes 32-63 elements 32-63 (64 contiguous bytes each), the
// same for both operands, so the contraction order is a fixed permutation of K.
// ---------------------------------------------------------------------------------------

struct GateGemmParams {
  const uint16_t* x;   // [T, d] bf16
  const uint16_t* wg;  // [S, E, d] bf16
  float* partial;      // [KS, T, E]
  int T, d, E, S;
  int chunks_per_block;  // 64-element chunks of K per block (grid.z slices)
};

template <int S>
__global__ __launch_bounds__(256) void gate_gemm_kernel(const GateGemmParams p) {
  __shared__ float red[3 * 16 * kWave];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int r = lane % 32, g = lane / 32;
  const int t0 = blockIdx.x * 32, e0 = blockIdx.y * 32;
  const int nchunks = p.d / 64;
  const int c_begin = blockIdx.z * p.chunks_per_block;
  const int c_end = min(nchunks, c_begin + p.chunks_per_block);
  const int per_wave = (c_end - c_begin + 3) / 4;
  int c = c_begin + wave * per_wave;
  const int c_stop = min(c_end, c + per_wave);

  const uint8_t* xp = (const uint8_t*)(p.x + (size_t)min(t0 + r, p.T - 1) * p.d) + g * 64;
  const uint8_t* wp[S];
#pragma unroll
  for (int s = 0; s < S; s++) wp[s] = (const uint8_t*)(p.wg + ((size_t)s * p.E + min(e0 + r, p.E - 1)) * p.d) + g * 64;

  v16f acc[S];
#pragma unroll
  for (int s = 0; s < S; s++)
#pragma unroll
    for (int i = 0; i < 16; i++) acc[s][i] = 0.f;

  auto step = [&](int c0, auto ucount) {
    constexpr int UC = decltype(ucount)::value;
    uint4 xr[UC][4], wr[UC][S][4];
#pragma unroll
    for (int u = 0; u < UC; u++) {
      const size_t off = (size_t)(c0 + u) * 128;
#pragma unroll
      for (int q = 0; q < 4; q++) xr[u][q] = *(const uint4*)(xp + off + q * 16);
#pragma unroll
      for (int s = 0; s < S; s++)
#pragma unroll
        for (int q = 0; q < 4; q++) wr[u][s][q] = *(const uint4*)(wp[s] + off + q * 16);
    }
#pragma unroll
    for (int u = 0; u < UC; u++)
#pragma unroll
      for (int q = 0; q < 4; q++)
#pragma unroll
        for (int s = 0; s < S; s++)
          acc[s] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, wr[u][s][q]), __builtin_bit_cast(v8bf, xr[u][q]),
                                                           acc[s], 0, 0, 0);
  };
  for (; c + 2 <= c_stop; c += 2) step(c, std::integral_constant<int, 2>{});
  for (; c < c_stop; c++) step(c, std::integral_constant<int, 1>{});

  // smallest term first, as one would add a float's low bits
  v16f sum = acc[S - 1];
#pragma unroll
  for (int s = S - 2; s >= 0; s--)
#pragma unroll
    for (int i = 0; i < 16; i++) sum[i] += acc[s][i];

  if (wave > 0) {
#pragma unroll
    for (int i = 0; i < 16; i++) red[((wave - 1) * 16 + i) * kWave + lane] = sum[i];
  }
  __syncthreads();
  if (wave > 0) return;
#pragma unroll
  for (int w = 0; w < 3; w++)
#pragma unroll
    for (int i = 0; i < 16; i++) sum[i] += red[(w * 16 + i) * kWave + lane];

  // D[i = expert][j = token]: lane holds token r and experts 8*q + 4*g + 0..3
  const int t = t0 + r;
  if (t >= p.T) return;
  float* out = p.partial + ((size_t)blockIdx.z * p.T + t) * p.E;
#pragma unroll
  for (int q = 0; q < 4; q++) {
    const int e = e0 + 8 * q + 4 * g;
    if (e < p.E) *(float4*)(out + e) = make_float4(sum[4 * q], sum[4 * q + 1], sum[4 * q + 2], sum[4 * q + 3]);
  }
}

// ---------------------------------------------------------------------------------------
// Stable counting sort of the flattened expert ids.
//   pass 1: per-wave-segment histograms; pass 2: exclusive scan over segments (one wave per expert);
//   pass 3: each wave re-reads its segment and ranks equal ids with ballots, in index order.
// ---------------------------------------------------------------------------------------

constexpr int kSortWaves = 4;
constexpr int kSortRounds = 4;
constexpr int kSortSeg = kSortRounds * kWave;    // entries per wave
constexpr int kSortChunk = kSortSeg * kSortWaves;  // entries per block
constexpr int kSortMaxE = 512;

__device__ __forceinline__ int clamp_expert(int e, int E) { return e < 0 ? 0 : (e >= E ? E - 1 : e); }
// sort key of expert id e: (e - roll) mod E (permute's roll_to_expert_id, moe.py:953-954; roll = 0: the id itself)
// the roll as given, or read from the device and taken mod E
__device__ __forceinline__ int resolve_roll(int roll, const int32_t* roll_dev, int E) {
  if (!roll_dev) return roll;
  const int r = *roll_dev % E;
  return r < 0 ? r + E : r;
}
__device__ __forceinline__ int sort_key(int e, int E, int roll) {
  e = clamp_expert(e, E) - roll;
  return e < 0 ? e + E : e;
}

__global__ __launch_bounds__(kSortWaves* kWave) void sort_hist_kernel(
    const int32_t* __restrict__ flat, int M, int E, int roll, const int32_t* __restrict__ roll_dev, int32_t* __restrict__ seg_hist) {
  roll = resolve_roll(roll, roll_dev, E);
  __shared__ int cnt[kSortWaves][kSortMaxE];
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  for (int e = lane; e < E; e += kWave) cnt[wave][e] = 0;
  __syncthreads();
  const int base = blockIdx.x * kSortChunk + wave * kSortSeg;
#pragma unroll
  for (int r = 0; r < kSortRounds; r++) {
    int i = base + r * kWave + lane;
    if (i < M) atomicAdd(&cnt[wave][sort_key(flat[i], E, roll)], 1);
  }
  __syncthreads();
  int32_t* dst = seg_hist + (size_t)(blockIdx.x * kSortWaves + wave) * E;
  for (int e = lane; e < E; e += kWave) dst[e] = cnt[wave][e];
}

// pass 2: one wave per expert turns its column of segment counts into exclusive prefixes (64 segments per step,
// a shuffle scan inside the wave) and writes the expert's total to group_sizes.
__global__ __launch_bounds__(kSortWaves* kWave) void sort_scan_kernel(int32_t* __restrict__ seg_hist, int nseg, int E,
                                                                     int32_t* __restrict__ group_sizes) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  const int e = blockIdx.x * kSortWaves + wave;
  if (e >= E) return;
  int running = 0;
  for (int s0 = 0; s0 < nseg; s0 += kWave) {
    const int s = s0 + lane;
    const int c = s < nseg ? seg_hist[(size_t)s * E + e] : 0;
    int incl = c;
#pragma unroll
    for (int o = 1; o < kWave; o <<= 1) {
      const int up = __shfl_up(incl, o);
      if (lane >= o) incl += up;
    }
    if (s < nseg) seg_hist[(size_t)s * E + e] = running + incl - c;
    running += __shfl(incl, kWave - 1);
  }
  if (lane == 0) group_sizes[e] = running;
}

__global__ __launch_bounds__(kSortWaves* kWave) void sort_scatter_kernel(
    const int32_t* __restrict__ flat, int M, int E, int roll, const int32_t* __restrict__ roll_dev, int ebits,
    const int32_t* __restrict__ seg_hist, const int32_t* __restrict__ group_sizes,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm,
    int32_t* __restrict__ sorted_experts) {
  __shared__ int run[kSortWaves][kSortMaxE];
  __shared__ int off[kSortMaxE];
  roll = resolve_roll(roll, roll_dev, E);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  // first row of every expert = exclusive scan of group_sizes, rebuilt by each block (E <= 512 values)
  for (int e = threadIdx.x; e < kSortMaxE; e += kSortWaves * kWave) off[e] = e < E ? group_sizes[e] : 0;
  __syncthreads();
  for (int o = 1; o < kSortMaxE; o <<= 1) {
    int add[kSortMaxE / (kSortWaves * kWave)];
#pragma unroll
    for (int q = 0; q < kSortMaxE / (kSortWaves * kWave); q++) {
      const int e = threadIdx.x + q * kSortWaves * kWave;
      add[q] = e >= o ? off[e - o] : 0;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < kSortMaxE / (kSortWaves * kWave); q++) off[threadIdx.x + q * kSortWaves * kWave] += add[q];
    __syncthreads();
  }
  const int32_t* seg = seg_hist + (size_t)(blockIdx.x * kSortWaves + wave) * E;
  for (int e = lane; e < E; e += kWave) run[wave][e] = (e > 0 ? off[e - 1] : 0) + seg[e];
  __syncthreads();
  const int base = blockIdx.x * kSortChunk + wave * kSortSeg;
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int r = 0; r < kSortRounds; r++) {
    const int i = base + r * kWave + lane;
    const bool valid = i < M;
    const int e = valid ? sort_key(flat[i], E, roll) : 0;
    unsigned long long mask = __ballot(valid);
    for (int b = 0; b < ebits; b++) {
      const bool bit = (e >> b) & 1;
      const unsigned long long bal = __ballot(valid && bit);
      mask &= bit ? bal : ~bal;
    }
    const int rank = __popcll(mask & lt);
    const int cnt = __popcll(mask);
    const int start = valid ? run[wave][e] : 0;
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == cnt - 1) run[wave][e] = start + cnt;
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      const int dest = start + rank;
      perm[dest] = i;
      if (inv_perm) inv_perm[i] = dest;
      if (sorted_experts) sorted_experts[dest] = e;
    }
  }
}

// All three passes in one block of NW waves for at most NW * kSortSeg entries (decode and small prefill: a launch costs
// as much as a pass; NW = 4 up to 1024 entries, 16 up to 4096): per-wave histograms in LDS, the prefixes over the
// segments and over the experts, then the same in-order ranking.
// The m-tile list of the grouped matmuls that follow, built behind the sort by the same block (tiles == NULL: not wanted).
struct SortMapArgs {
  TileInfo* tiles;
  int32_t* header;
  int G_local, group_offset, BM, zero_fill;
};

template <int NW>
__device__ __forceinline__ void sort_small_block(
    const int32_t* __restrict__ flat, int M, int E, int roll, const int32_t* __restrict__ roll_dev, int ebits, int32_t* __restrict__ group_sizes,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm, int32_t* __restrict__ sorted_experts, const SortMapArgs& mp) {
  __shared__ int run[NW][kSortMaxE];
  __shared__ int off[kSortMaxE];
  constexpr int NT = NW * kWave;
  roll = resolve_roll(roll, roll_dev, E);
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  if (M <= kWave && E <= kWave) {
    // The smallest decode steps (at most 64 routed rows over at most 64 experts): one wave holds an entry and an expert per
    // lane and sorts without a block barrier or a trip through memory: equal keys found by ballots, their count left in LDS
    // by the first of them, the experts' first rows by a scan over the lanes.  The tile list is then built from the counts in LDS.
    __shared__ int t_cnt[kWave], t_off[kWave];
    if (wave == 0) {
      const bool valid = lane < M;
      const int e = valid ? sort_key(flat[lane], E, roll) : 0;
      unsigned long long mask = __ballot(valid);
      for (int b = 0; b < ebits; b++) {
        const bool bit = (e >> b) & 1;
        const unsigned long long bal = __ballot(valid && bit);
        mask &= bit ? bal : ~bal;
      }
      const int rank = __popcll(mask & ((1ull << lane) - 1ull)), cnt = __popcll(mask);
      t_cnt[lane] = 0;
      __builtin_amdgcn_wave_barrier();
      if (valid && rank == 0) t_cnt[e] = cnt;
      __builtin_amdgcn_wave_barrier();
      const int c = lane < E ? t_cnt[lane] : 0;
      int incl = c;
#pragma unroll
      for (int o = 1; o < kWave; o <<= 1) {
        const int t = __shfl_up(incl, o);
        if (lane >= o) incl += t;
      }
      t_off[lane] = incl - c;
      if (lane < E) group_sizes[lane] = c;
      __builtin_amdgcn_wave_barrier();
      if (valid) {
        const int dest = t_off[e] + rank;
        perm[dest] = lane;
        if (inv_perm) inv_perm[lane] = dest;
        if (sorted_experts) sorted_experts[dest] = e;
      }
    }
    if (mp.tiles) {
      __syncthreads();
      build_tile_map<NT>(t_cnt, E, mp.group_offset, mp.G_local, M, mp.BM, mp.zero_fill, mp.header, mp.tiles, &run[0][0]);
    }
    return;
  }
  // (only the E counters that exist are cleared, scanned and offset: with 32 experts of at most 1024 that is 5 scan steps
  // instead of 10, each between two barriers)
  for (int e = threadIdx.x; e < NW * E; e += NT) run[e / E][e % E] = 0;
  __syncthreads();
  const int base = wave * kSortSeg;
#pragma unroll
  for (int r = 0; r < kSortRounds; r++) {
    const int i = base + r * kWave + lane;
    if (i < M) atomicAdd(&run[wave][sort_key(flat[i], E, roll)], 1);
  }
  __syncthreads();
  // counts of the segments -> exclusive prefixes over the segments; the expert's total goes to group_sizes and to off
  for (int e = threadIdx.x; e < E; e += NT) {
    int running = 0;
#pragma unroll
    for (int w = 0; w < NW; w++) {
      const int c = run[w][e];
      run[w][e] = running;
      running += c;
    }
    off[e] = running;
    group_sizes[e] = running;
  }
  __syncthreads();
  for (int o = 1; o < E; o <<= 1) {  // inclusive scan of the totals
    constexpr int Q = (kSortMaxE + NT - 1) / NT;
    int add[Q];
#pragma unroll
    for (int q = 0; q < Q; q++) {
      const int e = threadIdx.x + q * NT;
      add[q] = e >= o && e < E ? off[e - o] : 0;
    }
    __syncthreads();
#pragma unroll
    for (int q = 0; q < Q; q++)
      if (threadIdx.x + q * NT < E) off[threadIdx.x + q * NT] += add[q];
    __syncthreads();
  }
  for (int e = lane; e < E; e += kWave) run[wave][e] += e > 0 ? off[e - 1] : 0;
  __syncthreads();
  const unsigned long long lt = (1ull << lane) - 1ull;
  for (int r = 0; r < kSortRounds; r++) {
    const int i = base + r * kWave + lane;
    const bool valid = i < M;
    const int e = valid ? sort_key(flat[i], E, roll) : 0;
    unsigned long long mask = __ballot(valid);
    for (int b = 0; b < ebits; b++) {
      const bool bit = (e >> b) & 1;
      const unsigned long long bal = __ballot(valid && bit);
      mask &= bit ? bal : ~bal;
    }
    const int rank = __popcll(mask & lt);
    const int cnt = __popcll(mask);
    const int start = valid ? run[wave][e] : 0;
    __builtin_amdgcn_wave_barrier();
    if (valid && rank == cnt - 1) run[wave][e] = start + cnt;
    __builtin_amdgcn_wave_barrier();
    if (valid) {
      const int dest = start + rank;
      perm[dest] = i;
      if (inv_perm) inv_perm[i] = dest;
      if (sorted_experts) sorted_experts[dest] = e;
    }
  }
  if (mp.tiles) {
    __syncthreads();  // group_sizes, written above by this block, are read back from memory
    build_tile_map<NT>(group_sizes, E, mp.group_offset, mp.G_local, M, mp.BM, mp.zero_fill, mp.header, mp.tiles, &run[0][0]);
  }
}

template <int NW>
__global__ __launch_bounds__(NW* kWave) void sort_small_kernel(
    const int32_t* __restrict__ flat, int M, int E, int roll, const int32_t* __restrict__ roll_dev, int ebits, int32_t* __restrict__ group_sizes,
    int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm, int32_t* __restrict__ sorted_experts, const SortMapArgs mp) {
  sort_small_block<NW>(flat, M, E, roll, roll_dev, ebits, group_sizes, perm, inv_perm, sorted_experts, mp);
}

// Routing and the sort behind it in one block, for at most NW tokens (the smallest decode steps): every wave routes one
// token, the indices they wrote are read back by the block as the sort's keys.  One launch instead of two where a launch
// costs as much as the work; with more tokens than waves the routing of one block would take turns and lose to the
// many blocks of the kernel of its own.
struct RouteArgs {
  const float* logits;
  const float* pre_bias;
  int T, E, k, mode, norm, round_bf16;
  float scaling;
  int n_groups, topk_groups;
  float* w_out;
  int32_t* idx_out;
};

template <int NW>
__global__ __launch_bounds__(NW* kWave) void route_sort_small_kernel(
    const RouteArgs r, int roll, int ebits, int32_t* __restrict__ group_sizes, int32_t* __restrict__ perm, int32_t* __restrict__ inv_perm,
    int32_t* __restrict__ sorted_experts, const SortMapArgs mp) {
  const int wave = threadIdx.x / kWave, lane = threadIdx.x % kWave;
  // (one token per wave, all at once: r.T <= NW, no routing groups)
  route_token<false>(r.logits, r.pre_bias, r.T, r.E, r.k, r.mode, r.norm, r.round_bf16, r.scaling, 0, 0, r.w_out, r.idx_out, GateEpilogue{}, wave, lane,
                     nullptr, nullptr);
  __syncthreads();  // the indices, written above by this block, are read back from memory
  sort_small_block<NW>(r.idx_out, r.T * r.k, r.E, roll, nullptr, ebits, group_sizes, perm, inv_perm, sorted_experts, mp);
}

__global__ void invert_perm_kernel(const int32_t* __restrict__ perm, int M,
                                   int32_t* __restrict__ inv) {
  int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < M) {
    int p = perm[i];
    if (p >= 0 && p < M) inv[p] = i;
  }
}

// ---------------------------------------------------------------------------------------
// Row gather with optional quantisation: one 256-thread block per output row, the row is
// held in registers between the absmax pass and the quantise pass (one HBM read).
// ---------------------------------------------------------------------------------------

constexpr int kGqThreads = 256;
constexpr int kGqMaxChunks = 8;  // 16-byte chunks per thread -> d <= 256*8*8

enum { GQ_COPY = 0, GQ_INT8 = 1, GQ_FP8 = 2 };

__device__ __forceinline__ void unpack8(const uint4& u, float f[8]) {
  f[0] = bf16_bits_to_f32(u.x & 0xffffu);
  f[1] = bf16_bits_to_f32(u.x >> 16);
  f[2] = bf16_bits_to_f32(u.y & 0xffffu);
  f[3] = bf16_bits_to_f32(u.y >> 16);
  f[4] = bf16_bits_to_f32(u.z & 0xffffu);
  f[5] = bf16_bits_to_f32(u.z >> 16);
  f[6] = bf16_bits_to_f32(u.w & 0xffffu);
  f[7] = bf16_bits_to_f32(u.w >> 16);
}

__device__ __forceinline__ float absmax8(const uint4& u) {
  float f[8];
  unpack8(u, f);
  float m = 0.f;
#pragma unroll
  for (int i = 0; i < 8; i++) m = fmaxf(m, fabsf(f[i]));
  return m;
}

// Quantisation rules (moe_quant_rule).  RINT_DIV: scale = absmax / qmax, q = rint(x / scale) clipped, all in f32 (the
// rule adopted for the v1 path's third-party quantiser).  V2: the in-kernel quantiser of the reference's gmm_v2
// (pallas_mosaic_tpu_v2_gmm_kernel.py:528-542), whose every operation is carried out in the activation dtype, bf16:
// scale = bf16(absmax / qmax), inv = scale == 0 ? 0 : bf16(1 / scale), y = bf16(x * inv), then the cast of
// `.astype`: truncation toward zero for int8, round-to-nearest-even for fp8.  A bf16 op is an f32 op (correctly
// rounded, the default of hipcc for division) followed by a rounding to bf16, as XLA computes it.
struct QuantCfg {
  int rule;                   // moe_quant_rule
  int block_lanes;            // lanes that share a scale: 16 / 32 / 64 (K blocks of 128 / 256 / 512), 0 = the whole row
  int nkb;                    // scales per row
  const float* static_scale;  // [1] or NULL
  const float* row_weight;    // [R_out] or NULL: the gathered row is multiplied by its weight (rounded to bf16) first
  const int32_t* row_range;   // [2] (start, end) on the device or NULL: output rows outside [start, end) are zeros
};

template <int MODE>
__device__ __forceinline__ void quant_scale(float m, int rule, float& sc, float& inv) {
  const float qmax = MODE == GQ_INT8 ? 127.0f : 448.0f;
  if (rule == MOE_QUANT_V2) {
    sc = round_bf16_fn(m / qmax);
    inv = sc == 0.f ? 0.f : round_bf16_fn(1.0f / sc);
  } else {
    sc = m / qmax;
    inv = sc == 0.f ? 0.f : 1.0f / sc;  // this rule divides; the int8 path uses the reciprocal to find the values that need it
  }
}

template <int MODE>
__device__ __forceinline__ float quant_value(float f, float sc, float inv, int rule, bool is_static) {
  const float qmax = MODE == GQ_INT8 ? 127.0f : 448.0f;
  if (rule == MOE_QUANT_V2) {
    float y = round_bf16_fn(f * inv);
    // dynamic scales keep |y| <= 127.5 (450 for fp8), which the cast itself brings to qmax; the static branch
    // clips before the cast (:531)
    y = fminf(fmaxf(y, -qmax), qmax);
    (void)is_static;
    return MODE == GQ_INT8 ? truncf(y) : y;
  }
  if (MODE == GQ_INT8) {
    // rint(f / sc) without dividing: f * (1 / sc) is off the rounded quotient by at most 1.2e-7 of its value, 2.4e-5
    // for |q| < 200, so unless it lies within 1e-4 of k + 1/2 both round to the same integer; the few values that do lie
    // there (and those beyond 200, NaN included) take the division.  sc == 0 has inv == 0 and gives 0.
    float q = f * inv;
    if (fabsf(__builtin_amdgcn_fractf(q) - 0.5f) < 1e-4f || !(fabsf(q) < 200.0f)) q = sc == 0.f ? 0.f : f / sc;
    return fminf(fmaxf(rintf(q), -qmax), qmax);
  }
  const float q = sc == 0.f ? 0.f : f / sc;
  return fminf(fmaxf(q, -qmax), qmax);
}

template <int MODE>
__global__ __launch_bounds__(kGqThreads) void gather_rows_kernel(
    const uint4* __restrict__ x, const int32_t* __restrict__ row_idx, int idx_div, int R_in, int d,
    void* __restrict__ out, float* __restrict__ scale, const QuantCfg qc) {
  __shared__ float s_red[kGqThreads / kWave];
  const int r = blockIdx.x;
  const int src = row_idx ? row_idx[r] / idx_div : r;
  const int nch = d / 8;
  // an index outside the input (a malformed row_idx) reads nothing and yields a row of zeros, and so does an output
  // row outside the requested range (ragged_gather's [start, end), kernels/ragged/ragged_gather.py:357-376)
  bool in_range = src >= 0 && src < R_in;
  if (qc.row_range) in_range = in_range && r >= qc.row_range[0] && r < qc.row_range[1];
  const uint4* xrow = x + (size_t)(in_range ? src : 0) * nch;
  uint4 regs[kGqMaxChunks];
#pragma unroll
  for (int c = 0; c < kGqMaxChunks; c++) {
    int ci = threadIdx.x + c * kGqThreads;
    regs[c] = ci < nch && in_range ? xrow[ci] : make_uint4(0, 0, 0, 0);
  }
  if (qc.row_weight) {  // x[indices] * weights[:, None] (ragged_gather.py:316-319), product rounded to bf16
    const float w = qc.row_weight[r];
#pragma unroll
    for (int c = 0; c < kGqMaxChunks; c++) {
      float f[8];
      unpack8(regs[c], f);
      regs[c] = make_uint4(pack_bf16x2(f[0] * w, f[1] * w), pack_bf16x2(f[2] * w, f[3] * w), pack_bf16x2(f[4] * w, f[5] * w),
                           pack_bf16x2(f[6] * w, f[7] * w));
    }
  }

  if (MODE == GQ_COPY) {
    uint4* orow = (uint4*)out + (size_t)r * nch;
#pragma unroll
    for (int c = 0; c < kGqMaxChunks; c++) {
      int ci = threadIdx.x + c * kGqThreads;
      if (ci < nch) orow[ci] = regs[c];
    }
    return;
  }

  const bool is_static = qc.static_scale != nullptr;
  float row_sc = 0.f, row_inv = 0.f;
  if (is_static) {
    // one scale for the whole tensor: bf16(scale) and its bf16 inverse for the v2 rule (:528-529), the value itself otherwise
    const float s = *qc.static_scale;
    row_sc = qc.rule == MOE_QUANT_V2 ? round_bf16_fn(s) : s;
    row_inv = qc.rule == MOE_QUANT_V2 ? round_bf16_fn(1.0f / row_sc) : row_sc == 0.f ? 0.f : 1.0f / row_sc;
  } else if (qc.block_lanes == 0) {
    float m = 0.f;
#pragma unroll
    for (int c = 0; c < kGqMaxChunks; c++) m = fmaxf(m, absmax8(regs[c]));
    m = wave_max(m);
    if (threadIdx.x % kWave == 0) s_red[threadIdx.x / kWave] = m;
    __syncthreads();
    m = fmaxf(fmaxf(s_red[0], s_red[1]), fmaxf(s_red[2], s_red[3]));
    quant_scale<MODE>(m, qc.rule, row_sc, row_inv);
    if (threadIdx.x == 0) scale[r] = row_sc;
  }
  uint2* orow = (uint2*)out + (size_t)r * nch;
#pragma unroll
  for (int c = 0; c < kGqMaxChunks; c++) {
    int ci = threadIdx.x + c * kGqThreads;
    float sc = row_sc, inv = row_inv;
    if (!is_static && qc.block_lanes != 0) {
      // a K block is block_lanes consecutive 16-byte chunks == consecutive lanes of one wave
      float m = absmax8(regs[c]);
      for (int o = qc.block_lanes / 2; o > 0; o >>= 1) m = fmaxf(m, __shfl_xor(m, o));
      quant_scale<MODE>(m, qc.rule, sc, inv);
      if (ci < nch && (threadIdx.x & (qc.block_lanes - 1)) == 0) scale[(size_t)r * qc.nkb + ci / qc.block_lanes] = sc;
    }
    if (ci < nch) {
      float f[8];
      unpack8(regs[c], f);
#pragma unroll
      for (int i = 0; i < 8; i++) f[i] = quant_value<MODE>(f[i], sc, inv, qc.rule, is_static);
      if (MODE == GQ_INT8) {
        uint32_t b[8];
#pragma unroll
        for (int i = 0; i < 8; i++) b[i] = (uint32_t)((int)f[i]) & 0xffu;
        orow[ci] = make_uint2(b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24), b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24));
      } else {
        int lo = 0, hi = 0;
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], lo, false);
        lo = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], lo, true);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], hi, false);
        hi = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], hi, true);
        orow[ci] = make_uint2((uint32_t)lo, (uint32_t)hi);
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Unpermute + weighted combine: one block per token, f32 accumulation over the k rows.
// ---------------------------------------------------------------------------------------

constexpr int kCombineMaxK = 16;

__global__ __launch_bounds__(256) void combine_kernel(const uint4* __restrict__ y,
                                                      const int32_t* __restrict__ inv_perm,
                                                      const float* __restrict__ weights,
                                                      const uint8_t* __restrict__ valid, int k,
                                                      int d, uint4* __restrict__ out) {
  __shared__ int s_row[kCombineMaxK];
  __shared__ float s_w[kCombineMaxK];
  const int t = blockIdx.x;
  if (threadIdx.x < k) {
    // an index outside [0, M) (a malformed inv_perm) contributes nothing instead of reading out of bounds, and so does
    // a row that the caller masked out
    const int row = inv_perm[(size_t)t * k + threadIdx.x];
    const bool ok = row >= 0 && row < (int)gridDim.x * k && (!valid || valid[(size_t)t * k + threadIdx.x]);
    s_row[threadIdx.x] = ok ? row : -1;
    s_w[threadIdx.x] = weights ? weights[(size_t)t * k + threadIdx.x] : 1.0f;
  }
  __syncthreads();
  const int nch = d / 8;
  // (few tokens: gridDim.y blocks share a token's row, so that a decode-sized call still fills the chip)
  for (int ci = blockIdx.y * blockDim.x + threadIdx.x; ci < nch; ci += blockDim.x * gridDim.y) {
    float acc[8] = {0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f, 0.f};
    for (int s = 0; s < k; s++) {
      if (s_row[s] < 0) continue;
      uint4 u = y[(size_t)s_row[s] * nch + ci];
      float f[8];
      unpack8(u, f);
      const float w = s_w[s];
#pragma unroll
      for (int i = 0; i < 8; i++) acc[i] = fmaf(w, f[i], acc[i]);
    }
    uint4 o;
    o.x = pack_bf16x2(acc[0], acc[1]);
    o.y = pack_bf16x2(acc[2], acc[3]);
    o.z = pack_bf16x2(acc[4], acc[5]);
    o.w = pack_bf16x2(acc[6], acc[7]);
    out[(size_t)t * nch + ci] = o;
  }
}

// Gradient of the combine: one block per token.  dy[row_s] = bf16(w_s * dout[t]) for the k rows the token
// gathered, dw[t, s] = sum_d f32(y[row_s, d]) * f32(dout[t, d]).
__global__ __launch_bounds__(256) void combine_bwd_kernel(const uint4* __restrict__ dout, const uint4* __restrict__ y,
                                                          const int32_t* __restrict__ inv_perm,
                                                          const float* __restrict__ weights,
                                                          const uint8_t* __restrict__ valid, int k, int d,
                                                          uint4* __restrict__ dy, float* __restrict__ dw) {
  __shared__ int s_row[kCombineMaxK];
  __shared__ float s_w[kCombineMaxK];
  __shared__ bool s_masked[kCombineMaxK];
  __shared__ float s_part[kCombineMaxK][4];
  const int t = blockIdx.x;
  if (threadIdx.x < k) {
    const int row = inv_perm[(size_t)t * k + threadIdx.x];
    s_row[threadIdx.x] = row >= 0 && row < (int)gridDim.x * k ? row : -1;  // malformed index: no row is written
    s_w[threadIdx.x] = weights ? weights[(size_t)t * k + threadIdx.x] : 1.0f;
    s_masked[threadIdx.x] = valid && !valid[(size_t)t * k + threadIdx.x];  // a masked row took no part: zero gradients
  }
  __syncthreads();
  const int nch = d / 8;
  float dot[kCombineMaxK];
#pragma unroll
  for (int s = 0; s < kCombineMaxK; s++) dot[s] = 0.f;
  for (int ci = threadIdx.x; ci < nch; ci += blockDim.x) {
    float g[8];
    unpack8(dout[(size_t)t * nch + ci], g);
#pragma unroll
    for (int s = 0; s < kCombineMaxK; s++) {
      if (s >= k) break;
      if (s_row[s] < 0) continue;
      const size_t at = (size_t)s_row[s] * nch + ci;
      if (s_masked[s]) {
        dy[at] = make_uint4(0, 0, 0, 0);
        continue;
      }
      const float w = s_w[s];
      uint4 o;
      o.x = pack_bf16x2(w * g[0], w * g[1]);
      o.y = pack_bf16x2(w * g[2], w * g[3]);
      o.z = pack_bf16x2(w * g[4], w * g[5]);
      o.w = pack_bf16x2(w * g[6], w * g[7]);
      dy[at] = o;
      if (dw) {
        float f[8];
        unpack8(y[at], f);
#pragma unroll
        for (int i = 0; i < 8; i++) dot[s] = fmaf(f[i], g[i], dot[s]);
      }
    }
  }
  if (!dw) return;
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
#pragma unroll
  for (int s = 0; s < kCombineMaxK; s++) {
    if (s >= k) break;
    const float v = wave_sum(dot[s]);
    if (lane == 0) s_part[s][wave] = v;
  }
  __syncthreads();
  if (threadIdx.x < k) dw[(size_t)t * k + threadIdx.x] = s_part[threadIdx.x][0] + s_part[threadIdx.x][1] + s_part[threadIdx.x][2] + s_part[threadIdx.x][3];
}

// ---------------------------------------------------------------------------------------
// Gated activation on its own (training keeps both projections for the backward pass) and its gradient.
// 8 bf16 values per thread; all math in f32.
// ---------------------------------------------------------------------------------------

template <int ACT>
__global__ __launch_bounds__(256) void glu_fwd_kernel(const uint4* __restrict__ h0, const uint4* __restrict__ h1, size_t nvec,
                                                      float limit, uint4* __restrict__ out) {
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (size_t)gridDim.x * 256) {
    float g[8], u[8], y[8];
    unpack8(h0[i], g);
    unpack8(h1[i], u);
#pragma unroll
    for (int j = 0; j < 8; j++) y[j] = glu_act<ACT>(g[j], u[j], limit);
    out[i] = make_uint4(pack_bf16x2(y[0], y[1]), pack_bf16x2(y[2], y[3]), pack_bf16x2(y[4], y[5]), pack_bf16x2(y[6], y[7]));
  }
}

// y = gc * sigmoid(a * gc) * (uc + b) with gc = min(g, L), uc = clamp(u, -L, L) (no clipping for plain SiLU):
// dy/dg = [g <= L] (uc + b) s (1 + a gc (1 - s)),  dy/du = [-L <= u <= L] gc s,  s = sigmoid(a gc).
template <int ACT>
__global__ __launch_bounds__(256) void glu_bwd_kernel(const uint4* __restrict__ h0, const uint4* __restrict__ h1,
                                                      const uint4* __restrict__ dy, size_t nvec, float limit,
                                                      uint4* __restrict__ dh0, uint4* __restrict__ dh1) {
  constexpr bool CLIP = ACT != MOE_ACT_SILU;
  constexpr float a = ACT == MOE_ACT_SWIGLUOAI ? 1.702f : 1.0f;
  constexpr float b = ACT == MOE_ACT_SWIGLUOAI ? 1.0f : 0.0f;
  for (size_t i = (size_t)blockIdx.x * 256 + threadIdx.x; i < nvec; i += (size_t)gridDim.x * 256) {
    float g[8], u[8], d[8], dg[8], du[8];
    unpack8(h0[i], g);
    unpack8(h1[i], u);
    unpack8(dy[i], d);
#pragma unroll
    for (int j = 0; j < 8; j++) {
      const float gc = CLIP ? fminf(g[j], limit) : g[j];
      const float uc = CLIP ? fminf(fmaxf(u[j], -limit), limit) : u[j];
      const float s = 1.0f / (1.0f + expf(-a * gc));
      const bool g_in = !CLIP || g[j] <= limit, u_in = !CLIP || (u[j] >= -limit && u[j] <= limit);
      dg[j] = g_in ? d[j] * (uc + b) * s * (1.0f + a * gc * (1.0f - s)) : 0.f;
      du[j] = u_in ? d[j] * gc * s : 0.f;
    }
    dh0[i] = make_uint4(pack_bf16x2(dg[0], dg[1]), pack_bf16x2(dg[2], dg[3]), pack_bf16x2(dg[4], dg[5]), pack_bf16x2(dg[6], dg[7]));
    dh1[i] = make_uint4(pack_bf16x2(du[0], du[1]), pack_bf16x2(du[2], du[3]), pack_bf16x2(du[4], du[5]), pack_bf16x2(du[6], du[7]));
  }
}

// ---------------------------------------------------------------------------------------
// [G, K, N] -> [G, N, K] re-layout through a padded LDS tile.
// ---------------------------------------------------------------------------------------

template <typename T>
__global__ __launch_bounds__(256) void transpose_kernel(const T* __restrict__ in, int K, int N,
                                                        T* __restrict__ out) {
  __shared__ T tile[64][65];
  const size_t g = blockIdx.z;
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tx = threadIdx.x % 64, ty = threadIdx.x / 64;
  for (int i = ty; i < 64; i += 4) {
    int kk = k0 + i, nn = n0 + tx;
    if (kk < K && nn < N) tile[i][tx] = in[(g * K + kk) * N + nn];
  }
  __syncthreads();
  for (int i = ty; i < 64; i += 4) {
    int nn = n0 + i, kk = k0 + tx;
    if (kk < K && nn < N) out[(g * N + nn) * K + kk] = tile[tx][i];
  }
}

// 1-byte elements with K % 16 == 0 and N % 16 == 0 (the int8 / fp8 weights the quantised backward re-lays out on every
// step): a 128 x 128 tile goes through LDS with 16-byte loads along N and 16-byte stores along K, so that every request
// covers whole 128-byte lines on both sides; a lane gathers the 16 bytes of its output chunk with byte reads.  The chunk c
// of row k sits at slot c ^ (k / 16 % 8), which spreads the eight rows a store instruction's lanes read over the banks.
__global__ __launch_bounds__(256) void transpose8_kernel(const uint8_t* __restrict__ in, int K, int N, uint8_t* __restrict__ out) {
  __shared__ __attribute__((aligned(16))) uint8_t tile[128 * 128];
  const size_t g = blockIdx.z;
  const int k0 = blockIdx.y * 128, n0 = blockIdx.x * 128;
  const int tid = threadIdx.x;
  {
    const int c = tid % 8, r = tid / 8;
#pragma unroll
    for (int it = 0; it < 4; it++) {
      const int k = it * 32 + r;
      uint4 v = make_uint4(0, 0, 0, 0);
      if (k0 + k < K && n0 + c * 16 < N) v = *(const uint4*)(in + (g * K + k0 + k) * N + n0 + c * 16);
      *(uint4*)(tile + k * 128 + ((c ^ ((k >> 4) & 7)) << 4)) = v;
    }
  }
  __syncthreads();
  const int kc = tid % 8, nr = tid / 8;
  if (k0 + kc * 16 >= K) return;
#pragma unroll
  for (int it = 0; it < 4; it++) {
    const int n = it * 32 + nr;
    if (n0 + n >= N) continue;
    const uint8_t* src = tile + kc * 16 * 128 + (((n >> 4) ^ kc) << 4) + (n & 15);
    uint32_t w[4];
#pragma unroll
    for (int q = 0; q < 4; q++)
      w[q] = (uint32_t)src[(4 * q) * 128] | ((uint32_t)src[(4 * q + 1) * 128] << 8) | ((uint32_t)src[(4 * q + 2) * 128] << 16) |
             ((uint32_t)src[(4 * q + 3) * 128] << 24);
    *(uint4*)(out + (g * N + n0 + n) * K + k0 + kc * 16) = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// 2-byte elements with K % 8 == 0 and N % 8 == 0: 16-byte loads along N into LDS, then ds_read_b64_tr_b16 (the
// transposing LDS load: 16 lanes read a 4 x 16 block and lane L receives column L) twice per lane, which yields 8
// consecutive K values of one output row as one 16-byte store.
typedef short tr_v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) tr_v4s* tr_lds_ptr;

__global__ __launch_bounds__(256) void transpose16_kernel(const uint16_t* __restrict__ in, int K, int N,
                                                          uint16_t* __restrict__ out) {
  constexpr int kPitch = 64 * 2 + 16;  // bytes per LDS row
  __shared__ __attribute__((aligned(16))) uint8_t tile[64 * kPitch];
  const size_t g = blockIdx.z;
  const int k0 = blockIdx.y * 64, n0 = blockIdx.x * 64;
  const int tid = threadIdx.x;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int r = h * 32 + tid / 8, c8 = tid % 8;
    uint4 v = make_uint4(0, 0, 0, 0);
    if (k0 + r < K && n0 + c8 * 8 < N) v = *(const uint4*)(in + (g * K + k0 + r) * N + n0 + c8 * 8);
    *(uint4*)(tile + r * kPitch + c8 * 16) = v;
  }
  __syncthreads();
  const int s = tid % 16, grp = tid / 16;  // 16 lane groups
  const int n16 = grp % 4;
#pragma unroll
  for (int h = 0; h < 2; h++) {
    const int k8 = grp / 4 + h * 4;
    const uint8_t* p = tile + (k8 * 8 + s / 4) * kPitch + (n16 * 16 + 4 * (s % 4)) * 2;
    const tr_v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_lds_ptr)p);
    const tr_v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((tr_lds_ptr)(p + 4 * kPitch));
    const int n = n0 + n16 * 16 + s, k = k0 + k8 * 8;
    if (n < N && k < K) {
      typedef short v8s __attribute__((ext_vector_type(8)));
      const v8s v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
      *(uint4*)(out + (g * N + n) * K + k) = __builtin_bit_cast(uint4, v);
    }
  }
}

}  // namespace moe

using namespace moe;

extern "C" {

const char* moe_last_error(void) { return g_err; }
int moe_abi_version(void) { return 3; }

int moe_route_topk(const float* gate_logits, const float* pre_bias_logits, int T, int E, int k,
                   int mode, int norm_topk_prob, int weights_round_bf16,
                   float routed_scaling_factor, int n_routing_groups, int topk_routing_group,
                   float* topk_weights, int32_t* topk_idx, void* stream) {
  if (!gate_logits || !topk_weights || !topk_idx) return fail(MOE_ERR_INVALID_ARG, "route: NULL pointer");
  if (T < 0 || E <= 0 || k <= 0) return fail(MOE_ERR_INVALID_ARG, "route: bad sizes T=%d E=%d k=%d", T, E, k);
  if (E > kRouteMaxE || k > 16 || k > E) return fail(MOE_ERR_UNSUPPORTED, "route: need k<=16, k<=E<=512 (E=%d k=%d)", E, k);
  if (mode < MOE_ROUTE_SOFTMAX_TOPK || mode > MOE_ROUTE_SOFTMAX_ALL) return fail(MOE_ERR_INVALID_ARG, "route: bad mode %d", mode);
  if (mode == MOE_ROUTE_DEEPSEEK && !pre_bias_logits) return fail(MOE_ERR_INVALID_ARG, "route: DeepSeek mode needs pre_bias_logits");
  int ng = n_routing_groups > 0 ? n_routing_groups : 0;
  if (ng > 0) {
    if (mode != MOE_ROUTE_DEEPSEEK) return fail(MOE_ERR_INVALID_ARG, "route: routing groups need DeepSeek mode");
    if (ng > kWave || E % ng != 0 || E / ng < 2 || topk_routing_group <= 0 || topk_routing_group > ng)
      return fail(MOE_ERR_UNSUPPORTED, "route: bad routing groups %d/%d for E=%d", ng, topk_routing_group, E);
  }
  if (T == 0) return MOE_OK;
  route_topk_kernel<false><<<cdiv(T, kRouteWaves), kRouteWaves * kWave, 0, (hipStream_t)stream>>>(
      gate_logits, pre_bias_logits, T, E, k, mode, norm_topk_prob, weights_round_bf16,
      routed_scaling_factor, ng, topk_routing_group, topk_weights, topk_idx, GateEpilogue{});
  return check_launch("route_topk_kernel");
}

static int gate_k_splits(int T, int d, int E) {
  const int tiles = cdiv(T, 32) * cdiv(E, 32), nchunks = d / 64;
  int ks = 256 / tiles;
  ks = ks < 1 ? 1 : ks;
  const int cap = nchunks / 8 < 1 ? 1 : nchunks / 8;  // at least 8 chunks (2 per wave) per block
  ks = ks > cap ? cap : ks;
  return ks > 16 ? 16 : ks;
}

size_t moe_gate_route_workspace_bytes(int T, int d, int E) {
  if (T < 0 || d <= 0 || E <= 0) return 0;
  return (size_t)gate_k_splits(T, d, E) * T * E * sizeof(float) + 16;
}

int moe_gate_route(const void* x, const void* gate_kernel_terms, int num_terms, const float* gate_bias, int T, int d,
                   int E, int k, int score_func, int gate_round_bf16, int mode, int norm_topk_prob,
                   int weights_round_bf16, float routed_scaling_factor, int n_routing_groups, int topk_routing_group,
                   float* topk_weights, int32_t* topk_idx, float* gate_logits_out, float* pre_bias_logits_out,
                   void* workspace, size_t workspace_bytes, void* stream) {
  if (!x || !gate_kernel_terms || !topk_weights || !topk_idx || !workspace) return fail(MOE_ERR_INVALID_ARG, "gate_route: NULL pointer");
  if (T < 0 || d <= 0 || E <= 0 || k <= 0) return fail(MOE_ERR_INVALID_ARG, "gate_route: bad sizes T=%d d=%d E=%d k=%d", T, d, E, k);
  if (num_terms != 1 && num_terms != 3) return fail(MOE_ERR_INVALID_ARG, "gate_route: num_terms must be 1 or 3");
  if (d % 64 != 0 || E % 4 != 0) return fail(MOE_ERR_UNSUPPORTED, "gate_route: need d %% 64 == 0 and E %% 4 == 0 (d=%d E=%d)", d, E);
  if (E > kRouteMaxE || k > 16 || k > E) return fail(MOE_ERR_UNSUPPORTED, "gate_route: need k<=16, k<=E<=512 (E=%d k=%d)", E, k);
  if (score_func < 0 || score_func > 2) return fail(MOE_ERR_INVALID_ARG, "gate_route: bad score_func %d", score_func);
  if (mode < MOE_ROUTE_SOFTMAX_TOPK || mode > MOE_ROUTE_SOFTMAX_ALL) return fail(MOE_ERR_INVALID_ARG, "gate_route: bad mode %d", mode);
  int ng = n_routing_groups > 0 ? n_routing_groups : 0;
  if (ng > 0) {
    if (mode != MOE_ROUTE_DEEPSEEK) return fail(MOE_ERR_INVALID_ARG, "gate_route: routing groups need DeepSeek mode");
    if (ng > kWave || E % ng != 0 || E / ng < 2 || topk_routing_group <= 0 || topk_routing_group > ng)
      return fail(MOE_ERR_UNSUPPORTED, "gate_route: bad routing groups %d/%d for E=%d", ng, topk_routing_group, E);
  }
  if (workspace_bytes < moe_gate_route_workspace_bytes(T, d, E)) return fail(MOE_ERR_WORKSPACE, "gate_route: workspace too small");
  if (((uintptr_t)x | (uintptr_t)gate_kernel_terms | (uintptr_t)workspace) & 15) return fail(MOE_ERR_UNSUPPORTED, "gate_route: pointers must be 16-byte aligned");
  if (T == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const int ks = gate_k_splits(T, d, E);
  GateGemmParams gp;
  gp.x = (const uint16_t*)x; gp.wg = (const uint16_t*)gate_kernel_terms; gp.partial = (float*)workspace;
  gp.T = T; gp.d = d; gp.E = E; gp.S = num_terms; gp.chunks_per_block = cdiv(d / 64, ks);
  dim3 grid(cdiv(T, 32), cdiv(E, 32), ks);
  if (num_terms == 3)
    gate_gemm_kernel<3><<<grid, 256, 0, s>>>(gp);
  else
    gate_gemm_kernel<1><<<grid, 256, 0, s>>>(gp);
  GateEpilogue ge;
  ge.partials = (const float*)workspace; ge.bias = gate_bias; ge.logits_out = gate_logits_out; ge.pre_bias_out = pre_bias_logits_out;
  ge.num_partials = ks; ge.score_func = score_func; ge.round_bf16 = gate_round_bf16;
  route_topk_kernel<true><<<cdiv(T, kRouteWaves), kRouteWaves * kWave, 0, s>>>(
      nullptr, nullptr, T, E, k, mode, norm_topk_prob, weights_round_bf16, routed_scaling_factor, ng, topk_routing_group,
      topk_weights, topk_idx, ge);
  return check_launch("gate_route");
}

size_t moe_sort_workspace_bytes(int T, int k, int E) {
  if (T < 0 || k <= 0 || E <= 0) return 0;
  size_t M = (size_t)T * k;
  size_t nseg = (size_t)cdiv((int)M, kSortChunk) * kSortWaves;
  return (nseg * E + E) * sizeof(int32_t) + 256;
}

static int sort_impl(const int32_t* topk_idx, int T, int k, int E, int roll_to_expert_id, const int32_t* roll_dev, int32_t* perm,
                     int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                     void* workspace, size_t workspace_bytes, const SortMapArgs& mp, bool* mapped, void* stream) {
  if (!topk_idx || !perm || !group_sizes || !workspace) return fail(MOE_ERR_INVALID_ARG, "sort: NULL pointer");
  if (T < 0 || k <= 0 || E <= 0) return fail(MOE_ERR_INVALID_ARG, "sort: bad sizes");
  if (E > kSortMaxE) return fail(MOE_ERR_UNSUPPORTED, "sort: E=%d > %d", E, kSortMaxE);
  if (roll_to_expert_id < 0 || roll_to_expert_id >= E) return fail(MOE_ERR_INVALID_ARG, "sort: roll_to_expert_id %d outside [0, %d)", roll_to_expert_id, E);
  const int roll = roll_to_expert_id;
  if ((long long)T * k > INT_MAX / 2) return fail(MOE_ERR_UNSUPPORTED, "sort: T*k too large");
  if (workspace_bytes < moe_sort_workspace_bytes(T, k, E)) return fail(MOE_ERR_WORKSPACE, "sort: workspace too small");
  const int M = T * k;
  const int nblk = cdiv(M, kSortChunk);
  const int nseg = nblk * kSortWaves;
  int32_t* seg_hist = (int32_t*)workspace;
  hipStream_t s = (hipStream_t)stream;
  int ebits = 0;
  while ((1 << ebits) < E) ebits++;
  if (nblk <= 1) {  // also M == 0: group_sizes are all zero
    sort_small_kernel<kSortWaves><<<1, kSortWaves * kWave, 0, s>>>(topk_idx, M, E, roll, roll_dev, ebits, group_sizes, perm, inv_perm, sorted_experts, mp);
    *mapped = mp.tiles != nullptr;
    if (!*mapped) note_group_sizes_rewritten(group_sizes);
    return check_launch("sort_by_expert");
  }
  if (nblk <= 4) {  // up to 4096 entries: still one launch, with 16 waves
    sort_small_kernel<4 * kSortWaves><<<1, 4 * kSortWaves * kWave, 0, s>>>(topk_idx, M, E, roll, roll_dev, ebits, group_sizes, perm, inv_perm, sorted_experts, mp);
    *mapped = mp.tiles != nullptr;
    if (!*mapped) note_group_sizes_rewritten(group_sizes);
    return check_launch("sort_by_expert");
  }
  // (nothing is mapped from here on: a tile list recorded over this group_sizes buffer no longer describes it)
  note_group_sizes_rewritten(group_sizes);
  if (nblk > 0) sort_hist_kernel<<<nblk, kSortWaves * kWave, 0, s>>>(topk_idx, M, E, roll, roll_dev, seg_hist);
  sort_scan_kernel<<<cdiv(E, kSortWaves), kSortWaves * kWave, 0, s>>>(seg_hist, nseg, E, group_sizes);
  if (nblk > 0)
    sort_scatter_kernel<<<nblk, kSortWaves * kWave, 0, s>>>(topk_idx, M, E, roll, roll_dev, ebits, seg_hist, group_sizes,
                                                          perm, inv_perm, sorted_experts);
  return check_launch("sort_by_expert");
}

int moe_sort_by_expert_rolled(const int32_t* topk_idx, int T, int k, int E, int roll_to_expert_id, int32_t* perm,
                              int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                              void* workspace, size_t workspace_bytes, void* stream) {
  bool mapped = false;
  return sort_impl(topk_idx, T, k, E, roll_to_expert_id, nullptr, perm, inv_perm, group_sizes, sorted_experts, workspace, workspace_bytes,
                   SortMapArgs{nullptr, nullptr, 0, 0, 0, 0}, &mapped, stream);
}

int moe_sort_by_expert_rolled_dev(const int32_t* topk_idx, int T, int k, int E, const int32_t* roll_to_expert_id_dev, int32_t* perm,
                                  int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                                  void* workspace, size_t workspace_bytes, void* stream) {
  if (!roll_to_expert_id_dev) return fail(MOE_ERR_INVALID_ARG, "sort: NULL roll_to_expert_id_dev");
  bool mapped = false;
  return sort_impl(topk_idx, T, k, E, 0, roll_to_expert_id_dev, perm, inv_perm, group_sizes, sorted_experts, workspace, workspace_bytes,
                   SortMapArgs{nullptr, nullptr, 0, 0, 0, 0}, &mapped, stream);
}

int moe_sort_by_expert_mapped(const int32_t* topk_idx, int T, int k, int E, int roll_to_expert_id, int32_t* perm,
                              int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                              void* workspace, size_t workspace_bytes, int tile_rows, int num_groups_local, int group_offset,
                              int keep_other_rows, void* gmm_workspace, size_t gmm_workspace_bytes, void* stream) {
  if (!gmm_workspace) return fail(MOE_ERR_INVALID_ARG, "sort: NULL gmm_workspace");
  if (tile_rows <= 0 || num_groups_local <= 0 || group_offset < 0) return fail(MOE_ERR_INVALID_ARG, "sort: bad tile list arguments");
  const long long M = (long long)T * k;
  if (T >= 0 && k > 0 && M <= INT_MAX / 2 && gmm_workspace_bytes < moe_gmm_workspace_bytes((int)M, E))
    return fail(MOE_ERR_WORKSPACE, "sort: gmm_workspace too small");
  const int zero_fill = keep_other_rows ? 0 : 1;
  const SortMapArgs mp = {(TileInfo*)((uint8_t*)gmm_workspace + 16), (int32_t*)gmm_workspace, num_groups_local, group_offset, tile_rows, zero_fill};
  bool mapped = false;
  const int st = sort_impl(topk_idx, T, k, E, roll_to_expert_id, nullptr, perm, inv_perm, group_sizes, sorted_experts, workspace, workspace_bytes, mp,
                           &mapped, stream);
  if (st == MOE_OK && mapped) note_tile_map_built(gmm_workspace, group_sizes, (int)M, E, group_offset, num_groups_local, tile_rows, zero_fill);
  return st;
}

int moe_route_sort_mapped(const float* gate_logits, const float* pre_bias_logits, int T, int E, int k,
                          int mode, int norm_topk_prob, int weights_round_bf16, float routed_scaling_factor,
                          int n_routing_groups, int topk_routing_group, float* topk_weights, int32_t* topk_idx,
                          int roll_to_expert_id, int32_t* perm, int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                          void* workspace, size_t workspace_bytes, int tile_rows, int num_groups_local, int group_offset,
                          int keep_other_rows, void* gmm_workspace, size_t gmm_workspace_bytes, void* stream) {
  const long long M = (long long)T * k;
  // one launch for both when one block has a wave per token; two launches otherwise (the arguments are checked there)
  const bool one = T > 0 && T <= 4 * kSortWaves && k > 0 && E > 0 && E <= kSortMaxE && E <= kRouteMaxE && k <= 16 && k <= E && M <= kSortChunk && gate_logits && topk_weights &&
                   topk_idx && perm && group_sizes && workspace && gmm_workspace && roll_to_expert_id >= 0 && roll_to_expert_id < E &&
                   mode >= MOE_ROUTE_SOFTMAX_TOPK && mode <= MOE_ROUTE_SOFTMAX_ALL && (mode != MOE_ROUTE_DEEPSEEK || pre_bias_logits) &&
                   n_routing_groups <= 0 && tile_rows > 0 && num_groups_local > 0 && group_offset >= 0 &&
                   workspace_bytes >= moe_sort_workspace_bytes(T, k, E) && gmm_workspace_bytes >= moe_gmm_workspace_bytes((int)M, E);
  if (!one) {
    if (int st = moe_route_topk(gate_logits, pre_bias_logits, T, E, k, mode, norm_topk_prob, weights_round_bf16, routed_scaling_factor,
                                n_routing_groups, topk_routing_group, topk_weights, topk_idx, stream))
      return st;
    return moe_sort_by_expert_mapped(topk_idx, T, k, E, roll_to_expert_id, perm, inv_perm, group_sizes, sorted_experts, workspace, workspace_bytes,
                                     tile_rows, num_groups_local, group_offset, keep_other_rows, gmm_workspace, gmm_workspace_bytes, stream);
  }
  int ebits = 0;
  while ((1 << ebits) < E) ebits++;
  const int zero_fill = keep_other_rows ? 0 : 1;
  const SortMapArgs mp = {(TileInfo*)((uint8_t*)gmm_workspace + 16), (int32_t*)gmm_workspace, num_groups_local, group_offset, tile_rows, zero_fill};
  const RouteArgs r = {gate_logits, pre_bias_logits, T, E, k, mode, norm_topk_prob, weights_round_bf16, routed_scaling_factor, 0, 0, topk_weights, topk_idx};
  if (T <= kSortWaves)
    route_sort_small_kernel<kSortWaves><<<1, kSortWaves * kWave, 0, (hipStream_t)stream>>>(r, roll_to_expert_id, ebits, group_sizes, perm, inv_perm,
                                                                                            sorted_experts, mp);
  else
    route_sort_small_kernel<4 * kSortWaves><<<1, 4 * kSortWaves * kWave, 0, (hipStream_t)stream>>>(r, roll_to_expert_id, ebits, group_sizes, perm,
                                                                                                    inv_perm, sorted_experts, mp);
  if (int st = check_launch("route_sort_small_kernel")) return st;
  note_tile_map_built(gmm_workspace, group_sizes, (int)M, E, group_offset, num_groups_local, tile_rows, zero_fill);
  return MOE_OK;
}

int moe_sort_by_expert(const int32_t* topk_idx, int T, int k, int E, int32_t* perm,
                       int32_t* inv_perm, int32_t* group_sizes, int32_t* sorted_experts,
                       void* workspace, size_t workspace_bytes, void* stream) {
  return moe_sort_by_expert_rolled(topk_idx, T, k, E, 0, perm, inv_perm, group_sizes, sorted_experts, workspace, workspace_bytes, stream);
}

int moe_gather_rows(const void* x, const int32_t* row_idx, int idx_div, int R_in, int R_out, int d,
                    int out_dtype, int block_k, int rule, const float* static_scale, const float* row_weight,
                    const int32_t* row_range, void* out, float* scale, void* stream) {
  if (!x || !out) return fail(MOE_ERR_INVALID_ARG, "gather: NULL pointer");
  if (R_in <= 0 || R_out < 0 || d <= 0 || idx_div <= 0 || block_k < 0) return fail(MOE_ERR_INVALID_ARG, "gather: bad sizes");
  if (!row_idx && R_out > R_in) return fail(MOE_ERR_INVALID_ARG, "gather: R_out > R_in without row_idx");
  if (d % 8 != 0 || d > kGqThreads * kGqMaxChunks * 8) return fail(MOE_ERR_UNSUPPORTED, "gather: need d%%8==0 and d<=16384 (d=%d)", d);
  if (rule != MOE_QUANT_RINT_DIV && rule != MOE_QUANT_V2) return fail(MOE_ERR_INVALID_ARG, "gather: bad rule %d", rule);
  if (R_out == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const uint4* xs = (const uint4*)x;
  QuantCfg qc;
  qc.rule = rule; qc.block_lanes = 0; qc.nkb = 1; qc.static_scale = nullptr; qc.row_weight = row_weight; qc.row_range = row_range;
  if (out_dtype == MOE_BF16) {
    gather_rows_kernel<GQ_COPY><<<R_out, kGqThreads, 0, s>>>(xs, row_idx, idx_div, R_in, d, out, scale, qc);
    return check_launch("gather_rows_kernel");
  }
  if (out_dtype != MOE_INT8 && out_dtype != MOE_FP8_E4M3) return fail(MOE_ERR_UNSUPPORTED, "gather: out_dtype %d", out_dtype);
  if (static_scale) {
    qc.static_scale = static_scale;  // one scale for the tensor: block_k is not used and `scale` is not written
  } else {
    if (!scale) return fail(MOE_ERR_INVALID_ARG, "gather: quantised output needs a scale buffer");
    if (block_k != 0 && block_k != 128 && block_k != 256 && block_k != 512)
      return fail(MOE_ERR_UNSUPPORTED, "gather: block_k must be 0 (one scale per row), 128, 256 or 512 (block_k=%d)", block_k);
    qc.block_lanes = block_k / 8;
    qc.nkb = block_k ? cdiv(d, block_k) : 1;
  }
  if (out_dtype == MOE_INT8)
    gather_rows_kernel<GQ_INT8><<<R_out, kGqThreads, 0, s>>>(xs, row_idx, idx_div, R_in, d, out, scale, qc);
  else
    gather_rows_kernel<GQ_FP8><<<R_out, kGqThreads, 0, s>>>(xs, row_idx, idx_div, R_in, d, out, scale, qc);
  return check_launch("gather_rows_kernel");
}

int moe_unpermute_combine(const void* y, const int32_t* perm, const int32_t* inv_perm,
                          const float* weights, const uint8_t* valid_rows_mask, int T, int k, int d, void* out,
                          void* workspace, size_t workspace_bytes, void* stream) {
  if (!y || !out || (!perm && !inv_perm)) return fail(MOE_ERR_INVALID_ARG, "combine: NULL pointer");
  if (T < 0 || k <= 0 || d <= 0) return fail(MOE_ERR_INVALID_ARG, "combine: bad sizes");
  if (k > kCombineMaxK || d % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "combine: need k<=16, d%%8==0");
  if (T == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const int M = T * k;
  if (!inv_perm) {
    if (!workspace || workspace_bytes < (size_t)M * sizeof(int32_t)) return fail(MOE_ERR_WORKSPACE, "combine: workspace too small");
    invert_perm_kernel<<<cdiv(M, 256), 256, 0, s>>>(perm, M, (int32_t*)workspace);
    inv_perm = (const int32_t*)workspace;
  }
  const int splits = T < 2048 ? std::min(cdiv(d / 8, 256), 8) : 1;
  combine_kernel<<<dim3(T, splits), 256, 0, s>>>((const uint4*)y, inv_perm, weights, valid_rows_mask, k, d, (uint4*)out);
  return check_launch("combine_kernel");
}

int moe_unpermute_combine_bwd(const void* dout, const void* y, const int32_t* inv_perm, const float* weights,
                              const uint8_t* valid_rows_mask, int T, int k, int d, void* dy, float* dweights,
                              void* stream) {
  if (!dout || !inv_perm || !dy || (dweights && !y)) return fail(MOE_ERR_INVALID_ARG, "combine_bwd: NULL pointer");
  if (T < 0 || k <= 0 || d <= 0) return fail(MOE_ERR_INVALID_ARG, "combine_bwd: bad sizes");
  if (k > kCombineMaxK || d % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "combine_bwd: need k<=16, d%%8==0");
  if (T == 0) return MOE_OK;
  combine_bwd_kernel<<<T, 256, 0, (hipStream_t)stream>>>((const uint4*)dout, (const uint4*)y, inv_perm, weights,
                                                         valid_rows_mask, k, d, (uint4*)dy, dweights);
  return check_launch("combine_bwd_kernel");
}

int moe_glu_act(const void* h0, const void* h1, size_t n, int act, float act_limit, void* out, void* stream) {
  if (!h0 || !h1 || !out) return fail(MOE_ERR_INVALID_ARG, "glu_act: NULL pointer");
  if (act < MOE_ACT_SILU || act > MOE_ACT_SILU_CLIP) return fail(MOE_ERR_INVALID_ARG, "glu_act: bad act %d", act);
  if (n % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "glu_act: element count must be a multiple of 8");
  if (n == 0) return MOE_OK;
  const size_t nvec = n / 8;
  const unsigned blocks = (unsigned)(nvec / 256 + 1 < 8192 ? nvec / 256 + 1 : 8192);
  hipStream_t s = (hipStream_t)stream;
  if (act == MOE_ACT_SILU) glu_fwd_kernel<MOE_ACT_SILU><<<blocks, 256, 0, s>>>((const uint4*)h0, (const uint4*)h1, nvec, act_limit, (uint4*)out);
  else if (act == MOE_ACT_SWIGLUOAI) glu_fwd_kernel<MOE_ACT_SWIGLUOAI><<<blocks, 256, 0, s>>>((const uint4*)h0, (const uint4*)h1, nvec, act_limit, (uint4*)out);
  else glu_fwd_kernel<MOE_ACT_SILU_CLIP><<<blocks, 256, 0, s>>>((const uint4*)h0, (const uint4*)h1, nvec, act_limit, (uint4*)out);
  return check_launch("glu_fwd_kernel");
}

int moe_glu_act_bwd(const void* h0, const void* h1, const void* dout, size_t n, int act, float act_limit, void* dh0,
                    void* dh1, void* stream) {
  if (!h0 || !h1 || !dout || !dh0 || !dh1) return fail(MOE_ERR_INVALID_ARG, "glu_act_bwd: NULL pointer");
  if (act < MOE_ACT_SILU || act > MOE_ACT_SILU_CLIP) return fail(MOE_ERR_INVALID_ARG, "glu_act_bwd: bad act %d", act);
  if (n % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "glu_act_bwd: element count must be a multiple of 8");
  if (n == 0) return MOE_OK;
  const size_t nvec = n / 8;
  const unsigned blocks = (unsigned)(nvec / 256 + 1 < 8192 ? nvec / 256 + 1 : 8192);
  hipStream_t s = (hipStream_t)stream;
#define MOE_GLU_BWD(A) glu_bwd_kernel<A><<<blocks, 256, 0, s>>>((const uint4*)h0, (const uint4*)h1, (const uint4*)dout, nvec, act_limit, (uint4*)dh0, (uint4*)dh1)
  if (act == MOE_ACT_SILU) MOE_GLU_BWD(MOE_ACT_SILU);
  else if (act == MOE_ACT_SWIGLUOAI) MOE_GLU_BWD(MOE_ACT_SWIGLUOAI);
  else MOE_GLU_BWD(MOE_ACT_SILU_CLIP);
#undef MOE_GLU_BWD
  return check_launch("glu_bwd_kernel");
}

int moe_transpose_rhs(const void* rhs_gkn, int G, int K, int N, int elem_bytes, void* rhs_gnk,
                      void* stream) {
  if (!rhs_gkn || !rhs_gnk) return fail(MOE_ERR_INVALID_ARG, "transpose: NULL pointer");
  if (G <= 0 || K <= 0 || N <= 0) return fail(MOE_ERR_INVALID_ARG, "transpose: bad sizes");
  if (G > 65535 || cdiv(K, 64) > 65535) return fail(MOE_ERR_UNSUPPORTED, "transpose: grid too large");
  dim3 grid(cdiv(N, 64), cdiv(K, 64), G);
  hipStream_t s = (hipStream_t)stream;
  if (elem_bytes == 1 && K % 16 == 0 && N % 16 == 0 && (((uintptr_t)rhs_gkn | (uintptr_t)rhs_gnk) & 15) == 0)
    transpose8_kernel<<<dim3(cdiv(N, 128), cdiv(K, 128), G), 256, 0, s>>>((const uint8_t*)rhs_gkn, K, N, (uint8_t*)rhs_gnk);
  else if (elem_bytes == 1)
    transpose_kernel<uint8_t><<<grid, 256, 0, s>>>((const uint8_t*)rhs_gkn, K, N, (uint8_t*)rhs_gnk);
  else if (elem_bytes == 2 && K % 8 == 0 && N % 8 == 0 && (((uintptr_t)rhs_gkn | (uintptr_t)rhs_gnk) & 15) == 0)
    transpose16_kernel<<<grid, 256, 0, s>>>((const uint16_t*)rhs_gkn, K, N, (uint16_t*)rhs_gnk);
  else if (elem_bytes == 2)
    transpose_kernel<uint16_t><<<grid, 256, 0, s>>>((const uint16_t*)rhs_gkn, K, N, (uint16_t*)rhs_gnk);
  else
    return fail(MOE_ERR_UNSUPPORTED, "transpose: elem_bytes %d", elem_bytes);
  return check_launch("transpose_kernel");
}

}  // extern "C"
