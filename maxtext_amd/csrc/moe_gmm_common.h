// Shared pieces of the grouped-matmul kernels: the m-tile list, the parameter blocks, the epilogue, and the
// launchers each translation unit exports to the dispatcher (moe_gmm.hip).
#pragma once

#include <type_traits>

#include "moe_common.h"

namespace moe {

struct TileInfo {
  int32_t group;  // local group id, or -1: write zeros
  int32_t row0;
  int32_t nrows;
  int32_t pad;
};

// workspace: int32 header[4] (header[0] = number of tiles) | TileInfo tiles[max_tiles]
static inline int max_tiles_for(int M, int G, int bm) { return cdiv(M, bm) + G + 1; }

// Exclusive prefix sum over one value per thread of a THREADS-wide block; *total = the block's sum.  Each wave scans its
// values with lane shuffles, the waves' totals meet in s_buf: three barriers whatever the block's width.
template <int THREADS>
__device__ __forceinline__ int block_exclusive_scan(int v, int* s_buf, int* total) {
  static_assert(THREADS % kWave == 0, "whole waves");
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  int incl = v;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int t = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += t;
  }
  __syncthreads();  // (s_buf may still be read by the caller's previous use)
  if (lane == kWave - 1) s_buf[wave] = incl;
  __syncthreads();
  int base = 0, sum = 0;
#pragma unroll
  for (int w = 0; w < THREADS / kWave; w++) {
    const int c = s_buf[w];
    base += w < wave ? c : 0;
    sum += c;
  }
  *total = sum;
  __syncthreads();
  return base + incl - v;
}

// group_sizes (device) -> the list of (group, first row, rows) m-tiles of height BM that never straddle a group boundary,
// plus zero-fill tiles for the rows of groups held elsewhere and the rows past the groups' total; header[0] = tile count.
// One block of THREADS threads; s_buf holds THREADS ints.
template <int THREADS>
__device__ __forceinline__ void build_tile_map(const int32_t* __restrict__ group_sizes, int G_total, int group_offset, int G_local, int M,
                                               int BM, int zero_fill, int32_t* __restrict__ header, TileInfo* __restrict__ tiles, int* s_buf) {
  const int tid = threadIdx.x;
  const int per = (G_total + THREADS - 1) / THREADS;
  const int g0 = min(tid * per, G_total), g1 = min(g0 + per, G_total);
  long long rows = 0;
  for (int g = g0; g < g1; g++) rows += max(group_sizes[g], 0);
  int total_rows;
  int row_prefix = block_exclusive_scan<THREADS>((int)min(rows, (long long)M), s_buf, &total_rows);
  // clipped extents (reference_gmm: end = min(start + size, m)) and tile counts
  int ntiles = 0;
  {
    long long start = row_prefix;
    for (int g = g0; g < g1; g++) {
      long long end = start + max(group_sizes[g], 0);
      int s = (int)min(start, (long long)M), e = (int)min(end, (long long)M);
      const int local = g - group_offset;
      // rows of groups held elsewhere get zero-fill tiles, or none at all when the caller keeps what `out` holds
      if (zero_fill || (local >= 0 && local < G_local)) ntiles += (e - s + BM - 1) / BM;
      start = end;
    }
  }
  int total_tiles;
  int tile_prefix = block_exclusive_scan<THREADS>(ntiles, s_buf, &total_tiles);
  {
    long long start = row_prefix;
    int ti = tile_prefix;
    for (int g = g0; g < g1; g++) {
      long long end = start + max(group_sizes[g], 0);
      int s = (int)min(start, (long long)M), e = (int)min(end, (long long)M);
      int local = g - group_offset;
      int kind = (local >= 0 && local < G_local) ? local : -1;
      for (int r = s; r < e && (zero_fill || kind >= 0); r += BM) {
        TileInfo t;
        t.group = kind;
        t.row0 = r;
        t.nrows = min(BM, e - r);
        t.pad = 0;
        tiles[ti++] = t;
      }
      start = end;
    }
  }
  const int covered = min(total_rows, M);
  const int tail = zero_fill ? (M - covered + BM - 1) / BM : 0;
  for (int i = tid; i < tail; i += THREADS) {
    TileInfo t;
    t.group = -1;
    t.row0 = covered + i * BM;
    t.nrows = min(BM, M - t.row0);
    t.pad = 0;
    tiles[total_tiles + i] = t;
  }
  if (tid == 0) header[0] = total_tiles + tail;
}

// Tells moe_gmm that `workspace` holds the tile list of these groups at height bm (built by another entry point of the
// library), so that a call flagged MOE_GMM_SAME_GROUPS can use it.
void note_tile_map_built(const void* workspace, const int32_t* group_sizes, int M, int G_total, int group_offset, int G_local, int bm,
                         int zero_fill);

// Tells moe_gmm that a library entry has written new values into `group_sizes` without building a tile list: the
// record of a list over that buffer's old contents is dropped, so that a following call flagged MOE_GMM_SAME_GROUPS
// maps again instead of multiplying the new rows with the old group boundaries.
void note_group_sizes_rewritten(const int32_t* group_sizes);

// m-tiles per super-row of the persistent kernels' tile order (the tiles an XCD works on at a time are a patch of one
// super-row's m-tiles x a few n-tiles): as many as a group of average size plus three standard deviations of a
// multinomial draw has, so that a patch mostly stays inside one group and shares its weight panels; 8 for larger groups.
// Measured against 8 everywhere: Mixtral (8 or 9 tiles per group) first projection 1.81 -> 1.77 ms with 9, Qwen3 (4 or 5)
// second projection 0.56 -> 0.54 ms with 5.
static inline int default_super_row(int M, int G, int bm) {
  const double rows = (double)M / (G > 0 ? G : 1);
  const int t = (int)((rows + 3.0 * __builtin_sqrt(rows) + bm - 1) / bm);
  return t > 9 ? 8 : t < 4 ? 4 : t;
}

enum { OP_BF16 = 0, OP_I8 = 1, OP_F8 = 2 };      // MFMA operand type (= LDS element type)
enum { BSRC_SAME = 0, BSRC_I8 = 1, BSRC_I4 = 2, BSRC_MX4 = 3 };  // weight format in HBM

// Options every kernel family honours: activation rows read through an index (the permute of moe.py:956-959 fused into
// the matmul: row r of the product reads lhs row row_idx[r] / idx_div, and that row's scales), a factor per output row
// applied after the activation (routing weights before wo, models/deepseek_batchsplit_fp8.py:1049), f32 output.
struct RowOpts {
  const int32_t* row_idx;  // [M] or NULL
  int idx_div;
  int lhs_rows;            // rows of lhs; indices are clamped into [0, lhs_rows)
  int out_f32;             // out is [M, N] f32 instead of bf16
  const float* row_scale;  // [M] or NULL
};

__device__ __forceinline__ int lhs_row_of(const RowOpts& o, int r) {
  if (!o.row_idx) return r;
  const int s = o.row_idx[r] / o.idx_div;
  return min(max(s, 0), o.lhs_rows - 1);
}

// The same for a batch of rows: one uniform branch, the index loads issued back to back (a branch per row would put a
// full memory round trip between consecutive loads).
template <int NR>
__device__ __forceinline__ void lhs_rows_of(const RowOpts& o, int (&r)[NR]) {
  if (o.row_idx) {
    int s[NR];
#pragma unroll
    for (int i = 0; i < NR; i++) s[i] = o.row_idx[r[i]];
#pragma unroll
    for (int i = 0; i < NR; i++) r[i] = min(max(s[i] / o.idx_div, 0), o.lhs_rows - 1);
  }
}

// Four consecutive output values of one row: multiplied by the row's factor, then stored as bf16 (8 bytes) or f32.
__device__ __forceinline__ void store_out4(void* out, const RowOpts& o, size_t row, int N, int n, float (&v)[4]) {
  if (o.row_scale) {
    // the reference multiplies the finished result of the output type (models/deepseek_batchsplit_fp8.py:1048-1049):
    // a bf16 result is rounded before the multiplication and again after it
    const float w = o.row_scale[row];
#pragma unroll
    for (int r = 0; r < 4; r++) v[r] = (o.out_f32 ? v[r] : round_bf16_fn(v[r])) * w;
  }
  if (o.out_f32) {
    *(float4*)((float*)out + row * N + n) = make_float4(v[0], v[1], v[2], v[3]);
  } else {
    *(uint2*)((uint16_t*)out + row * N + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
  }
}

// Zeros for the `width` channels from n0 on of a tile's rows (rows of no local group).
__device__ __forceinline__ void zero_fill_tile(void* out, const RowOpts& o, int row0, int nrows, int n0, int width, int N, int tid,
                                               int nthreads) {
  const int qpr = width / 4;
  for (int i = tid; i < nrows * qpr; i += nthreads) {
    const int r = i / qpr, c = n0 + (i % qpr) * 4;
    if (c >= N) continue;
    if (o.out_f32)
      *(float4*)((float*)out + (size_t)(row0 + r) * N + c) = make_float4(0.f, 0.f, 0.f, 0.f);
    else
      *(uint2*)((uint16_t*)out + (size_t)(row0 + r) * N + c) = make_uint2(0, 0);
  }
}

struct TiledParams {
  const uint8_t* lhs;        // [M, K] elements of the MFMA operand type
  const float* lhs_scale;    // epilogue scale of the activations: [M] (stride 1) or one value (stride 0), or NULL
  const uint8_t* rhs;        // [G, N, K] (INT4: K/2 bytes per row)
  const uint8_t* rhs_up;     // same, or NULL
  const void* rhs_scale;     // f32 [G, N] (per channel) | bf16 [G, N, nkg] (INT4) | e8m0 bytes [G, N, K/32] (MXFP4)
  const void* rhs_up_scale;  //   (f32 per channel: element (g, n) at g * rhs_scale_gstride + n * rhs_scale_nstride)
  const float* rhs_bias;     // [G, N] f32 or NULL, added before the activation
  const float* rhs_up_bias;
  const uint16_t* partial_sum;     // [M, N] bf16 or NULL, added like the bias
  const uint16_t* partial_sum_up;
  const int32_t* header;
  const TileInfo* tiles;
  void* out;  // [M, N] bf16 (f32 with ro.out_f32)
  int M, K, N;
  int max_m_tiles, tiles_n;
  int act;
  float act_limit;
  int tune;  // > 0: m-tiles per raster super-row of the persistent kernel (tuning aid; 0 = default)
  int i4_group;  // values of K per int4 scale: 128 or 32
  int lhs_scale_stride;   // 1: one epilogue scale per row; 0: one for the tensor (static per-tensor scale)
  int rhs_scale_gstride;  // N: scales per expert; 0: one set shared by all experts ([1, 1, n], ops.py:250-260)
  int rhs_scale_nstride;  // 1: per output channel; 0: one per expert / tensor
  // K-block scales applied to the partial sums (block-scaled kernel; gmm_v2's layout): lhs_bs [M, lhs_nb] with one value
  // per lhs_qb values of K, rhs_bs [G, rhs_nb, N] (element (g, b, n) at g * rhs_bs_gstride + b * N + n) per rhs_qb values.
  // A side whose count is 1 has its scale in the epilogue fields above instead and a NULL pointer here.
  const float* lhs_bs;
  const float* rhs_bs;
  const float* rhs_up_bs;
  int lhs_nb, lhs_qb, rhs_nb, rhs_qb, rhs_bs_gstride;
  // weight-only int8 / int4 with K-major block scales [G, nb, N] (f32), multiplied in while the weights are widened
  int wq_kmajor;
  RowOpts ro;
};

__device__ __forceinline__ uint32_t i8x2_to_bf16x2(int lo, int hi) {
  // |value| <= 128 is exact in bf16, so truncating the f32 is the conversion
  return (__float_as_uint((float)lo) >> 16) | (__float_as_uint((float)hi) & 0xffff0000u);
}

// Bias of 4 consecutive output channels of one group (zeros without a bias).
__device__ __forceinline__ void load_bias4(const float* bias, int group, int N, int n, float (&b)[4]) {
  b[0] = b[1] = b[2] = b[3] = 0.f;
  if (bias) {
    const float4 v = *(const float4*)(bias + (size_t)group * N + n);
    b[0] = v.x; b[1] = v.y; b[2] = v.z; b[3] = v.w;
  }
}

// b += 4 consecutive bf16 values of row `row` of a [M, N] partial-sum matrix (nothing without one).
__device__ __forceinline__ void add_partial4(const uint16_t* ps, size_t row, int N, int n, float (&b)[4]) {
  if (ps) {
    const uint2 v = *(const uint2*)(ps + row * N + n);
    b[0] += bf16_bits_to_f32((uint16_t)(v.x & 0xffff));
    b[1] += bf16_bits_to_f32((uint16_t)(v.x >> 16));
    b[2] += bf16_bits_to_f32((uint16_t)(v.y & 0xffff));
    b[3] += bf16_bits_to_f32((uint16_t)(v.y >> 16));
  }
}

// Per-lane scales of the epilogue, fetched before the K loop so their latency hides behind it.  With
// weights as the MFMA "A" operand a lane owns row (lane % 32) of each 32-row tile and, per accumulator
// quad q, the 4 consecutive output channels 8*q + 4*(lane / 32) .. +3 of each 32-channel tile.  With the
// 16 x 16 instructions (MI = 16) it owns row (lane % 16) of each 16-row tile and the one quad of channels
// 4*(lane / 16) .. +3 of each 16-channel tile (only entry [.][0] of sg / su is used).
template <int MI>
__device__ __forceinline__ int epilogue_channel(int j, int q, int lane) {
  return MI == 32 ? j * 32 + 8 * q + 4 * (lane / 32) : j * 16 + 4 * (lane / 16);
}

template <int TM, int NT_OUT, bool GLU>
struct EpilogueScales {
  float sa[TM];
  float4 sg[NT_OUT][4], su[NT_OUT][4];
};

template <int TM, int NT_OUT, bool GLU, bool CHANNEL_SCALES, int MI = 32>
__device__ __forceinline__ void load_epilogue_scales(EpilogueScales<TM, NT_OUT, GLU>& e, const TiledParams& p, const TileInfo& tile,
                                                     int row_base, int n_base, int lane) {
  // every decision is uniform and taken once, so that the loads of a kind go out back to back
  const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
#pragma unroll
  for (int i = 0; i < TM; i++) e.sa[i] = 1.0f;
  if (p.lhs_scale) {
    int rows[TM];
#pragma unroll
    for (int i = 0; i < TM; i++) {
      const int lr = row_base + i * MI + (lane % MI);
      rows[i] = tile.row0 + (lr < tile.nrows ? lr : 0);
    }
    lhs_rows_of<TM>(p.ro, rows);
#pragma unroll
    for (int i = 0; i < TM; i++) e.sa[i] = p.lhs_scale[(size_t)rows[i] * p.lhs_scale_stride];
  }
#pragma unroll
  for (int j = 0; j < NT_OUT; j++)
#pragma unroll
    for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
      e.sg[j][q] = one;
      e.su[j][q] = one;
    }
  if (CHANNEL_SCALES && p.rhs_scale && !p.wq_kmajor) {  // (K-major block scales went in with the weights)
    const float* sg = (const float*)p.rhs_scale + (size_t)tile.group * p.rhs_scale_gstride;
    const float* su = GLU ? (const float*)p.rhs_up_scale + (size_t)tile.group * p.rhs_scale_gstride : nullptr;
    if (p.rhs_scale_nstride) {
#pragma unroll
      for (int j = 0; j < NT_OUT; j++)
#pragma unroll
        for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
          // channels past N (the last n-tile of a ragged N) read the scales of channel N - 4: they are never stored
          const int n = min(n_base + epilogue_channel<MI>(j, q, lane), p.N - 4);
          e.sg[j][q] = *(const float4*)(sg + n);
          if (GLU) e.su[j][q] = *(const float4*)(su + n);
        }
    } else {
      const float g1 = sg[0], u1 = GLU ? su[0] : 1.0f;
#pragma unroll
      for (int j = 0; j < NT_OUT; j++)
#pragma unroll
        for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
          e.sg[j][q] = make_float4(g1, g1, g1, g1);
          e.su[j][q] = make_float4(u1, u1, u1, u1);
        }
    }
  }
}

// Writes a wave's results.  The MFMA leaves lane l with 4 consecutive channels of row l % MI: 8-byte stores, neighbouring
// lanes in different rows; the plain bf16 case pairs tiles and stores 16 bytes per lane (below).  (Passing each row tile
// through LDS so that consecutive lanes store consecutive 16 bytes was measured and is slower.)
// (I_END < TM: only the wave's first I_END row tiles hold rows of this tile.)
template <int TM, int TN, int NT_OUT, bool GLU, int I_END = TM, typename acc_t>
__device__ __forceinline__ void store_epilogue(const acc_t (&acc)[TN][TM], const EpilogueScales<TM, NT_OUT, GLU>& e,
                                               const TiledParams& p, const TileInfo& tile, int row_base, int n_base, int lane) {
  constexpr int MI = sizeof(acc_t) == 16 ? 16 : 32;  // 4 accumulator registers per tile: the 16 x 16 instructions
  // Everything that needs a load is decided and loaded up front, by uniform branches, and the variants of the body are
  // separate straight-line instantiations: a branch or a load between two stores makes the compiler wait for ALL memory
  // operations in flight, the stores included, i.e. one memory round trip per store (measured on 256 x 256 tiles: 18 us
  // per tile, as much as ten K stages, against 6 us now).
  float rw[TM];
  const bool round_first = p.ro.row_scale && !p.ro.out_f32;
#pragma unroll
  for (int i = 0; i < TM; i++) rw[i] = 1.0f;
  if (p.ro.row_scale) {
#pragma unroll
    for (int i = 0; i < I_END; i++) {
      const int lr = row_base + i * MI + (lane % MI);
      rw[i] = p.ro.row_scale[tile.row0 + (lr < tile.nrows ? lr : 0)];
    }
  }
  // GENERAL: bias, partial sums, row factors, f32 output; otherwise bf16 results straight to memory
  auto body = [&](auto act_c, auto general_c) {
    constexpr int ACT = decltype(act_c)::value;
    constexpr bool GENERAL = decltype(general_c)::value;
    if constexpr (!GENERAL && MI == 16 && NT_OUT % 2 == 0) {
      // Two neighbouring 16-channel tiles at a time: lanes 16 apart trade halves (lane (row, q) gives its 4 channels of the
      // tile it does not keep and receives the neighbour's 4 of the one it keeps), so that every lane stores 16 bytes and a
      // row's 64 bytes of the pair leave in one instruction: half the store instructions and half the write requests
      // (256 x 256 int8 tiles, 14336-long K: 0.929 against 0.947 ms).
#pragma unroll
      for (int i = 0; i < I_END; i++) {
        const int lr = row_base + i * MI + (lane % MI);
        const bool row_ok = lr < tile.nrows;
#pragma unroll
        for (int j = 0; j < NT_OUT; j += 2) {
          uint32_t pk[2][2];
#pragma unroll
          for (int t = 0; t < 2; t++) {
            const float sg[4] = {e.sg[j + t][0].x, e.sg[j + t][0].y, e.sg[j + t][0].z, e.sg[j + t][0].w};
            const float su[4] = {e.su[j + t][0].x, e.su[j + t][0].y, e.su[j + t][0].z, e.su[j + t][0].w};
            float v[4];
#pragma unroll
            for (int r = 0; r < 4; r++) {
              const float g = fmaf((float)acc[j + t][i][r], e.sa[i] * sg[r], 0.f);
              v[r] = GLU ? glu_act<ACT>(g, fmaf((float)acc[j + t + NT_OUT][i][r], e.sa[i] * su[r], 0.f), p.act_limit) : g;
            }
            pk[t][0] = pack_bf16x2(v[0], v[1]);
            pk[t][1] = pack_bf16x2(v[2], v[3]);
          }
          const auto s0 = __builtin_amdgcn_permlane16_swap(pk[0][0], pk[1][0], false, false);
          const auto s1 = __builtin_amdgcn_permlane16_swap(pk[0][1], pk[1][1], false, false);
          const int qq = lane / 16;
          const int n8 = n_base + (j + (qq & 1)) * 16 + 4 * (qq & ~1);
          if (row_ok && n8 < p.N)
            *(uint4*)((uint16_t*)p.out + (size_t)(tile.row0 + lr) * p.N + n8) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
        }
      }
      return;
    }
#pragma unroll
    for (int i = 0; i < I_END; i++) {
      const int lr = row_base + i * MI + (lane % MI);
      const bool row_ok = lr < tile.nrows;
#pragma unroll
      for (int j = 0; j < NT_OUT; j++)
#pragma unroll
        for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
          const int n = n_base + epilogue_channel<MI>(j, q, lane);
          const bool ok = row_ok && n < p.N;
          const float sg[4] = {e.sg[j][q].x, e.sg[j][q].y, e.sg[j][q].z, e.sg[j][q].w};
          const float su[4] = {e.su[j][q].x, e.su[j][q].y, e.su[j][q].z, e.su[j][q].w};
          float bg[4] = {0.f, 0.f, 0.f, 0.f}, bu[4] = {0.f, 0.f, 0.f, 0.f};
          if (GENERAL && ok) {
            load_bias4(p.rhs_bias, tile.group, p.N, n, bg);
            load_bias4(GLU ? p.rhs_up_bias : nullptr, tile.group, p.N, n, bu);
            add_partial4(p.partial_sum, (size_t)(tile.row0 + lr), p.N, n, bg);
            add_partial4(GLU ? p.partial_sum_up : nullptr, (size_t)(tile.row0 + lr), p.N, n, bu);
          }
          float v[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const float g = fmaf((float)acc[j][i][4 * q + r], e.sa[i] * sg[r], bg[r]);
            float a = g;
            if (GLU) {
              const float u = fmaf((float)acc[j + NT_OUT][i][4 * q + r], e.sa[i] * su[r], bu[r]);
              a = glu_act<ACT>(g, u, p.act_limit);
            }
            // a row factor multiplies the finished result of the output type (store_out4 states the rule)
            if (GENERAL) a = (round_first ? round_bf16_fn(a) : a) * rw[i];
            v[r] = a;
          }
          if (ok) {
            if (GENERAL && p.ro.out_f32)
              *(float4*)((float*)p.out + (size_t)(tile.row0 + lr) * p.N + n) = make_float4(v[0], v[1], v[2], v[3]);
            else
              *(uint2*)((uint16_t*)p.out + (size_t)(tile.row0 + lr) * p.N + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
          }
        }
    }
  };
  const bool general = p.rhs_bias || p.rhs_up_bias || p.partial_sum || p.partial_sum_up || p.ro.out_f32 || p.ro.row_scale;
  dispatch_act(GLU ? p.act : MOE_ACT_NONE, [&](auto act_c) {
    if (general) body(act_c, std::true_type{});
    else body(act_c, std::false_type{});
  });
}

// ---- whole-line weight requests of the streaming kernels ----

// Weight fragment of one 128-byte k-block for 16 channels.  Each of the two requests covers whole 128-byte
// lines (8 channels x 128 B: lane (i, kq) asks for bytes (i/8)*64 + kq*16.. of channel i%8, then of channel
// i%8 + 8) and is non-temporal: weights are read once, and a streamed read that owns its lines runs about
// 12 % faster than one that leaves half of each line to the next request (STREAM = false keeps the lines
// cached, for tiles that share weights).  A rotation by 8 inside each row of 16 lanes then hands every lane
// the two 16-byte pieces of its own channel i.
template <bool STREAM>
__device__ __forceinline__ v4i load_w16(const uint8_t* p) {
  return STREAM ? __builtin_nontemporal_load((const v4i*)p) : *(const v4i*)p;
}

// a = request for channels i%8, b = request for channels i%8 + 8, each lane holding piece i/8 (the first or second
// 64 bytes of the 128-byte unit).  Returns in `first` / `second` the two pieces of the lane's own channel i.
__device__ __forceinline__ void own_channel_pieces(const v4i& a, const v4i& b, v4i& first, v4i& second) {
#pragma unroll
  for (int c = 0; c < 4; c++) {
    // lanes 8..15 of a row: the first piece of their channel sits in `b` of lane i-8; lanes 0..7 keep their `a`
    first[c] = __builtin_amdgcn_update_dpp(a[c], b[c], 0x128, 0xf, 0xc, false);
    // lanes 0..7: the second piece of their channel sits in `a` of lane i+8; lanes 8..15 keep their `b`
    second[c] = __builtin_amdgcn_update_dpp(b[c], a[c], 0x128, 0xf, 0x3, false);
  }
}

// ---- buffer descriptors and the untracked global -> LDS copy of the persistent stream kernels ----

// A raw buffer descriptor over `bytes` bytes at `base`: requests past the end return zeros instead of faulting, which
// is how rows past a tile's (or a weight matrix's) end are dealt with.
__device__ __forceinline__ v4i buffer_desc(const void* base, uint32_t bytes) {
  const uint64_t a = (uint64_t)base;
  return v4i{(int)(uint32_t)a, (int)(uint32_t)((a >> 32) & 0xffffu), (int)bytes, 0x00020000};
}
__device__ __forceinline__ uint32_t clamp_u32(size_t v) { return v > 0xffffffffull ? 0xffffffffu : (uint32_t)v; }

// global -> LDS copy of 16 bytes per lane through a buffer descriptor (1 KB per wave at lds_addr, a wave-uniform LDS byte
// address), written as asm: the compiler then neither waits for it before LDS accesses that follow nor gives up counting
// the LDS reads in flight.  Which buffer a copy writes and a read reads is settled by explicit waits and barriers.
__device__ __forceinline__ void dma16_buffer(const v4i& rsrc, uint32_t voff, uint32_t soff, uint32_t lds_addr) {
  asm volatile("" : "+s"(soff));  // (a literal offset is not an operand the instruction takes)
  asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_addr) : "memory", "m0");
}
// ---- the tile cursor of the persistent stream kernels -------------------------------------------------------------
// tile id -> (m-tile, n-tile): ids congruent mod 8 run on one XCD (persistent blocks are dealt round-robin to the XCDs
// and a block's ids advance by the grid size, a multiple of 8); each XCD owns a contiguous range of the order, which
// runs in super-rows of p.tune m-tiles with the m-tile index fastest, so that the 32 blocks of an XCD work on a patch
// of a super-row's m-tiles x a few n-tiles that shares activation and weight panels in that XCD's L2.
struct StreamTile {
  TileInfo info;
  int n0, id;
};
struct TilePeek {  // a tile record that has been requested but not looked at yet
  TileInfo ti;
  int n0, id;
  bool valid;
};
// The block's first id >= id0 that names an existing m-tile; its record is requested, not waited for.
template <int OUT_BN>
__device__ __forceinline__ TilePeek peek_tile(const TiledParams& p, int num_tiles, int id0) {
  // the order covers the tiles that exist (the count the tile map left on the device), not the host's upper bound: with
  // the bound, the ids of tiles that do not exist all fall into the last XCD's range and leave its blocks idle while the
  // other seven work through full ranges (GPT-OSS at 4096 tokens: 97 slots for 80 m-tiles, 8.7 rounds instead of 7.2)
  const int total = num_tiles * p.tiles_n;
  TilePeek pk;
  pk.valid = false;
  pk.n0 = 0;
  pk.id = total;
  pk.ti = TileInfo{-1, 0, 0, 0};
  const int q = total / 8, rem = total % 8;
  const int GSM = p.tune > 0 ? p.tune : 8;
  const int width = GSM * p.tiles_n;
  for (int id = id0; id < total; id += gridDim.x) {
    const int xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(num_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    pk.ti = p.tiles[m_idx];
    pk.n0 = ((logical % width) / gsz) * OUT_BN;
    pk.id = id;
    pk.valid = true;
    break;
  }
  return pk;
}
// Turns a requested record into the block's next tile that needs the matmul (its fields uniform, in scalar registers);
// tiles of rows that belong to no local group are written as zeros on the way, and the search goes on from there.
template <int OUT_BN, int THREADS>
__device__ __forceinline__ bool resolve_tile(const TiledParams& p, int num_tiles, TilePeek pk, StreamTile& t, int tid) {
  while (pk.valid) {
    t.info.group = __builtin_amdgcn_readfirstlane(pk.ti.group);
    t.info.row0 = __builtin_amdgcn_readfirstlane(pk.ti.row0);
    t.info.nrows = __builtin_amdgcn_readfirstlane(pk.ti.nrows);
    t.info.pad = 0;
    t.n0 = __builtin_amdgcn_readfirstlane(pk.n0);
    t.id = __builtin_amdgcn_readfirstlane(pk.id);
    if (t.info.group >= 0) return true;
    zero_fill_tile(p.out, p.ro, t.info.row0, t.info.nrows, t.n0, OUT_BN, p.N, tid, THREADS);
    pk = peek_tile<OUT_BN>(p, num_tiles, t.id + gridDim.x);
  }
  return false;
}

struct SkinnyParams {
  const uint8_t* lhs;      // [M, K] fp8
  const float* lhs_scale;  // [M, K/128]
  const uint8_t* rhs;      // [G, N, K] fp8
  const uint8_t* rhs_up;
  const float* rhs_scale;  // [G, ceil(N/128), K/128]
  const float* rhs_up_scale;
  const float* rhs_bias;   // [G, N] f32 or NULL
  const float* rhs_up_bias;
  const uint16_t* partial_sum;     // [M, N] bf16 or NULL, added like the bias
  const uint16_t* partial_sum_up;
  const int32_t* header;
  const TileInfo* tiles;
  void* out;
  int M, K, N;
  int n_blocks;  // blocks along N
  int min_rows, max_rows;  // only tiles with min_rows <= nrows <= max_rows are computed by this launch
  int act;
  float act_limit;
  // per-row x per-channel scales (ops.py:241-260: lhs [m, 1], rhs [1, 1, n]) instead of blocks: the block scales above
  // are NULL (taken as 1) and these are applied once to the finished sums
  const float* row_scale_lhs;  // [M] (stride 1) or one value (stride 0), or NULL
  const float* ch_scale;       // f32, element (g, n) at g * ch_gstride + n * ch_nstride, or NULL
  const float* ch_scale_up;
  int row_scale_lhs_stride, ch_gstride, ch_nstride;
  RowOpts ro;
};

struct Fp8TiledParams {
  TiledParams base;        // lhs / rhs / rhs_up fp8; its epilogue scales are NULL for block-scaled operands
  const float* a_scale;    // [M, K/128], or NULL: no block scales (per-row x per-channel scales sit in `base`)
  const float* w_scale;    // [G, ceil(N/128), K/128]
  const float* u_scale;
};

struct WqSkinnyParams {
  const uint8_t* lhs;       // [M, K] bf16
  const uint8_t* rhs;       // [G, N, K] int8 or [G, N, K/2] packed int4
  const uint8_t* rhs_up;
  const void* rhs_scale;    // int8: f32 [G, N]; int4: bf16 [G, N, ceil(K/128)]
  const void* rhs_up_scale;
  const float* rhs_bias;    // [G, N] f32 or NULL
  const float* rhs_up_bias;
  const uint16_t* partial_sum;     // [M, N] bf16 or NULL, added like the bias
  const uint16_t* partial_sum_up;
  const int32_t* header;
  const TileInfo* tiles;
  void* out;
  int M, K, N;
  int n_blocks;
  int act;
  float act_limit;
  int ch_gstride, ch_nstride;  // int8 per-channel scales: element (g, n) at g * ch_gstride + n * ch_nstride
  RowOpts ro;
};

// ---------------------------------------------------------------------------------------
// Host side shared by the launchers
// ---------------------------------------------------------------------------------------

// Per-device launch state: the attribute that lets a kernel use more than 64 KB of dynamic LDS belongs to a
// device's code object, and the CU count to the device, so both are kept per device ordinal.  A race between two
// host threads only repeats an idempotent call.
constexpr int kMaxDevices = 64;

int current_device(int* dev);
int device_cu_count(int* cus);

template <typename K>
static int reserve_lds(K kernel, int bytes, bool (&done)[kMaxDevices]) {
  int dev = 0;
  if (int st = current_device(&dev)) return st;
  if (done[dev]) return MOE_OK;
  hipError_t e = hipFuncSetAttribute((const void*)kernel, hipFuncAttributeMaxDynamicSharedMemorySize, bytes);
  if (e != hipSuccess) return fail(MOE_ERR_LAUNCH, "gmm: cannot reserve %d bytes of LDS: %s", bytes, hipGetErrorString(e));
  done[dev] = true;
  return MOE_OK;
}

// One "LDS limit raised" flag per device for each kernel instantiation.
template <typename Tag>
static bool (&lds_flags())[kMaxDevices] {
  static bool flags[kMaxDevices] = {};
  return flags;
}

// Raise the LDS limit of every instantiation of a family on the current device (moe_init: callers that must not
// touch function attributes later, e.g. while a stream is being captured, do it up front).
int prepare_tiled();
int prepare_dl();
int prepare_fp8();
int prepare_dlw();
int prepare_dls();
int prepare_tgmm();

// ---- launchers (one translation unit per kernel family) ----
// moe_gmm_tiled.hip: register-staged kernel, m-tile bm in {64, 128, 256}; block_scaled: int8 x int8 / fp8 x fp8 with K-block
// scales applied to the partial sums (bm 64 or 128)
int launch_tiled_bm(int op, int bsrc, bool glu, int bm, bool block_scaled, const TiledParams& p, int M, int G_total, hipStream_t s);
// moe_gmm_dl.hip: direct-to-LDS persistent kernel, 256 x 256 tiles; stage_bytes 128 or 64; rhs_kn: [G, K, N] bf16 weights
int launch_dl(int op, bool glu, int stage_bytes, bool rhs_kn, const TiledParams& p, int M, int G_total, hipStream_t s);
// moe_gmm_dlw.hip: the same pipeline for bf16 activations x int8 / int4 / mxfp4 weights (K % 64 == 0, default scale layouts)
// moe_gmm_dls.hip: the persistent 256 x 256 kernel for int8 x int8 / bf16 x bf16 with one request stream across tiles
// (fp8 x fp8 with epilogue scales too; lhs_e5m2: the activations are float8_e5m2, the weights e4m3)
int launch_dls(int op, bool glu, const TiledParams& p, int M, int G_total, hipStream_t s, int lhs_e5m2 = 0, int rhs_kn = 0);
bool dls_takes(int op, int K, int N, long long indexed_lhs_rows);
// moe_gmm_f8s.hip: the same stream for block-scaled fp8 (1 x 128 activation scales, 128 x 128 weight scales)
struct Fp8TiledParams;
int launch_f8s(bool glu, const Fp8TiledParams& P, int M, int G_total, hipStream_t s);
bool f8s_takes(int K, int N, long long M, long long indexed_lhs_rows);
int prepare_f8s();
int launch_dlw(int bsrc, bool glu, bool half, const TiledParams& p, int M, int G_total, hipStream_t s);
// whether that kernel takes the shape (indexed_lhs_rows: rows of lhs when a row index is used, else 0)
bool dlw_takes(int K, int N, long long indexed_lhs_rows, bool wq_kmajor);
// moe_gmm_fp8.hip
int launch_fp8_tiled(bool big, bool glu, bool vec4, const Fp8TiledParams& P, int M, int G_total, hipStream_t s);
int launch_fp8_skinny(bool few_rows, const SkinnyParams& p, bool glu, int max_tiles, hipStream_t s);
// moe_gmm_wq.hip: fmt is one of WQ_*; one_tile: 16-row tiles (else 32)
enum { WQ_I8 = 0, WQ_I4 = 1, WQ_MX4 = 2, WQ_I4G32 = 3 };  // weight formats of the streaming kernel (int4: group 128 / 32)
int launch_wq(int fmt, bool one_tile, const WqSkinnyParams& q, bool glu, int max_tiles, int tune, hipStream_t s);

}  // namespace moe
