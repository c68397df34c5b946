// Grouped matmul for gfx950.
//
//   tile_map_kernel   group_sizes (device) -> list of (group, first row, rows) m-tiles that never
//                     straddle a group boundary, plus zero-fill tiles for non-local / tail rows.
//   gmm_tiled_kernel  LDS-staged, double-buffered MFMA GEMM over that tile list.  Weights are the
//                     MFMA "A" operand (32 output channels per tile), activations the "B" operand
//                     (32 rows), so each lane ends up with 4 consecutive output channels of one
//                     row per accumulator quad and stores 8 bytes.  bf16 x {bf16, int8, int4}
//                     weights run on v_mfma_f32_32x32x16_bf16 (weights are widened to bf16 while
//                     they are copied into LDS), int8 x int8 on v_mfma_i32_32x32x32_i8.
//                     Used for weight-only formats, small problems and K tails.
//   gmm_dl_kernel     the prefill kernel for int8 x int8 and bf16 x bf16: persistent blocks, operands
//                     copied global -> LDS without passing through registers, 4 stages in flight.
//   gmm_fp8_skinny_kernel  block-scaled fp8 for few rows per expert (decode): no LDS, every wave
//                     streams 16 weight rows through v_mfma_f32_16x16x128_f8f6f4 and applies the
//                     per-128 K-block scales to the f32 partial sums.
//   gmm_fp8_tiled_kernel   block-scaled fp8 for 16 to 128 rows per expert: 128 x 128 tiles through LDS,
//                     v_mfma_f32_32x32x64_f8f6f4, one scaled accumulation per 128-wide K block.
//   gmm_fp8_big_kernel     block-scaled fp8 from 128 rows per expert (prefill): 256 x 256 tiles, one set of
//                     accumulators kept in units of the current K block's scale.
//   gmm_wq_skinny_kernel   the same streaming design for bf16 activations x int8 / int4 / mxfp4 weights,
//                     with K split over the waves of a block.

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

constexpr int kMapThreads = 256;

__device__ __forceinline__ int block_exclusive_scan(int v, int* s_buf, int* total) {
  const int tid = threadIdx.x;
  s_buf[tid] = v;
  __syncthreads();
  for (int o = 1; o < kMapThreads; o <<= 1) {
    int add = tid >= o ? s_buf[tid - o] : 0;
    __syncthreads();
    s_buf[tid] += add;
    __syncthreads();
  }
  int incl = s_buf[tid];
  *total = s_buf[kMapThreads - 1];
  __syncthreads();
  return incl - v;
}

__global__ __launch_bounds__(kMapThreads) void tile_map_kernel(
    const int32_t* __restrict__ group_sizes, int G_total, int group_offset, int G_local, int M,
    int BM, int zero_fill, int32_t* __restrict__ header, TileInfo* __restrict__ tiles) {
  __shared__ int s_buf[kMapThreads];
  const int tid = threadIdx.x;
  const int per = (G_total + kMapThreads - 1) / kMapThreads;
  const int g0 = min(tid * per, G_total), g1 = min(g0 + per, G_total);
  long long rows = 0;
  for (int g = g0; g < g1; g++) rows += max(group_sizes[g], 0);
  int total_rows;
  int row_prefix = block_exclusive_scan((int)min(rows, (long long)M), s_buf, &total_rows);
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
  int tile_prefix = block_exclusive_scan(ntiles, s_buf, &total_tiles);
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
  for (int i = tid; i < tail; i += kMapThreads) {
    TileInfo t;
    t.group = -1;
    t.row0 = covered + i * BM;
    t.nrows = min(BM, M - t.row0);
    t.pad = 0;
    tiles[total_tiles + i] = t;
  }
  if (tid == 0) header[0] = total_tiles + tail;
}

// ---------------------------------------------------------------------------------------
// Tiled MFMA kernel
// ---------------------------------------------------------------------------------------

enum { OP_BF16 = 0, OP_I8 = 1 };                 // MFMA operand type (= LDS element type)
enum { BSRC_SAME = 0, BSRC_I8 = 1, BSRC_I4 = 2, BSRC_MX4 = 3 };  // weight format in HBM

struct TiledParams {
  const uint8_t* lhs;        // [M, K] elements of the MFMA operand type
  const float* lhs_scale;    // [M] or NULL
  const uint8_t* rhs;        // [G, N, K] (INT4: K/2 bytes per row)
  const uint8_t* rhs_up;     // same, or NULL
  const void* rhs_scale;     // f32 [G, N] (per channel) | bf16 [G, N, nkg] (INT4) | e8m0 bytes [G, N, K/32] (MXFP4)
  const void* rhs_up_scale;
  const float* rhs_bias;     // [G, N] f32 or NULL, added before the activation
  const float* rhs_up_bias;
  const uint16_t* partial_sum;     // [M, N] bf16 or NULL, added like the bias
  const uint16_t* partial_sum_up;
  const int32_t* header;
  const TileInfo* tiles;
  uint16_t* out;  // [M, N] bf16
  int M, K, N;
  int max_m_tiles, tiles_n;
  int act;
  float act_limit;
  int tune;  // > 0: m-tiles per raster super-row of the persistent kernel (tuning aid; 0 = default)
  int i4_group;  // values of K per int4 scale: 128 or 32
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
  const float4 one = make_float4(1.f, 1.f, 1.f, 1.f);
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int lr = row_base + i * MI + (lane % MI);
    e.sa[i] = p.lhs_scale ? p.lhs_scale[tile.row0 + (lr < tile.nrows ? lr : 0)] : 1.0f;
  }
#pragma unroll
  for (int j = 0; j < NT_OUT; j++)
#pragma unroll
    for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
      const int n = n_base + epilogue_channel<MI>(j, q, lane);
      e.sg[j][q] = one;
      e.su[j][q] = one;
      if (CHANNEL_SCALES && p.rhs_scale && n < p.N) {
        e.sg[j][q] = *(const float4*)((const float*)p.rhs_scale + (size_t)tile.group * p.N + n);
        if (GLU) e.su[j][q] = *(const float4*)((const float*)p.rhs_up_scale + (size_t)tile.group * p.N + n);
      }
    }
}

template <int TM, int TN, int NT_OUT, bool GLU, typename acc_t>
__device__ __forceinline__ void store_epilogue(const acc_t (&acc)[TN][TM], const EpilogueScales<TM, NT_OUT, GLU>& e,
                                               const TiledParams& p, const TileInfo& tile, int row_base, int n_base, int lane) {
  constexpr int MI = sizeof(acc_t) == 16 ? 16 : 32;  // 4 accumulator registers per tile: the 16 x 16 instructions
  dispatch_act(GLU ? p.act : MOE_ACT_NONE, [&](auto act_c) {
  constexpr int ACT = decltype(act_c)::value;
#pragma unroll
  for (int i = 0; i < TM; i++) {
    const int lr = row_base + i * MI + (lane % MI);
    if (lr >= tile.nrows) continue;
    uint16_t* orow = p.out + (size_t)(tile.row0 + lr) * p.N;
#pragma unroll
    for (int j = 0; j < NT_OUT; j++)
#pragma unroll
      for (int q = 0; q < (MI == 32 ? 4 : 1); q++) {
        const int n = n_base + epilogue_channel<MI>(j, q, lane);
        if (n >= p.N) continue;
        const float sg[4] = {e.sg[j][q].x, e.sg[j][q].y, e.sg[j][q].z, e.sg[j][q].w};
        const float su[4] = {e.su[j][q].x, e.su[j][q].y, e.su[j][q].z, e.su[j][q].w};
        float bg[4], bu[4];
        load_bias4(p.rhs_bias, tile.group, p.N, n, bg);
        load_bias4(GLU ? p.rhs_up_bias : nullptr, tile.group, p.N, n, bu);
        add_partial4(p.partial_sum, (size_t)(tile.row0 + lr), p.N, n, bg);
        add_partial4(GLU ? p.partial_sum_up : nullptr, (size_t)(tile.row0 + lr), p.N, n, bu);
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const float g = fmaf((float)acc[j][i][4 * q + r], e.sa[i] * sg[r], bg[r]);
          if (GLU) {
            const float u = fmaf((float)acc[j + NT_OUT][i][4 * q + r], e.sa[i] * su[r], bu[r]);
            v[r] = glu_act<ACT>(g, u, p.act_limit);
          } else {
            v[r] = g;
          }
        }
        *(uint2*)(orow + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      }
  }
  });
}

template <int OP_, int BSRC_, int BM_, int BN_, int BKB_, int WAVES_M_, int WAVES_N_, bool GLU_>
struct TiledCfg {
  static constexpr int OP = OP_, BSRC = BSRC_, BM = BM_, BN = BN_, BKB = BKB_;
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool GLU = GLU_;
  static constexpr int THREADS = WAVES_M * WAVES_N * kWave;
  static constexpr int ESZ = OP == OP_I8 ? 1 : 2;
  static constexpr int BK = BKB / ESZ;
  static constexpr int LDR = BKB + 16;  // LDS row stride in bytes (pad keeps b128 reads conflict free)
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / 32, TN = WN / 32;
  static constexpr int KSUB = BKB / 32;  // MFMA steps per stage (32 bytes of K per row each)
  static constexpr int A_CPR = BKB / 16;
  static constexpr int A_CH = BM * A_CPR / THREADS;
  static constexpr bool NIBBLES = BSRC == BSRC_I4 || BSRC == BSRC_MX4;  // two weights per byte
  static constexpr int B_CHE = BSRC == BSRC_SAME ? 16 / ESZ : (BSRC == BSRC_I8 ? 16 : 32);  // elems per 16B
  static constexpr int B_CPR = BK / B_CHE;
  static constexpr int B_CH = BN * B_CPR / THREADS;
  static constexpr int STAGE = (BM + BN) * LDR;
  static constexpr int LDS_BYTES = 2 * STAGE;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(BM % (WAVES_M * 32) == 0 && BN % (WAVES_N * 32) == 0, "wave tiling");
  static_assert(!GLU || TN % 2 == 0, "GLU needs gate and up tiles in every wave");
  static_assert(BM * A_CPR % THREADS == 0 && A_CH >= 1, "A chunks");
  static_assert(BN * B_CPR % THREADS == 0 && B_CH >= 1, "B chunks");
  static_assert(BSRC == BSRC_SAME || OP == OP_BF16, "weight-only formats feed the bf16 MFMA");
};

template <typename C>
__global__ __launch_bounds__(C::THREADS) void gmm_tiled_kernel(const TiledParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int OP = C::OP;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;

  // ---- block -> (m-tile, n-tile): contiguous ids per XCD, then GSM x tiles_n super-rows ----
  int m_idx, n_idx;
  {
    const int nb = gridDim.x, pid = blockIdx.x;
    const int q = nb / 8, rem = nb % 8, xcd = pid % 8, loc = pid / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    constexpr int GSM = 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(p.max_m_tiles - first_m, GSM);
    m_idx = first_m + (logical % width) % gsz;
    n_idx = (logical % width) / gsz;
  }
  // the slot exists even when the tile does not (the list is sized for the worst case): both loads go out
  // together instead of one after the other
  const TileInfo tile = p.tiles[m_idx];
  if (m_idx >= p.header[0]) return;
  const int n0 = n_idx * C::OUT_BN;
  const int N = p.N, K = p.K;

  if (tile.group < 0) {  // rows of no local group: zeros
    constexpr int QPR = C::OUT_BN / 4;
    for (int i = tid; i < tile.nrows * QPR; i += C::THREADS) {
      int r = i / QPR, c = n0 + (i % QPR) * 4;
      if (c < N) *(uint2*)(p.out + (size_t)(tile.row0 + r) * N + c) = make_uint2(0, 0);
    }
    return;
  }

  // ---- global -> register staging -------------------------------------------------------
  const size_t a_row_bytes = (size_t)K * C::ESZ;
  const size_t b_row_bytes = C::NIBBLES ? (size_t)K / 2 : (size_t)K * (C::BSRC == BSRC_I8 ? 1 : C::ESZ);
  const uint8_t* a_ptr[C::A_CH];
  int a_k[C::A_CH], a_lds[C::A_CH];
#pragma unroll
  for (int i = 0; i < C::A_CH; i++) {
    int c = tid + i * C::THREADS;
    int r = c / C::A_CPR, col = c % C::A_CPR;
    int gr = tile.row0 + min(r, tile.nrows - 1);
    a_ptr[i] = p.lhs + (size_t)gr * a_row_bytes + col * 16;
    a_k[i] = col * (16 / C::ESZ);
    a_lds[i] = r * C::LDR + col * 16;
  }
  const uint8_t* b_ptr[C::B_CH];
  int b_k[C::B_CH], b_lds[C::B_CH], b_n[C::B_CH];
  bool b_up[C::B_CH];
#pragma unroll
  for (int i = 0; i < C::B_CH; i++) {
    int c = tid + i * C::THREADS;
    int vr = c / C::B_CPR, col = c % C::B_CPR;
    bool up = C::GLU && vr >= C::BN / 2;
    int n = n0 + (up ? vr - C::BN / 2 : vr);
    n = min(n, N - 1);
    const uint8_t* base = up ? p.rhs_up : p.rhs;
    b_ptr[i] = base + ((size_t)tile.group * N + n) * b_row_bytes + col * 16;
    b_k[i] = col * C::B_CHE;
    b_lds[i] = C::BM * C::LDR + vr * C::LDR + col * C::B_CHE * C::ESZ;
    b_n[i] = n;
    b_up[i] = up;
  }

  uint4 a_reg[C::A_CH], b_reg[C::B_CH];
  constexpr int B_GSZ = C::NIBBLES ? 1 : (C::BSRC == BSRC_I8 ? 2 : 2 * C::ESZ);  // half-bytes per element in HBM

  // Every chunk of a full stage is in range: plain loads that stay in flight during the MFMAs.
  auto load_stage = [&](int kt) {
    const size_t k0 = (size_t)kt * C::BK;
#pragma unroll
    for (int i = 0; i < C::A_CH; i++) a_reg[i] = *(const uint4*)(a_ptr[i] + k0 * C::ESZ);
#pragma unroll
    for (int i = 0; i < C::B_CH; i++) b_reg[i] = *(const uint4*)(b_ptr[i] + k0 * B_GSZ / 2);
  };
  // Last stage when K is not a multiple of BK: chunks past K read offset 0 and are zeroed by value.
  auto load_stage_tail = [&](int kt) {
    const int k0 = kt * C::BK;
#pragma unroll
    for (int i = 0; i < C::A_CH; i++) {
      const bool ok = k0 + a_k[i] < K;
      const uint4 v = *(const uint4*)(a_ptr[i] + (ok ? (size_t)k0 * C::ESZ : 0));
      const uint32_t m = ok ? 0xffffffffu : 0u;
      a_reg[i] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
    }
#pragma unroll
    for (int i = 0; i < C::B_CH; i++) {
      const bool ok = k0 + b_k[i] < K;
      const uint4 v = *(const uint4*)(b_ptr[i] + (ok ? (size_t)k0 * B_GSZ / 2 : 0));
      // INT4 stores value+8: a zero weight is the nibble 8 (MXFP4: nibble 0 is +0.0)
      const uint32_t z = C::BSRC == BSRC_I4 ? 0x88888888u : 0u;
      b_reg[i] = ok ? v : make_uint4(z, z, z, z);
    }
  };

  // single-chunk versions: MODE 1 = full stage, 2 = the stage that holds the K tail
  auto load_a_chunk = [&](int kt, int i, auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
    const int k0 = kt * C::BK;
    if constexpr (MODE == 1) {
      a_reg[i] = *(const uint4*)(a_ptr[i] + (size_t)k0 * C::ESZ);
    } else {
      const bool ok = k0 + a_k[i] < K;
      const uint4 v = *(const uint4*)(a_ptr[i] + (ok ? (size_t)k0 * C::ESZ : 0));
      const uint32_t m = ok ? 0xffffffffu : 0u;
      a_reg[i] = make_uint4(v.x & m, v.y & m, v.z & m, v.w & m);
    }
  };
  auto load_b_chunk = [&](int kt, int i, auto mode_c) {
    constexpr int MODE = decltype(mode_c)::value;
    const int k0 = kt * C::BK;
    if constexpr (MODE == 1) {
      b_reg[i] = *(const uint4*)(b_ptr[i] + (size_t)k0 * B_GSZ / 2);
    } else {
      const bool ok = k0 + b_k[i] < K;
      const uint4 v = *(const uint4*)(b_ptr[i] + (ok ? (size_t)k0 * B_GSZ / 2 : 0));
      const uint32_t z = C::BSRC == BSRC_I4 ? 0x88888888u : 0u;
      b_reg[i] = ok ? v : make_uint4(z, z, z, z);
    }
  };

  auto store_a_chunk = [&](int buf, int i) {
    uint8_t* s = smem + buf * C::STAGE;
    *(uint4*)(s + a_lds[i]) = a_reg[i];
  };
  // A weight chunk is converted and stored in 4 parts (one 32-bit word of the staged register each), so that the
  // conversions can be spread over the k sub-steps of a stage.  The chunk's scale is fetched with part 0.
  float b_scale[C::B_CH];
  auto store_b_part = [&](int buf, int kt, int i, int part) {
    uint8_t* s = smem + buf * C::STAGE;
    const uint32_t w4[4] = {b_reg[i].x, b_reg[i].y, b_reg[i].z, b_reg[i].w};
    const uint32_t w = w4[part];
    if (C::BSRC == BSRC_SAME) {  // nothing to convert: one 16-byte store with the last part
      if (part == 3) *(uint4*)(s + b_lds[i]) = b_reg[i];
    } else if (C::BSRC == BSRC_I8) {  // 4 int8 -> 4 bf16
      const int v = (int)w;
      *(uint2*)(s + b_lds[i] + 8 * part) = make_uint2(i8x2_to_bf16x2((v << 24) >> 24, (v << 16) >> 24), i8x2_to_bf16x2((v << 8) >> 24, v >> 24));
    } else if (C::BSRC == BSRC_MX4) {  // 8 e2m1 values of an MX block with its e8m0 scale 2^(s - 127)
      if (part == 0) {
        const int kk = kt * C::BK + b_k[i];
        const uint8_t* sc = (const uint8_t*)(b_up[i] ? p.rhs_up_scale : p.rhs_scale);
        const uint32_t sbyte = kk < K ? sc[((size_t)tile.group * N + b_n[i]) * (K / 32) + kk / 32] : 127u;
        b_scale[i] = __uint_as_float(sbyte << 23);
      }
      const float scale = b_scale[i];
      *(uint4*)(s + b_lds[i] + 16 * part) = make_uint4(
          __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 0)),
          __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 1)),
          __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 2)),
          __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, scale, 3)));
    } else {  // BSRC_I4: 8 values of one scale group (128 or 32 wide)
      if (part == 0) {
        const int kk = kt * C::BK + b_k[i];
        const int nkg = (K + p.i4_group - 1) / p.i4_group;
        const uint16_t* sc = (const uint16_t*)(b_up[i] ? p.rhs_up_scale : p.rhs_scale);
        b_scale[i] = kk < K ? bf16_bits_to_f32(sc[((size_t)tile.group * N + b_n[i]) * nkg + kk / p.i4_group]) : 0.f;
      }
      const float scale = b_scale[i];
      uint32_t o[4];
#pragma unroll
      for (int h = 0; h < 4; h++) {
        const int lo = (int)((w >> (8 * h)) & 0xf) - 8;
        const int hi = (int)((w >> (8 * h + 4)) & 0xf) - 8;
        o[h] = pack_bf16x2((float)lo * scale, (float)hi * scale);
      }
      *(uint4*)(s + b_lds[i] + 16 * part) = make_uint4(o[0], o[1], o[2], o[3]);
    }
  };
  auto store_b_chunk = [&](int buf, int kt, int i) {
#pragma unroll
    for (int part = 0; part < 4; part++) store_b_part(buf, kt, i, part);
  };
  auto store_stage = [&](int buf, int kt) {
#pragma unroll
    for (int i = 0; i < C::A_CH; i++) store_a_chunk(buf, i);
#pragma unroll
    for (int i = 0; i < C::B_CH; i++) store_b_chunk(buf, kt, i);
  };

  // ---- accumulators ---------------------------------------------------------------------
  typedef typename std::conditional<OP == OP_I8, v16i, v16f>::type acc_t;
  acc_t acc[C::TN][C::TM];
#pragma unroll
  for (int j = 0; j < C::TN; j++)
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][i][r] = 0;

  // LDS row of the wave's j-th weight tile: with GLU the first TN/2 tiles are gate channels,
  // the rest the matching up channels.
  int b_row[C::TN];
#pragma unroll
  for (int j = 0; j < C::TN; j++) {
    if (C::GLU) {
      constexpr int H = C::TN / 2;
      int jj = j < H ? j : j - H;
      b_row[j] = (j < H ? 0 : C::BN / 2) + wn * (C::WN / 2) + jj * 32;
    } else {
      b_row[j] = wn * C::WN + j * 32;
    }
  }
  const int frag_off = (lane % 32) * C::LDR + (lane / 32) * 16;

  auto compute_stage = [&](int buf) {
    const uint8_t* sa = smem + buf * C::STAGE + (wm * C::WM) * C::LDR + frag_off;
    const uint8_t* sb = smem + buf * C::STAGE + C::BM * C::LDR + frag_off;
#pragma unroll
    for (int ks = 0; ks < C::KSUB; ks++) {
      v4i af[C::TM], bf[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; i++) af[i] = *(const v4i*)(sa + i * 32 * C::LDR + ks * 32);
#pragma unroll
      for (int j = 0; j < C::TN; j++) bf[j] = *(const v4i*)(sb + b_row[j] * C::LDR + ks * 32);
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
          if constexpr (OP == OP_I8) {
            acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[j][i], 0, 0, 0);
          } else {
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(v8bf, bf[j]), __builtin_bit_cast(v8bf, af[i]), acc[j][i], 0, 0, 0);
          }
        }
    }
  };

  // MFMAs of the stage in `buf` with, after each k sub-step, a share of the register -> LDS stores (and weight
  // conversions) of stage kt_store into the other buffer; every register is refilled right after its store with
  // the same chunk of the stage after that (LOAD: 0 none, 1 full stage, 2 the stage holding the K tail), so a
  // load has a whole stage of MFMAs to land and the stores ride in the shadow of the MFMAs instead of forming a
  // phase of their own before the barrier.
  auto compute_and_store = [&](int buf, int kt_store, auto store_c, auto load_c) {
    constexpr bool STORE = decltype(store_c)::value;
    constexpr int LOAD = decltype(load_c)::value;
    const uint8_t* sa = smem + buf * C::STAGE + (wm * C::WM) * C::LDR + frag_off;
    const uint8_t* sb = smem + buf * C::STAGE + C::BM * C::LDR + frag_off;
    constexpr int A_PER = (C::A_CH + C::KSUB - 1) / C::KSUB;
#pragma unroll
    for (int ks = 0; ks < C::KSUB; ks++) {
      v4i af[C::TM], bf[C::TN];
#pragma unroll
      for (int i = 0; i < C::TM; i++) af[i] = *(const v4i*)(sa + i * 32 * C::LDR + ks * 32);
#pragma unroll
      for (int j = 0; j < C::TN; j++) bf[j] = *(const v4i*)(sb + b_row[j] * C::LDR + ks * 32);
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
          if constexpr (OP == OP_I8) {
            acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(bf[j], af[i], acc[j][i], 0, 0, 0);
          } else {
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
                __builtin_bit_cast(v8bf, bf[j]), __builtin_bit_cast(v8bf, af[i]), acc[j][i], 0, 0, 0);
          }
        }
      if constexpr (STORE) {
#pragma unroll
        for (int c = 0; c < A_PER; c++) {
          const int i = ks * A_PER + c;
          if (i < C::A_CH) {
            store_a_chunk(buf ^ 1, i);
            if constexpr (LOAD != 0) load_a_chunk(kt_store + 1, i, load_c);
          }
        }
        // part ks of every weight chunk; the register is refilled after its last part
        static_assert(C::KSUB == 4 || C::KSUB == 2, "weight chunks are stored in KSUB or 2 * KSUB parts");
#pragma unroll
        for (int i = 0; i < C::B_CH; i++) {
#pragma unroll
          for (int q = 0; q < 4 / C::KSUB; q++) store_b_part(buf ^ 1, kt_store, i, ks * (4 / C::KSUB) + q);
          if (ks == C::KSUB - 1) {
            if constexpr (LOAD != 0) load_b_chunk(kt_store + 1, i, load_c);
          }
        }
      }
      __builtin_amdgcn_sched_barrier(0);
    }
  };

  // ---- main loop: one barrier per stage --------------------------------------------------
  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;
  const int n_out0 = n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
  EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
  load_epilogue_scales<C::TM, NT_OUT, C::GLU, !C::NIBBLES>(esc, p, tile, wm * C::WM, n_out0, lane);

  // The steady-state loop only ever issues full-stage loads; the stage that may hold the K tail is
  // loaded in a peeled iteration so its masking code never merges into the loop body.
  const int nk = (K + C::BK - 1) / C::BK;
  const bool k_tail = (K % C::BK) != 0;
  const int full = k_tail ? nk - 1 : nk;  // stages 0 .. full-1 need no masking
  using L0 = std::integral_constant<int, 0>;
  using L1 = std::integral_constant<int, 1>;
  using L2 = std::integral_constant<int, 2>;
  if (nk == 1 && k_tail) load_stage_tail(0); else load_stage(0);
  store_stage(0, 0);
  if (nk > 1) {
    if (nk == 2 && k_tail) load_stage_tail(1); else load_stage(1);
  }
  __syncthreads();
  // LDS writes of this wave done, then the barrier; not __syncthreads(), whose fence would also wait for the global
  // loads that were just issued for the stage after next
  auto stage_barrier = [&]() { asm volatile("s_waitcnt lgkmcnt(0)\n\ts_barrier" ::: "memory"); };
  // Steady state: stage kt is computed, stage kt+1 moves from registers to LDS, stage kt+2 (a full one) is requested.
  int kt = 0;
  for (; kt + 2 < full; kt++) {
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L1{});
    stage_barrier();
  }
  if (kt + 2 < nk) {  // the stage after next is the one with the K tail
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L2{});
    stage_barrier();
    kt++;
  }
  if (kt + 1 < nk) {
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L0{});
    stage_barrier();
    kt++;
  }
  compute_stage(kt & 1);

  store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, tile, wm * C::WM, n_out0, lane);
}

// ---------------------------------------------------------------------------------------
// Direct-to-LDS variant of the tiled kernel for operands that need no conversion (int8 x int8,
// bf16 x bf16) and K * elem_size % BKB == 0.  global_load_lds_dwordx4 copies 16 bytes per lane
// straight into LDS (1 KB per wave instruction, no staging registers, no ds_write), NSTAGE
// buffers are kept in flight, and there is one barrier per K stage.  LDS rows are unpadded; the
// 16-byte chunk q of row r is stored at slot q ^ f(r), chosen so that the b128 fragment reads of
// 16 consecutive rows hit 16 different bank groups.  The permutation is applied on the global
// address side, because the LDS side of the instruction is fixed (base + 16 * lane).
// ---------------------------------------------------------------------------------------

template <int OP_, int BM_, int BN_, int BKB_, int WAVES_M_, int WAVES_N_, int NSTAGE_, bool GLU_, bool RHS_KN_ = false>
struct DlCfg {
  static constexpr int OP = OP_, BM = BM_, BN = BN_, BKB = BKB_, NSTAGE = NSTAGE_;
  // RHS_KN: the weights are given as [G, K, N] with N contiguous (the contraction index is the row).  A stage then
  // holds BK weight rows of BN channels instead of BN rows of BK values, and the weight fragments come out of it
  // through the transposing LDS read (ds_read_b64_tr_b16), as in the weight-gradient kernel.
  static constexpr bool RHS_KN = RHS_KN_;
  // rows (= columns) of the MFMA tile: 128-byte stages feed the 16 x 16 instructions (16x16x64 i8 / 16x16x32 bf16: 64
  // bytes of K per row), 64-byte stages the 32 x 32 ones (32x32x32 i8 / 32x32x16 bf16: 32 bytes of K per row)
  static constexpr int MI = BKB == 128 ? 16 : 32;
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_, NWAVES = WAVES_M_ * WAVES_N_;
  static constexpr bool GLU = GLU_;
  static constexpr int THREADS = NWAVES * kWave;
  static constexpr int ESZ = OP == OP_I8 ? 1 : 2;
  static constexpr int BK = BKB / ESZ;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N;
  static constexpr int TM = WM / MI, TN = WN / MI;
  static constexpr int KSUB = BKB / 32;
  static constexpr int CPR = BKB / 16;         // 16-byte chunks per row
  static constexpr int RPI = 1024 / BKB;       // rows per wave instruction
  static constexpr int A_IPW = BM / RPI / NWAVES, B_IPW = BN / RPI / NWAVES;  // instructions per wave per stage
  static constexpr int LPS = A_IPW + B_IPW;
  static constexpr int STAGE = (BM + BN) * BKB;
  static constexpr int LDS_BYTES = NSTAGE * STAGE;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(BKB == 64 || BKB == 128, "row swizzle is defined for 64 and 128 byte rows");
  static_assert(BM % (RPI * NWAVES) == 0 && BN % (RPI * NWAVES) == 0, "load split");
  static_assert(!GLU || ((BN / 2) % RPI == 0 && TN % 2 == 0), "GLU halves");
  static_assert((NSTAGE - 1) * LPS < 64, "vmcnt range");
  static_assert(MI == 32 || (NSTAGE == 2 && TM >= TN && TM * TN >= LPS), "16 x 16 pipeline shape");
  static_assert(!RHS_KN || (OP == 0 && MI == 16 && !GLU && BN == 256 && BK * BN * 2 == BN * BKB), "[G, K, N] weights: bf16, 256 channels");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS");
  __device__ static __forceinline__ int swz(int row) { return BKB == 128 ? (row >> 1) & 7 : (row >> 2) & 3; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, C::NWAVES >= 8 ? 2 : 1) void gmm_dl_kernel(const TiledParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  constexpr int OP = C::OP;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const size_t row_bytes = (size_t)K * C::ESZ;
  const int num_tiles = p.header[0];
  const int total = p.max_m_tiles * p.tiles_n;

  // Persistent blocks: block b works on tile ids b, b + gridDim.x, ...  A tile id is turned into (m-tile,
  // n-tile) so that ids that run at the same time on one XCD (ids congruent mod 8 go to the same XCD) form
  // a GSM x (32 / GSM) patch sharing activation and weight panels in that XCD's L2.
  struct Tile {
    TileInfo info;
    int n0;
  };
  auto locate = [&](int id, Tile& t) -> bool {
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 8;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(p.max_m_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    if (m_idx >= num_tiles) return false;
    t.info = p.tiles[m_idx];
    t.n0 = ((logical % width) / gsz) * C::OUT_BN;
    return true;
  };
  // Advances `id` to this block's next tile that needs the matmul; tiles of rows that belong to no local
  // group are written as zeros on the way.
  auto next_compute_tile = [&](int& id, Tile& t) -> bool {
    for (; id < total; id += gridDim.x) {
      if (!locate(id, t)) continue;
      if (t.info.group >= 0) return true;
      constexpr int QPR = C::OUT_BN / 4;
      for (int i = tid; i < t.info.nrows * QPR; i += C::THREADS) {
        int r = i / QPR, c = t.n0 + (i % QPR) * 4;
        if (c < N) *(uint2*)(p.out + (size_t)(t.info.row0 + r) * N + c) = make_uint2(0, 0);
      }
    }
    return false;
  };

  // ---- per-lane source addresses of this wave's load instructions ---------------------------
  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
  auto set_sources = [&](const Tile& t) {
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) {
      const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
      const int q = (lane % C::CPR) ^ C::swz(r);
      a_src[i] = p.lhs + (size_t)(t.info.row0 + min(r, t.info.nrows - 1)) * row_bytes + q * 16;
    }
#pragma unroll
    for (int i = 0; i < C::B_IPW; i++) {
      if constexpr (C::RHS_KN) {
        // a request covers two weight rows (contraction index) of the tile's 256 channels: 2 x 512 bytes
        const int r = 2 * (wave * C::B_IPW + i) + lane / 32;
        const int q = (lane % 32) ^ tr_swz(r);
        b_src[i] = p.rhs + (((size_t)t.info.group * K + r) * N + t.n0) * 2 + q * 16;
      } else {
        const int vr = (wave * C::B_IPW + i) * C::RPI + lane / C::CPR;
        const int q = (lane % C::CPR) ^ C::swz(vr);
        const bool up = C::GLU && vr >= C::BN / 2;
        const int n = min(t.n0 + (up ? vr - C::BN / 2 : vr), N - 1);
        b_src[i] = (up ? p.rhs_up : p.rhs) + ((size_t)t.info.group * N + n) * row_bytes + q * 16;
      }
    }
  };

  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;
  auto issue_one = [&](int kt, int buf, int idx) {
    const size_t koff = (size_t)kt * C::BKB;
    const int i = idx < C::A_IPW ? idx : idx - C::A_IPW;
    const uint8_t* src = idx < C::A_IPW ? a_src[i] + koff : b_src[i] + (C::RHS_KN ? (size_t)kt * C::BK * N * 2 : koff);
    const int off = buf * C::STAGE + (idx < C::A_IPW ? (wave * C::A_IPW + i) * 1024 : C::BM * C::BKB + (wave * C::B_IPW + i) * 1024);
    if constexpr (C::RHS_KN) {
      dma16_untracked(src, lds_base + off);  // the transposing reads below must not wait for the copies in flight
    } else {
      __builtin_amdgcn_global_load_lds((gbl_ptr_t)src, (lds_ptr_t)(smem + off), 16, 0, 0);
    }
  };

  typedef typename std::conditional<OP == OP_I8, v16i, v16f>::type acc32_t;
  typedef typename std::conditional<OP == OP_I8, v4i, v4f>::type acc16_t;
  typedef typename std::conditional<C::MI == 32, acc32_t, acc16_t>::type acc_t;
  constexpr int ACC_REGS = C::MI == 32 ? 16 : 4;
  acc_t acc[C::TN][C::TM];

  int b_row[C::TN];
#pragma unroll
  for (int j = 0; j < C::TN; j++) {
    if (C::GLU) {
      constexpr int H = C::TN / 2;
      b_row[j] = (j < H ? 0 : C::BN / 2) + wn * (C::WN / 2) + (j < H ? j : j - H) * C::MI;
    } else {
      b_row[j] = wn * C::WN + j * C::MI;
    }
  }
  // fragment of k-step ks: row (lane % 32), chunk q = 2*ks + lane/32, stored at slot q ^ swz(row)
  const int lrow = lane % 32;
  const int t16 = ((lane / 32) ^ C::swz(lrow)) * 16;
  const int row_off = lrow * C::BKB;

  // Fragments are double-buffered in registers: while the MFMAs of k-step ks run, the b128 reads of the
  // next k-step (possibly the first one of the next stage) are in flight.  LDS reads and global->LDS
  // requests are issued one at a time between MFMAs: a wave issues in order, so a burst of 4 loads + 6 reads
  // from all 8 waves right after the barrier would park every wave behind the address queues while the
  // MFMA pipes run dry.
  v4i fa[2][C::TM], fb[2][C::TN];
  auto read_frag = [&](int buf, int ks, int set, int f) {
    const int koff = t16 ^ (ks * 32);
    if (f < C::TM) {
      fa[set][f] = *(const v4i*)(smem + buf * C::STAGE + (wm * C::WM + f * 32) * C::BKB + row_off + koff);
    } else {
      fb[set][f - C::TM] = *(const v4i*)(smem + buf * C::STAGE + (C::BM + b_row[f - C::TM]) * C::BKB + row_off + koff);
    }
  };
  auto mfma_one = [&](int set, int idx) {
    const int j = idx / C::TM, i = idx % C::TM;
    if constexpr (C::MI != 32) {
      return;  // the 16 x 16 pipeline has its own k-step below
    } else if constexpr (OP == OP_I8) {
      acc[j][i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(fb[set][j], fa[set][i], acc[j][i], 0, 0, 0);
    } else {
      acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(
          __builtin_bit_cast(v8bf, fb[set][j]), __builtin_bit_cast(v8bf, fa[set][i]), acc[j][i], 0, 0, 0);
    }
  };
  constexpr int NMFMA = C::TM * C::TN, NFRAG = C::TM + C::TN;
  constexpr int HALF = C::LPS / 2;  // 64-byte stages: a stage's requests are split over two k-steps
  static_assert(NFRAG <= NMFMA && C::LPS % 2 == 0 && (C::MI == 16 || HALF <= NMFMA / 2), "interleave shape");
  // One k-step: MFMAs on register set SET with, slotted between them, the fragment reads of the next
  // k-step (RD) and HALF of a stage's requests (LD).  SET / RD / LD are compile-time so that the body is
  // straight-line code.
  auto kstep = [&](auto set_c, auto rd_c, auto ld_c, int rd_buf, int rd_ks, int ld_kt, int ld_buf, int ld_first) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value;
#pragma unroll
    for (int idx = 0; idx < NMFMA; idx++) {
      mfma_one(SET, idx);
      if (RD && idx < NFRAG) read_frag(rd_buf, rd_ks, SET ^ 1, idx);
      if (LD && (idx & 1) && idx / 2 < HALF) issue_one(ld_kt, ld_buf, ld_first + idx / 2);
      __builtin_amdgcn_sched_barrier(0);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): long satisfied by the time the last MFMA has issued
    __builtin_amdgcn_sched_barrier(0);
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // ---- the 16 x 16 instructions (16x16x64 i8, 16x16x32 bf16): 64 bytes of K per row and k-step, two k-steps per
  // 128-byte stage.  On changing operands the chip sustains about a fifth more of these than of the 32 x 32 ones
  // (a quarter of the accumulator registers read and written per instruction at half the work: the matrix pipes run
  // against the power limit, not the issue rate).  A wave's 128 x 64 tile takes 8 activation and 4 weight fragments
  // per k-step for 32 MFMAs.  The weight fragments are double-buffered; an activation fragment is reloaded for the
  // next k-step right after the four MFMAs that use it, so 12 fragments stay in registers instead of 24.
  // fragment of k-step ks: row (lane % 16), chunk q = 4*ks + lane/16, stored at slot q ^ swz(row)
  const int t16m = ((lane / 16) ^ C::swz(lane % 16)) * 16;
  const int row_off_m = (lane % 16) * C::BKB;
  v4i ga[C::TM], gb[2][C::TN];
  auto read_a16 = [&](int buf, int ks, int i) {
    ga[i] = *(const v4i*)(smem + buf * C::STAGE + (wm * C::WM + i * 16) * C::BKB + row_off_m + (t16m ^ (ks * 64)));
  };
  // [G, K, N] weights: the stage holds 64 rows of 512 bytes; lane (group gq, s16) addresses row 8 * gq + s16 / 4 (+ 4)
  // of the k-step's 32 rows and the 8 bytes 8 * (s16 % 4) of the fragment's 32-byte row slice; fragment j of the wave is
  // 32 * j bytes further along the row before the swizzle, which turns the step into an XOR of address bits 5 and 6
  const int kn_gq = lane / 16, kn_s16 = lane % 16;
  const int kn_base = (kn_gq * 8 + kn_s16 / 4) * (C::BN * 2) +
                      ((((8 * wn + (kn_s16 % 4) / 2) ^ (((kn_s16 / 4) << 2) ^ ((kn_gq & 1) << 1))) << 4) | ((kn_s16 & 1) << 3));
  auto read_b16 = [&](int buf, int ks, int set, int j) {
    if constexpr (C::RHS_KN) {
      int base = kn_base;
      asm volatile("" : "+v"(base));  // the address is formed here, not kept in a register across the loop
      gb[set][j] = __builtin_bit_cast(v4i, tr_read_frag(smem + buf * C::STAGE + C::BM * C::BKB + ks * 32 * (C::BN * 2) + (base ^ (32 * j)), C::BN * 2));
    } else {
      gb[set][j] = *(const v4i*)(smem + buf * C::STAGE + (C::BM + b_row[j]) * C::BKB + row_off_m + (t16m ^ (ks * 64)));
    }
  };
  auto kstep16 = [&](auto set_c, auto rd_c, auto ld_c, int rd_buf, int rd_ks, int ld_kt, int ld_buf) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value;
    if constexpr (C::MI == 16) {
#pragma unroll
      for (int i = 0; i < C::TM; i++) {
#pragma unroll
        for (int j = 0; j < C::TN; j++) {
          if constexpr (OP == OP_I8) {
            acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(gb[SET][j], ga[i], acc[j][i], 0, 0, 0);
          } else {
            acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(
                __builtin_bit_cast(v8bf, gb[SET][j]), __builtin_bit_cast(v8bf, ga[i]), acc[j][i], 0, 0, 0);
          }
          // the stage's requests go out one per MFMA from the start of the k-step: they have until the middle of the
          // next stage to land, and spreading them over the whole k-step measured 5 % slower
          if (LD && i * C::TN + j < C::LPS) issue_one(ld_kt, ld_buf, i * C::TN + j);
          if (RD && j == 1 && i < C::TN) read_b16(rd_buf, rd_ks, SET ^ 1, i);
          if (RD && j == C::TN - 1) read_a16(rd_buf, rd_ks, i);
          __builtin_amdgcn_sched_barrier(0);
        }
      }
    }
  };

  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;
  static_assert((C::MI == 32 && C::NSTAGE >= 3) || (C::MI == 16 && C::NSTAGE == 2), "pipeline shape");
  const int nk = K / C::BK;

  // Requests of a tile's first stages: stages 0..NSTAGE-3 in full and the first half of stage NSTAGE-2.
  auto issue_prologue = [&]() {
    if constexpr (C::MI == 16) {  // two buffers: both of the tile's first stages
#pragma unroll
      for (int s = 0; s < 2; s++)
#pragma unroll
        for (int i = 0; i < C::LPS; i++) issue_one(min(s, nk - 1), s, i);
      return;
    }
#pragma unroll
    for (int s = 0; s < C::NSTAGE - 2; s++)
#pragma unroll
      for (int i = 0; i < C::LPS; i++) issue_one(min(s, nk - 1), s, i);
#pragma unroll
    for (int i = 0; i < HALF; i++) issue_one(min(C::NSTAGE - 2, nk - 1), C::NSTAGE - 2, i);
  };

  // ---- pipeline -----------------------------------------------------------------------------------
  // A stage's requests are issued in two halves: the first during the last k-step of iteration kt (right
  // after the barrier that proves buffer (kt-1) % NSTAGE free), the second during the first k-step of
  // iteration kt+1.  Before the last k-step of iteration kt the wave waits for its own loads of stage
  // kt+1 and meets the others at a bare barrier: stage kt+1 is then complete in LDS and nobody reads stage
  // kt-1's buffer any more.  __syncthreads() is not used: its fence would drain vmcnt to 0 and with it the
  // loads that are meant to stay in flight.  Requests past the last stage re-read the last stage into a
  // buffer nobody reads again, which keeps the vmcnt bookkeeping uniform.
  // Across tiles: once a tile's last k-step has been issued, the first stages of the block's next tile are
  // requested, so they travel while the epilogue of the finished tile runs.
  int id = blockIdx.x;
  Tile cur;
  bool have = next_compute_tile(id, cur);
  if (have) {
    set_sources(cur);
    issue_prologue();
  }
  while (have) {
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int r = 0; r < ACC_REGS; r++) acc[j][i][r] = 0;
    // every request of the prologue (and every store of the previous epilogue) has completed
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    if constexpr (C::MI == 16) {
#pragma unroll
      for (int i = 0; i < C::TM; i++) read_a16(0, 0, i);
#pragma unroll
      for (int j = 0; j < C::TN; j++) read_b16(0, 0, 0, j);
    } else {
#pragma unroll
      for (int f = 0; f < NFRAG; f++) read_frag(0, 0, 0, f);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the loop is entered with no LDS read pending
    int kt = 0;
    const int n_out0 = cur.n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
    EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
    if constexpr (C::MI == 16) {
      // 128-byte stages, two buffers, stage kt in buffer kt % 2.  During a stage's first k-step the fragments of its
      // second one are read, after which no wave needs the buffer any more: once every wave has seen its own reads
      // return and its requests of stage kt+1 land, the block meets, and during the second k-step the fragments of
      // stage kt+1 are read from the other buffer while stage kt+2 is requested into this one.  A request carries a
      // whole 128-byte line: the L1 keeps a fixed number of requests in flight whatever their size.  The loop is cut
      // at the meeting point, where no LDS read may be pending anyway.
      kstep16(S0{}, T_{}, F_{}, 0, 1, 0, 0);
      for (; kt + 1 < nk; kt++) {
        const int buf = kt % 2;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        wait_vmcnt<0>();
        asm volatile("s_barrier" ::: "memory");
        kstep16(S1{}, T_{}, T_{}, buf ^ 1, 0, min(kt + 2, nk - 1), buf);
        kstep16(S0{}, T_{}, F_{}, buf ^ 1, 1, 0, 0);
      }
      load_epilogue_scales<C::TM, NT_OUT, C::GLU, true, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane);
      kstep16(S1{}, F_{}, F_{}, 0, 0, 0, 0);
    } else {
    for (; kt + 1 < nk; kt++) {
      const int buf = kt % C::NSTAGE;
      const int kb = kt + C::NSTAGE - 2, ka = kt + C::NSTAGE - 1;
      kstep(S0{}, T_{}, T_{}, buf, 1, min(kb, nk - 1), kb % C::NSTAGE, HALF);
      wait_vmcnt<(C::NSTAGE - 3) * C::LPS>();
      asm volatile("s_barrier" ::: "memory");
      kstep(S1{}, T_{}, T_{}, (kt + 1) % C::NSTAGE, 0, min(ka, nk - 1), ka % C::NSTAGE, 0);
    }
    // the epilogue's scales are fetched behind the last two k-steps
    load_epilogue_scales<C::TM, NT_OUT, C::GLU, true, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane);
    kstep(S0{}, T_{}, F_{}, kt % C::NSTAGE, 1, 0, 0, 0);
    kstep(S1{}, F_{}, F_{}, 0, 0, 0, 0, 0);
    }
    // all LDS reads of this tile are done in every wave and no request is still writing LDS: the buffers
    // can take the next tile's first stages
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    const Tile done = cur;
    id += gridDim.x;
    have = next_compute_tile(id, cur);
    if (have) {
      set_sources(cur);
      issue_prologue();
    }
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, done.info, wm * C::WM, n_out0, lane);
  }
  wait_vmcnt<0>();
}

// ---------------------------------------------------------------------------------------
// Block-scaled fp8 for few rows per expert.  One wave = 16 output channels x (16*MT) rows x all K.
// Weights and activations are read straight from global memory (activations hit in L2: every
// wave of a tile reads the same rows); nothing is shared between waves, so there are no barriers.
// ---------------------------------------------------------------------------------------

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
  uint16_t* out;
  int M, K, N;
  int n_blocks;  // blocks along N
  int min_rows, max_rows;  // only tiles with min_rows <= nrows <= max_rows are computed by this launch
  int act;
  float act_limit;
};

// Activation fragment of one 128-byte k-block: lane (j, kq) takes bytes kq*16.. and 64+kq*16.. of its row,
// the k order load_w128 leaves the weights in.
__device__ __forceinline__ v8i load_a128(const uint8_t* p) {
  const uint4 a = *(const uint4*)p, b = *(const uint4*)(p + 64);
  v8i r;
  r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w;
  r[4] = b.x; r[5] = b.y; r[6] = b.z; r[7] = b.w;
  return r;
}

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

template <bool STREAM>
__device__ __forceinline__ v8i load_w128(const uint8_t* lo_rows, const uint8_t* hi_rows) {
  const v4i a = load_w16<STREAM>(lo_rows), b = load_w16<STREAM>(hi_rows);
  v4i x, y;
  own_channel_pieces(a, b, x, y);
  v8i r;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    r[c] = x[c];
    r[4 + c] = y[c];
  }
  return r;
}

// One wave owns NT tiles of 16 output channels (x2 with GLU) and MT tiles of 16 rows, and walks K in
// steps of U 128-byte blocks whose loads are all issued before the first MFMA of the step.
template <int MT, int NT, int U, bool GLU>
__global__ __launch_bounds__(256) void gmm_fp8_skinny_kernel(const SkinnyParams p) {
  const int lane = threadIdx.x % kWave, wave = threadIdx.x / kWave;
  const int j = lane % 16, kq = lane / 16;
  const int m_idx = blockIdx.x / p.n_blocks;
  // the slot exists even when the tile does not (the list is sized for the worst case): both loads go out
  // together instead of one after the other
  const TileInfo tile = p.tiles[m_idx];
  if (m_idx >= p.header[0]) return;
  if (tile.group >= 0 ? (tile.nrows < p.min_rows || tile.nrows > p.max_rows) : p.min_rows > 1) return;
  const int N = p.N, K = p.K;
  constexpr int WN = 16 * NT;  // channels per wave
  const int n_w = (blockIdx.x % p.n_blocks) * (4 * WN) + wave * WN;
  if (n_w >= N) return;

  if (tile.group < 0) {
    for (int i = lane; i < tile.nrows * (WN / 4); i += kWave) {
      int r = i / (WN / 4), c = n_w + (i % (WN / 4)) * 4;
      if (c < N) *(uint2*)(p.out + (size_t)(tile.row0 + r) * N + c) = make_uint2(0, 0);
    }
    return;
  }

  const int nkb = K / 128;
  const int nnb = (N + 127) / 128;
  // offsets inside the expert's [N, K] matrix (the host checks N * K < 2^31), shared by rhs and rhs_up
  const uint8_t* wbase = p.rhs + (size_t)tile.group * N * K;
  const uint8_t* ubase = GLU ? p.rhs_up + (size_t)tile.group * N * K : nullptr;
  uint32_t wlo[NT], whi[NT];
  const float* wsp[NT];
  const float* usp[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int n16 = n_w + t * 16;
    const uint32_t in_line = (uint32_t)((j / 8) * 64 + kq * 16);
    wlo[t] = (uint32_t)min(n16 + j % 8, N - 1) * (uint32_t)K + in_line;
    whi[t] = (uint32_t)min(n16 + j % 8 + 8, N - 1) * (uint32_t)K + in_line;
    const size_t srow = ((size_t)tile.group * nnb + min(n16, N - 1) / 128) * nkb;
    wsp[t] = p.rhs_scale + srow;
    usp[t] = GLU ? p.rhs_up_scale + srow : nullptr;
  }
  const uint8_t* ap[MT];
  const float* asp[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int gr = tile.row0 + min(mt * 16 + j, tile.nrows - 1);
    ap[mt] = p.lhs + (size_t)gr * K + kq * 16;
    asp[mt] = p.lhs_scale + (size_t)gr * nkb;
  }
  v4f acc_g[NT][MT], acc_u[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      acc_g[t][mt] = v4f{0.f, 0.f, 0.f, 0.f};
      acc_u[t][mt] = v4f{0.f, 0.f, 0.f, 0.f};
    }
  const v4f zero = {0.f, 0.f, 0.f, 0.f};

  auto step = [&](int kb0, auto ucount) {
    constexpr int UC = decltype(ucount)::value;
    v8i wf[UC][NT], uf[UC][NT], af[UC][MT];
    float ws[UC][NT], us[UC][NT], as[UC][MT];
#pragma unroll
    for (int u = 0; u < UC; u++) {
      const size_t off = (size_t)(kb0 + u) * 128;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        wf[u][t] = load_w128<MT == 1>(wbase + wlo[t] + off, wbase + whi[t] + off);
        if (GLU) uf[u][t] = load_w128<MT == 1>(ubase + wlo[t] + off, ubase + whi[t] + off);
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) af[u][mt] = load_a128(ap[mt] + off);
    }
#pragma unroll
    for (int u = 0; u < UC; u++) {
#pragma unroll
      for (int t = 0; t < NT; t++) {
        ws[u][t] = wsp[t][kb0 + u];
        us[u][t] = GLU ? usp[t][kb0 + u] : 0.f;
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) as[u][mt] = asp[mt][kb0 + u];
    }
#pragma unroll
    for (int u = 0; u < UC; u++)
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          const v4f pg = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf[u][t], af[u][mt], zero, 0, 0, 0, 127, 0, 127);
          const float sg = as[u][mt] * ws[u][t];
#pragma unroll
          for (int r = 0; r < 4; r++) acc_g[t][mt][r] = fmaf(pg[r], sg, acc_g[t][mt][r]);
          if (GLU) {
            const v4f pu = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(uf[u][t], af[u][mt], zero, 0, 0, 0, 127, 0, 127);
            const float su = as[u][mt] * us[u][t];
#pragma unroll
            for (int r = 0; r < 4; r++) acc_u[t][mt][r] = fmaf(pu[r], su, acc_u[t][mt][r]);
          }
        }
  };

  int kb = 0;
  for (; kb + U <= nkb; kb += U) step(kb, std::integral_constant<int, U>{});
  for (; kb < nkb; kb++) step(kb, std::integral_constant<int, 1>{});

  dispatch_act(GLU ? p.act : MOE_ACT_NONE, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const int n = n_w + t * 16 + 4 * kq;
      if (n >= N) continue;
      float bg[4], bu[4];
      load_bias4(p.rhs_bias, tile.group, N, n, bg);
      load_bias4(GLU ? p.rhs_up_bias : nullptr, tile.group, N, n, bu);
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int lr = mt * 16 + j;
        if (lr >= tile.nrows) continue;
        float pg[4] = {bg[0], bg[1], bg[2], bg[3]}, pu[4] = {bu[0], bu[1], bu[2], bu[3]};
        add_partial4(p.partial_sum, (size_t)(tile.row0 + lr), N, n, pg);
        add_partial4(GLU ? p.partial_sum_up : nullptr, (size_t)(tile.row0 + lr), N, n, pu);
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; r++)
          v[r] = GLU ? glu_act<ACT>(acc_g[t][mt][r] + pg[r], acc_u[t][mt][r] + pu[r], p.act_limit) : acc_g[t][mt][r] + pg[r];
        *(uint2*)(p.out + (size_t)(tile.row0 + lr) * N + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      }
    }
  });
}

// ---------------------------------------------------------------------------------------
// Block-scaled fp8 for many rows per expert (prefill, training batches).  A block owns BM rows x 128 weight
// rows (with GLU: 64 gate + 64 up channels) and walks K in stages of one 128-wide scale block.  Operands go
// global -> LDS with global_load_lds_dwordx4 (8 rows x 128 bytes per wave instruction, the 16-byte chunk q of
// row r stored at slot q ^ ((r >> 1) & 7) so that fragment reads are conflict free), NSTAGE buffers deep.
// A wave owns 64 rows x 64 weight rows: per stage and 32 x 32 tile two chained v_mfma_f32_32x32x64_f8f6f4
// produce the block's partial sum, which is multiplied by a_scale[row, kb] * w_scale[n / 128, kb] and added to
// the f32 result: with weights as the "A" operand a lane holds one row of the tile, so the factor is one
// scalar per lane and tile.  Two waves per SIMD take turns on the matrix pipe, which hides the scaling FMAs
// of one behind the MFMAs of the other.
// ---------------------------------------------------------------------------------------

struct Fp8TiledParams {
  TiledParams base;        // lhs / rhs / rhs_up fp8; its scale pointers stay NULL (the epilogue applies none)
  const float* a_scale;    // [M, K/128]
  const float* w_scale;    // [G, ceil(N/128), K/128]
  const float* u_scale;
};

template <int BM_, int BKB_, int NSTAGE_, bool GLU_, bool VEC4_>
struct F8Cfg {
  static constexpr int BM = BM_, BN = 128, BKB = BKB_, NSTAGE = NSTAGE_;
  static constexpr bool GLU = GLU_, VEC4 = VEC4_;  // VEC4: a_scale is read four K blocks per load (K / 128 % 4 == 0)
  static constexpr int WAVES_M = BM / 64, WAVES_N = 2, NWAVES = WAVES_M * WAVES_N, THREADS = NWAVES * kWave;
  static constexpr int TM = 2, TN = 2;
  static constexpr int CPR = BKB / 16;     // 16-byte chunks per LDS row
  static constexpr int RPI = 1024 / BKB;   // rows per wave instruction
  static constexpr int SUBS = BKB / 64;    // MFMA k-steps (64 bytes of K) per stage
  static constexpr int A_IPW = BM / RPI / NWAVES, B_IPW = BN / RPI / NWAVES, LPS = A_IPW + B_IPW;
  static constexpr int STAGE = (BM + BN) * BKB;
  static constexpr int LDS_BYTES = NSTAGE * STAGE;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(BM == 128 || BM == 256, "row tile");
  static_assert(BKB == 64 || BKB == 128, "stage depth");
  static_assert(NSTAGE >= 2 && (NSTAGE - 2) * LPS < 64, "vmcnt range");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS");
  __device__ static __forceinline__ int swz(int row) { return BKB == 128 ? (row >> 1) & 7 : (row >> 2) & 3; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_fp8_tiled_kernel(const Fp8TiledParams P) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const TiledParams& p = P.base;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const int nkb = K / 128;          // scale blocks
  const int nst = K / C::BKB;       // stages

  // block -> (m-tile, n-tile): ids that run at the same time on one XCD (ids congruent mod 8) form a patch of
  // 4 m-tiles x 8 n-tiles that shares activation and weight panels in that XCD's L2
  const int total = p.max_m_tiles * p.tiles_n;
  TileInfo tile;
  int n0;
  {
    const int id = blockIdx.x;
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(p.max_m_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    n0 = ((logical % width) / gsz) * C::OUT_BN;
    tile = p.tiles[m_idx];  // the slot exists even when the tile does not
    if (m_idx >= p.header[0]) return;
  }
  if (tile.group < 0) {
    constexpr int QPR = C::OUT_BN / 4;
    for (int i = tid; i < tile.nrows * QPR; i += C::THREADS) {
      const int r = i / QPR, c = n0 + (i % QPR) * 4;
      if (c < N) *(uint2*)(p.out + (size_t)(tile.row0 + r) * N + c) = make_uint2(0, 0);
    }
    return;
  }

  // ---- per-lane sources of this wave's requests: lane l asks for row l / CPR, chunk (l % CPR) ^ swz(row) ----
  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
#pragma unroll
  for (int i = 0; i < C::A_IPW; i++) {
    const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(r);
    a_src[i] = p.lhs + (size_t)(tile.row0 + min(r, tile.nrows - 1)) * K + q * 16;
  }
#pragma unroll
  for (int i = 0; i < C::B_IPW; i++) {
    const int vr = (wave * C::B_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(vr);
    const bool up = C::GLU && vr >= C::BN / 2;
    const int n = min(n0 + (up ? vr - C::BN / 2 : vr), N - 1);
    b_src[i] = (up ? p.rhs_up : p.rhs) + ((size_t)tile.group * N + n) * K + q * 16;
  }
  auto issue_stage = [&](int kt, int buf) {
    const size_t koff = (size_t)kt * C::BKB;
    uint8_t* st = smem + buf * C::STAGE;
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++)
      __builtin_amdgcn_global_load_lds((gbl_ptr_t)(a_src[i] + koff), (lds_ptr_t)(st + (wave * C::A_IPW + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < C::B_IPW; i++)
      __builtin_amdgcn_global_load_lds((gbl_ptr_t)(b_src[i] + koff),
                                       (lds_ptr_t)(st + C::BM * C::BKB + (wave * C::B_IPW + i) * 1024), 16, 0, 0);
  };

  // ---- fragments: lane (row = lane % 32, kq = lane / 32) takes chunks 4h + 2kq, 4h + 2kq + 1 of k-step h ----
  const int lrow = lane % 32, kq = lane / 32, sw = C::swz(lrow);
  int choff[C::SUBS][2];
#pragma unroll
  for (int h = 0; h < C::SUBS; h++)
#pragma unroll
    for (int e = 0; e < 2; e++) choff[h][e] = lrow * C::BKB + (((4 * h + 2 * kq + e) ^ sw) * 16);
  int w_row[2];  // first LDS row of this wave's two weight tiles
  if (C::GLU) {
    w_row[0] = wn * 32;
    w_row[1] = C::BN / 2 + wn * 32;
  } else {
    w_row[0] = wn * 64;
    w_row[1] = wn * 64 + 32;
  }
  auto frag = [&](const uint8_t* base, int h) {
    const v4i a = *(const v4i*)(base + choff[h][0]), b = *(const v4i*)(base + choff[h][1]);
    v8i r;
    r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
    r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
    return r;
  };

  // ---- block scales ---------------------------------------------------------------------------------------
  const float* as_ptr[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int lr = wm * 64 + i * 32 + lrow;
    as_ptr[i] = P.a_scale + (size_t)(tile.row0 + min(lr, tile.nrows - 1)) * nkb;
  }
  const int nnb = (N + 127) / 128;
  const int n_out0 = n0 + (C::GLU ? wn * 32 : wn * 64);
  // both weight tiles of a wave lie in one 128-channel block (gate and up have tensors of their own)
  const float* ws_ptr[2];
  ws_ptr[0] = P.w_scale + ((size_t)tile.group * nnb + min(n_out0, N - 1) / 128) * nkb;
  ws_ptr[1] = C::GLU ? P.u_scale + ((size_t)tile.group * nnb + min(n_out0, N - 1) / 128) * nkb
                     : P.w_scale + ((size_t)tile.group * nnb + min(n_out0 + 32, N - 1) / 128) * nkb;

  v16f fin[2][2];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) fin[j][i][r] = 0.f;
  const v16f zero = fin[0][0];

  // ---- pipeline: stage kt is multiplied while stages kt+1 .. kt+NSTAGE-1 travel ---------------------------
  // The partial sum of a 128-wide K block (two k-steps) stays in `part` until the next block starts: each
  // tile's scaling FMAs are issued right before that tile's first MFMA of the next block, so they run in the
  // shadow of the previous tile's MFMAs.
  v16f part[2][2];
  float sc[2][2];
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++) {
      part[j][i] = zero;
      sc[j][i] = 0.f;
    }
  // a_scale: a lane's row differs from its neighbours', so a load touches 32 lines whatever its width; reading four K
  // blocks per load cuts the number of these loads by four.  The group buffer is refilled once its last value is taken.
  constexpr int GRP = C::VEC4 ? 4 : 1;
  float as_grp[2][GRP];
  auto load_a_scales = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      if constexpr (C::VEC4) {
        const float4 v = *(const float4*)(as_ptr[i] + kb);
        as_grp[i][0] = v.x; as_grp[i][1] = v.y; as_grp[i][2] = v.z; as_grp[i][3] = v.w;
      } else {
        as_grp[i][0] = as_ptr[i][kb];
      }
    }
  };
  load_a_scales(0);
  float as_cur[2];
  float ws_cur[2] = {ws_ptr[0][0], ws_ptr[1][0]};
#pragma unroll
  for (int s = 0; s < C::NSTAGE - 1; s++) issue_stage(min(s, nst - 1), s);

  // Opening stage kt: own requests of stage kt have landed (the newest NSTAGE-2 stages may still travel), then
  // everybody's have, and nobody reads stage kt-1 any more, so its buffer takes stage kt+NSTAGE-1.  The scales of
  // the NEXT K block are requested between the barrier and those requests: in vmcnt order they are then older than
  // the requests that stay in flight, so neither the wait of the next stage nor the compiler's wait for the scale
  // registers has to drain a stage that is still travelling.
  float ws_next[2];
  auto open_stage = [&](int kt, int next_kb, int next_group_kb) {
    wait_vmcnt<(C::NSTAGE - 2) * C::LPS>();
    asm volatile("s_barrier" ::: "memory");
    if (next_group_kb >= 0) load_a_scales(next_group_kb);
    if (next_kb >= 0) {
      ws_next[0] = ws_ptr[0][next_kb];
      ws_next[1] = ws_ptr[1][next_kb];
    }
    asm volatile("" ::: "memory");
    const int kl = kt + C::NSTAGE - 1;
    issue_stage(min(kl, nst - 1), kl % C::NSTAGE);
  };
  // one k-step (64 bytes of K) of all four tiles; FIRST: it opens a scale block
  auto kstep = [&](const uint8_t* st, int h, auto first_c) {
    constexpr bool FIRST = decltype(first_c)::value;
    v8i tf[2], wf[2];
#pragma unroll
    for (int i = 0; i < 2; i++) tf[i] = frag(st + (wm * 64 + i * 32) * C::BKB, h);
#pragma unroll
    for (int j = 0; j < 2; j++) wf[j] = frag(st + (C::BM + w_row[j]) * C::BKB, h);
#pragma unroll
    for (int j = 0; j < 2; j++)
#pragma unroll
      for (int i = 0; i < 2; i++) {
        if (FIRST) {
#pragma unroll
          for (int r = 0; r < 16; r++) fin[j][i][r] = fmaf(part[j][i][r], sc[j][i], fin[j][i][r]);
          sc[j][i] = as_cur[i] * ws_cur[j];
        }
        part[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j], tf[i], FIRST ? zero : part[j][i], 0, 0, 0, 127, 0, 127);
      }
  };
  static_assert(C::SUBS == 2, "a stage is one scale block");
  for (int kb = 0; kb < nkb; kb++) {
    const int kn = min(kb + 1, nkb - 1);
    const int c = C::VEC4 ? (kb & 3) : 0;  // uniform: which value of the group this block uses
#pragma unroll
    for (int i = 0; i < 2; i++) {
      as_cur[i] = as_grp[i][0];
      if constexpr (C::VEC4) as_cur[i] = c == 0 ? as_grp[i][0] : (c == 1 ? as_grp[i][1] : (c == 2 ? as_grp[i][2] : as_grp[i][3]));
    }
    open_stage(kb, kn, c == GRP - 1 ? min(kb + 1, nkb - GRP) : -1);
    const uint8_t* st = smem + (kb % C::NSTAGE) * C::STAGE;
    kstep(st, 0, std::true_type{});
    kstep(st, 1, std::false_type{});
    ws_cur[0] = ws_next[0];
    ws_cur[1] = ws_next[1];
  }
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) fin[j][i][r] = fmaf(part[j][i][r], sc[j][i], fin[j][i][r]);
  wait_vmcnt<0>();  // the last requests re-read the final stage into a buffer nobody reads

  constexpr int NT_OUT = C::GLU ? 1 : 2;
  EpilogueScales<2, NT_OUT, C::GLU> esc;
  load_epilogue_scales<2, NT_OUT, C::GLU, false>(esc, p, tile, wm * 64, n_out0, lane);
  store_epilogue<2, 2, NT_OUT, C::GLU>(fin, esc, p, tile, wm * 64, n_out0, lane);
}

// ---------------------------------------------------------------------------------------
// Block-scaled fp8, 256 x 256 tiles: half the operand bytes per flop of the 128 x 128 kernel above, which is
// what bounds that kernel.  A second set of accumulators for the per-block partial sums does not fit (a wave's
// 128 x 64 share of the tile is 128 registers), so there is ONE set, kept in units of the current block's scale:
// when K block kb starts the accumulators are multiplied by s[kb-1] / s[kb] (s = a_scale[row, kb] * w_scale[n/128, kb],
// one scalar per lane and tile) and the MFMAs of the block accumulate straight into them; the epilogue multiplies
// by the last block's scale.  sum_kb s[kb] P[kb] is unchanged, each block costs one more f32 rounding.  A block
// whose scale is zero (all-zero operands, so P = 0) keeps the previous unit.
// 8 waves (2 x 4), stages of one 128-byte scale block (the L1 keeps a fixed number of line requests in flight, so
// a request should carry a whole line), 2 buffers (128 KB), one block per CU; weights are the MFMA "A" operand.
// ---------------------------------------------------------------------------------------

template <bool GLU_, bool VEC4_>
struct F8BigCfg {
  static constexpr int BM = 256, BN = 256, BKB = 128, NSTAGE = 2;  // a stage is one scale block: 128-byte requests
  static constexpr bool GLU = GLU_, VEC4 = VEC4_;
  static constexpr int WAVES_M = 2, WAVES_N = 4, NWAVES = 8, THREADS = NWAVES * kWave;
  static constexpr int TM = 4, TN = 2;             // 32-row tiles of a wave: 128 rows x 64 weight rows
  static constexpr int CPR = BKB / 16, RPI = 1024 / BKB;
  static constexpr int A_IPW = BM / RPI / NWAVES, B_IPW = BN / RPI / NWAVES, LPS = A_IPW + B_IPW;
  static constexpr int STAGE = (BM + BN) * BKB;
  static constexpr int LDS_BYTES = NSTAGE * STAGE;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(LDS_BYTES <= 160 * 1024, "LDS");
  __device__ static __forceinline__ int swz(int row) { return (row >> 1) & 7; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_fp8_big_kernel(const Fp8TiledParams P) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const TiledParams& p = P.base;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const int nkb = K / 128, nst = K / C::BKB;

  // block -> (m-tile, n-tile): contiguous ids per XCD, super-rows of GSM m-tiles
  const int total = p.max_m_tiles * p.tiles_n;
  TileInfo tile;
  int n0;
  {
    const int id = blockIdx.x;
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(p.max_m_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    n0 = ((logical % width) / gsz) * C::OUT_BN;
    tile = p.tiles[m_idx];
    if (m_idx >= p.header[0]) return;
  }
  if (tile.group < 0) {
    constexpr int QPR = C::OUT_BN / 4;
    for (int i = tid; i < tile.nrows * QPR; i += C::THREADS) {
      const int r = i / QPR, c = n0 + (i % QPR) * 4;
      if (c < N) *(uint2*)(p.out + (size_t)(tile.row0 + r) * N + c) = make_uint2(0, 0);
    }
    return;
  }

  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
#pragma unroll
  for (int i = 0; i < C::A_IPW; i++) {
    const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(r);
    a_src[i] = p.lhs + (size_t)(tile.row0 + min(r, tile.nrows - 1)) * K + q * 16;
  }
#pragma unroll
  for (int i = 0; i < C::B_IPW; i++) {
    const int vr = (wave * C::B_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(vr);
    const bool up = C::GLU && vr >= C::BN / 2;
    const int n = min(n0 + (up ? vr - C::BN / 2 : vr), N - 1);
    b_src[i] = (up ? p.rhs_up : p.rhs) + ((size_t)tile.group * N + n) * K + q * 16;
  }
  auto issue_stage = [&](int kt, int buf) {
    const size_t koff = (size_t)kt * C::BKB;
    uint8_t* st = smem + buf * C::STAGE;
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++)
      __builtin_amdgcn_global_load_lds((gbl_ptr_t)(a_src[i] + koff), (lds_ptr_t)(st + (wave * C::A_IPW + i) * 1024), 16, 0, 0);
#pragma unroll
    for (int i = 0; i < C::B_IPW; i++)
      __builtin_amdgcn_global_load_lds((gbl_ptr_t)(b_src[i] + koff),
                                       (lds_ptr_t)(st + C::BM * C::BKB + (wave * C::B_IPW + i) * 1024), 16, 0, 0);
  };

  // fragment of a 32-row tile for k-step h (64 bytes of the 128-byte row): lane (row = lane % 32, kq = lane / 32)
  // takes chunks 4h + 2kq, 4h + 2kq + 1
  const int lrow = lane % 32, kq = lane / 32, sw = C::swz(lrow);
  int choff[2][2];
#pragma unroll
  for (int h = 0; h < 2; h++)
#pragma unroll
    for (int e = 0; e < 2; e++) choff[h][e] = lrow * C::BKB + (((4 * h + 2 * kq + e) ^ sw) * 16);
  auto frag = [&](const uint8_t* base, int h) {
    const v4i a = *(const v4i*)(base + choff[h][0]), b = *(const v4i*)(base + choff[h][1]);
    v8i r;
    r[0] = a[0]; r[1] = a[1]; r[2] = a[2]; r[3] = a[3];
    r[4] = b[0]; r[5] = b[1]; r[6] = b[2]; r[7] = b[3];
    return r;
  };
  int w_row[2];
  if (C::GLU) {
    w_row[0] = wn * 32;
    w_row[1] = C::BN / 2 + wn * 32;
  } else {
    w_row[0] = wn * 64;
    w_row[1] = wn * 64 + 32;
  }

  // ---- block scales: a_scale per lane and row tile, w_scale per weight tile -----------------------------------
  const float* as_ptr[C::TM];
#pragma unroll
  for (int i = 0; i < C::TM; i++) {
    const int lr = wm * 128 + i * 32 + lrow;
    as_ptr[i] = P.a_scale + (size_t)(tile.row0 + min(lr, tile.nrows - 1)) * nkb;
  }
  const int nnb = (N + 127) / 128;
  const int n_out0 = n0 + (C::GLU ? wn * 32 : wn * 64);
  const float* ws_ptr[2];
  ws_ptr[0] = P.w_scale + ((size_t)tile.group * nnb + min(n_out0, N - 1) / 128) * nkb;
  ws_ptr[1] = C::GLU ? P.u_scale + ((size_t)tile.group * nnb + min(n_out0, N - 1) / 128) * nkb
                     : P.w_scale + ((size_t)tile.group * nnb + min(n_out0 + 32, N - 1) / 128) * nkb;

  v16f acc[C::TN][C::TM];
#pragma unroll
  for (int j = 0; j < C::TN; j++)
#pragma unroll
    for (int i = 0; i < C::TM; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][i][r] = 0.f;

  // unit of the accumulators (the scale of the last block that had one) per row tile / weight tile
  float ua[C::TM], uw[2];
#pragma unroll
  for (int i = 0; i < C::TM; i++) ua[i] = 1.0f;
  uw[0] = uw[1] = 1.0f;
#pragma unroll
  for (int s = 0; s < C::NSTAGE - 1; s++) issue_stage(min(s, nst - 1), s);

  // a_scale is read four K blocks at a time: a lane's row differs from its neighbours', so every such load touches
  // 32 lines whatever its width, and the wide load cuts their number by four (VEC4: K / 128 is a multiple of 4, which
  // also makes the 16-byte loads aligned).  The next group is requested between a barrier and the stage requests
  // that follow it: in vmcnt order it is then older than everything that stays in flight.
  constexpr int GRP = C::VEC4 ? 4 : 1;
  float as_next[C::TM][GRP];  // one buffer: the next group is requested once the last value of this one has been read
  float ws_next[2];
  auto load_a_scales = [&](float (&dst)[C::TM][GRP], int kb) {
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
      if constexpr (C::VEC4) {
        const float4 v = *(const float4*)(as_ptr[i] + kb);
        dst[i][0] = v.x; dst[i][1] = v.y; dst[i][2] = v.z; dst[i][3] = v.w;
      } else {
        dst[i][0] = as_ptr[i][kb];
      }
    }
  };
  load_a_scales(as_next, 0);
  ws_next[0] = ws_ptr[0][0];
  ws_next[1] = ws_ptr[1][0];

  auto open_stage = [&](int kt, int next_group_kb, int next_kb) {
    wait_vmcnt<(C::NSTAGE - 2) * C::LPS>();
    asm volatile("s_barrier" ::: "memory");
    if (next_group_kb >= 0) load_a_scales(as_next, next_group_kb);
    if (next_kb >= 0) {
      ws_next[0] = ws_ptr[0][next_kb];
      ws_next[1] = ws_ptr[1][next_kb];
    }
    asm volatile("" ::: "memory");
    const int kl = kt + C::NSTAGE - 1;
    issue_stage(min(kl, nst - 1), kl % C::NSTAGE);
  };
  auto kstep = [&](int kt, int h) {
    const uint8_t* st = smem + (kt % C::NSTAGE) * C::STAGE;
    v8i tf[C::TM], wf[C::TN];
#pragma unroll
    for (int i = 0; i < C::TM; i++) tf[i] = frag(st + (wm * 128 + i * 32) * C::BKB, h);
#pragma unroll
    for (int j = 0; j < C::TN; j++) wf[j] = frag(st + (C::BM + w_row[j]) * C::BKB, h);
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int i = 0; i < C::TM; i++)
        acc[j][i] = __builtin_amdgcn_mfma_scale_f32_32x32x64_f8f6f4(wf[j], tf[i], acc[j][i], 0, 0, 0, 127, 0, 127);
  };
  for (int kb = 0; kb < nkb; kb++) {
    const int c = C::VEC4 ? (kb & 3) : 0;  // uniform: which of the group's values this block uses
    // scales of this block; a zero scale keeps the unit
    float ra[C::TM], rw[2];
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
      float sc = as_next[i][0];
      if constexpr (C::VEC4) sc = c == 0 ? as_next[i][0] : (c == 1 ? as_next[i][1] : (c == 2 ? as_next[i][2] : as_next[i][3]));
      const float nu = sc != 0.f ? sc : ua[i];
      ra[i] = ua[i] / nu;
      ua[i] = nu;
    }
#pragma unroll
    for (int j = 0; j < 2; j++) {
      const float sc = ws_next[j];
      const float nu = sc != 0.f ? sc : uw[j];
      rw[j] = uw[j] / nu;
      uw[j] = nu;
    }
    // the group's last value has been read above: its buffer takes the next group
    open_stage(kb, c == GRP - 1 ? min(kb + 1, nkb - GRP) : -1, min(kb + 1, nkb - 1));
    if (kb > 0) {
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int i = 0; i < C::TM; i++) {
          const float r_ = ra[i] * rw[j];
#pragma unroll
          for (int r = 0; r < 16; r++) acc[j][i][r] *= r_;
        }
    }
    kstep(kb, 0);
    kstep(kb, 1);
  }
  wait_vmcnt<0>();  // the last requests re-read the final stage into a buffer nobody reads

  // the epilogue's row and channel scales are the accumulators' unit
  constexpr int NT_OUT = C::GLU ? 1 : 2;
  EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
#pragma unroll
  for (int i = 0; i < C::TM; i++) esc.sa[i] = ua[i];
#pragma unroll
  for (int j = 0; j < NT_OUT; j++)
#pragma unroll
    for (int q = 0; q < 4; q++) {
      esc.sg[j][q] = make_float4(uw[C::GLU ? 0 : j], uw[C::GLU ? 0 : j], uw[C::GLU ? 0 : j], uw[C::GLU ? 0 : j]);
      esc.su[j][q] = make_float4(uw[1], uw[1], uw[1], uw[1]);
    }
  store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, tile, wm * 128, n_out0, lane);
}

// ---------------------------------------------------------------------------------------
// Weight-only int8 / int4 for few rows per expert (decode): bf16 activations, weights widened to bf16 in
// registers, v_mfma_f32_16x16x32_bf16.  Same streaming structure as the fp8 kernel: no LDS, one wave owns
// 16*NT output channels and walks K in 128-element blocks; lane (n = lane%16, kq = lane/16) holds 32 k values
// of the block for its channel (4-bit: kq*32.. ; int8: kq*16.. and 64 + kq*16..) and the matching 64 bytes of
// its activation row.  int4 weights are multiplied by their group-128 scale while
// they are widened; the int8 per-channel scale is applied once at the end.
// ---------------------------------------------------------------------------------------

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
  uint16_t* out;
  int M, K, N;
  int n_blocks;
  int act;
  float act_limit;
};

// Raw weight bytes of one lane for one 128-wide k block: 32 values = 16 bytes (int4) or 32 bytes (int8).
enum { WQ_I8 = 0, WQ_I4 = 1, WQ_MX4 = 2, WQ_I4G32 = 3 };  // weight formats of the streaming kernel (int4: group 128 / 32)

template <int FMT>
struct WqRaw {
  uint4 q0, q1;
};

template <int FMT>
__device__ __forceinline__ void widen32(const WqRaw<FMT>& raw, float scale, v8bf (&w)[4]) {
  if (FMT == WQ_MX4) {  // e2m1 pairs -> bf16 pairs times the block scale, one instruction per byte
    const uint32_t x[4] = {raw.q0.x, raw.q0.y, raw.q0.z, raw.q0.w};
#pragma unroll
    for (int s = 0; s < 4; s++)
      w[s] = __builtin_bit_cast(v8bf, make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x[s], scale, 0)),
                                                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x[s], scale, 1)),
                                                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x[s], scale, 2)),
                                                 __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(x[s], scale, 3))));
  } else if (FMT == WQ_I4 || FMT == WQ_I4G32) {  // (nibble - 8) * scale rounded to bf16, as the reference dequantises
    const uint32_t x[4] = {raw.q0.x, raw.q0.y, raw.q0.z, raw.q0.w};
#pragma unroll
    for (int s = 0; s < 4; s++) {
      uint32_t o[4];
#pragma unroll
      for (int h = 0; h < 4; h++) {
        const int lo = (int)((x[s] >> (8 * h)) & 0xf) - 8, hi = (int)((x[s] >> (8 * h + 4)) & 0xf) - 8;
        o[h] = pack_bf16x2((float)lo * scale, (float)hi * scale);
      }
      w[s] = __builtin_bit_cast(v8bf, make_uint4(o[0], o[1], o[2], o[3]));
    }
  } else {
    const uint32_t x[8] = {raw.q0.x, raw.q0.y, raw.q0.z, raw.q0.w, raw.q1.x, raw.q1.y, raw.q1.z, raw.q1.w};
#pragma unroll
    for (int s = 0; s < 4; s++) {
      uint32_t o[4];
#pragma unroll
      for (int h = 0; h < 2; h++) {
        const int v = (int)x[2 * s + h];
        o[2 * h] = i8x2_to_bf16x2((v << 24) >> 24, (v << 16) >> 24);
        o[2 * h + 1] = i8x2_to_bf16x2((v << 8) >> 24, v >> 24);
      }
      w[s] = __builtin_bit_cast(v8bf, make_uint4(o[0], o[1], o[2], o[3]));
    }
  }
}

// A block of 4 waves owns (4 / KSPLIT) * 16*NT output channels of one m-tile; KSPLIT waves share a channel
// group, split K into contiguous ranges of 128-wide blocks and add their partial sums through LDS at the
// end (with few tiles, a wave walking all of K alone leaves the memory system idle: KSPLIT = 4 for a handful
// of tokens, 1 once there are enough blocks).  Within its range a wave works in rounds of U blocks whose loads
// are all issued before the first block is converted and multiplied; other resident waves cover the rest of the
// latency (holding two rounds in registers halves the occupancy and measures slower).
//
// Weight requests cover 128 contiguous bytes of 8 channels each (one k-block of int8, two of a 4-bit format), two
// requests per 16 channels, like load_w128 of the fp8 kernel; 4-bit formats therefore walk K in pairs of blocks
// (U even) and keep the k order inside a block, int8 gets the order (kq*16.., 64 + kq*16..) inside its block and
// reads its activations to match.
//
// LINE = false (4-bit formats only) is the plain form: one 16-byte request per lane and k-block, 64 bytes per
// channel per request, no exchange, any U.
template <int FMT, int MT, int NT, bool GLU, int U, int KSPLIT, bool STREAM, bool PREFETCH, bool LINE>
__global__ __launch_bounds__(256) void gmm_wq_skinny_kernel(const WqSkinnyParams p) {
  constexpr bool INT4 = FMT == WQ_I4, MX4 = FMT == WQ_MX4, G32 = FMT == WQ_I4G32, NIB = FMT != WQ_I8;
  static_assert(LINE || NIB, "int8 always uses whole-line requests");
  constexpr int UB = NIB && LINE ? 2 : 1;  // k-blocks per weight request pair
  static_assert(U % UB == 0, "4-bit formats are loaded in pairs of k-blocks");
  constexpr int NACC = NT * MT * 4 * (GLU ? 2 : 1);
  constexpr int NSUB = 4 / KSPLIT;  // channel groups per block
  __shared__ float red[KSPLIT > 1 ? NSUB * (KSPLIT - 1) * NACC * kWave : 1];
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int ksub = wave % KSPLIT, nsub = wave / KSPLIT;
  const int j = lane % 16, kq = lane / 16;
  const int m_idx = blockIdx.x / p.n_blocks;
  // the slot exists even when the tile does not (the list is sized for the worst case): both loads go out
  // together instead of one after the other
  const TileInfo tile = p.tiles[m_idx];
  if (m_idx >= p.header[0]) return;
  const int N = p.N, K = p.K;
  constexpr int WN = 16 * NT;
  const int n_b = (blockIdx.x % p.n_blocks) * (NSUB * WN);
  const int n_w = n_b + nsub * WN;

  if (tile.group < 0) {
    for (int i = threadIdx.x; i < tile.nrows * (NSUB * WN / 4); i += 256) {
      int r = i / (NSUB * WN / 4), c = n_b + (i % (NSUB * WN / 4)) * 4;
      if (c < N) *(uint2*)(p.out + (size_t)(tile.row0 + r) * N + c) = make_uint2(0, 0);
    }
    return;
  }
  // a channel group past N has nothing to do, but its waves still meet the others at the barrier below
  const bool idle = n_w >= N;

  const int nkb = (K + 127) / 128;  // the last block may be partial (K % 32 == 0)
  const size_t wrow_bytes = NIB ? (size_t)K / 2 : (size_t)K;
  // the expert's matrix (the host checks N * K < 2^31) and, inside it, the rows of this lane's two requests
  const uint8_t* wbase = p.rhs + (size_t)tile.group * N * wrow_bytes;
  const uint8_t* ubase = GLU ? p.rhs_up + (size_t)tile.group * N * wrow_bytes : nullptr;
  const int piece = j / 8;
  uint32_t wlo[NT], whi[NT];
  const uint16_t* wsp[NT];
  const uint16_t* usp[NT];
  const uint8_t* wmx[NT];
  const uint8_t* umx[NT];
#pragma unroll
  for (int t = 0; t < NT; t++) {
    const int nw = min(n_w + t * 16 + j, N - 1);
    const size_t row = (size_t)tile.group * N + nw;
    wlo[t] = (uint32_t)min(n_w + t * 16 + (LINE ? j % 8 : j), N - 1) * (uint32_t)wrow_bytes;
    whi[t] = (uint32_t)min(n_w + t * 16 + j % 8 + 8, N - 1) * (uint32_t)wrow_bytes;
    wsp[t] = INT4 ? (const uint16_t*)p.rhs_scale + row * nkb : nullptr;
    usp[t] = INT4 && GLU ? (const uint16_t*)p.rhs_up_scale + row * nkb : nullptr;
    // MXFP4: one e8m0 byte per 32 values = per lane and k block
    wmx[t] = MX4 ? (const uint8_t*)p.rhs_scale + row * (size_t)(K / 32) + kq : nullptr;
    umx[t] = MX4 && GLU ? (const uint8_t*)p.rhs_up_scale + row * (size_t)(K / 32) + kq : nullptr;
    // int4 with group 32: one bf16 scale per lane and k block, indexed like the MXFP4 byte
    if (G32) {
      wsp[t] = (const uint16_t*)p.rhs_scale + row * (size_t)(K / 32) + kq;
      usp[t] = GLU ? (const uint16_t*)p.rhs_up_scale + row * (size_t)(K / 32) + kq : nullptr;
    }
  }
  const uint8_t* ap[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int gr = tile.row0 + min(mt * 16 + j, tile.nrows - 1);
    ap[mt] = p.lhs + (size_t)gr * K * 2;  // row start
  }
  v4f acc_g[NT][MT], acc_u[NT][MT];
#pragma unroll
  for (int t = 0; t < NT; t++)
#pragma unroll
    for (int mt = 0; mt < MT; mt++) {
      acc_g[t][mt] = v4f{0.f, 0.f, 0.f, 0.f};
      acc_u[t][mt] = v4f{0.f, 0.f, 0.f, 0.f};
    }

  // One round = U k-blocks held as raw bytes.
  struct WRound {
    v4i wa[U / UB][NT], wb[U / UB][NT], ua[U / UB][NT], ub[U / UB][NT];  // the two requests of each unit
    uint16_t wsc[U][NT], usc[U][NT];
  };
  struct ARound {
    uint4 araw[U][MT][4];
    bool live[U][2];  // first / second 16 k values of the lane (int8; one flag for the 4-bit formats)
  };
  const int chunk = (nkb + KSPLIT * UB - 1) / (KSPLIT * UB) * UB;  // whole units
  const int kb_begin = ksub * chunk;
  const int kb_end = idle ? kb_begin : min(nkb, kb_begin + chunk);

  // Blocks past the end of the range are loaded from the range's last block and flagged dead (their activations
  // are zeroed before use), so every round has the same instruction stream.
  // k index of a block's first value for this lane, or of one of its two 16-value pieces with int8
  auto lane_k = [&](int kb, int half) { return NIB ? kb * 128 + kq * 32 : kb * 128 + half * 64 + kq * 16; };
  auto load_w = [&](WRound& r, int kb0) {
#pragma unroll
    for (int un = 0; un < U / UB; un++) {
      // the piece of the unit this lane asks for: a whole block of a 4-bit format, half a block of int8
      const int kbp_raw = kb0 + un * UB + (NIB && LINE ? piece : 0);
      const int kbp = kbp_raw < kb_end ? kbp_raw : max(kb_end - 1, 0);
      const int kp = lane_k(kbp, LINE ? piece : 0);
      const uint32_t woff = kp < K ? (uint32_t)(NIB ? kp / 2 : kp) : 0u;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        r.wa[un][t] = load_w16<STREAM>(wbase + wlo[t] + woff);
        if (LINE) r.wb[un][t] = load_w16<STREAM>(wbase + whi[t] + woff);
        if (GLU) {
          r.ua[un][t] = load_w16<STREAM>(ubase + wlo[t] + woff);
          if (LINE) r.ub[un][t] = load_w16<STREAM>(ubase + whi[t] + woff);
        }
      }
    }
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool in_range = kb0 + u < kb_end;
      const int kb = in_range ? kb0 + u : max(kb_end - 1, 0);
      const bool addr_ok = lane_k(kb, 0) < K;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        if (INT4) {
          r.wsc[u][t] = wsp[t][kb];
          if (GLU) r.usc[u][t] = usp[t][kb];
        }
        if (MX4) {
          r.wsc[u][t] = addr_ok ? wmx[t][kb * 4] : (uint16_t)127;
          if (GLU) r.usc[u][t] = addr_ok ? umx[t][kb * 4] : (uint16_t)127;
        }
        if (G32) {
          r.wsc[u][t] = addr_ok ? wsp[t][kb * 4] : (uint16_t)0;
          if (GLU) r.usc[u][t] = addr_ok ? usp[t][kb * 4] : (uint16_t)0;
        }
      }
    }
  };
  auto load_a = [&](ARound& r, int kb0) {
#pragma unroll
    for (int u = 0; u < U; u++) {
      const bool in_range = kb0 + u < kb_end;
      const int kb = in_range ? kb0 + u : max(kb_end - 1, 0);
      // this lane's k values exist unless the block is the partial tail
      const bool ok0 = lane_k(kb, 0) < K, ok1 = lane_k(kb, 1) < K;
      r.live[u][0] = in_range && ok0;
      r.live[u][1] = in_range && ok1;
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        // 4-bit formats: 64 contiguous bytes; int8: 32 bytes for each of the two pieces.  A piece past K reads the row start.
        const uint8_t* a0 = ap[mt] + (ok0 ? (size_t)lane_k(kb, 0) * 2 : 0);
        const uint8_t* a1 = NIB ? a0 + 32 : ap[mt] + (ok1 ? (size_t)lane_k(kb, 1) * 2 : 0);
        r.araw[u][mt][0] = *(const uint4*)a0;
        r.araw[u][mt][1] = *(const uint4*)(a0 + 16);
        r.araw[u][mt][2] = *(const uint4*)a1;
        r.araw[u][mt][3] = *(const uint4*)(a1 + 16);
      }
    }
  };

  auto compute_round = [&](const WRound& r, const ARound& ar) {
    const auto& araw = ar.araw;
    const auto& wsc = r.wsc;
    const auto& usc = r.usc;
    const auto& live = ar.live;
    WqRaw<FMT> wraw[U][NT], uraw[U][NT];
#pragma unroll
    for (int un = 0; un < U / UB; un++)
#pragma unroll
      for (int t = 0; t < NT; t++) {
        if constexpr (!LINE) {
          wraw[un][t].q0 = __builtin_bit_cast(uint4, r.wa[un][t]);
          if (GLU) uraw[un][t].q0 = __builtin_bit_cast(uint4, r.ua[un][t]);
        } else {
          v4i x, y;
          own_channel_pieces(r.wa[un][t], r.wb[un][t], x, y);
          wraw[un * UB][t].q0 = __builtin_bit_cast(uint4, x);
          (NIB ? wraw[un * UB + UB - 1][t].q0 : wraw[un][t].q1) = __builtin_bit_cast(uint4, y);
          if (GLU) {
            own_channel_pieces(r.ua[un][t], r.ub[un][t], x, y);
            uraw[un * UB][t].q0 = __builtin_bit_cast(uint4, x);
            (NIB ? uraw[un * UB + UB - 1][t].q0 : uraw[un][t].q1) = __builtin_bit_cast(uint4, y);
          }
        }
      }
#pragma unroll
    for (int u = 0; u < U; u++) {
      if constexpr (INT4) {
        // A nibble n (stored value + 8) becomes the bf16 number 128 + n by OR-ing it into the mantissa of
        // 128.0 (0x4300): one AND-OR per pair of values, pairs (k, k+4) of each 8-nibble word.  The MFMA then
        // yields P = sum (128 + n_k) a_k; with SA = sum a_k from one more MFMA against a row of ones, the block's
        // contribution is scale * (P - 136 * SA), applied in f32.  The activations are permuted to the same
        // k order (k0,k4,k1,k5,k2,k6,k3,k7) with byte permutes.
        v8bf af[MT][4];
        v4f sa[MT];
        const v8bf ones = __builtin_bit_cast(v8bf, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          sa[mt] = v4f{0.f, 0.f, 0.f, 0.f};
#pragma unroll
          for (int s = 0; s < 4; s++) {
            const uint4 a = live[u][0] ? araw[u][mt][s] : make_uint4(0, 0, 0, 0);
            const uint4 q = make_uint4(__builtin_amdgcn_perm(a.z, a.x, 0x05040100u), __builtin_amdgcn_perm(a.z, a.x, 0x07060302u),
                                       __builtin_amdgcn_perm(a.w, a.y, 0x05040100u), __builtin_amdgcn_perm(a.w, a.y, 0x07060302u));
            af[mt][s] = __builtin_bit_cast(v8bf, q);
            sa[mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, af[mt][s], sa[mt], 0, 0, 0);
          }
        }
#pragma unroll
        for (int t = 0; t < NT; t++) {
          // scales of the 4 channels this lane holds in the accumulator layout: channel 4*kq + r lives in lane 4*kq + r
          const uint32_t mine = (uint32_t)wsc[u][t] | (GLU ? (uint32_t)usc[u][t] << 16 : 0u);
          float sg[4], su[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            const uint32_t v = (uint32_t)__builtin_amdgcn_ds_bpermute((4 * kq + r) * 4, (int)mine);
            sg[r] = __uint_as_float(v << 16);
            su[r] = __uint_as_float(v & 0xffff0000u);
          }
          const uint32_t xw[4] = {wraw[u][t].q0.x, wraw[u][t].q0.y, wraw[u][t].q0.z, wraw[u][t].q0.w};
          const uint32_t xu[4] = {uraw[u][t].q0.x, uraw[u][t].q0.y, uraw[u][t].q0.z, uraw[u][t].q0.w};
          constexpr uint32_t M4 = 0x000f000fu, C = 0x43004300u;
          v8bf wf[4], uf[4];
#pragma unroll
          for (int s = 0; s < 4; s++) {
            wf[s] = __builtin_bit_cast(v8bf, make_uint4((xw[s] & M4) | C, ((xw[s] >> 4) & M4) | C, ((xw[s] >> 8) & M4) | C, ((xw[s] >> 12) & M4) | C));
            if (GLU)
              uf[s] = __builtin_bit_cast(v8bf, make_uint4((xu[s] & M4) | C, ((xu[s] >> 4) & M4) | C, ((xu[s] >> 8) & M4) | C, ((xu[s] >> 12) & M4) | C));
          }
#pragma unroll
          for (int mt = 0; mt < MT; mt++) {
            v4f pg = {0.f, 0.f, 0.f, 0.f}, pu = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
            for (int s = 0; s < 4; s++) {
              pg = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s], af[mt][s], pg, 0, 0, 0);
              if (GLU) pu = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[s], af[mt][s], pu, 0, 0, 0);
            }
            const float off = 136.0f * sa[mt][0];
#pragma unroll
            for (int r = 0; r < 4; r++) {
              acc_g[t][mt][r] = fmaf(sg[r], pg[r] - off, acc_g[t][mt][r]);
              if (GLU) acc_u[t][mt][r] = fmaf(su[r], pu[r] - off, acc_u[t][mt][r]);
            }
          }
        }
      } else {
        v8bf af[MT][4];
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int s = 0; s < 4; s++) af[mt][s] = __builtin_bit_cast(v8bf, live[u][NIB ? 0 : s / 2] ? araw[u][mt][s] : make_uint4(0, 0, 0, 0));
#pragma unroll
        for (int t = 0; t < NT; t++) {
          v8bf wf[4], uf[4];
          widen32<FMT>(wraw[u][t], MX4 ? __uint_as_float((uint32_t)wsc[u][t] << 23) : (G32 ? bf16_bits_to_f32(wsc[u][t]) : 1.0f), wf);
          if (GLU) widen32<FMT>(uraw[u][t], MX4 ? __uint_as_float((uint32_t)usc[u][t] << 23) : (G32 ? bf16_bits_to_f32(usc[u][t]) : 1.0f), uf);
#pragma unroll
          for (int mt = 0; mt < MT; mt++)
#pragma unroll
            for (int s = 0; s < 4; s++) {
              acc_g[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf[s], af[mt][s], acc_g[t][mt], 0, 0, 0);
              if (GLU) acc_u[t][mt] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf[s], af[mt][s], acc_u[t][mt], 0, 0, 0);
            }
        }
      }
    }
  };

  if constexpr (PREFETCH) {
    // the weights of the next round are requested before the current one is multiplied
    WRound w0, w1;
    ARound a;
    if (kb_begin < kb_end) load_w(w0, kb_begin);
    for (int kb = kb_begin; kb < kb_end; kb += 2 * U) {
      load_a(a, kb);
      if (kb + U < kb_end) load_w(w1, kb + U);
      compute_round(w0, a);
      if (kb + U < kb_end) {
        load_a(a, kb + U);
        if (kb + 2 * U < kb_end) load_w(w0, kb + 2 * U);
        compute_round(w1, a);
      }
    }
  } else {
    WRound w;
    ARound a;
    for (int kb = kb_begin; kb < kb_end; kb += U) {
      load_w(w, kb);
      load_a(a, kb);
      compute_round(w, a);
    }
  }

  if constexpr (KSPLIT > 1) {
    // partial sums of the group's waves 1..KSPLIT-1 -> LDS -> its wave 0
    if (ksub > 0) {
      float* r = red + (size_t)(nsub * (KSPLIT - 1) + ksub - 1) * NACC * kWave + lane;
      int i = 0;
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int c = 0; c < 4; c++) {
            r[(i++) * kWave] = acc_g[t][mt][c];
            if (GLU) r[(i++) * kWave] = acc_u[t][mt][c];
          }
    }
    __syncthreads();
    if (ksub > 0) return;
#pragma unroll
    for (int w = 0; w < KSPLIT - 1; w++) {
      const float* r = red + (size_t)(nsub * (KSPLIT - 1) + w) * NACC * kWave + lane;
      int i = 0;
#pragma unroll
      for (int t = 0; t < NT; t++)
#pragma unroll
        for (int mt = 0; mt < MT; mt++)
#pragma unroll
          for (int c = 0; c < 4; c++) {
            acc_g[t][mt][c] += r[(i++) * kWave];
            if (GLU) acc_u[t][mt][c] += r[(i++) * kWave];
          }
    }
  }
  if (idle) return;

  dispatch_act(GLU ? p.act : MOE_ACT_NONE, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const int n = n_w + t * 16 + 4 * kq;
      if (n >= N) continue;
      float sg[4] = {1.f, 1.f, 1.f, 1.f}, su[4] = {1.f, 1.f, 1.f, 1.f};
      float bg[4], bu[4];
      load_bias4(p.rhs_bias, tile.group, N, n, bg);
      load_bias4(GLU ? p.rhs_up_bias : nullptr, tile.group, N, n, bu);
      if (FMT == WQ_I8) {
        const float4 a = *(const float4*)((const float*)p.rhs_scale + (size_t)tile.group * N + n);
        sg[0] = a.x; sg[1] = a.y; sg[2] = a.z; sg[3] = a.w;
        if (GLU) {
          const float4 b = *(const float4*)((const float*)p.rhs_up_scale + (size_t)tile.group * N + n);
          su[0] = b.x; su[1] = b.y; su[2] = b.z; su[3] = b.w;
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int lr = mt * 16 + j;
        if (lr >= tile.nrows) continue;
        float pg[4] = {bg[0], bg[1], bg[2], bg[3]}, pu[4] = {bu[0], bu[1], bu[2], bu[3]};
        add_partial4(p.partial_sum, (size_t)(tile.row0 + lr), N, n, pg);
        add_partial4(GLU ? p.partial_sum_up : nullptr, (size_t)(tile.row0 + lr), N, n, pu);
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; r++)
          v[r] = GLU ? glu_act<ACT>(fmaf(acc_g[t][mt][r], sg[r], pg[r]), fmaf(acc_u[t][mt][r], su[r], pu[r]), p.act_limit)
                     : fmaf(acc_g[t][mt][r], sg[r], pg[r]);
        *(uint2*)(p.out + (size_t)(tile.row0 + lr) * N + n) = make_uint2(pack_bf16x2(v[0], v[1]), pack_bf16x2(v[2], v[3]));
      }
    }
  });
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

// Per-device launch state: the attribute that lets a kernel use more than 64 KB of dynamic LDS belongs to a
// device's code object, and the CU count to the device, so both are kept per device ordinal.  A race between two
// host threads only repeats an idempotent call.
constexpr int kMaxDevices = 64;

static int current_device(int* dev) {
  if (hipGetDevice(dev) != hipSuccess || *dev < 0 || *dev >= kMaxDevices) return fail(MOE_ERR_LAUNCH, "gmm: cannot identify the current device");
  return MOE_OK;
}

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

template <typename C>
static int launch_tiled(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  static bool attr_set[kMaxDevices] = {};
  if (int st = reserve_lds(gmm_tiled_kernel<C>, C::LDS_BYTES, attr_set)) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long blocks = (long long)p.max_m_tiles * p.tiles_n;
  if (blocks > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_tiled_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_tiled_kernel");
}

template <typename C>
static int launch_dl(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  static bool attr_set[kMaxDevices] = {};
  if (int st = reserve_lds(gmm_dl_kernel<C>, C::LDS_BYTES, attr_set)) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  // one persistent block per CU (the LDS footprint allows no more); a multiple of 8 keeps "tile id mod 8"
  // equal to the XCD a block runs on
  static int cus_of[kMaxDevices] = {};
  int dev = 0;
  if (int st = current_device(&dev)) return st;
  if (cus_of[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return fail(MOE_ERR_LAUNCH, "gmm: cannot query the CU count");
    cus_of[dev] = n;
  }
  const int num_cus = cus_of[dev];
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  gmm_dl_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_dl_kernel");
}

template <int OP, int BSRC, bool GLU>
static int launch_tiled_by_rows(const TiledParams& p, int M, int G_total, int* bm_out, bool dry, hipStream_t s) {
  // rows per expert on average decides the m-tile: full 256-row tiles for prefill, 64 otherwise; a problem with
  // fewer 256 x 256 tiles than half the CUs of the chip also takes the 64-row tiles, which quadruples its blocks
  const long long tiles_big = (long long)max_tiles_for(M, G_total, 256) * cdiv(p.N, GLU ? 128 : 256);
  const bool big = (long long)M >= 128LL * G_total && tiles_big >= 128;
  // 32 to 128 rows per expert on average (200 for the weight-only formats, whose big kernel is the register-staged one:
  // level with the 256-row tiles at 192 rows per expert on the GPT-OSS shape, 12 % ahead at 256 on the skewed Qwen3 one):
  // 128-row tiles.  Measured against the 64-row tiles on the Mixtral, Qwen3 and GPT-OSS shapes they are 15-35 % faster
  // from 32 rows per expert on (one weight conversion / tile fetch serves twice the rows), and 256-row tiles would be
  // half empty; below 32 rows per expert the 64-row tiles stay.
  const bool mid = !big && (long long)M >= 32LL * G_total && (long long)M < 128LL * G_total;
  const bool mid_wq = BSRC != BSRC_SAME && (long long)M >= 32LL * G_total && (long long)M < 200LL * G_total;
  // one decision for the tile map (bm_out, on the dry run) and for the launch
  constexpr int ESZ = OP == OP_I8 ? 1 : 2;
  enum { K_T64, K_T128, K_T256, K_DL128, K_DL64 } kind = K_T64;
  if (mid || mid_wq) kind = K_T128;
  else if (big && BSRC == BSRC_SAME && (p.K * ESZ) % 128 == 0) kind = K_DL128;
  else if (big && BSRC == BSRC_SAME && (p.K * ESZ) % 64 == 0) kind = K_DL64;
  else if (big) kind = K_T256;
  *bm_out = kind == K_T64 ? 64 : kind == K_T128 ? 128 : 256;
  if (dry) return MOE_OK;
  if constexpr (BSRC == BSRC_SAME) {
    // operands that need no conversion stream straight into LDS when every stage is a full row slice: 128-byte stages
    // (two buffers, 16 x 16 MFMAs) when the rows allow it, 6-10 % faster than 64-byte stages (four buffers, 32 x 32 MFMAs)
    // on the Mixtral shape (tile variant 12 of the int8 path is the 64-byte pipeline, for comparison)
    if (kind == K_DL128) return launch_dl<DlCfg<OP, 256, 256, 128, 2, 4, 2, GLU>>(p, M, G_total, s);
    if (kind == K_DL64) return launch_dl<DlCfg<OP, 256, 256, 64, 2, 4, 4, GLU>>(p, M, G_total, s);
  }
  if (kind == K_T128) return launch_tiled<TiledCfg<OP, BSRC, 128, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
  if (kind == K_T256) return launch_tiled<TiledCfg<OP, BSRC, 256, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
  // (eight waves of 32 x 64: 3-5 % faster than four of 64 x 64 on the Mixtral int8 shape at 4 to 24 rows per expert)
  return launch_tiled<TiledCfg<OP, BSRC, 64, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
}

// Tile variants of the int8 kernel that reserved[0] can force (tuning aid); returns the m-tile.
template <bool GLU>
static int launch_i8_variant(int id, const TiledParams& p, int M, int G_total, int* bm_out, bool dry, hipStream_t s) {
#define MOE_VARIANT(ID, BM, BN, BKB, WM, WN)                                                        \
  if (id == ID) {                                                                                   \
    *bm_out = BM;                                                                                   \
    if (dry) return MOE_OK;                                                                         \
    return launch_tiled<TiledCfg<OP_I8, BSRC_SAME, BM, BN, BKB, WM, WN, GLU>>(p, M, G_total, s);    \
  }
  MOE_VARIANT(3, 256, 256, 64, 2, 4)  // the register-staged kernel on int8 x int8
#undef MOE_VARIANT
#define MOE_DL_VARIANT(ID, BM, BN, BKB, WM, WN, NS)                                                 \
  if (id == ID) {                                                                                   \
    *bm_out = BM;                                                                                   \
    if (dry) return MOE_OK;                                                                         \
    if (p.K % BKB) return fail(MOE_ERR_UNSUPPORTED, "gmm: variant needs K %% %d == 0", BKB);        \
    return launch_dl<DlCfg<OP_I8, BM, BN, BKB, WM, WN, NS, GLU>>(p, M, G_total, s);                 \
  }
  MOE_DL_VARIANT(12, 256, 256, 64, 2, 4, 4)  // the 64-byte-stage pipeline where the default is the 128-byte one
#undef MOE_DL_VARIANT
  return fail(MOE_ERR_INVALID_ARG, "gmm: unknown tile variant %d", id);
}

template <int OP, int BSRC>
static int launch_tiled_glu(const TiledParams& p, bool glu, int M, int G_total, int* bm_out, bool dry, hipStream_t s) {
  return glu ? launch_tiled_by_rows<OP, BSRC, true>(p, M, G_total, bm_out, dry, s)
             : launch_tiled_by_rows<OP, BSRC, false>(p, M, G_total, bm_out, dry, s);
}

template <int BM, int BKB, int NSTAGE, bool GLU, bool VEC4>
static int launch_fp8_tiled(Fp8TiledParams P, int M, int G_total, hipStream_t s) {
  using C = F8Cfg<BM, BKB, NSTAGE, GLU, VEC4>;
  static bool attr_set[kMaxDevices] = {};
  if (int st = reserve_lds(gmm_fp8_tiled_kernel<C>, C::LDS_BYTES, attr_set)) return st;
  P.base.max_m_tiles = max_tiles_for(M, G_total, BM);
  P.base.tiles_n = cdiv(P.base.N, C::OUT_BN);
  const long long tiles = (long long)P.base.max_m_tiles * P.base.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_fp8_tiled_kernel<C><<<(unsigned)tiles, C::THREADS, C::LDS_BYTES, s>>>(P);
  return check_launch("gmm_fp8_tiled_kernel");
}

template <bool GLU, bool VEC4>
static int launch_fp8_big(Fp8TiledParams P, int M, int G_total, hipStream_t s) {
  using C = F8BigCfg<GLU, VEC4>;
  static bool attr_set[kMaxDevices] = {};
  if (int st = reserve_lds(gmm_fp8_big_kernel<C>, C::LDS_BYTES, attr_set)) return st;
  P.base.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  P.base.tiles_n = cdiv(P.base.N, C::OUT_BN);
  const long long tiles = (long long)P.base.max_m_tiles * P.base.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_fp8_big_kernel<C><<<(unsigned)tiles, C::THREADS, C::LDS_BYTES, s>>>(P);
  return check_launch("gmm_fp8_big_kernel");
}

template <int MT, int NT, int U>
static int launch_skinny(SkinnyParams p, bool glu, int max_tiles, hipStream_t s) {
  p.n_blocks = cdiv(p.N, 64 * NT);
  const long long blocks = (long long)max_tiles * p.n_blocks;
  if (blocks > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  if (glu)
    gmm_fp8_skinny_kernel<MT, NT, U, true><<<(unsigned)blocks, 256, 0, s>>>(p);
  else
    gmm_fp8_skinny_kernel<MT, NT, U, false><<<(unsigned)blocks, 256, 0, s>>>(p);
  return check_launch("gmm_fp8_skinny_kernel");
}

// (NT, U) of the fp8 streaming kernel, from sweeps over NT in {1, 2, 4} and U in {1, 2, 4} on the DeepSeek-V3 shapes:
// 16-row tiles take 4 channel tiles per wave and one K block per step with fused GLU, 2 tiles and 4 blocks without;
// 64-row tiles take 2 tiles and one block.
template <int MT>
static int launch_skinny_default(const SkinnyParams& p, bool glu, int max_tiles, hipStream_t s) {
  if (MT > 1) return launch_skinny<MT, 2, 1>(p, glu, max_tiles, s);
  return glu ? launch_skinny<MT, 4, 1>(p, glu, max_tiles, s) : launch_skinny<MT, 2, 4>(p, glu, max_tiles, s);
}

template <int FMT, int MT, int KSPLIT, int NT, int U, bool LINE = true>
static int launch_wq_skinny_k(WqSkinnyParams p, bool glu, int max_tiles, hipStream_t s) {
  p.n_blocks = cdiv(p.N, (4 / KSPLIT) * 16 * NT);
  const long long blocks = (long long)max_tiles * p.n_blocks;
  if (blocks > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  // Weights are requested as ordinary loads: at decode sizes of a few hundred MB part of them is served by the
  // last-level cache on the next call, which a non-temporal request gives up; past those sizes the two measure the same.
  constexpr bool STREAM = false;
  // Requesting the next round's weights early pays where the extra registers leave the occupancy as it is
  // (measured: MXFP4 and group-32 int4 8 % faster, group-128 int4 without GLU 10 %; with GLU it drops to one wave
  // per SIMD and runs 25 % slower, int8 10 % slower).
  constexpr bool PF_GLU = LINE && MT == 1 && (FMT == WQ_MX4 || FMT == WQ_I4G32);
  constexpr bool PF_PLAIN = LINE && MT == 1 && FMT != WQ_I8;
  if (glu)
    gmm_wq_skinny_kernel<FMT, MT, NT, true, U, KSPLIT, STREAM, PF_GLU, LINE><<<(unsigned)blocks, 256, 0, s>>>(p);
  else
    gmm_wq_skinny_kernel<FMT, MT, NT, false, U, KSPLIT, STREAM, PF_PLAIN, LINE><<<(unsigned)blocks, 256, 0, s>>>(p);
  return check_launch("gmm_wq_skinny_kernel");
}

// K is split over the 4 waves of a block; `tune` == 1 (reserved[1] of the arguments) gives every wave all of K
// instead (measured slower up to 32 rows per expert; kept as a tuning aid).
template <int FMT, int MT>
static int launch_wq_skinny(const WqSkinnyParams& p, bool glu, int max_tiles, int tune, hipStream_t s) {
  // k-blocks per round: 2.  More raw bytes in flight per wave cost registers, and the occupancy lost with them costs
  // more than the longer rounds gain (4 measured 30-50 % slower on the 4-bit formats).
  constexpr int U = 2;
  if (tune == 1) return launch_wq_skinny_k<FMT, MT, 1, 2, U>(p, glu, max_tiles, s);
  if constexpr (FMT == WQ_I4 && MT == 1) {
    // Group-128 int4 with fused GLU holds the most registers of all variants and cannot afford the early request.
    // When the rows of the matrix do not start on 128-byte lines anyway (GPT-OSS: 1440-byte rows), rounds of three
    // k-blocks with plain 64-byte requests measure 8 % faster than rounds of two with request pairs.
    if (glu && (p.K / 2) % 128 != 0) return launch_wq_skinny_k<FMT, MT, 4, 2, 3, false>(p, glu, max_tiles, s);
  }
  return launch_wq_skinny_k<FMT, MT, 4, 2, U>(p, glu, max_tiles, s);
}

}  // namespace moe

using namespace moe;

extern "C" {

int moe_gmm_rhs_kn_supported(int M, int K, int N, int num_groups_total) {
  // the 256 x 256 direct-to-LDS kernel is the only one that reads [G, K, N]: whole 64-row stages of 256 channels, groups of
  // 128 rows and more on average, enough tiles for the chip (the rule by which moe_gmm picks that kernel for [G, N, K] too)
  if (M <= 0 || K <= 0 || N <= 0 || num_groups_total <= 0) return 0;
  if (K % 64 != 0 || N % 256 != 0 || (long long)M < 128LL * num_groups_total) return 0;
  return (long long)max_tiles_for(M, num_groups_total, 256) * (N / 256) >= 128 ? 1 : 0;
}

size_t moe_gmm_workspace_bytes(int M, int num_groups_total) {
  if (M < 0 || num_groups_total <= 0) return 0;
  return 16 + (size_t)max_tiles_for(M, num_groups_total, 16) * sizeof(TileInfo);
}

int moe_gmm(const moe_gmm_args* a, void* stream) {
  if (!a) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL args");
  if (a->struct_size != sizeof(moe_gmm_args)) return fail(MOE_ERR_INVALID_ARG, "gmm: struct_size %zu != %zu", a->struct_size, sizeof(moe_gmm_args));
  if (!a->lhs || !a->rhs || !a->group_sizes || !a->out || !a->workspace) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL pointer");
  if (a->M < 0 || a->K <= 0 || a->N <= 0 || a->num_groups_total <= 0 || a->num_groups_local <= 0 || a->group_offset < 0)
    return fail(MOE_ERR_INVALID_ARG, "gmm: bad sizes M=%d K=%d N=%d G=%d/%d", a->M, a->K, a->N, a->num_groups_local, a->num_groups_total);
  if (a->workspace_bytes < moe_gmm_workspace_bytes(a->M, a->num_groups_total)) return fail(MOE_ERR_WORKSPACE, "gmm: workspace too small");
  const bool glu = a->rhs_up != nullptr;
  if (glu && a->act == MOE_ACT_NONE) return fail(MOE_ERR_INVALID_ARG, "gmm: rhs_up needs an activation");
  if (!glu && a->act != MOE_ACT_NONE) return fail(MOE_ERR_INVALID_ARG, "gmm: activation needs rhs_up");
  if (a->act < MOE_ACT_NONE || a->act > MOE_ACT_SILU_CLIP) return fail(MOE_ERR_INVALID_ARG, "gmm: bad act %d", a->act);
  if (a->N % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "gmm: N %% 8 != 0 (N=%d)", a->N);
  if (a->rhs_up_bias && !glu) return fail(MOE_ERR_INVALID_ARG, "gmm: rhs_up_bias needs rhs_up");
  if (a->partial_sum_up && !glu) return fail(MOE_ERR_INVALID_ARG, "gmm: partial_sum_up needs rhs_up");
  if (((uintptr_t)a->partial_sum | (uintptr_t)a->partial_sum_up) & 7) return fail(MOE_ERR_UNSUPPORTED, "gmm: partial sums must be 8-byte aligned");
  if (a->partial_sum == a->out || a->partial_sum_up == a->out) return fail(MOE_ERR_INVALID_ARG, "gmm: partial sums must not alias out");
  if (((uintptr_t)a->rhs_bias | (uintptr_t)a->rhs_up_bias) & 15) return fail(MOE_ERR_UNSUPPORTED, "gmm: bias pointers must be 16-byte aligned");
  if (a->M == 0) return MOE_OK;
  const uintptr_t align = (uintptr_t)a->lhs | (uintptr_t)a->rhs | (uintptr_t)a->rhs_up | (uintptr_t)a->out |
                          (uintptr_t)a->rhs_scale | (uintptr_t)a->rhs_up_scale;
  if (align & 15) return fail(MOE_ERR_UNSUPPORTED, "gmm: pointers must be 16-byte aligned");

  hipStream_t s = (hipStream_t)stream;
  const int zero_fill = (a->flags & MOE_GMM_KEEP_OTHER_ROWS) ? 0 : 1;
  int32_t* header = (int32_t*)a->workspace;
  TileInfo* tiles = (TileInfo*)((uint8_t*)a->workspace + 16);

  const int L = a->lhs_dtype, R = a->rhs_dtype;
  int bm = 0;

  if (L == MOE_FP8_E4M3 && R == MOE_FP8_E4M3) {
    if (a->lhs_scale_block_k != 128 || a->rhs_scale_block_k != 128 || a->rhs_scale_block_n != 128 || !a->lhs_scale || !a->rhs_scale || (glu && !a->rhs_up_scale))
      return fail(MOE_ERR_UNSUPPORTED, "gmm: fp8 needs 1x128 lhs scales and 128x128 rhs scales");
    if (a->K % 128 != 0) return fail(MOE_ERR_UNSUPPORTED, "gmm: fp8 needs K %% 128 == 0 (K=%d)", a->K);
    if ((long long)a->N * a->K >= (1LL << 31)) return fail(MOE_ERR_UNSUPPORTED, "gmm: fp8 needs N * K < 2^31");
    // Up to 14 rows per expert on average (decode): the streaming kernel with 16-row tiles, one MFMA row tile per
    // wave; a group with more rows simply gets several tiles, which are adjacent in the grid, run at the same time
    // and share the group's weights through L2.  Beyond that the LDS-tiled kernel with 128 x 128 tiles (measured on
    // 256 experts of 7168 x 2048: at 12 rows per expert 1.27 against 1.52 ms, at 16, where half of the experts need a
    // second 16-row tile, 1.66 against 1.54 ms; the 256 x 256 kernel is within 5 % of it from 128
    // rows per expert on and behind it below, so it is not picked by default).  reserved[0] = 1 / 2 / 3 forces the
    // streaming kernel (64-row tiles past 16 rows per expert) / 128 x 128 tiles / 256 x 256 tiles (tuning aid).
    const int forced = a->reserved[0] >= 1 && a->reserved[0] <= 3 ? a->reserved[0] : 0;
    const bool few_rows = (long long)a->M <= 16LL * a->num_groups_total;
    const bool tiled = forced ? forced >= 2 : (long long)a->M > 14LL * a->num_groups_total;
    if (tiled) {
      const bool big = forced == 3;
      bm = big ? 256 : 128;
      tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, a->num_groups_total, a->group_offset, a->num_groups_local, a->M, bm, zero_fill, header, tiles);
      Fp8TiledParams P;
      TiledParams& q = P.base;
      q.lhs = (const uint8_t*)a->lhs; q.lhs_scale = nullptr;
      q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
      q.rhs_scale = nullptr; q.rhs_up_scale = nullptr;
      q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
      q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
      q.header = header; q.tiles = tiles; q.out = (uint16_t*)a->out;
      q.M = a->M; q.K = a->K; q.N = a->N; q.max_m_tiles = 0; q.tiles_n = 0;
      q.act = a->act; q.act_limit = a->act_limit; q.tune = a->reserved[1]; q.i4_group = 0;
      P.a_scale = a->lhs_scale; P.w_scale = (const float*)a->rhs_scale; P.u_scale = (const float*)a->rhs_up_scale;
      const int G = a->num_groups_total;
      const bool vec4 = (a->K / 128) % 4 == 0 && ((uintptr_t)a->lhs_scale & 15) == 0;
      if (big) {
        if (vec4) return glu ? launch_fp8_big<true, true>(P, a->M, G, s) : launch_fp8_big<false, true>(P, a->M, G, s);
        return glu ? launch_fp8_big<true, false>(P, a->M, G, s) : launch_fp8_big<false, false>(P, a->M, G, s);
      }
      if (vec4) return glu ? launch_fp8_tiled<128, 128, 2, true, true>(P, a->M, G, s) : launch_fp8_tiled<128, 128, 2, false, true>(P, a->M, G, s);
      return glu ? launch_fp8_tiled<128, 128, 2, true, false>(P, a->M, G, s) : launch_fp8_tiled<128, 128, 2, false, false>(P, a->M, G, s);
    }
    bm = few_rows ? 16 : 64;
    tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, a->num_groups_total, a->group_offset, a->num_groups_local, a->M, bm, zero_fill, header, tiles);
    SkinnyParams p;
    p.lhs = (const uint8_t*)a->lhs; p.lhs_scale = a->lhs_scale;
    p.rhs = (const uint8_t*)a->rhs; p.rhs_up = (const uint8_t*)a->rhs_up;
    p.rhs_scale = (const float*)a->rhs_scale; p.rhs_up_scale = (const float*)a->rhs_up_scale;
    p.rhs_bias = a->rhs_bias; p.rhs_up_bias = a->rhs_up_bias;
    p.partial_sum = (const uint16_t*)a->partial_sum; p.partial_sum_up = (const uint16_t*)a->partial_sum_up;
    p.header = header; p.tiles = tiles; p.out = (uint16_t*)a->out;
    p.M = a->M; p.K = a->K; p.N = a->N; p.n_blocks = 0;
    p.act = a->act; p.act_limit = a->act_limit;
    const int mx = max_tiles_for(a->M, a->num_groups_total, bm);
    p.min_rows = 1; p.max_rows = bm;
    if (few_rows) return launch_skinny_default<1>(p, glu, mx, s);
    return launch_skinny_default<4>(p, glu, mx, s);
  }

  TiledParams p;
  p.lhs = (const uint8_t*)a->lhs; p.lhs_scale = nullptr;
  p.rhs = (const uint8_t*)a->rhs; p.rhs_up = (const uint8_t*)a->rhs_up;
  p.rhs_scale = a->rhs_scale; p.rhs_up_scale = a->rhs_up_scale;
  p.rhs_bias = a->rhs_bias; p.rhs_up_bias = a->rhs_up_bias;
  p.partial_sum = (const uint16_t*)a->partial_sum; p.partial_sum_up = (const uint16_t*)a->partial_sum_up;
  p.header = header; p.tiles = tiles; p.out = (uint16_t*)a->out;
  p.M = a->M; p.K = a->K; p.N = a->N; p.max_m_tiles = 0; p.tiles_n = 0;
  p.act = a->act; p.act_limit = a->act_limit; p.tune = a->reserved[1]; p.i4_group = a->rhs_scale_block_k == 32 ? 32 : 128;

  enum { V_NONE, V_BF16, V_W8, V_W4, V_I8, V_MX4 } variant = V_NONE;
  if (L == MOE_BF16 && R == MOE_BF16) {
    if (a->K % 8) return fail(MOE_ERR_UNSUPPORTED, "gmm: bf16 needs K %% 8 == 0");
    p.rhs_scale = p.rhs_up_scale = nullptr;
    variant = V_BF16;
  } else if (L == MOE_BF16 && R == MOE_INT8) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale) || a->rhs_scale_block_n != 1 || a->rhs_scale_block_k != 0)
      return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 weights need per-channel f32 scales [G, N]");
    if (a->K % 16) return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 weights need K %% 16 == 0");
    variant = V_W8;
  } else if (L == MOE_BF16 && R == MOE_INT4) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale) || a->rhs_scale_block_n != 1 || (a->rhs_scale_block_k != 128 && a->rhs_scale_block_k != 32))
      return fail(MOE_ERR_UNSUPPORTED, "gmm: int4 weights need bf16 group scales [G, N, ceil(K/group)] with group 128 or 32");
    if (a->K % 32) return fail(MOE_ERR_UNSUPPORTED, "gmm: int4 weights need K %% 32 == 0");
    variant = V_W4;
  } else if (L == MOE_BF16 && R == MOE_MXFP4) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale) || a->rhs_scale_block_n != 1 || a->rhs_scale_block_k != 32)
      return fail(MOE_ERR_UNSUPPORTED, "gmm: mxfp4 weights need e8m0 block-32 scales [G, N, K/32]");
    if (a->K % 32) return fail(MOE_ERR_UNSUPPORTED, "gmm: mxfp4 weights need K %% 32 == 0");
    variant = V_MX4;
  } else if (L == MOE_INT8 && R == MOE_INT8) {
    if (!a->lhs_scale || a->lhs_scale_block_k != 0 || !a->rhs_scale || (glu && !a->rhs_up_scale) || a->rhs_scale_block_n != 1 || a->rhs_scale_block_k != 0)
      return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 x int8 needs per-row lhs scales [M] and per-channel rhs scales [G, N]");
    if (a->K % 16) return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 needs K %% 16 == 0");
    p.lhs_scale = a->lhs_scale;
    variant = V_I8;
  } else {
    return fail(MOE_ERR_UNSUPPORTED, "gmm: lhs_dtype %d x rhs_dtype %d", L, R);
  }

  const int M = a->M, G = a->num_groups_total;
  if (a->flags & MOE_GMM_RHS_KN) {
    if (variant != V_BF16 || glu || !moe_gmm_rhs_kn_supported(M, a->K, a->N, G))
      return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] weights need bf16 x bf16 without rhs_up and a shape moe_gmm_rhs_kn_supported accepts");
    tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->num_groups_local, M, 256, zero_fill, header, tiles);
    return launch_dl<DlCfg<OP_BF16, 256, 256, 128, 2, 4, 2, false, true>>(p, M, G, s);
  }
  const bool int4_g128 = variant == V_W4 && a->rhs_scale_block_k != 32;
  // rows per expert up to which the streaming kernel beats the register-staged one (measured on the GPT-OSS and Qwen3
  // shapes): 56 for group-128 int4, 64 for MXFP4 (0.38 / 0.41 / 0.49 ms at 320 / 384 / 512 tokens against 0.46 / 0.51 /
  // 0.53 ms), 32 for int8 and group-32 int4
  const long long stream_rows_hi = int4_g128 ? 56 : variant == V_MX4 ? 64 : 32;
  // few rows per expert with weight-only int8 / int4: the streaming kernel (decode is bound by weight bytes)
  // (a lane of that kernel owns 32 consecutive k values, so K must be a multiple of 32; other K take the tiled kernel)
  if ((variant == V_W8 || variant == V_W4 || variant == V_MX4) && (long long)M <= stream_rows_hi * G && a->K % 32 == 0 && a->reserved[0] != 1 &&
      (long long)a->N * a->K < (1LL << 31)) {
    // 16-row tiles up to 16 rows per expert on average, 32-row tiles above; group-128 int4 keeps the 16-row tiles over the
    // whole range (its 32-row variant runs at two waves per SIMD: 0.36 against 0.44 ms on the GPT-OSS shape at 256 tokens)
    // and stays on this kernel up to 56 rows per expert (0.43 / 0.48 ms at 320 / 384 tokens against 0.52 / 0.58 ms on
    // the 128-row tiles of the register-staged kernel; level at 512 tokens)
    const bool one = int4_g128 || (long long)M <= 16LL * G;
    bm = one ? 16 : 32;
    tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->num_groups_local, M, bm, zero_fill, header, tiles);
    WqSkinnyParams q;
    q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
    q.rhs_scale = a->rhs_scale; q.rhs_up_scale = a->rhs_up_scale;
    q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
    q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
    q.header = header; q.tiles = tiles; q.out = (uint16_t*)a->out;
    q.M = M; q.K = a->K; q.N = a->N; q.n_blocks = 0; q.act = a->act; q.act_limit = a->act_limit;
    const int mx = max_tiles_for(M, G, bm);
    const int kso = a->reserved[1];
    if (variant == V_W4 && a->rhs_scale_block_k == 32)
      return one ? launch_wq_skinny<WQ_I4G32, 1>(q, glu, mx, kso, s) : launch_wq_skinny<WQ_I4G32, 2>(q, glu, mx, kso, s);
    if (variant == V_W4) return one ? launch_wq_skinny<WQ_I4, 1>(q, glu, mx, kso, s) : launch_wq_skinny<WQ_I4, 2>(q, glu, mx, kso, s);
    if (variant == V_MX4) return one ? launch_wq_skinny<WQ_MX4, 1>(q, glu, mx, kso, s) : launch_wq_skinny<WQ_MX4, 2>(q, glu, mx, kso, s);
    return one ? launch_wq_skinny<WQ_I8, 1>(q, glu, mx, kso, s) : launch_wq_skinny<WQ_I8, 2>(q, glu, mx, kso, s);
  }
  // dry run to learn the m-tile, then build the tile list and launch
  const int forced = a->reserved[0];
  if (forced >= 3 && variant == V_I8) {
    int st = glu ? launch_i8_variant<true>(forced, p, M, G, &bm, true, s) : launch_i8_variant<false>(forced, p, M, G, &bm, true, s);
    if (st != MOE_OK) return st;
    tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->num_groups_local, M, bm, zero_fill, header, tiles);
    return glu ? launch_i8_variant<true>(forced, p, M, G, &bm, false, s) : launch_i8_variant<false>(forced, p, M, G, &bm, false, s);
  }
  auto run = [&](bool dry) -> int {
    switch (variant) {
      case V_BF16: return launch_tiled_glu<OP_BF16, BSRC_SAME>(p, glu, M, G, &bm, dry, s);
      case V_W8: return launch_tiled_glu<OP_BF16, BSRC_I8>(p, glu, M, G, &bm, dry, s);
      case V_W4: return launch_tiled_glu<OP_BF16, BSRC_I4>(p, glu, M, G, &bm, dry, s);
      case V_MX4: return launch_tiled_glu<OP_BF16, BSRC_MX4>(p, glu, M, G, &bm, dry, s);
      case V_I8: return launch_tiled_glu<OP_I8, BSRC_SAME>(p, glu, M, G, &bm, dry, s);
      default: break;
    }
    return fail(MOE_ERR_UNSUPPORTED, "gmm: no kernel");
  };
  if (int st = run(true)) return st;  // the m-tile this operand family takes for this shape
  tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->num_groups_local, M, bm, zero_fill, header, tiles);
  return run(false);
}

}  // extern "C"
