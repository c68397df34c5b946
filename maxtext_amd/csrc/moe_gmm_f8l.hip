// Grouped matmul, decode sizes: fp8 x fp8 or int8 x int8 with per-row x per-channel scales, weights and activations
// streamed through LDS.

#include "moe_gmm_f8d.h"

namespace moe {

// ---------------------------------------------------------------------------------------
// Operands with one scale per activation row and one per output channel (ops.py:241-260; float8_e4m3 or int8), applied to
// the finished sums.  The persistent stream of gmm_f8d_kernel (moe_gmm_f8d.hip: one 512-thread block per CU walks a run of
// items, a 16- or 32-row tile x 32 channels of both projections or 64 of one, and copies each item's weight rows global ->
// LDS in segments of 64 rows x 512 B ahead of the multiplication) with the tile's activations travelling beside the
// weights instead of staying in registers: a segment is the 64 weight rows, then the tile's 16 or 32 activation rows,
// 512 B of each (40 or 48 KB), in a ring of three (two in flight); an item re-reads its tile's activation rows, which
// come from L2.  Nothing is kept per k-block, so the segment loop is an ordinary one, K is any multiple of 512, and a
// second row tile costs 8 KB per segment and 16 accumulator registers.  The sums form in the MFMA accumulators (int32
// for int8: two v_mfma_i32_16x16x64_i8 per k-block), the row's scale is read with the tile, the item's channel scales
// are copied to LDS with its first segment.  Measured level with resident activations where both apply.  64-row tiles
// (25 to 48 rows per expert) run on segments half as wide, so that weights and activations of three segments in flight fit.
// ---------------------------------------------------------------------------------------

// MT row tiles of 16 per item (tiles of 16, 32 or 64 rows): a segment is 64 weight rows, then 16 * MT activation rows, KB
// k-blocks of 128 bytes of each.  16- and 32-row tiles: four k-blocks, one per wave of a channel tile, ring of three.  64-row
// tiles: two k-blocks (the rows would not fit otherwise), the four waves of a channel tile are two k-blocks x two pairs of row
// tiles, ring of four, so that the same 96 KB are in flight.
template <int MT>
struct F8lLds {
  static constexpr int kKb = MT == 4 ? 2 : 4;
  static constexpr int kRing = MT == 4 ? 4 : 3;
  static constexpr int kSegWidth = kKb * 128;
  static constexpr int kSegBytes = (64 + 16 * MT) * kSegWidth;
  static constexpr int kHalfFloats = MT == 2 ? 64 : 256;  // an item's channel scales per half: the KB a copy brings, or (32-row tiles:
                                                          // LDS is full) the 256 B that 16 lanes bring
  static constexpr int kScaleBuf = 2 * kHalfFloats * 4;
  static constexpr int kScale0 = kRing * kSegBytes;
  static constexpr int kRed0 = kScale0 + 3 * kScaleBuf;
  static constexpr int kBytes = kRed0 + kF8dRedBytes;  // 141312 / 161280 / 149504 bytes
  static_assert(kBytes <= 160 * 1024, "LDS");
};

template <bool GLU, bool NT, bool I8, int MT>
__global__ __launch_bounds__(kF8dThreads) void gmm_f8l_kernel(const SkinnyParams p, int num_groups) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  static_assert(MT == 1 || MT == 2 || MT == 4, "16-, 32- or 64-row tiles");
  using L = F8lLds<MT>;
  constexpr int KB = L::kKb, RING = L::kRing, AHEAD = RING - 1, SEGW = L::kSegWidth;
  constexpr int NRP = 4 / KB, MTW = MT / NRP;  // groups of row tiles among the waves of a channel tile, row tiles per wave
  constexpr int LPR = 8 * KB, RPI = kWave / LPR;  // lanes per segment row, rows per copy instruction
  constexpr int WCOP = 8 / RPI, ACOP = 2 * MT / RPI;  // a wave's copy instructions per segment: weights, activations
  constexpr int CH = GLU ? 32 : 64;
  constexpr int SRING = 3;  // scale buffers: a copy two positions ahead is at most two items ahead
  constexpr int HF = L::kHalfFloats;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int a = wave / 4, ksub = wave % KB, rp = (wave % 4) / KB;
  const int j = lane % 16, kq = lane / 16;
  const int N = p.N, K = p.K;
  const int nseg = K / SEGW;
  const uint32_t row_bytes = (uint32_t)K;
  const int ncg = (N + CH - 1) / CH;
  const int ntiles = __builtin_amdgcn_readfirstlane(p.header[0]);
  const long long total = (long long)ntiles * ncg;
  const int q0 = (int)(total * blockIdx.x / gridDim.x), q1 = (int)(total * (blockIdx.x + 1) / gridDim.x);
  if (q0 >= q1) return;
  const int nitems = q1 - q0, nstream = nitems * nseg;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  const uint32_t w_bytes = clamp_u32((size_t)num_groups * N * row_bytes);
  const uint32_t s_bytes = clamp_u32(((size_t)(num_groups - 1) * p.ch_gstride + N) * 4);
  const v4i desc_w = buffer_desc(p.rhs, w_bytes);
  const v4i desc_u = buffer_desc(GLU ? p.rhs_up : p.rhs, w_bytes);
  const v4i sdesc_w = buffer_desc(p.ch_scale, s_bytes);
  const v4i sdesc_u = buffer_desc(GLU ? p.ch_scale_up : p.ch_scale, s_bytes);
  const v4i desc_a = buffer_desc(p.lhs, clamp_u32((size_t)p.ro.lhs_rows * row_bytes));
  const bool up_half = wave >= 4;

  // ---- the tile the run is in and the one after it: experts, and where this lane's activation rows of each start ----
  // (lane: row 8 RPI t + RPI wave + lane / LPR of the tile for copy t, row 16 (MTW rp + t) + lane % 16 for the scale of the
  // finished sums)
  int m_cur = q0 / ncg;
  TileInfo tile;
  int g_cur = 0, g_next = 0;
  uint32_t aoff_cur[ACOP], aoff_next[ACOP];
  float rs[MTW];
  const int crow = RPI * wave + lane / LPR;
  const uint32_t achunk = (uint32_t)((lane % LPR) ^ (crow & 15)) * 16u;
  auto load_tile = [&](int m) {
    // (everything is read here, into registers that are used here: a load left pending would be waited for behind the copies)
    const TileInfo t = p.tiles[m];
    const TileInfo tn = p.tiles[min(m + 1, ntiles - 1)];
    tile.group = __builtin_amdgcn_readfirstlane(t.group);
    tile.row0 = __builtin_amdgcn_readfirstlane(t.row0);
    tile.nrows = __builtin_amdgcn_readfirstlane(t.nrows);
    const int n_row0 = __builtin_amdgcn_readfirstlane(tn.row0), n_nrows = __builtin_amdgcn_readfirstlane(tn.nrows);
    g_cur = max(tile.group, 0);
    g_next = m + 1 < ntiles ? max(__builtin_amdgcn_readfirstlane(tn.group), 0) : 0;
#pragma unroll
    for (int t2 = 0; t2 < ACOP; t2++) {
      aoff_cur[t2] = (uint32_t)lhs_row_of(p.ro, tile.row0 + min(8 * RPI * t2 + crow, tile.nrows - 1)) * row_bytes + achunk;
      aoff_next[t2] = (uint32_t)lhs_row_of(p.ro, n_row0 + min(8 * RPI * t2 + crow, n_nrows - 1)) * row_bytes + achunk;
      asm volatile("" : "+v"(aoff_cur[t2]), "+v"(aoff_next[t2]));
    }
#pragma unroll
    for (int t2 = 0; t2 < MTW; t2++) {
      const int gr = lhs_row_of(p.ro, tile.row0 + min(16 * (MTW * rp + t2) + j, tile.nrows - 1));
      rs[t2] = p.row_scale_lhs ? p.row_scale_lhs[(size_t)gr * p.row_scale_lhs_stride] : 1.0f;
      asm volatile("" : "+v"(rs[t2]));
    }
  };

  uint32_t lane_off[WCOP];
#pragma unroll
  for (int i = 0; i < WCOP; i++) {
    const int row = 8 * wave + RPI * i + lane / LPR;
    lane_off[i] = (uint32_t)(GLU ? row % 32 : row) * row_bytes + (uint32_t)((lane % LPR) ^ (row & 15)) * 16u;
  }
  auto issue = [&](int pos) {
    const int it = pos / nseg, s = pos - it * nseg;
    const int q = q0 + it;
    const int m = q / ncg, cg = q - m * ncg;
    const bool cur = m == m_cur;  // (the positions ahead, at most two items on, never leave the next tile: ncg >= 4)
    const int group = cur ? g_cur : g_next;
    if (s == 0 && wave % 4 == 0) {
      const uint32_t voff = (uint32_t)(group * p.ch_gstride + cg * CH) * 4u + (uint32_t)lane * 16u;
      const uint32_t dst = lds_base + L::kScale0 + (uint32_t)(it % SRING) * L::kScaleBuf + (up_half ? (uint32_t)HF * 4u : 0u);
      if (MT != 2) {
        f8d_copy<false>(up_half ? sdesc_u : sdesc_w, voff, dst);
      } else if (lane < 16) {  // (64 floats: the lanes that are switched off copy nothing)
        f8d_copy<false>(up_half ? sdesc_u : sdesc_w, voff, dst);
      }
    }
    const uint32_t slot = lds_base + (uint32_t)(pos % RING) * L::kSegBytes;
    const uint32_t base = (uint32_t)(group * N + cg * CH) * row_bytes + (uint32_t)(s * SEGW);
#pragma unroll
    for (int i = 0; i < WCOP; i++)
      f8d_copy<NT>(up_half ? desc_u : desc_w, base + lane_off[i], slot + (uint32_t)((8 * wave + RPI * i) * SEGW));
    // the tile's activation rows 8 RPI t + RPI wave and the RPI - 1 after it (read again by every item of the tile: temporal)
#pragma unroll
    for (int t2 = 0; t2 < ACOP; t2++)
      f8d_copy<false>(desc_a, (cur ? aoff_cur[t2] : aoff_next[t2]) + (uint32_t)(s * SEGW),
                      slot + (uint32_t)((64 + 8 * RPI * t2 + RPI * wave) * SEGW));
  };

  load_tile(m_cur);
#pragma unroll
  for (int pos = 0; pos < AHEAD; pos++)
    if (pos < nstream) issue(pos);

  float* const red = (float*)(smem + L::kRed0);
  for (int it = 0; it < nitems; it++) {
    const int q = q0 + it;
    const int m = q / ncg, cg = q - m * ncg;
    if (m != m_cur) {
      m_cur = m;
      load_tile(m);
    }
    v4f acc_g[MTW], acc_u[MTW];
    v4i ig[MTW], iu[MTW];
#pragma unroll
    for (int t2 = 0; t2 < MTW; t2++) {
      acc_g[t2] = acc_u[t2] = v4f{0.f, 0.f, 0.f, 0.f};
      ig[t2] = iu[t2] = v4i{0, 0, 0, 0};
    }
    const float* const sbuf = (const float*)(smem + L::kScale0 + (it % SRING) * L::kScaleBuf);
    for (int s = 0; s < nseg; s++) {
      const int pos = it * nseg + s;
      // this wave's copies of the segment (WCOP + ACOP, one more, ahead of them, with the scales) have landed once at most
      // those of the segments after it are outstanding
      if (pos + AHEAD - 1 < nstream) wait_vmcnt<(AHEAD - 1) * (WCOP + ACOP)>();
      else wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      if (pos + AHEAD < nstream) issue(pos + AHEAD);
      const uint8_t* slot = smem + (pos % RING) * L::kSegBytes;
      const int c0 = (ksub * 8 + kq) ^ j, c1 = (ksub * 8 + 4 + kq) ^ j;
      const uint8_t* wrow = slot + (a * 16 + j) * SEGW;
      const uint8_t* urow = slot + (32 + a * 16 + j) * SEGW;
      const uint4 w0 = *(const uint4*)(wrow + c0 * 16), w1 = *(const uint4*)(wrow + c1 * 16);
      const uint4 u0 = *(const uint4*)(urow + c0 * 16), u1 = *(const uint4*)(urow + c1 * 16);
#pragma unroll
      for (int t2 = 0; t2 < MTW; t2++) {
        const uint8_t* arow = slot + (64 + 16 * (MTW * rp + t2) + j) * SEGW;
        const uint4 x0 = *(const uint4*)(arow + c0 * 16), x1 = *(const uint4*)(arow + c1 * 16);
        if constexpr (I8) {
          const v4i a0 = {(int)x0.x, (int)x0.y, (int)x0.z, (int)x0.w}, a1 = {(int)x1.x, (int)x1.y, (int)x1.z, (int)x1.w};
          ig[t2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)w0.x, (int)w0.y, (int)w0.z, (int)w0.w}, a0, ig[t2], 0, 0, 0);
          iu[t2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)u0.x, (int)u0.y, (int)u0.z, (int)u0.w}, a0, iu[t2], 0, 0, 0);
          ig[t2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)w1.x, (int)w1.y, (int)w1.z, (int)w1.w}, a1, ig[t2], 0, 0, 0);
          iu[t2] = __builtin_amdgcn_mfma_i32_16x16x64_i8(v4i{(int)u1.x, (int)u1.y, (int)u1.z, (int)u1.w}, a1, iu[t2], 0, 0, 0);
        } else {
          v8i wf, uf, af;
          wf[0] = w0.x; wf[1] = w0.y; wf[2] = w0.z; wf[3] = w0.w; wf[4] = w1.x; wf[5] = w1.y; wf[6] = w1.z; wf[7] = w1.w;
          uf[0] = u0.x; uf[1] = u0.y; uf[2] = u0.z; uf[3] = u0.w; uf[4] = u1.x; uf[5] = u1.y; uf[6] = u1.z; uf[7] = u1.w;
          af[0] = x0.x; af[1] = x0.y; af[2] = x0.z; af[3] = x0.w; af[4] = x1.x; af[5] = x1.y; af[6] = x1.z; af[7] = x1.w;
          acc_g[t2] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, af, acc_g[t2], 0, 0, 0, 127, 0, 127);
          acc_u[t2] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(uf, af, acc_u[t2], 0, 0, 0, 127, 0, 127);
        }
      }
    }

    // ---- per row tile: sums of the waves ksub > 0 -> LDS -> wave (a, rp, 0), which runs the epilogue ----
#pragma unroll
    for (int t2 = 0; t2 < MTW; t2++) {
      if (t2 > 0) asm volatile("s_barrier" ::: "memory");  // the sums of the tile before have been read
      if (ksub > 0) {
        float* r = red + (size_t)(((a * NRP + rp) * (KB - 1) + ksub - 1) * 8) * kWave + lane;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          r[e * kWave] = I8 ? __int_as_float(ig[t2][e]) : acc_g[t2][e];
          r[(4 + e) * kWave] = I8 ? __int_as_float(iu[t2][e]) : acc_u[t2][e];
        }
      }
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the sums are in LDS (and this wave's reads of the tile before are done)
      asm volatile("s_barrier" ::: "memory");
      if (ksub == 0) {
        v4f sg = acc_g[t2], su = acc_u[t2];
        v4i jg = ig[t2], ju = iu[t2];
#pragma unroll
        for (int w = 0; w < KB - 1; w++) {
          const float* r = red + (size_t)(((a * NRP + rp) * (KB - 1) + w) * 8) * kWave + lane;
#pragma unroll
          for (int e = 0; e < 4; e++) {
            if (I8) {
              jg[e] += __float_as_int(r[e * kWave]);
              ju[e] += __float_as_int(r[(4 + e) * kWave]);
            } else {
              sg[e] += r[e * kWave];
              su[e] += r[(4 + e) * kWave];
            }
          }
        }
#pragma unroll
        for (int r = 0; r < 4; r++) {  // row scale x channel scale on the finished sums (int8: the exact integer sums, converted once)
          sg[r] = (I8 ? (float)jg[r] : sg[r]) * (rs[t2] * sbuf[a * 16 + 4 * kq + r]);
          su[r] = (I8 ? (float)ju[r] : su[r]) * (rs[t2] * sbuf[(GLU ? HF : 32) + a * 16 + 4 * kq + r]);
        }
        const int n = cg * CH + a * 16 + 4 * kq;
        const int jr = 16 * (MTW * rp + t2) + j;
        const size_t row = (size_t)(tile.row0 + jr);
        if (jr < tile.nrows && tile.group < 0) {  // rows of no local group: zeros
          float z[4] = {0.f, 0.f, 0.f, 0.f};
          if (n < N) store_out4(p.out, p.ro, row, N, n, z);
          if (!GLU && n + 32 < N) store_out4(p.out, p.ro, row, N, n + 32, z);
        } else if (jr < tile.nrows) {
          if (GLU) {
            if (n < N) {
              float bg[4], bu[4];
              load_bias4(p.rhs_bias, tile.group, N, n, bg);
              load_bias4(p.rhs_up_bias, tile.group, N, n, bu);
              add_partial4(p.partial_sum, row, N, n, bg);
              add_partial4(p.partial_sum_up, row, N, n, bu);
              dispatch_act(p.act, [&](auto act_c) {
                constexpr int ACT = decltype(act_c)::value;
                float v[4];
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = glu_act<ACT>(sg[r] + bg[r], su[r] + bu[r], p.act_limit);
                store_out4(p.out, p.ro, row, N, n, v);
              });
            }
          } else {
#pragma unroll
            for (int h = 0; h < 2; h++) {
              const int nh = n + 32 * h;
              if (nh < N) {
                float b4[4], v[4];
                load_bias4(p.rhs_bias, tile.group, N, nh, b4);
                add_partial4(p.partial_sum, row, N, nh, b4);
#pragma unroll
                for (int r = 0; r < 4; r++) v[r] = (h ? su[r] : sg[r]) + b4[r];
                store_out4(p.out, p.ro, row, N, nh, v);
              }
            }
          }
        }
      }
    }
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

// The per-row x per-channel kernel: K any multiple of 512, at least four channel groups per tile, weights and activations
// within 32-bit offsets
bool f8l_takes(int K, int N, int G_local, bool glu, long long lhs_rows) {
  const int ncg = cdiv(N, glu ? 32 : 64);
  return K % 512 == 0 && K >= 512 && N % 8 == 0 && ncg >= 4 && (long long)G_local * N * K + 65LL * K + 1024 < (1LL << 32) &&
         (lhs_rows + 1) * K + 1024 < (1LL << 32);
}

template <bool GLU, bool I8, int MT>
static int launch_f8l_one(const SkinnyParams& p, int num_groups, int blocks, hipStream_t s) {
  constexpr bool NT = MOE_F8D_NT != 0;
  if (int st = reserve_lds(gmm_f8l_kernel<GLU, NT, I8, MT>, F8lLds<MT>::kBytes,
                           lds_flags<std::integral_constant<int, 7700 + (GLU ? 1 : 0) + (I8 ? 2 : 0) + (MT - 1) * 4>>()))
    return st;
  gmm_f8l_kernel<GLU, NT, I8, MT><<<blocks, kF8dThreads, F8lLds<MT>::kBytes, s>>>(p, num_groups);
  return check_launch("gmm_f8l_kernel");
}

template <int MT>
static int launch_f8l_mt(const SkinnyParams& p, bool glu, bool int8, int num_groups, int blocks, hipStream_t s) {
  if (int8) return glu ? launch_f8l_one<true, true, MT>(p, num_groups, blocks, s) : launch_f8l_one<false, true, MT>(p, num_groups, blocks, s);
  return glu ? launch_f8l_one<true, false, MT>(p, num_groups, blocks, s) : launch_f8l_one<false, false, MT>(p, num_groups, blocks, s);
}

// tile_rows: the height of the tile list's tiles, 16, 32 or 64
int launch_f8l(const SkinnyParams& p, bool glu, bool int8, int tile_rows, int num_groups, hipStream_t s) {
  int cus = 0;
  if (int st = device_cu_count(&cus)) return st;
  if (tile_rows == 16) return launch_f8l_mt<1>(p, glu, int8, num_groups, cus, s);
  if (tile_rows == 32) return launch_f8l_mt<2>(p, glu, int8, num_groups, cus, s);
  if (tile_rows == 64) return launch_f8l_mt<4>(p, glu, int8, num_groups, cus, s);
  return fail(MOE_ERR_INVALID_ARG, "gmm: tiles of %d rows for the 8-bit decode kernel", tile_rows);
}

template <int MT>
static int prepare_f8l_mt() {
  constexpr bool NT = MOE_F8D_NT != 0;
  if (int st = reserve_lds(gmm_f8l_kernel<true, NT, true, MT>, F8lLds<MT>::kBytes, lds_flags<std::integral_constant<int, 7703 + (MT - 1) * 4>>())) return st;
  if (int st = reserve_lds(gmm_f8l_kernel<false, NT, true, MT>, F8lLds<MT>::kBytes, lds_flags<std::integral_constant<int, 7702 + (MT - 1) * 4>>())) return st;
  if (int st = reserve_lds(gmm_f8l_kernel<true, NT, false, MT>, F8lLds<MT>::kBytes, lds_flags<std::integral_constant<int, 7701 + (MT - 1) * 4>>())) return st;
  return reserve_lds(gmm_f8l_kernel<false, NT, false, MT>, F8lLds<MT>::kBytes, lds_flags<std::integral_constant<int, 7700 + (MT - 1) * 4>>());
}

int prepare_f8l() {
  if (int st = prepare_f8l_mt<1>()) return st;
  if (int st = prepare_f8l_mt<2>()) return st;
  return prepare_f8l_mt<4>();
}

}  // namespace moe
