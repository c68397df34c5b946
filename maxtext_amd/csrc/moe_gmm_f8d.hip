// Grouped matmul, decode sizes: block-scaled fp8 x fp8 with the weights streamed through LDS.

#include "moe_gmm_f8d.h"

namespace moe {

// ---------------------------------------------------------------------------------------
// The DeepSeek decode problem (float8_e4m3 activations with one scale per row and 128 values of K, float8_e4m3 weights with
// one scale per 128 x 128 block, a handful of rows per expert) is bound by the weight bytes.  The register-staged kernel
// (gmm_fp8_skinny_kernel) gives every wave its own 16 x 32 channel strip: each wave pays its own start-up, requests its
// own copy of the activations and scales, and the bytes in flight depend on the occupancy.  Here one persistent
// 512-thread block per CU walks a contiguous run of work items (a 16-row tile of one expert x 32 output channels of both
// projections, or 64 channels of one) and copies each item's weight rows global -> LDS in segments of four k-blocks
// (64 rows x 512 B = 32 KB), three segments ahead of the one being multiplied, exactly as the 4-bit decode kernel
// (moe_gmm_wqs.hip) does.  Loads complete in order, so nothing but the copies is loaded in the steady state:
//   * the tile's activations stay in registers across its channel groups: wave (a, ksub) keeps, for row lane % 16, the
//     k-blocks ksub, ksub + 4, ... (one per segment) with their scales;
//   * the block scales of an item's weights (one f32 per k-block and half) are copied to LDS with its first segment;
//   * tile records and activations are read when the run enters a new tile, in a side block that completes its loads.
// Wave (a, ksub) multiplies channels a*16 .. a*16+15 of both halves for its k-block of the segment: one
// v_mfma_f32_16x16x128_f8f6f4 per half, whose 16 x 16 sums are scaled by a_scale[row, kb] * w_scale[kb] and added in f32.
// The four ksub waves add their sums through LDS at the item's end and wave (a, 0) runs the epilogue.  LDS rows are 512 B
// with the 16-byte chunk index XOR-ed by row % 16.
// ---------------------------------------------------------------------------------------

constexpr int kF8dRing = 4;               // segment slots: one multiplied, three in flight
constexpr int kF8dSegBytes = 64 * 512;    // 64 rows x 4 k-blocks x 128 B
constexpr int kF8dMaxSeg = 14;            // K <= 7168: the activations of 14 k-blocks per wave fill 112 registers
constexpr int kF8dScaleBuf = 2 * 1024;    // an item's weight scales: the KB a copy brings for each half (K/128 floats used)
constexpr int f8d_scale_ring(int nseg) { return nseg == 1 ? 4 : nseg == 2 ? 3 : 2; }  // they arrive up to ceil(3 / NSEG) items ahead
constexpr int kF8dScale0 = kF8dRing * kF8dSegBytes;
constexpr int kF8dRed0 = kF8dScale0 + 4 * kF8dScaleBuf;
constexpr int kF8dLds = kF8dRed0 + kF8dRedBytes;     // 151552 bytes

template <int NSEG, bool GLU, bool NT>
__global__ __launch_bounds__(kF8dThreads) void gmm_f8d_kernel(const SkinnyParams p, int num_groups) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  static_assert(NSEG >= 1 && NSEG <= kF8dMaxSeg, "segments per item");
  constexpr int SRING = f8d_scale_ring(NSEG);
  constexpr int CH = GLU ? 32 : 64;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int a = wave / 4, ksub = wave % 4;
  const int j = lane % 16, kq = lane / 16;
  const int N = p.N, K = p.K;
  constexpr int nkb = 4 * NSEG;  // K == NSEG * 512 (the host checks)
  const uint32_t row_bytes = (uint32_t)K;
  const int ncg = (N + CH - 1) / CH;
  const int nnb = (N + 127) / 128;
  const int ntiles = __builtin_amdgcn_readfirstlane(p.header[0]);
  const long long total = (long long)ntiles * ncg;
  // ---- the run of items this block takes: an even split of the list, except ... ----
  // ... when the last expert has several tiles (the shared expert of a DeepSeek layer: every token's rows) and a tile is
  // about one block's share of the work.  Then its tiles go one each to blocks of one XCD (blocks are dealt round-robin to
  // the 8 XCDs: those with index 8k + 7), which walk the same channel groups side by side and find each item's weights in
  // that XCD's L2 after the first of them has read it; the other blocks split the other tiles' items evenly.
  const int nb = (int)gridDim.x, b = (int)blockIdx.x;
  int nsh = 0;
  if (ntiles >= 2 && nb % 8 == 0) {
    const int last = ntiles - 1;
    const int gl = __builtin_amdgcn_readfirstlane(p.tiles[last].group);
    const int gk = last - 1 - lane >= 0 ? p.tiles[last - 1 - lane].group : -3;  // lane k: the tile k + 1 before the last
    const unsigned long long same = __ballot(gk == gl && gl >= 0);
    const int run = same == ~0ull ? 64 : __builtin_ctzll(~same);  // tiles right before the last one that belong to its expert
    const long long share = total / nb;
    if (run >= 1 && run < 64 && run + 1 <= nb / 8 && 2LL * ncg >= share && 4LL * ncg <= 5 * share) nsh = run + 1;
  }
  int q0, q1;
  if (nsh && b % 8 == 7 && b / 8 < nsh) {
    q0 = (ntiles - nsh + b / 8) * ncg;
    q1 = q0 + ncg;
  } else if (nsh) {
    const int r = b - min(nsh, b / 8), nbo = nb - nsh;  // rank among the other blocks
    const long long others = (long long)(ntiles - nsh) * ncg;
    q0 = (int)(others * r / nbo);
    q1 = (int)(others * (r + 1) / nbo);
  } else {
    q0 = (int)(total * b / nb);
    q1 = (int)(total * (b + 1) / nb);
  }
  if (q0 >= q1) return;
  const int nitems = q1 - q0, nstream = nitems * NSEG;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  // weights and scales through buffer descriptors: a request past the end of a tensor returns zeros
  const uint32_t w_bytes = clamp_u32((size_t)num_groups * N * row_bytes);
  const uint32_t s_bytes = clamp_u32((size_t)num_groups * nnb * nkb * 4);
  const v4i desc_w = buffer_desc(p.rhs, w_bytes);
  const v4i desc_u = buffer_desc(GLU ? p.rhs_up : p.rhs, w_bytes);
  const v4i sdesc_w = buffer_desc(p.rhs_scale, s_bytes);
  const v4i sdesc_u = buffer_desc(GLU ? p.rhs_up_scale : p.rhs_scale, s_bytes);
  const bool up_half = wave >= 4;  // this wave copies rows 32..63 of a segment: the second projection / channels 32..63

  // ---- the tile the run is in: record, expert of the next tile, activations and scales of this wave's k-blocks ----
  int m_cur = q0 / ncg;
  TileInfo tile;
  int g_cur = 0, g_next = 0, shared_cur = 0, shared_next = 0;
  v8i act[NSEG];
  float as[NSEG];
  auto load_tile = [&](int m) {
    // (read into scalar registers here: a load left pending would be waited for at its first use, behind the copies)
    const TileInfo t = p.tiles[m];
    tile.group = __builtin_amdgcn_readfirstlane(t.group);
    tile.row0 = __builtin_amdgcn_readfirstlane(t.row0);
    tile.nrows = __builtin_amdgcn_readfirstlane(t.nrows);
    g_cur = max(tile.group, 0);
    const int gp = m > 0 ? p.tiles[m - 1].group : -2, gn = m + 1 < ntiles ? p.tiles[m + 1].group : -2, gnn = m + 2 < ntiles ? p.tiles[m + 2].group : -2;
    g_next = __builtin_amdgcn_readfirstlane(max(gn, 0));
    // an expert of several tiles (the shared expert of a DeepSeek layer: every token's rows) is read once per tile, by
    // blocks that walk its channel groups side by side: those copies stay temporal so that the later ones hit in the caches
    shared_cur = __builtin_amdgcn_readfirstlane((int)(tile.group >= 0 && (gp == tile.group || gn == tile.group)));
    shared_next = __builtin_amdgcn_readfirstlane((int)(gn >= 0 && (gn == tile.group || gnn == gn)));
  };
  auto load_acts = [&]() {
    // lane (j, kq) takes bytes kq*16.. and 64 + kq*16.. of its row's k-block: the order the weight fragments are read in
    const int gr = lhs_row_of(p.ro, tile.row0 + min(j, tile.nrows - 1));
    const uint8_t* arow = p.lhs + (size_t)gr * K + kq * 16;
    const float* asr = p.lhs_scale + (size_t)gr * nkb;
#pragma unroll
    for (int i = 0; i < NSEG; i++) {
      const int kb = 4 * i + ksub;
      const uint4 x = *(const uint4*)(arow + kb * 128), y = *(const uint4*)(arow + kb * 128 + 64);
      act[i][0] = x.x; act[i][1] = x.y; act[i][2] = x.z; act[i][3] = x.w;
      act[i][4] = y.x; act[i][5] = y.y; act[i][6] = y.z; act[i][7] = y.w;
      as[i] = asr[kb];
    }
    // the loads complete here (an empty statement that "uses" every register), not at their first use behind the copies
#pragma unroll
    for (int i = 0; i < NSEG; i++) {
      asm volatile("" : "+v"(act[i]));
      asm volatile("" : "+v"(as[i]));
    }
  };

  // ---- copies of one stream position: segment s of item q into ring slot `slot` ----
  // the lane's part of a copy's offset: row 8 * wave + 2 * i + lane / 32 of the segment (rows 0..31 the first half, 32..63
  // the second: the other projection, or channels 32..63), the 16-byte chunk XOR-ed with row % 16
  uint32_t lane_off[4];
#pragma unroll
  for (int i = 0; i < 4; i++) {
    const int row = 8 * wave + 2 * i + lane / 32;
    lane_off[i] = (uint32_t)(GLU ? row % 32 : row) * row_bytes + (uint32_t)((lane % 32) ^ (row & 15)) * 16u;
  }
  auto issue = [&](int pos) {
    const int it = pos / NSEG, s = pos - it * NSEG;
    const int q = q0 + it;
    const int m = q / ncg, cg = q - m * ncg;
    const int group = m == m_cur ? g_cur : g_next;  // (three positions ahead never leave the next tile: ncg >= 4)
    const bool temporal = !NT || (m == m_cur ? shared_cur : shared_next) != 0;
    if (s == 0 && wave % 4 == 0) {
      // the item's weight scales: the K/128 floats of its 128-channel block (a copy brings a whole KB: what follows
      // them is other blocks' scales, or zeros past the tensor)
      const uint32_t voff = (uint32_t)((group * nnb + cg * CH / 128) * nkb) * 4u + (uint32_t)lane * 16u;
      f8d_copy<false>(up_half ? sdesc_u : sdesc_w, voff, lds_base + kF8dScale0 + (uint32_t)(it % SRING) * kF8dScaleBuf + (up_half ? 1024u : 0u));
    }
    // (channels past N in an item's last rows are the next expert's first rows, or zeros past the tensor: never stored)
    const uint32_t slot = lds_base + (uint32_t)(pos % kF8dRing) * kF8dSegBytes;
    const uint32_t base = (uint32_t)(group * N + cg * CH) * row_bytes + (uint32_t)s * 512u;
    if (temporal) {
#pragma unroll
      for (int i = 0; i < 4; i++) f8d_copy<false>(up_half ? desc_u : desc_w, base + lane_off[i], slot + (uint32_t)(8 * wave + 2 * i) * 512u);
    } else {
#pragma unroll
      for (int i = 0; i < 4; i++) f8d_copy<true>(up_half ? desc_u : desc_w, base + lane_off[i], slot + (uint32_t)(8 * wave + 2 * i) * 512u);
    }
  };

  load_tile(m_cur);
#pragma unroll
  for (int pos = 0; pos < 3; pos++)
    if (pos < nstream) issue(pos);
  load_acts();

  float* const red = (float*)(smem + kF8dRed0);
  const v4f zero = {0.f, 0.f, 0.f, 0.f};

  for (int it = 0; it < nitems; it++) {
    const int q = q0 + it;
    const int m = q / ncg, cg = q - m * ncg;
    if (m != m_cur) {
      m_cur = m;
      load_tile(m);
      load_acts();
    }
    v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    const float* const sbuf = (const float*)(smem + kF8dScale0 + (it % SRING) * kF8dScaleBuf);
#pragma unroll
    for (int s = 0; s < NSEG; s++) {
      const int pos = it * NSEG + s;
      // this wave's copies of the segment have landed once at most the copies of the younger segments are outstanding
      const int younger = min(2, nstream - 1 - pos);
      if (younger == 2) wait_vmcnt<8>();
      else if (younger == 1) wait_vmcnt<4>();
      else wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      // every wave has left the slot of the segment before this one: it takes the segment three ahead
      if (pos + 3 < nstream) issue(pos + 3);
      const uint8_t* slot = smem + (pos % kF8dRing) * kF8dSegBytes;
      const int kb = 4 * s + ksub;
      const int c0 = (ksub * 8 + kq) ^ j, c1 = (ksub * 8 + 4 + kq) ^ j;
      const uint8_t* wrow = slot + (a * 16 + j) * 512;
      const uint8_t* urow = slot + (32 + a * 16 + j) * 512;
      const uint4 w0 = *(const uint4*)(wrow + c0 * 16), w1 = *(const uint4*)(wrow + c1 * 16);
      const uint4 u0 = *(const uint4*)(urow + c0 * 16), u1 = *(const uint4*)(urow + c1 * 16);
      v8i wf, uf;
      wf[0] = w0.x; wf[1] = w0.y; wf[2] = w0.z; wf[3] = w0.w; wf[4] = w1.x; wf[5] = w1.y; wf[6] = w1.z; wf[7] = w1.w;
      uf[0] = u0.x; uf[1] = u0.y; uf[2] = u0.z; uf[3] = u0.w; uf[4] = u1.x; uf[5] = u1.y; uf[6] = u1.z; uf[7] = u1.w;
      const v4f pg = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wf, act[s], zero, 0, 0, 0, 127, 0, 127);
      const v4f pu = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(uf, act[s], zero, 0, 0, 0, 127, 0, 127);
      const float fg = as[s] * sbuf[kb], fu = as[s] * sbuf[256 + kb];
#pragma unroll
      for (int r = 0; r < 4; r++) {
        acc_g[r] = fmaf(pg[r], fg, acc_g[r]);
        acc_u[r] = fmaf(pu[r], fu, acc_u[r]);
      }
      // (the sums are final here: left alone, the compiler keeps every segment's products to add them at the item's end)
      asm volatile("" : "+v"(acc_g), "+v"(acc_u));
    }

    // ---- sums of the waves ksub = 1..3 -> LDS -> wave (a, 0) ----
    if (ksub > 0) {
      float* r = red + (size_t)((a * 3 + ksub - 1) * 8) * kWave + lane;
#pragma unroll
      for (int e = 0; e < 4; e++) {
        r[e * kWave] = acc_g[e];
        r[(4 + e) * kWave] = acc_u[e];
      }
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0): the sums are in LDS
    asm volatile("s_barrier" ::: "memory");
    if (ksub == 0) {
#pragma unroll
      for (int w = 0; w < 3; w++) {
        const float* r = red + (size_t)((a * 3 + w) * 8) * kWave + lane;
#pragma unroll
        for (int e = 0; e < 4; e++) {
          acc_g[e] += r[e * kWave];
          acc_u[e] += r[(4 + e) * kWave];
        }
      }
      const int n = cg * CH + a * 16 + 4 * kq;
      const size_t row = (size_t)(tile.row0 + j);
      if (j < tile.nrows && tile.group < 0) {  // rows of no local group: zeros
        float z[4] = {0.f, 0.f, 0.f, 0.f};
        if (n < N) store_out4(p.out, p.ro, row, N, n, z);
        if (!GLU && n + 32 < N) store_out4(p.out, p.ro, row, N, n + 32, z);
      } else if (j < tile.nrows) {
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
              for (int r = 0; r < 4; r++) v[r] = glu_act<ACT>(acc_g[r] + bg[r], acc_u[r] + bu[r], p.act_limit);
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
              for (int r = 0; r < 4; r++) v[r] = (h ? acc_u[r] : acc_g[r]) + b4[r];
              store_out4(p.out, p.ro, row, N, nh, v);
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

// K a multiple of 512 up to 7168 (whole segments), at least four
// channel groups per tile (a copy issued three positions ahead then never looks past the next tile), 16-byte aligned
// scale rows (K % 512 == 0 gives that) and tensors within 32-bit offsets
bool f8d_takes(int K, int N, int G_local, bool glu) {
  const int ncg = cdiv(N, glu ? 32 : 64);
  return K % 512 == 0 && K / 512 <= kF8dMaxSeg && N % 8 == 0 && ncg >= 4 && (long long)G_local * N * K + 65LL * K + 1024 < (1LL << 32);  // (an item's last rows may lie up to 63 rows past N)
}


template <int NSEG, bool GLU>
static int launch_f8d_one(const SkinnyParams& p, int num_groups, int blocks, hipStream_t s) {
  constexpr bool NT = MOE_F8D_NT != 0;
  if (int st = reserve_lds(gmm_f8d_kernel<NSEG, GLU, NT>, kF8dLds, lds_flags<std::integral_constant<int, 7500 + NSEG * 2 + (GLU ? 1 : 0)>>())) return st;
  gmm_f8d_kernel<NSEG, GLU, NT><<<blocks, kF8dThreads, kF8dLds, s>>>(p, num_groups);
  return check_launch("gmm_f8d_kernel");
}

template <int NSEG>
static int launch_f8d_seg(const SkinnyParams& p, bool glu, int num_groups, int blocks, hipStream_t s) {
  return glu ? launch_f8d_one<NSEG, true>(p, num_groups, blocks, s) : launch_f8d_one<NSEG, false>(p, num_groups, blocks, s);
}

int launch_f8d(const SkinnyParams& p, bool glu, int num_groups, hipStream_t s) {
  int cus = 0;
  if (int st = device_cu_count(&cus)) return st;
  switch (p.K / 512) {
    case 1: return launch_f8d_seg<1>(p, glu, num_groups, cus, s);
    case 2: return launch_f8d_seg<2>(p, glu, num_groups, cus, s);
    case 3: return launch_f8d_seg<3>(p, glu, num_groups, cus, s);
    case 4: return launch_f8d_seg<4>(p, glu, num_groups, cus, s);
    case 5: return launch_f8d_seg<5>(p, glu, num_groups, cus, s);
    case 6: return launch_f8d_seg<6>(p, glu, num_groups, cus, s);
    case 7: return launch_f8d_seg<7>(p, glu, num_groups, cus, s);
    case 8: return launch_f8d_seg<8>(p, glu, num_groups, cus, s);
    case 9: return launch_f8d_seg<9>(p, glu, num_groups, cus, s);
    case 10: return launch_f8d_seg<10>(p, glu, num_groups, cus, s);
    case 11: return launch_f8d_seg<11>(p, glu, num_groups, cus, s);
    case 12: return launch_f8d_seg<12>(p, glu, num_groups, cus, s);
    case 13: return launch_f8d_seg<13>(p, glu, num_groups, cus, s);
    case 14: return launch_f8d_seg<14>(p, glu, num_groups, cus, s);
  }
  return fail(MOE_ERR_UNSUPPORTED, "gmm: K = %d is not a shape of the LDS-streamed fp8 decode kernel", p.K);
}

template <int NSEG>
static int prepare_f8d_pair() {
  constexpr bool NT = MOE_F8D_NT != 0;
  if (int st = reserve_lds(gmm_f8d_kernel<NSEG, true, NT>, kF8dLds, lds_flags<std::integral_constant<int, 7500 + NSEG * 2 + 1>>())) return st;
  return reserve_lds(gmm_f8d_kernel<NSEG, false, NT>, kF8dLds, lds_flags<std::integral_constant<int, 7500 + NSEG * 2>>());
}


int prepare_f8d() {
  if (int st = prepare_f8d_pair<1>()) return st;
  if (int st = prepare_f8d_pair<2>()) return st;
  if (int st = prepare_f8d_pair<3>()) return st;
  if (int st = prepare_f8d_pair<4>()) return st;
  if (int st = prepare_f8d_pair<5>()) return st;
  if (int st = prepare_f8d_pair<6>()) return st;
  if (int st = prepare_f8d_pair<7>()) return st;
  if (int st = prepare_f8d_pair<8>()) return st;
  if (int st = prepare_f8d_pair<9>()) return st;
  if (int st = prepare_f8d_pair<10>()) return st;
  if (int st = prepare_f8d_pair<11>()) return st;
  if (int st = prepare_f8d_pair<12>()) return st;
  if (int st = prepare_f8d_pair<13>()) return st;
  return prepare_f8d_pair<14>();
}

}  // namespace moe
