// Grouped matmul, decode sizes: bf16 activations x group-128 int4 weights with the weights streamed through LDS.

#include "moe_gmm_wqs.h"

namespace moe {

// ---------------------------------------------------------------------------------------
// With a handful of rows per expert the product is bound by the weight bytes, and what a kernel then needs is enough of
// them in flight.  The register-staged streaming kernel (moe_gmm_wq.hip) holds a wave's requests in its registers, so the
// bytes in flight are set by the occupancy; here they are set by LDS: one persistent 512-thread block per CU walks a
// contiguous run of work items (a 16-row tile of one expert x 32 output channels of both projections, or 64 channels
// of one) and copies each item's weight rows global -> LDS in segments of 8 k-blocks (64 rows x 512 B = 32 KB), three
// segments (96 KB per CU) ahead of the one being multiplied.  Nothing else is loaded in the steady state, because loads
// complete in order: a register load issued behind the copies could not be used before they land.  So
//   * the activations of the tile stay in registers for the whole run over its channel groups: wave (a, ksub) keeps, for
//     row lane%16, the k-blocks ksub, ksub + 4, ... (two per segment), already permuted to the k order of the widened
//     weights, and the row sums the offset removal needs;
//   * the group scales of an item (bf16 [channel, k-block]) are copied to LDS with its first segment;
//   * tile records and activations are read when the run enters a new tile, in a side block that completes its loads
//     (the copies in flight land meanwhile).
// Wave (a, ksub) multiplies channels a*16 .. a*16+15 of both halves of the item for its k-blocks; the four ksub waves add
// their sums through LDS at the item's end and wave (a, 0) runs the epilogue.  LDS rows are 512 B with the 16-byte chunk
// index XOR-ed by row % 16: the 16 lanes that read one chunk column of 16 rows hit 16 different bank groups.
//
// int4 values are widened as in the register-staged kernel: a nibble n (value + 8) is OR-ed into the mantissa of 128.0,
// the MFMA yields P = sum (128 + n_k) a_k, and the block's contribution is scale * (P - 136 * sum a_k) in f32.
// MXFP4 (e2m1 pairs, one e8m0 scale per 32 values = per lane and k-block) is widened by v_cvt_scalef32_pk_bf16_fp4, scale
// included, so its MFMAs add straight into the item's sums; its scales are the 32 x K/32 bytes of each half.
// ---------------------------------------------------------------------------------------

constexpr int kWqsThreads = 512;
constexpr int kWqsRing = 4;                           // segment slots: one multiplied, three in flight
constexpr int kWqsSegBytes = 64 * 512;                // 64 rows x 8 k-blocks x 64 B
// Scales of an item: two regions (one per half) of NSEG KB each (int4: 32 rows x nkb bf16 <= NSEG/2 KB; MXFP4: 32 rows x K/32
// bytes <= NSEG KB).  They arrive with the item's first segment, i.e. up to ceil(3 / NSEG) items ahead: 4, 3, 2 buffers
// for 1, 2, 3 segments per item, at most 12 KB.
constexpr int kWqsScaleArea = 16384;
constexpr int wqs_scale_ring(int nseg) { return nseg == 1 ? 4 : nseg == 2 ? 3 : 2; }
constexpr int kWqsRedBytes = 2 * 3 * 8 * kWave * 4;   // partial sums of the waves ksub = 1..3 of both channel halves
constexpr int kWqsScale0 = kWqsRing * kWqsSegBytes;
constexpr int kWqsRed0 = kWqsScale0 + kWqsScaleArea;
constexpr int kWqsLds = kWqsRed0 + kWqsRedBytes;      // 159744 bytes
constexpr int kWqsMaxKBlocks = 24;  // K <= 3072: eight k-blocks per wave (K up to 4096) do not fit the registers

// (x & mask) | c: one v_and_or_b32 when mask and c sit in registers (with literal constants the compiler emits two
// instructions, the fused one takes no literals).  Not written as asm: the hazard checks between matrix and vector
// instructions do not look inside asm statements.
__device__ __forceinline__ uint32_t and_or(uint32_t x, uint32_t mask, uint32_t c) { return (x & mask) | c; }

template <int FMT, int NSEG, bool GLU>
__global__ __launch_bounds__(kWqsThreads) void gmm_wqs_kernel(const WqSkinnyParams p, int num_groups) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  static_assert(FMT == WQ_I4 || FMT == WQ_MX4, "group-128 int4 or MXFP4");
  constexpr bool MX = FMT == WQ_MX4;
  constexpr int KBW = 2 * NSEG;  // k-blocks a wave owns
  constexpr int SRING = wqs_scale_ring(NSEG);
  constexpr int SHALF = NSEG * 1024;  // bytes of one half's scale region in LDS
  static_assert(SRING * 2 * SHALF <= kWqsScaleArea, "scale buffers");
  constexpr int CH = GLU ? 32 : 64;
  const int lane = threadIdx.x % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(threadIdx.x / kWave);
  const int a = wave / 4, ksub = wave % 4;
  const int j = lane % 16, kq = lane / 16;
  const int N = p.N, K = p.K;
  const int nkb = (K + 127) / 128;
  const uint32_t row_bytes = (uint32_t)K / 2;
  const int ncg = (N + CH - 1) / CH;
  const int ntiles = __builtin_amdgcn_readfirstlane(p.header[0]);
  const long long total = (long long)ntiles * ncg;
  const int q0 = (int)(total * blockIdx.x / gridDim.x), q1 = (int)(total * (blockIdx.x + 1) / gridDim.x);
  if (q0 >= q1) return;
  const int nitems = q1 - q0, nstream = nitems * NSEG;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  // weights and scales through buffer descriptors: a request past the end of a tensor returns zeros
  const uint32_t w_bytes = clamp_u32((size_t)num_groups * N * row_bytes);
  const uint32_t srow_bytes = MX ? (uint32_t)K / 32 : (uint32_t)nkb * 2;  // scale bytes of one channel
  const uint32_t s_bytes = clamp_u32((size_t)num_groups * N * srow_bytes);
  const v4i desc_w = buffer_desc(p.rhs, w_bytes);
  const v4i desc_u = buffer_desc(GLU ? p.rhs_up : p.rhs, w_bytes);
  const v4i sdesc_w = buffer_desc(p.rhs_scale, s_bytes);
  const v4i sdesc_u = buffer_desc(GLU ? p.rhs_up_scale : p.rhs_scale, s_bytes);
  const bool up_half = wave >= 4;  // this wave copies rows 32..63 of a segment: the second projection / channels 32..63

  // ---- the tile the run is in: record, expert of the next tile, activations of this wave's k-blocks ----
  int m_cur = q0 / ncg;
  TileInfo tile;
  int g_cur = 0, g_next = 0;
  uint4 act[KBW][4];
  float sa[KBW];
  auto load_tile = [&](int m) {
    // (read into scalar registers here: a load left pending would be waited for at its first use, behind the copies)
    const TileInfo t = p.tiles[m];
    tile.group = __builtin_amdgcn_readfirstlane(t.group);
    tile.row0 = __builtin_amdgcn_readfirstlane(t.row0);
    tile.nrows = __builtin_amdgcn_readfirstlane(t.nrows);
    g_cur = max(tile.group, 0);
    g_next = __builtin_amdgcn_readfirstlane(m + 1 < ntiles ? max(p.tiles[m + 1].group, 0) : 0);
  };
  auto load_acts = [&]() {
    const int gr = lhs_row_of(p.ro, tile.row0 + min(j, tile.nrows - 1));
    const uint8_t* arow = p.lhs + (size_t)gr * K * 2;
    const v8bf ones = __builtin_bit_cast(v8bf, make_uint4(0x3f803f80u, 0x3f803f80u, 0x3f803f80u, 0x3f803f80u));
    uint4 raw[KBW][4];
#pragma unroll
    for (int i = 0; i < KBW; i++) {
      const int k = (ksub + 4 * i) * 128 + kq * 32;
      const uint4* src = (const uint4*)(arow + (k < K ? (size_t)k * 2 : 0));
#pragma unroll
      for (int s = 0; s < 4; s++) raw[i][s] = src[s];
    }
#pragma unroll
    for (int i = 0; i < KBW; i++) {
      const bool ok = (ksub + 4 * i) * 128 + kq * 32 < K;  // the lane's 32 values exist (K % 32 == 0)
      v4f t = {0.f, 0.f, 0.f, 0.f};
#pragma unroll
      for (int s = 0; s < 4; s++) {
        const uint4 x = ok ? raw[i][s] : make_uint4(0, 0, 0, 0);
        if (MX) {
          act[i][s] = x;  // (the conversion hands out a word's values in their own order)
        } else {
          // k order (k0,k4,k1,k5,k2,k6,k3,k7): the order the nibbles of a word come out in
          act[i][s] = make_uint4(__builtin_amdgcn_perm(x.z, x.x, 0x05040100u), __builtin_amdgcn_perm(x.z, x.x, 0x07060302u),
                                 __builtin_amdgcn_perm(x.w, x.y, 0x05040100u), __builtin_amdgcn_perm(x.w, x.y, 0x07060302u));
          t = __builtin_amdgcn_mfma_f32_16x16x32_bf16(ones, __builtin_bit_cast(v8bf, act[i][s]), t, 0, 0, 0);
        }
      }
      sa[i] = -136.0f * t[0];  // what the sums of the k-block start at: the widened nibbles are 128 + 8 too large
    }
    // the loads complete here (an empty statement that "uses" every register), not at their first use behind the copies
#pragma unroll
    for (int i = 0; i < KBW; i++)
#pragma unroll
      for (int s = 0; s < 4; s++) asm volatile("" : "+v"(act[i][s].x), "+v"(act[i][s].y), "+v"(act[i][s].z), "+v"(act[i][s].w));
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
    if (s == 0 && (uint32_t)(wave % 4) * 1024u < 32u * srow_bytes) {
      // the item's scales: the rows of 32 channels of each half, contiguous in the [G, N, nkb] / [G, N, K/32] tensor (a
      // copy's last KB may run past them: what it brings is other channels' scales, or zeros past the tensor)
      const int ch0 = GLU ? cg * 32 : cg * 64 + (up_half ? 32 : 0);
      const uint32_t voff = (uint32_t)(group * N + ch0) * srow_bytes + (uint32_t)(wave % 4) * 1024u + (uint32_t)lane * 16u;
      dma16_buffer(up_half ? sdesc_u : sdesc_w, voff, 0u,
                   lds_base + kWqsScale0 + (uint32_t)(it % SRING) * (2u * SHALF) + (up_half ? (uint32_t)SHALF : 0u) + (uint32_t)(wave % 4) * 1024u);
    }
    // (channels past N in an item's last rows are the next expert's first rows, or zeros past the tensor: never stored)
    const uint32_t slot = lds_base + (uint32_t)(pos % kWqsRing) * kWqsSegBytes;
    const uint32_t base = (uint32_t)(group * N + cg * CH) * row_bytes + (uint32_t)s * 512u;
#pragma unroll
    for (int i = 0; i < 4; i++) dma16_buffer(up_half ? desc_u : desc_w, base + lane_off[i], 0u, slot + (uint32_t)(8 * wave + 2 * i) * 512u);
  };

  load_tile(m_cur);
#pragma unroll
  for (int pos = 0; pos < 3; pos++)
    if (pos < nstream) issue(pos);
  load_acts();

  float* const red = (float*)(smem + kWqsRed0);
  uint32_t M4 = 0x000f000fu, cbase = 0x43004300u;  // nibbles of a pair; two bf16 128.0: both opaque, i.e. in registers
  asm volatile("" : "+s"(M4));
  asm volatile("" : "+v"(cbase));

  for (int it = 0; it < nitems; it++) {
    const int q = q0 + it;
    const int m = q / ncg, cg = q - m * ncg;
    if (m != m_cur) {
      m_cur = m;
      load_tile(m);
      load_acts();
    }
    v4f acc_g = {0.f, 0.f, 0.f, 0.f}, acc_u = {0.f, 0.f, 0.f, 0.f};
    const uint8_t* const sbuf = smem + kWqsScale0 + (it % SRING) * (2 * SHALF);
    // int4: this lane's four channels (accumulator layout) of each half, at the wave's first k-block: the k-blocks that
    // follow are 4 entries apart.  MXFP4: the lane's own channel (operand layout), one byte per 32 values.
    const uint16_t* sc = (const uint16_t*)sbuf + (a * 16 + 4 * kq) * nkb + ksub;
    const uint8_t* scb = sbuf + (a * 16 + j) * (K / 32) + ksub * 4 + kq;
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
      const uint8_t* slot = smem + (pos % kWqsRing) * kWqsSegBytes;
      // A k-block past the last one (K not a multiple of 1024) is multiplied like the others: its activations are zeros, its
      // weights are whatever bytes follow the row, and the scale read in its place is a finite one (another channel's, or
      // the zeros a copy past the tensor's end returns), so it adds exact zeros.
#pragma unroll
      for (int b = 0; b < 2; b++) {
        const int i = 2 * s + b;
        const int c = ((ksub + 4 * b) * 4 + kq) ^ j;
        const uint4 wq = *(const uint4*)(slot + (a * 16 + j) * 512 + c * 16);
        const uint4 uq = *(const uint4*)(slot + (32 + a * 16 + j) * 512 + c * 16);
        const uint32_t xw[4] = {wq.x, wq.y, wq.z, wq.w};
        const uint32_t xu[4] = {uq.x, uq.y, uq.z, uq.w};
        if constexpr (MX) {
          // (a scale byte read past a row's end, for a k-block past the last, belongs to another channel: finite, and the
          // activations it meets are zeros)
          const float sg = __uint_as_float((uint32_t)scb[16 * i] << 23), su = __uint_as_float((uint32_t)scb[SHALF + 16 * i] << 23);
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const v8bf wf = __builtin_bit_cast(v8bf, make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xw[w], sg, 0)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xw[w], sg, 1)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xw[w], sg, 2)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xw[w], sg, 3))));
            const v8bf uf = __builtin_bit_cast(v8bf, make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xu[w], su, 0)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xu[w], su, 1)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xu[w], su, 2)),
                                                                __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(xu[w], su, 3))));
            const v8bf af = __builtin_bit_cast(v8bf, act[i][w]);
            acc_g = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af, acc_g, 0, 0, 0);
            acc_u = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf, af, acc_u, 0, 0, 0);
          }
        } else {
          float sg[4], su[4];
#pragma unroll
          for (int r = 0; r < 4; r++) {
            sg[r] = bf16_bits_to_f32(sc[r * nkb + 4 * i]);
            su[r] = bf16_bits_to_f32(sc[SHALF / 2 + r * nkb + 4 * i]);
          }
          v4f pg = {sa[i], sa[i], sa[i], sa[i]}, pu = pg;
#pragma unroll
          for (int w = 0; w < 4; w++) {
            const v8bf wf = __builtin_bit_cast(v8bf, make_uint4(and_or(xw[w], M4, cbase), and_or(xw[w] >> 4, M4, cbase), and_or(xw[w] >> 8, M4, cbase),
                                                                and_or(xw[w] >> 12, M4, cbase)));
            const v8bf uf = __builtin_bit_cast(v8bf, make_uint4(and_or(xu[w], M4, cbase), and_or(xu[w] >> 4, M4, cbase), and_or(xu[w] >> 8, M4, cbase),
                                                                and_or(xu[w] >> 12, M4, cbase)));
            const v8bf af = __builtin_bit_cast(v8bf, act[i][w]);
            pg = __builtin_amdgcn_mfma_f32_16x16x32_bf16(wf, af, pg, 0, 0, 0);
            pu = __builtin_amdgcn_mfma_f32_16x16x32_bf16(uf, af, pu, 0, 0, 0);
          }
#pragma unroll
          for (int r = 0; r < 4; r++) {
            acc_g[r] = fmaf(sg[r], pg[r], acc_g[r]);
            acc_u[r] = fmaf(su[r], pu[r], acc_u[r]);
          }
        }
      }
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

// group-128 int4 or MXFP4 with K up to 3072, at least four channel groups per tile (a copy issued three positions ahead
// then never looks past the next tile), scale rows that start on 16-byte boundaries and tensors within 32-bit offsets
bool wqs_takes(int fmt, int K, int N, int G_local, bool glu) {
  const int nkb = (K + 127) / 128;
  const int ncg = cdiv(N, glu ? 32 : 64);
  if (fmt != WQ_I4 && fmt != WQ_MX4) return false;
  const long long srow = fmt == WQ_MX4 ? K / 32 : nkb * 2;
  return K % 32 == 0 && nkb <= kWqsMaxKBlocks && N % 8 == 0 && ncg >= 4 && ((long long)N * srow) % 16 == 0 && (32 * srow) % 16 == 0 &&
         (long long)G_local * N * (K / 2) + 65LL * (K / 2) + 1024 < (1LL << 32);  // (an item's last rows may lie up to 63 rows past N)
}

template <int FMT, int NSEG, bool GLU>
static int launch_wqs_one(const WqSkinnyParams& p, int num_groups, int blocks, hipStream_t s) {
  if (int st = reserve_lds(gmm_wqs_kernel<FMT, NSEG, GLU>, kWqsLds, lds_flags<std::integral_constant<int, 7000 + FMT * 100 + NSEG * 2 + (GLU ? 1 : 0)>>()))
    return st;
  gmm_wqs_kernel<FMT, NSEG, GLU><<<blocks, kWqsThreads, kWqsLds, s>>>(p, num_groups);
  return check_launch("gmm_wqs_kernel");
}

template <int FMT>
static int launch_wqs_fmt(const WqSkinnyParams& p, bool glu, int num_groups, int blocks, hipStream_t s) {
  switch (cdiv(cdiv(p.K, 128), 8)) {
    case 1: return glu ? launch_wqs_one<FMT, 1, true>(p, num_groups, blocks, s) : launch_wqs_one<FMT, 1, false>(p, num_groups, blocks, s);
    case 2: return glu ? launch_wqs_one<FMT, 2, true>(p, num_groups, blocks, s) : launch_wqs_one<FMT, 2, false>(p, num_groups, blocks, s);
    case 3: return glu ? launch_wqs_one<FMT, 3, true>(p, num_groups, blocks, s) : launch_wqs_one<FMT, 3, false>(p, num_groups, blocks, s);
  }
  return fail(MOE_ERR_UNSUPPORTED, "gmm: K = %d is past the LDS-streamed decode kernel", p.K);
}

int launch_wqs(int fmt, const WqSkinnyParams& p, bool glu, int num_groups, hipStream_t s) {
  int cus = 0;
  if (int st = device_cu_count(&cus)) return st;
  return fmt == WQ_MX4 ? launch_wqs_fmt<WQ_MX4>(p, glu, num_groups, cus, s) : launch_wqs_fmt<WQ_I4>(p, glu, num_groups, cus, s);
}

template <int FMT, int NSEG>
static int prepare_wqs_pair() {
  if (int st = reserve_lds(gmm_wqs_kernel<FMT, NSEG, true>, kWqsLds, lds_flags<std::integral_constant<int, 7000 + FMT * 100 + NSEG * 2 + 1>>())) return st;
  return reserve_lds(gmm_wqs_kernel<FMT, NSEG, false>, kWqsLds, lds_flags<std::integral_constant<int, 7000 + FMT * 100 + NSEG * 2>>());
}

int prepare_wqs() {
  if (int st = prepare_wqs_pair<WQ_I4, 1>()) return st;
  if (int st = prepare_wqs_pair<WQ_I4, 2>()) return st;
  if (int st = prepare_wqs_pair<WQ_I4, 3>()) return st;
  if (int st = prepare_wqs_pair<WQ_MX4, 1>()) return st;
  if (int st = prepare_wqs_pair<WQ_MX4, 2>()) return st;
  return prepare_wqs_pair<WQ_MX4, 3>();
}

}  // namespace moe
