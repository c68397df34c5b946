// Grouped matmul: the streaming kernel for bf16 activations x int8 / int4 / mxfp4 weights (decode).

#include "moe_gmm_common.h"

namespace moe {

// ---------------------------------------------------------------------------------------
// Weight-only int8 / int4 for few rows per expert (decode): bf16 activations, weights widened to bf16 in
// registers, v_mfma_f32_16x16x32_bf16.  Same streaming structure as the fp8 kernel: no LDS, one wave owns
// 16*NT output channels and walks K in 128-element blocks; lane (n = lane%16, kq = lane/16) holds 32 k values
// of the block for its channel (4-bit: kq*32.. ; int8: kq*16.. and 64 + kq*16..) and the matching 64 bytes of
// its activation row.  int4 weights are multiplied by their group-128 scale while
// they are widened; the int8 per-channel scale is applied once at the end.
// ---------------------------------------------------------------------------------------


// Raw weight bytes of one lane for one 128-wide k block: 32 values = 16 bytes (int4) or 32 bytes (int8).

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
    zero_fill_tile(p.out, p.ro, tile.row0, tile.nrows, n_b, NSUB * WN, N, threadIdx.x, 256);
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
    const int gr = lhs_row_of(p.ro, tile.row0 + min(mt * 16 + j, tile.nrows - 1));
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
#pragma unroll
        for (int r = 0; r < 4; r++) {
          const size_t at = (size_t)tile.group * p.ch_gstride + (size_t)(n + r) * p.ch_nstride;
          sg[r] = ((const float*)p.rhs_scale)[at];
          if (GLU) su[r] = ((const float*)p.rhs_up_scale)[at];
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
        store_out4(p.out, p.ro, (size_t)(tile.row0 + lr), N, n, v);
      }
    }
  });
}


// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

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

// K is split over the 4 waves of a block; `tune` == 1 gives every wave all of K instead (measured slower up to 32 rows
// per expert; kept for the tuning entry point).
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

int launch_wq(int fmt, bool one_tile, const WqSkinnyParams& q, bool glu, int mx, int tune, hipStream_t s) {
#define MOE_WQ_CASE(FMT) \
  if (fmt == FMT) return one_tile ? launch_wq_skinny<FMT, 1>(q, glu, mx, tune, s) : launch_wq_skinny<FMT, 2>(q, glu, mx, tune, s);
  MOE_WQ_CASE(WQ_I8)
  MOE_WQ_CASE(WQ_I4)
  MOE_WQ_CASE(WQ_MX4)
  MOE_WQ_CASE(WQ_I4G32)
#undef MOE_WQ_CASE
  return fail(MOE_ERR_INVALID_ARG, "gmm: unknown streaming weight format %d", fmt);
}

}  // namespace moe
