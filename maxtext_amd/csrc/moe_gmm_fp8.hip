// Grouped matmul: the block-scaled fp8 kernels (streaming for decode, LDS-tiled for prefill).

#include "moe_gmm_common.h"

namespace moe {

// ---------------------------------------------------------------------------------------
// Block-scaled fp8 for few rows per expert.  One wave = 16 output channels x (16*MT) rows x all K.
// Weights and activations are read straight from global memory (activations hit in L2: every
// wave of a tile reads the same rows); nothing is shared between waves, so there are no barriers.
// ---------------------------------------------------------------------------------------


// Activation fragment of one 128-byte k-block: lane (j, kq) takes bytes kq*16.. and 64+kq*16.. of its row,
// the k order load_w128 leaves the weights in.
__device__ __forceinline__ v8i load_a128(const uint8_t* p) {
  const uint4 a = *(const uint4*)p, b = *(const uint4*)(p + 64);
  v8i r;
  r[0] = a.x; r[1] = a.y; r[2] = a.z; r[3] = a.w;
  r[4] = b.x; r[5] = b.y; r[6] = b.z; r[7] = b.w;
  return r;
}

// The two whole-line requests of a 128-byte weight k-block as they arrive (channels i%8 and i%8 + 8), and the
// fragment made of them once they are there.
struct RawW128 { v4i lo, hi; };
template <bool STREAM>
__device__ __forceinline__ RawW128 request_w128(const uint8_t* lo_rows, const uint8_t* hi_rows) {
  return RawW128{load_w16<STREAM>(lo_rows), load_w16<STREAM>(hi_rows)};
}
__device__ __forceinline__ v8i fragment_w128(const RawW128& w) {
  v4i x, y;
  own_channel_pieces(w.lo, w.hi, x, y);
  v8i r;
#pragma unroll
  for (int c = 0; c < 4; c++) {
    r[c] = x[c];
    r[4 + c] = y[c];
  }
  return r;
}

// One wave owns NT tiles of 16 output channels (x2 with GLU) and MT tiles of 16 rows, and walks K in
// steps of U 128-byte blocks whose loads are all issued before the first MFMA of the step (the compiler unrolls the
// loop and moves the next steps' requests ahead of the current step's MFMAs as far as the registers allow).
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
    zero_fill_tile(p.out, p.ro, tile.row0, tile.nrows, n_w, WN, N, lane, kWave);
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
    wsp[t] = p.rhs_scale ? p.rhs_scale + srow : nullptr;
    usp[t] = GLU && p.rhs_up_scale ? p.rhs_up_scale + srow : nullptr;
  }
  const uint8_t* ap[MT];
  const float* asp[MT];
#pragma unroll
  for (int mt = 0; mt < MT; mt++) {
    const int gr = lhs_row_of(p.ro, tile.row0 + min(mt * 16 + j, tile.nrows - 1));
    ap[mt] = p.lhs + (size_t)gr * K + kq * 16;
    asp[mt] = p.lhs_scale ? p.lhs_scale + (size_t)gr * nkb : nullptr;
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

  // operands of one step of UC k-blocks, as requested
  auto request = [&](int kb0, auto ucount, RawW128 (&wf)[U][NT], RawW128 (&uf)[U][GLU ? NT : 1], v8i (&af)[U][MT],
                     float (&ws)[U][NT], float (&us)[U][NT], float (&as)[U][MT]) {
    constexpr int UC = decltype(ucount)::value;
#pragma unroll
    for (int u = 0; u < UC; u++) {
      const size_t off = (size_t)(kb0 + u) * 128;
#pragma unroll
      for (int t = 0; t < NT; t++) {
        wf[u][t] = request_w128<MT == 1>(wbase + wlo[t] + off, wbase + whi[t] + off);
        if (GLU) uf[u][t] = request_w128<MT == 1>(ubase + wlo[t] + off, ubase + whi[t] + off);
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) af[u][mt] = load_a128(ap[mt] + off);
    }
#pragma unroll
    for (int u = 0; u < UC; u++) {
#pragma unroll
      for (int t = 0; t < NT; t++) {
        // no block scales (per-row x per-channel operands): every block counts as 1
        ws[u][t] = wsp[t] ? wsp[t][kb0 + u] : 1.0f;
        us[u][t] = GLU ? (usp[t] ? usp[t][kb0 + u] : 1.0f) : 0.f;
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) as[u][mt] = asp[mt] ? asp[mt][kb0 + u] : 1.0f;
    }
  };
  auto multiply = [&](auto ucount, const RawW128 (&wf)[U][NT], const RawW128 (&uf)[U][GLU ? NT : 1], const v8i (&af)[U][MT],
                      const float (&ws)[U][NT], const float (&us)[U][NT], const float (&as)[U][MT]) {
    constexpr int UC = decltype(ucount)::value;
#pragma unroll
    for (int u = 0; u < UC; u++)
#pragma unroll
      for (int t = 0; t < NT; t++) {
        const v8i w = fragment_w128(wf[u][t]);
        v8i wu = w;
        if (GLU) wu = fragment_w128(uf[u][t]);
#pragma unroll
        for (int mt = 0; mt < MT; mt++) {
          const v4f pg = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, af[u][mt], zero, 0, 0, 0, 127, 0, 127);
          const float sg = as[u][mt] * ws[u][t];
#pragma unroll
          for (int r = 0; r < 4; r++) acc_g[t][mt][r] = fmaf(pg[r], sg, acc_g[t][mt][r]);
          if (GLU) {
            const v4f pu = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(wu, af[u][mt], zero, 0, 0, 0, 127, 0, 127);
            const float su = as[u][mt] * us[u][t];
#pragma unroll
            for (int r = 0; r < 4; r++) acc_u[t][mt][r] = fmaf(pu[r], su, acc_u[t][mt][r]);
          }
        }
      }
  };

  RawW128 wf0[U][NT], uf0[U][GLU ? NT : 1];
  v8i af0[U][MT];
  float ws0[U][NT], us0[U][NT], as0[U][MT];
  constexpr std::integral_constant<int, U> full{};
  constexpr std::integral_constant<int, 1> one{};
  const int nfull = nkb / U;
  for (int s = 0; s < nfull; s++) {
    request(s * U, full, wf0, uf0, af0, ws0, us0, as0);
    multiply(full, wf0, uf0, af0, ws0, us0, as0);
  }
  for (int kb = nfull * U; kb < nkb; kb++) {
    request(kb, one, wf0, uf0, af0, ws0, us0, as0);
    multiply(one, wf0, uf0, af0, ws0, us0, as0);
  }

  dispatch_act(GLU ? p.act : MOE_ACT_NONE, [&](auto act_c) {
    constexpr int ACT = decltype(act_c)::value;
#pragma unroll
    for (int t = 0; t < NT; t++) {
      const int n = n_w + t * 16 + 4 * kq;
      if (n >= N) continue;
      float bg[4], bu[4];
      load_bias4(p.rhs_bias, tile.group, N, n, bg);
      load_bias4(GLU ? p.rhs_up_bias : nullptr, tile.group, N, n, bu);
      // per-channel scales of the finished sums (operands without block scales)
      float cg[4] = {1.f, 1.f, 1.f, 1.f}, cu[4] = {1.f, 1.f, 1.f, 1.f};
      if (p.ch_scale) {
#pragma unroll
        for (int r = 0; r < 4; r++) {
          cg[r] = p.ch_scale[(size_t)tile.group * p.ch_gstride + (size_t)(n + r) * p.ch_nstride];
          if (GLU) cu[r] = p.ch_scale_up[(size_t)tile.group * p.ch_gstride + (size_t)(n + r) * p.ch_nstride];
        }
      }
#pragma unroll
      for (int mt = 0; mt < MT; mt++) {
        const int lr = mt * 16 + j;
        if (lr >= tile.nrows) continue;
        float pg[4] = {bg[0], bg[1], bg[2], bg[3]}, pu[4] = {bu[0], bu[1], bu[2], bu[3]};
        add_partial4(p.partial_sum, (size_t)(tile.row0 + lr), N, n, pg);
        add_partial4(GLU ? p.partial_sum_up : nullptr, (size_t)(tile.row0 + lr), N, n, pu);
        const float sa = p.row_scale_lhs ? p.row_scale_lhs[(size_t)lhs_row_of(p.ro, tile.row0 + lr) * p.row_scale_lhs_stride] : 1.0f;
        float v[4];
#pragma unroll
        for (int r = 0; r < 4; r++)
          v[r] = GLU ? glu_act<ACT>(fmaf(acc_g[t][mt][r], sa * cg[r], pg[r]), fmaf(acc_u[t][mt][r], sa * cu[r], pu[r]), p.act_limit)
                     : fmaf(acc_g[t][mt][r], sa * cg[r], pg[r]);
        store_out4(p.out, p.ro, (size_t)(tile.row0 + lr), N, n, v);
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
  // (the order covers the tiles that exist, not the host's upper bound: see gmm_tiled_kernel)
  const int num_tiles = p.header[0];
  const int total = num_tiles * p.tiles_n;
  TileInfo tile;
  int n0;
  {
    const int id = blockIdx.x;
    if (id >= total) return;
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(num_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    n0 = ((logical % width) / gsz) * C::OUT_BN;
    tile = p.tiles[m_idx];
  }
  if (tile.group < 0) {
    zero_fill_tile(p.out, p.ro, tile.row0, tile.nrows, n0, C::OUT_BN, N, tid, C::THREADS);
    return;
  }

  // ---- per-lane sources of this wave's requests: lane l asks for row l / CPR, chunk (l % CPR) ^ swz(row) ----
  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
#pragma unroll
  for (int i = 0; i < C::A_IPW; i++) {
    const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(r);
    a_src[i] = p.lhs + (size_t)lhs_row_of(p.ro, tile.row0 + min(r, tile.nrows - 1)) * K + q * 16;
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
    as_ptr[i] = P.a_scale + (size_t)lhs_row_of(p.ro, tile.row0 + min(lr, tile.nrows - 1)) * nkb;
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
  // operands without block scales (per-row x per-channel scales, applied by the epilogue): every block counts as 1
  const bool unit = P.a_scale == nullptr;
  auto load_a_scales = [&](int kb) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      if (unit) {
#pragma unroll
        for (int c = 0; c < GRP; c++) as_grp[i][c] = 1.0f;
      } else if constexpr (C::VEC4) {
        const float4 v = *(const float4*)(as_ptr[i] + kb);
        as_grp[i][0] = v.x; as_grp[i][1] = v.y; as_grp[i][2] = v.z; as_grp[i][3] = v.w;
      } else {
        as_grp[i][0] = as_ptr[i][kb];
      }
    }
  };
  load_a_scales(0);
  float as_cur[2];
  float ws_cur[2] = {unit ? 1.0f : ws_ptr[0][0], unit ? 1.0f : ws_ptr[1][0]};
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
      ws_next[0] = unit ? 1.0f : ws_ptr[0][next_kb];
      ws_next[1] = unit ? 1.0f : ws_ptr[1][next_kb];
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
  load_epilogue_scales<2, NT_OUT, C::GLU, true>(esc, p, tile, wm * 64, n_out0, lane);
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
  // (the order covers the tiles that exist, not the host's upper bound: see gmm_tiled_kernel)
  const int num_tiles = p.header[0];
  const int total = num_tiles * p.tiles_n;
  TileInfo tile;
  int n0;
  {
    const int id = blockIdx.x;
    if (id >= total) return;
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(num_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    n0 = ((logical % width) / gsz) * C::OUT_BN;
    tile = p.tiles[m_idx];
  }
  if (tile.group < 0) {
    zero_fill_tile(p.out, p.ro, tile.row0, tile.nrows, n0, C::OUT_BN, N, tid, C::THREADS);
    return;
  }

  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
#pragma unroll
  for (int i = 0; i < C::A_IPW; i++) {
    const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
    const int q = (lane % C::CPR) ^ C::swz(r);
    a_src[i] = p.lhs + (size_t)lhs_row_of(p.ro, tile.row0 + min(r, tile.nrows - 1)) * K + q * 16;
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
    as_ptr[i] = P.a_scale + (size_t)lhs_row_of(p.ro, tile.row0 + min(lr, tile.nrows - 1)) * nkb;
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
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
static int prepare_fp8_tiled_cfg() {
  return reserve_lds(gmm_fp8_tiled_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

template <typename C>
static int prepare_fp8_big_cfg() {
  return reserve_lds(gmm_fp8_big_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

int prepare_fp8() {
  int st = MOE_OK;
#define MOE_PREP(GLU, VEC4)                                                          \
  if (!st) st = prepare_fp8_tiled_cfg<F8Cfg<128, 128, 2, GLU, VEC4>>();             \
  if (!st) st = prepare_fp8_big_cfg<F8BigCfg<GLU, VEC4>>();
  MOE_PREP(false, false) MOE_PREP(false, true) MOE_PREP(true, false) MOE_PREP(true, true)
#undef MOE_PREP
  return st;
}

template <int BM, int BKB, int NSTAGE, bool GLU, bool VEC4>
static int launch_fp8_tiled_cfg(Fp8TiledParams P, int M, int G_total, hipStream_t s) {
  using C = F8Cfg<BM, BKB, NSTAGE, GLU, VEC4>;
  if (int st = prepare_fp8_tiled_cfg<C>()) return st;
  P.base.max_m_tiles = max_tiles_for(M, G_total, BM);
  P.base.tiles_n = cdiv(P.base.N, C::OUT_BN);
  const long long tiles = (long long)P.base.max_m_tiles * P.base.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_fp8_tiled_kernel<C><<<(unsigned)tiles, C::THREADS, C::LDS_BYTES, s>>>(P);
  return check_launch("gmm_fp8_tiled_kernel");
}

template <bool GLU, bool VEC4>
static int launch_fp8_big_cfg(Fp8TiledParams P, int M, int G_total, hipStream_t s) {
  using C = F8BigCfg<GLU, VEC4>;
  if (int st = prepare_fp8_big_cfg<C>()) return st;
  P.base.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  P.base.tiles_n = cdiv(P.base.N, C::OUT_BN);
  const long long tiles = (long long)P.base.max_m_tiles * P.base.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_fp8_big_kernel<C><<<(unsigned)tiles, C::THREADS, C::LDS_BYTES, s>>>(P);
  return check_launch("gmm_fp8_big_kernel");
}

int launch_fp8_tiled(bool big, bool glu, bool vec4, const Fp8TiledParams& P, int M, int G, hipStream_t s) {
  if (big) {
    if (vec4) return glu ? launch_fp8_big_cfg<true, true>(P, M, G, s) : launch_fp8_big_cfg<false, true>(P, M, G, s);
    return glu ? launch_fp8_big_cfg<true, false>(P, M, G, s) : launch_fp8_big_cfg<false, false>(P, M, G, s);
  }
  if (vec4) return glu ? launch_fp8_tiled_cfg<128, 128, 2, true, true>(P, M, G, s) : launch_fp8_tiled_cfg<128, 128, 2, false, true>(P, M, G, s);
  return glu ? launch_fp8_tiled_cfg<128, 128, 2, true, false>(P, M, G, s) : launch_fp8_tiled_cfg<128, 128, 2, false, false>(P, M, G, s);
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

// (NT, U) of the fp8 streaming kernel, from sweeps over NT in {1, 2, 4, 8} and U in {1, 2, 4, 8} on the DeepSeek-V3 shapes
// (257 experts, 8 rows each): 16-row tiles take one K block per step, 2 channel tiles per wave with fused GLU (7168 -> 2048:
// 1.22 ms against 1.33 ms with 4 tiles, 1.28 ms with 1) and 4 tiles without (2048 -> 7168: 0.65 ms against 0.67 ms with
// 2 tiles and 4 blocks, 0.69 ms with 8 tiles); 64-row tiles take 2 tiles and one block.
int launch_fp8_skinny(bool few_rows, const SkinnyParams& p, bool glu, int max_tiles, hipStream_t s) {
  if (!few_rows) return launch_skinny<4, 2, 1>(p, glu, max_tiles, s);
  return glu ? launch_skinny<1, 2, 1>(p, glu, max_tiles, s) : launch_skinny<1, 4, 1>(p, glu, max_tiles, s);
}

}  // namespace moe
