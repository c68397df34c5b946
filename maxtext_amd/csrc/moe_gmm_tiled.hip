// Grouped matmul: the register-staged LDS-tiled MFMA kernel (weight-only formats, small problems, K tails).

#include "moe_gmm_common.h"

namespace moe {

template <int OP_, int BSRC_, int BM_, int BN_, int BKB_, int WAVES_M_, int WAVES_N_, bool GLU_, bool BS_ = false>
struct TiledCfg {
  static constexpr int OP = OP_, BSRC = BSRC_, BM = BM_, BN = BN_, BKB = BKB_;
  static constexpr int WAVES_M = WAVES_M_, WAVES_N = WAVES_N_;
  static constexpr bool GLU = GLU_;
  // BS: K-block scales (gmm_v2's [M, nb] / [G, nb, 1, N] layouts): the integer / f32 partial sums of a K block are
  // multiplied by the block's row and channel scales and added to a second, f32 set of accumulators
  static constexpr bool BS = BS_;
  static constexpr int THREADS = WAVES_M * WAVES_N * kWave;
  static constexpr int ESZ = OP == OP_BF16 ? 2 : 1;
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
  static_assert(!BS || (BSRC == BSRC_SAME && OP != OP_BF16 && BKB == 128 && BM <= 128), "block scales: 1-byte operands, 128-wide stages");
};

template <typename C>
__global__ __launch_bounds__(C::THREADS) void gmm_tiled_kernel(const TiledParams p) {
  extern __shared__ __attribute__((aligned(16))) uint8_t smem[];
  constexpr int OP = C::OP;
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;

  // ---- block -> (m-tile, n-tile): contiguous ids per XCD, then GSM x tiles_n super-rows ----
  // (over the tiles that exist, whose count the tile map left on the device: split over the grid, the host's upper
  // bound, the ids of tiles that do not exist would all fall to the last XCDs and leave them idle)
  const int num_tiles = p.header[0];
  int m_idx, n_idx;
  {
    const int nb = num_tiles * p.tiles_n, pid = blockIdx.x;
    if (pid >= nb) return;
    const int q = nb / 8, rem = nb % 8, xcd = pid % 8, loc = pid / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    constexpr int GSM = 4;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(num_tiles - first_m, GSM);
    m_idx = first_m + (logical % width) % gsz;
    n_idx = (logical % width) / gsz;
  }
  const TileInfo tile = p.tiles[m_idx];
  const int n0 = n_idx * C::OUT_BN;
  const int N = p.N, K = p.K;

  if (tile.group < 0) {  // rows of no local group: zeros
    zero_fill_tile(p.out, p.ro, tile.row0, tile.nrows, n0, C::OUT_BN, N, tid, C::THREADS);
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
    int gr = lhs_row_of(p.ro, tile.row0 + min(r, tile.nrows - 1));
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
      if (p.wq_kmajor) {  // scale of the chunk's K block (rhs_qb is a multiple of 16), multiplied in here
        if (part == 0) {
          const int kk = kt * C::BK + b_k[i];
          const float* sc = (const float*)(b_up[i] ? p.rhs_up_scale : p.rhs_scale);
          b_scale[i] = kk < K ? sc[(size_t)tile.group * p.rhs_scale_gstride + (size_t)(kk / p.rhs_qb) * N + b_n[i]] : 0.f;
        }
        const float sc_ = b_scale[i];
        *(uint2*)(s + b_lds[i] + 8 * part) = make_uint2(pack_bf16x2((float)((v << 24) >> 24) * sc_, (float)((v << 16) >> 24) * sc_),
                                                        pack_bf16x2((float)((v << 8) >> 24) * sc_, (float)(v >> 24) * sc_));
      } else {
        *(uint2*)(s + b_lds[i] + 8 * part) = make_uint2(i8x2_to_bf16x2((v << 24) >> 24, (v << 16) >> 24), i8x2_to_bf16x2((v << 8) >> 24, v >> 24));
      }
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
        if (p.wq_kmajor) {  // f32 [G, nb, N]
          const float* scf = (const float*)(b_up[i] ? p.rhs_up_scale : p.rhs_scale);
          b_scale[i] = kk < K ? scf[(size_t)tile.group * p.rhs_scale_gstride + (size_t)(kk / p.rhs_qb) * N + b_n[i]] : 0.f;
        } else {
          const uint16_t* sc = (const uint16_t*)(b_up[i] ? p.rhs_up_scale : p.rhs_scale);
          b_scale[i] = kk < K ? bf16_bits_to_f32(sc[((size_t)tile.group * N + b_n[i]) * nkg + kk / p.i4_group]) : 0.f;
        }
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
  // block-scaled operands: the f32 sums over finished K blocks
  v16f fin[C::BS ? C::TN : 1][C::BS ? C::TM : 1];
  if constexpr (C::BS) {
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int i = 0; i < C::TM; i++)
#pragma unroll
        for (int r = 0; r < 16; r++) fin[j][i][r] = 0.f;
  }
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
          } else if constexpr (OP == OP_F8) {
            // two instructions of 8 bytes per lane: both operands split their 16 bytes the same way, so the order of
            // the k values inside the 32-byte slice does not matter
            typedef long v2l __attribute__((ext_vector_type(2)));
            const v2l b2 = __builtin_bit_cast(v2l, bf[j]), a2 = __builtin_bit_cast(v2l, af[i]);
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b2[0], a2[0], acc[j][i], 0, 0, 0);
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b2[1], a2[1], acc[j][i], 0, 0, 0);
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
          } else if constexpr (OP == OP_F8) {
            // two instructions of 8 bytes per lane: both operands split their 16 bytes the same way, so the order of
            // the k values inside the 32-byte slice does not matter
            typedef long v2l __attribute__((ext_vector_type(2)));
            const v2l b2 = __builtin_bit_cast(v2l, bf[j]), a2 = __builtin_bit_cast(v2l, af[i]);
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b2[0], a2[0], acc[j][i], 0, 0, 0);
            acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_fp8_fp8(b2[1], a2[1], acc[j][i], 0, 0, 0);
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
  // Block scales: when stage kt ends a K block of either operand (a stage is 128 values of K, block sizes are
  // multiples of 128), the partial sums of the segment since the last flush are scaled and added to `fin`.
  int seg_start = 0;  // first k of the running segment
  auto flush_block = [&](int kt_done) {
    if constexpr (C::BS) {
      const int k_end = (kt_done + 1) * C::BK;
      const bool cut = kt_done == nk - 1 || (p.lhs_bs && k_end % p.lhs_qb == 0) || (p.rhs_bs && k_end % p.rhs_qb == 0);
      if (!cut) return;
      float la[C::TM];
#pragma unroll
      for (int i = 0; i < C::TM; i++) {
        const int lr = wm * C::WM + i * 32 + (lane % 32);
        la[i] = p.lhs_bs ? p.lhs_bs[(size_t)lhs_row_of(p.ro, tile.row0 + (lr < tile.nrows ? lr : 0)) * p.lhs_nb + seg_start / p.lhs_qb] : 1.0f;
      }
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
        const bool up = C::GLU && j >= NT_OUT;
        const float* rs = up ? p.rhs_up_bs : p.rhs_bs;
#pragma unroll
        for (int q = 0; q < 4; q++) {
          const int n = n_out0 + epilogue_channel<32>(up ? j - NT_OUT : j, q, lane);
          float4 r4 = make_float4(1.f, 1.f, 1.f, 1.f);
          if (rs && n < N) r4 = *(const float4*)(rs + (size_t)tile.group * p.rhs_bs_gstride + (size_t)(seg_start / p.rhs_qb) * N + n);
          const float rr[4] = {r4.x, r4.y, r4.z, r4.w};
#pragma unroll
          for (int i = 0; i < C::TM; i++)
#pragma unroll
            for (int r = 0; r < 4; r++) {
              fin[j][i][4 * q + r] = fmaf((float)acc[j][i][4 * q + r], la[i] * rr[r], fin[j][i][4 * q + r]);
              acc[j][i][4 * q + r] = 0;
            }
        }
      }
      seg_start = k_end;
    }
  };
  // Steady state: stage kt is computed, stage kt+1 moves from registers to LDS, stage kt+2 (a full one) is requested.
  int kt = 0;
  for (; kt + 2 < full; kt++) {
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L1{});
    flush_block(kt);
    stage_barrier();
  }
  if (kt + 2 < nk) {  // the stage after next is the one with the K tail
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L2{});
    flush_block(kt);
    stage_barrier();
    kt++;
  }
  if (kt + 1 < nk) {
    compute_and_store(kt & 1, kt + 1, std::true_type{}, L0{});
    flush_block(kt);
    stage_barrier();
    kt++;
  }
  compute_stage(kt & 1);
  flush_block(kt);

  if constexpr (C::BS)
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(fin, esc, p, tile, wm * C::WM, n_out0, lane);
  else
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, tile, wm * C::WM, n_out0, lane);
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
static int prepare_tiled_cfg() {
  return reserve_lds(gmm_tiled_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

template <typename C>
static int launch_tiled_cfg(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_tiled_cfg<C>()) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long blocks = (long long)p.max_m_tiles * p.tiles_n;
  if (blocks > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  gmm_tiled_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_tiled_kernel");
}

template <int OP, bool GLU>
static int launch_tiled_bs(int bm, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (p.K % 128 != 0) return fail(MOE_ERR_UNSUPPORTED, "gmm: K-block scales need K %% 128 == 0 (K=%d)", p.K);
  if (bm == 128) return launch_tiled_cfg<TiledCfg<OP, BSRC_SAME, 128, 256, 128, 2, 4, GLU, true>>(p, M, G_total, s);
  if (bm == 64) return launch_tiled_cfg<TiledCfg<OP, BSRC_SAME, 64, 256, 128, 2, 4, GLU, true>>(p, M, G_total, s);
  return fail(MOE_ERR_INVALID_ARG, "gmm: no block-scaled kernel with %d-row tiles", bm);
}

template <int OP, int BSRC, bool GLU>
static int launch_tiled_rows(int bm, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (bm == 128) return launch_tiled_cfg<TiledCfg<OP, BSRC, 128, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
  if (bm == 256) return launch_tiled_cfg<TiledCfg<OP, BSRC, 256, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
  // (eight waves of 32 x 64: 3-5 % faster than four of 64 x 64 on the Mixtral int8 shape at 4 to 24 rows per expert)
  if (bm == 64) return launch_tiled_cfg<TiledCfg<OP, BSRC, 64, 256, 128, 2, 4, GLU>>(p, M, G_total, s);
  return fail(MOE_ERR_INVALID_ARG, "gmm: no tiled kernel with %d-row tiles", bm);
}

template <int OP, int BSRC>
static int prepare_tiled_family() {
  int st = MOE_OK;
#define MOE_PREP(BM, GLU) if (!st) st = prepare_tiled_cfg<TiledCfg<OP, BSRC, BM, 256, 128, 2, 4, GLU>>();
  MOE_PREP(64, false) MOE_PREP(64, true) MOE_PREP(128, false) MOE_PREP(128, true) MOE_PREP(256, false) MOE_PREP(256, true)
#undef MOE_PREP
  return st;
}

template <int OP>
static int prepare_tiled_bs() {
  int st = MOE_OK;
#define MOE_PREP(BM, GLU) if (!st) st = prepare_tiled_cfg<TiledCfg<OP, BSRC_SAME, BM, 256, 128, 2, 4, GLU, true>>();
  MOE_PREP(64, false) MOE_PREP(64, true) MOE_PREP(128, false) MOE_PREP(128, true)
#undef MOE_PREP
  return st;
}

int prepare_tiled() {
  int st = prepare_tiled_family<OP_BF16, BSRC_SAME>();
  if (!st) st = prepare_tiled_family<OP_BF16, BSRC_I8>();
  if (!st) st = prepare_tiled_family<OP_BF16, BSRC_I4>();
  if (!st) st = prepare_tiled_family<OP_BF16, BSRC_MX4>();
  if (!st) st = prepare_tiled_family<OP_I8, BSRC_SAME>();
  if (!st) st = prepare_tiled_bs<OP_I8>();
  if (!st) st = prepare_tiled_bs<OP_F8>();
  return st;
}

int launch_tiled_bm(int op, int bsrc, bool glu, int bm, bool block_scaled, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (block_scaled) {
    if (bsrc != BSRC_SAME) return fail(MOE_ERR_UNSUPPORTED, "gmm: K-block scales on the partial sums need quantised activations");
    if (op == OP_I8) return glu ? launch_tiled_bs<OP_I8, true>(bm, p, M, G_total, s) : launch_tiled_bs<OP_I8, false>(bm, p, M, G_total, s);
    if (op == OP_F8) return glu ? launch_tiled_bs<OP_F8, true>(bm, p, M, G_total, s) : launch_tiled_bs<OP_F8, false>(bm, p, M, G_total, s);
    return fail(MOE_ERR_UNSUPPORTED, "gmm: no block-scaled kernel for operand %d", op);
  }
#define MOE_TILED_CASE(OP, BSRC)                                                         \
  if (op == OP && bsrc == BSRC)                                                          \
    return glu ? launch_tiled_rows<OP, BSRC, true>(bm, p, M, G_total, s) : launch_tiled_rows<OP, BSRC, false>(bm, p, M, G_total, s);
  MOE_TILED_CASE(OP_BF16, BSRC_SAME)
  MOE_TILED_CASE(OP_BF16, BSRC_I8)
  MOE_TILED_CASE(OP_BF16, BSRC_I4)
  MOE_TILED_CASE(OP_BF16, BSRC_MX4)
  MOE_TILED_CASE(OP_I8, BSRC_SAME)
#undef MOE_TILED_CASE
  return fail(MOE_ERR_UNSUPPORTED, "gmm: no tiled kernel for operand %d / weight format %d", op, bsrc);
}

}  // namespace moe
