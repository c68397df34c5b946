// Grouped matmul: the persistent 256 x 256 kernel for bf16 activations x int8 / int4 / mxfp4 weights (prefill).
//
// The pipeline of gmm_dl_kernel (moe_gmm_dl.hip) with a weight side of its own.  Activations go global -> LDS without
// passing through registers (global_load_lds_dwordx4, 8 rows x 128 B per wave instruction, XOR-swizzled unpadded rows, two
// buffers of 64 KB).  Weights cannot: their bytes have to become bf16 on the way.  Each thread therefore keeps the raw
// bytes of its share of one stage in registers (int8: 2 x 16 B, 4-bit formats: 16 B): they are requested one stage before
// they are needed, widened to bf16 (4-bit formats: multiplied by their group scale) and written into the swizzled LDS rows
// in the shadow of the MFMAs of the k-step in which the activation requests of the same stage go out, i.e. right after the
// barrier that proves the buffer free.  A weight is widened once per block (by one of 512 threads), not once per wave, and
// the fragment reads, the MFMA schedule and the epilogue are those of the bf16 x bf16 kernel.

#include "moe_gmm_common.h"

namespace moe {

template <int BSRC_, bool GLU_>
struct DlwCfg {
  static constexpr int BSRC = BSRC_;
  static constexpr bool GLU = GLU_;
  static constexpr int BM = 256, BN = 256, BKB = 128, BK = 64, MI = 16;
  static constexpr int WAVES_M = 2, WAVES_N = 4, NWAVES = 8, THREADS = NWAVES * kWave;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / MI, TN = WN / MI;
  static constexpr int CPR = BKB / 16, RPI = 1024 / BKB;
  static constexpr int A_IPW = BM / RPI / NWAVES;  // activation requests per wave per stage
  static constexpr int STAGE = (BM + BN) * BKB, LDS_BYTES = 2 * STAGE;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static constexpr bool NIBBLES = BSRC == BSRC_I4 || BSRC == BSRC_MX4;
  static constexpr int VPL = NIBBLES ? 32 : 16;          // weights per 16-byte load
  static constexpr int LPR = BK / VPL;                    // loads per weight row and stage
  static constexpr int B_LOADS = BN * LPR / THREADS;      // loads per thread and stage: 2 (int8) or 1
  static constexpr int SRC_STAGE_BYTES = NIBBLES ? BK / 2 : BK;  // bytes of a weight row per stage
  static constexpr int UNITS = 4;                         // 16-byte LDS chunks a thread writes per stage
  static_assert(BSRC != BSRC_SAME && B_LOADS * VPL * 2 / 16 == UNITS, "four chunks per thread");
  __device__ static __forceinline__ int swz(int row) { return (row >> 1) & 7; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_dlw_kernel(const TiledParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const size_t row_bytes = (size_t)K * 2;
  const size_t w_row_bytes = C::NIBBLES ? (size_t)K / 2 : (size_t)K;
  const int num_tiles = p.header[0];
  const int total = p.max_m_tiles * p.tiles_n;
  const int nk = K / C::BK;

  struct Tile {
    TileInfo info;
    int n0;
  };
  // tile id -> (m-tile, n-tile): ids congruent mod 8 run on one XCD and form an 8 x 4 patch that shares panels in its L2
  auto locate = [&](int id, Tile& t) -> bool {
    const int q = total / 8, rem = total % 8, xcd = id % 8, loc = id / 8;
    const int logical = xcd < rem ? xcd * (q + 1) + loc : rem * (q + 1) + (xcd - rem) * q + loc;
    const int GSM = p.tune > 0 ? p.tune : 8;
    const int width = GSM * p.tiles_n;
    const int sg = logical / width, first_m = sg * GSM;
    const int gsz = min(p.max_m_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    if (m_idx >= num_tiles) return false;
    // (uniform values: kept in scalar registers, so that a tile looked up ahead of time costs no vector registers)
    const TileInfo ti = p.tiles[m_idx];
    t.info.group = __builtin_amdgcn_readfirstlane(ti.group);
    t.info.row0 = __builtin_amdgcn_readfirstlane(ti.row0);
    t.info.nrows = __builtin_amdgcn_readfirstlane(ti.nrows);
    t.info.pad = 0;
    t.n0 = __builtin_amdgcn_readfirstlane(((logical % width) / gsz) * C::OUT_BN);
    return true;
  };
  auto next_compute_tile = [&](int& id, Tile& t) -> bool {
    for (; id < total; id += gridDim.x) {
      if (!locate(id, t)) continue;
      if (t.info.group >= 0) return true;
      zero_fill_tile(p.out, p.ro, t.info.row0, t.info.nrows, t.n0, C::OUT_BN, N, tid, C::THREADS);
    }
    return false;
  };

  // ---- activations: per-lane sources of this wave's requests --------------------------------------------------
  const uint8_t* a_src[C::A_IPW];
  // ---- weights: this thread's loads of a stage --------------------------------------------------------------
  // load l covers VPL consecutive k values of one weight row: row = idx / LPR, part = idx % LPR with idx = tid + l * THREADS
  const uint8_t* b_src[C::B_LOADS];
  const void* b_scale_row[C::B_LOADS];  // the row's scales (4-bit formats)
  int b_lds[C::B_LOADS];                // byte offset of the row inside a stage
  int b_sw[C::B_LOADS];                 // the row's swizzle
  int b_part[C::B_LOADS];
  auto set_sources = [&](const Tile& t) {
    int a_rows[C::A_IPW];
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) a_rows[i] = t.info.row0 + min((wave * C::A_IPW + i) * C::RPI + lane / C::CPR, t.info.nrows - 1);
    lhs_rows_of<C::A_IPW>(p.ro, a_rows);
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) {
      const int r = (wave * C::A_IPW + i) * C::RPI + lane / C::CPR;
      const int q = (lane % C::CPR) ^ C::swz(r);
      a_src[i] = p.lhs + (size_t)a_rows[i] * row_bytes + q * 16;
    }
#pragma unroll
    for (int l = 0; l < C::B_LOADS; l++) {
      const int idx = tid + l * C::THREADS;
      const int row = idx / C::LPR, part = idx % C::LPR;
      const bool up = C::GLU && row >= C::BN / 2;
      const int n = min(t.n0 + (up ? row - C::BN / 2 : row), N - 1);
      const size_t grow = (size_t)t.info.group * N + n;
      b_src[l] = (up ? p.rhs_up : p.rhs) + grow * w_row_bytes + part * 16;
      b_lds[l] = (C::BM + row) * C::BKB;
      b_sw[l] = C::swz(row);
      b_part[l] = part;
      if (C::BSRC == BSRC_I4) {
        const int nkg = (K + p.i4_group - 1) / p.i4_group;
        b_scale_row[l] = (const uint16_t*)(up ? p.rhs_up_scale : p.rhs_scale) + grow * nkg;
      } else if (C::BSRC == BSRC_MX4) {
        b_scale_row[l] = (const uint8_t*)(up ? p.rhs_up_scale : p.rhs_scale) + grow * (K / 32);
      } else {
        b_scale_row[l] = nullptr;
      }
    }
  };

  auto issue_a = [&](int kt, int buf, int i) {
    __builtin_amdgcn_global_load_lds((gbl_ptr_t)(a_src[i] + (size_t)kt * C::BKB), (lds_ptr_t)(smem + buf * C::STAGE + (wave * C::A_IPW + i) * 1024), 16,
                                     0, 0);
  };

  // raw weight bytes of one stage (and, for the 4-bit formats, the scale of each load's k range)
  struct WRegs {
    uint4 w[C::B_LOADS];
    float s[C::B_LOADS];
  };
  auto b_load = [&](WRegs& r, int kt) {
#pragma unroll
    for (int l = 0; l < C::B_LOADS; l++) {
      r.w[l] = *(const uint4*)(b_src[l] + (size_t)kt * C::SRC_STAGE_BYTES);
      const int k0 = kt * C::BK + b_part[l] * C::VPL;
      if (C::BSRC == BSRC_I4) r.s[l] = bf16_bits_to_f32(((const uint16_t*)b_scale_row[l])[p.i4_group == 32 ? k0 >> 5 : k0 >> 7]);
      else if (C::BSRC == BSRC_MX4) r.s[l] = __uint_as_float((uint32_t)((const uint8_t*)b_scale_row[l])[k0 / 32] << 23);
      else r.s[l] = 1.0f;
    }
  };
  // unit u of a stage: 8 weights -> one 16-byte chunk of the row in LDS
  auto b_store_unit = [&](const WRegs& r, int buf, int u) {
    constexpr int UPL = C::UNITS / C::B_LOADS;  // units per load: 2 (int8: 8 bytes each) or 4 (4-bit: one word each)
    const int l = u / UPL, h = u % UPL;
    const uint32_t w4[4] = {r.w[l].x, r.w[l].y, r.w[l].z, r.w[l].w};
    uint4 o;
    if (C::BSRC == BSRC_I8) {
      const int v0 = (int)w4[2 * h], v1 = (int)w4[2 * h + 1];
      o = make_uint4(i8x2_to_bf16x2((v0 << 24) >> 24, (v0 << 16) >> 24), i8x2_to_bf16x2((v0 << 8) >> 24, v0 >> 24),
                     i8x2_to_bf16x2((v1 << 24) >> 24, (v1 << 16) >> 24), i8x2_to_bf16x2((v1 << 8) >> 24, v1 >> 24));
    } else if (C::BSRC == BSRC_MX4) {
      const uint32_t w = w4[h];
      const float sc = r.s[l];
      o = make_uint4(__builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 0)),
                     __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 1)),
                     __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 2)),
                     __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(w, sc, 3)));
    } else {  // int4: (nibble - 8) * scale rounded to bf16, as the reference dequantises
      const uint32_t w = w4[h];
      const float sc = r.s[l];
      uint32_t x[4];
#pragma unroll
      for (int b = 0; b < 4; b++) {
        const int lo = (int)((w >> (8 * b)) & 0xf) - 8, hi = (int)((w >> (8 * b + 4)) & 0xf) - 8;
        x[b] = pack_bf16x2((float)lo * sc, (float)hi * sc);
      }
      o = make_uint4(x[0], x[1], x[2], x[3]);
    }
    const int q = b_part[l] * UPL + h;  // chunk of the 128-byte row
    *(uint4*)(smem + buf * C::STAGE + b_lds[l] + ((q ^ b_sw[l]) << 4)) = o;
  };

  typedef v4f acc_t;
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
  // fragment of k-step ks: row (lane % 16), chunk q = 4 * ks + lane / 16, stored at slot q ^ swz(row)
  const int t16m = ((lane / 16) ^ C::swz(lane % 16)) * 16;
  const int row_off_m = (lane % 16) * C::BKB;
  v4i ga[C::TM], gb[2][C::TN];
  auto read_a16 = [&](int buf, int ks, int i) {
    ga[i] = *(const v4i*)(smem + buf * C::STAGE + (wm * C::WM + i * 16) * C::BKB + row_off_m + (t16m ^ (ks * 64)));
  };
  auto read_b16 = [&](int buf, int ks, int set, int j) {
    gb[set][j] = *(const v4i*)(smem + buf * C::STAGE + (C::BM + b_row[j]) * C::BKB + row_off_m + (t16m ^ (ks * 64)));
  };

  WRegs wr;  // the stage after next (while the loop runs)
  // One k-step of 32 MFMAs.  RD: the fragments of the next k-step are read behind them.  LD: the k-step after the
  // barrier: the activation requests of stage ld_kt go out, the weights held in `wr` (the same stage) are widened and
  // written into the freed buffer, and the raw bytes of the stage after that are requested.
  auto kstep16 = [&](auto set_c, auto rd_c, auto ld_c, int rd_buf, int rd_ks, int ld_kt, int ld_buf) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value;
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, gb[SET][j]), __builtin_bit_cast(v8bf, ga[i]), acc[j][i], 0, 0, 0);
        const int slot = i * C::TN + j;
        if (LD && slot < C::A_IPW) issue_a(ld_kt, ld_buf, slot);
        // the four chunks of the weight stage, one every fourth MFMA from slot 6 on; then the next stage's raw bytes
        if (LD && slot >= 6 && slot < 6 + 4 * C::UNITS && (slot - 6) % 4 == 0) b_store_unit(wr, ld_buf, (slot - 6) / 4);
        if (LD && slot == 6 + 4 * C::UNITS) b_load(wr, min(ld_kt + 1, nk - 1));
        if (RD && j == 1 && i < C::TN) read_b16(rd_buf, rd_ks, SET ^ 1, i);
        if (RD && j == C::TN - 1) read_a16(rd_buf, rd_ks, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;

  // A tile's first two stages: activation requests, and the weights of both stages as raw bytes.
  WRegs w0, w1;
  auto issue_prologue = [&]() {
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) issue_a(min(s, nk - 1), s, i);
    b_load(w0, 0);
    b_load(w1, min(1, nk - 1));
  };
  // ... widened into the two buffers once they have arrived (and everything the previous tile read is done)
  auto finish_prologue = [&]() {
    wait_vmcnt<0>();
#pragma unroll
    for (int u = 0; u < C::UNITS; u++) b_store_unit(w0, 0, u);
#pragma unroll
    for (int u = 0; u < C::UNITS; u++) b_store_unit(w1, 1, u);
    b_load(wr, min(2, nk - 1));
  };

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
      for (int i = 0; i < C::TM; i++) acc[j][i] = v4f{0.f, 0.f, 0.f, 0.f};
    finish_prologue();
    // every activation request of the prologue has landed, every wave's weight chunks are written
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    asm volatile("s_barrier" ::: "memory");
#pragma unroll
    for (int i = 0; i < C::TM; i++) read_a16(0, 0, i);
#pragma unroll
    for (int j = 0; j < C::TN; j++) read_b16(0, 0, 0, j);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    const int n_out0 = cur.n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
    EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
    int kt = 0;
    kstep16(S0{}, T_{}, F_{}, 0, 1, 0, 0);
    for (; kt + 1 < nk; kt++) {
      const int buf = kt % 2;
      // own fragment reads of this stage done, own requests (activations of stage kt+1, raw weights of stage kt+2) landed,
      // own weight chunks of stage kt+1 written: then everybody's
      __builtin_amdgcn_s_waitcnt(0xC07F);
      wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      kstep16(S1{}, T_{}, T_{}, buf ^ 1, 0, min(kt + 2, nk - 1), buf);
      kstep16(S0{}, T_{}, F_{}, buf ^ 1, 1, 0, 0);
    }
    load_epilogue_scales<C::TM, NT_OUT, C::GLU, C::BSRC == BSRC_I8, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane);
    kstep16(S1{}, F_{}, F_{}, 0, 0, 0, 0);
    // all LDS reads of this tile are done in every wave and nothing is still writing LDS: the buffers can take the next tile
    // results first (the accumulators are then dead across the tile-boundary code), then the next tile
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, cur.info, wm * C::WM, n_out0, lane);
    __builtin_amdgcn_s_waitcnt(0xC07F);
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    id += gridDim.x;
    have = next_compute_tile(id, cur);
    if (have) {
      set_sources(cur);
      issue_prologue();
    }
  }
  wait_vmcnt<0>();
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
static int prepare_dlw_cfg() {
  return reserve_lds(gmm_dlw_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

int prepare_dlw() {
  int st = MOE_OK;
#define MOE_PREP(BSRC)                                       \
  if (!st) st = prepare_dlw_cfg<DlwCfg<BSRC, false>>();      \
  if (!st) st = prepare_dlw_cfg<DlwCfg<BSRC, true>>();
  MOE_PREP(BSRC_I8) MOE_PREP(BSRC_I4) MOE_PREP(BSRC_MX4)
#undef MOE_PREP
  return st;
}

template <typename C>
static int launch_dlw_cfg(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_dlw_cfg<C>()) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  int num_cus = 0;
  if (int st = device_cu_count(&num_cus)) return st;
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  gmm_dlw_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_dlw_kernel");
}

int launch_dlw(int bsrc, bool glu, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (p.K % 64 != 0 || p.wq_kmajor) return fail(MOE_ERR_UNSUPPORTED, "gmm: the weight-only direct-to-LDS kernel needs K %% 64 == 0 and scales in the default layout");
#define MOE_DLW_CASE(BSRC) \
  if (bsrc == BSRC) return glu ? launch_dlw_cfg<DlwCfg<BSRC, true>>(p, M, G_total, s) : launch_dlw_cfg<DlwCfg<BSRC, false>>(p, M, G_total, s);
  MOE_DLW_CASE(BSRC_I8)
  MOE_DLW_CASE(BSRC_I4)
  MOE_DLW_CASE(BSRC_MX4)
#undef MOE_DLW_CASE
  return fail(MOE_ERR_UNSUPPORTED, "gmm: no weight-only direct-to-LDS kernel for weight format %d", bsrc);
}

}  // namespace moe
