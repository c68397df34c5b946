// Grouped matmul: the direct-to-LDS persistent kernel (int8 x int8, bf16 x bf16 prefill).

#include "moe_gmm_common.h"

namespace moe {

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
  const int total = num_tiles * p.tiles_n;  // the tiles that exist, not the host's upper bound (see peek_tile)

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
    const int gsz = min(num_tiles - first_m, GSM);
    const int m_idx = first_m + (logical % width) % gsz;
    // (uniform values: kept in scalar registers, so that a tile looked up ahead of time costs no vector registers)
    const TileInfo ti = p.tiles[m_idx];
    t.info.group = __builtin_amdgcn_readfirstlane(ti.group);
    t.info.row0 = __builtin_amdgcn_readfirstlane(ti.row0);
    t.info.nrows = __builtin_amdgcn_readfirstlane(ti.nrows);
    t.info.pad = 0;
    t.n0 = __builtin_amdgcn_readfirstlane(((logical % width) / gsz) * C::OUT_BN);
    return true;
  };
  // Advances `id` to this block's next tile that needs the matmul; tiles of rows that belong to no local
  // group are written as zeros on the way.
  auto next_compute_tile = [&](int& id, Tile& t) -> bool {
    for (; id < total; id += gridDim.x) {
      if (!locate(id, t)) continue;
      if (t.info.group >= 0) return true;
      zero_fill_tile(p.out, p.ro, t.info.row0, t.info.nrows, t.n0, C::OUT_BN, N, tid, C::THREADS);
    }
    return false;
  };

  // ---- per-lane source addresses of this wave's load instructions ---------------------------
  const uint8_t* a_src[C::A_IPW];
  const uint8_t* b_src[C::B_IPW];
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
          // the stage's requests go out behind every third MFMA from the start of the k-step: one per MFMA fills the
          // address unit's queue, and the MFMAs behind a request that waits for a free entry wait with it (dlhs of the
          // Mixtral shape 1.71 -> 1.60 and 1.91 -> 1.83 ms); over the whole k-step they land too late (1.66 / 1.85 ms)
          if (LD && (i * C::TN + j) % 3 == 0 && (i * C::TN + j) / 3 < C::LPS) issue_one(ld_kt, ld_buf, (i * C::TN + j) / 3);
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
    // The results are stored before anything of the next tile is looked up: the accumulators are then dead across the
    // tile-boundary code.  (Requesting the next tile's first stages ahead of the stores, with the tile looked up before the
    // main loop, was measured 3 % slower: any code between the last k-step and the stores makes the compiler push
    // accumulators out to scratch memory and reload them between the stores, one memory round trip each.)
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, cur.info, wm * C::WM, n_out0, lane);
    // all LDS reads of this tile are done in every wave and no request is still writing LDS: the buffers can take the next tile
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
static int prepare_dl_cfg() {
  return reserve_lds(gmm_dl_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

int prepare_dl() {
  int st = MOE_OK;
#define MOE_PREP(OP, GLU)                                                            \
  if (!st) st = prepare_dl_cfg<DlCfg<OP, 256, 256, 128, 2, 4, 2, GLU>>();           \
  if (!st) st = prepare_dl_cfg<DlCfg<OP, 256, 256, 64, 2, 4, 4, GLU>>();
  MOE_PREP(OP_I8, false) MOE_PREP(OP_I8, true) MOE_PREP(OP_BF16, false) MOE_PREP(OP_BF16, true)
#undef MOE_PREP
  if (!st) st = prepare_dl_cfg<DlCfg<OP_BF16, 256, 256, 128, 2, 4, 2, false, true>>();
  return st;
}

template <typename C>
static int launch_dl_cfg(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_dl_cfg<C>()) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  // one persistent block per CU (the LDS footprint allows no more); a multiple of 8 keeps "tile id mod 8"
  // equal to the XCD a block runs on
  int num_cus = 0;
  if (int st = device_cu_count(&num_cus)) return st;
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  gmm_dl_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_dl_kernel");
}

template <int OP>
static int launch_dl_op(bool glu, int stage_bytes, const TiledParams& p, int M, int G_total, hipStream_t s) {
  // 128-byte stages (two buffers, 16 x 16 MFMAs) when the rows allow it: 6-10 % faster than 64-byte stages (four buffers,
  // 32 x 32 MFMAs) on the Mixtral shape
  if (stage_bytes == 128)
    return glu ? launch_dl_cfg<DlCfg<OP, 256, 256, 128, 2, 4, 2, true>>(p, M, G_total, s) : launch_dl_cfg<DlCfg<OP, 256, 256, 128, 2, 4, 2, false>>(p, M, G_total, s);
  if (stage_bytes == 64)
    return glu ? launch_dl_cfg<DlCfg<OP, 256, 256, 64, 2, 4, 4, true>>(p, M, G_total, s) : launch_dl_cfg<DlCfg<OP, 256, 256, 64, 2, 4, 4, false>>(p, M, G_total, s);
  return fail(MOE_ERR_INVALID_ARG, "gmm: stage of %d bytes", stage_bytes);
}

int launch_dl(int op, bool glu, int stage_bytes, bool rhs_kn, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (rhs_kn) {
    if (op != OP_BF16 || glu || stage_bytes != 128) return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] weights need bf16 x bf16 without rhs_up");
    return launch_dl_cfg<DlCfg<OP_BF16, 256, 256, 128, 2, 4, 2, false, true>>(p, M, G_total, s);
  }
  if (op == OP_I8) return launch_dl_op<OP_I8>(glu, stage_bytes, p, M, G_total, s);
  if (op == OP_BF16) return launch_dl_op<OP_BF16>(glu, stage_bytes, p, M, G_total, s);
  return fail(MOE_ERR_UNSUPPORTED, "gmm: no direct-to-LDS kernel for operand %d", op);
}

}  // namespace moe
