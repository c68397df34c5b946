// Grouped matmul: the persistent 256 x 256 kernel for operands that need no conversion (int8 x int8, bf16 x bf16 and
// fp8 x fp8 with per-row x per-channel scales, prefill) with the stages of a block's consecutive tiles as ONE request
// stream.
//
// Both operands go global -> LDS without passing through registers (buffer_load ... lds, 1 KB = 8 rows of 128 bytes per
// wave instruction; XOR-swizzled unpadded rows; two buffers of 64 KB; one barrier per stage).  8 waves as 2 x 4, each
// 128 x 64 of the tile in 16 x 16 MFMAs (16x16x64 i8 / 16x16x32 bf16); weight fragments double-buffered, an activation
// fragment reloaded for the next k-step right after the four MFMAs that use it.
//
// The requests run two stages ahead of the MFMAs ACROSS tile boundaries: a tile's first two stages arrive while the
// previous tile is still being multiplied, and the record of the next tile is read a whole tile ahead.  Addresses go
// through buffer descriptors that end where the tile's rows (the expert's weight matrix) end: rows past the end read as
// zeros, the lane-dependent part of an address is the same for every tile and the tile-dependent part is scalar, so
// moving the stream on to the next tile costs no vector work (with a row index: one index load per request).  What is
// left between two tiles is the epilogue.
//
// fp8 (e4m3 weights, e4m3 or e5m2 activations; scales per row / per tensor x per channel / per tensor, applied in the
// epilogue: what gmm() quantises to, kernels/megablox/ops.py:232-267, and the e5m2 gradient times e4m3 weights of its
// backward, ops.py:583-604) runs the same stream on v_mfma_f32_16x16x128_f8f6f4: a 128-byte stage is ONE instruction per
// 16 x 16 tile.  An operand fragment of that instruction is 8 registers, so only 4 of a wave's 8 activation fragments
// and its 4 weight fragments are live beside the 128 accumulators, and a stage is multiplied in two halves of 16 MFMAs:
// row tiles 0 .. 3 fragment by fragment (each slot reloaded with row tile + 4 after its four MFMAs), then row tiles
// 4 .. 7 weight fragment by weight fragment (each reloaded with the next stage's after its four MFMAs, the activation
// slots during the last four).  The stage barrier sits between the halves.

#include "moe_gmm_common.h"

namespace moe {

template <int OP_, bool GLU_, int LF_ = 0, bool KN_ = false>
struct DlsCfg {
  static constexpr int OP = OP_;
  static constexpr bool GLU = GLU_;
  static constexpr int LF = LF_;  // fp8 activations: 0 = e4m3, 1 = e5m2 (format selector of the MFMA's second operand)
  // fp8 weights given as [G, K, N] (the contraction index as the row: dlhs of a layer whose weights are [G, N, K], read as
  // they are).  The weight half of a stage then holds 128 contraction rows x 256 output channels (128 x 256 B, four rows per
  // wave instruction) and the weight fragments come out of it through ds_read_b64_tr_b8.
  static constexpr bool KN = KN_;
  static constexpr int BM = 256, BN = 256, BKB = 128, MI = 16;
  static constexpr int ESZ = OP == OP_BF16 ? 2 : 1, BK = BKB / ESZ;
  static constexpr int WAVES_M = 2, WAVES_N = 4, NWAVES = 8, THREADS = NWAVES * kWave;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / MI, TN = WN / MI;
  static constexpr int A_STAGE = BM * BKB, STAGE = (BM + BN) * BKB, LDS_BYTES = 2 * STAGE;
  static constexpr int A_IPW = BM / 8 / NWAVES, B_IPW = BN / 8 / NWAVES;  // requests per wave and stage: 4 + 4
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  // a stage's eight requests go out behind every REQ_STRIDE-th MFMA from the start of the k-step: one per MFMA fills the
  // address unit's queue and the MFMAs behind a request that waits for a free entry wait with it (Mixtral first projection
  // 1.707 -> 1.653 ms with 3; 2 and 4 in between; the fp8 loop, whose requests share 16 MFMAs, is fastest with 1)
  static constexpr int REQ_STRIDE = 3, REQ_STRIDE_F8 = 1;
  static_assert(OP == OP_I8 || OP == OP_BF16 || OP == OP_F8, "operands");
  static_assert(LF == 0 || OP == OP_F8, "only fp8 activations come in two formats");
  static_assert(!KN || (OP == OP_F8 && !GLU), "[G, K, N] weights: fp8 without rhs_up");
  // slot of the 16-byte chunk c of contraction row r in a [G, K, N] weight stage: c ^ kn_swz(r); the 8 rows of a transposing
  // read and those of the next lane group (16 rows further) then fall into 16 different 16-byte bank groups
  __device__ static __forceinline__ int kn_swz(int row) { return (row & 7) ^ (((row >> 4) & 1) << 3); }
  __device__ static __forceinline__ int swz(int row) { return (row >> 1) & 7; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_dls_kernel(const TiledParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  constexpr int OP = C::OP;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const uint32_t row_bytes = (uint32_t)K * C::ESZ;
  const int num_tiles = p.header[0];
  const int nk = K / C::BK;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  using Tile = StreamTile;
  using Peek = TilePeek;
  auto peek_from = [&](int id0) { return peek_tile<C::OUT_BN>(p, num_tiles, id0); };
  auto resolve = [&](Peek pk, Tile& t) { return resolve_tile<C::OUT_BN, C::THREADS>(p, num_tiles, pk, t, tid); };

  // ---- the loading side of the stream ---------------------------------------------------------------------------
  // request i of this wave covers rows (wave * 4 + i) * 8 .. + 7 of the tile's 256 activation (weight) rows, 128 bytes
  // of each; the lane's 16 bytes: global chunk = LDS slot ^ swizzle of the row
  auto lane_off = [&](int i, uint32_t row) {
    const int r = (wave * C::A_IPW + i) * 8 + lane / 8;
    return row * row_bytes + (uint32_t)(((lane % 8) ^ C::swz(r)) << 4);
  };
  v4i a_desc, b_desc;
  uint32_t a_voff[C::A_IPW], b_voff[C::B_IPW], b_soff = 0;
  auto set_a_sources = [&](const Tile& t) {
    if (p.ro.row_idx) {
      a_desc = buffer_desc(p.lhs, clamp_u32((size_t)p.ro.lhs_rows * row_bytes));
      int rows[C::A_IPW];
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) rows[i] = min(t.info.row0 + (wave * C::A_IPW + i) * 8 + lane / 8, p.M - 1);
      lhs_rows_of<C::A_IPW>(p.ro, rows);
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) a_voff[i] = lane_off(i, (uint32_t)rows[i]);
    } else {
      a_desc = buffer_desc(p.lhs + (size_t)t.info.row0 * row_bytes, clamp_u32((size_t)t.info.nrows * row_bytes));
    }
  };
  if (!p.ro.row_idx) {
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) a_voff[i] = lane_off(i, (uint32_t)((wave * C::A_IPW + i) * 8 + lane / 8));
  }
  // weights: with GLU the upper 128 of the tile's 256 rows are the second projection's, whose requests come from waves 4 .. 7
  const bool load_up = C::GLU && wave >= C::NWAVES / 2;
#pragma unroll
  for (int i = 0; i < C::B_IPW; i++) {
    if constexpr (C::KN) {
      // request i covers contraction rows (wave * 4 + i) * 4 + lane / 16 of the stage, the lane LDS slot lane % 16 of its row
      const int r = (wave * C::B_IPW + i) * 4 + lane / 16;
      b_voff[i] = (uint32_t)r * (uint32_t)N + (uint32_t)(((lane % 16) ^ C::kn_swz(r)) << 4);
    } else {
      const int r = (wave * C::B_IPW + i) * 8 + lane / 8;
      b_voff[i] = lane_off(i, (uint32_t)(C::GLU ? r % (C::BN / 2) : r));
    }
  }
  auto set_b_sources = [&](const Tile& t) {
    if constexpr (C::KN) {
      b_desc = buffer_desc(p.rhs + (size_t)t.info.group * N * row_bytes, clamp_u32((size_t)N * row_bytes));
      b_soff = (uint32_t)t.n0;  // the tile's first output channel: a byte offset inside every contraction row
    } else {
      b_desc = buffer_desc((load_up ? p.rhs_up : p.rhs) + (size_t)t.info.group * N * row_bytes, clamp_u32((size_t)N * row_bytes));
      b_soff = (uint32_t)t.n0 * row_bytes;
    }
  };
  // request idx of the stage: 0 .. 3 activations, 4 .. 7 weights
  auto issue_one = [&](int kt, int buf, int idx) {
    if (idx < C::A_IPW) dma16_buffer(a_desc, a_voff[idx], (uint32_t)kt * C::BKB, lds_base + buf * C::STAGE + (wave * C::A_IPW + idx) * 1024);
    else dma16_buffer(b_desc, b_voff[idx - C::A_IPW], b_soff + (uint32_t)kt * C::BKB * (C::KN ? (uint32_t)N : 1u), lds_base + buf * C::STAGE + C::A_STAGE + (wave * C::B_IPW + idx - C::A_IPW) * 1024);
  };


  using T_ = std::true_type;
  using F_ = std::false_type;
  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;
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
  // fragment of a 64-byte k-step ks: row (lane % 16), chunk q = 4 * ks + lane / 16, stored at slot q ^ swz(row)
  const int frag_lane = (lane % 16) * C::BKB + (((lane / 16) ^ C::swz(lane % 16)) << 4);

  if constexpr (OP == OP_F8) {
    // ---- the multiplying side, fp8 ---------------------------------------------------------------------------------
    constexpr int RING = C::TM / 2;
    static_assert(C::TM == 8 && C::TN == 4, "the two halves of a stage");
    v4f acc[C::TN][C::TM];
    // fragment: row (lane % 16), K bytes 16 q .. and 64 + 16 q .. with q = lane / 16 (both operands alike, so the order
    // of K inside the instruction does not matter)
    v8i ga[RING], gb[C::TN];
    auto read_frag = [&](v8i& f, const uint8_t* src) {
      const v4i lo = *(const v4i*)(src + frag_lane), hi = *(const v4i*)(src + (frag_lane ^ 64));
      f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
      f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
    };
    auto read_a = [&](int buf, int i, int slot) { read_frag(ga[slot], smem + buf * C::STAGE + (wm * C::WM + i * 16) * C::BKB); };
    // [G, K, N] weights: lane (s, q) addresses row 16 q + s / 2 (+ 8, 64, 72) of the stage's 128 contraction rows, i.e. the K
    // bytes 16 q .. and 64 + 16 q .. its activation fragment holds, and the 8 bytes s % 2 of the fragment's 16-byte channel block
    const int kn_base = C::A_STAGE + (16 * (lane / 16) + (lane % 16) / 2) * C::BN + ((((wn * C::TN) ^ ((lane % 16) / 2) ^ (((lane / 16) & 1) << 3))) << 4) + (lane % 2) * 8;
    auto read_b = [&](int buf, int j) {
      if constexpr (C::KN) {
        typedef int v2i_kn __attribute__((ext_vector_type(2)));
        typedef __attribute__((address_space(3))) v2i_kn* lds_v2i_kn;
        int base = kn_base;
        asm volatile("" : "+v"(base));
        const uint8_t* src = smem + buf * C::STAGE + (base ^ (j << 4));
#pragma unroll
        for (int t = 0; t < 4; t++) {
          const v2i_kn x = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_kn)(src + ((t & 1) * 8 + (t >> 1) * 64) * C::BN));
          gb[j][2 * t] = x[0];
          gb[j][2 * t + 1] = x[1];
        }
      } else {
        read_frag(gb[j], smem + buf * C::STAGE + C::A_STAGE + b_row[j] * C::BKB);
      }
    };
    const v4f zero = {0.f, 0.f, 0.f, 0.f};
    // First half of a stage (in buffer buf): row tiles 0 .. 3 from the ring, each slot reloaded with row tile + 4.
    // ZC: the tile's first stage starts from zero.
    auto half_lo = [&](auto zc_c, int buf) {
      constexpr bool ZC = decltype(zc_c)::value;
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int i = t / 4, j = t % 4;
        acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(gb[j], ga[i], ZC ? zero : acc[j][i], 0, C::LF, 0, 127, 0, 127);
        if (j == 3) read_a(buf, i + RING, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    // Second half: row tiles 4 .. 7 (in the ring), weight fragment by weight fragment.  RD: the next stage (buffer
    // rd_buf) is prepared behind it, its weight fragments and its row tiles 0 .. 3.  The eight requests of stage ld_kt go
    // out into ld_buf, one per MFMA from the start.
    auto half_hi = [&](auto rd_c, auto zc_c, int rd_buf, int ld_kt, int ld_buf) {
      constexpr bool RD = decltype(rd_c)::value, ZC = decltype(zc_c)::value;
#pragma unroll
      for (int t = 0; t < 16; t++) {
        const int j = t / 4, ii = t % 4;
        acc[j][RING + ii] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(gb[j], ga[ii], ZC ? zero : acc[j][RING + ii], 0, C::LF, 0, 127, 0, 127);
        if (t % C::REQ_STRIDE_F8 == 0 && t / C::REQ_STRIDE_F8 < C::A_IPW + C::B_IPW) issue_one(ld_kt, ld_buf, t / C::REQ_STRIDE_F8);
        if (RD && ii == 3) read_b(rd_buf, j);
        if (RD && j == 3) read_a(rd_buf, ii, ii);
        __builtin_amdgcn_sched_barrier(0);
      }
    };
    auto first_fragments = [&](int buf) {
#pragma unroll
      for (int i = 0; i < RING; i++) read_a(buf, i, i);
#pragma unroll
      for (int j = 0; j < C::TN; j++) read_b(buf, j);
    };

    Tile cur, nxt;
    if (!resolve(peek_from(blockIdx.x), cur)) return;
    set_a_sources(cur);
    set_b_sources(cur);
#pragma unroll
    for (int s = 0; s < 2; s++)
#pragma unroll
      for (int i = 0; i < C::A_IPW + C::B_IPW; i++) issue_one(s, s, i);
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    first_fragments(0);

    int base = 0;  // the buffer that holds stage 0 of the current tile
    while (true) {
      Peek pk = peek_from(cur.id + gridDim.x);
      bool have_n = false;
      const int n_out0 = cur.n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
      EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
      half_lo(T_{}, base);
      // Iteration `it`: the second half of stage it, then the first half of stage it + 1 (the schedule of the int8 / bf16
      // loop below with halves of a stage in place of its k-steps).
      auto stream_kt = [&](int s) { return s < nk ? s : (have_n ? s - nk : nk - 1); };
      int cb = base;
      auto iteration = [&](int it, auto last_c, auto zc_c) {
        constexpr bool LAST = decltype(last_c)::value;
        __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
        wait_vmcnt<0>();
        asm volatile("s_barrier" ::: "memory");
        if (LAST) {
          half_hi(F_{}, zc_c, 0, stream_kt(it + 2), cb);
        } else {
          half_hi(T_{}, zc_c, cb ^ 1, stream_kt(it + 2), cb);
          half_lo(F_{}, cb ^ 1);
        }
        cb ^= 1;
      };
      iteration(0, F_{}, T_{});
      for (int it = 1; it < nk - 2; it++) iteration(it, F_{}, F_{});
      have_n = resolve(pk, nxt);
      if (have_n) {
        set_a_sources(nxt);
        set_b_sources(nxt);
      }
      iteration(nk - 2, F_{}, F_{});
      iteration(nk - 1, T_{}, F_{});
      // (the sums are pinned to this point: their only readers sit behind the branches of the epilogue, and the compiler
      // otherwise moves the last MFMAs of every chain down there, away from the requests and reads they overlap, parking
      // the fragments in scratch memory on the way)
#pragma unroll
      for (int j = 0; j < C::TN; j++)
#pragma unroll
        for (int i = 0; i < C::TM; i++) asm volatile("" : "+v"(acc[j][i]));
      // (without the gated activation the epilogue's lane constants are made per tile: hoisted out of the tile loop they
      // are spilled over the main loop, 58 registers against 22, and the second projection of the Mixtral shape takes
      // 0.935 instead of 0.910 ms; with it the hoisted form is the faster one by 1 %)
      int lane_e = lane;
      if constexpr (!C::GLU) asm volatile("" : "+v"(lane_e));
      load_epilogue_scales<C::TM, NT_OUT, C::GLU, true, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane_e);
      store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, cur.info, wm * C::WM, n_out0, lane_e);
      if (!have_n) break;
      cur = nxt;
      base = cb;
      first_fragments(base);
    }
    __builtin_amdgcn_s_waitcnt(0xC07F);
    wait_vmcnt<0>();
  } else {
  // ---- the multiplying side, int8 / bf16 ------------------------------------------------------------------------
  typedef typename std::conditional<OP == OP_I8, v4i, v4f>::type acc_t;
  acc_t acc[C::TN][C::TM];
  v4i ga[C::TM], gb[2][C::TN];
  auto read_a = [&](int buf, int ks, int i) {
    ga[i] = *(const v4i*)(smem + buf * C::STAGE + (wm * C::WM + i * 16) * C::BKB + (frag_lane ^ (ks * 64)));
  };
  auto read_b = [&](int buf, int ks, int set, int j) {
    gb[set][j] = *(const v4i*)(smem + buf * C::STAGE + C::A_STAGE + b_row[j] * C::BKB + (frag_lane ^ (ks * 64)));
  };
  // One k-step of 32 MFMAs on the fragments in registers.  ZC: a tile's first k-step starts from zero.  RD: the fragments
  // of the next k-step (rd_buf, rd_ks) are read behind the MFMAs (the weights' into the other set, an activation fragment
  // in place once its four MFMAs are out).  LD: the eight requests of stage ld_kt of the loading tile go out into ld_buf,
  // one per MFMA from the start of the k-step.
  auto kstep = [&](auto set_c, auto rd_c, auto ld_c, auto zc_c, int rd_buf, int rd_ks, int ld_kt, int ld_buf) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value, ZC = decltype(zc_c)::value;
#pragma unroll
    for (int i = 0; i < C::TM; i++) {
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
        if constexpr (OP == OP_I8) {
          acc[j][i] = __builtin_amdgcn_mfma_i32_16x16x64_i8(gb[SET][j], ga[i], ZC ? v4i{0, 0, 0, 0} : acc[j][i], 0, 0, 0);
        } else {
          acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, gb[SET][j]), __builtin_bit_cast(v8bf, ga[i]),
                                                              ZC ? v4f{0.f, 0.f, 0.f, 0.f} : acc[j][i], 0, 0, 0);
        }
        const int slot = i * C::TN + j;
        if (LD && slot % C::REQ_STRIDE == 0 && slot / C::REQ_STRIDE < C::A_IPW + C::B_IPW) issue_one(ld_kt, ld_buf, slot / C::REQ_STRIDE);
        if (RD && j == 1 && i < C::TN) read_b(rd_buf, rd_ks, SET ^ 1, i);
        if (RD && j == C::TN - 1) read_a(rd_buf, rd_ks, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // The fragments of a tile's first k-step (stage 0 in buffer `buf`), with nothing to hide behind.
  auto first_fragments = [&](int buf) {
#pragma unroll
    for (int i = 0; i < C::TM; i++) read_a(buf, 0, i);
#pragma unroll
    for (int j = 0; j < C::TN; j++) read_b(buf, 0, 0, j);
  };

  Tile cur, nxt;
  if (!resolve(peek_from(blockIdx.x), cur)) return;
  // ---- head of the stream: the first tile's stages 0 and 1 ----
  set_a_sources(cur);
  set_b_sources(cur);
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int i = 0; i < C::A_IPW + C::B_IPW; i++) issue_one(s, s, i);
  wait_vmcnt<0>();
  asm volatile("s_barrier" ::: "memory");
  first_fragments(0);

  int base = 0;  // the buffer that holds stage 0 of the current tile
  while (true) {
    // the record of the block's next tile is requested now and looked at two stages before this tile ends
    Peek pk = peek_from(cur.id + gridDim.x);
    bool have_n = false;
    const int n_out0 = cur.n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
    EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
    // first half of stage 0; the fragments of its second half are read behind it
    kstep(S0{}, T_{}, F_{}, T_{}, base, 1, 0, 0);
    // Iteration `it`: the second half of stage it, then the first half of stage it + 1.  Every fragment of stage it is in
    // registers before the barrier, and stage it + 1 has landed at it: the buffer of stage it takes stage it + 2 of the
    // stream (from nk on: the next tile's).
    auto stream_kt = [&](int s) { return s < nk ? s : (have_n ? s - nk : nk - 1); };
    int cb = base;  // buffer of stage `it`
    auto iteration = [&](int it, auto last_c) {
      constexpr bool LAST = decltype(last_c)::value;  // the tile's last half stage: nothing is read behind it
      // own fragment reads done, own requests landed: then everybody's
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      if (LAST) {
        kstep(S1{}, F_{}, T_{}, F_{}, 0, 0, stream_kt(it + 2), cb);
      } else {
        kstep(S1{}, T_{}, T_{}, F_{}, cb ^ 1, 0, stream_kt(it + 2), cb);
        kstep(S0{}, T_{}, F_{}, F_{}, cb ^ 1, 1, 0, 0);
      }
      cb ^= 1;
    };
    for (int it = 0; it < nk - 2; it++) iteration(it, F_{});
    // the stream crosses into the next tile
    have_n = resolve(pk, nxt);
    if (have_n) {
      set_a_sources(nxt);
      set_b_sources(nxt);
    }
    iteration(nk - 2, F_{});
    iteration(nk - 1, T_{});
    // (requested only now: ahead of the last k-step the scales would push request offsets out to scratch memory, and
    // every reload between two requests waits for all requests in flight)
    load_epilogue_scales<C::TM, NT_OUT, C::GLU, true, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane);
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, cur.info, wm * C::WM, n_out0, lane);
    if (!have_n) break;
    cur = nxt;
    base = cb;  // the buffer of stage nk = the next tile's stage 0, landed before the last barrier
    first_fragments(base);
  }
  // nothing may still be writing LDS when the block ends
  __builtin_amdgcn_s_waitcnt(0xC07F);
  wait_vmcnt<0>();
  }
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
static int prepare_dls_cfg() {
  return reserve_lds(gmm_dls_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

int prepare_dls() {
  int st = MOE_OK;
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_I8, false>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_I8, true>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_BF16, false>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_BF16, true>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_F8, false>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_F8, true>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_F8, false, 1>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_F8, false, 0, true>>();
  if (!st) st = prepare_dls_cfg<DlsCfg<OP_F8, false, 1, true>>();
  return st;
}

template <typename C>
static int launch_dls_cfg(const TiledParams& p0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_dls_cfg<C>()) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  if (p.tune <= 0) p.tune = default_super_row(M, G_total, C::BM);
  // one persistent block per CU (the LDS footprint allows no more); a multiple of 8 keeps "tile id mod 8"
  // equal to the XCD a block runs on
  int num_cus = 0;
  if (int st = device_cu_count(&num_cus)) return st;
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  gmm_dls_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_dls_kernel");
}

bool dls_takes(int op, int K, int N, long long indexed_lhs_rows) {
  // whole 128-byte stages, at least three of them (the stream looks two stages ahead, into the next tile at most).  Byte
  // offsets are 32-bit: a weight request adds the lane's row (up to 255 rows past the last n-tile's first row, i.e. up to
  // N + 255 in all) times the row pitch to the descriptor's base, an activation request the lane's row of the 256-row
  // tile (or, with a row index, any of the indexed rows); each sum must stay below 2^32 so that a row past the end lands
  // beyond the descriptor's range and reads as zeros instead of wrapping around into it
  const long long esz = op == OP_BF16 ? 2 : 1, pitch = K * esz;
  return (op == OP_I8 || op == OP_BF16 || op == OP_F8) && pitch % 128 == 0 && pitch >= 384 && ((long long)N + 256) * pitch < (1LL << 32) &&
         (indexed_lhs_rows + 256) * pitch < (1LL << 32);
}

int launch_dls(int op, bool glu, const TiledParams& p, int M, int G_total, hipStream_t s, int lhs_e5m2, int rhs_kn) {
  if (!dls_takes(op, p.K, p.N, p.ro.row_idx ? p.ro.lhs_rows : 0))
    return fail(MOE_ERR_UNSUPPORTED, "gmm: the stream kernel needs int8, bf16 or fp8 operands, whole 128-byte stages (three or more) and 32-bit byte offsets");
  if (lhs_e5m2 && (op != OP_F8 || glu)) return fail(MOE_ERR_UNSUPPORTED, "gmm: e5m2 activations run against e4m3 weights without rhs_up");
  if (rhs_kn && (op != OP_F8 || glu || p.N % 256 != 0)) return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] weights on the stream kernel need fp8 operands, no rhs_up and N %% 256 == 0");
  if (op == OP_F8) {
    if (rhs_kn) return lhs_e5m2 ? launch_dls_cfg<DlsCfg<OP_F8, false, 1, true>>(p, M, G_total, s) : launch_dls_cfg<DlsCfg<OP_F8, false, 0, true>>(p, M, G_total, s);
    if (lhs_e5m2) return launch_dls_cfg<DlsCfg<OP_F8, false, 1>>(p, M, G_total, s);
    return glu ? launch_dls_cfg<DlsCfg<OP_F8, true>>(p, M, G_total, s) : launch_dls_cfg<DlsCfg<OP_F8, false>>(p, M, G_total, s);
  }
  if (op == OP_I8) return glu ? launch_dls_cfg<DlsCfg<OP_I8, true>>(p, M, G_total, s) : launch_dls_cfg<DlsCfg<OP_I8, false>>(p, M, G_total, s);
  return glu ? launch_dls_cfg<DlsCfg<OP_BF16, true>>(p, M, G_total, s) : launch_dls_cfg<DlsCfg<OP_BF16, false>>(p, M, G_total, s);
}

}  // namespace moe
