// Grouped matmul: the persistent 256 x 256 kernel for bf16 activations x int8 / int4 / mxfp4 weights (prefill).
//
// Both operands go global -> LDS without passing through registers (buffer_load ... lds, 1 KB per wave instruction):
// the activations as XOR-swizzled rows of 128 bytes (64 bf16 values of K), the weights as the RAW bytes of the
// checkpoint format (64 or 32 bytes per row and stage).  A weight becomes bf16 only in the registers of the wave that
// multiplies it: each of the 8 waves owns 32 of the tile's 256 weight rows for all 256 activation rows (16 x 2 MFMA
// tiles of 16 x 16 x 32), so every weight is widened exactly once per block, by the wave that needs it, in the shadow
// of that wave's own MFMAs, and no weight byte is ever written to LDS by a thread.  The fragments of the next k-step are
// read (and widened) behind the MFMAs of the current one: activations through a ring of four fragment registers,
// weights as two raw fragments.
//
// The stages of a block's consecutive tiles form ONE stream: the requests run two stages ahead of the MFMAs across tile
// boundaries, so a tile's first stages arrive while the previous tile is still being multiplied, and the record of the
// next tile is read a whole tile ahead.  Everything is addressed through buffer descriptors that end where the tile's
// rows (the expert's weight matrix) end: rows past the end read as zeros, the lane-dependent part of an address is the
// same for every tile and the tile-dependent part is scalar, so moving the stream on to the next tile costs no vector
// work (with a row index: one index load per request).  What is left between two tiles is the epilogue.

#include "moe_gmm_common.h"

namespace moe {

template <int BSRC_, bool GLU_>
struct DlwCfg {
  static constexpr int BSRC = BSRC_;
  static constexpr bool GLU = GLU_;
  static constexpr int BM = 256, BN = 256, BKB = 128, BK = 64, MI = 16;
  static constexpr int NWAVES = 8, THREADS = NWAVES * kWave;
  static constexpr int WN = BN / NWAVES, TM = BM / MI, TN = WN / MI;  // a wave: 256 rows x 32 weight rows
  // activation fragments in registers.  4, not 8: the longer ring is no faster (fragments are read four MFMA slots ahead
  // either way) and its 16 registers push lane-constant addresses of the int4 kernel out to scratch memory INSIDE the
  // main loop, where every reload waits for all requests in flight (GPT-OSS second projection: 0.74 ms against 0.48 ms)
  static constexpr int RING = 4;
  static constexpr bool NIBBLES = BSRC == BSRC_I4 || BSRC == BSRC_MX4;
  static constexpr int W_ROW = NIBBLES ? BK / 2 : BK;  // raw bytes of a weight row per stage: 32 or 64
  static constexpr int A_STAGE = BM * BKB, B_STAGE = BN * W_ROW, STAGE = A_STAGE + B_STAGE;
  static constexpr int NSTAGE = 3, LDS_BYTES = NSTAGE * STAGE;
  static constexpr int A_IPW = A_STAGE / 1024 / NWAVES;  // activation requests per wave and stage: 4
  static constexpr int B_IPW = B_STAGE / 1024 / NWAVES;  // weight requests per wave and stage: 2 (int8) or 1
  static constexpr int B_RPI = 1024 / W_ROW;             // weight rows per request: 16 or 32
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(BSRC != BSRC_SAME && TN == 2 && TM == 16 && LDS_BYTES <= 160 * 1024, "shape");
  // activations: chunk q of row r sits in slot q ^ swz_a(r) of the row's eight 16-byte slots
  __device__ static __forceinline__ int swz_a(int row) { return (row >> 1) & 7; }
  // weights: slot q ^ swz_b(r) of the row's four (int8) or two (4-bit) slots, so that the 16 rows a fragment read covers
  // spread over all banks
  __device__ static __forceinline__ int swz_b(int row) { return NIBBLES ? (row >> 3) & 1 : (row >> 2) & 3; }
};

// HALF: the tile list holds tiles of at most 128 rows (32 to 104 rows per expert on average): 8 row tiles per wave are
// multiplied instead of 16, with the work behind the MFMAs packed into half as many slots; the upper half of a stage's
// activation rows lies past the end of the tile's buffer descriptor and is neither fetched nor read.
template <typename C, bool HALF>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_dlw_kernel(const TiledParams p0) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  // (bf16 activations carry no scale: saying so here lets the epilogue fold the per-row factor away)
  TiledParams p = p0;
  p.lhs_scale = nullptr;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int N = p.N, K = p.K;
  const uint32_t row_bytes = (uint32_t)K * 2;
  const uint32_t w_row_bytes = C::NIBBLES ? (uint32_t)K / 2 : (uint32_t)K;
  const int num_tiles = p.header[0];
  const int nk = K / C::BK;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)smem;

  using Tile = StreamTile;
  using Peek = TilePeek;
  auto peek_from = [&](int id0) { return peek_tile<C::OUT_BN>(p, num_tiles, id0); };
  auto resolve = [&](Peek pk, Tile& t) { return resolve_tile<C::OUT_BN, C::THREADS>(p, num_tiles, pk, t, tid); };

  // ---- the loading side of the stream ---------------------------------------------------------------------------
  // activations: request i of this wave covers rows (wave * A_IPW + i) * 8 .. + 7 of the tile, 128 bytes of each
  v4i a_desc;
  uint32_t a_voff[C::A_IPW];
  auto a_lane_off = [&](int i, int row) {  // the lane's 16 bytes inside the row's 128: global chunk = LDS slot ^ swizzle
    const int r = (wave * C::A_IPW + i) * 8 + lane / 8;
    return (uint32_t)row * row_bytes + (uint32_t)(((lane % 8) ^ C::swz_a(r)) << 4);
  };
  auto set_a_sources = [&](const Tile& t) {
    if (p.ro.row_idx) {
      a_desc = buffer_desc(p.lhs, clamp_u32((size_t)p.ro.lhs_rows * row_bytes));
      int rows[C::A_IPW];
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) rows[i] = min(t.info.row0 + (wave * C::A_IPW + i) * 8 + lane / 8, p.M - 1);
      lhs_rows_of<C::A_IPW>(p.ro, rows);
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) a_voff[i] = a_lane_off(i, rows[i]);
    } else {
      a_desc = buffer_desc(p.lhs + (size_t)t.info.row0 * row_bytes, clamp_u32((size_t)t.info.nrows * row_bytes));
    }
  };
  if (!p.ro.row_idx) {
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) a_voff[i] = a_lane_off(i, (wave * C::A_IPW + i) * 8 + lane / 8);
  }
  // weights: request i of this wave covers the tile's weight rows (wave * B_IPW + i) * B_RPI .. + B_RPI - 1; with GLU the
  // upper 128 of the 256 rows are the second projection's, whose requests come from waves 4 .. 7
  const bool load_up = C::GLU && wave >= C::NWAVES / 2;
  v4i b_desc;
  uint32_t b_soff = 0;
  uint32_t b_voff[C::B_IPW];
#pragma unroll
  for (int i = 0; i < C::B_IPW; i++) {
    const int r = (wave * C::B_IPW + i) * C::B_RPI + lane / (C::W_ROW / 16);  // row of the tile
    const int pr = C::GLU ? r % (C::BN / 2) : r;                                // row of the projection's 128 / 256
    b_voff[i] = (uint32_t)pr * w_row_bytes + (uint32_t)(((lane % (C::W_ROW / 16)) ^ C::swz_b(r)) << 4);
  }
  auto set_b_sources = [&](const Tile& t) {
    b_desc = buffer_desc((load_up ? p.rhs_up : p.rhs) + (size_t)t.info.group * N * w_row_bytes, clamp_u32((size_t)N * w_row_bytes));
    b_soff = (uint32_t)t.n0 * w_row_bytes;
  };
  // (HALF: rows 128 .. 255 of a stage, the requests of waves 4 .. 7, are never read)
  const bool a_wanted = !HALF || wave < C::NWAVES / 2;
  auto issue_a = [&](int kt, int buf, int i) {
    if (a_wanted) dma16_buffer(a_desc, a_voff[i], (uint32_t)kt * C::BKB, lds_base + buf * C::STAGE + (wave * C::A_IPW + i) * 1024);
  };
  auto issue_b = [&](int kt, int buf, int i) {
    dma16_buffer(b_desc, b_voff[i], b_soff + (uint32_t)kt * C::W_ROW, lds_base + buf * C::STAGE + C::A_STAGE + (wave * C::B_IPW + i) * 1024);
  };

  // ---- the multiplying side ----------------------------------------------------------------------------------------
  // weight fragment j of this wave: rows frag_row(j) .. + 15 of the tile; the lane widens row + lane % 16
  auto frag_row = [&](int j) { return C::GLU ? j * (C::BN / 2) + wave * 16 : wave * C::WN + j * 16; };
  // scales of the 4-bit formats: per weight row and 32 (mxfp4, int4 group 32) or 128 values of K; the lane needs the ones
  // of its own row for the stage's two k-steps: one 2- or 4-byte load per fragment and stage
  __amdgpu_buffer_rsrc_t s_desc[C::TN];
  uint32_t s_soff = 0, s_voff = 0;
  const bool i4g32 = C::BSRC == BSRC_I4 && p.i4_group == 32;
  const uint32_t nkg = C::BSRC == BSRC_I4 ? (uint32_t)((K + p.i4_group - 1) / p.i4_group) : (uint32_t)(K / 32);
  const uint32_t s_row_bytes = C::BSRC == BSRC_I4 ? nkg * 2 : nkg;
  if (C::NIBBLES) s_voff = (uint32_t)((C::GLU ? wave * 16 : wave * C::WN) + lane % 16) * s_row_bytes;
  auto set_s_sources = [&](const Tile& t) {
    if (!C::NIBBLES) return;
#pragma unroll
    for (int j = 0; j < C::TN; j++)
      s_desc[j] = __builtin_amdgcn_make_buffer_rsrc((void*)((const uint8_t*)(C::GLU && j == 1 ? p.rhs_up_scale : p.rhs_scale) + (size_t)t.info.group * N * s_row_bytes),
                                                    0, (int)clamp_u32((size_t)N * s_row_bytes), 0x00020000);
    s_soff = (uint32_t)t.n0 * s_row_bytes;
  };
  // The raw scale bits of a stage are requested with its weights (ordinary loads: the compiler waits for them where they
  // are used) and turned into the factors of its two k-steps right after the barrier that also waits for the stage.
  uint32_t sc_raw[C::TN] = {0, 0};
  float sc_cur[C::TN][2] = {{1.0f, 1.0f}, {1.0f, 1.0f}};  // [fragment][k-step] of the stage being widened
  auto load_scales = [&](int kt) {
    if (!C::NIBBLES) return;
#pragma unroll
    for (int j = 0; j < C::TN; j++) {
      const uint32_t row_off = s_voff + (C::GLU ? 0u : (uint32_t)j * 16 * s_row_bytes);
      if (C::BSRC == BSRC_MX4) sc_raw[j] = __builtin_amdgcn_raw_buffer_load_b16(s_desc[j], row_off + (uint32_t)kt * 2, s_soff, 0);  // bytes 2 kt, 2 kt + 1
      else if (i4g32) sc_raw[j] = __builtin_amdgcn_raw_buffer_load_b32(s_desc[j], row_off + (uint32_t)kt * 4, s_soff, 0);            // bf16 2 kt, 2 kt + 1
      else sc_raw[j] = __builtin_amdgcn_raw_buffer_load_b16(s_desc[j], row_off + (uint32_t)(kt >> 1) * 2, s_soff, 0);                // bf16 kt / 2
    }
  };
  auto scales_to_current = [&]() {
    if (!C::NIBBLES) return;
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int ks = 0; ks < 2; ks++) {
        if (C::BSRC == BSRC_MX4) sc_cur[j][ks] = __uint_as_float(((sc_raw[j] >> (8 * ks)) & 0xffu) << 23);
        else if (i4g32) sc_cur[j][ks] = __uint_as_float(ks ? sc_raw[j] & 0xffff0000u : sc_raw[j] << 16);
        else sc_cur[j][ks] = __uint_as_float(sc_raw[j] << 16);
      }
  };

  typedef v4f acc_t;
  acc_t acc[C::TN][C::TM];
  // activation fragment of row tile i, k-step ks: row 16 i + lane % 16, chunk q = 4 ks + lane / 16, at slot q ^ swz_a(row)
  const int a_lane = (lane % 16) * C::BKB + (((lane / 16) ^ C::swz_a(lane % 16)) << 4);
  v4i ga[C::RING];
  auto read_a = [&](int buf, int ks, int i) {
    ga[i % C::RING] = *(const v4i*)(smem + buf * C::STAGE + i * 16 * C::BKB + (a_lane ^ (ks * 64)));
  };
  // raw weight fragment j, k-step ks: row frag_row(j) + lane % 16, the 8 values of K from 32 ks + 8 (lane / 16) on
  const int b_lane = C::NIBBLES ? (lane % 16) * C::W_ROW + (lane / 16) * 4 : (lane % 16) * C::W_ROW + ((lane / 16) & 1) * 8;
  const int b_sw = C::swz_b(lane % 16);
  typedef typename std::conditional<C::NIBBLES, uint32_t, uint2>::type raw_t;
  raw_t braw[C::TN];
  auto read_braw = [&](int buf, int ks, int j) {
    const int slot = C::NIBBLES ? ks : 2 * ks + (lane / 32);  // 16-byte slot of the row that holds the lane's bytes
    braw[j] = *(const raw_t*)(smem + buf * C::STAGE + C::A_STAGE + frag_row(j) * C::W_ROW + b_lane + ((slot ^ b_sw) << 4));
  };
  // widened weight fragments: the set of the current k-step and the one being built for the next
  v4i gb[2][C::TN];
  // int4: the fragment's low and high nibbles as bytes (values 0, 2, 4, 6 and 1, 3, 5, 7), taken apart once per fragment
  uint32_t nib_lo[C::TN], nib_hi[C::TN];
  // piece pc (0 .. 3) of fragment j: two of its eight values -> one register of gb[set][j]
  auto widen_piece = [&](int set, int j, int pc, float sc) {
    uint32_t o;
    if constexpr (C::BSRC == BSRC_I8) {
      const int w = (int)(pc < 2 ? braw[j].x : braw[j].y);
      const int sh = (pc & 1) * 16;
      o = pack_bf16x2((float)((w << (24 - sh)) >> 24), (float)((w << (16 - sh)) >> 24));
    } else if constexpr (C::BSRC == BSRC_MX4) {
      // (the byte selector is an immediate)
      o = pc == 0   ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(braw[j], sc, 0))
          : pc == 1 ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(braw[j], sc, 1))
          : pc == 2 ? __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(braw[j], sc, 2))
                    : __builtin_bit_cast(uint32_t, __builtin_amdgcn_cvt_scalef32_pk_bf16_fp4(braw[j], sc, 3));
    } else {  // int4: (nibble - 8) * scale rounded to bf16, as the reference dequantises
      // byte -> float is one instruction per value, and nibble * scale - 8 * scale is exact in f32 (12 significant bits),
      // so the fused multiply-add gives (nibble - 8) * scale bit for bit
      if (pc == 0) {
        nib_lo[j] = braw[j] & 0x0f0f0f0fu;
        nib_hi[j] = (braw[j] >> 4) & 0x0f0f0f0fu;
      }
      const float c8 = -8.0f * sc;
      o = pack_bf16x2(fmaf((float)((nib_lo[j] >> (8 * pc)) & 0xffu), sc, c8), fmaf((float)((nib_hi[j] >> (8 * pc)) & 0xffu), sc, c8));
    }
    gb[set][j][pc] = (int)o;
  };

  // One k-step of 32 MFMAs on the fragments of (cur_buf, cur_ks): row tiles 0 .. 7 sit in the ring, 8 .. 15 are read
  // behind the first half.  ZC: a tile's first k-step starts from zero.  RD: the next k-step (rd_buf, rd_ks) is prepared
  // behind the MFMAs: its raw weight fragments are read at the start and widened piece by piece into the other set (with
  // the scales in sc_cur), its row tiles 0 .. 7 are read behind the second half.  LD: the requests of stage ld_kt of the
  // loading tile go out into buffer ld_buf.
  auto kstep = [&](auto set_c, auto rd_c, auto ld_c, auto zc_c, int cur_buf, int cur_ks, int rd_buf, int rd_ks, int ld_kt, int ld_buf) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value, ZC = decltype(zc_c)::value;
    constexpr int TMX = HALF ? C::TM / 2 : C::TM;           // row tiles that are multiplied
    constexpr int W0 = HALF ? 4 : 8, WSTEP = HALF ? 1 : 2;  // slots of the eight widening pieces: W0, W0 + WSTEP, ...
    static_assert(2 * (C::A_IPW + C::B_IPW) <= TMX * C::TN && W0 + WSTEP * 4 * C::TN <= TMX * C::TN, "slots");
    float sc[C::TN] = {1.0f, 1.0f};
    if (RD && C::NIBBLES) {
#pragma unroll
      for (int j = 0; j < C::TN; j++) sc[j] = rd_ks ? sc_cur[j][1] : sc_cur[j][0];
    }
#pragma unroll
    for (int i = 0; i < TMX; i++) {
#pragma unroll
      for (int j = 0; j < C::TN; j++) {
        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(__builtin_bit_cast(v8bf, gb[SET][j]), __builtin_bit_cast(v8bf, ga[i % C::RING]),
                                                            ZC ? v4f{0.f, 0.f, 0.f, 0.f} : acc[j][i], 0, 0, 0);
        const int slot = i * C::TN + j;
        if (RD && slot < C::TN) read_braw(rd_buf, rd_ks, slot);
        // the eight pieces of the two fragments
        if (RD && slot >= W0 && slot < W0 + WSTEP * 4 * C::TN && (slot - W0) % WSTEP == 0) {
          const int q = (slot - W0) / WSTEP;
          widen_piece(SET ^ 1, q / 4, q % 4, sc[q / 4]);
        }
        if (LD && slot % 2 == 1 && slot / 2 < C::A_IPW) issue_a(ld_kt, ld_buf, slot / 2);
        if (LD && slot % 2 == 1 && slot / 2 >= C::A_IPW && slot / 2 < C::A_IPW + C::B_IPW) issue_b(ld_kt, ld_buf, slot / 2 - C::A_IPW);
        if (j == C::TN - 1 && i < TMX - C::RING) read_a(cur_buf, cur_ks, i + C::RING);
        if (RD && j == C::TN - 1 && i >= TMX - C::RING) read_a(rd_buf, rd_ks, i - (TMX - C::RING));
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;
  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;

  // The fragments of a tile's first k-step (stage 0 in buffer `buf`), read and widened with nothing to hide behind.
  auto first_fragments = [&](int buf) {
#pragma unroll
    for (int i = 0; i < C::RING; i++) read_a(buf, 0, i);
#pragma unroll
    for (int j = 0; j < C::TN; j++) read_braw(buf, 0, j);
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int pc = 0; pc < 4; pc++) widen_piece(0, j, pc, sc_cur[j][0]);
  };

  Tile cur, nxt;
  if (!resolve(peek_from(blockIdx.x), cur)) return;
  // ---- head of the stream: the first tile's stages 0 and 1 (scales: both into registers) ----
  set_a_sources(cur);
  set_b_sources(cur);
  set_s_sources(cur);
  load_scales(0);
#pragma unroll
  for (int s = 0; s < 2; s++) {
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) issue_a(s, s, i);
#pragma unroll
    for (int i = 0; i < C::B_IPW; i++) issue_b(s, s, i);
  }
  wait_vmcnt<0>();
  scales_to_current();
  load_scales(1);
  asm volatile("s_barrier" ::: "memory");
  first_fragments(0);

  int base = 0;  // the buffer that holds stage 0 of the current tile
  while (true) {
    // the record of the block's next tile is requested now and looked at two stages before this tile ends
    Peek pk = peek_from(cur.id + gridDim.x);
    bool have_n = false;
    const int n_out0 = cur.n0 + (C::GLU ? wave * 16 : wave * C::WN);
    EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
    // first half of stage 0; its second half is prepared behind it
    kstep(S0{}, T_{}, F_{}, T_{}, base, 0, base, 1, 0, 0);
    // Iteration `it`: the second half of stage it, then the first half of stage it + 1.  At its barrier stage it + 1 has
    // landed and nobody reads stage it - 1 any more: that buffer takes stage it + 2 of the stream (from nk on: the next
    // tile's).  The 4-bit formats' scales of stage it + 2 are requested with it; those of stage it + 1 become current.
    auto stream_kt = [&](int s) { return s < nk ? s : (have_n ? s - nk : nk - 1); };
    int cb = base;  // buffer of stage `it`
    auto iteration = [&](int it, auto last_c) {
      constexpr bool LAST = decltype(last_c)::value;  // the tile's last half stage: nothing is prepared behind it
      const int nb = cb == C::NSTAGE - 1 ? 0 : cb + 1, lb = nb == C::NSTAGE - 1 ? 0 : nb + 1;
      // own fragment reads done, own requests landed: then everybody's
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      scales_to_current();
      load_scales(stream_kt(it + 2));
      if (LAST) {
        kstep(S1{}, F_{}, T_{}, F_{}, cb, 1, 0, 0, stream_kt(it + 2), lb);
      } else {
        kstep(S1{}, T_{}, T_{}, F_{}, cb, 1, nb, 0, stream_kt(it + 2), lb);
        kstep(S0{}, T_{}, F_{}, F_{}, nb, 0, nb, 1, 0, 0);
      }
      cb = nb;
    };
    for (int it = 0; it < nk - 2; it++) iteration(it, F_{});
    // the stream crosses into the next tile
    have_n = resolve(pk, nxt);
    if (have_n) {
      set_a_sources(nxt);
      set_b_sources(nxt);
      set_s_sources(nxt);
    }
    iteration(nk - 2, F_{});
    // (the epilogue's lane constants are made per tile: hoisted out of the tile loop they are spilled over the main loop
    // and reloaded between the requests of a tile's last iterations, where every reload waits for the requests in flight;
    // Qwen3 second projection 0.437 -> 0.411 ms)
    int lane_e = lane;
    asm volatile("" : "+v"(lane_e));
    load_epilogue_scales<C::TM, NT_OUT, C::GLU, C::BSRC == BSRC_I8, C::MI>(esc, p, cur.info, 0, n_out0, lane_e);
    iteration(nk - 1, T_{});
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU, HALF ? C::TM / 2 : C::TM>(acc, esc, p, cur.info, 0, n_out0, lane_e);
    if (!have_n) break;
    cur = nxt;
    base = cb;  // (after the last iteration: the buffer of stage nk = the next tile's stage 0, landed before the last barrier)
    first_fragments(base);
  }
  // nothing may still be writing LDS when the block ends
  __builtin_amdgcn_s_waitcnt(0xC07F);
  wait_vmcnt<0>();
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
struct HalfTiles {};  // (a key for the second kernel's per-device set-up flags)

template <typename C>
static int prepare_dlw_cfg() {
  if (int st = reserve_lds(gmm_dlw_kernel<C, false>, C::LDS_BYTES, lds_flags<C>())) return st;
  return reserve_lds(gmm_dlw_kernel<C, true>, C::LDS_BYTES, lds_flags<HalfTiles<C>>());
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

// half: the tile list was built with 128-row tiles
template <typename C>
static int launch_dlw_cfg(bool half, const TiledParams& p0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_dlw_cfg<C>()) return st;
  TiledParams p = p0;
  p.max_m_tiles = max_tiles_for(M, G_total, half ? C::BM / 2 : C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  if (p.tune <= 0) p.tune = default_super_row(M, G_total, half ? C::BM / 2 : C::BM);
  int num_cus = 0;
  if (int st = device_cu_count(&num_cus)) return st;
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  if (half) gmm_dlw_kernel<C, true><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  else gmm_dlw_kernel<C, false><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(p);
  return check_launch("gmm_dlw_kernel");
}

bool dlw_takes(int K, int N, long long indexed_lhs_rows, bool wq_kmajor) {
  // whole 64-value stages, at least three of them (the stream looks two stages ahead, into the next tile at most); 32-bit
  // byte offsets: a request adds its lane's row (up to 255 rows past the last n-tile's first row; any indexed activation
  // row) times the row pitch to the descriptor's base, and the sum must not wrap around into the descriptor's range
  return K % 64 == 0 && K >= 192 && !wq_kmajor && ((long long)N + 256) * K < (1LL << 32) && (indexed_lhs_rows + 256) * K * 2 < (1LL << 32);
}

int launch_dlw(int bsrc, bool glu, bool half, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (!dlw_takes(p.K, p.N, p.ro.row_idx ? p.ro.lhs_rows : 0, p.wq_kmajor != 0))
    return fail(MOE_ERR_UNSUPPORTED, "gmm: the weight-only direct-to-LDS kernel needs K %% 64 == 0, K >= 192, scales in the default layout and 32-bit byte offsets");
#define MOE_DLW_CASE(BSRC) \
  if (bsrc == BSRC) return glu ? launch_dlw_cfg<DlwCfg<BSRC, true>>(half, p, M, G_total, s) : launch_dlw_cfg<DlwCfg<BSRC, false>>(half, p, M, G_total, s);
  MOE_DLW_CASE(BSRC_I8)
  MOE_DLW_CASE(BSRC_I4)
  MOE_DLW_CASE(BSRC_MX4)
#undef MOE_DLW_CASE
  return fail(MOE_ERR_UNSUPPORTED, "gmm: no weight-only direct-to-LDS kernel for weight format %d", bsrc);
}

}  // namespace moe
