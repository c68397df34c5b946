// Grouped matmul: block-scaled fp8 (1 x 128 activation scales, 128 x 128 weight scales; the DeepSeek-V3 recipe) for many
// rows per expert, on the persistent 256 x 256 stream of the int8 / bf16 prefill kernel.
//
// A stage is one 128-wide scale block: 128 bytes of K for 256 activation rows and 256 weight rows, global -> LDS without
// passing through registers (buffer_load ... lds, 8 rows x 128 bytes per wave instruction, XOR-swizzled unpadded rows, two
// buffers of 64 KB), requested two stages ahead of the MFMAs across tile boundaries.  8 waves as 2 x 4, each 128 rows x
// 64 channels in 8 x 4 tiles of v_mfma_f32_16x16x128_f8f6f4: ONE instruction per tile and stage gives the block's
// partial sum, which is multiplied by a_scale[row, kb] * w_scale[n / 128, kb] and added to the f32 result, exactly as the
// reference's block-scaled product is defined.  With weights as the first MFMA operand a lane holds 4 channels of ONE row
// per tile, so the factor is one register per row tile (two with GLU: gate and up have their own weight scales).
//
// Registers decide the schedule: a 16x16x128 operand fragment is 8 registers, so only 4 of a wave's 8 activation
// fragments and its 4 weight fragments are live (64 registers beside the 128 accumulators).  A stage is multiplied in two
// halves of 16 MFMAs: row tiles 0 .. 3 fragment by fragment (each reloaded with row tile + 4 right after its four MFMAs),
// then row tiles 4 .. 7 weight fragment by weight fragment (each weight fragment reloaded with the next stage's right
// after its four MFMAs, the activation fragments during the last four).  The stage barrier sits between the halves: by
// then every fragment of the stage is in registers and its buffer takes the stage after next.
//
// The activation scales of four stages (256 rows x 16 bytes) and the two weight-scale rows the tile needs travel the same
// way, into two small LDS buffers, so that nothing but LDS reads and the stream's own requests is ever waited for inside
// the loop.

#include "moe_gmm_common.h"

namespace moe {

template <bool GLU_>
struct F8sCfg {
  static constexpr bool GLU = GLU_;
  static constexpr int BM = 256, BN = 256, BKB = 128, MI = 16;
  static constexpr int WAVES_M = 2, WAVES_N = 4, NWAVES = 8, THREADS = NWAVES * kWave;
  static constexpr int WM = BM / WAVES_M, WN = BN / WAVES_N, TM = WM / MI, TN = WN / MI, RING = 4;
  static constexpr int A_STAGE = BM * BKB, STAGE = (BM + BN) * BKB;
  static constexpr int A_IPW = BM / 8 / NWAVES, B_IPW = BN / 8 / NWAVES;  // requests per wave and stage: 4 + 4
  // scales of four stages: 256 rows x 4 f32, then the two weight-scale rows (each lane of the request writes the same
  // 16 bytes: 1 KB per row)
  static constexpr int SC_A = BM * 16, SC_BYTES = SC_A + 2 * 1024, SC_OFF = 2 * STAGE;
  static constexpr int LDS_BYTES = 2 * STAGE + 2 * SC_BYTES;
  static constexpr int OUT_BN = GLU ? BN / 2 : BN;
  static_assert(TM == 8 && TN == 4 && 2 * RING == TM, "the two halves of a stage");
  static_assert(LDS_BYTES <= 160 * 1024, "LDS");
  __device__ static __forceinline__ int swz(int row) { return (row >> 1) & 7; }
};

template <typename C>
__global__ __launch_bounds__(C::THREADS, 2) void gmm_f8s_kernel(const Fp8TiledParams P) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t smem[];
  const TiledParams& p = P.base;
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wm = wave % C::WAVES_M, wn = wave / C::WAVES_M;
  const int N = p.N, K = p.K;
  const uint32_t row_bytes = (uint32_t)K;
  const int num_tiles = p.header[0];
  const int nk = K / C::BKB;  // stages = scale blocks
  const int nnb = (N + 127) / 128;
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
  v4i a_desc, b_desc, s_desc, w_desc = {0, 0, 0, 0};
  uint32_t a_voff[C::A_IPW], b_voff[C::B_IPW], b_soff = 0, s_voff = 0, w_soff = 0;
  const uint32_t scale_row_bytes = (uint32_t)nk * 4;
  auto set_a_sources = [&](const Tile& t) {
    if (p.ro.row_idx) {
      a_desc = buffer_desc(p.lhs, clamp_u32((size_t)p.ro.lhs_rows * row_bytes));
      s_desc = buffer_desc(P.a_scale, clamp_u32((size_t)p.ro.lhs_rows * scale_row_bytes));
      int rows[C::A_IPW];
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) rows[i] = min(t.info.row0 + (wave * C::A_IPW + i) * 8 + lane / 8, p.M - 1);
      lhs_rows_of<C::A_IPW>(p.ro, rows);
#pragma unroll
      for (int i = 0; i < C::A_IPW; i++) a_voff[i] = lane_off(i, (uint32_t)rows[i]);
      if (wave < 4) {  // the scale rows of tile rows wave * 64 + lane
        int srow[1] = {min(t.info.row0 + wave * 64 + lane, p.M - 1)};
        lhs_rows_of<1>(p.ro, srow);
        s_voff = (uint32_t)srow[0] * scale_row_bytes;
      }
    } else {
      a_desc = buffer_desc(p.lhs + (size_t)t.info.row0 * row_bytes, clamp_u32((size_t)t.info.nrows * row_bytes));
      s_desc = buffer_desc(P.a_scale + (size_t)t.info.row0 * nk, clamp_u32((size_t)t.info.nrows * scale_row_bytes));
    }
  };
  if (!p.ro.row_idx) {
#pragma unroll
    for (int i = 0; i < C::A_IPW; i++) a_voff[i] = lane_off(i, (uint32_t)((wave * C::A_IPW + i) * 8 + lane / 8));
    s_voff = (uint32_t)(wave * 64 + lane) * scale_row_bytes;
  }
  // weights: with GLU the upper 128 of the tile's 256 rows are the second projection's, whose requests come from waves 4 .. 7
  const bool load_up = C::GLU && wave >= C::NWAVES / 2;
#pragma unroll
  for (int i = 0; i < C::B_IPW; i++) {
    const int r = (wave * C::B_IPW + i) * 8 + lane / 8;
    b_voff[i] = lane_off(i, (uint32_t)(C::GLU ? r % (C::BN / 2) : r));
  }
  auto set_b_sources = [&](const Tile& t) {
    b_desc = buffer_desc((load_up ? p.rhs_up : p.rhs) + (size_t)t.info.group * N * row_bytes, clamp_u32((size_t)N * row_bytes));
    b_soff = (uint32_t)t.n0 * row_bytes;
    // the tile's two weight-scale rows: gate and up of its 128 channels, or its two blocks of 128 channels; waves 4 and 5
    // request one each
    if (wave == 4 || wave == 5) {
      const int sel = wave - 4;
      const float* base = C::GLU && sel ? P.u_scale : P.w_scale;
      const int nb = C::GLU ? t.n0 / 128 : min(t.n0 / 128 + sel, nnb - 1);
      w_desc = buffer_desc(base, 0xffffffffu);
      w_soff = (uint32_t)(((size_t)t.info.group * nnb + nb) * scale_row_bytes);
    }
  };
  // request idx of the stage: 0 .. 3 activations, 4 .. 7 weights
  auto issue_one = [&](int kt, int buf, int idx) {
    if (idx < C::A_IPW) dma16_buffer(a_desc, a_voff[idx], (uint32_t)kt * C::BKB, lds_base + buf * C::STAGE + (wave * C::A_IPW + idx) * 1024);
    else dma16_buffer(b_desc, b_voff[idx - C::A_IPW], b_soff + (uint32_t)kt * C::BKB, lds_base + buf * C::STAGE + C::A_STAGE + (wave * C::B_IPW + idx - C::A_IPW) * 1024);
  };
  // the scales of stages 4 * chunk .. + 3 into scale buffer sb
  auto issue_scales = [&](int chunk, int sb) {
    const uint32_t dst = lds_base + C::SC_OFF + sb * C::SC_BYTES;
    // one request with operands chosen per wave (two requests in the arms of a branch get merged by the compiler into
    // one whose scalar operands it can no longer keep in scalar registers)
    const bool is_w = wave >= 4;
    v4i d;
#pragma unroll
    for (int c = 0; c < 4; c++) d[c] = __builtin_amdgcn_readfirstlane(is_w ? w_desc[c] : s_desc[c]);
    const uint32_t so = (uint32_t)__builtin_amdgcn_readfirstlane((int)((is_w ? w_soff : 0u) + (uint32_t)chunk * 16));
    const uint32_t la = (uint32_t)__builtin_amdgcn_readfirstlane((int)(dst + (is_w ? C::SC_A + (wave - 4) * 1024 : wave * 1024)));
    if (wave < 6) dma16_buffer(d, is_w ? 0u : s_voff, so, la);
  };

  // ---- the multiplying side ----------------------------------------------------------------------------------------
  v4f acc[C::TN][C::TM];
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
  // which of the two weight-scale rows a weight fragment takes
  constexpr int NSEL = C::GLU ? 2 : 1;
  auto sel_of = [&](int j) { return C::GLU ? (j >= C::TN / 2 ? 1 : 0) : 0; };
  const int w_row_off = C::GLU ? 0 : (wn >= 2 ? 1024 : 0);
  // fragment: row (lane % 16), K bytes 16 q .. and 64 + 16 q .. with q = lane / 16 (both operands alike), i.e. the 16-byte
  // chunks q and 4 + q of the row, stored at slot chunk ^ swz(row)
  const int frag_lane = (lane % 16) * C::BKB + (((lane / 16) ^ C::swz(lane % 16)) << 4);
  v8i ga[C::RING], gb[C::TN];
  auto read_frag = [&](v8i& f, const uint8_t* base) {
    const v4i lo = *(const v4i*)(base + frag_lane), hi = *(const v4i*)(base + (frag_lane ^ 64));
    f[0] = lo[0]; f[1] = lo[1]; f[2] = lo[2]; f[3] = lo[3];
    f[4] = hi[0]; f[5] = hi[1]; f[6] = hi[2]; f[7] = hi[3];
  };
  auto read_a = [&](int buf, int i, int slot) { read_frag(ga[slot], smem + buf * C::STAGE + (wm * C::WM + i * 16) * C::BKB); };
  auto read_b = [&](int buf, int j) { read_frag(gb[j], smem + buf * C::STAGE + C::A_STAGE + b_row[j] * C::BKB); };
  // factors of the current stage per row tile: s_lo for row tiles 0 .. 3, s_hi for 4 .. 7
  float s_lo[NSEL][C::RING], s_hi[NSEL][C::RING];
  float a_raw[C::RING], w_raw[NSEL];
  const int scale_lane = (wm * C::WM + lane % 16) * 16;
  auto read_scales = [&](int sb, int col, int half) {
    const uint8_t* base = smem + C::SC_OFF + sb * C::SC_BYTES;
#pragma unroll
    for (int ii = 0; ii < C::RING; ii++) a_raw[ii] = *(const float*)(base + scale_lane + (half * C::RING + ii) * 256 + col * 4);
#pragma unroll
    for (int s = 0; s < NSEL; s++) w_raw[s] = *(const float*)(base + C::SC_A + w_row_off + s * 1024 + col * 4);
  };
  auto set_factors = [&](float (&dst)[NSEL][C::RING]) {
#pragma unroll
    for (int s = 0; s < NSEL; s++)
#pragma unroll
      for (int ii = 0; ii < C::RING; ii++) dst[s][ii] = a_raw[ii] * w_raw[s];
  };
  v4f pq[2];  // partial sums of the last two MFMAs
  const v4f zero = {0.f, 0.f, 0.f, 0.f};
  // (the empty asm statements pin a result to its place in the instruction stream: an MFMA whose sum is only used a slot
  // later and the FMAs that use it are otherwise placed wherever the instruction selector likes, which is not between
  // the requests and reads they are meant to overlap)
  auto add_scaled = [&](v4f& a, const v4f& part, float f) {
#pragma unroll
    for (int r = 0; r < 4; r++) a[r] = fmaf(part[r], f, a[r]);
    asm volatile("" : "+v"(a));
  };
  // slot t: the MFMA goes out first, then the FMAs of the slot before it
  auto mfma = [&](int t, const v8i& w, const v8i& x) {
    pq[t % 2] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(w, x, zero, 0, 0, 0, 127, 0, 127);
    asm volatile("" : "+v"(pq[0]), "+v"(pq[1]));
  };
  using T_ = std::true_type;
  using F_ = std::false_type;

  // First half of a stage (in buffer buf): row tiles 0 .. 3 from the ring, each slot reloaded with row tile + 4; the
  // factors of row tiles 4 .. 7 are read (scale buffer sb, column col).  PEND: the partial sum of the MFMA before this
  // half (weight fragment 3, row tile 7) is still to be added.
  auto half_lo = [&](auto pend_c, int buf, int sb, int col) {
    constexpr bool PEND = decltype(pend_c)::value;
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const int i = t / 4, j = t % 4;
      mfma(t, gb[j], ga[i]);
      if (t == 0) {
        if (PEND) add_scaled(acc[3][7], pq[1], s_hi[sel_of(3)][3]);
        read_scales(sb, col, 1);
      } else {
        add_scaled(acc[(t - 1) % 4][(t - 1) / 4], pq[(t - 1) % 2], s_lo[sel_of((t - 1) % 4)][(t - 1) / 4]);
      }
      if (t == 2) set_factors(s_hi);
      if (j == 3) read_a(buf, i + C::RING, i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // Second half of a stage: row tiles 4 .. 7 (in the ring), weight fragment by weight fragment.  RD: the next stage
  // (buffer rd_buf) is prepared behind it: its weight fragments, its row tiles 0 .. 3 and the factors of those (scale
  // buffer sb, column col).  LD: the eight requests of stage ld_kt go out into ld_buf, then the scales of chunk
  // sc_chunk into scale buffer sc_sb (sc_chunk < 0: none).
  auto half_hi = [&](auto rd_c, int rd_buf, int sb, int col, int ld_kt, int ld_buf, int sc_chunk, int sc_sb) {
    constexpr bool RD = decltype(rd_c)::value;
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const int j = t / 4, i = C::RING + t % 4;
      mfma(t, gb[j], ga[t % 4]);
      if (t == 0) {
        add_scaled(acc[3][3], pq[1], s_lo[sel_of(3)][3]);
        if (RD) read_scales(sb, col, 0);
      } else {
        add_scaled(acc[(t - 1) / 4][C::RING + (t - 1) % 4], pq[(t - 1) % 2], s_hi[sel_of((t - 1) / 4)][(t - 1) % 4]);
      }
      if (RD && t == 2) set_factors(s_lo);
      if (t < C::A_IPW + C::B_IPW) issue_one(ld_kt, ld_buf, t);
      if (t == C::A_IPW + C::B_IPW && sc_chunk >= 0) issue_scales(sc_chunk, sc_sb);
      if (RD && t % 4 == 3) read_b(rd_buf, j);
      if (RD && j == 3) read_a(rd_buf, t % 4, t % 4);
      (void)i;
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  constexpr int NT_OUT = C::GLU ? C::TN / 2 : C::TN;

  // What a tile's first half stage needs, with nothing to hide behind: zeroed sums, row tiles 0 .. 3 and the weight
  // fragments of stage 0 (buffer buf), the factors of row tiles 0 .. 3 (scale buffer sb, column 0).
  auto first_fragments = [&](int buf, int sb) {
#pragma unroll
    for (int j = 0; j < C::TN; j++)
#pragma unroll
      for (int i = 0; i < C::TM; i++) acc[j][i] = zero;
    read_scales(sb, 0, 0);
#pragma unroll
    for (int i = 0; i < C::RING; i++) read_a(buf, i, i);
#pragma unroll
    for (int j = 0; j < C::TN; j++) read_b(buf, j);
    set_factors(s_lo);
  };

  Tile cur, nxt;
  if (!resolve(peek_from(blockIdx.x), cur)) return;
  // ---- head of the stream: the first tile's stages 0 and 1 and its first scales ----
  set_a_sources(cur);
  set_b_sources(cur);
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int i = 0; i < C::A_IPW + C::B_IPW; i++) issue_one(s, s, i);
  issue_scales(0, 0);
  wait_vmcnt<0>();
  asm volatile("s_barrier" ::: "memory");
  first_fragments(0, 0);

  int base = 0;   // the buffer that holds stage 0 of the current tile
  int sbase = 0;  // the scale buffer that holds the current tile's stages 0 .. 3
  const int nchunk = nk / 4;
  while (true) {
    // the record of the block's next tile is requested now and looked at two stages before this tile ends
    Peek pk = peek_from(cur.id + gridDim.x);
    bool have_n = false;
    const int n_out0 = cur.n0 + (C::GLU ? wn * (C::WN / 2) : wn * C::WN);
    // first half of stage 0
    half_lo(F_{}, base, sbase, 0);
    // Iteration `it`: the second half of stage it, then the first half of stage it + 1.  Every fragment of stage it is in
    // registers before the barrier, and stage it + 1 has landed at it: the buffer of stage it takes stage it + 2 of the
    // stream (from nk on: the next tile's); every fourth iteration the scales of the four stages from it + 2 on follow.
    auto stream_kt = [&](int s) { return s < nk ? s : (have_n ? s - nk : nk - 1); };
    int cb = base;  // buffer of stage `it`
    auto iteration = [&](int it, auto last_c) {
      constexpr bool LAST = decltype(last_c)::value;  // the tile's last half stage: nothing is prepared behind it
      // own fragment reads done, own requests landed: then everybody's
      __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
      wait_vmcnt<0>();
      asm volatile("s_barrier" ::: "memory");
      const int s2 = it + 2;
      int sc_chunk = -1, sc_sb = 0;
      if (s2 % 4 == 0) {
        if (s2 < nk) {
          sc_chunk = s2 / 4;
          sc_sb = (sbase + sc_chunk) & 1;
        } else if (have_n) {
          sc_chunk = 0;
          sc_sb = (sbase + nchunk) & 1;
        }
      }
      const int s1 = it + 1;  // the stage prepared behind this half
      if (LAST) {
        half_hi(F_{}, 0, 0, 0, stream_kt(s2), cb, sc_chunk, sc_sb);
      } else {
        half_hi(T_{}, cb ^ 1, (sbase + s1 / 4) & 1, s1 % 4, stream_kt(s2), cb, sc_chunk, sc_sb);
        half_lo(T_{}, cb ^ 1, (sbase + s1 / 4) & 1, s1 % 4);
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
    add_scaled(acc[3][7], pq[1], s_hi[sel_of(3)][3]);
    EpilogueScales<C::TM, NT_OUT, C::GLU> esc;
    load_epilogue_scales<C::TM, NT_OUT, C::GLU, false, C::MI>(esc, p, cur.info, wm * C::WM, n_out0, lane);
    store_epilogue<C::TM, C::TN, NT_OUT, C::GLU>(acc, esc, p, cur.info, wm * C::WM, n_out0, lane);
    if (!have_n) break;
    cur = nxt;
    base = cb;  // the buffer of stage nk = the next tile's stage 0, landed before the last barrier
    sbase = (sbase + nchunk) & 1;
    first_fragments(base, sbase);
  }
  // nothing may still be writing LDS when the block ends
  __builtin_amdgcn_s_waitcnt(0xC07F);
  wait_vmcnt<0>();
}

// ---------------------------------------------------------------------------------------
// Host side
// ---------------------------------------------------------------------------------------

template <typename C>
static int prepare_f8s_cfg() {
  return reserve_lds(gmm_f8s_kernel<C>, C::LDS_BYTES, lds_flags<C>());
}

int prepare_f8s() {
  int st = prepare_f8s_cfg<F8sCfg<false>>();
  if (!st) st = prepare_f8s_cfg<F8sCfg<true>>();
  return st;
}

template <typename C>
static int launch_f8s_cfg(const Fp8TiledParams& P0, int M, int G_total, hipStream_t s) {
  if (int st = prepare_f8s_cfg<C>()) return st;
  Fp8TiledParams P = P0;
  TiledParams& p = P.base;
  p.max_m_tiles = max_tiles_for(M, G_total, C::BM);
  p.tiles_n = cdiv(p.N, C::OUT_BN);
  const long long tiles = (long long)p.max_m_tiles * p.tiles_n;
  if (tiles > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "gmm: grid too large");
  // m-tiles per super-row of the tile order: as many as a group has on average, so that the tiles an XCD works on at a
  // time share their weight panels (DeepSeek-V3 at 16384 tokens, 574 rows per expert: 5.6 ms with 3 against 6.0 ms with 8)
  if (p.tune <= 0) {
    const long long per_group = cdiv((int)cdiv(M, G_total), C::BM);
    p.tune = (int)(per_group < 1 ? 1 : per_group > 8 ? 8 : per_group);
  }
  // one persistent block per CU; a multiple of 8 keeps "tile id mod 8" equal to the XCD a block runs on
  int num_cus = 0;
  if (int st = device_cu_count(&num_cus)) return st;
  long long blocks = tiles < num_cus ? tiles : num_cus;
  if (blocks >= 8) blocks -= blocks % 8;
  gmm_f8s_kernel<C><<<(unsigned)blocks, C::THREADS, C::LDS_BYTES, s>>>(P);
  return check_launch("gmm_f8s_kernel");
}

bool f8s_takes(int K, int N, long long M, long long indexed_lhs_rows) {
  // stages in groups of four (the scales travel four stages at a time); byte offsets inside one expert's weight matrix,
  // inside the activations and inside their scales fit 32 bits
  const long long rows = indexed_lhs_rows > 0 ? indexed_lhs_rows : M;
  // (a request's lane row reaches up to 255 rows past the last n-tile's first row / the last indexed row: see dls_takes)
  return K % 512 == 0 && K >= 512 && ((long long)N + 256) * K < (1LL << 32) && (rows + 256) * K < (1LL << 32);
}

int launch_f8s(bool glu, const Fp8TiledParams& P, int M, int G_total, hipStream_t s) {
  const TiledParams& p = P.base;
  if (!P.a_scale || !P.w_scale || !f8s_takes(p.K, p.N, M, p.ro.row_idx ? p.ro.lhs_rows : 0))
    return fail(MOE_ERR_UNSUPPORTED, "gmm: the fp8 stream kernel needs block scales, K a multiple of 512 and 32-bit byte offsets");
  return glu ? launch_f8s_cfg<F8sCfg<true>>(P, M, G_total, s) : launch_f8s_cfg<F8sCfg<false>>(P, M, G_total, s);
}

}  // namespace moe
