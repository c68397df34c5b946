// Transposed grouped matmul (weight gradient): out[g][n][k] = sum over the rows m of group g of
// dout[m][n] * lhs[m][k].  Both operands are row-major with the contraction index m as the ROW index, the
// opposite of what an MFMA fragment wants (8 consecutive contraction values per lane).  The tiles are staged
// in LDS as they are and read back with ds_read_b64_tr_b16, gfx950's transposing LDS load: within 16 lanes,
// lane L receives the L-th 16-bit column of a 4 x 16 block whose rows are addressed by lanes 0-3, 4-7, ...
// Two such reads give a lane its 8 contraction values.  lhs is the MFMA "A" operand (32 k channels), dout
// the "B" operand (32 n channels), so a lane ends up with 4 consecutive k of one n: contiguous stores into
// the [G, N, K] weight layout.

#include "moe_gmm_common.h"

namespace moe {

constexpr int kTgBN = 128, kTgBK = 128, kTgBM = 32;  // output tile [BN x BK], contraction chunk BM rows
constexpr int kTgThreads = 256;
constexpr int kTgLdr = kTgBN * 2 + 32;  // LDS row stride in bytes (the pad spreads the 4 rows of a transposing read over the banks)

struct TgmmParams {
  const uint16_t* lhs;   // [M, K] bf16
  const uint16_t* dout;  // [M, N] bf16
  const int32_t* group_sizes;
  void* out;  // [G_local, N, K] bf16 or f32
  const void* existing;  // NULL, or [G_local, N, K] values added to the products before the store (may be `out` itself)
  const float* n_scale;  // NULL, or [N]: the products of output row n are multiplied by n_scale[n] first
  int M, K, N;
  int G_total, G_local, group_offset;
  int out_f32, existing_f32;
};

// out[off .. off+3] = v * n_scale[n] + existing[off .. off+3]: four values along K of output row n.  A lane reads the
// four values it is about to overwrite, so `existing` may be the output buffer.
__device__ __forceinline__ void tgmm_store4(const TgmmParams& p, size_t off, int n, float v0, float v1, float v2, float v3) {
  if (p.n_scale) {
    const float sc = p.n_scale[n];
    v0 *= sc; v1 *= sc; v2 *= sc; v3 *= sc;
  }
  if (p.existing) {
    if (p.existing_f32) {
      const float4 e = *(const float4*)((const float*)p.existing + off);
      v0 += e.x; v1 += e.y; v2 += e.z; v3 += e.w;
    } else {
      const uint2 e = *(const uint2*)((const uint16_t*)p.existing + off);
      v0 += bf16_bits_to_f32(e.x & 0xffffu); v1 += bf16_bits_to_f32(e.x >> 16);
      v2 += bf16_bits_to_f32(e.y & 0xffffu); v3 += bf16_bits_to_f32(e.y >> 16);
    }
  }
  if (p.out_f32) *(float4*)((float*)p.out + off) = make_float4(v0, v1, v2, v3);
  else *(uint2*)((uint16_t*)p.out + off) = make_uint2(pack_bf16x2(v0, v1), pack_bf16x2(v2, v3));
}

__device__ __forceinline__ v8bf read_tr_frag(const uint8_t* tile, int row0, int col0, int lane) {
  // 8 contraction values (rows row0 + 8*(lane/32) .. +7) of column col0 + lane%32
  const int s = lane % 16, cg = (lane / 16) % 2, half = lane / 32;
  const uint8_t* p = tile + (row0 + half * 8 + s / 4) * kTgLdr + (col0 + cg * 16 + 4 * (s % 4)) * 2;
  const v4s lo = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)p);
  const v4s hi = __builtin_amdgcn_ds_read_tr16_b64_v4i16((lds_v4s_t)(p + 4 * kTgLdr));
  typedef short v8s __attribute__((ext_vector_type(8)));
  const v8s v = {lo[0], lo[1], lo[2], lo[3], hi[0], hi[1], hi[2], hi[3]};
  return __builtin_bit_cast(v8bf, v);
}

__global__ __launch_bounds__(kTgThreads) void tgmm_kernel(const TgmmParams p) {
  __shared__ __attribute__((aligned(16))) uint8_t smem[2][2][kTgBM * kTgLdr];  // [buffer][lhs|dout]
  __shared__ int s_red[kTgThreads / kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  const int wk = wave % 2, wn = wave / 2;  // wave tile: 64 k x 64 n
  const int g_local = blockIdx.z, g = g_local + p.group_offset;
  const int n0 = blockIdx.y * kTgBN, k0 = blockIdx.x * kTgBK;
  const int N = p.N, K = p.K;

  // rows of group g: [start, start + size), clipped to M (sum of the sizes of the groups before it)
  long long part = 0;
  for (int i = tid; i < min(g, p.G_total); i += kTgThreads) part += max(p.group_sizes[i], 0);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
  if (lane == 0) s_red[wave] = (int)min(part, (long long)p.M);
  __syncthreads();
  long long start_ll = 0;
  for (int w = 0; w < kTgThreads / kWave; w++) start_ll += s_red[w];
  const int start = (int)min(start_ll, (long long)p.M);
  const int size = g < p.G_total ? min(max(p.group_sizes[g], 0), p.M - start) : 0;

  // staging: each tile is 32 rows x 256 bytes = 512 16-byte chunks, 2 per thread and operand
  int st_row[2], st_col[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int c = tid + i * kTgThreads;
    st_row[i] = c / 16;
    st_col[i] = (c % 16) * 8;  // element column within the tile
  }
  uint4 ra[2], rb[2];
  auto load_chunk = [&](int m0) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      const int r = m0 + st_row[i];
      const bool ok = r < size;
      const size_t row = (size_t)(start + (ok ? r : 0));
      const int kc = k0 + st_col[i], nc = n0 + st_col[i];
      uint4 a = make_uint4(0, 0, 0, 0), b = make_uint4(0, 0, 0, 0);
      if (ok && kc < K) a = *(const uint4*)(p.lhs + row * K + kc);
      if (ok && nc < N) b = *(const uint4*)(p.dout + row * N + nc);
      ra[i] = a;
      rb[i] = b;
    }
  };
  auto store_chunk = [&](int buf) {
#pragma unroll
    for (int i = 0; i < 2; i++) {
      *(uint4*)(&smem[buf][0][st_row[i] * kTgLdr + st_col[i] * 2]) = ra[i];
      *(uint4*)(&smem[buf][1][st_row[i] * kTgLdr + st_col[i] * 2]) = rb[i];
    }
  };

  v16f acc[2][2];  // [n tile][k tile]
#pragma unroll
  for (int j = 0; j < 2; j++)
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int r = 0; r < 16; r++) acc[j][i][r] = 0.f;

  const int nchunks = (size + kTgBM - 1) / kTgBM;
  if (nchunks > 0) {
    load_chunk(0);
    store_chunk(0);
  }
  __syncthreads();
  for (int c = 0; c < nchunks; c++) {
    const int cur = c & 1;
    if (c + 1 < nchunks) load_chunk((c + 1) * kTgBM);
#pragma unroll
    for (int ks = 0; ks < kTgBM / 16; ks++) {
      v8bf fk[2], fn[2];
#pragma unroll
      for (int i = 0; i < 2; i++) fk[i] = read_tr_frag(smem[cur][0], ks * 16, wk * 64 + i * 32, lane);
#pragma unroll
      for (int j = 0; j < 2; j++) fn[j] = read_tr_frag(smem[cur][1], ks * 16, wn * 64 + j * 32, lane);
#pragma unroll
      for (int j = 0; j < 2; j++)
#pragma unroll
        for (int i = 0; i < 2; i++) acc[j][i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(fk[i], fn[j], acc[j][i], 0, 0, 0);
    }
    if (c + 1 < nchunks) store_chunk(cur ^ 1);
    __syncthreads();
  }

  // D[i = k][j = n]: lane holds n = lane % 32 and k = 8*q + 4*(lane/32) + r
#pragma unroll
  for (int j = 0; j < 2; j++) {
    const int n = n0 + wn * 64 + j * 32 + (lane % 32);
    if (n >= N) continue;
#pragma unroll
    for (int i = 0; i < 2; i++)
#pragma unroll
      for (int q = 0; q < 4; q++) {
        const int k = k0 + wk * 64 + i * 32 + 8 * q + 4 * (lane / 32);
        if (k >= K) continue;
        const size_t off = ((size_t)g_local * N + n) * K + k;
        tgmm_store4(p, off, n, acc[j][i][4 * q], acc[j][i][4 * q + 1], acc[j][i][4 * q + 2], acc[j][i][4 * q + 3]);
      }
  }
}


// ---------------------------------------------------------------------------------------
// 256 (n) x 256 (k) output tiles for groups of many rows, on the pipeline of the direct-to-LDS GEMM: a stage is
// 64 contraction rows of both operands (64 x 512 bytes each), copied by global_load_lds_dwordx4 (a wave
// instruction moves two rows of 512 bytes: whole 128-byte lines) into two buffers of 64 KB; 8 waves of
// 64 (k) x 128 (n) on v_mfma_f32_16x16x32_bf16, two k-steps of 32 MFMAs per stage; the 4 lhs fragments of a wave
// are double-buffered in registers, each of its 8 dout fragments is reloaded for the next k-step right after the four
// MFMAs that use it.  Fragments come out of the row-major stage through ds_read_b64_tr_b16 as in tgmm_kernel.  LDS
// rows are unpadded, so the 16-byte chunk q of row r is stored at slot q ^ f(r), f(r) = 4 * (r % 4) ^ 2 * ((r / 8) % 2):
// the 4 rows x 32 bytes that 16 lanes of a transposing read address, and those of the next 16 lanes (8 rows further),
// then fall into 8 different 32-byte bank groups.  The permutation is applied on the global side (the LDS side of
// the copy is fixed at base + 16 * lane) and stays inside a row's 512 bytes, so every request still covers whole
// lines.  Rows past the end of the group are copied from a row of zeros.
// ---------------------------------------------------------------------------------------

constexpr int kTdTile = 256, kTdBM = 64;       // output tile edge, contraction rows per stage
constexpr int kTdThreads = 512, kTdWaves = 8;
constexpr int kTdRow = kTdTile * 2;            // bytes of one operand row in a stage
constexpr int kTdOperand = kTdBM * kTdRow;     // 32 KB
constexpr int kTdStage = 2 * kTdOperand;       // lhs rows | dout rows
constexpr int kTdLds = 2 * kTdStage;           // two buffers
constexpr int kTdIpw = kTdOperand / 1024 / kTdWaves;  // requests per wave, operand and stage
constexpr int kTdLps = 2 * kTdIpw;

__device__ __attribute__((aligned(512))) uint8_t tg_zero_row[kTdRow];

__global__ __launch_bounds__(kTdThreads, 2) void tgmm_dl_kernel(const TgmmParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t td_smem[];
  __shared__ int s_red[kTdWaves];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wk = wave % 4, wn = wave / 4;  // wave tile: 64 k x 128 n
  const int N = p.N, K = p.K;

  // Blocks b, b + 8, .. run on one XCD: give each XCD a contiguous range of tiles, walked in patches of 8 n-tiles x
  // 4 k-tiles of one group, so that the 32 blocks an XCD runs at a time share 8 dout and 4 lhs panels in its L2.
  const int tiles_k = K / kTdTile, tiles_n = N / kTdTile, per_group = tiles_k * tiles_n;
  const int total = per_group * p.G_local;
  const int q8 = total / 8, rem = total % 8, xcd = blockIdx.x % 8, loc = blockIdx.x / 8;
  const int logical = xcd < rem ? xcd * (q8 + 1) + loc : rem * (q8 + 1) + (xcd - rem) * q8 + loc;
  const int g_local = logical / per_group, t = logical % per_group, g = g_local + p.group_offset;
  constexpr int GSM = 8;
  const int width = GSM * tiles_k, first_n = (t / width) * GSM, gsz = min(tiles_n - first_n, GSM);
  const int n0 = (first_n + (t % width) % gsz) * kTdTile, k0 = ((t % width) / gsz) * kTdTile;

  // rows of group g: [start, start + size), clipped to M
  long long part = 0;
  for (int i = tid; i < min(g, p.G_total); i += kTdThreads) part += max(p.group_sizes[i], 0);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
  if (lane == 0) s_red[wave] = (int)min(part, (long long)p.M);
  __syncthreads();
  long long start_ll = 0;
  for (int w = 0; w < kTdWaves; w++) start_ll += s_red[w];
  // (uniform by construction; saying so lets the requests below use a scalar base address)
  const int start = __builtin_amdgcn_readfirstlane((int)min(start_ll, (long long)p.M));
  const int size = __builtin_amdgcn_readfirstlane(g < p.G_total ? min(max(p.group_sizes[g], 0), p.M - start) : 0);

  const int s16 = lane % 16, gq = lane / 16;
  if (size == 0) {  // an empty group's gradient is zero
    for (int i = tid; i < kTdTile * (kTdTile / 4); i += kTdThreads) {
      const size_t off = ((size_t)g_local * N + n0 + i / (kTdTile / 4)) * K + k0 + (i % (kTdTile / 4)) * 4;
      tgmm_store4(p, off, n0 + i / (kTdTile / 4), 0.f, 0.f, 0.f, 0.f);
    }
    return;
  }

  // ---- sources of this wave's requests: request i of an operand covers stage rows 2 * (4 * wave + i) + {0, 1}.  A
  // stage's first row is a scalar base, the lane adds a 32-bit offset.  Only a group's last stage can hold rows past its
  // end: requests of full stages (FULL) need no check, the others pick the row of zeros per lane, without a branch.
  // Requests i and i + 2 of a wave are 4 rows apart, which leaves the swizzle as it is: two per-lane offsets per operand.
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = 2 * (wave * kTdIpw + i) + lane / 32;
    const int chunk = (lane % 32) ^ tr_swz(r);
    a_off[i] = (uint32_t)r * K * 2 + chunk * 16;
    b_off[i] = (uint32_t)r * N * 2 + chunk * 16;
  }
  static_assert(kTdIpw == 4, "request i + 2 is request i four rows further down");
  const uint8_t* const a_base = (const uint8_t*)p.lhs + ((size_t)start * K + k0) * 2;
  const uint8_t* const b_base = (const uint8_t*)p.dout + ((size_t)start * N + n0) * 2;
  const size_t a_step = (size_t)kTdBM * K * 2, b_step = (size_t)kTdBM * N * 2;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)td_smem;
  auto issue_one = [&](auto full_c, int kt, int buf, int idx) {
    constexpr bool FULL = decltype(full_c)::value;
    const int i = idx % kTdIpw;
    const bool is_a = idx < kTdIpw;
    const uint8_t* src = is_a ? a_base + (kt * a_step + (size_t)(i / 2) * 8 * K) + a_off[i % 2]
                              : b_base + (kt * b_step + (size_t)(i / 2) * 8 * N) + b_off[i % 2];
    if constexpr (!FULL) {
      int l = lane;
      asm volatile("" : "+v"(l));  // keeps what follows inside the (short) loops that need it, out of the steady state's registers
      const int r = 2 * (wave * kTdIpw + i) + l / 32;
      const uint64_t keep = kt * kTdBM + r < size ? ~0ull : 0ull;
      const uint64_t zero = (uint64_t)(tg_zero_row + ((l % 32) ^ tr_swz(r)) * 16);
      src = (const uint8_t*)(((uint64_t)src & keep) | (zero & ~keep));
    }
    // (untracked: which buffer a copy writes and a read reads is settled by the explicit vmcnt waits and barriers below)
    dma16_untracked(src, lds_base + buf * kTdStage + (is_a ? 0 : kTdOperand) + (wave * kTdIpw + i) * 1024);
  };

  // ---- fragments: lane (group gq, s16) addresses row 8 * gq + s16 / 4 (+ 4) of the k-step's 32 rows and the 8 bytes
  // 8 * (s16 % 4) of the fragment's 32-byte row slice; fragment f of an operand is 32 * f bytes further along the row
  // before the swizzle, which turns the step into an XOR of address bits 5..7.
  const int xmask = ((s16 / 4) << 2) ^ ((gq & 1) << 1);
  const int row_part = (gq * 8 + s16 / 4) * kTdRow, piece = s16 % 4;
  const int k_base = row_part + ((((8 * wk + piece / 2) ^ xmask) << 4) | ((piece & 1) << 3));
  const int n_base = row_part + ((((16 * wn + piece / 2) ^ xmask) << 4) | ((piece & 1) << 3));
  v8bf fk[2][4], fn[8];
  // (the two bases pass through an empty asm so that the 12 fragment addresses are formed where they are used, an XOR
  // and an add each, instead of living in 12 registers across the loop: the kernel has none to spare)
  auto read_k = [&](int buf, int ks, int set, int f) {
    int base = k_base;
    asm volatile("" : "+v"(base));
    fk[set][f] = tr_read_frag(td_smem + buf * kTdStage + ks * 32 * kTdRow + (base ^ (32 * f)), kTdRow);
  };
  auto read_n = [&](int buf, int ks, int f) {
    int base = n_base;
    asm volatile("" : "+v"(base));
    fn[f] = tr_read_frag(td_smem + buf * kTdStage + kTdOperand + ks * 32 * kTdRow + (base ^ (32 * f)), kTdRow);
  };

  v4f acc[4][8];  // [k fragment][n fragment]
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[j][i][r] = 0.f;

  // One k-step: 32 MFMAs on lhs fragment set SET with, slotted between them, the fragment reads of the next k-step
  // (RD) and the requests of a stage (LD, spread over the k-step).
  auto kstep = [&](auto set_c, auto rd_c, auto ld_c, auto full_c, int rd_buf, int rd_ks, int ld_kt, int ld_buf) {
    constexpr int SET = decltype(set_c)::value;
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value;
#pragma unroll
    for (int i = 0; i < 8; i++) {
#pragma unroll
      for (int j = 0; j < 4; j++) {
        acc[j][i] = __builtin_amdgcn_mfma_f32_16x16x32_bf16(fk[SET][j], fn[i], acc[j][i], 0, 0, 0);
        // (behind every fourth MFMA: one request per MFMA fills the address unit's queue and stalls the MFMAs behind it;
        // both shapes of the Mixtral layer 1.86 -> 1.69 / 1.72 ms, every third 1.75 / 1.76 ms)
        if (LD && (i * 4 + j) % 4 == 0 && (i * 4 + j) / 4 < kTdLps) issue_one(full_c, ld_kt, ld_buf, (i * 4 + j) / 4);
        if (RD && j == 1 && i < 4) read_k(rd_buf, rd_ks, SET ^ 1, i);
        if (RD && j == 3) read_n(rd_buf, rd_ks, i);
        __builtin_amdgcn_sched_barrier(0);
      }
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;
  using S0 = std::integral_constant<int, 0>;
  using S1 = std::integral_constant<int, 1>;

  // Stage kt sits in buffer kt % 2.  During a stage's first k-step the fragments of its second one are read, after
  // which no wave needs the buffer any more: once every wave has seen its own reads return and its requests of stage
  // kt+1 land, the block meets, and during the second k-step the fragments of stage kt+1 are read from the other
  // buffer while stage kt+2 is requested into this one (past the last stage the last one is requested again, into a
  // buffer nobody reads any more, which keeps the bookkeeping uniform).
  const int nk = (size + kTdBM - 1) / kTdBM;
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int i = 0; i < kTdLps; i++) issue_one(F_{}, min(s, nk - 1), s, i);
  wait_vmcnt<0>();
  __syncthreads();
#pragma unroll
  for (int f = 0; f < 8; f++) read_n(0, 0, f);
#pragma unroll
  for (int f = 0; f < 4; f++) read_k(0, 0, 0, f);
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  kstep(S0{}, T_{}, F_{}, F_{}, 0, 1, 0, 0);
  int kt = 0;
  const int nfull = size / kTdBM;  // stages 0 .. nfull-1 hold 64 rows of the group
  for (; kt + 2 < nfull; kt++) {   // steady state: the stage requested is a full one
    const int buf = kt % 2;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    kstep(S1{}, T_{}, T_{}, T_{}, buf ^ 1, 0, kt + 2, buf);
    kstep(S0{}, T_{}, F_{}, F_{}, buf ^ 1, 1, 0, 0);
  }
  for (; kt + 1 < nk; kt++) {
    const int buf = kt % 2;
    __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    kstep(S1{}, T_{}, T_{}, F_{}, buf ^ 1, 0, min(kt + 2, nk - 1), buf);
    kstep(S0{}, T_{}, F_{}, F_{}, buf ^ 1, 1, 0, 0);
  }
  kstep(S1{}, F_{}, F_{}, F_{}, 0, 0, 0, 0);
  wait_vmcnt<0>();  // no request may still be writing LDS when the block ends

  // D[k][n]: the lane holds n = s16 and k = 4 * gq + r of each 16 x 16 tile
  if (!p.out_f32 && !p.existing) {
    // plain bf16 results: neighbouring k-tiles trade halves between lanes 16 apart, so that a lane stores 16 bytes and
    // the 64 bytes of a row n leave in one instruction
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int n = n0 + wn * 128 + i * 16 + s16;
      const float sc = p.n_scale ? p.n_scale[n] : 1.0f;
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        const auto s0 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(acc[j][i][0] * sc, acc[j][i][1] * sc),
                                                         pack_bf16x2(acc[j + 1][i][0] * sc, acc[j + 1][i][1] * sc), false, false);
        const auto s1 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(acc[j][i][2] * sc, acc[j][i][3] * sc),
                                                         pack_bf16x2(acc[j + 1][i][2] * sc, acc[j + 1][i][3] * sc), false, false);
        const int k = k0 + wk * 64 + (j + (gq & 1)) * 16 + 4 * (gq & ~1);
        *(uint4*)((uint16_t*)p.out + ((size_t)g_local * N + n) * K + k) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int n = n0 + wn * 128 + i * 16 + s16;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int k = k0 + wk * 64 + j * 16 + 4 * gq;
      const size_t off = ((size_t)g_local * N + n) * K + k;
      tgmm_store4(p, off, n, acc[j][i][0], acc[j][i][1], acc[j][i][2], acc[j][i][3]);
    }
  }
}


// ---------------------------------------------------------------------------------------
// The same 256 x 256 tiles for 1-byte operands: the drhs product of the fp8_full backward (kernels/megablox/ops.py:590-604:
// float8_e4m3fn activations x float8_e5m2 gradient, the contraction running over the rows of both) on
// v_mfma_scale_f32_16x16x128_f8f6f4, without widening either operand.  A stage is 128 contraction rows of both operands
// (128 x 256 bytes each, a wave instruction copies four rows), two buffers of 64 KB.  Fragments come out of the row-major
// stage through ds_read_b64_tr_b8: 16 lanes address an 8-row x 16-byte block (lane l: row l / 2, half l % 2) and lane l
// receives column l of the 8 rows; four such reads give a lane the 32 contraction values of its column that one
// 16 x 16 x 128 fragment holds.  Lane group q takes stage rows 32 q .. 32 q + 31 for BOTH operands, which is all the
// instruction needs (any order of the contraction index, as long as the two fragments agree).  A fragment is 8
// registers, so a wave (64 k x 128 n) keeps its 4 lhs fragments and a ring of 4 of its 8 dout fragments beside the 128
// accumulators and multiplies a stage in two halves of 16 MFMAs: dout fragments 0 .. 3 from the ring (each slot reloaded
// with fragment + 4 after its four MFMAs), then fragments 4 .. 7, lhs fragment by lhs fragment, with the next stage's
// fragments read behind them.  The 16-byte chunk c of stage row r sits at slot c ^ (r % 8) ^ 8 * ((r / 32) % 2): the 8 rows
// of a read and those of the next lane group fall into 16 different 16-byte bank groups.
// ---------------------------------------------------------------------------------------

constexpr int kT8BM = 128;                            // contraction rows per stage
constexpr int kT8Row = kTdTile;                       // bytes of one operand row in a stage
constexpr int kT8Operand = kT8BM * kT8Row;            // 32 KB
constexpr int kT8Stage = 2 * kT8Operand;              // lhs rows | dout rows
constexpr int kT8Lds = 2 * kT8Stage;                  // two buffers
constexpr int kT8Ipw = kT8Operand / 1024 / kTdWaves;  // requests per wave, operand and stage
constexpr int kT8Lps = 2 * kT8Ipw;
constexpr int kT8ReqStride = 2;                       // a stage's requests go out behind every second MFMA of a half

__device__ __forceinline__ int t8_swz(int row) { return (row & 7) ^ (((row >> 5) & 1) << 3); }

typedef int v2i_t8 __attribute__((ext_vector_type(2)));
typedef __attribute__((address_space(3))) v2i_t8* lds_v2i_t8;
__device__ __forceinline__ void tr8_read_frag(v8i& f, const uint8_t* p) {
#pragma unroll
  for (int t = 0; t < 4; t++) {
    const v2i_t8 x = __builtin_amdgcn_ds_read_tr8_b64_v2i32((lds_v2i_t8)(p + t * 8 * kT8Row));
    f[2 * t] = x[0];
    f[2 * t + 1] = x[1];
  }
}

template <int DF>  // element format of dout: 0 = e4m3, 1 = e5m2 (lhs is e4m3)
__global__ __launch_bounds__(kTdThreads, 2) void tgmm_f8_kernel(const TgmmParams p) {
  extern __shared__ __attribute__((aligned(1024))) uint8_t t8_smem[];
  __shared__ int s_red[kTdWaves];
  const int tid = threadIdx.x, lane = tid % kWave;
  const int wave = __builtin_amdgcn_readfirstlane(tid / kWave);
  const int wk = wave % 4, wn = wave / 4;  // wave tile: 64 k x 128 n
  const int N = p.N, K = p.K;

  // tile of this block: the order of tgmm_dl_kernel (XCD ranges, patches of 8 n-tiles x 4 k-tiles of one group)
  const int tiles_k = K / kTdTile, tiles_n = N / kTdTile, per_group = tiles_k * tiles_n;
  const int total = per_group * p.G_local;
  const int q8 = total / 8, rem = total % 8, xcd = blockIdx.x % 8, loc = blockIdx.x / 8;
  const int logical = xcd < rem ? xcd * (q8 + 1) + loc : rem * (q8 + 1) + (xcd - rem) * q8 + loc;
  const int g_local = logical / per_group, t = logical % per_group, g = g_local + p.group_offset;
  constexpr int GSM = 8;
  const int width = GSM * tiles_k, first_n = (t / width) * GSM, gsz = min(tiles_n - first_n, GSM);
  const int n0 = (first_n + (t % width) % gsz) * kTdTile, k0 = ((t % width) / gsz) * kTdTile;

  long long part = 0;
  for (int i = tid; i < min(g, p.G_total); i += kTdThreads) part += max(p.group_sizes[i], 0);
#pragma unroll
  for (int o = 32; o > 0; o >>= 1) part += __shfl_xor(part, o);
  if (lane == 0) s_red[wave] = (int)min(part, (long long)p.M);
  __syncthreads();
  long long start_ll = 0;
  for (int w = 0; w < kTdWaves; w++) start_ll += s_red[w];
  const int start = __builtin_amdgcn_readfirstlane((int)min(start_ll, (long long)p.M));
  const int size = __builtin_amdgcn_readfirstlane(g < p.G_total ? min(max(p.group_sizes[g], 0), p.M - start) : 0);

  const int s16 = lane % 16, gq = lane / 16;
  if (size == 0) {  // an empty group's gradient is zero
    for (int i = tid; i < kTdTile * (kTdTile / 4); i += kTdThreads) {
      const size_t off = ((size_t)g_local * N + n0 + i / (kTdTile / 4)) * K + k0 + (i % (kTdTile / 4)) * 4;
      tgmm_store4(p, off, n0 + i / (kTdTile / 4), 0.f, 0.f, 0.f, 0.f);
    }
    return;
  }

  // ---- requests: request i of an operand covers stage rows 4 * (4 * wave + i) + {0 .. 3}, lane l the 16 bytes of LDS
  // slot l % 16 of row l / 16.  Requests i and i + 2 of a wave are 8 rows apart inside one block of 32 rows, which leaves
  // the swizzle as it is: two per-lane offsets per operand.  Rows past the group's end come from a row of zeros.
  uint32_t a_off[2], b_off[2];
#pragma unroll
  for (int i = 0; i < 2; i++) {
    const int r = 4 * (wave * kT8Ipw + i) + lane / 16;
    const int chunk = (lane % 16) ^ t8_swz(r);
    a_off[i] = (uint32_t)r * K + chunk * 16;
    b_off[i] = (uint32_t)r * N + chunk * 16;
  }
  static_assert(kT8Ipw == 4, "request i + 2 is request i eight rows further down");
  const uint8_t* const a_base = (const uint8_t*)p.lhs + ((size_t)start * K + k0);
  const uint8_t* const b_base = (const uint8_t*)p.dout + ((size_t)start * N + n0);
  const size_t a_step = (size_t)kT8BM * K, b_step = (size_t)kT8BM * N;
  const uint32_t lds_base = (uint32_t)(uintptr_t)(__attribute__((address_space(3))) uint8_t*)t8_smem;
  auto issue_one = [&](auto full_c, int kt, int buf, int idx) {
    constexpr bool FULL = decltype(full_c)::value;
    const int i = idx % kT8Ipw;
    const bool is_a = idx < kT8Ipw;
    const uint8_t* src = is_a ? a_base + (kt * a_step + (size_t)(i / 2) * 8 * K) + a_off[i % 2]
                              : b_base + (kt * b_step + (size_t)(i / 2) * 8 * N) + b_off[i % 2];
    if constexpr (!FULL) {
      int l = lane;
      asm volatile("" : "+v"(l));
      const int r = 4 * (wave * kT8Ipw + i) + l / 16;
      const uint64_t keep = kt * kT8BM + r < size ? ~0ull : 0ull;
      const uint64_t zero = (uint64_t)(tg_zero_row + (l % 16) * 16);
      src = (const uint8_t*)(((uint64_t)src & keep) | (zero & ~keep));
    }
    dma16_untracked(src, lds_base + buf * kT8Stage + (is_a ? 0 : kT8Operand) + (wave * kT8Ipw + i) * 1024);
  };

  // ---- fragments: lane (group gq, s16) addresses row 32 * gq + s16 / 2 (+ 8, 16, 24) of the stage and the 8 bytes
  // s16 % 2 of the fragment's 16-byte column block c, stored at slot c ^ (s16 / 2) ^ 8 * (gq % 2); fragment f of an operand
  // is block c0 + f with c0 a multiple of 4 (lhs) or 8 (dout), so the step is an XOR of address bits 4 .. 6.
  const int xmask = (s16 / 2) ^ ((gq & 1) << 3);
  const int row_part = (32 * gq + s16 / 2) * kT8Row + (s16 % 2) * 8;
  const int k_base = row_part + (((4 * wk) ^ xmask) << 4);
  const int n_base = row_part + (((8 * wn) ^ xmask) << 4);
  constexpr int RING = 4;
  v8i fk[4], fn[RING];
  auto read_k = [&](int buf, int f) {
    int base = k_base;
    asm volatile("" : "+v"(base));
    tr8_read_frag(fk[f], t8_smem + buf * kT8Stage + (base ^ (16 * f)));
  };
  auto read_n = [&](int buf, int f, int slot) {
    int base = n_base;
    asm volatile("" : "+v"(base));
    tr8_read_frag(fn[slot], t8_smem + buf * kT8Stage + kT8Operand + (base ^ (16 * f)));
  };

  v4f acc[4][8];  // [k fragment][n fragment]
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 8; i++)
#pragma unroll
      for (int r = 0; r < 4; r++) acc[j][i][r] = 0.f;

  // first half of a stage (buffer buf): dout fragments 0 .. 3 from the ring, each slot reloaded with fragment + 4
  auto half_lo = [&](int buf) {
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const int i = t / 4, j = t % 4;
      acc[j][i] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fk[j], fn[i], acc[j][i], 0, DF, 0, 127, 0, 127);
      if (j == 3) read_n(buf, i + RING, i);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  // second half: dout fragments 4 .. 7, lhs fragment by lhs fragment.  RD: the next stage (rd_buf) is prepared behind it.
  // LD: the requests of stage ld_kt go out into ld_buf.
  auto half_hi = [&](auto rd_c, auto ld_c, auto full_c, int rd_buf, int ld_kt, int ld_buf) {
    constexpr bool RD = decltype(rd_c)::value, LD = decltype(ld_c)::value;
#pragma unroll
    for (int t = 0; t < 16; t++) {
      const int j = t / 4, ii = t % 4;
      acc[j][RING + ii] = __builtin_amdgcn_mfma_scale_f32_16x16x128_f8f6f4(fk[j], fn[ii], acc[j][RING + ii], 0, DF, 0, 127, 0, 127);
      if (LD && t % kT8ReqStride == 0 && t / kT8ReqStride < kT8Lps) issue_one(full_c, ld_kt, ld_buf, t / kT8ReqStride);
      if (RD && ii == 3) read_k(rd_buf, j);
      if (RD && j == 3) read_n(rd_buf, ii, ii);
      __builtin_amdgcn_sched_barrier(0);
    }
  };
  using T_ = std::true_type;
  using F_ = std::false_type;

  // Stage kt sits in buffer kt % 2.  After a stage's first half every fragment of it is in registers: the block meets
  // (own reads returned, own requests of stage kt + 1 landed), and during the second half the fragments of stage kt + 1
  // are read from the other buffer while stage kt + 2 is requested into this one.
  const int nk = (size + kT8BM - 1) / kT8BM;
#pragma unroll
  for (int s = 0; s < 2; s++)
#pragma unroll
    for (int i = 0; i < kT8Lps; i++) issue_one(F_{}, min(s, nk - 1), s, i);
  wait_vmcnt<0>();
  __syncthreads();
#pragma unroll
  for (int f = 0; f < RING; f++) read_n(0, f, f);
#pragma unroll
  for (int f = 0; f < 4; f++) read_k(0, f);
  __builtin_amdgcn_s_waitcnt(0xC07F);  // lgkmcnt(0)
  half_lo(0);
  int kt = 0;
  const int nfull = size / kT8BM;  // stages 0 .. nfull-1 hold 128 rows of the group
  for (; kt + 2 < nfull; kt++) {   // steady state: the stage requested is a full one
    const int buf = kt % 2;
    __builtin_amdgcn_s_waitcnt(0xC07F);
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    half_hi(T_{}, T_{}, T_{}, buf ^ 1, kt + 2, buf);
    half_lo(buf ^ 1);
  }
  for (; kt + 1 < nk; kt++) {
    const int buf = kt % 2;
    __builtin_amdgcn_s_waitcnt(0xC07F);
    wait_vmcnt<0>();
    asm volatile("s_barrier" ::: "memory");
    half_hi(T_{}, T_{}, F_{}, buf ^ 1, min(kt + 2, nk - 1), buf);
    half_lo(buf ^ 1);
  }
  __builtin_amdgcn_s_waitcnt(0xC07F);
  half_hi(F_{}, F_{}, F_{}, 0, 0, 0);
  wait_vmcnt<0>();  // no request may still be writing LDS when the block ends
  // (the sums are pinned to this point: their only readers sit behind the branches below)
#pragma unroll
  for (int j = 0; j < 4; j++)
#pragma unroll
    for (int i = 0; i < 8; i++) asm volatile("" : "+v"(acc[j][i]));

  // D[k][n]: the lane holds n = s16 and k = 4 * gq + r of each 16 x 16 tile
  if (!p.out_f32 && !p.existing) {
#pragma unroll
    for (int i = 0; i < 8; i++) {
      const int n = n0 + wn * 128 + i * 16 + s16;
      const float sc = p.n_scale ? p.n_scale[n] : 1.0f;
#pragma unroll
      for (int j = 0; j < 4; j += 2) {
        const auto s0 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(acc[j][i][0] * sc, acc[j][i][1] * sc),
                                                         pack_bf16x2(acc[j + 1][i][0] * sc, acc[j + 1][i][1] * sc), false, false);
        const auto s1 = __builtin_amdgcn_permlane16_swap(pack_bf16x2(acc[j][i][2] * sc, acc[j][i][3] * sc),
                                                         pack_bf16x2(acc[j + 1][i][2] * sc, acc[j + 1][i][3] * sc), false, false);
        const int k = k0 + wk * 64 + (j + (gq & 1)) * 16 + 4 * (gq & ~1);
        *(uint4*)((uint16_t*)p.out + ((size_t)g_local * N + n) * K + k) = make_uint4(s0[0], s1[0], s0[1], s1[1]);
      }
    }
    return;
  }
#pragma unroll
  for (int i = 0; i < 8; i++) {
    const int n = n0 + wn * 128 + i * 16 + s16;
#pragma unroll
    for (int j = 0; j < 4; j++) {
      const int k = k0 + wk * 64 + j * 16 + 4 * gq;
      const size_t off = ((size_t)g_local * N + n) * K + k;
      tgmm_store4(p, off, n, acc[j][i][0], acc[j][i][1], acc[j][i][2], acc[j][i][3]);
    }
  }
}

}  // namespace moe

using namespace moe;

namespace moe {
int prepare_tgmm() { return reserve_lds(tgmm_dl_kernel, kTdLds, lds_flags<TgmmParams>()); }
struct TgmmF8Tag0 {};
struct TgmmF8Tag1 {};
static int prepare_tgmm_f8(int df) {
  return df ? reserve_lds(tgmm_f8_kernel<1>, kT8Lds, lds_flags<TgmmF8Tag1>()) : reserve_lds(tgmm_f8_kernel<0>, kT8Lds, lds_flags<TgmmF8Tag0>());
}
}  // namespace moe

static bool tgmm_f8_takes(long long M, int K, int N, int G_total, int G_local) {
  const long long tiles = (long long)(K / kTdTile) * (N / kTdTile) * G_local;
  return K % kTdTile == 0 && N % kTdTile == 0 && K < (1 << 24) && N < (1 << 24) && M >= 128LL * G_total && tiles >= 128 && tiles <= 0x7fffffffLL;
}

extern "C" int moe_tgmm_fp8_supported(int M, int K, int N, int num_groups_total, int num_groups_local) {
  return M >= 0 && K > 0 && N > 0 && num_groups_total > 0 && num_groups_local > 0 && tgmm_f8_takes(M, K, N, num_groups_total, num_groups_local);
}

extern "C" int moe_tgmm_fp8(const void* lhs, const void* dout, int dout_dtype, const int32_t* group_sizes, int M, int K, int N,
                            int num_groups_total, int num_groups_local, int group_offset, const float* out_row_scale,
                            const void* existing_out, int existing_dtype, int out_dtype, void* out, void* stream) {
  if (!lhs || !dout || !group_sizes || !out) return fail(MOE_ERR_INVALID_ARG, "tgmm_fp8: NULL pointer");
  if (M < 0 || K <= 0 || N <= 0 || num_groups_total <= 0 || num_groups_local <= 0 || group_offset < 0)
    return fail(MOE_ERR_INVALID_ARG, "tgmm_fp8: bad sizes");
  if (dout_dtype != MOE_FP8_E4M3 && dout_dtype != MOE_FP8_E5M2) return fail(MOE_ERR_UNSUPPORTED, "tgmm_fp8: dout_dtype %d", dout_dtype);
  if (out_dtype != MOE_BF16 && out_dtype != MOE_F32) return fail(MOE_ERR_UNSUPPORTED, "tgmm_fp8: out_dtype %d", out_dtype);
  if (!tgmm_f8_takes(M, K, N, num_groups_total, num_groups_local))
    return fail(MOE_ERR_UNSUPPORTED, "tgmm_fp8: needs K and N multiples of 256, 128 rows per group on average and 128 output tiles "
                "(M=%d K=%d N=%d groups=%d); widen the operands to bf16 for moe_tgmm_scaled otherwise", M, K, N, num_groups_total);
  if (((uintptr_t)lhs | (uintptr_t)dout | (uintptr_t)out | (uintptr_t)existing_out) & 15) return fail(MOE_ERR_UNSUPPORTED, "tgmm_fp8: pointers must be 16-byte aligned");
  if (existing_out && existing_dtype != MOE_BF16 && existing_dtype != MOE_F32) return fail(MOE_ERR_UNSUPPORTED, "tgmm_fp8: existing_dtype %d", existing_dtype);
  if (existing_out == out && existing_dtype != out_dtype) return fail(MOE_ERR_INVALID_ARG, "tgmm_fp8: existing_out aliases out with another element type");
  TgmmParams p;
  p.lhs = (const uint16_t*)lhs; p.dout = (const uint16_t*)dout; p.group_sizes = group_sizes; p.out = out;
  p.M = M; p.K = K; p.N = N; p.G_total = num_groups_total; p.G_local = num_groups_local; p.group_offset = group_offset;
  p.out_f32 = out_dtype == MOE_F32;
  p.existing = existing_out; p.existing_f32 = existing_dtype == MOE_F32;
  p.n_scale = out_row_scale;
  const int df = dout_dtype == MOE_FP8_E5M2;
  if (int st = prepare_tgmm_f8(df)) return st;
  const unsigned tiles = (unsigned)((K / kTdTile) * (N / kTdTile) * num_groups_local);
  if (df) tgmm_f8_kernel<1><<<tiles, kTdThreads, kT8Lds, (hipStream_t)stream>>>(p);
  else tgmm_f8_kernel<0><<<tiles, kTdThreads, kT8Lds, (hipStream_t)stream>>>(p);
  return check_launch("tgmm_f8_kernel");
}

extern "C" int moe_tgmm_scaled(const void* lhs, const void* dout, const int32_t* group_sizes, int M, int K, int N,
                               int num_groups_total, int num_groups_local, int group_offset, const float* out_row_scale,
                               const void* existing_out, int existing_dtype, int out_dtype, void* out, void* stream) {
  if (!lhs || !dout || !group_sizes || !out) return fail(MOE_ERR_INVALID_ARG, "tgmm: NULL pointer");
  if (M < 0 || K <= 0 || N <= 0 || num_groups_total <= 0 || num_groups_local <= 0 || group_offset < 0)
    return fail(MOE_ERR_INVALID_ARG, "tgmm: bad sizes");
  if (K % 8 || N % 8) return fail(MOE_ERR_UNSUPPORTED, "tgmm: K and N must be multiples of 8");
  if (out_dtype != MOE_BF16 && out_dtype != MOE_F32) return fail(MOE_ERR_UNSUPPORTED, "tgmm: out_dtype %d", out_dtype);
  if (num_groups_local > 65535 || cdiv(N, kTgBN) > 65535) return fail(MOE_ERR_UNSUPPORTED, "tgmm: grid too large");
  if (((uintptr_t)lhs | (uintptr_t)dout | (uintptr_t)out) & 15) return fail(MOE_ERR_UNSUPPORTED, "tgmm: pointers must be 16-byte aligned");
  TgmmParams p;
  p.lhs = (const uint16_t*)lhs; p.dout = (const uint16_t*)dout; p.group_sizes = group_sizes; p.out = out;
  p.M = M; p.K = K; p.N = N; p.G_total = num_groups_total; p.G_local = num_groups_local; p.group_offset = group_offset;
  p.out_f32 = out_dtype == MOE_F32;
  if (existing_out && existing_dtype != MOE_BF16 && existing_dtype != MOE_F32)
    return fail(MOE_ERR_UNSUPPORTED, "tgmm: existing_dtype %d", existing_dtype);
  if ((uintptr_t)existing_out & 15) return fail(MOE_ERR_UNSUPPORTED, "tgmm: pointers must be 16-byte aligned");
  if (existing_out == out && existing_dtype != out_dtype)
    return fail(MOE_ERR_INVALID_ARG, "tgmm: existing_out aliases out with another element type");
  p.existing = existing_out; p.existing_f32 = existing_dtype == MOE_F32;
  p.n_scale = out_row_scale;
  // groups of 128 rows and more on average take the 256 x 256 tiles when the shape allows it
  const long long tiles = (long long)(K / kTdTile) * (N / kTdTile) * num_groups_local;
  if (K % kTdTile == 0 && N % kTdTile == 0 && K < (1 << 24) && N < (1 << 24) && (long long)M >= 128LL * num_groups_total && tiles >= 128 && tiles <= 0x7fffffffLL) {
    if (int st = prepare_tgmm()) return st;
    tgmm_dl_kernel<<<(unsigned)tiles, kTdThreads, kTdLds, (hipStream_t)stream>>>(p);
    return check_launch("tgmm_dl_kernel");
  }
  dim3 grid(cdiv(K, kTgBK), cdiv(N, kTgBN), num_groups_local);
  tgmm_kernel<<<grid, kTgThreads, 0, (hipStream_t)stream>>>(p);
  return check_launch("tgmm_kernel");
}

extern "C" int moe_tgmm(const void* lhs, const void* dout, const int32_t* group_sizes, int M, int K, int N,
                        int num_groups_total, int num_groups_local, int group_offset, const void* existing_out,
                        int existing_dtype, int out_dtype, void* out, void* stream) {
  return moe_tgmm_scaled(lhs, dout, group_sizes, M, K, N, num_groups_total, num_groups_local, group_offset, nullptr, existing_out,
                         existing_dtype, out_dtype, out, stream);
}
