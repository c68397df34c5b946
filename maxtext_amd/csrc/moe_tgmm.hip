// Transposed grouped matmul (weight gradient): out[g][n][k] = sum over the rows m of group g of
// dout[m][n] * lhs[m][k].  Both operands are row-major with the contraction index m as the ROW index, the
// opposite of what an MFMA fragment wants (8 consecutive contraction values per lane).  The tiles are staged
// in LDS as they are and read back with ds_read_b64_tr_b16, gfx950's transposing LDS load: within 16 lanes,
// lane L receives the L-th 16-bit column of a 4 x 16 block whose rows are addressed by lanes 0-3, 4-7, ...
// Two such reads give a lane its 8 contraction values.  lhs is the MFMA "A" operand (32 k channels), dout
// the "B" operand (32 n channels), so a lane ends up with 4 consecutive k of one n: contiguous stores into
// the [G, N, K] weight layout.

#include "moe_common.h"

namespace moe {

typedef short v4s __attribute__((ext_vector_type(4)));
typedef __attribute__((address_space(3))) v4s* lds_v4s_t;

constexpr int kTgBN = 128, kTgBK = 128, kTgBM = 32;  // output tile [BN x BK], contraction chunk BM rows
constexpr int kTgThreads = 256;
constexpr int kTgLdr = kTgBN * 2 + 32;  // LDS row stride in bytes (the pad spreads the 4 rows of a transposing read over the banks)

struct TgmmParams {
  const uint16_t* lhs;   // [M, K] bf16
  const uint16_t* dout;  // [M, N] bf16
  const int32_t* group_sizes;
  void* out;  // [G_local, N, K] bf16 or f32
  int M, K, N;
  int G_total, G_local, group_offset;
  int out_f32;
};

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
  for (int i = tid; i < g; i += kTgThreads) part += max(p.group_sizes[i], 0);
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
        const float v0 = acc[j][i][4 * q], v1 = acc[j][i][4 * q + 1], v2 = acc[j][i][4 * q + 2], v3 = acc[j][i][4 * q + 3];
        if (p.out_f32)
          *(float4*)((float*)p.out + off) = make_float4(v0, v1, v2, v3);
        else
          *(uint2*)((uint16_t*)p.out + off) = make_uint2(pack_bf16x2(v0, v1), pack_bf16x2(v2, v3));
      }
  }
}

}  // namespace moe

using namespace moe;

extern "C" int moe_tgmm(const void* lhs, const void* dout, const int32_t* group_sizes, int M, int K, int N,
                        int num_groups_total, int num_groups_local, int group_offset, int out_dtype, void* out,
                        void* stream) {
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
  dim3 grid(cdiv(K, kTgBK), cdiv(N, kTgBN), num_groups_local);
  tgmm_kernel<<<grid, kTgThreads, 0, (hipStream_t)stream>>>(p);
  return check_launch("tgmm_kernel");
}
