// The LDS-streamed 8-bit decode kernels, for a handful of rows per expert: weights copied global -> LDS by persistent
// blocks.
//   gmm_f8d_kernel (moe_gmm_f8d.hip): float8_e4m3 activations with 1 x 128 scales times float8_e4m3 weights with 128 x 128
//                   block scales, the tile's activations resident in registers (K a multiple of 512 up to 7168, 16-row tiles);
//   gmm_f8l_kernel (moe_gmm_f8l.hip): float8_e4m3 or int8 operands with one scale per row and one per output channel
//                   (row_scale_lhs / ch_scale of the parameters: per channel, n contiguous, the experts' rows a multiple of
//                   4 floats apart or shared, 16-byte aligned), the tile's activations copied beside the weights (K any
//                   multiple of 512, tiles of 16, 32 or 64 rows).
#pragma once

#include "moe_gmm_common.h"

namespace moe {

constexpr int kF8dThreads = 512;
constexpr int kF8dRedBytes = 2 * 3 * 8 * kWave * 4;  // partial sums of the waves ksub = 1..3 of both channel tiles
#ifndef MOE_F8D_NT
#define MOE_F8D_NT 1  // weights that are read once stream past the caches
#endif

// 16 bytes per lane, global -> LDS at lds_addr + lane * 16; NT: non-temporal (weights that are read once)
template <bool NT>
__device__ __forceinline__ void f8d_copy(const v4i& rsrc, uint32_t voff, uint32_t lds_addr) {
  uint32_t soff = 0;
  asm volatile("" : "+s"(soff));
  if (NT)
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen nt lds" : : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_addr) : "memory", "m0");
  else
    asm volatile("s_mov_b32 m0, %3\n\ts_nop 0\n\tbuffer_load_dwordx4 %0, %1, %2 offen lds" : : "v"(voff), "s"(rsrc), "s"(soff), "s"(lds_addr) : "memory", "m0");
}

bool f8d_takes(int K, int N, int G_local, bool glu);
int launch_f8d(const SkinnyParams& p, bool glu, int num_groups_local, hipStream_t s);
int prepare_f8d();
bool f8l_takes(int K, int N, int G_local, bool glu, long long lhs_rows);
int launch_f8l(const SkinnyParams& p, bool glu, bool int8, int tile_rows, int num_groups_local, hipStream_t s);  // tiles of 16, 32 or 64 rows
int prepare_f8l();

}  // namespace moe
