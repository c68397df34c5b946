// Launchers of the LDS-streamed 8-bit decode kernels (moe_gmm_f8d.hip), for a handful of rows per expert: weights copied
// global -> LDS by persistent blocks, 16-row tiles.
//   gmm_f8d_kernel: float8_e4m3 activations with 1 x 128 scales times float8_e4m3 weights with 128 x 128 block scales, the
//                   tile's activations resident in registers (K a multiple of 512 up to 7168);
//   gmm_f8l_kernel: float8_e4m3 or int8 operands with one scale per row and one per output channel (row_scale_lhs / ch_scale
//                   of the parameters: per channel, n contiguous, the experts' rows a multiple of 4 floats apart or
//                   shared, 16-byte aligned), the tile's activations copied beside the weights (K any multiple of 512).
#pragma once

#include "moe_gmm_common.h"

namespace moe {

bool f8d_takes(int K, int N, int G_local, bool glu);
int launch_f8d(const SkinnyParams& p, bool glu, int num_groups_local, hipStream_t s);
bool f8l_takes(int K, int N, int G_local, bool glu, long long lhs_rows);
int launch_f8l(const SkinnyParams& p, bool glu, bool int8, int tile_rows, int num_groups_local, hipStream_t s);  // tiles of 16 or 32 rows
int prepare_f8d();  // (both kernels)

}  // namespace moe
