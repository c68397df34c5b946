// Launcher of the LDS-streamed 8-bit decode kernel (moe_gmm_f8d.hip): float8_e4m3 activations times float8_e4m3 weights with
// 1 x 128 and 128 x 128 block scales, or float8_e4m3 / int8 operands with one scale per row and one per output channel, at
// a handful of rows per expert; weights copied global -> LDS by persistent blocks, 16-row tiles.
#pragma once

#include "moe_gmm_common.h"

namespace moe {

bool f8d_takes(int K, int N, int G_local, bool glu);
// kind: 0 = fp8 with block scales, 1 = fp8, 2 = int8 with per-row x per-channel scales (row_scale_lhs / ch_scale of the parameters)
int launch_f8d(const SkinnyParams& p, bool glu, int kind, int num_groups_local, hipStream_t s);
// The same operands (kinds 1 and 2) with rows of any multiple of 512 values: the activations travel beside the weights.
bool f8l_takes(int K, int N, int G_local, bool glu, long long lhs_rows);
int launch_f8l(const SkinnyParams& p, bool glu, bool int8, int num_groups_local, hipStream_t s);
int prepare_f8d();

}  // namespace moe
