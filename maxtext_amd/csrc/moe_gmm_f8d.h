// Launcher of the LDS-streamed fp8 decode kernel (moe_gmm_f8d.hip): float8_e4m3 activations with 1 x 128 scales times
// float8_e4m3 weights with 128 x 128 block scales at a handful of rows per expert, weights copied global -> LDS by
// persistent blocks, 16-row tiles.
#pragma once

#include "moe_gmm_common.h"

namespace moe {

bool f8d_takes(int K, int N, int G_local, bool glu);
int launch_f8d(const SkinnyParams& p, bool glu, int num_groups_local, hipStream_t s);
int prepare_f8d();

}  // namespace moe
