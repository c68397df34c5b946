// Launcher of the LDS-streamed decode kernel (moe_gmm_wqs.hip): group-128 int4 (WQ_I4) or MXFP4 (WQ_MX4) at decode sizes, weights copied
// global -> LDS by persistent blocks, 16-row tiles.
#pragma once

#include "moe_gmm_common.h"

namespace moe {

bool wqs_takes(int fmt, int K, int N, int G_local, bool glu);
int launch_wqs(int fmt, const WqSkinnyParams& q, bool glu, int num_groups_local, hipStream_t s);
int prepare_wqs();

}  // namespace moe
