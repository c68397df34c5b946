// Grouped matmul for gfx950.
//
//   tile_map_kernel   group_sizes (device) -> list of (group, first row, rows) m-tiles that never
//                     straddle a group boundary, plus zero-fill tiles for non-local / tail rows.
//   gmm_tiled_kernel  LDS-staged, double-buffered MFMA GEMM over that tile list.  Weights are the
//                     MFMA "A" operand (32 output channels per tile), activations the "B" operand
//                     (32 rows), so each lane ends up with 4 consecutive output channels of one
//                     row per accumulator quad and stores 8 bytes.  bf16 x {bf16, int8, int4}
//                     weights run on v_mfma_f32_32x32x16_bf16 (weights are widened to bf16 while
//                     they are copied into LDS), int8 x int8 on v_mfma_i32_32x32x32_i8.
//                     Used for weight-only formats, small problems and K tails.
//   gmm_dls_kernel    the prefill kernel for int8 x int8 and bf16 x bf16 (moe_gmm_dls.hip): persistent blocks, 256 x 256
//                     tiles, operands copied global -> LDS without passing through registers, the requests of a block's
//                     consecutive tiles as one stream.  gmm_dl_kernel (moe_gmm_dl.hip) is its predecessor, kept for the
//                     shapes the stream kernel does not take and for [G, K, N] weights.
//   gmm_dlw_kernel    the same stream for bf16 activations x int8 / int4 / mxfp4 weights (moe_gmm_dlw.hip): raw weight
//                     bytes through LDS, widened by the wave that multiplies them; on 128-row tiles (half of the row tiles
//                     multiplied) for int8 / int4 between the streaming kernel's range and prefill-sized groups.
//   gmm_f8s_kernel    the same stream for block-scaled fp8 (moe_gmm_f8s.hip): scales staged through LDS.
//   gmm_fp8_skinny_kernel  block-scaled fp8 for few rows per expert (decode): no LDS, every wave
//                     streams 16 weight rows through v_mfma_f32_16x16x128_f8f6f4 and applies the
//                     per-128 K-block scales to the f32 partial sums.
//   gmm_fp8_tiled_kernel   block-scaled fp8 for 16 to 128 rows per expert: 128 x 128 tiles through LDS,
//                     v_mfma_f32_32x32x64_f8f6f4, one scaled accumulation per 128-wide K block.
//   gmm_fp8_big_kernel     block-scaled fp8 from 128 rows per expert (prefill): 256 x 256 tiles, one set of
//                     accumulators kept in units of the current K block's scale.
//   gmm_wq_skinny_kernel   the same streaming design for bf16 activations x int8 / int4 / mxfp4 weights,
//                     with K split over the waves of a block.


#include "moe_gmm_common.h"
#include "moe_gmm_wqs.h"
#include "moe_gmm_f8d.h"

#include <cstring>
#include <mutex>

namespace moe {

constexpr int kMapThreads = 256;

__global__ __launch_bounds__(kMapThreads) void tile_map_kernel(
    const int32_t* __restrict__ group_sizes, int G_total, int group_offset, const int32_t* __restrict__ group_offset_dev, int G_local, int M,
    int BM, int zero_fill, int32_t* __restrict__ header, TileInfo* __restrict__ tiles) {
  __shared__ int s_buf[kMapThreads];
  if (group_offset_dev) group_offset = max(*group_offset_dev, 0);  // the shard's first group, held on the device
  build_tile_map<kMapThreads>(group_sizes, G_total, group_offset, G_local, M, BM, zero_fill, header, tiles, s_buf);
}

// The same list for a launch that hands the short last tiles of its groups to the decode kernel: a local group's rows
// are cut into tiles of BM rows as above, but a remainder of at most tail_rows rows becomes 16-row tiles of a second list
// (header[1] = their number, records from tiles + tail_base on).  A 256-row tile costs the persistent kernels the same
// whether it holds 256 rows or 5; the decode kernel streams the expert's weights once per 16 rows, about a quarter of
// that.  Zero-fill tiles (rows of groups held elsewhere, rows past the groups) stay in the first list.
constexpr int kTailTile = 16;
constexpr int kTailRows = 48;  // remainders up to three decode tiles (the two routes cost the same at about 58 rows on the GPT-OSS shape)
__global__ __launch_bounds__(kMapThreads) void tile_map_split_kernel(
    const int32_t* __restrict__ group_sizes, int G_total, int group_offset, const int32_t* __restrict__ group_offset_dev, int G_local, int M,
    int BM, int tail_rows, int tail_base, int zero_fill, int32_t* __restrict__ header, TileInfo* __restrict__ tiles) {
  __shared__ int s_buf[kMapThreads];
  if (group_offset_dev) group_offset = max(*group_offset_dev, 0);
  const int tid = threadIdx.x;
  const int per = (G_total + kMapThreads - 1) / kMapThreads;
  const int g0 = min(tid * per, G_total), g1 = min(g0 + per, G_total);
  long long rows = 0;
  for (int g = g0; g < g1; g++) rows += max(group_sizes[g], 0);
  int total_rows;
  const int row_prefix = block_exclusive_scan<kMapThreads>((int)min(rows, (long long)M), s_buf, &total_rows);
  // a group's clipped extent [s, e) -> (tiles of BM rows, 16-row tail tiles)
  auto split = [&](int s, int e, bool local, int& nmain, int& ntail) {
    const int n = e - s, rem = n % BM;
    nmain = n / BM;
    ntail = 0;
    if (rem > 0) {
      if (local && rem <= tail_rows) ntail = (rem + kTailTile - 1) / kTailTile;
      else nmain += 1;
    }
  };
  int my_main = 0, my_tail = 0;
  {
    long long start = row_prefix;
    for (int g = g0; g < g1; g++) {
      const long long end = start + max(group_sizes[g], 0);
      const int s = (int)min(start, (long long)M), e = (int)min(end, (long long)M);
      const int local = g - group_offset;
      const bool is_local = local >= 0 && local < G_local;
      if (zero_fill || is_local) {
        int a, b;
        split(s, e, is_local, a, b);
        my_main += a;
        my_tail += b;
      }
      start = end;
    }
  }
  int total_main, total_tail;
  const int main_prefix = block_exclusive_scan<kMapThreads>(my_main, s_buf, &total_main);
  const int tail_prefix = block_exclusive_scan<kMapThreads>(my_tail, s_buf, &total_tail);
  {
    long long start = row_prefix;
    int ti = main_prefix, tj = tail_base + tail_prefix;
    for (int g = g0; g < g1; g++) {
      const long long end = start + max(group_sizes[g], 0);
      const int s = (int)min(start, (long long)M), e = (int)min(end, (long long)M);
      const int local = g - group_offset;
      const bool is_local = local >= 0 && local < G_local;
      if (zero_fill || is_local) {
        int a, b;
        split(s, e, is_local, a, b);
        const int kind = is_local ? local : -1;
        for (int t = 0; t < a; t++) tiles[ti++] = TileInfo{kind, s + t * BM, min(BM, e - (s + t * BM)), 0};
        const int tail0 = e - (e - s) % BM;  // (b > 0 only with a remainder that went to the second list)
        for (int t = 0; t < b; t++) tiles[tj++] = TileInfo{kind, tail0 + t * kTailTile, min(kTailTile, e - (tail0 + t * kTailTile)), 0};
      }
      start = end;
    }
  }
  const int covered = min(total_rows, M);
  const int tail = zero_fill ? (M - covered + BM - 1) / BM : 0;
  for (int i = tid; i < tail; i += kMapThreads) tiles[total_main + i] = TileInfo{-1, covered + i * BM, min(BM, M - (covered + i * BM)), 0};
  if (tid == 0) {
    header[0] = total_main + tail;
    header[1] = total_tail;
  }
}

// What the last call on a device mapped, and into which buffer (MOE_GMM_SAME_GROUPS).
struct Mapped {
  const void* ws; const int32_t* gs; const int32_t* offset_dev; int M, G, offset, local, bm, zero_fill;
};
static Mapped g_last_map[kMaxDevices] = {};
static std::mutex g_last_map_lock;

// Records `now` as the device's current tile list; returns whether the list it replaces was the same one.
static bool note_tile_map(const Mapped& now) {
  int dev = 0;
  if (current_device(&dev) != MOE_OK) return false;
  std::lock_guard<std::mutex> hold(g_last_map_lock);
  const bool same = memcmp(&g_last_map[dev], &now, sizeof(Mapped)) == 0;
  g_last_map[dev] = now;
  return same;
}

void note_tile_map_built(const void* workspace, const int32_t* group_sizes, int M, int G_total, int group_offset, int G_local, int bm,
                         int zero_fill) {
  note_tile_map(Mapped{workspace, group_sizes, nullptr, M, G_total, group_offset, G_local, bm, zero_fill ? 1 : 0});
}

void note_group_sizes_rewritten(const int32_t* group_sizes) {
  int dev = 0;
  if (current_device(&dev) != MOE_OK) return;
  std::lock_guard<std::mutex> hold(g_last_map_lock);
  if (g_last_map[dev].gs == group_sizes) g_last_map[dev] = Mapped{};
}

// Tile list of moe_gmm_static_ws: one array per device, held until the process ends.  Its name is a host-side handle,
// not a device address: the address is looked up once per device (scratch_of) and passed to the kernels like any
// caller-supplied workspace.
constexpr size_t kStaticWsBytes = 1u << 20;
static __device__ __align__(256) uint8_t g_static_ws[kStaticWsBytes];

int current_device(int* dev) {
  if (hipGetDevice(dev) != hipSuccess || *dev < 0 || *dev >= kMaxDevices) return fail(MOE_ERR_LAUNCH, "gmm: cannot identify the current device");
  return MOE_OK;
}

int device_cu_count(int* cus) {
  static int cus_of[kMaxDevices] = {};
  int dev = 0;
  if (int st = current_device(&dev)) return st;
  if (cus_of[dev] == 0) {
    int n = 0;
    if (hipDeviceGetAttribute(&n, hipDeviceAttributeMultiprocessorCount, dev) != hipSuccess || n <= 0)
      return fail(MOE_ERR_LAUNCH, "gmm: cannot query the CU count");
    cus_of[dev] = n;
  }
  *cus = cus_of[dev];
  return MOE_OK;
}

static int scratch_of(void** ptr) {
  static void* ptr_of[kMaxDevices] = {};
  int dev = 0;
  if (int st = current_device(&dev)) return st;
  std::lock_guard<std::mutex> hold(g_last_map_lock);
  if (!ptr_of[dev]) {
    void* p = nullptr;
    hipError_t e = hipGetSymbolAddress(&p, HIP_SYMBOL(g_static_ws));
    if (e != hipSuccess || !p) return fail(MOE_ERR_LAUNCH, "gmm: cannot locate the static workspace: %s", hipGetErrorString(e));
    ptr_of[dev] = p;
  }
  *ptr = ptr_of[dev];
  return MOE_OK;
}

// Which kernel family takes a shape (rows per expert on average decide the m-tile) and its m-tile: one decision for the
// tile map and for the launch.
enum TiledKind { K_T64, K_T128, K_T256, K_DL128, K_DL64, K_DLW, K_DLW128 };

static TiledKind pick_tiled_kind(int op, int bsrc, bool glu, int M, int K, int N, int G_total, bool wq_kmajor = false, long long indexed_lhs_rows = 0) {
  // full 256-row tiles for prefill, 64 otherwise; a problem with fewer 256 x 256 tiles than half the CUs of the chip also
  // takes the 64-row tiles, which quadruples its blocks
  const long long tiles_big = (long long)max_tiles_for(M, G_total, 256) * cdiv(N, glu ? 128 : 256);
  const bool dlw_ok = bsrc != BSRC_SAME && dlw_takes(K, N, indexed_lhs_rows, wq_kmajor);
  // 256-row tiles from 128 rows per expert on average, where half of the routed groups no longer fit a 128-row tile (int8
  // x int8 on the Qwen3 shape: 0.106 against 0.126 ms at 112 rows, 0.133 against 0.131 at 128); the weight-only stream
  // kernel from 112: below, the same kernel runs on 128-row tiles (GPT-OSS int4 layer at 104 / 112 rows per expert 0.38 /
  // 0.45 ms on those, 0.44 / 0.44 on 256-row tiles)
  const bool big = (long long)M >= (dlw_ok ? 112LL : 128LL) * G_total && tiles_big >= 128;
  // 32 to 128 rows per expert on average: 128-row tiles; below 32, 64-row tiles.  With routed groups of near-equal size
  // the 64-row tiles are 5-10 % ahead up to 56 rows per expert (GPT-OSS shape, 384 tokens: 0.38 against 0.41 ms for the
  // layer) and collapse at 64, where half of the groups need a second tile (0.57 against 0.41 ms); with skewed routing
  // (Qwen3 shape, Zipf 1.2) the 128-row tiles are ahead from 12 rows per expert on (0.18 against 0.21 ms at 40, 0.20
  // against 0.26 ms at 56).  The weight-only shapes whose direct-to-LDS kernel does not apply follow the same rule:
  // their 256-row register-staged tiles pass the 128-row ones at 128 rows per expert as well.
  const bool mid = !big && (long long)M >= 32LL * G_total && (long long)M < 128LL * G_total;
  const int esz = op == OP_I8 ? 1 : 2;
  // weight-only formats between the streaming kernel's range and the 256-row tiles: the stream kernel on 128-row tiles
  // (half of its row tiles multiplied, nothing requested for the other half) is 10-15 % ahead of the register-staged
  // 128-row tiles for int8 and int4 (GPT-OSS int4 layer at 40 to 96 rows per expert 0.34-0.35 against 0.40-0.42 ms, Qwen3
  // int8 with Zipf routing at 20 to 80 rows 0.14-0.20 against 0.15-0.25 ms), 1-2 % for MXFP4 (0.338-0.352 against
  // 0.344-0.358 ms), and level with the 64-row tiles at 16 to 32 rows
  if (dlw_ok && !big && (long long)M >= 16LL * G_total && (long long)M < 128LL * G_total &&
      (long long)max_tiles_for(M, G_total, 128) * cdiv(N, glu ? 128 : 256) >= 128)
    return K_DLW128;
  if (mid) return K_T128;
  if (big && dlw_ok) return K_DLW;
  // operands that need no conversion stream straight into LDS when every stage is a full row slice
  if (big && bsrc == BSRC_SAME && (K * esz) % 128 == 0) return K_DL128;
  if (big && bsrc == BSRC_SAME && (K * esz) % 64 == 0) return K_DL64;
  if (big) return K_T256;
  return K_T64;
}

static int tiled_kind_bm(TiledKind k) { return k == K_T64 ? 64 : k == K_T128 || k == K_DLW128 ? 128 : 256; }  // (every direct-to-LDS kernel: 256)

static int launch_tiled_kind(TiledKind kind, int op, int bsrc, bool glu, const TiledParams& p, int M, int G_total, hipStream_t s) {
  if (kind == K_DL128) {
    // the stream kernel where its 32-bit offsets reach and K has three stages; the kernel that drains between tiles otherwise
    if (dls_takes(op, p.K, p.N, p.ro.row_idx ? p.ro.lhs_rows : 0)) return launch_dls(op, glu, p, M, G_total, s);
    return launch_dl(op, glu, 128, false, p, M, G_total, s);
  }
  if (kind == K_DL64) return launch_dl(op, glu, 64, false, p, M, G_total, s);
  if (kind == K_DLW || kind == K_DLW128) return launch_dlw(bsrc, glu, kind == K_DLW128, p, M, G_total, s);
  return launch_tiled_bm(op, bsrc, glu, tiled_kind_bm(kind), false, p, M, G_total, s);
}

}  // namespace moe

using namespace moe;

extern "C" {

int moe_gmm_rhs_kn_supported(int M, int K, int N, int num_groups_total) {
  // the 256 x 256 direct-to-LDS kernel is the only one that reads [G, K, N]: whole 64-row stages of 256 channels, groups of
  // 128 rows and more on average, enough tiles for the chip (the rule by which moe_gmm picks that kernel for [G, N, K] too)
  if (M <= 0 || K <= 0 || N <= 0 || num_groups_total <= 0) return 0;
  if (K % 64 != 0 || N % 256 != 0 || (long long)M < 128LL * num_groups_total) return 0;
  return (long long)max_tiles_for(M, num_groups_total, 256) * (N / 256) >= 128 ? 1 : 0;
}

int moe_gmm_lhs_e5m2_supported(int M, int K, int N, int num_groups_total) {
  // the rule by which moe_gmm sends fp8 operands with epilogue scales to the persistent stream kernel
  if (M <= 0 || K <= 0 || N <= 0 || num_groups_total <= 0 || N % 8 != 0) return 0;
  if (!dls_takes(OP_F8, K, N, 0) || (long long)N * K >= (1LL << 31) || (long long)M < 128LL * num_groups_total) return 0;
  return (long long)max_tiles_for(M, num_groups_total, 256) * cdiv(N, 256) >= 128 ? 1 : 0;
}

int moe_gmm_fp8_rhs_kn_supported(int M, int K, int N, int num_groups_total) {
  // fp8 weights as [G, K, N]: the persistent stream kernel reads them through the transposing 8-bit LDS load, 256 channels at a time
  return moe_gmm_lhs_e5m2_supported(M, K, N, num_groups_total) && N % 256 == 0 ? 1 : 0;
}

int moe_gmm_stream_kernel_takes(int lhs_dtype, int rhs_dtype, int K, int N, long long indexed_lhs_rows) {
  // which operand families the persistent stream kernels accept at this K, N (and number of indexed activation rows): the
  // shape half of moe_gmm's dispatch, exposed so that the 32-bit offset guards can be checked on the host
  if (K <= 0 || N <= 0 || indexed_lhs_rows < 0) return 0;
  if (lhs_dtype == MOE_INT8 && rhs_dtype == MOE_INT8) return dls_takes(OP_I8, K, N, indexed_lhs_rows) ? 1 : 0;
  if (lhs_dtype == MOE_BF16 && rhs_dtype == MOE_BF16) return dls_takes(OP_BF16, K, N, indexed_lhs_rows) ? 1 : 0;
  if ((lhs_dtype == MOE_FP8_E4M3 || lhs_dtype == MOE_FP8_E5M2) && rhs_dtype == MOE_FP8_E4M3) return dls_takes(OP_F8, K, N, indexed_lhs_rows) ? 1 : 0;
  if (lhs_dtype == MOE_BF16 && (rhs_dtype == MOE_INT8 || rhs_dtype == MOE_INT4 || rhs_dtype == MOE_MXFP4)) return dlw_takes(K, N, indexed_lhs_rows, false) ? 1 : 0;
  return 0;
}

size_t moe_gmm_workspace_bytes(int M, int num_groups_total) {
  if (M < 0 || num_groups_total <= 0) return 0;
  return 16 + (size_t)max_tiles_for(M, num_groups_total, 16) * sizeof(TileInfo);
}

// How the caller's scale arguments map onto the kernels.
struct ScalePlan {
  // lhs: epilogue scale (one per row, stride 1, or one for the tensor, stride 0) or K-block scales [M, nb]
  const float* lhs_epi; int lhs_epi_stride;
  const float* lhs_bs; int lhs_nb, lhs_qb;
  // rhs: epilogue scales (per channel or per tensor, per expert or shared) or K-major block scales [G, nb, N]
  bool rhs_epi; int rhs_gstride, rhs_nstride;
  bool rhs_bs; int rhs_nb, rhs_qb, rhs_bs_gstride;
};

static int gmm_impl(const moe_gmm_args* a, void* workspace, size_t workspace_bytes, int kernel, int raster, void* stream) {
  if (!a) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL args");
  if (a->struct_size != sizeof(moe_gmm_args)) return fail(MOE_ERR_INVALID_ARG, "gmm: struct_size %zu != %zu", a->struct_size, sizeof(moe_gmm_args));
  if (!a->lhs || !a->rhs || !a->group_sizes || !a->out || !workspace) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL pointer");
  if (a->M < 0 || a->K <= 0 || a->N <= 0 || a->num_groups_total <= 0 || a->num_groups_local <= 0 || a->group_offset < 0)
    return fail(MOE_ERR_INVALID_ARG, "gmm: bad sizes M=%d K=%d N=%d G=%d/%d", a->M, a->K, a->N, a->num_groups_local, a->num_groups_total);
  if (workspace_bytes < moe_gmm_workspace_bytes(a->M, a->num_groups_total)) return fail(MOE_ERR_WORKSPACE, "gmm: workspace too small");
  const bool glu = a->rhs_up != nullptr;
  if (glu && a->act == MOE_ACT_NONE) return fail(MOE_ERR_INVALID_ARG, "gmm: rhs_up needs an activation");
  if (!glu && a->act != MOE_ACT_NONE) return fail(MOE_ERR_INVALID_ARG, "gmm: activation needs rhs_up");
  if (a->act < MOE_ACT_NONE || a->act > MOE_ACT_SILU_CLIP) return fail(MOE_ERR_INVALID_ARG, "gmm: bad act %d", a->act);
  if (a->N % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "gmm: N %% 8 != 0 (N=%d)", a->N);
  if (a->rhs_up_bias && !glu) return fail(MOE_ERR_INVALID_ARG, "gmm: rhs_up_bias needs rhs_up");
  if (a->partial_sum_up && !glu) return fail(MOE_ERR_INVALID_ARG, "gmm: partial_sum_up needs rhs_up");
  if (((uintptr_t)a->partial_sum | (uintptr_t)a->partial_sum_up) & 7) return fail(MOE_ERR_UNSUPPORTED, "gmm: partial sums must be 8-byte aligned");
  if (a->partial_sum == a->out || a->partial_sum_up == a->out) return fail(MOE_ERR_INVALID_ARG, "gmm: partial sums must not alias out");
  if (((uintptr_t)a->rhs_bias | (uintptr_t)a->rhs_up_bias) & 15) return fail(MOE_ERR_UNSUPPORTED, "gmm: bias pointers must be 16-byte aligned");
  if (a->out_dtype != MOE_BF16 && a->out_dtype != MOE_F32) return fail(MOE_ERR_INVALID_ARG, "gmm: out_dtype must be MOE_BF16 or MOE_F32");
  if (a->reserved != 0) return fail(MOE_ERR_INVALID_ARG, "gmm: reserved field must be zero");
  if (a->lhs_row_idx && a->lhs_rows <= 0) return fail(MOE_ERR_INVALID_ARG, "gmm: lhs_row_idx needs lhs_rows");
  if (kernel < MOE_GMM_KERNEL_AUTO || kernel > MOE_GMM_KERNEL_STREAM_NOSPLIT) return fail(MOE_ERR_INVALID_ARG, "gmm: unknown kernel family %d", kernel);
  if (a->M == 0) return MOE_OK;
  const uintptr_t align = (uintptr_t)a->lhs | (uintptr_t)a->rhs | (uintptr_t)a->rhs_up | (uintptr_t)a->out |
                          (uintptr_t)a->rhs_scale | (uintptr_t)a->rhs_up_scale;
  if (align & 15) return fail(MOE_ERR_UNSUPPORTED, "gmm: pointers must be 16-byte aligned");

  hipStream_t s = (hipStream_t)stream;
  const int zero_fill = (a->flags & MOE_GMM_KEEP_OTHER_ROWS) ? 0 : 1;
  int32_t* header = (int32_t*)workspace;
  TileInfo* tiles = (TileInfo*)((uint8_t*)workspace + 16);
  const int M = a->M, K = a->K, N = a->N, G = a->num_groups_total;
  // float8_e5m2 activations (the quantised gradient of the backward, ops.py:583-604) against e4m3 weights: the fp8 path
  // with the other format selector on the MFMA's activation operand; only the persistent stream kernel carries it
  const bool lhs_e5m2 = a->lhs_dtype == MOE_FP8_E5M2;
  const int L = lhs_e5m2 ? MOE_FP8_E4M3 : a->lhs_dtype, R = a->rhs_dtype;
  const bool kmajor = (a->flags & MOE_GMM_RHS_SCALE_KMAJOR) != 0, shared = (a->flags & MOE_GMM_RHS_SCALE_SHARED) != 0;
  const int bn = a->rhs_scale_block_n, rbk = a->rhs_scale_block_k, lbk = a->lhs_scale_block_k;
  auto map_tiles = [&](int bm) {
    // (a device-held offset is part of the caller's promise like group_sizes: the record keeps its address)
    const bool same = note_tile_map(Mapped{workspace, a->group_sizes, a->group_offset_dev, M, G, a->group_offset_dev ? 0 : a->group_offset,
                                           a->num_groups_local, bm, zero_fill ? 1 : 0});
    if (!(same && (a->flags & MOE_GMM_SAME_GROUPS)))
      tile_map_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->group_offset_dev, a->num_groups_local, M, bm, zero_fill, header, tiles);
  };
  // (the split list is recorded under its own tile-height code: a plain list of the same height is another list)
  auto map_tiles_split = [&](int bm, int tail_rows, int tail_base) {
    const bool same = note_tile_map(Mapped{workspace, a->group_sizes, a->group_offset_dev, M, G, a->group_offset_dev ? 0 : a->group_offset,
                                           a->num_groups_local, bm | (tail_rows << 16), zero_fill ? 1 : 0});
    if (!(same && (a->flags & MOE_GMM_SAME_GROUPS)))
      tile_map_split_kernel<<<1, kMapThreads, 0, s>>>(a->group_sizes, G, a->group_offset, a->group_offset_dev, a->num_groups_local, M, bm, tail_rows,
                                                      tail_base, zero_fill, header, tiles);
  };
  RowOpts ro;
  ro.row_idx = a->lhs_row_idx; ro.idx_div = a->lhs_row_idx_div < 1 ? 1 : a->lhs_row_idx_div;
  ro.lhs_rows = a->lhs_row_idx ? a->lhs_rows : M; ro.out_f32 = a->out_dtype == MOE_F32; ro.row_scale = a->out_row_scale;

  const bool rhs_kn = (a->flags & MOE_GMM_RHS_KN) != 0;
  const bool kn_fp8 = rhs_kn && L == MOE_FP8_E4M3 && R == MOE_FP8_E4M3;
  if (rhs_kn && !kn_fp8 && (L != MOE_BF16 || R != MOE_BF16 || glu || !moe_gmm_rhs_kn_supported(M, K, N, G)))
    return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] weights need bf16 x bf16 (or fp8 x fp8) without rhs_up and a shape moe_gmm_rhs_kn_supported accepts");
  if (kn_fp8 && (glu || !moe_gmm_fp8_rhs_kn_supported(M, K, N, G) || a->lhs_row_idx))
    return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] fp8 weights need a shape moe_gmm_fp8_rhs_kn_supported accepts, no rhs_up and no row index");
  const bool quant_pair = (L == MOE_INT8 && R == MOE_INT8) || (L == MOE_FP8_E4M3 && R == MOE_FP8_E4M3);
  ScalePlan sp = {};
  // DeepSeek block scales: fp8 with [M, K/128] x [G, N/128, K/128]
  const bool fp8_blocks = !lhs_e5m2 && L == MOE_FP8_E4M3 && R == MOE_FP8_E4M3 && lbk == 128 && bn == 128 && rbk == 128 && !kmajor && !shared;
  if (quant_pair && !fp8_blocks) {
    if (!a->lhs_scale || !a->rhs_scale || (glu && !a->rhs_up_scale)) return fail(MOE_ERR_INVALID_ARG, "gmm: quantised operands need their scales");
    if (lbk == 0) { sp.lhs_epi = a->lhs_scale; sp.lhs_epi_stride = 1; }
    else if (lbk == MOE_SCALE_PER_TENSOR) { sp.lhs_epi = a->lhs_scale; sp.lhs_epi_stride = 0; }
    else if (lbk > 0 && lbk % 128 == 0) {
      sp.lhs_nb = cdiv(K, lbk); sp.lhs_qb = lbk;
      if (sp.lhs_nb == 1) { sp.lhs_epi = a->lhs_scale; sp.lhs_epi_stride = 1; } else sp.lhs_bs = a->lhs_scale;
    } else return fail(MOE_ERR_UNSUPPORTED, "gmm: lhs_scale_block_k must be 0, MOE_SCALE_PER_TENSOR or a multiple of 128 (got %d)", lbk);
    if (bn != 1 && bn != MOE_SCALE_PER_TENSOR) return fail(MOE_ERR_UNSUPPORTED, "gmm: quantised activations take per-channel or per-tensor weight scales, or fp8 128 x 128 blocks with 1 x 128 activation scales");
    const int nkb = rbk == 0 ? 1 : cdiv(K, rbk);
    if (rbk < 0 || (nkb > 1 && rbk % 128 != 0)) return fail(MOE_ERR_UNSUPPORTED, "gmm: rhs_scale_block_k must be 0 or a multiple of 128 (got %d)", rbk);
    if (nkb == 1) {
      sp.rhs_epi = true;
      sp.rhs_nstride = bn == 1 ? 1 : 0;
      sp.rhs_gstride = shared ? 0 : (bn == 1 ? N : 1);
    } else {
      if (!kmajor || bn != 1) return fail(MOE_ERR_UNSUPPORTED, "gmm: K-block weight scales of quantised activations must be [G, nkb, N] (MOE_GMM_RHS_SCALE_KMAJOR, per channel)");
      sp.rhs_bs = true; sp.rhs_nb = nkb; sp.rhs_qb = rbk; sp.rhs_bs_gstride = shared ? 0 : nkb * N;
    }
    if (K % 16) return fail(MOE_ERR_UNSUPPORTED, "gmm: quantised operands need K %% 16 == 0");
  }

  if (L == MOE_FP8_E4M3 && R == MOE_FP8_E4M3 && !(sp.lhs_bs || sp.rhs_bs)) {
    // fp8 kernels: block scales of the DeepSeek recipe, or (no block scales) per-row x per-channel in the epilogue
    if (fp8_blocks && (!a->lhs_scale || !a->rhs_scale || (glu && !a->rhs_up_scale)))
      return fail(MOE_ERR_INVALID_ARG, "gmm: fp8 block scales missing");
    if (K % 128 != 0) return fail(MOE_ERR_UNSUPPORTED, "gmm: fp8 needs K %% 128 == 0 (K=%d)", K);
    if ((long long)N * K >= (1LL << 31)) return fail(MOE_ERR_UNSUPPORTED, "gmm: fp8 needs N * K < 2^31");
    // Up to 14 rows per expert on average (decode): the streaming kernel with 16-row tiles, one MFMA row tile per
    // wave; a group with more rows simply gets several tiles, which are adjacent in the grid, run at the same time
    // and share the group's weights through L2.  Beyond that the LDS-tiled kernel with 128 x 128 tiles (measured on
    // 256 experts of 7168 x 2048: at 12 rows per expert 1.26 against 1.44 ms, at 16, where half of the experts need a
    // second 16-row tile, 1.66 against 1.43 ms), and from 128 rows per expert on the persistent 256 x 256 stream (with
    // groups of exactly 128 rows 1.94 against 1.70 ms, at 160 rows 2.05 against 2.54 ms; routed groups scatter around
    // their mean, and those over 128 rows cost the 128 x 128 kernel a second tile).
    const bool few_rows = (long long)M <= 16LL * G;
    // decode sizes: the LDS-streamed persistent kernels where they take the shape, one for block-scaled operands, one for
    // per-row x per-channel scales (MOE_GMM_KERNEL_STREAM keeps the register-staged kernel)
#ifndef MOE_F8D_ROWS_HI
#define MOE_F8D_ROWS_HI 14
#endif
    // (without block scales: per-channel weight scales with n contiguous, the experts' rows whole 16-byte units apart)
    const bool f8d_epi = !fp8_blocks && !lhs_e5m2 && !kn_fp8 && sp.rhs_epi && sp.rhs_nstride == 1 && sp.rhs_gstride % 4 == 0 &&
                         ((uintptr_t)a->rhs_scale & 15) == 0 && (!glu || ((uintptr_t)a->rhs_up_scale & 15) == 0);
    const bool f8d_ok = fp8_blocks && kernel == MOE_GMM_KERNEL_AUTO && f8d_takes(K, N, a->num_groups_local, glu);
    const bool f8l_ok = f8d_epi && kernel == MOE_GMM_KERNEL_AUTO && f8l_takes(K, N, a->num_groups_local, glu, ro.lhs_rows);
    // (the second of them also runs on 32- and 64-row tiles, several row tiles per weight segment)
#ifndef MOE_F8L_ROWS_HI
#define MOE_F8L_ROWS_HI 48  // 16-row tiles to 14 rows per expert on average, 32-row tiles to MOE_F8L_ROWS_32, 64-row tiles above
#endif
#ifndef MOE_F8L_ROWS_32
#define MOE_F8L_ROWS_32 24
#endif
    const bool tiled = kernel == MOE_GMM_KERNEL_AUTO ? (long long)M > (f8l_ok ? (long long)MOE_F8L_ROWS_HI : f8d_ok ? (long long)MOE_F8D_ROWS_HI : 14LL) * G
                                                     : kernel != MOE_GMM_KERNEL_STREAM;
    if (kernel > MOE_GMM_KERNEL_BIG) return fail(MOE_ERR_UNSUPPORTED, "gmm: kernel family %d does not take fp8 operands", kernel);
    // prefill-sized groups: the persistent 256 x 256 stream, where it takes the shape
    const bool chip_full = (long long)max_tiles_for(M, G, 256) * cdiv(N, glu ? 128 : 256) >= 128;
    const bool prefill = kernel == MOE_GMM_KERNEL_BIG || (kernel == MOE_GMM_KERNEL_AUTO && (long long)M >= 128LL * G && chip_full);
    // scales in the epilogue only (per row / per tensor x per channel / per tensor): the int8 x int8 problem on another MFMA
    const bool stream_epi = !fp8_blocks && prefill && dls_takes(OP_F8, K, N, ro.row_idx ? ro.lhs_rows : 0);
    if (kn_fp8 && !stream_epi) return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] fp8 weights run on the persistent 256 x 256 kernel only (no K-block scales)");
    if (lhs_e5m2 && !stream_epi)
      return fail(MOE_ERR_UNSUPPORTED, "gmm: float8_e5m2 activations run on the persistent 256 x 256 kernel only (128 rows per group on average, "
                  "K %% 128 == 0, K >= 384, no rhs_up, no K-block scales); widen them to bf16 for other shapes");
    if (stream_epi) {
      if (lhs_e5m2 && glu) return fail(MOE_ERR_UNSUPPORTED, "gmm: float8_e5m2 activations take no rhs_up");
      map_tiles(256);
      TiledParams q = {};
      q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
      q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
      q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
      q.header = header; q.tiles = tiles; q.out = a->out;
      q.M = M; q.K = K; q.N = N; q.act = a->act; q.act_limit = a->act_limit; q.tune = raster; q.ro = ro;
      q.lhs_scale = sp.lhs_epi; q.lhs_scale_stride = sp.lhs_epi_stride;
      q.rhs_scale = a->rhs_scale; q.rhs_up_scale = a->rhs_up_scale;
      q.rhs_scale_gstride = sp.rhs_gstride; q.rhs_scale_nstride = sp.rhs_nstride;
      return launch_dls(OP_F8, glu, q, M, G, s, lhs_e5m2 ? 1 : 0, kn_fp8 ? 1 : 0);
    }
    if (tiled) {
      const bool big = kernel == MOE_GMM_KERNEL_BIG;
      if (big && !fp8_blocks) return fail(MOE_ERR_UNSUPPORTED, "gmm: the 256 x 256 fp8 kernel takes block-scaled operands only");
      const bool stream = fp8_blocks && f8s_takes(K, N, M, ro.row_idx ? ro.lhs_rows : 0) && prefill;
      map_tiles(big || stream ? 256 : 128);
      Fp8TiledParams P = {};
      TiledParams& q = P.base;
      q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
      q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
      q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
      q.header = header; q.tiles = tiles; q.out = a->out;
      q.M = M; q.K = K; q.N = N; q.act = a->act; q.act_limit = a->act_limit; q.tune = raster; q.ro = ro;
      if (fp8_blocks) {
        P.a_scale = a->lhs_scale; P.w_scale = (const float*)a->rhs_scale; P.u_scale = (const float*)a->rhs_up_scale;
      } else {
        q.lhs_scale = sp.lhs_epi; q.lhs_scale_stride = sp.lhs_epi_stride;
        q.rhs_scale = a->rhs_scale; q.rhs_up_scale = a->rhs_up_scale;
        q.rhs_scale_gstride = sp.rhs_gstride; q.rhs_scale_nstride = sp.rhs_nstride;
      }
      if (stream) return launch_f8s(glu, P, M, G, s);
      const bool vec4 = fp8_blocks && (K / 128) % 4 == 0 && ((uintptr_t)a->lhs_scale & 15) == 0;
      return launch_fp8_tiled(big, glu, vec4, P, M, G, s);
    }
    const int bm = f8l_ok ? ((long long)M <= 14LL * G ? 16 : (long long)M <= (long long)MOE_F8L_ROWS_32 * G ? 32 : 64) : few_rows || f8d_ok ? 16 : 64;
    map_tiles(bm);
    SkinnyParams p = {};
    p.lhs = (const uint8_t*)a->lhs; p.rhs = (const uint8_t*)a->rhs; p.rhs_up = (const uint8_t*)a->rhs_up;
    if (fp8_blocks) {
      p.lhs_scale = a->lhs_scale; p.rhs_scale = (const float*)a->rhs_scale; p.rhs_up_scale = (const float*)a->rhs_up_scale;
    } else {
      p.row_scale_lhs = sp.lhs_epi; p.row_scale_lhs_stride = sp.lhs_epi_stride;
      p.ch_scale = (const float*)a->rhs_scale; p.ch_scale_up = (const float*)a->rhs_up_scale;
      p.ch_gstride = sp.rhs_gstride; p.ch_nstride = sp.rhs_nstride;
    }
    p.rhs_bias = a->rhs_bias; p.rhs_up_bias = a->rhs_up_bias;
    p.partial_sum = (const uint16_t*)a->partial_sum; p.partial_sum_up = (const uint16_t*)a->partial_sum_up;
    p.header = header; p.tiles = tiles; p.out = a->out;
    p.M = M; p.K = K; p.N = N; p.act = a->act; p.act_limit = a->act_limit; p.ro = ro;
    p.min_rows = 1; p.max_rows = bm;
    if (f8d_ok) return launch_f8d(p, glu, a->num_groups_local, s);
    if (f8l_ok) return launch_f8l(p, glu, false, bm, a->num_groups_local, s);
    return launch_fp8_skinny(few_rows, p, glu, max_tiles_for(M, G, bm), s);
  }

  TiledParams p = {};
  p.lhs = (const uint8_t*)a->lhs;
  p.rhs = (const uint8_t*)a->rhs; p.rhs_up = (const uint8_t*)a->rhs_up;
  p.rhs_scale = a->rhs_scale; p.rhs_up_scale = a->rhs_up_scale;
  p.rhs_bias = a->rhs_bias; p.rhs_up_bias = a->rhs_up_bias;
  p.partial_sum = (const uint16_t*)a->partial_sum; p.partial_sum_up = (const uint16_t*)a->partial_sum_up;
  p.header = header; p.tiles = tiles; p.out = a->out;
  p.M = M; p.K = K; p.N = N;
  p.act = a->act; p.act_limit = a->act_limit; p.tune = raster; p.i4_group = rbk == 32 ? 32 : 128;
  p.lhs_scale_stride = 1; p.rhs_scale_gstride = N; p.rhs_scale_nstride = 1; p.ro = ro;

  if (quant_pair) {
    // int8 x int8 with any of the layouts above, and fp8 x fp8 with K-block scales on per-channel weights
    const int op = L == MOE_INT8 ? OP_I8 : OP_F8;
    p.lhs_scale = sp.lhs_epi; p.lhs_scale_stride = sp.lhs_epi_stride;
    if (sp.rhs_epi) { p.rhs_scale_gstride = sp.rhs_gstride; p.rhs_scale_nstride = sp.rhs_nstride; }
    else { p.rhs_scale = nullptr; p.rhs_up_scale = nullptr; }
    if (sp.lhs_bs || sp.rhs_bs) {
      p.lhs_bs = sp.lhs_bs; p.lhs_nb = sp.lhs_nb ? sp.lhs_nb : 1; p.lhs_qb = sp.lhs_qb ? sp.lhs_qb : K;
      p.rhs_bs = sp.rhs_bs ? (const float*)a->rhs_scale : nullptr; p.rhs_up_bs = sp.rhs_bs ? (const float*)a->rhs_up_scale : nullptr;
      p.rhs_nb = sp.rhs_bs ? sp.rhs_nb : 1; p.rhs_qb = sp.rhs_bs ? sp.rhs_qb : K; p.rhs_bs_gstride = sp.rhs_bs_gstride;
      if (K % 128) return fail(MOE_ERR_UNSUPPORTED, "gmm: K-block scales need K %% 128 == 0 (K=%d)", K);
      if (kernel != MOE_GMM_KERNEL_AUTO && kernel != MOE_GMM_KERNEL_TILED) return fail(MOE_ERR_UNSUPPORTED, "gmm: K-block scales run on the LDS-tiled kernel");
      const int bm = (long long)M >= 32LL * G ? 128 : 64;
      map_tiles(bm);
      return launch_tiled_bm(op, BSRC_SAME, glu, bm, true, p, M, G, s);
    }
    // (fp8 without block scales was taken by the fp8 kernels above)
    if (kernel == MOE_GMM_KERNEL_BIG) {  // the register-staged kernel on 256 x 256 tiles
      map_tiles(256);
      return launch_tiled_bm(op, BSRC_SAME, glu, 256, false, p, M, G, s);
    }
    if (kernel == MOE_GMM_KERNEL_DL64) {
      if (K % 64) return fail(MOE_ERR_UNSUPPORTED, "gmm: 64-byte stages need K %% 64 == 0");
      map_tiles(256);
      return launch_dl(op, glu, 64, false, p, M, G, s);
    }
    if (kernel == MOE_GMM_KERNEL_STREAM || kernel == MOE_GMM_KERNEL_STREAM_NOSPLIT) return fail(MOE_ERR_UNSUPPORTED, "gmm: no streaming kernel for int8 x int8");
    // int8 x int8 at decode sizes (16-row tiles up to 14 rows per expert on average, 32- and 64-row tiles above): the LDS-streamed persistent kernel where it takes the
    // shape (per-channel weight scales with n contiguous, the experts' rows whole 16-byte units apart)
    if (op == OP_I8 && kernel == MOE_GMM_KERNEL_AUTO && (long long)M <= (long long)MOE_F8L_ROWS_HI * G && sp.rhs_epi && sp.rhs_nstride == 1 && sp.rhs_gstride % 4 == 0 &&
        ((uintptr_t)a->rhs_scale & 15) == 0 && (!glu || ((uintptr_t)a->rhs_up_scale & 15) == 0) &&
        f8l_takes(K, N, a->num_groups_local, glu, ro.lhs_rows)) {
      const int bm = (long long)M <= 14LL * G ? 16 : (long long)M <= (long long)MOE_F8L_ROWS_32 * G ? 32 : 64;
      map_tiles(bm);
      SkinnyParams q = {};
      q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
      q.row_scale_lhs = sp.lhs_epi; q.row_scale_lhs_stride = sp.lhs_epi_stride;
      q.ch_scale = (const float*)a->rhs_scale; q.ch_scale_up = (const float*)a->rhs_up_scale;
      q.ch_gstride = sp.rhs_gstride; q.ch_nstride = sp.rhs_nstride;
      q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
      q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
      q.header = header; q.tiles = tiles; q.out = a->out;
      q.M = M; q.K = K; q.N = N; q.act = a->act; q.act_limit = a->act_limit; q.ro = ro;
      q.min_rows = 1; q.max_rows = bm;
      return launch_f8l(q, glu, true, bm, a->num_groups_local, s);
    }
    TiledKind kind = pick_tiled_kind(op, BSRC_SAME, glu, M, K, N, G);
    if (kernel == MOE_GMM_KERNEL_TILED && (kind == K_DL128 || kind == K_DL64)) kind = K_T256;
    map_tiles(tiled_kind_bm(kind));
    return launch_tiled_kind(kind, op, BSRC_SAME, glu, p, M, G, s);
  }

  enum { V_NONE, V_BF16, V_W8, V_W4, V_MX4 } variant = V_NONE;
  bool wq_kmajor = false;
  if (L == MOE_BF16 && R == MOE_BF16) {
    if (K % 8) return fail(MOE_ERR_UNSUPPORTED, "gmm: bf16 needs K %% 8 == 0");
    p.rhs_scale = p.rhs_up_scale = nullptr;
    variant = V_BF16;
  } else if (L == MOE_BF16 && R == MOE_INT8) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale)) return fail(MOE_ERR_INVALID_ARG, "gmm: int8 weights need scales");
    if (K % 16) return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 weights need K %% 16 == 0");
    if (rbk == 0 && !kmajor && (bn == 1 || bn == MOE_SCALE_PER_TENSOR)) {
      p.rhs_scale_nstride = bn == 1 ? 1 : 0;
      p.rhs_scale_gstride = shared ? 0 : (bn == 1 ? N : 1);
    } else if (kmajor && bn == 1 && rbk > 0 && rbk % 16 == 0) {
      wq_kmajor = true;
      p.rhs_qb = rbk; p.rhs_nb = cdiv(K, rbk); p.rhs_scale_gstride = shared ? 0 : p.rhs_nb * N;
    } else {
      return fail(MOE_ERR_UNSUPPORTED, "gmm: int8 weights need f32 scales per channel / per tensor over all of K, or [G, nkb, N] with MOE_GMM_RHS_SCALE_KMAJOR");
    }
    variant = V_W8;
  } else if (L == MOE_BF16 && R == MOE_INT4) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale)) return fail(MOE_ERR_INVALID_ARG, "gmm: int4 weights need scales");
    if (K % 32) return fail(MOE_ERR_UNSUPPORTED, "gmm: int4 weights need K %% 32 == 0");
    if (kmajor && bn == 1 && rbk > 0 && rbk % 32 == 0) {
      wq_kmajor = true;
      p.rhs_qb = rbk; p.rhs_nb = cdiv(K, rbk); p.rhs_scale_gstride = shared ? 0 : p.rhs_nb * N;
    } else if (kmajor || shared || bn != 1 || (rbk != 128 && rbk != 32)) {
      return fail(MOE_ERR_UNSUPPORTED, "gmm: int4 weights need bf16 group scales [G, N, ceil(K/group)] with group 128 or 32, or f32 [G, nkb, N] with MOE_GMM_RHS_SCALE_KMAJOR");
    }
    variant = V_W4;
  } else if (L == MOE_BF16 && R == MOE_MXFP4) {
    if (!a->rhs_scale || (glu && !a->rhs_up_scale) || bn != 1 || rbk != 32 || kmajor || shared)
      return fail(MOE_ERR_UNSUPPORTED, "gmm: mxfp4 weights need e8m0 block-32 scales [G, N, K/32]");
    if (K % 32) return fail(MOE_ERR_UNSUPPORTED, "gmm: mxfp4 weights need K %% 32 == 0");
    variant = V_MX4;
  } else {
    return fail(MOE_ERR_UNSUPPORTED, "gmm: lhs_dtype %d x rhs_dtype %d", L, R);
  }
  p.wq_kmajor = wq_kmajor ? 1 : 0;

  if (a->flags & MOE_GMM_RHS_KN) {
    if (variant != V_BF16 || glu || !moe_gmm_rhs_kn_supported(M, K, N, G))
      return fail(MOE_ERR_UNSUPPORTED, "gmm: [G, K, N] weights need bf16 x bf16 without rhs_up and a shape moe_gmm_rhs_kn_supported accepts");
    map_tiles(256);
    return launch_dl(OP_BF16, false, 128, true, p, M, G, s);
  }
  const int bsrc = variant == V_BF16 ? BSRC_SAME : variant == V_W8 ? BSRC_I8 : variant == V_W4 ? BSRC_I4 : BSRC_MX4;
  const bool int4_g128 = variant == V_W4 && rbk != 32;
  // rows per expert up to which the streaming kernel beats the register-staged one (layer times on the GPT-OSS shape with
  // uniform routing): 32 for group-128 int4 (0.36 / 0.42 ms at 32 / 40 rows against 0.36 / 0.36 ms on the stream kernel's 128-row
  // tiles), 32 for MXFP4 (0.31 /
  // 0.38 against 0.34 / 0.35 ms).  Int8 and group-32 int4: 16, between the crossover with equal groups (30 on the Qwen3
  // shape, where both kernels then wait for the weights of all experts) and the one with Zipf-skewed routing (10: few
  // experts hold most rows and the tiled kernel converts their weights once per 128 rows instead of once per 32).
  // Group-128 int4 on shapes the LDS-streamed kernel takes: 48 (GPT-OSS shape, layer times at 40 / 48 / 64 rows per expert:
  // 0.28 / 0.32 / 0.38 ms against 0.33 ms on the 128-row tiles throughout).
  const int wq_fmt = variant == V_W8 ? WQ_I8 : variant == V_MX4 ? WQ_MX4 : (rbk == 32 ? WQ_I4G32 : WQ_I4);
  // (its copies move 16 bytes per lane; every pointer of the call has been checked for 16-byte alignment above)
  const bool wqs_ok = (int4_g128 || variant == V_MX4) && kernel == MOE_GMM_KERNEL_AUTO && wqs_takes(wq_fmt, K, N, a->num_groups_local, glu);
#ifndef MOE_WQS_MX_ROWS_HI
#define MOE_WQS_MX_ROWS_HI 48
#endif
  const long long stream_rows_hi = int4_g128 ? (wqs_ok ? 48 : 32) : variant == V_MX4 ? (wqs_ok ? MOE_WQS_MX_ROWS_HI : 32) : 16;
  // few rows per expert with weight-only int8 / int4: the streaming kernel (decode is bound by weight bytes)
  // (a lane of that kernel owns 32 consecutive k values, so K must be a multiple of 32; other K take the tiled kernel)
  const bool stream_ok = variant != V_BF16 && !wq_kmajor && K % 32 == 0 && (long long)N * K < (1LL << 31);
  const bool want_stream = kernel == MOE_GMM_KERNEL_STREAM || kernel == MOE_GMM_KERNEL_STREAM_NOSPLIT ||
                           (kernel == MOE_GMM_KERNEL_AUTO && (long long)M <= stream_rows_hi * G);
  if ((kernel == MOE_GMM_KERNEL_STREAM || kernel == MOE_GMM_KERNEL_STREAM_NOSPLIT) && !stream_ok)
    return fail(MOE_ERR_UNSUPPORTED, "gmm: the streaming kernel takes weight-only formats with K %% 32 == 0, N * K < 2^31 and no K-major scales");
  if (want_stream && stream_ok) {
    // 16-row tiles up to 16 rows per expert on average, 32-row tiles above; group-128 int4 keeps the 16-row tiles over the
    // whole range (its 32-row variant runs at two waves per SIMD: 0.36 against 0.44 ms on the GPT-OSS shape at 256 tokens)
    // and stays on this kernel up to 32 rows per expert
    const bool one = int4_g128 || wqs_ok || (long long)M <= 16LL * G;
    const int bm = one ? 16 : 32;
    map_tiles(bm);
    WqSkinnyParams q = {};
    q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
    q.rhs_scale = a->rhs_scale; q.rhs_up_scale = a->rhs_up_scale;
    q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
    q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
    q.header = header; q.tiles = tiles; q.out = a->out;
    q.M = M; q.K = K; q.N = N; q.act = a->act; q.act_limit = a->act_limit; q.ro = ro;
    q.ch_gstride = p.rhs_scale_gstride; q.ch_nstride = p.rhs_scale_nstride;
    const int fmt = wq_fmt;
    // group-128 int4: the LDS-streamed persistent kernel where it takes the shape (MOE_GMM_KERNEL_STREAM keeps the
    // register-staged one)
    if (wqs_ok) return launch_wqs(fmt, q, glu, a->num_groups_local, s);
    return launch_wq(fmt, one, q, glu, max_tiles_for(M, G, bm), kernel == MOE_GMM_KERNEL_STREAM_NOSPLIT ? 1 : 0, s);
  }
  const int op = OP_BF16;
  if (kernel == MOE_GMM_KERNEL_DL64) {
    if (variant != V_BF16 || (K * 2) % 64) return fail(MOE_ERR_UNSUPPORTED, "gmm: 64-byte stages need bf16 x bf16 with K %% 32 == 0");
    map_tiles(256);
    return launch_dl(op, glu, 64, false, p, M, G, s);
  }
  TiledKind kind = kernel == MOE_GMM_KERNEL_BIG ? K_T256 : pick_tiled_kind(op, bsrc, glu, M, K, N, G, wq_kmajor, a->lhs_row_idx ? ro.lhs_rows : 0);
  if (kernel == MOE_GMM_KERNEL_TILED && (kind == K_DL128 || kind == K_DL64 || kind == K_DLW || kind == K_DLW128)) kind = kind == K_DLW128 ? K_T128 : K_T256;
  // 4-bit weights on the persistent kernel: a group's last rows, when they are few, go to the decode kernel in a second
  // launch (16-row tiles of a second list) instead of filling a corner of one more 128- or 256-row tile
  const bool split_tails = (kind == K_DLW || kind == K_DLW128) && kernel == MOE_GMM_KERNEL_AUTO && (bsrc == BSRC_I4 || bsrc == BSRC_MX4) && !wq_kmajor &&
                           wqs_takes(wq_fmt, K, N, a->num_groups_local, glu);
  if (split_tails) {
    const int bm = tiled_kind_bm(kind);
    const int tail_base = max_tiles_for(M, G, bm);  // past every record the first list can hold
    if ((size_t)16 + ((size_t)tail_base + (size_t)G * cdiv(kTailRows, kTailTile)) * sizeof(TileInfo) <= workspace_bytes) {
      map_tiles_split(bm, kTailRows, tail_base);
      if (int st = launch_tiled_kind(kind, op, bsrc, glu, p, M, G, s)) return st;
      WqSkinnyParams q = {};
      q.lhs = (const uint8_t*)a->lhs; q.rhs = (const uint8_t*)a->rhs; q.rhs_up = (const uint8_t*)a->rhs_up;
      q.rhs_scale = a->rhs_scale; q.rhs_up_scale = a->rhs_up_scale;
      q.rhs_bias = a->rhs_bias; q.rhs_up_bias = a->rhs_up_bias;
      q.partial_sum = (const uint16_t*)a->partial_sum; q.partial_sum_up = (const uint16_t*)a->partial_sum_up;
      q.header = header + 1; q.tiles = tiles + tail_base; q.out = a->out;
      q.M = M; q.K = K; q.N = N; q.act = a->act; q.act_limit = a->act_limit; q.ro = ro;
      return launch_wqs(wq_fmt, q, glu, a->num_groups_local, s);
    }
  }
  map_tiles(tiled_kind_bm(kind));
  return launch_tiled_kind(kind, op, bsrc, glu, p, M, G, s);
}

int moe_gmm(const moe_gmm_args* a, void* stream) {
  if (!a) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL args");
  return gmm_impl(a, a->workspace, a->workspace_bytes, MOE_GMM_KERNEL_AUTO, 0, stream);
}

size_t moe_gmm_static_ws_capacity(void) { return kStaticWsBytes; }

int moe_gmm_static_ws(const moe_gmm_args* a, void* stream) {
  if (!a) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL args");
  if (a->M < 0 || a->num_groups_total <= 0 || moe_gmm_workspace_bytes(a->M, a->num_groups_total) > kStaticWsBytes)
    return fail(MOE_ERR_WORKSPACE, "gmm: M = %d rows in %d groups need a tile list of more than the %zu bytes of the static workspace", a->M,
                a->num_groups_total, kStaticWsBytes);
  void* ws = nullptr;
  if (int st = scratch_of(&ws)) return st;
  return gmm_impl(a, ws, kStaticWsBytes, MOE_GMM_KERNEL_AUTO, 0, stream);
}

int moe_init(void) {
  int cus = 0;
  void* ws = nullptr;
  if (int st = device_cu_count(&cus)) return st;
  if (int st = scratch_of(&ws)) return st;
  if (int st = prepare_tiled()) return st;
  if (int st = prepare_dl()) return st;
  if (int st = prepare_dlw()) return st;
  if (int st = prepare_dls()) return st;
  if (int st = prepare_wqs()) return st;
  if (int st = prepare_f8d()) return st;
  if (int st = prepare_f8l()) return st;
  if (int st = prepare_tgmm()) return st;
  if (int st = prepare_f8s()) return st;
  return prepare_fp8();
}

int moe_gmm_tuned(const moe_gmm_args* a, int kernel, int raster, void* stream) {
  if (!a) return fail(MOE_ERR_INVALID_ARG, "gmm: NULL args");
  return gmm_impl(a, a->workspace, a->workspace_bytes, kernel, raster < 0 ? 0 : raster, stream);
}

}  // extern "C"
