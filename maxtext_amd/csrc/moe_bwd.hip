// Gradient preparation of the quantised backward pass: the incoming gradient times the scale of the axis the product
// contracts away (_bwd_prepare_inputs, kernels/megablox/ops.py:530-580), optionally quantised to float8_e5m2 per row or
// per column (_bwd_quantize_gradient, ops.py:583-604).  The e5m2 values are written as bf16, in which they are exact, so
// that both gradient products can run on the bf16 kernels, or as float8_e5m2 bytes for the fp8 MFMA (e5m2 gradient x
// e4m3 weights).

#include "moe_common.h"

namespace moe {

constexpr float kE5m2Max = 57344.0f;

// absmax / 57344 rounded once (the quotient is formed in f64: one ulp of the scale moves values across e5m2 rounding
// boundaries)
__device__ __forceinline__ float e5m2_scale(float amax) { return (float)((double)amax / (double)kE5m2Max); }

// x / scale rounded to the float8_e5m2 grid, to nearest even (2 mantissa bits; subnormals are multiples of 2^-16); a
// zero scale gives zero
__device__ __forceinline__ float to_e5m2_grid(float x, float scale) {
  if (scale == 0.f) return 0.f;
  const float q = x / scale;
  const float a = fabsf(q);
  if (!(a < INFINITY)) return q;  // inf / nan as they are
  float r;
  if (a < 6.103515625e-05f) {  // below 2^-14
    r = rintf(a * 65536.0f) * (1.0f / 65536.0f);
  } else {
    uint32_t b = __float_as_uint(a);
    b += 0x000FFFFFu + ((b >> 21) & 1u);
    b &= 0xFFE00000u;
    r = __uint_as_float(b);
    if (r > kE5m2Max) r = INFINITY;  // what the cast gives beyond the largest finite value
  }
  return copysignf(r, q);
}

// A value on the e5m2 grid as its float8_e5m2 byte: the upper byte of the IEEE half of the same value (e5m2 is a half
// with 8 mantissa bits dropped; every grid value, inf and nan included, converts exactly).
__device__ __forceinline__ uint32_t e5m2_byte(float on_grid) {
  const _Float16 h = (_Float16)on_grid;
  return (uint32_t)(__builtin_bit_cast(uint16_t, h) >> 8);
}

// What the quantiser needs of a scale: the scale, its reciprocal rounded once, and whether every value takes the exact
// route (a zero or non-finite scale).
struct E5m2Scale {
  float s, inv;
  bool exact;
};
__device__ __forceinline__ E5m2Scale e5m2_prepare(float amax) {
  E5m2Scale r;
  r.s = e5m2_scale(amax);
  r.exact = !(r.s > 0.f && r.s < INFINITY);
  r.inv = 1.0f / r.s;
  return r;
}

// float8_e5m2 bytes of x0 / s0 and x1 / s1 (bits 0-7 and 8-15), equal to e5m2_byte(to_e5m2_grid(x, s)) bit for bit at a
// fraction of its instructions: the quotient is formed as x * (1 / s), which lies within 2 ulps of x / s, and rounded by
// v_cvt_pk_bf8_f32 (nearest even, OCP e5m2 on gfx950); only a product within 4 ulps of a tie of the grid, in the grid's
// subnormal range (below 2^-14, zero excepted) or not finite goes through the exact division and the rounding spelled
// out above, lane by lane.
__device__ __forceinline__ uint32_t e5m2_bytes2(float x0, float x1, const E5m2Scale& a, const E5m2Scale& b) {
  const float q0 = x0 * a.inv, q1 = x1 * b.inv;
  uint32_t pk = (uint32_t)__builtin_amdgcn_cvt_pk_bf8_f32(q0, q1, 0, false) & 0xffffu;
  const uint32_t b0 = __float_as_uint(q0) & 0x7fffffffu, b1 = __float_as_uint(q1) & 0x7fffffffu;
  const bool n0 = a.exact || ((b0 & 0x1fffffu) - 0xffffcu) <= 8u || (b0 - 1u) < 0x387fffffu || b0 >= 0x7f800000u;
  const bool n1 = b.exact || ((b1 & 0x1fffffu) - 0xffffcu) <= 8u || (b1 - 1u) < 0x387fffffu || b1 >= 0x7f800000u;
  if (n0) pk = (pk & 0xff00u) | e5m2_byte(to_e5m2_grid(x0, a.s));
  if (n1) pk = (pk & 0x00ffu) | (e5m2_byte(to_e5m2_grid(x1, b.s)) << 8);
  return pk;
}

// the value of a float8_e5m2 byte (the half whose upper byte it is)
__device__ __forceinline__ float e5m2_value(uint32_t byte) { return (float)__builtin_bit_cast(_Float16, (uint16_t)(byte << 8)); }

// 8 quantised results of one lane from their bytes (two per entry of pk): bf16 values or the bytes themselves
template <bool BYTES>
__device__ __forceinline__ void store8_e5m2(void* out, size_t idx, const uint32_t (&pk)[4]) {
  if (BYTES) {
    ((uint2*)out)[idx] = make_uint2(pk[0] | (pk[1] << 16), pk[2] | (pk[3] << 16));
  } else {
    uint32_t w[4];
#pragma unroll
    for (int e = 0; e < 4; e++) w[e] = pack_bf16x2(e5m2_value(pk[e] & 0xffu), e5m2_value(pk[e] >> 8));
    ((uint4*)out)[idx] = make_uint4(w[0], w[1], w[2], w[3]);
  }
}

// bf16(a), bf16(b) as floats: one v_cvt_pk_bf16_f32 for the pair
__device__ __forceinline__ void round_bf16_pair(float a, float b, float& ra, float& rb) {
  const uint32_t p = pack_bf16x2(a, b);
  ra = __uint_as_float(p << 16);
  rb = __uint_as_float(p & 0xffff0000u);
}

// 8 results of one lane: bf16 (16 bytes at `out` + 16 * idx) or, BYTES, float8_e5m2 (8 bytes at `out` + 8 * idx)
template <bool BYTES>
__device__ __forceinline__ void store8(void* out, size_t idx, const float (&o)[8]) {
  if (BYTES) {
    uint32_t lo = 0, hi = 0;
#pragma unroll
    for (int e = 0; e < 4; e++) {
      lo |= e5m2_byte(o[e]) << (8 * e);
      hi |= e5m2_byte(o[4 + e]) << (8 * e);
    }
    ((uint2*)out)[idx] = make_uint2(lo, hi);
  } else {
    ((uint4*)out)[idx] = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
  }
}

// expert of row m as the reference's backward sees it: the number of group ends <= m, taken relative to the first
// local group and clamped to the local range (rows of other shards and rows past the last group take the nearest
// local expert: their gradient rows do not reach the result)
__device__ __forceinline__ int local_group_of(const int* ends, int G_total, int m, int group_offset, int G_local) {
  int lo = 0, hi = G_total;  // first index with ends[i] > m
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (ends[mid] > m) hi = mid;
    else lo = mid + 1;
  }
  return min(max(lo - group_offset, 0), G_local - 1);
}

constexpr int kBwdThreads = 256;
constexpr int kBwdMaxChunks = 8;  // 8 bf16 per lane and chunk: rows of up to 16384 values
constexpr int kBwdMaxGroups = 1024;

// ends[g] = rows up to and including group g (negative sizes count as empty), built by the whole block: every thread
// loads up to four sizes at once and the partial sums meet in a scan, so a block pays one memory latency for the table
// instead of one per group.  Ends with a barrier.
__device__ __forceinline__ void block_group_ends(const int* __restrict__ group_sizes, int G_total, int* ends) {
  __shared__ int wave_sum[kBwdThreads / kWave];
  const int tid = threadIdx.x, lane = tid % kWave, wave = tid / kWave;
  constexpr int PER = kBwdMaxGroups / kBwdThreads;
  int loc[PER], sum = 0;
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int g = tid * PER + j;
    sum += g < G_total ? max(group_sizes[g], 0) : 0;
    loc[j] = sum;
  }
  int incl = sum;
#pragma unroll
  for (int o = 1; o < kWave; o <<= 1) {
    const int t = __shfl_up(incl, o, kWave);
    if (lane >= o) incl += t;
  }
  if (lane == kWave - 1) wave_sum[wave] = incl;
  __syncthreads();
  int base = incl - sum;
  for (int w = 0; w < wave; w++) base += wave_sum[w];
#pragma unroll
  for (int j = 0; j < PER; j++) {
    const int g = tid * PER + j;
    if (g < G_total) ends[g] = base + loc[j];
  }
  __syncthreads();
}

// One block per row: d = bf16(dout * bf16(factor)), factor = rhs_scale[group(row), n] (BY_CHANNEL) or lhs_scale[row];
// ROW_QUANT: the row's absmax, then the e5m2 values and the row's scale.
template <bool BY_CHANNEL, bool ROW_QUANT, bool BYTES = false>
__global__ __launch_bounds__(kBwdThreads) void bwd_scale_rows_kernel(const uint4* dout, int N, const float* factor, const int* group_sizes,
                                                                     int G_total, int G_local, int group_offset, void* out,
                                                                     float* scale_out, int factor_stride = 1) {
  __shared__ int ends[BY_CHANNEL ? kBwdMaxGroups : 1];
  __shared__ uint32_t wmax[kBwdThreads / kWave];
  const int m = blockIdx.x, tid = threadIdx.x;
  const float* f = factor;
  float row_f = 1.0f;
  if (BY_CHANNEL) {
    block_group_ends(group_sizes, G_total, ends);
    f = factor + (size_t)local_group_of(ends, G_total, m, group_offset, G_local) * N;
  } else {
    row_f = round_bf16_fn(factor[(size_t)m * factor_stride]);  // (stride 0: one factor for the tensor)
  }
  const int nvec = N / 8;
  float v[kBwdMaxChunks][8];
  uint32_t amax_bits = 0u;  // max of the bit patterns of |d|: orders like the values, and a NaN's pattern beats every number's
#pragma unroll
  for (int c = 0; c < kBwdMaxChunks; c++) {
    const int i = c * kBwdThreads + tid;
    if (i < nvec) {
      const uint4 x = dout[(size_t)m * nvec + i];
      const uint32_t w[4] = {x.x, x.y, x.z, x.w};
#pragma unroll
      for (int e = 0; e < 8; e += 2) {
        const float x0 = __uint_as_float(w[e / 2] << 16), x1 = __uint_as_float(w[e / 2] & 0xffff0000u);
        float f0 = row_f, f1 = row_f;
        if (BY_CHANNEL) round_bf16_pair(f[i * 8 + e], f[i * 8 + e + 1], f0, f1);
        round_bf16_pair(x0 * f0, x1 * f1, v[c][e], v[c][e + 1]);
        amax_bits = max(amax_bits, max(__float_as_uint(v[c][e]) & 0x7fffffffu, __float_as_uint(v[c][e + 1]) & 0x7fffffffu));
      }
    }
  }
  E5m2Scale sc = {1.0f, 1.0f, false};
  if (ROW_QUANT) {
#pragma unroll
    for (int o = kWave / 2; o > 0; o >>= 1) amax_bits = max(amax_bits, (uint32_t)__shfl_xor((int)amax_bits, o, kWave));
    if (tid % kWave == 0) wmax[tid / kWave] = amax_bits;
    __syncthreads();
    const float amax = __uint_as_float(max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
    sc = e5m2_prepare(amax);
    if (tid == 0) scale_out[m] = sc.s;
  }
#pragma unroll
  for (int c = 0; c < kBwdMaxChunks; c++) {
    const int i = c * kBwdThreads + tid;
    if (i < nvec) {
      if (ROW_QUANT) {
        uint32_t pk[4];
#pragma unroll
        for (int e = 0; e < 4; e++) pk[e] = e5m2_bytes2(v[c][2 * e], v[c][2 * e + 1], sc, sc);
        store8_e5m2<BYTES>(out, (size_t)m * nvec + i, pk);
      } else {
        store8<false>(out, (size_t)m * nvec + i, v[c]);
      }
    }
  }
}

// Column maxima of |d|, d = bf16(dout * bf16(lhs_scale[m])): a block walks a band of rows, a lane owns 8 columns; the
// bands meet in an atomic max on the bit patterns (non-negative floats order like integers; a NaN's pattern is larger
// than every number's and so survives, as it does in the reference's amax).
constexpr int kColBand = 64;
__global__ __launch_bounds__(kBwdThreads) void bwd_col_absmax_kernel(const uint4* dout, int M, int N, const float* lhs_scale, int scale_stride,
                                                                     uint32_t* colmax) {
  const int nvec = N / 8;
  const int i = blockIdx.x * kBwdThreads + threadIdx.x;
  if (i >= nvec) return;
  const int m0 = blockIdx.y * kColBand, m1 = min(m0 + kColBand, M);
  uint32_t mx[8] = {0u, 0u, 0u, 0u, 0u, 0u, 0u, 0u};
#pragma unroll 8
  for (int m = m0; m < m1; m++) {
    const uint4 x = dout[(size_t)m * nvec + i];
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
    const float fm = round_bf16_fn(lhs_scale[(size_t)m * scale_stride]);
#pragma unroll
    for (int e = 0; e < 8; e += 2) {
      float d0, d1;
      round_bf16_pair(__uint_as_float(w[e / 2] << 16) * fm, __uint_as_float(w[e / 2] & 0xffff0000u) * fm, d0, d1);
      // (the bit patterns of |d| order like the values, and a NaN's pattern beats every number's)
      mx[e] = max(mx[e], __float_as_uint(d0) & 0x7fffffffu);
      mx[e + 1] = max(mx[e + 1], __float_as_uint(d1) & 0x7fffffffu);
    }
  }
#pragma unroll
  for (int e = 0; e < 8; e++) atomicMax(colmax + i * 8 + e, mx[e] > 0x7f800000u ? 0x7fc00000u : mx[e]);
}

__global__ void bwd_clear_kernel(uint32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// d on the e5m2 grid of its column's scale; `colmax` still holds the maxima
template <bool BYTES>
__global__ __launch_bounds__(kBwdThreads) void bwd_col_quant_kernel(const uint4* dout, int M, int N, const float* lhs_scale, int scale_stride,
                                                                    const float* colmax, void* out) {
  const int nvec = N / 8;
  const int i = blockIdx.x * kBwdThreads + threadIdx.x;
  if (i >= nvec) return;
  const int m0 = blockIdx.y * kColBand, m1 = min(m0 + kColBand, M);
  E5m2Scale s[8];
#pragma unroll
  for (int e = 0; e < 8; e++) s[e] = e5m2_prepare(colmax[i * 8 + e]);
#pragma unroll 4
  for (int m = m0; m < m1; m++) {
    const uint4 x = dout[(size_t)m * nvec + i];
    const uint32_t w[4] = {x.x, x.y, x.z, x.w};
    const float fm = round_bf16_fn(lhs_scale[(size_t)m * scale_stride]);
    uint32_t pk[4];
#pragma unroll
    for (int e = 0; e < 4; e++) {
      float d0, d1;
      round_bf16_pair(__uint_as_float(w[e] << 16) * fm, __uint_as_float(w[e] & 0xffff0000u) * fm, d0, d1);
      pk[e] = e5m2_bytes2(d0, d1, s[2 * e], s[2 * e + 1]);
    }
    store8_e5m2<BYTES>(out, (size_t)m * nvec + i, pk);
  }
}

// Per-tensor quantisation: every column's maximum becomes the maximum of them all (one block; the patterns order like the
// values and a NaN's beats every number's, as above).
__global__ __launch_bounds__(kBwdThreads) void bwd_col_merge_kernel(uint32_t* colmax, int n) {
  __shared__ uint32_t wmax[kBwdThreads / kWave];
  uint32_t mx = 0u;
  for (int i = threadIdx.x; i < n; i += kBwdThreads) mx = max(mx, colmax[i]);
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) mx = max(mx, (uint32_t)__shfl_xor((int)mx, o, kWave));
  if (threadIdx.x % kWave == 0) wmax[threadIdx.x / kWave] = mx;
  __syncthreads();
  mx = max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]));
  for (int i = threadIdx.x; i < n; i += kBwdThreads) colmax[i] = mx;
}

__global__ void bwd_col_scale_kernel(float* colmax, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) colmax[i] = e5m2_scale(colmax[i]);
}

// h + bias[expert of the row] for the rows of local groups, the others copied as they are: one block per row.
__global__ __launch_bounds__(kBwdThreads) void add_group_bias_kernel(const uint4* h, int N, const float* bias, const int* group_sizes, int G_total,
                                                                     int G_local, int group_offset, uint4* out) {
  __shared__ int ends[kBwdMaxGroups];
  const int m = blockIdx.x, tid = threadIdx.x;
  block_group_ends(group_sizes, G_total, ends);
  int lo = 0, hi = G_total;  // first group whose end lies past the row (G_total: the row is in no group)
  while (lo < hi) {
    const int mid = (lo + hi) >> 1;
    if (ends[mid] > m) hi = mid;
    else lo = mid + 1;
  }
  const int local = lo - group_offset;
  const bool owned = lo < G_total && local >= 0 && local < G_local;
  const float* b = bias + (size_t)(owned ? local : 0) * N;
  const int nvec = N / 8;
  for (int i = tid; i < nvec; i += kBwdThreads) {
    const uint4 x = h[(size_t)m * nvec + i];
    uint4 y = x;
    if (owned) {
      const uint32_t w[4] = {x.x, x.y, x.z, x.w};
      float o[8];
#pragma unroll
      for (int e = 0; e < 8; e++) o[e] = bf16_bits_to_f32((w[e / 2] >> (16 * (e & 1))) & 0xffffu) + b[i * 8 + e];
      y = make_uint4(pack_bf16x2(o[0], o[1]), pack_bf16x2(o[2], o[3]), pack_bf16x2(o[4], o[5]), pack_bf16x2(o[6], o[7]));
    }
    out[(size_t)m * nvec + i] = y;
  }
}

}  // namespace moe

using namespace moe;

extern "C" {

int moe_bwd_scale_grad(const void* dout, int M, int N, int mode, int quantize, const float* factor, const int32_t* group_sizes,
                       int num_groups_total, int num_groups_local, int group_offset, void* out, float* scale_out, void* stream) {
  if (!dout || !factor || !out) return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: NULL pointer");
  if (M < 0 || N <= 0) return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: bad sizes");
  if (mode != MOE_BWD_FOR_DLHS && mode != MOE_BWD_FOR_DRHS && mode != MOE_BWD_PER_TENSOR) return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: bad mode %d", mode);
  if (quantize < 0 || quantize > 2) return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: quantize must be 0, 1 (e5m2 values as bf16) or 2 (float8_e5m2 bytes)");
  if (quantize && !scale_out) return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: the quantised gradient needs a scale buffer");
  const bool bytes = quantize == 2;
  if (N % 8 != 0 || N > kBwdThreads * kBwdMaxChunks * 8) return fail(MOE_ERR_UNSUPPORTED, "bwd_scale_grad: need N%%8==0 and N<=16384 (N=%d)", N);
  if (M == 0) return MOE_OK;
  hipStream_t s = (hipStream_t)stream;
  const uint4* x = (const uint4*)dout;
  if (mode == MOE_BWD_FOR_DLHS) {
    if (!group_sizes || num_groups_total <= 0 || num_groups_total > kBwdMaxGroups || num_groups_local <= 0 || group_offset < 0)
      return fail(MOE_ERR_INVALID_ARG, "bwd_scale_grad: bad groups (at most %d)", kBwdMaxGroups);
    if (bytes)
      bwd_scale_rows_kernel<true, true, true><<<M, kBwdThreads, 0, s>>>(x, N, factor, group_sizes, num_groups_total, num_groups_local, group_offset, out, scale_out);
    else if (quantize)
      bwd_scale_rows_kernel<true, true><<<M, kBwdThreads, 0, s>>>(x, N, factor, group_sizes, num_groups_total, num_groups_local, group_offset, out, scale_out);
    else
      bwd_scale_rows_kernel<true, false><<<M, kBwdThreads, 0, s>>>(x, N, factor, group_sizes, num_groups_total, num_groups_local, group_offset, out, scale_out);
    return check_launch("bwd_scale_rows_kernel");
  }
  // per tensor: one factor for every row, and the columns' maxima merged into one before they are used
  const bool tensor = mode == MOE_BWD_PER_TENSOR;
  const int fstride = tensor ? 0 : 1;
  if (!quantize) {
    bwd_scale_rows_kernel<false, false><<<M, kBwdThreads, 0, s>>>(x, N, factor, nullptr, 0, 0, 0, out, scale_out, fstride);
    return check_launch("bwd_scale_rows_kernel");
  }
  // per column: clear the maxima, take them, quantise with them, turn them into the scales
  const int nvec = N / 8;
  const dim3 grid(cdiv(nvec, kBwdThreads), cdiv(M, kColBand));
  if (grid.y > 65535) return fail(MOE_ERR_UNSUPPORTED, "bwd_scale_grad: too many rows (%d)", M);
  bwd_clear_kernel<<<cdiv(N, 256), 256, 0, s>>>((uint32_t*)scale_out, N);
  bwd_col_absmax_kernel<<<grid, kBwdThreads, 0, s>>>(x, M, N, factor, fstride, (uint32_t*)scale_out);
  if (tensor) bwd_col_merge_kernel<<<1, kBwdThreads, 0, s>>>((uint32_t*)scale_out, N);
  if (bytes) bwd_col_quant_kernel<true><<<grid, kBwdThreads, 0, s>>>(x, M, N, factor, fstride, scale_out, out);
  else bwd_col_quant_kernel<false><<<grid, kBwdThreads, 0, s>>>(x, M, N, factor, fstride, scale_out, out);
  bwd_col_scale_kernel<<<cdiv(N, 256), 256, 0, s>>>(scale_out, N);
  return check_launch("bwd_col_quant_kernel");
}

int moe_add_group_bias(const void* h, int M, int N, const float* bias, const int32_t* group_sizes, int num_groups_total,
                       int num_groups_local, int group_offset, void* out, void* stream) {
  if (!h || !bias || !group_sizes || !out) return fail(MOE_ERR_INVALID_ARG, "add_group_bias: NULL pointer");
  if (M < 0 || N <= 0 || N % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "add_group_bias: need N %% 8 == 0 (N=%d)", N);
  if (num_groups_total <= 0 || num_groups_total > kBwdMaxGroups || num_groups_local <= 0 || group_offset < 0)
    return fail(MOE_ERR_INVALID_ARG, "add_group_bias: bad groups (at most %d)", kBwdMaxGroups);
  if (M == 0) return MOE_OK;
  add_group_bias_kernel<<<M, kBwdThreads, 0, (hipStream_t)stream>>>((const uint4*)h, N, bias, group_sizes, num_groups_total, num_groups_local,
                                                                     group_offset, (uint4*)out);
  return check_launch("add_group_bias_kernel");
}

}  // extern "C"
