// On-the-fly weight quantiser of the training path: what gmm() does to its bf16 weights on every step,
// qpl.quantize(rhs, weight_qtype, channelwise_axes=[2]) (kernels/megablox/ops.py:250-260: one scale per output channel,
// shared by the experts and by K) or manual_quantize (layers/quantizations.py:961-991: one static scale for the tensor).
//
// Weights are [G, N, K] with K contiguous, so a channel's values are G rows of K.  Dynamic scales per channel are made
// and applied by one block per channel that sweeps its rows twice, the second time out of the caches (bf16 in once, 1 byte
// out: 3 bytes per value from HBM); a scale over more than a million values (per tensor, or hundreds of experts sharing
// long rows) takes two launches (5 bytes per value): every block reduces one row to its absmax and merges it into the
// scale's maximum with an atomic max on the bit pattern, the second pass divides by absmax / qmax and rounds.  A static
// scale needs the second pass only.

#include "moe_common.h"

namespace moe {

constexpr int kQThreads = 256;
constexpr int kQMaxChunks = 8;  // 8 bf16 per lane and chunk: rows of up to 16384 values

__device__ __forceinline__ void unpack_bf16x8(const uint4& u, float (&f)[8]) {
  const uint32_t w[4] = {u.x, u.y, u.z, u.w};
#pragma unroll
  for (int e = 0; e < 8; e++) f[e] = bf16_bits_to_f32((w[e / 2] >> (16 * (e & 1))) & 0xffffu);
}

__device__ __forceinline__ int scale_slot(int row, int N, int shared) { return shared == 2 ? 0 : shared ? row % N : row; }

// maxima[slot of the row] = max |w| over the row; slot = n (scales shared by the experts), g * N + n, or 0 (per tensor)
__global__ __launch_bounds__(kQThreads) void rhs_absmax_kernel(const uint4* __restrict__ w, int N, int K, int shared, uint32_t* __restrict__ maxima) {
  __shared__ uint32_t wmax[kQThreads / kWave];
  const int row = blockIdx.x, tid = threadIdx.x;
  const int nvec = K / 8;
  uint32_t m = 0u;  // bit patterns of non-negative floats order like the values; a NaN's pattern beats every number's
  for (int i = tid; i < nvec; i += kQThreads) {
    float f[8];
    unpack_bf16x8(w[(size_t)row * nvec + i], f);
#pragma unroll
    for (int e = 0; e < 8; e++) m = max(m, __float_as_uint(fabsf(f[e])));
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, o, kWave));
  if (tid % kWave == 0) wmax[tid / kWave] = m;
  __syncthreads();
  if (tid == 0) atomicMax(maxima + scale_slot(row, N, shared), max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3])));
}

// MODE 0: int8, 1: float8_e4m3fn.  STATIC: q = clip(bf16(w / bf16(scale)), +-bf16(qmax)) cast as `.astype` does (int8
// truncates, fp8 rounds to nearest even), manual_quantize's arithmetic for bf16 weights.  Otherwise scale = absmax / qmax
// and q = rint(w / scale) (int8) or the nearest-even cast of w / scale (fp8), in f32; a zero scale gives zeros.
template <int MODE, bool STATIC>
__global__ __launch_bounds__(kQThreads) void rhs_quant_kernel(const uint4* __restrict__ w, int N, int K, int shared, const float* __restrict__ maxima,
                                                               const float* __restrict__ static_scale, uint2* __restrict__ q) {
  const int row = blockIdx.x, tid = threadIdx.x;
  const int nvec = K / 8;
  const float qmax = MODE == 0 ? 127.0f : 448.0f;
  float sc;
  if (STATIC) sc = round_bf16_fn(*static_scale);
  else sc = maxima[scale_slot(row, N, shared)] / qmax;
  for (int i = tid; i < nvec; i += kQThreads) {
    float f[8];
    unpack_bf16x8(w[(size_t)row * nvec + i], f);
#pragma unroll
    for (int e = 0; e < 8; e++) {
      float y;
      if (STATIC) {
        y = fminf(fmaxf(round_bf16_fn(f[e] / sc), -qmax), qmax);  // (127 and 448 are bf16 values)
        if (MODE == 0) y = truncf(y);
      } else {
        y = sc == 0.f ? 0.f : f[e] / sc;
        y = fminf(fmaxf(MODE == 0 ? rintf(y) : y, -qmax), qmax);
      }
      f[e] = y;
    }
    uint32_t lo, hi;
    if (MODE == 0) {
      uint32_t b[8];
#pragma unroll
      for (int e = 0; e < 8; e++) b[e] = (uint32_t)((int)f[e]) & 0xffu;
      lo = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
      hi = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
    } else {
      int l = 0, h = 0;
      l = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], l, false);
      l = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], l, true);
      h = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], h, false);
      h = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], h, true);
      lo = (uint32_t)l;
      hi = (uint32_t)h;
    }
    q[(size_t)row * nvec + i] = make_uint2(lo, hi);
  }
}

// Dynamic scales per channel in one launch: a block owns one scale (a channel's G rows of K when the experts share it,
// one row otherwise), sweeps its rows once for the absmax and a second time, while they still sit in the caches (64 to
// 230 KB per block on the Mixtral shapes), to quantise them: the weights come from HBM once instead of twice.  Same
// arithmetic as the two kernels above.
template <int MODE>
__global__ __launch_bounds__(kQThreads) void rhs_quant_slot_kernel(const uint4* __restrict__ w, int G, int N, int K, int shared, uint2* __restrict__ q,
                                                                    float* __restrict__ scale) {
  __shared__ uint32_t wmax[kQThreads / kWave];
  const int slot = blockIdx.x, tid = threadIdx.x;
  const int nvec = K / 8, nrows = shared ? G : 1;
  const float qmax = MODE == 0 ? 127.0f : 448.0f;
  uint32_t m = 0u;
  for (int r = 0; r < nrows; r++) {
    const uint4* row = w + ((size_t)(shared ? r * N + slot : slot)) * nvec;
    for (int i = tid; i < nvec; i += kQThreads) {
      float f[8];
      unpack_bf16x8(row[i], f);
#pragma unroll
      for (int e = 0; e < 8; e++) m = max(m, __float_as_uint(fabsf(f[e])));
    }
  }
#pragma unroll
  for (int o = kWave / 2; o > 0; o >>= 1) m = max(m, (uint32_t)__shfl_xor((int)m, o, kWave));
  if (tid % kWave == 0) wmax[tid / kWave] = m;
  __syncthreads();
  const float sc = __uint_as_float(max(max(wmax[0], wmax[1]), max(wmax[2], wmax[3]))) / qmax;
  if (tid == 0) scale[slot] = sc;
  for (int r = 0; r < nrows; r++) {
    const size_t base = ((size_t)(shared ? r * N + slot : slot)) * nvec;
    for (int i = tid; i < nvec; i += kQThreads) {
      float f[8];
      unpack_bf16x8(w[base + i], f);
#pragma unroll
      for (int e = 0; e < 8; e++) {
        const float y = sc == 0.f ? 0.f : f[e] / sc;
        f[e] = fminf(fmaxf(MODE == 0 ? rintf(y) : y, -qmax), qmax);
      }
      uint32_t lo, hi;
      if (MODE == 0) {
        uint32_t b[8];
#pragma unroll
        for (int e = 0; e < 8; e++) b[e] = (uint32_t)((int)f[e]) & 0xffu;
        lo = b[0] | (b[1] << 8) | (b[2] << 16) | (b[3] << 24);
        hi = b[4] | (b[5] << 8) | (b[6] << 16) | (b[7] << 24);
      } else {
        int l = 0, h = 0;
        l = __builtin_amdgcn_cvt_pk_fp8_f32(f[0], f[1], l, false);
        l = __builtin_amdgcn_cvt_pk_fp8_f32(f[2], f[3], l, true);
        h = __builtin_amdgcn_cvt_pk_fp8_f32(f[4], f[5], h, false);
        h = __builtin_amdgcn_cvt_pk_fp8_f32(f[6], f[7], h, true);
        lo = (uint32_t)l;
        hi = (uint32_t)h;
      }
      q[base + i] = make_uint2(lo, hi);
    }
  }
}

__global__ void rhs_clear_kernel(uint32_t* p, int n) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = 0u;
}

// maxima -> scales, in place
__global__ void rhs_scale_kernel(float* p, int n, float qmax) {
  const int i = blockIdx.x * blockDim.x + threadIdx.x;
  if (i < n) p[i] = p[i] / qmax;
}

}  // namespace moe

using namespace moe;

extern "C" int moe_quantize_rhs(const void* w, int G, int N, int K, int out_dtype, int shared, const float* static_scale, void* q,
                                float* scale, void* stream) {
  if (!w || !q) return fail(MOE_ERR_INVALID_ARG, "quantize_rhs: NULL pointer");
  if (G <= 0 || N <= 0 || K <= 0) return fail(MOE_ERR_INVALID_ARG, "quantize_rhs: bad sizes");
  if (out_dtype != MOE_INT8 && out_dtype != MOE_FP8_E4M3) return fail(MOE_ERR_UNSUPPORTED, "quantize_rhs: out_dtype %d", out_dtype);
  if (K % 8 != 0) return fail(MOE_ERR_UNSUPPORTED, "quantize_rhs: K %% 8 != 0 (K=%d)", K);
  if ((long long)G * N > 0x7fffffffLL) return fail(MOE_ERR_UNSUPPORTED, "quantize_rhs: too many rows");
  if (!static_scale && !scale) return fail(MOE_ERR_INVALID_ARG, "quantize_rhs: dynamic scales need a scale buffer");
  if ((((uintptr_t)w) & 15) || (((uintptr_t)q) & 7)) return fail(MOE_ERR_UNSUPPORTED, "quantize_rhs: w must be 16-byte and q 8-byte aligned");
  hipStream_t s = (hipStream_t)stream;
  const int rows = G * N;
  const uint4* x = (const uint4*)w;
  if (static_scale) {
    if (out_dtype == MOE_INT8) rhs_quant_kernel<0, true><<<rows, kQThreads, 0, s>>>(x, N, K, 0, nullptr, static_scale, (uint2*)q);
    else rhs_quant_kernel<1, true><<<rows, kQThreads, 0, s>>>(x, N, K, 0, nullptr, static_scale, (uint2*)q);
    return check_launch("rhs_quant_kernel");
  }
  if (shared < 0 || shared > 2) return fail(MOE_ERR_INVALID_ARG, "quantize_rhs: shared must be 0 (per expert), 1 (shared by the experts) or 2 (per tensor)");
  const int ns = shared == 2 ? 1 : shared ? N : rows;
  // a scale whose values fit the caches between two sweeps of one block (2 MB: 128 experts of 8192) is made and applied in
  // one launch
  if (shared != 2 && (long long)(shared ? G : 1) * K <= (1LL << 20)) {
    if (out_dtype == MOE_INT8) rhs_quant_slot_kernel<0><<<ns, kQThreads, 0, s>>>(x, G, N, K, shared, (uint2*)q, scale);
    else rhs_quant_slot_kernel<1><<<ns, kQThreads, 0, s>>>(x, G, N, K, shared, (uint2*)q, scale);
    return check_launch("rhs_quant_slot_kernel");
  }
  rhs_clear_kernel<<<cdiv(ns, 256), 256, 0, s>>>((uint32_t*)scale, ns);
  rhs_absmax_kernel<<<rows, kQThreads, 0, s>>>(x, N, K, shared, (uint32_t*)scale);
  if (out_dtype == MOE_INT8) rhs_quant_kernel<0, false><<<rows, kQThreads, 0, s>>>(x, N, K, shared, scale, nullptr, (uint2*)q);
  else rhs_quant_kernel<1, false><<<rows, kQThreads, 0, s>>>(x, N, K, shared, scale, nullptr, (uint2*)q);
  rhs_scale_kernel<<<cdiv(ns, 256), 256, 0, s>>>(scale, ns, out_dtype == MOE_INT8 ? 127.0f : 448.0f);
  return check_launch("rhs_quant_kernel");
}

extern "C" int moe_tensor_scale(const void* x, long long rows, int K, float qmax, float* scale, void* stream) {
  if (!x || !scale) return fail(MOE_ERR_INVALID_ARG, "tensor_scale: NULL pointer");
  if (rows < 0 || rows > 0x7fffffffLL || K <= 0 || K % 8 != 0 || !(qmax > 0.f)) return fail(MOE_ERR_INVALID_ARG, "tensor_scale: bad sizes (K %% 8 == 0)");
  hipStream_t s = (hipStream_t)stream;
  rhs_clear_kernel<<<1, 64, 0, s>>>((uint32_t*)scale, 1);
  if (rows > 0) rhs_absmax_kernel<<<(unsigned)rows, kQThreads, 0, s>>>((const uint4*)x, 1, K, 2, (uint32_t*)scale);
  rhs_scale_kernel<<<1, 64, 0, s>>>(scale, 1, qmax);
  return check_launch("tensor_scale");
}
