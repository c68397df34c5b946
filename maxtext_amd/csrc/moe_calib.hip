// Calibration kernels: what the machine delivers with no memory system in the way (a register-only MFMA loop,
// with operands that stay constant or change every instruction) and with nothing but the memory system (a plain
// streaming read).  The benchmark reports them beside the roofline fractions of the real kernels, whose peaks are
// the published ones.

#include "moe_common.h"

namespace moe {

constexpr int kCalibAcc = 4;  // independent accumulators per wave: back-to-back MFMAs without dependency stalls

template <bool RANDOM>
__global__ __launch_bounds__(256) void calib_mfma_i8_kernel(int iters, int seed, int* __restrict__ sink) {
  v4i a = {seed + (int)threadIdx.x, seed * 3, seed * 5 + (int)threadIdx.x * 7, seed * 11};
  v4i b = {seed * 13, (int)threadIdx.x * 17, seed, seed * 23};
  v16i acc[kCalibAcc];
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < kCalibAcc; i++) {
      if (RANDOM) {  // one word of each operand moves every instruction (a linear congruential step)
        a[i & 3] = a[i & 3] * 1664525 + 1013904223;
        b[i & 3] = b[i & 3] * 22695477 + 1;
      }
      acc[i] = __builtin_amdgcn_mfma_i32_32x32x32_i8(a, b, acc[i], 0, 0, 0);
    }
  }
  int s = 0;
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = s;
}

template <bool RANDOM>
__global__ __launch_bounds__(256) void calib_mfma_bf16_kernel(int iters, int seed, int* __restrict__ sink) {
  v4i a = {0x3f803f80 + seed, 0x3f003f80, 0x40003f00 + (int)threadIdx.x, 0x3f803f00};
  v4i b = {0x3f003f80, 0x3f803f80 + (int)threadIdx.x, 0x3f803f00, 0x40003f80};
  v16f acc[kCalibAcc];
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) acc[i][r] = 0.f;
  for (int it = 0; it < iters; it++) {
#pragma unroll
    for (int i = 0; i < kCalibAcc; i++) {
      if (RANDOM) {  // mantissa and low exponent bits move, the values stay finite and of order one
        a[i & 3] = (a[i & 3] * 1664525 + 1013904223) & 0x00ff00ff | 0x3f003f00;
        b[i & 3] = (b[i & 3] * 22695477 + 1) & 0x00ff00ff | 0x3f003f00;
      }
      acc[i] = __builtin_amdgcn_mfma_f32_32x32x16_bf16(__builtin_bit_cast(v8bf, a), __builtin_bit_cast(v8bf, b), acc[i], 0, 0, 0);
    }
  }
  float s = 0.f;
#pragma unroll
  for (int i = 0; i < kCalibAcc; i++)
#pragma unroll
    for (int r = 0; r < 16; r++) s += acc[i][r];
  sink[blockIdx.x * 256 + threadIdx.x] = (int)s;
}

// every wave reads 8 KB per step with non-temporal requests of 1 KB (whole 128-byte lines: the request shape that
// streams fastest on this part), the grid strides over the buffer once
__global__ __launch_bounds__(256) void calib_read_kernel(const v4i* __restrict__ src, size_t nvec, int* __restrict__ sink) {
  constexpr int U = 8;
  const size_t stride = (size_t)gridDim.x * 256 * U;
  v4i s = {0, 0, 0, 0};
  for (size_t i = ((size_t)blockIdx.x * 256 + threadIdx.x / kWave * kWave) * U + threadIdx.x % kWave; i + (U - 1) * kWave < nvec; i += stride) {
    v4i v[U];
#pragma unroll
    for (int j = 0; j < U; j++) v[j] = __builtin_nontemporal_load(src + i + j * kWave);
#pragma unroll
    for (int j = 0; j < U; j++) s ^= v[j];
  }
  if ((s[0] ^ s[1] ^ s[2] ^ s[3]) == 0x12345678) sink[0] = 1;
}

constexpr int kCalibBlocks = 256 * 8;  // 2 waves per SIMD on 256 CUs

}  // namespace moe

using namespace moe;

extern "C" {

size_t moe_calib_scratch_bytes(void) { return (size_t)kCalibBlocks * 256 * sizeof(int); }

double moe_calib_mfma_ops(int dtype, int iters) {
  const double per_mfma = dtype == MOE_INT8 ? 2.0 * 32 * 32 * 32 : 2.0 * 32 * 32 * 16;
  return (double)kCalibBlocks * 4 * (double)iters * kCalibAcc * per_mfma;
}

int moe_calib_mfma(int dtype, int random_operands, int iters, void* scratch, void* stream) {
  if (!scratch || iters <= 0) return fail(MOE_ERR_INVALID_ARG, "calib_mfma: bad arguments");
  hipStream_t s = (hipStream_t)stream;
  int* sink = (int*)scratch;
  if (dtype == MOE_INT8) {
    if (random_operands) calib_mfma_i8_kernel<true><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
    else calib_mfma_i8_kernel<false><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
  } else if (dtype == MOE_BF16) {
    if (random_operands) calib_mfma_bf16_kernel<true><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
    else calib_mfma_bf16_kernel<false><<<kCalibBlocks, 256, 0, s>>>(iters, 12345, sink);
  } else {
    return fail(MOE_ERR_UNSUPPORTED, "calib_mfma: dtype %d", dtype);
  }
  return check_launch("calib_mfma_kernel");
}

int moe_calib_read(const void* src, size_t bytes, void* scratch, void* stream) {
  if (!src || !scratch || bytes < 65536 || ((uintptr_t)src & 15)) return fail(MOE_ERR_INVALID_ARG, "calib_read: bad arguments");
  calib_read_kernel<<<kCalibBlocks, 256, 0, (hipStream_t)stream>>>((const v4i*)src, bytes / 16, (int*)scratch);
  return check_launch("calib_read_kernel");
}

}  // extern "C"
